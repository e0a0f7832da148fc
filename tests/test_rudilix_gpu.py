"""Rudilix through the engine against the plain implementation (``plain_rudilix.py``,
float64, whole sequences, one function per mechanism).

float32 runs are held to the plain logits row by row (root mean square of the
difference over the vocabulary, relative to the logits' own spread): measured 1e-6 to
7e-6, bound 1e-4.  That is the bound that can fail, and every schedule, cut and batch is
held to it.  A bfloat16 run is chaotic at single rows: the delta rule's read-out is divided
by its own root mean square, which for a request's first tokens is a multiple of q . k, a
number that may be as small as its rounding error, and the weights here are drawn sharp on
purpose.  So bfloat16 rows are held to the plain logits by their median and their ninth
decile, and the worst row only to a bound that says that nothing is grossly wrong; the
bounds were measured first (median 0.009 to 0.011, ninth decile 0.015 to 0.02, worst row
0.07 and 0.28) and then set with margins.  How a bfloat16 request was cut and batched must
not show beyond rounding either: every schedule is held to the whole prompts' run."""

import math

import pytest
import torch

import engine_util as eu
import plain_rudilix as plain
import rudilix_util as ru

pytestmark = pytest.mark.gpu

F32_BOUND = 1e-4
BF16_MEDIAN, BF16_DECILE, BF16_WORST = 0.04, 0.12, 0.6
BF16_BETWEEN_MEDIAN, BF16_BETWEEN_WORST = 1e-3, 0.03      # one schedule against another (measured 0 and 0.006)


def build(cfg, seed=0, dtype="float32", tensors=None):
    from zig_ai_amd.engine import DecoderModel
    d, tensors = ru.folder(cfg, seed, tensors)
    return DecoderModel.from_folder(d, dtype), tensors


def runner_for(model, page_size=4, tokens=256, slots=4, graphs=True):
    from zig_ai_amd.engine import ModelRunner
    return ModelRunner(model, page_size=page_size, num_pages=max(1, -(-tokens // page_size)),
                       num_slots=slots, use_graphs=graphs)


def plain_logits(cfg, tensors, prompts):
    return [plain.forward(cfg, tensors, p).float() for p in prompts]


def worst(got, want):
    return float(ru.row_error(got, want).max())


def assert_bfloat16_close(got, want, what=None):
    e = ru.row_error(got, want)
    found = (float(e.median()), float(e.quantile(0.9)), float(e.max()))
    assert found[0] < BF16_MEDIAN and found[1] < BF16_DECILE and found[2] < BF16_WORST, (what, found)


# ----------------------------------------------------------- each mechanism alone
ALONE = {
    "ssd": ru.one_layer("mamba2", ru.ssd()),
    "ssd one group": ru.one_layer("mamba2", ru.ssd(heads=2, vdim=24, state=72, groups=1,
                                                     norm_groups=1, conv=2), ff=0),
    "delta": ru.one_layer("channel_delta", ru.delta()),
    "delta wide": ru.one_layer("channel_delta", ru.delta(heads=2, kv_heads=1, dim=40, vdim=72,
                                                          conv=4), ff=0),
    "delta one tap": ru.one_layer("channel_delta", ru.delta(heads=3, kv_heads=3, dim=16, vdim=16,
                                                             conv=1)),
    "attention + delta": ru.one_layer("parallel", ru.parallel()),
    "attention alone": ru.one_layer("parallel", ru.parallel(right_scale=0.0), ff=0),
    "attention, full rotation, no window": ru.one_layer("parallel", ru.parallel(
        ru.attention(heads=6, kv_heads=2, dim=16, vdim=16, window=0, rot_dims=16, scale=0.4),
        right_scale=0.0)),
}


@pytest.mark.parametrize("name", sorted(ALONE))
def test_mechanism_alone(name):
    cfg = ALONE[name]
    model, tensors = build(cfg, seed=3)
    prompts = [ru.tokens(70, cfg["vocab"], 1), ru.tokens(5, cfg["vocab"], 2)]
    want = plain_logits(cfg, tensors, prompts)
    runner = runner_for(model)
    got = eu.run_schedule(runner, prompts, eu.whole([len(p) for p in prompts]))
    for g, w in zip(got, want):
        assert worst(g, w) < F32_BOUND
    # the same, token by token from the first token on: the state and the cache alone
    got = eu.run_schedule(runner, prompts, eu.bulk_then_single([len(p) for p in prompts], tail=10 ** 6))
    for g, w in zip(got, want):
        assert worst(g, w) < F32_BOUND


# -------------------------------------------------------- schedules of whole models
LENGTHS = [150, 37, 9, 1, 75, 130, 2]


def schedules(lengths):
    return {
        "whole": eu.whole(lengths),
        "bulk + tail": eu.bulk_then_single(lengths, tail=40),
        "portions": eu.changing_portions(lengths, seed=1),
        "portions of two": eu.changing_portions(lengths, seed=0, sizes=(2, 2, 3, 2, 17)),
        "mixed": eu.mixed(lengths, seed=2, max_live=4, decode_tail=20),
        "mixed, three live": eu.mixed(lengths, seed=5, max_live=3, decode_tail=45),
    }


@pytest.mark.parametrize("which", ["all", "other"])
@pytest.mark.parametrize("page_size", [4, 16])
def test_schedules_float32(which, page_size):
    cfg = ru.TINY_ALL if which == "all" else ru.TINY_OTHER
    model, tensors = build(cfg, seed=11)
    prompts = [ru.tokens(n, cfg["vocab"], 20 + i) for i, n in enumerate(LENGTHS)]
    want = plain_logits(cfg, tensors, prompts)
    for name, schedule in schedules(LENGTHS).items():
        # a pool for the most tokens live at any time: pages and slots are used again
        peak = eu.peak_tokens(LENGTHS, schedule, round_to=max(16, page_size))
        runner = runner_for(model, page_size=page_size, tokens=peak, slots=4)
        got = eu.run_schedule(runner, prompts, schedule)
        for i, (g, w) in enumerate(zip(got, want)):
            assert worst(g, w) < F32_BOUND, (name, i)
        if "mixed" in name:
            assert runner.cache.pages_reused > 0
        assert len(runner.cache.requests) == 0


@pytest.mark.parametrize("which", ["all", "other"])
def test_schedules_bfloat16(which):
    cfg = ru.TINY_ALL if which == "all" else ru.TINY_OTHER
    model, tensors = build(cfg, seed=11, dtype="bfloat16")
    prompts = [ru.tokens(n, cfg["vocab"], 20 + i) for i, n in enumerate(LENGTHS)]
    want = plain_logits(cfg, tensors, prompts)
    base = None
    for name, schedule in schedules(LENGTHS).items():
        peak = eu.peak_tokens(LENGTHS, schedule, round_to=16)
        runner = runner_for(model, page_size=16, tokens=peak, slots=4)
        got = eu.run_schedule(runner, prompts, schedule)
        assert_bfloat16_close(torch.cat(got), torch.cat(want), name)
        if base is None:
            base = got
        e = ru.row_error(torch.cat(got), torch.cat(base))
        assert float(e.median()) < BF16_BETWEEN_MEDIAN and float(e.max()) < BF16_BETWEEN_WORST, \
            (name, float(e.median()), float(e.max()))


# ---------------------------------------- configurations drawn at random, both types
@pytest.mark.parametrize("seed", range(12))
def test_random_configurations(seed):
    cfg = ru.random_config(seed)
    lengths = [70, 1, 33, 12, 2]
    prompts = [ru.tokens(n, cfg["vocab"], 90 + i) for i, n in enumerate(lengths)]
    model, tensors = build(cfg, seed=seed)
    want = plain_logits(cfg, tensors, prompts)
    for name, schedule in (("whole", eu.whole(lengths)),
                           ("portions", eu.changing_portions(lengths, seed=seed)),
                           ("mixed", eu.mixed(lengths, seed=seed, max_live=3, decode_tail=9))):
        peak = eu.peak_tokens(lengths, schedule, round_to=16)
        runner = runner_for(model, page_size=4 if seed % 2 else 16, tokens=peak, slots=3)
        got = eu.run_schedule(runner, prompts, schedule)
        # (a model drawn with hardly any spread in its logits is measured against that
        # spread all the same; the bound allows for it)
        for i, (g, w) in enumerate(zip(got, want)):
            assert worst(g, w) < 3 * F32_BOUND, (name, i, cfg)
    # the same model in bfloat16 runs (odd widths fall back to 32-bit weights) and agrees
    # with itself across schedules
    model16, _ = build(cfg, seed=seed, dtype="bfloat16")
    base = None
    for schedule in (eu.whole(lengths), eu.mixed(lengths, seed=seed, max_live=3, decode_tail=9)):
        got = eu.run_schedule(runner_for(model16, page_size=16, tokens=256, slots=3), prompts, schedule)
        assert all(torch.isfinite(g).all() for g in got)
        base = base or got
        e = ru.row_error(torch.cat(got), torch.cat(base))
        assert float(e.median()) < BF16_BETWEEN_MEDIAN, float(e.median())


# --------------------------------------------- window edges, with scores that stand out
def sharp_window_cfg(window, rot):
    # a scale that makes the softmax all but choose one key: a key wrongly seen or wrongly
    # hidden then takes or loses nearly all of a query's weight
    att = ru.attention(heads=2, kv_heads=1, dim=16, vdim=16, window=window, rot_dims=rot,
                       base=100.0, scale=2.5)
    return ru.one_layer("parallel", ru.parallel(att, left_scale=1.0, right_scale=0.0), ff=0)


@pytest.mark.parametrize("window,rot", [(7, 0), (16, 8), (1, 16), (21, 4)])
def test_window_edges(window, rot):
    cfg = sharp_window_cfg(window, rot)
    model, tensors = build(cfg, seed=5)
    n = 90
    prompts = [ru.tokens(n, cfg["vocab"], 7)]
    want = plain_logits(cfg, tensors, prompts)[0]
    # the test can see an edge that is one token off: the plain implementation itself,
    # one key more or one fewer, is far from what it gives with the right window
    for other in (window - 1, window + 1):
        if other >= 1:
            off = sharp_window_cfg(other, rot)
            assert worst(plain.forward(off, tensors, prompts[0]).float(), want) > 0.05
    for page_size in (4, 16):
        for name, schedule in (("whole", eu.whole([n])),
                               ("decoded", eu.bulk_then_single([n], tail=n - 3)),
                               ("portions", eu.changing_portions([n], sizes=(5, 2, window, 3, window + 1)))):
            runner = runner_for(model, page_size=page_size, tokens=128)
            got = eu.run_schedule(runner, prompts, schedule)[0]
            assert worst(got, want) < 2e-3, (name, page_size)


# ------------------- key and value widths that the matrix-core attention kernels take
@pytest.mark.parametrize("dim,window,rot", [(64, 40, 32), (128, 0, 128), (64, 130, 0)])
def test_matrix_core_attention_with_gate(dim, window, rot):
    att = ru.attention(heads=4, kv_heads=2, dim=dim, vdim=dim, window=window, rot_dims=rot,
                       base=1000.0, scale=dim ** -0.5)
    cfg = ru.config([ru.layer("parallel", ru.parallel(att, ru.delta(), 1.0, 0.5), ff=64)], width=128)
    model, tensors = build(cfg, seed=6, dtype="bfloat16")
    assert model.blocks[0].parts["left"].mfma
    lengths = [200, 70, 3]
    prompts = [ru.tokens(n, cfg["vocab"], 50 + i) for i, n in enumerate(lengths)]
    want = plain_logits(cfg, tensors, prompts)
    base = None
    for name, schedule in (("whole", eu.whole(lengths)),
                           ("bulk + tail", eu.bulk_then_single(lengths, tail=60)),
                           ("portions", eu.changing_portions(lengths, seed=3)),
                           ("mixed", eu.mixed(lengths, seed=1, max_live=3, decode_tail=30))):
        runner = runner_for(model, page_size=16, tokens=512, slots=3)
        got = eu.run_schedule(runner, prompts, schedule)
        assert_bfloat16_close(torch.cat(got), torch.cat(want), name)
        base = base or got
        e = ru.row_error(torch.cat(got), torch.cat(base))
        assert float(e.median()) < BF16_BETWEEN_MEDIAN and float(e.max()) < BF16_BETWEEN_WORST, \
            (name, float(e.median()), float(e.max()))


# ---------------- a width at which a decode batch's opening products run the norm themselves
def test_decode_batches_at_a_width_of_512():
    from zig_ai_amd.kernels import ops
    cfg = ru.config([ru.layer("parallel", ru.parallel()), ru.layer("mamba2", ru.ssd()),
                     ru.layer("channel_delta", ru.delta(), ff=0)], width=512)
    model, tensors = build(cfg, seed=13, dtype="bfloat16")
    assert ops.normed_rows_fusable(3, 512)
    lengths = [60, 25, 8]
    prompts = [ru.tokens(n, cfg["vocab"], 70 + i) for i, n in enumerate(lengths)]
    want = plain_logits(cfg, tensors, prompts)
    whole = eu.run_schedule(runner_for(model, page_size=16, tokens=256), prompts, eu.whole(lengths))
    # all three decode together from their fifth token on: steps of three rows
    steps = [([(i, 0, 4) for i in range(3)], [])]
    steps += [([(i, p, p + 1) for i, n in enumerate(lengths) if p < n],
               [i for i, n in enumerate(lengths) if p == n - 1]) for p in range(4, max(lengths))]
    got = eu.run_schedule(runner_for(model, page_size=16, tokens=256, graphs=False), prompts, steps)
    # (such a step does take that form)
    from zig_ai_amd.engine import StepEntry
    runner = runner_for(model, page_size=16, tokens=64, graphs=False)
    runner.admit("x")
    runner.step([StepEntry("x", prompts[2][:4], [])])
    ops.form_log = []
    try:
        runner.step([StepEntry("x", prompts[2][4:5], [0])])
        assert any(r.get("norm_in_product") for r in ops.form_log if r["op"] == "linear")
    finally:
        ops.form_log = None
    assert_bfloat16_close(torch.cat(got), torch.cat(want))
    # (a product that runs the norm rounds x * weight and scales its sums, the norm as a
    # kernel rounds x * scale * weight: the two runs differ as two roundings do, measured
    # median 0.010, worst 0.038)
    assert_bfloat16_close(torch.cat(got), torch.cat(whole))
    # and replayed from graphs
    again = eu.run_schedule(runner_for(model, page_size=16, tokens=256), prompts, steps)
    e = ru.row_error(torch.cat(again), torch.cat(got))
    assert float(e.max()) < BF16_BETWEEN_WORST


# ----------------------------------------------------------------- far tokens count
@pytest.mark.parametrize("kind", ["mamba2", "channel_delta"])
def test_far_tokens_reach_the_end(kind):
    mixer = ru.ssd(heads=2, vdim=16, state=16, groups=1, norm_groups=1, conv=2) \
        if kind == "mamba2" else ru.delta(heads=2, kv_heads=2, dim=16, vdim=16, conv=2)
    cfg = ru.one_layer(kind, mixer, ff=0)
    tensors = ru.make_tensors(cfg, seed=9)
    tensors["l0.mix.A_log"] = torch.full_like(tensors["l0.mix.A_log"], -8.0)   # all but no decay
    model, tensors = build(cfg, tensors=tensors)
    # (the delta rule overwrites: its state of 16 key channels keeps a token for some tens of
    # steps whatever the decay)
    n = 400 if kind == "mamba2" else 40
    a = ru.tokens(n, cfg["vocab"], 3)
    b = list(a)
    b[1] = (b[1] + 1) % cfg["vocab"]
    wa, wb = plain.forward(cfg, tensors, a).float(), plain.forward(cfg, tensors, b).float()
    assert worst(wb[-8:], wa[-8:]) > 1e-2          # the second token still shows at the end
    for prompt, want in ((a, wa), (b, wb)):
        for schedule in (eu.whole([n]), eu.bulk_then_single([n], tail=64),
                         eu.changing_portions([n], sizes=(33, 2, 64, 17))):
            got = eu.run_schedule(runner_for(model, tokens=512), [prompt], schedule)[0]
            assert worst(got, want) < F32_BOUND
    # nothing is left of a request whose slot is taken again: b after a in a pool of one slot
    runner = runner_for(model, tokens=512, slots=1)
    for prompt, want in ((a, wa), (b, wb), (a, wa)):
        got = eu.run_schedule(runner, [prompt], eu.bulk_then_single([n], tail=5))[0]
        assert worst(got, want) < F32_BOUND


# ------------------------------------- a long context cut into ranges, with the gate
def test_long_context_without_window():
    cfg = ru.TINY_OTHER
    model, tensors = build(cfg, seed=4)
    n = 700
    prompts = [ru.tokens(n, cfg["vocab"], 1), ru.tokens(30, cfg["vocab"], 2)]
    want = plain_logits(cfg, tensors, prompts)
    runner = runner_for(model, page_size=16, tokens=1024)
    wants = [list(range(n - 90, n)), list(range(30))]
    steps = [([(0, 0, n - 80)], [])]
    # the long request decodes beside the short one's portions and single tokens
    steps += [([(0, n - 80 + i, n - 79 + i)] + ([(1, 3 * i, 3 * i + 3)] if i < 10 else []),
               [1] if i == 9 else []) for i in range(80)]
    steps[-1] = (steps[-1][0], [0])
    got = eu.run_schedule(runner, prompts, steps, wants=wants)
    assert worst(got[0], want[0][n - 90:]) < F32_BOUND
    assert worst(got[1], want[1]) < F32_BOUND


# ------------------------------------------------------------------- long decoding
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(dtype):
    cfg = ru.TINY_ALL
    model, tensors = build(cfg, seed=21, dtype=dtype)
    n = 330
    prompts = [ru.tokens(n, cfg["vocab"], 5)]
    want = plain_logits(cfg, tensors, prompts)[0]
    runner = runner_for(model, page_size=16, tokens=512)       # decode steps replay from graphs
    got = eu.run_schedule(runner, prompts, eu.bulk_then_single([n], tail=300))[0]
    if dtype == "float32":
        assert worst(got, want) < F32_BOUND
    else:
        assert_bfloat16_close(got, want)


# ------------------------------------------- unequal requests together and alone
def test_batch_against_each_alone():
    cfg = ru.TINY_ALL
    model, tensors = build(cfg, seed=2, dtype="bfloat16")
    lengths = [64, 3, 41, 17]
    prompts = [ru.tokens(n, cfg["vocab"], 40 + i) for i, n in enumerate(lengths)]
    alone = eu.run_schedule(runner_for(model, tokens=256), prompts, eu.whole(lengths))
    together = [([(i, 0, n) for i, n in enumerate(lengths)], list(range(len(lengths))))]
    got = eu.run_schedule(runner_for(model, tokens=256), prompts, together)
    assert_bfloat16_close(torch.cat(got), torch.cat(alone))


# ------------------------------------------- generation through engine and scheduler
def test_greedy_generation():
    from zig_ai_amd.engine import Engine
    cfg = ru.TINY_ALL
    d, tensors = ru.folder(cfg, seed=8)
    engine = Engine(d, dtype="float32", page_size=4, num_pages=128, max_num_seqs=3,
                    max_num_batched_tokens=48, chunk_size=20, max_model_len=256)
    prompts = [ru.tokens(n, cfg["vocab"], 60 + i) for i, n in enumerate([33, 5, 70, 12, 1])]
    outs = engine.generate(prompts, max_new_tokens=20, temperature=0.0)
    assert all(len(o) == 20 for o in outs)
    for p, o in zip(prompts, outs):
        # every chosen token is the plain implementation's choice for the same history
        logits = plain.forward(cfg, tensors, p + o)
        for j, tok in enumerate(o):
            row = logits[len(p) + j - 1]
            assert float(row.max() - row[tok]) <= 1e-3 * float(row.abs().max()), (j, tok)
    assert len(engine.runner.cache.requests) == 0
    engine.runner.cache.check()


def test_generation_bfloat16_runs_through_graphs():
    from zig_ai_amd.engine import Engine
    cfg = ru.TINY_OTHER
    d, tensors = ru.folder(cfg, seed=8)
    engine = Engine(d, dtype="bfloat16", page_size=16, num_pages=64, max_num_seqs=4,
                    max_model_len=256)
    assert engine.runner.graphs is not None        # every part can be recorded
    prompts = [ru.tokens(n, cfg["vocab"], 80 + i) for i, n in enumerate([40, 7, 19])]
    outs = engine.generate(prompts, max_new_tokens=24, temperature=0.0)
    for p, o in zip(prompts, outs):
        logits = plain.forward(cfg, tensors, p + o)
        for j, tok in enumerate(o):
            row = logits[len(p) + j - 1]
            spread = float(row.max() - row.min())
            assert float(row.max() - row[tok]) <= 0.1 * spread, (j, tok)


# ------------------------------------------------------------------ kernels alone
def _slots(n_slots, floats, device):
    # rows spaced wider than their length, as the cache manager's slot rows are
    mem = torch.zeros((n_slots, floats + 12), dtype=torch.float32, device=device)
    return mem, mem[:, :floats]


def _step_arrays(lengths, slots, device):
    seq = [i for i, n in enumerate(lengths) for _ in range(n)]
    start = [0]
    for n in lengths:
        start.append(start[-1] + n)
    mk = lambda v: torch.tensor(v, dtype=torch.int32, device=device)
    return mk(seq), mk(start), mk(slots)


@pytest.mark.parametrize("taps,dtype", [(4, torch.float32), (2, torch.bfloat16), (1, torch.float32),
                                        (8, torch.bfloat16)])
def test_causal_conv_kernel(taps, dtype):
    from zig_ai_amd.kernels import ops
    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(taps)
    C, col0, width = 70, 5, 90
    lengths_a, lengths_b = [13, 1, 2, 40], [1, 5, 1, 3]      # two steps of the same requests
    n_a, n_b = sum(lengths_a), sum(lengths_b)
    x = torch.randn(n_a + n_b, width, generator=g).to(dtype)
    w = torch.randn(C, taps, generator=g)
    bias = torch.randn(C, generator=g)
    mem, state = _slots(6, C * (taps - 1) + 7, dev)
    slots = [4, 0, 5, 2]
    xa, xb = x[:n_a].to(dev).contiguous(), x[n_a:].to(dev).contiguous()
    ya = ops.causal_conv_silu(xa, col0, w.to(dev), bias.to(dev), state, 7,
                              *_step_arrays(lengths_a, slots, dev)).cpu()
    yb = ops.causal_conv_silu(xb, col0, w.to(dev), bias.to(dev), state, 7,
                              *_step_arrays(lengths_b, slots, dev)).cpu()
    a0 = b0 = 0
    for la, lb in zip(lengths_a, lengths_b):
        whole = torch.cat([x[a0:a0 + la], x[n_a + b0:n_a + b0 + lb]]).double()[:, col0:col0 + C]
        want = plain.silu(plain.causal_conv(whole, w.double(), bias.double()))
        got = torch.cat([ya[a0:a0 + la], yb[b0:b0 + lb]]).double()
        assert float((got - want).abs().max()) < 1e-5
        a0, b0 = a0 + la, b0 + lb
    assert float(mem[:, C * (taps - 1) + 7:].abs().max()) == 0.0     # nothing beyond the window
    assert float(state[1].abs().max()) == 0.0                        # a slot nobody uses


def _plain_delta(q, k, v, beta, decay):
    T, H, d = decay.shape
    G, dv = q.shape[1], v.shape[2]
    out = torch.zeros((T, H, dv), dtype=torch.float64)
    for h in range(H):
        g = h // (H // G)
        S = torch.zeros((d, dv), dtype=torch.float64)
        for t in range(T):
            S = decay[t, h][:, None] * S
            u = beta[t, h] * (v[t, h] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            out[t, h] = S.T @ q[t, g]
    return out


@pytest.mark.parametrize("H,G,d,dv", [(2, 1, 16, 8), (3, 3, 40, 72), (2, 2, 128, 128), (4, 2, 64, 256),
                                      (1, 1, 256, 64)])
def test_delta_recurrence_kernel(H, G, d, dv):
    from zig_ai_amd.kernels import ops
    dev = torch.device("cuda")
    gen = torch.Generator().manual_seed(d + dv)
    lengths = [37, 1, 18]
    T = sum(lengths)
    conv = torch.randn(T, 2 * G * d + H * dv + 3, generator=gen)
    proj = torch.randn(T, H + 5, generator=gen)
    decay_raw = torch.randn(T, H * d + 9, generator=gen)
    dt_bias = torch.randn(H * d, generator=gen)
    A_log = torch.rand(H, generator=gen) * 4 - 4
    mem, state = _slots(5, 11 + H * d * dv, dev)
    slots = [3, 0, 4]
    seq, start, slot_id = _step_arrays(lengths, slots, dev)
    # in two steps: the first tokens of every request, then the rest, through the state
    cut = [20, 0, 7]
    rows_a = [r for i, n in enumerate(lengths) for r in range(int(start[i]), int(start[i]) + cut[i])]
    rows_b = [r for i, n in enumerate(lengths) for r in range(int(start[i]) + cut[i], int(start[i + 1]))]
    got = torch.zeros((T, H * dv), dtype=torch.float64)
    for rows, lens, used in ((rows_a, [c for c in cut if c], [s for s, c in zip(slots, cut) if c]),
                             (rows_b, [n - c for n, c in zip(lengths, cut)], slots)):
        idx = torch.tensor(rows)
        _, st, sl = _step_arrays(lens, used, dev)
        out = ops.matrix_recurrence("delta", conv[idx].to(dev).contiguous(), 3, 3 + G * d,
                                    3 + 2 * G * d, proj[idx].to(dev).contiguous(), 5,
                                    decay_raw[idx].to(dev).contiguous(), dt_bias.to(dev),
                                    A_log.to(dev), None, state, 11, st, sl, H, G, d, dv)
        got[idx] = out.cpu().double()
    c = conv.double()
    for i in range(len(lengths)):
        a, b = int(start[i]), int(start[i + 1])
        q = c[a:b, 3:3 + G * d].view(-1, G, d)
        k = c[a:b, 3 + G * d:3 + 2 * G * d].view(-1, G, d)
        v = c[a:b, 3 + 2 * G * d:].view(-1, H, dv)
        q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
        k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
        beta = torch.sigmoid(proj[a:b, 5:5 + H].double())
        decay = torch.exp(-torch.exp(A_log.double())[None, :, None] * plain.softplus(
            (decay_raw[a:b, :H * d].double() + dt_bias.double()).view(-1, H, d)))
        want = _plain_delta(q, k, v, beta, decay).reshape(b - a, H * dv)
        assert float((got[a:b] - want).abs().max()) < 2e-5 * max(1.0, float(want.abs().max()))
    assert float(mem[:, 11 + H * d * dv:].abs().max()) == 0.0
    assert float(state[:, :11].abs().max()) == 0.0


@pytest.mark.parametrize("H,G,N,P", [(4, 2, 24, 16), (3, 1, 128, 64), (2, 2, 16, 40)])
def test_ssd_recurrence_kernel(H, G, N, P):
    from zig_ai_amd.kernels import ops
    dev = torch.device("cuda")
    gen = torch.Generator().manual_seed(N + P)
    lengths = [29, 2, 1]
    T = sum(lengths)
    conv = torch.randn(T, H * P + 2 * G * N, generator=gen)
    proj = torch.randn(T, 4 + H, generator=gen).to(torch.bfloat16)
    dt_bias, D = torch.randn(H, generator=gen), torch.randn(H, generator=gen)
    A_log = torch.rand(H, generator=gen) * 3 - 3
    mem, state = _slots(4, H * N * P, dev)
    seq, start, slot_id = _step_arrays(lengths, [2, 3, 0], dev)
    out = ops.matrix_recurrence("ssd", conv.to(dev), H * P + G * N, H * P, 0, proj.to(dev), 4, None,
                                dt_bias.to(dev), A_log.to(dev), D.to(dev), state, 0, start, slot_id,
                                H, G, N, P).cpu().double()
    c = conv.double()
    for i in range(len(lengths)):
        a, b = int(start[i]), int(start[i + 1])
        x = c[a:b, :H * P].view(-1, H, P)
        B = c[a:b, H * P:H * P + G * N].view(-1, G, N)
        C = c[a:b, H * P + G * N:].view(-1, G, N)
        dt = plain.softplus(proj[a:b, 4:].double() + dt_bias.double())
        for h in range(H):
            S = torch.zeros((N, P), dtype=torch.float64)
            for t in range(b - a):
                S = torch.exp(-torch.exp(A_log[h].double()) * dt[t, h]) * S \
                    + dt[t, h] * torch.outer(B[t, h // (H // G)], x[t, h])
                want = S.T @ C[t, h // (H // G)] + D[h].double() * x[t, h]
                assert float((out[a + t, h * P:(h + 1) * P] - want).abs().max()) < 2e-5 * max(
                    1.0, float(want.abs().max()))
    assert float(state[1].abs().max()) == 0.0


def test_small_kernels():
    from zig_ai_amd.kernels import ops
    dev = torch.device("cuda")
    gen = torch.Generator().manual_seed(0)
    T = 9
    for I in (52, 56):          # element by element, and eight at a time
        gu = (torch.randn(T, 2 * I, generator=gen) * 3).to(torch.bfloat16)
        got = ops.clamped_glu(gu.to(dev), 2.0, 1.702, 1.0).cpu().double()
        g = gu[:, :I].double().clamp(max=2.0)
        u = gu[:, I:].double().clamp(-2.0, 2.0)
        want = g * torch.sigmoid(1.702 * g) * (u + 1.0)
        assert float((got - want).abs().max()) < 0.04
        got = ops.clamped_glu(gu.float().to(dev), 2.0, 1.702, 1.0).cpu().double()
        assert float((got - want).abs().max()) < 1e-5
    # gated group norm, both orders
    y = torch.randn(T, 96, generator=gen)
    gate = torch.randn(T, 96 + 8, generator=gen)
    w = torch.randn(96, generator=gen)
    got = ops.gated_group_norm(y.to(dev), gate.to(dev), 8, w.to(dev), 32, 1e-5, "silu", True).cpu()
    v = (y.double() * plain.silu(gate[:, 8:].double())).view(T, 3, 32)
    want = (plain.rms(v, 1e-5).reshape(T, 96) * w.double())
    assert float((got.double() - want).abs().max()) < 1e-5
    got = ops.gated_group_norm(y.to(dev), gate.to(dev), 8, w[:24].contiguous().to(dev), 24, 1e-5,
                               "sigmoid", False).cpu()
    want = (plain.rms(y.double().view(T, 4, 24), 1e-5) * w[:24].double()).reshape(T, 96) \
        * torch.sigmoid(gate[:, 8:].double())
    assert float((got.double() - want).abs().max()) < 1e-5
    # weighted additions to the stream, with and without the norm
    x = torch.randn(T, 80, generator=gen)
    a, b = torch.randn(T, 80, generator=gen), torch.randn(T, 80, generator=gen)
    nw = torch.randn(80, generator=gen)
    res = x.to(dev).clone()
    out = ops.scaled_add_rmsnorm(res, a.to(dev), 0.3, b.to(dev), -1.1, nw.to(dev), 1e-6).cpu()
    s = x.double() + 0.3 * a.double() - 1.1 * b.double()
    assert float((res.cpu().double() - s).abs().max()) < 1e-5
    assert float((out.double() - plain.rms(s, 1e-6) * nw.double()).abs().max()) < 1e-5
    assert ops.scaled_add_rmsnorm(res, a.to(torch.bfloat16).to(dev), 2.0) is None
    s = s + 2.0 * a.to(torch.bfloat16).double()
    assert float((res.cpu().double() - s).abs().max()) < 1e-5
