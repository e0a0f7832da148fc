"""Ranesun through the engine against the plain implementation (``plain_ranesun.py``,
float64, whole sequences, one function per mechanism).

float32 runs are held to the plain logits row by row (root mean square of the difference
over the vocabulary, relative to the logits' own spread): measured 1e-6 to 1e-5, bound
1e-4; every schedule, cut and batch is held to it.  bfloat16 rows are held to the plain
logits by their median, their ninth decile and, loosely, their worst row (the weights here
are drawn sharp on purpose), and every schedule to the whole prompts' run: how a request
was cut and batched must not show beyond rounding."""

import pytest
import torch

import engine_util as eu
import plain_ranesun as plain
import ranesun_util as ru

pytestmark = pytest.mark.gpu

F32_BOUND = 1e-4
BF16_MEDIAN, BF16_DECILE, BF16_WORST = 0.04, 0.1, 0.5
BF16_BETWEEN_MEDIAN, BF16_BETWEEN_WORST = 0.02, 0.2


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
    "retention": ru.one_layer("retention", ru.retention()),
    "retention, whole rotation, wide": ru.one_layer(
        "retention", ru.retention(heads=2, dim=40, vdim=72, rot_dims=40, base=1e6)),
    "retention, no rotation, no decay": ru.one_layer(
        "retention", ru.retention(heads=2, dim=16, vdim=16, decay=[1.0, 0.25], rot_dims=0)),
    "attention": ru.one_layer("attention", ru.attention()),
    "attention, one kv head, temperature every token": ru.one_layer(
        "attention", ru.attention(heads=8, kv_heads=1, dim=32, scale=0.4, softcap=3.0, coef=0.5,
                                  every=1)),
    "attention, no cap, no temperature": ru.one_layer(
        "attention", ru.attention(heads=2, kv_heads=2, dim=24, softcap=0.0, every=0)),
    "dense": ru.one_layer("retention", ru.retention(), ru.dense()),
    "experts": ru.one_layer("retention", ru.retention(), ru.moe()),
    "experts, one of one": ru.one_layer("attention", ru.attention(), ru.moe(ff=40, experts=1, top=1)),
    "experts, all of four": ru.one_layer("attention", ru.attention(), ru.moe(ff=8, experts=4, top=4)),
    "loop of one layer, three times": ru.one_layer("retention", ru.retention(), ru.dense(16),
                                                   loop=(0, 1, 3)),
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


def test_streams_after_every_layer_run():
    cfg = ru.TINY_ALL
    model, tensors = build(cfg, seed=4)
    prompt = ru.tokens(21, cfg["vocab"], 3)
    streams = []
    plain.forward(cfg, tensors, prompt, streams)
    from zig_ai_amd.engine import StepEntry
    runner = runner_for(model)
    runner.admit("a")
    taps = []
    runner.step([StepEntry("a", prompt, [])], taps=taps)
    assert len(taps) == len(streams) + 1 == 12       # the embedding, then eleven layer runs
    for i, s in enumerate(streams):
        got = taps[i + 1]["stream"].double().cpu()
        assert float((got - s).abs().max()) < 1e-4 * float(s.abs().max()), i


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


@pytest.mark.parametrize("which", ["all", "other", "loop twice"])
@pytest.mark.parametrize("page_size", [4, 16])
def test_schedules_float32(which, page_size):
    cfg = {"all": ru.TINY_ALL, "other": ru.TINY_OTHER, "loop twice": ru.TINY_LOOP_TWICE}[which]
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
@pytest.mark.parametrize("seed", range(10))
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
        for i, (g, w) in enumerate(zip(got, want)):
            assert worst(g, w) < 3 * F32_BOUND, (name, i, cfg)
    # the same model in bfloat16 runs and agrees with itself across schedules
    model16, _ = build(cfg, seed=seed, dtype="bfloat16")
    base = None
    for schedule in (eu.whole(lengths), eu.mixed(lengths, seed=seed, max_live=3, decode_tail=9)):
        got = eu.run_schedule(runner_for(model16, page_size=16, tokens=256, slots=3), prompts, schedule)
        assert all(torch.isfinite(g).all() for g in got)
        base = base or got
        e = ru.row_error(torch.cat(got), torch.cat(base))
        assert float(e.median()) < BF16_BETWEEN_MEDIAN, float(e.median())


# ------------------------------ one far key among hundreds, with a score that stands out
def far_key_model(dtype, dim):
    """An attention layer whose scores are all but flat, but for ONE key far back: its key
    vector and the last query are made long along one direction, so that the last token's
    output is that key's value if and only if the key is found."""
    cfg = ru.one_layer("attention", ru.attention(heads=2, kv_heads=1, dim=dim, scale=1.0,
                                                 softcap=50.0, coef=0.2, every=48),
                       width=64, vocab=300)
    t = ru.make_tensors(cfg, seed=7)
    t["l0.mix.q"] *= 0.05
    t["l0.mix.k"] *= 0.05
    t["l0.norm1"] = torch.ones_like(t["l0.norm1"])
    t["l0.norm1.b"] = torch.zeros_like(t["l0.norm1.b"])
    t["l0.mix.sink"] = torch.tensor([-3.0, 0.5])
    # token 299 is the one to find and token 298 the one that asks: the key's first element
    # reads the stream's first channel, where 299 is long, the queries' first elements read
    # the second channel, where 298 is long (298's own key is short)
    t["embed"][299] = 0.0
    t["embed"][299, 0] = 8.0
    t["embed"][298] = 0.0
    t["embed"][298, 1] = 8.0
    t["l0.mix.k"][0, :] = 0.0
    t["l0.mix.k"][0, 0] = 1.0
    for h in range(2):
        t["l0.mix.q"][h * dim, :] = 0.0
        t["l0.mix.q"][h * dim, 1] = 1.0
    t["l0.mix.o"] *= 4.0
    # (what the folder will hold: values that bfloat16 has)
    return cfg, {k: v if v.dtype == torch.int32 else v.to(torch.bfloat16).float() for k, v in t.items()}


@pytest.mark.parametrize("dtype,dim", [("float32", 16), ("bfloat16", 64), ("bfloat16", 128),
                                       ("bfloat16", 32)])
def test_a_far_key_is_found(dtype, dim):
    cfg, tensors = far_key_model(dtype, dim)
    model, _ = build(cfg, tensors=tensors, dtype=dtype)
    n = 700
    for place in (0, 1, 15, 16, 63, 64, 333):           # first tokens, page and tile borders
        prompt = [t % 298 for t in ru.tokens(n, 298, place)]
        prompt[place] = 299
        prompt[-1] = 298
        other = list(prompt)
        other[place] = 5                                 # the same prompt without the key
        want = plain.forward(cfg, tensors, prompt).float()
        assert worst(plain.forward(cfg, tensors, other).float()[-1:], want[-1:]) > 0.05
        for schedule in (eu.whole([n]), eu.bulk_then_single([n], tail=3),
                         eu.changing_portions([n], sizes=(64, 2, 130, 17, 256))):
            got = eu.run_schedule(runner_for(model, page_size=16, tokens=1024), [prompt], schedule)[0]
            if dtype == "float32":
                assert worst(got, want) < F32_BOUND, place
            else:
                assert worst(got[-1:], want[-1:]) < 0.02, place


# --------------------------------------------------------------- the sink's share
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_sink_counts_once_however_the_context_is_cut(dtype):
    # sinks about as large as the logarithm of the keys' summed weights, so that they take
    # about half of every head's weight: left out, counted per range of a cut context, or
    # scaled, they would move every output by tens of percent
    cfg = ru.one_layer("attention", ru.attention(heads=4, kv_heads=1, dim=64, scale=0.11,
                                                 softcap=25.0, coef=0.4, every=48),
                       width=64, vocab=97)
    tensors = ru.make_tensors(cfg, seed=5)
    n = 1300
    prompt = ru.tokens(n, cfg["vocab"], 1)
    tensors["l0.mix.o"] *= 16.0
    tensors["l0.mix.sink"] = torch.tensor([14.0, 15.0, 13.0, 16.0])
    want = plain.forward(cfg, tensors, prompt).float()
    without = dict(tensors)
    without["l0.mix.sink"] = torch.full((4,), -60.0)
    assert worst(plain.forward(cfg, without, prompt).float()[-40:], want[-40:]) > 0.05
    model, _ = build(cfg, tensors=tensors, dtype=dtype)
    bound = F32_BOUND if dtype == "float32" else 0.03
    # one request decoding at 1,300 keys: its context is cut into ranges that are merged
    for schedule in (eu.whole([n]), eu.bulk_then_single([n], tail=40),
                     eu.changing_portions([n], sizes=(600, 2, 500, 64, 100, 3))):
        got = eu.run_schedule(runner_for(model, page_size=16, tokens=2048), [prompt], schedule)[0]
        assert worst(got[-40:], want[-40:]) < bound
        assert worst(got[:8], want[:8]) < bound                    # the first tokens


def test_the_query_temperature_changes_where_it_should():
    # a coefficient so large that a position on the wrong side of a step of the temperature
    # has scores that differ by a factor
    cfg = ru.one_layer("attention", ru.attention(heads=2, kv_heads=2, dim=16, scale=0.7,
                                                 softcap=0.0, coef=3.0, every=16))
    model, tensors = build(cfg, seed=6)
    n = 70
    prompt = ru.tokens(n, cfg["vocab"], 2)
    want = plain.forward(cfg, tensors, prompt).float()
    off = ru.one_layer("attention", ru.attention(heads=2, kv_heads=2, dim=16, scale=0.7,
                                                 softcap=0.0, coef=3.0, every=17))
    assert worst(plain.forward(off, tensors, prompt).float(), want) > 0.05
    for schedule in (eu.whole([n]), eu.bulk_then_single([n], tail=60),
                     eu.changing_portions([n], sizes=(15, 2, 16, 1, 17))):
        got = eu.run_schedule(runner_for(model), [prompt], schedule)[0]
        assert worst(got, want) < F32_BOUND


# ----------------------------------------------------------------- far tokens count
def test_far_tokens_reach_the_end_through_the_state():
    cfg = ru.one_layer("retention", ru.retention(heads=2, dim=16, vdim=16,
                                                 decay=[0.99951171875, 1.0], rot_dims=8))
    model, tensors = build(cfg, seed=9)
    n = 600
    a = ru.tokens(n, cfg["vocab"], 3)
    b = list(a)
    b[1] = (b[1] + 1) % cfg["vocab"]
    wa, wb = plain.forward(cfg, tensors, a).float(), plain.forward(cfg, tensors, b).float()
    assert worst(wb[-8:], wa[-8:]) > 1e-2          # the second token still shows at the end
    for prompt, want in ((a, wa), (b, wb)):
        for schedule in (eu.whole([n]), eu.bulk_then_single([n], tail=64),
                         eu.changing_portions([n], sizes=(33, 2, 64, 17, 300))):
            got = eu.run_schedule(runner_for(model, tokens=1024), [prompt], schedule)[0]
            assert worst(got, want) < F32_BOUND
    # nothing is left of a request whose slot is taken again: b after a in a pool of one slot
    runner = runner_for(model, tokens=1024, slots=1)
    for prompt, want in ((a, wa), (b, wb), (a, wa)):
        got = eu.run_schedule(runner, [prompt], eu.bulk_then_single([n], tail=5))[0]
        assert worst(got, want) < F32_BOUND


# ------------------------------------------------------------------- long decoding
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(dtype):
    cfg = ru.TINY_ALL
    model, tensors = build(cfg, seed=21, dtype=dtype)
    n = 330
    prompts = [ru.tokens(n, cfg["vocab"], 5)]
    want = plain_logits(cfg, tensors, prompts)[0]
    runner = runner_for(model, page_size=16, tokens=512)       # decode steps replay from graphs
    assert runner.graphs is not None
    got = eu.run_schedule(runner, prompts, eu.bulk_then_single([n], tail=300))[0]
    if dtype == "float32":
        assert worst(got, want) < F32_BOUND
    else:
        assert_bfloat16_close(got, want)
    # the same steps issued kernel by kernel
    again = eu.run_schedule(runner_for(model, page_size=16, tokens=512, graphs=False), prompts,
                            eu.bulk_then_single([n], tail=300))[0]
    assert worst(again, got) < (1e-5 if dtype == "float32" else BF16_BETWEEN_WORST)


# ------------------------------------------- unequal requests together and alone
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_batch_against_each_alone(dtype):
    cfg = ru.TINY_ALL
    model, tensors = build(cfg, seed=2, dtype=dtype)
    lengths = [64, 3, 41, 17]
    prompts = [ru.tokens(n, cfg["vocab"], 40 + i) for i, n in enumerate(lengths)]
    alone = eu.run_schedule(runner_for(model, tokens=256), prompts, eu.whole(lengths))
    together = [([(i, 0, n) for i, n in enumerate(lengths)], list(range(len(lengths))))]
    got = eu.run_schedule(runner_for(model, tokens=256), prompts, together)
    if dtype == "float32":
        assert worst(torch.cat(got), torch.cat(alone)) < 1e-5
    else:
        e = ru.row_error(torch.cat(got), torch.cat(alone))
        assert float(e.median()) < BF16_BETWEEN_MEDIAN and float(e.max()) < BF16_BETWEEN_WORST


# ------------------- sizes that the matrix-core kernels take, at widths of real layers
@pytest.mark.parametrize("dim,heads,kv", [(64, 8, 2), (128, 4, 1), (64, 16, 4)])
def test_matrix_core_paths(dim, heads, kv):
    cfg = ru.config([
        ru.layer("attention", ru.attention(heads=heads, kv_heads=kv, dim=dim, scale=dim ** -0.5,
                                           softcap=20.0, coef=0.3, every=50),
                 ru.moe(ff=64, experts=6, top=2)),
        ru.layer("retention", ru.retention(heads=3, dim=64, vdim=32, rot_dims=16), ru.dense(256)),
    ], width=256, vocab=211, loop=(0, 2, 2))
    model, tensors = build(cfg, seed=6, dtype="bfloat16")
    assert model.blocks[0].parts["mixer"].mfma
    lengths = [300, 70, 3]
    prompts = [ru.tokens(n, cfg["vocab"], 50 + i) for i, n in enumerate(lengths)]
    want = plain_logits(cfg, tensors, prompts)
    base = None
    for name, schedule in (("whole", eu.whole(lengths)),
                           ("bulk + tail", eu.bulk_then_single(lengths, tail=60)),
                           ("portions", eu.changing_portions(lengths, seed=3)),
                           ("mixed", eu.mixed(lengths, seed=1, max_live=3, decode_tail=30))):
        runner = runner_for(model, page_size=16, tokens=768, slots=3)
        got = eu.run_schedule(runner, prompts, schedule)
        assert_bfloat16_close(torch.cat(got), torch.cat(want), name)
        base = base or got
        e = ru.row_error(torch.cat(got), torch.cat(base))
        assert float(e.median()) < BF16_BETWEEN_MEDIAN and float(e.max()) < BF16_BETWEEN_WORST, \
            (name, float(e.median()), float(e.max()))


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


def test_trace_replay_and_command_line(tmp_path):
    import json
    import os
    import subprocess
    import sys
    cfg = ru.TINY_LOOP_TWICE
    d, tensors = ru.folder(cfg, seed=12)
    prompt = ru.tokens(40, cfg["vocab"], 9)
    want = plain.forward(cfg, tensors, prompt).float()
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": prompt[:25], "want": [3, 24]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": prompt[25:27], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": prompt[27:], "want": [12]}], "end": ["a"]}]
    out = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", d,
                          "--dtype", "float32", "--out", str(tmp_path), "--max-tokens", "64"],
                         input="\n".join(json.dumps(s) for s in steps) + "\n", text=True,
                         capture_output=True, timeout=600)
    assert out.returncode == 0, out.stderr[-2000:]
    assert [l for l in out.stdout.split("\n") if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    import numpy as np
    first = torch.from_numpy(np.fromfile(tmp_path / "0.f32", dtype="<f4").reshape(2, -1))
    last = torch.from_numpy(np.fromfile(tmp_path / "2.f32", dtype="<f4").reshape(1, -1))
    assert not (tmp_path / "1.f32").exists()
    assert worst(torch.cat([first, last]), want[[3, 24, 39]]) < F32_BOUND
    gen = subprocess.run([sys.executable, "-m", "zig_ai_amd", "--model", d, "--dtype", "float32",
                          "--prompt-ids", ",".join(map(str, prompt[:9])), "-n", "5",
                          "--temperature", "0", "--json"], cwd=root, text=True, capture_output=True,
                         timeout=600)
    assert gen.returncode == 0, gen.stderr[-2000:]
    outputs = json.loads(gen.stdout.strip().split("\n")[-1])["outputs"]
    assert len(outputs) == 1 and len(outputs[0]) == 5
    logits = plain.forward(cfg, tensors, prompt[:9] + outputs[0])
    for j, tok in enumerate(outputs[0]):
        row = logits[9 + j - 1]
        assert float(row.max() - row[tok]) <= 1e-3 * float(row.abs().max()), (j, tok)


# ------------------------------------------------------------------ kernels alone
def _slots(n_slots, floats, device):
    # rows spaced wider than their length, as the cache manager's slot rows are
    mem = torch.zeros((n_slots, floats + 12), dtype=torch.float32, device=device)
    return mem, mem[:, :floats]


def _step_arrays(lengths, slots, device):
    start = [0]
    for n in lengths:
        start.append(start[-1] + n)
    mk = lambda v: torch.tensor(v, dtype=torch.int32, device=device)
    return mk(start), mk(slots)


@pytest.mark.parametrize("width,dtype", [(48, torch.float32), (1024, torch.bfloat16), (70, torch.bfloat16),
                                         (5000, torch.float32)])
def test_layer_norm_kernel(width, dtype):
    from zig_ai_amd.kernels import ops
    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(width)
    x = torch.randn(9, width, generator=g) * 3 + 1.5
    stack = torch.randn(3, 9, width, generator=g)
    w, b = torch.randn(width, generator=g), torch.randn(width, generator=g)
    res = x.to(dev)
    out = ops.add_layernorm(res, stack.to(dev), w.to(dev), b.to(dev), 1e-5, dtype)
    total = x.double() + stack.double().sum(0)
    want = plain.layer_norm(total, w.double(), b.double(), 1e-5)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert float((out.double().cpu() - want).abs().max()) < tol * float(want.abs().max())
    assert float((res.double().cpu() - total).abs().max()) < 1e-5      # the sum was stored
    rows = torch.tensor([7, 2], dtype=torch.int32, device=dev)
    some = ops.add_layernorm(res, None, w.to(dev), None, 1e-5, torch.float32, rows=rows)
    want = plain.layer_norm(total[[7, 2]], w.double(), torch.zeros(width, dtype=torch.float64), 1e-5)
    assert float((some.double().cpu() - want).abs().max()) < 1e-5 * float(want.abs().max())
    # between two passes: the stream takes what is pending, the origin and one row of a table
    res2 = x.to(dev)
    ops.stream_add_(res2, stack.to(dev), x.to(dev), w.to(dev))
    assert float((res2.double().cpu() - (2 * x.double() + stack.double().sum(0) + w.double())).abs().max()) < 1e-5


@pytest.mark.parametrize("H,d,dv,rot", [(2, 16, 8, 8), (3, 40, 72, 40), (2, 128, 128, 64),
                                        (1, 256, 64, 0), (6, 32, 64, 32)])
def test_retention_kernels(H, d, dv, rot):
    from zig_ai_amd.kernels import ops
    dev = torch.device("cuda")
    gen = torch.Generator().manual_seed(d + dv)
    lengths, positions0 = [37, 1, 18], [5, 0, 130]
    T = sum(lengths)
    stride = 2 * H * d + 2 * H * dv + 3
    proj = torch.randn(T, stride, generator=gen)
    decay = torch.rand(H, generator=gen) * 0.2 + 0.8
    inv_freq = (100.0 ** (-torch.arange(rot // 2, dtype=torch.float64) * 2 / rot)).float() if rot else None
    pos = torch.tensor([p0 + j for p0, n in zip(positions0, lengths) for j in range(n)], dtype=torch.int32)
    mem, state = _slots(5, 11 + H * d * dv, dev)
    slots = [3, 0, 4]
    start, slot_id = _step_arrays(lengths, slots, dev)
    # in two steps: the first tokens of every request, then the rest, through the state
    cut = [20, 0, 7]
    rows_a = [r for i in range(3) for r in range(int(start[i]), int(start[i]) + cut[i])]
    rows_b = [r for i in range(3) for r in range(int(start[i]) + cut[i], int(start[i + 1]))]
    got = torch.zeros((T, H * dv), dtype=torch.float64)
    for rows, lens, used in ((rows_a, [c for c in cut if c], [s for s, c in zip(slots, cut) if c]),
                             (rows_b, [n - c for n, c in zip(lengths, cut)], slots)):
        idx = torch.tensor(rows)
        st, sl = _step_arrays(lens, used, dev)
        vec = ops.retention_prepare(proj[idx].to(dev).contiguous(), 3, 3 + H * d, 3 + 2 * H * d,
                                    pos[idx].to(dev), inv_freq.to(dev) if rot else None, H, d, dv,
                                    rot, d ** -0.5)
        out = ops.matrix_recurrence("fixed", vec, 0, H * d, 2 * H * d, None, 0, decay.to(dev), None,
                                    None, None, state, 11, st, sl, H, H, d, dv)
        got[idx] = out.double().cpu()
    p64 = proj.double()
    r0 = 0
    for n, p0 in zip(lengths, positions0):
        q = p64[r0:r0 + n, 3:3 + H * d].view(n, H, d)
        k = p64[r0:r0 + n, 3 + H * d:3 + 2 * H * d].view(n, H, d)
        v = p64[r0:r0 + n, 3 + 2 * H * d:3 + 2 * H * d + H * dv].view(n, H, dv)
        if rot:
            q = plain.rotate_half(q, torch.arange(p0, p0 + n), rot, 100.0)
            k = plain.rotate_half(k, torch.arange(p0, p0 + n), rot, 100.0)
        k = k * d ** -0.5
        S = torch.zeros(H, d, dv, dtype=torch.float64)
        for t in range(n):
            S = decay.double()[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
            want = torch.einsum("hdv,hd->hv", S, q[t]).reshape(-1)
            assert float((got[r0 + t] - want).abs().max()) < 2e-4 * max(1.0, float(want.abs().max()))
        r0 += n
    assert float(mem[:, 11 + H * d * dv:].abs().max()) == 0.0     # nothing beyond the window
    assert float(mem[:, :11].abs().max()) == 0.0                   # nor before it
    assert float(state[1].abs().max()) == 0.0                      # a slot nobody uses


@pytest.mark.parametrize("T,E,top,K,N,dtype", [(70, 5, 2, 48, 24, torch.float32),
                                                (300, 8, 2, 320, 96, torch.bfloat16),
                                                (3, 8, 2, 320, 96, torch.bfloat16),
                                                (130, 3, 3, 40, 72, torch.bfloat16),
                                                (9, 1, 1, 24, 8, torch.float32),
                                                (600, 64, 4, 64, 40, torch.bfloat16),
                                                (1200, 4, 2, 72, 136, torch.bfloat16),
                                                (700, 2, 1, 256, 200, torch.bfloat16)])
def test_expert_kernels(T, E, top, K, N, dtype):
    from zig_ai_amd.kernels import ops
    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(T + E)
    vocab = 50
    table = torch.rand(vocab, E, generator=g).argsort(dim=1)[:, :top].to(torch.int32)
    ids = torch.randint(0, vocab, (T,), generator=g, dtype=torch.int32)
    lists, counts = ops.expert_lists(ids.to(dev), table.to(dev), T, E)
    picks = table[ids.long()]                                     # [T, top]
    for e in range(E):
        want = [t * top + j for t in range(T) for j in range(top) if int(picks[t, j]) == e]
        assert int(counts[e]) == len(want)
        assert lists[e, :len(want)].tolist() == want
    x = (torch.randn(T, K, generator=g)).to(dtype)
    w_up = (torch.randn(E, N, K, generator=g) * K ** -0.5).to(dtype)
    w_down = (torch.randn(E, K, N, generator=g) * N ** -0.5).to(dtype)
    a = ops.grouped_linear(x.to(dev), w_up.to(dev), lists, counts, T, per_token=True,
                           activation="relu2")
    want_a = torch.stack([torch.relu(x[t].double() @ w_up[int(picks[t, j])].double().T) ** 2
                          for t in range(T) for j in range(top)])
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert float((a.double().cpu() - want_a).abs().max()) < tol * float(want_a.abs().max())
    y = ops.grouped_linear(a, w_down.to(dev), lists, counts, T, per_token=False, stacked=True,
                           out_scale=1.0 / top)
    assert tuple(y.shape) == (top, T, K) and y.dtype == torch.float32
    a64 = a.double().cpu().view(T, top, N)
    want_y = torch.stack([torch.stack([a64[t, j] @ w_down[int(picks[t, j])].double().T / top
                                       for t in range(T)]) for j in range(top)])
    assert float((y.double().cpu() - want_y).abs().max()) < tol * float(want_y.abs().max())
    # a token's result does not depend on who shares its expert: the first three tokens alone
    l3, c3 = ops.expert_lists(ids[:3].to(dev).contiguous(), table.to(dev), 3, E)
    a3 = ops.grouped_linear(x[:3].to(dev).contiguous(), w_up.to(dev), l3, c3, 3, per_token=True,
                            activation="relu2")
    assert torch.equal(a3, a[:3 * top])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gated_unit_and_scale_kernels(dtype):
    from zig_ai_amd.kernels import ops
    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(1)
    for inter in (24, 7):
        gu = (torch.randn(11, 2 * inter, generator=g) * 3).to(dtype)
        out = ops.gated_unit(gu.to(dev), "gelu_tanh").double().cpu()
        want = plain.gelu_tanh(gu[:, :inter].double()) * gu[:, inter:].double()
        tol = 1e-6 if dtype == torch.float32 else 5e-3       # of the largest value
        assert float((out - want).abs().max()) < tol * float(want.abs().max())
        out = ops.gated_unit(gu.to(dev), "silu").double().cpu()
        want = plain.silu(gu[:, :inter].double()) * gu[:, inter:].double()
        assert float((out - want).abs().max()) < tol * float(want.abs().max())
    x = torch.randn(5, 9, generator=g)
    assert torch.allclose(ops.scale_(x.to(dev), 2.5).cpu(), x * 2.5)


@pytest.mark.parametrize("M,K,I", [(1, 320, 256), (8, 2048, 1024), (16, 512, 136)])
def test_gate_in_the_product_of_a_decode_batch(M, K, I):
    """The gate|up product that applies the gate to its own sums, with the tanh form of gelu,
    against the plain formula on the 32-bit products."""
    from zig_ai_amd.kernels import ops
    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(M + K)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(2 * I, K, generator=g) * 2.0 * K ** -0.5).to(torch.bfloat16)
    for act, fn in (("gelu_tanh", plain.gelu_tanh), ("silu", plain.silu)):
        got = ops.linear_swiglu(x.to(dev), w.to(dev), act).double().cpu()
        gu = x.double() @ w.double().T
        want = fn(gu[:, :I]) * gu[:, I:]
        assert float((got - want).abs().max()) < 1e-2 * float(want.abs().max()), act


@pytest.mark.parametrize("H,d,dv", [(2, 16, 8), (3, 64, 128), (1, 128, 40)])
def test_retention_in_chunks_against_the_plain_walk(H, d, dv):
    """Long portions walked as chunks side by side: against float64, in two steps so that the
    second starts from carried states, with portions of exactly one chunk, one more and one
    fewer, and a decay of one and of a half."""
    from zig_ai_amd.kernels import ops
    dev = torch.device("cuda")
    gen = torch.Generator().manual_seed(d + dv)
    C = ops.RETENTION_CHUNK
    steps = [[2 * C + 70, 1, C, C + 1], [C - 1, 3 * C, 5, 1]]
    decay = torch.tensor(([1.0, 0.5, 0.99609375] * H)[:H])
    mem, state = _slots(6, 7 + H * d * dv, dev)
    slots = [4, 0, 5, 2]
    S64 = [torch.zeros(H, d, dv, dtype=torch.float64) for _ in slots]
    for lengths in steps:
        T = sum(lengths)
        vec = torch.randn(T, 2 * H * d + H * dv, generator=gen)
        vec[:, H * d:2 * H * d] *= d ** -0.5
        start, slot_id = _step_arrays(lengths, slots, dev)
        seq, row0, cnt = [], [], []
        r = 0
        for i, n in enumerate(lengths):
            for a in range(0, n, C):
                seq.append(i); row0.append(r + a); cnt.append(min(C, n - a))
            r += n
        mk = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)
        items = (mk(seq), mk(row0), mk(cnt), len(seq))
        got = ops.fixed_decay_recurrence_chunked(vec.to(dev), 0, H * d, 2 * H * d, decay.to(dev),
                                                 state, 7, slot_id, items, H, d, dv).double().cpu()
        v64 = vec.double()
        r = 0
        for i, n in enumerate(lengths):
            q = v64[r:r + n, :H * d].view(n, H, d)
            k = v64[r:r + n, H * d:2 * H * d].view(n, H, d)
            v = v64[r:r + n, 2 * H * d:].view(n, H, dv)
            for t in range(n):
                S64[i] = decay.double()[:, None, None] * S64[i] + k[t][:, :, None] * v[t][:, None, :]
                want = torch.einsum("hdv,hd->hv", S64[i], q[t]).reshape(-1)
                assert float((got[r + t] - want).abs().max()) < 3e-4 * max(1.0, float(want.abs().max())), (i, t)
            r += n
        for i, slot in enumerate(slots):
            kept = state[slot, 7:].double().cpu().view(H, dv, d).transpose(1, 2)
            assert float((kept - S64[i]).abs().max()) < 3e-4 * max(1.0, float(S64[i].abs().max()))
    assert float(mem[:, :7].abs().max()) == 0.0 and float(mem[:, 7 + H * d * dv:].abs().max()) == 0.0
