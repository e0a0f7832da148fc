"""Ranesun's configuration and description as parts (no GPU), and what pins the plain
implementation's mechanisms: identities that a consistent mistake would break."""

import math

import pytest
import torch

import plain_ranesun as plain
import ranesun_util as ru
from zig_ai_amd.config import ConfigError, config_from_dict, known_architectures
from zig_ai_amd.weights.loader import expected_tensors


def test_registered_and_round_trip():
    assert "Ranesun" in known_architectures()
    for cfg in (ru.TINY_ALL, ru.TINY_OTHER, ru.TINY_LOOP_ONCE, ru.TINY_LOOP_TWICE):
        typed = config_from_dict(cfg)
        assert config_from_dict(typed.to_dict()) == typed
        assert typed.hidden_size == cfg["width"] and typed.vocab_size == cfg["vocab"]


def test_every_tensor_is_named_with_its_shape():
    cfg = ru.TINY_ALL
    tensors = ru.make_tensors(cfg)
    spec = config_from_dict(cfg).to_spec()
    expected = {e.names[0]: tuple(e.rule.shapes[0]) for e in expected_tensors(spec)}
    assert set(expected) == set(tensors)
    for name, shape in expected.items():
        assert tuple(tensors[name].shape) == shape, name
    # a layer without a feed-forward may carry its second norm
    assert "l2.norm2" in spec.ignored_tensors and "l2.norm2.b" in spec.ignored_tensors


def test_run_order_of_the_loop():
    spec = config_from_dict(ru.TINY_ALL).to_spec()       # layers 1..3 three times
    order = [(c.layer, None if c.before is None else dict(c.before.args)) for c in spec.schedule]
    assert [l for l, _ in order] == [0, 1, 2, 3, 1, 2, 3, 1, 2, 3, 4]
    assert order[1][1] == {"row": 0, "add_origin": False}
    assert order[4][1] == {"row": 1, "add_origin": True}
    assert order[7][1] == {"row": 2, "add_origin": True}
    assert all(b is None for i, (_, b) in enumerate(order) if i not in (1, 4, 7))
    # every time a layer runs it has a cache entry of its own
    caches = [c.cache for c in spec.resolved_schedule()]
    assert len(set(caches)) == len(caches)
    assert [c.layer for c in config_from_dict(ru.TINY_OTHER).to_spec().schedule] == [0, 1, 2]
    assert config_from_dict(ru.TINY_OTHER).to_spec().stream_parts == ()
    once = config_from_dict(ru.TINY_LOOP_ONCE).to_spec()
    assert [c.layer for c in once.schedule] == [0, 1] and once.schedule[0].before is not None
    assert plain.run_order(ru.TINY_ALL) == [(c.layer,
                                             None if (c.layer < 1 or c.layer > 3) else t,
                                             c.before is not None)
                                            for c, t in zip(spec.schedule,
                                                            [None, 0, 0, 0, 1, 1, 1, 2, 2, 2, None])]


def test_constants_reach_the_parts():
    spec = config_from_dict(ru.TINY_ALL).to_spec()
    att = spec.layers[2].parts["mixer"].params
    assert att["values"] == "keys" and att["sink"] and att["softcap"] == 2.5
    assert att["query_temperature"] == (0.7, 3) and att["softmax_scale"] == 0.8
    assert att["num_heads"] == 6 and att["num_kv_heads"] == 1 and att["position"] is None
    plain_att = spec.layers[4].parts["mixer"].params
    assert plain_att["softcap"] == 0.0 and plain_att["query_temperature"] is None
    ret = spec.layers[3].parts["mixer"].params
    assert ret["decay"] == tuple(ru.TINY_ALL["layers"][3]["mixer"]["decay"])
    assert ret["position"].params["pairing"] == "half" and ret["position"].params["rotary_dim"] == 24
    assert spec.layers[0].parts["feed_forward"].params["activation"] == "gelu_tanh"
    experts = spec.layers[1].parts["feed_forward"]
    assert experts.kind == "table_experts" and experts.params["experts"] == 5 \
        and experts.params["top"] == 2 and experts.params["activation"] == "relu2"
    assert spec.layers[2].arrangement == "pre_norm_residual_no_ff"
    assert spec.lm_head.params["tied"] and spec.lm_head.params["logit_scale"] == 1.5
    assert spec.final_norm.kind == "layer_norm"


@pytest.mark.parametrize("breakage", [
    lambda c: c["layers"][0].update(type="mamba2"),
    lambda c: c["layers"][1]["mixer"].update(decay=[0.5]),
    lambda c: c["layers"][0]["mixer"].update(vdim=8),
    lambda c: c["layers"][0]["mixer"].update(kv_heads=3),
    lambda c: c["layers"][1]["mlp"]["router"].update(top=9),
    lambda c: c["layers"][1]["mixer"]["rot"].update(dims=18),
    lambda c: c.update(loop={"start": 2, "stop": 2, "times": 2}),
    lambda c: c.update(loop={"start": 0, "stop": 9, "times": 1}),
    lambda c: c.pop("norm"),
    lambda c: c.update(layers=[]),
])
def test_malformed_configurations(breakage):
    import copy
    cfg = copy.deepcopy(ru.TINY_ALL)
    breakage(cfg)
    with pytest.raises(ConfigError):
        config_from_dict(cfg)


def test_random_model_folder_has_usable_tables(tmp_path):
    from zig_ai_amd.weights.random_init import write_random_model
    from zig_ai_amd.weights.safetensors_io import Checkpoint
    write_random_model(ru.TINY_ALL, str(tmp_path), seed=3)
    ckpt = Checkpoint(str(tmp_path))
    table = ckpt.tensor("l1.mlp.table")
    assert table.dtype == torch.int32 and tuple(table.shape) == (ru.TINY_ALL["vocab"], 2)
    assert int(table.min()) >= 0 and int(table.max()) < 5
    assert bool((table[:, 0] != table[:, 1]).all())
    assert len({tuple(r) for r in table.tolist()}) > 5          # not one pick for everybody


# ----------------------------------------------- what pins the plain implementation
def test_layer_norm_against_the_library():
    x = torch.randn(5, 24, dtype=torch.float64)
    w, b = torch.randn(24, dtype=torch.float64), torch.randn(24, dtype=torch.float64)
    want = torch.nn.functional.layer_norm(x, (24,), w, b, eps=1e-3)
    assert torch.allclose(plain.layer_norm(x, w, b, 1e-3), want, atol=1e-12)


def test_gelu_tanh_against_the_library():
    z = torch.linspace(-6, 6, 101, dtype=torch.float64)
    assert torch.allclose(plain.gelu_tanh(z), torch.nn.functional.gelu(z, approximate="tanh"),
                          atol=1e-12)


def test_rotation_keeps_lengths_and_depends_on_distance_only():
    g = torch.Generator().manual_seed(0)
    q = torch.randn(1, 2, 16, generator=g, dtype=torch.float64)
    k = torch.randn(1, 2, 16, generator=g, dtype=torch.float64)
    def dot(pq, pk):
        a = plain.rotate_half(q, torch.tensor([pq]), 8, 100.0)
        b = plain.rotate_half(k, torch.tensor([pk]), 8, 100.0)
        return (a * b).sum(-1)
    assert torch.allclose(dot(5, 3), dot(105, 103), atol=1e-9)
    assert not torch.allclose(dot(5, 3), dot(5, 4), atol=1e-3)
    r = plain.rotate_half(q, torch.tensor([11]), 8, 100.0)
    assert torch.allclose(r[..., 8:], q[..., 8:])                 # the rest passes unchanged
    assert torch.allclose(r.norm(dim=-1), q.norm(dim=-1))
    # element i turns with element i + dims/2
    e = torch.zeros(1, 1, 16, dtype=torch.float64)
    e[0, 0, 1] = 1.0
    r = plain.rotate_half(e, torch.tensor([1]), 8, 100.0)
    ang = 100.0 ** (-2.0 / 8)
    assert abs(float(r[0, 0, 1]) - math.cos(ang)) < 1e-12 and abs(float(r[0, 0, 5]) - math.sin(ang)) < 1e-12


def test_retention_is_a_decaying_sum_of_outer_products():
    cfg = ru.one_layer("retention", ru.retention(heads=2, dim=8, vdim=4, decay=[0.5, 1.0], rot_dims=0))
    t = ru.make_tensors(cfg, seed=1)
    m = cfg["layers"][0]["mixer"]
    h = torch.randn(6, cfg["width"], dtype=torch.float64)
    S = torch.zeros(2, 8, 4, dtype=torch.float64)
    plain.retention(h, t, "l0.mix.", m, 1e-5, state=S)
    k = (h @ t["l0.mix.k"].double().T).view(6, 2, 8) * 8 ** -0.5
    v = (h @ t["l0.mix.v"].double().T).view(6, 2, 4)
    for head, a in ((0, 0.5), (1, 1.0)):
        want = sum(a ** (5 - j) * torch.outer(k[j, head], v[j, head]) for j in range(6))
        assert torch.allclose(S[head], want, atol=1e-10)
    # two portions through the state give what one gives
    S2 = torch.zeros_like(S)
    a = plain.retention(h[:4], t, "l0.mix.", m, 1e-5, state=S2)
    b = plain.retention(h[4:], t, "l0.mix.", m, 1e-5, positions=torch.arange(4, 6), state=S2)
    whole = plain.retention(h, t, "l0.mix.", m, 1e-5)
    assert torch.allclose(torch.cat([a, b]), whole, atol=1e-10)


def test_sink_takes_its_share_and_the_cap_bounds_the_scores():
    cfg = ru.one_layer("attention", ru.attention(heads=2, kv_heads=1, dim=16, softcap=0.0, every=0))
    t = ru.make_tensors(cfg, seed=2)
    h = torch.randn(9, cfg["width"], dtype=torch.float64)
    m = cfg["layers"][0]["mixer"]
    base = plain.sink_attention(h, t, "l0.mix.", m)
    # a sink far below every score changes nothing; a sink far above takes everything
    t["l0.mix.sink"] = torch.full((2,), -80.0)
    no_sink = plain.sink_attention(h, t, "l0.mix.", m)
    k = h @ t["l0.mix.k"].double().T
    # the first token sees only itself: without a sink its output is its own key, projected
    want0 = torch.cat([k[0], k[0]]) @ t["l0.mix.o"].double().T
    assert torch.allclose(no_sink[0], want0, atol=1e-9)
    t["l0.mix.sink"] = torch.full((2,), 80.0)
    assert float(plain.sink_attention(h, t, "l0.mix.", m).abs().max()) < 1e-9
    assert not torch.allclose(base, no_sink, atol=1e-3)
    # with a tiny cap every score is nearly the same: the weights become uniform
    t["l0.mix.sink"] = torch.full((2,), -80.0)
    capped = plain.sink_attention(h, t, "l0.mix.", dict(m, softcap=1e-6))
    mean_k = torch.stack([k[:i + 1].mean(0) for i in range(9)])
    assert torch.allclose(capped, torch.cat([mean_k, mean_k], dim=1) @ t["l0.mix.o"].double().T,
                          atol=1e-5)


def test_query_temperature_steps_with_the_position():
    pos = torch.arange(0, 200)
    f = plain.query_temperature(pos, 0.25, 40)
    assert float(f[0]) == 1.0 and float(f[38]) == 1.0
    assert abs(float(f[39]) - (1 + 0.25 * math.log(2))) < 1e-12      # (39 + 1) / 40 = 1
    assert abs(float(f[79]) - (1 + 0.25 * math.log(3))) < 1e-12
    assert float(f[78]) == float(f[39])


def test_table_experts_average_their_experts():
    cfg = ru.one_layer("retention", ru.retention(), ru.moe(ff=8, experts=3, top=2))
    t = ru.make_tensors(cfg, seed=3)
    h = torch.randn(4, cfg["width"], dtype=torch.float64)
    ids = [0, 1, 2, 0]
    got = plain.table_experts(h, ids, t, "l0.mlp.", 2)
    assert torch.allclose(got[0] - got[3], plain.table_experts(h[[0]] - 0, [0], t, "l0.mlp.", 2)[0]
                          - plain.table_experts(h[[3]], [0], t, "l0.mlp.", 2)[0], atol=1e-12)
    e0, e1 = t["l0.mlp.table"][1].tolist()
    one = lambda e: (torch.relu(h[1] @ t[f"l0.mlp.e{e}.up"].double().T) ** 2) @ t[f"l0.mlp.e{e}.down"].double().T
    assert torch.allclose(got[1], 0.5 * (one(e0) + one(e1)), atol=1e-12)
