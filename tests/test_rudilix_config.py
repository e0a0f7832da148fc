"""Rudilix without a GPU: its configuration and the description it turns into, and what
pins the plain implementation (library routines and invariants, not the engine)."""

import math

import pytest
import torch

import plain_rudilix as plain
import rudilix_util as ru
from zig_ai_amd.config import ConfigError, config_from_dict, known_architectures
from zig_ai_amd.weights.loader import expected_tensors


def test_registered_and_round_trip():
    assert "Rudilix" in known_architectures()
    for cfg in (ru.TINY_ALL, ru.TINY_OTHER):
        c = config_from_dict(cfg)
        assert config_from_dict(c.to_dict()) == c
        assert [l.type for l in c.layers] == [l["type"] for l in cfg["layers"]]


def test_spec_names_every_tensor_with_its_shape():
    for cfg in (ru.TINY_ALL, ru.TINY_OTHER):
        tensors = ru.make_tensors(cfg, seed=1)
        c = config_from_dict(cfg).with_shapes(
            lambda name: tuple(tensors[name].shape) if name in tensors else None)
        expected = expected_tensors(c.to_spec())
        names = {e.names[0] for e in expected}
        assert names == set(tensors)
        for e in expected:
            assert tuple(tensors[e.names[0]].shape) in e.rule.shapes, e.names[0]


def test_spec_carries_the_constants():
    c = config_from_dict(ru.TINY_ALL)
    spec = c.to_spec()
    first, third = spec.layers[0], spec.layers[2]
    assert first.arrangement == "scaled_residual_parallel"
    assert first.params == {"residual_scale": 0.8, "mixer_scales": (0.7, 1.3)}
    left = first.parts["left"].params
    assert (left["window"], left["softmax_scale"], left["value_dim"], left["gate"]) == (9, 0.6, 24, "head")
    assert left["position"].params["rotary_dim"] == 8 and left["position"].params["pairing"] == "adjacent"
    assert third.arrangement == "scaled_residual_no_ff" and "feed_forward" not in third.parts
    assert spec.final_norm.params["weight_offset"] == 1.0
    other = config_from_dict(ru.TINY_OTHER).to_spec()
    att = other.layers[2].parts["left"].params
    assert att["window"] == 0 and att["position"] is None


@pytest.mark.parametrize("change,message", [
    (lambda c: c["layers"][0].update(type="conv"), "type must be one of"),
    (lambda c: c["layers"][1]["mixer"].update(groups=3), "do not divide"),
    (lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=7), "must be even"),
    (lambda c: c.pop("norm"), "no norm object"),
    (lambda c: c.pop("width"), "no width"),
])
def test_bad_configurations(change, message):
    import copy
    cfg = copy.deepcopy(ru.TINY_ALL)
    change(cfg)
    with pytest.raises(ConfigError, match=message):
        config_from_dict(cfg)


# ------------------------------------------------- what pins the plain implementation
def test_plain_convolution_against_the_library():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(19, 6, generator=g, dtype=torch.float64)
    w = torch.randn(6, 4, generator=g, dtype=torch.float64)
    b = torch.randn(6, generator=g, dtype=torch.float64)
    want = torch.nn.functional.conv1d(torch.nn.functional.pad(x.T[None], (3, 0)), w[:, None, :], b,
                                      groups=6)[0].T
    assert torch.allclose(plain.causal_conv(x, w, b), want, atol=1e-12)


def test_plain_rotation_depends_on_distance_only():
    g = torch.Generator().manual_seed(1)
    q = torch.randn(1, 1, 12, generator=g, dtype=torch.float64)
    k = torch.randn(1, 1, 12, generator=g, dtype=torch.float64)

    def score(pq, pk):
        a = plain.rotate_adjacent(q, torch.tensor([pq]), 8, 300.0)
        b = plain.rotate_adjacent(k, torch.tensor([pk]), 8, 300.0)
        return float((a * b).sum())
    assert abs(score(5, 2) - score(40, 37)) < 1e-10
    assert abs(score(5, 2) - score(5, 3)) > 1e-6
    r = plain.rotate_adjacent(q, torch.tensor([9]), 8, 300.0)
    assert torch.equal(r[..., 8:], q[..., 8:])                  # beyond rot.dims: unchanged
    assert abs(float(r.norm()) - float(q.norm())) < 1e-12
    # pair (0, 1) at position 1 turns by the angle 1 * base^0 = 1
    e = torch.zeros(1, 1, 12, dtype=torch.float64)
    e[..., 0] = 1.0
    r = plain.rotate_adjacent(e, torch.tensor([1]), 8, 300.0)
    assert abs(float(r[0, 0, 0]) - math.cos(1.0)) < 1e-12 and abs(float(r[0, 0, 1]) - math.sin(1.0)) < 1e-12


def test_plain_delta_rule_recalls_what_it_stored():
    """With no decay and beta = 1, writing (k, v) and reading with q = k gives v back;
    writing the same key again replaces the value."""
    cfg = ru.one_layer("channel_delta", ru.delta(heads=1, kv_heads=1, dim=4, vdim=3, conv=1), ff=0)
    d, dv = 4, 3
    S = torch.zeros((d, dv), dtype=torch.float64)
    k = torch.tensor([0.6, 0.0, 0.8, 0.0], dtype=torch.float64)
    for v in (torch.tensor([1.0, 2.0, 3.0], dtype=torch.float64),
              torch.tensor([-1.0, 0.5, 0.0], dtype=torch.float64)):
        u = 1.0 * (v - S.T @ k)
        S = S + torch.outer(k, u)
        assert torch.allclose(S.T @ k, v, atol=1e-12)
    assert cfg["layers"][0]["type"] == "channel_delta"


def test_plain_model_is_causal_and_windowed():
    cfg = ru.one_layer("parallel", ru.parallel(ru.attention(window=5), right_scale=0.0), ff=0)
    tensors = ru.make_tensors(cfg, seed=2)
    a = ru.tokens(30, cfg["vocab"], 1)
    b = list(a)
    b[10] = (b[10] + 1) % cfg["vocab"]
    la, lb = plain.forward(cfg, tensors, a), plain.forward(cfg, tensors, b)
    changed = ((la - lb).abs().max(dim=1).values > 1e-9).nonzero().flatten().tolist()
    assert changed == [10, 11, 12, 13, 14]          # itself and the window - 1 = 4 after it


def test_plain_softplus_and_norms():
    x = torch.tensor([-50.0, -1.0, 0.0, 2.0, 90.0], dtype=torch.float64)
    assert torch.allclose(plain.softplus(x), torch.nn.functional.softplus(x, threshold=1e9), atol=1e-12)
    v = torch.tensor([[3.0, 4.0]], dtype=torch.float64)
    assert torch.allclose(plain.rms(v, 0.0), v / math.sqrt(12.5))
    assert torch.allclose(plain.offset_norm(v, torch.tensor([0.5, -1.0], dtype=torch.float64), 0.0),
                          v / math.sqrt(12.5) * torch.tensor([1.5, 0.0], dtype=torch.float64))
