"""Small Rudilix configurations and weights for tests, made here: none of them is a
model anybody ships.  The weights are drawn so that faults show: attention scores spread
over several units (a lost key, or one too many, moves the output), decays from fast to
very slow (a far token still counts in some heads), filters, gates and norms that are not
near-trivial."""

import json
import math
import os
import tempfile

import torch

FOLDERS = {}


def attention(heads=4, kv_heads=2, dim=16, vdim=24, window=9, rot_dims=8, base=500.0, scale=0.6):
    out = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        out["mask"] = {"size": window}
    if rot_dims:
        out["rot"] = {"dims": rot_dims, "base": base}
    return out


def delta(heads=4, kv_heads=2, dim=16, vdim=24, conv=3):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}


def ssd(heads=4, vdim=16, state=24, groups=2, norm_groups=2, conv=4):
    return {"heads": heads, "vdim": vdim, "state": state, "groups": groups,
            "norm_groups": norm_groups, "conv": conv}


def layer(kind, mixer, ff=96, limit=1.5):
    return {"type": kind, "mixer": mixer,
            "mlp": {"kind": "dense", "ff": ff, "limit": limit} if ff else None}


def parallel(left=None, right=None, left_scale=0.7, right_scale=1.3):
    return {"left": left or attention(), "right": right or delta(),
            "left_scale": left_scale, "right_scale": right_scale}


def config(layers, width=64, vocab=160, residual_mult=0.8, eps=1e-5):
    return {"architecture": "Rudilix", "vocab": vocab, "width": width,
            "residual_mult": residual_mult, "norm": {"eps": eps}, "layers": layers}


# every layer type, sizes that differ from one another wherever two could be equal:
# grouped key/value heads in both the attention and the delta rule, several groups and
# norm groups in the state-space layer, a layer without a feed-forward, two filter lengths
TINY_ALL = config([
    layer("parallel", parallel()),
    layer("mamba2", ssd()),
    layer("channel_delta", delta(heads=6, kv_heads=3, dim=8, vdim=16, conv=2), ff=0),
    layer("parallel", parallel(attention(heads=2, kv_heads=1, dim=24, vdim=8, window=33,
                                         rot_dims=24, base=10000.0, scale=0.3),
                               delta(heads=2, kv_heads=2, dim=24, vdim=8, conv=4),
                               left_scale=1.0, right_scale=0.4), ff=40, limit=0.8),
    layer("mamba2", ssd(heads=3, vdim=8, state=40, groups=1, norm_groups=3, conv=2), ff=72),
])

# another order, other sizes: equal key and value widths, one head, residual weight 1,
# an attention without a window and without rotation, a filter of one tap
TINY_OTHER = config([
    layer("channel_delta", delta(heads=1, kv_heads=1, dim=32, vdim=32, conv=1)),
    layer("mamba2", ssd(heads=1, vdim=32, state=16, groups=1, norm_groups=1, conv=3), ff=0),
    layer("parallel", parallel(attention(heads=3, kv_heads=3, dim=16, vdim=16, window=0,
                                         rot_dims=0, scale=0.5),
                               delta(heads=3, kv_heads=1, dim=16, vdim=8, conv=5),
                               left_scale=1.0, right_scale=1.0)),
], width=48, vocab=97, residual_mult=1.0, eps=1e-6)


def one_layer(kind, mixer, **kw):
    return config([layer(kind, mixer, **kw)])


def low_rank(cfg_layer):
    return 8 if cfg_layer["heads"] % 2 == 0 else 12


def make_tensors(cfg, seed=0, ranks=None):
    """name -> float32 tensor (values representable in bfloat16) for ``cfg``."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def normal(*shape, std=1.0, mean=0.0):
        t = torch.randn(*shape, generator=g) * std + mean
        return t.to(torch.bfloat16).to(torch.float32)

    def uniform(*shape, lo=0.0, hi=1.0):
        t = torch.rand(*shape, generator=g) * (hi - lo) + lo
        return t.to(torch.bfloat16).to(torch.float32)

    out = {"embed": normal(cfg["vocab"], W), "head": normal(cfg["vocab"], W, std=W ** -0.5),
           "final.norm": normal(W, std=0.3)}

    def add_delta(p, m):
        H, G, d, dv, L = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
        r = (ranks or {}).get(p, low_rank(m))
        for name, rows in (("q", G * d), ("k", G * d), ("v", H * dv)):
            out[p + name] = normal(rows, W, std=2.0 * W ** -0.5)
            out[p + name + ".conv"] = normal(rows, L, std=0.6)
        out[p + "b"] = normal(H, W, std=2.0 * W ** -0.5)
        out[p + "A_log"] = uniform(H, lo=-6.0, hi=0.5)
        out[p + "norm"] = normal(dv, std=0.3, mean=1.0)
        out[p + "a1"] = normal(r, W, std=W ** -0.5)
        out[p + "a2"] = normal(H * d, r, std=1.5 * r ** -0.5)
        out[p + "dt_bias"] = normal(H * d, std=1.0)
        out[p + "g1"] = normal(r + 4, W, std=W ** -0.5)
        out[p + "g2"] = normal(H * dv, r + 4, std=1.5 * (r + 4) ** -0.5)
        out[p + "o"] = normal(W, H * dv, std=(H * dv) ** -0.5)

    def add_attention(p, m):
        H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        for name, rows in (("q", H * d), ("k", G * d), ("v", G * dv)):
            out[p + name] = normal(rows, W, std=W ** -0.5)
            out[p + name + ".b"] = normal(rows, std=0.3)
        out[p + "q.norm"] = normal(d, std=0.3, mean=1.2)
        out[p + "k.norm"] = normal(d, std=0.3, mean=1.2)
        out[p + "g"] = normal(H, W, std=2.0 * W ** -0.5)
        out[p + "o"] = normal(W, H * dv, std=(H * dv) ** -0.5)

    def add_ssd(p, m):
        H, P, N, G, L = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
        inner, C = H * P, H * P + 2 * G * N
        out[p + "in"] = normal(2 * inner + 2 * G * N + H, W, std=1.5 * W ** -0.5)
        out[p + "conv"] = normal(C, L, std=0.6)
        out[p + "conv.b"] = normal(C, std=0.2)
        out[p + "dt_bias"] = normal(H, std=1.0)
        out[p + "A_log"] = uniform(H, lo=-5.0, hi=1.0)
        out[p + "D"] = normal(H, std=0.5, mean=1.0)
        out[p + "norm"] = normal(inner, std=0.3, mean=1.0)
        out[p + "o"] = normal(W, inner, std=inner ** -0.5)

    for i, lay in enumerate(cfg["layers"]):
        p = f"l{i}."
        out[p + "norm1"] = normal(W, std=0.3)
        if lay["type"] == "mamba2":
            add_ssd(p + "mix.", lay["mixer"])
        elif lay["type"] == "channel_delta":
            add_delta(p + "mix.", lay["mixer"])
        else:
            add_attention(p + "mix.left.", lay["mixer"]["left"])
            add_delta(p + "mix.right.", lay["mixer"]["right"])
        if lay["mlp"]:
            F = lay["mlp"]["ff"]
            out[p + "norm2"] = normal(W, std=0.3)
            out[p + "mlp.gate"] = normal(F, W, std=2.0 * W ** -0.5)
            out[p + "mlp.up"] = normal(F, W, std=2.0 * W ** -0.5)
            out[p + "mlp.down"] = normal(W, F, std=F ** -0.5)
    return out


def folder(cfg, seed=0, tensors=None):
    """A model folder (config.json, model.safetensors in bfloat16) in a temporary place;
    returns (folder, tensors as float32)."""
    from safetensors.torch import save_file
    key = (json.dumps(cfg, sort_keys=True), seed) if tensors is None else None
    if key is not None and key in FOLDERS:
        return FOLDERS[key]
    if tensors is None:
        tensors = make_tensors(cfg, seed)
    d = tempfile.mkdtemp(prefix="rudilix_model_")
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in tensors.items()},
              os.path.join(d, "model.safetensors"))
    if key is not None:
        FOLDERS[key] = (d, tensors)
    return d, tensors


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(1000 + seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def row_error(got, want):
    """Per row: the root mean square of the difference (means taken off) relative to the
    root mean square of the wanted logits over all rows."""
    got, want = got.double(), want.double()
    assert got.shape == want.shape, (got.shape, want.shape)
    assert torch.isfinite(got).all(), "non-finite logits"
    d = got - want
    d = d - d.mean(dim=1, keepdim=True)
    scale = (want - want.mean(dim=1, keepdim=True)).pow(2).mean().sqrt()
    return d.pow(2).mean(dim=1).sqrt() / scale


def random_config(seed):
    """A configuration drawn at random: layer order, every size and every constant."""
    import random
    rng = random.Random(seed)

    def pick(*values):
        return rng.choice(values)

    def rand_delta():
        kv = pick(1, 2, 3)
        return delta(heads=kv * pick(1, 2), kv_heads=kv, dim=pick(8, 12, 16, 40, 72),
                     vdim=pick(4, 8, 12, 24, 40), conv=pick(1, 2, 3, 4, 5))

    def rand_attention():
        kv = pick(1, 2, 3)
        dim = pick(8, 16, 24, 40)
        return attention(heads=kv * pick(1, 2, 4), kv_heads=kv, dim=dim, vdim=pick(8, 16, 32, 48),
                         window=pick(0, 1, 2, 5, 17, 64, 500), rot_dims=pick(0, 2, dim // 2 // 2 * 2, dim),
                         base=pick(10.0, 1000.0, 50000.0), scale=pick(0.1, 0.35, 0.7))

    def rand_ssd():
        groups = pick(1, 2, 3)
        heads = groups * pick(1, 2)
        vdim = pick(4, 8, 12, 24)
        norm_groups = pick(*[g for g in (1, 2, 3, 4, heads) if (heads * vdim) % g == 0])
        return ssd(heads=heads, vdim=vdim, state=pick(4, 8, 20, 48, 136), groups=groups,
                   norm_groups=norm_groups, conv=pick(2, 3, 4, 6))

    layers = []
    for _ in range(pick(1, 2, 3, 4, 6)):
        kind = pick("mamba2", "channel_delta", "parallel")
        if kind == "mamba2":
            mixer = rand_ssd()
        elif kind == "channel_delta":
            mixer = rand_delta()
        else:
            mixer = parallel(rand_attention(), rand_delta(), pick(0.3, 1.0, -0.8), pick(0.5, 1.0, 1.6))
        layers.append(layer(kind, mixer, ff=pick(0, 8, 24, 100), limit=pick(0.3, 1.0, 4.0)))
    return config(layers, width=pick(16, 24, 40, 64, 104), vocab=pick(11, 50, 203),
                  residual_mult=pick(0.25, 1.0, 1.5), eps=pick(1e-6, 1e-5, 1e-3))
