"""Small Ranesun configurations and weights for tests, made here: none of them is a model
anybody ships.  The weights are drawn so that faults show: attention scores spread over
several units and reach the cap, sinks that take a visible share of a head's weight,
decays from fast to very slow, norms with biases, tables that send neighbouring token ids
to different experts."""

import json
import os
import tempfile

import torch

FOLDERS = {}


def retention(heads=3, dim=16, vdim=24, decay=None, rot_dims=8, base=300.0):
    out = {"heads": heads, "dim": dim, "vdim": vdim,
           "decay": list(decay) if decay is not None
           else [1.0 - 2.0 ** -(3 + 2 * h) for h in range(heads)]}
    if rot_dims:
        out["rot"] = {"dims": rot_dims, "base": base}
    return out


def attention(heads=4, kv_heads=2, dim=16, scale=0.5, softcap=4.0, coef=0.3, every=7):
    out = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale}
    if softcap:
        out["softcap"] = softcap
    if every:
        out["q_temp"] = {"coef": coef, "every": every}
    return out


def dense(ff=72):
    return {"kind": "dense", "ff": ff}


def moe(ff=24, experts=5, top=2):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def layer(kind, mixer, mlp=None):
    return {"type": kind, "mixer": mixer, "mlp": mlp}


def config(layers, width=48, vocab=131, eps=1e-5, logit_scale=1.5, loop=None):
    out = {"architecture": "Ranesun", "vocab": vocab, "width": width, "norm": {"eps": eps},
           "logit_scale": logit_scale, "layers": layers}
    if loop is not None:
        out["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return out


# both mixers, all three kinds of feed-forward (and none), a loop over the middle that
# starts behind the first layer and runs three times; sizes differ wherever two could be
# equal (query/key width against value width, heads against key/value heads)
TINY_ALL = config([
    layer("attention", attention(), dense()),
    layer("retention", retention(), moe()),
    layer("attention", attention(heads=6, kv_heads=1, dim=8, scale=0.8, softcap=2.5, coef=0.7,
                                 every=3), None),
    layer("retention", retention(heads=2, dim=24, vdim=8, rot_dims=24, base=10000.0),
          moe(ff=16, experts=3, top=1)),
    layer("attention", attention(heads=2, kv_heads=2, dim=32, scale=0.3, softcap=0.0, every=0),
          dense(40)),
], loop=(1, 4, 3))

# another order and other sizes: no loop at all, one head, top = experts, no rotation,
# a rotation of two elements, logit scale 1, query/key width equal to the value width
TINY_OTHER = config([
    layer("retention", retention(heads=1, dim=32, vdim=32, decay=[0.96875], rot_dims=0), dense(56)),
    layer("retention", retention(heads=4, dim=8, vdim=16, rot_dims=2, base=50.0), None),
    layer("attention", attention(heads=3, kv_heads=3, dim=16, scale=0.45, softcap=9.0, coef=0.1,
                                 every=50), moe(ff=32, experts=2, top=2)),
], width=40, vocab=67, eps=1e-6, logit_scale=1.0)

# a loop that is the whole model and runs once, and one that runs twice from layer 0
TINY_LOOP_ONCE = config([layer("retention", retention(), dense(24)),
                         layer("attention", attention(), None)], loop=(0, 2, 1))
TINY_LOOP_TWICE = config([layer("attention", attention(), moe()),
                          layer("retention", retention(), dense(24))], loop=(0, 1, 2))


def one_layer(kind, mixer, mlp=None, **kw):
    return config([layer(kind, mixer, mlp)], **kw)


def make_tensors(cfg, seed=0):
    """name -> float32 tensor (values representable in bfloat16; tables int32) for ``cfg``."""
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]

    def normal(*shape, std=1.0, mean=0.0):
        t = torch.randn(*shape, generator=g) * std + mean
        return t.to(torch.bfloat16).to(torch.float32)

    out = {"embed": normal(V, W), "final.norm": normal(W, std=0.3, mean=1.0),
           "final.norm.b": normal(W, std=0.3)}
    if cfg.get("loop"):
        out["loop.step"] = normal(cfg["loop"]["times"], W, std=0.7)
    for i, lay in enumerate(cfg["layers"]):
        p, m = f"l{i}.", lay["mixer"]
        out[p + "norm1"] = normal(W, std=0.3, mean=1.0)
        out[p + "norm1.b"] = normal(W, std=0.3)
        if lay["type"] == "retention":
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            out[p + "mix.q"] = normal(H * d, W, std=2.0 * W ** -0.5)
            out[p + "mix.k"] = normal(H * d, W, std=2.0 * W ** -0.5)
            out[p + "mix.v"] = normal(H * dv, W, std=W ** -0.5)
            out[p + "mix.g"] = normal(H * dv, W, std=2.0 * W ** -0.5)
            out[p + "mix.o"] = normal(W, H * dv, std=(H * dv) ** -0.5)
        else:
            H, G, d = m["heads"], m["kv_heads"], m["dim"]
            out[p + "mix.q"] = normal(H * d, W, std=2.0 * W ** -0.5)
            out[p + "mix.k"] = normal(G * d, W, std=2.0 * W ** -0.5)
            out[p + "mix.sink"] = normal(H, std=1.5, mean=1.0)
            out[p + "mix.o"] = normal(W, H * d, std=(H * d) ** -0.5)
        mlp = lay["mlp"]
        if mlp is None:
            continue
        out[p + "norm2"] = normal(W, std=0.3, mean=1.0)
        out[p + "norm2.b"] = normal(W, std=0.3)
        if mlp["kind"] == "dense":
            F = mlp["ff"]
            out[p + "mlp.gate"] = normal(F, W, std=2.0 * W ** -0.5)
            out[p + "mlp.up"] = normal(F, W, std=2.0 * W ** -0.5)
            out[p + "mlp.down"] = normal(W, F, std=F ** -0.5)
        else:
            F, E, top = mlp["expert"]["ff"], mlp["router"]["experts"], mlp["router"]["top"]
            for e in range(E):
                out[f"{p}mlp.e{e}.up"] = normal(F, W, std=2.0 * W ** -0.5)
                out[f"{p}mlp.e{e}.down"] = normal(W, F, std=2.0 * F ** -0.5)
            noise = torch.rand(V, E, generator=g)
            out[p + "mlp.table"] = noise.argsort(dim=1)[:, :top].to(torch.int32).contiguous()
    return out


def folder(cfg, seed=0, tensors=None):
    """A model folder (config.json, model.safetensors: bfloat16, tables int32) in a
    temporary place; returns (folder, tensors)."""
    from safetensors.torch import save_file
    key = (json.dumps(cfg, sort_keys=True), seed) if tensors is None else None
    if key is not None and key in FOLDERS:
        return FOLDERS[key]
    if tensors is None:
        tensors = make_tensors(cfg, seed)
    d = tempfile.mkdtemp(prefix="ranesun_model_")
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: (v if v.dtype == torch.int32 else v.to(torch.bfloat16)).contiguous()
               for k, v in tensors.items()}, os.path.join(d, "model.safetensors"))
    if key is not None:
        FOLDERS[key] = (d, tensors)
    return d, tensors


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(2000 + seed)
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

    def rand_retention():
        heads, dim = pick(1, 2, 3, 5), pick(8, 16, 24, 40, 72)
        return retention(heads=heads, dim=dim, vdim=pick(8, 16, 24, 40),
                         decay=[pick(0.5, 0.9, 0.96875, 0.99951171875, 1.0) for _ in range(heads)],
                         rot_dims=pick(0, 2, dim // 4 * 2, dim), base=pick(10.0, 1000.0, 5e5))

    def rand_attention():
        kv = pick(1, 2, 3)
        return attention(heads=kv * pick(1, 2, 4), kv_heads=kv, dim=pick(16, 32, 48, 64),
                         scale=pick(0.1, 0.35, 0.7), softcap=pick(0.0, 1.0, 5.0, 20.0),
                         coef=pick(-0.2, 0.25, 1.0), every=pick(0, 1, 2, 16, 48))

    def rand_mlp():
        kind = pick("none", "dense", "moe", "moe")
        if kind == "none":
            return None
        if kind == "dense":
            return dense(pick(8, 24, 100))
        experts = pick(1, 2, 4, 9)
        return moe(ff=pick(8, 16, 40), experts=experts, top=pick(*range(1, min(experts, 3) + 1)))

    n = pick(1, 2, 3, 4, 5)
    layers = [layer(*pick(("retention", rand_retention()), ("attention", rand_attention())),
                    rand_mlp()) for _ in range(n)]
    loop = None
    if pick(True, True, False):
        start = rng.randrange(n)
        loop = (start, rng.randrange(start + 1, n + 1), pick(1, 2, 3))
    return config(layers, width=pick(16, 24, 40, 64, 104), vocab=pick(11, 50, 203),
                  eps=pick(1e-6, 1e-5, 1e-3), logit_scale=pick(0.5, 1.0, 3.0), loop=loop)
