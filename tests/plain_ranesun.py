"""A plain, slow Ranesun: whole sequences, no cache, no batching, one function per
mechanism, on the CPU in float64.  It shares no code with the engine: it takes the
config.json dictionary and a mapping from tensor names to tensors.  The retention is
walked token by token.

Notation: ``h`` is a mixer's input ``[T, width]``; weights are ``[out, in]`` and applied
as ``h @ W.T``; positions count from 0.
"""

from __future__ import annotations

import math
from typing import Dict, List, Mapping, Optional

import torch

DT = torch.float64


def _w(tensors: Mapping[str, torch.Tensor], name: str) -> torch.Tensor:
    return tensors[name].to(DT)


# ------------------------------------------------------------------ small pieces
def layer_norm(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float) -> torch.Tensor:
    """(x - mean) / sqrt(mean((x - mean)^2) + eps) * w + b over the last axis."""
    mu = x.mean(dim=-1, keepdim=True)
    c = x - mu
    return c / torch.sqrt((c * c).mean(dim=-1, keepdim=True) + eps) * w + b


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def silu(x: torch.Tensor) -> torch.Tensor:
    return x * torch.sigmoid(x)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rotate_half(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """Rotary positions on the first ``dims`` elements of each head, element i paired with
    i + dims/2, angle = position * base^(-2i / dims).  ``x``: [T, heads, dim]."""
    out = x.clone()
    half = dims // 2
    i = torch.arange(half, dtype=DT)
    freq = torch.pow(torch.tensor(base, dtype=DT), -2.0 * i / dims)
    ang = positions.to(DT)[:, None] * freq[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    a, b = x[..., :half], x[..., half:dims]
    out[..., :half] = a * c - b * s
    out[..., half:dims] = b * c + a * s
    return out


# -------------------------------------------------------------------- retention
def retention(h: torch.Tensor, tensors, p: str, m: Mapping, eps: float,
              positions: Optional[torch.Tensor] = None,
              state: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Linear attention with one fixed decay per head: S <- decay S + k v^T, o = S^T q;
    no softmax, no denominator.  ``state`` ([heads, dim, vdim], updated in place) lets a
    caller go on from an earlier portion."""
    T = h.shape[0]
    H, d, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    pos = torch.arange(T) if positions is None else positions
    q = (h @ _w(tensors, p + "q").T).view(T, H, d)
    k = (h @ _w(tensors, p + "k").T).view(T, H, d)
    v = (h @ _w(tensors, p + "v").T).view(T, H, dv)
    rot = m.get("rot")
    if rot:
        q = rotate_half(q, pos, int(rot["dims"]), float(rot["base"]))
        k = rotate_half(k, pos, int(rot["dims"]), float(rot["base"]))
    k = k * d ** -0.5
    decay = torch.tensor([float(x) for x in m["decay"]], dtype=DT)
    S = torch.zeros((H, d, dv), dtype=DT) if state is None else state
    o = torch.zeros((T, H, dv), dtype=DT)
    for t in range(T):
        S.mul_(decay[:, None, None])
        S.add_(k[t][:, :, None] * v[t][:, None, :])
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    o = unit_rms(o, eps).reshape(T, H * dv)
    return (o * silu(h @ _w(tensors, p + "g").T)) @ _w(tensors, p + "o").T


# -------------------------------------------------------------------- attention
def query_temperature(positions: torch.Tensor, coef: float, every: int) -> torch.Tensor:
    """1 + coef * ln(floor((p + 1) / every) + 1)."""
    return 1.0 + coef * torch.log(torch.div(positions + 1, every, rounding_mode="floor").to(DT) + 1.0)


def sink_attention(h: torch.Tensor, tensors, p: str, m: Mapping) -> torch.Tensor:
    """Causal attention whose values are its keys, with a capped score and one more term
    exp(sink_h) in the softmax's denominator."""
    T = h.shape[0]
    H, G, d = int(m["heads"]), int(m["kv_heads"]), int(m["dim"])
    q = (h @ _w(tensors, p + "q").T).view(T, H, d)
    k = (h @ _w(tensors, p + "k").T).view(T, G, d)
    pos = torch.arange(T)
    temp = m.get("q_temp")
    if temp:
        q = q * query_temperature(pos, float(temp["coef"]), int(temp["every"]))[:, None, None]
    sink = _w(tensors, p + "sink")
    cap = float(m.get("softcap") or 0.0)
    out = torch.zeros((T, H, d), dtype=DT)
    causal = pos[None, :] <= pos[:, None]
    for hh in range(H):
        kk = k[:, hh // (H // G)]
        s = (q[:, hh] @ kk.T) * float(m["scale"])
        if cap:
            s = cap * torch.tanh(s / cap)
        s = s.masked_fill(~causal, -math.inf)
        top = torch.maximum(s.max(dim=-1, keepdim=True).values, sink[hh])
        e = torch.exp(s - top)
        out[:, hh] = (e / (e.sum(dim=-1, keepdim=True) + torch.exp(sink[hh] - top))) @ kk
    return out.reshape(T, H * d) @ _w(tensors, p + "o").T


# ----------------------------------------------------------------- feed-forward
def dense_ff(h: torch.Tensor, tensors, p: str) -> torch.Tensor:
    a = gelu_tanh(h @ _w(tensors, p + "gate").T) * (h @ _w(tensors, p + "up").T)
    return a @ _w(tensors, p + "down").T


def table_experts(h: torch.Tensor, token_ids: List[int], tensors, p: str, top: int) -> torch.Tensor:
    """Every token id names its experts in a table; each counts 1/top."""
    table = tensors[p + "table"].to(torch.int64)
    out = torch.zeros_like(h)
    for t, tok in enumerate(token_ids):
        for e in table[tok].tolist():
            u = torch.relu(h[t] @ _w(tensors, f"{p}e{e}.up").T) ** 2
            out[t] += (u @ _w(tensors, f"{p}e{e}.down").T) / top
    return out


# ------------------------------------------------------------------- the model
def run_order(config: Mapping) -> List[tuple]:
    """[(layer, number of the pass or None, first of its pass)]"""
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return [(i, None, False) for i in range(n)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    order = [(i, None, False) for i in range(a)]
    for t in range(times):
        order += [(i, t, i == a) for i in range(a, b)]
    return order + [(i, None, False) for i in range(b, n)]


def forward(config: Mapping, tensors: Mapping[str, torch.Tensor], token_ids: List[int],
            streams: Optional[List[torch.Tensor]] = None) -> torch.Tensor:
    """Logits [T, vocab] in float64.  ``streams`` receives the residual stream after
    every layer run."""
    eps = float(config["norm"]["eps"])
    x0 = _w(tensors, "embed")[torch.tensor(token_ids)]
    x = x0.clone()
    for i, t, first in run_order(config):
        if first:
            if t > 0:
                x = x + x0
            x = x + _w(tensors, "loop.step")[t]
        layer, p = config["layers"][i], f"l{i}."
        h = layer_norm(x, _w(tensors, p + "norm1"), _w(tensors, p + "norm1.b"), eps)
        if layer["type"] == "retention":
            x = x + retention(h, tensors, p + "mix.", layer["mixer"], eps)
        elif layer["type"] == "attention":
            x = x + sink_attention(h, tensors, p + "mix.", layer["mixer"])
        else:
            raise ValueError(layer["type"])
        mlp = layer.get("mlp")
        if mlp is not None:
            h = layer_norm(x, _w(tensors, p + "norm2"), _w(tensors, p + "norm2.b"), eps)
            if mlp["kind"] == "dense":
                x = x + dense_ff(h, tensors, p + "mlp.")
            else:
                x = x + table_experts(h, token_ids, tensors, p + "mlp.", int(mlp["router"]["top"]))
        if streams is not None:
            streams.append(x.clone())
    x = layer_norm(x, _w(tensors, "final.norm"), _w(tensors, "final.norm.b"), eps)
    return (x @ _w(tensors, "embed").T) * float(config.get("logit_scale", 1.0))
