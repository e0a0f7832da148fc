"""A plain, slow Rudilix: whole sequences, no cache, no batching, one function per
mechanism, on the CPU in float64.  It shares no code with the engine: it takes the
config.json dictionary and a mapping from tensor names to tensors and walks the
sequence token by token wherever the design has a recurrence.

Notation: ``h`` is a mixer's input ``[T, width]``; weights are ``[out, in]`` and
applied as ``h @ W.T``; positions count from 0.
"""

from __future__ import annotations

import math
from typing import Dict, List, Mapping, Optional

import torch

DT = torch.float64


def _w(tensors: Mapping[str, torch.Tensor], name: str) -> torch.Tensor:
    return tensors[name].to(DT)


# ------------------------------------------------------------------ small pieces
def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def offset_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """The block's norm: its weight is stored around zero and used as 1 + w."""
    return rms(x, eps) * (1.0 + w)


def silu(x: torch.Tensor) -> torch.Tensor:
    return x * torch.sigmoid(x)


def softplus(x: torch.Tensor) -> torch.Tensor:
    return torch.log1p(torch.exp(-x.abs())) + torch.clamp(x, min=0.0)


def causal_conv(x: torch.Tensor, taps: torch.Tensor, bias: Optional[torch.Tensor]) -> torch.Tensor:
    """Per channel: y[t, c] = sum_j taps[c, j] * x[t - (L - 1 - j), c], zeros before the
    start; the last column of ``taps`` meets the current token."""
    T, C = x.shape
    L = taps.shape[1]
    y = torch.zeros((T, C), dtype=DT)
    for j in range(L):
        back = L - 1 - j
        if back < T:
            y[back:] += x[:T - back] * taps[:, j]
    if bias is not None:
        y = y + bias
    return y


def rotate_adjacent(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """Rotary positions on the first ``dims`` elements of each head, element 2i paired
    with 2i + 1, angle = position * base^(-2i / dims).  ``x``: [T, heads, dim]."""
    out = x.clone()
    i = torch.arange(dims // 2, dtype=DT)
    freq = torch.pow(torch.tensor(base, dtype=DT), -2.0 * i / dims)
    ang = positions.to(DT)[:, None] * freq[None, :]                 # [T, dims/2]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    a, b = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = a * c - b * s
    out[..., 1:dims:2] = b * c + a * s
    return out


# ---------------------------------------------------------------- feed-forward
def clamped_glu(h: torch.Tensor, tensors, prefix: str, limit: float) -> torch.Tensor:
    g = torch.clamp(h @ _w(tensors, prefix + "gate").T, max=limit)
    u = torch.clamp(h @ _w(tensors, prefix + "up").T, min=-limit, max=limit)
    y = g * torch.sigmoid(1.702 * g) * (u + 1.0)
    return y @ _w(tensors, prefix + "down").T


# --------------------------------------------------- sliding-window attention
def window_attention(h: torch.Tensor, tensors, p: str, cfg: Mapping, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, G, d, dv = cfg["heads"], cfg["kv_heads"], cfg["dim"], cfg["vdim"]
    q = (h @ _w(tensors, p + "q").T + _w(tensors, p + "q.b")).view(T, H, d)
    k = (h @ _w(tensors, p + "k").T + _w(tensors, p + "k.b")).view(T, G, d)
    v = (h @ _w(tensors, p + "v").T + _w(tensors, p + "v.b")).view(T, G, dv)
    q = rms(q, eps) * _w(tensors, p + "q.norm")
    k = rms(k, eps) * _w(tensors, p + "k.norm")
    pos = torch.arange(T)
    rot = cfg.get("rot")
    if rot:
        q = rotate_adjacent(q, pos, int(rot["dims"]), float(rot["base"]))
        k = rotate_adjacent(k, pos, int(rot["dims"]), float(rot["base"]))
    mask = cfg.get("mask")
    window = int(mask["size"]) if mask else 0
    gate = torch.sigmoid(h @ _w(tensors, p + "g").T)                # [T, H]
    out = torch.zeros((T, H, dv), dtype=DT)
    for head in range(H):
        kvh = head // (H // G)
        s = (q[:, head] @ k[:, kvh].T) * float(cfg["scale"])      # [T, T]
        i, j = pos[:, None], pos[None, :]
        seen = (j <= i)
        if window:
            seen = seen & (i - j < window)
        s = s.masked_fill(~seen, -math.inf)
        out[:, head] = torch.softmax(s, dim=-1) @ v[:, kvh]
    out = out * gate[:, :, None]
    return out.reshape(T, H * dv) @ _w(tensors, p + "o").T


# ---------------------------------------------------------- gated delta rule
def channel_delta(h: torch.Tensor, tensors, p: str, cfg: Mapping, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, G, d, dv = cfg["heads"], cfg["kv_heads"], cfg["dim"], cfg["vdim"]
    q = silu(causal_conv(h @ _w(tensors, p + "q").T, _w(tensors, p + "q.conv"), None)).view(T, G, d)
    k = silu(causal_conv(h @ _w(tensors, p + "k").T, _w(tensors, p + "k.conv"), None)).view(T, G, d)
    v = silu(causal_conv(h @ _w(tensors, p + "v").T, _w(tensors, p + "v.conv"), None)).view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ _w(tensors, p + "b").T)                # [T, H]
    a = (h @ _w(tensors, p + "a1").T) @ _w(tensors, p + "a2").T + _w(tensors, p + "dt_bias")
    decay = torch.exp(-torch.exp(_w(tensors, p + "A_log"))[None, :, None]
                      * softplus(a).view(T, H, d))                  # [T, H, d]
    o = torch.zeros((T, H, dv), dtype=DT)
    for head in range(H):
        kvh = head // (H // G)
        S = torch.zeros((d, dv), dtype=DT)
        for t in range(T):
            S = decay[t, head][:, None] * S
            u = beta[t, head] * (v[t, head] - S.T @ k[t, kvh])
            S = S + torch.outer(k[t, kvh], u)
            o[t, head] = S.T @ q[t, kvh]
    gate = torch.sigmoid((h @ _w(tensors, p + "g1").T) @ _w(tensors, p + "g2").T).view(T, H, dv)
    o = rms(o, eps) * _w(tensors, p + "norm") * gate
    return o.reshape(T, H * dv) @ _w(tensors, p + "o").T


# ------------------------------------------------------------------- mamba2
def mamba2(h: torch.Tensor, tensors, p: str, cfg: Mapping, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, P, N, G = cfg["heads"], cfg["vdim"], cfg["state"], cfg["groups"]
    inner = H * P
    zxbcdt = h @ _w(tensors, p + "in").T
    z = zxbcdt[:, :inner]
    xbc = zxbcdt[:, inner:2 * inner + 2 * G * N]
    dt = zxbcdt[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, _w(tensors, p + "conv"), _w(tensors, p + "conv.b")))
    x = xbc[:, :inner].view(T, H, P)
    B = xbc[:, inner:inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + _w(tensors, p + "dt_bias"))                  # [T, H]
    A = torch.exp(_w(tensors, p + "A_log"))
    D = _w(tensors, p + "D")
    y = torch.zeros((T, H, P), dtype=DT)
    for head in range(H):
        g = head // (H // G)
        S = torch.zeros((N, P), dtype=DT)
        for t in range(T):
            S = torch.exp(-A[head] * dt[t, head]) * S + dt[t, head] * torch.outer(B[t, g], x[t, head])
            y[t, head] = S.T @ C[t, g] + D[head] * x[t, head]
    y = y.reshape(T, inner) * silu(z)
    parts = int(cfg["norm_groups"])
    y = rms(y.view(T, parts, inner // parts), eps).reshape(T, inner) * _w(tensors, p + "norm")
    return y @ _w(tensors, p + "o").T


# ------------------------------------------------------------------ the model
def mixer(kind: str, h, tensors, prefix: str, cfg: Mapping, eps: float) -> torch.Tensor:
    if kind == "mamba2":
        return mamba2(h, tensors, prefix, cfg, eps)
    if kind == "channel_delta":
        return channel_delta(h, tensors, prefix, cfg, eps)
    if kind == "parallel":
        left = window_attention(h, tensors, prefix + "left.", cfg["left"], eps)
        right = channel_delta(h, tensors, prefix + "right.", cfg["right"], eps)
        return float(cfg["left_scale"]) * left + float(cfg["right_scale"]) * right
    raise ValueError(kind)


def forward(config: Mapping, tensors: Mapping[str, torch.Tensor], tokens: List[int],
            streams: Optional[list] = None) -> torch.Tensor:
    """Logits ``[T, vocab]`` of one whole sequence.  ``streams`` receives the residual
    stream after every layer."""
    eps = float(config["norm"]["eps"])
    m = float(config["residual_mult"])
    x = _w(tensors, "embed")[torch.tensor(tokens, dtype=torch.long)]
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        h = offset_norm(x, _w(tensors, p + "norm1"), eps)
        x = x + m * mixer(layer["type"], h, tensors, p + "mix.", layer["mixer"], eps)
        if layer.get("mlp"):
            h = offset_norm(x, _w(tensors, p + "norm2"), eps)
            x = x + m * clamped_glu(h, tensors, p + "mlp.", float(layer["mlp"]["limit"]))
        if streams is not None:
            streams.append(x.clone())
    x = offset_norm(x, _w(tensors, "final.norm"), eps)
    return x @ _w(tensors, "head").T
