"""Typed configuration of Rudilix, a decoder whose layers mix tokens in one of three
ways, listed layer by layer in config.json:

  ``mamba2``         a state-space-duality mixer (``parts/recurrent.py``, ``ssd``)
  ``channel_delta``  the gated delta rule with one decay per key channel (``gated_delta``)
  ``parallel``       sliding-window attention with a gate per head (``gqa_attention`` with
                     ``value_dim`` and ``gate``) beside a ``channel_delta`` mixer, both on
                     the same normed input, added with ``left_scale`` / ``right_scale``

Each layer is pre-norm with a residual weight (``residual_mult``), norms store their
weight around zero, and the feed-forward (``mlp``, may be absent) is a gated unit with
bounded inputs.  config.json keys: ``architecture``, ``vocab``, ``width``,
``residual_mult``, ``norm.eps`` and ``layers[i] = {type, mixer, mlp}``; tensor names:
``embed``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``,
``final.norm``, ``head``.  The low-rank widths of the delta mixer's decay and gate are
not in config.json; the loader reads them from the stored shapes (``with_shapes``).
"""

from __future__ import annotations

from dataclasses import dataclass, field, replace
from typing import Any, Callable, Dict, Mapping, Optional, Tuple

from .fields import read_float, read_int
from .spec import ConfigError, LayerCall, LayerSpec, ModelSpec, PartSpec

LAYER_TYPES = ("mamba2", "channel_delta", "parallel")
# constants of the design's feed-forward: y = g * sigmoid(GLU_ALPHA * g) * (u + GLU_UP_OFFSET)
GLU_ALPHA = 1.702
GLU_UP_OFFSET = 1.0
DEFAULT_LOW_RANK = 32      # of a model that is made from sizes alone


def _mapping(data: Mapping[str, Any], key: str, where: str) -> Mapping[str, Any]:
    value = data.get(key)
    if not isinstance(value, Mapping):
        raise ConfigError(f"{where} has no {key} object")
    return value


@dataclass(frozen=True)
class DeltaSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    decay_rank: int = DEFAULT_LOW_RANK
    gate_rank: int = DEFAULT_LOW_RANK

    @classmethod
    def read(cls, m: Mapping[str, Any], where: str) -> "DeltaSizes":
        heads = read_int(m, ["heads"], minimum=1)
        kv = read_int(m, ["kv_heads"], default=heads, minimum=1)
        if heads % kv:
            raise ConfigError(f"{where}: {heads} heads do not divide into {kv} kv_heads")
        return cls(heads, kv, read_int(m, ["dim"], minimum=1), read_int(m, ["vdim"], minimum=1),
                   read_int(m, ["conv"], minimum=1),
                   read_int(m, ["decay_rank"], default=DEFAULT_LOW_RANK, minimum=1),
                   read_int(m, ["gate_rank"], default=DEFAULT_LOW_RANK, minimum=1))

    def to_dict(self) -> dict:
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim,
                "vdim": self.vdim, "conv": self.conv}


@dataclass(frozen=True)
class AttentionSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int                      # 0: every earlier key
    rot_dims: int                    # 0: no rotation
    rot_base: float

    @classmethod
    def read(cls, m: Mapping[str, Any], where: str) -> "AttentionSizes":
        heads = read_int(m, ["heads"], minimum=1)
        kv = read_int(m, ["kv_heads"], default=heads, minimum=1)
        if heads % kv:
            raise ConfigError(f"{where}: {heads} heads do not divide into {kv} kv_heads")
        dim = read_int(m, ["dim"], minimum=1)
        mask, rot = m.get("mask"), m.get("rot")
        window = read_int(mask, ["size"], minimum=1) if isinstance(mask, Mapping) else 0
        dims, base = 0, 10000.0
        if isinstance(rot, Mapping):
            dims = read_int(rot, ["dims"], minimum=2)
            base = read_float(rot, ["base"], positive=True)
            if dims % 2 or dims > dim:
                raise ConfigError(f"{where}: rot.dims {dims} must be even and at most dim {dim}")
        return cls(heads, kv, dim, read_int(m, ["vdim"], default=dim, minimum=1),
                   read_float(m, ["scale"], default=dim ** -0.5, positive=True), window, dims, base)

    def to_dict(self) -> dict:
        out: Dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim,
                               "vdim": self.vdim, "scale": self.scale}
        if self.window:
            out["mask"] = {"size": self.window}
        if self.rot_dims:
            out["rot"] = {"dims": self.rot_dims, "base": self.rot_base}
        return out


@dataclass(frozen=True)
class SsdSizes:
    heads: int
    vdim: int
    state: int
    groups: int
    norm_groups: int
    conv: int

    @classmethod
    def read(cls, m: Mapping[str, Any], where: str) -> "SsdSizes":
        heads = read_int(m, ["heads"], minimum=1)
        groups = read_int(m, ["groups"], default=1, minimum=1)
        norm_groups = read_int(m, ["norm_groups"], default=1, minimum=1)
        vdim = read_int(m, ["vdim"], minimum=1)
        if heads % groups:
            raise ConfigError(f"{where}: {heads} heads do not divide into {groups} groups")
        if (heads * vdim) % norm_groups:
            raise ConfigError(f"{where}: {heads * vdim} channels do not divide into "
                              f"{norm_groups} norm_groups")
        return cls(heads, vdim, read_int(m, ["state"], minimum=1), groups, norm_groups,
                   read_int(m, ["conv"], minimum=1))

    def to_dict(self) -> dict:
        return {"heads": self.heads, "vdim": self.vdim, "state": self.state,
                "groups": self.groups, "norm_groups": self.norm_groups, "conv": self.conv}


@dataclass(frozen=True)
class RudilixLayer:
    type: str
    ssd: Optional[SsdSizes] = None
    delta: Optional[DeltaSizes] = None          # the layer's own, or the parallel layer's right
    attention: Optional[AttentionSizes] = None  # the parallel layer's left
    left_scale: float = 1.0
    right_scale: float = 1.0
    ff: int = 0                                 # 0: no feed-forward
    ff_limit: float = 0.0


@dataclass(frozen=True)
class RudilixConfig:
    architecture: str
    vocab_size: int
    hidden_size: int
    residual_mult: float
    norm_eps: float
    layers: Tuple[RudilixLayer, ...]
    max_position_embeddings: int = 0
    eos_token_id: Optional[int] = None

    # ---------------------------------------------------------------- parsing
    @classmethod
    def from_dict(cls, data: Mapping[str, Any]) -> "RudilixConfig":
        entries = data.get("layers")
        if not isinstance(entries, (list, tuple)) or not entries:
            raise ConfigError("config.json has no layers list")
        layers = []
        for i, entry in enumerate(entries):
            where = f"layers[{i}]"
            if not isinstance(entry, Mapping) or entry.get("type") not in LAYER_TYPES:
                raise ConfigError(f"{where}.type must be one of {', '.join(LAYER_TYPES)}, got "
                                  f"{entry.get('type') if isinstance(entry, Mapping) else entry!r}")
            kind = entry["type"]
            m = _mapping(entry, "mixer", where)
            kw: Dict[str, Any] = {}
            if kind == "mamba2":
                kw["ssd"] = SsdSizes.read(m, where)
            elif kind == "channel_delta":
                kw["delta"] = DeltaSizes.read(m, where)
            else:
                kw["attention"] = AttentionSizes.read(_mapping(m, "left", where + ".mixer"),
                                                      where + ".mixer.left")
                kw["delta"] = DeltaSizes.read(_mapping(m, "right", where + ".mixer"),
                                              where + ".mixer.right")
                kw["left_scale"] = read_float(m, ["left_scale"], default=1.0)
                kw["right_scale"] = read_float(m, ["right_scale"], default=1.0)
            mlp = entry.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, Mapping) or mlp.get("kind", "dense") != "dense":
                    raise ConfigError(f"{where}.mlp must be null or a dense feed-forward")
                kw["ff"] = read_int(mlp, ["ff"], minimum=1)
                kw["ff_limit"] = read_float(mlp, ["limit"], default=0.0)
            layers.append(RudilixLayer(kind, **kw))
        eos = data.get("eos_token_id")
        return cls(
            architecture=str(data.get("architecture") or "Rudilix"),
            vocab_size=read_int(data, ["vocab"], minimum=1),
            hidden_size=read_int(data, ["width"], minimum=1),
            residual_mult=read_float(data, ["residual_mult"], default=1.0),
            norm_eps=read_float(_mapping(data, "norm", "config.json"), ["eps"], positive=True),
            layers=tuple(layers),
            max_position_embeddings=read_int(data, ["max_position_embeddings"], default=0, minimum=0),
            eos_token_id=eos if isinstance(eos, int) and not isinstance(eos, bool) else None)

    def to_dict(self) -> dict:
        layers = []
        for layer in self.layers:
            if layer.type == "mamba2":
                mixer = layer.ssd.to_dict()
            elif layer.type == "channel_delta":
                mixer = layer.delta.to_dict()
            else:
                mixer = {"left": layer.attention.to_dict(), "left_scale": layer.left_scale,
                         "right": layer.delta.to_dict(), "right_scale": layer.right_scale}
            if layer.type != "mamba2":
                d = mixer["right"] if layer.type == "parallel" else mixer
                d.update(decay_rank=layer.delta.decay_rank, gate_rank=layer.delta.gate_rank)
            mlp = {"kind": "dense", "ff": layer.ff, "limit": layer.ff_limit} if layer.ff else None
            layers.append({"type": layer.type, "mixer": mixer, "mlp": mlp})
        out = {"architecture": self.architecture, "vocab": self.vocab_size,
               "width": self.hidden_size, "residual_mult": self.residual_mult,
               "norm": {"eps": self.norm_eps}, "layers": layers}
        if self.max_position_embeddings:
            out["max_position_embeddings"] = self.max_position_embeddings
        if self.eos_token_id is not None:
            out["eos_token_id"] = self.eos_token_id
        return out

    # ---------------------------------------------- sizes only the tensors give
    def with_shapes(self, shape_of: Callable[[str], Optional[Tuple[int, ...]]]) -> "RudilixConfig":
        """The configuration with the delta mixers' low-rank widths taken from a
        checkpoint: ``shape_of(name)`` is a stored tensor's shape, or None."""
        layers = []
        for i, layer in enumerate(self.layers):
            if layer.delta is not None:
                p = f"l{i}.mix." + ("right." if layer.type == "parallel" else "")
                a, g = shape_of(p + "a1"), shape_of(p + "g1")
                layer = replace(layer, delta=replace(
                    layer.delta,
                    decay_rank=int(a[0]) if a else layer.delta.decay_rank,
                    gate_rank=int(g[0]) if g else layer.delta.gate_rank))
            layers.append(layer)
        return replace(self, layers=tuple(layers))

    # ------------------------------------------------------------ translation
    def _delta_spec(self, s: DeltaSizes, p: str) -> PartSpec:
        return PartSpec(
            "gated_delta",
            {"hidden_size": self.hidden_size, "num_heads": s.heads, "num_kv_heads": s.kv_heads,
             "head_dim": s.dim, "value_dim": s.vdim, "kernel_size": s.conv,
             "decay_rank": s.decay_rank, "gate_rank": s.gate_rank, "norm_eps": self.norm_eps},
            {"q_proj.weight": (p + "q",), "k_proj.weight": (p + "k",), "v_proj.weight": (p + "v",),
             "q_conv.weight": (p + "q.conv",), "k_conv.weight": (p + "k.conv",),
             "v_conv.weight": (p + "v.conv",), "beta_proj.weight": (p + "b",),
             "A_log": (p + "A_log",), "dt_bias": (p + "dt_bias",),
             "decay_down.weight": (p + "a1",), "decay_up.weight": (p + "a2",),
             "gate_down.weight": (p + "g1",), "gate_up.weight": (p + "g2",),
             "norm.weight": (p + "norm",), "out_proj.weight": (p + "o",)})

    def _attention_spec(self, s: AttentionSizes, p: str) -> PartSpec:
        rope = None
        if s.rot_dims:
            rope = PartSpec("rope", {"head_dim": s.dim, "rotary_dim": s.rot_dims,
                                     "theta": s.rot_base, "pairing": "adjacent"})
        return PartSpec(
            "gqa_attention",
            {"hidden_size": self.hidden_size, "num_heads": s.heads, "num_kv_heads": s.kv_heads,
             "head_dim": s.dim, "value_dim": s.vdim, "qk_norm": True, "norm_eps": self.norm_eps,
             "window": s.window, "softmax_scale": s.scale, "bias": "qkv", "gate": "head",
             "position": rope},
            {"q_proj.weight": (p + "q",), "k_proj.weight": (p + "k",), "v_proj.weight": (p + "v",),
             "q_proj.bias": (p + "q.b",), "k_proj.bias": (p + "k.b",), "v_proj.bias": (p + "v.b",),
             "q_norm.weight": (p + "q.norm",), "k_norm.weight": (p + "k.norm",),
             "gate_proj.weight": (p + "g",), "out_proj.weight": (p + "o",)})

    def _ssd_spec(self, s: SsdSizes, p: str) -> PartSpec:
        return PartSpec(
            "ssd",
            {"hidden_size": self.hidden_size, "num_heads": s.heads, "head_dim": s.vdim,
             "state_size": s.state, "groups": s.groups, "norm_groups": s.norm_groups,
             "kernel_size": s.conv, "norm_eps": self.norm_eps},
            {"in_proj.weight": (p + "in",), "conv.weight": (p + "conv",),
             "conv.bias": (p + "conv.b",), "dt_bias": (p + "dt_bias",), "A_log": (p + "A_log",),
             "D": (p + "D",), "norm.weight": (p + "norm",), "out_proj.weight": (p + "o",)})

    def _norm_spec(self, name: str) -> PartSpec:
        return PartSpec("rms_norm", {"width": self.hidden_size, "eps": self.norm_eps,
                                     "weight_offset": 1.0}, {"weight": (name,)})

    def to_spec(self) -> ModelSpec:
        H = self.hidden_size
        layers = []
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            parts: Dict[str, PartSpec] = {"mixer_norm": self._norm_spec(p + "norm1")}
            params: Dict[str, Any] = {"residual_scale": self.residual_mult}
            if layer.type == "parallel":
                parts["left"] = self._attention_spec(layer.attention, p + "mix.left.")
                parts["right"] = self._delta_spec(layer.delta, p + "mix.right.")
                params["mixer_scales"] = (layer.left_scale, layer.right_scale)
                kind = "scaled_residual_parallel"
            else:
                parts["mixer"] = self._ssd_spec(layer.ssd, p + "mix.") if layer.type == "mamba2" \
                    else self._delta_spec(layer.delta, p + "mix.")
                kind = "scaled_residual"
            if layer.ff:
                parts["feed_forward_norm"] = self._norm_spec(p + "norm2")
                parts["feed_forward"] = PartSpec(
                    "clamped_glu",
                    {"hidden_size": H, "intermediate_size": layer.ff, "limit": layer.ff_limit,
                     "alpha": GLU_ALPHA, "up_offset": GLU_UP_OFFSET},
                    {"gate.weight": (p + "mlp.gate",), "up.weight": (p + "mlp.up",),
                     "down.weight": (p + "mlp.down",)})
            else:
                kind += "_no_ff"
            layers.append(LayerSpec(parts, kind, params))
        embedding = PartSpec("token_embedding", {"vocab_size": self.vocab_size, "hidden_size": H},
                             {"weight": ("embed",)})
        lm_head = PartSpec("linear_head", {"vocab_size": self.vocab_size, "hidden_size": H,
                                           "tied": False}, {"weight": ("head",)})
        schedule = tuple(LayerCall(i) for i in range(len(self.layers)))
        # a layer without a feed-forward may still carry its second norm; it is not read
        ignored = tuple(f"l{i}.norm2" for i, layer in enumerate(self.layers) if not layer.ff)
        return ModelSpec(self.architecture, H, self.vocab_size, embedding, tuple(layers), schedule,
                         self._norm_spec("final.norm"), lm_head, self.max_position_embeddings,
                         ignored)
