"""Typed configuration of Ranesun, a decoder whose layers mix tokens in one of two ways,
listed layer by layer in config.json:

  ``retention``  linear attention with one fixed decay a head and rotary positions
                 (``parts/recurrent.py``, ``retention``)
  ``attention``  causal grouped-query attention whose values are its keys, without
                 rotation, with a temperature on the queries by position, capped scores
                 and a sink a head in the softmax (``gqa_attention`` with ``values="keys"``,
                 ``softcap``, ``sink`` and ``query_temperature``)

Each layer is pre-norm with layer norms (weight and bias).  Its feed-forward (``mlp``,
may be absent) is either dense, a gated unit with the tanh form of gelu on the gate
(``swiglu`` with ``activation="gelu_tanh"``), or a set of small experts that a table picks
by token id (``table_experts``).  A span of layers (``loop``: ``start``, ``stop``, ``times``) may
run several times in a row with the same weights, every pass with caches and states of
its own; before each pass the stream takes a row of ``loop.step`` and, from the second
pass on, the embedding's output once more (``parts/stream.py``, ``pass_offset``).  The head
is the embedding table, its logits times ``logit_scale``.

config.json keys: ``architecture``, ``vocab``, ``width``, ``norm.eps``, ``logit_scale``,
``loop``, ``layers[i] = {type, mixer, mlp}``; tensor names: ``embed``, ``loop.step``,
``l<i>.norm1`` (+ ``.b``), ``l<i>.norm2`` (+ ``.b``), ``l<i>.mix.*``, ``l<i>.mlp.*``,
``final.norm`` (+ ``.b``).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Mapping, Optional, Tuple

from .fields import read_float, read_int
from .spec import ConfigError, LayerCall, LayerSpec, ModelSpec, PartSpec, StreamStep

LAYER_TYPES = ("retention", "attention")
# constants of the design
DENSE_ACTIVATION = "gelu_tanh"      # on the gate of a dense feed-forward
EXPERT_ACTIVATION = "relu2"         # inside an expert


def _mapping(data: Mapping[str, Any], key: str, where: str) -> Mapping[str, Any]:
    value = data.get(key)
    if not isinstance(value, Mapping):
        raise ConfigError(f"{where} has no {key} object")
    return value


@dataclass(frozen=True)
class RetentionSizes:
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]
    rot_dims: int                    # 0: no rotation
    rot_base: float

    @classmethod
    def read(cls, m: Mapping[str, Any], where: str) -> "RetentionSizes":
        heads = read_int(m, ["heads"], minimum=1)
        dim = read_int(m, ["dim"], minimum=1)
        decay = m.get("decay")
        if not isinstance(decay, (list, tuple)) or len(decay) != heads or not all(
                isinstance(x, (int, float)) and not isinstance(x, bool) for x in decay):
            raise ConfigError(f"{where}.decay must list one number for each of the {heads} heads")
        rot = m.get("rot")
        dims, base = 0, 10000.0
        if isinstance(rot, Mapping):
            dims = read_int(rot, ["dims"], minimum=2)
            base = read_float(rot, ["base"], positive=True)
            if dims % 2 or dims > dim:
                raise ConfigError(f"{where}: rot.dims {dims} must be even and at most dim {dim}")
        return cls(heads, dim, read_int(m, ["vdim"], default=dim, minimum=1),
                   tuple(float(x) for x in decay), dims, base)

    def to_dict(self) -> dict:
        out: Dict[str, Any] = {"heads": self.heads, "dim": self.dim, "vdim": self.vdim,
                               "decay": list(self.decay)}
        if self.rot_dims:
            out["rot"] = {"dims": self.rot_dims, "base": self.rot_base}
        return out


@dataclass(frozen=True)
class SinkAttentionSizes:
    heads: int
    kv_heads: int
    dim: int
    scale: float
    softcap: float                   # 0: no cap
    temp_coef: float
    temp_every: int                  # 0: no temperature

    @classmethod
    def read(cls, m: Mapping[str, Any], where: str) -> "SinkAttentionSizes":
        heads = read_int(m, ["heads"], minimum=1)
        kv = read_int(m, ["kv_heads"], default=heads, minimum=1)
        if heads % kv:
            raise ConfigError(f"{where}: {heads} heads do not divide into {kv} kv_heads")
        dim = read_int(m, ["dim"], minimum=1)
        vdim = read_int(m, ["vdim"], default=dim, minimum=1)
        if vdim != dim:
            raise ConfigError(f"{where}: the values are the keys, so vdim {vdim} must equal dim {dim}")
        temp = m.get("q_temp")
        coef, every = 0.0, 0
        if isinstance(temp, Mapping):
            coef = read_float(temp, ["coef"])
            every = read_int(temp, ["every"], minimum=1)
        return cls(heads, kv, dim, read_float(m, ["scale"], default=dim ** -0.5, positive=True),
                   read_float(m, ["softcap"], default=0.0), coef, every)

    def to_dict(self) -> dict:
        out: Dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim,
                               "vdim": self.dim, "scale": self.scale}
        if self.softcap:
            out["softcap"] = self.softcap
        if self.temp_every:
            out["q_temp"] = {"coef": self.temp_coef, "every": self.temp_every}
        return out


@dataclass(frozen=True)
class RanesunLayer:
    type: str
    retention: Optional[RetentionSizes] = None
    attention: Optional[SinkAttentionSizes] = None
    mlp: Optional[str] = None        # None, "dense" or "moe"
    ff: int = 0                      # of the dense feed-forward, or of one expert
    experts: int = 0
    top: int = 0


@dataclass(frozen=True)
class RanesunConfig:
    architecture: str
    vocab_size: int
    hidden_size: int
    norm_eps: float
    logit_scale: float
    layers: Tuple[RanesunLayer, ...]
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 0              # 0: no loop (and no ``loop.step`` tensor)
    max_position_embeddings: int = 0
    eos_token_id: Optional[int] = None

    # ---------------------------------------------------------------- parsing
    @classmethod
    def from_dict(cls, data: Mapping[str, Any]) -> "RanesunConfig":
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
            if kind == "retention":
                kw["retention"] = RetentionSizes.read(m, where + ".mixer")
            else:
                kw["attention"] = SinkAttentionSizes.read(m, where + ".mixer")
            mlp = entry.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, Mapping) or mlp.get("kind") not in ("dense", "moe"):
                    raise ConfigError(f"{where}.mlp must be null, or of kind dense or moe")
                kw["mlp"] = mlp["kind"]
                if mlp["kind"] == "dense":
                    kw["ff"] = read_int(mlp, ["ff"], minimum=1)
                else:
                    router = _mapping(mlp, "router", where + ".mlp")
                    kw["ff"] = read_int(_mapping(mlp, "expert", where + ".mlp"), ["ff"], minimum=1)
                    kw["experts"] = read_int(router, ["experts"], minimum=1)
                    kw["top"] = read_int(router, ["top"], minimum=1)
                    if kw["top"] > kw["experts"]:
                        raise ConfigError(f"{where}.mlp.router: top {kw['top']} of "
                                          f"{kw['experts']} experts")
            layers.append(RanesunLayer(kind, **kw))
        loop = data.get("loop")
        start = stop = times = 0
        if loop is not None:
            if not isinstance(loop, Mapping):
                raise ConfigError("loop must be an object with start, stop and times")
            start = read_int(loop, ["start"], minimum=0)
            stop = read_int(loop, ["stop"], minimum=0)
            times = read_int(loop, ["times"], minimum=1)
            if not start < stop <= len(layers):
                raise ConfigError(f"loop spans layers {start}..{stop - 1} of {len(layers)}")
        eos = data.get("eos_token_id")
        return cls(
            architecture=str(data.get("architecture") or "Ranesun"),
            vocab_size=read_int(data, ["vocab"], minimum=1),
            hidden_size=read_int(data, ["width"], minimum=1),
            norm_eps=read_float(_mapping(data, "norm", "config.json"), ["eps"], positive=True),
            logit_scale=read_float(data, ["logit_scale"], default=1.0),
            layers=tuple(layers), loop_start=start, loop_stop=stop, loop_times=times,
            max_position_embeddings=read_int(data, ["max_position_embeddings"], default=0, minimum=0),
            eos_token_id=eos if isinstance(eos, int) and not isinstance(eos, bool) else None)

    def to_dict(self) -> dict:
        layers = []
        for layer in self.layers:
            mixer = (layer.retention if layer.type == "retention" else layer.attention).to_dict()
            if layer.mlp == "dense":
                mlp: Any = {"kind": "dense", "ff": layer.ff}
            elif layer.mlp == "moe":
                mlp = {"kind": "moe", "expert": {"ff": layer.ff},
                       "router": {"experts": layer.experts, "top": layer.top}}
            else:
                mlp = None
            layers.append({"type": layer.type, "mixer": mixer, "mlp": mlp})
        out: Dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab_size,
                               "width": self.hidden_size, "norm": {"eps": self.norm_eps},
                               "logit_scale": self.logit_scale, "layers": layers}
        if self.loop_times:
            out["loop"] = {"start": self.loop_start, "stop": self.loop_stop,
                           "times": self.loop_times}
        if self.max_position_embeddings:
            out["max_position_embeddings"] = self.max_position_embeddings
        if self.eos_token_id is not None:
            out["eos_token_id"] = self.eos_token_id
        return out

    # ------------------------------------------------------------ translation
    def _norm_spec(self, name: str) -> PartSpec:
        return PartSpec("layer_norm", {"width": self.hidden_size, "eps": self.norm_eps},
                        {"weight": (name,), "bias": (name + ".b",)})

    def _retention_spec(self, s: RetentionSizes, p: str) -> PartSpec:
        rope = None
        if s.rot_dims:
            rope = PartSpec("rope", {"head_dim": s.dim, "rotary_dim": s.rot_dims,
                                     "theta": s.rot_base, "pairing": "half"})
        return PartSpec(
            "retention",
            {"hidden_size": self.hidden_size, "num_heads": s.heads, "head_dim": s.dim,
             "value_dim": s.vdim, "decay": s.decay, "norm_eps": self.norm_eps, "position": rope},
            {"q_proj.weight": (p + "q",), "k_proj.weight": (p + "k",), "v_proj.weight": (p + "v",),
             "gate_proj.weight": (p + "g",), "out_proj.weight": (p + "o",)})

    def _attention_spec(self, s: SinkAttentionSizes, p: str) -> PartSpec:
        return PartSpec(
            "gqa_attention",
            {"hidden_size": self.hidden_size, "num_heads": s.heads, "num_kv_heads": s.kv_heads,
             "head_dim": s.dim, "qk_norm": False, "window": 0, "softmax_scale": s.scale,
             "values": "keys", "softcap": s.softcap, "sink": True,
             "query_temperature": (s.temp_coef, s.temp_every) if s.temp_every else None,
             "position": None},
            {"q_proj.weight": (p + "q",), "k_proj.weight": (p + "k",), "sink": (p + "sink",),
             "out_proj.weight": (p + "o",)})

    def _mlp_spec(self, layer: RanesunLayer, p: str) -> PartSpec:
        H = self.hidden_size
        if layer.mlp == "dense":
            return PartSpec("swiglu", {"hidden_size": H, "intermediate_size": layer.ff,
                                       "activation": DENSE_ACTIVATION},
                            {"gate.weight": (p + "gate",), "up.weight": (p + "up",),
                             "down.weight": (p + "down",)})
        names = {"table": (p + "table",)}
        for e in range(layer.experts):
            names[f"experts.{e}.up.weight"] = (f"{p}e{e}.up",)
            names[f"experts.{e}.down.weight"] = (f"{p}e{e}.down",)
        return PartSpec("table_experts",
                        {"hidden_size": H, "intermediate_size": layer.ff, "experts": layer.experts,
                         "top": layer.top, "vocab_size": self.vocab_size,
                         "activation": EXPERT_ACTIVATION}, names)

    def run_order(self) -> Tuple[LayerCall, ...]:
        """Every layer once, the loop's span ``times`` times in a row; each time a layer runs
        it has a cache entry of its own, and the first layer of every pass is preceded by
        the pass's offset."""
        n = len(self.layers)
        if not self.loop_times:
            return tuple(LayerCall(i) for i in range(n))
        calls = [LayerCall(i) for i in range(self.loop_start)]
        for t in range(self.loop_times):
            for i in range(self.loop_start, self.loop_stop):
                before = StreamStep(0, {"row": t, "add_origin": t > 0}) \
                    if i == self.loop_start else None
                calls.append(LayerCall(i, before=before))
        calls += [LayerCall(i) for i in range(self.loop_stop, n)]
        return tuple(calls)

    def to_spec(self) -> ModelSpec:
        H = self.hidden_size
        layers = []
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            parts: Dict[str, PartSpec] = {"mixer_norm": self._norm_spec(p + "norm1")}
            parts["mixer"] = self._retention_spec(layer.retention, p + "mix.") \
                if layer.type == "retention" else self._attention_spec(layer.attention, p + "mix.")
            kind = "pre_norm_residual"
            if layer.mlp:
                parts["feed_forward_norm"] = self._norm_spec(p + "norm2")
                parts["feed_forward"] = self._mlp_spec(layer, p + "mlp.")
            else:
                kind = "pre_norm_residual_no_ff"
            layers.append(LayerSpec(parts, kind))
        embedding = PartSpec("token_embedding", {"vocab_size": self.vocab_size, "hidden_size": H},
                             {"weight": ("embed",)})
        lm_head = PartSpec("linear_head", {"vocab_size": self.vocab_size, "hidden_size": H,
                                           "tied": True, "logit_scale": self.logit_scale}, {})
        stream_parts = ()
        if self.loop_times:
            stream_parts = (PartSpec("pass_offset", {"passes": self.loop_times, "width": H},
                                     {"table": ("loop.step",)}),)
        # a layer without a feed-forward may still carry its second norm; it is not read
        ignored = tuple(name for i, layer in enumerate(self.layers) if not layer.mlp
                        for name in (f"l{i}.norm2", f"l{i}.norm2.b"))
        return ModelSpec(self.architecture, H, self.vocab_size, embedding, tuple(layers),
                         self.run_order(), self._norm_spec("final.norm"), lm_head,
                         self.max_position_embeddings, ignored, stream_parts)
