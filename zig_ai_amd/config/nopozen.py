"""Typed configuration of Nopozen, a decoder whose layers mix tokens in one of three ways,
listed layer by layer in config.json:

  ``lightning``    lightning attention: linear attention with one fixed decay a head, silu on
                   q, k and v, one norm over all heads and a sigmoid gate an element
                   (``retention`` with ``activation="silu"``, ``key_scale=1``,
                   ``output_norm="all"``, ``gate="sigmoid"``)
  ``attention``    grouped-query attention with biases, a per-head norm of q and k, rotary
                   positions in halves with frequencies rescaled by wavelength, a mask in
                   chunks and a sigmoid gate a head (``gqa_attention`` with ``bias``,
                   ``qk_norm``, ``chunk``, ``gate="head"``)
  ``attention_2``  grouped-query attention without biases whose q, k and v pass a short
                   causal convolution over time, partial rotation, every earlier key, a sink
                   of score zero in the softmax and a sigmoid gate an element
                   (``gqa_attention`` with ``conv``, ``sink_value=0``, ``gate="element"``)

A layer is parallel: one RMS norm, and mixer and feed-forward both on its output
(``parallel_residual``).  The feed-forward (``mlp``, may be absent) is dense without a gate,
``W_down relu(W_up h)^2`` (``activated_mlp``), or a set of small gated experts of which a
router with a bias picks ``top``, weighted by the softmax over the chosen logits
(``routed_experts`` with ``router_bias`` and ``renormalize``).  A span of layers (``loop``:
``start``, ``stop``, ``times``) may run several times in a row with the same weights, every
pass with caches and states of its own; each pass starts from ``loop.in`` applied to the
stream and the embedding's output side by side (``pass_mix``).  The head is a matrix of its
own.

config.json keys: ``architecture``, ``vocab``, ``width``, ``norm.eps``, ``loop``,
``layers[i] = {type, mixer, mlp}``; tensor names: ``embed``, ``loop.in``, ``l<i>.norm1``,
``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``, ``head``.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Mapping, Optional, Tuple

from .fields import read_float, read_int
from .spec import ConfigError, LayerCall, LayerSpec, ModelSpec, PartSpec, StreamStep

LAYER_TYPES = ("lightning", "attention", "attention_2")
# constants of the design
DENSE_ACTIVATION = "relu2"          # of a dense feed-forward (no gate)
EXPERT_ACTIVATION = "silu"          # on the gate inside an expert
LIGHTNING_ACTIVATION = "silu"       # on q, k and v of the lightning mixer
LIGHTNING_KEY_SCALE = 1.0           # the lightning mixer's keys are not scaled
SINK_SCORE = 0.0                    # attention_2: the softmax's denominator takes exp(0) more


def _mapping(data: Mapping[str, Any], key: str, where: str) -> Mapping[str, Any]:
    value = data.get(key)
    if not isinstance(value, Mapping):
        raise ConfigError(f"{where} has no {key} object")
    return value


@dataclass(frozen=True)
class RotarySizes:
    dims: int
    base: float
    scaling: Optional[Tuple[float, float, float, float]] = None   # factor, low, high, original

    @classmethod
    def read(cls, m: Mapping[str, Any], dim: int, where: str) -> "RotarySizes":
        if m.get("rot") is None:
            return cls(0, 10000.0)                     # no rotation at all
        rot = _mapping(m, "rot", where)
        dims = read_int(rot, ["dims"], minimum=0)
        if dims == 0:
            return cls(0, read_float(rot, ["base"], default=10000.0, positive=True))
        if dims % 2 or dims > dim:
            raise ConfigError(f"{where}: rot.dims {dims} must be even and at most dim {dim}")
        scaling = None
        sc = rot.get("scaling")
        if sc is not None:
            if not isinstance(sc, Mapping):
                raise ConfigError(f"{where}.rot.scaling must be an object")
            scaling = (read_float(sc, ["factor"], positive=True), read_float(sc, ["low"]),
                       read_float(sc, ["high"]), read_float(sc, ["original"], positive=True))
            if not scaling[2] > scaling[1]:
                raise ConfigError(f"{where}.rot.scaling: high must exceed low")
        return cls(dims, read_float(rot, ["base"], positive=True), scaling)

    def to_dict(self) -> dict:
        out: Dict[str, Any] = {"dims": self.dims, "base": self.base}
        if self.scaling:
            out["scaling"] = dict(zip(("factor", "low", "high", "original"), self.scaling))
        return out

    def spec(self, head_dim: int) -> Optional[PartSpec]:
        if not self.dims:
            return None
        params: Dict[str, Any] = {"head_dim": head_dim, "rotary_dim": self.dims,
                                  "theta": self.base, "pairing": "half"}
        if self.scaling:
            params["scaling"] = dict(zip(("factor", "low", "high", "original"), self.scaling))
        return PartSpec("rope", params)


@dataclass(frozen=True)
class LightningSizes:
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]

    @classmethod
    def read(cls, m: Mapping[str, Any], where: str) -> "LightningSizes":
        heads = read_int(m, ["heads"], minimum=1)
        dim = read_int(m, ["dim"], minimum=1)
        decay = m.get("decay")
        if not isinstance(decay, (list, tuple)) or len(decay) != heads or not all(
                isinstance(x, (int, float)) and not isinstance(x, bool) for x in decay):
            raise ConfigError(f"{where}.decay must list one number for each of the {heads} heads")
        return cls(heads, dim, read_int(m, ["vdim"], default=dim, minimum=1),
                   tuple(float(x) for x in decay))

    def to_dict(self) -> dict:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "decay": list(self.decay)}


@dataclass(frozen=True)
class AttentionSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: RotarySizes
    chunk: int = 0                   # attention: mask.size (0: every earlier key)
    conv: int = 0                    # attention_2: taps of the convolution over time

    @classmethod
    def read(cls, m: Mapping[str, Any], kind: str, where: str) -> "AttentionSizes":
        heads = read_int(m, ["heads"], minimum=1)
        kv = read_int(m, ["kv_heads"], default=heads, minimum=1)
        if heads % kv:
            raise ConfigError(f"{where}: {heads} heads do not divide into {kv} kv_heads")
        dim = read_int(m, ["dim"], minimum=1)
        chunk = conv = 0
        if kind == "attention":
            mask = m.get("mask")
            if mask is not None:
                if not isinstance(mask, Mapping):
                    raise ConfigError(f"{where}.mask must be an object with size")
                chunk = read_int(mask, ["size"], minimum=1)
        else:
            conv = read_int(m, ["conv"], minimum=1)
        return cls(heads, kv, dim, read_int(m, ["vdim"], default=dim, minimum=1),
                   read_float(m, ["scale"], default=dim ** -0.5, positive=True),
                   RotarySizes.read(m, dim, where), chunk, conv)

    def to_dict(self) -> dict:
        out: Dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim,
                               "vdim": self.vdim, "scale": self.scale}
        if self.rot.dims:
            out["rot"] = self.rot.to_dict()
        if self.chunk:
            out["mask"] = {"size": self.chunk}
        if self.conv:
            out["conv"] = self.conv
        return out


@dataclass(frozen=True)
class NopozenLayer:
    type: str
    lightning: Optional[LightningSizes] = None
    attention: Optional[AttentionSizes] = None
    mlp: Optional[str] = None        # None, "dense" or "moe"
    ff: int = 0                      # of the dense feed-forward, or of one expert
    experts: int = 0
    top: int = 0


@dataclass(frozen=True)
class NopozenConfig:
    architecture: str
    vocab_size: int
    hidden_size: int
    norm_eps: float
    layers: Tuple[NopozenLayer, ...]
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 0              # 0: no loop (and no ``loop.in`` tensor)
    max_position_embeddings: int = 0
    eos_token_id: Optional[int] = None

    # ---------------------------------------------------------------- parsing
    @classmethod
    def from_dict(cls, data: Mapping[str, Any]) -> "NopozenConfig":
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
            if kind == "lightning":
                kw["lightning"] = LightningSizes.read(m, where + ".mixer")
            else:
                kw["attention"] = AttentionSizes.read(m, kind, where + ".mixer")
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
            layers.append(NopozenLayer(kind, **kw))
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
            architecture=str(data.get("architecture") or "Nopozen"),
            vocab_size=read_int(data, ["vocab"], minimum=1),
            hidden_size=read_int(data, ["width"], minimum=1),
            norm_eps=read_float(_mapping(data, "norm", "config.json"), ["eps"], positive=True),
            layers=tuple(layers), loop_start=start, loop_stop=stop, loop_times=times,
            max_position_embeddings=read_int(data, ["max_position_embeddings"], default=0, minimum=0),
            eos_token_id=eos if isinstance(eos, int) and not isinstance(eos, bool) else None)

    def to_dict(self) -> dict:
        layers = []
        for layer in self.layers:
            mixer = (layer.lightning if layer.type == "lightning" else layer.attention).to_dict()
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
                               "layers": layers}
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
        return PartSpec("rms_norm", {"width": self.hidden_size, "eps": self.norm_eps},
                        {"weight": (name,)})

    def _lightning_spec(self, s: LightningSizes, p: str) -> PartSpec:
        return PartSpec(
            "retention",
            {"hidden_size": self.hidden_size, "num_heads": s.heads, "head_dim": s.dim,
             "value_dim": s.vdim, "decay": s.decay, "norm_eps": self.norm_eps, "position": None,
             "activation": LIGHTNING_ACTIVATION, "key_scale": LIGHTNING_KEY_SCALE,
             "output_norm": "all", "gate": "sigmoid"},
            {"q_proj.weight": (p + "q",), "k_proj.weight": (p + "k",), "v_proj.weight": (p + "v",),
             "gate_proj.weight": (p + "g",), "norm.weight": (p + "norm",),
             "out_proj.weight": (p + "o",)})

    def _attention_spec(self, kind: str, s: AttentionSizes, p: str) -> PartSpec:
        params: Dict[str, Any] = {
            "hidden_size": self.hidden_size, "num_heads": s.heads, "num_kv_heads": s.kv_heads,
            "head_dim": s.dim, "value_dim": s.vdim, "norm_eps": self.norm_eps, "window": 0,
            "softmax_scale": s.scale, "position": s.rot.spec(s.dim)}
        names = {"q_proj.weight": (p + "q",), "k_proj.weight": (p + "k",),
                 "v_proj.weight": (p + "v",), "gate_proj.weight": (p + "g",),
                 "out_proj.weight": (p + "o",)}
        if kind == "attention":
            params.update(qk_norm=True, bias=True, gate="head", chunk=s.chunk)
            names.update({"q_proj.bias": (p + "q.b",), "k_proj.bias": (p + "k.b",),
                          "v_proj.bias": (p + "v.b",), "out_proj.bias": (p + "o.b",),
                          "q_norm.weight": (p + "q.norm",), "k_norm.weight": (p + "k.norm",)})
        else:
            params.update(qk_norm=False, gate="element", conv=s.conv, sink_value=SINK_SCORE)
            names.update({"q_conv.weight": (p + "q.conv",), "k_conv.weight": (p + "k.conv",),
                          "v_conv.weight": (p + "v.conv",)})
        return PartSpec("gqa_attention", params, names)

    def _mlp_spec(self, layer: NopozenLayer, p: str) -> PartSpec:
        H = self.hidden_size
        if layer.mlp == "dense":
            return PartSpec("activated_mlp", {"hidden_size": H, "intermediate_size": layer.ff,
                                              "activation": DENSE_ACTIVATION},
                            {"up.weight": (p + "up",), "down.weight": (p + "down",)})
        names = {"router.weight": (p + "router",), "router.bias": (p + "router.b",)}
        for e in range(layer.experts):
            names[f"experts.{e}.gate.weight"] = (f"{p}e{e}.gate",)
            names[f"experts.{e}.up.weight"] = (f"{p}e{e}.up",)
            names[f"experts.{e}.down.weight"] = (f"{p}e{e}.down",)
        return PartSpec("routed_experts",
                        {"hidden_size": H, "intermediate_size": layer.ff, "experts": layer.experts,
                         "top": layer.top, "scores": "softmax", "renormalize": True,
                         "router_bias": True, "activation": EXPERT_ACTIVATION}, names)

    def run_order(self) -> Tuple[LayerCall, ...]:
        """Every layer once, the loop's span ``times`` times in a row; each time a layer runs
        it has a cache entry of its own, and the first layer of every pass (the first pass
        too) is preceded by the pass's projection."""
        n = len(self.layers)
        if not self.loop_times:
            return tuple(LayerCall(i) for i in range(n))
        calls = [LayerCall(i) for i in range(self.loop_start)]
        for _ in range(self.loop_times):
            for i in range(self.loop_start, self.loop_stop):
                calls.append(LayerCall(i, before=StreamStep(0) if i == self.loop_start else None))
        calls += [LayerCall(i) for i in range(self.loop_stop, n)]
        return tuple(calls)

    def to_spec(self) -> ModelSpec:
        H = self.hidden_size
        layers = []
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            parts: Dict[str, PartSpec] = {"norm": self._norm_spec(p + "norm1")}
            if layer.type == "lightning":
                parts["mixer"] = self._lightning_spec(layer.lightning, p + "mix.")
            else:
                parts["mixer"] = self._attention_spec(layer.type, layer.attention, p + "mix.")
            kind = "parallel_residual_no_ff"
            if layer.mlp:
                parts["feed_forward"] = self._mlp_spec(layer, p + "mlp.")
                kind = "parallel_residual"
            layers.append(LayerSpec(parts, kind))
        embedding = PartSpec("token_embedding", {"vocab_size": self.vocab_size, "hidden_size": H},
                             {"weight": ("embed",)})
        lm_head = PartSpec("linear_head", {"vocab_size": self.vocab_size, "hidden_size": H,
                                           "tied": False}, {"weight": ("head",)})
        stream_parts = ()
        if self.loop_times:
            stream_parts = (PartSpec("pass_mix", {"width": H}, {"weight": ("loop.in",)}),)
        return ModelSpec(self.architecture, H, self.vocab_size, embedding, tuple(layers),
                         self.run_order(), self._norm_spec("final.norm"), lm_head,
                         self.max_position_embeddings, (), stream_parts)
