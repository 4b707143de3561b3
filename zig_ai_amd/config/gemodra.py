"""Typed configuration of Gemodra, a decoder whose layers all mix tokens by attention over
one small latent vector a token, in one of two forms listed layer by layer in config.json:

  ``latent_attention``    queries through a normed latent; keys and values of every head are
                          expansions of one normed latent a token, beside a rotated key part
                          that all heads share (rotary positions in adjacent pairs); a sink a
                          head in the softmax; an output gate an element
  ``latent_attention_2``  the same without positions and without the rotated part, with an
                          output gate a head

(both ``parts/latent_attention.py``, ``latent_attention``).  Each layer is pre-norm with RMS
norms and a weight ``residual_mult`` on what enters the stream (``scaled_residual``).  Its
feed-forward (``mlp``, may be absent) is a set of small gated experts chosen by a router
(``routed_experts``): softmax scores, a correction added for the choice only, the choice
limited to the best groups of neighbouring experts, identity experts that hand the input
on, and a shared expert with a gate a token.  After the feed-forward every layer takes an
input of its own from the tokens themselves (``token_side``: a slice of a second embedding
table, gated by the stream, projected, normed).  The embedding's output is normed, the head
is a matrix of its own and its logits are capped (``cap * tanh(logits / cap)``).

config.json keys: ``architecture``, ``vocab``, ``width``, ``norm.eps``, ``residual_mult``,
``logit_softcap``, ``token_side.dim``, ``layers[i] = {type, mixer, mlp}``; tensor names:
``embed``, ``embed.norm``, ``side.embed``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.*``,
``l<i>.mlp.*``, ``l<i>.side.*``, ``final.norm``, ``head``.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Mapping, Optional, Tuple

from .fields import read_float, read_int
from .spec import ConfigError, LayerCall, LayerSpec, ModelSpec, PartSpec, StreamStep

LAYER_TYPES = ("latent_attention", "latent_attention_2")
# constants of the design
EXPERT_ACTIVATION = "silu"          # on the gate of an expert and of the shared expert
SIDE_ACTIVATION = "gelu_tanh"       # on the gate of the per-layer token input
ROTARY_PAIRING = "adjacent"         # element 2i with 2i + 1
# which gate each form has on the attention's output
OUTPUT_GATE = {"latent_attention": "element", "latent_attention_2": "head"}


def _mapping(data: Mapping[str, Any], key: str, where: str) -> Mapping[str, Any]:
    value = data.get(key)
    if not isinstance(value, Mapping):
        raise ConfigError(f"{where} has no {key} object")
    return value


@dataclass(frozen=True)
class LatentSizes:
    heads: int
    dim: int                         # unrotated query/key elements a head
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    rot_dim: int = 0                 # rotated query/key elements (0: no positions)
    rot_dims: int = 0                # how many of them the rotation turns
    rot_base: float = 10000.0

    @classmethod
    def read(cls, m: Mapping[str, Any], where: str, rotated: bool) -> "LatentSizes":
        heads = read_int(m, ["heads"], minimum=1)
        dim = read_int(m, ["dim"], minimum=1)
        rot_dim = rot_dims = 0
        base = 10000.0
        if rotated:
            rot_dim = read_int(m, ["rot_dim"], minimum=2)
            rot = _mapping(m, "rot", where)
            rot_dims = read_int(rot, ["dims"], minimum=2)
            base = read_float(rot, ["base"], positive=True)
            if rot_dims % 2 or rot_dims > rot_dim:
                raise ConfigError(f"{where}: rot.dims {rot_dims} must be even and at most rot_dim "
                                  f"{rot_dim}")
        elif m.get("rot_dim"):
            raise ConfigError(f"{where}: this form of the mixer has no rotated part")
        return cls(heads, dim, read_int(m, ["vdim"], default=dim, minimum=1),
                   read_int(m, ["kv_rank"], minimum=1), read_int(m, ["q_rank"], minimum=1),
                   read_float(m, ["scale"], default=(dim + rot_dim) ** -0.5, positive=True),
                   rot_dim, rot_dims, base)

    def to_dict(self) -> dict:
        out: Dict[str, Any] = {"heads": self.heads, "dim": self.dim, "vdim": self.vdim,
                               "kv_rank": self.kv_rank, "q_rank": self.q_rank, "scale": self.scale}
        if self.rot_dim:
            out["rot_dim"] = self.rot_dim
            out["rot"] = {"dims": self.rot_dims, "base": self.rot_base}
        return out


@dataclass(frozen=True)
class RouterSizes:
    experts: int                     # experts that have weights
    identity: int                    # router outputs beyond them that hand the input on
    top: int
    scale: float
    groups: int = 0                  # 0: the choice is not limited to groups
    keep: int = 0
    ff: int = 0                      # width inside an expert
    shared_ff: int = 0               # 0: no shared expert

    @classmethod
    def read(cls, mlp: Mapping[str, Any], where: str) -> "RouterSizes":
        router = _mapping(mlp, "router", where)
        experts = read_int(router, ["experts"], minimum=0)
        identity = read_int(router, ["identity"], default=0, minimum=0)
        total = experts + identity
        top = read_int(router, ["top"], minimum=1)
        if top > total:
            raise ConfigError(f"{where}.router: top {top} of {total} router outputs")
        groups = keep = 0
        g = router.get("groups")
        if g is not None:
            if not isinstance(g, Mapping):
                raise ConfigError(f"{where}.router.groups must be an object with count and keep")
            groups = read_int(g, ["count"], minimum=1)
            keep = read_int(g, ["keep"], minimum=1)
            if total % groups or keep > groups:
                raise ConfigError(f"{where}.router: {total} router outputs in {groups} groups, "
                                  f"{keep} kept")
            if keep * (total // groups) < top:
                raise ConfigError(f"{where}.router: {keep} groups of {total // groups} cannot "
                                  f"yield {top} experts")
        ff = read_int(_mapping(mlp, "expert", where), ["ff"], minimum=1) if experts else 0
        shared = mlp.get("shared")
        shared_ff = 0
        if shared is not None:
            if not isinstance(shared, Mapping):
                raise ConfigError(f"{where}.shared must be an object with ff, or null")
            shared_ff = read_int(shared, ["ff"], minimum=1)
        return cls(experts, identity, top, read_float(router, ["scale"], default=1.0), groups,
                   keep, ff, shared_ff)

    def to_dict(self) -> dict:
        router: Dict[str, Any] = {"experts": self.experts, "identity": self.identity,
                                  "top": self.top, "scale": self.scale}
        if self.groups:
            router["groups"] = {"count": self.groups, "keep": self.keep}
        out: Dict[str, Any] = {"kind": "moe", "router": router}
        if self.experts:
            out["expert"] = {"ff": self.ff}
        if self.shared_ff:
            out["shared"] = {"ff": self.shared_ff}
        return out


@dataclass(frozen=True)
class GemodraLayer:
    type: str
    mixer: LatentSizes
    mlp: Optional[RouterSizes] = None


@dataclass(frozen=True)
class GemodraConfig:
    architecture: str
    vocab_size: int
    hidden_size: int
    norm_eps: float
    residual_mult: float
    logit_softcap: float             # 0: none
    side_dim: int                    # 0: no per-layer token input
    layers: Tuple[GemodraLayer, ...]
    max_position_embeddings: int = 0
    eos_token_id: Optional[int] = None

    # ---------------------------------------------------------------- parsing
    @classmethod
    def from_dict(cls, data: Mapping[str, Any]) -> "GemodraConfig":
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
            mixer = LatentSizes.read(_mapping(entry, "mixer", where), where + ".mixer",
                                     rotated=kind == "latent_attention")
            mlp = entry.get("mlp")
            sizes = None
            if mlp is not None:
                if not isinstance(mlp, Mapping) or mlp.get("kind") != "moe":
                    raise ConfigError(f"{where}.mlp must be null or of kind moe")
                sizes = RouterSizes.read(mlp, where + ".mlp")
            layers.append(GemodraLayer(kind, mixer, sizes))
        side = data.get("token_side")
        side_dim = 0
        if side is not None:
            if not isinstance(side, Mapping):
                raise ConfigError("token_side must be an object with dim, or null")
            side_dim = read_int(side, ["dim"], minimum=1)
        eos = data.get("eos_token_id")
        return cls(
            architecture=str(data.get("architecture") or "Gemodra"),
            vocab_size=read_int(data, ["vocab"], minimum=1),
            hidden_size=read_int(data, ["width"], minimum=1),
            norm_eps=read_float(_mapping(data, "norm", "config.json"), ["eps"], positive=True),
            residual_mult=read_float(data, ["residual_mult"], default=1.0),
            logit_softcap=read_float(data, ["logit_softcap"], default=0.0),
            side_dim=side_dim, layers=tuple(layers),
            max_position_embeddings=read_int(data, ["max_position_embeddings"], default=0, minimum=0),
            eos_token_id=eos if isinstance(eos, int) and not isinstance(eos, bool) else None)

    def to_dict(self) -> dict:
        layers = [{"type": layer.type, "mixer": layer.mixer.to_dict(),
                   "mlp": layer.mlp.to_dict() if layer.mlp is not None else None}
                  for layer in self.layers]
        out: Dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab_size,
                               "width": self.hidden_size, "norm": {"eps": self.norm_eps},
                               "residual_mult": self.residual_mult, "layers": layers}
        if self.logit_softcap:
            out["logit_softcap"] = self.logit_softcap
        if self.side_dim:
            out["token_side"] = {"dim": self.side_dim}
        if self.max_position_embeddings:
            out["max_position_embeddings"] = self.max_position_embeddings
        if self.eos_token_id is not None:
            out["eos_token_id"] = self.eos_token_id
        return out

    # ------------------------------------------------------------ translation
    def _norm_spec(self, name: str) -> PartSpec:
        return PartSpec("rms_norm", {"width": self.hidden_size, "eps": self.norm_eps},
                        {"weight": (name,)})

    def _mixer_spec(self, kind: str, s: LatentSizes, p: str) -> PartSpec:
        rope = None
        if s.rot_dim:
            rope = PartSpec("rope", {"head_dim": s.rot_dim, "rotary_dim": s.rot_dims,
                                     "theta": s.rot_base, "pairing": ROTARY_PAIRING})
        return PartSpec(
            "latent_attention",
            {"hidden_size": self.hidden_size, "num_heads": s.heads, "head_dim": s.dim,
             "rotated_dim": s.rot_dim, "value_dim": s.vdim, "kv_rank": s.kv_rank,
             "q_rank": s.q_rank, "softmax_scale": s.scale, "norm_eps": self.norm_eps,
             "sink": True, "gate": OUTPUT_GATE[kind], "position": rope},
            {"q_down.weight": (p + "dq",), "q_norm.weight": (p + "dq.norm",),
             "q_up.weight": (p + "uq",), "kv_down.weight": (p + "dkv",),
             "kv_norm.weight": (p + "dkv.norm",), "k_up.weight": (p + "uk",),
             "v_up.weight": (p + "uv",), "sink": (p + "sink",), "gate_proj.weight": (p + "g",),
             "out_proj.weight": (p + "o",)})

    def _mlp_spec(self, s: RouterSizes, p: str) -> PartSpec:
        names = {"router.weight": (p + "router",), "correction": (p + "correction",)}
        for e in range(s.experts):
            for w in ("gate", "up", "down"):
                names[f"experts.{e}.{w}.weight"] = (f"{p}e{e}.{w}",)
        if s.shared_ff:
            for w in ("gate", "up", "down"):
                names[f"shared.{w}.weight"] = (f"{p}shared.{w}",)
            names["shared.token_gate.weight"] = (p + "shared.sg",)
        return PartSpec(
            "routed_experts",
            {"hidden_size": self.hidden_size, "intermediate_size": s.ff, "experts": s.experts,
             "identity_experts": s.identity, "top": s.top, "route_scale": s.scale,
             "groups": s.groups, "groups_kept": s.keep, "scores": "softmax", "correction": True,
             "renormalize": False, "shared_size": s.shared_ff, "shared_gate": bool(s.shared_ff),
             "activation": EXPERT_ACTIVATION}, names)

    def run_order(self) -> Tuple[LayerCall, ...]:
        """Every layer once; with a token input, each followed by its own."""
        if not self.side_dim:
            return tuple(LayerCall(i) for i in range(len(self.layers)))
        return tuple(LayerCall(i, after=StreamStep(0, {"layer": i}))
                     for i in range(len(self.layers)))

    def to_spec(self) -> ModelSpec:
        H = self.hidden_size
        layers = []
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            parts: Dict[str, PartSpec] = {"mixer_norm": self._norm_spec(p + "norm1"),
                                          "mixer": self._mixer_spec(layer.type, layer.mixer,
                                                                    p + "mix.")}
            kind = "scaled_residual_no_ff"
            if layer.mlp is not None:
                parts["feed_forward_norm"] = self._norm_spec(p + "norm2")
                parts["feed_forward"] = self._mlp_spec(layer.mlp, p + "mlp.")
                kind = "scaled_residual"
            layers.append(LayerSpec(parts, kind, {"residual_scale": self.residual_mult}))
        embedding = PartSpec("token_embedding",
                             {"vocab_size": self.vocab_size, "hidden_size": H, "norm": True,
                              "norm_eps": self.norm_eps},
                             {"weight": ("embed",), "norm.weight": ("embed.norm",)})
        lm_head = PartSpec("linear_head", {"vocab_size": self.vocab_size, "hidden_size": H,
                                           "tied": False, "softcap": self.logit_softcap},
                           {"weight": ("head",)})
        stream_parts = ()
        if self.side_dim:
            names = {"table": ("side.embed",)}
            for i in range(len(self.layers)):
                names[f"layers.{i}.gate.weight"] = (f"l{i}.side.gate",)
                names[f"layers.{i}.proj.weight"] = (f"l{i}.side.proj",)
                names[f"layers.{i}.norm.weight"] = (f"l{i}.side.norm",)
            stream_parts = (PartSpec(
                "token_side", {"layers": len(self.layers), "dim": self.side_dim, "width": H,
                               "vocab_size": self.vocab_size, "eps": self.norm_eps,
                               "scale": self.residual_mult, "activation": SIDE_ACTIVATION},
                names),)
        # a layer without a feed-forward may still carry its second norm; it is not read
        ignored = tuple(f"l{i}.norm2" for i, layer in enumerate(self.layers) if layer.mlp is None)
        return ModelSpec(self.architecture, H, self.vocab_size, embedding, tuple(layers),
                         self.run_order(), self._norm_spec("final.norm"), lm_head,
                         self.max_position_embeddings, ignored, stream_parts)
