"""Fazopel: a decoder whose config.json lists its layers one by one.  A layer's two halves read the residual stream as it
is and pass their outputs through a norm before they join it (parts/block.py, "prenorm" with the norm kind "none" in
front and output norms behind):

    x += norm1(mixer(x));   x += norm2(ff(x))                         plain RMSNorms with weights [width]

Two kinds of mixers:

  "lightning"   linear attention with a matrix state per head and a decay that is a constant of the head; q, k, v pass a
                silu, the heads' outputs are normed together and gated by a sigmoid (parts/recurrent.py)
  "attention"   grouped-query causal attention whose values are the key projections themselves (there is no value
                matrix); an RMSNorm over every query and key head, a rotation of the first rot.dims dimensions of a head
                in split-half pairs with the frequency scaling of long wavelengths, and one more term of score 0 in the
                softmax (parts/attention.py)

and two kinds of feed-forwards: "dense" (squared relu, no gate) and "moe" (gated experts with clamped arguments, chosen
by softmax score + a correction, weighted by the plain scores of the chosen over their sum times a constant; optionally a
shared expert with a sigmoid gate of one number per token; parts/moe.py); "mlp": null leaves the second half out.  A
layer with "weights_of": j has no tensors of its own: it runs layer j's weights with a cache or state of its own, which
the plan's schedule says by naming layer j twice.

config.json keys: architecture, vocab, width, norm.eps, layers[] = {type, mixer, mlp, weights_of?} with
  lightning mixer   {heads, dim, vdim, decay: [one per head]}
  attention mixer   {heads, kv_heads, dim, vdim, scale, rot: {base, dims, scaling: {factor, low, high, original}}}
  mlp               {kind: "dense", ff} | {kind: "moe", expert: {ff, limit}, router: {experts, top, scale},
                    shared: {ff, limit}} | null

Tensor names of the folder (linear weights [out, in]): embed, head, final.norm, and for layer i under l<i>.:
  norm1, norm2
  lightning:  mix.{q,k,v,g,o}, mix.norm
  attention:  mix.{q,k,o}, mix.q.norm, mix.k.norm
  dense:      mlp.{up,down}
  moe:        mlp.router, mlp.correction, mlp.e<n>.{gate,up,down}, mlp.shared.{gate,up,down,sg}
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple, Union

from ..engine.plan import LayerPlan, ModelPlan, ScheduleEntry
from ..parts.base import PartSpec
from .base import Architecture, ConfigError, _positive_int, register_architecture

NAME = "Fazopel"

# Constants of the design (the same in every model of it)
GATE_SLOPE = 1.702            # an expert's gate is g sigmoid(GATE_SLOPE g)
UP_SHIFT = 1.0                # and multiplies (u + UP_SHIFT)
WEIGHT_FLOOR = 1e-20          # joins the sum of the chosen scores that the weights are divided by


def _number(raw: dict, key: str, what: str, positive: bool = True) -> float:
    v = raw.get(key)
    if isinstance(v, bool) or not isinstance(v, (int, float)) or (positive and not v > 0):
        raise ConfigError(f"config.json: {what}.{key} must be a {'positive ' if positive else ''}number, got {v!r}")
    return float(v)


def _object(raw, what: str) -> dict:
    if not isinstance(raw, dict):
        raise ConfigError(f"config.json: {what} must be an object, got {raw!r}")
    return raw


@dataclass(frozen=True)
class LightningSizes:
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]

    def to_dict(self):
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "decay": list(self.decay)}


@dataclass(frozen=True)
class FrequencyScaling:
    factor: float
    low: float
    high: float
    original: float

    def to_dict(self):
        return {"factor": self.factor, "low": self.low, "high": self.high, "original": self.original}


@dataclass(frozen=True)
class SinkAttentionSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_base: float
    rot_dims: int               # 0: no rotation
    rot_scaling: Optional[FrequencyScaling] = None

    def to_dict(self):
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.rot_dims:
            d["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
            if self.rot_scaling is not None:
                d["rot"]["scaling"] = self.rot_scaling.to_dict()
        return d


@dataclass(frozen=True)
class DenseSizes:
    ff: int

    def to_dict(self):
        return {"kind": "dense", "ff": self.ff}


@dataclass(frozen=True)
class MoeSizes:
    experts: int
    top: int
    scale: float
    ff: int
    limit: float
    shared_ff: int = 0          # 0: no shared expert
    shared_limit: float = 0.0

    def to_dict(self):
        d = {"kind": "moe", "expert": {"ff": self.ff, "limit": self.limit},
             "router": {"experts": self.experts, "top": self.top, "scale": self.scale}}
        if self.shared_ff:
            d["shared"] = {"ff": self.shared_ff, "limit": self.shared_limit}
        return d


@dataclass(frozen=True)
class FazopelLayer:
    type: str                                                   # "lightning" | "attention"
    mixer: Union[LightningSizes, SinkAttentionSizes]
    mlp: Union[DenseSizes, MoeSizes, None]
    weights_of: Optional[int] = None

    def to_dict(self):
        d = {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}
        if self.weights_of is not None:
            d["weights_of"] = self.weights_of
        return d


@dataclass(frozen=True)
class FazopelConfig:
    vocab: int
    width: int
    eps: float
    layers: Tuple[FazopelLayer, ...]

    MIXER_TYPES = ("lightning", "attention")
    MLP_KINDS = ("dense", "moe")

    @staticmethod
    def _mixer(kind: str, raw, where: str):
        m = _object(raw, where + ".mixer")
        heads, dim = _positive_int(m, "heads"), _positive_int(m, "dim")
        vdim = _positive_int(m, "vdim", dim)
        if kind == "lightning":
            decay = m.get("decay")
            if (not isinstance(decay, list) or len(decay) != heads
                    or any(isinstance(d, bool) or not isinstance(d, (int, float)) or not 0.0 <= d <= 1.0 for d in decay)):
                raise ConfigError(f"config.json: {where}.mixer.decay must list one number in [0, 1] for each of the {heads} heads")
            return LightningSizes(heads, dim, vdim, tuple(float(d) for d in decay))
        kv_heads = _positive_int(m, "kv_heads", heads)
        if heads % kv_heads:
            raise ConfigError(f"config.json: {where}: {heads} heads are not a multiple of {kv_heads} kv_heads")
        if vdim != dim:
            raise ConfigError(f"config.json: {where}.mixer: the values are the keys, so vdim {vdim} must equal dim {dim}")
        base, dims, scaling = 0.0, 0, None
        if m.get("rot") is not None:
            rot = _object(m["rot"], where + ".mixer.rot")
            base, dims = _number(rot, "base", where + ".mixer.rot"), _positive_int(rot, "dims")
            if dims % 2 or dims > dim:
                raise ConfigError(f"config.json: {where}.mixer.rot.dims {dims} must be even and at most dim {dim}")
            if rot.get("scaling") is not None:
                sc, w = _object(rot["scaling"], where + ".mixer.rot.scaling"), where + ".mixer.rot.scaling"
                scaling = FrequencyScaling(_number(sc, "factor", w), _number(sc, "low", w), _number(sc, "high", w),
                                           _number(sc, "original", w))
                if scaling.high == scaling.low:
                    raise ConfigError(f"config.json: {w}: high and low must differ")
        return SinkAttentionSizes(heads, kv_heads, dim, vdim, _number(m, "scale", where + ".mixer"), base, dims, scaling)

    @classmethod
    def _mlp(cls, raw, where: str):
        if raw is None:
            return None
        m = _object(raw, where + ".mlp")
        kind = m.get("kind")
        if kind == "dense":
            return DenseSizes(_positive_int(m, "ff"))
        if kind == "moe":
            router = _object(m.get("router"), where + ".mlp.router")
            expert = _object(m.get("expert"), where + ".mlp.expert")
            experts, top = _positive_int(router, "experts"), _positive_int(router, "top")
            if top > experts:
                raise ConfigError(f"config.json: {where}.mlp.router: top {top} of {experts} experts")
            scale = _number(router, "scale", where + ".mlp.router") if "scale" in router else 1.0
            shared_ff, shared_limit = 0, 0.0
            if m.get("shared") is not None:
                sh = _object(m["shared"], where + ".mlp.shared")
                shared_ff, shared_limit = _positive_int(sh, "ff"), _number(sh, "limit", where + ".mlp.shared")
            return MoeSizes(experts, top, scale, _positive_int(expert, "ff"), _number(expert, "limit", where + ".mlp.expert"),
                            shared_ff, shared_limit)
        raise ConfigError(f"config.json: {where}.mlp.kind {kind!r} is not one of {cls.MLP_KINDS}")

    @classmethod
    def from_dict(cls, raw: dict) -> "FazopelConfig":
        norm = _object(raw.get("norm"), "norm")
        layers_raw = raw.get("layers")
        if not isinstance(layers_raw, list) or not layers_raw:
            raise ConfigError("config.json: layers must be a list with at least one entry")
        layers = []
        for i, L in enumerate(layers_raw):
            where = f"layers[{i}]"
            L = _object(L, where)
            kind = L.get("type")
            if kind not in cls.MIXER_TYPES:
                raise ConfigError(f"config.json: {where}.type {kind!r} is not one of {cls.MIXER_TYPES}")
            wo = L.get("weights_of")
            if wo is not None and (isinstance(wo, bool) or not isinstance(wo, int) or not 0 <= wo < len(layers_raw) or wo == i):
                raise ConfigError(f"config.json: {where}.weights_of {wo!r} names no other layer")
            layers.append(FazopelLayer(kind, cls._mixer(kind, L.get("mixer"), where), cls._mlp(L.get("mlp"), where), wo))
        for i, L in enumerate(layers):
            if L.weights_of is not None:
                src = layers[L.weights_of]
                if src.weights_of is not None:
                    raise ConfigError(f"config.json: layers[{i}] uses the weights of layers[{L.weights_of}], which has none of its own")
                if (src.type, src.mixer, src.mlp) != (L.type, L.mixer, L.mlp):
                    raise ConfigError(f"config.json: layers[{i}] uses the weights of layers[{L.weights_of}] but differs from it")
        return cls(vocab=_positive_int(raw, "vocab"), width=_positive_int(raw, "width"), eps=_number(norm, "eps", "norm"),
                   layers=tuple(layers))

    def to_dict(self) -> dict:
        return {"architecture": NAME, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
                "layers": [L.to_dict() for L in self.layers]}


def _mixer_spec(c: FazopelConfig, L: FazopelLayer):
    """(mixer spec, the mixer's local tensor names -> names under l<i>.mix.)"""
    m = L.mixer
    if L.type == "lightning":
        spec = PartSpec.of("lightning", hidden=c.width, n_heads=m.heads, head_dim=m.dim, v_head_dim=m.vdim, decay=m.decay,
                           eps=c.eps, gate_activation="sigmoid")
        return spec, {"wq": "q", "wk": "k", "wv": "v", "wg": "g", "wo": "o", "norm": "norm"}
    if m.rot_dims:
        scaling = None
        if m.rot_scaling is not None:
            s = m.rot_scaling
            scaling = (("rope_type", "llama3"), ("factor", s.factor), ("low_freq_factor", s.low), ("high_freq_factor", s.high),
                       ("original_max_position_embeddings", s.original))
        position = PartSpec.of("rope", head_dim=m.dim, theta=m.rot_base, rope_dims=m.rot_dims, scaling=scaling)
    else:
        position = PartSpec.of("none")
    spec = PartSpec.of("attention", hidden=c.width, n_heads=m.heads, n_kv_heads=m.kv_heads, head_dim=m.dim, scale=m.scale,
                       position=position, qk_norm_eps=c.eps, qk_norm_span="head", sink=True, value_is_key=True)
    return spec, {"wq": "q", "wk": "k", "wo": "o", "q_norm": "q.norm", "k_norm": "k.norm"}


def _ffn_spec(c: FazopelConfig, mlp, prefix: str):
    """(feed-forward spec, its local tensor names -> names of the folder)"""
    if isinstance(mlp, DenseSizes):
        return (PartSpec.of("dense", hidden=c.width, intermediate=mlp.ff, activation="relu2"),
                {"w_up": prefix + "up", "w_down": prefix + "down"})
    spec = PartSpec.of("moe", hidden=c.width, n_experts=mlp.experts, top_k=mlp.top, intermediate=mlp.ff, scoring="softmax",
                       renormalize=True, weight_on="output", expert_limit=mlp.limit, gate_slope=GATE_SLOPE, up_shift=UP_SHIFT,
                       choice_bias=True, weight_floor=WEIGHT_FLOOR, weight_scale=mlp.scale,
                       shared_intermediate=mlp.shared_ff, shared_limit=mlp.shared_limit)
    names = {"router": prefix + "router", "correction": prefix + "correction"}
    for e in range(mlp.experts):
        names.update({f"e{e}.w_gate": f"{prefix}e{e}.gate", f"e{e}.w_up": f"{prefix}e{e}.up", f"e{e}.w_down": f"{prefix}e{e}.down"})
    if mlp.shared_ff:
        names.update({"shared.w_gate": prefix + "shared.gate", "shared.w_up": prefix + "shared.up",
                      "shared.w_down": prefix + "shared.down", "shared.gate": prefix + "shared.sg"})
    return spec, names


def build_fazopel_plan(c: FazopelConfig) -> ModelPlan:
    norm, reads_stream = PartSpec.of("rmsnorm", dim=c.width, eps=c.eps), PartSpec.of("none", dim=c.width)
    layers, index = [], {}                  # index: config layer -> its place among the layers that own tensors
    for i, L in enumerate(c.layers):
        if L.weights_of is not None:
            continue
        p = f"l{i}."
        mixer, mixer_names = _mixer_spec(c, L)
        names = {"mixer_out_norm.weight": p + "norm1"}
        names.update({"mixer." + local: p + "mix." + name for local, name in mixer_names.items()})
        ffn = None
        if L.mlp is not None:
            ffn, ffn_names = _ffn_spec(c, L.mlp, p + "mlp.")
            names["ffn_out_norm.weight"] = p + "norm2"
            names.update({"ffn." + local: name for local, name in ffn_names.items()})
        block = PartSpec.of("prenorm", mixer=mixer, ffn=ffn, mixer_norm=reads_stream,
                            ffn_norm=reads_stream if ffn is not None else None, mixer_out_norm=norm,
                            ffn_out_norm=norm if ffn is not None else None)
        index[i] = len(layers)
        layers.append(LayerPlan(block=block, names=names))
    schedule = [ScheduleEntry(index[L.weights_of if L.weights_of is not None else i]) for i, L in enumerate(c.layers)]
    plan = ModelPlan(vocab_size=c.vocab, hidden_size=c.width, layers=layers, schedule=schedule, final_norm=norm,
                     embedding_name="embed", final_norm_names={"weight": "final.norm"}, lm_head_name="head")
    plan.validate()
    return plan


FAZOPEL = register_architecture(Architecture(name=NAME, config_cls=FazopelConfig, build_plan=build_fazopel_plan,
                                             aliases=("fazopel",)))
