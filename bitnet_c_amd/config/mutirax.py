"""Mutirax: a decoder whose config.json lists its layers one by one, over a residual of several streams.

A layer is pre-norm, each sublayer's output times a constant m (`residual_mult`): x += m mixer(norm1(x)), x += m ff(norm2(x)),
with the norm tanh(alpha x) * w + b (no statistics; parts/hyper.py "dyt").  With `streams` in config.json the residual is
that many copies of the embedding's rows; sublayer q of a layer reads sum_s in_q[s] x_s and rebuilds every copy,
x_t <- sum_s mix_q[s, t] x_s + m out_q[t] y; the model's norm reads their sum (parts/hyper.py, block "hyper").

Three kinds of mixers:

  "gla"               gated linear attention: a float32 matrix state per head with a decay per key channel and token
                      (parts/recurrent.py "gla")
  "latent_attention"  causal attention whose queries pass a normed latent and whose keys and values are projections of one
                      normed latent per token, beside one rotated key part that all heads share (frequencies rescaled
                      the "yarn" way); one sigmoid gate number per head (parts/latent.py)
  "parallel"          half the sum of two mixers' outputs, each under an RMSNorm of its own (parts/parallel.py): left,
                      grouped-query attention without a value matrix (the values are the keys as they leave a short
                      convolution over time on the query and key projections; norms over the whole projections; a
                      rotation of the first rot.dims dimensions of a head; a learned term per head in the softmax's
                      denominator; parts/attention.py); right, a recurrent block around a real-gated linear recurrent
                      unit with a short convolution (parts/recurrent.py "rglru")

and two kinds of feed-forwards: "dense" (a gated unit with bounded arguments, parts/ffn.py "gated_clamped") and "moe"
(silu-gated experts; a router with a bias; the chosen logits' softmax as weights; parts/moe.py); "mlp": null leaves the
second sublayer out.  `loop` {start, stop, times} runs layers start .. stop - 1 `times` times in a row, as a block, with
the same weights and a cache or state of its own for every run: the plan's schedule names those layers several times.

config.json keys: architecture, vocab, width, norm.eps, residual_mult, streams, loop, layers[] = {type, mixer, mlp} with
  gla mixer         {heads, dim, vdim, tau}                          (the decay's rank is the shape of its tensor a1)
  latent mixer      {heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, rot: {base, dims, scaling: {factor, original, fast, slow}}}
  parallel mixer    {left: {heads, kv_heads, dim, vdim, conv, scale, rot: {base, dims}}, right: {width, blocks, conv}}
  mlp               {kind: "dense", ff, limit} | {kind: "moe", expert: {ff}, router: {experts, top}} | null

Tensor names of the folder (linear weights [out, in]): embed, head, final.norm{,.b,.alpha}, and for layer i under l<i>.:
  norm1{,.b,.alpha}, norm2{,.b,.alpha}, hc1.{in,out,mix}, hc2.{in,out,mix}
  gla:       mix.{q,k,v,g,o}, mix.norm, mix.a1, mix.a2, mix.a2.b
  latent:    mix.dq, mix.dq.norm, mix.uq, mix.dkv, mix.dkv.norm, mix.uk, mix.uv, mix.g, mix.o
  parallel:  mix.left.{q,k,o}, mix.left.{q,k}.norm, mix.left.{q,k}.conv, mix.left.sink, mix.left.out,
             mix.right.{y,x,o}, mix.right.{y,x}.b, mix.right.conv, mix.right.conv.b, mix.right.{ra,ri}, mix.right.{ra,ri}.b,
             mix.right.lam, mix.right.out
  dense:     mlp.{gate,up,down}
  moe:       mlp.router, mlp.router.b, mlp.e<n>.{gate,up,down}
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple, Union

from ..engine.plan import LayerPlan, ModelPlan, ScheduleEntry
from ..parts.base import PartSpec
from .base import Architecture, ConfigError, _positive_int, register_architecture
from .fazopel import _number, _object

NAME = "Mutirax"

# Constants of the design (the same in every model of it)
GATE_SLOPE = 1.702            # the dense unit's gate is g sigmoid(GATE_SLOPE g)
UP_SHIFT = 1.0                # and multiplies (u + UP_SHIFT)
LRU_SHARPNESS = 8.0           # log a = -LRU_SHARPNESS r softplus(lam)


@dataclass(frozen=True)
class Rotation:
    base: float
    dims: int
    scaling: Optional[Tuple[Tuple[str, float], ...]] = None       # "yarn": factor, original, fast, slow

    def to_dict(self):
        d = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            d["scaling"] = dict(self.scaling)
        return d


def _rotation(raw, where: str, limit: int) -> Optional[Rotation]:
    if raw is None:
        return None
    rot = _object(raw, where)
    base, dims = _number(rot, "base", where), _positive_int(rot, "dims")
    if dims % 2 or dims > limit or base == 1.0:
        raise ConfigError(f"config.json: {where}.dims {dims} must be even and at most {limit}, and the base not 1")
    scaling = None
    if rot.get("scaling") is not None:
        sc, w = _object(rot["scaling"], where + ".scaling"), where + ".scaling"
        scaling = tuple((k, _number(sc, k, w)) for k in ("factor", "original", "fast", "slow"))
    return Rotation(base, dims, scaling)


@dataclass(frozen=True)
class GlaSizes:
    heads: int
    dim: int
    vdim: int
    tau: float
    decay_rank: int

    def to_dict(self):
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "tau": self.tau}


@dataclass(frozen=True)
class LatentSizes:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    rot: Optional[Rotation]

    def to_dict(self):
        d = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "kv_rank": self.kv_rank,
             "q_rank": self.q_rank, "scale": self.scale}
        if self.rot is not None:
            d["rot"] = self.rot.to_dict()
        return d


@dataclass(frozen=True)
class LeftSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    scale: float
    rot: Optional[Rotation]

    def to_dict(self):
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "conv": self.conv,
             "scale": self.scale}
        if self.rot is not None:
            d["rot"] = self.rot.to_dict()
        return d


@dataclass(frozen=True)
class RightSizes:
    width: int
    blocks: int
    conv: int

    def to_dict(self):
        return {"width": self.width, "blocks": self.blocks, "conv": self.conv}


@dataclass(frozen=True)
class ParallelSizes:
    left: LeftSizes
    right: RightSizes

    def to_dict(self):
        return {"left": self.left.to_dict(), "right": self.right.to_dict()}


@dataclass(frozen=True)
class DenseSizes:
    ff: int
    limit: float

    def to_dict(self):
        return {"kind": "dense", "ff": self.ff, "limit": self.limit}


@dataclass(frozen=True)
class MoeSizes:
    experts: int
    top: int
    ff: int

    def to_dict(self):
        return {"kind": "moe", "expert": {"ff": self.ff}, "router": {"experts": self.experts, "top": self.top}}


@dataclass(frozen=True)
class MutiraxLayer:
    type: str
    mixer: Union[GlaSizes, LatentSizes, ParallelSizes]
    mlp: Union[DenseSizes, MoeSizes, None]

    def to_dict(self):
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclass(frozen=True)
class MutiraxConfig:
    vocab: int
    width: int
    eps: float
    residual_mult: float
    streams: Optional[int]                     # None: one plain residual without connection tensors
    loop: Optional[Tuple[int, int, int]]       # (start, stop, times)
    layers: Tuple[MutiraxLayer, ...]

    MIXER_TYPES = ("gla", "latent_attention", "parallel")
    MLP_KINDS = ("dense", "moe")
    DEFAULT_DECAY_RANK = 16

    @staticmethod
    def sizes_from_tensors(raw: dict, shapes: dict) -> dict:
        """config.json does not say how wide the low-rank input of a gla layer's decay is: the tensor a1 does."""
        raw = dict(raw)
        layers = []
        for i, L in enumerate(raw.get("layers") or []):
            if isinstance(L, dict) and L.get("type") == "gla" and isinstance(L.get("mixer"), dict) and "decay_rank" not in L["mixer"]:
                shape = shapes.get(f"l{i}.mix.a1")
                if shape:
                    L = dict(L, mixer=dict(L["mixer"], decay_rank=int(shape[0])))
            layers.append(L)
        raw["layers"] = layers
        return raw

    @classmethod
    def _mixer(cls, kind: str, raw, where: str):
        m = _object(raw, where + ".mixer")
        if kind == "gla":
            heads, dim = _positive_int(m, "heads"), _positive_int(m, "dim")
            return GlaSizes(heads, dim, _positive_int(m, "vdim", dim), _number(m, "tau", where + ".mixer"),
                            _positive_int(m, "decay_rank", cls.DEFAULT_DECAY_RANK))
        if kind == "latent_attention":
            heads, dim = _positive_int(m, "heads"), _positive_int(m, "dim")
            rot_dim = m.get("rot_dim", 0)
            if isinstance(rot_dim, bool) or not isinstance(rot_dim, int) or rot_dim < 0 or rot_dim % 2:
                raise ConfigError(f"config.json: {where}.mixer.rot_dim must be an even number, got {rot_dim!r}")
            rot = _rotation(m.get("rot"), where + ".mixer.rot", max(rot_dim, 2)) if rot_dim else None
            if rot_dim and rot is None:
                raise ConfigError(f"config.json: {where}.mixer: a rotated part of {rot_dim} dimensions needs rot")
            if rot is not None and rot.dims != rot_dim:
                rot = Rotation(rot.base, rot_dim, rot.scaling)          # the rotated vector is the rot_dim part, whole
            return LatentSizes(heads, dim, rot_dim, _positive_int(m, "vdim", dim), _positive_int(m, "kv_rank"),
                               _positive_int(m, "q_rank"), _number(m, "scale", where + ".mixer"), rot)
        left, right = _object(m.get("left"), where + ".mixer.left"), _object(m.get("right"), where + ".mixer.right")
        heads, dim = _positive_int(left, "heads"), _positive_int(left, "dim")
        kv_heads = _positive_int(left, "kv_heads", heads)
        if heads % kv_heads:
            raise ConfigError(f"config.json: {where}: {heads} heads are not a multiple of {kv_heads} kv_heads")
        vdim = _positive_int(left, "vdim", dim)
        if vdim != dim:
            raise ConfigError(f"config.json: {where}.mixer.left: the values are the keys, so vdim {vdim} must equal dim {dim}")
        ls = LeftSizes(heads, kv_heads, dim, vdim, _positive_int(left, "conv"), _number(left, "scale", where + ".mixer.left"),
                       _rotation(left.get("rot"), where + ".mixer.left.rot", dim))
        rs = RightSizes(_positive_int(right, "width"), _positive_int(right, "blocks"), _positive_int(right, "conv"))
        if rs.width % rs.blocks:
            raise ConfigError(f"config.json: {where}.mixer.right: {rs.width} channels are not {rs.blocks} equal parts")
        return ParallelSizes(ls, rs)

    @classmethod
    def _mlp(cls, raw, where: str):
        if raw is None:
            return None
        m = _object(raw, where + ".mlp")
        kind = m.get("kind")
        if kind == "dense":
            return DenseSizes(_positive_int(m, "ff"), _number(m, "limit", where + ".mlp"))
        if kind == "moe":
            router = _object(m.get("router"), where + ".mlp.router")
            experts, top = _positive_int(router, "experts"), _positive_int(router, "top")
            if top > experts:
                raise ConfigError(f"config.json: {where}.mlp.router: top {top} of {experts} experts")
            return MoeSizes(experts, top, _positive_int(_object(m.get("expert"), where + ".mlp.expert"), "ff"))
        raise ConfigError(f"config.json: {where}.mlp.kind {kind!r} is not one of {cls.MLP_KINDS}")

    @classmethod
    def from_dict(cls, raw: dict) -> "MutiraxConfig":
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
            layers.append(MutiraxLayer(kind, cls._mixer(kind, L.get("mixer"), where), cls._mlp(L.get("mlp"), where)))
        loop = None
        if raw.get("loop") is not None:
            lp = _object(raw["loop"], "loop")
            start, stop, times = lp.get("start"), lp.get("stop"), lp.get("times")
            for v in (start, stop, times):
                if isinstance(v, bool) or not isinstance(v, int):
                    raise ConfigError(f"config.json: loop needs whole numbers start, stop and times, got {lp!r}")
            if not (0 <= start < stop <= len(layers)) or times < 1:
                raise ConfigError(f"config.json: loop {lp!r} names no run of the {len(layers)} layers, or repeats it less than once")
            loop = (start, stop, times)
        streams = raw.get("streams")
        if streams is not None and (isinstance(streams, bool) or not isinstance(streams, int) or streams < 1):
            raise ConfigError(f"config.json: streams must be a positive whole number, got {streams!r}")
        mult = _number(raw, "residual_mult", "config") if "residual_mult" in raw else 1.0
        return cls(vocab=_positive_int(raw, "vocab"), width=_positive_int(raw, "width"), eps=_number(norm, "eps", "norm"),
                   residual_mult=mult, streams=streams, loop=loop, layers=tuple(layers))

    def to_dict(self) -> dict:
        d = {"architecture": NAME, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
             "residual_mult": self.residual_mult, "layers": [L.to_dict() for L in self.layers]}
        for i, L in enumerate(self.layers):
            if L.type == "gla":
                d["layers"][i]["mixer"]["decay_rank"] = L.mixer.decay_rank
        if self.streams is not None:
            d["streams"] = self.streams
        if self.loop is not None:
            d["loop"] = {"start": self.loop[0], "stop": self.loop[1], "times": self.loop[2]}
        return d

    def layer_runs(self):
        """The layers in the order they run."""
        n = len(self.layers)
        if self.loop is None:
            return list(range(n))
        a, b, times = self.loop
        return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def _rope(rot: Optional[Rotation], head_dim: int) -> PartSpec:
    if rot is None:
        return PartSpec.of("none")
    return PartSpec.of("rope", head_dim=head_dim, theta=rot.base, rope_dims=rot.dims)


def _mixer_spec(c: MutiraxConfig, L: MutiraxLayer):
    """(mixer spec, the mixer's local tensor names -> names under l<i>.mix.)"""
    m = L.mixer
    if L.type == "gla":
        spec = PartSpec.of("gla", hidden=c.width, n_heads=m.heads, head_dim=m.dim, v_head_dim=m.vdim, decay_rank=m.decay_rank,
                           tau=m.tau, eps=c.eps)
        return spec, {"wq": "q", "wk": "k", "wv": "v", "wg": "g", "wo": "o", "norm": "norm", "wa1": "a1", "wa2": "a2",
                      "a2_bias": "a2.b"}
    if L.type == "latent_attention":
        scaling = None
        if m.rot is not None and m.rot.scaling is not None:
            scaling = (("rope_type", "yarn"),) + m.rot.scaling
        spec = PartSpec.of("latent_attention", hidden=c.width, n_heads=m.heads, head_dim=m.dim, v_head_dim=m.vdim,
                           kv_rank=m.kv_rank, scale=m.scale, eps=c.eps, gate="head", q_rank=m.q_rank, rot_dim=m.rot_dim,
                           rot_theta=m.rot.base if m.rot is not None else 10000.0, rot_scaling=scaling)
        return spec, {"wdq": "dq", "dq_norm": "dq.norm", "wuq": "uq", "wdkv": "dkv", "dkv_norm": "dkv.norm", "wuk": "uk",
                      "wuv": "uv", "wg": "g", "wo": "o"}
    left = PartSpec.of("attention", hidden=c.width, n_heads=m.left.heads, n_kv_heads=m.left.kv_heads, head_dim=m.left.dim,
                       scale=m.left.scale, position=_rope(m.left.rot, m.left.dim), qk_norm_eps=c.eps, qk_norm_span="projection",
                       sink="learned", value_is_key=True, conv_taps=m.left.conv)
    right = PartSpec.of("rglru", hidden=c.width, width=m.right.width, blocks=m.right.blocks, conv_taps=m.right.conv,
                        sharpness=LRU_SHARPNESS)
    spec = PartSpec.of("parallel", hidden=c.width, left=left, right=right, eps=c.eps)
    names = {"left.wq": "left.q", "left.wk": "left.k", "left.wo": "left.o", "left.q_norm": "left.q.norm",
             "left.k_norm": "left.k.norm", "left.q_conv": "left.q.conv", "left.k_conv": "left.k.conv", "left.sink": "left.sink",
             "left_out": "left.out", "right_out": "right.out",
             "right.wy": "right.y", "right.by": "right.y.b", "right.wx": "right.x", "right.bx": "right.x.b",
             "right.conv": "right.conv", "right.conv_bias": "right.conv.b", "right.ra": "right.ra", "right.ra_bias": "right.ra.b",
             "right.ri": "right.ri", "right.ri_bias": "right.ri.b", "right.lam": "right.lam", "right.wo": "right.o"}
    return spec, names


def _ffn_spec(c: MutiraxConfig, mlp, prefix: str):
    """(feed-forward spec, its local tensor names -> names of the folder)"""
    if isinstance(mlp, DenseSizes):
        spec = PartSpec.of("gated_clamped", hidden=c.width, intermediate=mlp.ff, limit=mlp.limit, slope=GATE_SLOPE, shift=UP_SHIFT)
        return spec, {"w_gate": prefix + "gate", "w_up": prefix + "up", "w_down": prefix + "down"}
    spec = PartSpec.of("moe", hidden=c.width, n_experts=mlp.experts, top_k=mlp.top, intermediate=mlp.ff, activation="silu",
                       scoring="softmax", renormalize=True, weight_on="output", gated=True, router_bias=True)
    names = {"router": prefix + "router", "router_bias": prefix + "router.b"}
    for e in range(mlp.experts):
        names.update({f"e{e}.w_gate": f"{prefix}e{e}.gate", f"e{e}.w_up": f"{prefix}e{e}.up", f"e{e}.w_down": f"{prefix}e{e}.down"})
    return spec, names


_NORM_NAMES = {"weight": "", "bias": ".b", "alpha": ".alpha"}


def build_mutirax_plan(c: MutiraxConfig) -> ModelPlan:
    norm = PartSpec.of("dyt", dim=c.width)
    learned = c.streams is not None
    n_streams = c.streams if learned else 1
    layers = []
    for i, L in enumerate(c.layers):
        p = f"l{i}."
        mixer, mixer_names = _mixer_spec(c, L)
        names = {"mixer_norm." + local: p + "norm1" + tail for local, tail in _NORM_NAMES.items()}
        names.update({"mixer." + local: p + "mix." + name for local, name in mixer_names.items()})
        ffn = None
        if L.mlp is not None:
            ffn, ffn_names = _ffn_spec(c, L.mlp, p + "mlp.")
            names.update({"ffn_norm." + local: p + "norm2" + tail for local, tail in _NORM_NAMES.items()})
            names.update({"ffn." + local: name for local, name in ffn_names.items()})
        if learned:
            for q in ("hc1", "hc2") if ffn is not None else ("hc1",):
                names.update({f"{q}.{n}": f"{p}{q}.{n}" for n in ("in", "out", "mix")})
        block = PartSpec.of("hyper", mixer=mixer, ffn=ffn, mixer_norm=norm, ffn_norm=norm if ffn is not None else None,
                            streams=n_streams, mult=c.residual_mult, learned=learned)
        layers.append(LayerPlan(block=block, names=names))
    schedule = [ScheduleEntry(i) for i in c.layer_runs()]
    plan = ModelPlan(vocab_size=c.vocab, hidden_size=c.width, layers=layers, schedule=schedule, final_norm=norm,
                     embedding_name="embed", final_norm_names={local: "final.norm" + tail for local, tail in _NORM_NAMES.items()},
                     lm_head_name="head", residual_streams=n_streams)
    plan.validate()
    return plan


MUTIRAX = register_architecture(Architecture(name=NAME, config_cls=MutiraxConfig, build_plan=build_mutirax_plan,
                                             aliases=("mutirax",)))
