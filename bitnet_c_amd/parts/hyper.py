"""A residual that is several streams ("hyper-connections"), the block that reads and writes it, and a norm without
statistics.

Instead of one residual x there are n copies x_1 .. x_n, all equal to the embedding's rows at the start.  Sublayer q of a
layer (1: the mixer, 2: the feed-forward) reads a weighted sum of them, and its output rebuilds all of them at once from
the old ones:

    u = sum_s in_q[s] x_s;   y = sublayer(norm(u));   x_t <- sum_s mix_q[s, t] x_s + mult * out_q[t] * y

(mix is indexed [from, to]; mult is a constant of the model).  What leaves the model is the sum of the streams.  With
one stream and in = out = mix = 1 this is the plain residual x <- x + mult * sublayer(norm(x)); a block built with
learned=False is that, without tensors.

The write of a sublayer is held back and done by the kernel that reads for the next one (ops.hc_step): the streams are
read once and written once per sublayer, and the read's norm rides along.

"dyt": the norm tanh(alpha x) * w + b with one number alpha, a weight and a bias vector; no mean, no variance, no eps.
"""
from __future__ import annotations

import torch

from .. import ops
from .base import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, ParamSpec, Part, PartSpec
from .linear import upload


@NORMS.register("dyt")
class DynamicTanh(Part):
    prompt_capturable = True    # a prompt step is read from the context's device tensors alone

    def __init__(self, dim: int):
        self.dim = int(dim)
        self.weight = self.bias = self.alpha = None

    def tensors(self):
        return {"weight": ParamSpec((self.dim,), "ones"), "bias": ParamSpec((self.dim,), "zeros"), "alpha": ParamSpec((), "ones")}

    def load(self, tensors, device, dtype):
        self.weight = upload(tensors["weight"], device, torch.float32)
        self.bias = upload(tensors["bias"], device, torch.float32)
        self.alpha = upload(tensors["alpha"], device, torch.float32).reshape(1).contiguous()

    @property
    def tanh_triple(self):
        """(weight, bias, alpha): what a kernel that applies this norm on its way needs (ops.hc_step)."""
        return self.weight, self.bias, self.alpha

    def apply(self, x, delta, out_dtype, rows=None):
        return ops.add_dyt_norm(x, delta, self.weight, self.bias, self.alpha, out_dtype, rows)


class HyperStream:
    """The residual of a step as n float32 streams.  Until the first write every stream is the embedding's rows
    (`base`, read n times by the first kernel); `lanes` [n, T, D] afterwards.  A sublayer's output is held back with its
    coefficients (`pending`) and folded in by the next read."""

    def __init__(self, x: torch.Tensor, n: int):
        if not 1 <= n <= ops.HC_MAX_STREAMS:
            raise ValueError(f"a residual of {n} streams (at most {ops.HC_MAX_STREAMS})")
        self.base, self.n = x, int(n)
        self.lanes = None
        self.pending = None                      # (delta, mix, out_coef, mult)

    def write(self, delta, mix, out_coef, mult: float) -> None:
        if self.pending is not None:
            self._pass(read=False)
        self.pending = (delta, mix, out_coef, float(mult))

    def _pass(self, read: bool, in_coef=None, norm=None, out_dtype=None, rows=None):
        src = self.lanes if self.lanes is not None else self.base
        kw = {}
        store = None
        if self.pending is not None:
            delta, mix, out_coef, mult = self.pending
            kw = dict(delta=delta, mix=mix, out_coef=out_coef, mult=mult)
            if rows is None:
                store = self.lanes if self.lanes is not None else torch.empty((self.n,) + tuple(self.base.shape),
                                                                              dtype=torch.float32, device=self.base.device)
        triple = getattr(norm, "tanh_triple", None) if norm is not None else None
        h = ops.hc_step(src, store, self.n, in_coef=in_coef, norm=triple, rows=rows, read=read,
                        out_dtype=out_dtype if (norm is None or triple is not None) else torch.float32, **kw)
        if store is not None:
            self.lanes, self.pending = store, None
        if read and norm is not None and triple is None:
            h = norm.apply(h, None, out_dtype)       # a norm that the kernel does not know: on the sum that it formed
        return h

    def read(self, in_coef, norm, out_dtype):
        """norm(sum_s in_coef[s] x_s) for the next sublayer, after the held-back write."""
        return self._pass(True, in_coef, norm, out_dtype)

    def normed(self, norm, out_dtype, rows=None, consumer=None, ctx=None):
        """The model's end: the sum of the streams (at `rows`) under `norm`."""
        return self._pass(True, None, norm, out_dtype, rows)

    def flush(self) -> torch.Tensor:
        """The sum of the streams, [T, D] float32 (diagnostics, and a model without a final norm)."""
        return self._pass(True, None, None, torch.float32)

    @property
    def x(self):
        return self.flush()


@BLOCKS.register("hyper")
class HyperBlock(Part):
    """norm -> mixer and norm -> feed-forward over a residual of `streams` streams, each sublayer's output times `mult`.
    learned: the coefficients are tensors hc1.in / hc1.out [n], hc1.mix [n, n] (and hc2.* with a feed-forward); else one
    stream with coefficients 1."""

    def __init__(self, mixer: PartSpec, ffn: PartSpec | None, mixer_norm: PartSpec, ffn_norm: PartSpec | None = None,
                 streams: int = 1, mult: float = 1.0, learned: bool = True):
        if (ffn is None) != (ffn_norm is None):
            raise ValueError("hyper block: a feed-forward and its norm come together or not at all")
        self.n, self.mult, self.learned = int(streams), float(mult), bool(learned)
        if not 1 <= self.n <= ops.HC_MAX_STREAMS or (not self.learned and self.n != 1):
            raise ValueError(f"hyper block: {streams} streams (at most {ops.HC_MAX_STREAMS}; one when nothing is learned)")
        self.mixer = MIXERS.build(mixer)
        self.ffn = FEED_FORWARDS.build(ffn) if ffn is not None else None
        self.mixer_norm = NORMS.build(mixer_norm)
        self.ffn_norm = NORMS.build(ffn_norm) if ffn_norm is not None else None
        self.coef = {}                            # "hc1" / "hc2" -> (in, out, mix) float32 on the device

    @property
    def prompt_capturable(self) -> bool:
        return all(getattr(c, "prompt_capturable", False) for c in self.children().values())

    def children(self):
        c = {"mixer": self.mixer, "ffn": self.ffn, "mixer_norm": self.mixer_norm, "ffn_norm": self.ffn_norm}
        return {k: v for k, v in c.items() if v is not None}

    def _sublayers(self):
        return ("hc1", "hc2") if self.ffn is not None else ("hc1",)

    def linears(self):
        return [l for part in self.children().values() for l in getattr(part, "linears", list)()]

    def tensors(self):
        t = {f"{cn}.{tn}": spec for cn, c in self.children().items() for tn, spec in c.tensors().items()}
        if self.learned:
            for q in self._sublayers():
                t.update({f"{q}.in": ParamSpec((self.n,), "ones"), f"{q}.out": ParamSpec((self.n,), "ones"),
                          f"{q}.mix": ParamSpec((self.n, self.n), "normal")})
        return t

    def load(self, tensors, device, dtype):
        for cn, c in self.children().items():
            c.load({k[len(cn) + 1:]: v for k, v in tensors.items() if k.startswith(cn + ".")}, device, dtype)
        for q in self._sublayers():
            if self.learned:
                self.coef[q] = tuple(upload(tensors[f"{q}.{n}"], device, torch.float32).contiguous() for n in ("in", "out", "mix"))
            else:
                one = torch.ones(1, dtype=torch.float32, device=device)
                self.coef[q] = (one, one, one.reshape(1, 1))

    def cache_need(self):
        return self.mixer.cache_need()

    def forward(self, stream, ctx, kv):
        if not isinstance(stream, HyperStream) or stream.n != self.n:
            raise TypeError(f"hyper block: the model's residual must be {self.n} streams (ModelPlan.residual_streams)")
        tap = getattr(ctx, "tap", None)
        if tap is not None:
            tap("layer_in", ctx.entry, stream, ctx)
        c_in, c_out, c_mix = self.coef["hc1"]
        h = stream.read(c_in, self.mixer_norm, ctx.act_dtype)
        stream.write(self.mixer.forward(h, ctx, kv), c_mix, c_out, self.mult)
        if tap is not None:
            tap("ffn_in", ctx.entry, stream, ctx)
        if self.ffn is not None:
            c_in, c_out, c_mix = self.coef["hc2"]
            h = stream.read(c_in, self.ffn_norm, ctx.act_dtype)
            stream.write(self.ffn.forward(h, ctx), c_mix, c_out, self.mult)
        if tap is not None:
            tap("layer_out", ctx.entry, stream, ctx)
