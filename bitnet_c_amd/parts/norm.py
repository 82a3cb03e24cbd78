"""RMSNorm: out = x * 1/sqrt(mean(x^2) + eps) * w, eps inside the root
(src/transformer/rmsnorm_scalar.c:4-13).  Computed in float32 whatever the activation
type; the weight is kept in float32.  `scalar`: the model folder holds one number for all
coordinates (a tensor without dimensions); it is spread over the coordinates at load, and
every kernel that takes this norm, folded into a product or not, sees a weight vector.

"none": no norm at all: the part behind it reads the stream itself, in the activations' type (a block whose norms sit on
its parts' outputs only)."""
from __future__ import annotations

import torch

from .. import ops
from .base import NORMS, ParamSpec, Part
from .linear import upload


@NORMS.register("rmsnorm")
class RMSNorm(Part):
    prompt_capturable = True    # a prompt step is read from the context's device tensors alone
    deferrable = True        # a product may fold this norm around itself (weight and eps are all it needs)
    takes_partial_sums = True    # apply() accepts ops.PartialSums as the delta
    normed_delta = True          # weight and eps are all that ops.add_normed_rmsnorm needs: it may be a block's output norm

    def __init__(self, dim: int, eps: float, scalar: bool = False):
        self.dim, self.eps, self.scalar = int(dim), float(eps), bool(scalar)
        self.weight = None

    def tensors(self):
        return {"weight": ParamSpec(() if self.scalar else (self.dim,), init="ones")}

    def load(self, tensors, device, dtype):
        w = upload(tensors["weight"], device, torch.float32)
        self.weight = w.reshape(1).expand(self.dim).contiguous() if self.scalar else w

    def apply(self, x, delta, out_dtype, rows=None):
        return ops.add_rmsnorm(x, delta, self.weight, self.eps, out_dtype, rows)


@NORMS.register("none")
class NoNorm(Part):
    """The stream as it is.  A held-back output that has a norm of its own is added by the same kernel that hands the
    rows on (ResidualStream.normed)."""
    prompt_capturable = True
    passes_rows = True           # ResidualStream: no weight, no factor: the rows themselves

    def __init__(self, dim: int = 0):
        self.dim = int(dim)

    def apply(self, x, delta, out_dtype, rows=None):
        if rows is not None:
            if delta is not None:
                raise ValueError("a choice of rows leaves the stream as it is")
            return ops.gather_rows(x, rows, out_dtype)
        if delta is not None:
            ops.residual_add(x, delta)
        return ops.stream_rows(x, out_dtype)
