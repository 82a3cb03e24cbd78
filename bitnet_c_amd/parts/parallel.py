"""Two mixers side by side: both read the same input, each output goes through an RMSNorm of its own over the model
width (plain weights "left_out" / "right_out", eps inside the root), and the result is half their sum:

    y = 1/2 (rmsnorm(left(h)) * w_left + rmsnorm(right(h)) * w_right)

The two are any registered mixers; between them they may keep one set of keys and values (the cache gives an entry of
the schedule one).  Each may keep a state of fixed size: two float32 states addressed by the step's slot ids lie side by
side in the entry's one state row, the left mixer's first, and each mixer sees its own columns.
"""
from __future__ import annotations

import dataclasses

import torch

from .. import ops
from .base import MIXERS, CacheNeed, ParamSpec, Part, PartSpec, StateNeed
from .linear import upload


@MIXERS.register("parallel")
class ParallelMixer(Part):
    def __init__(self, hidden: int, left: PartSpec, right: PartSpec, eps: float):
        self.hidden, self.eps = int(hidden), float(eps)
        self.left, self.right = MIXERS.build(left), MIXERS.build(right)
        needs = [self.left.cache_need(), self.right.cache_need()]
        if sum(n.kv is not None for n in needs) > 1:
            raise ValueError("parallel mixer: its two mixers may keep one set of keys and values between them")
        self.state_split = None                  # floats of the left mixer's state when both keep one
        if all(n.state is not None for n in needs):
            for n in needs:
                if len(n.state.shape) != 1 or n.state.dtype != torch.float32:
                    raise ValueError("parallel mixer: two states share a row only as flat float32 states")
            self.state_split = int(needs[0].state.shape[0])
        self.w_left = self.w_right = None

    @property
    def prompt_capturable(self) -> bool:
        return all(getattr(m, "prompt_capturable", False) for m in (self.left, self.right))

    def children(self):
        return {"left": self.left, "right": self.right}

    def tensors(self):
        t = {f"{cn}.{tn}": spec for cn, c in self.children().items() for tn, spec in c.tensors().items()}
        t.update({"left_out": ParamSpec((self.hidden,), "ones"), "right_out": ParamSpec((self.hidden,), "ones")})
        return t

    def load(self, tensors, device, dtype):
        for cn, c in self.children().items():
            c.load({k[len(cn) + 1:]: v for k, v in tensors.items() if k.startswith(cn + ".")}, device, dtype)
        self.w_left = upload(tensors["left_out"], device, torch.float32)
        self.w_right = upload(tensors["right_out"], device, torch.float32)

    def linears(self):
        return [l for c in self.children().values() for l in c.linears()]

    def cache_need(self) -> CacheNeed:
        a, b = self.left.cache_need(), self.right.cache_need()
        state = a.state or b.state
        if self.state_split is not None:
            state = StateNeed((a.state.shape[0] + b.state.shape[0],), torch.float32,
                              device_addressed=a.state.device_addressed and b.state.device_addressed)
        return CacheNeed(kv=a.kv or b.kv, state=state)

    def forward(self, h, ctx, kv):
        kv_a = kv_b = kv
        if self.state_split is not None:
            kv_a = dataclasses.replace(kv, state=kv.state[:, :self.state_split])
            kv_b = dataclasses.replace(kv, state=kv.state[:, self.state_split:])
        a = self.left.forward(h, ctx, kv_a)
        b = self.right.forward(h, ctx, kv_b)
        return ops.rmsnorm_mean(a, self.w_left, b, self.w_right, self.eps)
