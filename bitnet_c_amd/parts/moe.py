"""Mixture-of-experts feed-forward: n_experts small feed-forwards, of which every token uses top_k.

    z = W_router h                         float32 (h in the activations' type)
    s = sigmoid(z)   or   softmax(z)       `scoring`
    the top_k experts with the largest scores; their weights w are the scores themselves, or, with `renormalize`, the
    scores divided by their sum
    y = sum over the chosen e of  W_down,e act(W_up,e (w_e h))     weight_on "input": the weight multiplies what the expert reads
      = sum over the chosen e of  w_e W_down,e act(W_up,e h)       weight_on "output"

Options beside that form, each off by default:
  expert_limit     the experts are gated units instead: W_down,e unit(W_gate,e x, W_up,e x) with
                   unit(g, u) = g' sigmoid(slope g') (u' + shift), g' = min(g, limit), u' = clamp(u, -limit, limit)
                   (gate_slope 1.702 and up_shift 1 unless said otherwise; tensors e<n>.w_gate beside w_up, w_down)
  choice_bias      a tensor `correction` [n_experts]: the experts with the largest score + correction are chosen; the
                   weights stay the plain scores
  weight_floor     joins the sum that `renormalize` divides by;  weight_scale multiplies the weights
  gated            (without expert_limit) the experts are plain gated units W_down,e (act(W_gate,e x) * (W_up,e x)) with
                   act = silu: the unit above without bounds, slope 1 and shift 0
  router_bias      a tensor `router_bias` [n_experts] added to the logits themselves, before scoring and choice
  shared_intermediate (with shared_limit)   one more gated unit of that width that every token runs (shared.w_gate,
                   shared.w_up, shared.w_down), its output times sigmoid(shared.gate . h), one number per token

The experts' matrices are stacked on the device ([E, F, D] and [E, D, F]); the model folder holds them one by one
(e<n>.w_up [F, D], e<n>.w_down [D, F]).  The router runs one workgroup a token and chooses on the device; steps of few rows
read each chosen expert once per (token, choice) pair (ops.moe_experts), steps of many rows order the pairs by expert and
run the two products as grouped matrix products over tiles whose rows share an expert (ops.moe_experts_grouped).  Nothing waits
for the host, so the part's steps are captured like any other.  The result is handed on as the top_k slabs of float32
rows (ops.PartialSums) that the consumer's kernel adds.
"""
from __future__ import annotations

import torch

from .. import ops
from .base import FEED_FORWARDS, ParamSpec, Part
from .linear import Linear, upload


@FEED_FORWARDS.register("moe")
class MoEFFN(Part):
    prompt_capturable = True    # a prompt step is read from the context's device tensors alone

    def __init__(self, hidden: int, n_experts: int, top_k: int, intermediate: int, activation: str = "relu2",
                 scoring: str = "sigmoid", renormalize: bool = False, weight_on: str = "input", expert_limit: float = 0.0,
                 gate_slope: float = 1.702, up_shift: float = 1.0, choice_bias: bool = False, weight_floor: float = 0.0,
                 weight_scale: float = 1.0, shared_intermediate: int = 0, shared_limit: float = 0.0, gated: bool = False,
                 router_bias: bool = False):
        if activation not in ops.UNARY_ACTIVATIONS:
            raise ValueError(f"moe: unknown activation {activation!r}; known: {sorted(ops.UNARY_ACTIVATIONS)}")
        if scoring not in ops.MOE_SCORINGS:
            raise ValueError(f"moe: unknown scoring {scoring!r}; known: {sorted(ops.MOE_SCORINGS)}")
        if weight_on not in ("input", "output"):
            raise ValueError(f"moe: weight_on {weight_on!r} is neither 'input' nor 'output'")
        self.hidden, self.E, self.K, self.F = int(hidden), int(n_experts), int(top_k), int(intermediate)
        if not 1 <= self.K <= self.E or self.E > ops.MOE_MAX_EXPERTS:
            raise ValueError(f"moe: top_k {self.K} of {self.E} experts (at most {ops.MOE_MAX_EXPERTS})")
        self.activation, self.scoring, self.renormalize = activation, scoring, bool(renormalize)
        self.weight_on_input = weight_on == "input"
        self.unit = ops.ClampedUnit(float(expert_limit), float(gate_slope), float(up_shift)) if expert_limit else None
        if gated and self.unit is None:
            if activation != "silu":
                raise ValueError(f"moe: gated experts without bounds take the activation 'silu', got {activation!r}")
            self.unit = ops.ClampedUnit(float("inf"), 1.0, 0.0)
        self.has_router_bias = bool(router_bias)
        self.has_choice_bias, self.weight_floor, self.weight_scale = bool(choice_bias), float(weight_floor), float(weight_scale)
        if self.weight_floor < 0 or not self.weight_scale > 0:
            raise ValueError(f"moe: weight_floor {weight_floor} must not be negative and weight_scale {weight_scale} be positive")
        self.Fs = int(shared_intermediate)
        if self.Fs < 0 or (self.Fs > 0) != (shared_limit > 0):
            raise ValueError("moe: a shared expert has a width and a limit, or there is none")
        self.shared_unit = ops.ClampedUnit(float(shared_limit), float(gate_slope), float(up_shift)) if self.Fs else None
        self.shared_up, self.shared_down = Linear(), Linear()
        self.router = self.w_up = self.w_down = self.choice_bias = self.shared_gate = self.router_bias = None

    def tensors(self):
        t = {"router": ParamSpec((self.E, self.hidden))}
        if self.has_choice_bias:
            t["correction"] = ParamSpec((self.E,), "normal")
        if self.has_router_bias:
            t["router_bias"] = ParamSpec((self.E,), "normal")
        for e in range(self.E):
            if self.unit is not None:
                t[f"e{e}.w_gate"] = ParamSpec((self.F, self.hidden))
            t[f"e{e}.w_up"] = ParamSpec((self.F, self.hidden))
            t[f"e{e}.w_down"] = ParamSpec((self.hidden, self.F))
        if self.Fs:
            t.update({"shared.w_gate": ParamSpec((self.Fs, self.hidden)), "shared.w_up": ParamSpec((self.Fs, self.hidden)),
                      "shared.w_down": ParamSpec((self.hidden, self.Fs)), "shared.gate": ParamSpec((1, self.hidden))})
        return t

    def load(self, tensors, device, dtype):
        self.router = upload(tensors["router"], device, torch.float32)
        F, gated = self.F, self.unit is not None
        self.w_up = torch.empty((self.E, 2 * F if gated else F, self.hidden), dtype=dtype, device=device)
        self.w_down = torch.empty((self.E, self.hidden, F), dtype=dtype, device=device)
        for e in range(self.E):                              # one by one: the host holds no stacked copy
            if gated:                                        # an expert's gate rows, then its up rows
                self.w_up[e, :F].copy_(upload(tensors[f"e{e}.w_gate"], device, dtype))
            self.w_up[e, F if gated else 0:].copy_(upload(tensors[f"e{e}.w_up"], device, dtype))
            self.w_down[e].copy_(upload(tensors[f"e{e}.w_down"], device, dtype))
        if self.has_choice_bias:
            self.choice_bias = upload(tensors["correction"], device, torch.float32)
        if self.has_router_bias:
            self.router_bias = upload(tensors["router_bias"], device, torch.float32)
        if self.Fs:
            w = torch.cat([upload(tensors[n], device, dtype) for n in ("shared.w_gate", "shared.w_up")], dim=0).contiguous()
            self.shared_up.load(w, None, device, dtype)
            self.shared_down.load(tensors["shared.w_down"], None, device, dtype)
            self.shared_gate = upload(tensors["shared.gate"], device, torch.float32).reshape(-1).contiguous()

    def linears(self):
        return [self.shared_up, self.shared_down] if self.Fs else []

    def forward(self, h, ctx, lazy_ok: bool = False):
        if isinstance(h, ops.DeferredNorm):
            h = h.materialize()
        routed = ops.moe_route(h, self.router, self.K, self.scoring, self.renormalize, choice_bias=self.choice_bias,
                               weight_floor=self.weight_floor, weight_scale=self.weight_scale, gate=self.shared_gate,
                               logit_bias=self.router_bias)
        ids, wts = routed[0], routed[1]
        experts = ops.moe_experts_grouped if ops.moe_grouped_supported(h.shape[0], self.hidden, self.F, h.dtype) else ops.moe_experts
        y = experts(h, self.w_up, self.w_down, ids, wts, self.activation, self.weight_on_input, gated=self.unit,
                    extra_slabs=1 if self.Fs else 0)
        if self.Fs:
            # the shared expert: its gate (one number a token, formed beside the router's logits) multiplies the unit's
            # output where that is rounded to the activations' type; its result is one more slab of the sum
            act = ops.gated_unit(self.shared_up(h), self.shared_unit, routed[2])
            y.slabs[self.K].copy_(self.shared_down(act, out_dtype=torch.float32))
        return y
