"""Mixers that carry a state of fixed size per sequence instead of keys and values.  The state lives in the cache's
state area (float32, a row per sequence slot, zero when a slot is handed out) and is addressed through the step's
device-side slot ids alone, so decode steps and prompt steps of models with these mixers are captured like any other.
Whatever enters a recurrence is float32 (decays, gates, exponentials, the state); the projections run in the
activations' type.  The kernels are csrc/state_mixers.hip.

"wkv": time mixing with a matrix state per head and a decay that depends on the token.  With h' the previous token's
input (zero before the first token; the last h of a step is part of the state):
    x_s = h + (h' - h) * mu_s                     for s in r, k, v, g, w  (five mixes of the same two rows)
    r, k, v = W_r x_r, W_k x_k, W_v x_v           heads x head_dim each;  gate = silu(W_g x_g)
    w = exp(-exp(W_w2 tanh(W_w1 x_w) + w0))       per head and key channel, in (0, 1)
    o_t = (S + diag(u) k_t v_t^T)^T r_t           the bonus u counts for the current token alone
    S  <- diag(w_t) S + k_t v_t^T
    y = W_o (o / rms_head(o) * norm * gate)       every head divided by its own root mean square (eps inside the root)

"mingru": a gated recurrence whose gates read the current token alone:
    z = sigmoid(W_z h + b_z);  c = W_x h + b_x;  cand = c + 1/2 where c >= 0, sigmoid(c) below
    S <- (1 - z) S + z cand   element by element;   y = W_o (S * silu(W_g h))

"lightning": linear attention with a matrix state per head and a decay that is a constant of the head (csrc/lightning.hip):
    q, k = silu(W_q h), silu(W_k h)   heads x head_dim;   v = silu(W_v h)   heads x v_head_dim
    S <- decay_head S + k_t v_t^T;    o_t = S^T q_t                       no other scale
    y = W_o (o / rms_row(o) * norm * sigmoid(W_g h))                     the heads' outputs normed together, eps inside the root
"""
from __future__ import annotations

import torch

from .. import ops
from .base import MIXERS, CacheNeed, ParamSpec, Part, StateNeed
from .linear import Linear, upload


def _sequences(ctx):
    """How a kernel that walks a sequence's tokens finds them: one tile a sequence in a prompt step, the lengths in a
    decode step (row b is sequence b's one token)."""
    if ctx.is_decode:
        return dict(seq_lens=ctx.seq_lens)
    return dict(tiles=ctx.tiles(ops.SEQUENCE_TILE))


@MIXERS.register("wkv")
class WKV(Part):
    prompt_capturable = True    # a prompt step is read from the context's device tensors alone

    MIXES = ("r", "k", "v", "g", "w")

    def __init__(self, hidden: int, n_heads: int, head_dim: int, decay_rank: int, eps: float):
        self.hidden, self.H, self.hs, self.rank, self.eps = int(hidden), int(n_heads), int(head_dim), int(decay_rank), float(eps)
        if not ops.wkv_supported(self.hs, self.hs):
            raise ValueError(f"wkv: head_dim {self.hs} is not supported by the kernel (at most {ops.WKV_MAX_DIM})")
        self.r, self.k, self.v, self.g, self.w1, self.w2, self.o = (Linear() for _ in range(7))
        self.mu = self.w0 = self.u = self.norm = None

    @property
    def inner(self):
        return self.H * self.hs

    @property
    def state_floats(self):
        return ops.wkv_state_floats(self.H, self.hs, self.hs)

    def tensors(self):
        D, A = self.hidden, self.inner
        t = {f"mu_{s}": ParamSpec((D,), "normal") for s in self.MIXES}
        t.update({"wr": ParamSpec((A, D)), "wk": ParamSpec((A, D)), "wv": ParamSpec((A, D)), "wg": ParamSpec((A, D)),
                  "w1": ParamSpec((self.rank, D)), "w2": ParamSpec((A, self.rank)), "w0": ParamSpec((A,), "normal"),
                  "u": ParamSpec((self.H, self.hs), "normal"), "norm": ParamSpec((A,), "ones"), "wo": ParamSpec((D, A))})
        return t

    def load(self, tensors, device, dtype):
        for lin, n in ((self.r, "wr"), (self.k, "wk"), (self.v, "wv"), (self.g, "wg"), (self.w1, "w1"), (self.w2, "w2"),
                       (self.o, "wo")):
            lin.load(tensors[n], None, device, dtype)
        self.mu = torch.stack([upload(tensors[f"mu_{s}"], device, torch.float32) for s in self.MIXES]).contiguous()
        self.w0 = upload(tensors["w0"], device, torch.float32)
        self.u = upload(tensors["u"], device, torch.float32).reshape(-1).contiguous()
        self.norm = upload(tensors["norm"], device, torch.float32)

    def linears(self):
        return [self.r, self.k, self.v, self.g, self.o]

    def cache_need(self) -> CacheNeed:
        # per head a [head_dim, head_dim] matrix (in the kernel's own order and rounding of its rows), then the last input row
        return CacheNeed(state=StateNeed((self.state_floats + self.hidden,), torch.float32, device_addressed=True))

    def forward(self, h, ctx, kv):
        H, hs = self.H, self.hs
        state = kv.state
        mixes = ops.token_shift(h, self.mu, state[:, self.state_floats:], ctx.positions, ctx.seq_index, ctx.slot_ids)
        r, k, v, g = self.r(mixes[0]), self.k(mixes[1]), self.v(mixes[2]), self.g(mixes[3])
        low = self.w1(mixes[4])
        ops.unary_act(low, "tanh", out=low)
        d = self.w2(low)
        o = ops.wkv_scan(r, k, v, d, self.w0, self.u, h, state, ctx.slot_ids, H, hs, hs, **_sequences(ctx))
        y = ops.head_norm_gate(o, g, self.norm, H, hs, self.eps)
        return self.o(y)


@MIXERS.register("mingru")
class MinGRU(Part):
    prompt_capturable = True    # a prompt step is read from the context's device tensors alone

    def __init__(self, hidden: int, width: int, bias: bool = True):
        self.hidden, self.W, self.has_bias = int(hidden), int(width), bool(bias)
        self.zxg, self.o = Linear(), Linear()         # the three projections stacked: one product
        self.bz = self.bx = None

    def tensors(self):
        D, W = self.hidden, self.W
        t = {"wz": ParamSpec((W, D)), "wx": ParamSpec((W, D)), "wg": ParamSpec((W, D)), "wo": ParamSpec((D, W))}
        if self.has_bias:
            t.update({"bz": ParamSpec((W,), "normal"), "bx": ParamSpec((W,), "normal")})
        return t

    def load(self, tensors, device, dtype):
        w = torch.cat([upload(tensors[n], device, dtype) for n in ("wz", "wx", "wg")], dim=0).contiguous()
        self.zxg.load(w, None, device, dtype)
        self.o.load(tensors["wo"], None, device, dtype)
        if self.has_bias:
            self.bz, self.bx = (upload(tensors[n], device, torch.float32) for n in ("bz", "bx"))

    def linears(self):
        return [self.zxg, self.o]

    def cache_need(self) -> CacheNeed:
        return CacheNeed(state=StateNeed((self.W,), torch.float32, device_addressed=True))

    def forward(self, h, ctx, kv):
        zxg = self.zxg(h)
        y = ops.mingru_scan(zxg, self.bz, self.bx, kv.state, ctx.slot_ids, self.W, **_sequences(ctx))
        return self.o(y)


@MIXERS.register("lightning")
class Lightning(Part):
    prompt_capturable = True    # a prompt step is read from the context's device tensors alone

    def __init__(self, hidden: int, n_heads: int, head_dim: int, decay, eps: float, v_head_dim: int = 0,
                 gate_activation: str = "sigmoid"):
        self.hidden, self.H, self.hs, self.eps = int(hidden), int(n_heads), int(head_dim), float(eps)
        self.vd = int(v_head_dim) or self.hs
        self.decay_values = tuple(float(d) for d in decay)
        if len(self.decay_values) != self.H or not all(0.0 <= d <= 1.0 for d in self.decay_values):
            raise ValueError(f"lightning: one decay in [0, 1] per head, got {len(self.decay_values)} for {self.H} heads")
        if not ops.lightning_supported(self.hs, self.vd):
            raise ValueError(f"lightning: head_dim {self.hs} is not supported by the kernel (at most {ops.LIGHTNING_MAX_DIM})")
        if gate_activation not in ops.UNARY_ACTIVATIONS:
            raise ValueError(f"lightning: unknown gate activation {gate_activation!r}; known: {sorted(ops.UNARY_ACTIVATIONS)}")
        self.gate_activation = gate_activation
        self.qkvg, self.o = Linear(), Linear()        # the four projections stacked: one product
        self.decay = self.norm = None

    @property
    def k_col(self):
        return self.H * self.hs

    @property
    def v_col(self):
        return 2 * self.H * self.hs

    @property
    def g_col(self):
        return 2 * self.H * self.hs + self.H * self.vd

    def tensors(self):
        D, A, B = self.hidden, self.H * self.hs, self.H * self.vd
        return {"wq": ParamSpec((A, D)), "wk": ParamSpec((A, D)), "wv": ParamSpec((B, D)), "wg": ParamSpec((B, D)),
                "norm": ParamSpec((B,), "ones"), "wo": ParamSpec((D, B))}

    def load(self, tensors, device, dtype):
        w = torch.cat([upload(tensors[n], device, dtype) for n in ("wq", "wk", "wv", "wg")], dim=0).contiguous()
        self.qkvg.load(w, None, device, dtype)
        self.o.load(tensors["wo"], None, device, dtype)
        self.norm = upload(tensors["norm"], device, torch.float32)
        self.decay = torch.tensor(self.decay_values, dtype=torch.float64).to(torch.float32).to(device)

    def linears(self):
        return [self.qkvg, self.o]

    def cache_need(self) -> CacheNeed:
        # per head a [head_dim, v_head_dim] matrix, float32
        return CacheNeed(state=StateNeed((self.H * self.hs * self.vd,), torch.float32, device_addressed=True))

    def forward(self, h, ctx, kv):
        x = self.qkvg(h)
        o = ops.lightning_scan(x, 0, self.k_col, self.v_col, self.decay, kv.state, ctx.slot_ids, self.H, self.hs, self.vd,
                               **_sequences(ctx))
        y = ops.row_norm_gate(o, x[:, self.g_col:], self.norm, self.eps, self.gate_activation)
        return self.o(y)


@MIXERS.register("gla")
class GatedLinearAttention(Part):
    """Linear attention with a matrix state per head and a decay per key channel that depends on the token
    (csrc/conv_scans.hip):
        q = W_q h / sqrt(head_dim), k = W_k h   heads x head_dim;   v = W_v h   heads x v_head_dim
        alpha = sigmoid(W_a2 (W_a1 h) + b)^(1 / tau)                 heads x head_dim, float32
        S <- diag(alpha_t) S + k_t v_t^T;   o_t = S^T q_t            the decay acts on the rows of the key channels
        y = W_o (o / rms_head(o) * norm * silu(W_g h))               every head by its own root mean square, norm [v_head_dim]
    The decay's low-rank input rides in the stacked projection; its logits leave their product as float32."""
    prompt_capturable = True    # a prompt step is read from the context's device tensors alone

    def __init__(self, hidden: int, n_heads: int, head_dim: int, v_head_dim: int, decay_rank: int, tau: float, eps: float):
        self.hidden, self.H, self.hs, self.vd = int(hidden), int(n_heads), int(head_dim), int(v_head_dim) or int(head_dim)
        self.rank, self.tau, self.eps = int(decay_rank), float(tau), float(eps)
        if not ops.gla_supported(self.hs, self.vd):
            raise ValueError(f"gla: head_dim {self.hs} is not supported by the kernel (at most {ops.GLA_MAX_DIM})")
        if not self.tau > 0 or self.rank < 1:
            raise ValueError(f"gla: tau {tau} must be positive and the decay's rank {decay_rank} at least 1")
        self.proj, self.a2, self.o = Linear(), Linear(), Linear()        # proj: [W_a1; W_q; W_k; W_v; W_g] stacked
        self.norm = None

    @property
    def q_col(self):
        return self.rank

    @property
    def k_col(self):
        return self.rank + self.H * self.hs

    @property
    def v_col(self):
        return self.rank + 2 * self.H * self.hs

    @property
    def g_col(self):
        return self.rank + 2 * self.H * self.hs + self.H * self.vd

    def tensors(self):
        D, A, B = self.hidden, self.H * self.hs, self.H * self.vd
        return {"wq": ParamSpec((A, D)), "wk": ParamSpec((A, D)), "wv": ParamSpec((B, D)), "wg": ParamSpec((B, D)),
                "wa1": ParamSpec((self.rank, D)), "wa2": ParamSpec((A, self.rank)), "a2_bias": ParamSpec((A,), "normal"),
                "norm": ParamSpec((self.vd,), "ones"), "wo": ParamSpec((D, B))}

    def load(self, tensors, device, dtype):
        w = torch.cat([upload(tensors[n], device, dtype) for n in ("wa1", "wq", "wk", "wv", "wg")], dim=0).contiguous()
        self.proj.load(w, None, device, dtype)
        self.a2.load(tensors["wa2"], tensors["a2_bias"], device, dtype)
        self.o.load(tensors["wo"], None, device, dtype)
        self.norm = upload(tensors["norm"], device, torch.float32).repeat(self.H).contiguous()      # the same for every head

    def linears(self):
        return [self.proj, self.o]

    def cache_need(self) -> CacheNeed:
        # per head a [head_dim, v_head_dim] matrix, float32, row-major
        return CacheNeed(state=StateNeed((self.H * self.hs * self.vd,), torch.float32, device_addressed=True))

    def forward(self, h, ctx, kv):
        x = self.proj(h)
        low = x[:, :self.rank]
        if x.shape[0] > 1 and (x.stride(0) * x.element_size()) % 16:
            low = low.contiguous()
        z = self.a2(low, out_dtype=torch.float32)
        o = ops.gla_scan(x, self.q_col, self.k_col, self.v_col, z, kv.state, ctx.slot_ids, self.H, self.hs, self.vd,
                         self.hs ** -0.5, 1.0 / self.tau, **_sequences(ctx))
        y = ops.head_norm_gate(o, x[:, self.g_col:], self.norm, self.H, self.vd, self.eps)
        return self.o(y)


@MIXERS.register("rglru")
class RealGatedLRU(Part):
    """A recurrent block around a real-gated linear recurrent unit, `width` channels wide (csrc/conv_scans.hip):
        y = gelu_tanh(W_y h + b_y);   u = conv(W_x h + b_x)      a causal convolution per channel with a bias, no activation
        r = sigmoid(A_b u_b + a_b),  i = sigmoid(I_b u_b + i_b)  u in `blocks` equal parts, a square matrix per part
        log a = -sharpness r softplus(lam);  S <- a S + sqrt(1 - a^2) i u     from S = 0, the first token like any other
        out = W_o (S * y)
    The gates, a, the unit's operands and S are float32 (the gate matrices are kept in float32, turned to [in, out]); the
    state row holds S, then the convolution's last taps - 1 inputs."""
    prompt_capturable = True    # a prompt step is read from the context's device tensors alone

    def __init__(self, hidden: int, width: int, blocks: int, conv_taps: int, sharpness: float = 8.0):
        self.hidden, self.W, self.blocks, self.taps = int(hidden), int(width), int(blocks), int(conv_taps)
        self.sharpness = float(sharpness)
        if self.blocks < 1 or self.W % self.blocks:
            raise ValueError(f"rglru: {width} channels are not {blocks} equal parts")
        if not 1 <= self.taps <= ops.CONV_MAX_TAPS:
            raise ValueError(f"rglru: conv_taps {conv_taps} (1 to {ops.CONV_MAX_TAPS})")
        self.yx, self.o = Linear(), Linear()          # yx: [W_y; W_x] stacked with their biases
        self.conv_w = self.conv_b = self.wa_t = self.wi_t = self.ba = self.bi = self.c_neg = None

    def tensors(self):
        D, W, B, bw = self.hidden, self.W, self.blocks, self.W // self.blocks
        return {"wy": ParamSpec((W, D)), "by": ParamSpec((W,), "normal"), "wx": ParamSpec((W, D)), "bx": ParamSpec((W,), "normal"),
                "conv": ParamSpec((W, self.taps)), "conv_bias": ParamSpec((W,), "normal"),
                "ra": ParamSpec((B, bw, bw)), "ra_bias": ParamSpec((B, bw), "normal"),
                "ri": ParamSpec((B, bw, bw)), "ri_bias": ParamSpec((B, bw), "normal"),
                "lam": ParamSpec((W,), "normal"), "wo": ParamSpec((D, W))}

    def load(self, tensors, device, dtype):
        w = torch.cat([upload(tensors[n], device, dtype) for n in ("wy", "wx")], dim=0).contiguous()
        b = torch.cat([upload(tensors[n], device, torch.float32) for n in ("by", "bx")])
        self.yx.load(w, b, device, dtype)
        self.o.load(tensors["wo"], None, device, dtype)
        self.conv_w = upload(tensors["conv"], device, torch.float32)
        self.conv_b = upload(tensors["conv_bias"], device, torch.float32)
        self.wa_t = upload(tensors["ra"], device, torch.float32).transpose(1, 2).contiguous()
        self.wi_t = upload(tensors["ri"], device, torch.float32).transpose(1, 2).contiguous()
        self.ba = upload(tensors["ra_bias"], device, torch.float32).reshape(-1).contiguous()
        self.bi = upload(tensors["ri_bias"], device, torch.float32).reshape(-1).contiguous()
        lam = tensors["lam"].detach().to("cpu").to(torch.float64)
        self.c_neg = (-self.sharpness * torch.nn.functional.softplus(lam)).to(torch.float32).to(device)

    def linears(self):
        return [self.yx, self.o]

    def cache_need(self) -> CacheNeed:
        return CacheNeed(state=StateNeed((self.W * self.taps,), torch.float32, device_addressed=True))

    def forward(self, h, ctx, kv):
        W = self.W
        yx = self.yx(h)                                   # [T, 2 W]: the y branch before its gelu, then the convolution's input
        seqs = _sequences(ctx)
        conv_state = kv.state[:, W:] if self.taps > 1 else kv.state
        u = ops.short_conv(yx, W, self.conv_w, self.conv_b, conv_state, ctx.positions, ctx.seq_index, ctx.slot_ids,
                           out_dtype=torch.float32, **seqs)
        a, b = ops.lru_gates(u, self.wa_t, self.ba, self.wi_t, self.bi, self.c_neg)
        out = ops.lru_scan(a, b, yx[:, :W], kv.state, ctx.slot_ids, **seqs)
        return self.o(out)
