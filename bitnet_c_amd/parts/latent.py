"""Latent attention: causal attention without positions whose keys and values are projections of one vector per token.

With h the mixer's input, per head i of n_heads (query/key size head_dim, value size v_head_dim):
    q_i = W_q,i h
    c   = rmsnorm(W_dkv h) * dkv_norm          the latent, kv_rank wide; eps inside the root, float32
    k_i = W_uk,i c;   v_i = W_uv,i c
    o_i = sum_j softmax_j((q_i . k_i,j) * scale) v_i,j       over the positions j <= the query's
    y   = W_o (concat(o) * sigmoid(W_g h))     the gate reads the mixer's input (gate False: no gate)

Only c is kept: the cache holds it as the one "kv head" of an attention whose keys and values are the same vectors
(a key row per position and, for the kernels' second product, the same numbers transposed inside the page).  Since k and
v are linear in c the mixer never forms them: the query goes into the latent's space, q'_i = W_uk,i^T q_i, all heads attend
over the cached c (score = q'_i . c_j), and the value projection runs on the attended latent, o_i = W_uv,i (sum_j p_j c_j).
That is the same sum in another order; scores, softmax and the norm are float32, the products accumulate in float32.
The attention itself is the attention mixer's general form (ops.attention / ops.attention_general_prompt) with one kv
head of size kv_rank and values as wide.

Options, each off by default:
  q_rank      the queries go through a latent of their own: c_q = rmsnorm(W_dq h) * dq_norm, q = W_uq c_q (tensors wdq, dq_norm,
              wuq instead of wq)
  rot_dim     every query head is [head_dim plain, rot_dim rotated] and W_dkv h has rot_dim more rows behind the latent's: one
              rotated key part that all heads share, not normed.  The score is (q_plain . k_plain + q_rot . k_rot) * scale.  The
              rotation turns dimension i with dimension i + rot_dim / 2 by position * f_i (rot_theta, rot_scaling as
              parts/position.py's; a "yarn" scaling also multiplies cosine and sine).  The cache's key row is then
              [c, k_rot] (kv_rank + rot_dim wide) and the query in the latent's space [W_uk^T q_plain, q_rot]; values stay c.
  gate        "head": one gate number per head, sigmoid(W_g h)_i multiplies head i's output (wg [heads, hidden])

own_latent False: the layer has no W_dkv; its schedule entry reads the cache of the entry that has (ScheduleEntry.kv_from),
with its own W_uk and W_uv, queries, gate and output projection.
"""
from __future__ import annotations

import torch

from .. import ops
from .base import MIXERS, CacheNeed, KVNeed, ParamSpec, Part
from .linear import Linear, upload
from .position import rope_frequencies, rope_magnitude


@MIXERS.register("latent_attention")
class LatentAttention(Part):
    prompt_capturable = True    # a prompt step is read from the context's device tensors alone

    def __init__(self, hidden: int, n_heads: int, head_dim: int, kv_rank: int, scale: float, eps: float,
                 v_head_dim: int = 0, own_latent: bool = True, gate=True, q_rank: int = 0, rot_dim: int = 0,
                 rot_theta: float = 10000.0, rot_scaling=None):
        self.hidden, self.H, self.hs, self.rank = int(hidden), int(n_heads), int(head_dim), int(kv_rank)
        self.vd = int(v_head_dim) or self.hs
        if gate not in (False, True, "head"):
            raise ValueError(f"latent attention: gate {gate!r} is neither False, True nor 'head'")
        self.scale, self.eps, self.own, self.gated = float(scale), float(eps), bool(own_latent), bool(gate)
        self.gate_per_head = gate == "head"
        self.q_rank, self.rot = int(q_rank), int(rot_dim)
        if self.rot % 2 or self.rot < 0 or self.q_rank < 0:
            raise ValueError(f"latent attention: rot_dim {rot_dim} must be even and q_rank {q_rank} not negative")
        self.kw = self.rank + self.rot               # width of a cached key row: the latent, then the rotated part
        if self.rank % 2 or self.rank < 2 or self.kw > ops.MAX_HEAD_DIM:
            raise ValueError(f"latent attention: kv_rank {self.rank} (+ rot_dim {self.rot}) is not supported by the attention "
                             f"kernels (even, at most {ops.MAX_HEAD_DIM})")
        if max(self.hs + self.rot, self.rank) > ops.HEAD_LINEAR_MAX_IN:
            raise ValueError(f"latent attention: head_dim {self.hs} / kv_rank {self.rank} above {ops.HEAD_LINEAR_MAX_IN}")
        self.rot_scaling = dict(rot_scaling) if rot_scaling else None
        self.rot_mult = rope_magnitude(self.rot_scaling)
        self._freq_host = rope_frequencies(self.rot, float(rot_theta), self.rot_scaling) if self.rot else None
        self.inv_freq = self.dq_norm = None
        self.uq = Linear()                          # W_uq when the queries have a latent of their own
        self.proj, self.o = Linear(), Linear()      # proj: [W_q (or W_dq); W_g; W_dkv] stacked, one product
        self.uk = self.uv_t = self.dkv_norm = None   # [H, head_dim, rank] and [H, rank, v_head_dim]: both [head, in, out]

    @property
    def q_dim(self):
        return self.H * (self.hs + self.rot)

    @property
    def g_dim(self):
        return 0 if not self.gated else self.H if self.gate_per_head else self.o_dim

    @property
    def o_dim(self):
        return self.H * self.vd

    def tensors(self):
        D = self.hidden
        if self.q_rank:
            t = {"wdq": ParamSpec((self.q_rank, D)), "dq_norm": ParamSpec((self.q_rank,), "ones"),
                 "wuq": ParamSpec((self.q_dim, self.q_rank))}
        else:
            t = {"wq": ParamSpec((self.q_dim, D))}
        t.update({"wuk": ParamSpec((self.H * self.hs, self.rank)), "wuv": ParamSpec((self.o_dim, self.rank)),
                  "wo": ParamSpec((D, self.o_dim))})
        if self.gated:
            t["wg"] = ParamSpec((self.g_dim, D))
        if self.own:
            t.update({"wdkv": ParamSpec((self.kw, D)), "dkv_norm": ParamSpec((self.rank,), "ones")})
        return t

    def load(self, tensors, device, dtype):
        # the products that read h, stacked: [W_dq or W_q; W_g; W_dkv]
        names = ["wdq" if self.q_rank else "wq"] + (["wg"] if self.gated else []) + (["wdkv"] if self.own else [])
        w = torch.cat([upload(tensors[n], device, dtype) for n in names], dim=0).contiguous()
        self.proj.load(w, None, device, dtype)
        if self.q_rank:
            self.uq.load(tensors["wuq"], None, device, dtype)
            self.dq_norm = upload(tensors["dq_norm"], device, torch.float32)
        self.o.load(tensors["wo"], None, device, dtype)
        # W_uk of head i is [head_dim, rank]: already [in, out] for q' = W_uk^T q; W_uv of head i is [v_head_dim, rank]:
        # turned once to [rank, v_head_dim].  With a rotated part a head's matrix gets rot_dim more rows and columns that
        # hand the rotated query dimensions on as they are (an identity block), so one product per head makes the whole
        # query of the latent's space.
        uk = upload(tensors["wuk"], device, dtype).reshape(self.H, self.hs, self.rank)
        if self.rot:
            full = torch.zeros((self.H, self.hs + self.rot, self.kw), dtype=dtype, device=uk.device)
            full[:, :self.hs, :self.rank] = uk
            full[:, self.hs:, self.rank:] = torch.eye(self.rot, dtype=dtype, device=uk.device)
            uk = full
            self.inv_freq = self._freq_host.to(device).contiguous()
        self.uk = uk.contiguous()
        self.uv_t = upload(tensors["wuv"], device, dtype).reshape(self.H, self.vd, self.rank).transpose(1, 2).contiguous()
        if self.own:
            self.dkv_norm = upload(tensors["dkv_norm"], device, torch.float32)

    def linears(self):
        return [self.proj, self.o] + ([self.uq] if self.q_rank else [])

    def cache_need(self) -> CacheNeed:
        return CacheNeed(kv=KVNeed(1, self.kw, 0, v_head_dim=self.rank, v_layout="transposed"))

    def forward(self, h, ctx, kv):
        H, hs, vd, R = self.H, self.hs, self.vd, self.rank
        if isinstance(h, ops.DeferredNorm):
            h = h.materialize()
        if kv.writes != self.own:
            raise ValueError("latent attention: a layer with a down-projection writes its own cache, one without reads another's")
        p = self.proj(h)                                    # [T, q columns (+ gate columns) (+ R + rot)]
        q_cols = self.q_rank or self.q_dim
        if self.own:
            ops.latent_store(p, q_cols + self.g_dim, R, self.dkv_norm, self.eps, ctx.positions,
                             ctx.seq_index, kv.block_table, kv.k_pages, kv.v_pages, rot_dims=self.rot, inv_freq=self.inv_freq,
                             rot_mult=self.rot_mult)
        if self.q_rank:
            cq = p[:, :q_cols].contiguous() if p.shape[1] != q_cols else p
            qh = self.uq(ops.rmsnorm_mean(cq, self.dq_norm, None, None, self.eps))       # [T, H (hs + rot)]
        else:
            qh = p[:, :q_cols]
        KW = self.kw
        q = ops.head_linear(qh, self.uk)                     # [T, H KW]: the queries in the latent's space
        if self.rot:
            ops.rope_heads(q, ctx.positions, self.inv_freq, H, KW, R, self.rot, self.rot_mult)
        out = torch.empty((h.shape[0], H * R), dtype=h.dtype, device=h.device)
        on_matrix_cores = ops.attention_general_supported(h.dtype, KW, R) and ops.GENERAL_PROMPT_ON_MATRIX_CORES
        if ctx.is_decode and on_matrix_cores:
            n_splits, chunk, _ = ops.general_decode_plan(ctx.n_rows, H, 1, kv.max_len)
            ops.attention_general_decode(q, out, kv.k_pages, kv.v_pages, kv.block_table, ctx.seq_lens, H, 1, KW, R, self.scale,
                                         n_splits=n_splits, chunk=chunk, max_len_dev=ctx.max_len_dev if n_splits > 1 else None)
        elif ctx.is_decode:
            n_splits, chunk = ops.decode_splits(ctx.n_rows, H, 1, kv.max_len, h.dtype, target_wgs=ops.VECTOR_DECODE_TARGET_WGS)
            ops.attention(q, out, kv.k_pages, kv.v_pages, kv.block_table, H, 1, KW, self.scale, seq_lens=ctx.seq_lens,
                          n_splits=n_splits, chunk=chunk, max_len_dev=ctx.max_len_dev if n_splits > 1 else None,
                          v_transposed=True, blocked=False, v_dim=R)
        elif on_matrix_cores:
            ops.attention_general_prompt(q, out, kv.k_pages, kv.v_pages, kv.block_table, H, 1, KW, R, self.scale,
                                         ctx.tiles(ops.GENERAL_PROMPT_TILE))
        else:
            _, _, qt = ops.attention_row_shape(H, 1, False)
            ops.attention(q, out, kv.k_pages, kv.v_pages, kv.block_table, H, 1, KW, self.scale, tiles=ctx.tiles(qt), qt=qt,
                          v_transposed=True, blocked=False, v_dim=R)
        gate = p[:, q_cols:q_cols + self.g_dim] if self.gated else None
        return self.o(ops.head_linear(out, self.uv_t, gate, gate_per_head=self.gate_per_head))
