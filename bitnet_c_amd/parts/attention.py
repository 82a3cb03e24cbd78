"""Attention mixer: grouped-query attention over the paged cache.

Order of the reference's layer (src/transformer/cpu.c:770-939): Q, K, V projections
(+ bias when the tensors exist) -> position encoding of Q and K -> K, V into the cache
-> for head h, kv head h / (H/Hkv): scores (q.k) * scale over the visible keys, softmax,
weighted sum of values -> output projection.  scale is a parameter (1/sqrt(head_dim)
for this architecture, src/model_arch.c:141-145); `window` > 0 limits the visible keys
to the last `window` positions.

The three projections are stored stacked ([Wq; Wk; Wv], as the reference's GPU upload
stacks them, include/backend_model.h:21-22) so that one product computes them.
A schedule entry that reads another entry's cache computes Q only.

What other architectures put into the same mixer, each a parameter that is off by default; any of them takes the
mixer to its general form: one kernel norms, rotates and stores (ops.qk_norm_store), attention reads pages with a key
row per position and transposed values, in both types.  The general form rotates by itself (any "rope" position, in
split-half or in neighbouring pairs, over the first rope_dims dimensions) and takes a window:
  v_head_dim     value heads of another width than the query/key heads
  qk_norm_eps    an RMSNorm over every query and every key head before they meet (tensors q_norm, k_norm [head_dim],
                 shared by the heads, plain weights); with qk_norm_span "projection" one norm over the whole query
                 projection and one over the whole key projection instead (q_norm [heads head_dim], k_norm
                 [kv heads head_dim]), before the heads are split and before the rotation
  a "rope" position with interleaved=True: pairs (2i, 2i + 1) instead of (i, i + rope_dims / 2)
  q_temp_coef, q_temp_every   the query at position p times 1 + coef * ln(floor((p + 1) / every) + 1)
  distance_bias  tensors dist_a, dist_b [heads]: dist_a[h] * ln(1 + dist_b[h] * (i - j)) is taken off the score of
                 query i and key j
  sink           the softmax has one more term of score 0 and no value: p_j = exp(s_j) / (1 + sum exp(s)); "learned": the
                 term's score is a number per head (tensor sink [heads]): p_j = exp(s_j) / (exp(sink_h) + sum exp(s))
  conv_taps      a short causal convolution over time on every channel of the query and key projections, directly behind the
                 projection (tensors q_conv [heads head_dim, taps], k_conv [kv heads head_dim, taps], no bias; the last
                 column meets the current token, zeros before a sequence's first token); with value_is_key the values are
                 the keys as they leave it.  A sequence's last taps - 1 projected rows are a state beside its pages.
  value_is_key   there is no value projection: kv head g's value is its key projection as projected, before the key's norm
                 and rotation (the tensor wv does not exist; the value heads are as wide as the key heads)
"""
from __future__ import annotations

import torch

from .. import ops
from .base import MIXERS, POSITION_ENCODINGS, CacheNeed, KVNeed, ParamSpec, Part, PartSpec, StateNeed
from .linear import Linear, upload


@MIXERS.register("attention")
class Attention(Part):
    @property
    def prompt_capturable(self) -> bool:      # a prompt step is read from the context's device tensors alone
        return getattr(self.position, "prompt_capturable", False)

    takes_deferred_norm = True      # forward accepts an ops.DeferredNorm for h
    gives_lazy_delta = True         # forward(..., lazy_ok=True) may return a LazyDelta

    def __init__(self, hidden: int, n_heads: int, n_kv_heads: int, head_dim: int, scale: float,
                 position: PartSpec, window: int = 0, bias: bool = False, v_head_dim: int = 0,
                 qk_norm_eps: float | None = None, q_temp_coef: float = 0.0, q_temp_every: int = 0,
                 distance_bias: bool = False, sink=False, qk_norm_span: str = "head", value_is_key: bool = False,
                 conv_taps: int = 0):
        if n_heads % n_kv_heads:
            raise ValueError(f"attention: {n_heads} heads are not a multiple of {n_kv_heads} kv heads")
        if head_dim % 2 or head_dim < 2 or head_dim > ops.MAX_HEAD_DIM:
            raise ValueError(f"attention: head_dim {head_dim} is not supported by the kernels "
                             f"(even, at most {ops.MAX_HEAD_DIM})")
        self.hidden, self.H, self.Hkv, self.hs = int(hidden), int(n_heads), int(n_kv_heads), int(head_dim)
        self.scale, self.window, self.has_bias = float(scale), int(window), bool(bias)
        self.position = POSITION_ENCODINGS.build(position)
        self.qkv, self.o = Linear(), Linear()
        self.vd = int(v_head_dim) or self.hs
        self.value_is_key = bool(value_is_key)
        if self.value_is_key and self.vd != self.hs:
            raise ValueError(f"attention: values that are the keys are as wide as the keys, got {self.vd} and {self.hs}")
        self.qk_norm_eps = None if qk_norm_eps is None else float(qk_norm_eps)
        self.q_temp_coef, self.q_temp_every = float(q_temp_coef), int(q_temp_every)
        if sink not in (False, True, "learned"):
            raise ValueError(f"attention: sink {sink!r} is neither False, True nor 'learned'")
        self.distance_bias, self.sink, self.sink_learned = bool(distance_bias), bool(sink), sink == "learned"
        self.conv_taps = int(conv_taps)
        if self.conv_taps < 0 or self.conv_taps > ops.CONV_MAX_TAPS:
            raise ValueError(f"attention: conv_taps {conv_taps} (at most {ops.CONV_MAX_TAPS})")
        if qk_norm_span not in ("head", "projection"):
            raise ValueError(f"attention: qk_norm_span {qk_norm_span!r} is neither 'head' nor 'projection'")
        self.norm_projection = qk_norm_span == "projection"
        if self.norm_projection and self.qk_norm_eps is None:
            raise ValueError("attention: a norm over the whole projection needs qk_norm_eps")
        self.general = (self.vd != self.hs or self.qk_norm_eps is not None or self.q_temp_every > 0
                        or self.distance_bias or self.sink or getattr(self.position, "interleaved", False)
                        or self.value_is_key or self.conv_taps > 0)
        if self.general:
            if self.vd % 2 or self.vd < 2 or self.vd > ops.MAX_HEAD_DIM:
                raise ValueError(f"attention: v_head_dim {self.vd} is not supported by the kernels (even, at most {ops.MAX_HEAD_DIM})")
            if self.has_bias:
                raise ValueError("attention: head norms, a query temperature, a distance bias, a sink, a rotation in neighbouring "
                                 "pairs, values of another width or values that are the keys come without projection biases")
            self.takes_deferred_norm = self.gives_lazy_delta = False
        self.q_norm = self.k_norm = self.dist_a = self.dist_b = self.sink_values = self.conv_w = None

    @property
    def q_dim(self):
        return self.H * self.hs

    @property
    def kv_dim(self):
        return self.Hkv * self.hs

    def tensors(self):
        t = {"wq": ParamSpec((self.q_dim, self.hidden)), "wk": ParamSpec((self.kv_dim, self.hidden)),
             "wv": ParamSpec((self.Hkv * self.vd, self.hidden)), "wo": ParamSpec((self.hidden, self.H * self.vd))}
        if self.value_is_key:
            del t["wv"]
        if self.qk_norm_eps is not None:
            nq, nk = (self.q_dim, self.kv_dim) if self.norm_projection else (self.hs, self.hs)
            t.update({"q_norm": ParamSpec((nq,), "ones"), "k_norm": ParamSpec((nk,), "ones")})
        if self.distance_bias:
            t.update({"dist_a": ParamSpec((self.H,), "normal"), "dist_b": ParamSpec((self.H,), "ones")})
        if self.sink_learned:
            t["sink"] = ParamSpec((self.H,), "normal")
        if self.conv_taps:
            t.update({"q_conv": ParamSpec((self.q_dim, self.conv_taps)), "k_conv": ParamSpec((self.kv_dim, self.conv_taps))})
        if self.has_bias:
            t.update({"bq": ParamSpec((self.q_dim,), "normal"), "bk": ParamSpec((self.kv_dim,), "normal"),
                      "bv": ParamSpec((self.kv_dim,), "normal"), "bo": ParamSpec((self.hidden,), "normal")})
        return t

    def load(self, tensors, device, dtype):
        # stacked on the device: the host holds no copy beside the file's own bytes
        stacked = ("wq", "wk") if self.value_is_key else ("wq", "wk", "wv")
        w = torch.cat([upload(tensors[n], device, dtype) for n in stacked], dim=0).contiguous()
        b = None
        if self.has_bias:
            b = torch.cat([upload(tensors[n], device, torch.float32) for n in ("bq", "bk", "bv")])
        self.qkv.load(w, b, device, dtype)
        self.o.load(tensors["wo"], tensors.get("bo") if self.has_bias else None, device, dtype)
        self.position.prepare(device)
        if self.qk_norm_eps is not None:
            self.q_norm, self.k_norm = (upload(tensors[n], device, torch.float32) for n in ("q_norm", "k_norm"))
        if self.distance_bias:
            self.dist_a, self.dist_b = (upload(tensors[n], device, torch.float32) for n in ("dist_a", "dist_b"))
        if self.sink_learned:
            self.sink_values = upload(tensors["sink"], device, torch.float32)
        if self.conv_taps:
            self.conv_w = torch.cat([upload(tensors[n], device, torch.float32) for n in ("q_conv", "k_conv")], dim=0).contiguous()

    def linears(self):
        return [self.qkv, self.o]

    def cache_need(self) -> CacheNeed:
        if self.general:                  # keys a row per position, values transposed inside a page, in both types: what the
            # vector kernel and the general prompt kernel on the matrix cores both read
            state = None
            if self.conv_taps > 1:        # the projected query and key rows of the last taps - 1 positions, float32
                state = StateNeed(((self.conv_taps - 1) * (self.q_dim + self.kv_dim),), torch.float32, device_addressed=True)
            return CacheNeed(kv=KVNeed(self.Hkv, self.hs, self.window, v_head_dim=self.vd, v_layout="transposed"), state=state)
        return CacheNeed(kv=KVNeed(self.Hkv, self.hs, self.window))

    def wants_deferred_norm(self, ctx, rows: int) -> bool:
        """With more rows than the fused product takes, the norm's factor can only go into the decode kernel that
        rotates by itself (forward); a prompt step is better served by the plain norm."""
        if rows <= ops.FUSED_ROWS:
            return True
        fuse_ok, inv_freq = self.position.fusable(self.hs)
        return bool(ctx.is_decode and fuse_ok and inv_freq is not None and not self.has_bias and ops.LIBRARY_PRODUCTS
                    and ops.can_fuse_decode(self.qkv.weight.dtype, self.H, self.Hkv, self.hs))

    def _forward_general(self, h, ctx, kv):
        """Projections; norms, rotation and temperature with the cache write (one kernel); attention with its window,
        distance bias and sink (prompt steps on the matrix cores where the sizes allow, else the vector kernel); the
        output projection."""
        H, Hkv, hs, vd = self.H, self.Hkv, self.hs, self.vd
        if isinstance(h, ops.DeferredNorm):
            h = h.materialize()
        width = H * hs + Hkv * (hs if self.value_is_key else hs + vd)
        if kv.writes:
            qkv = self.qkv(h)
        else:
            qkv = torch.empty((h.shape[0], width), dtype=h.dtype, device=h.device)
            qkv[:, :self.q_dim] = self.qkv(h, rows=slice(0, self.q_dim))
        if self.conv_taps:
            if not kv.writes:
                raise ValueError("attention: a convolution on the projections needs the layer's own keys")
            seqs = dict(seq_lens=ctx.seq_lens) if ctx.is_decode else dict(tiles=ctx.tiles(ops.SEQUENCE_TILE))
            state = kv.state if kv.state is not None else self._no_state(qkv.device)     # one tap keeps nothing
            qk = ops.short_conv(qkv, 0, self.conv_w, None, state, ctx.positions, ctx.seq_index, ctx.slot_ids, **seqs)
            if self.value_is_key:
                qkv = qk
            else:
                qkv[:, :self.q_dim + self.kv_dim].copy_(qk)
        ops.qk_norm_store(qkv, ctx.positions, H, Hkv, hs, v_dim=vd, q_weight=self.q_norm, k_weight=self.k_norm,
                          eps=self.qk_norm_eps or 0.0, temp_coef=self.q_temp_coef, temp_every=self.q_temp_every,
                          norm_projection=self.norm_projection, inv_freq=self.position.inv_freq,
                          rope_dims=self.position.rope_dims, rope_interleaved=getattr(self.position, "interleaved", False),
                          seq_index=ctx.seq_index if kv.writes else None, block_table=kv.block_table if kv.writes else None,
                          k_pages=kv.k_pages if kv.writes else None, v_pages=kv.v_pages if kv.writes else None,
                          v_transposed=True, v_from_k=self.value_is_key)
        out = torch.empty((h.shape[0], H * vd), dtype=h.dtype, device=h.device)
        bias = (self.dist_a, self.dist_b) if self.distance_bias else None
        on_matrix_cores = (ops.attention_general_supported(h.dtype, hs, vd) and ops.GENERAL_PROMPT_ON_MATRIX_CORES
                           and width % 8 == 0 and qkv.data_ptr() % 16 == 0)
        if ctx.is_decode and on_matrix_cores:
            n_splits, chunk, follows = ops.general_decode_plan(ctx.n_rows, H, Hkv, kv.max_len, self.window)
            ops.attention_general_decode(qkv, out, kv.k_pages, kv.v_pages, kv.block_table, ctx.seq_lens, H, Hkv, hs, vd, self.scale,
                                         window=self.window, n_splits=n_splits, chunk=chunk,
                                         max_len_dev=ctx.max_len_dev if follows and n_splits > 1 else None,
                                         distance_bias=bias, sink=self._sink())
        elif ctx.is_decode:
            if not self.window:
                n_splits, chunk = ops.decode_splits(ctx.n_rows, H, Hkv, kv.max_len, h.dtype, target_wgs=ops.VECTOR_DECODE_TARGET_WGS)
            elif h.dtype == torch.bfloat16 and self.window >= 4 * ops.PAGE:
                # a long window is cut like a sequence of its own length: the kernel counts the splits from the window's
                # first page, so the plan depends on the window alone and serves every length (also a captured step's)
                n_splits, chunk = ops.decode_splits(ctx.n_rows, H, Hkv, self.window + ops.PAGE, h.dtype,
                                                    target_wgs=ops.VECTOR_DECODE_TARGET_WGS)
            else:
                n_splits, chunk = 1, 0                    # a short window is not split; a float32 cache sums in runs from position 0
            ops.attention(qkv, out, kv.k_pages, kv.v_pages, kv.block_table, H, Hkv, hs, self.scale, window=self.window,
                          seq_lens=ctx.seq_lens, n_splits=n_splits, chunk=chunk,
                          max_len_dev=ctx.max_len_dev if n_splits > 1 and not self.window else None, v_transposed=True, blocked=False,
                          v_dim=vd, distance_bias=bias, sink=self._sink())
        elif on_matrix_cores:
            ops.attention_general_prompt(qkv, out, kv.k_pages, kv.v_pages, kv.block_table, H, Hkv, hs, vd, self.scale,
                                         ctx.tiles(ops.GENERAL_PROMPT_TILE), distance_bias=bias, sink=self._sink(),
                                         window=self.window)
        else:
            _, _, qt = ops.attention_row_shape(H, Hkv, False)
            ops.attention(qkv, out, kv.k_pages, kv.v_pages, kv.block_table, H, Hkv, hs, self.scale, window=self.window,
                          tiles=ctx.tiles(qt), qt=qt, v_transposed=True, blocked=False, v_dim=vd, distance_bias=bias,
                          sink=self._sink())
        return self.o(out)

    def _sink(self):
        return self.sink_values if self.sink_learned else self.sink

    def _no_state(self, device):
        """What a convolution of one tap is handed for a state when the entry has none: it is never read."""
        if getattr(self, "_empty_state", None) is None:
            self._empty_state = torch.zeros((1, 1), dtype=torch.float32, device=device)
        return self._empty_state

    def forward(self, h, ctx, kv, lazy_ok: bool = False):
        if self.general:
            return self._forward_general(h, ctx, kv)
        H, Hkv, hs = self.H, self.Hkv, self.hs
        last = self.o.lazy if lazy_ok else self.o
        fuse_ok, inv_freq = self.position.fusable(hs)
        vt, blocked = kv.v_transposed, bool(kv.blocked)
        decode_fused = (ctx.is_decode and fuse_ok and ops.can_fuse_decode(self.qkv.weight.dtype, H, Hkv, hs)
                        and blocked)                            # the matrix-core kernels read blocked pages
        row_scale = None
        if isinstance(h, ops.DeferredNorm) and h.shape[0] > ops.FUSED_ROWS:
            # More rows than the fused product takes.  When the decode kernel rotates by itself it can apply the norm's
            # factor as well (it multiplies whole rows of q, k and v): the library's product of the copy, then that
            # kernel.  Else the norm is applied the plain way.
            if decode_fused and inv_freq is not None and not self.has_bias and kv.writes and ops.LIBRARY_PRODUCTS:
                row_scale, h = h, h.scaled
            else:
                h = h.materialize()
        if kv.writes:
            qkv = self.qkv(h)                                   # [T, (H + 2 Hkv) hs]
        else:
            qkv = self.qkv(h, rows=slice(0, self.q_dim))        # Q alone
            pad = torch.empty((h.shape[0], (H + 2 * Hkv) * hs), dtype=h.dtype, device=h.device)
            pad[:, :self.q_dim] = qkv
            qkv = pad
        out = torch.empty((h.shape[0], self.q_dim), dtype=h.dtype, device=h.device)
        if decode_fused:
            # one kernel: rotation of Q and the new K, the cache write, attention, merge of the splits
            if self.window:
                n_splits, chunk = 1, 0
            else:
                n_splits, chunk = ops.decode_splits(ctx.n_rows, H, Hkv, kv.max_len, h.dtype)
            ops.attention(qkv, out, kv.k_pages, kv.v_pages, kv.block_table, H, Hkv, hs, self.scale,
                          window=self.window, seq_lens=ctx.seq_lens, n_splits=n_splits, chunk=chunk,
                          fused_rotate=inv_freq, fused_write=kv.writes, by_length=ctx.by_length,
                          max_len_dev=ctx.max_len_dev if n_splits > 1 else None, v_transposed=vt, blocked=blocked,
                          row_scale=row_scale)
            return last(out)
        self.position.encode_and_store(qkv, ctx, H, Hkv, hs, kv)
        if ctx.is_decode:
            if self.window:                   # a window is short; its keys are not split
                n_splits, chunk = 1, 0
            else:
                n_splits, chunk = ops.decode_splits(ctx.n_rows, H, Hkv, kv.max_len, h.dtype)
            ops.attention(qkv, out, kv.k_pages, kv.v_pages, kv.block_table, H, Hkv, hs, self.scale,
                          window=self.window, seq_lens=ctx.seq_lens, n_splits=n_splits, chunk=chunk,
                          by_length=ctx.by_length, max_len_dev=ctx.max_len_dev if n_splits > 1 else None,
                          v_transposed=vt, blocked=blocked)
        else:
            # pages in another order than the matrix-core kernels' own: the vector kernel, with its tiles
            _, _, qt = ops.attention_row_shape(H, Hkv, False, h.dtype if blocked else None, hs)
            ops.attention(qkv, out, kv.k_pages, kv.v_pages, kv.block_table, H, Hkv, hs, self.scale,
                          window=self.window, tiles=ctx.tiles(qt), qt=qt, v_transposed=vt, blocked=blocked)
        return last(out)
