"""Checked Python entry points of the HIP kernels.

Every function here validates shapes, dtypes, devices and strides on the host before it
launches anything: a kernel is never handed operands that its indexing does not expect.
There is no other implementation behind these functions: without a GPU, or when the
kernels cannot be compiled, they raise.  Kernels run on torch's current stream, so a
step can be captured into a HIP graph.
"""
from __future__ import annotations

import os
from ctypes import c_float, c_int, c_longlong, c_void_p
from dataclasses import dataclass
from typing import Optional

import torch

from .csrc import build as _build

PAGE = _build.header_constant("BN_PAGE")                         # tokens per cache page: defined once, in csrc/common.h
F32_FOLD_KEYS = _build.header_constant("BN_F32_FOLD_KEYS")       # a float32 cache's keys are summed in runs of this many
SPLIT_MIN_PAGES = _build.header_constant("BN_SPLIT_MIN_PAGES")   # shortest run of pages that decode attention splits off
_DT = {torch.float32: 0, torch.bfloat16: 1}


class KernelError(RuntimeError):
    pass


_SIGNATURES = {
    "elementwise": {
        "bn_embed_gather": [c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_float, c_void_p],
        "bn_softcap": [c_void_p, c_longlong, c_float, c_void_p],
        "bn_gather_rows": [c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p],
        "bn_add_rmsnorm": [c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_float, c_void_p],
        "bn_residual_add": [c_int, c_void_p, c_void_p, c_longlong, c_void_p],
        "bn_add_rmsnorm_parts": [c_int, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                 c_float, c_void_p],
        "bn_residual_add_parts": [c_void_p, c_void_p, c_int, c_longlong, c_void_p],
        "bn_add_rmsnorm_parts_pieces": [c_int],
        "bn_add_rmsnorm_parts_wide": [c_int, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_int, c_float,
                                      c_void_p],
        "bn_swiglu": [c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
        "bn_sum_deferred": [c_int, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p],
        "bn_swiglu_scaled": [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_int, c_float, c_void_p],
        "bn_bias_add": [c_int, c_void_p, c_void_p, c_int, c_int, c_void_p],
        "bn_embed_gather_sinusoid": [c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_float,
                                     c_void_p],
        "bn_unary_act_apply": [c_int, c_void_p, c_void_p, c_longlong, c_int, c_void_p],
        "bn_scale": [c_void_p, c_longlong, c_float, c_void_p],
        "bn_rmsnorm_mean": [c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_float, c_void_p],
        "bn_add_normed_rmsnorm": [c_int, c_void_p, c_void_p, c_int, c_int, c_void_p, c_float, c_void_p, c_void_p, c_int, c_int,
                                  c_float, c_void_p],
    },
    "qk_norm": {
        "bn_qk_norm_store": [c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p,
                             c_void_p, c_int, c_int, c_int, c_int, c_int, c_float, c_float, c_int, c_int, c_int, c_void_p, c_int,
                             c_int, c_int, c_void_p],
    },
    "latent": {
        "bn_latent_store": [c_int, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p,
                            c_int, c_int, c_float, c_int, c_void_p, c_float, c_void_p],
        "bn_head_linear": [c_int, c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                           c_void_p],
        "bn_sigmoid_gate": [c_int, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
        "bn_rope_heads": [c_int, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_float, c_void_p],
    },
    "moe": {
        "bn_moe_route": [c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                         c_void_p, c_float, c_float, c_void_p, c_void_p, c_void_p, c_void_p],
        "bn_moe_experts": [c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                           c_int, c_int, c_int, c_int, c_int, c_float, c_float, c_float, c_void_p],
        "bn_gated_unit": [c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_float, c_float, c_float, c_void_p],
        "bn_moe_grouped_tiles": [c_int, c_int, c_int],
        "bn_moe_group": [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                         c_int, c_void_p],
    },
    "attn_mfma_general": {
        "bn_attn_general_supports": [c_int, c_int],
        "bn_attn_general_prompt": [c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int,
                                   c_int, c_int, c_int, c_float, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p],
        "bn_attn_general_decode": [c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int,
                                   c_int, c_int, c_int, c_float, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_void_p,
                                   c_void_p, c_void_p, c_void_p],
    },
    "hyper": {
        "bn_hc_step": [c_int, c_int, c_void_p, c_longlong, c_void_p, c_longlong, c_void_p, c_int, c_longlong, c_void_p, c_void_p,
                       c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
        "bn_dyt_norm": [c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p],
    },
    "conv_scans": {
        "bn_short_conv": [c_int, c_int, c_void_p, c_int, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_longlong,
                          c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
        "bn_lru_gates": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                         c_void_p],
        "bn_lru_scan": [c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_longlong, c_void_p, c_int, c_void_p,
                        c_void_p, c_int, c_void_p],
        "bn_lru_scan_pieces": [c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_longlong, c_void_p, c_int, c_void_p,
                               c_int, c_int, c_int, c_void_p, c_void_p],
        "bn_gla_supports": [c_int, c_int],
        "bn_gla_scan": [c_int, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_longlong, c_void_p, c_int,
                        c_void_p, c_void_p, c_int, c_int, c_int, c_float, c_float, c_void_p],
        "bn_gla_scan_pieces": [c_int, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_longlong, c_void_p,
                               c_int, c_void_p, c_int, c_int, c_int, c_float, c_float, c_int, c_int, c_void_p, c_void_p, c_void_p],
    },
    "lightning": {
        "bn_lightning_supports": [c_int, c_int],
        "bn_lightning_chunked": [c_int, c_int],
        "bn_lightning_prefers_chunks": [c_int, c_int, c_int, c_int],
        "bn_lightning_scan": [c_int, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_longlong, c_void_p,
                              c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p],
        "bn_row_norm_gate": [c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_float, c_int, c_void_p],
    },
    "state_mixers": {
        "bn_token_shift": [c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_longlong, c_void_p, c_void_p, c_void_p, c_int,
                           c_int, c_int, c_void_p],
        "bn_wkv_supports": [c_int, c_int],
        "bn_wkv_state_floats": [c_int, c_int],
        "bn_wkv_scan": [c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p,
                        c_void_p, c_void_p, c_void_p, c_longlong, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int,
                        c_int, c_void_p],
        "bn_head_norm_gate": [c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_float, c_void_p],
        "bn_mingru_scan": [c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_longlong, c_void_p, c_int,
                           c_void_p, c_void_p, c_int, c_void_p],
    },
    "rope_kv": {
        "bn_v_transposed_write": [c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_int, c_int,
                                  c_int, c_void_p],
        "bn_rope_kv_write": [c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                             c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
        "bn_rope_kv_write_tiles": [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p,
                                   c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_int, c_void_p],
    },
    "attn_rows": {
        "bn_attn_rows_key_tile": [c_int, c_int],
        "bn_attn_rows": [c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                         c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int,
                         c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p],
    },
    "attn_mfma": {
        "bn_attn_mfma_supports": [c_int],
        "bn_attn_mfma_prompt_tokens": [c_int, c_int],
        "bn_attn_mfma_scaled": [c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int,
                                c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_void_p, c_void_p, c_void_p, c_int,
                                c_void_p, c_void_p, c_void_p, c_int, c_int, c_float, c_void_p],
        "bn_attn_mfma": [c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                         c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_void_p, c_void_p,
                         c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p],
    },
    "gemm_tiled": {
        "bn_gemm_tiled": [c_int, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                          c_void_p],
    },
    "gemm_mfma": {
        "bn_gemm_mfma_supports": [c_int, c_int, c_int, c_int, c_int],
        "bn_gemm_mfma": [c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                         c_int, c_void_p],
        "bn_gemm_mfma_grouped": [c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_longlong,
                                 c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    },
    "skinny_gemm": {
        "bn_skinny_gemm_supports": [c_int, c_int, c_int, c_int, c_int],
        "bn_skinny_gemm": [c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                           c_int, c_int, c_int, c_void_p],
        "bn_skinny_gemm_fused_tile_cols": [c_int],
        "bn_skinny_gemm_fused_tiles": [c_int, c_int],
        "bn_skinny_gemm_fused": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                 c_void_p, c_int, c_int, c_float, c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p,
                                 c_int, c_void_p],
    },
    "splitk_gemm": {
        "bn_splitk_gemm_supports": [c_int, c_int, c_int, c_int, c_int, c_int],
        "bn_splitk_gemm_splits": [c_int, c_int, c_int],
        "bn_splitk_gemm": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
        "bn_splitk_gemm_swiglu": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_int,
                                  c_int, c_float, c_int, c_void_p],
    },
    "sampling": {
        "bn_argmax": [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p],
        "bn_repeat_penalty": [c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_float, c_void_p],
        "bn_sample": [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_float, c_float, c_void_p, c_void_p],
        "bn_sample_wide": [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_float, c_float, c_void_p, c_void_p],
    },
}
_fns = {}


def _fn(lib: str, name: str):
    f = _fns.get(name)
    if f is None:
        handle = _build.load(lib)
        f = getattr(handle, name)
        f.argtypes = _SIGNATURES[lib][name]
        f.restype = c_int
        _fns[name] = f
    return f


_gpu_seen = False


def require_gpu() -> None:
    global _gpu_seen
    if _gpu_seen:                      # asked before every launch: a GPU that was there stays
        return
    if not torch.cuda.is_available():
        raise KernelError("no GPU: the kernels of this library are HIP code for gfx950 and there is "
                          "no CPU implementation behind them")
    _gpu_seen = True


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """The current HIP stream's handle (it changes under a graph capture, so it is asked for at every launch; the
    raw query costs a fraction of building a torch.cuda.Stream object)."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _check(rc: int, what: str) -> None:
    if rc == 0:
        return
    if rc == -1:
        raise KernelError(f"{what}: the kernel refuses these sizes or this alignment")
    if rc == -2:
        raise KernelError(f"{what}: unsupported dtype")
    raise KernelError(f"{what}: HIP error {rc}")


def _dev(t: torch.Tensor, name: str, dtype=None, dims=None) -> None:
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise KernelError(f"{name}: expected a GPU tensor")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name}: expected {dtype}, got {t.dtype}")
    if dims is not None and t.dim() != dims:
        raise KernelError(f"{name}: expected {dims} dimensions, got shape {tuple(t.shape)}")


def _rows(t: torch.Tensor, name: str) -> int:
    """Row stride of a 2-D tensor whose rows are contiguous."""
    if t.dim() != 2 or (t.shape[1] > 1 and t.stride(1) != 1):
        raise KernelError(f"{name}: expected a 2-D tensor with contiguous rows, got shape "
                          f"{tuple(t.shape)} strides {t.stride()}")
    return t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1])


def _code(dtype) -> int:
    if dtype not in _DT:
        raise KernelError(f"unsupported dtype {dtype}")
    return _DT[dtype]


# The gate's activation of a gated feed-forward, out = act(gate) * up (BN_ACT_* of csrc/common.h): every kernel that
# ends in a gated unit takes the kind as an argument.
ACTIVATIONS = {"silu": _build.header_constant("BN_ACT_SILU"), "gelu_tanh": _build.header_constant("BN_ACT_GELU_TANH"),
               "relu2": _build.header_constant("BN_ACT_RELU2")}


def _act(name: str) -> int:
    if name not in ACTIVATIONS:
        raise KernelError(f"unknown gate activation {name!r}; the kernels take {sorted(ACTIVATIONS)}")
    return ACTIVATIONS[name]


# --------------------------------------------------------------------------------------
# row-wise kernels
# --------------------------------------------------------------------------------------

def embed_gather(table: torch.Tensor, tokens: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """float32 rows of the embedding table for int32 token ids, times `scale` (an architecture's embedding
    multiplier; 1 changes no bit)."""
    require_gpu()
    _dev(table, "table", dims=2)
    _dev(tokens, "tokens", torch.int32, 1)
    if not table.is_contiguous() or not tokens.is_contiguous():
        raise KernelError("embed_gather: table and tokens must be contiguous")
    n, dim = tokens.numel(), table.shape[1]
    x = torch.empty((n, dim), dtype=torch.float32, device=table.device)
    _check(_fn("elementwise", "bn_embed_gather")(_code(table.dtype), x.data_ptr(), table.data_ptr(),
                                                 tokens.data_ptr(), n, dim, table.shape[0], float(scale), _stream()),
           "embed_gather")
    return x


def gather_rows(x: torch.Tensor, rows: torch.Tensor, out_dtype) -> torch.Tensor:
    """The rows `rows` (int32) of the float32 stream x [T, D], in out_dtype: what an output matrix reads when the
    architecture puts no norm in front of it."""
    require_gpu()
    _dev(x, "x", torch.float32, 2)
    _dev(rows, "rows", torch.int32, 1)
    if not x.is_contiguous() or not rows.is_contiguous():
        raise KernelError("gather_rows: x and rows must be contiguous")
    out = torch.empty((rows.numel(), x.shape[1]), dtype=out_dtype, device=x.device)
    if rows.numel():
        _check(_fn("elementwise", "bn_gather_rows")(_code(out_dtype), out.data_ptr(), x.data_ptr(), rows.data_ptr(), rows.numel(),
                                                    x.shape[1], _stream()), "gather_rows")
    return out


def stream_rows(x: torch.Tensor, out_dtype) -> torch.Tensor:
    """Every row of the float32 stream x [T, D] in out_dtype (a copy): what a part reads when no norm stands in front
    of it."""
    require_gpu()
    _dev(x, "x", torch.float32, 2)
    if not x.is_contiguous():
        raise KernelError("stream_rows: x must be contiguous")
    out = torch.empty(tuple(x.shape), dtype=out_dtype, device=x.device)
    if x.shape[0]:
        _check(_fn("elementwise", "bn_gather_rows")(_code(out_dtype), out.data_ptr(), x.data_ptr(), None, x.shape[0], x.shape[1],
                                                    _stream()), "stream_rows")
    return out


def softcap_(logits: torch.Tensor, cap: float) -> None:
    """In place: cap * tanh(logits / cap), float32 (an architecture's bound on its logits; cap > 0)."""
    require_gpu()
    _dev(logits, "logits", torch.float32)
    if not logits.is_contiguous() or not cap > 0:
        raise KernelError("softcap: contiguous float32 logits and a positive cap")
    if logits.numel():
        _check(_fn("elementwise", "bn_softcap")(logits.data_ptr(), logits.numel(), float(cap), _stream()), "softcap")


def add_rmsnorm(x: torch.Tensor, delta, weight: torch.Tensor, eps: float, out_dtype,
                rows=None) -> torch.Tensor:
    """x (float32, [T, D]) += delta (if given), and the RMS-normed rows in out_dtype.
    With `rows` (int32 indices) only those rows are normed and x is left as it is."""
    require_gpu()
    _dev(x, "x", torch.float32, 2)
    _dev(weight, "weight", torch.float32, 1)
    T, D = x.shape
    if not x.is_contiguous() or weight.numel() != D or not weight.is_contiguous():
        raise KernelError(f"add_rmsnorm: x {tuple(x.shape)} must be contiguous and weight have {D} elements")
    parts = delta if isinstance(delta, PartialSums) else None
    if parts is not None:
        if parts.shape != x.shape:
            raise KernelError(f"add_rmsnorm: partial sums {tuple(parts.shape)} do not match x {tuple(x.shape)}")
    elif delta is not None:
        _dev(delta, "delta", out_dtype, 2)
        if delta.shape != x.shape or not delta.is_contiguous():
            raise KernelError(f"add_rmsnorm: delta {tuple(delta.shape)} does not match x {tuple(x.shape)}")
    n = T
    if rows is not None:
        _dev(rows, "rows", torch.int32, 1)
        if not rows.is_contiguous():
            raise KernelError("add_rmsnorm: rows must be contiguous")
        n = rows.numel()
    out = torch.empty((n, D), dtype=out_dtype, device=x.device)
    if n == 0:
        return out
    if parts is not None and rows is None and D % 4 == 0 and parts.slabs.shape[0] > 2 and T <= 65535:
        # many slabs: the sum over the whole chip first, then the norm (one workgroup a row would pull all of its slabs alone)
        ssq = torch.empty((T, _fn("elementwise", "bn_add_rmsnorm_parts_pieces")(D)), dtype=torch.float32, device=x.device)
        _check(_fn("elementwise", "bn_add_rmsnorm_parts_wide")(_code(out_dtype), x.data_ptr(), parts.slabs.data_ptr(),
                                                               parts.slabs.shape[0], T, weight.data_ptr(), out.data_ptr(),
                                                               ssq.data_ptr(), D, float(eps), _stream()), "add_rmsnorm")
        return out
    if parts is not None:
        _check(_fn("elementwise", "bn_add_rmsnorm_parts")(_code(out_dtype), x.data_ptr(), parts.slabs.data_ptr(),
                                                          parts.slabs.shape[0], T, weight.data_ptr(), out.data_ptr(),
                                                          rows.data_ptr() if rows is not None else None,
                                                          n, D, float(eps), _stream()), "add_rmsnorm")
        return out
    _check(_fn("elementwise", "bn_add_rmsnorm")(_code(out_dtype), x.data_ptr(),
                                                delta.data_ptr() if delta is not None else None,
                                                weight.data_ptr(), out.data_ptr(),
                                                rows.data_ptr() if rows is not None else None,
                                                n, D, float(eps), _stream()), "add_rmsnorm")
    return out


def residual_add(x: torch.Tensor, delta) -> None:
    """x (float32) += delta (a tensor of x's shape, or PartialSums)."""
    require_gpu()
    _dev(x, "x", torch.float32)
    if isinstance(delta, PartialSums):
        if tuple(delta.shape) != tuple(x.shape) or not x.is_contiguous():
            raise KernelError("residual_add: partial sums do not match x, or x is not contiguous")
        _check(_fn("elementwise", "bn_residual_add_parts")(x.data_ptr(), delta.slabs.data_ptr(), delta.slabs.shape[0],
                                                           x.numel(), _stream()), "residual_add")
        return
    _dev(delta, "delta")
    if x.shape != delta.shape or not x.is_contiguous() or not delta.is_contiguous():
        raise KernelError("residual_add: shapes differ or tensors are not contiguous")
    _check(_fn("elementwise", "bn_residual_add")(_code(delta.dtype), x.data_ptr(), delta.data_ptr(),
                                                 x.numel(), _stream()), "residual_add")


def swiglu(gu: torch.Tensor, interleaved: bool = False, activation: str = "silu") -> torch.Tensor:
    """[T, 2F] (gate | up) -> act(gate) * up, [T, F].  interleaved: gate and up columns
    alternate in blocks of 8 (see interleave_gate_up).  activation: one of ACTIVATIONS."""
    require_gpu()
    _dev(gu, "gu", dims=2)
    if not gu.is_contiguous() or gu.shape[1] % 2:
        raise KernelError(f"swiglu: expected a contiguous [T, 2F] tensor, got {tuple(gu.shape)}")
    T, F = gu.shape[0], gu.shape[1] // 2
    out = torch.empty((T, F), dtype=gu.dtype, device=gu.device)
    if interleaved and F % 8:
        raise KernelError("swiglu: the interleaved layout needs F to be a multiple of 8")
    _check(_fn("elementwise", "bn_swiglu")(_code(gu.dtype), out.data_ptr(), gu.data_ptr(), T, F, int(interleaved),
                                           _act(activation), _stream()), "swiglu")
    return out


def bias_add(y: torch.Tensor, bias: torch.Tensor) -> None:
    require_gpu()
    _dev(y, "y", dims=2)
    _dev(bias, "bias", torch.float32, 1)
    if not y.is_contiguous() or bias.numel() != y.shape[1] or not bias.is_contiguous():
        raise KernelError("bias_add: y must be contiguous [T, N] and bias have N elements")
    _check(_fn("elementwise", "bn_bias_add")(_code(y.dtype), y.data_ptr(), bias.data_ptr(), y.shape[0],
                                             y.shape[1], _stream()), "bias_add")


# --------------------------------------------------------------------------------------
# matrix products
# --------------------------------------------------------------------------------------

def _tiled(x, w, out_dtype):
    M, K = x.shape
    N = w.shape[0]
    y = torch.empty((M, N), dtype=out_dtype, device=x.device)
    _check(_fn("gemm_tiled", "bn_gemm_tiled")(_code(x.dtype), _code(out_dtype), x.data_ptr(), w.data_ptr(),
                                              y.data_ptr(), M, N, K, _rows(x, "x"), _rows(w, "w"), N,
                                              _stream()), "gemm_tiled")
    return y


def gemm_mfma(x: torch.Tensor, w: torch.Tensor, out_dtype=None, glu8: bool = False, activation: str = "silu",
              width: int = 0) -> torch.Tensor:
    """The library-free bf16 product for many rows: y[M, N] = x[M, K] . w[N, K]^T on the matrix cores,
    or with glu8 act(gate) * up for w = gate and up rows interleaved in blocks of 8 ([2N, K]).
    width: the tile's rows of w (256, 192 or 128); 0 lets the kernel pick by the shape."""
    require_gpu()
    if width not in (0, 256, 192, 128):
        raise KernelError(f"gemm_mfma: the tile width is 256, 192, 128 or 0 (any), not {width}")
    _dev(x, "x", torch.bfloat16, 2)
    _dev(w, "w", torch.bfloat16, 2)
    M, K = x.shape
    rows = w.shape[0]
    if w.shape[1] != K or (glu8 and rows % 16):
        raise KernelError(f"gemm_mfma: x {tuple(x.shape)} and w {tuple(w.shape)} do not agree")
    N = rows // 2 if glu8 else rows
    out_dtype = out_dtype or torch.bfloat16
    y = torch.empty((M, N), dtype=out_dtype, device=x.device)
    if M == 0:
        return y
    _check(_fn("gemm_mfma", "bn_gemm_mfma")(_code(out_dtype), x.data_ptr(), w.data_ptr(), y.data_ptr(), M, N, K,
                                            _rows(x, "x"), _rows(w, "w"), N, int(glu8), _act(activation), int(width),
                                            _stream()),
           "gemm_mfma")
    return y


def gemm_mfma_supported(M: int, N: int, K: int, ldx: int, ldw: int) -> bool:
    """The conditions of bn_gemm_mfma_supports, checked here so that asking does not load (and at
    first use compile) a kernel that a model may never need."""
    return M >= 1 and N >= 1 and K >= 8 and K % 8 == 0 and ldx % 8 == 0 and ldw % 8 == 0 and ldx >= K and ldw >= K


SKINNY_ROWS = 16      # bf16 products with more rows than this go to the library


def skinny_supported(M: int, N: int, K: int, ldx: int, ldw: int) -> bool:
    return bool(_fn("skinny_gemm", "bn_skinny_gemm_supports")(M, N, K, ldx, ldw))


# --------------------------------------------------------------------------------------
# the streamed copy of a weight matrix
# --------------------------------------------------------------------------------------
STREAM_TILE_ROWS = _build.header_constant("BN_STREAM_TILE_ROWS")
STREAM_TILE_COLS = _build.header_constant("BN_STREAM_TILE_COLS")


@dataclass
class StreamedWeight:
    """A bf16 weight matrix [N, K] in the order in which the kernels that read it once per call load it (csrc/common.h):
    tiles of tile_rows (at most 16) rows x 32 columns, each the run of bytes that one load of a wave takes (lane r + 16 g:
    columns 8 g .. 8 g + 7 of row r), [ceil(N / tile_rows), ceil(K / 32), 32 tile_rows], rows past N and columns past K zero.
    A second copy beside the row-major matrix, which the products of many rows (the library's) and everything else keep
    reading: the kernels of up to 128 rows take it through their `streamed` argument and give the same result bit for
    bit, 5 to 15 % sooner.  The kernel of up to 16 rows gives a workgroup one row of tiles, so fewer than 16 rows a tile
    are chosen where that spreads the tiles more evenly over the CUs (stream_tile_rows)."""
    tiles: torch.Tensor
    N: int
    K: int
    tile_rows: int = STREAM_TILE_ROWS

    @property
    def k_tiles(self) -> int:
        return self.tiles.shape[1]

    def nbytes(self) -> int:
        return self.tiles.numel() * self.tiles.element_size()


def stream_tile_rows(N: int) -> int:
    """The rows per tile with which a matrix of N rows is best streamed: the columns that the fused product of up to 16
    rows gives a workgroup over the row-major matrix (16, or fewer when that leaves the busiest CU at least 15 % fewer
    columns: 12 for 6,144 rows on 256 CUs, 10 for 5,120)."""
    return int(_fn("skinny_gemm", "bn_skinny_gemm_fused_tile_cols")(int(N)))


def stream_copy(w: torch.Tensor, tile_rows: Optional[int] = None) -> StreamedWeight:
    """The streamed copy of w [N, K] (bf16, on the device; made there).  tile_rows None: stream_tile_rows(N); a matrix
    with gate and up rows interleaved in blocks of 8 needs 16."""
    require_gpu()
    _dev(w, "w", torch.bfloat16, 2)
    N, K = w.shape
    R, C = (stream_tile_rows(N) if tile_rows is None else int(tile_rows)), STREAM_TILE_COLS
    if not 1 <= R <= STREAM_TILE_ROWS:
        raise KernelError(f"stream_copy: a tile has 1 to {STREAM_TILE_ROWS} rows, not {R}")
    nt, kt = (N + R - 1) // R, (K + C - 1) // C
    if nt * R != N or kt * C != K:
        padded = torch.zeros((nt * R, kt * C), dtype=w.dtype, device=w.device)
        padded[:N, :K] = w
        w = padded
    # [nt, r, kt, g, 8] -> [nt, kt, g, r, 8]: lane r + 16 g of tile (nt, kt)
    tiles = w.view(nt, R, kt, C // 8, 8).permute(0, 2, 3, 1, 4).contiguous().view(nt, kt, R * C)
    return StreamedWeight(tiles, N, K, R)


def unstream(sw: StreamedWeight) -> torch.Tensor:
    """The row-major matrix [N, K] that a streamed copy holds."""
    R, C = sw.tile_rows, STREAM_TILE_COLS
    nt, kt = sw.tiles.shape[:2]
    return sw.tiles.view(nt, kt, C // 8, R, 8).permute(0, 3, 1, 2, 4).reshape(nt * R, kt * C)[:sw.N, :sw.K].contiguous()


def _weight_arg(w: torch.Tensor, streamed: Optional[StreamedWeight], what: str, need_rows: int = 0):
    """(pointer, row stride or tiles along K, rows per tile or 0) of the weights that a kernel is to read: the streamed
    copy if one is given (checked against w; need_rows: the only tile height the kernel takes, else w is read), else
    w itself."""
    if streamed is not None and need_rows and getattr(streamed, "tile_rows", 0) != need_rows:
        streamed = None
    if streamed is None:
        return w.data_ptr(), _rows(w, "w"), 0
    t = streamed.tiles
    R = streamed.tile_rows
    if (not isinstance(streamed, StreamedWeight) or (streamed.N, streamed.K) != tuple(w.shape) or t.device != w.device
            or t.dtype != torch.bfloat16 or not t.is_contiguous() or t.dim() != 3 or not 1 <= R <= STREAM_TILE_ROWS
            or tuple(t.shape) != ((streamed.N + R - 1) // R, (streamed.K + STREAM_TILE_COLS - 1) // STREAM_TILE_COLS,
                                  R * STREAM_TILE_COLS)):
        raise KernelError(f"{what}: the streamed copy does not belong to w {tuple(w.shape)}")
    return t.data_ptr(), t.shape[1], R


# bf16 products with many rows: the library's matrix product (as the reference hands its batched
# products to a library, src/gpu_cuda.cu:11571) unless this is False or BITNET_NO_LIBRARY is set;
# then this library's own matrix-core kernel (gemm_mfma) does them.
LIBRARY_PRODUCTS = os.environ.get("BITNET_NO_LIBRARY", "") in ("", "0")


def linear(x: torch.Tensor, w: torch.Tensor, out_dtype=None, *, allow_library: Optional[bool] = None,
           streamed: Optional[StreamedWeight] = None) -> torch.Tensor:
    """y[M, N] = x[M, K] . w[N, K]^T.  streamed: w's streamed copy, which the kernel of up to 16 rows reads instead.

    float32: the tiled kernel (plain fmaf, a fixed order of summation).
    bf16: up to 16 rows (one MFMA tile of activations) the matrix-core kernel that streams
    the weights once; above that the library's matrix product, which from 32 rows on is about
    twice as fast as the streaming kernel, with a bf16 or a float32 result (logits).  Without the
    library (allow_library False; None follows LIBRARY_PRODUCTS) the streaming kernel takes up to 64
    rows and the tiled matrix-core kernel (gemm_mfma) everything above; shapes that none of them
    takes (rows that are not 16-byte aligned) go to the plain tiled kernel."""
    require_gpu()
    _dev(x, "x", dims=2)
    _dev(w, "w", x.dtype, 2)
    M, K = x.shape
    N = w.shape[0]
    if w.shape[1] != K:
        raise KernelError(f"linear: x {tuple(x.shape)} and w {tuple(w.shape)} do not agree")
    out_dtype = out_dtype or x.dtype
    if allow_library is None:
        allow_library = LIBRARY_PRODUCTS
    if M == 0:
        return torch.empty((0, N), dtype=out_dtype, device=x.device)
    ldx, ldw = _rows(x, "x"), _rows(w, "w")
    if x.dtype == torch.float32:
        if out_dtype != torch.float32:
            raise KernelError("linear: float32 inputs give float32 outputs")
        return _tiled(x, w, torch.float32)
    if x.dtype != torch.bfloat16:
        raise KernelError(f"linear: unsupported dtype {x.dtype}")
    aligned = (x.data_ptr() % 16 == 0) and (w.data_ptr() % 16 == 0)
    small = M <= SKINNY_ROWS or (M <= 64 and not allow_library)
    if small and aligned and skinny_supported(M, N, K, ldx, ldw):
        y = torch.empty((M, N), dtype=out_dtype, device=x.device)
        wp, wl, tiled = _weight_arg(w, streamed if M <= SKINNY_ROWS else None, "linear")
        _check(_fn("skinny_gemm", "bn_skinny_gemm")(_code(out_dtype), x.data_ptr(), wp, y.data_ptr(),
                                                    M, N, K, ldx, wl, N, 0, 0, 0, tiled, _stream()), "skinny_gemm")
        return y
    if M > SKINNY_ROWS and allow_library:
        if out_dtype == torch.bfloat16:
            return torch.matmul(x, w.t())
        if out_dtype == torch.float32:
            return torch.mm(x, w.t(), out_dtype=torch.float32)
    if aligned and gemm_mfma_supported(M, N, K, ldx, ldw):
        return gemm_mfma(x, w, out_dtype)
    return _tiled(x, w, out_dtype)


def interleave_gate_up(w_gate: torch.Tensor, w_up: torch.Tensor) -> torch.Tensor:
    """[2F, K] with gate and up rows alternating in blocks of 8 (F a multiple of 8): rows
    16t..16t+7 are gate rows 8t..8t+7, rows 16t+8..16t+15 the up rows of the same columns.  A
    16-row tile of the decode kernel then holds both halves of 8 result columns."""
    F, K = w_gate.shape
    if F % 8 or w_up.shape != w_gate.shape:
        raise KernelError("interleave_gate_up: F must be a multiple of 8 and the shapes equal")
    return torch.stack([w_gate.reshape(F // 8, 8, K), w_up.reshape(F // 8, 8, K)], dim=1).reshape(2 * F, K).contiguous()


# The interleaved gate/up product with its SwiGLU epilogue in the kernel that stages the activations once per 64 or 112
# columns (splitk_gemm.hip).  Without the library it is the kernel of 17 to 128 rows.  With the library it takes the row
# counts at which it was measured faster than what else there is (the fused streaming kernel up to 16 rows, whose every
# workgroup stages all rows for its 16 columns; above that the library's product and the kernel of the gated unit) on
# matrices of at least STAGED_MIN_TILES_PER_CU column tiles per CU (smaller ones leave it too few waves): 13 to 16 rows,
# and up to 64 rows over a streamed copy of the weights (us at 16 / 32 / 64 rows, streamed: 8B 45.6 / 45.7 / 50.9 against
# 47.8 / 55.4 / 54.3; 13B 53.2 / 53.7 / 61.5 against 57.9 / 56.1 / 59.7; 70B 163 / 169 / 190 against 175 / 196 / 216;
# at a hidden size of 3,072 and below the others win by 5 to 15 %).
SWIGLU_STAGED_ROWS = (17, 128)
SWIGLU_STAGED_LIBRARY_ROWS = (13, 16)
SWIGLU_STAGED_STREAMED_ROWS = (13, 64)
STAGED_MIN_TILES_PER_CU = 6


_CUS = None


def _compute_units() -> int:
    global _CUS
    if _CUS is None:
        _CUS = int(torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count)
    return _CUS


def _staged_swiglu_rows(M: int, allow_library: bool, w_rows: int, streamed) -> bool:
    if not allow_library:
        lo, hi = SWIGLU_STAGED_ROWS
        return lo <= M <= hi
    lo, hi = SWIGLU_STAGED_STREAMED_ROWS if streamed is not None else SWIGLU_STAGED_LIBRARY_ROWS
    return lo <= M <= hi and w_rows // 16 >= STAGED_MIN_TILES_PER_CU * _compute_units()


def _staged_swiglu(x, w_gate_up, pre, activation, streamed=None):
    """The staged kernel's gate/up product with the gated unit (and a deferred norm's factor) in its epilogue; None if
    it does not take the shape."""
    M, K = x.shape
    F = w_gate_up.shape[0] // 2
    ldx = _rows(x, "x")
    wp, wl, tiled = _weight_arg(w_gate_up, streamed, "linear_swiglu", need_rows=STREAM_TILE_ROWS)
    if F % 8 or not _fn("splitk_gemm", "bn_splitk_gemm_supports")(M, 2 * F, K, ldx, wl, tiled):
        return None
    if pre is not None:          # what the kernel's passes over the parts of the sums of squares hold (SG_NORM_*)
        n = pre.slots.shape[1]
        per = min(64, 1 << max(0, n - 1).bit_length())
        if -(-M // (4 * (64 // per))) > 4 or -(-n // per) > 8:
            return None
    y = torch.empty((M, F), dtype=x.dtype, device=x.device)
    _check(_fn("splitk_gemm", "bn_splitk_gemm_swiglu")(
        x.data_ptr(), wp, y.data_ptr(), M, F, K, ldx, wl, F, _act(activation),
        pre.slots.data_ptr() if pre is not None else None, pre.slots.shape[1] if pre is not None else 0,
        pre.stream.shape[1] if pre is not None else 0, float(pre.eps) if pre is not None else 0.0, int(tiled != 0), _stream()),
        "splitk_gemm(glu)")
    return y


def linear_swiglu(x: torch.Tensor, w_gate_up: torch.Tensor, interleaved: bool = False, *,
                  allow_library: Optional[bool] = None, activation: str = "silu",
                  streamed: Optional[StreamedWeight] = None) -> torch.Tensor:
    """act(x.Wg^T) * (x.Wu^T) for w_gate_up = [Wg; Wu] ([2F, K]), or the two interleaved in
    blocks of 8 rows (interleave_gate_up); act is silu unless `activation` names another of
    ACTIVATIONS.  The decode-sized bf16 case is one kernel, and so is the interleaved case without
    the library; every other case is the product followed by the gated-unit kernel."""
    require_gpu()
    _dev(x, "x", dims=2)
    _dev(w_gate_up, "w_gate_up", x.dtype, 2)
    M, K = x.shape
    if w_gate_up.shape[0] % 2 or w_gate_up.shape[1] != K:
        raise KernelError(f"linear_swiglu: x {tuple(x.shape)} and w {tuple(w_gate_up.shape)} do not agree")
    F = w_gate_up.shape[0] // 2
    if interleaved and F % 8:
        raise KernelError("linear_swiglu: the interleaved layout needs F to be a multiple of 8")
    if allow_library is None:
        allow_library = LIBRARY_PRODUCTS
    if M == 0:
        return torch.empty((0, F), dtype=x.dtype, device=x.device)
    ldx, ldw = _rows(x, "x"), _rows(w_gate_up, "w_gate_up")
    aligned = x.data_ptr() % 16 == 0 and w_gate_up.data_ptr() % 16 == 0
    if x.dtype == torch.bfloat16 and interleaved and aligned and _staged_swiglu_rows(M, allow_library, 2 * F, streamed):
        y = _staged_swiglu(x, w_gate_up, None, activation, streamed)
        if y is not None:
            return y
    if (x.dtype == torch.bfloat16 and (M <= SKINNY_ROWS or (M <= 64 and not allow_library))
            and aligned and skinny_supported(M, F, K, ldx, ldw)):
        y = torch.empty((M, F), dtype=x.dtype, device=x.device)
        _check(_fn("skinny_gemm", "bn_skinny_gemm")(_code(x.dtype), x.data_ptr(), w_gate_up.data_ptr(),
                                                    y.data_ptr(), M, F, K, ldx, ldw, F, 2 if interleaved else 1, F,
                                                    _act(activation), 0, _stream()), "skinny_gemm(glu)")
        return y
    if (x.dtype == torch.bfloat16 and interleaved and not allow_library and aligned
            and gemm_mfma_supported(M, 2 * F, K, ldx, ldw)):
        return gemm_mfma(x, w_gate_up, x.dtype, glu8=True, activation=activation)
    return swiglu(linear(x, w_gate_up, allow_library=allow_library), interleaved, activation)


# --------------------------------------------------------------------------------------
# decode products with the neighbouring RMSNorm folded in
# --------------------------------------------------------------------------------------
# Set False (or BITNET_NO_FUSED_NORM=1) to keep every norm a kernel of its own.
SPLIT_SUMS = os.environ.get("BITNET_NO_SPLIT_SUMS", "") in ("", "0")
# Where a product that ends a part is left as partial sums (splitk_gemm) instead of going to the library: from 17 to 128
# rows when K is at least twice N, the shape of a feed-forward's last product.  Measured on nine layer shapes (hidden 2,048
# to 8,192) with the kernels of the next norm included: from 64 rows on it is 15 to 45 % faster than the library's product
# (8B: 36 us against 45 at 64 rows, 44 against 80 at 128; 70B: 119 against 148, 141 against 210); below 64 rows the two
# products are equal within a tenth, and the partial sums win by the kernel that they save: one kernel adds them to
# the stream and leaves the next norm to its consumer (sum_deferred), where the library's product needs the add and the
# norm.  Square products (an output projection) as well up to SPLIT_SUM_SQUARE_WIDTH columns: 12 + 5 us against 15 + 5 at
# 64 rows of the 8B shape; at widths of 5,120 and 8,192 whole decode steps were equal within the noise of a run or slower.
SPLIT_SUM_ROWS = (17, 128)
SPLIT_SUM_SQUARE_WIDTH = int(os.environ.get("BITNET_SPLIT_SQUARE_WIDTH", "4096"))


@dataclass
class PartialSums:
    """A product that is still a sum to be formed: `slabs` [S, M, N] float32, the products over S ranges of K
    (splitk_gemm).  add_rmsnorm and residual_add take it in place of a delta and add the slabs in order."""
    slabs: torch.Tensor

    @property
    def shape(self):
        return self.slabs.shape[1:]

    @property
    def device(self):
        return self.slabs.device


def can_split_sums(M: int, N: int, K: int, dtype) -> bool:
    """Whether a product of these sizes whose result goes to the residual stream is done as partial sums."""
    if not (SPLIT_SUMS and dtype == torch.bfloat16 and SPLIT_SUM_ROWS[0] <= M <= SPLIT_SUM_ROWS[1] and K % 8 == 0 and N >= 1):
        return False
    return K >= 2 * N or (K >= N and N <= SPLIT_SUM_SQUARE_WIDTH)


def linear_partial_sums(x: torch.Tensor, w: torch.Tensor, streamed: Optional[StreamedWeight] = None) -> PartialSums:
    """x [M, K] . w[N, K]^T as float32 partial sums over ranges of K (bf16 operands, 1 to 128 rows).  streamed: w's
    streamed copy, read instead of w."""
    require_gpu()
    _dev(x, "x", torch.bfloat16, 2)
    _dev(w, "w", torch.bfloat16, 2)
    ldx = _rows(x, "x")
    M, K = x.shape
    N = w.shape[0]
    if w.shape[1] != K:
        raise KernelError(f"linear_partial_sums: x {tuple(x.shape)} and w {tuple(w.shape)} do not fit")
    wp, wl, tiled = _weight_arg(w, streamed, "linear_partial_sums")
    if not _fn("splitk_gemm", "bn_splitk_gemm_supports")(M, N, K, ldx, wl, tiled) or (x.data_ptr() | wp) % 16:
        raise KernelError(f"linear_partial_sums: the kernel takes 1 to 128 rows, K a multiple of 8 and 16-byte aligned "
                          f"operands, not x {tuple(x.shape)} (row stride {ldx}), w {tuple(w.shape)} (row stride {wl})")
    S = _fn("splitk_gemm", "bn_splitk_gemm_splits")(N, K, tiled)
    slabs = torch.empty((S, M, N), dtype=torch.float32, device=x.device)
    _check(_fn("splitk_gemm", "bn_splitk_gemm")(x.data_ptr(), wp, slabs.data_ptr(), M, N, K, ldx, wl, S, tiled,
                                                _stream()), "splitk_gemm")
    return PartialSums(slabs)


FUSE_NORMS = os.environ.get("BITNET_NO_FUSED_NORM", "") in ("", "0")
FUSED_ROWS = 16           # rows the fused products take (one MFMA tile of activations)
FUSED_SLOTS = 512         # column tiles of 16 whose sums of squares a consumer adds up: streams up to 8,192 wide


@dataclass
class DeferredNorm:
    """An RMSNorm that has not been applied yet.  `scaled` is the bf16 copy of the stream already
    multiplied by the norm's weights, `slots` [M, n] the sums of squares of the stream's rows in
    parts; a product that consumes it (linear_prenorm, linear_swiglu_prenorm) multiplies its
    result's rows by 1/sqrt(mean + eps).  `stream`, `weight`, `eps` are what the plain kernel needs
    when the consumer cannot take it (materialize)."""
    scaled: torch.Tensor
    slots: torch.Tensor
    stream: torch.Tensor
    weight: torch.Tensor
    eps: float

    @property
    def shape(self):
        return self.scaled.shape

    @property
    def dtype(self):
        return self.scaled.dtype

    @property
    def device(self):
        return self.scaled.device

    def materialize(self, out_dtype=None, rows=None) -> torch.Tensor:
        return add_rmsnorm(self.stream, None, self.weight, self.eps, out_dtype or self.scaled.dtype, rows)


DEFER_ROWS = (17, 128)    # row counts at which a norm is left to its consumer through sum_deferred (below: the fused products)


def can_sum_deferred(M: int, D: int, dtype) -> bool:
    """Whether the residual stream of M rows of D columns leaves the norm of a consumer that asks for it undone
    (sum_deferred) instead of norming the rows itself."""
    return FUSE_NORMS and dtype == torch.bfloat16 and DEFER_ROWS[0] <= M <= DEFER_ROWS[1] and D % 8 == 0 and D >= 8


def sum_deferred(x: torch.Tensor, delta, weight: torch.Tensor, eps: float) -> DeferredNorm:
    """x (float32 [M, D], in place) += delta (a bf16 or float32 tensor, PartialSums, or None), and what the next norm
    (weights `weight`, `eps`) needs of the new x for a consumer that applies it itself: the bf16 copy times the weights
    and the rows' sums of squares in pieces of 1,024 columns.  One kernel over the whole chip."""
    require_gpu()
    _dev(x, "x", torch.float32, 2)
    _dev(weight, "weight", torch.float32, 1)
    M, D = x.shape
    if not x.is_contiguous() or weight.numel() != D or not weight.is_contiguous() or D % 4 or M < 1 or M > 65535:
        raise KernelError(f"sum_deferred: x {tuple(x.shape)} must be contiguous with a width that is a multiple of 4, "
                          f"weight have {D} elements")
    n_parts, dptr, ddt = 0, None, 0
    if isinstance(delta, PartialSums):
        if tuple(delta.shape) != (M, D) or not delta.slabs.is_contiguous():
            raise KernelError(f"sum_deferred: partial sums {tuple(delta.shape)} do not match x {tuple(x.shape)}")
        n_parts, dptr, ddt = delta.slabs.shape[0], delta.slabs.data_ptr(), _DT[torch.float32]
    elif delta is not None:
        _dev(delta, "delta", dims=2)
        if tuple(delta.shape) != (M, D) or not delta.is_contiguous() or delta.dtype not in _DT:
            raise KernelError(f"sum_deferred: delta {tuple(delta.shape)} ({delta.dtype}) does not match x {tuple(x.shape)}")
        n_parts, dptr, ddt = 1, delta.data_ptr(), _DT[delta.dtype]
    scaled = torch.empty((M, D), dtype=torch.bfloat16, device=x.device)
    slots = torch.empty((M, _fn("elementwise", "bn_add_rmsnorm_parts_pieces")(D)), dtype=torch.float32, device=x.device)
    _check(_fn("elementwise", "bn_sum_deferred")(ddt, x.data_ptr(), dptr, n_parts, M, weight.data_ptr(), scaled.data_ptr(),
                                                 slots.data_ptr(), D, _stream()), "sum_deferred")
    return DeferredNorm(scaled, slots, x, weight, float(eps))


def swiglu_scaled(gu: torch.Tensor, pre: DeferredNorm, activation: str = "silu") -> torch.Tensor:
    """act(s * gate) * (s * up) for gu = [T, 2F] (bf16, gate and up interleaved in blocks of 8) that is the product of a
    deferred norm's copy with the gate and up weights; s the rows' 1/sqrt(mean + eps)."""
    require_gpu()
    _dev(gu, "gu", torch.bfloat16, 2)
    T, F = gu.shape[0], gu.shape[1] // 2
    if not gu.is_contiguous() or gu.shape[1] % 16 or pre.slots.shape[0] != T or not pre.slots.is_contiguous():
        raise KernelError(f"swiglu_scaled: gu {tuple(gu.shape)} / slots {tuple(pre.slots.shape)} do not fit")
    out = torch.empty((T, F), dtype=gu.dtype, device=gu.device)
    if T:
        _check(_fn("elementwise", "bn_swiglu_scaled")(out.data_ptr(), gu.data_ptr(), T, F, _act(activation), pre.slots.data_ptr(),
                                                      pre.slots.shape[1], pre.stream.shape[1], float(pre.eps), _stream()),
               "swiglu_scaled")
    return out


def can_fuse_norm(M: int, N: int, K: int, dtype) -> bool:
    """Whether a product of these sizes can take a norm into its kernel (either side of it)."""
    return (dtype == torch.bfloat16 and 1 <= M <= FUSED_ROWS and K % 8 == 0 and N >= 1
            and torch.cuda.is_available() and skinny_supported(M, N, K, K, K))


def _fused_call(x, w, y, M, N, K, glu8, pre: Optional[DeferredNorm], resid, resid_bf16, next_weight, slots_out,
                activation: str = "silu", streamed: Optional[StreamedWeight] = None):
    wp, wl, tiled = _weight_arg(w, streamed, "fused product", need_rows=STREAM_TILE_ROWS if glu8 else 0)
    _check(_fn("skinny_gemm", "bn_skinny_gemm_fused")(
        x.data_ptr(), wp, y.data_ptr() if y is not None else None, M, N, K, _rows(x, "x"), wl,
        N if y is not None else 0, int(glu8), _act(activation),
        pre.slots.data_ptr() if pre is not None else None, pre.slots.shape[1] if pre is not None else 0,
        pre.stream.shape[1] if pre is not None else 0, float(pre.eps) if pre is not None else 0.0,
        resid.data_ptr() if resid is not None else None, _rows(resid, "resid") if resid is not None else 0,
        resid_bf16.data_ptr() if resid_bf16 is not None else None, N if resid_bf16 is not None else 0,
        next_weight.data_ptr() if next_weight is not None else None,
        slots_out.data_ptr() if slots_out is not None else None, tiled, _stream()), "skinny_gemm(fused)")


def _check_deferred(pre: DeferredNorm, K: int) -> int:
    _dev(pre.scaled, "deferred norm: scaled", torch.bfloat16, 2)
    _dev(pre.slots, "deferred norm: slots", torch.float32, 2)
    M = pre.scaled.shape[0]
    if (pre.scaled.shape[1] != K or pre.stream.shape[1] != K or pre.slots.shape[0] != M
            or not pre.slots.is_contiguous() or pre.slots.shape[1] > FUSED_SLOTS or pre.scaled.data_ptr() % 16):
        raise KernelError(f"deferred norm: copy {tuple(pre.scaled.shape)}, slots {tuple(pre.slots.shape)} do not fit "
                          f"an input width of {K}")
    return M


def linear_prenorm(pre: DeferredNorm, w: torch.Tensor, streamed: Optional[StreamedWeight] = None) -> torch.Tensor:
    """linear(rmsnorm(stream), w) for a deferred norm, in one kernel (bf16, up to 16 rows).  streamed: w's streamed
    copy, read instead of w."""
    require_gpu()
    _dev(w, "w", torch.bfloat16, 2)
    N, K = w.shape
    M = _check_deferred(pre, K)
    if not can_fuse_norm(M, N, K, torch.bfloat16) or w.data_ptr() % 16:
        raise KernelError(f"linear_prenorm: {M} rows, w {tuple(w.shape)} cannot be fused")
    y = torch.empty((M, N), dtype=torch.bfloat16, device=w.device)
    _fused_call(pre.scaled, w, y, M, N, K, False, pre, None, None, None, None, streamed=streamed)
    return y


def linear_swiglu_prenorm(pre: DeferredNorm, w_gate_up: torch.Tensor, activation: str = "silu",
                          streamed: Optional[StreamedWeight] = None) -> torch.Tensor:
    """linear_swiglu(rmsnorm(stream), w) for gate and up interleaved in blocks of 8, in one kernel.  streamed: w's
    streamed copy, read instead of w."""
    require_gpu()
    _dev(w_gate_up, "w_gate_up", torch.bfloat16, 2)
    F, K = w_gate_up.shape[0] // 2, w_gate_up.shape[1]
    M = _check_deferred(pre, K)
    if (w_gate_up.shape[0] % 16 == 0 and w_gate_up.data_ptr() % 16 == 0
            and _staged_swiglu_rows(M, LIBRARY_PRODUCTS, w_gate_up.shape[0], streamed)):
        y = _staged_swiglu(pre.scaled, w_gate_up, pre, activation, streamed)
        if y is not None:
            return y
    if M > FUSED_ROWS and w_gate_up.shape[0] % 16 == 0 and LIBRARY_PRODUCTS:
        # more rows than the fused kernel takes: the library's product of the copy, and the norm's factor in the
        # kernel of the gated unit, which runs anyway
        return swiglu_scaled(torch.matmul(pre.scaled, w_gate_up.t()), pre, activation)
    if w_gate_up.shape[0] % 16 or not can_fuse_norm(M, F, K, torch.bfloat16) or w_gate_up.data_ptr() % 16:
        raise KernelError(f"linear_swiglu_prenorm: {M} rows, w {tuple(w_gate_up.shape)} cannot be fused")
    y = torch.empty((M, F), dtype=torch.bfloat16, device=w_gate_up.device)
    _fused_call(pre.scaled, w_gate_up, y, M, F, K, True, pre, None, None, None, None, activation, streamed)
    return y


def _fused_tiles(N: int, tile_rows: int = 0) -> int:
    """Column tiles of the fused product kernel for N columns (over a streamed copy with tile_rows rows a tile if that
    is not 0): one partial sum of squares per row and tile."""
    return int(_fn("skinny_gemm", "bn_skinny_gemm_fused_tiles")(int(N), int(tile_rows)))


def can_defer_norm(M: int, N: int, K: int, dtype) -> bool:
    """Whether linear_into_stream takes a product of these sizes (N is the stream's width)."""
    return FUSE_NORMS and can_fuse_norm(M, N, K, dtype) and _fused_tiles(N) <= FUSED_SLOTS


def linear_into_stream(x: torch.Tensor, w: torch.Tensor, stream: torch.Tensor, weight: torch.Tensor,
                       eps: float, streamed: Optional[StreamedWeight] = None) -> DeferredNorm:
    """stream += linear(x, w) (float32 stream [M, N], in place), and what the next norm (weights
    `weight`, `eps`) needs: the bf16 copy of the new stream times the weights and the rows' sums of
    squares in parts.  Returns that norm, deferred."""
    require_gpu()
    _dev(x, "x", torch.bfloat16, 2)
    _dev(w, "w", torch.bfloat16, 2)
    _dev(stream, "stream", torch.float32, 2)
    _dev(weight, "weight", torch.float32, 1)
    M, K = x.shape
    N = w.shape[0]
    if w.shape[1] != K or tuple(stream.shape) != (M, N) or weight.numel() != N or not weight.is_contiguous():
        raise KernelError(f"linear_into_stream: x {tuple(x.shape)}, w {tuple(w.shape)}, stream {tuple(stream.shape)}, "
                          f"weight {tuple(weight.shape)} do not agree")
    if not can_defer_norm(M, N, K, torch.bfloat16) or x.data_ptr() % 16 or w.data_ptr() % 16:
        raise KernelError(f"linear_into_stream: {M} rows, w {tuple(w.shape)} cannot be fused")
    if streamed is not None and _fused_tiles(N, streamed.tile_rows) > FUSED_SLOTS:
        streamed = None                       # more rows of tiles than a consumer adds up slots
    scaled = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    slots = torch.empty((M, _fused_tiles(N, streamed.tile_rows if streamed is not None else 0)), dtype=torch.float32,
                        device=x.device)
    _fused_call(x, w, None, M, N, K, False, None, stream, scaled, weight, slots, streamed=streamed)
    return DeferredNorm(scaled, slots, stream, weight, float(eps))


# --------------------------------------------------------------------------------------
# position encoding + cache write, attention
# --------------------------------------------------------------------------------------

KV_BLOCK = _build.header_constant("BN_KV_BLOCK")       # positions in a block of a blocked page


def kernel_v_layout(dtype, head_dim: int = 0) -> str:
    """The page layout (KVNeed.v_layout) that the attention kernels of this library read fastest at a cache type and
    head size: "blocked" for bf16 at the head sizes of the matrix-core kernels (keys and values of a page in those
    kernels' own order, blocked_page_index), else bf16 values transposed inside a page ([pages, Hkv, hs, PAGE]) and
    float32 values like the keys ([pages, Hkv, PAGE, hs]).  Without a head size: "transposed" or "rows".  The vector
    kernel and the cache write take rows and transposed values at either type; the matrix-core kernels take blocked
    pages alone."""
    if dtype != torch.bfloat16:
        return "rows"
    return "blocked" if head_dim and mfma_attention(dtype, head_dim) else "transposed"


def _page_layout(dtype, hs: int, v_transposed, blocked) -> str:
    """The layout that a caller names with v_transposed (None, False, True) and blocked (None, False, True); neither:
    kernel_v_layout."""
    if blocked:
        if v_transposed is False or dtype != torch.bfloat16 or hs % 32:
            raise KernelError(f"blocked pages are bf16 pages of head sizes that are multiples of 32 (got {dtype}, {hs})")
        return "blocked"
    if v_transposed is None:
        return kernel_v_layout(dtype, hs if blocked is None else 0)
    return "transposed" if v_transposed else "rows"


_LAYOUT_CODES = {"rows": 0, "transposed": 1, "blocked": 2}       # BN_KV_* of csrc/rope_kv.hip; + 4: values by page tiles


def _check_pages(k_pages, v_pages, Hkv, hs, dtype, v_transposed=None, blocked=None, vd: int = 0) -> str:
    """Checks both page tensors against the layout that the caller names (_page_layout) and returns it.  vd: the width
    of a value head (0: the keys'; the vector attention kernel and qk_norm_store take another, the rest want values as
    wide as keys).  Blocked pages have the shapes of pages with transposed values."""
    vd = vd or hs
    layout = _page_layout(dtype, hs, v_transposed, blocked)
    if layout == "blocked" and vd != hs:
        raise KernelError("blocked pages hold values as wide as keys")
    v_shape = (Hkv, PAGE, vd) if layout == "rows" else (Hkv, vd, PAGE)
    for t, nm, shape in ((k_pages, "k_pages", (Hkv, PAGE, hs)), (v_pages, "v_pages", v_shape)):
        _dev(t, nm, dtype, 4)
        if tuple(t.shape[1:]) != shape or not t.is_contiguous():
            raise KernelError(f"{nm}: expected contiguous [pages, {', '.join(map(str, shape))}], got {tuple(t.shape)}")
    if k_pages.shape[0] != v_pages.shape[0]:
        raise KernelError("k_pages and v_pages differ in their number of pages")
    if k_pages.data_ptr() % 16 or v_pages.data_ptr() % 16:
        raise KernelError("k_pages and v_pages must start at multiples of 16 bytes (the kernels load 16 bytes at a time)")
    return layout


def blocked_page_index(hs: int):
    """Where the elements of a (page, kv head) lie in a blocked page (csrc/common.h), as two int64 tensors: k_index[p, d]
    = the place of dimension d of the key at position p, v_index[d, p] = the place of dimension d of the value at
    position p, both counted in elements from the beginning of the (page, kv head).  Position p = 32 b + r: the keys'
    operand tiles hold the block's positions 8 (i / 4) + i % 4 (tile 0) and 4 further (tile 1) in tile row i, a lane
    group g the dimensions 32 c + 8 g .. + 7; the values' tiles hold dimension 16 t + i in row i, a lane group the
    positions 8 g .. 8 g + 7 of the block."""
    if hs % 32:
        raise KernelError(f"blocked pages need a head size that is a multiple of 32, got {hs}")
    p = torch.arange(PAGE).view(PAGE, 1)
    d = torch.arange(hs).view(1, hs)
    b, r = p // 32, p % 32
    tile, i = (r // 4) % 2, (r // 8) * 4 + r % 4
    k_index = 32 * hs * b + 8 * (64 * (2 * (d // 32) + tile) + 16 * ((d // 8) % 4) + i) + d % 8
    v_index = 32 * hs * b + 8 * (64 * (d // 16) + 16 * ((p // 8) % 4) + d % 16) + p % 8
    return k_index.contiguous(), v_index.t().contiguous()


def to_blocked_pages(k_rows: torch.Tensor, v_transposed: torch.Tensor):
    """Pages [n, Hkv, PAGE, hs] of keys and [n, Hkv, hs, PAGE] of transposed values as blocked pages (the same shapes)."""
    hs = k_rows.shape[-1]
    ki, vi = (t.to(k_rows.device).reshape(-1) for t in blocked_page_index(hs))
    k = torch.empty_like(k_rows).view(*k_rows.shape[:2], -1)
    v = torch.empty_like(v_transposed).view(*v_transposed.shape[:2], -1)
    k[..., ki] = k_rows.reshape(*k_rows.shape[:2], -1)
    v[..., vi] = v_transposed.reshape(*v_transposed.shape[:2], -1)
    return k.view(k_rows.shape), v.view(v_transposed.shape)


def from_blocked_pages(k_blocked: torch.Tensor, v_blocked: torch.Tensor):
    """The inverse of to_blocked_pages: keys as rows, values transposed."""
    hs = k_blocked.shape[-1]
    ki, vi = (t.to(k_blocked.device).reshape(-1) for t in blocked_page_index(hs))
    k = k_blocked.reshape(*k_blocked.shape[:2], -1)[..., ki].view(k_blocked.shape)
    v = v_blocked.reshape(*v_blocked.shape[:2], -1)[..., vi].view(v_blocked.shape)
    return k.contiguous(), v.contiguous()


def rope_kv_write(qkv: torch.Tensor, positions: torch.Tensor, H: int, Hkv: int, hs: int, *,
                  inv_freq=None, rope_dims: int = 0, seq_index=None, block_table=None,
                  k_pages=None, v_pages=None, page_tiles=None, v_transposed=None, blocked=None) -> None:
    """Rotate the Q heads of qkv ([T, (H+2Hkv)*hs]) in place, rotate the K heads and store
    them and the V heads at each token's position of its sequence's pages.
    k_pages None: rotate Q only.  rope_dims 0: no rotation.  positions < 0: padding rows.
    page_tiles (optional, [n, 4] int32 = sequence, first row, rows, position of the first; each
    tile inside one page, all rows covered): transposed or blocked V pages are then filled by a kernel
    that stores runs of positions instead of single elements.
    v_transposed, blocked: the layout of the pages (neither: kernel_v_layout of qkv's type and hs)."""
    require_gpu()
    _dev(qkv, "qkv", dims=2)
    _dev(positions, "positions", torch.int32, 1)
    T = qkv.shape[0]
    stride = _rows(qkv, "qkv")
    if qkv.shape[1] < (H + 2 * Hkv) * hs or positions.numel() != T or not positions.is_contiguous():
        raise KernelError(f"rope_kv_write: qkv {tuple(qkv.shape)} / positions {tuple(positions.shape)} do not "
                          f"fit H={H} Hkv={Hkv} hs={hs}")
    if rope_dims:
        _dev(inv_freq, "inv_freq", torch.float32, 1)
        if rope_dims % 2 or rope_dims > hs or inv_freq.numel() != rope_dims // 2 or not inv_freq.is_contiguous():
            raise KernelError(f"rope_kv_write: rope_dims {rope_dims} does not fit hs={hs} / inv_freq "
                              f"{tuple(inv_freq.shape)}")
    bt_stride = 0
    layout = "rows"
    if k_pages is not None:
        layout = _check_pages(k_pages, v_pages, Hkv, hs, qkv.dtype, v_transposed, blocked)
        _dev(seq_index, "seq_index", torch.int32, 1)
        _dev(block_table, "block_table", torch.int32, 2)
        if seq_index.numel() != T or not seq_index.is_contiguous() or not block_table.is_contiguous():
            raise KernelError("rope_kv_write: seq_index must have one entry per token; tables contiguous")
        bt_stride = block_table.shape[1]
    if T == 0:
        return
    tiled_v = (page_tiles is not None and k_pages is not None and layout != "rows" and qkv.dtype == torch.bfloat16     # a bf16 kernel
               and hs % 8 == 0 and stride % 8 == 0
               and qkv.data_ptr() % 16 == 0 and hs * (PAGE + 2) * 2 <= 65536 and Hkv <= 65535)
    if tiled_v:
        _dev(page_tiles, "page_tiles", torch.int32, 2)
        if page_tiles.shape[1] != 4 or not page_tiles.is_contiguous() or page_tiles.shape[0] == 0:
            raise KernelError("rope_kv_write: page_tiles must be a contiguous [n, 4] tensor")
    if (tiled_v and rope_dims > 0 and rope_dims % 16 == 0
            and (k_pages.data_ptr() | v_pages.data_ptr()) % 16 == 0):
        # the rows that the 16-byte kernel takes: rotation, keys and the values' tiles in one launch
        _check(_fn("rope_kv", "bn_rope_kv_write_tiles")(
            qkv.data_ptr(), stride, positions.data_ptr(), seq_index.data_ptr(), block_table.data_ptr(), bt_stride,
            k_pages.data_ptr(), v_pages.data_ptr(), inv_freq.data_ptr(), rope_dims, T, H, Hkv, hs, _LAYOUT_CODES[layout],
            page_tiles.data_ptr(), page_tiles.shape[0], _stream()), "rope_kv_write(tiles)")
        return
    _check(_fn("rope_kv", "bn_rope_kv_write")(
        _code(qkv.dtype), qkv.data_ptr(), stride, positions.data_ptr(),
        seq_index.data_ptr() if k_pages is not None else None,
        block_table.data_ptr() if k_pages is not None else None, bt_stride,
        k_pages.data_ptr() if k_pages is not None else None,
        v_pages.data_ptr() if k_pages is not None else None,
        inv_freq.data_ptr() if rope_dims else None, rope_dims, T, H, Hkv, hs,
        _LAYOUT_CODES[layout] + (4 if tiled_v else 0), _stream()), "rope_kv_write")
    if tiled_v:
        _check(_fn("rope_kv", "bn_v_transposed_write")(
            qkv.data_ptr(), stride, page_tiles.data_ptr(), page_tiles.shape[0], block_table.data_ptr(), bt_stride,
            v_pages.data_ptr(), H, Hkv, hs, int(layout == "blocked"), _stream()), "v_transposed_write")


MAX_HEAD_DIM = _build.header_constant("BN_MAX_HEAD_DIM")    # the attention kernels take every even head size up to this


def _pow2_at_least(n: int) -> int:
    p = 1
    while p < n:
        p *= 2
    return p


MFMA_HEAD_DIMS = (_build.header_constant("BN_MFMA_HEAD_DIM_SMALL"), _build.header_constant("BN_MFMA_HEAD_DIM_LARGE"))


def mfma_attention(dtype, hs: int) -> bool:
    """Whether the matrix-core attention kernels take this cache type and head size (bn_attn_mfma_supports, answered
    from the header so that asking loads no kernel)."""
    return dtype == torch.bfloat16 and int(hs) in MFMA_HEAD_DIMS


def attention_row_shape(H: int, Hkv: int, decode: bool, dtype=None, hs: int = 0):
    """(RT, GT, QT): what one workgroup covers: QT query tokens x GT heads of one kv group
    (RT = QT * GT rows for the vector kernel)."""
    G = H // Hkv
    GT = min(_pow2_at_least(G), 16)
    if decode:
        return GT, GT, 1
    if dtype is not None and mfma_attention(dtype, hs):
        qt = _fn("attn_mfma", "bn_attn_mfma_prompt_tokens")(int(hs), GT)
        return qt * GT, GT, qt
    return 16, GT, 16 // GT


def pair_tiles(rows: list) -> list:
    """The order in which the prompt form of the matrix-core attention wants its tiles (sequence, first row, rows,
    position of the first): it gives a workgroup two consecutive tiles of the list when there are more tiles than
    CUs, and a causal tile's work grows with its position.  So a sequence's tile with the most keys is followed by
    its tile with the fewest, the second by the last but one, and so on (equal work per workgroup); sequences follow
    each other, longest first, so that workgroups that run together walk the same keys; the middle tiles of
    sequences with an odd number of them are paired with each other at the end.  The result of the attention does
    not depend on the order."""
    by_seq = {}
    for r in rows:
        by_seq.setdefault(r[0], []).append(r)
    keys = lambda r: r[3] + r[2]
    out, single = [], []
    for seq in sorted(by_seq, key=lambda q: -max(keys(r) for r in by_seq[q])):
        ts = sorted(by_seq[seq], key=lambda r: -keys(r))
        n = len(ts)
        for p in range(n // 2):
            out += [ts[p], ts[n - 1 - p]]
        if n % 2:
            single.append(ts[n // 2])
    single.sort(key=lambda r: -keys(r))
    n = len(single)
    for p in range(n // 2):
        out += [single[p], single[n - 1 - p]]
    if n % 2:
        out.append(single[n // 2])
    return out


# Workgroups that a decode attention launch aims for when it cuts the keys: one for every CU of this chip.  (Measured at
# 8,000 and 32,000 cached tokens a sequence and 1 to 8 sequences of the 8B shape: about 256 workgroups are fastest
# whatever the batch, 29 us against 35 for 504 at one sequence of 32,000 tokens, 183 against 188 at eight.)
DECODE_TARGET_WGS = int(os.environ.get("BITNET_DECODE_WGS", "256"))


VECTOR_DECODE_TARGET_WGS = int(os.environ.get("BITNET_VECTOR_DECODE_WGS", "1024"))     # see decode_splits


def decode_splits(n_seqs: int, H: int, Hkv: int, max_len: int, dtype=None, target_wgs: int = 0):
    """(n_splits, chunk): how the keys of a decode step are cut so that the launch fills the
    chip.  A function of the batch's shape and of max_len alone.  A float32 cache is cut in runs of F32_FOLD_KEYS
    positions whatever the batch: both forms of the float32 kernel sum a query's keys run by run and fold the runs in
    order, so a decode step may give every run a workgroup and float32 logits stay equal bit for bit under every cut."""
    if dtype == torch.float32:
        return max(1, (max_len + F32_FOLD_KEYS - 1) // F32_FOLD_KEYS), F32_FOLD_KEYS
    RT, GT, _ = attention_row_shape(H, Hkv, True)
    G = H // Hkv
    wgs = max(1, n_seqs * Hkv * ((G + GT - 1) // GT))
    pages = max(1, (max_len + PAGE - 1) // PAGE)
    # about DECODE_TARGET_WGS workgroups, but no split shorter than SPLIT_MIN_PAGES pages: below that the merging costs
    # more than the parallelism gains (measured at batch 1, 8 and 64 of the 8B shape)
    # target_wgs: another aim than DECODE_TARGET_WGS (the vector kernel's workgroups are small, several fit on a CU and
    # hide each other's waits: VECTOR_DECODE_TARGET_WGS)
    target = target_wgs or DECODE_TARGET_WGS
    want = max(1, min(pages // SPLIT_MIN_PAGES, 64, (target + wgs - 1) // wgs))
    chunk = ((pages + want - 1) // want) * PAGE
    n_splits = (pages * PAGE + chunk - 1) // chunk
    return n_splits, chunk


def split_chunk(max_len: int, n_splits: int) -> int:
    """Keys per split when a launch of n_splits splits meets sequences of up to max_len keys (bn_split_chunk of
    csrc/common.h): what the kernels compute themselves when the length comes in device memory."""
    pages = max(1, (max_len + PAGE - 1) // PAGE)
    return max(SPLIT_MIN_PAGES, (pages + n_splits - 1) // n_splits) * PAGE


def can_fuse_decode(dtype, H: int, Hkv: int, hs: int) -> bool:
    """Whether decode attention can rotate Q and K and store the new K, V itself."""
    return mfma_attention(dtype, hs) and H // Hkv <= 16


def _sink_args(sink, H: int, what: str):
    """(flag, address) of a softmax's sink as the kernels take it: False or None, no sink; True, one more term of score
    0; a float32 tensor [H], one more term of that score per head."""
    if sink is None or sink is False:
        return 0, None
    if sink is True:
        return 1, None
    _dev(sink, "sink", torch.float32, 1)
    if sink.numel() != H or not sink.is_contiguous():
        raise KernelError(f"{what}: a sink with scores holds one float32 per head ({H}), got {tuple(sink.shape)}")
    return 1, sink.data_ptr()


def attention(qkv: torch.Tensor, out: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
              block_table: torch.Tensor, H: int, Hkv: int, hs: int, scale: float, *, window: int = 0,
              tiles=None, qt: int = 0, seq_lens=None, n_splits: int = 1, chunk: int = 0,
              force_vector: bool = False, fused_rotate=None, fused_write: bool = False, by_length=None,
              max_len_dev=None, v_transposed=None, row_scale: Optional["DeferredNorm"] = None, blocked=None,
              v_dim: int = 0, distance_bias=None, sink: bool = False) -> None:
    """Causal attention of the (rotated) Q heads in qkv over the paged cache.

    Prompt form: `tiles` [n, 4] int32 = (sequence, first token row, tokens (<= qt), position of
    the first), qt = the QT of attention_row_shape(H, Hkv, False, dtype, hs).
    Decode form: tiles None, seq_lens [B] int32 (keys in the cache, the new one included; 0 for a
    padding row); row b of qkv is sequence b's token; n_splits/chunk from decode_splits.  Every entry of
    block_table names a page of the pool, also those behind a sequence's last page (0 will do): the
    matrix-core kernel asks for a workgroup's first block of keys before it knows the sequence's length.
    bf16 with head size 64 or 128 over blocked pages runs on the matrix cores, everything else on the vector ALUs,
    which read rows and transposed values (force_vector: say so where the pages are not blocked and the head size
    would be the other kernel's; its qt then is that of attention_row_shape without dtype).
    Decode on the matrix cores can do the work of rope_kv_write itself (can_fuse_decode):
    fused_rotate = inv_freq [hs/2]: qkv arrives unrotated, Q and the new K are rotated inside;
    fused_write: the new K, V of every row (from qkv) are stored at position seq_lens - 1 first.
    by_length (decode form, optional): [B] int32, a permutation of the rows, longest sequence
    first; the matrix-core kernel hands out its workgroups in that order when a launch puts several
    on every CU, so that long and short sequences share CUs.  It changes no result.
    max_len_dev (decode form, optional): a device int32 holding the longest sequence's key count; with
    n_splits > 1 the kernels then cut the keys into n_splits runs of split_chunk(max_len, n_splits) and
    `chunk` is not used, so that one captured launch serves every length up to the block table's width.
    v_transposed, blocked: the layout of the pages (neither: kernel_v_layout of qkv's type and hs).
    window with n_splits > 1 (decode form on the vector kernel, bf16): the splits are counted from the page that holds the
    window's first key, so n_splits * chunk need only cover window + PAGE positions, whatever the sequences' lengths.
    row_scale (decode form on the matrix cores with fused_rotate): a DeferredNorm whose factor the rows of qkv still
    lack (qkv is the product of its bf16 copy with the stacked weights); the kernel multiplies q and the new key and
    value of every row by it.
    What only the vector kernel does (pages that are not blocked): v_dim, value heads of another width than the keys'
    (out is then [T, H * v_dim]); distance_bias = (a, b), two float32 tensors [H]: a[h] * ln(1 + b[h] * (i - j)) is taken
    off the score of query position i and key position j; sink: the softmax has one more term without a value: True, of
    score 0 (1 is added to its denominator); a float32 tensor [H], of that score per head (exp(sink[h]) is added)."""
    require_gpu()
    _dev(qkv, "qkv", dims=2)
    _dev(out, "out", qkv.dtype, 2)
    vd = int(v_dim) or hs
    layout = _check_pages(k_pages, v_pages, Hkv, hs, qkv.dtype, v_transposed, blocked, vd)
    vt = layout != "rows"
    _dev(block_table, "block_table", torch.int32, 2)
    T = qkv.shape[0]
    if H % Hkv or qkv.shape[1] < H * hs or out.shape != (T, H * vd) or not out.is_contiguous():
        raise KernelError(f"attention: qkv {tuple(qkv.shape)} / out {tuple(out.shape)} do not fit H={H} hs={hs} v_dim={vd}")
    if vd % 2 or vd < 2 or vd > MAX_HEAD_DIM:
        raise KernelError(f"attention: value width {vd} is not supported (even, at most {MAX_HEAD_DIM})")
    sink_flag, sink_ptr = _sink_args(sink, H, "attention")
    extras = vd != hs or distance_bias is not None or bool(sink_flag)
    if extras and layout == "blocked":
        raise KernelError("attention: another value width, a distance bias and a sink are the vector kernel's, which reads "
                          "pages with a row per position or transposed values")
    da = db = None
    if distance_bias is not None:
        da, db = distance_bias
        for t, nm in ((da, "distance_bias[0]"), (db, "distance_bias[1]")):
            _dev(t, nm, torch.float32, 1)
            if t.numel() != H or not t.is_contiguous():
                raise KernelError(f"attention: {nm} must hold one float32 per head")
    if hs % 2 or hs < 2 or hs > MAX_HEAD_DIM:
        raise KernelError(f"attention: head size {hs} is not supported (even, at most {MAX_HEAD_DIM})")
    if not block_table.is_contiguous():
        raise KernelError("attention: block_table must be contiguous")
    decode = tiles is None
    use_mfma = layout == "blocked"
    if use_mfma and (force_vector or not mfma_attention(qkv.dtype, hs)):
        raise KernelError(f"attention: blocked pages are read by the matrix-core kernels alone (head size {hs}, "
                          f"force_vector={force_vector})")
    if not use_mfma and mfma_attention(qkv.dtype, hs) and not force_vector:
        force_vector = True          # pages in another order than the matrix-core kernels': the vector kernel reads them
    RT, GT, QT = attention_row_shape(H, Hkv, decode, qkv.dtype if use_mfma else None, hs)
    if decode:
        _dev(seq_lens, "seq_lens", torch.int32, 1)
        if seq_lens.numel() != T or block_table.shape[0] < T or not seq_lens.is_contiguous():
            raise KernelError("attention(decode): one seq_lens entry and one block_table row per token")
        n_tiles = T
    else:
        _dev(tiles, "tiles", torch.int32, 2)
        if tiles.shape[1] != 4 or not tiles.is_contiguous() or qt != QT:
            raise KernelError(f"attention(prompt): tiles must be [n, 4] built for qt={QT}, got qt={qt}")
        n_tiles = tiles.shape[0]
        n_splits, chunk = 1, 0
    if T == 0 or n_tiles == 0:
        return
    part_o = part_ml = None
    fold = F32_FOLD_KEYS if qkv.dtype == torch.float32 else 0       # float32: runs of keys folded in order, in both forms
    if fold:
        if decode and n_splits > 1 and chunk != fold:
            raise KernelError(f"attention: a float32 cache's keys are split in runs of {fold}, not {chunk}")
        max_len_dev = None                                          # and the runs do not follow the longest sequence
    if max_len_dev is not None:
        _dev(max_len_dev, "max_len_dev", torch.int32)
        if not decode or max_len_dev.numel() != 1:
            raise KernelError("attention: max_len_dev is one int32 and belongs to the decode form")
        chunk = split_chunk(block_table.shape[1] * PAGE, n_splits)         # of the longest sequence the table can hold
    if n_splits > 1:
        if chunk <= 0 or chunk % PAGE:
            raise KernelError(f"attention: chunk {chunk} must be a positive multiple of {PAGE}")
        cover = block_table.shape[1] * PAGE
        if window and decode and not use_mfma:           # the vector kernel counts a windowed step's splits from the window's first page
            cover = min(cover, window + PAGE)
        if n_splits * chunk < cover:
            raise KernelError(f"attention: {n_splits} splits of {chunk} keys do not cover the "
                              f"{block_table.shape[1]} pages of the block table")
        if n_splits > (1024 if fold else 64):
            raise KernelError("attention: at most 64 splits (1,024 runs of a float32 cache)")
        part_o = torch.empty((T * H * n_splits, vd), dtype=torch.float32, device=qkv.device)
        part_ml = torch.empty((T * H * n_splits, 2), dtype=torch.float32, device=qkv.device)
    po = part_o.data_ptr() if part_o is not None else None
    pm = part_ml.data_ptr() if part_ml is not None else None
    sl = seq_lens.data_ptr() if decode else None
    tl = tiles.data_ptr() if not decode else None
    if by_length is not None:
        _dev(by_length, "by_length", torch.int32, 1)
        if not decode or by_length.numel() != T or not by_length.is_contiguous():
            raise KernelError("attention: by_length is one entry per row of the decode form")
    fused = fused_rotate is not None or fused_write
    if fused and not (use_mfma and decode and can_fuse_decode(qkv.dtype, H, Hkv, hs)):
        raise KernelError("attention: rotation / cache write inside the kernel needs the decode form on the "
                          "matrix cores with at most 16 heads per kv head")
    if fused_rotate is not None:
        _dev(fused_rotate, "fused_rotate", torch.float32, 1)
        if fused_rotate.numel() != hs // 2 or not fused_rotate.is_contiguous():
            raise KernelError(f"attention: fused rotation needs {hs // 2} frequencies (full rotary)")
    if fused_write and qkv.shape[1] < (H + 2 * Hkv) * hs:
        raise KernelError("attention: fused cache write needs the K and V heads in qkv")
    if row_scale is not None:
        if not (use_mfma and decode and fused_rotate is not None):
            raise KernelError("attention: a deferred norm's factor is applied by the decode form on the matrix cores "
                              "with the rotation inside the kernel, and by nothing else")
        _dev(row_scale.slots, "row_scale.slots", torch.float32, 2)
        if row_scale.slots.shape[0] != T or not row_scale.slots.is_contiguous() or not 1 <= row_scale.slots.shape[1] <= 64:
            raise KernelError(f"attention: row_scale slots {tuple(row_scale.slots.shape)} do not fit {T} rows (1 to 64 pieces)")
        _check(_fn("attn_mfma", "bn_attn_mfma_scaled")(
            qkv.data_ptr(), _rows(qkv, "qkv"), out.data_ptr(), H * hs, k_pages.data_ptr(), v_pages.data_ptr(),
            block_table.data_ptr(), block_table.shape[1], sl, T, H, Hkv, hs, GT, int(window), float(scale), int(n_splits),
            int(chunk), po, pm, fused_rotate.data_ptr(), int(bool(fused_write)),
            by_length.data_ptr() if by_length is not None else None,
            max_len_dev.data_ptr() if max_len_dev is not None else None, row_scale.slots.data_ptr(),
            row_scale.slots.shape[1], row_scale.stream.shape[1], float(row_scale.eps), _stream()), "attention(mfma, scaled)")
        return
    if use_mfma:
        _check(_fn("attn_mfma", "bn_attn_mfma")(
            qkv.data_ptr(), _rows(qkv, "qkv"), out.data_ptr(), H * hs, k_pages.data_ptr(), v_pages.data_ptr(),
            block_table.data_ptr(), block_table.shape[1], sl, tl, n_tiles, T, H, Hkv, hs, GT, int(window),
            float(scale), int(n_splits), int(chunk), po, pm,
            fused_rotate.data_ptr() if fused_rotate is not None else None, int(fused_rotate is not None),
            int(bool(fused_write)), by_length.data_ptr() if by_length is not None else None,
            max_len_dev.data_ptr() if max_len_dev is not None else None, _stream()),
            "attention(mfma)")
        return
    _check(_fn("attn_rows", "bn_attn_rows")(
        _code(qkv.dtype), qkv.data_ptr(), _rows(qkv, "qkv"), out.data_ptr(), H * vd,
        k_pages.data_ptr(), v_pages.data_ptr(), block_table.data_ptr(), block_table.shape[1],
        sl, tl, n_tiles, T, H, Hkv, hs, RT, GT, int(window), float(scale), int(n_splits), int(chunk),
        po, pm, int(vt), max_len_dev.data_ptr() if max_len_dev is not None else None, int(fold), vd,
        da.data_ptr() if da is not None else None, db.data_ptr() if db is not None else None, sink_flag, sink_ptr, _stream()),
        "attention")



# --------------------------------------------------------------------------------------
# attention without a rotation: head norms, query temperature, cache write
# --------------------------------------------------------------------------------------

def qk_norm_store(qkv: torch.Tensor, positions: torch.Tensor, H: int, Hkv: int, hs: int, *, v_dim: int = 0,
                  q_weight=None, k_weight=None, eps: float = 0.0, temp_coef: float = 0.0, temp_every: int = 0,
                  seq_index=None, block_table=None, k_pages=None, v_pages=None, v_transposed: bool = False,
                  norm_projection: bool = False, inv_freq=None, rope_dims: int = 0, rope_interleaved: bool = False,
                  v_from_k: bool = False) -> None:
    """In place on qkv [T, H hs + Hkv (hs + v_dim)]: every query and key head under an RMSNorm of its own (weights
    [hs] float32, shared by the heads; both or neither), or, with norm_projection, one RMSNorm over the whole query
    projection and one over the whole key projection (weights [H hs] and [Hkv hs]); then the first rope_dims dimensions
    of every query and key head rotated by the position (inv_freq [rope_dims / 2] float32; pairs (2i, 2i + 1) when
    rope_interleaved, (i, i + rope_dims / 2) otherwise; inv_freq None: no rotation); the queries times
    1 + temp_coef ln(floor((p + 1) / temp_every) + 1) at position p (temp_every 0: no temperature); the keys and the
    values go into the pages when pages are given (keys a row per position; values the same way, or transposed inside a
    page when v_transposed).  Rows with position < 0 are left alone.  v_from_k: the values are the key projections as
    they arrived (before norm and rotation); qkv is [T, (H + Hkv) hs] then and v_dim equals hs."""
    require_gpu()
    _dev(qkv, "qkv", dims=2)
    _dev(positions, "positions", torch.int32, 1)
    vd = int(v_dim) or hs
    T = qkv.shape[0]
    if v_from_k and vd != hs:
        raise KernelError(f"qk_norm_store: values that are the keys are as wide as the keys, got {vd} and {hs}")
    if (positions.numel() != T or qkv.shape[1] < H * hs + Hkv * (hs if v_from_k else hs + vd)
            or (q_weight is None) != (k_weight is None)):
        raise KernelError(f"qk_norm_store: qkv {tuple(qkv.shape)} does not fit H={H} Hkv={Hkv} hs={hs} v_dim={vd}")
    for w, nm, heads in ((q_weight, "q_weight", H), (k_weight, "k_weight", Hkv)):
        if w is not None:
            _dev(w, nm, torch.float32, 1)
            want = hs * heads if norm_projection else hs
            if w.numel() != want or not w.is_contiguous():
                raise KernelError(f"qk_norm_store: {nm} must hold {want} float32 values")
    if hs > MAX_HEAD_DIM:
        raise KernelError(f"qk_norm_store: head size {hs} is above {MAX_HEAD_DIM}")
    if inv_freq is not None:
        _dev(inv_freq, "inv_freq", torch.float32, 1)
        if rope_dims <= 0 or rope_dims % 2 or rope_dims > hs or inv_freq.numel() != rope_dims // 2 or not inv_freq.is_contiguous():
            raise KernelError(f"qk_norm_store: rope_dims {rope_dims} does not fit hs={hs} / inv_freq {tuple(inv_freq.shape)}")
    if k_pages is not None:
        _check_pages(k_pages, v_pages, Hkv, hs, qkv.dtype, bool(v_transposed), False, vd)
        _dev(seq_index, "seq_index", torch.int32, 1)
        _dev(block_table, "block_table", torch.int32, 2)
        if seq_index.numel() != T or not block_table.is_contiguous():
            raise KernelError("qk_norm_store: one seq_index entry per row and a contiguous block table")
    if T == 0:
        return
    _check(_fn("qk_norm", "bn_qk_norm_store")(
        _code(qkv.dtype), qkv.data_ptr(), _rows(qkv, "qkv"), positions.data_ptr(),
        seq_index.data_ptr() if k_pages is not None else None, block_table.data_ptr() if k_pages is not None else None,
        block_table.shape[1] if k_pages is not None else 0, k_pages.data_ptr() if k_pages is not None else None,
        v_pages.data_ptr() if k_pages is not None else None, q_weight.data_ptr() if q_weight is not None else None,
        k_weight.data_ptr() if k_weight is not None else None, T, H, Hkv, hs, vd, float(eps), float(temp_coef),
        int(temp_every), int(bool(v_transposed)), int(bool(norm_projection)),
        inv_freq.data_ptr() if inv_freq is not None else None, int(rope_dims), int(bool(rope_interleaved)),
        int(bool(v_from_k)), _stream()), "qk_norm_store")


GENERAL_PROMPT_TILE = 16       # query tokens of a tile of attention_general_prompt
# BITNET_NO_GENERAL_MFMA=1 keeps the attention mixer's general form on the vector kernel in prompt steps too
GENERAL_PROMPT_ON_MATRIX_CORES = os.environ.get("BITNET_NO_GENERAL_MFMA", "") in ("", "0")
_GENERAL_SIZES = (32, 64, 96, 128, 256)        # key widths; values may also be 192 wide (a latent beside a rotated key part)


def attention_general_supported(dtype, hs: int, v_dim: int) -> bool:
    """Whether attention_general_prompt takes this type and these head sizes (bn_attn_general_supports, answered here so
    that asking loads no kernel)."""
    return dtype == torch.bfloat16 and int(hs) in _GENERAL_SIZES and int(v_dim) in _GENERAL_SIZES + (192,)


def attention_general_prompt(qkv: torch.Tensor, out: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                             block_table: torch.Tensor, H: int, Hkv: int, hs: int, v_dim: int, scale: float, tiles: torch.Tensor,
                             *, distance_bias=None, sink: bool = False, window: int = 0) -> None:
    """Causal prompt attention on the matrix cores for what attention() leaves to the vector kernel: bf16, keys 32, 64,
    96, 128 or 256 wide, values of a width of their own from the same list, a distance bias and a sink (as attention()'s),
    a window (> 0: a query sees the last `window` positions, its own included).  qkv's row stride is a multiple of 8.
    Pages: keys a row per position, values transposed.  tiles [n, 4] int32: (sequence, first row, rows <= 16, position of
    the first), any order, tiles of no rows skipped.  out [T, H v_dim]."""
    require_gpu()
    _dev(qkv, "qkv", torch.bfloat16, 2)
    _dev(out, "out", torch.bfloat16, 2)
    if not attention_general_supported(qkv.dtype, hs, v_dim):
        raise KernelError(f"attention_general_prompt: bf16 with head sizes from {_GENERAL_SIZES}, got {hs} and {v_dim}")
    _check_pages(k_pages, v_pages, Hkv, hs, qkv.dtype, True, False, v_dim)
    _dev(block_table, "block_table", torch.int32, 2)
    _dev(tiles, "tiles", torch.int32, 2)
    T = qkv.shape[0]
    if (H % Hkv or qkv.shape[1] < H * hs or out.shape != (T, H * v_dim) or not out.is_contiguous() or tiles.shape[1] != 4
            or not tiles.is_contiguous() or not block_table.is_contiguous()):
        raise KernelError(f"attention_general_prompt: qkv {tuple(qkv.shape)} / out {tuple(out.shape)} / tiles {tuple(tiles.shape)} "
                          f"do not fit H={H} hs={hs} v_dim={v_dim}")
    da = db = None
    if distance_bias is not None:
        da, db = distance_bias
        for t, nm in ((da, "distance_bias[0]"), (db, "distance_bias[1]")):
            _dev(t, nm, torch.float32, 1)
            if t.numel() != H or not t.is_contiguous():
                raise KernelError(f"attention_general_prompt: {nm} must hold one float32 per head")
    if window < 0 or _rows(qkv, "qkv") % 8 or qkv.data_ptr() % 16:
        raise KernelError(f"attention_general_prompt: window {window} / row stride {_rows(qkv, 'qkv')} (a multiple of 8, 16-byte aligned)")
    if T == 0 or tiles.shape[0] == 0:
        return
    _check(_fn("attn_mfma_general", "bn_attn_general_prompt")(
        qkv.data_ptr(), _rows(qkv, "qkv"), out.data_ptr(), H * v_dim, k_pages.data_ptr(), v_pages.data_ptr(),
        block_table.data_ptr(), block_table.shape[1], tiles.data_ptr(), tiles.shape[0], H, Hkv, hs, v_dim, float(scale),
        da.data_ptr() if da is not None else None, db.data_ptr() if db is not None else None,
        *_sink_args(sink, H, "attention_general_prompt"), int(window), _stream()), "attention_general_prompt")


def general_decode_plan(n_seqs: int, H: int, Hkv: int, max_len: int, window: int = 0):
    """(n_splits, chunk, follows_length) for attention_general_decode: how a decode step's keys are cut so that the launch
    fills the chip with its one-wave workgroups.  Without a window the plan follows max_len (the cache's bound in a
    captured step: pass max_len_dev then, and the keys per split follow the longest sequence of each replay); with a window
    it depends on the window alone, because the kernel counts the splits from the window's first page."""
    if window:
        n_splits, chunk = decode_splits(n_seqs, H, Hkv, window + PAGE, torch.bfloat16, target_wgs=VECTOR_DECODE_TARGET_WGS)
        return n_splits, chunk, False
    n_splits, chunk = decode_splits(n_seqs, H, Hkv, max_len, torch.bfloat16, target_wgs=VECTOR_DECODE_TARGET_WGS)
    return n_splits, chunk, True


def attention_general_decode(qkv: torch.Tensor, out: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                             block_table: torch.Tensor, seq_lens: torch.Tensor, H: int, Hkv: int, hs: int, v_dim: int, scale: float,
                             *, window: int = 0, n_splits: int = 1, chunk: int = 0, max_len_dev=None, distance_bias=None,
                             sink: bool = False) -> None:
    """The decode form of attention_general_prompt (bf16, the same head sizes and pages): row b of qkv is sequence b's new
    token, seq_lens [B] its keys in the cache (0: a padding row, whose output is zeros).  A wave takes the heads that share
    a kv head together, so their keys and values are read once.  n_splits > 1 cuts the keys into runs of `chunk` positions
    (a multiple of PAGE; with max_len_dev, a device int32, into runs of split_chunk(longest sequence, n_splits)), merged in
    index order; with a window the runs are counted from the page of the window's first key and need only cover
    window + PAGE positions.  distance_bias, sink: as attention()'s."""
    require_gpu()
    _dev(qkv, "qkv", torch.bfloat16, 2)
    _dev(out, "out", torch.bfloat16, 2)
    if not attention_general_supported(qkv.dtype, hs, v_dim):
        raise KernelError(f"attention_general_decode: bf16 with head sizes from {_GENERAL_SIZES}, got {hs} and {v_dim}")
    _check_pages(k_pages, v_pages, Hkv, hs, qkv.dtype, True, False, v_dim)
    _dev(block_table, "block_table", torch.int32, 2)
    _dev(seq_lens, "seq_lens", torch.int32, 1)
    T = qkv.shape[0]
    if (H % Hkv or qkv.shape[1] < H * hs or out.shape != (T, H * v_dim) or not out.is_contiguous() or seq_lens.numel() != T
            or block_table.shape[0] < T or not block_table.is_contiguous() or not seq_lens.is_contiguous()):
        raise KernelError(f"attention_general_decode: qkv {tuple(qkv.shape)} / out {tuple(out.shape)} / seq_lens "
                          f"{tuple(seq_lens.shape)} do not fit H={H} hs={hs} v_dim={v_dim}")
    if window < 0 or _rows(qkv, "qkv") % 8 or qkv.data_ptr() % 16:
        raise KernelError(f"attention_general_decode: window {window} / row stride {_rows(qkv, 'qkv')} (a multiple of 8, 16-byte aligned)")
    da = db = None
    if distance_bias is not None:
        da, db = distance_bias
        for t, nm in ((da, "distance_bias[0]"), (db, "distance_bias[1]")):
            _dev(t, nm, torch.float32, 1)
            if t.numel() != H or not t.is_contiguous():
                raise KernelError(f"attention_general_decode: {nm} must hold one float32 per head")
    part_o = part_ml = None
    if n_splits > 1:
        if max_len_dev is not None:
            _dev(max_len_dev, "max_len_dev", torch.int32)
            if max_len_dev.numel() != 1 or window:
                raise KernelError("attention_general_decode: max_len_dev is one int32 and belongs to steps without a window")
            chunk = split_chunk(block_table.shape[1] * PAGE, n_splits)
        if chunk <= 0 or chunk % PAGE or n_splits > 64:
            raise KernelError(f"attention_general_decode: chunk {chunk} must be a positive multiple of {PAGE}, at most 64 splits")
        cover = min(block_table.shape[1] * PAGE, window + PAGE) if window else block_table.shape[1] * PAGE
        if n_splits * chunk < cover:
            raise KernelError(f"attention_general_decode: {n_splits} splits of {chunk} keys do not cover {cover} positions")
        part_o = torch.empty((T * H * n_splits, v_dim), dtype=torch.float32, device=qkv.device)
        part_ml = torch.empty((T * H * n_splits, 2), dtype=torch.float32, device=qkv.device)
    if T == 0:
        return
    _check(_fn("attn_mfma_general", "bn_attn_general_decode")(
        qkv.data_ptr(), _rows(qkv, "qkv"), out.data_ptr(), H * v_dim, k_pages.data_ptr(), v_pages.data_ptr(),
        block_table.data_ptr(), block_table.shape[1], seq_lens.data_ptr(), T, H, Hkv, hs, v_dim, float(scale),
        da.data_ptr() if da is not None else None, db.data_ptr() if db is not None else None,
        *_sink_args(sink, H, "attention_general_decode"), int(window), int(n_splits), int(chunk), part_o.data_ptr() if part_o is not None else None,
        part_ml.data_ptr() if part_ml is not None else None,
        max_len_dev.data_ptr() if (max_len_dev is not None and n_splits > 1) else None, _stream()), "attention_general_decode")


# --------------------------------------------------------------------------------------
# row-wise kernels of other architectures' parts
# --------------------------------------------------------------------------------------

UNARY_ACTIVATIONS = {n: _build.header_constant("BN_UNARY_" + n.upper()) for n in
                     ("gelu_erf", "gelu_tanh", "silu", "relu2", "tanh", "sigmoid")}


def unary_act(x: torch.Tensor, activation: str, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """activation(x) element by element (float32 arithmetic); one of UNARY_ACTIVATIONS.  out: where to (x itself will do)."""
    require_gpu()
    _dev(x, "x")
    if activation not in UNARY_ACTIVATIONS:
        raise KernelError(f"unknown activation {activation!r}; known: {sorted(UNARY_ACTIVATIONS)}")
    if out is None:
        out = torch.empty_like(x)
    if not x.is_contiguous() or not out.is_contiguous() or out.shape != x.shape or out.dtype != x.dtype:
        raise KernelError("unary_act: x and out must be contiguous and alike")
    if x.numel():
        _check(_fn("elementwise", "bn_unary_act_apply")(_code(x.dtype), out.data_ptr(), x.data_ptr(), x.numel(),
                                                        UNARY_ACTIVATIONS[activation], _stream()), "unary_act")
    return out


def scale_(x: torch.Tensor, factor: float) -> None:
    """In place: float32 x times a constant (an architecture's multiplier of its logits)."""
    require_gpu()
    _dev(x, "x", torch.float32)
    if not x.is_contiguous():
        raise KernelError("scale_: a contiguous float32 tensor")
    if x.numel():
        _check(_fn("elementwise", "bn_scale")(x.data_ptr(), x.numel(), float(factor), _stream()), "scale")


def sinusoid_frequencies(dim: int, base: float) -> torch.Tensor:
    """base^(-2i/dim) for i < ceil(dim / 2), formed in double and rounded to float32 once."""
    i = torch.arange((dim + 1) // 2, dtype=torch.float64)
    return torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / dim).to(torch.float32)


def embed_gather_sinusoid(table: torch.Tensor, tokens: torch.Tensor, positions: torch.Tensor, freq: torch.Tensor,
                          scale: float = 1.0) -> torch.Tensor:
    """embed_gather plus a sinusoidal position vector: entry 2i gets sin(p freq[i]), entry 2i + 1 cos(p freq[i])."""
    require_gpu()
    _dev(table, "table", dims=2)
    _dev(tokens, "tokens", torch.int32, 1)
    _dev(positions, "positions", torch.int32, 1)
    _dev(freq, "freq", torch.float32, 1)
    n, dim = tokens.numel(), table.shape[1]
    if (not table.is_contiguous() or not tokens.is_contiguous() or not positions.is_contiguous() or positions.numel() != n
            or freq.numel() != (dim + 1) // 2 or not freq.is_contiguous()):
        raise KernelError("embed_gather_sinusoid: contiguous inputs, a position per token and ceil(dim / 2) frequencies")
    x = torch.empty((n, dim), dtype=torch.float32, device=table.device)
    if n:
        _check(_fn("elementwise", "bn_embed_gather_sinusoid")(
            _code(table.dtype), x.data_ptr(), table.data_ptr(), tokens.data_ptr(), positions.data_ptr(), freq.data_ptr(),
            n, dim, table.shape[0], float(scale), _stream()), "embed_gather_sinusoid")
    return x


def rmsnorm_mean(a: torch.Tensor, wa: torch.Tensor, b: Optional[torch.Tensor], wb: Optional[torch.Tensor],
                 eps: float) -> torch.Tensor:
    """The mean of two branches [T, D], each under an RMSNorm of its own (float32 weights [D]); b None: a alone."""
    require_gpu()
    _dev(a, "a", dims=2)
    _dev(wa, "wa", torch.float32, 1)
    T, D = a.shape
    if not a.is_contiguous() or wa.numel() != D or not wa.is_contiguous():
        raise KernelError("rmsnorm_mean: a contiguous [T, D] and D weights")
    if b is not None:
        _dev(b, "b", a.dtype, 2)
        _dev(wb, "wb", torch.float32, 1)
        if b.shape != a.shape or not b.is_contiguous() or wb.numel() != D or not wb.is_contiguous():
            raise KernelError("rmsnorm_mean: the branches must be alike")
    out = torch.empty_like(a)
    if T:
        _check(_fn("elementwise", "bn_rmsnorm_mean")(_code(a.dtype), out.data_ptr(), a.data_ptr(),
                                                     b.data_ptr() if b is not None else None, wa.data_ptr(),
                                                     wb.data_ptr() if b is not None else None, T, D, float(eps), _stream()),
               "rmsnorm_mean")
    return out


# --------------------------------------------------------------------------------------
# mixers with a state of fixed size (csrc/state_mixers.hip)
# --------------------------------------------------------------------------------------

SEQUENCE_TILE = 1 << 30          # StepContext.tiles(SEQUENCE_TILE): one tile a sequence, for kernels that walk a sequence's tokens
WKV_MAX_DIM = _build.header_constant("WKV_MAX_DIM", "state_mixers.hip")


def _seq_args(tiles, seq_lens, what: str):
    """(tiles pointer, number of tiles, seq_lens pointer): a prompt step names its sequences by tiles [n, 4], a decode
    step by seq_lens [B] (row b = sequence b's one token)."""
    if tiles is not None:
        _dev(tiles, "tiles", torch.int32, 2)
        if tiles.shape[1] != 4 or not tiles.is_contiguous():
            raise KernelError(f"{what}: tiles must be contiguous [n, 4]")
        return tiles.data_ptr(), tiles.shape[0], None
    _dev(seq_lens, "seq_lens", torch.int32, 1)
    if not seq_lens.is_contiguous():
        raise KernelError(f"{what}: seq_lens must be contiguous")
    return None, seq_lens.numel(), seq_lens.data_ptr()


def _state_rows(state: torch.Tensor, need: int, what: str) -> int:
    _dev(state, "state", torch.float32, 2)
    if state.stride(1) != 1 or state.shape[1] < need:
        raise KernelError(f"{what}: the state must be float32 [slots, >= {need}] with contiguous rows, got {tuple(state.shape)}")
    return state.stride(0)


def token_shift(h: torch.Tensor, mu: torch.Tensor, state: torch.Tensor, positions, seq_index, slot_ids) -> torch.Tensor:
    """[n_mix, T, D]: h[t] + (h[t-1] - h[t]) * mu[s] for every mix s; the token before a step's first is read from the
    first D values of the sequence's state row (state: [slots, >= D], a view that starts at those values), and is 0 at
    position 0.  Reads the state only."""
    require_gpu()
    _dev(h, "h", dims=2)
    _dev(mu, "mu", torch.float32, 2)
    T, D = h.shape
    if not h.is_contiguous() or mu.shape[1] != D or not mu.is_contiguous():
        raise KernelError("token_shift: h contiguous [T, D], mu contiguous [n_mix, D]")
    stride = _state_rows(state, D, "token_shift")
    for t, nm, n in ((positions, "positions", T), (seq_index, "seq_index", T)):
        _dev(t, nm, torch.int32, 1)
        if t.numel() != n or not t.is_contiguous():
            raise KernelError(f"token_shift: {nm} has one entry per row")
    _dev(slot_ids, "slot_ids", torch.int32, 1)
    out = torch.empty((mu.shape[0], T, D), dtype=h.dtype, device=h.device)
    if T:
        _check(_fn("state_mixers", "bn_token_shift")(_code(h.dtype), out.data_ptr(), h.data_ptr(), mu.data_ptr(), state.data_ptr(),
                                                     stride, positions.data_ptr(), seq_index.data_ptr(),
                                                     slot_ids.data_ptr(), T, D, mu.shape[0], _stream()), "token_shift")
    return out


def wkv_supported(dk: int, dv: int) -> bool:
    return 1 <= dk <= WKV_MAX_DIM and 1 <= dv <= WKV_MAX_DIM


WKV_ROWS_PER_THREAD = _build.header_constant("WKV_KR", "state_mixers.hip")


def wkv_state_floats(H: int, dk: int, dv: int) -> int:
    """float32 values of the matrix states of H heads as wkv_scan keeps them: the dk rows of a head are rounded up to a
    power of two times the rows a thread holds (the kernel spreads a column's rows over that many neighbouring lanes and
    stores the state in the lanes' order, which no one else reads)."""
    if not wkv_supported(dk, dv):
        raise KernelError(f"wkv: head sizes up to {WKV_MAX_DIM}, got {dk} x {dv}")
    p = 1
    while p * WKV_ROWS_PER_THREAD < dk:
        p *= 2
    return H * p * WKV_ROWS_PER_THREAD * dv


def wkv_scan(r, k, v, d, w0, u, h, state, slot_ids, H: int, dk: int, dv: int, *, tiles=None, seq_lens=None) -> torch.Tensor:
    """The wkv recurrence over every sequence of a step; float32 [T, H dv].  r, k, d: [T, H dk] (rows contiguous, any row
    stride), v: [T, H dv], in the activations' type; w0, u: float32 [H dk] (the decay's offset, the current token's
    bonus); h [T, D]: the mixer's input.  state [slots, >= wkv_state_floats(H, dk, dv) + D] float32: the heads' matrices
    in the kernel's own order, then the last h, both updated in place.  Per head, in float32:
        w_t = exp(-exp(d_t + w0));  o_t = (S + diag(u) k_t v_t^T)^T r_t;  S <- diag(w_t) S + k_t v_t^T."""
    require_gpu()
    _dev(h, "h", dims=2)
    T, D = h.shape
    if not wkv_supported(dk, dv):
        raise KernelError(f"wkv_scan: head sizes up to {WKV_MAX_DIM}, got {dk} x {dv}")
    for t, nm, n in ((r, "r", H * dk), (k, "k", H * dk), (v, "v", H * dv), (d, "d", H * dk)):
        _dev(t, nm, h.dtype, 2)
        if t.shape != (T, n):
            raise KernelError(f"wkv_scan: {nm} must be [{T}, {n}], got {tuple(t.shape)}")
    for t, nm in ((w0, "w0"), (u, "u")):
        _dev(t, nm, torch.float32, 1)
        if t.numel() != H * dk or not t.is_contiguous():
            raise KernelError(f"wkv_scan: {nm} must hold {H * dk} float32 values")
    if not h.is_contiguous():
        raise KernelError("wkv_scan: h must be contiguous")
    stride = _state_rows(state, wkv_state_floats(H, dk, dv) + D, "wkv_scan")
    _dev(slot_ids, "slot_ids", torch.int32, 1)
    tl, n_tiles, sl = _seq_args(tiles, seq_lens, "wkv_scan")
    o = torch.empty((T, H * dv), dtype=torch.float32, device=h.device)
    if T and n_tiles:
        _check(_fn("state_mixers", "bn_wkv_scan")(
            _code(h.dtype), r.data_ptr(), _rows(r, "r"), k.data_ptr(), _rows(k, "k"), v.data_ptr(), _rows(v, "v"),
            d.data_ptr(), _rows(d, "d"), w0.data_ptr(), u.data_ptr(), o.data_ptr(), h.data_ptr(), state.data_ptr(), stride,
            tl, n_tiles, sl, slot_ids.data_ptr(), H, dk, dv, D, _stream()), "wkv_scan")
    return o


def head_norm_gate(o: torch.Tensor, gate: torch.Tensor, weight: torch.Tensor, H: int, dv: int, eps: float) -> torch.Tensor:
    """o [T, H dv] float32, each head divided by its root mean square (eps inside the root), times weight [H dv]
    (float32), times silu(gate) (gate [T, H dv] in the activations' type, which is the result's)."""
    require_gpu()
    _dev(o, "o", torch.float32, 2)
    _dev(gate, "gate", dims=2)
    _dev(weight, "weight", torch.float32, 1)
    T = o.shape[0]
    if o.shape[1] != H * dv or not o.is_contiguous() or gate.shape != o.shape or weight.numel() != H * dv or not weight.is_contiguous():
        raise KernelError("head_norm_gate: o and gate [T, H dv], weight [H dv]")
    y = torch.empty((T, H * dv), dtype=gate.dtype, device=o.device)
    if T:
        _check(_fn("state_mixers", "bn_head_norm_gate")(_code(gate.dtype), y.data_ptr(), o.data_ptr(), gate.data_ptr(),
                                                        _rows(gate, "gate"), weight.data_ptr(), T, H, dv, float(eps), _stream()),
               "head_norm_gate")
    return y


def mingru_scan(zxg: torch.Tensor, bias_z, bias_x, state: torch.Tensor, slot_ids, W: int, *, tiles=None,
                seq_lens=None) -> torch.Tensor:
    """The min-GRU recurrence over every sequence of a step.  zxg [T, 3 W]: the projections of the update gate, the
    candidate and the output gate side by side, without biases (bias_z, bias_x: float32 [W] or None).  state
    [slots, >= W] float32, updated in place.  Per channel, in float32: z = sigmoid(a + bias_z); c = b + bias_x;
    cand = c + 1/2 where c >= 0, sigmoid(c) below; S <- (1 - z) S + z cand; result S * silu(g), [T, W]."""
    require_gpu()
    _dev(zxg, "zxg", dims=2)
    T = zxg.shape[0]
    if zxg.shape[1] != 3 * W:
        raise KernelError(f"mingru_scan: zxg must be [T, {3 * W}], got {tuple(zxg.shape)}")
    for t, nm in ((bias_z, "bias_z"), (bias_x, "bias_x")):
        if t is not None:
            _dev(t, nm, torch.float32, 1)
            if t.numel() != W or not t.is_contiguous():
                raise KernelError(f"mingru_scan: {nm} must hold {W} float32 values")
    stride = _state_rows(state, W, "mingru_scan")
    _dev(slot_ids, "slot_ids", torch.int32, 1)
    tl, n_tiles, sl = _seq_args(tiles, seq_lens, "mingru_scan")
    y = torch.empty((T, W), dtype=zxg.dtype, device=zxg.device)
    if T and n_tiles:
        _check(_fn("state_mixers", "bn_mingru_scan")(
            _code(zxg.dtype), y.data_ptr(), zxg.data_ptr(), _rows(zxg, "zxg"),
            bias_z.data_ptr() if bias_z is not None else None, bias_x.data_ptr() if bias_x is not None else None,
            state.data_ptr(), stride, tl, n_tiles, sl, slot_ids.data_ptr(), W, _stream()), "mingru_scan")
    return y


# --------------------------------------------------------------------------------------
# a part's output with a norm of its own; latent attention; mixture of experts
# --------------------------------------------------------------------------------------

LIGHTNING_MAX_DIM = _build.header_constant("LA_MAX_DIM", "lightning.hip")


def lightning_supported(dk: int, dv: int) -> bool:
    return 1 <= dk <= LIGHTNING_MAX_DIM and dv >= 1


def lightning_chunked(dk: int, dv: int) -> bool:
    """Whether prompt steps of these head sizes take the chunked form of the recurrence."""
    return bool(_fn("lightning", "bn_lightning_chunked")(int(dk), int(dv)))


def lightning_scan(x: torch.Tensor, q_col: int, k_col: int, v_col: int, decay: torch.Tensor, state: torch.Tensor, slot_ids,
                   H: int, dk: int, dv: int, *, tiles=None, seq_lens=None, chain: Optional[bool] = None) -> torch.Tensor:
    """Linear attention with a fixed decay per head over every sequence of a step; float32 [T, H dv].  x [T, >= ...] in
    the activations' type holds the projections side by side: queries at column q_col and keys at k_col (H dk wide),
    values at v_col (H dv wide); each passes silu in float32.  decay [H] float32.  state [slots, >= H dk dv] float32, the
    heads' matrices [H][dk][dv], updated in place; a sequence at position 0 starts from zeros.  Per head, in float32:
        S <- decay S + k_t v_t^T;  o_t = S^T q_t.
    A prompt step (tiles) of a key width that lightning_chunked() takes can run the same sums chunk by chunk on the matrix
    cores, in float32, instead of token by token as decode steps do.  chain: True the token-by-token kernel, False the
    chunks where they can be, None whichever is the faster for this many sequences and heads."""
    require_gpu()
    _dev(x, "x", dims=2)
    _dev(decay, "decay", torch.float32, 1)
    T = x.shape[0]
    if not lightning_supported(dk, dv):
        raise KernelError(f"lightning_scan: key width up to {LIGHTNING_MAX_DIM}, got {dk} x {dv}")
    ld = _rows(x, "x")
    if (decay.numel() != H or not decay.is_contiguous() or min(q_col, k_col, v_col) < 0
            or max(q_col + H * dk, k_col + H * dk, v_col + H * dv) > x.shape[1]):
        raise KernelError(f"lightning_scan: x {tuple(x.shape)} does not hold H={H} heads of {dk} / {dv} at columns "
                          f"{q_col}, {k_col}, {v_col}, or decay is not [H]")
    stride = _state_rows(state, H * dk * dv, "lightning_scan")
    _dev(slot_ids, "slot_ids", torch.int32, 1)
    tl, n_seqs, sl = _seq_args(tiles, seq_lens, "lightning_scan")
    if tiles is None and n_seqs != T:
        raise KernelError("lightning_scan: a decode step has one length per row")
    o = torch.empty((T, H * dv), dtype=torch.float32, device=x.device)
    if T and n_seqs:
        prepared = None
        if tiles is not None and chain is not True and lightning_chunked(dk, dv) and (
                chain is False or _fn("lightning", "bn_lightning_prefers_chunks")(n_seqs, H, dk, dv)):
            # the chunked form's own copy of the step's q, k and v: silu applied, float32, head by head
            prepared = torch.empty(H * T * (2 * ((dk + 3) // 4 * 4) + (dv + 3) // 4 * 4), dtype=torch.float32, device=x.device)
        _check(_fn("lightning", "bn_lightning_scan")(_code(x.dtype), x.data_ptr(), ld, int(q_col), int(k_col), int(v_col),
                                                     decay.data_ptr(), o.data_ptr(), state.data_ptr(), stride, tl, n_seqs, sl,
                                                     slot_ids.data_ptr(), H, dk, dv, T,
                                                     prepared.data_ptr() if prepared is not None else None, _stream()),
               "lightning_scan")
    return o


def row_norm_gate(o: torch.Tensor, gate: torch.Tensor, weight: torch.Tensor, eps: float, activation: str = "sigmoid") -> torch.Tensor:
    """o [T, W] float32 divided by its rows' root mean square (eps inside the root), times weight [W] (float32), times
    act(gate) (gate [T, W] in the activations' type, which is the result's; act one of UNARY_ACTIVATIONS)."""
    require_gpu()
    _dev(o, "o", torch.float32, 2)
    _dev(gate, "gate", dims=2)
    _dev(weight, "weight", torch.float32, 1)
    T, W = o.shape
    if not o.is_contiguous() or tuple(gate.shape) != (T, W) or weight.numel() != W or not weight.is_contiguous():
        raise KernelError("row_norm_gate: o and gate [T, W], weight [W]")
    if activation not in UNARY_ACTIVATIONS:
        raise KernelError(f"unknown activation {activation!r}; known: {sorted(UNARY_ACTIVATIONS)}")
    y = torch.empty((T, W), dtype=gate.dtype, device=o.device)
    if T:
        _check(_fn("lightning", "bn_row_norm_gate")(_code(gate.dtype), y.data_ptr(), o.data_ptr(), gate.data_ptr(),
                                                    _rows(gate, "gate"), weight.data_ptr(), T, W, float(eps),
                                                    UNARY_ACTIVATIONS[activation], _stream()), "row_norm_gate")
    return y


def add_normed_rmsnorm(x: torch.Tensor, delta, out_weight: torch.Tensor, out_eps: float, weight: Optional[torch.Tensor] = None,
                       eps: float = 0.0, out_dtype=None, rows_out: bool = False):
    """x (float32, [T, D]) += out_weight * delta / sqrt(mean(delta^2) + out_eps), row by row in float32; delta [T, D]
    in x's or the activations' type, or PartialSums (its slabs are added first).  With `weight`, also returns the rows of
    the new x under an RMSNorm (weight, eps) in out_dtype: a block's output norm, the residual sum and the next part's
    norm in one kernel.  rows_out (without weight): returns the rows of the new x themselves in out_dtype, for a next part
    that reads the stream as it is."""
    require_gpu()
    _dev(x, "x", torch.float32, 2)
    _dev(out_weight, "out_weight", torch.float32, 1)
    T, D = x.shape
    parts = delta if isinstance(delta, PartialSums) else None
    d = parts.slabs if parts is not None else delta
    _dev(d, "delta")
    if tuple(parts.shape if parts is not None else d.shape) != (T, D) or not d.is_contiguous() or not x.is_contiguous():
        raise KernelError(f"add_normed_rmsnorm: delta does not match x {tuple(x.shape)}, or is not contiguous")
    if out_weight.numel() != D or not out_weight.is_contiguous() or D > 16384:
        raise KernelError(f"add_normed_rmsnorm: the output norm's weight must hold {D} (at most 16,384) values")
    if parts is None and d.dtype not in _DT:
        raise KernelError(f"add_normed_rmsnorm: unsupported delta type {d.dtype}")
    out = None
    if weight is not None and rows_out:
        raise KernelError("add_normed_rmsnorm: either the rows under a norm (weight) or the rows themselves (rows_out)")
    if weight is not None:
        _dev(weight, "weight", torch.float32, 1)
        if weight.numel() != D or not weight.is_contiguous():
            raise KernelError(f"add_normed_rmsnorm: weight must hold {D} values")
    if weight is not None or rows_out:
        out = torch.empty((T, D), dtype=out_dtype or (torch.float32 if parts is not None else d.dtype), device=x.device)
    # the kernel's type names the type of out and of a delta that is no float32 slab
    code = _code(out.dtype) if out is not None else (_code(torch.float32) if parts is not None else _code(d.dtype))
    if parts is None and out is not None and out.dtype != d.dtype:
        raise KernelError("add_normed_rmsnorm: delta and the normed rows have one type")
    if T == 0:
        return out
    _check(_fn("elementwise", "bn_add_normed_rmsnorm")(
        code, x.data_ptr(), d.data_ptr(), parts.slabs.shape[0] if parts is not None else 1, int(parts is not None),
        out_weight.data_ptr(), float(out_eps), weight.data_ptr() if weight is not None else None,
        out.data_ptr() if out is not None else None, T, D, float(eps), _stream()), "add_normed_rmsnorm")
    return out


def latent_store(x: torch.Tensor, col: int, rank: int, weight: torch.Tensor, eps: float, positions, seq_index, block_table,
                 k_pages: torch.Tensor, v_pages: torch.Tensor, *, rot_dims: int = 0, inv_freq: Optional[torch.Tensor] = None,
                 rot_mult: float = 1.0) -> None:
    """Columns col .. col + rank of every row of x under an RMSNorm (weight [rank] float32, eps inside the root, float32
    arithmetic), stored at the row's position of its sequence's pages: as a key row ([pages, 1, PAGE, rank]) and into the
    transposed value page ([pages, 1, rank, PAGE]).  Rows with position < 0 store nothing.
    rot_dims > 0: the next rot_dims columns of x are one more key part, not normed, dimension i turned with dimension
    i + rot_dims / 2 by position * inv_freq[i] (cosine and sine times rot_mult); a key row is then rank + rot_dims wide
    and holds it behind the latent, the value page stays rank wide."""
    require_gpu()
    _dev(x, "x", dims=2)
    _dev(weight, "weight", torch.float32, 1)
    _dev(positions, "positions", torch.int32, 1)
    _dev(seq_index, "seq_index", torch.int32, 1)
    _dev(block_table, "block_table", torch.int32, 2)
    T = x.shape[0]
    rot_dims = int(rot_dims)
    _check_pages(k_pages, v_pages, 1, rank + rot_dims, x.dtype, True, False, rank)
    if rot_dims:
        _dev(inv_freq, "inv_freq", torch.float32, 1)
        if rot_dims % 2 or inv_freq.numel() != rot_dims // 2 or not inv_freq.is_contiguous():
            raise KernelError(f"latent_store: {rot_dims} rotated dimensions need {rot_dims // 2} frequencies")
    if (col < 0 or x.shape[1] < col + rank + rot_dims or weight.numel() != rank or not weight.is_contiguous() or positions.numel() != T
            or seq_index.numel() != T or not block_table.is_contiguous()):
        raise KernelError(f"latent_store: x {tuple(x.shape)} / columns {col}..{col + rank} / weight {tuple(weight.shape)} do not fit")
    if T == 0:
        return
    _check(_fn("latent", "bn_latent_store")(_code(x.dtype), x.data_ptr(), _rows(x, "x"), int(col), positions.data_ptr(),
                                            seq_index.data_ptr(), block_table.data_ptr(), block_table.shape[1],
                                            k_pages.data_ptr(), v_pages.data_ptr(), weight.data_ptr(), T, int(rank), float(eps),
                                            rot_dims, inv_freq.data_ptr() if rot_dims else None, float(rot_mult),
                                            _stream()), "latent_store")


def rope_heads(x: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor, H: int, head_stride: int, offset: int,
               rot_dims: int, mult: float = 1.0) -> None:
    """In place on x [T, >= (H - 1) head_stride + offset + rot_dims]: in every head (head h starts at column
    h * head_stride) the rot_dims columns from `offset` on are rotated, dimension i with dimension i + rot_dims / 2, by
    position * inv_freq[i]; cosine and sine times `mult`.  Rows with position < 0 are left alone."""
    require_gpu()
    _dev(x, "x", dims=2)
    _dev(positions, "positions", torch.int32, 1)
    _dev(inv_freq, "inv_freq", torch.float32, 1)
    T = x.shape[0]
    if (rot_dims <= 0 or rot_dims % 2 or inv_freq.numel() != rot_dims // 2 or not inv_freq.is_contiguous() or offset < 0
            or head_stride < offset + rot_dims or x.shape[1] < (H - 1) * head_stride + offset + rot_dims or positions.numel() != T):
        raise KernelError(f"rope_heads: x {tuple(x.shape)} does not fit {H} heads of stride {head_stride} with {rot_dims} "
                          f"rotated columns from {offset}")
    if T:
        _check(_fn("latent", "bn_rope_heads")(_code(x.dtype), x.data_ptr(), _rows(x, "x"), positions.data_ptr(),
                                              inv_freq.data_ptr(), T, int(H), int(head_stride), int(offset), int(rot_dims),
                                              float(mult), _stream()), "rope_heads")


HEAD_LINEAR_MAX_IN = 1792          # the kernel stages 8 rows of a head's input as float32 beside its partial sums in 64 KB of shared memory


def head_linear(x: torch.Tensor, w: torch.Tensor, gate: Optional[torch.Tensor] = None, *,
                allow_library: Optional[bool] = None, gate_per_head: bool = False) -> torch.Tensor:
    """A product per head: y[t, h, :] = x[t, h, :] . w[h] with x [T, H I] (rows contiguous), w [H, I, O] -> y [T, H O];
    with `gate` [T, H O] (rows contiguous) y is multiplied by sigmoid(gate) element by element, or, with gate_per_head,
    head h of y by sigmoid of the one number gate[t, h] (gate [T, H]).  float32 accumulation.
    bf16 with more than SKINNY_ROWS rows goes to the library's batched product (allow_library as linear's), everything else
    to a kernel that reads every head's matrix once for 8 rows."""
    require_gpu()
    _dev(x, "x", dims=2)
    _dev(w, "w", x.dtype, 3)
    T = x.shape[0]
    H, I, O = w.shape
    if x.shape[1] != H * I or not w.is_contiguous():
        raise KernelError(f"head_linear: x {tuple(x.shape)} and w {tuple(w.shape)} do not fit")
    if gate is not None:
        _dev(gate, "gate", x.dtype, 2)
        if tuple(gate.shape) != (T, H if gate_per_head else H * O):
            raise KernelError(f"head_linear: gate {tuple(gate.shape)} is not [{T}, {H if gate_per_head else H * O}]")
    group = O if gate_per_head else 1
    y = torch.empty((T, H * O), dtype=x.dtype, device=x.device)
    if T == 0:
        return y
    if allow_library is None:
        allow_library = LIBRARY_PRODUCTS
    ldx = _rows(x, "x")
    if x.dtype == torch.bfloat16 and T > SKINNY_ROWS and allow_library:
        xv = x.as_strided((H, T, I), (I, ldx, 1))
        torch.bmm(xv, w, out=y.view(T, H, O).transpose(0, 1))
        if gate is not None:
            _check(_fn("latent", "bn_sigmoid_gate")(_code(y.dtype), y.data_ptr(), H * O, gate.data_ptr(), _rows(gate, "gate"),
                                                    group, T, H * O, _stream()), "sigmoid_gate")
        return y
    if I > HEAD_LINEAR_MAX_IN:
        raise KernelError(f"head_linear: a head's input of {I} values is above {HEAD_LINEAR_MAX_IN}")
    _check(_fn("latent", "bn_head_linear")(_code(x.dtype), x.data_ptr(), ldx, w.data_ptr(), y.data_ptr(), H * O,
                                           gate.data_ptr() if gate is not None else None,
                                           _rows(gate, "gate") if gate is not None else 0, group, T, H, I, O, _stream()),
           "head_linear")
    return y


# --------------------------------------------------------------------------------------
# a residual of several streams and the norm without statistics (csrc/hyper.hip)
# --------------------------------------------------------------------------------------

HC_MAX_STREAMS = _build.header_constant("BN_HC_MAX_STREAMS", "hyper.hip")


def hc_step(lanes_in: torch.Tensor, lanes_out: Optional[torch.Tensor], n: int, *, delta=None, mix=None, out_coef=None,
            mult: float = 1.0, in_coef=None, norm=None, out_dtype=None, rows=None, read: bool = True):
    """One pass over a residual of n streams.  lanes_in: [n, T, D] float32, or [T, D] read as every stream.  With `delta`
    (a sublayer's output [T, D], float32 or bf16, or PartialSums) the streams are rebuilt first, x_t <- sum_s mix[s, t] x_s +
    mult out_coef[t] delta, and stored in lanes_out [n, T, D] (which may be lanes_in; None: not stored).  Then, with `read`,
    u = sum_s in_coef[s] x_s (in_coef None: the plain sum) is returned as [T or len(rows), D]: under norm = (weight, bias,
    alpha) as tanh(alpha u) weight + bias in out_dtype, else u itself in out_dtype (float32 unless said).  rows: a choice of
    rows (int32) for the result; the streams are then not stored.  mix [n, n], out_coef [n], in_coef [n] float32."""
    require_gpu()
    _dev(lanes_in, "lanes_in", torch.float32)
    if lanes_in.dim() == 2:
        T, D = lanes_in.shape
        in_stride = 0
    else:
        if lanes_in.dim() != 3 or lanes_in.shape[0] != n:
            raise KernelError(f"hc_step: {n} streams do not fit {tuple(lanes_in.shape)}")
        _, T, D = lanes_in.shape
        in_stride = T * D
    if not lanes_in.is_contiguous() or not 1 <= n <= HC_MAX_STREAMS:
        raise KernelError(f"hc_step: contiguous streams, at most {HC_MAX_STREAMS}")
    if lanes_out is not None:
        _dev(lanes_out, "lanes_out", torch.float32, 3)
        if tuple(lanes_out.shape) != (n, T, D) or not lanes_out.is_contiguous() or rows is not None:
            raise KernelError(f"hc_step: lanes_out {tuple(lanes_out.shape)} is not [{n}, {T}, {D}], or a choice of rows stores streams")
    d_ptr, d_code, n_slabs = None, 0, 0
    if delta is not None:
        slabs = delta.slabs if isinstance(delta, PartialSums) else delta
        _dev(slabs, "delta")
        if tuple(slabs.shape[-2:]) != (T, D) or not slabs.is_contiguous() or slabs.dim() not in (2, 3):
            raise KernelError(f"hc_step: delta {tuple(slabs.shape)} does not match the streams [{T}, {D}]")
        n_slabs = slabs.shape[0] if slabs.dim() == 3 else 1
        if slabs.dtype != torch.float32 and n_slabs != 1:
            raise KernelError("hc_step: several slabs are float32 slabs")
        d_ptr, d_code = slabs.data_ptr(), _code(slabs.dtype)
        for t, nm, cnt in ((mix, "mix", n * n), (out_coef, "out_coef", n)):
            _dev(t, nm, torch.float32)
            if t.numel() != cnt or not t.is_contiguous():
                raise KernelError(f"hc_step: {nm} must hold {cnt} float32 values")
    if in_coef is not None:
        _dev(in_coef, "in_coef", torch.float32, 1)
        if in_coef.numel() != n or not in_coef.is_contiguous():
            raise KernelError(f"hc_step: in_coef must hold {n} float32 values")
    n_rows = T
    if rows is not None:
        _dev(rows, "rows", torch.int32, 1)
        if not rows.is_contiguous():
            raise KernelError("hc_step: rows must be contiguous")
        n_rows = rows.numel()
    w = b = alpha = None
    if norm is not None:
        w, b, alpha = norm
        for t, nm, cnt in ((w, "norm weight", D), (b, "norm bias", D), (alpha, "norm alpha", 1)):
            _dev(t, nm, torch.float32)
            if t.numel() != cnt or not t.is_contiguous():
                raise KernelError(f"hc_step: {nm} must hold {cnt} float32 values")
    h = None
    if read:
        h = torch.empty((n_rows, D), dtype=out_dtype or torch.float32, device=lanes_in.device)
    if n_rows == 0 or T == 0:
        return h
    _check(_fn("hyper", "bn_hc_step")(
        d_code, _code(h.dtype) if h is not None else 0, lanes_in.data_ptr(), in_stride,
        lanes_out.data_ptr() if lanes_out is not None else None, T * D, d_ptr, n_slabs, T * D,
        mix.data_ptr() if delta is not None else None, out_coef.data_ptr() if delta is not None else None, float(mult),
        in_coef.data_ptr() if in_coef is not None else None, w.data_ptr() if w is not None else None,
        b.data_ptr() if b is not None else None, alpha.data_ptr() if alpha is not None else None,
        h.data_ptr() if h is not None else None, rows.data_ptr() if rows is not None else None, n_rows, T, D, int(n),
        _stream()), "hc_step")
    return h


def add_dyt_norm(x: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, bias: torch.Tensor, alpha: torch.Tensor,
                 out_dtype, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x (float32 [T, D]) += delta (out_dtype, optional; not with a choice of rows), then tanh(alpha x) * weight + bias of
    all rows or of `rows`, in out_dtype.  weight, bias [D] and alpha (one number) float32 on the device."""
    require_gpu()
    _dev(x, "x", torch.float32, 2)
    T, D = x.shape
    for t, nm, cnt in ((weight, "weight", D), (bias, "bias", D), (alpha, "alpha", 1)):
        _dev(t, nm, torch.float32)
        if t.numel() != cnt or not t.is_contiguous():
            raise KernelError(f"add_dyt_norm: {nm} must hold {cnt} float32 values")
    if not x.is_contiguous() or (rows is not None and delta is not None):
        raise KernelError("add_dyt_norm: x contiguous; a choice of rows leaves the stream as it is")
    if delta is not None:
        _dev(delta, "delta", out_dtype, 2)
        if delta.shape != x.shape or not delta.is_contiguous():
            raise KernelError(f"add_dyt_norm: delta {tuple(delta.shape)} does not match x {tuple(x.shape)}")
    n = T
    if rows is not None:
        _dev(rows, "rows", torch.int32, 1)
        n = rows.numel()
    out = torch.empty((n, D), dtype=out_dtype, device=x.device)
    if n:
        _check(_fn("hyper", "bn_dyt_norm")(_code(out_dtype), x.data_ptr(), delta.data_ptr() if delta is not None else None,
                                           weight.data_ptr(), bias.data_ptr(), alpha.data_ptr(), out.data_ptr(),
                                           rows.data_ptr() if rows is not None else None, n, D, _stream()), "add_dyt_norm")
    return out


# --------------------------------------------------------------------------------------
# short convolutions and recurrences with a float32 state (csrc/conv_scans.hip)
# --------------------------------------------------------------------------------------

CONV_MAX_TAPS = _build.header_constant("BN_CONV_MAX_TAPS", "conv_scans.hip")
GLA_MAX_DIM = _build.header_constant("GLA_MAX_DIM", "conv_scans.hip")


def short_conv(x: torch.Tensor, col: int, weight: torch.Tensor, bias: Optional[torch.Tensor], state: torch.Tensor, positions,
               seq_index, slot_ids, *, tiles=None, seq_lens=None, out_dtype=None) -> torch.Tensor:
    """A causal convolution over time on C channels of x (columns col .. col + C): y_t = sum_j weight[:, j] u_(t - taps + 1 + j)
    (+ bias), zeros before a sequence's first token.  weight [C, taps], bias [C] float32.  state: float32
    [slots, >= (taps - 1) C] (a view that starts at this convolution's values): a sequence's inputs before the step's
    first token, oldest first; read for a step's first tokens and left holding the step's last inputs.  tiles (one a
    sequence) in a prompt step, seq_lens in a decode step.  Returns y [T, C] in out_dtype (x's unless said)."""
    require_gpu()
    _dev(x, "x", dims=2)
    _dev(weight, "weight", torch.float32, 2)
    T = x.shape[0]
    C, taps = weight.shape
    if not weight.is_contiguous() or not 1 <= taps <= CONV_MAX_TAPS or col < 0 or x.shape[1] < col + C:
        raise KernelError(f"short_conv: x {tuple(x.shape)} / columns {col}..{col + C} / weight {tuple(weight.shape)} do not fit "
                          f"(at most {CONV_MAX_TAPS} taps)")
    if bias is not None:
        _dev(bias, "bias", torch.float32, 1)
        if bias.numel() != C or not bias.is_contiguous():
            raise KernelError(f"short_conv: bias must hold {C} float32 values")
    stride = _state_rows(state, (taps - 1) * C, "short_conv")
    for t, nm in ((positions, "positions"), (seq_index, "seq_index")):
        _dev(t, nm, torch.int32, 1)
        if t.numel() != T or not t.is_contiguous():
            raise KernelError(f"short_conv: {nm} must hold one int32 per row")
    _dev(slot_ids, "slot_ids", torch.int32, 1)
    tl, n_seqs, sl = _seq_args(tiles, seq_lens, "short_conv")
    if tl is None and n_seqs != T:
        raise KernelError("short_conv: a decode step has one row a sequence")
    y = torch.empty((T, C), dtype=out_dtype or x.dtype, device=x.device)
    if T and n_seqs:
        _check(_fn("conv_scans", "bn_short_conv")(
            _code(x.dtype), _code(y.dtype), x.data_ptr(), _rows(x, "x"), int(col), y.data_ptr(), C, weight.data_ptr(),
            bias.data_ptr() if bias is not None else None, state.data_ptr(), stride, positions.data_ptr(), seq_index.data_ptr(),
            slot_ids.data_ptr(), tl, sl, n_seqs, T, C, taps, _stream()), "short_conv")
    return y


def lru_gates(u: torch.Tensor, wa_t: torch.Tensor, ba: torch.Tensor, wi_t: torch.Tensor, bi: torch.Tensor,
              c_neg: torch.Tensor):
    """The operands of a real-gated linear recurrent unit from its input u [T, W] float32: u in `blocks` equal parts, in
    part b r = sigmoid(u_b . wa_t[b] + ba), i = sigmoid(u_b . wi_t[b] + bi) (wa_t, wi_t [blocks, in, out] float32, the
    biases [W]); a = exp(c_neg r) (c_neg [W], the channel's -8 softplus(lam)).  Returns (a, sqrt(1 - a^2) i u), float32
    [T, W] each.  All of it in float32."""
    require_gpu()
    _dev(u, "u", torch.float32, 2)
    T, W = u.shape
    _dev(wa_t, "wa_t", torch.float32, 3)
    _dev(wi_t, "wi_t", torch.float32, 3)
    blocks = wa_t.shape[0]
    bw = W // max(blocks, 1)
    if (blocks < 1 or W % blocks or tuple(wa_t.shape) != (blocks, bw, bw) or tuple(wi_t.shape) != (blocks, bw, bw)
            or not (u.is_contiguous() and wa_t.is_contiguous() and wi_t.is_contiguous()) or bw * 32 + 32768 > 64 * 1024):
        raise KernelError(f"lru_gates: u {tuple(u.shape)} and gate matrices {tuple(wa_t.shape)} / {tuple(wi_t.shape)} do not fit")
    for t, nm in ((ba, "ba"), (bi, "bi"), (c_neg, "c_neg")):
        _dev(t, nm, torch.float32, 1)
        if t.numel() != W or not t.is_contiguous():
            raise KernelError(f"lru_gates: {nm} must hold {W} float32 values")
    a = torch.empty((T, W), dtype=torch.float32, device=u.device)
    b = torch.empty((T, W), dtype=torch.float32, device=u.device)
    if T:
        _check(_fn("conv_scans", "bn_lru_gates")(u.data_ptr(), wa_t.data_ptr(), ba.data_ptr(), wi_t.data_ptr(), bi.data_ptr(),
                                                 c_neg.data_ptr(), a.data_ptr(), b.data_ptr(), T, W, blocks, _stream()), "lru_gates")
    return a, b


def lru_scan(a: torch.Tensor, b: torch.Tensor, y_pre: torch.Tensor, state: torch.Tensor, slot_ids, *, tiles=None,
             seq_lens=None, pieces: Optional[bool] = None) -> torch.Tensor:
    """S <- a_t S + b_t per channel over every sequence's tokens (a, b [T, W] float32; S from the sequence's state row,
    zeros at position 0, left there afterwards), the result times gelu_tanh(y_pre) (y_pre [T, W] in the activations'
    type, which is the result's).  pieces (prompt form): as gla_scan's, with pieces of LRU_PIECE tokens; None: for steps of
    at least GLA_PIECES_MIN_ROWS rows."""
    require_gpu()
    _dev(a, "a", torch.float32, 2)
    _dev(b, "b", torch.float32, 2)
    _dev(y_pre, "y_pre", dims=2)
    T, W = a.shape
    if tuple(b.shape) != (T, W) or tuple(y_pre.shape) != (T, W) or not (a.is_contiguous() and b.is_contiguous()):
        raise KernelError(f"lru_scan: a {tuple(a.shape)}, b {tuple(b.shape)}, y_pre {tuple(y_pre.shape)} do not fit")
    stride = _state_rows(state, W, "lru_scan")
    _dev(slot_ids, "slot_ids", torch.int32, 1)
    tl, n_seqs, sl = _seq_args(tiles, seq_lens, "lru_scan")
    out = torch.empty((T, W), dtype=y_pre.dtype, device=a.device)
    if pieces is None:
        pieces = tl is not None and T >= GLA_PIECES_MIN_ROWS
    if pieces and tl is not None and T and n_seqs:
        max_pieces = -(-T // LRU_PIECE)
        carry = torch.empty((n_seqs * max_pieces, 2, W), dtype=torch.float32, device=a.device)
        _check(_fn("conv_scans", "bn_lru_scan_pieces")(_code(y_pre.dtype), a.data_ptr(), b.data_ptr(), y_pre.data_ptr(),
                                                       _rows(y_pre, "y_pre"), out.data_ptr(), state.data_ptr(), stride, tl, n_seqs,
                                                       slot_ids.data_ptr(), W, LRU_PIECE, max_pieces, carry.data_ptr(), _stream()),
               "lru_scan(pieces)")
        return out
    if T and n_seqs:
        _check(_fn("conv_scans", "bn_lru_scan")(_code(y_pre.dtype), a.data_ptr(), b.data_ptr(), y_pre.data_ptr(), _rows(y_pre, "y_pre"),
                                                out.data_ptr(), state.data_ptr(), stride, tl, n_seqs, sl, slot_ids.data_ptr(), W,
                                                _stream()), "lru_scan")
    return out


def gla_supported(dk: int, dv: int) -> bool:
    return bool(_fn("conv_scans", "bn_gla_supports")(int(dk), int(dv)))


GLA_PIECE = 64                  # tokens of a piece of a long prompt
LRU_PIECE = 64                  # the same for the recurrent unit's chain
GLA_PIECES_MIN_ROWS = 256       # prompt steps of at least this many rows walk their sequences in pieces side by side


def gla_scan(x: torch.Tensor, q_col: int, k_col: int, v_col: int, z: torch.Tensor, state: torch.Tensor, slot_ids, H: int,
             dk: int, dv: int, q_scale: float, inv_tau: float, *, tiles=None, seq_lens=None, pieces: Optional[bool] = None) -> torch.Tensor:
    """Gated linear attention over every sequence's tokens: per head S <- diag(alpha_t) S + k_t v_t^T, o_t = S^T (q_scale q_t)
    with alpha = sigmoid(z)^inv_tau per key channel.  x [T, ld] holds q at q_col, k at k_col (heads of dk) and v at v_col
    (heads of dv); z [T, H dk] float32.  state: float32 [slots, >= H dk dv], a head's matrix [dk, dv] row-major; zeros at
    position 0.  Returns o [T, H dv] float32.
    pieces (prompt form): cut every sequence into pieces of GLA_PIECE tokens that are walked side by side: every piece's
    own sum from nothing, the sequence's state carried through the pieces' sums and the products of their decays, then
    every piece's outputs from what it starts with.  Twice the arithmetic on many times the workgroups; the results differ
    from the plain walk's by rounding alone.  None: for steps of at least GLA_PIECES_MIN_ROWS rows."""
    require_gpu()
    _dev(x, "x", dims=2)
    _dev(z, "z", torch.float32, 2)
    T = x.shape[0]
    if (not gla_supported(dk, dv) or x.shape[1] < max(q_col + H * dk, k_col + H * dk, v_col + H * dv) or min(q_col, k_col, v_col) < 0
            or tuple(z.shape) != (T, H * dk) or not z.is_contiguous()):
        raise KernelError(f"gla_scan: x {tuple(x.shape)} / z {tuple(z.shape)} do not fit H={H} dk={dk} dv={dv} (dk at most {GLA_MAX_DIM})")
    stride = _state_rows(state, H * dk * dv, "gla_scan")
    _dev(slot_ids, "slot_ids", torch.int32, 1)
    tl, n_seqs, sl = _seq_args(tiles, seq_lens, "gla_scan")
    o = torch.empty((T, H * dv), dtype=torch.float32, device=x.device)
    if pieces is None:                                   # long steps, as long as the pieces' matrices stay below 2 GB
        pieces = (tl is not None and T >= GLA_PIECES_MIN_ROWS
                  and n_seqs * -(-T // GLA_PIECE) * H * dk * dv * 4 <= 2 << 30)
    if pieces and tl is not None and T and n_seqs:
        max_pieces = -(-T // GLA_PIECE)                  # no sequence of the step has more rows than the step
        carry = torch.empty((n_seqs * max_pieces, H * dk * dv), dtype=torch.float32, device=x.device)
        fade = torch.empty((n_seqs * max_pieces, H * dk), dtype=torch.float32, device=x.device)
        _check(_fn("conv_scans", "bn_gla_scan_pieces")(_code(x.dtype), x.data_ptr(), _rows(x, "x"), int(q_col), int(k_col), int(v_col),
                                                       z.data_ptr(), o.data_ptr(), state.data_ptr(), stride, tl, n_seqs,
                                                       slot_ids.data_ptr(), H, dk, dv, float(q_scale), float(inv_tau), GLA_PIECE,
                                                       max_pieces, carry.data_ptr(), fade.data_ptr(), _stream()), "gla_scan(pieces)")
        return o
    if T and n_seqs:
        _check(_fn("conv_scans", "bn_gla_scan")(_code(x.dtype), x.data_ptr(), _rows(x, "x"), int(q_col), int(k_col), int(v_col),
                                                z.data_ptr(), o.data_ptr(), state.data_ptr(), stride, tl, n_seqs, sl,
                                                slot_ids.data_ptr(), H, dk, dv, float(q_scale), float(inv_tau), _stream()), "gla_scan")
    return o


MOE_MAX_EXPERTS = _build.header_constant("MOE_MAX_EXPERTS", "moe.hip")
MOE_SCORINGS = {"sigmoid": _build.header_constant("MOE_SCORE_SIGMOID", "moe.hip"),
                "softmax": _build.header_constant("MOE_SCORE_SOFTMAX", "moe.hip")}


def moe_route(h: torch.Tensor, router: torch.Tensor, top_k: int, scoring: str = "sigmoid", renormalize: bool = False, *,
              choice_bias: Optional[torch.Tensor] = None, weight_floor: float = 0.0, weight_scale: float = 1.0,
              gate: Optional[torch.Tensor] = None, logit_bias: Optional[torch.Tensor] = None):
    """(ids [T, top_k] int32, weights [T, top_k] float32): router logits z = router . h (+ logit_bias [E] float32) in
    float32 (router [E, D] float32, h in the activations' type), scores sigmoid(z) or softmax(z) over the experts, the top_k largest in
    descending order (ties: the lower index); renormalize divides the chosen scores by their sum (+ weight_floor);
    weight_scale multiplies the weights.  choice_bias [E] float32: the experts are chosen by score + bias, the weights
    stay the plain scores.  gate [D] float32: a third result [T] float32, sigmoid(gate . h), a shared expert's gate."""
    require_gpu()
    _dev(h, "h", dims=2)
    _dev(router, "router", torch.float32, 2)
    T, D = h.shape
    E = router.shape[0]
    if scoring not in MOE_SCORINGS:
        raise KernelError(f"moe_route: unknown scoring {scoring!r}; known: {sorted(MOE_SCORINGS)}")
    if router.shape[1] != D or not router.is_contiguous() or not 1 <= top_k <= E or E > MOE_MAX_EXPERTS or D > 16384:
        raise KernelError(f"moe_route: h {tuple(h.shape)}, router {tuple(router.shape)}, top_k {top_k} do not fit "
                          f"(at most {MOE_MAX_EXPERTS} experts, 16,384 columns)")
    for t, nm, n in ((choice_bias, "choice_bias", E), (gate, "gate", D), (logit_bias, "logit_bias", E)):
        if t is not None:
            _dev(t, nm, torch.float32, 1)
            if t.numel() != n or not t.is_contiguous():
                raise KernelError(f"moe_route: {nm} must hold {n} float32 values")
    if not weight_floor >= 0.0:
        raise KernelError(f"moe_route: weight_floor {weight_floor} must not be negative")
    ids = torch.empty((T, top_k), dtype=torch.int32, device=h.device)
    wts = torch.empty((T, top_k), dtype=torch.float32, device=h.device)
    gate_out = torch.empty((T,), dtype=torch.float32, device=h.device) if gate is not None else None
    if T:
        _check(_fn("moe", "bn_moe_route")(_code(h.dtype), h.data_ptr(), _rows(h, "h"), router.data_ptr(), ids.data_ptr(),
                                          wts.data_ptr(), T, D, E, int(top_k), MOE_SCORINGS[scoring], int(bool(renormalize)),
                                          choice_bias.data_ptr() if choice_bias is not None else None, float(weight_floor),
                                          float(weight_scale), gate.data_ptr() if gate is not None else None,
                                          gate_out.data_ptr() if gate is not None else None,
                                          logit_bias.data_ptr() if logit_bias is not None else None, _stream()), "moe_route")
    return (ids, wts) if gate is None else (ids, wts, gate_out)


@dataclass(frozen=True)
class ClampedUnit:
    """The gated unit glu(g, u) = g' sigmoid(slope g') (u' + shift) with g' = min(g, limit), u' = clamp(u, -limit, limit)."""
    limit: float
    slope: float = 1.702
    shift: float = 1.0

    def __post_init__(self):
        if not self.limit > 0:
            raise KernelError(f"a clamped unit's limit must be positive, got {self.limit}")


def _expert_shapes(h, w_up, w_down, ids, wts, gated, what: str):
    T, D = h.shape
    E, F = w_down.shape[0], w_down.shape[2]
    K = ids.shape[1]
    up_rows = 2 * F if gated else F
    if (tuple(w_up.shape) != (E, up_rows, D) or tuple(w_down.shape) != (E, D, F) or tuple(ids.shape) != (T, K) or tuple(wts.shape) != (T, K)
            or not (w_up.is_contiguous() and w_down.is_contiguous() and ids.is_contiguous() and wts.is_contiguous())):
        raise KernelError(f"{what}: h {tuple(h.shape)}, w_up {tuple(w_up.shape)}, w_down {tuple(w_down.shape)}, ids "
                          f"{tuple(ids.shape)} do not fit ({'gate and up rows stacked' if gated else 'experts without a gate'})")
    return T, D, E, F, K


def gated_unit(gu: torch.Tensor, unit: ClampedUnit, row_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
    """gu [T, 2 F] (gate columns, then up columns) -> [T, F] in gu's type: the clamped unit of every pair, times
    row_scale[t] (float32) when given, rounded once."""
    require_gpu()
    _dev(gu, "gu", dims=2)
    T, F2 = gu.shape
    if F2 % 2 or gu.dtype not in _DT:
        raise KernelError(f"gated_unit: gate and up columns side by side, got {tuple(gu.shape)} {gu.dtype}")
    if row_scale is not None:
        _dev(row_scale, "row_scale", torch.float32, 1)
        if row_scale.numel() != T or not row_scale.is_contiguous():
            raise KernelError("gated_unit: one factor per row")
    out = torch.empty((T, F2 // 2), dtype=gu.dtype, device=gu.device)
    if T:
        _check(_fn("moe", "bn_gated_unit")(_code(gu.dtype), out.data_ptr(), gu.data_ptr(), _rows(gu, "gu"),
                                           row_scale.data_ptr() if row_scale is not None else None, T, F2 // 2,
                                           float(unit.limit), float(unit.slope), float(unit.shift), _stream()), "gated_unit")
    return out


def moe_experts(h: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor, ids: torch.Tensor, wts: torch.Tensor,
                activation: str = "relu2", weight_on_input: bool = True, *, gated: Optional[ClampedUnit] = None,
                extra_slabs: int = 0) -> PartialSums:
    """The chosen experts' outputs, expert e being w_down[e] act(w_up[e] x) (w_up [E, F, D], w_down [E, D, F], act one of
    UNARY_ACTIVATIONS), or, with `gated`, w_down[e] unit(gate rows . x, up rows . x) (w_up [E, 2 F, D]: F gate rows, then F
    up rows): slab j of the result [top_k, T, D] (float32) holds every token's j-th choice, computed on w h
    (weight_on_input) or scaled by w afterwards.  The feed-forward's output is the sum of the slabs.  extra_slabs: that
    many more slabs behind the experts', left for the caller to fill."""
    require_gpu()
    _dev(h, "h", dims=2)
    _dev(w_up, "w_up", h.dtype, 3)
    _dev(w_down, "w_down", h.dtype, 3)
    _dev(ids, "ids", torch.int32, 2)
    _dev(wts, "wts", torch.float32, 2)
    T, D, E, F, K = _expert_shapes(h, w_up, w_down, ids, wts, gated is not None, "moe_experts")
    if gated is None and activation not in UNARY_ACTIVATIONS:
        raise KernelError(f"unknown activation {activation!r}; known: {sorted(UNARY_ACTIVATIONS)}")
    if max(D, F) > 16384 or K > 65535:
        raise KernelError(f"moe_experts: width {D} / expert width {F} above 16,384 values")
    y = torch.empty((K + int(extra_slabs), T, D), dtype=torch.float32, device=h.device)
    unit = gated or ClampedUnit(1.0)
    run = 65535 // K                                      # tokens of one launch: a pair a row of the grid
    ld = _rows(h, "h")
    for t0 in range(0, T, run):
        n = min(run, T - t0)
        hidden = torch.empty((n * K, F), dtype=torch.float32, device=h.device)
        _check(_fn("moe", "bn_moe_experts")(_code(h.dtype), h.data_ptr() + t0 * ld * h.element_size(), ld, w_up.data_ptr(),
                                            w_down.data_ptr(), ids.data_ptr() + t0 * K * 4, wts.data_ptr() + t0 * K * 4,
                                            y.data_ptr() + t0 * D * 4, hidden.data_ptr(), n, T, D, F, K,
                                            0 if gated is not None else UNARY_ACTIVATIONS[activation], int(bool(weight_on_input)),
                                            int(gated is not None), float(unit.limit), float(unit.slope), float(unit.shift),
                                            _stream()), "moe_experts")
    return PartialSums(y)


MOE_GROUPED_MIN_ROWS = 17           # rows from which a bf16 step's experts run as grouped products (below: a pair at a time)
MOE_TILE_ROWS = _build.header_constant("GM_BM", "gemm_mfma.hip")     # rows of a tile of the grouped products


def moe_grouped_supported(T: int, D: int, F: int, dtype) -> bool:
    """Whether moe_experts_grouped takes a step of T rows of these sizes and is the faster of the two: bf16, rows of whole
    16-byte groups, and enough rows for experts to be shared."""
    return dtype == torch.bfloat16 and T >= MOE_GROUPED_MIN_ROWS and D % 8 == 0 and F % 8 == 0


def moe_experts_grouped(h: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor, ids: torch.Tensor, wts: torch.Tensor,
                        activation: str = "relu2", weight_on_input: bool = True, *, gated: Optional[ClampedUnit] = None,
                        extra_slabs: int = 0) -> PartialSums:
    """What moe_experts computes, for bf16 steps of many rows: the (token, choice) pairs are ordered by expert on the
    device and cut into tiles of up to MOE_TILE_ROWS rows of one expert, the inputs are gathered in that order (scaled
    and rounded there when the weight multiplies the input), and both products run as grouped matrix products on the matrix
    cores (the tiled kernel of gemm_mfma with a list of tiles).  Nothing comes back to the host; the launches' sizes depend
    on the step's shape alone.  gated, extra_slabs: as moe_experts's; the gate and up rows of an expert run as one grouped
    product and the unit follows in a kernel of its own."""
    require_gpu()
    _dev(h, "h", torch.bfloat16, 2)
    _dev(w_up, "w_up", torch.bfloat16, 3)
    _dev(w_down, "w_down", torch.bfloat16, 3)
    _dev(ids, "ids", torch.int32, 2)
    _dev(wts, "wts", torch.float32, 2)
    T, D, E, F, K = _expert_shapes(h, w_up, w_down, ids, wts, gated is not None, "moe_experts_grouped")
    if gated is None and activation not in UNARY_ACTIVATIONS:
        raise KernelError(f"unknown activation {activation!r}; known: {sorted(UNARY_ACTIVATIONS)}")
    ld = _rows(h, "h")
    if D % 8 or F % 8 or E > MOE_MAX_EXPERTS or ld % 8 or (h.data_ptr() | w_up.data_ptr() | w_down.data_ptr()) % 16:
        raise KernelError(f"moe_experts_grouped: widths {D} and {F} must be multiples of 8, rows 16-byte aligned, at most "
                          f"{MOE_MAX_EXPERTS} experts")
    y = torch.empty((K + int(extra_slabs), T, D), dtype=torch.float32, device=h.device)
    if T == 0:
        return PartialSums(y)
    n = T * K
    max_tiles = -(-n // MOE_TILE_ROWS) + E
    work = torch.empty((2 * n + 3 * max_tiles + 1,), dtype=torch.int32, device=h.device)
    row_scale = torch.empty((n,), dtype=torch.float32, device=h.device)
    xg = torch.empty((n, D), dtype=torch.bfloat16, device=h.device)
    hidden = torch.empty((n, 2 * F if gated is not None else F), dtype=torch.bfloat16, device=h.device)
    _check(_fn("moe", "bn_moe_group")(h.data_ptr(), ld, ids.data_ptr(), wts.data_ptr(), work.data_ptr(), row_scale.data_ptr(),
                                      xg.data_ptr(), T, D, E, K, MOE_TILE_ROWS, int(bool(weight_on_input)), _stream()),
           "moe_group")
    row_map, tiles = work.data_ptr() + 4 * n, work.data_ptr() + 8 * n
    n_tiles = tiles + 12 * max_tiles
    grouped = _fn("gemm_mfma", "bn_gemm_mfma_grouped")
    if gated is not None:
        _check(grouped(_code(torch.bfloat16), xg.data_ptr(), w_up.data_ptr(), hidden.data_ptr(), tiles, n_tiles, max_tiles, None, None,
                       2 * F * D, -1, n, 2 * F, D, D, D, 2 * F, _stream()), "moe_experts_grouped(gate and up)")
        hidden = gated_unit(hidden, gated)
    else:
        _check(grouped(_code(torch.bfloat16), xg.data_ptr(), w_up.data_ptr(), hidden.data_ptr(), tiles, n_tiles, max_tiles, None, None,
                       F * D, UNARY_ACTIVATIONS[activation], n, F, D, D, D, F, _stream()), "moe_experts_grouped(up)")
    _check(grouped(_code(torch.float32), hidden.data_ptr(), w_down.data_ptr(), y.data_ptr(), tiles, n_tiles, max_tiles, row_map,
                   None if weight_on_input else row_scale.data_ptr(), D * F, -1, n, D, F, F, F, D, _stream()),
           "moe_experts_grouped(down)")
    return PartialSums(y)


# --------------------------------------------------------------------------------------
# sampling
# --------------------------------------------------------------------------------------

def _logits_ok(logits):
    _dev(logits, "logits", torch.float32, 2)
    return _rows(logits, "logits")


def argmax(logits: torch.Tensor) -> torch.Tensor:
    require_gpu()
    ld = _logits_ok(logits)
    B, V = logits.shape
    out = torch.empty((B,), dtype=torch.int32, device=logits.device)
    if B:
        wv = wi = None
        if B <= 256 and V >= 16384:          # few rows of a large vocabulary: two stages
            wv = torch.empty((B, 64), dtype=torch.float32, device=logits.device)
            wi = torch.empty((B, 64), dtype=torch.int32, device=logits.device)
        _check(_fn("sampling", "bn_argmax")(logits.data_ptr(), ld, B, V, out.data_ptr(),
                                            wv.data_ptr() if wv is not None else None,
                                            wi.data_ptr() if wi is not None else None, _stream()), "argmax")
    return out


def repeat_penalty_(logits: torch.Tensor, recent: torch.Tensor, penalty: float) -> None:
    """In place: every distinct token id of a row of `recent` (int32, -1 = none) is penalised once."""
    require_gpu()
    ld = _logits_ok(logits)
    _dev(recent, "recent", torch.int32, 2)
    if recent.shape[0] != logits.shape[0] or not recent.is_contiguous():
        raise KernelError("repeat_penalty: one contiguous row of recent tokens per row of logits")
    if logits.shape[0] and recent.shape[1]:
        _check(_fn("sampling", "bn_repeat_penalty")(logits.data_ptr(), ld, logits.shape[0], logits.shape[1],
                                                    recent.data_ptr(), recent.shape[1], float(penalty),
                                                    _stream()), "repeat_penalty")


WIDE_SAMPLE_VOCAB = 16384                 # from this many logits a row on, sampling spreads a row over 32 workgroups
_WIDE_ROW_WORDS = 2 * 4 * 256 + 3 * 32    # WIDE_ROW_WORDS of csrc/sampling.hip


def sample(logits: torch.Tensor, temperature: float, top_p: float, uniforms=None, *,
           force_one_workgroup: bool = False) -> torch.Tensor:
    """One token id per row.  temperature 0: argmax.  uniforms: float32 [B] in [0, 1)."""
    require_gpu()
    if temperature == 0.0:
        return argmax(logits)                 # the same first maximum, in two stages for a large vocabulary
    ld = _logits_ok(logits)
    B, V = logits.shape
    out = torch.empty((B,), dtype=torch.int32, device=logits.device)
    if B == 0:
        return out
    _dev(uniforms, "uniforms", torch.float32, 1)
    if uniforms.numel() != B or not uniforms.is_contiguous():
        raise KernelError("sample: one uniform number per row")
    if V >= WIDE_SAMPLE_VOCAB and B <= 65535 and not force_one_workgroup:
        # a large vocabulary: every pass over a row is spread over 32 workgroups
        ws = torch.zeros((B, _WIDE_ROW_WORDS), dtype=torch.int64, device=logits.device)
        _check(_fn("sampling", "bn_sample_wide")(logits.data_ptr(), ld, B, V, ws.data_ptr(), uniforms.data_ptr(),
                                                 float(temperature), float(top_p), out.data_ptr(), _stream()),
               "sample(wide)")
        return out
    probs = torch.empty((B, V), dtype=torch.float32, device=logits.device)
    _check(_fn("sampling", "bn_sample")(logits.data_ptr(), ld, B, V, probs.data_ptr(), uniforms.data_ptr(),
                                        float(temperature), float(top_p), out.data_ptr(), _stream()), "sample")
    return out
