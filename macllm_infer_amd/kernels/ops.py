"""The operations the parts are made of, each a hand-written HIP kernel for gfx950
(matrix products of the bfloat16 path go to the BLAS library, as the reference's do:
src/model_weights.rs:307-415 hands them to its tensor library).

Every wrapper checks operand shapes, dtypes and devices on the host before the launch,
and raises ``KernelError`` when a kernel refuses a size.  There is no other code path:
without a GPU and the built modules these functions fail.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import Optional, Sequence

import torch

from . import build

_c_int = ctypes.c_int
_c_long = ctypes.c_long
_c_float = ctypes.c_float
_c_ptr = ctypes.c_void_p

DT_F32, DT_BF16 = 0, 1


class KernelError(RuntimeError):
    pass


_SIGNATURES = {
    "common": {
        "mi_embed": [_c_ptr, _c_ptr, _c_int, _c_float, _c_ptr, _c_int, _c_int, _c_ptr],
        "mi_feed_tokens": [_c_ptr, _c_int, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, _c_ptr],
        "mi_add_rmsnorm": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_float, _c_ptr, _c_int, _c_ptr, _c_int,
                           _c_int, _c_ptr],
        "mi_add_partials_rmsnorm": [_c_ptr, _c_ptr, _c_int, _c_ptr, _c_float, _c_ptr, _c_int, _c_ptr, _c_int, _c_int,
                                    _c_int, _c_ptr],
        "mi_swiglu": [_c_ptr, _c_int, _c_long, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
        "mi_scale_to_f32": [_c_ptr, _c_int, _c_float, _c_ptr, _c_long, _c_ptr],
        "mi_tanh_softcap": [_c_ptr, _c_float, _c_long, _c_ptr],
        "mi_add_bias_round": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr],
    },
    "attention": {
        "mi_rope_kv_store": [_c_ptr, _c_int, _c_long, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_int,
                             _c_ptr, _c_ptr, _c_ptr, _c_long, _c_int, _c_ptr],
        "mi_paged_attention": [_c_ptr, _c_int, _c_long, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_long,
                               _c_int, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_float, _c_int, _c_ptr, _c_int, _c_ptr, _c_long,
                               _c_ptr, _c_long, _c_ptr, _c_int, _c_int, _c_ptr, _c_ptr],
        "mi_paged_attention_workspace": [_c_int, _c_int, _c_int, _c_int],
        "mi_prefill_attention": [_c_ptr, _c_long, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_long, _c_int, _c_ptr,
                                 _c_int, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_float, _c_int, _c_int, _c_ptr, _c_long,
                                 _c_ptr],
        "mi_decode_attention": [_c_ptr, _c_long, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_long, _c_int,
                                _c_ptr, _c_int, _c_ptr, _c_ptr, _c_float, _c_int, _c_int, _c_int, _c_ptr, _c_ptr,
                                _c_ptr, _c_long, _c_ptr],
    },
    "mamba2": {
        "mi_conv1d_silu": [_c_ptr, _c_int, _c_long, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr,
                           _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr],
        "mi_conv_state_update": [_c_ptr, _c_int, _c_long, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int,
                                 _c_ptr],
        "mi_conv_step": [_c_ptr, _c_int, _c_long, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr],
        "mi_ssm_scan": [_c_ptr, _c_int, _c_long, _c_ptr, _c_long, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                        _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_long, _c_ptr, _c_long, _c_ptr],
        "mi_gate_norm": [_c_ptr, _c_long, _c_ptr, _c_int, _c_long, _c_ptr, _c_int, _c_float, _c_ptr, _c_long,
                         _c_int, _c_int, _c_ptr],
    },
    "ssd": {
        "mi_ssd_supported": [_c_int, _c_int, _c_int, _c_int, _c_int],
        "mi_ssd_prefill": [_c_ptr, _c_long, _c_ptr, _c_long, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr,
                           _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr,
                           _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_long, _c_ptr, _c_long, _c_ptr, _c_long,
                           _c_ptr, _c_long, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr],
    },
    "gemm": {
        "mi_gemm_f32": [_c_ptr, _c_long, _c_ptr, _c_long, _c_ptr, _c_ptr, _c_long, _c_int, _c_int, _c_int, _c_ptr],
    },
    "decode": {
        "mi_fused_gemm": [_c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_float, _c_ptr, _c_long, _c_ptr,
                          _c_ptr, _c_int, _c_int, _c_int, _c_ptr, _c_long, _c_int, _c_float, _c_int, _c_int, _c_int,
                          _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr, _c_int, _c_int, _c_float, _c_int,
                          _c_ptr],
        "mi_fused_gemm_residual": [_c_ptr, _c_long, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_long,
                                   _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr],
        "mi_fused_gemm_supported": [_c_int, _c_int, _c_int],
        "mi_fused_gemm_split": [_c_ptr, _c_long, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr, _c_int, _c_int, _c_int,
                                _c_ptr],
        "mi_shared_rows_gemm_split": [_c_ptr, _c_long, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr, _c_int, _c_int,
                                      _c_int, _c_ptr],
        "mi_mixer_split_keys": [_c_int, _c_int, _c_int, _c_long],
        "mi_mixer_runs": [_c_int, _c_int, _c_int, _c_long, _c_ptr, _c_ptr],
        "mi_fused_gemm_merge": [_c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_long, _c_ptr,
                                _c_ptr, _c_int, _c_int, _c_int, _c_ptr, _c_long, _c_int, _c_ptr, _c_ptr, _c_long, _c_ptr,
                                _c_ptr, _c_ptr],
        "mi_mixer_decode": [_c_ptr, _c_long, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_int,
                            _c_ptr, _c_ptr, _c_long, _c_int, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_float, _c_int,
                            _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                            _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_long, _c_ptr, _c_long,
                            _c_int, _c_ptr],
    },
    "microbench": {
        "mi_stream_read": [_c_ptr, _c_long, _c_ptr, _c_int, _c_ptr],
        "mi_stream_rmw": [_c_ptr, _c_long, _c_float, _c_int, _c_ptr],
    },
    "sampling": {
        "mi_apply_penalties": [_c_ptr, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                               _c_ptr, _c_ptr, _c_ptr, _c_ptr],
        "mi_argmax": [_c_ptr, _c_int, _c_int, _c_ptr, _c_ptr],
        "mi_keep_allowed": [_c_ptr, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_long, _c_ptr],
        "mi_sample": [_c_ptr, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                      _c_ptr, _c_ptr],
    },
}

_functions = {}


def _fn(module: str, name: str, restype=_c_int):
    key = (module, name)
    if key not in _functions:
        library = build.load_module(module)
        function = getattr(library, name)
        function.argtypes = _SIGNATURES[module][name]
        function.restype = restype
        _functions[key] = function
    return _functions[key]


def require_gpu(device) -> torch.device:
    device = torch.device(device)
    if device.type != "cuda" or not torch.cuda.is_available():
        raise KernelError("the HIP kernels need a GPU (device 'cuda:N'); there is no CPU path")
    return device


def _dt(tensor: torch.Tensor) -> int:
    if tensor.dtype == torch.float32:
        return DT_F32
    if tensor.dtype == torch.bfloat16:
        return DT_BF16
    raise KernelError(f"unsupported dtype {tensor.dtype}; kernels take float32 or bfloat16")


def _p(tensor: Optional[torch.Tensor]):
    return None if tensor is None else tensor.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)      # the handle without a Stream object around it


def _stream():
    """The current HIP stream of the current device, as the integer the launchers take."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _check(code: int, name: str, detail: str = "") -> None:
    if code == 0:
        return
    if code == -1:
        raise KernelError(f"{name}: bad argument {detail}")
    if code == -2:
        raise KernelError(f"{name}: size not supported by this kernel {detail}")
    raise KernelError(f"{name}: HIP launch failed with error {code} {detail}")


def _need(condition: bool, message: str) -> None:
    if not condition:
        raise KernelError(message)


def _i32(tensor: torch.Tensor, name: str) -> None:
    _need(tensor.dtype == torch.int32 and tensor.is_contiguous() and tensor.is_cuda,
          f"{name} must be a contiguous int32 GPU tensor")


def _row_major(tensor: torch.Tensor, name: str) -> int:
    """A 2-D tensor whose rows are contiguous; returns the row stride in elements."""
    _need(tensor.dim() == 2 and tensor.stride(1) == 1 and tensor.is_cuda,
          f"{name} must be a 2-D GPU tensor with contiguous rows")
    return tensor.stride(0) if tensor.shape[0] > 1 else max(tensor.stride(0), tensor.shape[1])


# --------------------------------------------------------------------------- common
def embed(token_ids: torch.Tensor, table: torch.Tensor, multiplier: float, out: torch.Tensor) -> None:
    """out[t] = table[token_ids[t]] * multiplier, out float32 [T, d]."""
    _i32(token_ids, "token_ids")
    T, d = out.shape
    _need(token_ids.numel() == T and table.dim() == 2 and table.shape[1] == d and table.is_contiguous(),
          "embed: shapes do not match")
    _need(out.dtype == torch.float32 and out.is_contiguous(), "embed: out must be contiguous float32")
    _check(_fn("common", "mi_embed")(_p(token_ids), _p(table), _dt(table), float(multiplier), _p(out), T, d,
                                     _stream()), "embed")


def feed_tokens(token_ids: torch.Tensor, source: torch.Tensor, dst: Sequence[int], src: Sequence[int]) -> None:
    """token_ids[dst[i]] = source[src[i]] on the device (both int32): tokens that a sampler left on the
    device go into a step's token ids without passing through the host."""
    _i32(token_ids, "token_ids")
    _i32(source, "source")
    count = len(dst)
    _need(len(src) == count, "feed_tokens: as many sources as places")
    if count == 0:
        return
    places = (ctypes.c_int * count)(*[int(value) for value in dst])
    sources = (ctypes.c_int * count)(*[int(value) for value in src])
    _check(_fn("common", "mi_feed_tokens")(_p(token_ids), token_ids.numel(), _p(source), source.numel(),
                                           ctypes.addressof(places), ctypes.addressof(sources), count, _stream()),
           "feed_tokens")


def add_rmsnorm(h: torch.Tensor, deltas: Sequence[torch.Tensor], weight: torch.Tensor, eps: float,
                out: Optional[torch.Tensor], rows: Optional[torch.Tensor] = None) -> None:
    """h += sum(deltas) (float32, in place); out = h / sqrt(mean(h^2) + eps) * weight.

    With ``rows`` (int32 indices) only those rows are read, ``out[i]`` gets row ``rows[i]``
    and ``h`` is left as it is.  ``out`` may be None when only the sum is wanted."""
    _need(h.dtype == torch.float32 and h.dim() == 2 and h.is_contiguous() and h.is_cuda,
          "add_rmsnorm: h must be contiguous float32 [T, d]")
    T, d = h.shape
    _need(len(deltas) <= 2, "add_rmsnorm: at most two deltas")
    for delta in deltas:
        _need(delta.shape == h.shape and delta.is_contiguous() and delta.dtype == deltas[0].dtype,
              "add_rmsnorm: deltas must be contiguous [T, d] of one dtype")
    _need(weight.dtype == torch.float32 and weight.numel() == d and weight.is_contiguous(),
          "add_rmsnorm: weight must be float32 [d]")
    n_rows = T
    if rows is not None:
        _i32(rows, "rows")
        n_rows = rows.numel()
    if out is not None:
        _need(out.shape == (n_rows, d) and out.is_contiguous(), "add_rmsnorm: out must be contiguous [rows, d]")
    delta_dtype = _dt(deltas[0]) if deltas else DT_F32
    out_dtype = _dt(out) if out is not None else DT_F32
    _check(_fn("common", "mi_add_rmsnorm")(
        _p(h), _p(deltas[0]) if len(deltas) > 0 else None, _p(deltas[1]) if len(deltas) > 1 else None,
        delta_dtype, _p(weight), float(eps), _p(out), out_dtype, _p(rows), n_rows, d, _stream()),
        "add_rmsnorm", f"(d={d})")


def add_partials_rmsnorm(h: torch.Tensor, partial: torch.Tensor, weight: torch.Tensor, eps: float,
                         out: Optional[torch.Tensor]) -> None:
    """``add_rmsnorm`` for a branch that arrives as float32 partial sums ``partial`` [S, T, d] (the
    slabs of ``fused_gemm_split``): h += sum of the slabs (in slab order), and, with ``out``,
    out = RMSNorm(h) * weight."""
    T, d = h.shape
    _need(h.dtype == torch.float32 and h.is_contiguous() and h.is_cuda, "add_partials_rmsnorm: h must be contiguous float32")
    _need(partial.dtype == torch.float32 and partial.dim() == 3 and partial.shape[1:] == (T, d)
          and partial.is_contiguous(), "add_partials_rmsnorm: partial must be contiguous float32 [S, T, d]")
    _need(weight.dtype == torch.float32 and weight.numel() == d and weight.is_contiguous(),
          "add_partials_rmsnorm: weight must be float32 [d]")
    _need(out is None or (out.shape == (T, d) and out.is_contiguous()), "add_partials_rmsnorm: bad out")
    _check(_fn("common", "mi_add_partials_rmsnorm")(
        _p(h), _p(partial), partial.shape[0], _p(weight), float(eps), _p(out), _dt(out) if out is not None else DT_F32,
        None, T, T, d, _stream()), "add_partials_rmsnorm", f"(d={d}, S={partial.shape[0]})")


def swiglu(gate_up: torch.Tensor, out: torch.Tensor, tile: int = 0) -> None:
    """out[t, i] = SiLU(g[t, i]) * u[t, i] with a row of ``gate_up`` holding [g | u] (``tile`` 0) or
    g and u interleaved in tiles of ``tile`` columns: [g[0:tile] | u[0:tile] | g[tile:2 tile] | ...]."""
    ld = _row_major(gate_up, "gate_up")
    T, two_i = gate_up.shape
    _need(two_i % 2 == 0 and out.shape == (T, two_i // 2) and out.is_contiguous() and out.dtype == gate_up.dtype,
          "swiglu: out must be contiguous [T, I] of the input's dtype")
    _need(tile >= 0 and (tile == 0 or (two_i // 2) % tile == 0), "swiglu: the tile must divide the width")
    _check(_fn("common", "mi_swiglu")(_p(gate_up), _dt(gate_up), ld, _p(out), T, two_i // 2, int(tile), _stream()),
           "swiglu")


def scale_to_f32(values: torch.Tensor, multiplier: float, out: torch.Tensor) -> None:
    _need(values.is_contiguous() and out.is_contiguous() and out.dtype == torch.float32
          and out.numel() == values.numel() and values.is_cuda, "scale_to_f32: shapes do not match")
    _check(_fn("common", "mi_scale_to_f32")(_p(values), _dt(values), float(multiplier), _p(out), values.numel(),
                                            _stream()), "scale_to_f32")


def tanh_softcap(logits: torch.Tensor, cap: float) -> None:
    """logits <- cap * tanh(logits / cap), in place (float32)."""
    _need(logits.is_contiguous() and logits.dtype == torch.float32 and logits.is_cuda and cap > 0,
          "tanh_softcap: contiguous float32 logits on the GPU and a positive cap")
    if logits.numel():
        _check(_fn("common", "mi_tanh_softcap")(_p(logits), float(cap), logits.numel(), _stream()), "tanh_softcap")


# --------------------------------------------------------------------------- matrix products
def linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], keep_float32: bool = False) -> torch.Tensor:
    """x [M, K] . weight[N, K]^T (+ bias float32 [N]) -> [M, N] in x's dtype, or, with
    ``keep_float32`` and no bias, in float32 whatever the operands are (the library writes its
    float32 sums without rounding them to bfloat16: the logits).

    float32 operands: the hand-written float32 FMA kernel (true 32-bit).  bfloat16 operands:
    the BLAS library with float32 accumulation.  A float32 weight with bfloat16 activations
    (a tensor that was stored in 32-bit) runs in float32 and the result is rounded once."""
    _need(x.dim() == 2 and weight.dim() == 2 and x.shape[1] == weight.shape[1], "linear: shapes do not match")
    if weight.dtype == torch.float32:
        xf = x if x.dtype == torch.float32 else x.float()
        ldx = _row_major(xf, "x")
        ldw = _row_major(weight, "weight")
        M, K = xf.shape
        N = weight.shape[0]
        out = torch.empty((M, N), dtype=torch.float32, device=x.device)
        if bias is not None:
            _need(bias.dtype == torch.float32 and bias.numel() == N, "linear: bias must be float32 [N]")
        _check(_fn("gemm", "mi_gemm_f32")(_p(xf), ldx, _p(weight), ldw, _p(bias), _p(out), N, M, N, K, _stream()),
               "gemm_f32", f"(M={M}, N={N}, K={K})")
        return out if x.dtype == torch.float32 or keep_float32 else out.to(x.dtype)
    _need(x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16, "linear: operands must share a dtype")
    if keep_float32:
        _need(bias is None, "linear: float32 results of bfloat16 operands come without a bias")
        return torch.mm(x, weight.t(), out_dtype=torch.float32)
    if bias is None:
        return torch.mm(x, weight.t())
    # the bias stays float32: it is added to the product's float32 sums, and the result is rounded once
    _need(bias.dtype == torch.float32 and bias.numel() == weight.shape[0] and bias.is_contiguous(),
          "linear: bias must be float32 [N]")
    sums = torch.mm(x, weight.t(), out_dtype=torch.float32)
    out = torch.empty(sums.shape, dtype=torch.bfloat16, device=x.device)
    _check(_fn("common", "mi_add_bias_round")(_p(sums), _p(bias), _p(out), sums.shape[0], sums.shape[1], _stream()),
           "add_bias_round")
    return out


# --------------------------------------------------------------------------- attention
def rope_kv_store(qkv: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int,
                  positions: torch.Tensor, inv_freq: Optional[torch.Tensor], rotary_dim: int,
                  slot_mapping: Optional[torch.Tensor], k_cache: Optional[torch.Tensor],
                  v_cache: Optional[torch.Tensor]) -> None:
    """Rotate q (in place) and k of every token; store rotated k and raw v into the cache.

    ``qkv`` [T, >= (Hq+2Hkv)*dh] holds q heads, k heads, v heads.  ``k_cache`` [pages, Hkv,
    page_size, dh] and ``v_cache`` [pages, Hkv, dh, page_size] are one layer's views of the pool;
    ``slot_mapping[t] = page*page_size + offset``.  Without ``slot_mapping`` nothing is stored."""
    ld = _row_major(qkv, "qkv")
    T = qkv.shape[0]
    _need(qkv.shape[1] >= (num_heads + 2 * num_kv_heads) * head_dim, "rope_kv_store: qkv is too narrow")
    _i32(positions, "positions")
    _need(positions.numel() == T, "rope_kv_store: one position per token")
    if inv_freq is not None:
        _need(inv_freq.dtype == torch.float32 and inv_freq.numel() == rotary_dim // 2 and inv_freq.is_cuda,
              "rope_kv_store: inv_freq must be float32 [rotary_dim/2]")
    page_stride, page_size = 0, 0
    if slot_mapping is not None:
        _i32(slot_mapping, "slot_mapping")
        _need(slot_mapping.numel() == T, "rope_kv_store: one cache cell per token")
        page_stride, page_size = _cache_view(k_cache, v_cache, num_kv_heads, head_dim, qkv.dtype)
    _check(_fn("attention", "mi_rope_kv_store")(
        _p(qkv), _dt(qkv), ld, T, num_heads, num_kv_heads, head_dim, _p(positions), _p(inv_freq),
        rotary_dim if inv_freq is not None else 0, _p(slot_mapping),
        _p(k_cache) if slot_mapping is not None else None, _p(v_cache) if slot_mapping is not None else None,
        page_stride, page_size, _stream()), "rope_kv_store")


def _cache_view(k_cache, v_cache, num_kv_heads, head_dim, dtype):
    """K pages are [pages, Hkv, page_size, dh]; V pages are transposed, [pages, Hkv, dh, page_size]."""
    _need(k_cache is not None and v_cache is not None and k_cache.dim() == 4 and v_cache.dim() == 4,
          "k_cache must be [pages, Hkv, page_size, dh] and v_cache [pages, Hkv, dh, page_size]")
    page_size = k_cache.shape[2]
    _need(k_cache.shape[1] == num_kv_heads and k_cache.shape[3] == head_dim
          and v_cache.shape == (k_cache.shape[0], num_kv_heads, head_dim, page_size),
          "k_cache must be [pages, Hkv, page_size, dh] and v_cache [pages, Hkv, dh, page_size]")
    for name, cache in (("k_cache", k_cache), ("v_cache", v_cache)):
        _need(cache.dtype == dtype and cache.is_cuda, f"{name} must be a GPU tensor of the activation dtype")
        _need(cache.stride(3) == 1 and cache.stride(2) == cache.shape[3]
              and cache.stride(1) == page_size * head_dim, f"{name}: a page's block per kv head must be dense")
    _need(k_cache.stride(0) == v_cache.stride(0), "k_cache and v_cache must share a page stride")
    return k_cache.stride(0), page_size


def paged_attention(q: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int,
                    k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                    lane_of_token: torch.Tensor, positions: torch.Tensor, scale: float,
                    window: Optional[int], out: torch.Tensor, max_seq_len: Optional[int] = None,
                    slopes: Optional[torch.Tensor] = None, query_tiles: Optional[torch.Tensor] = None,
                    tile_tokens: int = 0, cu_seqlens: Optional[torch.Tensor] = None) -> None:
    """Causal attention of every token over its request's cached keys (its own included).

    ``q`` [T, >= Hq*dh] (rotated); ``block_tables`` [lanes, max_pages] page ids by logical
    page; a key at position p is visible to a query at position s when p <= s and, with a
    window w, s - p < w.  ``out`` [T, Hq*dh].  ``max_seq_len``: an upper bound of position + 1 over
    the step's tokens (what the block tables can hold if it is not given); it sizes the launch and
    the work area, never the result.  ``slopes`` (float32 [Hq]): a bias on the scores by distance,
    ``score -= slopes[head] * (s - p)``.  ``query_tiles`` [tiles, 2] = (lane or -1, first token row) of runs of
    up to ``tile_tokens`` tokens of one lane, with ``cu_seqlens`` [lanes + 1]: for steps whose lanes hold several
    tokens, a kernel that fetches a run of keys once for sixteen queries (the same bits as without)."""
    q_ld = _row_major(q, "q")
    out_ld = _row_major(out, "out")
    T = q.shape[0]
    _need(q.shape[1] >= num_heads * head_dim and out.shape == (T, num_heads * head_dim)
          and out.dtype == q.dtype, "paged_attention: q/out shapes do not match")
    page_stride, page_size = _cache_view(k_cache, v_cache, num_kv_heads, head_dim, q.dtype)
    _i32(block_tables, "block_tables")
    _i32(lane_of_token, "lane_of_token")
    _i32(positions, "positions")
    _need(block_tables.dim() == 2 and lane_of_token.numel() == T and positions.numel() == T,
          "paged_attention: metadata shapes do not match")
    _need(slopes is None or (slopes.dtype == torch.float32 and slopes.numel() == num_heads and slopes.is_contiguous()
                             and slopes.is_cuda), "paged_attention: slopes must be float32 [Hq] on the GPU")
    holds = block_tables.shape[1] * page_size
    span = holds if max_seq_len is None else max(1, min(int(max_seq_len), holds))
    floats = _fn("attention", "mi_paged_attention_workspace", _c_long)(T, num_heads, head_dim, span)
    partial = torch.empty((max(int(floats), 1),), dtype=torch.float32, device=q.device)
    tiles = 0
    if query_tiles is not None and tile_tokens and tile_tokens % 16 == 0 and cu_seqlens is not None:
        _i32(query_tiles, "query_tiles")
        _i32(cu_seqlens, "cu_seqlens")
        _need(query_tiles.dim() == 2 and query_tiles.shape[1] == 2 and cu_seqlens.numel() == block_tables.shape[0] + 1,
              "paged_attention: the table of runs or the lanes' offsets do not fit the step")
        tiles = query_tiles.shape[0]
    _check(_fn("attention", "mi_paged_attention")(
        _p(q), _dt(q), q_ld, T, num_heads, num_kv_heads, head_dim, _p(k_cache), _p(v_cache), page_stride,
        page_size, _p(block_tables), block_tables.shape[1], _p(lane_of_token), _p(positions), float(scale),
        int(window or 0), _p(slopes), span, _p(partial), partial.numel(), _p(out), out_ld,
        _p(query_tiles) if tiles else None, tiles, int(tile_tokens) if tiles else 0, _p(cu_seqlens) if tiles else None,
        _stream()), "paged_attention", f"(head_dim={head_dim})")


def prefill_attention_supported(dtype, num_heads: int, num_kv_heads: int, head_dim: int, page_size: int) -> bool:
    """Whether the matrix-core attention kernel covers this geometry."""
    return (dtype == torch.bfloat16 and head_dim in (64, 128) and page_size % 4 == 0
            and num_heads // num_kv_heads <= 64)


def prefill_attention(q: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int, k_cache: torch.Tensor,
                      v_cache: torch.Tensor, block_tables: torch.Tensor, query_tiles: torch.Tensor,
                      cu_seqlens: torch.Tensor, start_pos: torch.Tensor, scale: float, window: Optional[int],
                      out: torch.Tensor, max_seq_len: int = 0) -> None:
    """``paged_attention`` on the matrix cores for bfloat16 (flash-style, online softmax in
    float32).  ``query_tiles`` [tiles, 2]: (lane, first token row) of runs of up to 64 tokens of
    one lane; the keys and values of the step's own tokens must be in the cache already.
    ``max_seq_len``: an upper bound of the step's longest context if known (it picks how many heads share
    a key fragment, never the result)."""
    q_ld = _row_major(q, "q")
    out_ld = _row_major(out, "out")
    T = q.shape[0]
    _need(q.dtype == torch.bfloat16 and out.dtype == torch.bfloat16, "prefill_attention: bfloat16 only")
    _need(q.shape[1] >= num_heads * head_dim and out.shape == (T, num_heads * head_dim) and q_ld % 8 == 0
          and q.data_ptr() % 16 == 0 and out_ld % 4 == 0 and out.data_ptr() % 8 == 0,
          "prefill_attention: q/out shapes or alignment do not fit")
    page_stride, page_size = _cache_view(k_cache, v_cache, num_kv_heads, head_dim, q.dtype)
    _need(prefill_attention_supported(q.dtype, num_heads, num_kv_heads, head_dim, page_size),
          "prefill_attention: geometry not covered; use paged_attention")
    for name, tensor in (("block_tables", block_tables), ("query_tiles", query_tiles), ("cu_seqlens", cu_seqlens),
                         ("start_pos", start_pos)):
        _i32(tensor, name)
    _need(block_tables.dim() == 2 and query_tiles.dim() == 2 and query_tiles.shape[1] == 2
          and cu_seqlens.numel() == start_pos.numel() + 1, "prefill_attention: metadata shapes do not match")
    _check(_fn("attention", "mi_prefill_attention")(
        _p(q), q_ld, num_heads, num_kv_heads, head_dim, _p(k_cache), _p(v_cache), page_stride, page_size,
        _p(block_tables), block_tables.shape[1], _p(query_tiles), query_tiles.shape[0], _p(cu_seqlens),
        _p(start_pos), float(scale), int(window or 0), int(max_seq_len or 0), _p(out), out_ld, _stream()),
        "prefill_attention")


def decode_attention_supported(dtype, num_heads: int, num_kv_heads: int, head_dim: int, page_size: int) -> bool:
    """Whether the split-context kernel for single-token queries covers this geometry."""
    return (dtype == torch.bfloat16 and head_dim in (64, 128) and num_heads // num_kv_heads <= 8
            and page_size % 8 == 0 and page_size <= 512)


def decode_attention(q: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int, k_cache: torch.Tensor,
                     v_cache: torch.Tensor, block_tables: torch.Tensor, lane_of_token: torch.Tensor,
                     positions: torch.Tensor, scale: float, window: Optional[int], max_seq_len: int,
                     out: torch.Tensor) -> None:
    """``paged_attention`` for batches of single decoded tokens in bfloat16: the context of each
    request is split over many workgroups and the G query heads of a kv head share its K/V
    loads.  ``max_seq_len``: an upper bound of the longest context in the batch."""
    q_ld = _row_major(q, "q")
    out_ld = _row_major(out, "out")
    T = q.shape[0]
    _need(q.dtype == torch.bfloat16 and out.dtype == torch.bfloat16, "decode_attention: bfloat16 only")
    _need(q.shape[1] >= num_heads * head_dim and out.shape == (T, num_heads * head_dim) and q_ld % 8 == 0
          and q.data_ptr() % 16 == 0, "decode_attention: q/out shapes or alignment do not fit")
    page_stride, page_size = _cache_view(k_cache, v_cache, num_kv_heads, head_dim, q.dtype)
    _need(decode_attention_supported(q.dtype, num_heads, num_kv_heads, head_dim, page_size),
          "decode_attention: geometry not covered; use paged_attention")
    _i32(block_tables, "block_tables")
    _i32(lane_of_token, "lane_of_token")
    _i32(positions, "positions")
    _need(block_tables.dim() == 2 and lane_of_token.numel() == T and positions.numel() == T,
          "decode_attention: metadata shapes do not match")
    span = max_seq_len if not window else min(max_seq_len, window + page_size)
    split_keys = 64
    while split_keys < 512 and span * T * num_kv_heads > 1024 * split_keys:
        split_keys *= 2
    split_keys = max(split_keys, page_size)
    splits = max(1, -(-span // split_keys))
    partial_o = torch.empty((T, num_heads, splits, head_dim), dtype=torch.float32, device=q.device)
    partial_ml = torch.empty((T, num_heads, splits, 2), dtype=torch.float32, device=q.device)
    _check(_fn("attention", "mi_decode_attention")(
        _p(q), q_ld, T, num_heads, num_kv_heads, head_dim, _p(k_cache), _p(v_cache), page_stride, page_size,
        _p(block_tables), block_tables.shape[1], _p(lane_of_token), _p(positions), float(scale), int(window or 0),
        split_keys, splits, _p(partial_o), _p(partial_ml), _p(out), out_ld, _stream()), "decode_attention")


# --------------------------------------------------------------------------- mamba2
def conv1d_silu(u: torch.Tensor, col_offset: int, width: int, weight: torch.Tensor,
                bias: Optional[torch.Tensor], conv_state: torch.Tensor, lane_of_token: torch.Tensor,
                cu_seqlens: torch.Tensor, slot_ids: torch.Tensor, out: torch.Tensor) -> None:
    """out[t] = SiLU(causal depthwise conv of u[:, col_offset:col_offset+width]) per lane,
    the K-1 rows before a lane's first token coming from ``conv_state[slot]`` [K-1, width]."""
    ld = _row_major(u, "u")
    T = u.shape[0]
    K = weight.shape[1]
    _need(weight.shape == (width, K) and weight.dtype == torch.float32 and weight.is_contiguous(),
          "conv1d_silu: weight must be float32 [C, K]")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == width), "conv1d_silu: bad bias")
    _need(conv_state.dim() == 3 and conv_state.shape[1:] == (max(K - 1, 0), width)
          and conv_state.dtype == u.dtype and conv_state.is_contiguous(), "conv1d_silu: bad conv_state")
    _need(out.shape == (T, width) and out.is_contiguous() and out.dtype == u.dtype, "conv1d_silu: bad out")
    _need(u.shape[1] >= col_offset + width, "conv1d_silu: u is too narrow")
    for name, tensor in (("lane_of_token", lane_of_token), ("cu_seqlens", cu_seqlens), ("slot_ids", slot_ids)):
        _i32(tensor, name)
    _check(_fn("mamba2", "mi_conv1d_silu")(
        _p(u), _dt(u), ld, col_offset, T, width, K, _p(weight), _p(bias), _p(conv_state), _p(lane_of_token),
        _p(cu_seqlens), _p(slot_ids), _p(out), _stream()), "conv1d_silu", f"(K={K})")


def conv_state_update(u: torch.Tensor, col_offset: int, width: int, kernel: int, conv_state: torch.Tensor,
                      cu_seqlens: torch.Tensor, slot_ids: torch.Tensor) -> None:
    """conv_state[slot] = last K-1 rows of [conv_state[slot] ; the lane's rows of u]."""
    ld = _row_major(u, "u")
    num_lanes = slot_ids.numel()
    _need(conv_state.dim() == 3 and conv_state.shape[1:] == (max(kernel - 1, 0), width)
          and conv_state.dtype == u.dtype and conv_state.is_contiguous(), "conv_state_update: bad conv_state")
    _need(cu_seqlens.numel() == num_lanes + 1, "conv_state_update: cu_seqlens must have lanes+1 entries")
    _i32(cu_seqlens, "cu_seqlens")
    _i32(slot_ids, "slot_ids")
    _check(_fn("mamba2", "mi_conv_state_update")(
        _p(u), _dt(u), ld, col_offset, width, kernel, _p(conv_state), _p(cu_seqlens), _p(slot_ids), num_lanes,
        _stream()), "conv_state_update", f"(K={kernel})")


def conv_step(u: torch.Tensor, col_offset: int, width: int, weight: torch.Tensor, bias: Optional[torch.Tensor],
              conv_state: torch.Tensor, slot_ids: torch.Tensor) -> None:
    """One conv step of single-token lanes, in place: row m of ``u`` is the new token of the request in
    ``slot_ids[m]``; columns [col_offset, col_offset + width) become SiLU(conv over [tail ; sample]) and the
    tail ``conv_state[slot]`` [K-1, width] is rolled by one and takes the sample."""
    ld = _row_major(u, "u")
    M = u.shape[0]
    K = weight.shape[1]
    _need(weight.shape == (width, K) and weight.dtype == torch.float32 and weight.is_contiguous(),
          "conv_step: weight must be float32 [C, K]")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == width), "conv_step: bad bias")
    _need(conv_state.dim() == 3 and conv_state.shape[1:] == (max(K - 1, 0), width)
          and conv_state.dtype == u.dtype and conv_state.is_contiguous(), "conv_step: bad conv_state")
    _need(u.shape[1] >= col_offset + width, "conv_step: u is too narrow")
    _i32(slot_ids, "slot_ids")
    _need(slot_ids.numel() >= M, "conv_step: one slot per row")
    _check(_fn("mamba2", "mi_conv_step")(_p(u), _dt(u), ld, col_offset, M, width, K, _p(weight), _p(bias),
                                         _p(conv_state), _p(slot_ids), _stream()), "conv_step", f"(K={K})")


def ssm_scan(xbc: torch.Tensor, dt: torch.Tensor, dt_bias: torch.Tensor, A: torch.Tensor, D: torch.Tensor,
             ssm_state: torch.Tensor, cu_seqlens: torch.Tensor, slot_ids: torch.Tensor, num_groups: int,
             y: torch.Tensor, longest: int = 0) -> None:
    """Selective scan of every lane from and into ``ssm_state[slot]`` [H, P, N] (float32).

    ``xbc`` [T, E + 2*G*N] = post-conv x | B | C; ``dt`` [T, H] raw (a column view is fine);
    ``y`` float32 [T, E] gets s.C + D*x.  ``longest``: an upper bound of the tokens of a lane if known (it
    sizes the blocks of tokens a workgroup stages, never the result)."""
    xbc_ld = _row_major(xbc, "xbc")
    dt_ld = _row_major(dt, "dt")
    y_ld = _row_major(y, "y")
    _need(ssm_state.dim() == 4 and ssm_state.dtype == torch.float32 and ssm_state.is_contiguous(),
          "ssm_scan: state must be contiguous float32 [slots, H, P, N]")
    _, H, P, N = ssm_state.shape
    T = xbc.shape[0]
    _need(xbc.shape[1] == H * P + 2 * num_groups * N and dt.shape == (T, H) and dt.dtype == xbc.dtype
          and y.shape == (T, H * P) and y.dtype == torch.float32, "ssm_scan: shapes do not match")
    for name, vector in (("dt_bias", dt_bias), ("A", A), ("D", D)):
        _need(vector.dtype == torch.float32 and vector.numel() == H and vector.is_contiguous() and vector.is_cuda,
              f"ssm_scan: {name} must be float32 [H]")
    _i32(cu_seqlens, "cu_seqlens")
    _i32(slot_ids, "slot_ids")
    num_lanes = slot_ids.numel()
    _need(cu_seqlens.numel() == num_lanes + 1, "ssm_scan: cu_seqlens must have lanes+1 entries")
    longest = min(int(longest), T) if longest and longest > 0 else T
    # lanes of several tokens: every token's delta and decay are formed once, ahead of the scan, into a work area
    delta_decay = None if longest == 1 else torch.empty((T, H, 2), dtype=torch.float32, device=xbc.device)
    _check(_fn("mamba2", "mi_ssm_scan")(
        _p(xbc), _dt(xbc), xbc_ld, _p(dt), dt_ld, _p(dt_bias), _p(A), _p(D), _p(ssm_state), _p(cu_seqlens),
        _p(slot_ids), num_lanes, longest, H, P, N, num_groups, _p(delta_decay), T, _p(y), y_ld,
        _stream()), "ssm_scan", f"(N={N})")


class SsdChunks:
    """The chunk table of one step for chunks of ``chunk_size`` tokens: every lane is cut from its
    first token into chunks (the last one may be short).  ``chunks`` int32 [n, 4] = (lane, first
    token row, length, index within the lane); ``lane_chunks`` int32 [lanes, 2] = (first chunk,
    number of chunks)."""

    def __init__(self, lane_lengths: Sequence[int], chunk_size: int, device):
        _need(chunk_size > 0 and len(lane_lengths) > 0 and all(length > 0 for length in lane_lengths),
              "ssd: lanes and the chunk size must be positive")
        rows, lanes, first = [], [], 0
        for lane, length in enumerate(lane_lengths):
            count = -(-length // chunk_size)
            lanes.append((len(rows), count))
            for index in range(count):
                rows.append((lane, first + index * chunk_size, min(chunk_size, length - index * chunk_size), index))
            first += length
        self.chunk_size = chunk_size
        self.num_tokens = first
        self.num_lanes = len(lane_lengths)
        self.num_chunks = len(rows)
        flat = [value for row in rows for value in row] + [value for row in lanes for value in row]
        packed = torch.tensor(flat, dtype=torch.int32)
        packed = packed.to(device, non_blocking=True)
        self.chunks = packed[:4 * len(rows)]
        self.lane_chunks = packed[4 * len(rows):]


def ssd_supported(chunk_size: int, head_dim: int, state_size: int, num_groups: int, inner_size: int) -> bool:
    """Whether ``ssd_prefill`` covers these sizes (otherwise ``ssm_scan`` does)."""
    return bool(_fn("ssd", "mi_ssd_supported")(chunk_size, head_dim, state_size, num_groups, inner_size))


def ssd_prefill(xbc: torch.Tensor, dt: torch.Tensor, dt_bias: torch.Tensor, A: torch.Tensor, D: torch.Tensor,
                ssm_state: torch.Tensor, table: SsdChunks, slot_ids: torch.Tensor, num_groups: int,
                y: Optional[torch.Tensor], z: Optional[torch.Tensor] = None,
                gated: Optional[torch.Tensor] = None, conv: Optional[dict] = None) -> None:
    """The selective scan of ``ssm_scan`` (same arguments and results beyond rounding) for bfloat16,
    in chunks on the matrix cores.  ``table`` cuts this step's lanes into chunks.  With ``z`` and
    ``gated`` (bfloat16 [T, E], column views are fine) it writes gated = y * SiLU(z) and no y.
    With ``conv`` = {u, weight, bias, state} the conv runs here too: ``xbc`` is then written (what
    ``conv1d_silu`` would put there from the raw rows ``u`` [T, C]) and the tails ``state`` updated
    (as ``conv_state_update`` would); see ``ssd_conv_supported``."""
    xbc_ld = _row_major(xbc, "xbc")
    dt_ld = _row_major(dt, "dt")
    fused_gate = z is not None
    _need((gated is not None) == fused_gate and (y is None) == fused_gate,
          "ssd_prefill: give either y, or z and gated")
    if fused_gate:
        z_ld, gated_ld, y_ld = _row_major(z, "z"), _row_major(gated, "gated"), 0
        _need(z.dtype == torch.bfloat16 and gated.dtype == torch.bfloat16 and z.shape == gated.shape
              and z.data_ptr() % 8 == 0 and gated.data_ptr() % 8 == 0, "ssd_prefill: z/gated do not fit")
    else:
        z_ld = gated_ld = 0
        y_ld = _row_major(y, "y")
    _need(ssm_state.dim() == 4 and ssm_state.dtype == torch.float32 and ssm_state.is_contiguous(),
          "ssd_prefill: state must be contiguous float32 [slots, H, P, N]")
    _, H, P, N = ssm_state.shape
    T = xbc.shape[0]
    E, GN = H * P, num_groups * N
    _need(xbc.dtype == torch.bfloat16 and xbc.shape[1] == E + 2 * GN and dt.shape == (T, H)
          and dt.dtype == xbc.dtype, "ssd_prefill: shapes do not match (bfloat16 only)")
    result = gated if fused_gate else y
    _need(result.shape == (T, E) and (fused_gate or y.dtype == torch.float32), "ssd_prefill: output shape")
    _need(table.num_tokens == T and table.num_lanes == slot_ids.numel(),
          "ssd_prefill: the chunk table was made for another step")
    for name, vector in (("dt_bias", dt_bias), ("A", A), ("D", D)):
        _need(vector.dtype == torch.float32 and vector.numel() == H and vector.is_contiguous() and vector.is_cuda,
              f"ssd_prefill: {name} must be float32 [H]")
    _i32(slot_ids, "slot_ids")
    _need(xbc.data_ptr() % 16 == 0 and (fused_gate or y.data_ptr() % 16 == 0),
          "ssd_prefill: xbc and y must be 16-byte aligned")
    Q, chunks = table.chunk_size, table.num_chunks
    device = xbc.device
    delta = torch.empty((2, T, H), dtype=torch.float32, device=device)
    transposed = torch.empty((chunks * (E + GN) * Q,), dtype=torch.bfloat16, device=device)
    chunk_state = torch.empty((chunks * H * P * N + chunks * H,), dtype=torch.float32, device=device)
    state_in = torch.empty((chunks * H * P * N,), dtype=torch.bfloat16, device=device)
    decay = chunk_state[chunks * H * P * N:]
    raw = conv_w = conv_b = conv_state = None
    raw_ld = taps = 0
    if conv is not None:
        raw, conv_w, conv_b, conv_state = conv["u"], conv["weight"], conv.get("bias"), conv["state"]
        raw_ld = _row_major(raw, "conv u")
        C = E + 2 * GN
        taps = conv_w.shape[1]
        _need(raw.dtype == torch.bfloat16 and raw.shape == (T, C), "ssd_prefill: conv u must be bfloat16 [T, C]")
        _need(conv_w.dtype == torch.float32 and conv_w.shape == (C, taps) and conv_w.is_contiguous(),
              "ssd_prefill: conv weight must be float32 [C, K]")
        _need(conv_b is None or (conv_b.dtype == torch.float32 and conv_b.numel() == C), "ssd_prefill: bad conv bias")
        _need(conv_state.dim() == 3 and conv_state.shape[1:] == (taps - 1, C) and conv_state.dtype == torch.bfloat16
              and conv_state.is_contiguous(), "ssd_prefill: bad conv state")
        _need(ssd_conv_supported(taps, C, raw), "ssd_prefill: the conv does not fit (see ssd_conv_supported)")
    _check(_fn("ssd", "mi_ssd_prefill")(
        _p(xbc), xbc_ld, _p(dt), dt_ld, _p(dt_bias), _p(A), _p(D), _p(ssm_state), _p(table.chunks), chunks,
        _p(table.lane_chunks), _p(slot_ids), table.num_lanes, Q, H, P, N, num_groups, _p(delta[0]), _p(delta[1]),
        _p(transposed), _p(chunk_state), _p(decay), _p(state_in), _p(y), y_ld, _p(z), z_ld, _p(gated), gated_ld,
        _p(raw), raw_ld, _p(conv_w), _p(conv_b), _p(conv_state), int(taps), _stream()),
        "ssd_prefill", f"(Q={Q}, P={P}, N={N})")


def ssd_conv_supported(taps: int, channels: int, u: torch.Tensor) -> bool:
    """Whether ``ssd_prefill`` can run the conv itself: 2 to 4 taps, channels in eights, 16-byte rows."""
    return (2 <= taps <= 4 and channels % 8 == 0 and u.dim() == 2 and u.stride(1) == 1 and u.stride(0) % 8 == 0
            and u.data_ptr() % 16 == 0)


def gate_norm(y: torch.Tensor, z: torch.Tensor, weight: Optional[torch.Tensor], num_groups: int, eps: float,
              out: torch.Tensor) -> None:
    """out = y * SiLU(z), then (with a weight) RMSNorm over each group of E/G channels."""
    y_ld = _row_major(y, "y")
    z_ld = _row_major(z, "z")
    out_ld = _row_major(out, "out")
    T, E = y.shape
    _need(y.dtype == torch.float32 and z.shape == (T, E) and out.shape == (T, E) and out.dtype == z.dtype,
          "gate_norm: shapes do not match")
    _need(weight is None or (weight.dtype == torch.float32 and weight.numel() == E and weight.is_contiguous()),
          "gate_norm: weight must be float32 [E]")
    _check(_fn("mamba2", "mi_gate_norm")(_p(y), y_ld, _p(z), _dt(z), z_ld, _p(weight), num_groups, float(eps),
                                         _p(out), out_ld, T, E, _stream()), "gate_norm")


# --------------------------------------------------------------------------- fused decode kernels
PRO_NORM, PRO_PLAIN = 0, 1
EPI_PLAIN, EPI_SWIGLU, EPI_CONV = 0, 1, 2


def fused_gemm_supported(normed: bool, rows: int, in_features: int) -> bool:
    """Whether ``fused_gemm`` covers a batch of ``rows`` rows of ``in_features`` inputs."""
    return bool(_fn("decode", "mi_fused_gemm_supported")(PRO_NORM if normed else PRO_PLAIN, rows, in_features))


def fragment_order(weight: torch.Tensor) -> torch.Tensor:
    """A copy of weight [N, K] (K a multiple of 32) in the order in which the skinny kernels' waves read it:
    [ceil(N / 16), K / 32, 4, 16, 8] with element [n, c, q, r, j] = weight[16 n + r, 32 c + 8 q + j], rows past N
    zero.  A wave's load of a fragment is then one run of 1 KiB."""
    _need(weight.dim() == 2 and weight.shape[1] % 32 == 0, "fragment_order: weight must be [N, K] with K a multiple of 32")
    N, K = weight.shape
    if N % 16:
        weight = torch.cat([weight, weight.new_zeros((-N % 16, K))])
    return weight.view(-1, 16, K // 32, 4, 8).permute(0, 2, 3, 1, 4).contiguous()


def _weight_operand(weight: torch.Tensor, fragments: Optional[torch.Tensor], name: str) -> torch.Tensor:
    if fragments is None:
        return weight
    N, K = weight.shape
    _need(fragments.dtype == torch.bfloat16 and fragments.is_contiguous() and fragments.is_cuda
          and fragments.shape == (-(-N // 16), K // 32, 4, 16, 8), f"{name}: fragments do not fit the weight")
    return fragments


@dataclass(frozen=True)
class AttentionRuns:
    """What ``mixer_decode(merge=False)`` leaves of the attended heads: ``partial`` float32
    [M, heads, runs, head_dim + 2], (maximum, normalizer, sums) per run of ``run_keys`` keys."""
    partial: torch.Tensor
    positions: torch.Tensor
    heads: int
    head_dim: int
    runs: int
    run_keys: int
    page_size: int
    window: int


def fused_gemm_merge_supported(M: int, K: int, heads: int, head_dim: int) -> bool:
    """Whether ``fused_gemm_merge`` takes a step of M rows (the merged heads sit in LDS beside the waves' sums)."""
    merged = heads * head_dim
    waves = 8 if K // 32 > 32 else 4
    return (M <= 16 and K % 32 == 0 and merged % 32 == 0 and merged <= K
            and waves * 1024 + 1024 + M * (merged + 8) * 2 <= 64 * 1024)


def fused_gemm_merge(weight: torch.Tensor, bias: Optional[torch.Tensor], out: Optional[torch.Tensor], x: torch.Tensor,
                     attended: AttentionRuns, fragments: Optional[torch.Tensor] = None,
                     residual: Optional[tuple] = None) -> None:
    """out[M, N] = x [M, K] . weight[N, K]^T (+ bias) in bfloat16 for a step of up to 16 rows, where the first
    heads * head_dim columns of x are not read but merged from the runs of keys that ``mixer_decode(merge=False)``
    left: the merge of the runs and the product in one launch.  With ``residual`` = (h, hb, next norm's weight,
    ssq) the result is added to the residual stream as ``fused_gemm_residual`` does it, and ``out`` is None."""
    _need(weight.dtype == torch.bfloat16 and weight.dim() == 2 and weight.is_contiguous() and weight.is_cuda,
          "fused_gemm_merge: weight must be contiguous bfloat16 [N, K]")
    N, K = weight.shape
    x_ld = _row_major(x, "x")
    M = x.shape[0]
    _need(x.dtype == torch.bfloat16 and x.shape == (M, K) and x.data_ptr() % 16 == 0, "fused_gemm_merge: bad x")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == N and bias.is_contiguous()),
          "fused_gemm_merge: bias must be float32 [N]")
    h = hb = next_weight = ssq = None
    hb_ld = out_ld = 0
    if residual is not None:
        h, hb, next_weight, ssq = residual
        hb_ld = _residual_arguments(h, hb, next_weight, ssq, M, N, "fused_gemm_merge")
    else:
        _need(out.dtype == torch.bfloat16 and out.shape == (M, N), "fused_gemm_merge: out must be bfloat16 [M, N]")
        out_ld = _row_major(out, "out")
    _need(attended.partial.dtype == torch.float32 and attended.partial.is_contiguous()
          and attended.partial.numel() >= M * attended.heads * attended.runs * (attended.head_dim + 2),
          "fused_gemm_merge: the partial results do not cover the step")
    _i32(attended.positions, "positions")
    _need(attended.positions.numel() == M, "fused_gemm_merge: one position per row")
    operand = _weight_operand(weight, fragments, "fused_gemm_merge")
    _check(_fn("decode", "mi_fused_gemm_merge")(
        _p(attended.partial), _p(attended.positions), attended.heads, attended.head_dim, attended.runs,
        attended.run_keys, attended.page_size, attended.window, _p(x), x_ld, _p(operand), _p(bias), M, N, K, _p(out),
        out_ld, int(fragments is not None), _p(h), _p(hb), hb_ld, _p(next_weight), _p(ssq), _stream()),
        "fused_gemm_merge", f"(M={M}, N={N}, K={K})")


def fused_gemm_split(weight: torch.Tensor, bias: Optional[torch.Tensor], x: torch.Tensor, partial: torch.Tensor,
                     feature_tiles: int = 1, fragments: Optional[torch.Tensor] = None,
                     shared_rows: bool = False) -> None:
    """x [M, K] . weight[N, K]^T (+ bias) for a small batch in bfloat16, split over K: slab s of
    ``partial`` (float32 [S, M, N], contiguous) receives the sums over the s-th run of K, the bias
    in slab 0.  The product is the sum of the slabs (``add_partials_rmsnorm`` adds them to the
    residual stream): many rows, a long K and few output features fill the GPU this way.
    ``shared_rows`` (up to 128 rows, one feature tile a wave beyond 64; K >= 128): the kernel whose four waves
    share the step's rows through LDS instead of fetching them each."""
    _need(weight.dtype == torch.bfloat16 and weight.dim() == 2 and weight.is_contiguous() and weight.is_cuda,
          "fused_gemm_split: weight must be contiguous bfloat16 [N, K]")
    N, K = weight.shape
    x_ld = _row_major(x, "x")
    M = x.shape[0]
    _need(x.dtype == torch.bfloat16 and x.shape == (M, K) and x.data_ptr() % 16 == 0, "fused_gemm_split: bad x")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == N and bias.is_contiguous()),
          "fused_gemm_split: bias must be float32 [N]")
    _need(partial.dtype == torch.float32 and partial.dim() == 3 and partial.shape[1:] == (M, N)
          and partial.is_contiguous() and partial.is_cuda, "fused_gemm_split: partial must be contiguous float32 [S, M, N]")
    operand = _weight_operand(weight, fragments, "fused_gemm_split")
    entry = "mi_shared_rows_gemm_split" if shared_rows else "mi_fused_gemm_split"
    _check(_fn("decode", entry)(_p(x), x_ld, _p(operand), _p(bias), M, N, K, _p(partial), partial.shape[0],
                                int(feature_tiles), int(fragments is not None), _stream()),
           "fused_gemm_split", f"(M={M}, N={N}, K={K}, S={partial.shape[0]}, shared_rows={shared_rows})")


def fused_gemm(weight: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor, *, out_scale: float = 1.0,
               x: Optional[torch.Tensor] = None, h_in: Optional[torch.Tensor] = None,
               deltas: Sequence[torch.Tensor] = (), h_out: Optional[torch.Tensor] = None,
               norm_weight: Optional[torch.Tensor] = None, eps: float = 0.0, epilogue: int = EPI_PLAIN,
               conv: Optional[dict] = None, feature_tiles: int = 1, fragments: Optional[torch.Tensor] = None,
               row_scale: Optional["RowScale"] = None, shared_rows: bool = False, row_tiles: int = 1) -> None:
    """out[M, N'] = epilogue(prologue . weight[N, K]^T + bias) for a small batch in bfloat16.

    Prologue: ``x`` [M, K] bfloat16, or ``h_in`` float32 [M, K] with up to two bfloat16 ``deltas``:
    the rows are summed (the sum goes to ``h_out``, a different tensor, if given), RMS-normed
    with ``norm_weight`` and ``eps``.  Epilogue PLAIN: bfloat16 or float32 ``out`` [M, N] times
    ``out_scale``.  SWIGLU: weight rows in tiles of 8 gate + 8 up rows, ``out`` [M, N/2].
    CONV: ``conv`` = {lo, hi, taps, weight [C, taps], bias, state [slots, taps-1, C], slot_ids}:
    rows lo..hi-1 go through the causal depthwise conv step of their channel with the request's
    tail (which is rolled) and SiLU.  ``feature_tiles`` (1, 2 or 4; more than one with ``x`` only): how many
    tiles of 16 output features a workgroup owns; the rows of x cross the caches once per workgroup, so
    steps of many rows gain from more.  ``fragments``: ``fragment_order(weight)``, read instead of the weight.
    ``row_scale`` (with ``x``): x holds rows times a norm's weight that are not divided by their root mean
    square yet; the sums of row m are multiplied by 1 / sqrt(sum of squares of the row / width + eps) before the
    bias, from the partial sums of squares that ``fused_gemm_residual`` left.  ``shared_rows`` (``x``, K >= 128,
    bfloat16 ``out``, 1 or 2 feature tiles a wave): the kernel whose four waves own feature tiles
    and share the step's rows through LDS instead of fetching them each.  ``row_tiles`` (1 to 4; more than one
    with ``x``, one feature tile, not ``shared_rows``): the step's tiles of 16 rows are dealt out to that many
    workgroups per tile of features, each of which fetches its own rows only."""
    _need(weight.dtype == torch.bfloat16 and weight.dim() == 2 and weight.is_contiguous() and weight.is_cuda,
          "fused_gemm: weight must be contiguous bfloat16 [N, K]")
    _need(row_scale is None or x is not None, "fused_gemm: a row scale needs x")
    _need(1 <= row_tiles <= 4 and (row_tiles == 1 or (x is not None and feature_tiles == 1 and not shared_rows)),
          "fused_gemm: row_tiles is 1 to 4, and more than 1 needs x, one feature tile and the skinny kernel")
    if row_scale is not None:
        _need(row_scale.ssq.dtype == torch.float32 and row_scale.ssq.is_contiguous() and row_scale.ssq.dim() == 2
              and row_scale.ssq.shape[1] == 16 * (-(-out.shape[0] // 16)), "fused_gemm: the partial sums of squares do not fit the step")
    _need(feature_tiles in (1, 2, 4) and (feature_tiles == 1 or x is not None),
          "fused_gemm: feature_tiles is 1, 2 or 4, and more than 1 needs x")
    _need(not shared_rows or (x is not None and out.dtype == torch.bfloat16 and feature_tiles in (1, 2)),
          "fused_gemm: shared_rows takes x, writes bfloat16 and has 1 or 2 feature tiles a wave")
    N, K = weight.shape
    M = out.shape[0]
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == N and bias.is_contiguous()),
          "fused_gemm: bias must be float32 [N]")
    out_ld = _row_major(out, "out")
    _need(out.dtype in (torch.bfloat16, torch.float32), "fused_gemm: out must be bfloat16 or float32")
    _need(out.shape[1] == (N // 2 if epilogue == EPI_SWIGLU else N), "fused_gemm: out has the wrong width")
    if x is not None:
        pro = PRO_PLAIN
        x_ld = _row_major(x, "x")
        _need(x.dtype == torch.bfloat16 and x.shape == (M, K) and x.data_ptr() % 16 == 0, "fused_gemm: bad x")
    else:
        pro = PRO_NORM
        x_ld = 0
        _need(h_in is not None and h_in.dtype == torch.float32 and h_in.shape == (M, K) and h_in.is_contiguous(),
              "fused_gemm: h_in must be contiguous float32 [M, K]")
        _need(len(deltas) <= 2 and all(d.dtype == torch.bfloat16 and d.shape == (M, K) and d.is_contiguous()
                                       for d in deltas), "fused_gemm: deltas must be contiguous bfloat16 [M, K]")
        _need(h_out is None or (h_out.shape == (M, K) and h_out.dtype == torch.float32 and h_out.is_contiguous()
                                and h_out.data_ptr() != h_in.data_ptr()), "fused_gemm: bad h_out")
        _need(norm_weight is not None and norm_weight.dtype == torch.float32 and norm_weight.numel() == K,
              "fused_gemm: norm_weight must be float32 [K]")
    lo = hi = taps = 0
    conv_w = conv_b = conv_state = slot_ids = None
    if epilogue == EPI_CONV:
        lo, hi, taps = conv["lo"], conv["hi"], conv["taps"]
        conv_w, conv_b, conv_state, slot_ids = conv["weight"], conv.get("bias"), conv["state"], conv["slot_ids"]
        channels = hi - lo
        _need(conv_w.dtype == torch.float32 and conv_w.shape == (channels, taps) and conv_w.is_contiguous(),
              "fused_gemm: conv weight must be float32 [C, taps]")
        _need(conv_b is None or (conv_b.dtype == torch.float32 and conv_b.numel() == channels), "fused_gemm: bad conv bias")
        _need(conv_state.dtype == torch.bfloat16 and conv_state.shape[1:] == (max(taps - 1, 0), channels)
              and conv_state.is_contiguous(), "fused_gemm: bad conv state")
        _i32(slot_ids, "slot_ids")
        _need(slot_ids.numel() >= M, "fused_gemm: one slot per row")
    _check(_fn("decode", "mi_fused_gemm")(
        pro, epilogue, _p(h_in), _p(deltas[0]) if len(deltas) > 0 else None, _p(deltas[1]) if len(deltas) > 1 else None,
        _p(h_out), _p(norm_weight), float(eps), _p(x), x_ld, _p(_weight_operand(weight, fragments, "fused_gemm")),
        _p(bias), M, N, K, _p(out), out_ld,
        1 if out.dtype == torch.float32 else 0, float(out_scale), lo, hi, taps, _p(conv_w), _p(conv_b), _p(conv_state),
        _p(slot_ids), -int(feature_tiles) if shared_rows else int(feature_tiles), int(fragments is not None),
        _p(row_scale.ssq) if row_scale is not None else None, row_scale.ssq.shape[0] if row_scale is not None else 0,
        int(row_scale.width) if row_scale is not None else 0, float(row_scale.eps) if row_scale is not None else 0.0,
        int(row_tiles), _stream()), "fused_gemm", f"(M={M}, N={N}, K={K})")


@dataclass(frozen=True)
class RowScale:
    """Partial sums of squares ``ssq`` float32 [workgroups, 16 ceil(M / 16)] of rows of ``width`` elements, and the
    ``eps`` of the norm they belong to: what ``fused_gemm_residual`` leaves for the product behind the norm."""
    ssq: torch.Tensor
    width: int
    eps: float


def residual_workspace(M: int, N: int, device) -> torch.Tensor:
    """The partial sums of squares of a step of M rows of N elements, for ``fused_gemm_residual`` to fill."""
    return torch.empty((-(-N // 16), 16 * (-(-M // 16))), dtype=torch.float32, device=device)


def _residual_arguments(h, hb, next_weight, ssq, M, N, name):
    _need(h.dtype == torch.float32 and h.shape == (M, N) and h.is_contiguous(), f"{name}: h must be contiguous float32 [M, N]")
    _need(hb.dtype == torch.bfloat16 and hb.shape == (M, N), f"{name}: hb must be bfloat16 [M, N]")
    _need(next_weight.dtype == torch.float32 and next_weight.numel() == N and next_weight.is_contiguous(),
          f"{name}: the next norm's weight must be float32 [N]")
    _need(ssq.dtype == torch.float32 and ssq.is_contiguous() and ssq.shape == (-(-N // 16), 16 * (-(-M // 16))),
          f"{name}: ssq must be float32 [ceil(N / 16), 16 ceil(M / 16)]")
    return _row_major(hb, "hb")


def fused_gemm_residual(weight: torch.Tensor, bias: Optional[torch.Tensor], x: torch.Tensor, h: torch.Tensor,
                        hb: torch.Tensor, next_weight: torch.Tensor, ssq: torch.Tensor,
                        fragments: Optional[torch.Tensor] = None, row_tiles: int = 1) -> None:
    """h += x [M, K] . weight[N, K]^T (+ bias), float32 in place: a projection whose result joins the residual
    stream.  Beside it ``hb`` = bfloat16(h * next_weight), the new rows times the next norm's weight, and ``ssq``
    (``residual_workspace``), the sums of squares of the new rows over every 16 features: what ``fused_gemm`` with
    ``row_scale`` needs to be the product behind that norm, without a pass for the norm.  ``row_tiles`` (1 to 4):
    the step's tiles of 16 rows dealt out to that many workgroups per tile of features (a projection into the
    stream has few features: 64 workgroups for 1,024 of them, 256 with the 64 rows of a step over four)."""
    _need(1 <= row_tiles <= 4, "fused_gemm_residual: row_tiles is 1 to 4")
    _need(weight.dtype == torch.bfloat16 and weight.dim() == 2 and weight.is_contiguous() and weight.is_cuda,
          "fused_gemm_residual: weight must be contiguous bfloat16 [N, K]")
    N, K = weight.shape
    x_ld = _row_major(x, "x")
    M = x.shape[0]
    _need(x.dtype == torch.bfloat16 and x.shape == (M, K) and x.data_ptr() % 16 == 0, "fused_gemm_residual: bad x")
    _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == N and bias.is_contiguous()),
          "fused_gemm_residual: bias must be float32 [N]")
    hb_ld = _residual_arguments(h, hb, next_weight, ssq, M, N, "fused_gemm_residual")
    _check(_fn("decode", "mi_fused_gemm_residual")(
        _p(x), x_ld, _p(_weight_operand(weight, fragments, "fused_gemm_residual")), _p(bias), M, N, K, _p(h), _p(hb),
        hb_ld, _p(next_weight), _p(ssq), int(fragments is not None), int(row_tiles), _stream()), "fused_gemm_residual",
        f"(M={M}, N={N}, K={K})")


def mixer_decode_supported(num_heads: int, num_kv_heads: int, head_dim: int, page_size: int, state_size: int,
                           max_seq_len: int = 1, window: Optional[int] = None, rotary_dim: int = 0) -> bool:
    return (head_dim in (64, 128) and num_heads // num_kv_heads <= 8 and page_size % 8 == 0 and page_size <= 512
            and state_size <= 512 and rotary_dim % 16 == 0)


MERGE_AT_ONCE = 8          # runs of keys a merge asks for at once (decode.hip)


def mixer_runs(M: int, num_kv_heads: int, page_size: int, span: int):
    """(keys of a run, runs per token and kv head) as ``mixer_decode`` cuts the contexts of a step of M tokens
    whose requests hold up to ``span`` keys."""
    run_keys, runs = ctypes.c_int(0), ctypes.c_int(0)
    _check(_fn("decode", "mi_mixer_runs")(M, num_kv_heads, page_size, span, ctypes.addressof(run_keys),
                                          ctypes.addressof(runs)), "mixer_decode", "(no run length for these sizes)")
    return run_keys.value, runs.value


def mixer_decode(u: torch.Tensor, *, num_heads: int, num_kv_heads: int, head_dim: int, q_col: int, k_col: int,
                 v_col: int, inv_freq: Optional[torch.Tensor], rotary_dim: int, k_cache: torch.Tensor,
                 v_cache: torch.Tensor, block_tables: torch.Tensor, positions: torch.Tensor,
                 slot_mapping: torch.Tensor, scale: float, window: Optional[int], max_seq_len: int,
                 ssm_heads: int, ssm_head_dim: int, state_size: int, num_groups: int,
                 z_col: int, x_col: int, dt_col: int, dt_bias: torch.Tensor, A: torch.Tensor, D: torch.Tensor,
                 ssm_state: torch.Tensor, slot_ids: torch.Tensor, out: torch.Tensor,
                 ssm_y: Optional[torch.Tensor], merge: bool = True) -> Optional[AttentionRuns]:
    """Both mixers of a decode step in one launch.  ``u`` [M, >=cols] holds each token's projected
    row (q, k, v unrotated; x, B, C after the conv).  Attention: rotates q and the new key, writes
    the new K/V into the cache cell ``slot_mapping``, attends over the request's pages, writes
    ``out[:, :Hq*dh]``.  State space: one scan step from and into ``ssm_state[slot_ids]``, writes
    ``y * SiLU(z)`` to ``out[:, Hq*dh:]``, or float32 ``y`` to ``ssm_y`` when a grouped norm
    follows.  ``max_seq_len``: an upper bound of the longest context in the batch.  With ``merge=False``
    ``out[:, :Hq*dh]`` is not written: the runs of keys are returned unmerged, for ``fused_gemm_merge``."""
    u_ld = _row_major(u, "u")
    out_ld = _row_major(out, "out")
    M = u.shape[0]
    E = ssm_heads * ssm_head_dim
    _need(u.dtype == torch.bfloat16 and out.dtype == torch.bfloat16 and out.shape == (M, num_heads * head_dim + E),
          "mixer_decode: u/out shapes do not match")
    page_stride, page_size = _cache_view(k_cache, v_cache, num_kv_heads, head_dim, u.dtype)
    _need(mixer_decode_supported(num_heads, num_kv_heads, head_dim, page_size, state_size, max_seq_len, window,
                                 rotary_dim if inv_freq is not None else 0), "mixer_decode: geometry not covered")
    for name, tensor in (("block_tables", block_tables), ("positions", positions), ("slot_mapping", slot_mapping),
                         ("slot_ids", slot_ids)):
        _i32(tensor, name)
    _need(block_tables.dim() == 2 and block_tables.shape[0] >= M and positions.numel() == M
          and slot_mapping.numel() == M and slot_ids.numel() == M, "mixer_decode: metadata shapes do not match")
    _need(ssm_state.dtype == torch.float32 and ssm_state.shape[1:] == (ssm_heads, ssm_head_dim, state_size)
          and ssm_state.is_contiguous(), "mixer_decode: bad state")
    for name, vector in (("dt_bias", dt_bias), ("A", A), ("D", D)):
        _need(vector.dtype == torch.float32 and vector.numel() == ssm_heads, f"mixer_decode: {name} must be float32 [H]")
    _need(ssm_y is None or (ssm_y.dtype == torch.float32 and ssm_y.shape == (M, E) and ssm_y.is_contiguous()),
          "mixer_decode: bad ssm_y")
    widest = max(q_col + num_heads * head_dim, k_col + num_kv_heads * head_dim, v_col + num_kv_heads * head_dim,
                 z_col + E, x_col + E + 2 * num_groups * state_size, dt_col + ssm_heads)
    _need(u.shape[1] >= widest, "mixer_decode: u is too narrow")
    span = max(1, int(max_seq_len)) if not window else window + page_size
    run_keys, runs = mixer_runs(M, num_kv_heads, page_size, span)        # the launcher's own rule
    partial = torch.empty((M * num_heads * runs * (head_dim + 2),), dtype=torch.float32, device=u.device)
    _check(_fn("decode", "mi_mixer_decode")(
        _p(u), u_ld, M, num_heads, num_kv_heads, head_dim, q_col, k_col, v_col, _p(inv_freq), rotary_dim,
        _p(k_cache), _p(v_cache), page_stride, page_size, _p(block_tables), block_tables.shape[1], _p(positions),
        _p(slot_mapping), float(scale), int(window or 0), int(max_seq_len), ssm_heads, ssm_head_dim, state_size,
        num_groups, z_col, x_col, dt_col, _p(dt_bias), _p(A), _p(D), _p(ssm_state), _p(slot_ids), _p(out),
        out.data_ptr() + 2 * num_heads * head_dim,
        _p(ssm_y), out_ld, _p(partial), partial.numel(), int(merge), _stream()), "mixer_decode")
    if merge or runs == 1:                  # one workgroup per token and kv head has written the heads itself
        return None
    return AttentionRuns(partial, positions, num_heads, head_dim, runs, run_keys, page_size, int(window or 0))


# --------------------------------------------------------------------------- memory microbenchmarks
def stream_read(data: torch.Tensor, sink: torch.Tensor, blocks: int = 4096) -> None:
    """Read ``data`` (contiguous, a multiple of 16 bytes) once; ``sink``: an int32 GPU tensor."""
    _need(data.is_cuda and data.is_contiguous() and (data.numel() * data.element_size()) % 16 == 0,
          "stream_read: data must be a contiguous GPU tensor of a multiple of 16 bytes")
    _i32(sink, "sink")
    _check(_fn("microbench", "mi_stream_read")(_p(data), data.numel() * data.element_size(), _p(sink), int(blocks),
                                               _stream()), "stream_read")


def stream_rmw(data: torch.Tensor, scale: float = 1.0, blocks: int = 4096) -> None:
    """data *= scale in place, float32, read once and written once."""
    _need(data.is_cuda and data.is_contiguous() and data.dtype == torch.float32 and data.numel() % 4 == 0,
          "stream_rmw: data must be a contiguous float32 GPU tensor of a multiple of 4 elements")
    _check(_fn("microbench", "mi_stream_rmw")(_p(data), data.numel() * 4, float(scale), int(blocks), _stream()),
           "stream_rmw")


# --------------------------------------------------------------------------- sampling
def apply_penalties(logits, tokens, offsets, prompt_lens, repetition, presence, frequency, count_all, count_gen,
                    extra_source=None, extra_rows=None):
    """Repetition, presence and frequency penalties over each row's history ``tokens[offsets[b]:offsets[b + 1]]``
    (its first ``prompt_lens[b]`` tokens are the prompt).  A row's newest generated token may be on the device
    only: ``extra_rows[b]`` (int32, -1 = none) is then its place in ``extra_source`` (int32)."""
    B, V = logits.shape
    _need(logits.dtype == torch.float32 and logits.is_contiguous() and logits.is_cuda, "penalties: bad logits")
    for name, tensor in (("tokens", tokens), ("offsets", offsets), ("prompt_lens", prompt_lens),
                         ("count_all", count_all), ("count_gen", count_gen)):
        _i32(tensor, name)
    _need(count_all.numel() >= B * V and count_gen.numel() >= B * V, "penalties: work areas are too small")
    _need(offsets.numel() == B + 1 and prompt_lens.numel() == B, "penalties: bad history layout")
    _need((extra_source is None) == (extra_rows is None), "penalties: extra tokens need their source and their rows")
    if extra_source is not None:
        _i32(extra_source, "extra_source")
        _i32(extra_rows, "extra_rows")
        _need(extra_rows.numel() == B, "penalties: one extra row index per row")
    _check(_fn("sampling", "mi_apply_penalties")(
        _p(logits), B, V, _p(tokens), _p(offsets), _p(prompt_lens), _p(repetition), _p(presence), _p(frequency),
        _p(count_all), _p(count_gen), _p(extra_source), _p(extra_rows), _stream()), "apply_penalties")


def keep_allowed(logits: torch.Tensor, ids: torch.Tensor, offsets: torch.Tensor, keep: torch.Tensor) -> None:
    """Rows ``b`` with a list of allowed tokens ``ids[offsets[b]:offsets[b + 1]]`` keep those logits and get -inf
    everywhere else; rows whose list is empty stay as they are.  ``keep``: a work area with a row of at least
    ``V`` 32-bit words for each row of ``logits``."""
    B, V = logits.shape
    _need(logits.dtype == torch.float32 and logits.is_contiguous() and logits.is_cuda, "keep_allowed: bad logits")
    _i32(ids, "ids")
    _i32(offsets, "offsets")
    _need(offsets.numel() == B + 1, "keep_allowed: one offset a row and one more")
    _need(keep.is_cuda and keep.dim() == 2 and keep.stride(1) == 1 and keep.shape[0] >= B
          and keep.element_size() in (4, 8), "keep_allowed: bad work area")
    words = keep.element_size() // 4
    _need(keep.shape[1] * words >= V, "keep_allowed: the work area's rows are too short")
    _check(_fn("sampling", "mi_keep_allowed")(_p(logits), B, V, _p(ids), _p(offsets), _p(keep),
                                              keep.stride(0) * words, _stream()), "keep_allowed")


def argmax(logits: torch.Tensor, out: torch.Tensor) -> None:
    B, V = logits.shape
    _need(logits.dtype == torch.float32 and logits.is_contiguous() and logits.is_cuda, "argmax: bad logits")
    _i32(out, "out")
    _need(out.numel() == B, "argmax: one output per row")
    _check(_fn("sampling", "mi_argmax")(_p(logits), B, V, _p(out), _stream()), "argmax")


def sample(logits, temperature, top_k, top_p, seeds, draw_index, keys, out, done=None) -> None:
    """One token per row; may overwrite ``logits``.  ``keys`` int64 [B, padded] work area.  With
    ``done`` (int32 [B] work area) the rows that need no full sort (all but a top-k above 1 024) are
    drawn by selection; without it every row is sorted."""
    B, V = logits.shape
    _need(logits.dtype == torch.float32 and logits.is_contiguous() and logits.is_cuda, "sample: bad logits")
    padded = keys.shape[1]
    _need(keys.dtype == torch.int64 and keys.shape[0] >= B and keys.is_contiguous(), "sample: bad work area")
    _need(temperature.dtype == torch.float32 and top_p.dtype == torch.float32 and seeds.dtype == torch.int64,
          "sample: bad parameter dtypes")
    _i32(top_k, "top_k")
    _i32(draw_index, "draw_index")
    _i32(out, "out")
    if done is not None:
        _i32(done, "done")
        _need(done.numel() >= B, "sample: done must hold one flag per row")
    _check(_fn("sampling", "mi_sample")(_p(logits), B, V, padded, _p(temperature), _p(top_k), _p(top_p),
                                        _p(seeds), _p(draw_index), _p(keys), _p(out), _p(done), _stream()), "sample")
