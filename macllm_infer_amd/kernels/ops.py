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
                           _c_int, _c_float, _c_float, _c_ptr],
        "mi_add_partials_rmsnorm": [_c_ptr, _c_ptr, _c_int, _c_ptr, _c_float, _c_ptr, _c_int, _c_ptr, _c_int, _c_int,
                                    _c_int, _c_ptr],
        "mi_swiglu": [_c_ptr, _c_int, _c_long, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr],
        "mi_cast_rows": [_c_ptr, _c_ptr, _c_int, _c_long, _c_int, _c_int, _c_ptr],
        "mi_scale_to_f32": [_c_ptr, _c_int, _c_float, _c_ptr, _c_long, _c_ptr],
        "mi_tanh_softcap": [_c_ptr, _c_float, _c_long, _c_ptr],
        "mi_add_bias_round": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr],
        "mi_add_scaled_rmsnorm": [_c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_float, _c_ptr, _c_int, _c_ptr, _c_int, _c_int,
                                  _c_ptr],
        "mi_polynorm": [_c_ptr, _c_int, _c_long, _c_ptr, _c_float, _c_ptr, _c_long, _c_int, _c_int, _c_ptr],
        "mi_embed_bigram": [_c_ptr, _c_ptr, _c_int, _c_float, _c_ptr, _c_int, _c_long, _c_long, _c_ptr, _c_ptr, _c_ptr,
                            _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
        "mi_stream_add": [_c_ptr, _c_ptr, _c_int, _c_float, _c_ptr, _c_int, _c_int, _c_ptr],
        "mi_normed_sum": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_int, _c_int, _c_ptr],
        "mi_add_layernorm": [_c_ptr, _c_ptr, _c_int, _c_float, _c_ptr, _c_int, _c_float, _c_ptr, _c_int, _c_float, _c_ptr,
                             _c_ptr, _c_ptr, _c_float, _c_ptr, _c_ptr, _c_float, _c_ptr, _c_int, _c_ptr, _c_int, _c_int,
                             _c_ptr],
        "mi_clamped_glu": [_c_ptr, _c_int, _c_long, _c_ptr, _c_long, _c_int, _c_int, _c_float, _c_float, _c_float, _c_ptr],
    },
    "latent": {
        "mi_latent_prepare": [_c_ptr, _c_int, _c_long, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_float, _c_ptr,
                              _c_ptr, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_long, _c_int, _c_ptr, _c_long, _c_ptr],
        "mi_rotate_heads": [_c_ptr, _c_int, _c_long, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_int, _c_int,
                            _c_ptr, _c_long, _c_int, _c_int, _c_int, _c_ptr],
        "mi_head_gemm": [_c_ptr, _c_int, _c_long, _c_long, _c_ptr, _c_long, _c_long, _c_ptr, _c_long, _c_long, _c_int,
                         _c_int, _c_int, _c_int, _c_ptr],
        "mi_latent_attention": [_c_ptr, _c_long, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_long, _c_int, _c_ptr, _c_int,
                                _c_ptr, _c_int, _c_ptr, _c_ptr, _c_float, _c_int, _c_ptr, _c_long, _c_ptr],
        "mi_latent_attention_supported": [_c_int, _c_int],
        "mi_latent_decode_attention": [_c_ptr, _c_long, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_long, _c_int,
                                       _c_ptr, _c_int, _c_ptr, _c_ptr, _c_float, _c_int, _c_int, _c_int, _c_ptr, _c_ptr,
                                       _c_ptr, _c_long, _c_ptr],
    },
    "moe": {
        "mi_moe_route": [_c_ptr, _c_long, _c_int, _c_int, _c_int, _c_ptr, _c_float, _c_float, _c_int, _c_ptr, _c_ptr, _c_ptr,
                         _c_ptr],
        "mi_moe_plan": [_c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr],
        "mi_moe_expert_gemm": [_c_ptr, _c_int, _c_long, _c_int, _c_ptr, _c_long, _c_long, _c_int, _c_int, _c_ptr, _c_ptr,
                               _c_int, _c_int, _c_int, _c_int, _c_float, _c_float, _c_float, _c_ptr, _c_int, _c_long,
                               _c_ptr],
        "mi_moe_combine": [_c_ptr, _c_long, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_int, _c_long, _c_ptr, _c_ptr, _c_int, _c_int,
                           _c_ptr],
    },
    "linear_state": {
        "mi_linear_state_scan": [_c_ptr, _c_int, _c_long, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr,
                                 _c_ptr, _c_ptr, _c_int, _c_ptr, _c_long, _c_int, _c_ptr, _c_float, _c_ptr, _c_ptr, _c_int,
                                 _c_ptr, _c_long, _c_ptr, _c_float, _c_float, _c_float, _c_float, _c_ptr],
        "mi_linear_state_scan_chunked": [_c_ptr, _c_int, _c_long, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                                         _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_long, _c_int, _c_ptr, _c_float, _c_ptr,
                                         _c_ptr, _c_int, _c_ptr, _c_long, _c_ptr, _c_float, _c_float, _c_float, _c_float,
                                         _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr],
        "mi_linear_state_local_floats": [_c_int, _c_int, _c_int, _c_int, _c_int],
        "mi_linear_state_start_floats": [_c_int, _c_int, _c_int, _c_int],
        "mi_head_norm_gate": [_c_ptr, _c_long, _c_ptr, _c_int, _c_long, _c_ptr, _c_int, _c_int, _c_float, _c_int, _c_ptr,
                              _c_long, _c_int, _c_ptr],
        "mi_tanh_rows": [_c_ptr, _c_int, _c_long, _c_ptr, _c_long, _c_int, _c_int, _c_ptr],
    },
    "attention": {
        "mi_rope_kv_store": [_c_ptr, _c_int, _c_long, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_int,
                             _c_ptr, _c_ptr, _c_ptr, _c_long, _c_int, _c_ptr],
        "mi_paged_attention": [_c_ptr, _c_int, _c_long, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_long,
                               _c_int, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_float, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr,
                               _c_float, _c_int, _c_int,
                               _c_ptr, _c_long, _c_ptr, _c_long, _c_ptr, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int,
                               _c_ptr],
        "mi_attention_prepare": [_c_ptr, _c_int, _c_long, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr,
                                 _c_int, _c_int, _c_float, _c_ptr, _c_ptr, _c_float, _c_int, _c_ptr, _c_ptr, _c_float,
                                 _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_long, _c_int, _c_ptr],
        "mi_paged_attention_workspace": [_c_int, _c_int, _c_int, _c_int],
        "mi_prefill_attention": [_c_ptr, _c_long, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_long, _c_int, _c_ptr,
                                 _c_int, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_float, _c_int, _c_int, _c_ptr, _c_long,
                                 _c_ptr, _c_ptr, _c_int, _c_ptr],
        "mi_prefill_attention_forms": [_c_ptr, _c_long, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_long, _c_int,
                                       _c_ptr, _c_int, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_float, _c_int, _c_int, _c_ptr,
                                       _c_long, _c_int, _c_ptr, _c_ptr, _c_ptr],
        "mi_decode_attention": [_c_ptr, _c_long, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_long, _c_int,
                                _c_ptr, _c_int, _c_ptr, _c_ptr, _c_float, _c_int, _c_int, _c_int, _c_ptr, _c_ptr,
                                _c_ptr, _c_long, _c_ptr],
        "mi_decode_attention_forms": [_c_ptr, _c_long, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_long,
                                      _c_int, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_float, _c_int, _c_int, _c_int, _c_ptr,
                                      _c_ptr, _c_ptr, _c_long, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr, _c_ptr],
    },
    "mamba2": {
        "mi_conv1d_silu": [_c_ptr, _c_int, _c_long, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr,
                           _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr],
        "mi_conv_state_update": [_c_ptr, _c_int, _c_long, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int,
                                 _c_ptr],
        "mi_conv_step": [_c_ptr, _c_int, _c_long, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int,
                         _c_ptr],
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
                out: Optional[torch.Tensor], rows: Optional[torch.Tensor] = None,
                factors: Optional[Sequence[float]] = None) -> None:
    """h += sum(deltas) (float32, in place); out = h / sqrt(mean(h^2) + eps) * weight.  With ``factors`` (a number
    for each delta) h += sum of factor * delta, the products in float32.

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
    _need(factors is None or len(factors) == len(deltas), "add_rmsnorm: one factor for each delta")
    scales = [float(factor) for factor in (factors or ())] + [1.0, 1.0]
    _check(_fn("common", "mi_add_rmsnorm")(
        _p(h), _p(deltas[0]) if len(deltas) > 0 else None, _p(deltas[1]) if len(deltas) > 1 else None,
        delta_dtype, _p(weight), float(eps), _p(out), out_dtype, _p(rows), n_rows, d, scales[0], scales[1], _stream()),
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


GATE_ACTIVATIONS = {"silu": 0, "gelu_tanh": 1}


def swiglu(gate_up: torch.Tensor, out: torch.Tensor, tile: int = 0, activation: str = "silu") -> None:
    """out[t, i] = act(g[t, i]) * u[t, i] with a row of ``gate_up`` holding [g | u] (``tile`` 0) or
    g and u interleaved in tiles of ``tile`` columns: [g[0:tile] | u[0:tile] | g[tile:2 tile] | ...]; act is SiLU
    or ("gelu_tanh") 0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3)))."""
    _need(activation in GATE_ACTIVATIONS, f"swiglu: the activation {activation!r} is not known")
    ld = _row_major(gate_up, "gate_up")
    T, two_i = gate_up.shape
    _need(two_i % 2 == 0 and out.shape == (T, two_i // 2) and out.is_contiguous() and out.dtype == gate_up.dtype,
          "swiglu: out must be contiguous [T, I] of the input's dtype")
    _need(tile >= 0 and (tile == 0 or (two_i // 2) % tile == 0), "swiglu: the tile must divide the width")
    _check(_fn("common", "mi_swiglu")(_p(gate_up), _dt(gate_up), ld, _p(out), T, two_i // 2, int(tile),
                                      GATE_ACTIVATIONS[activation], _stream()), "swiglu")


def cast_rows(source: torch.Tensor, out: torch.Tensor) -> None:
    """out[t, :] = source[t, :] in ``out``'s dtype: the float32 stream's rows into (a column block of) a matrix of
    activations."""
    _need(source.dtype == torch.float32 and source.dim() == 2 and source.is_contiguous() and source.is_cuda,
          "cast_rows: the source must be contiguous float32 [T, d] on the GPU")
    ld = _row_major(out, "out")
    _need(out.shape == source.shape, "cast_rows: out must have the source's shape")
    if source.numel():
        _check(_fn("common", "mi_cast_rows")(_p(source), _p(out), _dt(out), ld, source.shape[0], source.shape[1],
                                             _stream()), "cast_rows")


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


def add_scaled_rmsnorm(h: torch.Tensor, delta: torch.Tensor, scale: torch.Tensor, weight: torch.Tensor, eps: float,
                       out: Optional[torch.Tensor], rows: Optional[torch.Tensor] = None) -> None:
    """h += scale * delta (float32, in place; ``scale`` float32 [d], one factor a feature);
    out = h / sqrt(mean(h^2) + eps) * weight.  With ``rows`` only those rows are read, ``out[i]`` gets row
    ``rows[i]`` and ``h`` is left as it is.  ``out`` may be None when only the sum is wanted."""
    _need(h.dtype == torch.float32 and h.dim() == 2 and h.is_contiguous() and h.is_cuda,
          "add_scaled_rmsnorm: h must be contiguous float32 [T, d]")
    T, d = h.shape
    _need(delta.shape == h.shape and delta.is_contiguous(), "add_scaled_rmsnorm: delta must be contiguous [T, d]")
    for name, vector in (("scale", scale), ("weight", weight)):
        _need(vector.dtype == torch.float32 and vector.numel() == d and vector.is_contiguous() and vector.is_cuda,
              f"add_scaled_rmsnorm: {name} must be float32 [d] on the GPU")
    n_rows = T
    if rows is not None:
        _i32(rows, "rows")
        n_rows = rows.numel()
        _need(out is not None, "add_scaled_rmsnorm: a gather needs somewhere to put its rows")
    if out is not None:
        _need(out.shape == (n_rows, d) and out.is_contiguous(), "add_scaled_rmsnorm: out must be contiguous [rows, d]")
    _check(_fn("common", "mi_add_scaled_rmsnorm")(
        _p(h), _p(delta), _dt(delta), _p(scale), _p(weight), float(eps), _p(out),
        _dt(out) if out is not None else DT_F32, _p(rows), n_rows, d, _stream()), "add_scaled_rmsnorm", f"(d={d})")


def polynorm(z: torch.Tensor, coefficients: torch.Tensor, eps: float, out: torch.Tensor) -> None:
    """out = c0 z/rms(z) + c1 z^2/rms(z^2) + c2 z^3/rms(z^3) + c3 row by row, rms(x) = sqrt(mean(x^2) + eps)
    over the row; ``coefficients`` float32 [4]."""
    ld = _row_major(z, "z")
    out_ld = _row_major(out, "out")
    _need(out.shape == z.shape and out.dtype == z.dtype, "polynorm: out must have the input's shape and dtype")
    _need(coefficients.dtype == torch.float32 and coefficients.numel() == 4 and coefficients.is_cuda
          and coefficients.is_contiguous(), "polynorm: coefficients must be float32 [4] on the GPU")
    _check(_fn("common", "mi_polynorm")(_p(z), _dt(z), ld, _p(coefficients), float(eps), _p(out), out_ld, z.shape[0],
                                        z.shape[1], _stream()), "polynorm")


# --------------------------------------------------------------------------- bigram embedding, layer norm, clamped GLU
def embed_bigram(token_ids: torch.Tensor, table: torch.Tensor, multiplier: float, bigram: torch.Tensor, buckets: int,
                 mul_prev: int, mul_cur: int, positions: torch.Tensor, lane_of_token: torch.Tensor,
                 cu_seqlens: torch.Tensor, slot_ids: torch.Tensor, previous: torch.Tensor, out: torch.Tensor) -> None:
    """out[t] = table[token] * multiplier + bigram[row]: row = (token before * mul_prev + token * mul_cur) mod
    ``buckets``, or ``buckets`` (the table's last row) at position 0.  The token before a lane's first one is
    ``previous[slot of the lane]`` (int32 [slots, 1]); a second launch then leaves the lane's last token there."""
    T, d = out.shape
    for name, tensor in (("token_ids", token_ids), ("positions", positions), ("lane_of_token", lane_of_token),
                         ("cu_seqlens", cu_seqlens), ("slot_ids", slot_ids), ("previous", previous)):
        _i32(tensor, name)
    lanes = slot_ids.numel()
    _need(token_ids.numel() == T and positions.numel() == T and lane_of_token.numel() == T
          and cu_seqlens.numel() == lanes + 1, "embed_bigram: the step's arrays do not fit its tokens and lanes")
    _need(table.dim() == 2 and table.shape[1] == d and table.is_contiguous() and bigram.shape == (buckets + 1, d)
          and bigram.is_contiguous() and bigram.dtype == table.dtype, "embed_bigram: tables do not fit")
    _need(out.dtype == torch.float32 and out.is_contiguous(), "embed_bigram: out must be contiguous float32")
    _check(_fn("common", "mi_embed_bigram")(
        _p(token_ids), _p(table), _dt(table), float(multiplier), _p(bigram), int(buckets), int(mul_prev), int(mul_cur),
        _p(positions), _p(lane_of_token), _p(cu_seqlens), _p(slot_ids), _p(previous), _p(out), T, d, lanes, _stream()),
        "embed_bigram")


def stream_add(h: torch.Tensor, rows: Optional[torch.Tensor], factor: float, vector: Optional[torch.Tensor]) -> None:
    """h += factor * rows (+ vector on every row), in float32, in place."""
    _need(h.dtype == torch.float32 and h.dim() == 2 and h.is_contiguous() and h.is_cuda,
          "stream_add: h must be contiguous float32 [T, d]")
    T, d = h.shape
    _need(rows is None or (rows.shape == h.shape and rows.is_contiguous()), "stream_add: rows must be contiguous [T, d]")
    _need(vector is None or (vector.dtype == torch.float32 and vector.numel() == d and vector.is_contiguous()),
          "stream_add: the vector must be float32 [d]")
    if rows is None and vector is None:
        return
    _check(_fn("common", "mi_stream_add")(_p(h), _p(rows), _dt(rows) if rows is not None else DT_F32, float(factor),
                                          _p(vector), T, d, _stream()), "stream_add")


NORMED_SUM_MOST = 4          # branches that ``normed_sum`` takes in one launch


def normed_sum(branches: Sequence[tuple], out: torch.Tensor) -> None:
    """out = sum over ``branches`` [(rows [T, d], factor, weight float32 [d], eps)], in their order, of
    factor * rows / sqrt(mean(rows^2) + eps) * weight, float32: every branch through an RMS norm of its own."""
    _need(0 < len(branches) <= NORMED_SUM_MOST, f"normed_sum: one to {NORMED_SUM_MOST} branches")
    _need(out.dtype == torch.float32 and out.dim() == 2 and out.is_contiguous() and out.is_cuda,
          "normed_sum: out must be contiguous float32 [T, d]")
    T, d = out.shape
    count = len(branches)
    rows = (ctypes.c_void_p * count)()
    weights = (ctypes.c_void_p * count)()
    dtypes = (ctypes.c_int * count)()
    lds = (ctypes.c_long * count)()
    factors = (ctypes.c_float * count)()
    epsilons = (ctypes.c_float * count)()
    for index, (tensor, factor, weight, eps) in enumerate(branches):
        lds[index] = _row_major(tensor, "a branch")
        _need(tensor.shape == (T, d), "normed_sum: branches must be [T, d]")
        _need(weight.dtype == torch.float32 and weight.numel() == d and weight.is_contiguous() and weight.is_cuda,
              "normed_sum: a weight must be float32 [d] on the GPU")
        rows[index], weights[index], dtypes[index] = tensor.data_ptr(), weight.data_ptr(), _dt(tensor)
        factors[index], epsilons[index] = float(factor), float(eps)
    _check(_fn("common", "mi_normed_sum")(rows, dtypes, lds, weights, factors, epsilons, count, _p(out), T, d, _stream()),
           "normed_sum")


def add_layernorm(h: torch.Tensor, branches: Sequence[tuple], vector: Optional[torch.Tensor],
                  weight: Optional[torch.Tensor], bias: Optional[torch.Tensor], eps: float, out: Optional[torch.Tensor],
                  rows: Optional[torch.Tensor] = None, branch_norm: Optional[tuple] = None) -> None:
    """h += sum of factor * branch over ``branches`` [(tensor [T, d], factor)] (at most three) + ``vector`` [d]
    (float32, in place); out = (h - mean) / sqrt(variance + eps) * weight + bias, statistics in float32, the
    variance from the deviations.  With ``rows`` only those rows are read, ``out[i]`` gets row ``rows[i]`` and
    ``h`` is left as it is.  ``branch_norm`` (weight, bias, eps): the branches' weighted sum goes through a layer
    norm of its own before it is added, h += LN(sum) * weight + bias.  Without ``out`` nothing is normed behind
    the add, and ``weight`` and ``bias`` may be None."""
    _need(h.dtype == torch.float32 and h.dim() == 2 and h.is_contiguous() and h.is_cuda,
          "add_layernorm: h must be contiguous float32 [T, d]")
    T, d = h.shape
    _need(len(branches) <= 3, "add_layernorm: at most three branches")
    for tensor, _ in branches:
        _need(tensor.shape == h.shape and tensor.is_contiguous(), "add_layernorm: branches must be contiguous [T, d]")
    named = [("weight", weight), ("bias", bias)] if out is not None or weight is not None else []
    if branch_norm is not None:
        _need(rows is None and len(branches) > 0, "add_layernorm: a norm on the branches needs branches and all rows")
        named += [("the branches' weight", branch_norm[0]), ("the branches' bias", branch_norm[1])]
    for name, one in named:
        _need(one is not None and one.dtype == torch.float32 and one.numel() == d and one.is_contiguous(),
              f"add_layernorm: {name} must be float32 [d]")
    _need(vector is None or (vector.dtype == torch.float32 and vector.numel() == d and vector.is_contiguous()),
          "add_layernorm: the vector must be float32 [d]")
    n_rows = T
    if rows is not None:
        _i32(rows, "rows")
        n_rows = rows.numel()
        _need(out is not None, "add_layernorm: a gather needs somewhere to put its rows")
    if out is not None:
        _need(out.shape == (n_rows, d) and out.is_contiguous(), "add_layernorm: out must be contiguous [rows, d]")
    if n_rows == 0:
        return
    flat = []
    for index in range(3):
        if index < len(branches):
            tensor, factor = branches[index]
            flat += [_p(tensor), _dt(tensor), float(factor)]
        else:
            flat += [None, DT_F32, 0.0]
    post = branch_norm if branch_norm is not None else (None, None, 0.0)
    _check(_fn("common", "mi_add_layernorm")(
        _p(h), *flat, _p(vector), _p(weight), _p(bias), float(eps), _p(post[0]), _p(post[1]), float(post[2]), _p(out),
        _dt(out) if out is not None else DT_F32, _p(rows), n_rows, d, _stream()), "add_layernorm", f"(d={d})")


def clamped_glu(gate_up: torch.Tensor, limit: float, alpha: float, up_offset: float, out: torch.Tensor) -> None:
    """out = g * sigmoid(alpha g) * (u + up_offset) with g = min(gate, limit), u = clamp(up, -limit, limit); a row of
    ``gate_up`` holds [gate | up]."""
    ld = _row_major(gate_up, "gate_up")
    out_ld = _row_major(out, "out")
    T, two_i = gate_up.shape
    _need(two_i % 2 == 0 and out.shape == (T, two_i // 2) and out.dtype == gate_up.dtype,
          "clamped_glu: out must be [T, I] of the input's dtype")
    _check(_fn("common", "mi_clamped_glu")(_p(gate_up), _dt(gate_up), ld, _p(out), out_ld, T, two_i // 2, float(limit),
                                           float(alpha), float(up_offset), _stream()), "clamped_glu")


# --------------------------------------------------------------------------- latent attention
def latent_prepare(down: torch.Tensor, q_rank: int, kv_rank: int, rope_dim: int, q_norm: Optional[torch.Tensor],
                   kv_norm: torch.Tensor, eps: float, positions: torch.Tensor, inv_freq: Optional[torch.Tensor],
                   rotary_dim: int, interleaved: bool, slot_mapping: Optional[torch.Tensor],
                   k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                   query_latent: Optional[torch.Tensor]) -> None:
    """From a token's down-projected row [query latent | key/value latent | key part to turn]: the query latent's
    RMS norm (times ``q_norm``) into ``query_latent``; the key/value latent's RMS norm (times ``kv_norm``) and the
    key part, its first ``rotary_dim`` dimensions turned by the token's position, into the token's cache cell: K
    pages [pages, 1, page_size, kv_rank + rope_dim] get [latent | turned part], V pages [pages, 1, kv_rank,
    page_size] the latent.  Norms, angles and the turn are float32.  Without ``slot_mapping`` nothing is stored."""
    ld = _row_major(down, "down")
    T = down.shape[0]
    _need(down.shape[1] >= q_rank + kv_rank + rope_dim, "latent_prepare: the projected rows are too narrow")
    _i32(positions, "positions")
    _need(positions.numel() == T, "latent_prepare: one position per token")
    _need(q_rank >= 0 and (q_rank > 0) == (q_norm is not None) == (query_latent is not None),
          "latent_prepare: a query latent comes with its norm and its place, or not at all")
    for name, vector, size in (("q_norm", q_norm, q_rank), ("kv_norm", kv_norm, kv_rank)):
        if vector is None:
            continue
        _need(vector.dtype == torch.float32 and vector.numel() == size and vector.is_contiguous() and vector.is_cuda,
              f"latent_prepare: {name} must be float32 [{size}] on the GPU")
    turned = int(rotary_dim) if inv_freq is not None else 0
    _need(turned % 2 == 0 and turned <= rope_dim, "latent_prepare: the turned dimensions are pairs within the key part")
    if inv_freq is not None:
        _need(inv_freq.dtype == torch.float32 and inv_freq.numel() == turned // 2 and inv_freq.is_cuda,
              "latent_prepare: inv_freq must be float32 [rotary_dim / 2]")
    q_ld = 0
    if query_latent is not None:
        q_ld = _row_major(query_latent, "query_latent")
        _need(query_latent.shape == (T, q_rank) and query_latent.dtype == down.dtype,
              "latent_prepare: query_latent must be [T, q_rank]")
    page_stride, page_size = 0, 0
    if slot_mapping is not None:
        _i32(slot_mapping, "slot_mapping")
        _need(slot_mapping.numel() == T, "latent_prepare: one cache cell per token")
        page_stride, page_size = _cache_view(k_cache, v_cache, 1, kv_rank + rope_dim, down.dtype, kv_rank)
    _check(_fn("latent", "mi_latent_prepare")(
        _p(down), _dt(down), ld, T, q_rank, kv_rank, rope_dim, _p(q_norm), _p(kv_norm), float(eps), _p(positions),
        _p(inv_freq), turned, 1 if interleaved else 0, _p(slot_mapping),
        _p(k_cache) if slot_mapping is not None else None, _p(v_cache) if slot_mapping is not None else None,
        page_stride, page_size, _p(query_latent), q_ld, _stream()), "latent_prepare")


def rotate_heads(x: torch.Tensor, col: int, head_stride: int, num_heads: int, width: int, positions: torch.Tensor,
                 inv_freq: Optional[torch.Tensor], rotary_dim: int, interleaved: bool, out: torch.Tensor, out_col: int,
                 out_head_stride: int) -> None:
    """out[t, out_col + h * out_head_stride + j] = the turned x[t, col + h * head_stride + j], j below ``width``: the
    first ``rotary_dim`` of the ``width`` dimensions turned in pairs by the token's position, the rest copied."""
    ld = _row_major(x, "x")
    out_ld = _row_major(out, "out")
    T = x.shape[0]
    _i32(positions, "positions")
    turned = int(rotary_dim) if inv_freq is not None else 0
    _need(out.shape[0] == T and positions.numel() == T and out.dtype == x.dtype and turned % 2 == 0 and turned <= width
          and col + (num_heads - 1) * head_stride + width <= x.shape[1]
          and out_col + (num_heads - 1) * out_head_stride + width <= out.shape[1], "rotate_heads: shapes do not fit")
    if inv_freq is not None:
        _need(inv_freq.dtype == torch.float32 and inv_freq.numel() == turned // 2 and inv_freq.is_cuda,
              "rotate_heads: inv_freq must be float32 [rotary_dim / 2]")
    _check(_fn("latent", "mi_rotate_heads")(
        _p(x), _dt(x), ld, int(col), int(head_stride), num_heads, width, _p(positions), _p(inv_freq), turned,
        1 if interleaved else 0, _p(out), out_ld, int(out_col), int(out_head_stride), T, _stream()), "rotate_heads")


def head_linear(x: torch.Tensor, x_col: int, x_head_stride: int, weight: torch.Tensor, out: torch.Tensor, out_col: int,
                out_head_stride: int) -> None:
    """One product per head: out[:, out_col + h * out_head_stride : + N] = x[:, x_col + h * x_head_stride : + K] .
    weight[h]^T, ``weight`` [heads, N, K], float32 sums on the matrix cores (float32 operands: true 32-bit)."""
    ldx = _row_major(x, "x")
    ldo = _row_major(out, "out")
    _need(weight.dim() == 3 and weight.is_contiguous() and weight.is_cuda, "head_linear: weight must be contiguous [heads, N, K]")
    heads, N, K = weight.shape
    T = x.shape[0]
    _need(out.shape[0] == T and x_col + (heads - 1) * x_head_stride + K <= x.shape[1]
          and out_col + (heads - 1) * out_head_stride + N <= out.shape[1], "head_linear: shapes do not fit")
    rows = x if x.dtype == weight.dtype else x.to(weight.dtype)
    target = out if out.dtype == weight.dtype else torch.empty(out.shape, dtype=weight.dtype, device=out.device)
    if rows is not x:
        ldx = _row_major(rows, "x")
    if target is not out:
        ldo = _row_major(target, "out")
    _check(_fn("latent", "mi_head_gemm")(
        _p(rows), _dt(rows), ldx, int(x_col), _p(weight), int(x_head_stride), int(out_head_stride), _p(target), ldo,
        int(out_col), T, N, K, heads, _stream()), "head_linear", f"(N={N}, K={K})")
    if target is not out:
        width = (heads - 1) * out_head_stride + N
        out[:, out_col:out_col + width] = target[:, out_col:out_col + width].to(out.dtype)


def latent_attention_supported(dtype, num_heads: int, kv_rank: int, rope_dim: int, page_size: int) -> bool:
    """Whether the matrix-core kernel for prompt portions of latent attention covers this geometry."""
    return (dtype == torch.bfloat16 and page_size % 4 == 0
            and bool(_fn("latent", "mi_latent_attention_supported")(int(kv_rank), int(rope_dim))))


def latent_attention(q: torch.Tensor, num_heads: int, kv_rank: int, rope_dim: int, k_cache: torch.Tensor,
                     v_cache: torch.Tensor, block_tables: torch.Tensor, query_tiles: torch.Tensor, cu_seqlens: torch.Tensor,
                     start_pos: torch.Tensor, scale: float, window: Optional[int], out: torch.Tensor) -> None:
    """Causal attention of prompt portions over cached latent rows on the matrix cores (bfloat16, online softmax in
    float32).  ``q`` [T, heads * (kv_rank + rope_dim)]: every head's query in the latent space beside its turned
    part; K pages [pages, 1, page_size, kv_rank + rope_dim], V pages [pages, 1, kv_rank, page_size];
    ``query_tiles`` [tiles, 2]: (lane, first token row) of runs of up to 64 tokens of one lane; the step's own rows
    must be in the cache already.  ``out`` [T, heads * kv_rank]: the attended latents."""
    q_ld = _row_major(q, "q")
    out_ld = _row_major(out, "out")
    T = q.shape[0]
    width = kv_rank + rope_dim
    _need(q.dtype == torch.bfloat16 and out.dtype == torch.bfloat16, "latent_attention: bfloat16 only")
    _need(q.shape[1] >= num_heads * width and out.shape == (T, num_heads * kv_rank) and q_ld % 8 == 0
          and q.data_ptr() % 16 == 0 and out_ld % 4 == 0 and out.data_ptr() % 8 == 0,
          "latent_attention: q/out shapes or alignment do not fit")
    page_stride, page_size = _cache_view(k_cache, v_cache, 1, width, q.dtype, kv_rank)
    _need(latent_attention_supported(q.dtype, num_heads, kv_rank, rope_dim, page_size),
          "latent_attention: geometry not covered; use paged_attention")
    for name, tensor in (("block_tables", block_tables), ("query_tiles", query_tiles), ("cu_seqlens", cu_seqlens),
                         ("start_pos", start_pos)):
        _i32(tensor, name)
    _need(block_tables.dim() == 2 and query_tiles.dim() == 2 and query_tiles.shape[1] == 2
          and cu_seqlens.numel() == start_pos.numel() + 1, "latent_attention: metadata shapes do not match")
    _check(_fn("latent", "mi_latent_attention")(
        _p(q), q_ld, num_heads, kv_rank, rope_dim, _p(k_cache), _p(v_cache), page_stride, page_size, _p(block_tables),
        block_tables.shape[1], _p(query_tiles), query_tiles.shape[0], _p(cu_seqlens), _p(start_pos), float(scale),
        int(window or 0), _p(out), out_ld, _stream()), "latent_attention")


def latent_decode_attention(q: torch.Tensor, num_heads: int, kv_rank: int, rope_dim: int, k_cache: torch.Tensor,
                            v_cache: torch.Tensor, block_tables: torch.Tensor, lane_of_token: torch.Tensor,
                            positions: torch.Tensor, scale: float, window: Optional[int], max_seq_len: int,
                            out: torch.Tensor) -> None:
    """``latent_attention`` for steps of single decoded tokens: a request's context is split over many waves, and
    the heads, which all read the same cached rows, are the columns of the matrix cores' products.
    ``max_seq_len``: an upper bound of the longest context in the step."""
    q_ld = _row_major(q, "q")
    out_ld = _row_major(out, "out")
    T = q.shape[0]
    width = kv_rank + rope_dim
    _need(q.dtype == torch.bfloat16 and out.dtype == torch.bfloat16, "latent_decode_attention: bfloat16 only")
    _need(q.shape[1] >= num_heads * width and out.shape == (T, num_heads * kv_rank) and q_ld % 8 == 0
          and q.data_ptr() % 16 == 0, "latent_decode_attention: q/out shapes or alignment do not fit")
    page_stride, page_size = _cache_view(k_cache, v_cache, 1, width, q.dtype, kv_rank)
    _need(latent_attention_supported(q.dtype, num_heads, kv_rank, rope_dim, page_size),
          "latent_decode_attention: geometry not covered; use paged_attention")
    _i32(block_tables, "block_tables")
    _i32(lane_of_token, "lane_of_token")
    _i32(positions, "positions")
    _need(block_tables.dim() == 2 and lane_of_token.numel() == T and positions.numel() == T,
          "latent_decode_attention: metadata shapes do not match")
    holds = block_tables.shape[1] * page_size
    span = max(1, min(int(max_seq_len), holds)) if max_seq_len else holds
    if window:
        span = min(span, int(window) + 32)
    # runs of 64 keys while that leaves the step a few thousand waves, longer ones beyond; at most 256 runs a request
    split_keys = 64
    while (split_keys < 1024 and T * -(-span // split_keys) > 4096) or -(-span // split_keys) + 1 > 256:
        split_keys *= 2
    splits = max(1, -(-span // split_keys) + (1 if window else 0))
    partial_o = torch.empty((T, num_heads, splits, kv_rank), dtype=torch.float32, device=q.device)
    partial_ml = torch.empty((T, num_heads, splits, 2), dtype=torch.float32, device=q.device)
    _check(_fn("latent", "mi_latent_decode_attention")(
        _p(q), q_ld, T, num_heads, kv_rank, rope_dim, _p(k_cache), _p(v_cache), page_stride, page_size, _p(block_tables),
        block_tables.shape[1], _p(lane_of_token), _p(positions), float(scale), int(window or 0), split_keys, splits,
        _p(partial_o), _p(partial_ml), _p(out), out_ld, _stream()), "latent_decode_attention")


# --------------------------------------------------------------------------- routed experts
MOE_TILE_ROWS = 16          # places of a tile of the grouped products: steps of few rows
MOE_WIDE_TILE_ROWS = 64     # steps whose experts get 64 rows or more each on average
MOE_WIDEST_TILE_ROWS = 128  # and 256 or more, if rows and matrices are whole 16-byte pieces (``whole_pieces``)


def moe_tile_rows(tokens: int, top_k: int, num_experts: int, whole_pieces: bool = False) -> int:
    """The tile of the grouped products for a step: it depends on the step's size alone, never on its tokens."""
    if whole_pieces and tokens * top_k >= 2 * MOE_WIDEST_TILE_ROWS * num_experts:
        return MOE_WIDEST_TILE_ROWS
    return MOE_WIDE_TILE_ROWS if tokens * top_k >= MOE_WIDE_TILE_ROWS * num_experts else MOE_TILE_ROWS


def moe_route(logits: torch.Tensor, num_experts: int, top_k: int, correction: torch.Tensor, scale: float, eps: float,
              shared_gate: bool, routing: str = "softmax_then_top"):
    """From float32 router logits [T, >= num_experts (+ 1)]: s = softmax over the experts; the ``top_k`` largest of
    s + correction (ties to the lower number) are the token's experts (int32 [T, top_k]), their weights (float32
    [T, top_k]) s / (sum of the chosen s + eps) * scale; with ``shared_gate`` also sigmoid of column
    ``num_experts`` (float32 [T]), else None.  ``routing`` "top_then_softmax": the ``top_k`` largest of
    logits + correction (the correction is then a bias of the logits) are chosen, and their weights are the softmax
    over these alone, times scale."""
    _need(routing in ("softmax_then_top", "top_then_softmax"), f"moe_route: routing {routing!r} is not known")
    ld = _row_major(logits, "logits")
    T = logits.shape[0]
    _need(logits.dtype == torch.float32 and logits.shape[1] >= num_experts + (1 if shared_gate else 0),
          "moe_route: float32 logits of every expert")
    _need(correction.dtype == torch.float32 and correction.numel() == num_experts and correction.is_cuda,
          "moe_route: the correction must be float32 [experts] on the GPU")
    _need(0 < top_k <= num_experts, "moe_route: a token uses at least one and at most all experts")
    chosen = torch.empty((T, top_k), dtype=torch.int32, device=logits.device)
    weights = torch.empty((T, top_k), dtype=torch.float32, device=logits.device)
    gate = torch.empty((T,), dtype=torch.float32, device=logits.device) if shared_gate else None
    _check(_fn("moe", "mi_moe_route")(_p(logits), ld, T, num_experts, top_k, _p(correction), float(scale), float(eps),
                                      0 if routing == "softmax_then_top" else 1, _p(chosen), _p(weights), _p(gate),
                                      _stream()), "moe_route", f"(experts={num_experts})")
    return chosen, weights, gate


class MoePlan:
    """The rows of a step grouped by expert, on the device: ``source`` int32 [capacity] = the token whose row
    stands at a place (-1: padding), ``place`` int32 [T * top_k] = where a token's choice stands, ``tile_expert``
    int32 [capacity / pad] = the expert of every tile of ``pad`` places (-1: an unused tile).  Every expert's rows
    start a tile; ``capacity`` depends on the number of tokens alone."""

    def __init__(self, chosen: torch.Tensor, num_experts: int, pad: Optional[int] = None):
        _i32(chosen, "chosen")
        tokens, top_k = chosen.shape
        pad = moe_tile_rows(tokens, top_k, num_experts) if pad is None else int(pad)
        self.pad, self.tokens, self.top_k = pad, tokens, top_k
        self.capacity = -(-(tokens * top_k + num_experts * (pad - 1)) // pad) * pad
        device = chosen.device
        self.source = torch.empty((self.capacity,), dtype=torch.int32, device=device)
        self.place = torch.empty((tokens * top_k,), dtype=torch.int32, device=device)
        self.tile_expert = torch.empty((self.capacity // pad,), dtype=torch.int32, device=device)
        ranks = torch.empty((tokens * top_k,), dtype=torch.int32, device=device)
        _check(_fn("moe", "mi_moe_plan")(_p(chosen), tokens * top_k, top_k, num_experts, pad, self.capacity,
                                         _p(self.source), _p(self.place), _p(self.tile_expert), _p(ranks), _stream()),
               "moe_plan", f"(experts={num_experts})")


def moe_plan(chosen: torch.Tensor, num_experts: int, pad: Optional[int] = None) -> MoePlan:
    return MoePlan(chosen, num_experts, pad)


def moe_expert_gemm(x: torch.Tensor, plan: MoePlan, weight: torch.Tensor, out: torch.Tensor, gather: bool, glu,
                    squared_relu: bool = False) -> None:
    """The grouped product of a plan's rows with their experts' matrices ``weight`` [experts, N, K]: the row at a
    place is ``x[source[place]]`` (``gather``) or ``x[place]``; out[place] = weight[expert] . row, or with ``glu``
    (limit, alpha, up_offset; N = 2 I, gate rows then up rows) the clamped gated activation of the two halves,
    [capacity, I]; or with ``squared_relu`` max(weight[expert] . row, 0)^2.  Float32 sums on the matrix cores;
    float32 operands give a true 32-bit product."""
    _need(not (squared_relu and glu is not None), "moe_expert_gemm: one activation")
    ldx = _row_major(x, "x")
    ldo = _row_major(out, "out")
    _need(weight.dim() == 3 and weight.is_contiguous() and weight.is_cuda and x.dtype == weight.dtype,
          "moe_expert_gemm: weight must be contiguous [experts, N, K] of the rows' dtype")
    experts, N, K = weight.shape
    width = N // 2 if glu is not None else N
    _need(x.shape[1] == K and out.shape == (plan.capacity, width) and (gather or x.shape[0] == plan.capacity)
          and (not gather or x.shape[0] == plan.tokens), "moe_expert_gemm: shapes do not fit the plan")
    _check(_fn("moe", "mi_moe_expert_gemm")(
        _p(x), _dt(x), ldx, x.shape[0], _p(weight), N * K, K, N, K, _p(plan.source), _p(plan.tile_expert),
        plan.tile_expert.numel(), plan.pad, 1 if gather else 0, 1 if glu is not None else (2 if squared_relu else 0),
        float(glu.limit) if glu is not None else 0.0, float(glu.alpha) if glu is not None else 0.0,
        float(glu.up_offset) if glu is not None else 0.0, _p(out), _dt(out), ldo, _stream()),
        "moe_expert_gemm", f"(N={N}, K={K})")


def moe_combine(down: torch.Tensor, plan: MoePlan, weights: torch.Tensor, shared_rows: Optional[torch.Tensor],
                shared_gate: Optional[torch.Tensor], out: torch.Tensor) -> None:
    """out[t] = sum over the token's choices k, in their order, of weights[t, k] * down[place[t, k]]
    (+ shared_gate[t] * shared_rows[t]), float32."""
    T, d = out.shape
    ld = _row_major(down, "down")
    _need(down.dtype == torch.float32 and out.dtype == torch.float32 and out.is_contiguous() and down.shape[1] == d
          and weights.dtype == torch.float32 and weights.shape == (T, plan.top_k) and weights.is_contiguous()
          and T == plan.tokens, "moe_combine: shapes do not fit the plan")
    shared_ld = 0
    if shared_rows is not None:
        shared_ld = _row_major(shared_rows, "shared_rows")
        _need(shared_rows.shape == (T, d) and shared_gate is not None and shared_gate.dtype == torch.float32
              and shared_gate.numel() == T, "moe_combine: the shared rows and their gate do not fit")
    _check(_fn("moe", "mi_moe_combine")(
        _p(down), ld, _p(plan.place), _p(weights), plan.top_k, _p(shared_rows),
        _dt(shared_rows) if shared_rows is not None else DT_F32, shared_ld, _p(shared_gate), _p(out), T, d, _stream()),
        "moe_combine")


# --------------------------------------------------------------------------- mixers with a matrix-valued state
def tanh_rows(x: torch.Tensor, out: torch.Tensor) -> None:
    """out = tanh(x) for a block of columns (``x`` may be a column view of a wider matrix)."""
    ld = _row_major(x, "x")
    out_ld = _row_major(out, "out")
    _need(out.shape == x.shape and out.dtype == x.dtype, "tanh_rows: out must have the input's shape and dtype")
    _check(_fn("linear_state", "mi_tanh_rows")(_p(x), _dt(x), ld, _p(out), out_ld, x.shape[0], x.shape[1], _stream()),
           "tanh_rows")


def head_norm_gate(raw: torch.Tensor, gate: torch.Tensor, weight: Optional[torch.Tensor], num_heads: int, eps: float,
                   activation: str, out: torch.Tensor) -> None:
    """out[t, head] = raw[t, head] / rms(raw[t, head]) (* weight) * act(gate[t, head]) with rms over the head's
    columns and act "silu" or "sigmoid".  ``raw`` float32 [T, H * dv]; ``gate`` and ``out`` [T, H * dv] of the
    activation dtype (column views allowed); ``weight`` float32 [H * dv] or None."""
    raw_ld = _row_major(raw, "raw")
    gate_ld = _row_major(gate, "gate")
    out_ld = _row_major(out, "out")
    T, width = raw.shape
    _need(raw.dtype == torch.float32 and width % num_heads == 0 and gate.shape == raw.shape and out.shape == raw.shape
          and gate.dtype == out.dtype, "head_norm_gate: shapes or dtypes do not match")
    _need(weight is None or (weight.dtype == torch.float32 and weight.numel() == width and weight.is_contiguous()
                             and weight.is_cuda), "head_norm_gate: weight must be float32 [H * dv] on the GPU")
    _need(activation in ("silu", "sigmoid"), "head_norm_gate: the gate's activation is 'silu' or 'sigmoid'")
    _check(_fn("linear_state", "mi_head_norm_gate")(
        _p(raw), raw_ld, _p(gate), _dt(gate), gate_ld, _p(weight), num_heads, width // num_heads, float(eps),
        0 if activation == "silu" else 1, _p(out), out_ld, T, _stream()), "head_norm_gate")


def linear_state_scan(u: torch.Tensor, *, q_col: int, k_col: int, v_col: int, num_heads: int, key_dim: int,
                      value_dim: int, state: torch.Tensor, cu_seqlens: torch.Tensor, slot_ids: torch.Tensor,
                      out: torch.Tensor, max_query_len: int = 0, head_decay: Optional[torch.Tensor] = None,
                      key_scale: float = 1.0, positions: Optional[torch.Tensor] = None,
                      inv_freq: Optional[torch.Tensor] = None, rotary_dim: int = 0, removal_col: int = -1,
                      decay_logits: Optional[torch.Tensor] = None, decay_bias: Optional[torch.Tensor] = None,
                      decay_floor: float = 0.0, key_eps: float = 0.0, chunks=None, gate_power: float = 0.0,
                      query_scale: float = 1.0) -> None:
    """The scan of a mixer whose state is a matrix per head, from and into ``state`` [slots, H, dv, dk] (float32, the
    state of a head transposed), for every lane of the step from its slot; ``out`` float32 [T, H * dv] = S^T q.

    ``u`` [T, ...]: the projection's rows with q heads at ``q_col``, k heads at ``k_col`` (H * dk columns each) and
    v heads at ``v_col`` (H * dv).  Retention (``head_decay`` float32 [H]): S <- decay S + k v^T after q and k were
    turned by ``positions`` (``inv_freq``, ``rotary_dim``; None: no rotation) and k multiplied by ``key_scale``.
    Delta rule (``removal_col`` >= 0: the columns of the removal rate's logits; ``decay_logits`` float32 [T, H * dk],
    ``decay_bias`` float32 [H * dk]): w = exp(-decay_floor * sigmoid(logits + bias)), a = sigmoid(removal),
    u = k / sqrt(sum k^2 + key_eps), S <- diag(w) S - (a u)(u^T S) + k v^T.  Gated decay (``gate_power`` > 0, no
    removal; ``decay_logits`` and ``decay_bias`` as above): w = sigmoid(logits + bias)^gate_power per head and key
    channel, S <- diag(w) S + k v^T.  ``query_scale`` multiplies q.  ``max_query_len``: the longest lane
    (1 picks small workgroups; 0: not known).  ``chunks`` (a table of the step's lanes cut into chunks: ``chunks``
    int32 [n, 4], ``lane_chunks`` int32 [lanes, 2], ``num_chunks``, ``chunk_size``): the scan runs chunk by chunk in
    three passes (the chunks' own states and transitions side by side, the carry from chunk to chunk, the outputs
    side by side), the same sums in another order: for long portions."""
    ld = _row_major(u, "u")
    T = u.shape[0]
    H, dk, dv = int(num_heads), int(key_dim), int(value_dim)
    delta = removal_col >= 0
    gated = not delta and gate_power > 0
    widest = max(q_col + H * dk, k_col + H * dk, v_col + H * dv, removal_col + H * dk if delta else 0)
    _need(min(q_col, k_col, v_col) >= 0 and u.shape[1] >= widest, "linear_state_scan: u is too narrow for its columns")
    _need(state.dtype == torch.float32 and state.dim() == 4 and state.shape[1:] == (H, dv, dk) and state.is_contiguous()
          and state.is_cuda, "linear_state_scan: state must be contiguous float32 [slots, H, dv, dk] on the GPU")
    _i32(cu_seqlens, "cu_seqlens")
    _i32(slot_ids, "slot_ids")
    lanes = slot_ids.numel()
    _need(cu_seqlens.numel() == lanes + 1, "linear_state_scan: one offset more than lanes")
    _need(out.dtype == torch.float32 and out.shape == (T, H * dv) and out.is_contiguous(),
          "linear_state_scan: out must be contiguous float32 [T, H * dv]")
    logits_ld = 0
    if delta or gated:
        _need(decay_logits is not None and decay_logits.dtype == torch.float32 and decay_logits.shape == (T, H * dk),
              "linear_state_scan: decay_logits must be float32 [T, H * dk]")
        logits_ld = _row_major(decay_logits, "decay_logits")
        _need(decay_bias is not None and decay_bias.dtype == torch.float32 and decay_bias.numel() == H * dk
              and decay_bias.is_contiguous() and decay_bias.is_cuda, "linear_state_scan: decay_bias must be float32 [H * dk]")
    if not delta and not gated:
        _need(head_decay is not None and head_decay.dtype == torch.float32 and head_decay.numel() == H
              and head_decay.is_cuda, "linear_state_scan: head_decay must be float32 [H] on the GPU")
    if inv_freq is not None:
        _i32(positions, "positions")
        _need(positions.numel() == T and inv_freq.dtype == torch.float32 and inv_freq.numel() == rotary_dim // 2
              and inv_freq.is_cuda and 0 < rotary_dim <= dk, "linear_state_scan: the rotation does not fit the heads")
    if chunks is not None:
        _i32(chunks.chunks, "chunks")
        _i32(chunks.lane_chunks, "lane_chunks")
        count = int(chunks.num_chunks)
        _need(chunks.chunks.numel() >= 4 * count and chunks.lane_chunks.numel() >= 2 * lanes and count > 0,
              "linear_state_scan: the chunk table does not cover the step")
        floats = _fn("linear_state", "mi_linear_state_local_floats", _c_long)(count, H, dk, dv, 1 if delta else 2 if gated else 0)
        local = torch.empty((floats,), dtype=torch.float32, device=u.device)
        start = torch.empty((_fn("linear_state", "mi_linear_state_start_floats", _c_long)(count, H, dk, dv),),
                            dtype=torch.float32, device=u.device)
        _check(_fn("linear_state", "mi_linear_state_scan_chunked")(
            _p(u), _dt(u), ld, int(q_col), int(k_col), int(v_col), int(removal_col), H, dk, dv, _p(state),
            _p(cu_seqlens), _p(slot_ids), lanes, _p(out), out.stride(0), int(chunks.chunk_size), _p(head_decay),
            float(key_scale), _p(positions) if inv_freq is not None else None, _p(inv_freq),
            int(rotary_dim) if inv_freq is not None else 0, _p(decay_logits), logits_ld, _p(decay_bias),
            float(decay_floor), float(key_eps), float(gate_power) if gated else 0.0, float(query_scale),
            _p(chunks.chunks), _p(chunks.lane_chunks), count, _p(local), _p(start),
            _stream()), "linear_state_scan_chunked", f"(dk={dk}, dv={dv}, chunks={count})")
        return
    _check(_fn("linear_state", "mi_linear_state_scan")(
        _p(u), _dt(u), ld, int(q_col), int(k_col), int(v_col), int(removal_col), H, dk, dv, _p(state), _p(cu_seqlens),
        _p(slot_ids), lanes, _p(out), out.stride(0), int(max_query_len), _p(head_decay), float(key_scale),
        _p(positions) if inv_freq is not None else None, _p(inv_freq), int(rotary_dim) if inv_freq is not None else 0,
        _p(decay_logits), logits_ld, _p(decay_bias), float(decay_floor), float(key_eps),
        float(gate_power) if gated else 0.0, float(query_scale), _stream()),
        "linear_state_scan", f"(dk={dk}, dv={dv})")


# --------------------------------------------------------------------------- matrix products
SKINNY_ROWS = 16          # steps of up to this many rows take the skinny kernel in ``linear``


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
    M, K = x.shape
    if (M <= SKINNY_ROWS and x.is_cuda and K % 32 == 0 and weight.is_contiguous() and x.stride(1) == 1
            and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and fused_gemm_supported(False, M, K)):
        # a step of a few rows waits for the weights: the skinny kernel streams them once, bias and rounding in
        # its epilogue (the library takes 8 us for such a product where this takes 5)
        out = torch.empty((M, weight.shape[0]), dtype=torch.float32 if keep_float32 else torch.bfloat16, device=x.device)
        fused_gemm(weight, bias, out, x=x)
        return out
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
                  v_cache: Optional[torch.Tensor], value_dim: Optional[int] = None) -> None:
    """Rotate q (in place) and k of every token; store rotated k and raw v into the cache.

    ``qkv`` [T, >= (Hq+Hkv)*dh + Hkv*dv] holds q heads, k heads, v heads (``value_dim`` dv: the width of a value
    head, the keys' if not given).  ``k_cache`` [pages, Hkv,
    page_size, dh] and ``v_cache`` [pages, Hkv, dv, page_size] are one layer's views of the pool;
    ``slot_mapping[t] = page*page_size + offset``.  Without ``slot_mapping`` nothing is stored."""
    ld = _row_major(qkv, "qkv")
    T = qkv.shape[0]
    value_dim = head_dim if value_dim is None else int(value_dim)
    _need(qkv.shape[1] >= (num_heads + num_kv_heads) * head_dim + num_kv_heads * value_dim,
          "rope_kv_store: qkv is too narrow")
    _i32(positions, "positions")
    _need(positions.numel() == T, "rope_kv_store: one position per token")
    if inv_freq is not None:
        _need(inv_freq.dtype == torch.float32 and inv_freq.numel() == rotary_dim // 2 and inv_freq.is_cuda,
              "rope_kv_store: inv_freq must be float32 [rotary_dim/2]")
    page_stride, page_size = 0, 0
    if slot_mapping is not None:
        _i32(slot_mapping, "slot_mapping")
        _need(slot_mapping.numel() == T, "rope_kv_store: one cache cell per token")
        page_stride, page_size = _cache_view(k_cache, v_cache, num_kv_heads, head_dim, qkv.dtype, value_dim)
    _check(_fn("attention", "mi_rope_kv_store")(
        _p(qkv), _dt(qkv), ld, T, num_heads, num_kv_heads, head_dim, value_dim, _p(positions), _p(inv_freq),
        rotary_dim if inv_freq is not None else 0, _p(slot_mapping),
        _p(k_cache) if slot_mapping is not None else None, _p(v_cache) if slot_mapping is not None else None,
        page_stride, page_size, _stream()), "rope_kv_store")


def _cache_view(k_cache, v_cache, num_kv_heads, head_dim, dtype, value_dim=None):
    """K pages are [pages, Hkv, page_size, dh]; V pages are transposed, [pages, Hkv, dv, page_size] (dv the
    width of a value head: ``value_dim``, or the keys')."""
    value_dim = head_dim if value_dim is None else value_dim
    _need(k_cache is not None and v_cache is not None and k_cache.dim() == 4 and v_cache.dim() == 4,
          "k_cache must be [pages, Hkv, page_size, dh] and v_cache [pages, Hkv, dv, page_size]")
    page_size = k_cache.shape[2]
    _need(k_cache.shape[1] == num_kv_heads and k_cache.shape[3] == head_dim
          and v_cache.shape == (k_cache.shape[0], num_kv_heads, value_dim, page_size),
          "k_cache must be [pages, Hkv, page_size, dh] and v_cache [pages, Hkv, dv, page_size]")
    for name, cache, width in (("k_cache", k_cache, head_dim), ("v_cache", v_cache, value_dim)):
        _need(cache.dtype == dtype and cache.is_cuda, f"{name} must be a GPU tensor of the activation dtype")
        _need(cache.stride(3) == 1 and cache.stride(2) == cache.shape[3]
              and cache.stride(1) == page_size * width, f"{name}: a page's block per kv head must be dense")
    _need(k_cache.stride(0) == v_cache.stride(0), "k_cache and v_cache must share a page stride")
    return k_cache.stride(0), page_size


def paged_attention(q: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int,
                    k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                    lane_of_token: torch.Tensor, positions: torch.Tensor, scale: float,
                    window: Optional[int], out: torch.Tensor, max_seq_len: Optional[int] = None,
                    slopes: Optional[torch.Tensor] = None, query_tiles: Optional[torch.Tensor] = None,
                    tile_tokens: int = 0, cu_seqlens: Optional[torch.Tensor] = None,
                    log_bias: Optional[torch.Tensor] = None, sinks: Optional[torch.Tensor] = None,
                    value_dim: Optional[int] = None, head_scales: Optional[torch.Tensor] = None,
                    score_bias: Optional[torch.Tensor] = None, sigmoid: bool = False, keep_first: int = 0,
                    fixed_sink: Optional[float] = None) -> None:
    """Causal attention of every token over its request's cached keys (its own included).

    ``q`` [T, >= Hq*dh] (rotated); ``block_tables`` [lanes, max_pages] page ids by logical
    page; a key at position p is visible to a query at position s when p <= s and, with a
    window w, s - p < w.  ``out`` [T, Hq*dh].  ``max_seq_len``: an upper bound of position + 1 over
    the step's tokens (what the block tables can hold if it is not given); it sizes the launch and
    the work area, never the result.  ``slopes`` (float32 [Hq]): a bias on the scores by distance,
    ``score -= slopes[head] * (s - p)``.  ``query_tiles`` [tiles, 2] = (lane or -1, first token row) of runs of
    up to ``tile_tokens`` tokens of one lane, with ``cu_seqlens`` [lanes + 1]: for steps whose lanes hold several
    tokens, a kernel that fetches a run of keys once for sixteen queries (the same bits as without).
    ``log_bias`` (float32 [Hq, 2] = (r1, r2)): ``score -= r1 * ln(1 + r2 * (s - p))``.  ``sinks`` (float32 [Hq]):
    exp(sink) is one more term of the softmax's denominator, with no key and no value.  ``value_dim``: the
    width of a value head if it is not the keys'; ``out`` is then [T, Hq * value_dim].  ``head_scales`` (float32
    [Hq]): every head's scores are multiplied by its number (after ``scale``).  ``sigmoid``: a visible key weighs
    sigmoid(score + ``score_bias[head]``) (float32 [Hq] or None) on its own and nothing is normalized.
    ``keep_first`` (with a window): keys at positions below it stay visible behind the window.  ``fixed_sink``: a
    sink of this score for every head, in place of ``sinks``."""
    _need(keep_first >= 0 and (keep_first == 0 or window), "paged_attention: first keys are kept behind a window")
    _need(fixed_sink is None or (sinks is None and not sigmoid), "paged_attention: one sink, in a softmax")
    q_ld = _row_major(q, "q")
    out_ld = _row_major(out, "out")
    T = q.shape[0]
    value_dim = head_dim if value_dim is None else int(value_dim)
    _need(q.shape[1] >= num_heads * head_dim and out.shape == (T, num_heads * value_dim)
          and out.dtype == q.dtype, "paged_attention: q/out shapes do not match")
    page_stride, page_size = _cache_view(k_cache, v_cache, num_kv_heads, head_dim, q.dtype, value_dim)
    _i32(block_tables, "block_tables")
    _i32(lane_of_token, "lane_of_token")
    _i32(positions, "positions")
    _need(block_tables.dim() == 2 and lane_of_token.numel() == T and positions.numel() == T,
          "paged_attention: metadata shapes do not match")
    _need(slopes is None or (slopes.dtype == torch.float32 and slopes.numel() == num_heads and slopes.is_contiguous()
                             and slopes.is_cuda), "paged_attention: slopes must be float32 [Hq] on the GPU")
    _need(log_bias is None or (log_bias.dtype == torch.float32 and log_bias.shape == (num_heads, 2)
                               and log_bias.is_contiguous() and log_bias.is_cuda),
          "paged_attention: log_bias must be float32 [Hq, 2] on the GPU")
    _need(sinks is None or (sinks.dtype == torch.float32 and sinks.numel() == num_heads and sinks.is_contiguous()
                            and sinks.is_cuda), "paged_attention: sinks must be float32 [Hq] on the GPU")
    for name, one in (("head_scales", head_scales), ("score_bias", score_bias)):
        _need(one is None or (one.dtype == torch.float32 and one.numel() == num_heads and one.is_contiguous()
                              and one.is_cuda), f"paged_attention: {name} must be float32 [Hq] on the GPU")
    _need(sigmoid or score_bias is None, "paged_attention: a bias per head is for sigmoid weights")
    _need(not (sigmoid and sinks is not None), "paged_attention: a sink belongs to a softmax")
    holds = block_tables.shape[1] * page_size
    span = holds if max_seq_len is None else max(1, min(int(max_seq_len), holds))
    floats = _fn("attention", "mi_paged_attention_workspace", _c_long)(T, num_heads, value_dim, span)
    partial = torch.empty((max(int(floats), 1),), dtype=torch.float32, device=q.device)
    tiles = 0
    if query_tiles is not None and tile_tokens and tile_tokens % 16 == 0 and cu_seqlens is not None:
        _i32(query_tiles, "query_tiles")
        _i32(cu_seqlens, "cu_seqlens")
        _need(query_tiles.dim() == 2 and query_tiles.shape[1] == 2 and cu_seqlens.numel() == block_tables.shape[0] + 1,
              "paged_attention: the table of runs or the lanes' offsets do not fit the step")
        tiles = query_tiles.shape[0]
    _check(_fn("attention", "mi_paged_attention")(
        _p(q), _dt(q), q_ld, T, num_heads, num_kv_heads, head_dim, value_dim, _p(k_cache), _p(v_cache), page_stride,
        page_size, _p(block_tables), block_tables.shape[1], _p(lane_of_token), _p(positions), float(scale),
        int(window or 0), int(keep_first), _p(slopes), _p(log_bias), _p(sinks),
        float(fixed_sink or 0.0), 0 if fixed_sink is None else 1, span, _p(partial), partial.numel(), _p(out), out_ld,
        _p(query_tiles) if tiles else None, tiles, int(tile_tokens) if tiles else 0, _p(cu_seqlens) if tiles else None,
        _p(head_scales), _p(score_bias), 1 if sigmoid else 0, _stream()), "paged_attention", f"(head_dim={head_dim})")


def attention_prepare(qkv: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int,
                      positions: torch.Tensor, inv_freq: Optional[torch.Tensor], rotary_dim: int,
                      slot_mapping: Optional[torch.Tensor], k_cache: Optional[torch.Tensor],
                      v_cache: Optional[torch.Tensor], *, values_from_keys: bool = False,
                      q_norm: Optional[torch.Tensor] = None, k_norm: Optional[torch.Tensor] = None,
                      norm_eps: float = 0.0, value_inv_freq: Optional[torch.Tensor] = None,
                      interleaved: bool = False, turn_scale: float = 1.0, head_norm: Optional[str] = None,
                      q_head_weight: Optional[torch.Tensor] = None, k_head_weight: Optional[torch.Tensor] = None,
                      head_eps: float = 0.0) -> None:
    """A token's projected row made ready for attention, one launch: ``qkv`` [T, >= Hq*dh + Hkv*dh (+ Hkv*dv)]
    holds q heads, k heads and (unless ``values_from_keys``) v heads.

    * ``q_norm`` / ``k_norm`` (float32 [Hq*dh] / [Hkv*dh]): the whole q projection, and the whole k projection, is
      divided by its root mean square (``norm_eps`` inside the root) and multiplied by the weight, before rotation;
    * ``head_norm`` ("before_rotation" / "after_rotation"): every q head and every k head is divided by its own root
      mean square over dh (``head_eps`` inside the root) and multiplied by ``q_head_weight`` / ``k_head_weight``
      (float32 [dh], shared by all heads; None: the bare division);
    * q and k are turned by the token's position over the first ``rotary_dim`` dims, angle = position * inv_freq[j],
      pairs (j, j + rotary_dim / 2) or, ``interleaved``, (2j, 2j + 1), cosines and sines times ``turn_scale``; q is
      written back in place, k goes to the token's cache cell;
    * the values are the v heads, or with ``values_from_keys`` the k heads as projected (before norm and rotation);
      with ``value_inv_freq`` (float32 [dv / 2]) they are turned by the position over all their dims (half-split
      pairs); they go to the token's (transposed) cache cell.

    Norms, angles and rotations are float32.  Without ``slot_mapping`` nothing is stored."""
    ld = _row_major(qkv, "qkv")
    T = qkv.shape[0]
    value_dim = int(value_dim)
    q_cols, k_cols = num_heads * head_dim, num_kv_heads * head_dim
    v_cols = 0 if values_from_keys else num_kv_heads * value_dim
    _need(qkv.shape[1] >= q_cols + k_cols + v_cols, "attention_prepare: qkv is too narrow")
    _need(not values_from_keys or value_dim == head_dim, "attention_prepare: values that are the keys have their width")
    _i32(positions, "positions")
    _need(positions.numel() == T, "attention_prepare: one position per token")
    if inv_freq is not None:
        _need(inv_freq.dtype == torch.float32 and inv_freq.numel() == rotary_dim // 2 and inv_freq.is_cuda
              and 0 < rotary_dim <= head_dim and rotary_dim % 2 == 0,
              "attention_prepare: inv_freq must be float32 [rotary_dim / 2]")
    if value_inv_freq is not None:
        _need(value_inv_freq.dtype == torch.float32 and value_dim % 2 == 0 and value_inv_freq.numel() == value_dim // 2
              and value_inv_freq.is_cuda, "attention_prepare: value_inv_freq must be float32 [value_dim / 2]")
    _need((q_norm is None) == (k_norm is None), "attention_prepare: both projections are normed or neither")
    if q_norm is not None:
        _need(q_norm.dtype == torch.float32 and q_norm.numel() == q_cols and q_norm.is_contiguous() and q_norm.is_cuda
              and k_norm.dtype == torch.float32 and k_norm.numel() == k_cols and k_norm.is_contiguous()
              and k_norm.is_cuda and norm_eps > 0, "attention_prepare: the norms' weights must be float32 [Hq*dh], [Hkv*dh]")
    _need(head_norm in (None, "before_rotation", "after_rotation") and (head_norm is None or q_norm is None),
          "attention_prepare: heads are normed before or after the rotation, and not beside a norm of the projections")
    _need((q_head_weight is None) == (k_head_weight is None) and (q_head_weight is None or head_norm is not None),
          "attention_prepare: the heads' norm has both weights or none")
    for one in (q_head_weight, k_head_weight):
        _need(one is None or (one.dtype == torch.float32 and one.numel() == head_dim and one.is_contiguous() and one.is_cuda),
              "attention_prepare: a weight of the heads' norm must be float32 [dh] on the GPU")
    _need(head_norm is None or head_eps > 0, "attention_prepare: the heads' norm needs its eps")
    page_stride, page_size = 0, 0
    if slot_mapping is not None:
        _i32(slot_mapping, "slot_mapping")
        _need(slot_mapping.numel() == T, "attention_prepare: one cache cell per token")
        page_stride, page_size = _cache_view(k_cache, v_cache, num_kv_heads, head_dim, qkv.dtype, value_dim)
    _check(_fn("attention", "mi_attention_prepare")(
        _p(qkv), _dt(qkv), ld, T, num_heads, num_kv_heads, head_dim, value_dim, 1 if values_from_keys else 0,
        _p(positions), _p(inv_freq), int(rotary_dim) if inv_freq is not None else 0, 1 if interleaved else 0,
        float(turn_scale), _p(q_norm), _p(k_norm), float(norm_eps),
        {None: 0, "before_rotation": 1, "after_rotation": 2}[head_norm], _p(q_head_weight), _p(k_head_weight),
        float(head_eps), _p(value_inv_freq), _p(slot_mapping), _p(k_cache) if slot_mapping is not None else None,
        _p(v_cache) if slot_mapping is not None else None, page_stride, page_size, _stream()), "attention_prepare")


def prefill_attention_supported(dtype, num_heads: int, num_kv_heads: int, head_dim: int, page_size: int) -> bool:
    """Whether the matrix-core attention kernel covers this geometry."""
    return (dtype == torch.bfloat16 and head_dim in (64, 128) and page_size % 4 == 0
            and num_heads // num_kv_heads <= 64)


def prefill_attention(q: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int, k_cache: torch.Tensor,
                      v_cache: torch.Tensor, block_tables: torch.Tensor, query_tiles: torch.Tensor,
                      cu_seqlens: torch.Tensor, start_pos: torch.Tensor, scale: float, window: Optional[int],
                      out: torch.Tensor, max_seq_len: int = 0, log_bias: Optional[torch.Tensor] = None,
                      sinks: Optional[torch.Tensor] = None, keep_first: int = 0) -> None:
    """``paged_attention`` on the matrix cores for bfloat16 (flash-style, online softmax in
    float32).  ``query_tiles`` [tiles, 2]: (lane, first token row) of runs of up to 64 tokens of
    one lane; the keys and values of the step's own tokens must be in the cache already.
    ``max_seq_len``: an upper bound of the step's longest context if known (it picks how many heads share
    a key fragment, never the result).  ``keep_first`` (with a window): keys at positions below it stay visible."""
    _need(keep_first >= 0 and (keep_first == 0 or window), "prefill_attention: first keys are kept behind a window")
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
    # the same two terms as ``paged_attention``'s: a bias by the logarithm of the distance, a sink in the denominator
    _need(log_bias is None or (log_bias.dtype == torch.float32 and log_bias.shape == (num_heads, 2)
                               and log_bias.is_contiguous() and log_bias.is_cuda),
          "prefill_attention: log_bias must be float32 [Hq, 2] on the GPU")
    _need(sinks is None or (sinks.dtype == torch.float32 and sinks.numel() == num_heads and sinks.is_contiguous()
                            and sinks.is_cuda), "prefill_attention: sinks must be float32 [Hq] on the GPU")
    _check(_fn("attention", "mi_prefill_attention")(
        _p(q), q_ld, num_heads, num_kv_heads, head_dim, _p(k_cache), _p(v_cache), page_stride, page_size,
        _p(block_tables), block_tables.shape[1], _p(query_tiles), query_tiles.shape[0], _p(cu_seqlens),
        _p(start_pos), float(scale), int(window or 0), int(max_seq_len or 0), _p(out), out_ld, _p(log_bias),
        _p(sinks), int(keep_first), _stream()), "prefill_attention")


PREFILL_VALUE_WIDTH_MOST = 256      # the widest values the matrix-core kernel computes with


def prefill_attention_forms_supported(dtype, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int,
                                      page_size: int, sigmoid: bool, per_head: bool) -> bool:
    """Whether the matrix-core kernel's further forms cover this: sigmoid weights (with a multiplier and a bias per
    head, ``per_head``) over values as wide as the keys, or a softmax over values of another width."""
    if not (dtype == torch.bfloat16 and head_dim in (64, 128) and page_size % 4 == 0
            and num_heads // num_kv_heads <= 64 and value_dim % 4 == 0):
        return False
    if sigmoid:
        return value_dim == head_dim
    return value_dim != head_dim and value_dim <= PREFILL_VALUE_WIDTH_MOST and not per_head


def prefill_attention_forms(q: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int,
                            k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                            query_tiles: torch.Tensor, cu_seqlens: torch.Tensor, start_pos: torch.Tensor, scale: float,
                            window: Optional[int], out: torch.Tensor, max_seq_len: int = 0, sigmoid: bool = False,
                            head_scales: Optional[torch.Tensor] = None, score_bias: Optional[torch.Tensor] = None) -> None:
    """``prefill_attention`` for values of another width than the keys (``out`` [T, Hq * value_dim]), or, with
    ``sigmoid``, for weights sigmoid(score * scale * head_scales[h] + score_bias[h]) that are not normalized."""
    q_ld = _row_major(q, "q")
    out_ld = _row_major(out, "out")
    T = q.shape[0]
    _need(q.dtype == torch.bfloat16 and out.dtype == torch.bfloat16, "prefill_attention_forms: bfloat16 only")
    _need(q.shape[1] >= num_heads * head_dim and out.shape == (T, num_heads * value_dim) and q_ld % 8 == 0
          and q.data_ptr() % 16 == 0 and out_ld % 4 == 0 and out.data_ptr() % 8 == 0,
          "prefill_attention_forms: q/out shapes or alignment do not fit")
    page_stride, page_size = _cache_view(k_cache, v_cache, num_kv_heads, head_dim, q.dtype, value_dim)
    _need(prefill_attention_forms_supported(q.dtype, num_heads, num_kv_heads, head_dim, value_dim, page_size, sigmoid,
                                            head_scales is not None or score_bias is not None),
          "prefill_attention_forms: not covered; use paged_attention")
    for name, tensor in (("block_tables", block_tables), ("query_tiles", query_tiles), ("cu_seqlens", cu_seqlens),
                         ("start_pos", start_pos)):
        _i32(tensor, name)
    _need(block_tables.dim() == 2 and query_tiles.dim() == 2 and query_tiles.shape[1] == 2
          and cu_seqlens.numel() == start_pos.numel() + 1, "prefill_attention_forms: metadata shapes do not match")
    for name, tensor in (("head_scales", head_scales), ("score_bias", score_bias)):
        _need(tensor is None or (tensor.dtype == torch.float32 and tensor.numel() == num_heads and tensor.is_contiguous()
                                 and tensor.is_cuda), f"prefill_attention_forms: {name} must be float32 [Hq] on the GPU")
    _check(_fn("attention", "mi_prefill_attention_forms")(
        _p(q), q_ld, num_heads, num_kv_heads, head_dim, int(value_dim), _p(k_cache), _p(v_cache), page_stride,
        page_size, _p(block_tables), block_tables.shape[1], _p(query_tiles), query_tiles.shape[0], _p(cu_seqlens),
        _p(start_pos), float(scale), int(window or 0), int(max_seq_len or 0), _p(out), out_ld, 1 if sigmoid else 0,
        _p(head_scales), _p(score_bias), _stream()), "prefill_attention_forms")


DECODE_KEEP_FIRST_MOST = 512        # DEC_MAX_SPLIT in attention.hip: the kept first keys are one block's work


def decode_attention_supported(dtype, num_heads: int, num_kv_heads: int, head_dim: int, page_size: int,
                               value_dim: Optional[int] = None, keep_first: int = 0) -> bool:
    """Whether the split-context kernel for single-token queries covers this geometry."""
    return (dtype == torch.bfloat16 and head_dim in (64, 128) and num_heads // num_kv_heads <= 8
            and page_size % 8 == 0 and page_size <= 512 and (value_dim is None or 0 < value_dim <= 256)
            and keep_first <= DECODE_KEEP_FIRST_MOST)


def decode_attention(q: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int, k_cache: torch.Tensor,
                     v_cache: torch.Tensor, block_tables: torch.Tensor, lane_of_token: torch.Tensor,
                     positions: torch.Tensor, scale: float, window: Optional[int], max_seq_len: int,
                     out: torch.Tensor, value_dim: Optional[int] = None, head_scales: Optional[torch.Tensor] = None,
                     score_bias: Optional[torch.Tensor] = None, sigmoid: bool = False, keep_first: int = 0,
                     sinks: Optional[torch.Tensor] = None) -> None:
    """``paged_attention`` for batches of single decoded tokens in bfloat16: the context of each
    request is split over many workgroups and the G query heads of a kv head share its K/V
    loads.  ``max_seq_len``: an upper bound of the longest context in the batch.  ``value_dim``,
    ``head_scales``, ``score_bias``, ``sigmoid``, ``keep_first`` and ``sinks`` as in ``paged_attention``."""
    _need(keep_first >= 0 and (keep_first == 0 or window), "decode_attention: first keys are kept behind a window")
    _need(sinks is None or (sinks.dtype == torch.float32 and sinks.numel() == num_heads and sinks.is_contiguous()
                            and sinks.is_cuda and not sigmoid), "decode_attention: sinks must be float32 [Hq] on the GPU")
    q_ld = _row_major(q, "q")
    out_ld = _row_major(out, "out")
    T = q.shape[0]
    value_dim = head_dim if value_dim is None else int(value_dim)
    _need(q.dtype == torch.bfloat16 and out.dtype == torch.bfloat16, "decode_attention: bfloat16 only")
    _need(q.shape[1] >= num_heads * head_dim and out.shape == (T, num_heads * value_dim) and q_ld % 8 == 0
          and q.data_ptr() % 16 == 0, "decode_attention: q/out shapes or alignment do not fit")
    page_stride, page_size = _cache_view(k_cache, v_cache, num_kv_heads, head_dim, q.dtype, value_dim)
    _need(decode_attention_supported(q.dtype, num_heads, num_kv_heads, head_dim, page_size, value_dim, keep_first),
          "decode_attention: geometry not covered; use paged_attention")
    _i32(block_tables, "block_tables")
    _i32(lane_of_token, "lane_of_token")
    _i32(positions, "positions")
    _need(block_tables.dim() == 2 and lane_of_token.numel() == T and positions.numel() == T,
          "decode_attention: metadata shapes do not match")
    for name, one in (("head_scales", head_scales), ("score_bias", score_bias)):
        _need(one is None or (one.dtype == torch.float32 and one.numel() == num_heads and one.is_contiguous()
                              and one.is_cuda), f"decode_attention: {name} must be float32 [Hq] on the GPU")
    _need(sigmoid or score_bias is None, "decode_attention: a bias per head is for sigmoid weights")
    span = max_seq_len if not window else min(max_seq_len, window + page_size)
    split_keys = 64
    while split_keys < 512 and span * T * num_kv_heads > 1024 * split_keys:
        split_keys *= 2
    split_keys = max(split_keys, page_size)
    splits = max(1, -(-span // split_keys))
    blocks = splits + (1 if keep_first else 0)         # the kept first keys are the work of one more block
    partial_o = torch.empty((T, num_heads, blocks, value_dim), dtype=torch.float32, device=q.device)
    partial_ml = torch.empty((T, num_heads, blocks, 2), dtype=torch.float32, device=q.device)
    _check(_fn("attention", "mi_decode_attention_forms")(
        _p(q), q_ld, T, num_heads, num_kv_heads, head_dim, value_dim, _p(k_cache), _p(v_cache), page_stride, page_size,
        _p(block_tables), block_tables.shape[1], _p(lane_of_token), _p(positions), float(scale), int(window or 0),
        split_keys, splits, _p(partial_o), _p(partial_ml), _p(out), out_ld, _p(head_scales), _p(score_bias),
        1 if sigmoid else 0, int(keep_first), _p(sinks), _stream()), "decode_attention")


# --------------------------------------------------------------------------- mamba2
def conv1d_silu(u: torch.Tensor, col_offset: int, width: int, weight: torch.Tensor,
                bias: Optional[torch.Tensor], conv_state: torch.Tensor, lane_of_token: torch.Tensor,
                cu_seqlens: torch.Tensor, slot_ids: torch.Tensor, out: torch.Tensor, activation: bool = True) -> None:
    """out[t] = SiLU(causal depthwise conv of u[:, col_offset:col_offset+width]) per lane,
    the K-1 rows before a lane's first token coming from ``conv_state[slot]`` [K-1, width].
    ``activation`` False: the convolution's sums as they are, without the SiLU."""
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
        _p(cu_seqlens), _p(slot_ids), _p(out), 1 if activation else 0, _stream()), "conv1d_silu", f"(K={K})")


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
              conv_state: torch.Tensor, slot_ids: torch.Tensor, activation: bool = True) -> None:
    """One conv step of single-token lanes, in place: row m of ``u`` is the new token of the request in
    ``slot_ids[m]``; columns [col_offset, col_offset + width) become SiLU(conv over [tail ; sample]) and the
    tail ``conv_state[slot]`` [K-1, width] is rolled by one and takes the sample.  ``activation`` False: no SiLU."""
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
                                         _p(conv_state), _p(slot_ids), 1 if activation else 0, _stream()),
           "conv_step", f"(K={K})")


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
               row_scale: Optional["RowScale"] = None, shared_rows: bool = False, row_tiles: int = 1,
               gate_activation: str = "silu") -> None:
    """out[M, N'] = epilogue(prologue . weight[N, K]^T + bias) for a small batch in bfloat16.

    Prologue: ``x`` [M, K] bfloat16, or ``h_in`` float32 [M, K] with up to two bfloat16 ``deltas``:
    the rows are summed (the sum goes to ``h_out``, a different tensor, if given), RMS-normed
    with ``norm_weight`` and ``eps``.  Epilogue PLAIN: bfloat16 or float32 ``out`` [M, N] times
    ``out_scale``.  SWIGLU: weight rows in tiles of 8 gate + 8 up rows, ``out`` [M, N/2] = act(gate) * up with
    act = SiLU or, ``gate_activation`` "gelu_tanh", the tanh form of GELU.
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
    _need(gate_activation in GATE_ACTIVATIONS and (gate_activation == "silu" or epilogue == EPI_SWIGLU),
          "fused_gemm: the gate's activation is silu or gelu_tanh, and belongs to the SWIGLU epilogue")
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
        pro, epilogue | (GATE_ACTIVATIONS[gate_activation] << 8), _p(h_in), _p(deltas[0]) if len(deltas) > 0 else None, _p(deltas[1]) if len(deltas) > 1 else None,
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
