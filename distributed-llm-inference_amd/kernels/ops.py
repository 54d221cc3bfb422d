"""Typed wrappers around the library's ``extern "C"`` entry points.

Every wrapper checks on the host that the operands have the device, type, layout and sizes that
its kernel and launch grid assume, and raises :class:`KernelArgumentError` otherwise: a kernel is
never launched on operands it was not written for. torch supplies device memory and the current
stream; nothing here computes with torch.
"""

from __future__ import annotations

import ctypes
from typing import Optional, Sequence

import torch

from . import build

_c_int, _c_i64, _c_float, _c_ptr = ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_void_p


class KernelArgumentError(ValueError):
    """Operands that a kernel does not take."""


class KernelLaunchError(RuntimeError):
    """The HIP runtime refused a launch."""


_SIGNATURES = {
    "dli_embedding": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
    "dli_rms_norm": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_float, _c_int, _c_ptr],
    "dli_silu_mul": [_c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
    "dli_add": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
    "dli_gather_rows": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
    "dli_to_float": [_c_ptr, _c_ptr, _c_i64, _c_int, _c_ptr],
    "dli_copy_pages": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_i64, _c_i64, _c_int, _c_ptr],
    "dli_fill": [_c_ptr, _c_float, _c_i64, _c_int, _c_ptr],
    "dli_skinny4_gemm": [_c_ptr, _c_i64, _c_ptr, _c_int, _c_ptr, _c_float, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_ptr,
                         _c_i64, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "dli_skinny4_tile_features": [_c_int, _c_int],
    "dli_rope_kv_write": [_c_ptr, _c_i64, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int,
                          _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "dli_gemm_f32_nt": [_c_ptr, _c_i64, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_i64, _c_ptr, _c_i64, _c_int,
                        _c_int, _c_int, _c_ptr],
    "dli_sample": [_c_ptr, _c_i64, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                   _c_ptr],
    "dli_sample_scratch_per_row": [],
    "dli_sample_and_advance": [_c_ptr, _c_i64, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                               _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int,
                               _c_int, _c_ptr],
    "dli_decode_advance": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int,
                           _c_int, _c_int, _c_ptr],
    "dli_skinny_gemm_max_rows": [],
    "dli_skinny_gemm": [_c_ptr, _c_i64, _c_ptr, _c_int, _c_ptr, _c_float, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_ptr,
                        _c_i64, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "dli_skinny_gemm_qkv_rope": [_c_ptr, _c_i64, _c_ptr, _c_int, _c_ptr, _c_float, _c_ptr, _c_ptr, _c_ptr, _c_i64,
                                 _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                                 _c_int, _c_ptr],
    "dli_head_gemm_supports": [_c_int, _c_int, _c_int],
    "dli_head_gemm": [_c_ptr, _c_i64, _c_ptr, _c_int, _c_ptr, _c_float, _c_ptr, _c_ptr, _c_i64, _c_int, _c_int, _c_int,
                      _c_int, _c_ptr, _c_ptr, _c_ptr],
    "dli_head_gemm_workgroups": [_c_int, _c_int],
    "dli_skinny_gemm_merged": [_c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_ptr, _c_int,
                               _c_int, _c_int, _c_ptr],
    "dli_mid_gemm": [_c_ptr, _c_i64, _c_ptr, _c_int, _c_ptr, _c_float, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_i64, _c_int,
                     _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "dli_mid_finish_residual": [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_i64, _c_ptr, _c_int, _c_int, _c_ptr],
    "dli_mid_finish_residual_normed": [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_float, _c_ptr, _c_i64,
                                       _c_int, _c_int, _c_ptr],
    "dli_mid_finish_qkv": [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_int, _c_int,
                           _c_int, _c_int, _c_int, _c_ptr],
    "dli_gemm_bf16": [_c_ptr, _c_i64, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_i64, _c_i64, _c_i64, _c_i64, _c_ptr, _c_i64,
                      _c_int, _c_ptr],
    "dli_gemm_bf16_f32": [_c_ptr, _c_i64, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_i64, _c_i64, _c_i64, _c_i64, _c_ptr, _c_i64,
                      _c_int, _c_ptr],
    "dli_gemm_bf16_usable": [_c_i64, _c_i64, _c_i64, _c_i64, _c_i64, _c_i64, _c_int, _c_i64, _c_int],
    "dli_prenorm_blocks_bf16": [_c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr],
    "dli_embedding_ssq": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr],
    "dli_attention_generic_tile_rows": [_c_int],
    "dli_attention_mfma_supports": [_c_int, _c_int],
    "dli_attention_prefill_tile_rows": [_c_int, _c_int, _c_int],
    "dli_attention_decode_bf16": [_c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                                  _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int, _c_ptr],
    "dli_attention_decode_self_merging_bf16": [_c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr,
                                               _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                                               _c_float, _c_int, _c_int, _c_ptr],
    "dli_attention_decode_partial_bf16": [_c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int,
                                          _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int, _c_ptr],
    "dli_attention_decode_bf16_static": [_c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_int,
                                         _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int, _c_ptr],
    "dli_rope_angles": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
    "dli_attention_prefill_bf16": [_c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_int,
                                   _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_ptr,
                                   _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr],
    "dli_attention_prefill_cut_floats": [_c_int, _c_int, _c_int],
    "dli_attention_prefill_max_cuts": [],
    "dli_attention_generic": [_c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr,
                              _c_int, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float,
                              _c_int, _c_int, _c_ptr],
    "dli_attention_scored": [_c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr,
                             _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int, _c_int, _c_ptr,
                             _c_ptr, _c_ptr, _c_i64, _c_int, _c_int, _c_ptr, _c_int, _c_ptr],
    "dli_attention_scored_splits": [_c_int, _c_int, _c_int],
    "dli_attention_scored_single": [_c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int,
                                    _c_int, _c_int, _c_int, _c_float, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_i64,
                                    _c_int, _c_int, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr],
    "dli_attention_scored_mfma_supports": [_c_int, _c_int, _c_int],
    "dli_attention_scored_mfma": [_c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr,
                                  _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_int, _c_int, _c_ptr,
                                  _c_ptr, _c_ptr, _c_i64, _c_int, _c_int, _c_ptr, _c_ptr],
    "dli_embed_sinusoid": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
    "dli_cast_from_f32": [_c_ptr, _c_ptr, _c_i64, _c_int, _c_ptr],
    "dli_norm_into_stream": [_c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_float, _c_int, _c_ptr],
    "dli_rms_norm_from_f32": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_float, _c_int, _c_ptr],
    "dli_softcap": [_c_ptr, _c_i64, _c_float, _c_ptr],
    "dli_post_norm_stream": [_c_ptr, _c_i64, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_float,
                             _c_float, _c_int, _c_ptr],
    "dli_causal_conv": [_c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_i64,
                        _c_ptr, _c_i64, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "dli_selective_scan_max_states": [],
    "dli_selective_scan": [_c_ptr, _c_i64, _c_ptr, _c_i64, _c_ptr, _c_i64, _c_int, _c_int, _c_ptr, _c_i64, _c_ptr, _c_ptr,
                           _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_int, _c_int, _c_int, _c_int, _c_int,
                           _c_ptr],
    "dli_bounded_gates": [_c_ptr, _c_i64, _c_int, _c_int, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr],
    "dli_gated_linear_scan": [_c_ptr, _c_i64, _c_int, _c_int, _c_int, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                              _c_i64, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "dli_latent_norm_cache": [_c_ptr, _c_i64, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_float, _c_ptr, _c_ptr,
                              _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
    "dli_head_products": [_c_ptr, _c_i64, _c_ptr, _c_ptr, _c_i64, _c_ptr, _c_i64, _c_int, _c_int, _c_int, _c_int, _c_int,
                          _c_ptr],
    "dli_token_shift": [_c_ptr, _c_ptr, _c_int, _c_ptr, _c_i64, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int,
                        _c_int, _c_ptr],
    "dli_lowrank_out": [_c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_i64,
                        _c_ptr, _c_ptr],
    "dli_qk_unit_cache": [_c_ptr, _c_i64, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                          _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _c_ptr],
    "dli_recurrent_scan_supports": [_c_int],
    "dli_recurrent_scan": [_c_ptr, _c_i64, _c_ptr, _c_i64, _c_ptr, _c_i64, _c_ptr, _c_i64, _c_ptr, _c_i64, _c_ptr, _c_ptr,
                           _c_i64, _c_ptr, _c_ptr, _c_float, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_ptr,
                           _c_i64, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "dli_rotary_cache": [_c_ptr, _c_i64, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr,
                         _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "dli_diff_head_norm": [_c_ptr, _c_i64, _c_float, _c_float, _c_float, _c_ptr, _c_i64, _c_ptr, _c_i64, _c_int, _c_int,
                           _c_int, _c_int, _c_ptr],
    "dli_branch_weighted_sum": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_int, _c_int, _c_ptr],
    "dli_scale_f32": [_c_ptr, _c_i64, _c_float, _c_ptr],
    "dli_silu_columns": [_c_ptr, _c_i64, _c_int, _c_int, _c_ptr],
    "dli_rms_norm_pair": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_float, _c_int, _c_ptr],
    "dli_add_pair_into_stream": [_c_ptr, _c_ptr, _c_ptr, _c_i64, _c_ptr],
    "dli_table_choose": [_c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr],
    "dli_exp_gates": [_c_ptr, _c_i64, _c_int, _c_int, _c_ptr, _c_ptr, _c_float, _c_ptr, _c_i64, _c_i64, _c_ptr, _c_ptr,
                      _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr],
    "dli_scalar_gate_scan": [_c_ptr, _c_i64, _c_ptr, _c_i64, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr,
                             _c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_int, _c_int, _c_int, _c_int,
                             _c_int, _c_float, _c_int, _c_int, _c_ptr],
    "dli_group_norm": [_c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_float, _c_int, _c_ptr],
    "dli_branch_norm_mean": [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_int, _c_int, _c_float, _c_ptr],
    "dli_head_norm_gate": [_c_ptr, _c_i64, _c_ptr, _c_i64, _c_ptr, _c_float, _c_ptr, _c_i64, _c_int, _c_int, _c_int, _c_int,
                           _c_ptr, _c_int, _c_ptr],
    "dli_gated_delta_max_taps": [],
    "dli_conv_prepare": [_c_ptr, _c_i64, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_i64, _c_ptr, _c_ptr,
                         _c_ptr, _c_ptr, _c_i64, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    "dli_gated_delta_scan": [_c_ptr, _c_i64, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_int, _c_int, _c_int,
                             _c_int, _c_int, _c_int, _c_ptr],
    "dli_poly_norm": [_c_ptr, _c_i64, _c_ptr, _c_ptr, _c_i64, _c_int, _c_int, _c_float, _c_int, _c_ptr],
    "dli_clamped_glu": [_c_ptr, _c_i64, _c_ptr, _c_int, _c_int, _c_float, _c_float, _c_float, _c_int, _c_ptr],
    "dli_router_choose": [_c_ptr, _c_i64, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_ptr, _c_ptr,
                          _c_ptr],
    "dli_expert_tile_rows": [_c_int, _c_int, _c_int],
    "dli_expert_products": [_c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int,
                            _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_float, _c_float, _c_int,
                            _c_ptr],
    "dli_expert_combine": [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_i64, _c_ptr, _c_i64, _c_ptr, _c_i64, _c_ptr, _c_int, _c_int,
                           _c_int, _c_int, _c_int, _c_ptr],
}

_lib: Optional[ctypes.CDLL] = None


def library() -> ctypes.CDLL:
    """The loaded HIP library with argument types declared (compiled at the first call if absent)."""
    global _lib
    if _lib is None:
        lib = build.load()
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(lib, name, None)
            if fn is None:
                raise build.KernelBuildError(f"{build.loaded_path()} lacks the entry point {name}")
            fn.argtypes = argtypes
            fn.restype = _c_int
        _lib = lib
    return _lib


def _check(status: int, name: str) -> None:
    if status == 0:
        return
    if status == -1:
        raise KernelArgumentError(f"{name}: the kernel does not take these sizes")
    raise KernelLaunchError(f"{name}: launch failed (status {status})")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> _c_ptr:
    """The current stream's handle. The raw getter skips the Stream object that
    ``torch.cuda.current_stream()`` builds at every call (a hundred calls a step)."""
    if _raw_stream is not None:
        return _c_ptr(_raw_stream(torch.cuda.current_device()))
    return _c_ptr(torch.cuda.current_stream().cuda_stream)


def _is_bf16(dtype: torch.dtype) -> int:
    if dtype == torch.bfloat16:
        return 1
    if dtype == torch.float32:
        return 0
    raise KernelArgumentError(f"activation type {dtype} is neither float32 nor bfloat16")


def _ptr(t: Optional[torch.Tensor]) -> _c_ptr:
    return _c_ptr(0 if t is None else t.data_ptr())


def _require(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelArgumentError(msg)


def _dense(t: torch.Tensor, name: str, dtype: Optional[torch.dtype] = None, ndim: Optional[int] = None) -> None:
    # the messages are put together only when a check fails: this runs hundreds of times a step
    if t.is_cuda and t.is_contiguous() and (dtype is None or t.dtype == dtype) and (ndim is None or t.dim() == ndim):
        return
    _require(t.is_cuda, f"{name} is not on the GPU")
    _require(t.is_contiguous(), f"{name} is not contiguous")
    _require(dtype is None or t.dtype == dtype, f"{name} has type {t.dtype}, expected {dtype}")
    _require(ndim is None or t.dim() == ndim, f"{name} has {t.dim()} dimensions, expected {ndim}")


def _rows(t: torch.Tensor, name: str, dtype: torch.dtype) -> None:
    """A 2-D operand whose rows are contiguous (a row stride larger than the width is allowed)."""
    if t.is_cuda and t.dim() == 2 and t.stride(1) == 1 and t.stride(0) >= t.shape[1] and t.dtype == dtype:
        return
    _require(t.is_cuda, f"{name} is not on the GPU")
    _require(t.dim() == 2 and t.stride(1) == 1 and t.stride(0) >= t.shape[1],
             f"{name} is not a matrix with contiguous rows")
    _require(t.dtype == dtype, f"{name} has type {t.dtype}, expected {dtype}")


# ----------------------------------------------------------------------------- element-wise

def embedding(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor) -> None:
    """``out[t] = table[ids[t]]``; ids int32 and already checked against the table's rows."""
    _dense(table, "table", ndim=2)
    _dense(ids, "ids", torch.int32, 1)
    _dense(out, "out", table.dtype, 2)
    _require(out.shape == (ids.shape[0], table.shape[1]), "out must be [len(ids), width]")
    _check(library().dli_embedding(_ptr(table), _ptr(ids), _ptr(out), ids.shape[0], table.shape[1],
                                   _is_bf16(table.dtype), _stream()), "embedding")


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor,
             delta: Optional[torch.Tensor] = None, sum_out: Optional[torch.Tensor] = None) -> None:
    """``out = weight * cast(x * rsqrt(mean(x^2) + eps))``. With ``delta``: x is first replaced by
    ``x + delta`` (written to ``sum_out``, which may be ``x`` itself)."""
    _dense(x, "x", ndim=2)
    _dense(weight, "weight", torch.float32, 1)
    _dense(out, "out", x.dtype, 2)
    _require(weight.shape[0] == x.shape[1], "weight length differs from the row width")
    _require(out.shape == x.shape, "out differs from x in shape")
    if delta is not None:
        _dense(delta, "delta", x.dtype, 2)
        _require(sum_out is not None, "delta needs sum_out")
        _dense(sum_out, "sum_out", x.dtype, 2)
        _require(delta.shape == x.shape and sum_out.shape == x.shape, "delta/sum_out differ from x in shape")
    _check(library().dli_rms_norm(_ptr(x), _ptr(delta), _ptr(weight), _ptr(sum_out), _ptr(out), x.shape[0],
                                  x.shape[1], float(eps), _is_bf16(x.dtype), _stream()), "rms_norm")


def silu_mul(gate_up: torch.Tensor, out: torch.Tensor) -> None:
    """``out = silu(gate_up[:, :I]) * gate_up[:, I:]``."""
    _dense(gate_up, "gate_up", ndim=2)
    _dense(out, "out", gate_up.dtype, 2)
    _require(gate_up.shape[1] == 2 * out.shape[1] and gate_up.shape[0] == out.shape[0],
             "gate_up must be [rows, 2*I] for out [rows, I]")
    _check(library().dli_silu_mul(_ptr(gate_up), _ptr(out), out.shape[0], out.shape[1],
                                  _is_bf16(out.dtype), _stream()), "silu_mul")


def add(a: torch.Tensor, b: Optional[torch.Tensor], out: torch.Tensor,
        bias: Optional[torch.Tensor] = None) -> None:
    """``out = (a + bias) + b``; sums in 32-bit. ``out`` may alias ``a`` or ``b``."""
    _dense(a, "a", ndim=2)
    _dense(out, "out", a.dtype, 2)
    _require(out.shape == a.shape, "out differs from a in shape")
    if b is not None:
        _dense(b, "b", a.dtype, 2)
        _require(b.shape == a.shape, "b differs from a in shape")
    if bias is not None:
        _dense(bias, "bias", a.dtype, 1)
        _require(bias.shape[0] == a.shape[1], "bias length differs from the row width")
    _check(library().dli_add(_ptr(a), _ptr(b), _ptr(bias), _ptr(out), a.shape[0], a.shape[1],
                             _is_bf16(a.dtype), _stream()), "add")


def gather_rows(x: torch.Tensor, rows: torch.Tensor, out: torch.Tensor) -> None:
    """``out[i] = x[rows[i]]``; rows int32, already checked against x's rows."""
    _dense(x, "x", ndim=2)
    _dense(rows, "rows", torch.int32, 1)
    _dense(out, "out", x.dtype, 2)
    _require(out.shape == (rows.shape[0], x.shape[1]), "out must be [len(rows), width]")
    _check(library().dli_gather_rows(_ptr(x), _ptr(rows), _ptr(out), rows.shape[0], x.shape[1],
                                     _is_bf16(x.dtype), _stream()), "gather_rows")


def to_float(x: torch.Tensor, out: torch.Tensor) -> None:
    _dense(x, "x")
    _dense(out, "out", torch.float32)
    _require(out.numel() == x.numel(), "out differs from x in size")
    _check(library().dli_to_float(_ptr(x), _ptr(out), x.numel(), _is_bf16(x.dtype), _stream()), "to_float")


def fill(x: torch.Tensor, value: float) -> None:
    _dense(x, "x")
    _check(library().dli_fill(_ptr(x), float(value), x.numel(), _is_bf16(x.dtype), _stream()), "fill")


def copy_pages(pool: torch.Tensor, src: torch.Tensor, dst: torch.Tensor) -> None:
    """Copy page ``src[i]`` onto page ``dst[i]`` in every layer, keys and values.

    ``pool`` is ``[layers, 2, pages, ...]`` (or ``[layers, 1, pages, ...]`` where keys and values
    live in tensors of their own); the page ids are int32 and already range-checked.
    """
    _dense(pool, "pool")
    _require(pool.dim() >= 4 and pool.shape[1] in (1, 2), "pool must be [layers, 1 or 2, pages, ...]")
    _dense(src, "src", torch.int32, 1)
    _dense(dst, "dst", torch.int32, 1)
    _require(src.shape == dst.shape, "src and dst differ in length")
    pages = pool.shape[2]
    page_elems = pool[0, 0, 0].numel()
    _check(library().dli_copy_pages(_ptr(pool), _ptr(src), _ptr(dst), src.shape[0], pool.shape[0] * pool.shape[1], pages,
                                    page_elems, _is_bf16(pool.dtype), _stream()), "copy_pages")


# ----------------------------------------------------------------------------- position + cache write

def rope_kv_write(qkv: torch.Tensor, positions: torch.Tensor, inv_freq: Optional[torch.Tensor],
                  rotary_dim: int, slots: Optional[torch.Tensor], k_pages: Optional[torch.Tensor],
                  v_pages: Optional[torch.Tensor], q_heads: int, kv_heads: int, head_dim: int) -> None:
    """Rotate q (in place) and k, and write rotated k and raw v at each token's cache slot.

    ``qkv`` is ``[tokens, (q_heads + 2*kv_heads) * head_dim]``; ``k_pages`` is
    ``[pages, kv_heads, page_size, head_dim]`` and ``v_pages`` ``[pages, kv_heads, head_dim,
    page_size]``; ``slots[t] = page * page_size + offset`` (negative: the token is not cached).
    """
    _rows(qkv, "qkv", qkv.dtype)
    n = qkv.shape[0]
    _require(qkv.shape[1] == (q_heads + 2 * kv_heads) * head_dim, "qkv width differs from (q+2kv)*head_dim")
    _dense(positions, "positions", torch.int32, 1)
    _require(positions.shape[0] == n, "positions differ from qkv in rows")
    page_size = 1
    if inv_freq is not None:
        _dense(inv_freq, "inv_freq", torch.float32, 1)
        _require(inv_freq.shape[0] * 2 == rotary_dim, "inv_freq must hold rotary_dim/2 frequencies")
    if kv_heads > 0:
        _require(slots is not None and k_pages is not None and v_pages is not None,
                 "kv heads need slots and pages")
        _dense(slots, "slots", torch.int32, 1)
        _require(slots.shape[0] == n, "slots differ from qkv in rows")
        _dense(k_pages, "k_pages", qkv.dtype, 4)
        _dense(v_pages, "v_pages", qkv.dtype, 4)
        page_size = k_pages.shape[2]
        _require(k_pages.shape[1] == kv_heads and k_pages.shape[3] == head_dim,
                 "k_pages must be [pages, kv_heads, page_size, head_dim]")
        _require(v_pages.shape == (k_pages.shape[0], kv_heads, head_dim, page_size),
                 "v_pages must be [pages, kv_heads, head_dim, page_size]")
    _check(library().dli_rope_kv_write(
        _ptr(qkv), qkv.stride(0), _ptr(positions), _ptr(inv_freq), rotary_dim, _ptr(slots), _ptr(k_pages),
        _ptr(v_pages), n, q_heads, kv_heads, head_dim, page_size, _is_bf16(qkv.dtype), _stream()),
        "rope_kv_write")


# ----------------------------------------------------------------------------- matrix products

def gemm_f32(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, bias: Optional[torch.Tensor] = None,
             residual: Optional[torch.Tensor] = None) -> None:
    """``out = a @ w.T (+ bias) (+ residual)`` in IEEE single precision; ``w`` is ``[n, k]``."""
    _rows(a, "a", torch.float32)
    _rows(w, "w", torch.float32)
    _rows(out, "out", torch.float32)
    m, k = a.shape
    n = w.shape[0]
    _require(w.shape[1] == k, "a and w differ in inner size")
    _require(out.shape == (m, n), "out must be [rows of a, rows of w]")
    if bias is not None:
        _dense(bias, "bias", torch.float32, 1)
        _require(bias.shape[0] == n, "bias length differs from rows of w")
    ldr = 0
    if residual is not None:
        _rows(residual, "residual", torch.float32)
        _require(residual.shape == (m, n), "residual differs from out in shape")
        ldr = residual.stride(0)
    _check(library().dli_gemm_f32_nt(_ptr(a), a.stride(0), _ptr(w), w.stride(0), _ptr(bias), _ptr(residual),
                                     ldr, _ptr(out), out.stride(0), m, n, k, _stream()), "gemm_f32")


SKINNY_STORE, SKINNY_SWIGLU, SKINNY_RESIDUAL, SKINNY_F32 = 0, 1, 2, 3


def skinny_gemm_supports(rows: int, k: int, dtype: torch.dtype) -> bool:
    """Whether the decode product kernel takes ``rows`` activation rows of width ``k``."""
    return dtype == torch.bfloat16 and 0 < rows <= 64 and k > 0 and k % 32 == 0


def skinny_gemm_shape(n: int, k: int, tiled: bool = False, units: int = 256) -> int:
    """Workgroup shape for ``n`` output features of depth ``k``: with few tiles of 16 features the
    waves of a workgroup split k, with many they split the tiles so that the activations are read
    once per 8 tiles. From cold-cache timings on MI355X (``units`` compute units); with tiled
    weights at the 1B, 1.7B and 3B sizes: four k-waves on one tile each where the tiles are no
    more than the compute units or fill them evenly with short rows (6.5 us against 6.8 and 7.4
    for q/k/v at the 1B sizes, 16.2 against 16.8 for gate and up), else on two tiles each, which
    halves the workgroups and with them the uneven last round (11.5 us against 13.9 for q/k/v
    at the 3B sizes, 8.6 against 10.1 at the 1.7B sizes)."""
    tiles = -(-n // 16)
    if tiled:
        if tiles >= 2048 and k >= 3072:
            return 2   # a vocabulary with long rows: no split of k
        if tiles <= units or (tiles % units == 0 and k <= 2048):
            return 0
        return 4
    if tiles >= 768:   # a vocabulary
        return 3
    return 1 if k >= 4096 else 0


def tiled_weights_help(w_rows: int, k: int, epilogue: int, device: torch.device) -> bool:
    """Whether a second copy of a ``[w_rows, k]`` weight in tile order (:func:`tile_weights`)
    would be used: the sizes allow it and steps of 5 to 16 rows run this product on the
    16x16-tile kernel."""
    n = w_rows // 2 if epilogue == SKINNY_SWIGLU else w_rows
    if k % 128 != 0 or n % 16 != 0 or n == 0:
        return False
    return skinny_gemm_plan(8, n, k, epilogue, device)[0] == "tiles16"


def tile_weights(w: torch.Tensor, whole_blocks: bool = True) -> torch.Tensor:
    """``w [n, k]`` (bfloat16, n % 16 == 0, k % 128 == 0) in the order in which the 16x16-tile
    kernel's lanes read it: ``t[tile][block][q][g][c][8] = w[16*tile + c][128*block + 32*g + 8*q + ...]``,
    so that each load of a wave is 1 KB of consecutive memory. Same number of elements, flat.
    ``whole_blocks=False`` takes any k % 8 == 0 and fills the last block of 128 with zeros (the copy
    then has ``n * padded_k(k)`` elements; only :func:`mid_gemm` reads such a copy)."""
    _dense(w, "w", torch.bfloat16, 2)
    n, k = w.shape
    if k % 128 != 0 and not whole_blocks:
        _require(k % 8 == 0, "tile order needs k % 8 == 0")
        w = torch.nn.functional.pad(w, (0, padded_k(k) - k))
        k = w.shape[1]
    _require(n % 16 == 0 and k % 128 == 0, "tile order needs n % 16 == 0 and k % 128 == 0")
    t = w.view(n // 16, 16, k // 128, 4, 4, 8)       # tile, c, block, g, q, 8
    return t.permute(0, 2, 4, 3, 1, 5).contiguous().view(-1)


def padded_k(k: int) -> int:
    """``k`` rounded up to whole blocks of 128."""
    return -(-k // 128) * 128


_compute_units: dict[int, int] = {}


def compute_units(device: torch.device) -> int:
    """Compute units of the device (256 on MI355X)."""
    return _units(device)


def _units(device: torch.device) -> int:
    index = device.index if device.index is not None else torch.cuda.current_device()
    if index not in _compute_units:
        _compute_units[index] = torch.cuda.get_device_properties(index).multi_processor_count
    return _compute_units[index]


def skinny_gemm_plan(rows: int, n: int, k: int, epilogue: int, device: torch.device,
                     blocks4: Optional[int] = None, tiled: bool = False) -> tuple[str, int, int]:
    """How :func:`skinny_gemm` runs a product: ``(kernel, shape, parts)``.

    ``"blocks4"`` is the 4x4-block kernel (at most 16 rows), ``"tiles16"`` the 16x16-tile kernel
    (at most 64 rows); ``shape`` is that kernel's workgroup shape. ``parts`` is the number of parts
    that the residual epilogue leaves of each row's sum of squares. The choice follows cold-cache
    timings on MI355X: the block kernel reads whole cache lines of the weights and only the rows of
    activations that exist, which wins for one to four rows; with more rows the activations'
    traffic grows and the tile kernel, which reads them once per 16 features, is ahead.
    ``tiled``: a copy of the weights in tile order is at hand (at most 16 rows); the tile kernel
    then reads whole lines too and takes over from two rows on, and below that where the
    product has few features.
    """
    if blocks4 is None and rows <= 16 and k % 8 == 0:
        # long rows and so few features that tiles of 16 would leave half the compute units idle
        # (2048 at the 1B sizes; not 3072 at the 3B sizes, where the tile kernel is ahead from 4 rows on)
        deep = k >= 4096 and -(-n // 16) * 2 <= _units(device)
        if deep:
            blocks4 = 1   # (the shape of 16 k-waves was ahead for one to four rows until the loads of
            #               a wave's chunks overlapped: now 9.8 against 10.8 us for down at the 1B sizes)
        elif rows <= 4:
            out_feats = n * (2 if epilogue == SKINNY_SWIGLU else 1)
            few = out_feats <= 16 * _units(device)
            if not (tiled and (rows >= 2 or few)):
                blocks4 = 1 if few else 0
    if blocks4 is not None:
        feats = int(library().dli_skinny4_tile_features(blocks4, epilogue))
        return "blocks4", blocks4, -(-n // feats)
    shape = skinny_gemm_shape(n, k, tiled and rows <= 16, _units(device))
    if tiled and rows <= MERGED_ROWS and shape == 0 and -(-n // 16) <= _units(device):
        # Few tiles and very few rows: eight k-waves are as fast as four (4.3 against 4.4 us for o at
        # the 1B sizes), and the o projection that merges the attention's runs of keys itself, whose
        # waves each merge the k they multiply, is faster with them; it has to add in the same order
        # as this one to give the same bits.
        shape = 1
    return "tiles16", shape, -(-n // 16)


def skinny_gemm(x: torch.Tensor, w: torch.Tensor, *, epilogue: int, out: Optional[torch.Tensor] = None,
                bias: Optional[torch.Tensor] = None, norm_w: Optional[torch.Tensor] = None, eps: float = 0.0,
                ssq_in: Optional[torch.Tensor] = None, stream: Optional[torch.Tensor] = None,
                ssq_out: Optional[torch.Tensor] = None, shape: Optional[int] = None,
                blocks4: Optional[int] = None, w_tiled: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """``y = xhat @ w.T`` for at most 64 rows of bfloat16 ``x``, with fused surroundings.

    ``norm_w``/``eps``/``ssq_in [parts, rows]``: xhat is the RMSNorm of x, the row sums of squares
    being given in parts. Epilogues: ``SKINNY_STORE`` (``out`` bfloat16 ``[rows, n]``),
    ``SKINNY_SWIGLU`` (``w`` is ``[2n, k]``: gate rows then up rows; ``out [rows, n]`` gets
    ``silu(gate) * up``), ``SKINNY_RESIDUAL`` (``stream [rows, n]`` becomes ``stream + y`` in place;
    the parts of its row sums of squares are returned as ``[parts, rows]``, in ``ssq_out`` if that
    is given with the shape :func:`skinny_gemm_plan` names), ``SKINNY_F32`` (``out`` float32).
    ``shape`` forces the 16x16-tile kernel with that workgroup shape, ``blocks4`` the 4x4-block
    kernel with that one (at most 16 rows). ``w_tiled``: the same weights in tile order
    (:func:`tile_weights`), read instead of ``w`` when the 16x16-tile kernel runs at most 16 rows.
    """
    _rows(x, "x", torch.bfloat16)
    _dense(w, "w", torch.bfloat16, 2)
    m, k = x.shape
    _require(w.shape[1] == k, "x and w differ in inner size")
    _require(skinny_gemm_supports(m, k, x.dtype), f"the decode product takes 1..64 rows and k % 32 == 0, not {m} x {k}")
    _require(x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0, "operands must be 16-byte aligned")
    n = w.shape[0] // 2 if epilogue == SKINNY_SWIGLU else w.shape[0]
    up_offset = n if epilogue == SKINNY_SWIGLU else 0
    if epilogue == SKINNY_SWIGLU:
        _require(w.shape[0] == 2 * n, "swiglu needs gate rows and up rows")
    if bias is not None:
        _dense(bias, "bias", torch.bfloat16, 1)
        _require(bias.shape[0] == w.shape[0], "bias length differs from rows of w")
    if k % 128 != 0:
        w_tiled = None   # a copy in whole blocks with a zero-filled last one: the 17-to-64-row kernel's alone
    if shape is not None:
        _require(shape in (0, 1, 2, 3, 4), "shape must be 0..4")
        kernel, a, n_parts = "tiles16", shape, -(-n // 16)
    else:
        if blocks4 is not None:
            _require(blocks4 in (0, 1, 2) and m <= 16 and k % 8 == 0, "blocks4 must be 0..2, with at most 16 rows")
        kernel, a, n_parts = skinny_gemm_plan(m, n, k, epilogue, x.device, blocks4,
                                              tiled=w_tiled is not None and m <= 16)
    tiled = w_tiled is not None and kernel == "tiles16" and m <= 16
    if tiled:
        _dense(w_tiled, "w_tiled", torch.bfloat16, 1)
        _require(w_tiled.numel() == w.numel() and k % 128 == 0 and n % 16 == 0 and w_tiled.data_ptr() % 16 == 0,
                 "w_tiled must hold the same weights in tile order (n % 16 == 0, k % 128 == 0)")
    parts = 0
    if norm_w is not None:
        _require(epilogue != SKINNY_RESIDUAL, "the residual epilogue takes no fused norm")
        _dense(norm_w, "norm_w", torch.float32, 1)
        _require(norm_w.shape[0] == k and norm_w.data_ptr() % 16 == 0, "norm weight must have k aligned values")
        _require(ssq_in is not None, "a fused norm needs the sums of squares")
        _dense(ssq_in, "ssq_in", torch.float32, 2)
        _require(ssq_in.shape[1] == m and ssq_in.shape[0] >= 1, "ssq_in must be [parts, rows]")
        parts = ssq_in.shape[0]
    ldo = lds = 0
    if epilogue == SKINNY_RESIDUAL:
        _require(stream is not None, "the residual epilogue needs stream")
        _rows(stream, "stream", torch.bfloat16)
        _require(stream.shape == (m, n), "stream must be [rows, n]")
        if ssq_out is None:
            ssq_out = torch.empty(n_parts, m, device=x.device, dtype=torch.float32)
        _dense(ssq_out, "ssq_out", torch.float32, 2)
        _require(ssq_out.shape == (n_parts, m), f"ssq_out must be [{n_parts}, rows] for this product")
        _require(stream.data_ptr() % 8 == 0, "stream must be 8-byte aligned")
        lds = stream.stride(0)
    else:
        _require(out is not None, "this epilogue needs out")
        _rows(out, "out", torch.float32 if epilogue == SKINNY_F32 else torch.bfloat16)
        _require(out.shape == (m, n), "out must be [rows, n]")
        _require(out.data_ptr() % 16 == 0, "out must be 16-byte aligned")
        ldo = out.stride(0)
    if kernel == "tiles16":
        _check(library().dli_skinny_gemm(
            _ptr(x), x.stride(0), _ptr(ssq_in), parts, _ptr(norm_w), float(eps), _ptr(w_tiled if tiled else w),
            _ptr(bias), _ptr(out), ldo, _ptr(stream), lds, _ptr(ssq_out), m, n, k, up_offset, epilogue, a,
            int(tiled), _stream()), "skinny_gemm")
    else:
        _check(library().dli_skinny4_gemm(
            _ptr(x), x.stride(0), _ptr(ssq_in), parts, _ptr(norm_w), float(eps), _ptr(w), _ptr(bias), _ptr(out), ldo,
            _ptr(stream), lds, _ptr(ssq_out), m, n, k, up_offset, epilogue, a, _stream()), "skinny4_gemm")
    return ssq_out if epilogue == SKINNY_RESIDUAL else None


def head_gemm_supports(rows: int, n: int, k: int, dtype: torch.dtype) -> bool:
    """Whether :func:`head_gemm` takes this product (at most 16 rows, ``n % 16 == 0``, ``k`` one
    of 1024, 2048, 3072, 4096)."""
    return dtype == torch.bfloat16 and bool(library().dli_head_gemm_supports(int(rows), int(n), int(k)))


def head_gemm(x: torch.Tensor, w_tiled: torch.Tensor, out: torch.Tensor, norm_w: Optional[torch.Tensor] = None,
              eps: float = 0.0, ssq_in: Optional[torch.Tensor] = None, workgroups: int = 0,
              best: Optional[tuple[torch.Tensor, torch.Tensor]] = None) -> int:
    """``out = xhat @ w.T`` as float32 for at most 16 rows and the many rows of a vocabulary:
    workgroups that stay for the whole launch walk the tiles of ``w_tiled`` (:func:`tile_weights`
    of ``w [n, k]``) in turn, each wave keeping its normalised activations in registers. ``norm_w``,
    ``eps``, ``ssq_in [parts, rows]``: the RMSNorm of ``x`` as in :func:`skinny_gemm`. The sums are
    those of :func:`skinny_gemm` with ``shape=4``, to the bit. ``workgroups``: how many (0: one per
    compute unit). ``best``: float32 values and int32 indices (the scratch of :func:`sample_scratch`); each
    workgroup then leaves every row's best logit and its lowest index among the logits it made, as
    ``[rows, parts]`` at the start of both, and the number of parts comes back (the first stage of
    :func:`sample_and_advance`'s argmax); without it 0."""
    _rows(x, "x", torch.bfloat16)
    m, k = x.shape
    _rows(out, "out", torch.float32)
    n = out.shape[1]
    _require(out.shape[0] == m, "out must be [rows, n]")
    _require(head_gemm_supports(m, n, k, x.dtype), f"the logits kernel takes 1..16 rows, n % 16 == 0 and k of 1024 to "
             f"4096 in steps of 1024, not {m} x {k} -> {n}")
    _dense(w_tiled, "w_tiled", torch.bfloat16, 1)
    _require(w_tiled.numel() == n * k and w_tiled.data_ptr() % 16 == 0, "w_tiled must hold [n, k] in tile order")
    _require(x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and out.stride(0) % 4 == 0 and out.data_ptr() % 16 == 0,
             "operands must be 16-byte aligned")
    parts = 0
    if norm_w is not None:
        _dense(norm_w, "norm_w", torch.float32, 1)
        _require(norm_w.shape[0] == k and norm_w.data_ptr() % 16 == 0, "norm weight must have k aligned values")
        _require(ssq_in is not None, "a fused norm needs the sums of squares")
        _dense(ssq_in, "ssq_in", torch.float32, 2)
        _require(ssq_in.shape[1] == m and ssq_in.shape[0] >= 1, "ssq_in must be [parts, rows]")
        parts = ssq_in.shape[0]
    groups = 0
    if best is not None:
        groups = int(library().dli_head_gemm_workgroups(n, int(workgroups)))
        _dense(best[0], "best values", torch.float32)
        _dense(best[1], "best indices", torch.int32)
        _require(best[0].numel() >= m * groups and best[1].numel() >= m * groups, "the argmax's scratch is too small")
    _check(library().dli_head_gemm(_ptr(x), x.stride(0), _ptr(ssq_in), parts, _ptr(norm_w), float(eps), _ptr(w_tiled),
                                   _ptr(out), out.stride(0), m, n, k, int(workgroups),
                                   _ptr(best[0]) if best is not None else None,
                                   _ptr(best[1]) if best is not None else None, _stream()), "head_gemm")
    return groups


MERGED_ROWS, MERGED_SPLITS, _MERGED_RANGE = 4, 16, 512  # csrc/skinny_gemm.hip: MERGE_ROWS, MERGE_SPLITS, MERGE_RANGE


def skinny_gemm_merged_supports(rows: int, n: int, heads: int, head_dim: int, splits: int,
                                device: torch.device) -> bool:
    """Whether :func:`skinny_gemm_merged` takes this o projection: few rows, few runs of keys, a
    product that the 16x16-tile kernel runs with k split over the waves of a workgroup."""
    k = heads * head_dim
    if not (0 < rows <= MERGED_ROWS and 2 <= splits <= MERGED_SPLITS and head_dim % 4 == 0 and k % 128 == 0
            and n % 16 == 0):
        return False
    return _merged_shape(rows, n, k, device) is not None


def _merged_shape(rows: int, n: int, k: int, device: torch.device) -> Optional[int]:
    """The workgroup shape (0: four k-waves, 1: eight) with which the merging o projection runs:
    that of the plain product with the residual sum, so that both add in the same order, or None
    if that one runs on another kernel or a wave's run of k does not fit the merge's buffer."""
    kernel, shape, _ = skinny_gemm_plan(rows, n, k, SKINNY_RESIDUAL, device, tiled=True)
    if kernel != "tiles16" or shape not in (0, 1):
        return None
    return shape if -(-(k // 128) // (4 if shape == 0 else 8)) * 128 <= _MERGED_RANGE else None


def skinny_gemm_merged(part_o: torch.Tensor, part_ml: torch.Tensor, splits: int, heads: int, head_dim: int,
                       w_tiled: torch.Tensor, stream: torch.Tensor, bias: Optional[torch.Tensor] = None,
                       ssq_out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``stream += merge(part_o, part_ml) @ w.T (+ bias)`` for at most four rows: the o projection
    of a decode step fed with the partial results that :func:`attention_decode` leaves with
    ``merge=False`` (``part_o [rows, heads, splits, head_dim]``, ``part_ml [rows, heads, splits, 2]``),
    merged inside the product's kernel with the arithmetic of the merge kernel. Returns the parts
    of the rows' sums of squares like the residual epilogue of :func:`skinny_gemm`."""
    _rows(stream, "stream", torch.bfloat16)
    m, n = stream.shape
    k = heads * head_dim
    _require(skinny_gemm_merged_supports(m, n, heads, head_dim, splits, stream.device),
             f"the merging o projection takes 1..{MERGED_ROWS} rows and 2..{MERGED_SPLITS} runs of keys, "
             f"not {m} rows, {splits} runs, {heads} heads of {head_dim}")
    _dense(part_o, "part_o", torch.float32)
    _dense(part_ml, "part_ml", torch.float32)
    _require(part_o.numel() >= m * heads * splits * head_dim and part_ml.numel() >= m * heads * splits * 2,
             "partial-result buffers are too small")
    _require(part_o.data_ptr() % 16 == 0 and part_ml.data_ptr() % 8 == 0, "partial results must be 16-byte aligned")
    _dense(w_tiled, "w_tiled", torch.bfloat16, 1)
    _require(w_tiled.numel() == n * k and w_tiled.data_ptr() % 16 == 0, "w_tiled must hold [n, heads*head_dim] in tile order")
    if bias is not None:
        _dense(bias, "bias", torch.bfloat16, 1)
        _require(bias.shape[0] == n, "bias length differs from rows of w")
    _, _, n_parts = skinny_gemm_plan(m, n, k, SKINNY_RESIDUAL, stream.device, tiled=True)
    shape = _merged_shape(m, n, k, stream.device)
    if ssq_out is None:
        ssq_out = torch.empty(n_parts, m, device=stream.device, dtype=torch.float32)
    _dense(ssq_out, "ssq_out", torch.float32, 2)
    _require(ssq_out.shape == (n_parts, m), f"ssq_out must be [{n_parts}, rows] for this product")
    _require(stream.data_ptr() % 8 == 0, "stream must be 8-byte aligned")
    _check(library().dli_skinny_gemm_merged(
        _ptr(part_o), _ptr(part_ml), int(splits), int(heads), int(head_dim), _ptr(w_tiled), _ptr(bias), _ptr(stream),
        stream.stride(0), _ptr(ssq_out), m, n, shape, _stream()), "skinny_gemm_merged")
    return ssq_out


_GEMM_WORKSPACE_BYTES = 64 << 20
_gemm_workspaces: dict[int, torch.Tensor] = {}


MID_PARTIAL, MID_SWIGLU, MID_STORE = 0, 1, 2
MID_ROWS = 64


def mid_gemm_supports(rows: int, k: int, dtype: torch.dtype) -> bool:
    """Whether the product kernel for decode steps of up to 64 rows takes this shape."""
    return dtype == torch.bfloat16 and 0 < rows <= MID_ROWS and k > 0 and k % 8 == 0


MID_SHAPES = ((4, 1), (4, 2))              # (waves, kwaves) that are built for the plain products
MID_SHAPES_GATED = ((2, 1), (2, 2), (2, 4))  # and for the gated one


def mid_gemm_plan(n: int, k: int, epilogue: int, units: int, rows: int = 64) -> tuple[int, int, int]:
    """``(waves, kwaves, splits)`` for a product of ``n`` output features of depth ``k``.

    A workgroup has ``waves`` feature tiles of 16 and ``kwaves`` waves on each, which split its
    range of k; ``splits`` workgroups share a feature tile's whole k (a gated product is never
    split: its epilogue needs whole sums). These launches last a few trips to memory, so the plan
    aims at one workgroup on every compute unit with eight to sixteen waves, each with few blocks
    of 128 k to fetch."""
    tiles, blocks = -(-n // 16), -(-k // 128)
    if epilogue == MID_SWIGLU:
        # (two against four k-waves a tile, cold weights: 21.1 and 21.4 us at 32 rows, 23.4 and 23.0
        # at 48, 28.7 and 26.1 at 64 at the 1B sizes; with k of 3072 24.8 and 24.5, 29.9 and 27.2, 37.4
        # and 31.9. In a decode step of 64 rows, where part of the weights is warm: 2.93 to 2.96 ms with
        # either at the 1B sizes, 5.48 against 5.39 ms at the 3B sizes. Four tiles a workgroup, or one,
        # were behind at every number of rows.)
        return 2, (4 if rows > 32 and blocks >= 24 else 2) if blocks >= 2 else 1, 1
    if epilogue == MID_STORE:
        return 4, 2 if blocks >= 2 else 1, 1
    waves = 4
    groups = -(-tiles // waves)
    splits = max(1, min(blocks, round(units / groups)))
    kwaves = 2 if blocks // splits >= 2 else 1
    return waves, kwaves, splits


def mid_tiles_help(w_rows: int, k: int, epilogue: int) -> bool:
    """Whether decode steps of 17 to 64 rows would read a copy of a ``[w_rows, k]`` weight in tile
    order (:func:`tile_weights`, of whole blocks of k, zero-filled): the layer products do, where
    the features tile."""
    n = w_rows // 2 if epilogue == SKINNY_SWIGLU else w_rows
    return epilogue in (SKINNY_STORE, SKINNY_SWIGLU, SKINNY_RESIDUAL) and k % 8 == 0 and n % 16 == 0 and n > 0


def mid_gemm(x: torch.Tensor, w: torch.Tensor, *, epilogue: int, tiled: bool = False, n: Optional[int] = None,
             out: Optional[torch.Tensor] = None, bias: Optional[torch.Tensor] = None,
             norm_w: Optional[torch.Tensor] = None, eps: float = 0.0, ssq_in: Optional[torch.Tensor] = None,
             splits: Optional[int] = None, waves: Optional[int] = None,
             kwaves: Optional[int] = None) -> torch.Tensor:
    """``y = xhat @ w.T`` for at most 64 rows of bfloat16 ``x [rows, k]``, k a multiple of 8.

    ``w`` is ``[n, k]`` (``[2n, k]``, gate rows then up rows, for ``MID_SWIGLU``), or the same in
    tile order (:func:`tile_weights`, flat; of whole blocks, zero-filled where k is no multiple
    of 128) with ``tiled`` and ``n`` given. ``norm_w``/``eps``/
    ``ssq_in [parts, rows]``: xhat is the RMSNorm of x. ``MID_PARTIAL`` returns float32
    ``[splits, rows, n]`` whose sum over the splits, in their order, is the product (no bias; the
    finishing kernels add them up); ``MID_STORE`` and ``MID_SWIGLU`` return bfloat16 ``[rows, n]``.
    """
    _rows(x, "x", torch.bfloat16)
    m, k = x.shape
    _require(mid_gemm_supports(m, k, x.dtype), f"this product takes 1..64 rows and k % 8 == 0, not {m} x {k}")
    _require(x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0, "operands must be 16-byte aligned")
    sets = 2 if epilogue == MID_SWIGLU else 1
    if tiled:
        _dense(w, "w", torch.bfloat16, 1)
        _require(n is not None and n % 16 == 0 and w.numel() == sets * n * padded_k(k),
                 "tiled weights need n % 16 == 0 features of depth k, in whole blocks of 128")
    else:
        _dense(w, "w", torch.bfloat16, 2)
        _require(w.shape[1] == k and w.shape[0] % sets == 0, "x and w differ in inner size")
        n = w.shape[0] // sets
    _require(epilogue in (MID_PARTIAL, MID_SWIGLU, MID_STORE), "unknown epilogue")
    plan_waves, plan_kwaves, plan_splits = mid_gemm_plan(n, k, epilogue, _units(x.device), m)
    waves = plan_waves if waves is None else waves
    kwaves = plan_kwaves if kwaves is None else kwaves
    splits = plan_splits if splits is None else splits
    built = MID_SHAPES_GATED if epilogue == MID_SWIGLU else MID_SHAPES
    _require((waves, kwaves) in built and 1 <= splits <= -(-k // 128),
             f"(waves, kwaves) must be one of {built}, splits 1..k/128")
    if epilogue == MID_PARTIAL:
        _require(bias is None and n % 4 == 0, "partial products take no bias, n % 4 == 0")
        if out is None:
            out = torch.empty(splits, m, n, device=x.device, dtype=torch.float32)
        _dense(out, "out", torch.float32, 3)
        _require(out.shape == (splits, m, n), "out must be [splits, rows, n]")
        ldo = n
    else:
        _require(splits == 1, "only partial products are split")
        if out is None:
            out = torch.empty(m, n, device=x.device, dtype=torch.bfloat16)
        _rows(out, "out", torch.bfloat16)
        _require(out.shape == (m, n) and out.stride(0) % 4 == 0 and out.data_ptr() % 8 == 0, "out must be [rows, n], rows 8-byte aligned")
        ldo = out.stride(0)
    if bias is not None:
        _dense(bias, "bias", torch.bfloat16, 1)
        _require(bias.shape[0] == sets * n, "bias length differs from rows of w")
    parts = 0
    if norm_w is not None:
        _dense(norm_w, "norm_w", torch.float32, 1)
        _require(norm_w.shape[0] == k and norm_w.data_ptr() % 16 == 0, "norm weight must have k aligned values")
        _require(ssq_in is not None, "a fused norm needs the sums of squares")
        _dense(ssq_in, "ssq_in", torch.float32, 2)
        _require(ssq_in.shape[1] == m and ssq_in.shape[0] >= 1, "ssq_in must be [parts, rows]")
        parts = ssq_in.shape[0]
    _check(library().dli_mid_gemm(
        _ptr(x), x.stride(0), _ptr(ssq_in) if norm_w is not None else None, parts, _ptr(norm_w), float(eps), _ptr(w),
        int(tiled), _ptr(bias), _ptr(out), ldo, m, n, k, n if epilogue == MID_SWIGLU else 0, epilogue, splits, waves,
        kwaves, _stream()), "mid_gemm")
    return out


MID_NORMED_WIDTH = 8192  # the widest row that the normalising finish holds in one workgroup


def mid_finish_residual(partial: torch.Tensor, stream: torch.Tensor, bias: Optional[torch.Tensor] = None,
                        ssq_out: Optional[torch.Tensor] = None, norm_w: Optional[torch.Tensor] = None,
                        eps: float = 0.0, normed_out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``stream += sum over splits of partial (+ bias)`` in place (32-bit sum, the product rounded
    to bfloat16 first, as the fused epilogue of the few-row product does), and each row's sum of
    squares of the new stream, in parts of 1024 features, as float32 ``[parts, rows]`` for the norm
    that follows.

    With ``norm_w`` (float32 ``[n]``, ``n <= MID_NORMED_WIDTH``), ``eps`` and ``normed_out``
    (bfloat16 ``[rows, n]``) that norm is applied here as well: ``normed_out`` gets the RMSNorm of
    the new stream with the two roundings of the fused norm prologues, for a product that then
    reads it as it is; the sums of squares come back whole, as ``[1, rows]``."""
    _dense(partial, "partial", torch.float32, 3)
    _rows(stream, "stream", torch.bfloat16)
    splits, m, n = partial.shape
    _require(stream.shape == (m, n) and n % 4 == 0 and stream.stride(0) % 4 == 0 and stream.data_ptr() % 8 == 0,
             "stream must be [rows, n] with n % 4 == 0")
    if bias is not None:
        _dense(bias, "bias", torch.bfloat16, 1)
        _require(bias.shape[0] == n, "bias length differs from n")
    parts = 1 if norm_w is not None else -(-n // 1024)
    if ssq_out is None:
        ssq_out = torch.empty(parts, m, device=stream.device, dtype=torch.float32)
    _dense(ssq_out, "ssq_out", torch.float32, 2)
    _require(ssq_out.shape == (parts, m), f"ssq_out must be [{parts}, rows]")
    if norm_w is not None:
        _dense(norm_w, "norm_w", torch.float32, 1)
        _require(norm_w.shape[0] == n and norm_w.data_ptr() % 16 == 0, "norm weight must have n aligned values")
        _require(n <= MID_NORMED_WIDTH, f"rows wider than {MID_NORMED_WIDTH} are normalised by the product that reads them")
        _require(normed_out is not None, "the normalised rows need normed_out")
        _rows(normed_out, "normed_out", torch.bfloat16)
        _require(normed_out.shape == (m, n) and normed_out.stride(0) % 4 == 0 and normed_out.data_ptr() % 8 == 0,
                 "normed_out must be [rows, n]")
        _check(library().dli_mid_finish_residual_normed(
            _ptr(partial), splits, _ptr(bias), _ptr(stream), stream.stride(0), _ptr(ssq_out), _ptr(norm_w), float(eps),
            _ptr(normed_out), normed_out.stride(0), m, n, _stream()), "mid_finish_residual")
        return ssq_out
    _check(library().dli_mid_finish_residual(_ptr(partial), splits, _ptr(bias), _ptr(stream), stream.stride(0),
                                             _ptr(ssq_out), m, n, _stream()), "mid_finish_residual")
    return ssq_out


def mid_finish_qkv(partial: torch.Tensor, out: torch.Tensor, angles: torch.Tensor, slots: torch.Tensor,
                   k_pages: torch.Tensor, v_pages: torch.Tensor, q_heads: int,
                   bias: Optional[torch.Tensor] = None) -> None:
    """The fused q/k/v projection's partial products ``[splits, rows, (q + 2 kv) * head_dim]``, in
    the feature order of :func:`tile_weights_qkv_rope` (``bias`` too): summed over the splits,
    rotated, q written to ``out[:, :q_heads * head_dim]`` in the usual order, rotated k and v into
    the cache pages at ``slots`` (negative: not cached). ``angles``: :func:`rope_angles`."""
    _dense(partial, "partial", torch.float32, 3)
    _rows(out, "out", torch.bfloat16)
    splits, m, n = partial.shape
    _dense(k_pages, "k_pages", torch.bfloat16, 4)
    _dense(v_pages, "v_pages", torch.bfloat16, 4)
    _, kv_heads, page_size, head_dim = k_pages.shape
    _require(v_pages.shape == (k_pages.shape[0], kv_heads, head_dim, page_size), "v_pages must be [pages, kv_heads, head_dim, page_size]")
    _require(head_dim % 16 == 0 and n == (q_heads + 2 * kv_heads) * head_dim, "partial width differs from (q + 2 kv) * head_dim")
    _require(out.shape[0] == m and out.shape[1] >= q_heads * head_dim and out.stride(0) % 4 == 0 and out.data_ptr() % 8 == 0,
             "out must hold the q heads of every row")
    _dense(angles, "angles", torch.float32, 3)
    _require(angles.shape == (m, 2, head_dim // 2), "angles must be [rows, 2, head_dim / 2]")
    _dense(slots, "slots", torch.int32, 1)
    _require(slots.shape[0] == m, "slots differ from partial in rows")
    if bias is not None:
        _dense(bias, "bias", torch.bfloat16, 1)
        _require(bias.shape[0] == n, "bias length differs from the features")
    _check(library().dli_mid_finish_qkv(_ptr(partial), splits, _ptr(bias), _ptr(angles), _ptr(slots), _ptr(out),
                                        out.stride(0), _ptr(k_pages), _ptr(v_pages), m, q_heads, kv_heads, head_dim,
                                        page_size, _stream()), "mid_finish_qkv")


def gemm_workspace(device: torch.device) -> tuple[torch.Tensor, int]:
    """The device buffer that the vendor library's products may use, and its size in bytes."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    workspace = _gemm_workspaces.get(index)
    if workspace is None:
        workspace = _gemm_workspaces[index] = torch.empty(_GEMM_WORKSPACE_BYTES, dtype=torch.uint8, device=device)
    return workspace, _GEMM_WORKSPACE_BYTES


def prenorm_blocks(x: torch.Tensor, blocks, count: int, step) -> bool:
    """Run ``count`` pre-norm blocks (ctypes array of ``parts.native.BlockArgs``) on the residual
    stream ``x`` for the step described by ``step`` (``parts.native.StepArgs``), all launches
    issued from C. Whoever fills the structures has checked shapes and sizes. False, with nothing
    launched, where an argument or a product's shape is refused."""
    _rows(x, "x", torch.bfloat16)
    status = library().dli_prenorm_blocks_bf16(_ptr(x), ctypes.cast(blocks, ctypes.c_void_p), int(count),
                                               ctypes.cast(ctypes.pointer(step), ctypes.c_void_p), _stream())
    if status == -1:
        return False
    _check(status, "prenorm_blocks")
    return True


def gemm_bf16(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, bias: Optional[torch.Tensor] = None) -> bool:
    """``out = x @ w.T (+ bias)`` for bfloat16 matrices with contiguous rows through the vendor
    library, 32-bit accumulation, the bias added before the one rounding (``out`` float32: the
    sums as they are, unrounded). The library's choice
    of kernel is looked up once per shape. Returns False where the library has no kernel for the
    shape (nothing was computed then)."""
    _rows(x, "x", torch.bfloat16)
    _rows(w, "w", torch.bfloat16)
    _require(out.dtype in (torch.bfloat16, torch.float32), "out must be bfloat16 or float32")
    _rows(out, "out", out.dtype)
    rows, k = x.shape
    feats = w.shape[0]
    _require(w.shape[1] == k and out.shape == (rows, feats), "x [n, k], w [m, k] and out [n, m] do not fit")
    if bias is not None:
        _dense(bias, "bias", torch.bfloat16, 1)
        _require(bias.shape[0] == feats, "bias length differs from rows of w")
    index = x.device.index if x.device.index is not None else torch.cuda.current_device()
    workspace = _gemm_workspaces.get(index)
    if workspace is None:
        workspace = _gemm_workspaces[index] = torch.empty(_GEMM_WORKSPACE_BYTES, dtype=torch.uint8, device=x.device)
    call = library().dli_gemm_bf16 if out.dtype == torch.bfloat16 else library().dli_gemm_bf16_f32
    status = call(_ptr(x), x.stride(0), _ptr(w), w.stride(0), _ptr(bias), _ptr(out), out.stride(0),
                  rows, feats, k, _ptr(workspace), _GEMM_WORKSPACE_BYTES, index, _stream())
    if status == -1:
        return False
    _check(status, "gemm_bf16")
    return True


def qkv_rope_feature_order(q_heads: int, kv_heads: int, head_dim: int) -> torch.Tensor:
    """The order of the fused projection's features in which :func:`skinny_gemm_qkv_rope` wants
    its weights and bias: tile ``t`` of a q or k head holds the head's dimensions ``8t..8t+7`` and
    ``half+8t..half+8t+7`` (eight rotary pairs); v heads keep their order. int64 ``[features]``."""
    _require(head_dim % 16 == 0 and q_heads > 0 and kv_heads > 0, "heads of a multiple of 16 dimensions")
    half = head_dim // 2
    within = torch.tensor([(8 * (f // 16) + f % 8) + (half if f % 16 >= 8 else 0) for f in range(head_dim)])
    heads = []
    for h in range(q_heads + 2 * kv_heads):
        local = within if h < q_heads + kv_heads else torch.arange(head_dim)
        heads.append(h * head_dim + local)
    return torch.cat(heads)


def tile_weights_qkv_rope(w: torch.Tensor, q_heads: int, kv_heads: int, head_dim: int) -> torch.Tensor:
    """The fused q/k/v matrix in tile order (:func:`tile_weights`) with the features in
    :func:`qkv_rope_feature_order`."""
    _dense(w, "w", torch.bfloat16, 2)
    _require(w.shape[0] == (q_heads + 2 * kv_heads) * head_dim, "w must hold the q, k and v heads")
    order = qkv_rope_feature_order(q_heads, kv_heads, head_dim).to(w.device)
    return tile_weights(w[order].contiguous(), whole_blocks=False)


def skinny_gemm_qkv_rope(x: torch.Tensor, w_tiled: torch.Tensor, q_out: torch.Tensor, angles: torch.Tensor,
                         slots: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, q_heads: int, *,
                         bias: Optional[torch.Tensor] = None, norm_w: Optional[torch.Tensor] = None,
                         eps: float = 0.0, ssq_in: Optional[torch.Tensor] = None,
                         shape: Optional[int] = None) -> None:
    """The fused q/k/v projection of at most 16 decode rows with rotation and cache write inside:
    ``q_out[row, head*head_dim + dim]`` (a ``[rows, >= q_heads*head_dim]`` bfloat16 buffer) gets the
    rotated queries; the rotated keys and the values go to the pages at ``slots[row]`` (negative:
    not cached). ``w_tiled`` comes from :func:`tile_weights_qkv_rope`, ``bias`` (optional) is in
    :func:`qkv_rope_feature_order`, ``angles [rows, 2, head_dim/2]`` from :func:`rope_angles`.
    ``norm_w``/``eps``/``ssq_in`` as in :func:`skinny_gemm`."""
    _rows(x, "x", torch.bfloat16)
    m, k = x.shape
    _dense(k_pages, "k_pages", torch.bfloat16, 4)
    _dense(v_pages, "v_pages", torch.bfloat16, 4)
    pages, kv_heads, page_size, head_dim = k_pages.shape
    _require(v_pages.shape == (pages, kv_heads, head_dim, page_size), "v_pages must be [pages, kv_heads, head_dim, page_size]")
    n = (q_heads + 2 * kv_heads) * head_dim
    _require(0 < m <= 16 and k % 128 == 0 and head_dim % 16 == 0 and q_heads > 0,
             f"this product takes 1..16 rows, k % 128 == 0 and head_dim % 16 == 0, not {m} x {k}, {head_dim}")
    _dense(w_tiled, "w_tiled", torch.bfloat16, 1)
    _require(w_tiled.numel() == n * k and w_tiled.data_ptr() % 16 == 0, "w_tiled must hold [(q + 2 kv) * head_dim, k]")
    _require(x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0, "x must be 16-byte aligned")
    _rows(q_out, "q_out", torch.bfloat16)
    _require(q_out.shape[0] == m and q_out.shape[1] >= q_heads * head_dim and q_out.stride(0) % 8 == 0
             and q_out.data_ptr() % 16 == 0, "q_out must be [rows, >= q_heads * head_dim], 16-byte aligned")
    _dense(angles, "angles", torch.float32, 3)
    _require(angles.shape == (m, 2, head_dim // 2) and angles.data_ptr() % 16 == 0, "angles must be [rows, 2, head_dim/2]")
    _dense(slots, "slots", torch.int32, 1)
    _require(slots.shape[0] == m, "one slot per row")
    if bias is not None:
        _dense(bias, "bias", torch.bfloat16, 1)
        _require(bias.shape[0] == n, "bias length differs from the features")
    parts = 0
    if norm_w is not None:
        _dense(norm_w, "norm_w", torch.float32, 1)
        _require(norm_w.shape[0] == k and norm_w.data_ptr() % 16 == 0, "norm weight must have k aligned values")
        _require(ssq_in is not None, "a fused norm needs the sums of squares")
        _dense(ssq_in, "ssq_in", torch.float32, 2)
        _require(ssq_in.shape[1] == m and ssq_in.shape[0] >= 1, "ssq_in must be [parts, rows]")
        parts = ssq_in.shape[0]
    if shape is None:
        shape = skinny_gemm_shape(n, k, tiled=True, units=_units(x.device))
        if shape == 0:
            shape = 1  # with the rotation in its epilogue eight k-waves are ahead (7.0 against 7.7 us at the 1B sizes)
    _require(shape in (0, 1, 2, 3, 4), "shape must be 0..4")
    _check(library().dli_skinny_gemm_qkv_rope(
        _ptr(x), x.stride(0), _ptr(ssq_in), parts, _ptr(norm_w), float(eps), _ptr(w_tiled), _ptr(bias), _ptr(q_out),
        q_out.stride(0), _ptr(angles), _ptr(slots), _ptr(k_pages), _ptr(v_pages), m, k, q_heads, kv_heads, head_dim,
        page_size, shape, _stream()), "skinny_gemm_qkv_rope")


def embedding_ssq(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor, ssq: torch.Tensor) -> None:
    """``out[t] = table[ids[t]]`` and ``ssq[0, t] = sum(out[t]^2)`` (bfloat16 table)."""
    _dense(table, "table", torch.bfloat16, 2)
    _dense(ids, "ids", torch.int32, 1)
    _dense(out, "out", torch.bfloat16, 2)
    _dense(ssq, "ssq", torch.float32, 2)
    _require(out.shape == (ids.shape[0], table.shape[1]) and ssq.shape == (1, ids.shape[0]),
             "out [len(ids), width], ssq [1, len(ids)]")
    _check(library().dli_embedding_ssq(_ptr(table), _ptr(ids), _ptr(out), _ptr(ssq), ids.shape[0], table.shape[1],
                                       _stream()), "embedding_ssq")

# ----------------------------------------------------------------------------- attention

def attention_generic_tile_rows(head_dim: int) -> int:
    rows = library().dli_attention_generic_tile_rows(head_dim)
    if rows <= 0:
        raise KernelArgumentError(
            f"attention takes head_dim in steps of 16 up to 256, not {head_dim}")
    return rows


def attention_generic(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, out: torch.Tensor,
                      q_start: torch.Tensor, kv_len: torch.Tensor, block_tables: torch.Tensor,
                      tile_entry: torch.Tensor, tile_q0: torch.Tensor, q_heads: int, scale: float,
                      window: int = 0) -> None:
    """Paged causal attention for a batch of portions (vector units, 32-bit arithmetic).

    ``q`` and ``out`` are ``[tokens, q_heads*head_dim]`` (rows contiguous, any row stride);
    ``q_start [entries+1]``, ``kv_len [entries]``, ``block_tables [entries, width]`` describe the
    requests; ``tile_entry/tile_q0`` list the query tiles of ``attention_generic_tile_rows`` rows.
    """
    _dense(k_pages, "k_pages", ndim=4)
    dtype = k_pages.dtype
    _rows(q, "q", dtype)
    _rows(out, "out", dtype)
    pages, kv_heads, page_size, head_dim = k_pages.shape
    _dense(v_pages, "v_pages", dtype, 4)
    _require(v_pages.shape == (pages, kv_heads, head_dim, page_size),
             "v_pages must be [pages, kv_heads, head_dim, page_size]")
    _require(q.shape[1] == q_heads * head_dim and out.shape == q.shape, "q/out must be [tokens, q_heads*head_dim]")
    _require(q_heads % kv_heads == 0, "query heads are not a multiple of kv heads")
    for name, t in (("q_start", q_start), ("kv_len", kv_len), ("tile_entry", tile_entry), ("tile_q0", tile_q0)):
        _dense(t, name, torch.int32, 1)
    _dense(block_tables, "block_tables", torch.int32, 2)
    entries = kv_len.shape[0]
    _require(q_start.shape[0] == entries + 1 and block_tables.shape[0] >= entries,
             "q_start/kv_len/block_tables disagree on the number of requests")
    _require(tile_entry.shape == tile_q0.shape, "tile lists differ in length")
    _check(library().dli_attention_generic(
        _ptr(q), q.stride(0), _ptr(k_pages), _ptr(v_pages), _ptr(out), out.stride(0), _ptr(q_start),
        _ptr(kv_len), _ptr(block_tables), block_tables.stride(0), _ptr(tile_entry), _ptr(tile_q0),
        tile_entry.shape[0], q_heads, kv_heads, head_dim, page_size, float(scale), int(window),
        _is_bf16(dtype), _stream()), "attention_generic")



def attention_mfma_supports(head_dim: int, page_size: int, dtype: torch.dtype) -> bool:
    """Whether the matrix-core attention kernels take this shape (else: the generic kernel)."""
    return dtype == torch.bfloat16 and bool(library().dli_attention_mfma_supports(head_dim, page_size))


def attention_prefill_tile_rows(head_dim: int, q_heads: int, kv_heads: int) -> int:
    """Queries per tile of the tile list that :func:`attention_prefill` expects for this shape."""
    rows = int(library().dli_attention_prefill_tile_rows(head_dim, q_heads, kv_heads))
    _require(rows > 0, "query heads are not a multiple of kv heads")
    return rows


def attention_prefill_cut_floats(head_dim: int, q_heads: int, kv_heads: int) -> int:
    """float32 values that :func:`attention_prefill` wants in ``cut_buf`` per run of a tile whose
    keys are cut into runs; 0 where this shape's kernel cuts no tiles."""
    n = int(library().dli_attention_prefill_cut_floats(head_dim, q_heads, kv_heads))
    _require(n >= 0, "query heads are not a multiple of kv heads")
    return n


def attention_prefill_max_cuts() -> int:
    """The most runs that :func:`attention_prefill` lets a tile's keys be cut into."""
    return int(library().dli_attention_prefill_max_cuts())


def _check_paged(q, k_pages, v_pages, out, q_heads):
    _dense(k_pages, "k_pages", torch.bfloat16, 4)
    _rows(q, "q", torch.bfloat16)
    _rows(out, "out", torch.bfloat16)
    pages, kv_heads, page_size, head_dim = k_pages.shape
    _dense(v_pages, "v_pages", torch.bfloat16, 4)
    _require(v_pages.shape == (pages, kv_heads, head_dim, page_size),
             "v_pages must be [pages, kv_heads, head_dim, page_size]")
    _require(q.shape[1] == q_heads * head_dim and out.shape == q.shape, "q/out must be [rows, q_heads*head_dim]")
    _require(q_heads % kv_heads == 0, "query heads are not a multiple of kv heads")
    _require(q.stride(0) % 4 == 0 and out.stride(0) % 4 == 0 and q.data_ptr() % 8 == 0 and out.data_ptr() % 8 == 0,
             "q/out rows must be 8-byte aligned")
    _require(bool(library().dli_attention_mfma_supports(head_dim, page_size)),
             f"the matrix-core attention takes head_dim 16..128 in steps of 16 and pages of a multiple of 16, "
             f"not head_dim {head_dim}, page size {page_size}")
    return kv_heads, page_size, head_dim


def attention_decode(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, out: Optional[torch.Tensor],
                     kv_len: torch.Tensor, block_tables: torch.Tensor, q_heads: int, scale: float,
                     window: int = 0, splits: int = 1, part_o: Optional[torch.Tensor] = None,
                     part_ml: Optional[torch.Tensor] = None, merge: bool = True,
                     arrivals: Optional[torch.Tensor] = None) -> None:
    """Decode attention: row ``e`` of ``q`` is request ``e``'s single query over its ``kv_len[e]`` keys.

    With ``splits > 1`` each request's keys are cut into that many runs whose partial results go
    through ``part_o [rows, q_heads, splits, head_dim]`` and ``part_ml [rows, q_heads, splits, 2]``
    (float32) and are merged by a second kernel; with ``merge=False`` (``splits > 1`` only) they
    are left there for :func:`skinny_gemm_merged` and ``out`` is not written (it may be None).
    ``arrivals``: int32 counters (one per request, kv head and 16 query heads of its group; zero before
    the first launch, and every launch leaves them zero) with which the launch merges by itself, the
    workgroup that finishes last doing the second kernel's work with the same result to the bit
    (up to :data:`SELF_MERGING_SPLITS` runs; beyond that the second kernel runs as without them).
    """
    _require(merge or splits > 1, "without a merge there must be two or more runs of keys")
    kv_heads, page_size, head_dim = _check_paged(q, k_pages, v_pages, out if out is not None else q, q_heads)
    _require(merge is False or out is not None, "out is needed unless the partial results are left unmerged")
    rows = q.shape[0]
    _dense(kv_len, "kv_len", torch.int32, 1)
    _dense(block_tables, "block_tables", torch.int32, 2)
    _require(kv_len.shape[0] >= rows and block_tables.shape[0] >= rows, "one kv_len and table row per request")
    _require(1 <= splits <= 65535 and rows <= 65535, "splits and requests must fit the grid")
    if splits > 1:
        _require(part_o is not None and part_ml is not None, "splits > 1 needs the partial-result buffers")
        _dense(part_o, "part_o", torch.float32)
        _dense(part_ml, "part_ml", torch.float32)
        _require(part_o.numel() >= rows * q_heads * splits * head_dim and part_ml.numel() >= rows * q_heads * splits * 2,
                 "partial-result buffers are too small")
    if not merge:
        _check(library().dli_attention_decode_partial_bf16(
            _ptr(q), q.stride(0), _ptr(k_pages), _ptr(v_pages), _ptr(part_o), _ptr(part_ml), _ptr(kv_len),
            _ptr(block_tables), block_tables.stride(0), rows, q_heads, kv_heads, head_dim, page_size, float(scale),
            int(window), int(splits), _stream()), "attention_decode")
        return
    if arrivals is not None and splits > 1:
        _dense(arrivals, "arrivals", torch.int32, 1)
        _require(arrivals.numel() >= rows * kv_heads * ((q_heads // kv_heads + 15) // 16),
                 "one arrival counter per request, kv head and tile of 16 heads")
        _check(library().dli_attention_decode_self_merging_bf16(
            _ptr(q), q.stride(0), _ptr(k_pages), _ptr(v_pages), _ptr(out), out.stride(0), _ptr(part_o), _ptr(part_ml),
            _ptr(arrivals), _ptr(kv_len), _ptr(block_tables), block_tables.stride(0), rows, q_heads, kv_heads,
            head_dim, page_size, float(scale), int(window), int(splits), _stream()), "attention_decode")
        return
    _check(library().dli_attention_decode_bf16(
        _ptr(q), q.stride(0), _ptr(k_pages), _ptr(v_pages), _ptr(out), out.stride(0), _ptr(part_o), _ptr(part_ml),
        _ptr(kv_len), _ptr(block_tables), block_tables.stride(0), rows, q_heads, kv_heads, head_dim, page_size,
        float(scale), int(window), int(splits), _stream()), "attention_decode")


SELF_MERGING_SPLITS = 16  # csrc/merge_splits.h: MERGE_SPLITS

STATIC_SCRATCH_FLOATS = 2 * 1024 * 1024  # csrc/no_alloc.h: DLI_STATIC_SCRATCH_FLOATS


def attention_decode_static(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, out: torch.Tensor,
                            kv_len: torch.Tensor, block_tables: torch.Tensor, q_heads: int, scale: float,
                            window: int = 0, splits: int = 1) -> None:
    """:func:`attention_decode` for callers that cannot allocate: the partial results of the key
    splits live in a static device array of :data:`STATIC_SCRATCH_FLOATS` floats inside the
    library (one per GPU, shared by every call on it: calls that overlap on one GPU race)."""
    kv_heads, page_size, head_dim = _check_paged(q, k_pages, v_pages, out, q_heads)
    rows = q.shape[0]
    _dense(kv_len, "kv_len", torch.int32, 1)
    _dense(block_tables, "block_tables", torch.int32, 2)
    _require(kv_len.shape[0] >= rows and block_tables.shape[0] >= rows, "one kv_len and table row per request")
    _require(1 <= splits <= 65535 and rows <= 65535, "splits and requests must fit the grid")
    status = library().dli_attention_decode_bf16_static(
        _ptr(q), q.stride(0), _ptr(k_pages), _ptr(v_pages), _ptr(out), out.stride(0), _ptr(kv_len),
        _ptr(block_tables), block_tables.stride(0), rows, q_heads, kv_heads, head_dim, page_size, float(scale),
        int(window), int(splits), _stream())
    if status == -3:
        raise KernelArgumentError(
            f"attention_decode_static: {rows} requests x {q_heads} heads x {splits} splits x {head_dim} need more "
            f"than the {STATIC_SCRATCH_FLOATS} floats of static scratch")
    _check(status, "attention_decode_static")


def rope_angles(positions: torch.Tensor, inv_freq: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """``[tokens, 2, half]`` float32: cos and sin of ``float(position) * inv_freq``, rounded to
    ``dtype`` as the rotation kernels round them. One table serves every layer of a step."""
    _dense(positions, "positions", torch.int32, 1)
    _dense(inv_freq, "inv_freq", torch.float32, 1)
    n, half = positions.shape[0], inv_freq.shape[0]
    table = torch.empty(n, 2, half, device=positions.device, dtype=torch.float32)
    _check(library().dli_rope_angles(_ptr(positions), _ptr(inv_freq), _ptr(table), n, half, _is_bf16(dtype),
                                     _stream()), "rope_angles")
    return table


def attention_prefill(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, out: torch.Tensor,
                      q_start: torch.Tensor, kv_len: torch.Tensor, block_tables: torch.Tensor,
                      tile_entry: torch.Tensor, tile_q0: torch.Tensor, q_heads: int, scale: float,
                      window: int = 0, tile_cut: Optional[torch.Tensor] = None, cut_tiles: int = 0, cut_room: int = 0,
                      cut_buf: Optional[torch.Tensor] = None, cut_count: Optional[torch.Tensor] = None) -> None:
    """Matrix-core attention for portions; operands as :func:`attention_generic`, tiles of
    :func:`attention_prefill_tile_rows` queries (the tile list must be built with that height, in
    any order: every tile has a workgroup of its own and workgroups start in the list's order, so
    the tiles with the most keys belong first).

    ``tile_cut`` (int32, one per list entry; only without a window and where
    :func:`attention_prefill_cut_floats` is not 0): -1 for a whole tile, or ``run | runs << 4 |
    place << 8`` for one of the 2 to :func:`attention_prefill_max_cuts` runs of a tile that is
    listed once per run and whose keys that many workgroups share, ``place`` numbering the
    ``cut_tiles`` cut tiles from 0. ``cut_room``: the most runs of any tile; ``cut_buf``: float32,
    ``cut_tiles * cut_room * attention_prefill_cut_floats(...)`` values; ``cut_count``: int32,
    ``cut_tiles * q_heads`` counters, zero before the first launch (every launch leaves them zero;
    launches that share them must not overlap)."""
    kv_heads, page_size, head_dim = _check_paged(q, k_pages, v_pages, out, q_heads)
    for name, t in (("q_start", q_start), ("kv_len", kv_len), ("tile_entry", tile_entry), ("tile_q0", tile_q0)):
        _dense(t, name, torch.int32, 1)
    _dense(block_tables, "block_tables", torch.int32, 2)
    entries = kv_len.shape[0]
    _require(q_start.shape[0] == entries + 1 and block_tables.shape[0] >= entries,
             "q_start/kv_len/block_tables disagree on the number of requests")
    _require(tile_entry.shape == tile_q0.shape, "tile lists differ in length")
    if tile_cut is not None:
        _dense(tile_cut, "tile_cut", torch.int32, 1)
        _require(tile_cut.shape == tile_entry.shape, "tile_cut differs in length from the tile list")
        per = attention_prefill_cut_floats(head_dim, q_heads, kv_heads)
        _require(per > 0 and window == 0, "this shape's kernel cuts no tiles, or a window is set")
        _require(cut_buf is not None and cut_count is not None and cut_tiles > 0, "cut tiles need their buffers")
        _require(2 <= cut_room <= attention_prefill_max_cuts(), "cut_room outside what the kernel takes")
        _dense(cut_buf, "cut_buf", torch.float32, 1)
        _dense(cut_count, "cut_count", torch.int32, 1)
        _require(cut_buf.shape[0] >= cut_tiles * cut_room * per and cut_count.shape[0] >= cut_tiles * q_heads,
                 "cut_buf or cut_count too small for the cut tiles")
    _check(library().dli_attention_prefill_bf16(
        _ptr(q), q.stride(0), _ptr(k_pages), _ptr(v_pages), _ptr(out), out.stride(0), _ptr(q_start), _ptr(kv_len),
        _ptr(block_tables), block_tables.stride(0), _ptr(tile_entry), _ptr(tile_q0), tile_entry.shape[0], q_heads,
        kv_heads, head_dim, page_size, float(scale), int(window), _ptr(tile_cut), int(cut_tiles), int(cut_room),
        _ptr(cut_buf), _ptr(cut_count), _stream()), "attention_prefill")

# ----------------------------------------------------------------------------- sampling

def sample_scratch(rows: int, device: torch.device) -> tuple[torch.Tensor, torch.Tensor]:
    """Scratch that :func:`sample` needs for ``rows`` rows (values and indices of the argmax's
    first stage: its own chunks, or one part per workgroup of a logits kernel that does that stage)."""
    per = max(int(library().dli_sample_scratch_per_row()), compute_units(device))
    return (torch.empty(rows * per, device=device, dtype=torch.float32),
            torch.empty(rows * per, device=device, dtype=torch.int32))


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
           seeds: torch.Tensor, counters: torch.Tensor, out: torch.Tensor,
           scratch: Optional[tuple[torch.Tensor, torch.Tensor]] = None) -> None:
    """One token per row of float32 ``logits [rows, vocab]``.

    Rows with ``temperature == 0`` or ``top_k == 1`` take the argmax (lowest id on ties); the others
    apply temperature, top-k (``<= 0``: off), top-p and draw with Philox(seed, counter).
    """
    _rows(logits, "logits", torch.float32)
    rows, vocab = logits.shape
    _dense(temperature, "temperature", torch.float32, 1)
    _dense(top_k, "top_k", torch.int32, 1)
    _dense(top_p, "top_p", torch.float32, 1)
    _dense(seeds, "seeds", torch.int64, 1)
    _dense(counters, "counters", torch.int64, 1)
    _dense(out, "out", torch.int32, 1)
    for name, t in (("temperature", temperature), ("top_k", top_k), ("top_p", top_p), ("seeds", seeds),
                    ("counters", counters), ("out", out)):
        _require(t.shape[0] == rows, f"{name} must have one value per row")
    if scratch is None:
        scratch = sample_scratch(rows, logits.device)
    per = int(library().dli_sample_scratch_per_row())
    _dense(scratch[0], "scratch values", torch.float32)
    _dense(scratch[1], "scratch indices", torch.int32)
    _require(scratch[0].numel() >= rows * per and scratch[1].numel() >= rows * per, "sampling scratch is too small")
    _check(library().dli_sample(_ptr(logits), logits.stride(0), rows, vocab, _ptr(temperature), _ptr(top_k),
                                _ptr(top_p), _ptr(seeds), _ptr(counters), _ptr(scratch[0]), _ptr(scratch[1]),
                                _ptr(out), _stream()), "sample")


def sample_and_advance(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
                       seeds: torch.Tensor, counters: torch.Tensor, out: torch.Tensor,
                       scratch: tuple[torch.Tensor, torch.Tensor], parts: int, tokens_out: torch.Tensor,
                       token_ids: torch.Tensor, positions: torch.Tensor, kv_len: torch.Tensor,
                       slots: Sequence[torch.Tensor], tables: Sequence[torch.Tensor], page_size: int,
                       advance: bool) -> None:
    """:func:`sample` and :func:`decode_advance` in one launch (for decode steps recorded into a
    graph): the thread that chooses a row's token hands it on. ``parts`` > 0: ``scratch`` already
    holds the first stage of every row's argmax as ``[rows, parts]`` (:func:`head_gemm` with
    ``best``), and the kernel that reads all logits for it does not run."""
    _rows(logits, "logits", torch.float32)
    rows, vocab = logits.shape
    _dense(temperature, "temperature", torch.float32, 1)
    _dense(top_p, "top_p", torch.float32, 1)
    _dense(seeds, "seeds", torch.int64, 1)
    _dense(counters, "counters", torch.int64, 1)
    for name, t in (("top_k", top_k), ("out", out), ("tokens_out", tokens_out), ("token_ids", token_ids),
                    ("positions", positions), ("kv_len", kv_len)):
        _dense(t, name, torch.int32, 1)
    for name, t in (("temperature", temperature), ("top_k", top_k), ("top_p", top_p), ("seeds", seeds),
                    ("counters", counters), ("out", out), ("tokens_out", tokens_out), ("token_ids", token_ids),
                    ("positions", positions), ("kv_len", kv_len)):
        _require(t.shape[0] == rows, f"{name} must have one value per row")
    per = int(library().dli_sample_scratch_per_row())
    _dense(scratch[0], "scratch values", torch.float32)
    _dense(scratch[1], "scratch indices", torch.int32)
    need = rows * (parts if parts > 0 else per)
    _require(0 <= parts <= 1024 and scratch[0].numel() >= need and scratch[1].numel() >= need,
             "sampling scratch is too small")
    _require(len(slots) == len(tables) <= 4, "one slot vector and one table per group, at most 4 groups")
    width = 1
    for g, (sl, tb) in enumerate(zip(slots, tables)):
        _dense(sl, f"slots[{g}]", torch.int32, 1)
        _dense(tb, f"tables[{g}]", torch.int32, 2)
        _require(sl.shape[0] == rows and tb.shape[0] == rows, "slots and tables must have one row per request")
        _require(g == 0 or tb.shape[1] == width, "the groups' tables differ in width")
        width = tb.shape[1]
    n = len(slots)
    slot_ptrs = (ctypes.c_void_p * 4)(*([t.data_ptr() for t in slots] + [None] * (4 - n)))
    table_ptrs = (ctypes.c_void_p * 4)(*([t.data_ptr() for t in tables] + [None] * (4 - n)))
    _check(library().dli_sample_and_advance(
        _ptr(logits), logits.stride(0), rows, vocab, _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(seeds),
        _ptr(counters), _ptr(scratch[0]), _ptr(scratch[1]), int(parts), _ptr(out), _ptr(tokens_out), _ptr(token_ids),
        _ptr(positions), _ptr(kv_len), ctypes.cast(slot_ptrs, ctypes.c_void_p), ctypes.cast(table_ptrs, ctypes.c_void_p),
        n, width, int(page_size), int(bool(advance)), _stream()), "sample_and_advance")


def decode_advance(sampled: torch.Tensor, tokens_out: torch.Tensor, token_ids: torch.Tensor,
                   positions: torch.Tensor, kv_len: torch.Tensor, counters: torch.Tensor,
                   slots: Sequence[torch.Tensor], tables: Sequence[torch.Tensor], page_size: int,
                   advance: bool) -> None:
    """Hand the sampled tokens of a decode step to the next one on the device.

    ``tokens_out[i] = sampled[i]``; with ``advance`` every row that has keys gets its sampled token
    as next input, position, key count and draw counter plus one, and in each group of layers the
    cache slot of the new position from its block-table row (``tables[g]`` is ``[rows, width]``).
    """
    rows = sampled.shape[0]
    for name, t in (("sampled", sampled), ("tokens_out", tokens_out), ("token_ids", token_ids),
                    ("positions", positions), ("kv_len", kv_len)):
        _dense(t, name, torch.int32, 1)
        _require(t.shape[0] == rows, f"{name} must have one entry per row")
    _dense(counters, "counters", torch.int64, 1)
    _require(counters.shape[0] == rows, "counters must have one entry per row")
    _require(len(slots) == len(tables) <= 4, "one slot vector and one table per group, at most 4 groups")
    width = 1
    for g, (sl, tb) in enumerate(zip(slots, tables)):
        _dense(sl, f"slots[{g}]", torch.int32, 1)
        _dense(tb, f"tables[{g}]", torch.int32, 2)
        _require(sl.shape[0] == rows and tb.shape[0] == rows, "slots and tables must have one row per request")
        _require(g == 0 or tb.shape[1] == width, "the groups' tables differ in width")
        width = tb.shape[1]
    n = len(slots)
    slot_ptrs = (ctypes.c_void_p * 4)(*([t.data_ptr() for t in slots] + [None] * (4 - n)))
    table_ptrs = (ctypes.c_void_p * 4)(*([t.data_ptr() for t in tables] + [None] * (4 - n)))
    _check(library().dli_decode_advance(
        _ptr(sampled), _ptr(tokens_out), _ptr(token_ids), _ptr(positions), _ptr(kv_len), _ptr(counters),
        ctypes.cast(slot_ptrs, ctypes.c_void_p), ctypes.cast(table_ptrs, ctypes.c_void_p), n, width,
        int(page_size), rows, int(bool(advance)), _stream()), "decode_advance")


# ----------------------------------------------------------------------------- a 32-bit residual stream

def _f32_rows(t: torch.Tensor, name: str) -> None:
    _rows(t, name, torch.float32)


def _rounded_copy(rounded: Optional[torch.Tensor], like: torch.Tensor) -> None:
    if rounded is not None:
        _dense(rounded, "rounded", torch.bfloat16, 2)
        _require(rounded.shape == like.shape, "the rounded copy differs from the stream in shape")


def embed_sinusoid(table: torch.Tensor, ids: torch.Tensor, positions: torch.Tensor, inv_freq: Optional[torch.Tensor],
                   out: torch.Tensor, rounded: Optional[torch.Tensor] = None) -> None:
    """``out[t] = table[ids[t]] + pe(positions[t])`` in float32, ``pe[2i] = sin(p f_i)``,
    ``pe[2i+1] = cos(p f_i)`` with ``f = inv_freq [ceil(width/2)]`` (``None``: the token's row alone, widened
    to float32). ``rounded``: the same rows once more in bfloat16."""
    _rounded_copy(rounded, out)
    _dense(table, "table", ndim=2)
    _dense(ids, "ids", torch.int32, 1)
    _dense(positions, "positions", torch.int32, 1)
    _dense(out, "out", torch.float32, 2)
    n, width = ids.shape[0], table.shape[1]
    _require(positions.shape[0] == n and out.shape == (n, width), "ids, positions and out disagree on the rows")
    if inv_freq is not None:
        _dense(inv_freq, "inv_freq", torch.float32, 1)
        _require(inv_freq.shape[0] * 2 >= width, "inv_freq must hold a frequency for every pair of columns")
    _check(library().dli_embed_sinusoid(_ptr(table), _ptr(ids), _ptr(positions), _ptr(inv_freq), _ptr(out), _ptr(rounded), n, width,
                                        _is_bf16(table.dtype), _stream()), "embed_sinusoid")


def cast_from_f32(x: torch.Tensor, out: torch.Tensor) -> None:
    """``out = x`` rounded to ``out``'s type (float32 or bfloat16)."""
    _dense(x, "x", torch.float32)
    _dense(out, "out")
    _require(out.numel() == x.numel(), "out differs from x in size")
    _check(library().dli_cast_from_f32(_ptr(x), _ptr(out), x.numel(), _is_bf16(out.dtype), _stream()), "cast_from_f32")


def norm_into_stream(y: torch.Tensor, weight: torch.Tensor, eps: float, x: torch.Tensor,
                     rounded: Optional[torch.Tensor] = None) -> None:
    """``x += weight * y / sqrt(mean(y^2) + eps)`` row by row: ``x`` float32 ``[n, width]``, ``y`` float32
    or bfloat16 with contiguous rows, statistics and sum in 32-bit. ``rounded``: the new ``x`` once more
    in bfloat16 (what the next product reads)."""
    _rounded_copy(rounded, x)
    _rows(y, "y", y.dtype)
    _dense(x, "x", torch.float32, 2)
    _dense(weight, "weight", torch.float32, 1)
    _require(y.shape == x.shape and weight.shape[0] == x.shape[1], "y, x and weight disagree on the sizes")
    _check(library().dli_norm_into_stream(_ptr(y), y.stride(0), _ptr(weight), _ptr(x), _ptr(rounded), x.shape[0], x.shape[1],
                                          float(eps), _is_bf16(y.dtype), _stream()), "norm_into_stream")


def post_norm_stream(x: torch.Tensor, y: torch.Tensor, weight: torch.Tensor, alpha: float, eps: float,
                     gate: Optional[torch.Tensor] = None, gate_bias: Optional[torch.Tensor] = None,
                     rounded: Optional[torch.Tensor] = None) -> None:
    """``x <- weight * s / sqrt(mean(s^2) + eps)`` with ``s = alpha x + r y`` row by row, where
    ``r = sigmoid(gate + gate_bias)`` element by element (``gate`` float32 ``[n, width]``, rows contiguous;
    ``None``: ``r = 1``): the norm after a residual sum. ``x`` float32 ``[n, width]``, ``y`` float32 or bfloat16
    with contiguous rows; sums and statistics in 32-bit. ``rounded``: the new ``x`` once more in bfloat16."""
    _rounded_copy(rounded, x)
    _rows(y, "y", y.dtype)
    _dense(x, "x", torch.float32, 2)
    _dense(weight, "weight", torch.float32, 1)
    _require(y.shape == x.shape and weight.shape[0] == x.shape[1], "y, x and weight disagree on the sizes")
    g_stride = 0
    if gate is not None:
        _f32_rows(gate, "gate")
        _require(gate.shape == x.shape, "gate differs from x in shape")
        g_stride = gate.stride(0)
        if gate_bias is not None:
            _dense(gate_bias, "gate_bias", torch.float32, 1)
            _require(gate_bias.shape[0] == x.shape[1], "gate_bias must hold a value per column")
    else:
        _require(gate_bias is None, "a gate's bias comes with a gate")
    _check(library().dli_post_norm_stream(_ptr(y), y.stride(0), _ptr(gate), g_stride, _ptr(gate_bias), _ptr(weight), _ptr(x),
                                          _ptr(rounded), x.shape[0], x.shape[1], float(alpha), float(eps),
                                          _is_bf16(y.dtype), _stream()), "post_norm_stream")


def rms_norm_from_f32(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor) -> None:
    """``out = weight * x / sqrt(mean(x^2) + eps)`` for a float32 ``x``, rounded once to ``out``'s type."""
    _dense(x, "x", torch.float32, 2)
    _dense(weight, "weight", torch.float32, 1)
    _dense(out, "out", ndim=2)
    _require(out.shape == x.shape and weight.shape[0] == x.shape[1], "out, x and weight disagree on the sizes")
    _check(library().dli_rms_norm_from_f32(_ptr(x), _ptr(weight), _ptr(out), x.shape[0], x.shape[1], float(eps),
                                           _is_bf16(out.dtype), _stream()), "rms_norm_from_f32")


def softcap(y: torch.Tensor, cap: float) -> None:
    """``y <- cap * tanh(y / cap)`` in place (float32)."""
    _dense(y, "y", torch.float32)
    _require(cap > 0, "the cap must be positive")
    _check(library().dli_softcap(_ptr(y), y.numel(), float(cap), _stream()), "softcap")


def token_shift(x: torch.Tensor, mu: torch.Tensor, state: torch.Tensor, q_start: torch.Tensor,
                positions: torch.Tensor, state_slots: torch.Tensor, out: torch.Tensor) -> None:
    """``out[s, t] = x[t] + (x[t-1] - x[t]) * mu[s]`` for every mix ``s``; the row before an entry's
    first row is the request's kept row, the first ``width`` floats of ``state[slot]`` (zeros at
    position 0), which then receives the entry's last row. ``x`` float32 ``[n, width]``, ``mu`` float32
    ``[mixes, width]``, ``state`` float32 ``[slots, >= width]``, ``out [mixes, n, width]``."""
    _dense(x, "x", torch.float32, 2)
    _dense(mu, "mu", torch.float32, 2)
    _dense(out, "out", ndim=3)
    n, width = x.shape
    _require(mu.shape[1] == width and out.shape == (mu.shape[0], n, width), "x, mu and out disagree on the sizes")
    _require(state.is_cuda and state.dtype == torch.float32 and state.dim() == 2 and state.stride(1) == 1
             and state.shape[1] >= width, "state must be float32 [slots, >= width]")
    for name, t in (("q_start", q_start), ("positions", positions), ("state_slots", state_slots)):
        _dense(t, name, torch.int32, 1)
    entries = state_slots.shape[0]
    _require(q_start.shape[0] == entries + 1 and positions.shape[0] == n, "q_start/state_slots/positions disagree")
    _check(library().dli_token_shift(_ptr(x), _ptr(mu), mu.shape[0], _ptr(state), state.stride(0), _ptr(q_start),
                                     entries, _ptr(positions), _ptr(state_slots), _ptr(out), n, width,
                                     _is_bf16(out.dtype), _stream()), "token_shift")


LOWRANK_OUT_ACTS = {"none": 0, "delta_decay": 1, "double_exp_decay": 2, "softplus": 3}


def lowrank_out(t: torch.Tensor, w2t: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                act: str = "tanh", out_act: str = "none", rate: Optional[torch.Tensor] = None,
                rate_bias: Optional[torch.Tensor] = None) -> None:
    """``out = out_act(act(t) @ w2t + bias)`` in 32-bit: ``t`` float32 ``[n, rank]`` (rows contiguous, any
    row stride), ``w2t`` float32 ``[rank, features]`` (the projection's second matrix transposed);
    ``act`` ``"tanh"`` or ``"none"``; ``out_act`` ``"none"``, ``"delta_decay"`` (``exp(-exp(-1/2) sigmoid(y))``)
    or ``"double_exp_decay"`` (``exp(-exp(y))``). ``rate`` (float32 ``[n, features]``, rows contiguous)
    becomes ``sigmoid(rate + rate_bias)`` in place in the same launch."""
    _require(out_act in LOWRANK_OUT_ACTS, f"out_act must be one of {sorted(LOWRANK_OUT_ACTS)}")
    _f32_rows(t, "t")
    _dense(w2t, "w2t", torch.float32, 2)
    _dense(out, "out", torch.float32, 2)
    _require(act in ("tanh", "none"), "act must be 'tanh' or 'none'")
    n, rank = t.shape
    feats = w2t.shape[1]
    _require(w2t.shape[0] == rank and out.shape == (n, feats), "t, w2t and out disagree on the sizes")
    if bias is not None:
        _dense(bias, "bias", torch.float32, 1)
        _require(bias.shape[0] == feats, "bias length differs from the features")
    rate_stride = 0
    if rate is not None:
        _f32_rows(rate, "rate")
        _require(rate.shape == (n, feats), "rate must be [n, features]")
        rate_stride = rate.stride(0)
        if rate_bias is not None:
            _dense(rate_bias, "rate_bias", torch.float32, 1)
            _require(rate_bias.shape[0] == feats, "rate_bias length differs from the features")
    _check(library().dli_lowrank_out(_ptr(t), t.stride(0), _ptr(w2t), _ptr(bias), _ptr(out), n, feats, rank,
                                     1 if act == "tanh" else 0, LOWRANK_OUT_ACTS[out_act], _ptr(rate), rate_stride,
                                     _ptr(rate_bias), _stream()), "lowrank_out")


def qk_unit_cache(proj: torch.Tensor, q_off: int, k_off: int, v_off: int, q_out: torch.Tensor,
                  slots: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, q_heads: int, eps: float,
                  mix: Optional[torch.Tensor] = None, v_first_in: Optional[torch.Tensor] = None,
                  v_first_out: Optional[torch.Tensor] = None) -> None:
    """From the float32 projections ``proj [n, >= ...]`` (q at ``q_off``, k at ``k_off``, v at
    ``v_off``): q and k divided by their root mean square per head, ``q_out [n, q_heads*dim]``; with
    ``mix`` (a float32 scalar on the device) ``v <- (1 - mix) v + mix v_first_in``; ``v_first_out``
    receives this layer's v; k and v are written at each token's cache slot."""
    _f32_rows(proj, "proj")
    _dense(k_pages, "k_pages", ndim=4)
    dtype = k_pages.dtype
    pages, kv_heads, page_size, dim = k_pages.shape
    _dense(v_pages, "v_pages", dtype, 4)
    vdim = v_pages.shape[2]
    _require(v_pages.shape == (pages, kv_heads, vdim, page_size), "v_pages must be [pages, kv_heads, vdim, page_size]")
    n = proj.shape[0]
    _dense(q_out, "q_out", dtype, 2)
    _require(q_out.shape == (n, q_heads * dim), "q_out must be [n, q_heads*dim]")
    _dense(slots, "slots", torch.int32, 1)
    _require(slots.shape[0] == n, "slots differ from proj in rows")
    for off, size in ((q_off, q_heads * dim), (k_off, kv_heads * dim), (v_off, kv_heads * vdim)):
        _require(0 <= off and off + size <= proj.shape[1], "a projection lies outside proj's columns")
    for t in (v_first_in, v_first_out):
        if t is not None:
            _dense(t, "v_first", torch.float32, 2)
            _require(t.shape == (n, kv_heads * vdim), "v_first must be [n, kv_heads*vdim]")
    if mix is not None:
        _require(mix.is_cuda and mix.dtype == torch.float32 and mix.numel() == 1 and v_first_in is not None,
                 "mix must be one float32 on the device, with v_first_in")
    _check(library().dli_qk_unit_cache(
        _ptr(proj), proj.stride(0), q_off, k_off, v_off, _ptr(q_out), _ptr(mix), _ptr(v_first_in), _ptr(v_first_out),
        _ptr(slots), _ptr(k_pages), _ptr(v_pages), n, q_heads, kv_heads, dim, vdim, page_size, float(eps),
        _is_bf16(dtype), _stream()), "qk_unit_cache")


def attention_scored(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, out: torch.Tensor,
                     q_start: torch.Tensor, kv_len: torch.Tensor, block_tables: torch.Tensor,
                     tile_entry: Optional[torch.Tensor], tile_q0: Optional[torch.Tensor], q_heads: int, scale: float,
                     *, window: int = 0, chunk: int = 0, sink: bool = False, r1: Optional[torch.Tensor] = None,
                     r2: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None, keep_first: int = 0) -> None:
    """Paged causal attention on the vector units (32-bit arithmetic) with changes to the scores
    as parameters: ``window`` and ``chunk`` restrict the keys a query sees (under a window the first
    ``keep_first`` positions stay visible from any distance), ``r1, r2`` (float32
    ``[q_heads]``) take ``r1 log(1 + r2 (p - j))`` off the scaled score, ``sink`` adds ``exp(0)`` to the
    softmax's denominator, ``gate`` (float32 ``[tokens, q_heads*value_dim]``, rows contiguous)
    multiplies the result by its sigmoid. Values may differ from keys in size (``v_pages``), and the
    value pages may hold fewer heads than the key pages, a divisor of their number: kv head ``g`` then
    reads the values of head ``g % value_heads`` (several score maps over one set of values). ``out`` is
    of the pages' type, or float32 (the result unrounded).
    Without tile lists every entry is one row (a step of single tokens)."""
    _dense(k_pages, "k_pages", ndim=4)
    dtype = k_pages.dtype
    _rows(q, "q", dtype)
    out32 = out.dtype == torch.float32 and dtype != torch.float32
    _rows(out, "out", torch.float32 if out32 else dtype)
    pages, kv_heads, page_size, head_dim = k_pages.shape
    _dense(v_pages, "v_pages", dtype, 4)
    v_heads, value_dim = v_pages.shape[1], v_pages.shape[2]
    _require(v_pages.shape == (pages, v_heads, value_dim, page_size) and v_heads > 0 and kv_heads % v_heads == 0,
             "v_pages must be [pages, value heads, value_dim, page_size], the value heads a divisor of the kv heads")
    _require(keep_first >= 0, "keep_first must not be negative")
    _require(q.shape[1] == q_heads * head_dim and out.shape == (q.shape[0], q_heads * value_dim),
             "q must be [tokens, q_heads*head_dim] and out [tokens, q_heads*value_dim]")
    _require(q_heads % kv_heads == 0, "query heads are not a multiple of kv heads")
    _require(max(head_dim, value_dim) <= 256, "heads of at most 256")
    _dense(q_start, "q_start", torch.int32, 1)
    _dense(kv_len, "kv_len", torch.int32, 1)
    _dense(block_tables, "block_tables", torch.int32, 2)
    entries = kv_len.shape[0]
    _require(q_start.shape[0] == entries + 1 and block_tables.shape[0] >= entries,
             "q_start/kv_len/block_tables disagree on the number of requests")
    if tile_entry is None:
        _require(tile_q0 is None and q.shape[0] == entries, "without tile lists every entry must be one row")
        tiles = entries
    else:
        _dense(tile_entry, "tile_entry", torch.int32, 1)
        _dense(tile_q0, "tile_q0", torch.int32, 1)
        _require(tile_entry.shape == tile_q0.shape, "tile lists differ in length")
        tiles = tile_entry.shape[0]
    _require((r1 is None) == (r2 is None), "r1 and r2 come together")
    for name, t in (("r1", r1), ("r2", r2)):
        if t is not None:
            _dense(t, name, torch.float32, 1)
            _require(t.shape[0] == q_heads, f"{name} must hold one value per query head")
    gate_stride = 0
    if gate is not None:
        _f32_rows(gate, "gate")
        _require(gate.shape == out.shape, "gate differs from out in shape")
        gate_stride = gate.stride(0)
    if tile_entry is None:
        # few (kv head, group of query heads) pairs an entry: an entry's keys are cut over several workgroups
        # (a number that the heads and the number of entries decide), whose shares a second kernel adds up
        splits = int(library().dli_attention_scored_splits(q_heads, kv_heads, entries))
        if splits > 1:
            parts = torch.empty(entries * q_heads * splits * (value_dim + 2), device=q.device, dtype=torch.float32)
            _check(library().dli_attention_scored_single(
                _ptr(q), q.stride(0), _ptr(k_pages), _ptr(v_pages), _ptr(out), out.stride(0), _ptr(kv_len),
                _ptr(block_tables), block_tables.stride(0), entries, q_heads, kv_heads, head_dim, value_dim, page_size,
                float(scale), int(window), int(chunk), int(bool(sink)), _ptr(r1), _ptr(r2), _ptr(gate), gate_stride,
                int(keep_first), v_heads, _ptr(out if out32 else None), _ptr(parts), splits, _is_bf16(dtype), _stream()),
                "attention_scored_single")
            return
    _check(library().dli_attention_scored(
        _ptr(q), q.stride(0), _ptr(k_pages), _ptr(v_pages), _ptr(out), out.stride(0), _ptr(q_start), _ptr(kv_len),
        _ptr(block_tables), block_tables.stride(0), _ptr(tile_entry), _ptr(tile_q0), tiles, q_heads, kv_heads,
        head_dim, value_dim, page_size, float(scale), int(window), int(chunk), int(bool(sink)), _ptr(r1), _ptr(r2),
        _ptr(gate), gate_stride, int(keep_first), v_heads, _ptr(out if out32 else None), _is_bf16(dtype), _stream()),
        "attention_scored")


SCORED_MFMA_TILE_ROWS = 64  # queries of a tile of the matrix-core kernel (four waves of 16)


def attention_scored_mfma_supports(head_dim: int, value_dim: int, page_size: int, dtype: torch.dtype) -> bool:
    return dtype == torch.bfloat16 and bool(
        library().dli_attention_scored_mfma_supports(int(head_dim), int(value_dim), int(page_size)))


def attention_scored_mfma(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, out: torch.Tensor,
                          q_start: torch.Tensor, kv_len: torch.Tensor, block_tables: torch.Tensor,
                          tile_entry: torch.Tensor, tile_q0: torch.Tensor, q_heads: int, scale: float, *,
                          window: int = 0, chunk: int = 0, sink: bool = False, r1: Optional[torch.Tensor] = None,
                          r2: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None, keep_first: int = 0) -> None:
    """:func:`attention_scored` for the portions of a bfloat16 step on the matrix cores: the same
    operands and parameters, tiles of ``SCORED_MFMA_TILE_ROWS`` queries, sizes that
    :func:`attention_scored_mfma_supports` takes."""
    _dense(k_pages, "k_pages", torch.bfloat16, 4)
    _rows(q, "q", torch.bfloat16)
    out32 = out.dtype == torch.float32
    _rows(out, "out", torch.float32 if out32 else torch.bfloat16)
    pages, kv_heads, page_size, head_dim = k_pages.shape
    _dense(v_pages, "v_pages", torch.bfloat16, 4)
    v_heads, value_dim = v_pages.shape[1], v_pages.shape[2]
    _require(v_pages.shape == (pages, v_heads, value_dim, page_size) and v_heads > 0 and kv_heads % v_heads == 0,
             "v_pages must be [pages, value heads, value_dim, page_size], the value heads a divisor of the kv heads")
    _require(keep_first >= 0, "keep_first must not be negative")
    _require(attention_scored_mfma_supports(head_dim, value_dim, page_size, k_pages.dtype),
             "the matrix-core kernel does not take these sizes")
    _require(q.shape[1] == q_heads * head_dim and out.shape == (q.shape[0], q_heads * value_dim),
             "q must be [tokens, q_heads*head_dim] and out [tokens, q_heads*value_dim]")
    _require(q_heads % kv_heads == 0, "query heads are not a multiple of kv heads")
    _require(q.stride(0) % 4 == 0 and out.stride(0) % 4 == 0 and q.data_ptr() % 8 == 0
             and out.data_ptr() % (16 if out32 else 8) == 0, "q and out must be aligned for four values at once, row by row")
    for name, t in (("q_start", q_start), ("kv_len", kv_len), ("tile_entry", tile_entry), ("tile_q0", tile_q0)):
        _dense(t, name, torch.int32, 1)
    _dense(block_tables, "block_tables", torch.int32, 2)
    entries = kv_len.shape[0]
    _require(q_start.shape[0] == entries + 1 and block_tables.shape[0] >= entries,
             "q_start/kv_len/block_tables disagree on the number of requests")
    _require(tile_entry.shape == tile_q0.shape, "tile lists differ in length")
    _require((r1 is None) == (r2 is None), "r1 and r2 come together")
    for name, t in (("r1", r1), ("r2", r2)):
        if t is not None:
            _dense(t, name, torch.float32, 1)
            _require(t.shape[0] == q_heads, f"{name} must hold one value per query head")
    gate_stride = 0
    if gate is not None:
        _f32_rows(gate, "gate")
        _require(gate.shape == out.shape, "gate differs from out in shape")
        gate_stride = gate.stride(0)
    _check(library().dli_attention_scored_mfma(
        _ptr(q), q.stride(0), _ptr(k_pages), _ptr(v_pages), _ptr(out), out.stride(0), _ptr(q_start), _ptr(kv_len),
        _ptr(block_tables), block_tables.stride(0), _ptr(tile_entry), _ptr(tile_q0), tile_entry.shape[0], q_heads,
        kv_heads, head_dim, value_dim, page_size, float(scale), int(window), int(chunk), int(bool(sink)), _ptr(r1),
        _ptr(r2), _ptr(gate), gate_stride, int(keep_first), v_heads, _ptr(out if out32 else None), _stream()),
        "attention_scored_mfma")


RULE_DELTA, RULE_BONUS = 0, 1


def recurrent_scan_supports(dim: int) -> bool:
    return bool(library().dli_recurrent_scan_supports(int(dim)))


def recurrent_scan(r: torch.Tensor, k: torch.Tensor, v: torch.Tensor, w: torch.Tensor, g_pre: torch.Tensor,
                   norm_w: torch.Tensor, eps: float, state: torch.Tensor, q_start: torch.Tensor,
                   positions: torch.Tensor, state_slots: torch.Tensor, out: torch.Tensor, heads: int, dim: int,
                   rule: int, a: Optional[torch.Tensor] = None, bonus: Optional[torch.Tensor] = None) -> None:
    """A matrix-state recurrence per request and head, with the per-head norm and the gate of its
    output (``csrc/recurrent_scan.hip`` states both rules). ``r, k, v``, the decay ``w``, the gate's
    pre-activation ``g_pre`` and (delta rule) the removal rate ``a`` are float32 ``[n, heads*dim]`` with
    contiguous rows (any row stride); ``state`` is float32 ``[slots, >= heads*dim*dim]``, row
    ``state_slots[e]`` being entry ``e``'s; ``out [n, heads*dim]`` float32 or bfloat16."""
    n, width = out.shape[0], heads * dim
    w_pre, a_pre, a_bias = w, a, None
    for name, t in (("r", r), ("k", k), ("v", v), ("w", w), ("g_pre", g_pre), ("a", a)):
        if t is not None:
            _f32_rows(t, name)
            _require(t.shape == (n, width), f"{name} must be [n, heads*dim]")
    _rows(out, "out", out.dtype)
    _require(out.shape[1] == width, "out must be [n, heads*dim]")
    _require(recurrent_scan_supports(dim), f"the recurrence kernels take heads of 1 to 1024, not {dim}")
    _dense(norm_w, "norm_w", torch.float32, 1)
    _require(norm_w.shape[0] == width, "norm_w must hold heads*dim values")
    _require(state.is_cuda and state.dtype == torch.float32 and state.dim() == 2 and state.stride(1) == 1
             and state.shape[1] >= heads * dim * dim, "state must be float32 [slots, >= heads*dim*dim]")
    for name, t in (("q_start", q_start), ("positions", positions), ("state_slots", state_slots)):
        _dense(t, name, torch.int32, 1)
    entries = state_slots.shape[0]
    _require(q_start.shape[0] == entries + 1 and positions.shape[0] == n, "q_start/state_slots/positions disagree")
    if rule == RULE_DELTA:
        _require(a is not None, "the delta rule needs the removal rate")
    else:
        _require(rule == RULE_BONUS and bonus is not None, "the bonus rule needs bonus")
        _dense(bonus, "bonus", torch.float32)
        _require(bonus.numel() == width, "bonus must hold heads*dim values")
    sa = a_pre.stride(0) if a_pre is not None else 0
    o_raw = torch.empty(n, width, device=out.device, dtype=torch.float32)  # the recurrence's output before norm and gate
    _check(library().dli_recurrent_scan(
        _ptr(r), r.stride(0), _ptr(k), k.stride(0), _ptr(v), v.stride(0), _ptr(w_pre), w_pre.stride(0), _ptr(a_pre), sa,
        _ptr(a_bias), _ptr(g_pre), g_pre.stride(0), _ptr(bonus), _ptr(norm_w), float(eps), _ptr(state), state.stride(0),
        _ptr(q_start), _ptr(positions), _ptr(state_slots), _ptr(o_raw), o_raw.stride(0), _ptr(out), out.stride(0), entries,
        n, heads, dim, int(rule), _is_bf16(out.dtype), _stream()), "recurrent_scan")


# ----------------------------------------------------------------------------- rotary keys from 32-bit projections

def rotary_cache(proj: torch.Tensor, q_off: int, k_off: int, v_off: int, positions: torch.Tensor,
                 inv_freq: Optional[torch.Tensor], rot_dims: int, interleaved: bool, q_out: torch.Tensor,
                 slots: Optional[torch.Tensor], k_pages: Optional[torch.Tensor], v_pages: Optional[torch.Tensor], q_heads: int,
                 bias: Optional[torch.Tensor] = None) -> None:
    """From the float32 projections ``proj [n, >= ...]`` (q at ``q_off``, k at ``k_off``, v at ``v_off``):
    the first ``rot_dims`` components of every q and k head rotated by ``position * inv_freq[i]`` (pair
    ``i`` is ``(2i, 2i+1)`` where ``interleaved``, else ``(i, i + rot_dims/2)``; 32-bit angles),
    ``q_out [n, q_heads*dim]``; rotated k and v written at each token's cache slot. ``bias`` (float32, a
    value for every column of ``proj``) is added first. The value pages may hold fewer heads than the key
    pages; without pages (``None``: the mixer reads another's) only q is made."""
    _f32_rows(proj, "proj")
    n = proj.shape[0]
    dtype = q_out.dtype
    _dense(q_out, "q_out", dtype, 2)
    _require(q_out.shape[0] == n and q_out.shape[1] % q_heads == 0, "q_out must be [n, q_heads*dim]")
    dim = q_out.shape[1] // q_heads
    kv_heads = v_heads = 0
    page_size = vdim = 1
    if k_pages is not None:
        _dense(k_pages, "k_pages", dtype, 4)
        pages, kv_heads, page_size, kdim = k_pages.shape
        _require(kdim == dim, "keys and queries differ in size")
        _dense(v_pages, "v_pages", dtype, 4)
        v_heads, vdim = v_pages.shape[1], v_pages.shape[2]
        _require(v_pages.shape == (pages, v_heads, vdim, page_size), "v_pages must be [pages, value heads, vdim, page_size]")
        _dense(slots, "slots", torch.int32, 1)
        _require(slots.shape[0] == n, "slots differ from proj in rows")
    else:
        _require(v_pages is None, "value pages come with key pages")
    _dense(positions, "positions", torch.int32, 1)
    _require(positions.shape[0] == n, "positions differ from proj in rows")
    for off, size in ((q_off, q_heads * dim), (k_off, kv_heads * dim), (v_off, v_heads * vdim)):
        _require(0 <= off and off + size <= proj.shape[1], "a projection lies outside proj's columns")
    if bias is not None:
        _dense(bias, "bias", torch.float32, 1)
        _require(bias.shape[0] >= max(q_off + q_heads * dim, k_off + kv_heads * dim, v_off + v_heads * vdim),
                 "bias must hold a value for every projected column")
    _require(0 <= rot_dims <= dim and rot_dims % 2 == 0, "the rotated components must be an even number within the head")
    if rot_dims:
        _dense(inv_freq, "inv_freq", torch.float32, 1)
        _require(inv_freq.shape[0] * 2 == rot_dims, "inv_freq must hold rot_dims/2 frequencies")
    _check(library().dli_rotary_cache(
        _ptr(proj), proj.stride(0), q_off, k_off, v_off, _ptr(bias), _ptr(positions), _ptr(inv_freq if rot_dims else None),
        int(rot_dims), int(bool(interleaved)), _ptr(q_out), _ptr(slots if k_pages is not None else None), _ptr(k_pages),
        _ptr(v_pages), n, q_heads, kv_heads, v_heads, dim, vdim, page_size, _is_bf16(dtype), _stream()), "rotary_cache")


def group_norm(x: torch.Tensor, weight: torch.Tensor, groups: int, eps: float, out: torch.Tensor,
               delta: Optional[torch.Tensor] = None) -> None:
    """``out = weight * n(x)`` for a float32 ``x [rows, width]``, ``n`` dividing each of ``groups`` equal
    consecutive parts of a row by its own root mean square (eps inside the root); 32-bit, rounded once
    to ``out``'s type. With ``delta`` (float32, rows contiguous): ``x += delta`` first, in place."""
    _dense(x, "x", torch.float32, 2)
    _dense(weight, "weight", torch.float32, 1)
    _dense(out, "out", ndim=2)
    _require(out.shape == x.shape and weight.shape[0] == x.shape[1], "out, x and weight disagree on the sizes")
    _require(groups >= 1 and x.shape[1] % groups == 0, "the row does not split into that many equal parts")
    stride = 0
    if delta is not None:
        _f32_rows(delta, "delta")
        _require(delta.shape == x.shape, "delta differs from x in shape")
        stride = delta.stride(0)
    _check(library().dli_group_norm(_ptr(x), _ptr(delta), stride, _ptr(weight), _ptr(out), x.shape[0], x.shape[1],
                                    int(groups), float(eps), _is_bf16(out.dtype), _stream()), "group_norm")


def branch_norm_mean(branches: Sequence[torch.Tensor], weights: Sequence[torch.Tensor], eps: float,
                     out: torch.Tensor) -> None:
    """``out = mean_j(weights[j] * branches[j] / sqrt(mean(branches[j]^2) + eps))`` row by row: up to four
    float32 ``[rows, width]`` branches (rows contiguous), each normalised over the whole row."""
    _dense(out, "out", torch.float32, 2)
    count = len(branches)
    _require(1 <= count <= 4 and len(weights) == count, "one to four branches, each with its weight")
    for y, w in zip(branches, weights):
        _f32_rows(y, "branch")
        _dense(w, "weight", torch.float32, 1)
        _require(y.shape == out.shape and w.shape[0] == out.shape[1], "a branch or its weight differs from out in size")
    ys = (ctypes.c_void_p * count)(*[y.data_ptr() for y in branches])
    strides = (ctypes.c_int64 * count)(*[y.stride(0) for y in branches])
    ws = (ctypes.c_void_p * count)(*[w.data_ptr() for w in weights])
    _check(library().dli_branch_norm_mean(ctypes.cast(ys, _c_ptr), ctypes.cast(strides, _c_ptr), ctypes.cast(ws, _c_ptr),
                                          count, _ptr(out), out.shape[0], out.shape[1], float(eps), _stream()),
           "branch_norm_mean")


# ----------------------------------------------------------------------------- the gated delta rule

def gated_delta_max_taps() -> int:
    return int(library().dli_gated_delta_max_taps())


def conv_prepare(proj: torch.Tensor, b_off: int, a_off: int, conv_w: torch.Tensor, a_log: torch.Tensor,
                 dt_bias: torch.Tensor, state: torch.Tensor, kept_offset: int, q_start: torch.Tensor,
                 positions: torch.Tensor, state_slots: torch.Tensor, out: torch.Tensor, heads: int, kv_heads: int,
                 dim: int, vdim: int) -> None:
    """What the gated delta rule reads, from a step's float32 projections ``proj [n, >=]`` (columns: q and
    k, ``kv_heads x dim`` each, then v, ``heads x vdim``; beta's and the decay's pre-activations at ``b_off``
    and ``a_off``): the short causal convolution per channel (``conv_w [channels, taps]``, the inputs before
    the step's first row from ``state[slot, kept_offset:]``, which then receives the step's last
    ``taps - 1`` inputs), silu, unit q and k per head (q times ``dim^-1/2``), ``beta = sigmoid(b)``,
    ``g = exp(-exp(a_log) softplus(a + dt_bias))``; ``out [n, channels + 2 heads]`` float32."""
    _f32_rows(proj, "proj")
    _dense(conv_w, "conv_w", torch.float32, 2)
    channels, taps = conv_w.shape
    _require(channels == 2 * kv_heads * dim + heads * vdim, "conv_w must hold a row per channel of q, k and v")
    _require(1 <= taps <= gated_delta_max_taps(), "too many taps")
    for name, t in (("a_log", a_log), ("dt_bias", dt_bias)):
        _dense(t, name, torch.float32, 1)
        _require(t.shape[0] == heads, f"{name} must hold a value per head")
    _dense(out, "out", torch.float32, 2)
    n = proj.shape[0]
    _require(out.shape == (n, channels + 2 * heads), "out must be [n, channels + 2 heads]")
    _require(state.is_cuda and state.dtype == torch.float32 and state.dim() == 2 and state.stride(1) == 1
             and state.shape[1] >= kept_offset + (taps - 1) * channels, "state must be float32 [slots, >= kept inputs]")
    for name, t in (("q_start", q_start), ("positions", positions), ("state_slots", state_slots)):
        _dense(t, name, torch.int32, 1)
    entries = state_slots.shape[0]
    _require(q_start.shape[0] == entries + 1 and positions.shape[0] == n, "q_start/state_slots/positions disagree")
    _require(channels <= b_off and b_off + heads <= proj.shape[1] and channels <= a_off and a_off + heads <= proj.shape[1],
             "beta's or the decay's columns lie outside proj")
    _check(library().dli_conv_prepare(
        _ptr(proj), proj.stride(0), int(b_off), int(a_off), _ptr(conv_w), _ptr(a_log), _ptr(dt_bias), _ptr(state),
        state.stride(0), int(kept_offset), _ptr(q_start), _ptr(positions), _ptr(state_slots), _ptr(out), out.stride(0),
        entries, n, heads, kv_heads, dim, vdim, taps, _stream()), "conv_prepare")


def gated_delta_scan(prep: torch.Tensor, state: torch.Tensor, q_start: torch.Tensor, positions: torch.Tensor,
                     state_slots: torch.Tensor, o: torch.Tensor, heads: int, kv_heads: int, dim: int, vdim: int) -> None:
    """Per request and head ``S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q`` over the step's rows
    in order, ``S`` float32 ``[heads][vdim][dim]`` at the start of ``state[slot]`` (zeros at position 0);
    ``prep`` as :func:`conv_prepare` leaves it; ``o [n, heads*vdim]`` float32."""
    _f32_rows(prep, "prep")
    _f32_rows(o, "o")
    n = prep.shape[0]
    _require(prep.shape[1] == 2 * kv_heads * dim + heads * vdim + 2 * heads, "prep must be [n, q | k | v | beta | g]")
    _require(o.shape == (n, heads * vdim), "o must be [n, heads*vdim]")
    _require(heads % kv_heads == 0, "heads do not group onto kv_heads")
    _require(state.is_cuda and state.dtype == torch.float32 and state.dim() == 2 and state.stride(1) == 1
             and state.shape[1] >= heads * vdim * dim, "state must be float32 [slots, >= heads*vdim*dim]")
    for name, t in (("q_start", q_start), ("positions", positions), ("state_slots", state_slots)):
        _dense(t, name, torch.int32, 1)
    entries = state_slots.shape[0]
    _require(q_start.shape[0] == entries + 1 and positions.shape[0] == n, "q_start/state_slots/positions disagree")
    _check(library().dli_gated_delta_scan(
        _ptr(prep), prep.stride(0), _ptr(state), state.stride(0), _ptr(q_start), _ptr(positions), _ptr(state_slots),
        _ptr(o), o.stride(0), entries, n, heads, kv_heads, dim, vdim, _stream()), "gated_delta_scan")


HEAD_GATES = {"sigmoid": 0, "silu": 1, "none": 2}


def head_norm_gate(o: torch.Tensor, g_pre: Optional[torch.Tensor], norm_w: torch.Tensor, eps: float, out: torch.Tensor,
                   heads: int, dim: int, gate: str = "silu", den: Optional[torch.Tensor] = None) -> None:
    """``out = o / sqrt(mean_head(o^2) + eps) * norm_w * gate(g_pre)`` head by head: ``o`` and ``g_pre`` float32
    ``[n, heads*dim]`` (rows contiguous), ``norm_w`` float32 ``[heads*dim]``, ``gate`` ``"silu"``, ``"sigmoid"`` or
    ``"none"`` (the per-head norm alone; ``g_pre`` is then ``None``)."""
    _f32_rows(o, "o")
    _rows(out, "out", out.dtype)
    _dense(norm_w, "norm_w", torch.float32, 1)
    n, width = o.shape[0], heads * dim
    _require(gate in HEAD_GATES, f"gate must be one of {sorted(HEAD_GATES)}")
    _require((g_pre is None) == (gate == "none"), "g_pre comes with a gate, and only with one")
    if g_pre is not None:
        _f32_rows(g_pre, "g_pre")
        _require(g_pre.shape == (n, width), "g_pre must be [n, heads*dim]")
    _require(o.shape == (n, width) and out.shape == (n, width) and norm_w.shape[0] == width,
             "o, out and norm_w must be [n, heads*dim]")
    if den is not None:   # every head of ``o`` is divided by its value first
        _dense(den, "den", torch.float32, 2)
        _require(den.shape == (n, heads), "den must be [n, heads]")
    _check(library().dli_head_norm_gate(_ptr(o), o.stride(0), _ptr(g_pre), 0 if g_pre is None else g_pre.stride(0),
                                        _ptr(norm_w), float(eps), _ptr(out), out.stride(0), n, heads, dim,
                                        HEAD_GATES[gate], _ptr(den), _is_bf16(out.dtype), _stream()), "head_norm_gate")


# ----------------------------------------------------------------------------- feed-forward: polynomial activation, experts

def poly_norm(z: torch.Tensor, coef: torch.Tensor, eps: float, out: torch.Tensor) -> None:
    """``out = a N(z) + b N(z^2) + c N(z^3) + e`` row by row, ``coef = (a, b, c, e)`` float32 on the device,
    ``N(x) = x / sqrt(mean(x^2) + eps)``; ``z`` float32, ``out`` float32 or bfloat16."""
    _f32_rows(z, "z")
    _rows(out, "out", out.dtype)
    _dense(coef, "coef", torch.float32, 1)
    _require(coef.shape[0] == 4 and out.shape == z.shape, "four coefficients; out like z")
    _check(library().dli_poly_norm(_ptr(z), z.stride(0), _ptr(coef), _ptr(out), out.stride(0), z.shape[0], z.shape[1],
                                   float(eps), _is_bf16(out.dtype), _stream()), "poly_norm")


def clamped_glu(gate_up: torch.Tensor, out: torch.Tensor, limit: float, alpha: float, up_shift: float = 1.0) -> None:
    """``out = g sigmoid(alpha g) (u + up_shift)`` with ``g = min(gate, limit)``, ``u = clamp(up, -limit, limit)``
    (an infinite limit, ``alpha = 1`` and ``up_shift = 0``: ``silu(gate) * up``);
    ``gate_up [n, >= 2 ff]`` holds gate then up (rows contiguous), ``out [n, ff]`` of the same type."""
    _rows(gate_up, "gate_up", out.dtype)
    _dense(out, "out", ndim=2)
    n, ff = out.shape
    _require(gate_up.shape[0] == n and gate_up.shape[1] >= 2 * ff, "gate_up must hold gate and up for every row")
    _check(library().dli_clamped_glu(_ptr(gate_up), gate_up.stride(0), _ptr(out), n, ff, float(limit), float(alpha),
                                     float(up_shift), _is_bf16(out.dtype), _stream()), "clamped_glu")


def router_choose(logits: torch.Tensor, total: int, correction: Optional[torch.Tensor], groups: int, keep: int, top: int,
                  scale: float, ids: torch.Tensor, weights: torch.Tensor, bias: Optional[torch.Tensor] = None) -> None:
    """The router's choice per row of float32 ``logits [n, >= total]``: scores ``softmax`` over the first
    ``total`` columns (plus ``bias``, float32 ``[total]``, where the router has one); choice scores add ``correction``; with ``groups`` > 1 only the ``keep`` groups of
    neighbours with the largest best choice score can be chosen; ``ids [n, top]`` int32 are the largest
    choice scores (lowest index on a tie), ``weights [n, top]`` their scores (without correction) divided
    by their sum + 1e-20, times ``scale``."""
    _f32_rows(logits, "logits")
    n = logits.shape[0]
    _require(logits.shape[1] >= total, "logits must hold every router output")
    if correction is not None:
        _dense(correction, "correction", torch.float32, 1)
        _require(correction.shape[0] == total, "correction must hold a value per router output")
    if bias is not None:
        _dense(bias, "bias", torch.float32, 1)
        _require(bias.shape[0] == total, "bias must hold a value per router output")
    _dense(ids, "ids", torch.int32, 2)
    _dense(weights, "weights", torch.float32, 2)
    _require(ids.shape == (n, top) and weights.shape == (n, top), "ids and weights must be [n, top]")
    _require(1 <= top <= min(total, 64) and groups >= 1 and total % groups == 0 and 1 <= keep <= groups
             and keep * (total // groups) >= top, "the router's sizes do not fit each other")
    _check(library().dli_router_choose(_ptr(logits), logits.stride(0), _ptr(bias), _ptr(correction), n, int(total), int(groups),
                                       int(keep), int(top), float(scale), _ptr(ids), _ptr(weights), _stream()),
           "router_choose")


def expert_products(ids: torch.Tensor, h: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor,
                    limit: float, alpha: float, up_shift: float = 1.0) -> torch.Tensor:
    """The chosen experts' results for every (token, choice): ``z [n * top, width]`` float32, row
    ``t * top + j`` holding ``w_down[e] clamped_glu(w_gate[e] h_t, w_up[e] h_t)`` for ``e = ids[t, j]`` (rows of
    ids at or above the number of experts are left unwritten). ``w_gate, w_up [experts, ff, width]``,
    ``w_down [experts, width, ff]`` of ``h``'s type. Nothing here waits for the device: the rows are
    sorted by expert and cut into tiles on the device."""
    _dense(ids, "ids", torch.int32, 2)
    n, top = ids.shape
    _rows(h, "h", h.dtype)
    for name, w in (("w_gate", w_gate), ("w_up", w_up), ("w_down", w_down)):
        _dense(w, name, h.dtype, 3)
    experts, ff, width = w_gate.shape
    _require(w_up.shape == w_gate.shape and w_down.shape == (experts, width, ff) and h.shape == (n, width),
             "h [n, width], w_gate/w_up [experts, ff, width], w_down [experts, width, ff] do not fit")
    slots = n * top
    tile_rows = int(library().dli_expert_tile_rows(width, ff, _is_bf16(h.dtype)))
    max_tiles = max(1, min(slots, slots // tile_rows + experts))
    ints = torch.empty(experts + 1 + slots + 2 * max_tiles + 1, device=h.device, dtype=torch.int32)
    offsets, order = ints[:experts + 1], ints[experts + 1:experts + 1 + slots]
    tiles = ints[experts + 1 + slots:]
    tile_expert, tile_row0, tile_count = tiles[:max_tiles], tiles[max_tiles:2 * max_tiles], tiles[2 * max_tiles:]
    y = torch.empty(slots, ff, device=h.device, dtype=h.dtype)
    z = torch.empty(slots, width, device=h.device, dtype=torch.float32)
    _check(library().dli_expert_products(
        _ptr(ids), _ptr(h), h.stride(0), _ptr(w_gate), _ptr(w_up), _ptr(w_down), _ptr(offsets), _ptr(order),
        _ptr(tile_expert), _ptr(tile_row0), _ptr(tile_count), max_tiles, _ptr(y), _ptr(z), n, top, experts, width, ff,
        float(limit), float(alpha), float(up_shift), _is_bf16(h.dtype), _stream()), "expert_products")
    return z


def expert_combine(ids: torch.Tensor, weights: torch.Tensor, z: Optional[torch.Tensor], h: torch.Tensor, experts: int,
                   out: torch.Tensor, shared: Optional[torch.Tensor] = None,
                   shared_gate: Optional[torch.Tensor] = None) -> None:
    """``out[t] = sum_j weights[t, j] * (z[t * top + j] if ids[t, j] < experts else h[t])
    + sigmoid(shared_gate[t]) * shared[t]``; ``out`` float32 ``[n, width]``, ``shared`` float32 ``[n, width]``
    and ``shared_gate`` float32 ``[n, 1]`` (a column of a wider matrix will do), both optional."""
    _dense(ids, "ids", torch.int32, 2)
    _dense(weights, "weights", torch.float32, 2)
    n, top = ids.shape
    _rows(h, "h", h.dtype)
    _dense(out, "out", torch.float32, 2)
    width = out.shape[1]
    _require(weights.shape == (n, top) and h.shape == (n, width) and out.shape[0] == n, "ids, weights, h and out disagree")
    if z is not None:
        _dense(z, "z", torch.float32, 2)
        _require(z.shape == (n * top, width), "z must be [n * top, width]")
    else:
        _require(experts == 0, "without z every chosen id must be an identity expert")
    s_stride = g_stride = 0
    if shared is not None:
        _f32_rows(shared, "shared")
        _require(shared.shape == (n, width), "shared must be [n, width]")
        s_stride = shared.stride(0)
    if shared_gate is not None:
        _require(shared is not None and shared_gate.is_cuda and shared_gate.dtype == torch.float32
                 and shared_gate.dim() == 2 and shared_gate.shape == (n, 1), "shared_gate must be float32 [n, 1] beside shared")
        g_stride = shared_gate.stride(0)
    _check(library().dli_expert_combine(_ptr(ids), _ptr(weights), _ptr(z), _ptr(h), h.stride(0), _ptr(shared_gate), g_stride,
                                        _ptr(shared), s_stride, _ptr(out), n, top, int(experts), width, _is_bf16(h.dtype),
                                        _stream()), "expert_combine")


# ----------------------------------------------------------------------------- short convolutions, the selective scan

def _step_arrays(q_start: torch.Tensor, positions: torch.Tensor, state_slots: torch.Tensor, n: int) -> int:
    for name, t in (("q_start", q_start), ("positions", positions), ("state_slots", state_slots)):
        _dense(t, name, torch.int32, 1)
    entries = state_slots.shape[0]
    _require(q_start.shape[0] == entries + 1 and positions.shape[0] == n, "q_start/state_slots/positions disagree")
    return entries


def _state_rows(state: torch.Tensor, floats: int) -> None:
    _require(state.is_cuda and state.dtype == torch.float32 and state.dim() == 2 and state.stride(1) == 1
             and state.shape[1] >= floats, f"state must be float32 [slots, >= {floats}]")


def causal_conv(x: torch.Tensor, conv_w: torch.Tensor, bias: Optional[torch.Tensor], state: torch.Tensor, kept_offset: int,
                q_start: torch.Tensor, positions: torch.Tensor, state_slots: torch.Tensor, out: torch.Tensor,
                rounded: Optional[torch.Tensor] = None, act: str = "silu") -> None:
    """A short causal convolution over time per channel: ``out[t, c] = act(bias[c] + sum_j conv_w[c, taps-1-j] x[t-j, c])``
    with zeros before position 0. ``x`` float32 ``[n, >= channels]`` (rows contiguous; the channels from
    column 0), ``conv_w`` float32 ``[channels, taps]`` (the last column is the current token's). The inputs
    before an entry's first row come from ``state[slot, kept_offset:]`` (``[taps-1, channels]``, the newest
    last), which then receives the entry's last ``taps - 1`` inputs. ``out`` float32 ``[n, channels]``;
    ``rounded``: the result once more (float32 or bfloat16), for the product that reads it next.
    ``act``: ``"silu"`` or ``"none"``."""
    _f32_rows(x, "x")
    _dense(conv_w, "conv_w", torch.float32, 2)
    channels, taps = conv_w.shape
    n = x.shape[0]
    _require(x.shape[1] >= channels, "x must hold every channel")
    _require(1 <= taps <= gated_delta_max_taps(), "too many taps")
    if bias is not None:
        _dense(bias, "bias", torch.float32, 1)
        _require(bias.shape[0] == channels, "bias must hold a value per channel")
    _f32_rows(out, "out")
    _require(out.shape == (n, channels), "out must be [n, channels]")
    r_stride, r_bf16 = 0, 0
    if rounded is not None:
        _rows(rounded, "rounded", rounded.dtype)
        _require(rounded.shape == (n, channels), "the rounded copy must be [n, channels]")
        r_stride, r_bf16 = rounded.stride(0), _is_bf16(rounded.dtype)
    _require(act in ("silu", "none"), "act must be 'silu' or 'none'")
    _state_rows(state, kept_offset + (taps - 1) * channels)
    entries = _step_arrays(q_start, positions, state_slots, n)
    _check(library().dli_causal_conv(
        _ptr(x), x.stride(0), _ptr(conv_w), _ptr(bias), _ptr(state), state.stride(0), int(kept_offset), _ptr(q_start),
        _ptr(positions), _ptr(state_slots), _ptr(out), out.stride(0), _ptr(rounded), r_stride, r_bf16, entries, n,
        channels, taps, int(act == "silu"), _stream()), "causal_conv")


def selective_scan_max_states() -> int:
    return int(library().dli_selective_scan_max_states())


def selective_scan(x: torch.Tensor, dt: torch.Tensor, bc: torch.Tensor, b_off: int, c_off: int, z: Optional[torch.Tensor],
                   a_log: torch.Tensor, d: Optional[torch.Tensor], state: torch.Tensor, q_start: torch.Tensor,
                   positions: torch.Tensor, state_slots: torch.Tensor, out: torch.Tensor) -> None:
    """Per request and channel ``S[n] <- exp(dt A[n]) S[n] + dt x B[n]``, ``y = sum_n S[n] C[n] + d x``,
    ``out = y silu(z)`` over the step's rows in order, ``A = -exp(a_log)``. ``x``, ``dt`` (positive step sizes)
    and ``z`` (``None``: no gate) float32 ``[n, channels]`` (rows contiguous), ``bc`` float32 ``[n, >=]`` with the
    token's B and C (``states`` values each) at columns ``b_off`` and ``c_off``, ``a_log`` float32
    ``[channels, states]``, ``d`` float32 ``[channels]`` or ``None``. ``S`` float32 ``[channels][states]`` at
    the start of ``state[slot]`` (zeros at position 0). ``out [n, channels]``, float32 or bfloat16."""
    _f32_rows(x, "x")
    _f32_rows(dt, "dt")
    _f32_rows(bc, "bc")
    _dense(a_log, "a_log", torch.float32, 2)
    channels, states = a_log.shape
    n = x.shape[0]
    _require(x.shape == (n, channels) and dt.shape == (n, channels), "x and dt must be [n, channels]")
    _require(1 <= states <= selective_scan_max_states(), "too many states a channel")
    _require(bc.shape[0] == n and 0 <= b_off and b_off + states <= bc.shape[1] and 0 <= c_off
             and c_off + states <= bc.shape[1], "B or C lie outside bc")
    if z is not None:
        _f32_rows(z, "z")
        _require(z.shape == (n, channels), "z must be [n, channels]")
    if d is not None:
        _dense(d, "d", torch.float32, 1)
        _require(d.shape[0] == channels, "d must hold a value per channel")
    _rows(out, "out", out.dtype)
    _require(out.shape == (n, channels), "out must be [n, channels]")
    _state_rows(state, channels * states)
    entries = _step_arrays(q_start, positions, state_slots, n)
    _check(library().dli_selective_scan(
        _ptr(x), x.stride(0), _ptr(dt), dt.stride(0), _ptr(bc), bc.stride(0), int(b_off), int(c_off), _ptr(z),
        0 if z is None else z.stride(0), _ptr(a_log), _ptr(d), _ptr(state), state.stride(0), _ptr(q_start), _ptr(positions),
        _ptr(state_slots), _ptr(out), out.stride(0), entries, n, channels, states, _is_bf16(out.dtype), _stream()),
        "selective_scan")


# ----------------------------------------------------------------------------- the gated linear recurrence

def bounded_gates(proj: torch.Tensor, q_off: int, f_off: int, width: int, f_bias: Optional[torch.Tensor],
                  lower: Optional[torch.Tensor]) -> None:
    """In place on float32 ``proj [n, >=]``: the ``width`` columns from ``q_off`` become ``silu`` of themselves,
    those from ``f_off`` become ``lower + (1 - lower) sigmoid(. + f_bias)`` (``lower``, ``f_bias`` float32
    ``[width]``; ``None``: zeros)."""
    _f32_rows(proj, "proj")
    for name, t in (("f_bias", f_bias), ("lower", lower)):
        if t is not None:
            _dense(t, name, torch.float32, 1)
            _require(t.shape[0] == width, f"{name} must hold a value per column")
    _require(0 <= q_off and q_off + width <= proj.shape[1] and 0 <= f_off and f_off + width <= proj.shape[1]
             and (q_off + width <= f_off or f_off + width <= q_off), "the columns lie outside proj or overlap")
    _check(library().dli_bounded_gates(_ptr(proj), proj.stride(0), int(q_off), int(f_off), _ptr(f_bias), _ptr(lower),
                                       proj.shape[0], int(width), _stream()), "bounded_gates")


def gated_linear_scan(proj: torch.Tensor, q_off: int, f_off: int, v_off: int, state: torch.Tensor, q_start: torch.Tensor,
                      positions: torch.Tensor, state_slots: torch.Tensor, o: torch.Tensor, heads: int, dim: int,
                      vdim: int) -> None:
    """Per request and head ``S <- diag(f) S + (1 - f) v^T``, ``o = S^T q`` over the step's rows in order:
    float32 ``proj [n, >=]`` holds q and f (``heads x dim`` each, as :func:`bounded_gates` leaves them) and v
    (``heads x vdim``) at their columns; ``S`` float32 ``[heads][vdim][dim]`` at the start of ``state[slot]``
    (zeros at position 0); ``o [n, heads*vdim]`` float32."""
    _f32_rows(proj, "proj")
    _f32_rows(o, "o")
    n = proj.shape[0]
    _require(o.shape == (n, heads * vdim), "o must be [n, heads*vdim]")
    _require(all(0 <= off and off + heads * size <= proj.shape[1]
                 for off, size in ((q_off, dim), (f_off, dim), (v_off, vdim))), "q, f or v lie outside proj")
    _state_rows(state, heads * vdim * dim)
    entries = _step_arrays(q_start, positions, state_slots, n)
    _check(library().dli_gated_linear_scan(
        _ptr(proj), proj.stride(0), int(q_off), int(f_off), int(v_off), _ptr(state), state.stride(0), _ptr(q_start),
        _ptr(positions), _ptr(state_slots), _ptr(o), o.stride(0), entries, n, heads, dim, vdim, _stream()),
        "gated_linear_scan")


# ----------------------------------------------------------------------------- attention through a latent

def latent_norm_cache(proj: torch.Tensor, q_off: int, q_rank: int, c_off: int, rank: int, q_weight: torch.Tensor,
                      c_weight: torch.Tensor, eps: float, q_out: torch.Tensor, slots: torch.Tensor, k_pages: torch.Tensor,
                      v_pages: torch.Tensor) -> None:
    """From float32 ``proj [n, >=]``: the ``q_rank`` columns from ``q_off`` and the ``rank`` columns from ``c_off``
    each divided by their root mean square (eps inside the root) and multiplied by their weight; the first
    goes to ``q_out [n, q_rank]``, the second into the token's cache slot (negative: not cached) as a key,
    ``k_pages [pages, 1, page_size, rank]``, and as a value, ``v_pages [pages, 1, rank, page_size]``."""
    _f32_rows(proj, "proj")
    n = proj.shape[0]
    _dense(q_weight, "q_weight", torch.float32, 1)
    _dense(c_weight, "c_weight", torch.float32, 1)
    _require(q_weight.shape[0] == q_rank and c_weight.shape[0] == rank, "the weights must fit the latents")
    _require(0 <= q_off and q_off + q_rank <= proj.shape[1] and 0 <= c_off and c_off + rank <= proj.shape[1],
             "the latents lie outside proj")
    _dense(q_out, "q_out", ndim=2)
    _require(q_out.shape == (n, q_rank), "q_out must be [n, q_rank]")
    _dense(k_pages, "k_pages", q_out.dtype, 4)
    _dense(v_pages, "v_pages", q_out.dtype, 4)
    pages, _, page_size, _ = k_pages.shape
    _require(k_pages.shape == (pages, 1, page_size, rank) and v_pages.shape == (pages, 1, rank, page_size),
             "the pages must hold one latent a token: k [pages, 1, page_size, rank], v [pages, 1, rank, page_size]")
    _dense(slots, "slots", torch.int32, 1)
    _require(slots.shape[0] == n, "a cache slot per row")
    _check(library().dli_latent_norm_cache(
        _ptr(proj), proj.stride(0), int(q_off), int(q_rank), int(c_off), int(rank), _ptr(q_weight), _ptr(c_weight),
        float(eps), _ptr(q_out), _ptr(slots), _ptr(k_pages), _ptr(v_pages), n, page_size, _is_bf16(q_out.dtype),
        _stream()), "latent_norm_cache")


def head_products(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, gate: Optional[torch.Tensor] = None) -> None:
    """``out[t, h] = w[h] x[t, h]`` for every head (32-bit sums, ascending k): ``x [n, heads*k]``,
    ``w [heads, m, k]``, ``out [n, heads*m]``, all of one type (float32 or bfloat16, rows contiguous);
    ``gate`` (float32 ``[n, heads*m]``): the result is multiplied by its sigmoid."""
    _dense(w, "w", ndim=3)
    heads, m, k = w.shape
    _rows(x, "x", w.dtype)
    _rows(out, "out", w.dtype)
    n = x.shape[0]
    _require(x.shape == (n, heads * k) and out.shape == (n, heads * m), "x must be [n, heads*k] and out [n, heads*m]")
    g_stride = 0
    if gate is not None:
        _f32_rows(gate, "gate")
        _require(gate.shape == out.shape, "gate differs from out in shape")
        g_stride = gate.stride(0)
    _check(library().dli_head_products(_ptr(x), x.stride(0), _ptr(w), _ptr(out), out.stride(0), _ptr(gate), g_stride, n,
                                       heads, m, k, _is_bf16(w.dtype), _stream()), "head_products")


# ----------------------------------------------------------------------------- recurrences under scalar gates, differential maps

def exp_gates(pre: torch.Tensor, i_off: int, f_off: int, i_bias: Optional[torch.Tensor], f_bias: Optional[torch.Tensor],
              cap: float, state: torch.Tensor, m_off: int, q_start: torch.Tensor, positions: torch.Tensor,
              state_slots: torch.Tensor, heads: int) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """The factors of a matrix memory with exponential gates, per row and head of the step: from the float32
    pre-activations ``pre [n, >=]`` (input gate of head ``h`` at column ``i_off + h``, forget gate at
    ``f_off + h``; biases float32 ``[heads]``) the log gates ``i = cap tanh(. / cap)`` (``cap`` 0: as they are) and
    ``f = logsigmoid(cap tanh(. / cap))``, the running reference point ``m <- max(f + m, i)`` (kept at
    ``state[slot][m_off + h]``, 0 at position 0), and ``keep = exp(f + m_old - m)``, ``write = exp(i - m)``,
    ``floor = exp(-m)``, and the logarithm of ``keep`` (never above zero): four float32 ``[n, heads]``."""
    _f32_rows(pre, "pre")
    n = pre.shape[0]
    _require(0 <= i_off and i_off + heads <= pre.shape[1] and 0 <= f_off and f_off + heads <= pre.shape[1],
             "the gates lie outside pre's columns")
    for name, t in (("i_bias", i_bias), ("f_bias", f_bias)):
        if t is not None:
            _dense(t, name, torch.float32, 1)
            _require(t.shape[0] == heads, f"{name} must hold a value per head")
    _state_rows(state, m_off + heads)
    entries = _step_arrays(q_start, positions, state_slots, n)
    out = torch.empty(4, n, heads, device=pre.device, dtype=torch.float32)
    _check(library().dli_exp_gates(_ptr(pre), pre.stride(0), int(i_off), int(f_off), _ptr(i_bias), _ptr(f_bias), float(cap),
                                   _ptr(state), state.stride(0), int(m_off), _ptr(q_start), _ptr(positions), _ptr(state_slots),
                                   _ptr(out[0]), _ptr(out[1]), _ptr(out[2]), _ptr(out[3]), entries, n, heads, _stream()),
           "exp_gates")
    return out[0], out[1], out[2], out[3]


def scalar_gate_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, state: torch.Tensor, q_start: torch.Tensor,
                     positions: torch.Tensor, state_slots: torch.Tensor, o: torch.Tensor, heads: int, dim: int, vdim: int, *,
                     keep: Optional[torch.Tensor] = None, write: Optional[torch.Tensor] = None,
                     decay: Optional[torch.Tensor] = None, floor: Optional[torch.Tensor] = None,
                     den: Optional[torch.Tensor] = None, q_scale: float = 1.0, silu: bool = False,
                     log_keep: Optional[torch.Tensor] = None, chunked: bool = True) -> None:
    """Per request and head ``S <- a S + b k v^T``, ``o = S^T q`` over the step's rows in order, with
    ``a, b = keep, write`` (float32 ``[n, heads]``) or ``a = decay[head]``, ``b = 1``. ``q, k [n, heads*dim]`` and
    ``v [n, heads*vdim]`` are float32 with contiguous rows (columns of a wider matrix will do); with ``silu`` all
    three pass through silu first; q is multiplied by ``q_scale``. With ``floor`` (float32 ``[n, heads]``) the state
    has one more column a head, for a value that is always one, and ``den [n, heads]`` receives
    ``max(|that column's result|, floor) + 1e-6``. ``S`` float32 ``[heads][vdim (+ 1)][dim]`` at the start of
    ``state[slot]`` (zeros at position 0); ``o [n, heads*vdim]`` float32. A step with portions whose heads hold 16 to 64
    keys in steps of 16 runs 64 tokens at a time on the matrix cores, in 32-bit (``chunked``; under gates it needs
    ``log_keep``, the logarithm of ``keep``; not with ``silu``); any other walks the tokens one by one."""
    for name, t, width in (("q", q, heads * dim), ("k", k, heads * dim), ("v", v, heads * vdim), ("o", o, heads * vdim)):
        _f32_rows(t, name)
        _require(t.shape[1] == width, f"{name} must hold {width} columns")
    n = q.shape[0]
    _require(k.shape[0] == n and v.shape[0] == n and o.shape[0] == n, "q, k, v and o differ in rows")
    _require((keep is None) == (write is None) and (keep is not None or decay is not None), "keep and write, or decay")
    _require((floor is None) == (den is None) and (floor is None or keep is not None), "floor and den come with the gates")
    for name, t in (("keep", keep), ("write", write), ("floor", floor), ("den", den), ("log_keep", log_keep)):
        if t is not None:
            _dense(t, name, torch.float32, 2)
            _require(t.shape == (n, heads), f"{name} must be [n, heads]")
    if decay is not None:
        _dense(decay, "decay", torch.float32, 1)
        _require(decay.shape[0] == heads, "decay must hold a value per head")
    _state_rows(state, heads * (vdim + (floor is not None)) * dim)
    entries = _step_arrays(q_start, positions, state_slots, n)
    _check(library().dli_scalar_gate_scan(
        _ptr(q), q.stride(0), _ptr(k), k.stride(0), _ptr(v), v.stride(0), _ptr(keep), _ptr(write), _ptr(log_keep), heads,
        _ptr(decay), _ptr(floor), _ptr(den), _ptr(state), state.stride(0), _ptr(q_start), _ptr(positions), _ptr(state_slots),
        _ptr(o), o.stride(0), entries, n, heads, dim, vdim, float(q_scale), int(bool(silu)), int(bool(chunked)), _stream()),
        "scalar_gate_scan")


def diff_head_norm(a: torch.Tensor, lam: float, after: float, eps: float, gate: Optional[torch.Tensor], out: torch.Tensor,
                   heads: int, vdim: int) -> None:
    """Two attention maps over the same values combined head by head: ``a`` float32 ``[n, 2*heads*vdim]`` holds the
    first map's heads, then the second's; ``out[:, h] = d / sqrt(mean(d^2) + eps) * after * sigmoid(gate[:, h])`` with
    ``d = a1_h - lam a2_h`` (``gate`` float32 ``[n, heads]``, a column range of a wider matrix will do; ``None``: 1)."""
    _f32_rows(a, "a")
    _rows(out, "out", out.dtype)
    n = a.shape[0]
    _require(a.shape[1] == 2 * heads * vdim and out.shape == (n, heads * vdim), "a [n, 2*heads*vdim], out [n, heads*vdim]")
    if gate is not None:
        _f32_rows(gate, "gate")
        _require(gate.shape == (n, heads), "gate must be [n, heads]")
    _check(library().dli_diff_head_norm(_ptr(a), a.stride(0), float(lam), float(after), float(eps), _ptr(gate),
                                        0 if gate is None else gate.stride(0), _ptr(out), out.stride(0), n, heads, vdim,
                                        _is_bf16(out.dtype), _stream()), "diff_head_norm")


def branch_weighted_sum(branches: Sequence[torch.Tensor], scales: Sequence[float], out: torch.Tensor) -> None:
    """``out = sum_b scales[b] * branches[b]``: one to four float32 ``[n, width]`` matrices (rows contiguous)."""
    _dense(out, "out", torch.float32, 2)
    _require(1 <= len(branches) <= 4 and len(scales) == len(branches), "one to four branches, a scale each")
    for i, y in enumerate(branches):
        _f32_rows(y, f"branch {i}")
        _require(y.shape == out.shape, "a branch differs from out in shape")
    count = len(branches)
    ptrs = (ctypes.c_void_p * count)(*[y.data_ptr() for y in branches])
    strides = (ctypes.c_int64 * count)(*[y.stride(0) for y in branches])
    sc = (ctypes.c_float * count)(*[float(x) for x in scales])
    _check(library().dli_branch_weighted_sum(ptrs, strides, sc, count, _ptr(out), out.shape[0], out.shape[1], _stream()),
           "branch_weighted_sum")


def scale_f32(y: torch.Tensor, scale: float) -> None:
    """``y *= scale`` in place (float32)."""
    _dense(y, "y", torch.float32)
    _check(library().dli_scale_f32(_ptr(y), y.numel(), float(scale), _stream()), "scale_f32")


def table_choose(table: torch.Tensor, token_ids: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor) -> None:
    """A router that is a table: ``ids[t] = table[token_ids[t]]`` (``table`` int32 ``[vocabulary, top]``), every
    weight ``1 / top``."""
    _dense(table, "table", torch.int32, 2)
    _dense(token_ids, "token_ids", torch.int32, 1)
    _dense(ids, "ids", torch.int32, 2)
    _dense(weights, "weights", torch.float32, 2)
    n, top = ids.shape
    _require(table.shape[1] == top and token_ids.shape[0] == n and weights.shape == (n, top), "table, ids and weights disagree")
    _check(library().dli_table_choose(_ptr(table), _ptr(token_ids), n, top, table.shape[0], _ptr(ids), _ptr(weights), _stream()),
           "table_choose")


def rms_norm_pair(x: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, eps: float, out1: torch.Tensor, out2: torch.Tensor) -> None:
    """``out1 = w1 * x / sqrt(mean(x^2) + eps)`` and ``out2`` alike with ``w2``: two norms of one float32 ``x`` that
    agree on eps, from one pass over the rows' statistics; both rounded once to the outputs' type."""
    _dense(x, "x", torch.float32, 2)
    for name, w in (("w1", w1), ("w2", w2)):
        _dense(w, name, torch.float32, 1)
        _require(w.shape[0] == x.shape[1], f"{name} must hold a value per column")
    _dense(out1, "out1", ndim=2)
    _dense(out2, "out2", out1.dtype, 2)
    _require(out1.shape == x.shape and out2.shape == x.shape, "the outputs differ from x in shape")
    _check(library().dli_rms_norm_pair(_ptr(x), _ptr(w1), _ptr(w2), _ptr(out1), _ptr(out2), x.shape[0], x.shape[1], float(eps),
                                       _is_bf16(out1.dtype), _stream()), "rms_norm_pair")


def add_pair_into_stream(x: torch.Tensor, a: torch.Tensor, b: torch.Tensor) -> None:
    """``x += a + b`` (all float32, equal shapes): the two results are added to each other first."""
    for name, t in (("x", x), ("a", a), ("b", b)):
        _dense(t, name, torch.float32, 2)
    _require(a.shape == x.shape and b.shape == x.shape, "a and b differ from x in shape")
    _check(library().dli_add_pair_into_stream(_ptr(x), _ptr(a), _ptr(b), x.numel(), _stream()), "add_pair_into_stream")


def silu_columns(x: torch.Tensor) -> None:
    """``x <- silu(x)`` in place: float32 ``[n, width]`` with contiguous rows (columns of a wider matrix will do)."""
    _f32_rows(x, "x")
    _check(library().dli_silu_columns(_ptr(x), x.stride(0), x.shape[0], x.shape[1], _stream()), "silu_columns")
