"""Python face of the HIP kernels: one function per kernel.

Each wrapper checks on the host that the operands are what the kernel and its
grid assume (device, dtype, contiguity, shapes) and then launches on torch's
current stream.  There is no other implementation behind these functions: without
the library, or on a tensor that is not on the GPU, they raise.
"""
from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_void_p

import torch

from ..errors import KernelError, ShapeError
from .build import load

F32, BF16 = 0, 1
_CODES = {torch.float32: F32, torch.bfloat16: BF16}

_SIGNATURES = {
    "ri_embed_gather": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_void_p],
    "ri_add_rmsnorm": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_float, c_void_p, c_int,
                       c_int, c_int, c_void_p],
    "ri_add_rows": [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_void_p],
    "ri_qk_norm_rope_kv_write": [c_void_p, c_int, c_void_p, c_void_p, c_float, c_void_p, c_int, c_void_p, c_void_p,
                                 c_void_p, c_int, c_int, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int,
                                 c_int, c_int, c_int, c_int, c_void_p],
    "ri_attention": [c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int,
                     c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_float, c_void_p, c_void_p],
    "ri_qk_norm_temper_kv_write": [c_void_p, c_int, c_void_p, c_void_p, c_float, c_float, c_int, c_void_p, c_void_p,
                                   c_void_p, c_int, c_int, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int,
                                   c_int, c_int, c_int, c_int, c_void_p],
    "ri_streams_read_norm": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_void_p,
                             c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_int, c_void_p, c_int, c_int, c_void_p],
    "ri_embed_positions_norm": [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_float,
                                c_int, c_int, c_int, c_void_p],
    "ri_gla_scan": [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_float, c_float,
                    c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "ri_gla_step_fits": [c_int, c_int],
    "ri_decay_chunks_fit": [c_int, c_int],
    "ri_gla_step": [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_float, c_float,
                    c_void_p, c_void_p, c_void_p, c_float, c_int, c_int, c_int, c_int, c_void_p],
    "ri_gla_norm_gate": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_float, c_int, c_int, c_int,
                         c_void_p],
    "ri_relu_squared": [c_void_p, c_void_p, c_int, ctypes.c_long, c_void_p],
    "ri_gelu_tanh": [c_void_p, c_void_p, c_int, ctypes.c_long, c_void_p],
    "ri_gelu_erf": [c_void_p, c_void_p, c_int, ctypes.c_long, c_void_p],
    "ri_delta_prepare": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p,
                         c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "ri_delta_max_dim": [],
    "ri_delta_scan": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                      c_int, c_void_p],
    "ri_delta_step_fits": [c_int, c_int],
    "ri_delta_step": [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                      c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "ri_experts_route": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p],
    "ri_experts_activate": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_float, c_void_p],
    "ri_experts_sort": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p],
    "ri_experts_gather": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p],
    "ri_experts_combine": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p],
    "ri_experts_few_tokens": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                              c_int, c_float, c_void_p],
    "ri_attention_prefill_bf16": [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                                  c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_float, c_void_p, c_void_p],
    "ri_attention_decode_bf16": [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                 c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_float, c_void_p, c_int,
                                 c_void_p],
    "ri_attention_decode_kept_bf16": [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                      c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_float, c_void_p, c_int,
                                      c_int, c_void_p, c_void_p],
    "ri_attention_decode_fused_bf16": [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_float,
                                       c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                       c_int, c_int, c_int, c_int, c_float, c_int, c_void_p],
    "ri_gemm_f32": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
    "ri_gemv_bf16": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
    "ri_sample": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_float, c_int, c_float, c_float,
                  c_void_p],
    "ri_mark_seen": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p],
    "ri_sample_split": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_float, c_int,
                        c_float, c_float, c_void_p],
    "ri_gemm_skinny_packed_bf16": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "ri_gemm_mid_packed_bf16": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "ri_gemm_wide_packed_bf16": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                 c_int, c_void_p],
    "ri_gemm_wide_packed_bf16_plan": [c_int, c_int, c_int, c_void_p, c_void_p],
    "ri_gemm_wide_stretch_plan": [c_int, c_int, c_int, c_void_p, c_void_p],
    "ri_compute_units": [],
    "ri_sum_parts": [c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "ri_attention_decode_chunks": [c_int],
    "ri_attention_decode_streams": [c_int, c_int, c_int],
    "ri_attention_decode_pieces": [c_int, c_int, c_int, c_int],
    "ri_gemv_bf16_partials": [c_int, c_int],
    "ri_gemm_skinny_packed_bf16_partials": [c_int],
    "ri_gemv_bf16_linked": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_int, c_float,
                            c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p],
    "ri_gemm_skinny_packed_bf16_linked": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p,
                                          c_int, c_float, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p],
    "ri_swiglu": [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
    "ri_add_bias": [c_void_p, c_int, c_void_p, c_int, c_int, c_void_p],
    "ri_finish_norm": [c_void_p, c_void_p, c_void_p, c_int, c_float, c_int, c_int, c_int, c_void_p],
    "ri_argmax": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p],
    "ri_attention_prefill_kept_bf16": [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                                       c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_float, c_void_p, c_int,
                                       c_void_p, c_void_p],
    "ri_attention_kept": [c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int,
                          c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_float, c_void_p, c_int, c_void_p,
                          c_void_p],
    "ri_qk_pairs_norm_kv_write": [c_void_p, c_int, ctypes.c_long, c_int, c_int, c_int, c_void_p, c_int, c_void_p, c_void_p,
                                  c_int, c_float, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_int, c_void_p,
                                  c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "ri_decay_step": [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_float, c_void_p, c_void_p, c_int, c_int,
                      c_int, c_int, c_void_p],
    "ri_decay_scan": [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_float, c_void_p, c_void_p,
                      c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "ri_decay_scan_chunked": [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_float, c_void_p, c_void_p,
                              c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, ctypes.c_long, c_void_p],
    "ri_embed_scaled": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_float, c_int, c_int, c_void_p],
    "ri_branch_norm_add": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_void_p, c_void_p, c_float, c_int, c_void_p,
                           c_int, c_int, c_void_p],
    "ri_gate_rows": [c_void_p, c_int, c_int, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_float, c_int, c_int, c_int,
                     c_void_p],
    "ri_row_norm_gate": [c_void_p, c_int, c_int, c_void_p, c_void_p, c_float, c_void_p, c_int, c_int, c_int, c_float, c_int,
                         c_int, c_int, c_void_p],
    "ri_experts_route_general": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int,
                                 c_int, c_int, c_int, c_int, c_int, c_void_p],
    "ri_experts_activate_strided": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_float, c_void_p],
    "ri_experts_finish": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_int, c_void_p, c_int, c_int,
                          c_void_p],
    "ri_scaled_sum_norm": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_void_p, c_float, c_void_p, c_void_p, c_float,
                           c_int, c_int, c_int, c_void_p],
    "ri_glu_clamped_bias": [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_float, c_int, c_int, c_void_p],
    "ri_experts_activate_plain": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "ri_softcap_rows": [c_void_p, c_float, ctypes.c_long, c_void_p],
    "ri_latent_prepare": [c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_void_p,
                          c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "ri_latent_attention_mfma_fits": [c_int, c_int, c_int],
    "ri_latent_attention_mfma": [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                 c_int, c_int, c_int, c_float, c_void_p, c_void_p, c_int, c_int, c_void_p],
    "ri_head_products": [c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_int, c_void_p,
                         c_int, c_int, c_float, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "ri_whole_norm_kv_write": [c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_void_p,
                               c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "ri_talking_attention_shares": [c_int, c_int],
    "ri_talking_attention": [c_void_p, c_int, c_int, c_int, c_float, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p,
                             c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                             c_float, c_void_p, c_void_p, c_void_p, c_void_p],
    "ri_talking_attention_mfma_fits": [c_int, c_int, c_int, c_int],
    "ri_talking_attention_mfma": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                                  c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_void_p, c_void_p, c_void_p,
                                  c_void_p],
    "ri_shift_mix": [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p],
    "ri_shift_keep": [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p],
    "ri_timemix_max_dim": [],
    "ri_tanh_rows": [c_void_p, c_int, c_void_p, ctypes.c_long, c_void_p],
    "ri_timemix_scan": [c_void_p, c_int, c_int, c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                        c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p],
    "ri_timemix_scan_cols_fits": [c_int],
    "ri_timemix_scan_cols": [c_void_p, c_int, c_int, c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                             c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                             c_void_p],
    "ri_causal_conv_silu": [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                            c_void_p, c_int, c_int, c_int, c_int, c_void_p],
    "ri_ssd_scan": [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p,
                    c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "ri_ssd_scan_cols_fits": [c_int, c_int],
    "ri_ssd_scan_cols": [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p,
                         c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "ri_group_rms_norm": [c_void_p, c_int, c_void_p, c_void_p, c_float, c_int, c_int, c_int, c_void_p],
}

_fn = {}


def _get(name: str):
    f = _fn.get(name)
    if f is None:
        lib = load()
        try:
            f = getattr(lib, name)
        except AttributeError:
            raise KernelError(f"the kernel library has no {name}: it is older than this package, build it again") from None
        f.argtypes = _SIGNATURES[name]
        f.restype = c_int
        _fn[name] = f
    return f


def _call(name: str, *args) -> None:
    rc = _get(name)(*args)
    if rc != 0:
        raise KernelError(load().ri_last_error().decode())


def _stream() -> int:
    """The current device's current stream, as the raw handle the kernels are launched on (torch's
    ``current_stream()`` builds a Python object through several layers for the same number: 5 us a call)."""
    return torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice())


def code(dtype: torch.dtype) -> int:
    try:
        return _CODES[dtype]
    except KeyError:
        raise ShapeError(f"dtype {dtype} is not float32 or bfloat16") from None


def _dev(t: torch.Tensor, name: str, dtype=None, shape=None) -> int:
    """Checks a tensor and returns its device address."""
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise KernelError(f"{name}: the kernels run on the GPU only, got "
                          f"{t.device if isinstance(t, torch.Tensor) else type(t).__name__}")
    if not t.is_contiguous():
        raise ShapeError(f"{name} must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise ShapeError(f"{name} must be {dtype}, got {t.dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise ShapeError(f"{name} must have shape {list(shape)}, got {list(t.shape)}")
    return t.data_ptr()


def _opt(t, name: str, dtype=None, shape=None):
    return None if t is None else _dev(t, name, dtype, shape)


# ---------------------------------------------------------------- row-wise
GATE_SIGMOID, GATE_SILU = 0, 1


def embed_scaled(table: torch.Tensor, ids: torch.Tensor, scale: float, act_dtype=None):
    """float32 ``E[ids] * scale`` and, with ``act_dtype``, the same rows in that format (else None)."""
    tokens, dim = ids.shape[0], table.shape[1]
    out = torch.empty((tokens, dim), dtype=torch.float32, device=table.device)
    act = torch.empty((tokens, dim), dtype=act_dtype, device=table.device) if act_dtype is not None else None
    _call("ri_embed_scaled", _dev(out, "out"), _opt(act, "act"), code(act_dtype or torch.float32), _dev(table, "table"),
          code(table.dtype), _dev(ids, "ids", torch.int32, (tokens,)), float(scale), tokens, dim, _stream())
    return out, act


def branch_norm_add(residual: torch.Tensor, y: torch.Tensor, gain, bias, eps: float, norm_kind: int, layer_scale,
                    act_dtype=None):
    """``residual += layer_scale * norm(y)`` in place (float32), the norm a layer norm (``NORM_LAYER``, with ``bias``) or an
    RMS norm (``NORM_RMS``) over ``y``'s rows with ``gain``; ``y`` is ``[T, dim]`` or float32 ``[parts, T, dim]`` (added in
    order).  With ``act_dtype`` the new residual is also returned in that format."""
    rows, dim = residual.shape
    parts = y.shape[0] if y.dim() == 3 else 1
    if tuple(y.shape[-2:]) != (rows, dim):
        raise ShapeError(f"a branch output of {list(y.shape)} for a residual of {list(residual.shape)}")
    act = torch.empty((rows, dim), dtype=act_dtype, device=residual.device) if act_dtype is not None else None
    _call("ri_branch_norm_add", _dev(residual, "residual", torch.float32), _opt(act, "act"), code(act_dtype or torch.float32),
          _dev(y, "y"), code(y.dtype), parts, _dev(gain, "gain", torch.float32, (dim,)),
          _opt(bias, "bias", torch.float32, (dim,)), float(eps), int(norm_kind),
          _opt(layer_scale, "layer_scale", torch.float32, (dim,)), rows, dim, _stream())
    return act


def gate_rows(out: torch.Tensor, out_off: int, x: torch.Tensor, proj: torch.Tensor, g_off: int, scale: float,
              kind: int = GATE_SIGMOID) -> None:
    """``out[:, out_off : out_off + w] = scale * x * gate(proj[:, g_off : g_off + w])`` for ``x [T, w]``; the gate is a
    sigmoid or silu; ``out`` and ``proj`` share a format.  ``proj`` None: no gate, the scaled copy alone."""
    rows, width = x.shape
    if out.shape[0] != rows or (proj is not None and (out.dtype != proj.dtype or proj.shape[0] != rows)):
        raise ShapeError(f"gate_rows: out {list(out.shape)} {out.dtype}, x {list(x.shape)}, gates "
                         f"{None if proj is None else list(proj.shape)}")
    _call("ri_gate_rows", _dev(out, "out"), out.shape[1], int(out_off), _dev(x, "x"), code(x.dtype), _opt(proj, "proj"),
          proj.shape[1] if proj is not None else 0, int(g_off), code(out.dtype), float(scale), int(kind), rows, width, _stream())


def row_norm_gate(out: torch.Tensor, out_off: int, x: torch.Tensor, gain, eps: float, proj, g_off: int, scale: float,
                  kind: int = GATE_SIGMOID) -> None:
    """``out[:, out_off : out_off + w] = scale * x / sqrt(mean(x^2) + eps) * gain * gate(proj[:, g_off : g_off + w])``, the
    mean over the whole row of ``x [T, w]`` float32; ``gain`` and ``proj`` may be None."""
    rows, width = x.shape
    if out.shape[0] != rows or (proj is not None and (proj.dtype != out.dtype or proj.shape[0] != rows)):
        raise ShapeError(f"row_norm_gate: out {list(out.shape)}, x {list(x.shape)}")
    _call("ri_row_norm_gate", _dev(out, "out"), out.shape[1], int(out_off), _dev(x, "x", torch.float32),
          _opt(gain, "gain", torch.float32, (width,)), float(eps), _opt(proj, "proj"),
          proj.shape[1] if proj is not None else 0, int(g_off), code(out.dtype), float(scale), int(kind), rows, width, _stream())


def embed_gather(table: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
    """float32 rows ``table[ids]``; ids int32 ``[T]``, already checked to be inside the table."""
    tokens, dim = ids.shape[0], table.shape[1]
    out = torch.empty((tokens, dim), dtype=torch.float32, device=table.device)
    _call("ri_embed_gather", _dev(out, "out"), _dev(table, "table"), code(table.dtype),
          _dev(ids, "ids", torch.int32, (tokens,)), tokens, dim, _stream())
    return out


def add_rmsnorm(residual: torch.Tensor, pending, gain: torch.Tensor, eps: float, out_dtype,
                rows: torch.Tensor | None = None, tiled: bool = False):
    """``residual += pending`` (in place, when ``rows`` is None) and the RMSNorm of the sum.
    With ``rows`` the sum and norm are taken of those rows only and nothing is written back.
    ``pending`` may be ``[parts, T, dim]``: the parts of a product split along K, added in order.
    With ``tiled`` the normed rows (bfloat16, at most 64) come as ``TiledRows``."""
    t, dim = residual.shape
    n = t if rows is None else rows.shape[0]
    parts = 1
    if pending is not None and pending.dim() == 3:
        parts = pending.shape[0]
        if tuple(pending.shape[1:]) != (t, dim):
            raise ShapeError(f"pending parts are {list(pending.shape)}, the stream is {[t, dim]}")
    elif pending is not None and tuple(pending.shape) != (t, dim):
        raise ShapeError(f"pending is {list(pending.shape)}, the stream is {[t, dim]}")
    out = TiledRows.empty(n, dim, residual.device) if tiled else torch.empty((n, dim), dtype=out_dtype,
                                                                             device=residual.device)
    _call("ri_add_rmsnorm", _dev(out.data if tiled else out, "out"), code(out_dtype),
          _dev(residual, "residual", torch.float32),
          _opt(pending, "pending"), code(pending.dtype) if pending is not None else F32, parts, t,
          _dev(gain, "gain", torch.float32, (dim,)), float(eps), _opt(rows, "rows", torch.int32), n, dim, int(tiled),
          _stream())
    return out


def add_rows(residual: torch.Tensor, pending, rows: torch.Tensor | None = None, in_place: bool = False) -> torch.Tensor:
    """float32 ``residual[rows] + pending[rows]`` without a norm; with ``in_place`` (all rows) the sum is
    written into ``residual`` itself."""
    t, dim = residual.shape
    n = t if rows is None else rows.shape[0]
    if in_place and rows is not None:
        raise ShapeError("an add in place takes all rows")
    out = residual if in_place else torch.empty((n, dim), dtype=torch.float32, device=residual.device)
    _call("ri_add_rows", _dev(out, "out"), _dev(residual, "residual", torch.float32),
          _opt(pending, "pending", None, (t, dim)), code(pending.dtype) if pending is not None else F32,
          _opt(rows, "rows", torch.int32), n, dim, _stream())
    return out


def add_bias(x: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """``x[t, :] += bias`` in place (float32 bias, the sum in float32); returns ``x``."""
    rows, dim = x.shape
    _call("ri_add_bias", _dev(x, "x"), code(x.dtype), _dev(bias, "bias", torch.float32, (dim,)), rows, dim, _stream())
    return x


def swiglu(y: torch.Tensor, tiled_out: bool = False):
    """``silu(y[:, :I]) * y[:, I:]`` for ``y: [T, 2 I]``; ``tiled_out``: the bfloat16 result as ``TiledRows``
    (at most 64 rows, ``I`` a multiple of 8)."""
    tokens, two_i = y.shape
    if two_i % 2:
        raise ShapeError(f"swiglu input has an odd width {two_i}")
    inter = two_i // 2
    tiled_out = tiled_out and y.dtype == torch.bfloat16 and tokens <= 64 and inter % 8 == 0
    out = TiledRows.empty(tokens, inter, y.device) if tiled_out else torch.empty((tokens, inter), dtype=y.dtype,
                                                                                   device=y.device)
    _call("ri_swiglu", _dev(out.data if tiled_out else out, "out"), _dev(y, "y"), code(y.dtype), tokens, inter,
          int(tiled_out), _stream())
    return out


def argmax(logits: torch.Tensor) -> torch.Tensor:
    """int32 index of the first maximum of every row of float32 ``logits``."""
    rows, vocab = logits.shape
    ids = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    ws = torch.empty((rows * 64 * 2,), dtype=torch.int32, device=logits.device)      # 64 (value, index) pairs a row
    _call("ri_argmax", _dev(ids, "ids"), _dev(logits, "logits", torch.float32), _dev(ws, "workspace"), rows, vocab,
          _stream())
    return ids


# From this vocabulary size on a sampled row is cut over many workgroups (at 151,936 entries: 8 short
# launches instead of one long one).
SPLIT_SAMPLER_MIN_VOCAB = 16384


def sample(logits: torch.Tensor, uniform, temperature: float, top_k: int = 0, top_p: float = 1.0,
           penalty: float = 1.0, seen: torch.Tensor | None = None, seen_rows: torch.Tensor | None = None,
           split: bool | None = None) -> torch.Tensor:
    """int32 token per row of float32 ``logits``: repetition penalty over the ids marked in ``seen``
    (uint8 ``[*, vocab]``), greedy when the temperature is not positive, else temperature, top-k, top-p
    and one draw with ``uniform[r]`` in [0, 1).  ``split``: the many-workgroups form (the same token;
    by default for large vocabularies)."""
    rows, vocab = logits.shape
    out = torch.empty((rows,), dtype=torch.int32, device=logits.device)
    if split is None:
        split = vocab >= SPLIT_SAMPLER_MIN_VOCAB
    if split and temperature > 0:
        lib = load()
        lib.ri_sample_split_workspace_bytes.restype = ctypes.c_long
        lib.ri_sample_split_workspace_bytes.argtypes = [c_int]
        ws = torch.empty((lib.ri_sample_split_workspace_bytes(rows),), dtype=torch.uint8, device=logits.device)
        _call("ri_sample_split", _dev(out, "out"), _dev(logits, "logits", torch.float32),
              _opt(seen, "seen", torch.uint8), _opt(seen_rows, "seen_rows", torch.int32, (rows,)),
              _dev(uniform, "uniform", torch.float32, (rows,)), _dev(ws, "workspace"), rows, vocab, float(temperature),
              int(top_k), float(top_p), float(penalty), _stream())
        return out
    _call("ri_sample", _dev(out, "out"), _dev(logits, "logits", torch.float32),
          _opt(seen, "seen", torch.uint8), _opt(seen_rows, "seen_rows", torch.int32, (rows,)),
          _opt(uniform, "uniform", torch.float32, (rows,)), rows, vocab, float(temperature), int(top_k), float(top_p),
          float(penalty), _stream())
    return out


def mark_seen(seen: torch.Tensor, rows: torch.Tensor, tokens: torch.Tensor) -> None:
    """``seen[rows[i], tokens[i]] = 1``."""
    n = rows.shape[0]
    _call("ri_mark_seen", _dev(seen, "seen", torch.uint8), _dev(rows, "rows", torch.int32, (n,)),
          _dev(tokens, "tokens", torch.int32, (n,)), n, seen.shape[1], _stream())


# ---------------------------------------------------------------- attention
def qk_norm_rope_kv_write(qkv, q_gain, k_gain, eps, inv_freq, tok_pos, tok_seq, page_table, k_pages, v_pages,
                          heads: int, kv_heads: int, head_dim: int, cu_seqlens=None, max_new: int = 0) -> None:
    """In place on ``qkv: [T, (H + 2 Hkv) dh]``: per-head norm and rotation of q and k; k and v go to their
    pages.  ``inv_freq`` (float32 ``[r]``, ``r <= dh / 2``) rotates the first ``2 r`` elements of every head in
    pairs ``(i, i + r)``; what lies behind them is normed only.  With ``cu_seqlens`` (int32 ``[seqs + 1]``) and
    ``max_new`` values are written a page at a time."""
    tokens = qkv.shape[0]
    width = (heads + 2 * kv_heads) * head_dim
    if k_pages is None:                       # nothing goes to the cache: k is changed in place like q
        if v_pages is not None:
            raise ShapeError("key pages and value pages come together or not at all")
        num_pages, page_size = 0, 0
    else:
        num_pages, hkv, page_size, dh = k_pages.shape
        if (hkv, dh) != (kv_heads, head_dim) or tuple(v_pages.shape) != (num_pages, hkv, dh, page_size):
            raise ShapeError(f"pages are {list(k_pages.shape)} / {list(v_pages.shape)}, the mixer has {kv_heads} kv "
                             f"heads of {head_dim}")
    rot_dim = head_dim if inv_freq is None else 2 * inv_freq.shape[0]
    if inv_freq is not None and (inv_freq.dim() != 1 or not 2 <= rot_dim <= head_dim):
        raise ShapeError(f"inv_freq is {list(inv_freq.shape)}: a head of {head_dim} takes 1 to {head_dim // 2} frequencies")
    _call("ri_qk_norm_rope_kv_write", _dev(qkv, "qkv", None, (tokens, width)), code(qkv.dtype),
          _opt(q_gain, "q_gain", torch.float32, (head_dim,)), _opt(k_gain, "k_gain", torch.float32, (head_dim,)),
          float(eps), _opt(inv_freq, "inv_freq", torch.float32), rot_dim,
          _dev(tok_pos, "tok_pos", torch.int32, (tokens,)), _dev(tok_seq, "tok_seq", torch.int32, (tokens,)),
          _opt(cu_seqlens, "cu_seqlens", torch.int32), 0 if cu_seqlens is None else cu_seqlens.shape[0] - 1,
          int(max_new), _dev(page_table, "page_table", torch.int32), page_table.shape[1],
          _opt(k_pages, "k_pages"), _opt(v_pages, "v_pages"), code(qkv.dtype if k_pages is None else k_pages.dtype),
          tokens, heads, kv_heads, head_dim, page_size, num_pages, _stream())


def attention(qkv, k_pages, v_pages, tok_pos, tok_seq, page_table, heads: int, kv_heads: int, head_dim: int,
              window: int | None, scale: float, softcap: float | None = None, slopes: torch.Tensor | None = None,
              keep_first: int = 0, sinks: torch.Tensor | None = None, q_off: int = 0) -> torch.Tensor:
    """Attention of every new token over its sequence's pages; q is the first ``H dh`` columns of ``qkv``.
    With a window, ``keep_first`` first tokens of the sequence stay visible behind it; ``sinks`` (float32 ``[heads]``)
    adds ``exp(sinks[h])`` to the denominator of head ``h``'s softmax.  ``q_off``: the queries' first column in ``qkv``'s rows
    where it is not 0.
    The size of a value head is read from ``v_pages [pages, kv_heads, v_dim, page]``; with ``softcap`` a score
    ``s`` becomes ``softcap * tanh(s / softcap)`` before the softmax; with ``slopes`` (float32 ``[heads]``) the score of
    head ``h`` at position ``p`` for the key at ``j`` then loses ``slopes[h] * (p - j)``."""
    tokens, stride = qkv.shape
    if q_off < 0 or q_off + heads * head_dim > stride:
        raise ShapeError(f"attention: queries at column {q_off} of rows of {stride} for {heads} heads of {head_dim}")
    v_dim = v_pages.shape[2]
    if tuple(k_pages.shape[:2]) != tuple(v_pages.shape[:2]) or k_pages.shape[2] != v_pages.shape[3] or k_pages.shape[3] != head_dim:
        raise ShapeError(f"attention: key pages {list(k_pages.shape)} and value pages {list(v_pages.shape)} for heads of {head_dim}")
    out = torch.empty((tokens, heads * v_dim), dtype=qkv.dtype, device=qkv.device)
    _call("ri_attention_kept", _dev(out, "out"), _dev(qkv, "qkv") + int(q_off) * qkv.element_size(), code(qkv.dtype), stride, _dev(k_pages, "k_pages"),
          _dev(v_pages, "v_pages"), code(k_pages.dtype), _dev(tok_pos, "tok_pos", torch.int32, (tokens,)),
          _dev(tok_seq, "tok_seq", torch.int32, (tokens,)), _dev(page_table, "page_table", torch.int32),
          page_table.shape[1], tokens, heads, kv_heads, head_dim, v_dim, k_pages.shape[2], int(window or 0),
          float(scale), float(softcap or 0.0), _opt(slopes, "slopes", torch.float32, (heads,)), int(keep_first or 0),
          _opt(sinks, "sinks", torch.float32, (heads,)), _stream())
    return out


def qk_pairs_norm_kv_write(proj, q_off: int, k_off: int, v_off: int, inv_freq, q_gain, k_gain, norm: bool, eps: float,
                           tok_pos, tok_seq, page_table, k_pages, v_pages, heads: int, kv_heads: int, dim: int, vdim: int,
                           cu_seqlens=None, max_new: int = 0) -> None:
    """In place on the projection rows ``proj [T, row]`` (q heads at column ``q_off``, k heads at ``k_off``, v heads at
    ``v_off``): the neighbours ``(2i, 2i + 1)`` of the first ``2 len(inv_freq)`` elements of every q and k head turn by
    ``pos * inv_freq[i]``, then, with ``norm``, every head is divided by its root mean square (and multiplied by the
    gains, where given); q stays in ``proj``, k and v go to their pages."""
    tokens, row = proj.shape
    pages, _, page_size, _ = k_pages.shape
    seqs = cu_seqlens.shape[0] - 1 if cu_seqlens is not None else 0
    rot = 0 if inv_freq is None else 2 * inv_freq.shape[0]
    _call("ri_qk_pairs_norm_kv_write", _dev(proj, "proj"), code(proj.dtype), row, int(q_off), int(k_off), int(v_off),
          _opt(inv_freq, "inv_freq", torch.float32), rot, _opt(q_gain, "q_gain", torch.float32, (dim,)),
          _opt(k_gain, "k_gain", torch.float32, (dim,)), int(bool(norm)), float(eps),
          _dev(tok_pos, "tok_pos", torch.int32, (tokens,)), _dev(tok_seq, "tok_seq", torch.int32, (tokens,)),
          _opt(cu_seqlens, "cu_seqlens", torch.int32), seqs, int(max_new),
          _dev(page_table, "page_table", torch.int32), page_table.shape[1],
          _dev(k_pages, "k_pages", proj.dtype, (pages, kv_heads, page_size, dim)),
          _dev(v_pages, "v_pages", proj.dtype, (pages, kv_heads, vdim, page_size)), code(k_pages.dtype),
          tokens, heads, kv_heads, dim, vdim, page_size, _stream())


def qk_norm_temper_kv_write(qkv, q_gain, k_gain, eps: float, temper, tok_pos, tok_seq, page_table, k_pages, v_pages,
                            heads: int, kv_heads: int, dim: int, vdim: int, cu_seqlens=None, max_new: int = 0) -> None:
    """Per-head RMS norm of q and k (gains may be None), the query temperature ``temper = (coef, every)`` or None
    (``q *= 1 + coef * ln(floor((pos + 1) / every) + 1)``, q in place), k and v into their pages.
    ``qkv: [T, heads * dim + kv_heads * dim + kv_heads * vdim]``.  With ``cu_seqlens`` (``[seqs + 1]``) and
    ``max_new`` (the most new tokens of any sequence) a prompt's values go into their pages a page at a time."""
    tokens, stride = qkv.shape
    seqs = cu_seqlens.shape[0] - 1 if cu_seqlens is not None else 0
    if stride != (heads + kv_heads) * dim + kv_heads * vdim:
        raise ShapeError(f"qkv rows of {stride} for {heads} + {kv_heads} heads of {dim} and {kv_heads} of {vdim}")
    pages, _, page_size, _ = k_pages.shape
    coef, every = (float(temper[0]), int(temper[1])) if temper else (0.0, 1)
    _call("ri_qk_norm_temper_kv_write", _dev(qkv, "qkv"), code(qkv.dtype), _opt(q_gain, "q_gain", torch.float32, (dim,)),
          _opt(k_gain, "k_gain", torch.float32, (dim,)), float(eps), coef, every,
          _dev(tok_pos, "tok_pos", torch.int32, (tokens,)), _dev(tok_seq, "tok_seq", torch.int32, (tokens,)),
          _opt(cu_seqlens, "cu_seqlens", torch.int32), seqs, int(max_new),
          _dev(page_table, "page_table", torch.int32), page_table.shape[1],
          _dev(k_pages, "k_pages", None, (pages, kv_heads, page_size, dim)),
          _dev(v_pages, "v_pages", k_pages.dtype, (pages, kv_heads, vdim, page_size)), code(k_pages.dtype),
          tokens, heads, kv_heads, dim, vdim, page_size, _stream())


NORM_NONE, NORM_RMS, NORM_LAYER = 0, 1, 2
MAX_STREAMS = 16


def streams_read_norm(streams, pending, mix, out_coef, in_coef, gain, bias, eps: float, norm_kind: int, out_dtype,
                      rows: torch.Tensor | None = None, fresh: torch.Tensor | None = None) -> torch.Tensor:
    """The write that waits for the residual streams, the read and the norm, in one kernel.
    ``streams: [T, S, dim]`` float32.  With ``pending`` (``[T, dim]`` or ``[parts, T, dim]``):
    ``x_t <- sum_s mix[s, t] x_s + out_coef[t] * pending``; then ``u = sum_t in_coef[t] x_t`` and the norm of ``u``
    (``NORM_NONE``, ``NORM_RMS`` or ``NORM_LAYER`` with ``gain`` and optional ``bias``).  Coefficients that are
    None are the identity and ones.  With ``rows`` only those rows are read and nothing is stored.  ``fresh``
    (``[T, dim]``): the one row all streams start from, spread into ``streams`` by this call."""
    t, n, dim = streams.shape
    count = t if rows is None else rows.shape[0]
    parts = 1
    if pending is not None:
        if pending.dim() == 3:
            parts = pending.shape[0]
        if tuple(pending.shape[-2:]) != (t, dim):
            raise ShapeError(f"pending is {list(pending.shape)}, the streams are {list(streams.shape)}")
    out = torch.empty((count, dim), dtype=out_dtype, device=streams.device)
    if count == 0:
        return out
    _call("ri_streams_read_norm", _dev(out, "out"), code(out_dtype), _dev(streams, "streams", torch.float32),
          _opt(fresh, "fresh", torch.float32, (t, dim)), n,
          _opt(pending, "pending"), code(pending.dtype) if pending is not None else F32, parts, t,
          _opt(mix, "mix", torch.float32, (n, n)), _opt(out_coef, "out_coef", torch.float32, (n,)),
          _opt(in_coef, "in_coef", torch.float32, (n,)), _opt(gain, "gain", torch.float32, (dim,)),
          _opt(bias, "bias", torch.float32, (dim,)), float(eps), int(norm_kind),
          _opt(rows, "rows", torch.int32), count, dim, _stream())
    return out


def embed_positions_norm(table, positions, ids, tok_pos, gain, bias, eps: float, norm_kind: int) -> torch.Tensor:
    """float32 rows ``norm(table[ids] + positions[tok_pos])`` (``positions`` may be None)."""
    tokens, dim = ids.shape[0], table.shape[1]
    out = torch.empty((tokens, dim), dtype=torch.float32, device=table.device)
    if positions is not None and (positions.dtype != table.dtype or positions.shape[1] != dim):
        raise ShapeError("the table of positions must have the token table's dtype and width")
    _call("ri_embed_positions_norm", _dev(out, "out"), _dev(table, "table"), _opt(positions, "positions"),
          code(table.dtype), _dev(ids, "ids", torch.int32, (tokens,)), _dev(tok_pos, "tok_pos", torch.int32, (tokens,)),
          _opt(gain, "gain", torch.float32, (dim,)), _opt(bias, "bias", torch.float32, (dim,)), float(eps),
          int(norm_kind), tokens, dim, _stream())
    return out


GLA_MAX_DIM = 512


def gla_scan(proj, q_off: int, k_off: int, v_off: int, z, z_bias, tau: float, q_scale: float, state, cu_seqlens,
             slots, heads: int, dim: int, vdim: int) -> torch.Tensor:
    """The gated linear recurrence over every sequence's new tokens; float32 ``[T, heads * vdim]``.
    ``proj: [T, row]`` holds q, k (``heads * dim``) and v (``heads * vdim``) at the given columns; ``z``
    (float32 ``[T, heads * dim]``) and ``z_bias`` give the decay ``exp(log_sigmoid(z + bias) / tau)``;
    ``state: [slots, heads, dim, vdim]`` float32 is read and written at the sequences' slots.  In a step with more
    tokens than sequences ``z`` is overwritten (by the decays, made for all tokens at once before the walk)."""
    tokens, row = proj.shape
    seqs = slots.shape[0]
    if state.dim() != 4 or tuple(state.shape[1:]) != (heads, dim, vdim):
        raise ShapeError(f"the state is {list(state.shape)}, not [slots, {heads}, {dim}, {vdim}]")
    out = torch.empty((tokens, heads * vdim), dtype=torch.float32, device=proj.device)
    _call("ri_gla_scan", _dev(out, "out"), _dev(proj, "proj"), code(proj.dtype), row, q_off, k_off, v_off,
          _dev(z, "z", torch.float32, (tokens, heads * dim)), _opt(z_bias, "z_bias", torch.float32, (heads * dim,)),
          float(tau), float(q_scale), _dev(state, "state", torch.float32),
          _dev(cu_seqlens, "cu_seqlens", torch.int32, (seqs + 1,)), _dev(slots, "slots", torch.int32, (seqs,)),
          seqs, tokens, heads, dim, vdim, _stream())
    return out


def decay_scan(proj, q_off: int, k_off: int, v_off: int, head_decay, q_scale: float, state, cu_seqlens, slots,
               heads: int, dim: int, vdim: int) -> torch.Tensor:
    """Linear attention with one fixed decay per head over the new tokens of every sequence, from the state its slot
    holds: ``S <- decay_h S + k v^T``, ``o = S^T q`` with ``q = silu(.) * q_scale``, ``k = silu(.)``, ``v = silu(.)`` of the
    projection's columns at ``q_off``, ``k_off``, ``v_off``; ``head_decay`` float32 ``[heads]``; ``state`` float32
    ``[slots, heads, dim, vdim]``, updated in place.  Returns float32 ``[T, heads * vdim]``."""
    tokens, row = proj.shape
    seqs = slots.shape[0]
    out = torch.empty((tokens, heads * vdim), dtype=torch.float32, device=proj.device)
    _call("ri_decay_scan", _dev(out, "out"), _dev(proj, "proj"), code(proj.dtype), row, int(q_off), int(k_off), int(v_off),
          _dev(head_decay, "head_decay", torch.float32, (heads,)), float(q_scale),
          _dev(state, "state", torch.float32, (state.shape[0], heads, dim, vdim)),
          _dev(cu_seqlens, "cu_seqlens", torch.int32, (seqs + 1,)), _dev(slots, "slots", torch.int32, (seqs,)),
          seqs, tokens, heads, dim, vdim, _stream())
    return out


DECAY_CHUNKS_FROM = 128       # new tokens of a step's longest sequence from which the chunked form is the faster one
DECAY_CHUNKS_FORCED = None    # True or False: every step of two tokens and more, or none, goes in chunks (tests, measurements)


def decay_chunks_pay(seqs: int, tokens: int, max_new: int, heads: int, dim: int, vdim: int) -> bool:
    """Whether ``decay_scan_chunked`` is expected to take less time than ``decay_scan`` for this step (host arithmetic
    only).  Measured on 256 compute units with heads of 64 x 32 to 128 x 128, 1 to 32 sequences and 128 to 8,192
    tokens: the walk takes a token's latency (0.2 to 0.33 us) times the longest sequence, the chunks a workgroup's time
    (25 to 45 us in all three launches) for as many (chunk, head) pairs as the machine holds at once; they are even at
    128 tokens and the chunks ahead from there on, for one prompt (2,048 tokens: 67 against 672 us) and for batches of
    prompts (32 of 1,024: 0.74 against 1.32 ms)."""
    if DECAY_CHUNKS_FORCED is not None:
        return bool(DECAY_CHUNKS_FORCED) and max_new >= 2
    return max_new >= DECAY_CHUNKS_FROM


def decay_chunks_fit(dim: int, vdim: int, row: int, offsets: tuple) -> bool:
    """Whether ``decay_scan_chunked`` takes these head sizes and this place in the projection's rows (host code only)."""
    return bool(_get("ri_decay_chunks_fit")(int(dim), int(vdim))) and row % 4 == 0 and all(o % 4 == 0 for o in offsets)


def decay_scan_chunked(proj, q_off: int, k_off: int, v_off: int, head_decay, q_scale: float, state, cu_seqlens, slots,
                       heads: int, dim: int, vdim: int, max_new: int) -> torch.Tensor:
    """``decay_scan`` for prompts, in chunks of 64 tokens: with a constant decay a chunk's tokens do not wait for one
    another (``o_i = sum_{j <= i} d^(i - j) (q_i . k_j) v_j + d^(i + 1) S0^T q_i``), so every chunk's own sum, the walk
    from chunk to chunk and every chunk's outputs are three launches whatever the number of tokens.  float32
    throughout; differs from ``decay_scan`` by rounding alone.  ``max_new``: the most new tokens of a sequence."""
    tokens, row = proj.shape
    seqs = slots.shape[0]
    out = torch.empty((tokens, heads * vdim), dtype=torch.float32, device=proj.device)
    need = (tokens // 64 + seqs) * heads * dim * vdim
    work = torch.empty((need,), dtype=torch.float32, device=proj.device)
    _call("ri_decay_scan_chunked", _dev(out, "out"), _dev(proj, "proj"), code(proj.dtype), row, int(q_off), int(k_off),
          int(v_off), _dev(head_decay, "head_decay", torch.float32, (heads,)), float(q_scale),
          _dev(state, "state", torch.float32, (state.shape[0], heads, dim, vdim)),
          _dev(cu_seqlens, "cu_seqlens", torch.int32, (seqs + 1,)), _dev(slots, "slots", torch.int32, (seqs,)),
          seqs, tokens, int(max_new), heads, dim, vdim, _dev(work, "workspace"), need, _stream())
    return out


def decay_step(proj, q_off: int, k_off: int, v_off: int, head_decay, q_scale: float, state, slots, heads: int, dim: int,
               vdim: int) -> torch.Tensor:
    """``decay_scan`` for one new token a sequence (row ``b`` of ``proj`` belongs to ``slots[b]``), where ``gla_step_fits``
    says the head sizes are taken: the state's trip from memory and back in 16-byte pieces.  float32 ``[seqs, heads * vdim]``."""
    seqs, row = proj.shape
    out = torch.empty((seqs, heads * vdim), dtype=torch.float32, device=proj.device)
    _call("ri_decay_step", _dev(out, "out"), _dev(proj, "proj"), code(proj.dtype), row, int(q_off), int(k_off), int(v_off),
          _dev(head_decay, "head_decay", torch.float32, (heads,)), float(q_scale),
          _dev(state, "state", torch.float32, (state.shape[0], heads, dim, vdim)), _dev(slots, "slots", torch.int32, (seqs,)),
          seqs, heads, dim, vdim, _stream())
    return out


def gla_step_fits(dim: int, vdim: int) -> bool:
    """Whether ``gla_step`` takes these head sizes (host code only: it needs no GPU)."""
    return bool(_get("ri_gla_step_fits")(int(dim), int(vdim)))


def gla_step(proj, q_off: int, k_off: int, v_off: int, g_off: int, z, z_bias, tau: float, q_scale: float, state, slots,
             gain, eps: float, heads: int, dim: int, vdim: int) -> torch.Tensor:
    """One new token a sequence (row ``b`` of ``proj`` and ``z`` belongs to ``slots[b]``): the recurrence's step on
    the state, the per-head RMS norm and the gate ``silu(g)`` in one kernel; ``[seqs, heads * vdim]`` in the dtype
    of ``proj``."""
    seqs, row = proj.shape
    if state.dim() != 4 or tuple(state.shape[1:]) != (heads, dim, vdim):
        raise ShapeError(f"the state is {list(state.shape)}, not [slots, {heads}, {dim}, {vdim}]")
    out = torch.empty((seqs, heads * vdim), dtype=proj.dtype, device=proj.device)
    _call("ri_gla_step", _dev(out, "out"), _dev(proj, "proj"), code(proj.dtype), row, q_off, k_off, v_off, g_off,
          _dev(z, "z", torch.float32, (seqs, heads * dim)), _opt(z_bias, "z_bias", torch.float32, (heads * dim,)),
          float(tau), float(q_scale), _dev(state, "state", torch.float32), _dev(slots, "slots", torch.int32, (seqs,)),
          _dev(gain, "gain", torch.float32, (vdim,)), float(eps), seqs, heads, dim, vdim, _stream())
    return out


def gla_norm_gate(o, proj, g_off: int, gain, eps: float, heads: int, vdim: int) -> torch.Tensor:
    """``rms_norm(o[t, h]) * gain * silu(gate[t, h])`` in the dtype of ``proj``, whose rows hold the gate at column
    ``g_off``; ``o``: float32 ``[T, heads * vdim]``."""
    tokens, row = proj.shape
    out = torch.empty((tokens, heads * vdim), dtype=proj.dtype, device=proj.device)
    _call("ri_gla_norm_gate", _dev(out, "out"), _dev(o, "o", torch.float32, (tokens, heads * vdim)), _dev(proj, "proj"),
          code(proj.dtype), row, g_off, _dev(gain, "gain", torch.float32, (vdim,)), float(eps), tokens, heads, vdim,
          _stream())
    return out


def relu_squared(y: torch.Tensor) -> torch.Tensor:
    """``max(y, 0)^2`` elementwise."""
    out = torch.empty(y.shape, dtype=y.dtype, device=y.device)
    if y.numel():
        _call("ri_relu_squared", _dev(out, "out"), _dev(y, "y"), code(y.dtype), y.numel(), _stream())
    return out


def gelu_tanh(y: torch.Tensor) -> torch.Tensor:
    """``0.5 y (1 + tanh(sqrt(2 / pi) (y + 0.044715 y^3)))`` elementwise, taken in float32."""
    out = torch.empty(y.shape, dtype=y.dtype, device=y.device)
    if y.numel():
        _call("ri_gelu_tanh", _dev(out, "out"), _dev(y, "y"), code(y.dtype), y.numel(), _stream())
    return out


def gelu_erf(y: torch.Tensor) -> torch.Tensor:
    """``0.5 y (1 + erf(y / sqrt(2)))`` elementwise, taken in float32."""
    out = torch.empty(y.shape, dtype=y.dtype, device=y.device)
    if y.numel():
        _call("ri_gelu_erf", _dev(out, "out"), _dev(y, "y"), code(y.dtype), y.numel(), _stream())
    return out


ACTIVATIONS = {"relu2": relu_squared, "gelu_tanh": gelu_tanh, "gelu_erf": gelu_erf}      # what a dense feed-forward may name

DELTA_MAX_DIM = 256
DELTA_MAX_TAPS = 16


def delta_prepare(proj, q_off: int, taps, tails, ab, a_log, dt_bias, tok_seq, cu_seqlens, slots, heads: int,
                  kv_heads: int, dim: int, vdim: int):
    """What the gated delta rule's walk reads, for all tokens of a step: float32 ``qkv [T, channels]`` (q and k of
    ``kv_heads`` heads of ``dim``, v of ``heads`` heads of ``vdim``: the projections at column ``q_off`` of ``proj``
    through their short convolutions (``taps [channels, K]``, the inputs before the step from ``tails [slots, K - 1,
    channels]``) and silu, q and k as unit vectors per head, q times ``dim^(-1/2)``) and ``gates [T, 2 heads]``
    (``g = exp(-exp(a_log) softplus(a + dt_bias))`` then ``beta = sigmoid(b)`` from ``ab [T, 2 heads]``).  The tails
    are moved on by the step's tokens."""
    tokens, row = proj.shape
    seqs = slots.shape[0]
    channels = 2 * kv_heads * dim + heads * vdim
    ntaps = taps.shape[1]
    if tails.dim() != 3 or tuple(tails.shape[1:]) != (ntaps - 1, channels):
        raise ShapeError(f"the convolutions' tails are {list(tails.shape)}, not [slots, {ntaps - 1}, {channels}]")
    qkv = torch.empty((tokens, channels), dtype=torch.float32, device=proj.device)
    gates = torch.empty((tokens, 2 * heads), dtype=torch.float32, device=proj.device)
    _call("ri_delta_prepare", _dev(qkv, "qkv"), _dev(gates, "gates"), _dev(proj, "proj"), code(proj.dtype), row, q_off,
          _dev(taps, "taps", torch.float32, (channels, ntaps)), ntaps, _dev(tails, "tails", torch.float32),
          _dev(ab, "ab", torch.float32, (tokens, 2 * heads)), _dev(a_log, "a_log", torch.float32, (heads,)),
          _dev(dt_bias, "dt_bias", torch.float32, (heads,)), _dev(tok_seq, "tok_seq", torch.int32, (tokens,)),
          _dev(cu_seqlens, "cu_seqlens", torch.int32, (seqs + 1,)), _dev(slots, "slots", torch.int32, (seqs,)),
          seqs, tokens, heads, kv_heads, dim, vdim, _stream())
    return qkv, gates


def delta_scan(qkv, gates, state, cu_seqlens, slots, heads: int, kv_heads: int, dim: int, vdim: int,
               slices: int = 0) -> torch.Tensor:
    """The gated delta rule over every sequence's new tokens, ``S <- g S; u = beta (v - S^T k); S <- S + k u^T;
    o = S^T q``; float32 ``[T, heads * vdim]``.  ``state: [slots, heads, dim, vdim]`` float32 is read and written at
    the sequences' slots.  ``slices``: the lanes a column's rows are spread over, 4 or 8 (0: chosen by the size of the
    launch, which depends on the sequences and heads and not on their tokens)."""
    tokens = qkv.shape[0]
    seqs = slots.shape[0]
    channels = 2 * kv_heads * dim + heads * vdim
    if state.dim() != 4 or tuple(state.shape[1:]) != (heads, dim, vdim):
        raise ShapeError(f"the state is {list(state.shape)}, not [slots, {heads}, {dim}, {vdim}]")
    out = torch.empty((tokens, heads * vdim), dtype=torch.float32, device=qkv.device)
    _call("ri_delta_scan", _dev(out, "out"), _dev(qkv, "qkv", torch.float32, (tokens, channels)),
          _dev(gates, "gates", torch.float32, (tokens, 2 * heads)), _dev(state, "state", torch.float32),
          _dev(cu_seqlens, "cu_seqlens", torch.int32, (seqs + 1,)), _dev(slots, "slots", torch.int32, (seqs,)),
          seqs, tokens, heads, kv_heads, dim, vdim, int(slices), _stream())
    return out


def delta_step_fits(dim: int, vdim: int) -> bool:
    """Whether ``delta_step`` takes these head sizes (host code only: it needs no GPU)."""
    return bool(_get("ri_delta_step_fits")(int(dim), int(vdim)))


def delta_step(proj, q_off: int, g_off: int, taps, tails, ab, a_log, dt_bias, state, cu_seqlens, slots, gain, eps: float,
               heads: int, kv_heads: int, dim: int, vdim: int) -> torch.Tensor:
    """One new token a sequence (row ``b`` of ``proj`` and ``ab`` belongs to ``slots[b]``): what ``delta_prepare`` and
    ``delta_scan`` compute, the per-head RMS norm and the gate ``silu(g)`` (at column ``g_off`` of ``proj``) in one
    kernel, and the tails moved on; ``[seqs, heads * vdim]`` in the dtype of ``proj``."""
    seqs, row = proj.shape
    channels = 2 * kv_heads * dim + heads * vdim
    ntaps = taps.shape[1]
    if state.dim() != 4 or tuple(state.shape[1:]) != (heads, dim, vdim):
        raise ShapeError(f"the state is {list(state.shape)}, not [slots, {heads}, {dim}, {vdim}]")
    if tails.dim() != 3 or tuple(tails.shape[1:]) != (ntaps - 1, channels):
        raise ShapeError(f"the convolutions' tails are {list(tails.shape)}, not [slots, {ntaps - 1}, {channels}]")
    out = torch.empty((seqs, heads * vdim), dtype=proj.dtype, device=proj.device)
    _call("ri_delta_step", _dev(out, "out"), _dev(proj, "proj"), code(proj.dtype), row, q_off, g_off,
          _dev(taps, "taps", torch.float32, (channels, ntaps)), ntaps, _dev(tails, "tails", torch.float32),
          _dev(ab, "ab", torch.float32, (seqs, 2 * heads)), _dev(a_log, "a_log", torch.float32, (heads,)),
          _dev(dt_bias, "dt_bias", torch.float32, (heads,)), _dev(state, "state", torch.float32),
          _dev(cu_seqlens, "cu_seqlens", torch.int32, (seqs + 1,)), _dev(slots, "slots", torch.int32, (seqs,)),
          _dev(gain, "gain", torch.float32, (vdim,)), float(eps), seqs, heads, kv_heads, dim, vdim, _stream())
    return out


EXPERTS_MAX = 1024


def experts_route(z: torch.Tensor, correction: torch.Tensor, top: int):
    """The router of a mixture of experts from its float32 logits ``z [T, E]``: ``s = sigmoid(z)``, the ``top``
    experts with the largest ``s + correction`` (the lower index on a tie), weights ``s / (sum of the chosen s +
    1e-20)``.  Returns ``ids [T, top]`` int32, ``weights [T, top]`` and ``dense [T, E]`` (zero where not chosen)."""
    tokens, experts = z.shape
    ids = torch.empty((tokens, top), dtype=torch.int32, device=z.device)
    weights = torch.empty((tokens, top), dtype=torch.float32, device=z.device)
    dense = torch.empty((tokens, experts), dtype=torch.float32, device=z.device)
    _call("ri_experts_route", _dev(ids, "ids"), _dev(weights, "weights"), _dev(dense, "dense"),
          _dev(z, "z", torch.float32), _dev(correction, "correction", torch.float32, (experts,)), tokens, experts,
          int(top), _stream())
    return ids, weights, dense


ROUTE_SIGMOID, ROUTE_SOFTMAX = 0, 1


def experts_route_general(z: torch.Tensor, correction: torch.Tensor, outs: int, experts: int, top: int, kind: int,
                          normalize: bool, groups: int = 1, keep: int = 1):
    """The general router from float32 logits ``z [T, >= outs]``: scores ``s`` are the sigmoid or the softmax over the
    ``outs`` outputs (``experts`` real ones, then identity experts); the choice is by ``s + correction`` among the outputs of
    the ``keep`` best of ``groups`` equal runs of neighbours (a group's score: its largest choice score); weights are the
    chosen ``s``, over their sum with ``normalize``.  Returns ``ids``, ``weights`` ``[T, top]``, ``dense [T, outs]`` and
    ``extra [T, 2]`` (the identity experts' weight; the sigmoid of column ``outs`` of ``z`` where it has one)."""
    tokens, stride = z.shape
    ids = torch.empty((tokens, top), dtype=torch.int32, device=z.device)
    weights = torch.empty((tokens, top), dtype=torch.float32, device=z.device)
    dense = torch.empty((tokens, outs), dtype=torch.float32, device=z.device)
    extra = torch.empty((tokens, 2), dtype=torch.float32, device=z.device)
    _call("ri_experts_route_general", _dev(ids, "ids"), _dev(weights, "weights"), _dev(dense, "dense"), _dev(extra, "extra"),
          _dev(z, "z", torch.float32), stride, _dev(correction, "correction", torch.float32, (outs,)), tokens, outs, experts,
          int(top), int(kind), int(bool(normalize)), int(groups), int(keep), _stream())
    return ids, weights, dense, extra


def experts_finish(routed: torch.Tensor, x, shared, extra: torch.Tensor) -> torch.Tensor:
    """float32 ``routed + extra[:, 0] * x + extra[:, 1] * shared`` row by row; ``routed`` (float32) and ``shared`` may
    be ``[parts, T, dim]`` (added in order); ``x`` and ``shared`` may be None."""
    tokens, dim = routed.shape[-2:]
    parts = routed.shape[0] if routed.dim() == 3 else 1
    shared_parts = shared.shape[0] if shared is not None and shared.dim() == 3 else 1
    out = torch.empty((tokens, dim), dtype=torch.float32, device=routed.device)
    _call("ri_experts_finish", _dev(out, "out"), _dev(routed, "routed", torch.float32), parts, _opt(x, "x"),
          code(x.dtype) if x is not None else F32, _opt(shared, "shared"), code(shared.dtype) if shared is not None else F32,
          shared_parts, _dev(extra, "extra", torch.float32, (tokens, 2)), tokens, dim, _stream())
    return out


def experts_sort(ids: torch.Tensor, experts: int):
    """The assignments ``ids [T, top]`` sorted by expert and, inside an expert, by token: ``dest [T * top]`` (the row
    of assignment ``t * top + k``) and ``offsets [experts + 1]`` (where every expert's rows begin), int32."""
    pairs = ids.numel()
    dest = torch.empty((pairs,), dtype=torch.int32, device=ids.device)
    rank = torch.empty((pairs,), dtype=torch.int32, device=ids.device)
    offsets = torch.empty((experts + 1,), dtype=torch.int32, device=ids.device)
    counts = torch.empty((experts,), dtype=torch.int32, device=ids.device)
    _call("ri_experts_sort", _dev(dest, "dest"), _dev(offsets, "offsets"), _dev(rank, "rank"), _dev(counts, "counts"),
          _dev(ids, "ids", torch.int32), pairs, experts, _stream())
    return dest, offsets


def experts_gather(x: torch.Tensor, dest: torch.Tensor, top: int) -> torch.Tensor:
    """``rows[dest[t * top + k]] = x[t]``: every assignment's token row at its place among its expert's rows."""
    tokens, dim = x.shape
    rows = torch.empty((tokens * top, dim), dtype=x.dtype, device=x.device)
    _call("ri_experts_gather", _dev(rows, "rows"), _dev(x, "x", torch.bfloat16), _dev(dest, "dest", torch.int32, (tokens * top,)),
          tokens * top, top, dim, _stream())
    return rows


def experts_combine(y: torch.Tensor, dest: torch.Tensor, weights: torch.Tensor) -> torch.Tensor:
    """float32 ``out[t] = sum_k weights[t, k] * y[dest[t * top + k]]``, the sum in the order chosen."""
    tokens, top = weights.shape
    dim = y.shape[1]
    out = torch.empty((tokens, dim), dtype=torch.float32, device=y.device)
    _call("ri_experts_combine", _dev(out, "out"), _dev(y, "y", torch.bfloat16, (tokens * top, dim)),
          _dev(dest, "dest", torch.int32, (tokens * top,)), _dev(weights, "weights", torch.float32), tokens, top, dim, _stream())
    return out


def experts_activate(gu: torch.Tensor, dense, ff: int, limit: float) -> torch.Tensor:
    """``dense[t, e] * g sigmoid(1.702 g) (u + 1)`` with ``g = min(gate, limit)``, ``u = clamp(up, -limit, limit)``
    for ``gu [T, E * 2 * ff]`` (every expert's gate then up); ``[T, E * ff]``, zero for experts not chosen.  ``dense``
    None: rows of one expert each (``gu [T, 2 * ff]``), every weight 1.  ``limit <= 0``: the plain gated form
    ``silu(gate) * up``.  ``dense`` may have more columns than there are experts (a router with outputs that are no
    experts): the first ``E`` are read."""
    if dense is None:
        tokens = gu.shape[0]
        out = torch.empty((tokens, ff), dtype=gu.dtype, device=gu.device)
        if tuple(gu.shape) != (tokens, 2 * ff):
            raise ShapeError(f"gate|up rows are {list(gu.shape)} for experts of {ff}")
        _call("ri_experts_activate", _dev(out, "out"), _dev(gu, "gu"), code(gu.dtype), None, tokens, 1, ff, float(limit), _stream())
        return out
    tokens, outs = dense.shape
    experts = gu.shape[1] // (2 * ff)
    if tuple(gu.shape) != (tokens, experts * 2 * ff) or experts > outs:
        raise ShapeError(f"gate|up rows are {list(gu.shape)} for experts of {ff}, weights {list(dense.shape)}")
    out = torch.empty((tokens, experts * ff), dtype=gu.dtype, device=gu.device)
    _call("ri_experts_activate_strided", _dev(out, "out"), _dev(gu, "gu"), code(gu.dtype), _dev(dense, "dense", torch.float32),
          outs, tokens, experts, ff, float(limit), _stream())
    return out


def experts_few_tokens(x, gate_up, down, ids, weights, ff: int, limit: float) -> torch.Tensor:
    """The weighted sum of the chosen experts' outputs for a few tokens, reading only the chosen experts' rows
    (bfloat16): ``x [T, dim]``, ``gate_up [E * 2 * ff, dim]``, ``down [dim, E * ff]``, ``ids`` and ``weights``
    ``[T, top]`` from ``experts_route``; float32 ``[T, dim]``."""
    tokens, dim = x.shape
    top = ids.shape[1]
    experts = gate_up.shape[0] // (2 * ff)
    if tuple(gate_up.shape) != (experts * 2 * ff, dim) or tuple(down.shape) != (dim, experts * ff):
        raise ShapeError(f"experts' matrices {list(gate_up.shape)} and {list(down.shape)} for rows of {dim} and experts of {ff}")
    out = torch.empty((tokens, dim), dtype=torch.float32, device=x.device)
    act = torch.empty((tokens * top, ff), dtype=torch.bfloat16, device=x.device)
    _call("ri_experts_few_tokens", _dev(out, "out"), _dev(act, "act"), _dev(x, "x", torch.bfloat16),
          _dev(gate_up, "gate_up", torch.bfloat16), _dev(down, "down", torch.bfloat16),
          _dev(ids, "ids", torch.int32, (tokens, top)), _dev(weights, "weights", torch.float32, (tokens, top)),
          tokens, experts, top, ff, dim, float(limit), _stream())
    return out


MFMA_HEAD_DIMS = (32, 64, 128)
MAX_HEAD_DIM = 512          # what the general attention and q/k kernels take (any size from 1 up to it)


def mfma_attention_fits(dtype, head_dim: int, group: int, page_size: int, decode: bool) -> bool:
    """Whether the matrix-core attention kernels take this case (else the generic kernel does)."""
    return (dtype == torch.bfloat16 and head_dim in MFMA_HEAD_DIMS and page_size == 32
            and group <= (16 if decode else (64 if head_dim <= 64 else 32)))


def attention_prefill_bf16(qkv, k_pages, v_pages, cu_seqlens, tok_pos, page_table, seqs: int, max_new: int,
                           heads: int, kv_heads: int, head_dim: int, window: int | None, scale: float,
                           softcap: float | None = None, slopes: torch.Tensor | None = None, keep_first: int = 0,
                           sinks: torch.Tensor | None = None, q_off: int = 0) -> torch.Tensor:
    """Matrix-core attention for any number of new tokens per sequence (bfloat16, pages of 32).  With ``softcap`` a
    score ``s`` becomes ``softcap * tanh(s / softcap)`` before the softmax; with ``slopes`` (float32 ``[heads]``) head
    ``h``'s score at position ``p`` for the key at ``j`` then loses ``slopes[h] * (p - j)``.  ``keep_first``, ``sinks`` and
    ``q_off`` as in ``attention``."""
    tokens, stride = qkv.shape
    if q_off < 0 or q_off + heads * head_dim > stride or q_off % 8:
        raise ShapeError(f"attention: queries at column {q_off} of rows of {stride} for {heads} heads of {head_dim}")
    out = torch.empty((tokens, heads * head_dim), dtype=torch.bfloat16, device=qkv.device)
    _call("ri_attention_prefill_kept_bf16", _dev(out, "out"), _dev(qkv, "qkv", torch.bfloat16) + 2 * int(q_off), stride,
          _dev(k_pages, "k_pages", torch.bfloat16), _dev(v_pages, "v_pages", torch.bfloat16),
          _dev(cu_seqlens, "cu_seqlens", torch.int32, (seqs + 1,)), _dev(tok_pos, "tok_pos", torch.int32, (tokens,)),
          _dev(page_table, "page_table", torch.int32), page_table.shape[1], seqs, max_new, heads, kv_heads, head_dim,
          k_pages.shape[2], int(window or 0), float(scale), float(softcap or 0.0),
          _opt(slopes, "slopes", torch.float32, (heads,)), int(keep_first or 0), _opt(sinks, "sinks", torch.float32, (heads,)),
          _stream())
    return out


def decode_attention_runs(seqs: int, kv_heads: int, max_len: int) -> int:
    """The runs per sequence in which the decode attention's streaming kernel walks a step of this size, or 0
    where it takes one workgroup per chunk of 256 keys instead (host code only: it needs no GPU)."""
    chunks = _get("ri_attention_decode_chunks")(int(max_len))
    return _get("ri_attention_decode_streams")(int(seqs), int(kv_heads), chunks)


def decode_attention_streams(seqs: int, kv_heads: int, max_len: int) -> bool:
    """Whether ``attention_decode_bf16`` walks a step of this size with its streaming kernel (whole runs of a
    sequence's pages per workgroup) rather than with one workgroup per chunk of 256 keys."""
    return decode_attention_runs(seqs, kv_heads, max_len) > 0


def attention_decode_bf16(qkv, k_pages, v_pages, cu_seqlens, tok_pos, page_table, seqs: int, max_len: int,
                          heads: int, kv_heads: int, head_dim: int, window: int | None, scale: float,
                          tiled_out: bool = False, softcap: float | None = None, slopes: torch.Tensor | None = None,
                          keep_first: int = 0, sinks: torch.Tensor | None = None, q_off: int = 0):
    """Matrix-core attention for one new token per sequence; ``max_len`` bounds every sequence's length
    after this step (it sizes the grid and the workspace, not the result).  ``tiled_out``: the result as
    ``TiledRows`` (at most 64 sequences).  ``softcap`` and ``slopes`` as in ``attention_prefill_bf16``; ``keep_first``,
    ``sinks`` and ``q_off`` as in ``attention`` (in steps for which ``decode_attention_streams`` is false)."""
    tokens, stride = qkv.shape
    if tokens != seqs:
        raise ShapeError(f"decode attention takes one token per sequence, got {tokens} tokens for {seqs} sequences")
    if q_off < 0 or q_off + heads * head_dim > stride or q_off % 8:
        raise ShapeError(f"attention: queries at column {q_off} of rows of {stride} for {heads} heads of {head_dim}")
    chunks = _get("ri_attention_decode_chunks")(int(max_len))      # the kernels' own chunk size
    out = (TiledRows.empty(tokens, heads * head_dim, qkv.device) if tiled_out else
           torch.empty((tokens, heads * head_dim), dtype=torch.bfloat16, device=qkv.device))
    pieces = _get("ri_attention_decode_pieces")(int(seqs), int(kv_heads), int(heads), chunks)
    ws = torch.empty((seqs, heads, chunks * pieces, head_dim + 2), dtype=torch.float32, device=qkv.device)
    _call("ri_attention_decode_kept_bf16", _dev(out.data if tiled_out else out, "out"), _dev(ws, "workspace"),
          _dev(qkv, "qkv", torch.bfloat16) + 2 * int(q_off), stride,
          _dev(k_pages, "k_pages", torch.bfloat16), _dev(v_pages, "v_pages", torch.bfloat16),
          _dev(cu_seqlens, "cu_seqlens", torch.int32, (seqs + 1,)), _dev(tok_pos, "tok_pos", torch.int32, (tokens,)),
          _dev(page_table, "page_table", torch.int32), page_table.shape[1], seqs, chunks, heads, kv_heads, head_dim,
          k_pages.shape[2], int(window or 0), float(scale), float(softcap or 0.0),
          _opt(slopes, "slopes", torch.float32, (heads,)), int(tiled_out), int(keep_first or 0),
          _opt(sinks, "sinks", torch.float32, (heads,)), _stream())
    return out


def attention_decode_fused_bf16(qkv, q_gain, k_gain, eps, inv_freq, k_pages, v_pages, tok_pos, page_table, seqs: int,
                                max_len: int, heads: int, kv_heads: int, head_dim: int, window: int | None,
                                scale: float, tiled_out: bool = False):
    """A layer's decode attention from the raw ``qkv: [seqs, (H + 2 Hkv) dh]``: q/k norm, rotation, the new
    token's k and v into their pages and attention in one kernel, then the join.  ``tiled_out``: the result
    as ``TiledRows``."""
    tokens, stride = qkv.shape
    if tokens != seqs:
        raise ShapeError(f"decode attention takes one token per sequence, got {tokens} tokens for {seqs} sequences")
    num_pages, hkv, page_size, dh = k_pages.shape
    if (hkv, dh) != (kv_heads, head_dim) or tuple(v_pages.shape) != (num_pages, hkv, dh, page_size):
        raise ShapeError(f"pages are {list(k_pages.shape)} / {list(v_pages.shape)}, the mixer has {kv_heads} kv heads "
                         f"of {head_dim}")
    chunks = _get("ri_attention_decode_chunks")(int(max_len))      # the kernels' own chunk size
    out = (TiledRows.empty(tokens, heads * head_dim, qkv.device) if tiled_out else
           torch.empty((tokens, heads * head_dim), dtype=torch.bfloat16, device=qkv.device))
    pieces = _get("ri_attention_decode_pieces")(int(seqs), int(kv_heads), int(heads), chunks)
    ws = torch.empty((seqs, heads, chunks * pieces, head_dim + 2), dtype=torch.float32, device=qkv.device)
    half = head_dim // 2
    _call("ri_attention_decode_fused_bf16", _dev(out.data if tiled_out else out, "out"), _dev(ws, "workspace"),
          _dev(qkv, "qkv", torch.bfloat16), stride, _opt(q_gain, "q_gain", torch.float32, (head_dim,)),
          _opt(k_gain, "k_gain", torch.float32, (head_dim,)), float(eps),
          _opt(inv_freq, "inv_freq", torch.float32, (half,)), _dev(k_pages, "k_pages", torch.bfloat16),
          _dev(v_pages, "v_pages", torch.bfloat16), _dev(tok_pos, "tok_pos", torch.int32, (tokens,)),
          _dev(page_table, "page_table", torch.int32), page_table.shape[1], seqs, chunks, heads, kv_heads, head_dim,
          page_size, int(window or 0), float(scale), int(tiled_out), _stream())
    return out


# ---------------------------------------------------------------- products
def gemm_f32(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """``x @ w.T`` in true 32-bit arithmetic; ``x`` float32 ``[M, K]``, ``w`` float32 or bfloat16 ``[N, K]``."""
    m, k = x.shape
    n = w.shape[0]
    out = torch.empty((m, n), dtype=torch.float32, device=x.device)
    _call("ri_gemm_f32", _dev(out, "out"), _dev(x, "x", torch.float32), _dev(w, "w", None, (n, k)), code(w.dtype),
          m, n, k, _stream())
    return out


def gemv_bf16(x: torch.Tensor, w: torch.Tensor, out_dtype=torch.bfloat16, swiglu: bool = False) -> torch.Tensor:
    """``x @ w.T`` for up to 8 bfloat16 rows; with ``swiglu`` ``w`` is gate rows then up rows and the
    result is ``silu(gate) * up``."""
    m, k = x.shape
    n = w.shape[0] // 2 if swiglu else w.shape[0]
    out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    _call("ri_gemv_bf16", _dev(out, "out"), code(out_dtype), _dev(x, "x", torch.bfloat16),
          _dev(w, "w", torch.bfloat16, (w.shape[0], k)), m, n, k, int(swiglu), _stream())
    return out


def pack_for_mfma(w: torch.Tensor, swiglu: bool = False) -> torch.Tensor:
    """A bfloat16 weight ``[N, K]`` cut into MFMA A-operand tiles: ``[ceil(N/16), ceil(K/32), 64, 8]``, lane
    ``l`` of a tile holding row ``l % 16`` and ``k = 8 * (l // 16) ..+8``, zero beyond N and K.  With
    ``swiglu`` the gate half and the up half of ``[2 N, K]`` are packed one after the other."""
    if swiglu:
        half = w.shape[0] // 2
        return torch.cat([pack_for_mfma(w[:half]), pack_for_mfma(w[half:])], 0)
    n, k = w.shape
    n16, k32 = -(-n // 16) * 16, -(-k // 32) * 32
    if (n16, k32) != (n, k):
        padded = torch.zeros((n16, k32), dtype=w.dtype, device=w.device)
        padded[:n, :k] = w
        w = padded
    tiles = w.view(n16 // 16, 16, k32 // 32, 4, 8).permute(0, 2, 3, 1, 4)      # [row tile, k tile, k group, row, 8]
    return tiles.reshape(n16 // 16, k32 // 32, 64, 8).contiguous()


TILED_X, TILED_OUT = 1, 2


class TiledRows:
    """Up to 64 bfloat16 rows of ``k`` columns in the order the matrix cores take them as an operand:
    ``data[ceil(m / 16), ceil(k / 32), 64, 8]``, lane ``l`` of a tile holding row ``l % 16`` of its 16 rows and
    the columns ``8 * (l // 16) ..+8`` of its 32.  A packed product, a norm or the decode attention writes its
    result this way for the packed product after it, which then loads a tile as one kilobyte in a row; rows
    beyond ``m`` and columns beyond ``k`` are never read."""

    def __init__(self, data: torch.Tensor, m: int, k: int):
        self.data, self.shape = data, (m, k)
        self.dtype, self.device = data.dtype, data.device

    @staticmethod
    def empty(m: int, k: int, device) -> "TiledRows":
        if not 1 <= m <= 64:
            raise ShapeError(f"tiled rows hold 1 to 64 rows, not {m}")
        return TiledRows(torch.empty((-(-m // 16), -(-k // 32), 64, 8), dtype=torch.bfloat16, device=device), m, k)

    def rows(self) -> torch.Tensor:
        """The same values row-major, ``[m, k]``."""
        m, k = self.shape
        row_tiles, tiles = self.data.shape[:2]
        return (self.data.view(row_tiles, tiles, 4, 16, 8).permute(0, 3, 1, 2, 4)
                .reshape(row_tiles * 16, tiles * 32)[:m, :k].contiguous())


def as_rows(x):
    """A tensor for code that wants plain rows."""
    return x.rows() if isinstance(x, TiledRows) else x


def gemm_skinny_packed_bf16(x, wpacked: torch.Tensor, n: int, out_dtype=torch.bfloat16,
                            swiglu: bool = False, parts: int = 1, tiled_out: bool = False):
    """``x @ w.T`` for up to 16 bfloat16 rows (a tensor or ``TiledRows``) with ``w`` packed by
    ``pack_for_mfma``; ``n`` is the number of output columns (rows of w; of its gate half with ``swiglu``).
    With ``parts > 1`` K is cut into that many pieces and the result is their float32 sums ``[parts, M, n]``,
    for a consumer that adds them.  With ``tiled_out`` the bfloat16 result comes as ``TiledRows``."""
    m, k = x.shape
    row_tiles = -(-n // 16)
    want = (row_tiles * (2 if swiglu else 1), -(-k // 32), 64, 8)
    if tuple(wpacked.shape) != want:
        raise ShapeError(f"packed weight is {list(wpacked.shape)}, a product with n {n}, k {k} wants {list(want)}")
    if tiled_out and (parts != 1 or out_dtype != torch.bfloat16):
        raise ShapeError("a tiled result is bfloat16 and whole")
    flags = (TILED_X if isinstance(x, TiledRows) else 0) | (TILED_OUT if tiled_out else 0)
    xd = _dev(x.data, "x", torch.bfloat16) if isinstance(x, TiledRows) else _dev(x, "x", torch.bfloat16)
    if tiled_out:
        out = TiledRows.empty(m, n, x.device)
        od = _dev(out.data, "out")
    else:
        out = torch.empty((m, n) if parts == 1 else (parts, m, n), dtype=out_dtype, device=x.device)
        od = _dev(out, "out")
    _call("ri_gemm_skinny_packed_bf16", od, code(out_dtype), xd, _dev(wpacked, "wpacked", torch.bfloat16), m, n, k,
          int(swiglu), int(parts), flags, _stream())
    return out


class NormedLater:
    """Rows of a residual stream whose RMSNorm is left to the product that reads them:
    ``xg = bfloat16(r * gain)`` and partial sums of ``r^2`` per row, ``[M, partials]``; the
    normed rows are ``xg / sqrt(ssq.sum(1) / dim + eps)``.  ``xg`` is a tensor or ``TiledRows``."""

    def __init__(self, xg, ssq: torch.Tensor, eps: float, dim: int):
        self.xg, self.ssq, self.eps, self.dim = xg, ssq, float(eps), int(dim)
        self.shape, self.dtype, self.device = xg.shape, xg.dtype, xg.device


def finish_norm(later: NormedLater) -> torch.Tensor:
    """The normed bfloat16 rows ``[M, dim]`` of a ``NormedLater``, for a reader that cannot take the norm
    over (``xg`` was rounded once already, so this differs from the plain norm by one more rounding)."""
    xg = later.xg
    tiled = isinstance(xg, TiledRows)
    m, dim = xg.shape
    out = torch.empty((m, dim), dtype=torch.bfloat16, device=later.device)
    _call("ri_finish_norm", _dev(out, "out"), _dev(xg.data if tiled else xg, "xg", torch.bfloat16),
          _dev(later.ssq, "ssq", torch.float32, (m, later.ssq.shape[1])), later.ssq.shape[1], later.eps, later.dim, m,
          int(tiled), _stream())
    return out


def gemm_mid_packed_bf16(x, wpacked: torch.Tensor, n: int, out_dtype=torch.bfloat16, swiglu: bool = False,
                         tiled_out: bool = False):
    """``x @ w.T`` for up to 64 bfloat16 rows (a tensor or ``TiledRows``) with ``w`` packed by
    ``pack_for_mfma``: the packed product for the steps of 17 to 64 tokens.  ``tiled_out``: the bfloat16
    result as ``TiledRows``."""
    m, k = x.shape
    row_tiles = -(-n // 16)
    want = (row_tiles * (2 if swiglu else 1), -(-k // 32), 64, 8)
    if tuple(wpacked.shape) != want:
        raise ShapeError(f"packed weight is {list(wpacked.shape)}, a product with n {n}, k {k} wants {list(want)}")
    if tiled_out and out_dtype != torch.bfloat16:
        raise ShapeError("a tiled result is bfloat16")
    x_tiled = isinstance(x, TiledRows)
    out = TiledRows.empty(m, n, x.device) if tiled_out else torch.empty((m, n), dtype=out_dtype, device=x.device)
    _call("ri_gemm_mid_packed_bf16", _dev(out.data if tiled_out else out, "out"), code(out_dtype),
          _dev(x.data if x_tiled else x, "x", torch.bfloat16), _dev(wpacked, "wpacked", torch.bfloat16), m, n, k,
          int(swiglu), (TILED_X if x_tiled else 0) | (TILED_OUT if tiled_out else 0), _stream())
    return out


def compute_units() -> int:
    """Compute units of the current device (256 where there is none): what the rules that size launches
    count workgroups against."""
    return int(_get("ri_compute_units")())


def wide_product_plan(n: int, k: int, swiglu: bool = False, rows: int = 64) -> tuple[int, int]:
    """``(waves, parts)``: how many wavefronts a workgroup of ``gemm_wide_packed_bf16`` should have and into how
    many stretches of K it should cut a product of ``rows`` rows with an ``n x k`` matrix (host code only): with the
    activation K whole and the wavefronts that fill the compute units more evenly; without it, from 17 rows on,
    what makes a compute unit fetch the fewest bytes."""
    waves, parts = ctypes.c_int(0), ctypes.c_int(0)
    if swiglu:
        if rows > 64:
            raise ShapeError("more than 64 rows go without the activation")
        _call("ri_gemm_wide_packed_bf16_plan", int(n), int(k), 1, ctypes.addressof(waves), ctypes.addressof(parts))
    else:
        _call("ri_gemm_wide_stretch_plan", int(rows), int(n), int(k), ctypes.addressof(waves), ctypes.addressof(parts))
    return waves.value, parts.value


def gemm_wide_packed_bf16(x, wpacked: torch.Tensor, n: int, out_dtype=torch.bfloat16, swiglu: bool = False,
                          parts: int = 1, tiled_out: bool = False, depth: int = 2, waves: int = 4):
    """``x @ w.T`` for up to 64 bfloat16 rows (a tensor or ``TiledRows``) with ``w`` packed by ``pack_for_mfma``,
    the tiles of x shared by a workgroup's wavefronts through LDS: the product for steps of 17 to 64 tokens.
    65 to 256 plain rows (past 128 in two passes over the weights): float32 sums in rows (``waves`` and ``parts``
    from ``wide_product_plan(..., rows=m)``), ``depth`` 1; with ``swiglu`` 65 to 128 plain rows where the plan says
    five to eight wavefronts, K whole.
    ``parts > 1``: K in that many stretches, the result their float32 sums ``[parts, M, n]`` for a reader
    that adds them (with ``swiglu`` ``[parts, M, 2 n]``, gate sums then up sums, the activation left to
    ``sum_parts``).  ``tiled_out``: the bfloat16 result as ``TiledRows``.  ``waves``: wavefronts (row tiles) a
    workgroup, 3 or 4, with the activation at ``depth`` 1 up to 8 (``wide_product_plan``); the sums do not depend on it."""
    m, k = x.shape
    row_tiles = -(-n // 16)
    want = (row_tiles * (2 if swiglu else 1), -(-k // 32), 64, 8)
    if tuple(wpacked.shape) != want:
        raise ShapeError(f"packed weight is {list(wpacked.shape)}, a product with n {n}, k {k} wants {list(want)}")
    if m > 64:
        if tiled_out or isinstance(x, TiledRows) or (not swiglu and out_dtype != torch.float32) or (swiglu and (parts != 1 or m > 128)):
            raise ShapeError("more than 64 rows: plain rows in and out; float32 sums without the activation, "
                             "or up to 128 rows with it and K whole")
        depth = 1
    if parts != 1 and (out_dtype != torch.float32 or tiled_out):
        raise ShapeError("a product in parts has float32 sums in rows")
    if tiled_out and out_dtype != torch.bfloat16:
        raise ShapeError("a tiled result is bfloat16")
    x_tiled = isinstance(x, TiledRows)
    if tiled_out:
        out = TiledRows.empty(m, n, x.device)
    else:
        out = torch.empty((m, n) if parts == 1 else (parts, m, 2 * n if swiglu else n), dtype=out_dtype, device=x.device)
    _call("ri_gemm_wide_packed_bf16", _dev(out.data if tiled_out else out, "out"), code(out_dtype),
          _dev(x.data if x_tiled else x, "x", torch.bfloat16), _dev(wpacked, "wpacked", torch.bfloat16), m, n, k,
          int(swiglu), int(parts), (TILED_X if x_tiled else 0) | (TILED_OUT if tiled_out else 0), int(depth),
          int(waves), _stream())
    return out


def sum_parts(parts: torch.Tensor, out_dtype=torch.bfloat16, tiled_out: bool = False, swiglu: bool = False):
    """``parts.sum(0)`` of float32 ``[parts, M, n]``, added in order, as ``out_dtype`` (bfloat16 also as
    ``TiledRows``); with ``swiglu`` the rows are gate sums then up sums and the result ``silu(gate) * up``."""
    p, m, n = parts.shape
    if swiglu:
        if n % 2:
            raise ShapeError(f"gate and up sums side by side have an even width, not {n}")
        n //= 2
    out = TiledRows.empty(m, n, parts.device) if tiled_out else torch.empty((m, n), dtype=out_dtype, device=parts.device)
    _call("ri_sum_parts", _dev(out.data if tiled_out else out, "out"), code(torch.bfloat16 if tiled_out else out_dtype),
          _dev(parts, "parts", torch.float32), p, m, n, int(swiglu), int(tiled_out), _stream())
    return out


def linked_product(x, w: torch.Tensor, n: int, packed: bool, out_dtype=torch.bfloat16, swiglu: bool = False,
                   residual: torch.Tensor | None = None, next_gain: torch.Tensor | None = None,
                   next_eps: float = 0.0, tiled_out: bool = False):
    """A decode-size product that does the RMSNorm before it, the residual add and the RMSNorm's
    preparation after it, or both, in the same kernel.

    ``x`` is bfloat16 rows (a tensor or ``TiledRows``) or a ``NormedLater``; ``w`` the row-major weight
    (``packed`` false: up to 8 rows, one wavefront per weight row) or its MFMA tiles (``packed`` true: up to
    16 rows).  With ``residual`` (float32 ``[M, n]``, updated in place to ``residual + x @ w.T``) the result
    is the ``NormedLater`` of the new residual for a norm with ``next_gain`` and ``next_eps``; else the
    product.  ``tiled_out`` (packed only) asks for the bfloat16 rows of the result as ``TiledRows``."""
    later = x if isinstance(x, NormedLater) else None
    xr = later.xg if later else x
    if not packed:
        xr, tiled_out = as_rows(xr), False
    m, k = xr.shape
    name = "ri_gemm_skinny_packed_bf16" if packed else "ri_gemv_bf16"
    if packed:
        want = (-(-n // 16) * (2 if swiglu else 1), -(-k // 32), 64, 8)
        if tuple(w.shape) != want:
            raise ShapeError(f"packed weight is {list(w.shape)}, a product with n {n}, k {k} wants {list(want)}")
        wd = _dev(w, "wpacked", torch.bfloat16)
    else:
        wd = _dev(w, "w", torch.bfloat16, (n * (2 if swiglu else 1), k))
    x_tiled = isinstance(xr, TiledRows)
    xd = _dev(xr.data, "x", torch.bfloat16) if x_tiled else _dev(xr, "x", torch.bfloat16, (m, k))
    # the packed kernel takes the layouts of x and of its result as one more argument
    layout = ((TILED_X if x_tiled else 0) | (TILED_OUT if tiled_out else 0),) if packed else ()
    if later is not None:
        ssq_in = _dev(later.ssq, "ssq", torch.float32, (m, later.ssq.shape[1]))
        n_in, eps, dim = later.ssq.shape[1], later.eps, later.dim
        if dim != k:
            raise ShapeError(f"rows normed over {dim} elements into a product over {k}")
    else:
        ssq_in, n_in, eps, dim = None, 0, 0.0, 0
    if residual is None:
        if tiled_out and out_dtype != torch.bfloat16:
            raise ShapeError("a tiled result is bfloat16")
        out = TiledRows.empty(m, n, xr.device) if tiled_out else torch.empty((m, n), dtype=out_dtype, device=xr.device)
        _call(name + "_linked", _dev(out.data if tiled_out else out, "out"), code(out_dtype), xd, wd, m, n, k,
              int(swiglu), ssq_in, n_in, eps, dim, None, None, None, None, *layout, _stream())
        return out
    if swiglu:
        raise ShapeError("a gate|up product does not feed the residual stream")
    partials = _get("ri_gemm_skinny_packed_bf16_partials")(n) if packed else _get("ri_gemv_bf16_partials")(n, k)
    xg = TiledRows.empty(m, n, xr.device) if tiled_out else torch.empty((m, n), dtype=torch.bfloat16, device=xr.device)
    ssq = torch.empty((m, partials), dtype=torch.float32, device=xr.device)
    _call(name + "_linked", None, code(torch.bfloat16), xd, wd, m, n, k, 0,
          ssq_in, n_in, eps, dim, _dev(residual, "residual", torch.float32, (m, n)),
          _dev(next_gain, "next_gain", torch.float32, (n,)), _dev(xg.data if tiled_out else xg, "xg"), _dev(ssq, "ssq"),
          *layout, _stream())
    return NormedLater(xg, ssq, next_eps, n)


# ---------------------------------------------------------------- layers whose norm sits behind the residual sum
def scaled_sum_norm(residual: torch.Tensor, y: torch.Tensor, y_bias, alpha: float, gain, bias, eps: float, norm_kind: int,
                    act_dtype=None):
    """``residual <- norm(alpha * residual + y + y_bias)`` in place (float32), the norm a layer norm (``NORM_LAYER``, with
    ``bias``) or an RMS norm (``NORM_RMS``) with ``gain``; ``y`` is ``[T, dim]`` or float32 ``[parts, T, dim]`` (added in
    order), ``y_bias`` a float32 row or None.  With ``act_dtype`` the new residual is also returned in that format."""
    rows, dim = residual.shape
    parts = y.shape[0] if y.dim() == 3 else 1
    if tuple(y.shape[-2:]) != (rows, dim):
        raise ShapeError(f"a branch output of {list(y.shape)} for a residual of {list(residual.shape)}")
    act = torch.empty((rows, dim), dtype=act_dtype, device=residual.device) if act_dtype is not None else None
    _call("ri_scaled_sum_norm", _dev(residual, "residual", torch.float32), _opt(act, "act"), code(act_dtype or torch.float32),
          _dev(y, "y"), code(y.dtype), parts, _opt(y_bias, "y_bias", torch.float32, (dim,)), float(alpha),
          _dev(gain, "gain", torch.float32, (dim,)), _opt(bias, "bias", torch.float32, (dim,)), float(eps), int(norm_kind),
          rows, dim, _stream())
    return act


def glu_clamped_bias(gu: torch.Tensor, b_gate, b_up, limit: float) -> torch.Tensor:
    """``g sigmoid(1.702 g) (u + 1)`` with ``g = min(gate + b_gate, limit)``, ``u = clamp(up + b_up, -limit, limit)`` for rows
    ``gu [T, gate | up]``; the biases are float32 rows or None."""
    rows, two = gu.shape
    ff = two // 2
    if two != 2 * ff:
        raise ShapeError(f"gate|up rows of {two} elements")
    out = torch.empty((rows, ff), dtype=gu.dtype, device=gu.device)
    _call("ri_glu_clamped_bias", _dev(out, "out"), _dev(gu, "gu"), code(gu.dtype), _opt(b_gate, "b_gate", torch.float32, (ff,)),
          _opt(b_up, "b_up", torch.float32, (ff,)), float(limit), rows, ff, _stream())
    return out


PLAIN_ACTIVATIONS = {"gelu_erf": 0, "gelu_tanh": 1, "relu2": 2}      # what experts without a gate may name


def experts_activate_plain(u: torch.Tensor, dense, ff: int, activation: str) -> torch.Tensor:
    """``dense[t, e] * act(u[t, e, :])`` for ``u [T, E * ff]``, zero for the experts a token did not choose; ``dense`` None:
    every weight 1."""
    tokens, wide = u.shape
    experts = wide // ff
    if wide != experts * ff or (dense is not None and (dense.shape[0] != tokens or dense.shape[1] < experts)):
        raise ShapeError(f"up rows are {list(u.shape)} for experts of {ff}, weights {None if dense is None else list(dense.shape)}")
    out = torch.empty_like(u)
    _call("ri_experts_activate_plain", _dev(out, "out"), _dev(u, "u"), code(u.dtype), _opt(dense, "dense", torch.float32),
          dense.shape[1] if dense is not None else experts, tokens, experts, ff, PLAIN_ACTIVATIONS[activation], _stream())
    return out


def softcap_rows(x: torch.Tensor, cap: float) -> torch.Tensor:
    """``x <- cap * tanh(x / cap)`` in place (float32); returns ``x``."""
    if x.numel():
        _call("ri_softcap_rows", _dev(x, "x", torch.float32), float(cap), x.numel(), _stream())
    return x


# ---------------------------------------------------------------- attention over a cached latent
GENERIC_MAX_HEAD_DIM = 1024      # what the general attention kernel alone takes


def latent_prepare(proj, q_off: int, kv_off: int, gain, eps: float, inv_freq, tok_pos, tok_seq, page_table, k_pages, v_pages,
                   heads: int, dim: int, rot: int, rank: int) -> None:
    """In rows ``proj [T, ...]``: the latent (``rank`` columns from ``kv_off``) is RMS-normed with ``gain`` and written, with
    the rotated ``rot`` columns behind it, as the token's key row ``[rank + rot]`` of one key/value head, and alone as its
    value row; the last ``rot`` elements of every query head (``heads`` of ``dim + rot`` from ``q_off``) are rotated in place."""
    tokens, stride = proj.shape
    if tuple(k_pages.shape[1:]) != (1, v_pages.shape[3], rank + rot) or tuple(v_pages.shape[1:3]) != (1, rank):
        raise ShapeError(f"latent_prepare: key pages {list(k_pages.shape)}, value pages {list(v_pages.shape)} for a latent of "
                         f"{rank} + {rot}")
    _call("ri_latent_prepare", _dev(proj, "proj"), code(proj.dtype), stride, int(q_off), int(kv_off),
          _dev(gain, "gain", torch.float32, (rank,)), float(eps), _opt(inv_freq, "inv_freq", torch.float32, (rot // 2,)),
          _dev(tok_pos, "tok_pos", torch.int32, (tokens,)), _dev(tok_seq, "tok_seq", torch.int32, (tokens,)),
          _dev(page_table, "page_table", torch.int32), page_table.shape[1], _dev(k_pages, "k_pages"), _dev(v_pages, "v_pages"),
          code(k_pages.dtype), k_pages.shape[2], tokens, heads, dim, rot, rank, _stream())


def latent_attention_mfma_fits(dtype, key_dim: int, rank: int, page_size: int) -> bool:
    return dtype == torch.bfloat16 and bool(_get("ri_latent_attention_mfma_fits")(key_dim, rank, page_size))


def latent_attention_mfma(q, k_pages, v_pages, tok_pos, tok_seq, page_table, heads: int, scale: float, sinks,
                          max_len: int = 0) -> torch.Tensor:
    """bfloat16 ``[T, heads * rank]``: causal attention on the matrix cores of every new token's ``heads`` query rows (``q [T,
    heads * key_dim]``) over its sequence's single key/value head (``k_pages [pages, 1, 32, key_dim]``, ``v_pages [pages, 1, rank,
    32]``), with a sink per head in the softmax's denominator (or None).  ``max_len``: a bound on the sequences' lengths; given, a
    step of few tokens cuts every token's pages into chunks that run side by side and are joined by a second launch."""
    tokens = q.shape[0]
    key_dim, rank, page = k_pages.shape[3], v_pages.shape[2], k_pages.shape[2]
    if k_pages.shape[1] != 1 or v_pages.shape[1] != 1 or v_pages.shape[3] != page or q.shape[1] != heads * key_dim:
        raise ShapeError(f"latent_attention_mfma: q {list(q.shape)}, key pages {list(k_pages.shape)}, value pages {list(v_pages.shape)}")
    out = torch.empty((tokens, heads * rank), dtype=torch.bfloat16, device=q.device)
    chunks, chunk_pages, partial = 1, 0, None
    units = tokens * -(-heads // 16)
    if max_len and units < 256:                      # fewer wavefronts than half the machine's SIMDs: chunks of pages side by side
        pages = -(-int(max_len) // page)
        chunks = max(1, min(pages, 512 // units, 64))
        chunk_pages = -(-pages // chunks)
        chunks = -(-pages // chunk_pages)
        if chunks > 1:
            partial = torch.empty((tokens, heads, chunks, rank + 2), dtype=torch.float32, device=q.device)
    _call("ri_latent_attention_mfma", _dev(out, "out"), _dev(q, "q", torch.bfloat16), q.shape[1],
          _dev(k_pages, "k_pages", torch.bfloat16), _dev(v_pages, "v_pages", torch.bfloat16),
          _dev(tok_pos, "tok_pos", torch.int32, (tokens,)), _dev(tok_seq, "tok_seq", torch.int32, (tokens,)),
          _dev(page_table, "page_table", torch.int32), page_table.shape[1], tokens, heads, key_dim, rank, page, float(scale),
          _opt(sinks, "sinks", torch.float32, (heads,)), _opt(partial, "partial"), chunks, chunk_pages, _stream())
    return out


def head_products(x, x_off: int, x_head: int, w, heads: int, k: int, n: int, extra: int = 0, out=None, out_off: int = 0,
                  out_head: int | None = None, gates=None, g_off: int = 0, scale: float = 1.0, out_dtype=None):
    """``out[t, out_off + h * out_head + (0..n)] = scale * sigmoid(gates[t, g_off + h]) * x[t, x_off + h * x_head + (0..k)] @ w[h]``
    for a stack of matrices ``w [heads, k, n]``; the ``extra`` elements of ``x`` behind ``k`` are copied behind ``n`` (times
    the same factors).  ``out`` None: a new tensor ``[T, heads * (n + extra)]`` of ``out_dtype`` (default: ``x``'s)."""
    tokens = x.shape[0]
    if tuple(w.shape) != (heads, k, n):
        raise ShapeError(f"head_products: matrices {list(w.shape)} for {heads} heads of {k} x {n}")
    if out is None:
        out_head = n + extra
        out = torch.empty((tokens, heads * out_head), dtype=out_dtype or x.dtype, device=x.device)
    if out.shape[0] != tokens or (gates is not None and (gates.shape[0] != tokens or gates.dtype != x.dtype)):
        raise ShapeError(f"head_products: out {list(out.shape)}, x {list(x.shape)}")
    _call("ri_head_products", _dev(out, "out"), code(out.dtype), out.shape[1], int(out_off), int(out_head), _dev(x, "x"),
          code(x.dtype), x.shape[1], int(x_off), int(x_head), _dev(w, "w"), code(w.dtype), _opt(gates, "gates"),
          gates.shape[1] if gates is not None else 0, int(g_off), float(scale), tokens, heads, k, n, int(extra), _stream())
    return out


def head_gate_copy(out, out_off: int, out_head: int, x, x_off: int, x_head: int, heads: int, width: int, gates=None,
                   g_off: int = 0, scale: float = 1.0) -> None:
    """``out[t, out_off + h * out_head + (0..width)] = scale * sigmoid(gates[t, g_off + h]) * x[t, x_off + h * x_head + (0..width)]``:
    the copying half of ``head_products`` alone (no matrices)."""
    tokens = x.shape[0]
    if out.shape[0] != tokens or (gates is not None and (gates.shape[0] != tokens or gates.dtype != x.dtype)):
        raise ShapeError(f"head_gate_copy: out {list(out.shape)}, x {list(x.shape)}")
    _call("ri_head_products", _dev(out, "out"), code(out.dtype), out.shape[1], int(out_off), int(out_head), _dev(x, "x"),
          code(x.dtype), x.shape[1], int(x_off), int(x_head), _dev(x, "x"), code(x.dtype), _opt(gates, "gates"),
          gates.shape[1] if gates is not None else 0, int(g_off), float(scale), tokens, heads, 0, 0, int(width), _stream())


BATCHED_HEAD_PRODUCTS_FROM = 128       # tokens of a step from which the products per head go to the library


def head_products_batched(x, x_off: int, x_head: int, w, heads: int, k: int, n: int, extra: int = 0, gates=None,
                          g_off: int = 0) -> torch.Tensor:
    """What ``head_products`` gives for bfloat16 rows, with the products as one batched product of the library over the
    heads (float32 sums, rounded once); the copied elements and the gates go through ``head_gate_copy``.  For steps of
    many tokens: the library's product runs on the matrix cores, ``head_products`` on the vector units."""
    tokens = x.shape[0]
    if tuple(w.shape) != (heads, k, n) or x.dim() != 2 or x.stride(1) != 1 or not w.is_contiguous():
        raise ShapeError(f"head_products_batched: matrices {list(w.shape)} for {heads} heads of {k} x {n}, rows {list(x.shape)}")
    if x_off < 0 or x_head < k + extra or x_off + (heads - 1) * x_head + k + extra > x.shape[1]:
        raise ShapeError(f"head_products_batched: heads of {x_head} at column {x_off} of rows of {x.shape[1]}")
    out_head = n + extra
    out = torch.empty((tokens, heads * out_head), dtype=x.dtype, device=x.device)
    xv = x.as_strided((heads, tokens, k), (x_head, x.stride(0), 1), x.storage_offset() + x_off)
    if gates is None:
        torch.bmm(xv, w, out=out.as_strided((heads, tokens, n), (out_head, out.stride(0), 1)))
        if extra:
            head_gate_copy(out, n, out_head, x, x_off + k, x_head, heads, extra)
        return out
    plain = torch.empty_like(out)
    torch.bmm(xv, w, out=plain.as_strided((heads, tokens, n), (out_head, plain.stride(0), 1)))
    if extra:
        head_gate_copy(plain, n, out_head, x, x_off + k, x_head, heads, extra)
    head_gate_copy(out, 0, out_head, plain, 0, out_head, heads, out_head, gates=gates, g_off=g_off)
    return out


# ---------------------------------------------------------------- windowed attention whose heads talk
def whole_norm_kv_write(proj, q_off: int, k_off: int, q_gain, k_gain, eps: float, tok_pos, tok_seq, page_table, k_pages,
                        v_pages, heads: int, kv_heads: int, dim: int) -> None:
    """q (``heads * dim`` columns from ``q_off``) and k (``kv_heads * dim`` from ``k_off``) of every row are RMS-normed over
    the whole projection with a gain an element; q stays in place, the normed k goes to the key pages and k as projected
    to the value pages."""
    tokens, stride = proj.shape
    if tuple(k_pages.shape[1:]) != (kv_heads, v_pages.shape[3], dim) or tuple(v_pages.shape[1:3]) != (kv_heads, dim):
        raise ShapeError(f"whole_norm_kv_write: key pages {list(k_pages.shape)}, value pages {list(v_pages.shape)}")
    _call("ri_whole_norm_kv_write", _dev(proj, "proj"), code(proj.dtype), stride, int(q_off), int(k_off),
          _dev(q_gain, "q_gain", torch.float32, (heads * dim,)), _dev(k_gain, "k_gain", torch.float32, (kv_heads * dim,)),
          float(eps), _dev(tok_pos, "tok_pos", torch.int32, (tokens,)), _dev(tok_seq, "tok_seq", torch.int32, (tokens,)),
          _dev(page_table, "page_table", torch.int32), page_table.shape[1], _dev(k_pages, "k_pages"), _dev(v_pages, "v_pages"),
          code(k_pages.dtype), k_pages.shape[2], tokens, heads, kv_heads, dim, _stream())


def talking_attention_shares(tokens: int, longest: int) -> int:
    """Into how many shares a step of ``tokens`` tokens that see up to ``longest`` keys each cuts its walk over the keys."""
    return _get("ri_talking_attention_shares")(int(tokens), int(longest))


def talking_attention(proj, q_off: int, k_pages, v_pages, tok_pos, tok_seq, page_table, heads: int, kv_heads: int, dim: int,
                      window: int | None, scale: float, r1, r2, talk, shares: int = 1) -> torch.Tensor:
    """Windowed attention of every new token over its sequence's pages with the distance bias ``r1_h ln(1 + r2_h (i - j))``
    taken off the scores and the heads' weights mixed by ``talk [heads, heads]`` after the softmax: ``[T, heads * dim]``, the
    heads side by side.  ``r1``/``r2`` and ``talk`` may be None.  With ``shares > 1`` (a step of few tokens) the walk over the
    keys is cut into that many shares that run side by side, and the result is float32."""
    tokens = proj.shape[0]
    width = heads * dim
    stats = torch.empty((tokens, heads, 2), dtype=torch.float32, device=proj.device)
    out = (torch.empty((tokens, width), dtype=proj.dtype, device=proj.device) if shares == 1
           else torch.empty((shares, tokens, width), dtype=torch.float32, device=proj.device))
    _call("ri_talking_attention", _dev(out, "out"), code(out.dtype), width, 0, 1.0, int(shares), _dev(stats, "stats"),
          _dev(proj, "proj"), code(proj.dtype), proj.shape[1], int(q_off), _dev(k_pages, "k_pages"), _dev(v_pages, "v_pages"),
          code(k_pages.dtype), _dev(tok_pos, "tok_pos", torch.int32, (tokens,)), _dev(tok_seq, "tok_seq", torch.int32, (tokens,)),
          _dev(page_table, "page_table", torch.int32), page_table.shape[1], tokens, heads, kv_heads, dim, k_pages.shape[2],
          int(window or 0), float(scale), _opt(r1, "r1", torch.float32, (heads,)), _opt(r2, "r2", torch.float32, (heads,)),
          _opt(talk, "talk", torch.float32, (heads, heads)), _stream())
    return out if shares == 1 else sum_parts(out, torch.float32)


def talking_attention_mfma_fits(dtype, heads: int, kv_heads: int, dim: int, page_size: int) -> bool:
    return dtype == torch.bfloat16 and bool(_get("ri_talking_attention_mfma_fits")(heads, kv_heads, dim, page_size))


def talking_attention_mfma(proj, q_off: int, k_pages, v_pages, tok_pos, cu_seqlens, new_counts, page_table, heads: int,
                           kv_heads: int, dim: int, window: int | None, scale: float, r1, r2, talk) -> torch.Tensor:
    """The same attention on the matrix cores, for prompts in bfloat16: ``[T, heads * dim]``.  ``new_counts``: every
    sequence's number of new tokens (the host's list), by which the launch counts its tiles of 16 tokens."""
    tokens = proj.shape[0]
    seqs = len(new_counts)
    tiles = sum(-(-int(n) // 16) for n in new_counts)
    out = torch.empty((tokens, heads * dim), dtype=torch.bfloat16, device=proj.device)
    if tiles == 0:
        return out
    stats = torch.empty((tokens, heads, 2), dtype=torch.float32, device=proj.device)
    _call("ri_talking_attention_mfma", _dev(out, "out"), _dev(stats, "stats"), _dev(proj, "proj", torch.bfloat16), proj.shape[1],
          int(q_off), _dev(k_pages, "k_pages", torch.bfloat16), _dev(v_pages, "v_pages", torch.bfloat16),
          _dev(tok_pos, "tok_pos", torch.int32, (tokens,)), _dev(cu_seqlens, "cu_seqlens", torch.int32, (seqs + 1,)), seqs,
          _dev(page_table, "page_table", torch.int32), page_table.shape[1], tiles, heads, kv_heads, dim, k_pages.shape[2],
          int(window or 0), float(scale), _opt(r1, "r1", torch.float32, (heads,)), _opt(r2, "r2", torch.float32, (heads,)),
          _opt(talk, "talk", torch.float32, (heads, heads)), _stream())
    return out


# ---------------------------------------------------------------- time mixing
def timemix_max_dim() -> int:
    return _get("ri_timemix_max_dim")()


def shift_mix(x32, kept, mu, tok_seq, cu_seqlens, slots, out_dtype) -> torch.Tensor:
    """``[n, T, width]``: for every mixing vector ``mu[s]`` the rows ``h + (h' - h) * mu[s]``, ``h'`` the row before (the
    sequence's kept row ``kept[slot]`` for the first token of the step)."""
    tokens, width = x32.shape
    n = mu.shape[0]
    out = torch.empty((n, tokens, width), dtype=out_dtype, device=x32.device)
    _call("ri_shift_mix", _dev(out, "out"), code(out_dtype), _dev(x32, "x", torch.float32), _dev(kept, "kept", torch.float32),
          _dev(mu, "mu", torch.float32, (n, width)), n, _dev(tok_seq, "tok_seq", torch.int32, (tokens,)),
          _dev(cu_seqlens, "cu_seqlens", torch.int32), _dev(slots, "slots", torch.int32), tokens, width, _stream())
    return out


def tanh_rows(x: torch.Tensor, out_dtype) -> torch.Tensor:
    """``tanh(x)`` of float32 ``x``, taken in float32 and written as ``out_dtype``."""
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    if x.numel():
        _call("ri_tanh_rows", _dev(out, "out"), code(out_dtype), _dev(x, "x", torch.float32), x.numel(), _stream())
    return out


def shift_keep(kept, x32, cu_seqlens, slots) -> None:
    """Every sequence's last row of the step becomes its kept row."""
    seqs = slots.shape[0]
    _call("ri_shift_keep", _dev(kept, "kept", torch.float32), _dev(x32, "x", torch.float32),
          _dev(cu_seqlens, "cu_seqlens", torch.int32, (seqs + 1,)), _dev(slots, "slots", torch.int32), seqs, x32.shape[1], _stream())


def timemix_scan(out, out_off: int, out_scale: float, r, k, v, g, z, w0, u, gain, eps: float, state, cu_seqlens, slots,
                 heads: int, dim: int, columns: bool | None = None) -> None:
    """The walk of the time mixing over every sequence's new tokens on ``state [slots, heads, dim, dim]`` (float32, in
    place); ``r, k, v, g [T, heads * dim]``, ``z`` float32 the decay's pre-activation without its bias ``w0``; the normed and
    gated heads, times ``out_scale``, go to the columns ``out_off ..`` of ``out``.  ``columns``: the form in which a thread holds a
    whole column of the state (heads of up to 128; the default where it fits), else the form that cuts the rows into slices;
    the two differ by rounding alone.  The first form overwrites ``z`` with the decays."""
    tokens, width = r.shape
    seqs = slots.shape[0]
    for name, t in (("k", k), ("v", v), ("g", g)):
        if tuple(t.shape) != (tokens, width) or t.dtype != r.dtype:
            raise ShapeError(f"timemix_scan: {name} is {list(t.shape)} {t.dtype}, r {list(r.shape)} {r.dtype}")
    if width != heads * dim or tuple(state.shape[1:]) != (heads, dim, dim) or out.shape[0] != tokens or out.dtype != r.dtype:
        raise ShapeError(f"timemix_scan: rows of {width}, state {list(state.shape)}, out {list(out.shape)}")
    fits = bool(_get("ri_timemix_scan_cols_fits")(dim))
    if fits if columns is None else (columns and fits):
        o = torch.empty((tokens, width), dtype=torch.float32, device=r.device)
        _call("ri_timemix_scan_cols", _dev(out, "out"), out.shape[1], int(out_off), float(out_scale), _dev(o, "o"), _dev(r, "r"),
              _dev(k, "k"), _dev(v, "v"), _dev(g, "g"), code(r.dtype), _dev(z, "z", torch.float32, (tokens, width)),
              _dev(w0, "w0", torch.float32, (width,)), _dev(u, "u", torch.float32, (width,)),
              _dev(gain, "gain", torch.float32, (width,)), float(eps), _dev(state, "state", torch.float32),
              _dev(cu_seqlens, "cu_seqlens", torch.int32, (seqs + 1,)), _dev(slots, "slots", torch.int32), tokens, seqs, heads, dim,
              _stream())
        return
    _call("ri_timemix_scan", _dev(out, "out"), out.shape[1], int(out_off), float(out_scale), _dev(r, "r"), _dev(k, "k"),
          _dev(v, "v"), _dev(g, "g"), code(r.dtype), _dev(z, "z", torch.float32, (tokens, width)),
          _dev(w0, "w0", torch.float32, (width,)), _dev(u, "u", torch.float32, (width,)),
          _dev(gain, "gain", torch.float32, (width,)), float(eps), _dev(state, "state", torch.float32),
          _dev(cu_seqlens, "cu_seqlens", torch.int32, (seqs + 1,)), _dev(slots, "slots", torch.int32), seqs, heads, dim, _stream())


# ---------------------------------------------------------------- the state-space mixer
SSD_MAX_TAPS = 16


def causal_conv_silu(proj, col0: int, channels: int, taps_w, bias, tails, tok_seq, cu_seqlens, slots) -> torch.Tensor:
    """float32 ``[T, channels]``: ``silu`` of every channel's causal convolution (``taps_w [channels, taps]``, the last
    column the current token's) over the columns ``col0 ..`` of ``proj``, the inputs before a step from ``tails [slots, taps -
    1, channels]``; then the tails are moved on by the step's tokens."""
    tokens = proj.shape[0]
    seqs, taps = slots.shape[0], taps_w.shape[1]
    if tuple(taps_w.shape) != (channels, taps) or (taps > 1 and tuple(tails.shape[1:]) != (taps - 1, channels)):
        raise ShapeError(f"causal_conv_silu: taps {list(taps_w.shape)}, tails {list(tails.shape)} for {channels} channels")
    out = torch.empty((tokens, channels), dtype=torch.float32, device=proj.device)
    for update in (0, 1):
        _call("ri_causal_conv_silu", _dev(out, "out"), _dev(proj, "proj"), code(proj.dtype), proj.shape[1], int(col0),
              _dev(taps_w, "taps", torch.float32), _opt(bias, "bias", torch.float32, (channels,)),
              _opt(tails if taps > 1 else None, "tails", torch.float32), taps, _dev(tok_seq, "tok_seq", torch.int32, (tokens,)),
              _dev(cu_seqlens, "cu_seqlens", torch.int32, (seqs + 1,)), _dev(slots, "slots", torch.int32), tokens, seqs,
              channels, update, _stream())
    return out


def ssd_scan(xbc, b_off: int, c_off: int, proj, z_off: int, dt_off: int, dt_bias, a_log, d_skip, state, cu_seqlens, slots,
             heads: int, groups: int, n: int, vdim: int, columns: bool | None = None) -> torch.Tensor:
    """float32 ``[T, heads * vdim]``: the walk ``S <- exp(-exp(A_log) dt) S + dt B x^T``, ``y = S^T C + D x`` over every
    sequence's new tokens on ``state [slots, heads, n, vdim]`` (float32, in place), times ``silu(z)``; x, B and C are
    columns of ``xbc`` (float32), z and the raw step sizes columns of ``proj``.  ``columns``: the form in which a thread holds a
    whole column of the state (states of up to 128 rows; the default where it fits), else the form that cuts the rows into
    slices; the two differ by rounding alone."""
    tokens, channels = xbc.shape
    seqs = slots.shape[0]
    if tuple(state.shape[1:]) != (heads, n, vdim) or proj.shape[0] != tokens:
        raise ShapeError(f"ssd_scan: state {list(state.shape)} for {heads} heads of {n} x {vdim}")
    out = torch.empty((tokens, heads * vdim), dtype=torch.float32, device=xbc.device)
    fits = bool(_get("ri_ssd_scan_cols_fits")(n, vdim))
    columns = fits if columns is None else (columns and fits)
    _call("ri_ssd_scan_cols" if columns else "ri_ssd_scan", _dev(out, "out"), _dev(xbc, "xbc", torch.float32), channels, int(b_off), int(c_off), _dev(proj, "proj"),
          code(proj.dtype), proj.shape[1], int(z_off), int(dt_off), _opt(dt_bias, "dt_bias", torch.float32, (heads,)),
          _dev(a_log, "a_log", torch.float32, (heads,)), _opt(d_skip, "d_skip", torch.float32, (heads,)),
          _dev(state, "state", torch.float32), _dev(cu_seqlens, "cu_seqlens", torch.int32, (seqs + 1,)),
          _dev(slots, "slots", torch.int32), seqs, heads, groups, n, vdim, _stream())
    return out


def group_rms_norm(x, gain, eps: float, parts: int, out_dtype) -> torch.Tensor:
    """Rows of float32 ``x [T, width]`` in ``parts`` equal parts, each divided by its root mean square, times ``gain``."""
    rows, width = x.shape
    out = torch.empty((rows, width), dtype=out_dtype, device=x.device)
    _call("ri_group_rms_norm", _dev(out, "out"), code(out_dtype), _dev(x, "x", torch.float32),
          _opt(gain, "gain", torch.float32, (width,)), float(eps), rows, width, int(parts), _stream())
    return out
