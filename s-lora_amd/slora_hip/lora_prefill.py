"""Prefill-time operator surface: ``lora_get_qkvo_fwd_shrink`` and
``lora_get_qkvo_fwd_expand`` with the reference's exact positional signatures
(slora/models/peft/triton_kernel/lora/lora_prefill.py:139 and :105), bound to
the segmented gather-GEMM HIP kernels of libslora_hip.so.

Note the argument order: these take ``(b_loc, b_lora_start, b_lora_ranks)``
while ``dispatch_bgmv`` takes ``(start, ranks, loc)``.  ``x``, ``w`` and ``o``
are 2-D and may be row-strided views (the reference passes ``stride(0)`` and
``stride(1)``; a column stride other than 1 is rejected here).
"""
from __future__ import annotations

import ctypes as C

import torch

from . import _cabi
from ._kernels import _DTYPE_CODE, _stream

_F16_BF16 = (torch.float16, torch.bfloat16)


def _check_2d(t, name):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if t.dim() != 2:
        raise RuntimeError(f"{name} must be a 2D tensor")
    if t.size(1) > 1 and t.stride(1) != 1:
        raise RuntimeError(f"{name} must have unit column stride, got {t.stride(1)}")


def _check_1d(t, name, dtype):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if t.dim() != 1 or not t.is_contiguous():
        raise RuntimeError(f"{name} must be a contiguous 1D tensor")
    if t.dtype != dtype:
        raise RuntimeError(f"{name} must be {dtype}, got {t.dtype}")


def _common(x, w, o, b_loc, b_lora_start, b_lora_ranks, b_start_loc, b_seq_len, b_indicies):
    _check_2d(x, "x")
    _check_2d(w, "w")
    _check_2d(o, "o")
    _check_1d(b_loc, "b_loc", torch.int64)
    _check_1d(b_lora_start, "b_lora_start", torch.int64)
    _check_1d(b_lora_ranks, "b_lora_ranks", torch.int64)
    _check_1d(b_indicies, "b_indicies", torch.int64)
    _check_1d(b_start_loc, "b_start_loc", torch.int32)
    _check_1d(b_seq_len, "b_seq_len", torch.int32)
    if x.dtype not in _F16_BF16 or w.dtype != x.dtype or o.dtype != x.dtype:
        raise RuntimeError(f"x, w and o must share a dtype of float16 or bfloat16, got {x.dtype}, {w.dtype}, {o.dtype}")
    if not (b_start_loc.numel() == b_seq_len.numel() == b_indicies.numel()):
        raise RuntimeError("b_start_loc, b_seq_len and b_indicies must have one entry per request")
    if b_lora_start.numel() != b_lora_ranks.numel():
        raise RuntimeError("b_lora_start and b_lora_ranks must have one entry per adapter")
    if x.size(0) != o.size(0):
        raise RuntimeError(f"x and o must have the same number of rows, got {x.size(0)} and {o.size(0)}")
    return _cabi.SloraTables(b_lora_start.data_ptr(), b_lora_ranks.data_ptr(), b_loc.data_ptr(),
                             b_lora_start.numel(), b_loc.numel())


@torch.inference_mode()
def lora_get_qkvo_fwd_shrink(x, w, o, b_loc, b_lora_start, b_lora_ranks, b_start_loc, b_seq_len, b_indicies,
                             hidden_size, qkvo, max_rank, max_input_len) -> None:
    """``o[rows_i, :r] = x[rows_i] @ A_i`` per request i (rows ``b_start_loc[i] +
    [0, b_seq_len[i])``), zeros in columns ``r..max_rank``."""
    tables = _common(x, w, o, b_loc, b_lora_start, b_lora_ranks, b_start_loc, b_seq_len, b_indicies)
    if x.size(1) < hidden_size or w.size(1) < hidden_size or o.size(1) < max_rank:
        raise RuntimeError("x/w narrower than hidden_size or o narrower than max_rank")
    lib = _cabi.load_library()
    rc = lib.slora_sgmm_shrink(o.data_ptr(), x.data_ptr(), w.data_ptr(), C.byref(tables), b_start_loc.data_ptr(),
                               b_seq_len.data_ptr(), b_indicies.data_ptr(), b_seq_len.numel(), int(max_input_len),
                               x.size(0), int(hidden_size), int(max_rank), x.stride(0), w.stride(0), o.stride(0),
                               w.size(0), int(qkvo), _DTYPE_CODE[x.dtype], _stream(x))
    _cabi.check(rc, "lora_get_qkvo_fwd_shrink", f"(hidden_size={hidden_size} max_rank={max_rank} qkvo={qkvo})")


@torch.inference_mode()
def lora_get_qkvo_fwd_expand(x, w, o, scale, b_loc, b_lora_start, b_lora_ranks, b_start_loc, b_seq_len, b_indicies,
                             feat_out, qkvo, max_rank, max_input_len) -> None:
    """``o[rows_i] += (x[rows_i, :r] @ B_i) * scale[a_i]`` per request i."""
    tables = _common(x, w, o, b_loc, b_lora_start, b_lora_ranks, b_start_loc, b_seq_len, b_indicies)
    if not isinstance(scale, torch.Tensor) or not scale.is_cuda or not scale.is_contiguous():
        raise RuntimeError("scale must be a contiguous CUDA tensor")
    if scale.dtype not in _DTYPE_CODE:
        raise RuntimeError(f"scale must be float16, bfloat16 or float32, got {scale.dtype}")
    if scale.numel() < b_lora_start.numel():
        raise RuntimeError("scale must have one entry per adapter")
    if o.size(1) < feat_out or x.size(1) < max_rank:
        raise RuntimeError("o narrower than feat_out or x narrower than max_rank")
    lib = _cabi.load_library()
    rc = lib.slora_sgmm_expand(o.data_ptr(), x.data_ptr(), w.data_ptr(), C.byref(tables), scale.data_ptr(),
                               _DTYPE_CODE[scale.dtype], b_start_loc.data_ptr(), b_seq_len.data_ptr(),
                               b_indicies.data_ptr(), b_seq_len.numel(), int(max_input_len), x.size(0),
                               int(feat_out), w.size(1), int(max_rank), x.stride(0), w.stride(0), o.stride(0),
                               w.size(0), int(qkvo), _DTYPE_CODE[x.dtype], _stream(x))
    _cabi.check(rc, "lora_get_qkvo_fwd_expand", f"(feat_out={feat_out} max_rank={max_rank} qkvo={qkvo})")
