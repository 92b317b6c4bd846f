"""Argument checks shared by the ops: same conditions and ``RuntimeError`` as the reference's
CHECK_INPUT / CHECK_DIM macros (csrc/src/pytorch_extension_utils.h:220-239)."""
from __future__ import annotations

import torch

from .._lib import TWL_BF16, TWL_F16, TWL_F32


def check_cuda(x: torch.Tensor, name: str) -> None:
    if not isinstance(x, torch.Tensor):
        raise RuntimeError(f"{name} must be a torch.Tensor")
    if not x.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")


def check_contiguous(x: torch.Tensor, name: str) -> None:
    if not x.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")


def check_input(x: torch.Tensor, name: str) -> None:
    check_cuda(x, name)
    check_contiguous(x, name)


def check_dim(d: int, x: torch.Tensor, name: str) -> None:
    if x.dim() != d:
        raise RuntimeError(f"{name} must be a {d}D tensor")


def check_dtype(x: torch.Tensor, dtype: torch.dtype, name: str) -> None:
    if x.dtype != dtype:
        raise RuntimeError(f"{name} must have dtype {dtype}, got {x.dtype}")


def check_same_device(ref: torch.Tensor, *others) -> None:
    for name, t in others:
        if t is not None and t.device != ref.device:
            raise RuntimeError(f"{name} must be on {ref.device}, got {t.device}")


def dtype_code(dt: torch.dtype, name: str) -> int:
    if dt == torch.float16:
        return TWL_F16
    if dt == torch.bfloat16:
        return TWL_BF16
    if dt == torch.float32:
        return TWL_F32
    raise RuntimeError(f"{name}: unsupported dtype {dt}")


def ptr(x) -> int:
    return 0 if x is None else x.data_ptr()


def stream_of(x: torch.Tensor) -> int:
    """The current stream of ``x``'s device (kernel/cuda/sampling.py:78,98 pass the same)."""
    return torch.cuda.current_stream(x.device).cuda_stream
