"""Small tensor helpers shared by the HIP operator wrappers."""
from __future__ import annotations

import torch

from .. import _lib


def dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return _lib.F32
    if t.dtype == torch.bfloat16:
        return _lib.BF16
    if t.dtype == torch.float16:
        return _lib.F16
    raise TypeError(f"unsupported dtype {t.dtype}: the HIP kernels take float32, bfloat16 or float16 tensors")


def state_dtype_code(t: torch.Tensor) -> int:
    """dtype code of a recurrent state tensor (float32, bfloat16 or float16)."""
    return dtype_code(t)


def ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


def require_gpu(*tensors: torch.Tensor) -> torch.device:
    dev = tensors[0].device
    if dev.type != "cuda":
        raise RuntimeError(
            "the 'hip' mLSTM kernels run on an AMD GPU only (got a tensor on "
            f"'{dev}'); there is no CPU fallback in mlstm_kernels_amd"
        )
    for t in tensors:
        if t is not None and t.device != dev:
            raise RuntimeError("all tensors must be on the same device")
    return dev


def current_stream_ptr(dev: torch.device) -> int:
    return torch.cuda.current_stream(dev).cuda_stream
