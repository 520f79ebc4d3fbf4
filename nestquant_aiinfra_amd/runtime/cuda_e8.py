"""Stand-alone E8 projection under the reference's names (nestquant/runtime/cuda_e8.py:13-43),
over the library's nq_e8_nearest.  Unlike the reference's extension, which launches on the
default stream (nestquant/runtime/cuda_e8.cu:55), this one uses the current stream."""

from __future__ import annotations

import torch

from .. import _native


def cuda_e8_available() -> bool:
    """Whether a GPU and the HIP library are there to run e8_nearest_cuda."""
    return bool(torch.cuda.is_available()) and _native.LIBRARY_PATH.exists()


def e8_nearest_cuda(x: torch.Tensor) -> torch.Tensor:
    """Project a ``[N, 8]`` float32 GPU tensor onto E8 (ties go to the half-integer coset)."""
    if not isinstance(x, torch.Tensor) or not x.is_cuda:
        raise ValueError("x must be a CUDA tensor")
    if x.dtype != torch.float32 or x.ndim != 2 or x.shape[1] != 8:
        raise ValueError("x must have dtype float32 and shape [N, 8]")
    points = x.contiguous()
    out = torch.empty_like(points)
    if points.shape[0]:
        _native.check(_native.library().nq_e8_nearest(points.data_ptr(), out.data_ptr(), points.shape[0],
                                                      _native.stream_handle(points.device)))
    return out
