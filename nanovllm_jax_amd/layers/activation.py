"""SiLU-and-multiply of the fused gate/up projection.

Host-side mirror of the reference's ``SiluAndMul`` (``layers/activation.py:12-33``):
the first half of the last dimension is the gate, the second half the up
projection; one launch of ``nvj_silu_and_mul_launch``, no CPU implementation.
"""
from __future__ import annotations

import torch

from .. import _lib

__all__ = ["silu_and_mul", "SiluAndMul"]


def _require(cond: bool, msg: str) -> None:
    if not cond:
        raise ValueError(msg)


def silu_and_mul(x, out=None):
    """``x`` ``[..., 2 * intermediate]`` bf16 -> ``[..., intermediate]`` bf16 =
    ``silu(x[..., :intermediate]) * x[..., intermediate:]``."""
    lib = _lib.load()
    _require(isinstance(x, torch.Tensor), "x must be a torch.Tensor")
    _require(x.is_cuda, f"x must live on the GPU (got {x.device}); this op has no CPU "
                        "implementation")
    _require(x.dtype == torch.bfloat16, f"x must be bfloat16, got {x.dtype}")
    _require(x.dim() >= 1 and x.shape[-1] % 2 == 0 and x.is_contiguous(),
             "x must be contiguous with an even last dimension")
    inter = x.shape[-1] // 2
    num_tokens = x.numel() // (2 * inter) if inter else 0
    shape = tuple(x.shape[:-1]) + (inter,)
    y = torch.empty(shape, dtype=x.dtype, device=x.device) if out is None else out
    _require(tuple(y.shape) == shape and y.dtype == x.dtype and y.is_contiguous()
             and y.device == x.device, "out must be [..., intermediate] bf16 on x's device")
    with torch.cuda.device(x.device):
        stream = torch.cuda.current_stream().cuda_stream
        _lib.check(lib.nvj_silu_and_mul_launch(stream, x.data_ptr(), 2 * inter, y.data_ptr(),
                                               num_tokens, inter),
                   "nvj_silu_and_mul_launch")
    return y


class SiluAndMul:
    def __call__(self, x):
        return silu_and_mul(x)
