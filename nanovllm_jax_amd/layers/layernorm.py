"""RMSNorm, optionally fused with the residual add.

Host-side mirror of the reference's ``RMSNorm`` (``layers/layernorm.py:11-90``):
``RMSNorm(hidden, eps)(x)`` returns the normalised tensor,
``RMSNorm(hidden, eps)(x, residual)`` returns ``(normalised, new_residual)``.
Both run as one launch of ``nvj_add_rms_norm_launch``; there is no CPU
implementation.
"""
from __future__ import annotations

import torch

from .. import _lib

__all__ = ["rms_norm", "RMSNorm"]


def _require(cond: bool, msg: str) -> None:
    if not cond:
        raise ValueError(msg)


def rms_norm(x, weight, eps, residual=None, out=None, residual_out=None):
    """``x`` and ``residual`` ``[..., hidden]`` bf16, ``weight`` ``[hidden]`` float32.

    Without ``residual``: returns ``bf16(x * rsqrt(mean(x^2) + eps) * weight)``.
    With it: ``s = float(x) + float(residual)``; returns ``(bf16(s * rsqrt(mean(s^2)
    + eps) * weight), bf16(s))`` (``layers/layernorm.py:50-79``).  ``residual_out``
    may be ``residual`` itself (updated in place).
    """
    lib = _lib.load()
    tensors = [("x", x), ("weight", weight)]
    if residual is not None:
        tensors.append(("residual", residual))
    for name, t in tensors:
        _require(isinstance(t, torch.Tensor), f"{name} must be a torch.Tensor")
        _require(t.is_cuda, f"{name} must live on the GPU (got {t.device}); "
                            "this op has no CPU implementation")
        _require(t.device == x.device, f"{name} is on {t.device}, x on {x.device}")
    _require(x.dtype == torch.bfloat16, f"x must be bfloat16, got {x.dtype}")
    _require(weight.dtype == torch.float32, f"weight must be float32, got {weight.dtype}")
    _require(x.dim() >= 1 and x.is_contiguous(), "x must be contiguous")
    hidden = x.shape[-1]
    _require(weight.shape == (hidden,) and weight.is_contiguous(),
             f"weight must be [{hidden}] contiguous")
    if residual is not None:
        _require(residual.dtype == torch.bfloat16 and residual.shape == x.shape
                 and residual.is_contiguous(), "residual must match x (bf16, contiguous)")
    num_tokens = x.numel() // hidden if hidden else 0
    y = torch.empty_like(x) if out is None else out
    _require(y.shape == x.shape and y.dtype == x.dtype and y.is_contiguous()
             and y.device == x.device, "out must match x")
    r_out = None
    if residual is not None:
        r_out = torch.empty_like(x) if residual_out is None else residual_out
        _require(r_out.shape == x.shape and r_out.dtype == x.dtype and r_out.is_contiguous()
                 and r_out.device == x.device, "residual_out must match x")
    with torch.cuda.device(x.device):
        stream = torch.cuda.current_stream().cuda_stream
        _lib.check(lib.nvj_add_rms_norm_launch(
            stream, x.data_ptr(), residual.data_ptr() if residual is not None else None,
            weight.data_ptr(), float(eps), y.data_ptr(),
            r_out.data_ptr() if r_out is not None else None, num_tokens, hidden),
            "nvj_add_rms_norm_launch")
    return y if residual is None else (y, r_out)


class RMSNorm:
    """``RMSNorm(hidden_size, eps)``; ``weight`` is a float32 tensor of ones until
    assigned (``layers/layernorm.py:22-29``)."""

    def __init__(self, hidden_size: int, eps: float = 1e-6, device=None):
        self.eps = eps
        self.weight = torch.ones(hidden_size, dtype=torch.float32, device=device)

    def __call__(self, x, residual=None):
        return rms_norm(x, self.weight, self.eps, residual)
