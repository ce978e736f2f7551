"""RMSNorm module (reference lit_gpt/rmsnorm.py:6-28) backed by the ``lga_rmsnorm`` HIP kernel."""

from __future__ import annotations

import torch
import torch.nn as nn

from lit_gpt import ops


def _gpu_only(what: str) -> None:
    raise RuntimeError(f"{what}: this build computes on the MI355X only (no CPU path); move the model to 'cuda'")


class RMSNorm(nn.Module):
    """lit_gpt/rmsnorm.py:6-28 on the GPU (``lga_rmsnorm``): fp32 math, one cast back to bf16."""

    def __init__(self, size: int, dim: int = -1, eps: float = 1e-5) -> None:
        super().__init__()
        self.weight = nn.Parameter(torch.ones(size))
        self.eps = eps
        self.dim = dim

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if not x.is_cuda:
            _gpu_only("RMSNorm")
        return ops.rmsnorm(x.contiguous(), self.weight, self.eps)

    def reset_parameters(self) -> None:
        torch.nn.init.ones_(self.weight)


class StreamRMSNorm(nn.Module):
    """RMS norm over rows of the fp32 residual stream (``lgs_rmsnorm``): x / sqrt(mean(x^2) + eps) * (offset + w).
    ``offset`` 1.0 serves checkpoints whose norm weight is stored around zero, 0.0 the plain weight; the weight is
    kept in fp32 whatever the model's compute dtype."""

    def __init__(self, size: int, eps: float = 1e-5, offset: float = 0.0) -> None:
        super().__init__()
        self.register_buffer("weight", torch.zeros(size) if offset else torch.ones(size))
        self.eps, self.offset = eps, offset

    def forward(self, x: torch.Tensor, bf16_copy: bool = False):
        """``bf16_copy``: (y, y rounded to bf16) — the second is what a bf16 MFMA product reads."""
        from lit_gpt import seq_ops

        if not x.is_cuda:
            _gpu_only("StreamRMSNorm")
        return seq_ops.rmsnorm(x, self.weight, offset=self.offset, eps=self.eps, bf16_copy=bf16_copy)
