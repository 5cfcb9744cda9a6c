"""SwiGLU: silu(gate) * up over the two halves of the last dim (reference "native" backend,
lightvllm/layers/activation.py:7-29), and the clamped gated unit with a sigmoid of slope alpha."""
import torch
import torch.nn.functional as F
from torch import nn

from .. import mix_ops, ops
from .fused import use_fused


class SiluAndMul(nn.Module):

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if use_fused(x):
            return ops.silu_and_mul(x)
        gate, up = torch.chunk(x, 2, dim=-1)
        return F.silu(gate) * up


class ClampedGLU(nn.Module):
    """min(g, L) * sigmoid(alpha * g) * (clamp(u, -L, L) + 1) over [gate | up] halves of the last dim."""

    def __init__(self, limit: float, alpha: float = 1.702):
        super().__init__()
        self.limit, self.alpha = float(limit), float(alpha)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return mix_ops.clamped_glu(x, self.limit, self.alpha)
