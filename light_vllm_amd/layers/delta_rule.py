"""Gated delta rule mixer: a linear-attention layer whose state S [D, Dv] per head is decayed,
corrected towards the new value along the new key, and read with the query:

    S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q

with q, k, v from projections that pass a short causal convolution and silu, q and k scaled to unit
length per head (q also by D^-1/2), beta = sigmoid(W_b h), g = exp(-exp(A_log) softplus(W_a h +
dt_bias)); each head's o is RMS-normed over Dv, weighted, gated by silu(W_g h) and projected out.

Serving state per sequence (one slot of the engine's state manager): S in f32 and the last
taps - 1 convolution inputs. A ragged step carries any number of new tokens per sequence from that
state; a sequence without context starts from zeros without the slot being cleared.
All six input projections are one GEMM; everything between it and the output GEMM is four launches
(mix_ops: delta_prep, conv_state_update, gated_delta_rule, head_norm_gate).
"""
from __future__ import annotations

import torch
from torch import nn

from .. import mix_ops
from ..utils.context import get_context
from .linear import MergedColumnParallelLinear, RowParallelLinear
from .tp import tp_size


class GatedDeltaRule(nn.Module):
    uses_state_slots = True

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, conv_taps: int,
                 norm_eps: float = 1e-6, unit_eps: float = 1e-6):
        super().__init__()
        assert tp_size() == 1, "the delta-rule mixer is not sharded: run it with tensor_parallel_size 1"
        assert heads % kv_heads == 0 and conv_taps >= 1
        self.H, self.G, self.D, self.Dv, self.taps = heads, kv_heads, dim, vdim, conv_taps
        self.norm_eps, self.unit_eps = norm_eps, unit_eps
        gd, hv = kv_heads * dim, heads * vdim
        self.channels = 2 * gd + hv                                     # convolution channels: q | k | v
        self.sizes = [gd, gd, hv, hv, heads, heads]                     # q | k | v | gate | b | a
        self.off_gate, self.off_b, self.off_a = self.channels, self.channels + hv, self.channels + hv + heads
        self.in_proj = MergedColumnParallelLinear(width, self.sizes, bias=False)
        self.o_proj = RowParallelLinear(hv, width, bias=False)
        f32 = dict(dtype=torch.float32)
        self.conv_weight = nn.Parameter(torch.zeros(self.channels, conv_taps, **f32))   # last column: current token
        self.A_log = nn.Parameter(torch.zeros(heads, **f32))
        self.dt_bias = nn.Parameter(torch.zeros(heads, **f32))
        self.out_norm_weight = nn.Parameter(torch.ones(vdim, **f32))
        self.conv_state = torch.tensor([])      # [slots, taps-1, channels] act; bound by the runner
        self.state = torch.tensor([])           # [slots, H, D, Dv] f32

    # -- cache protocol of the model runner
    def cache_bytes(self, block_size: int, act_bytes: int) -> tuple[int, int]:
        """(bytes per cache page, bytes per state slot)."""
        return 0, self.H * self.D * self.Dv * 4 + max(self.taps - 1, 1) * self.channels * act_bytes

    def bind_cache(self, num_blocks: int, block_size: int, num_slots: int, device, dtype) -> None:
        self._conv_buf = torch.zeros(num_slots, max(self.taps - 1, 1), self.channels, dtype=dtype, device=device)
        self.conv_state = self._conv_buf[:, :self.taps - 1]      # taps == 1: an empty view that still has an address
        self.state = torch.zeros(num_slots, self.H, self.D, self.Dv, dtype=torch.float32, device=device)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        step = get_context().ragged
        proj = self.in_proj(h)
        qn, kn, v, beta, decay = mix_ops.delta_prep(proj, self.conv_weight, self.conv_state, self.A_log, self.dt_bias,
                                                    step, self.G, self.H, self.D, self.Dv, self.taps, self.off_b,
                                                    self.off_a, self.unit_eps)
        mix_ops.conv_state_update(proj, self.conv_state, step, self.channels, self.taps)
        o = mix_ops.gated_delta_rule(qn, kn, v, beta, decay, self.state, step)
        gate = proj[:, self.off_gate:self.off_gate + self.H * self.Dv]
        y = mix_ops.head_norm_gate(o, gate, self.out_norm_weight, self.norm_eps, h.dtype)
        return self.o_proj(y)
