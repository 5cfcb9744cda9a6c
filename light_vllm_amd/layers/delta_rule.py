"""Gated delta rule mixer: a linear-attention layer whose state S [D, Dv] per head is decayed,
corrected towards the new value along the new key, and read with the query:

    S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q

with q, k, v from projections that pass a short causal convolution and silu, q and k scaled to unit
length per head (q also by D^-1/2), beta = sigmoid(W_b h), g = exp(-exp(A_log) softplus(a + dt_bias));
each head's o is RMS-normed over Dv, weighted, gated and projected out.

Variants, chosen by the constructor:
  * decay="head": one g per head, a = W_a h (H numbers); decay="channel": every key channel of a
    head has a g of its own, which scales its row of S (a and dt_bias are H*D wide, A_log stays per head);
  * decay_rank / gate_rank: a (the gate) is a product of two thin matrices, W_2 (W_1 h), instead of
    one projection; the first factors ride in the fused input GEMM;
  * gate_act: the output gate is silu or sigmoid of its projection.

Serving state per sequence (one slot of the engine's state manager): S in f32 and the last
taps - 1 convolution inputs. A ragged step carries any number of new tokens per sequence from that
state; a sequence without context starts from zeros without the slot being cleared.
All input projections are one GEMM; everything between it and the output GEMM is four launches
(mix_ops: delta_prep, conv_state_update, gated_delta_rule, head_norm_gate) and the thin second factors.
"""
from __future__ import annotations

import torch
from torch import nn

from .. import mix_ops
from ..utils.context import get_context
from .linear import ColumnParallelLinear, MergedColumnParallelLinear, RowParallelLinear
from .tp import tp_size


class GatedDeltaRule(nn.Module):
    uses_state_slots = True

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, conv_taps: int,
                 norm_eps: float = 1e-6, unit_eps: float = 1e-6, decay: str = "head", decay_rank: int | None = None,
                 gate_rank: int | None = None, gate_act: str = "silu", share: "GatedDeltaRule | None" = None):
        super().__init__()
        assert tp_size() == 1, "the delta-rule mixer is not sharded: run it with tensor_parallel_size 1"
        assert heads % kv_heads == 0 and conv_taps >= 1 and decay in ("head", "channel") and gate_act in ("silu", "sigmoid")
        self.H, self.G, self.D, self.Dv, self.taps = heads, kv_heads, dim, vdim, conv_taps
        self.norm_eps, self.unit_eps, self.gate_act = norm_eps, unit_eps, gate_act
        self.decay_per_channel = decay == "channel"
        gd, hv = kv_heads * dim, heads * vdim
        decay_width = heads * dim if self.decay_per_channel else heads
        self.channels = 2 * gd + hv                                     # convolution channels: q | k | v
        gate_in = gate_rank if gate_rank is not None else hv
        decay_in = decay_rank if decay_rank is not None else decay_width
        self.sizes = [gd, gd, hv, gate_in, heads, decay_in]             # q | k | v | gate (or its first factor) | b | a (or its first factor)
        self.off_gate, self.off_b, self.off_a = self.channels, self.channels + gate_in, self.channels + gate_in + heads
        self.gate_in, self.decay_in = gate_in, decay_in
        if share is None:
            f32 = dict(dtype=torch.float32)
            self.in_proj = MergedColumnParallelLinear(width, self.sizes, bias=False)
            self.gate_up = ColumnParallelLinear(gate_rank, hv, bias=False) if gate_rank is not None else None
            self.decay_up = ColumnParallelLinear(decay_rank, decay_width, bias=False) if decay_rank is not None else None
            self.o_proj = RowParallelLinear(hv, width, bias=False)
            self.conv_weight = nn.Parameter(torch.zeros(self.channels, conv_taps, **f32))   # last column: current token
            self.A_log = nn.Parameter(torch.zeros(heads, **f32))
            self.dt_bias = nn.Parameter(torch.zeros(decay_width, **f32))
            self.out_norm_weight = nn.Parameter(torch.ones(vdim, **f32))
        else:       # the same weights as another layer; the state is this layer's own
            assert share.sizes == self.sizes and share.taps == conv_taps
            self.in_proj, self.gate_up, self.decay_up, self.o_proj = share.in_proj, share.gate_up, share.decay_up, share.o_proj
            self.conv_weight, self.A_log, self.dt_bias = share.conv_weight, share.A_log, share.dt_bias
            self.out_norm_weight = share.out_norm_weight
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
        a = proj[:, self.off_a:self.off_a + self.decay_in]
        if self.decay_up is not None:
            a = self.decay_up(a)
        qn, kn, v, beta, decay = mix_ops.delta_prep(proj, self.conv_weight, self.conv_state, self.A_log, self.dt_bias,
                                                    step, self.G, self.H, self.D, self.Dv, self.taps, self.off_b, a,
                                                    self.unit_eps, self.decay_per_channel)
        mix_ops.conv_state_update(proj, self.conv_state, step, self.channels, self.taps)
        o = mix_ops.gated_delta_rule(qn, kn, v, beta, decay, self.state, step)
        gate = proj[:, self.off_gate:self.off_gate + self.gate_in]
        if self.gate_up is not None:
            gate = self.gate_up(gate)
        y = mix_ops.head_norm_gate(o, gate, self.out_norm_weight, self.norm_eps, h.dtype, self.gate_act)
        return self.o_proj(y)
