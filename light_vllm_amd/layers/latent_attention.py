"""Latent attention: keys and values of all heads are up-projections of one small latent vector per
token, and only that latent (plus, optionally, one rotated positional key part shared by all heads)
is cached.

    c_q = rms_norm(W_dq h) * w_q          q_h = W_uq,h c_q            = [q_h^n (dim) | q_h^r (rot_dim)]
    [c' | k^r'] = W_dkv h                 c = rms_norm(c') * w_kv     k^r = rotate(k^r', position)
    k_h = W_uk,h c,   v_h = W_uv,h c      score_h(i, j) = (q_h^n(i) . k_h(j) + rotate(q_h^r(i)) . k^r(j)) * scale
    o_h = softmax_j<=i(score_h) v_h,      y = W_o [gate_h * o_h]_h,   gate = sigmoid(W_g h)

Served in the absorbed form: q_h^n . (W_uk,h c) = (W_uk,h^T q_h^n) . c, and sum_j p_j W_uv,h c_j =
W_uv,h sum_j p_j c_j, so every head attends to the cached rows [c | k^r] themselves (keys: the whole
row, values: its first kv_rank entries) and the per-head matrices act on queries and outputs only,
as two batched GEMMs. A decoded token therefore reads kv_rank + rot_dim numbers per cached token
instead of heads * (dim + vdim), and one attention kernel serves prompts, portions and single tokens:
the paged windowed kernel with one kv head, a window no sequence reaches, no pooled blocks and no sink.

The output gate is one number per head (`gate="head"`) or one per output channel (`gate="channel"`).
Rotation: the first rot_dims entries of the rot_dim-wide positional part, entries i and i + rot_dims/2
form a pair, angle = position * base^(-2i/rot_dims); rot_dim = 0 gives position-free attention.
"""
from __future__ import annotations

import torch
from torch import nn

from .. import mix_ops
from ..utils.context import get_context
from .linear import ColumnParallelLinear, MergedColumnParallelLinear, RowParallelLinear
from .tp import tp_size

NO_WINDOW = 1 << 30       # a window no sequence reaches: plain causal attention


class LatentAttention(nn.Module):
    uses_pages = True

    def __init__(self, width: int, heads: int, dim: int, vdim: int, q_rank: int, kv_rank: int, scale: float,
                 rot_dim: int = 0, rot_dims: int = 0, rot_base: float = 10000.0, gate: str = "head",
                 norm_eps: float = 1e-6, share: "LatentAttention | None" = None):
        super().__init__()
        assert tp_size() == 1, "latent attention is not sharded: run it with tensor_parallel_size 1"
        assert gate in ("head", "channel") and 0 <= rot_dims <= rot_dim and rot_dims % 2 == 0
        self.H, self.Dn, self.Dr, self.Dv, self.Rq, self.R = heads, dim, rot_dim, vdim, q_rank, kv_rank
        self.rot_dims, self.rot_base, self.scale, self.norm_eps = rot_dims, float(rot_base), float(scale), norm_eps
        self.gate_per_channel = gate == "channel"
        self.sizes = [q_rank, kv_rank + rot_dim, heads * vdim if self.gate_per_channel else heads]   # dq | dkv | gate
        if share is None:
            f32 = dict(dtype=torch.float32)
            self.in_proj = MergedColumnParallelLinear(width, self.sizes, bias=False)
            self.uq = ColumnParallelLinear(q_rank, heads * (dim + rot_dim), bias=False)
            self.uk = nn.Parameter(torch.empty(heads, dim, kv_rank))        # W_uk per head, [dim, kv_rank]
            self.uv = nn.Parameter(torch.empty(heads, vdim, kv_rank))       # W_uv per head, [vdim, kv_rank]
            self.o_proj = RowParallelLinear(heads * vdim, width, bias=False)
            self.q_norm_weight = nn.Parameter(torch.ones(q_rank, **f32))
            self.kv_norm_weight = nn.Parameter(torch.ones(kv_rank, **f32))
        else:       # the same weights as another layer; cache and position in the model are this layer's own
            assert (share.sizes, share.H, share.Dn, share.Dr, share.Dv) == (self.sizes, heads, dim, rot_dim, vdim)
            self.in_proj, self.uq, self.uk, self.uv, self.o_proj = share.in_proj, share.uq, share.uk, share.uv, share.o_proj
            self.q_norm_weight, self.kv_norm_weight = share.q_norm_weight, share.kv_norm_weight
        self.inv_freq = None          # f32 [rot_dims/2], made with the cache
        self.cache = torch.tensor([])  # [pages, page, kv_rank + rot_dim]; bound by the runner

    # -- cache protocol of the model runner
    def cache_bytes(self, block_size: int, act_bytes: int) -> tuple[int, int]:
        return block_size * (self.R + self.Dr) * act_bytes, 0

    def bind_cache(self, num_blocks: int, block_size: int, num_slots: int, device, dtype) -> None:
        self.cache = torch.zeros(num_blocks, block_size, self.R + self.Dr, dtype=dtype, device=device)
        self.inv_freq = mix_ops.rotary_inv_freq(max(self.rot_dims, 2), self.rot_base, device)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        step = get_context().ragged
        T, H, R, Dn, Dr = h.size(0), self.H, self.R, self.Dn, self.Dr
        proj = self.in_proj(h)
        cq = mix_ops.latent_prep(proj, 0, self.Rq, self.q_norm_weight, self.kv_norm_weight, self.inv_freq, self.cache,
                                 step, self.Rq, R, Dr, self.rot_dims, self.norm_eps)
        q = self.uq(cq)
        q_lat = torch.bmm(q.view(T, H, Dn + Dr)[:, :, :Dn].transpose(0, 1), self.uk)              # [H, T, R]
        q_abs = mix_ops.latent_q_finish(q, q_lat, self.inv_freq, step, H, Dn, Dr, R, self.rot_dims)
        rows = self.cache.unsqueeze(2)                                                              # [pages, page, 1, R + Dr]
        o_lat = mix_ops.window_pool_attention(q_abs, rows, rows[..., :R], None, None, None, step, H, 1, R + Dr, R,
                                              NO_WINDOW, 0, self.scale, has_sink=False)
        o = torch.bmm(o_lat.view(T, H, R).transpose(0, 1), self.uv.transpose(1, 2))                 # [H, T, Dv]
        gate = proj[:, self.sizes[0] + self.sizes[1]:]
        return self.o_proj(mix_ops.latent_out_gate(o, gate, self.gate_per_channel))
