"""Sliding-window attention whose far past is kept as pooled blocks.

Position i sees the tokens j with 0 <= i - j < window and, for every block of `pool` tokens that lies
wholly before the window (b * pool + pool - 1 <= i - window), one key and one value: the means of the
block's cached keys and values. Tokens that have left the window while their block is not yet
wholly outside are not seen. Tokens and blocks share one softmax, optionally with a sink (a term of
score 0 and no value, i.e. 1 added to the denominator). No positional rotation: the scores do not
depend on positions. Options used by the models: RMS norm over the whole q and k projections before
the split into heads, a sigmoid output gate from the layer input, separate key and value head sizes.

Cache: the engine's pages hold K and V rows of all tokens ([pages, page, G, D] / [.., Dv]); the
pooled entries live in two companion tensors indexed by the same page ids (a block is stored with
the page of its last token), so one block table serves both and pages are freed together.
Three launches between the input GEMM and the output GEMM (mix_ops: qk_fullnorm_store, pool_update,
window_pool_attention).
"""
from __future__ import annotations

import torch
from torch import nn

from .. import mix_ops
from ..utils.context import get_context
from .linear import MergedColumnParallelLinear, RowParallelLinear
from .tp import tp_size


class WindowPoolAttention(nn.Module):
    uses_pages = True

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, window: int, pool: int,
                 scale: float, norm_eps: float = 1e-6, sink: bool = True, gated: bool = True):
        super().__init__()
        assert tp_size() == 1, "the windowed pooled attention is not sharded: run it with tensor_parallel_size 1"
        assert heads % kv_heads == 0 and window >= 1 and pool >= 0
        self.H, self.G, self.D, self.Dv = heads, kv_heads, dim, vdim
        self.window, self.pool, self.scale, self.norm_eps, self.sink, self.gated = window, pool, scale, norm_eps, sink, gated
        self.sizes = [heads * dim, kv_heads * dim, kv_heads * vdim] + ([heads * vdim] if gated else [])
        self.in_proj = MergedColumnParallelLinear(width, self.sizes, bias=False)     # q | k | v | gate
        self.o_proj = RowParallelLinear(heads * vdim, width, bias=False)
        f32 = dict(dtype=torch.float32)
        self.q_norm_weight = nn.Parameter(torch.ones(heads * dim, **f32))
        self.k_norm_weight = nn.Parameter(torch.ones(kv_heads * dim, **f32))
        self.k_cache = self.v_cache = self.k_pool = self.v_pool = torch.tensor([])

    def cache_bytes(self, block_size: int, act_bytes: int) -> tuple[int, int]:
        rows = block_size + mix_ops.pooled_slots(block_size, self.pool)
        return rows * self.G * (self.D + self.Dv) * act_bytes, 0

    def bind_cache(self, num_blocks: int, block_size: int, num_slots: int, device, dtype) -> None:
        pp = max(mix_ops.pooled_slots(block_size, self.pool), 1)
        kw = dict(dtype=dtype, device=device)
        self.k_cache = torch.zeros(num_blocks, block_size, self.G, self.D, **kw)
        self.v_cache = torch.zeros(num_blocks, block_size, self.G, self.Dv, **kw)
        self.k_pool = torch.zeros(num_blocks, pp, self.G, self.D, **kw)
        self.v_pool = torch.zeros(num_blocks, pp, self.G, self.Dv, **kw)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        step = get_context().ragged
        proj = self.in_proj(h)
        a, b, c = self.sizes[0], self.sizes[0] + self.sizes[1], self.sizes[0] + self.sizes[1] + self.sizes[2]
        q = mix_ops.qk_fullnorm_store(proj[:, :a], proj[:, a:b], proj[:, b:c], self.q_norm_weight, self.k_norm_weight,
                                      self.k_cache, self.v_cache, step, self.H, self.G, self.D, self.Dv, self.norm_eps)
        mix_ops.pool_update(self.k_cache, self.v_cache, self.k_pool, self.v_pool, step, self.G, self.D, self.Dv, self.pool)
        gate = proj[:, c:] if self.gated else None
        o = mix_ops.window_pool_attention(q, self.k_cache, self.v_cache, self.k_pool, self.v_pool, gate, step, self.H,
                                          self.G, self.D, self.Dv, self.window, self.pool, self.scale, self.sink)
        return self.o_proj(o)
