"""Hyper-connections: S parallel residual streams instead of one.

A sublayer reads u = sum_s in[s] x_s, and its output y comes back as
x_t <- sum_s mix[s, t] x_s + out[t] * y for all streams at once (mix indexed [from, to]); the
model's result is the sum of the streams. With S = 1, in = out = mix = 1 this is the plain pre-norm
residual. Streams and the three small parameter tensors are f32 whatever the activation dtype.

`advance` is the one device step between two sublayers: the update for the sublayer that has just
run fused with the read-out and grouped RMS norm for the one that runs next (mix_ops.hc_update_norm).
"""
from __future__ import annotations

import torch
from torch import nn

from .. import mix_ops


class HyperConnection(nn.Module):
    """Parameters of one sublayer's connection to the streams."""

    def __init__(self, streams: int):
        super().__init__()
        f32 = dict(dtype=torch.float32)
        self.streams = streams
        self.read = nn.Parameter(torch.ones(streams, **f32))           # in[s]
        self.write = nn.Parameter(torch.ones(streams, **f32))          # out[t]
        self.mix = nn.Parameter(torch.eye(streams, **f32))             # mix[from, to]


class GroupedRMSNorm(nn.Module):
    """RMS norm in `groups` equal consecutive parts of the vector, each divided by its own
    sqrt(mean(part^2) + eps), then one weight over the whole vector. f32 weight."""

    def __init__(self, hidden_size: int, groups: int = 1, eps: float = 1e-6):
        super().__init__()
        assert hidden_size % groups == 0, f"{groups} norm groups do not divide {hidden_size}"
        self.hidden_size, self.groups, self.eps = hidden_size, groups, eps
        self.weight = nn.Parameter(torch.ones(hidden_size, dtype=torch.float32))


def open_streams(embedded: torch.Tensor, streams: int) -> torch.Tensor:
    """[T, W] activations -> [T, S, W] f32 streams, every stream a copy of the embedding output."""
    return embedded.float().unsqueeze(1).repeat(1, streams, 1)


def advance(x: torch.Tensor, y, done: HyperConnection | None, nxt_read: torch.Tensor | None,
            nxt_norm: GroupedRMSNorm | None, act_dtype) -> torch.Tensor | None:
    """Write sublayer output y back through `done` (None: nothing to write, the first read-out), then
    read out and norm for the next sublayer (nxt_read None: no read-out)."""
    return mix_ops.hc_update_norm(
        x, y,
        done.mix if done is not None else None, done.write if done is not None else None,
        nxt_read, nxt_norm.weight if nxt_norm is not None else None,
        nxt_norm.groups if nxt_norm is not None else 1, nxt_norm.eps if nxt_norm is not None else 0.0,
        act_dtype)
