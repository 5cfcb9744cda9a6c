"""Kagalorn: a decoder-only model of delta-rule and windowed-attention layers on hyper-connected
residual streams.

config.json (`architecture: "Kagalorn"`) lists the layers; each names its mixer type ("delta": gated
delta rule with short convolutions, "attention": sliding window with pooled blocks, sink softmax,
whole-projection q/k norm and an output gate), the mixer's sizes and its feed-forward (a dense
clamped gated unit, or none). Every sublayer is pre-normed in groups and tied to `streams` residual
streams by its own hyper-connection; the model ends with the grouped norm of the summed streams and
the output head. Sizes, layer order and constants all come from the config; nothing here assumes a
particular model.

The model runs ragged steps only (utils.context.RaggedStep): prompts, portions of prompts and single
decoded tokens are one code path, from the paged K/V cache and the per-sequence state slot.
Checkpoint tensors: embed, head, final.norm, l<i>.norm1|norm2, l<i>.hc1|hc2.in|out|mix,
l<i>.mix.* and l<i>.mlp.gate|up|down, linear weights stored [out, in].
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import Any, Optional

import torch
from torch import nn

from ..layers.activation import ClampedGLU
from ..layers.delta_rule import GatedDeltaRule
from ..layers.embed_head import ParallelLMHead, VocabParallelEmbedding
from ..layers.hyper_connections import GroupedRMSNorm, HyperConnection, advance, open_streams
from ..layers.linear import MergedColumnParallelLinear, RowParallelLinear
from ..layers.window_pool_attention import WindowPoolAttention

GLU_ALPHA = 1.702          # slope of the sigmoid in the feed-forward gate
UNIT_NORM_EPS = 1e-6       # inside the root of the delta rule's unit norms


@dataclass
class KagalornConfig:
    """config.json of a Kagalorn checkpoint. Attribute names the engine reads from any model config
    (vocab_size, hidden_size, max_position_embeddings, torch_dtype) are provided as well."""
    vocab: int
    width: int
    streams: int
    norm_eps: float
    norm_groups: int
    layers: list = field(default_factory=list)
    torch_dtype: Any = torch.bfloat16
    max_position_embeddings: int = 1 << 30       # no positional table: any length the cache holds
    architectures: tuple = ("Kagalorn",)

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, d: dict) -> "KagalornConfig":
        for key in ("vocab", "width", "layers", "norm"):
            if key not in d:
                raise ValueError(f"Kagalorn config lacks '{key}'")
        layers = []
        for i, L in enumerate(d["layers"]):
            kind, m = L["type"], dict(L["mixer"])
            if kind == "delta":
                need = ("heads", "kv_heads", "dim", "vdim", "conv")
            elif kind == "attention":
                need = ("heads", "kv_heads", "dim", "vdim", "scale", "mask")
            else:
                raise ValueError(f"layer {i}: unknown mixer type '{kind}'")
            missing = [k for k in need if k not in m]
            if missing:
                raise ValueError(f"layer {i} ({kind}): mixer lacks {missing}")
            mlp = L.get("mlp")
            if mlp is not None and mlp.get("kind", "dense") != "dense":
                raise ValueError(f"layer {i}: unknown feed-forward kind '{mlp.get('kind')}'")
            layers.append({"type": kind, "mixer": m, "mlp": dict(mlp) if mlp is not None else None})
        return cls(vocab=int(d["vocab"]), width=int(d["width"]), streams=int(d.get("streams", 1)),
                   norm_eps=float(d["norm"]["eps"]), norm_groups=int(d["norm"].get("groups", 1)), layers=layers)

    @classmethod
    def from_pretrained(cls, path: str) -> "KagalornConfig":
        with open(os.path.join(path, "config.json")) as f:
            return cls.from_dict(json.load(f))


class ClampedGLUMLP(nn.Module):

    def __init__(self, width: int, ff: int, limit: float):
        super().__init__()
        self.gate_up_proj = MergedColumnParallelLinear(width, [ff, ff], bias=False)
        self.down_proj = RowParallelLinear(ff, width, bias=False)
        self.act_fn = ClampedGLU(limit, GLU_ALPHA)

    def forward(self, x):
        return self.down_proj(self.act_fn(self.gate_up_proj(x)))


class KagalornLayer(nn.Module):

    def __init__(self, config: KagalornConfig, spec: dict):
        super().__init__()
        m, W = spec["mixer"], config.width
        if spec["type"] == "delta":
            self.mix = GatedDeltaRule(W, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"],
                                      norm_eps=config.norm_eps, unit_eps=UNIT_NORM_EPS)
        else:
            self.mix = WindowPoolAttention(W, m["heads"], m["kv_heads"], m["dim"], m["vdim"], int(m["mask"]["size"]),
                                           int(m["mask"].get("pool", 0)), float(m["scale"]), norm_eps=config.norm_eps,
                                           sink=True, gated=True)
        self.norm1 = GroupedRMSNorm(W, config.norm_groups, config.norm_eps)
        self.hc1 = HyperConnection(config.streams)
        self.mlp = None
        if spec["mlp"] is not None:
            self.mlp = ClampedGLUMLP(W, int(spec["mlp"]["ff"]), float(spec["mlp"]["limit"]))
            self.norm2 = GroupedRMSNorm(W, config.norm_groups, config.norm_eps)
            self.hc2 = HyperConnection(config.streams)

    def sublayers(self):
        yield self.hc1, self.norm1, self.mix
        if self.mlp is not None:
            yield self.hc2, self.norm2, self.mlp


class KagalornForCausalLM(nn.Module):
    ragged_steps = True           # the runner feeds utils.context.RaggedStep batches
    config_class = KagalornConfig

    def __init__(self, config: KagalornConfig):
        super().__init__()
        self.config = config
        self.embed = VocabParallelEmbedding(config.vocab, config.width)
        self.layers = nn.ModuleList([KagalornLayer(config, spec) for spec in config.layers])
        self.final_norm = GroupedRMSNorm(config.width, config.norm_groups, config.norm_eps)
        self.lm_head = ParallelLMHead(config.vocab, config.width)
        self.register_buffer("sum_read", torch.ones(config.streams, dtype=torch.float32), persistent=False)
        self.layer_outputs: Optional[list] = None     # set to [] to record the summed streams after every layer

    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        emb = self.embed(input_ids)
        act = emb.dtype
        x = open_streams(emb, self.config.streams)
        subs = [s for layer in self.layers for s in layer.sublayers()]
        ends = set()
        n = 0
        for layer in self.layers:
            n += 1 if layer.mlp is None else 2
            ends.add(n - 1)
        h = advance(x, None, None, subs[0][0].read, subs[0][1], act) if subs else None
        for i, (hc, _, fn) in enumerate(subs):
            y = fn(h)
            if i + 1 < len(subs):
                h = advance(x, y, hc, subs[i + 1][0].read, subs[i + 1][1], act)
            else:
                h = advance(x, y, hc, self.sum_read, self.final_norm, act)
            if self.layer_outputs is not None and i in ends:
                self.layer_outputs.append(x.sum(1))
        if not subs:
            h = advance(x, None, None, self.sum_read, self.final_norm, act)
        return h

    def compute_logits(self, hidden_states):
        return self.lm_head(hidden_states)

    def greedy_tokens(self, hidden_states):
        return self.lm_head.greedy_tokens(hidden_states)

    # ------------------------------------------------------------------ checkpoint
    def weight_targets(self) -> dict:
        """checkpoint tensor name -> (parameter, where, shape): where is None (the whole parameter), the
        index of a part of a merged projection, or ("rows", offset, size)."""
        t = {}

        def whole(name, param):
            t[name] = (param, None, tuple(param.shape))

        def part(name, linear, j):
            t[name] = (linear.weight, j, (linear.output_sizes[j], linear.weight.shape[1]))

        whole("embed", self.embed.weight)
        whole("head", self.lm_head.weight)
        whole("final.norm", self.final_norm.weight)
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            whole(p + "norm1", layer.norm1.weight)
            for q, hc in ((1, layer.hc1),) + (((2, layer.hc2),) if layer.mlp is not None else ()):
                whole(p + f"hc{q}.in", hc.read)
                whole(p + f"hc{q}.out", hc.write)
                whole(p + f"hc{q}.mix", hc.mix)
            mix = layer.mix
            if isinstance(mix, GatedDeltaRule):
                for j, nm in enumerate(("q", "k", "v", "g", "b", "a")):
                    part(p + "mix." + nm, mix.in_proj, j)
                gd, hv = mix.G * mix.D, mix.H * mix.Dv
                for nm, off, size in (("q", 0, gd), ("k", gd, gd), ("v", 2 * gd, hv)):
                    t[p + f"mix.{nm}.conv"] = (mix.conv_weight, ("rows", off, size), (size, mix.taps))
                whole(p + "mix.A_log", mix.A_log)
                whole(p + "mix.dt_bias", mix.dt_bias)
                whole(p + "mix.norm", mix.out_norm_weight)
            else:
                for j, nm in enumerate(("q", "k", "v", "g")):
                    part(p + "mix." + nm, mix.in_proj, j)
                whole(p + "mix.q.norm", mix.q_norm_weight)
                whole(p + "mix.k.norm", mix.k_norm_weight)
            whole(p + "mix.o", mix.o_proj.weight)
            if layer.mlp is not None:
                whole(p + "norm2", layer.norm2.weight)
                part(p + "mlp.gate", layer.mlp.gate_up_proj, 0)
                part(p + "mlp.up", layer.mlp.gate_up_proj, 1)
                whole(p + "mlp.down", layer.mlp.down_proj.weight)
        return t

    def load_weights(self, tensors) -> None:
        """tensors: iterable of (checkpoint name, tensor). Every parameter must be covered."""
        targets = self.weight_targets()
        seen = set()
        for name, tensor in tensors:
            if name not in targets:
                raise KeyError(f"checkpoint tensor '{name}' has no place in this Kagalorn configuration")
            param, where, shape = targets[name]
            if tuple(tensor.shape) != shape:
                raise ValueError(f"'{name}': shape {tuple(tensor.shape)} does not fit {shape}")
            if where is None:
                loader = getattr(param, "weight_loader", None)
                if loader is not None:
                    loader(param, tensor)
                else:
                    param.data.copy_(tensor)
            elif isinstance(where, tuple):
                param.data[where[1]:where[1] + where[2]].copy_(tensor)
            else:
                param.weight_loader(param, tensor, where)
            seen.add(name)
        missing = sorted(set(targets) - seen)
        if missing:
            raise KeyError(f"checkpoint lacks {missing[:8]}{' ...' if len(missing) > 8 else ''}")

    @torch.no_grad()
    def init_random_on_device(self, seed: int = 0) -> None:
        """Fast random fill on the parameters' own device (benchmarks: values differ between devices)."""
        S = self.config.streams
        gens = {}
        for name, (param, where, _) in self.weight_targets().items():
            if where is not None and not (isinstance(where, int) and where == 0) and not (isinstance(where, tuple) and where[1] == 0):
                continue                    # merged tensors are filled once, through their first part
            g = gens.get(param.device)
            if g is None:
                g = gens[param.device] = torch.Generator(device=param.device).manual_seed(seed)
            leaf = name.rsplit(".", 1)[-1]
            if "norm" in leaf:
                param.fill_(1.0)
            elif ".hc" in name:
                param.copy_(torch.eye(S) if leaf == "mix" else torch.full((S,), 1.0 / S if leaf == "in" else 1.0))
            elif leaf in ("conv", "A_log", "dt_bias"):
                param.normal_(0.0, 0.5, generator=g)
            else:
                param.normal_(0.0, param.shape[-1] ** -0.5, generator=g)

    def random_weights(self, seed: int = 0):
        """(name, tensor) pairs of a seeded random checkpoint of this configuration, for runs without
        weights on disk. Scales keep activations of order one through any depth."""
        from ..utils.loader import full_random_tensor
        S = self.config.streams
        for name, (_, _, shape) in self.weight_targets().items():
            leaf = name.rsplit(".", 1)[-1]
            if "norm" in leaf:
                yield name, 1.0 + full_random_tensor(name, shape, seed, 0.1)
            elif ".hc" in name and leaf == "mix":
                yield name, torch.eye(S) * 0.8 + full_random_tensor(name, shape, seed, 0.1)
            elif ".hc" in name:
                yield name, (1.0 / S if leaf == "in" else 1.0) + full_random_tensor(name, shape, seed, 0.1)
            elif leaf in ("conv", "A_log", "dt_bias"):
                yield name, full_random_tensor(name, shape, seed, 0.5)
            elif len(shape) == 2:
                yield name, full_random_tensor(name, shape, seed, shape[1] ** -0.5)
            else:
                yield name, full_random_tensor(name, shape, seed, 0.5)
