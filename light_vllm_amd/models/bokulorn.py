"""Bokulorn: a decoder-only model of latent-attention and channel-wise delta-rule layers with
mixture-of-experts feed-forwards on one f32 residual.

config.json (`architecture: "Bokulorn"`) lists the layers. Each names its mixer type:
  "latent_attention"    latent attention with a rotated positional part and one output gate per head,
  "latent_attention_2"  position-free latent attention, gated per output channel,
  "channel_delta"       gated delta rule in which every key channel of every head decays at its own rate, with
                        thin two-factor projections for the decay and the output gate,
the mixer's sizes, and its feed-forward (a mixture of squared-relu experts behind a sigmoid router
with a selection-only correction and a group limit, or none). A layer is parallel: mixer and
feed-forward take the same normed input h = norm(x) and x += mix(h) + ffn(h). Norm weights are
held as offsets from one, i.e. applied as (1 + w); the embedding is multiplied by a constant. A layer with
`weights_of: j` reuses the parameters of layer j while keeping separate cache pages and state slots.

Sizes, layer order and constants come from the config; the ranks of the delta rule's thin factors,
which the config does not name, come from the checkpoint's tensor shapes (or from the optional mixer
keys `decay_rank` / `gate_rank` when a model is built without a checkpoint).

The model runs ragged steps only (utils.context.RaggedStep). Checkpoint tensors: embed, head,
final.norm, l<i>.norm1, l<i>.mix.*, l<i>.mlp.e<j>.up|down, l<i>.mlp.router|correction; linear weights
stored [out, in].
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from glob import glob
from typing import Any, Optional

import torch
from torch import nn

from ..layers.delta_rule import GatedDeltaRule
from ..layers.embed_head import ParallelLMHead, VocabParallelEmbedding
from ..layers.latent_attention import LatentAttention
from ..layers.layernorm import OffsetRMSNorm
from ..layers.moe import SparseMoE

UNIT_NORM_EPS = 1e-6       # inside the root of the delta rule's unit norms
NORM_WEIGHT_OFFSET = 1.0   # norm weights are offsets from one
LATENT_TYPES = ("latent_attention", "latent_attention_2")


def _tensor_shapes(path: str) -> dict:
    """name -> shape of every tensor in the *.safetensors files of a directory (headers only)."""
    from safetensors import safe_open
    shapes = {}
    for file in sorted(glob(os.path.join(path, "*.safetensors"))):
        with safe_open(file, "pt", "cpu") as f:
            for name in f.keys():
                shapes[name] = tuple(f.get_slice(name).get_shape())
    return shapes


@dataclass
class BokulornConfig:
    """config.json of a Bokulorn checkpoint. Attribute names the engine reads from any model config
    (vocab_size, hidden_size, max_position_embeddings, torch_dtype) are provided as well."""
    vocab: int
    width: int
    norm_eps: float
    embedding_scale: float = 1.0
    layers: list = field(default_factory=list)
    torch_dtype: Any = torch.bfloat16
    max_position_embeddings: int = 1 << 30       # positions are rotated on the fly: any length the cache holds
    architectures: tuple = ("Bokulorn",)

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    def source_of(self, i: int) -> int:
        """The layer whose weights layer i runs with (itself unless it names another)."""
        seen = set()
        while self.layers[i].get("weights_of") is not None:
            assert i not in seen, "weights_of forms a loop"
            seen.add(i)
            i = int(self.layers[i]["weights_of"])
        return i

    @classmethod
    def from_dict(cls, d: dict, shapes: Optional[dict] = None) -> "BokulornConfig":
        for key in ("vocab", "width", "layers", "norm"):
            if key not in d:
                raise ValueError(f"Bokulorn config lacks '{key}'")
        layers = []
        for i, L in enumerate(d["layers"]):
            kind, m = L["type"], dict(L["mixer"])
            if kind in LATENT_TYPES:
                need = ("heads", "dim", "vdim", "q_rank", "kv_rank", "scale")
                if kind == "latent_attention" and int(m.get("rot_dim", 0)) > 0:
                    need += ("rot",)
            elif kind == "channel_delta":
                need = ("heads", "kv_heads", "dim", "vdim", "conv")
            else:
                raise ValueError(f"layer {i}: unknown mixer type '{kind}'")
            missing = [k for k in need if k not in m]
            if missing:
                raise ValueError(f"layer {i} ({kind}): mixer lacks {missing}")
            mlp = L.get("mlp")
            if mlp is not None:
                if mlp.get("kind") != "moe":
                    raise ValueError(f"layer {i}: unknown feed-forward kind '{mlp.get('kind')}'")
                mlp = {"kind": "moe", "expert": dict(mlp["expert"]), "router": dict(mlp["router"])}
            spec = {"type": kind, "mixer": m, "mlp": mlp}
            if L.get("weights_of") is not None:
                j = int(L["weights_of"])
                if not 0 <= j < len(d["layers"]) or j == i:
                    raise ValueError(f"layer {i}: weights_of {j}")
                spec["weights_of"] = j
            layers.append(spec)
        cfg = cls(vocab=int(d["vocab"]), width=int(d["width"]), norm_eps=float(d["norm"]["eps"]),
                  embedding_scale=float(d.get("embedding", {}).get("scale", 1.0)), layers=layers)
        for i, spec in enumerate(layers):
            j = cfg.source_of(i)
            if layers[j]["type"] != spec["type"]:
                raise ValueError(f"layer {i}: weights_of names a layer of another type")
            if spec["type"] == "channel_delta":       # thin-factor ranks: the tensors' shapes, else the optional keys
                m = spec["mixer"]
                for key, tensor in (("decay_rank", f"l{j}.mix.a1"), ("gate_rank", f"l{j}.mix.g1")):
                    if shapes is not None and tensor in shapes:
                        m[key] = int(shapes[tensor][0])
                    elif key not in m:
                        raise ValueError(f"layer {i}: '{key}' is neither in the config nor given by a tensor '{tensor}'")
        return cfg

    @classmethod
    def from_pretrained(cls, path: str) -> "BokulornConfig":
        with open(os.path.join(path, "config.json")) as f:
            return cls.from_dict(json.load(f), _tensor_shapes(path))


def _make_mixer(config: BokulornConfig, spec: dict, share):
    m, W = spec["mixer"], config.width
    if spec["type"] == "channel_delta":
        return GatedDeltaRule(W, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"], norm_eps=config.norm_eps,
                              unit_eps=UNIT_NORM_EPS, decay="channel", decay_rank=int(m["decay_rank"]),
                              gate_rank=int(m["gate_rank"]), gate_act="sigmoid", share=share)
    positional = spec["type"] == "latent_attention"
    rot_dim = int(m.get("rot_dim", 0)) if positional else 0
    rot = m.get("rot") or {}
    return LatentAttention(W, m["heads"], m["dim"], m["vdim"], m["q_rank"], m["kv_rank"], float(m["scale"]),
                           rot_dim=rot_dim, rot_dims=int(rot.get("dims", rot_dim)) if rot_dim else 0,
                           rot_base=float(rot.get("base", 10000.0)), gate="head" if positional else "channel",
                           norm_eps=config.norm_eps, share=share)


class BokulornLayer(nn.Module):

    def __init__(self, config: BokulornConfig, spec: dict, source: "BokulornLayer | None" = None):
        super().__init__()
        self.mix = _make_mixer(config, spec, source.mix if source is not None else None)
        self.norm1 = source.norm1 if source is not None else OffsetRMSNorm(config.width, config.norm_eps, NORM_WEIGHT_OFFSET)
        self.mlp = None
        if spec["mlp"] is not None:
            r = spec["mlp"]["router"]
            groups = r.get("groups") or {}
            self.mlp = SparseMoE(config.width, int(spec["mlp"]["expert"]["ff"]), int(r["experts"]), int(r["top"]),
                                 int(groups.get("count", 1)), int(groups.get("keep", groups.get("count", 1))),
                                 share=source.mlp if source is not None else None)


class BokulornForCausalLM(nn.Module):
    ragged_steps = True           # the runner feeds utils.context.RaggedStep batches
    config_class = BokulornConfig

    def __init__(self, config: BokulornConfig):
        super().__init__()
        self.config = config
        self.embed = VocabParallelEmbedding(config.vocab, config.width)
        # a layer may name a later one: build the owners first, then the layers that borrow
        built: dict[int, BokulornLayer] = {}
        for i, spec in enumerate(config.layers):
            if config.source_of(i) == i:
                built[i] = BokulornLayer(config, spec)
        for i, spec in enumerate(config.layers):
            if i not in built:
                built[i] = BokulornLayer(config, spec, built[config.source_of(i)])
        self.layers = nn.ModuleList([built[i] for i in range(len(config.layers))])
        self.final_norm = OffsetRMSNorm(config.width, config.norm_eps, NORM_WEIGHT_OFFSET)
        self.lm_head = ParallelLMHead(config.vocab, config.width)
        self.layer_outputs: Optional[list] = None     # set to [] to record the residual after every layer

    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        emb = self.embed(input_ids)
        act = emb.dtype
        x = emb.float().mul_(self.config.embedding_scale)           # the residual, f32 throughout
        norms = [layer.norm1 for layer in self.layers] + [self.final_norm]
        h = norms[0](x, act_dtype=act)
        for i, layer in enumerate(self.layers):
            y1 = layer.mix(h)
            y2 = layer.mlp(h) if layer.mlp is not None else None
            h = norms[i + 1](x, y1, y2, act_dtype=act)              # x += y1 + y2, then the next layer's norm
            if self.layer_outputs is not None:
                self.layer_outputs.append(x.clone())
        return h

    def compute_logits(self, hidden_states):
        return self.lm_head(hidden_states)

    def greedy_tokens(self, hidden_states):
        return self.lm_head.greedy_tokens(hidden_states)

    # ------------------------------------------------------------------ checkpoint
    def weight_targets(self) -> dict:
        """checkpoint tensor name -> (parameter, where, shape): where is None (the whole parameter), the
        index of a part of a merged projection, ("rows", offset, size) or ("cols", offset, size)."""
        t = {}

        def whole(name, param, shape=None):
            t[name] = (param, None, tuple(shape or param.shape))

        def part(name, linear, j):
            t[name] = (linear.weight, j, (linear.output_sizes[j], linear.weight.shape[1]))

        whole("embed", self.embed.weight)
        whole("head", self.lm_head.weight)
        whole("final.norm", self.final_norm.weight)
        for i, layer in enumerate(self.layers):
            if self.config.source_of(i) != i:
                continue                      # runs with another layer's tensors
            p = f"l{i}."
            whole(p + "norm1", layer.norm1.weight)
            mix = layer.mix
            if isinstance(mix, GatedDeltaRule):
                for j, nm in enumerate(("q", "k", "v", "g1", "b", "a1")):
                    part(p + "mix." + nm, mix.in_proj, j)
                whole(p + "mix.g2", mix.gate_up.weight)
                whole(p + "mix.a2", mix.decay_up.weight)
                gd, hv = mix.G * mix.D, mix.H * mix.Dv
                for nm, off, size in (("q", 0, gd), ("k", gd, gd), ("v", 2 * gd, hv)):
                    t[p + f"mix.{nm}.conv"] = (mix.conv_weight, ("rows", off, size), (size, mix.taps))
                whole(p + "mix.A_log", mix.A_log)
                whole(p + "mix.dt_bias", mix.dt_bias)
                whole(p + "mix.norm", mix.out_norm_weight)
            else:
                for j, nm in enumerate(("dq", "dkv", "g")):
                    part(p + "mix." + nm, mix.in_proj, j)
                whole(p + "mix.dq.norm", mix.q_norm_weight)
                whole(p + "mix.dkv.norm", mix.kv_norm_weight)
                whole(p + "mix.uq", mix.uq.weight)
                whole(p + "mix.uk", mix.uk, (mix.H * mix.Dn, mix.R))       # head by head: a view of [H, dim, R]
                whole(p + "mix.uv", mix.uv, (mix.H * mix.Dv, mix.R))
            whole(p + "mix.o", mix.o_proj.weight)
            if layer.mlp is not None:
                moe = layer.mlp
                whole(p + "mlp.router", moe.router_weight)
                whole(p + "mlp.correction", moe.correction)
                for e in range(moe.E):
                    t[p + f"mlp.e{e}.up"] = (moe.up_weight, ("rows", e * moe.ff, moe.ff), (moe.ff, moe.width))
                    t[p + f"mlp.e{e}.down"] = (moe.down_weight, ("cols", e * moe.ff, moe.ff), (moe.width, moe.ff))
        return t

    def load_weights(self, tensors) -> None:
        """tensors: iterable of (checkpoint name, tensor). Every parameter must be covered."""
        targets = self.weight_targets()
        seen = set()
        for name, tensor in tensors:
            if name not in targets:
                raise KeyError(f"checkpoint tensor '{name}' has no place in this Bokulorn configuration")
            param, where, shape = targets[name]
            if tuple(tensor.shape) != shape:
                raise ValueError(f"'{name}': shape {tuple(tensor.shape)} does not fit {shape}")
            if where is None:
                loader = getattr(param, "weight_loader", None)
                if loader is not None:
                    loader(param, tensor)
                else:
                    param.data.copy_(tensor.reshape(param.shape))
            elif isinstance(where, tuple) and where[0] == "rows":
                param.data[where[1]:where[1] + where[2]].copy_(tensor)
            elif isinstance(where, tuple):
                param.data[:, where[1]:where[1] + where[2]].copy_(tensor)
            else:
                param.weight_loader(param, tensor, where)
            seen.add(name)
        missing = sorted(set(targets) - seen)
        if missing:
            raise KeyError(f"checkpoint lacks {missing[:8]}{' ...' if len(missing) > 8 else ''}")

    @staticmethod
    def _random_std(name: str, shape) -> Optional[float]:
        """Standard deviation of a random stand-in for checkpoint tensor `name` (None: a norm weight,
        drawn near 0). Scales keep activations of order one through any depth."""
        leaf = name.rsplit(".", 1)[-1]
        if "norm" in leaf:
            return None
        if leaf in ("conv", "A_log", "dt_bias", "correction"):
            return 0.5
        return shape[-1] ** -0.5 if len(shape) == 2 else 0.5

    @torch.no_grad()
    def init_random_on_device(self, seed: int = 0) -> None:
        """Fast random fill on the parameters' own device (benchmarks: values differ between devices)."""
        gens, done = {}, set()
        for name, (param, _, shape) in self.weight_targets().items():
            if id(param) in done:
                continue                    # merged tensors are filled once
            done.add(id(param))
            g = gens.get(param.device)
            if g is None:
                g = gens[param.device] = torch.Generator(device=param.device).manual_seed(seed)
            std = self._random_std(name, shape)
            if std is None:
                param.zero_()
            else:
                param.normal_(0.0, std, generator=g)

    def random_weights(self, seed: int = 0):
        """(name, tensor) pairs of a seeded random checkpoint of this configuration, for runs without
        weights on disk."""
        from ..utils.loader import full_random_tensor
        for name, (_, _, shape) in self.weight_targets().items():
            std = self._random_std(name, shape)
            yield name, full_random_tensor(name, shape, seed, 0.1 if std is None else std)
