"""Shared cases of the Kagalorn tests: small configurations and random weights made here, the engine
(or single kernels) on one side, oracle/kagalorn_oracle.py on the other. The CPU test file runs them
through the package's torch restatement of the kernels (host logic: pages, slots, ragged batching),
the GPU test file through the HIP kernels."""
from __future__ import annotations

import json
import os

import torch

from oracle import kagalorn_oracle as oracle

ATT_A = {"heads": 4, "kv_heads": 2, "dim": 12, "vdim": 8, "scale": 0.3, "mask": {"size": 6, "pool": 4}}
ATT_B = {"heads": 3, "kv_heads": 3, "dim": 8, "vdim": 16, "scale": 0.25, "mask": {"size": 9, "pool": 5}}
DEL_A = {"heads": 4, "kv_heads": 2, "dim": 8, "vdim": 12, "conv": 3}
DEL_B = {"heads": 2, "kv_heads": 2, "dim": 20, "vdim": 6, "conv": 5}

CFG_MAIN = {
    "architecture": "Kagalorn", "vocab": 61, "width": 48, "streams": 3, "norm": {"eps": 1e-5, "groups": 3},
    "layers": [
        {"type": "attention", "mixer": ATT_A, "mlp": {"kind": "dense", "ff": 40, "limit": 2.0}},
        {"type": "delta", "mixer": DEL_A, "mlp": None},
        {"type": "delta", "mixer": DEL_B, "mlp": {"kind": "dense", "ff": 24, "limit": 0.7}},
        {"type": "attention", "mixer": ATT_B, "mlp": {"kind": "dense", "ff": 40, "limit": 1.5}},
    ],
}
# values that a model may happen to make 1 or equal: one stream, one norm group, one tap, one kv head under ten
# query heads, a pool of one token, no pool at all, a window of one, value size above one wave, key size 40
CFG_ODD = {
    "architecture": "Kagalorn", "vocab": 37, "width": 40, "streams": 1, "norm": {"eps": 1e-6, "groups": 1},
    "layers": [
        {"type": "delta", "mixer": {"heads": 2, "kv_heads": 1, "dim": 40, "vdim": 70, "conv": 1}, "mlp": None},
        {"type": "attention", "mixer": {"heads": 10, "kv_heads": 1, "dim": 16, "vdim": 4, "scale": 0.5,
                                        "mask": {"size": 4, "pool": 1}}, "mlp": {"kind": "dense", "ff": 16, "limit": 1.0}},
        {"type": "attention", "mixer": {"heads": 2, "kv_heads": 2, "dim": 8, "vdim": 8, "scale": 0.4,
                                        "mask": {"size": 1, "pool": 0}}, "mlp": None},
        {"type": "attention", "mixer": {"heads": 2, "kv_heads": 1, "dim": 8, "vdim": 8, "scale": 0.4,
                                        "mask": {"size": 3, "pool": 21}}, "mlp": None},
    ],
}


# head sizes in multiples of 16 (in bf16 the attention layers then run on the matrix cores), five query heads a kv head
CFG_WIDE = {
    "architecture": "Kagalorn", "vocab": 83, "width": 64, "streams": 2, "norm": {"eps": 1e-6, "groups": 2},
    "layers": [
        {"type": "attention", "mixer": {"heads": 5, "kv_heads": 1, "dim": 32, "vdim": 16, "scale": 0.18,
                                        "mask": {"size": 20, "pool": 6}}, "mlp": {"kind": "dense", "ff": 96, "limit": 3.0}},
        {"type": "delta", "mixer": {"heads": 2, "kv_heads": 1, "dim": 16, "vdim": 32, "conv": 4}, "mlp": None},
        {"type": "attention", "mixer": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 48, "scale": 0.25,
                                        "mask": {"size": 17, "pool": 3}}, "mlp": {"kind": "dense", "ff": 96, "limit": 3.0}},
    ],
}


def write_model(path, cfg: dict, weights: dict) -> str:
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in weights.items()}, os.path.join(path, "model.safetensors"))
    return str(path)


def tokens_for(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def replay(model_dir, dtype, device, prompts: dict, schedule: list, max_tokens: int, page: int = 16, slots: int = 4):
    """Feeds `schedule` (steps of [(id, count), ...]) through the engine's trace replayer asking for the
    logits of every token; a request ends with its last token. Returns id -> [len, vocab] f32."""
    from light_vllm_amd.engine.trace_replay import TraceReplayer
    rp = TraceReplayer(model_dir, dtype, max_tokens, device=device, slots=slots, page=page)
    at = {i: 0 for i in prompts}
    got = {i: [] for i in prompts}
    try:
        for step in schedule:
            entries, end = [], []
            for i, n in step:
                lo, hi = at[i], at[i] + n
                entries.append({"id": i, "tokens": prompts[i][lo:hi], "want": list(range(n))})
                at[i] = hi
                if hi == len(prompts[i]):
                    end.append(i)
            logits = rp.step(entries, end)
            row = 0
            for i, n in step:
                got[i].append(logits[row:row + n].clone())
                row += n
    finally:
        rp.close()
    return {i: torch.cat(v) if v else torch.empty(0, 0) for i, v in got.items()}


def rel_err(got, want):
    """Per-row error the way a logit comparison should see it: mean removed, relative to the rows' spread."""
    d = got.double() - want.double()
    d = d - d.mean(-1, keepdim=True)
    w = want.double() - want.double().mean(-1, keepdim=True)
    return (d.pow(2).mean(-1).sqrt() / w.pow(2).mean().sqrt()).max().item()


# f32 runs are the sharp comparison. A model this narrow averages little rounding away, so in bf16 single
# positions are a tenth off the oracle; those runs guard the bf16 kernels against gross faults, the
# beacon cases (single kernels, scores that stand out) against fine ones.
TOL = {"float32": 3e-4, "bfloat16": 0.5}
TOL_MEDIAN = {"float32": 1e-4, "bfloat16": 0.12}


def assert_close(got, want, dtype, what):
    d = got.double() - want.double()
    d = d - d.mean(-1, keepdim=True)
    w = want.double() - want.double().mean(-1, keepdim=True)
    e = d.pow(2).mean(-1).sqrt() / w.pow(2).mean().sqrt()
    assert e.max().item() <= TOL[dtype] and e.median().item() <= TOL_MEDIAN[dtype], (what, e.max().item(), e.median().item())


def make_step(lens_q, ctx_lens, slots, tables, device):
    from light_vllm_amd.utils.context import RaggedStep
    cu = [0]
    tok_seq = []
    for b, n in enumerate(lens_q):
        cu.append(cu[-1] + n)
        tok_seq += [b] * n
    width = max(len(t) for t in tables)
    padded = [list(t) + [-1] * (width - len(t)) for t in tables]
    i32 = dict(dtype=torch.int32, device=device)
    return RaggedStep(torch.tensor(cu, **i32), torch.tensor(ctx_lens, **i32), torch.tensor(slots, **i32),
                      torch.tensor(tok_seq, **i32), torch.tensor(padded, **i32), list(lens_q), list(ctx_lens),
                      list(slots), [list(t) for t in tables])
