"""Replay of a recorded schedule: given token ids are fed through the engine step by step and the
logits of chosen positions are written out; nothing is sampled.

A step names, for each request, its next tokens and the places among them whose logits are wanted;
all requests of a step run as one ragged batch (portions of prompts beside single tokens). A request
is admitted at its first step (state slot), takes pages as it grows, may sit out steps, and gives
everything back when the step that ends it is done. The replayer owns no model code, cache or
loader: it drives the engine's scheduler state (page pool, state slots) and the model runner's
ragged step.

Input: one JSON object per line, {"step": n, "entries": [{"id", "tokens", "want"}], "end": [ids]}.
Output: <out>/<step>.f32 (little-endian f32 [wanted, vocab], in the order of entries and wants) for
steps that want something, and a line "done <step>" on standard output after every step.
"""
from __future__ import annotations

import json
import os
import sys

import numpy as np

from ..sampling_params import SamplingParams
from .llm_engine import LLMEngine
from .sequence import Sequence

PAGE_TOKENS = 64          # page size of replay runs: live tokens are counted in multiples of it
STATE_SLOTS = 4           # live requests at any time


class TraceReplayer:

    def __init__(self, model: str, dtype: str, max_tokens: int, device: str = "cuda", slots: int = STATE_SLOTS,
                 page: int = PAGE_TOKENS):
        self.engine = LLMEngine(model, dtype=dtype, device=device, kvcache_block_size=page, max_num_seqs=slots,
                                max_cache_tokens=max_tokens, max_num_batched_tokens=max(max_tokens, page),
                                max_model_len=max(max_tokens, page), enforce_eager=True)
        if not self.engine.config.ragged:
            raise RuntimeError("trace replay needs a model that runs ragged steps")
        self.live: dict[str, Sequence] = {}

    def step(self, entries: list, end: list):
        sched, runner = self.engine.scheduler, self.engine.model_runner
        seqs, rows, at = [], [], 0
        for e in entries:
            tokens = [int(t) for t in e["tokens"]]
            if not tokens:
                continue
            seq = self.live.get(e["id"])
            if seq is None:
                seq = Sequence(tokens, SamplingParams(temperature=0.0, max_tokens=1 << 30, ignore_eos=True))
                sched.admit(seq)
                self.live[e["id"]] = seq
            else:
                seq.extend_tokens(tokens)
            sched.block_manager.extend(seq, len(seq))
            seq.num_scheduled_tokens = len(tokens)
            seqs.append(seq)
            rows.extend(at + int(w) for w in e.get("want", ()))
            at += len(tokens)
        logits = runner.call("run_rows", seqs, rows) if seqs else None
        for seq in seqs:
            seq.num_computed_tokens += seq.num_scheduled_tokens
            seq.num_scheduled_tokens = 0
        for rid in end:
            seq = self.live.pop(rid, None)
            if seq is not None:
                sched.release(seq)
        return logits if rows else None

    def close(self):
        self.engine.exit()


def main(argv=None) -> int:
    import argparse
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=("bfloat16", "float32"))
    ap.add_argument("--out", required=True, help="folder for the <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True, help="most tokens live requests hold at any time")
    ap.add_argument("--device", default="cuda")
    a = ap.parse_args(argv)
    os.makedirs(a.out, exist_ok=True)
    rp = TraceReplayer(a.model, a.dtype, a.max_tokens, device=a.device)
    try:
        for line in sys.stdin:
            line = line.strip()
            if not line:
                continue
            msg = json.loads(line)
            logits = rp.step(msg.get("entries", []), msg.get("end", []))
            if logits is not None:
                tmp = os.path.join(a.out, f".{msg['step']}.part")
                np.ascontiguousarray(logits.numpy(), dtype="<f4").tofile(tmp)
                os.replace(tmp, os.path.join(a.out, f"{msg['step']}.f32"))
            sys.stdout.write(f"done {msg['step']}\n")
            sys.stdout.flush()
    finally:
        rp.close()
    return 0
