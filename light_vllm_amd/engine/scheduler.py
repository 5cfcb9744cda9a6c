"""Prefill-first continuous batching with LIFO preemption.

Same policy as the reference's Scheduler (lightvllm/engine/scheduler.py:55-134): a step is either a
prefill of as many waiting sequences as fit (`max_num_seqs`, `max_num_batched_tokens` counting only
un-cached tokens, free KV blocks), or one decode token for the running sequences, preempting from
the tail of the running queue when the KV pool cannot grow. It decides the batch composition that
the attention kernels see; nothing here touches the device.

Models that run ragged steps (config.ragged) are scheduled differently: one step mixes single decode
tokens with portions of prompts under the same token budget (`max_num_batched_tokens`, a prompt longer
than the budget or than `long_prefill_token_threshold` is computed over several steps), pages are taken
as a sequence grows, without the prefix cache, and every live sequence holds a state slot.
"""
from __future__ import annotations

from collections import deque

from .block_manager import BlockManager
from .sequence import Sequence, SequenceStatus
from .state_manager import StateSlotManager


class Scheduler:

    def __init__(self, config):
        self.max_num_seqs = config.max_num_seqs
        self.max_num_batched_tokens = config.max_num_batched_tokens
        self.eos = config.eos
        self.block_manager = BlockManager(config.num_kvcache_blocks, config.kvcache_block_size,
                                          getattr(config, "strict_reference", False))
        self.ragged = bool(getattr(config, "ragged", False))
        self.state_slots = StateSlotManager(config.max_num_seqs) if self.ragged else None
        self.prefill_cap = getattr(config, "long_prefill_token_threshold", 0)
        self.waiting: deque[Sequence] = deque()
        self.running: deque[Sequence] = deque()

    def is_finished(self) -> bool:
        return not self.waiting and not self.running

    def add(self, seq: Sequence) -> None:
        self.waiting.append(seq)

    def preempt(self, seq: Sequence) -> None:
        seq.status = SequenceStatus.WAITING
        seq.needs_prefill = True          # recomputed from all its tokens when it is scheduled again
        self.block_manager.deallocate(seq)
        if self.ragged:
            self.state_slots.release(seq)
            seq.num_computed_tokens = 0
        self.waiting.appendleft(seq)

    # ------------------------------------------------------------------ ragged steps
    def admit(self, seq: Sequence) -> None:
        """A sequence becomes live: it gets a state slot; pages follow as its tokens are scheduled."""
        self.state_slots.acquire(seq)
        seq.status = SequenceStatus.RUNNING
        self.running.append(seq)

    def release(self, seq: Sequence) -> None:
        """Give back what a live sequence holds (finished, or ended by the caller)."""
        self.block_manager.deallocate(seq)
        self.state_slots.release(seq)
        seq.status = SequenceStatus.FINISHED
        self.running.remove(seq)

    def _portion(self, seq: Sequence, budget: int) -> int:
        n = min(len(seq) - seq.num_computed_tokens, budget)
        if self.prefill_cap > 0 and n > 1:
            n = min(n, self.prefill_cap)
        return n

    def _schedule_ragged(self) -> tuple[list[Sequence], bool]:
        budget = self.max_num_batched_tokens
        batch: list[Sequence] = []
        # running sequences, those that decode first (one token each), then portions of prompts
        order = sorted(self.running, key=lambda q: len(q) - q.num_computed_tokens > 1)
        for seq in order:
            if not seq.is_running:
                continue                  # preempted below while an earlier one was served
            n = self._portion(seq, budget)
            if n <= 0:
                continue
            while not self.block_manager.can_extend(seq, seq.num_computed_tokens + n):
                victim = next((v for v in reversed(self.running) if v is not seq and v not in batch), seq)
                self.running.remove(victim)
                self.preempt(victim)
                if victim is seq:
                    break
            else:
                self.block_manager.extend(seq, seq.num_computed_tokens + n)
                seq.num_scheduled_tokens = n
                budget -= n
                batch.append(seq)
        while self.waiting and budget > 0 and len(self.running) < self.max_num_seqs and self.state_slots.num_free:
            seq = self.waiting[0]
            n = self._portion(seq, budget)
            if not self.block_manager.can_extend(seq, n):
                break
            self.waiting.popleft()
            self.admit(seq)
            self.block_manager.extend(seq, n)
            seq.num_scheduled_tokens = n
            budget -= n
            batch.append(seq)
        assert batch, "nothing could be scheduled: the page pool is smaller than one sequence needs"
        return batch, any(seq.num_scheduled_tokens > 1 for seq in batch)

    def _postprocess_ragged(self, seqs: list[Sequence], token_ids: list) -> None:
        for seq, token_id in zip(seqs, token_ids):
            seq.num_computed_tokens += seq.num_scheduled_tokens
            seq.num_scheduled_tokens = 0
            if token_id is None:          # a portion that does not end the known tokens: nothing was sampled
                continue
            seq.append_token(token_id)
            seq.needs_prefill = False
            if (not seq.ignore_eos and token_id == self.eos) or seq.num_completion_tokens == seq.max_tokens:
                self.release(seq)

    def schedule(self) -> tuple[list[Sequence], bool]:
        if self.ragged:
            return self._schedule_ragged()
        batch: list[Sequence] = []
        num_batched_tokens = 0
        # prefill
        while self.waiting and len(batch) < self.max_num_seqs:
            seq = self.waiting[0]
            if (num_batched_tokens + len(seq) > self.max_num_batched_tokens
                    or not self.block_manager.can_allocate(seq)):
                break
            self.block_manager.allocate(seq)
            num_batched_tokens += len(seq) - seq.num_cached_tokens
            seq.status = SequenceStatus.RUNNING
            self.waiting.popleft()
            self.running.append(seq)
            batch.append(seq)
        if batch:
            return batch, True
        # decode
        while self.running and len(batch) < self.max_num_seqs:
            seq = self.running.popleft()
            while not self.block_manager.can_append(seq):
                if self.running:
                    self.preempt(self.running.pop())
                else:
                    self.preempt(seq)
                    break
            else:
                self.block_manager.may_append(seq)
                batch.append(seq)
        assert batch, "decode step scheduled nothing"
        self.running.extendleft(reversed(batch))
        return batch, False

    def postprocess(self, seqs: list[Sequence], token_ids: list[int]) -> None:
        if self.ragged:
            return self._postprocess_ragged(seqs, token_ids)
        for seq, token_id in zip(seqs, token_ids):
            seq.append_token(token_id)
            seq.needs_prefill = False
            if (not seq.ignore_eos and token_id == self.eos) or seq.num_completion_tokens == seq.max_tokens:
                seq.status = SequenceStatus.FINISHED
                self.block_manager.deallocate(seq)
                self.running.remove(seq)
