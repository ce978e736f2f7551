"""Batched serving of the layered models: a slot scheduler over the model's caches and states.

``BatchEngine`` owns the mapping request -> cache slot. A step takes, per request, its next tokens (a whole prompt,
or one decoded token), packs them into one ``StepBatch`` — no padding: the kernels take per-token slots and
positions — runs the model's step function once, and returns the logits of the rows asked for. A finished request
gives its slot back; the lowest free slot is handed out next, and the caches grow when more requests are live than
ever before. ``generate`` runs greedy or sampled continuation of several prompts through the same steps and
``generate.base.sample``.
"""

from __future__ import annotations

import sys
from pathlib import Path
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import torch

wd = Path(__file__).parent.parent.resolve()
if str(wd) not in sys.path:
    sys.path.append(str(wd))

from lit_gpt.mixers import StepBatch  # noqa: E402


class SlotPool:
    """Cache slots by number: ``take`` hands out the lowest free one, ``give`` returns it."""

    def __init__(self) -> None:
        self.free: List[int] = []
        self.size = 0

    def take(self) -> int:
        if self.free:
            self.free.sort()
            return self.free.pop(0)
        self.size += 1
        return self.size - 1

    def give(self, slot: int) -> None:
        if slot in self.free or not 0 <= slot < self.size:
            raise ValueError(f"slot {slot} is not in use")
        self.free.append(slot)


class BatchEngine:
    def __init__(self, model, max_seq_length: int, slots: int = 4) -> None:
        self.model = model
        self.device = model.device
        model.set_kv_cache(max(1, slots), max_seq_length)
        self.pool = SlotPool()
        self.live: Dict[Hashable, Tuple[int, int]] = {}  # request -> (slot, tokens held so far)

    def step(self, entries: Sequence[Tuple[Hashable, Sequence[int], Sequence[int]]],
             end: Sequence[Hashable] = ()) -> Optional[torch.Tensor]:
        """entries: (request, its next token ids, indices among them whose logits are wanted). Returns the wanted
        logits (n, vocab) fp32 in the order of the entries, or None. ``end``: requests finished after this step."""
        model = self.model
        table, rows, at = [], [], 0
        for req, tokens, want in entries:
            if req not in self.live:
                self.live[req] = (self.pool.take(), 0)
            slot, held = self.live[req]
            if held + len(tokens) > model.max_seq_length:
                raise ValueError(f"request {req!r} would hold {held + len(tokens)} tokens, the cache has room for "
                                 f"{model.max_seq_length}")
            for t in tokens:
                if not 0 <= int(t) < model.config.vocab:
                    raise ValueError(f"token id {t} outside the vocabulary")
            table.append((slot, held, tokens))
            rows += [at + int(k) for k in want]
            at += len(tokens)
            self.live[req] = (slot, held + len(tokens))
        if self.pool.size > model.slots:
            model.grow_slots(max(self.pool.size, 2 * model.slots))
        out = None
        if table:
            x = model.forward_step(StepBatch.build(table, self.device))
            if rows:
                out = model.logits(x, torch.tensor(rows, dtype=torch.int32).to(self.device))
        for req in end:
            slot, _ = self.live.pop(req)
            self.pool.give(slot)
        return out

    @torch.inference_mode()
    def generate(self, prompts: Sequence[Sequence[int]], max_new_tokens: int, *, temperature: float = 0.0,
                 top_k: Optional[int] = None, eos_id: Optional[int] = None) -> List[List[int]]:
        """Continue every prompt by up to ``max_new_tokens`` tokens: one prompt step for all, then one-token steps
        for those still running (a request that drew ``eos_id`` leaves the batch). Returns prompt + continuation."""
        from generate.base import sample

        ids = [object() for _ in prompts]
        seqs = [list(p) for p in prompts]
        running = list(range(len(prompts)))
        feed = {i: seqs[i] for i in running}
        for n in range(max_new_tokens):
            entries = [(ids[i], feed[i], [len(feed[i]) - 1]) for i in running]
            last = n == max_new_tokens - 1
            logits = self.step(entries, end=[ids[i] for i in running] if last else ())
            nxt, done = {}, []
            for row, i in enumerate(running):
                tok = int(sample(logits[row].view(1, 1, -1), temperature=temperature, top_k=top_k))
                seqs[i].append(tok)
                nxt[i] = [tok]
                if eos_id is not None and tok == eos_id and not last:
                    done.append(i)
            if done:
                self.step([], end=[ids[i] for i in done])
                running = [i for i in running if i not in done]
            feed = nxt
            if not running:
                break
        return seqs
