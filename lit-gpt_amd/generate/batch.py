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

    def decode_graph(self, requests: Sequence[Hashable], tokens: Sequence[int]) -> "GreedyDecodeGraph":
        """A captured greedy decode step for these live requests, whose next input tokens are ``tokens``."""
        return GreedyDecodeGraph(self, requests, tokens)

    @torch.inference_mode()
    def generate(self, prompts: Sequence[Sequence[int]], max_new_tokens: int, *, temperature: float = 0.0,
                 top_k: Optional[int] = None, eos_id: Optional[int] = None, use_graph: bool = False) -> List[List[int]]:
        """Continue every prompt by up to ``max_new_tokens`` tokens: one prompt step for all, then one-token steps
        for those still running (a request that drew ``eos_id`` leaves the batch). Returns prompt + continuation.
        ``use_graph`` (greedy, no eos): the one-token steps run as replays of one captured HIP graph."""
        from generate.base import sample

        if use_graph and temperature == 0.0 and eos_id is None and max_new_tokens > 1:
            ids = [object() for _ in prompts]
            logits = self.step([(ids[i], list(p), [len(p) - 1]) for i, p in enumerate(prompts)])
            first = [int(sample(logits[i].view(1, 1, -1), temperature=0.0)) for i in range(len(prompts))]
            graph = self.decode_graph(ids, first)
            new = torch.stack([graph.step().clone() for _ in range(max_new_tokens - 1)]).cpu()
            self.step([], end=ids)
            return [list(p) + [first[i]] + new[:, i].tolist() for i, p in enumerate(prompts)]

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


class GreedyDecodeGraph:
    """One-token greedy steps of a fixed set of live requests as replays of one HIP graph: the step's table (tokens,
    slots, positions) lives in static device buffers; the captured chain runs the model's step function, the output
    product, the framework's argmax per row (which writes the next input token in place) and advances the positions
    on the device, so a replay needs no host work. ``step()`` returns the (B,) device tensor of the tokens drawn."""

    def __init__(self, engine: BatchEngine, requests: Sequence[Hashable], tokens: Sequence[int]) -> None:
        from lit_gpt import ops

        model, dev = engine.model, engine.device
        self.engine, self.requests = engine, list(requests)
        B = len(self.requests)
        table = [(engine.live[r][0], engine.live[r][1], [int(t)]) for r, t in zip(self.requests, tokens)]
        self.batch = StepBatch.build(table, dev)
        self.drawn = torch.zeros(B, dtype=torch.int64, device=dev)
        self.steps_done = 0
        self.room = min(model.max_seq_length - engine.live[r][1] for r in self.requests)

        def body() -> None:
            b = self.batch
            logits = model.logits(model.forward_step(b))
            for i in range(B):
                ops.argmax(logits[i], out_idx=self.drawn[i:i + 1], token_out=b.tokens[i:i + 1])
            b.pos.add_(1)
            b.seq_pos0.add_(1)

        with torch.inference_mode():
            body()  # the first step runs eagerly (it also builds every kernel's device object)
            self._advance()
            self.first = self.drawn.clone()
            torch.cuda.synchronize(dev)
            self.graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(self.graph):
                body()
        self._pending_first = True

    def _advance(self) -> None:
        if self.steps_done >= self.room:
            raise ValueError("a request would outgrow the cache")
        self.steps_done += 1
        for r in self.requests:
            slot, held = self.engine.live[r]
            self.engine.live[r] = (slot, held + 1)

    def step(self) -> torch.Tensor:
        if self._pending_first:  # the eager step's tokens
            self._pending_first = False
            return self.first
        self._advance()
        self.graph.replay()
        return self.drawn
