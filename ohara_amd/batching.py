"""Continuous batching on the decode path: sequences of different lengths share one batch, join
when a slot is free and leave when they finish.

The reference drives `Llama.forward` with a single scalar position for the whole batch
(ohara/models/llama.py:287-299, ohara/chat_engine.py:395-405), so all sequences of a batch must
have the same length and start together.  Here every slot of the KV caches has its own length: a
prompt is prefilled into its slot alone, and one decode step advances every active slot at its own
position (`Llama.forward` with one position per sequence).  Selection is greedy or the fused
temperature / top-k / top-p sampler of ohara/chat_engine.py:51-82.
"""

from __future__ import annotations

import torch

from . import ops
from .llama import BF16, Llama


class ContinuousBatcher:
    def __init__(self, model: Llama, slots: int, sampling=None, valid_vocab: int = 0, generator=None, int8: bool = False):
        if slots < 1:
            raise ValueError("batch_size must be at least 1")
        self.model, self.slots = model, slots
        self.sampling = sampling if (sampling is not None and sampling.temperature > 0) else None
        self.valid_vocab = valid_vocab
        self.generator = generator
        self.cache = model.build_kv_cache(slots, int8=int8)  # int8: the caches of ohara/modules/kv_cache.py:15-32
        for c in self.cache:
            c._commit_ragged(slots, [0] * slots)
        self.active = [False] * slots
        self.lengths = [0] * slots
        self.last = torch.zeros(slots, dtype=torch.int64, device=model.device)
        self.seq_pos = torch.zeros(slots, dtype=torch.int32, device=model.device)
        self.active_dev = torch.zeros(slots, dtype=torch.uint8, device=model.device)
        self._toks = self._u = self._graph = None

    def free_slots(self) -> list[int]:
        return [b for b in range(self.slots) if not self.active[b]]

    def _select(self, logits: torch.Tensor) -> torch.Tensor:
        """logits (rows, V) -> ids (rows,) on the device."""
        vv = self.valid_vocab or None
        if self.sampling is None:
            return ops.argmax(logits, valid_vocab=vv)
        u = torch.rand(logits.shape[0], device=logits.device, dtype=torch.float32, generator=self.generator)
        return ops.sample_topk_topp(logits, self.sampling.temperature, self.sampling.top_k, self.sampling.top_p, u,
                                    valid_vocab=vv)

    @torch.no_grad()
    def add(self, prompt_ids) -> tuple[int, int]:
        """Prefill a prompt (1-D ids) into a free slot -> (slot, first generated id)."""
        free = self.free_slots()
        if not free:
            raise RuntimeError("no free slot")
        ids = torch.as_tensor(prompt_ids, dtype=torch.int64).reshape(1, -1)
        if ids.shape[1] < 1:
            raise ValueError("input sequence cannot be empty")
        if ids.shape[1] >= self.model.config.max_sequence_length:
            raise ValueError("input exceeds max_sequence_length")
        b = free[0]
        for c in self.cache:
            c.lengths[b] = 0
        views = [c._row_view(b) for c in self.cache]
        logits = self.model.forward(ids.to(self.model.device), views, 0, last_only=True)
        tok = self._select(logits.view(1, -1))
        n = ids.shape[1]
        for c in self.cache:
            c.lengths[b] = n
            c.length = max(c.lengths)
        self.lengths[b] = n
        self.active[b] = True
        self.last[b:b + 1] = tok
        self.seq_pos[b] = n
        self.active_dev[b] = 1
        return b, int(tok.item())

    def remove(self, slot: int) -> None:
        self.active[slot] = False
        self.lengths[slot] = 0
        self.last[slot] = 0
        self.seq_pos[slot] = 0
        self.active_dev[slot] = 0
        for c in self.cache:
            c.lengths[slot] = 0

    def _device_step(self) -> None:
        """Everything of a step that runs on the device, with no host synchronisation: forward at
        the slots' own positions, selection, position advance, next inputs.  Capturable."""
        logits = self.model.forward(self.last.view(self.slots, 1), self.cache, list(self.lengths), last_only=True,
                                    seq_pos=self.seq_pos)
        vv = self.valid_vocab or None
        if self.sampling is None:
            ops.argmax(logits.view(self.slots, -1), valid_vocab=vv, next_ids=self._toks)
        else:
            ops.sample_topk_topp(logits.view(self.slots, -1), self.sampling.temperature, self.sampling.top_k,
                                 self.sampling.top_p, self._u, valid_vocab=vv, out=self._toks)
        # idle slots stay at position 0 and are fed id 0; active ones advance and are fed what they selected
        ops.advance_ragged(self.seq_pos, self.active_dev, self._toks, self.last, 1)

    def _enqueue_step(self, use_graph: bool) -> None:
        """One decode step of every active slot, enqueued; the host books advance, nothing is read back."""
        if max(n for n, a in zip(self.lengths, self.active) if a) + 1 > self.model.config.max_sequence_length:
            raise ValueError("input exceeds max_sequence_length")
        if self._toks is None:
            self._toks = torch.zeros(self.slots, dtype=torch.int64, device=self.model.device)
            self._u = torch.zeros(self.slots, dtype=torch.float32, device=self.model.device)
        if self.sampling is not None:
            self._u.copy_(torch.rand(self.slots, device=self.model.device, dtype=torch.float32, generator=self.generator))
        if use_graph and self._graph is None:
            # the capture itself executes nothing: the books it touches are restored, and the step
            # is then replayed like any other
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                self._device_step()
            self._graph = g
        if use_graph:
            self._graph.replay()
        else:
            self._device_step()
        for b in range(self.slots):
            if self.active[b]:
                self.lengths[b] += 1
        for c in self.cache:
            c.lengths = list(self.lengths)
            c.length = max(self.lengths)

    @torch.no_grad()
    def step(self, use_graph: bool = True) -> dict[int, int]:
        """One decode step for every active slot -> {slot: new id}.  Idle slots ride along at
        position 0 of their own cache rows (overwritten when the slot is taken again).  The device
        work is captured once into a HIP graph (positions, inputs and the active mask live in
        device tensors, so joins and leaves need no re-capture) and replayed per step."""
        if not any(self.active):
            return {}
        self._enqueue_step(use_graph)
        host = self._toks.tolist()
        return {b: host[b] for b in range(self.slots) if self.active[b]}

    @torch.no_grad()
    def steps(self, n: int, use_graph: bool = True) -> dict[int, list[int]]:
        """``n`` decode steps of every active slot with ONE read-back at the end -> {slot: its n new ids}: the
        chunked read-back of the single-sequence engines (a stop id is looked for in the chunk afterwards; a
        slot that met one has run on to the end of the chunk and is trimmed and removed by the caller)."""
        if n < 1 or not any(self.active):
            return {}
        if max(m for m, a in zip(self.lengths, self.active) if a) + n > self.model.config.max_sequence_length:
            raise ValueError("input exceeds max_sequence_length")
        rows = torch.empty(n, self.slots, dtype=torch.int64, device=self.model.device)
        for i in range(n):
            self._enqueue_step(use_graph)
            rows[i].copy_(self._toks)
        host = rows.t().tolist()
        return {b: host[b] for b in range(self.slots) if self.active[b]}
