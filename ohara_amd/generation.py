"""Token sources for the generate loops of ``Inference`` and ``ChatEngine``.

A *token source* is an iterator over the ids a model produces after a prompt.  The engines only
consume ids (stop checks, detokenisation, printing); how the ids are produced is decided here:

* ``device_tokens`` - the fast path for the kernel-backed dense ``Llama``: the prompt is prefilled
  once, then every token is one replay of a captured graph (persistent decode step + selection, or
  + the fused sampler walking a pre-drawn tensor of uniforms by itself), launched in chunks.  The
  ids of a chunk travel to pinned host memory behind the chunk; while the host looks at them the
  next chunk is already running, so the GPU never waits for the stop check or the detokeniser.
  Tokens launched past a stop id are simply not looked at.
* ``stepwise_tokens`` - any object with the reference's forward signature (other model families,
  the dummy models of the host tests): one forward and one selection per requested token, in the
  reference's call pattern (the whole prompt at position 0, then single tokens at P, P+1, ...;
  ohara/inference.py:102-121, ohara/chat_engine.py:388-405).  Being a generator, nothing is
  computed past the token at which the consumer stops.
"""

from __future__ import annotations

from collections import deque
from typing import Callable, Iterator, Sequence

import torch


def supports_device_loop(model) -> bool:
    """True for models that own a device-resident decode loop (``Llama.session``)."""
    return callable(getattr(model, "session", None)) and callable(getattr(model, "supports_persistent", None))


class DeviceLoop:
    """One reusable single-sequence decode session per (model, selection rule).

    Building a session allocates the KV caches, captures a graph and, for the persistent kernel,
    sets up its workspace; a chat engine answers many requests with the same rule, so the session is
    kept and restarted.  The sampling parameters are baked into the captured graph: another
    temperature / top-k / top-p means another session (the previous one is dropped)."""

    FIRST_CHUNK = 4    # tokens of the first chunk (short: the first text appears early)
    MAX_CHUNK = 32     # later chunks double up to this many

    def __init__(self, model, valid_vocab: int = 0):
        self.model = model
        self.valid_vocab = int(valid_vocab)
        self._key = None
        self.session = None
        self._pinned = None
        self._pinned_err = None
        self._busy = False

    def _rule_key(self, sampling):
        if sampling is None or sampling.temperature <= 0:
            return None
        return (float(sampling.temperature), int(sampling.top_k), float(sampling.top_p))

    def _get_session(self, sampling):
        key = self._rule_key(sampling)
        if self.session is None or key != self._key:
            cap = self.model.config.max_sequence_length
            self.session = self.model.session(1, cap, self.valid_vocab, sampling=sampling if key else None)
            self._key = key
            self._pinned = torch.empty(cap, dtype=torch.int64, pin_memory=True)
            self._pinned_err = torch.zeros(4, dtype=torch.int32, pin_memory=True)
        return self.session

    def tokens(self, prompt_ids: Sequence[int], limit: int, sampling=None, u: torch.Tensor | None = None,
               generator: torch.Generator | None = None) -> Iterator[int]:
        """Up to ``limit`` ids after ``prompt_ids``.  ``u``: (limit,) uniform draws, one per token
        (drawn from ``generator`` / the global generator when omitted); ignored when greedy."""
        model = self.model
        if limit < 1:
            return
        if self._busy:
            # one session, one KV cache (the reference serialises requests with a lock for the same
            # reason, ohara/webui/server.py:143-147): a second generation would restart the session
            # under the first one's feet
            raise RuntimeError("this engine is still generating: finish or close the previous stream first")
        self._busy = True
        try:
            yield from self._tokens(prompt_ids, limit, sampling, u, generator)
        finally:
            self._busy = False

    def _tokens(self, prompt_ids, limit, sampling, u, generator) -> Iterator[int]:
        model = self.model
        sess = self._get_session(sampling)
        draws = None
        if sess.sampling is not None:
            if u is None:
                gdev = generator.device if generator is not None else model.device
                u = torch.rand(limit, generator=generator, device=gdev, dtype=torch.float32)
            if u.numel() < limit:
                raise ValueError("u must hold one uniform draw per generated token")
            draws = u.reshape(-1)[:limit].to(device=model.device, dtype=torch.float32).view(limit, 1)
        sess.restart(draws)
        prompt = torch.as_tensor(list(prompt_ids), dtype=torch.int64).view(1, -1)
        sess.prefill(prompt)  # produces token 0
        history, pinned, pinned_err = sess.history, self._pinned, self._pinned_err
        err_word = sess.error_word()  # device view of the persistent kernel's sticky error word, or None
        inflight: deque = deque()  # (first, last, slot, event) of chunks whose ids are on their way to the host
        launched, chunk, nchunks = 1, self.FIRST_CHUNK, 0

        def ship(first: int, last: int) -> None:
            # the error word travels with every chunk: the usual consumer stops at a stop id and never
            # drains the generator, so a check after the last chunk would not run
            nonlocal nchunks
            slot = nchunks % pinned_err.numel()
            nchunks += 1
            pinned[first:last].copy_(history[first:last, 0], non_blocking=True)
            if err_word is not None:
                pinned_err[slot : slot + 1].copy_(err_word, non_blocking=True)
            ev = torch.cuda.Event()
            ev.record()
            inflight.append((first, last, slot, ev))

        ship(0, 1)
        while inflight:
            # keep one chunk running behind the one the host is about to read
            if launched < limit and len(inflight) < 2:
                n = min(chunk, limit - launched)
                sess.run(n)
                ship(launched, launched + n)
                launched += n
                chunk = min(2 * chunk, self.MAX_CHUNK)
            first, last, slot, ev = inflight.popleft()
            ev.synchronize()
            if err_word is not None and int(pinned_err[slot]) != 0:
                torch.cuda.current_stream().synchronize()  # the chunk launched behind this one
                sess.reset_error()  # the barrier counters are mixed after an expiry: start them over
                raise RuntimeError("persistent decode kernel: a grid barrier wait expired")
            for tok in pinned[first:last].tolist():
                yield tok


def stepwise_tokens(model, prompt_ids: Sequence[int], limit: int, select: Callable[[torch.Tensor, int], torch.Tensor],
                    device, cache=None, use_cache: bool = True, last_only: bool | None = None) -> Iterator[int]:
    """One forward and one ``select(logits, step)`` per token.  With a cache the model sees the whole
    prompt at position 0 and then single tokens; without one it sees the growing sequence every time
    (ohara/inference.py:111-114)."""
    seq = torch.as_tensor(list(prompt_ids), dtype=torch.long, device=device).view(1, -1)
    if last_only is None:
        last_only = bool(getattr(model, "supports_last_only", False))
    feed, position = seq, 0
    for step in range(limit):
        if use_cache:
            logits = model(feed, cache, position, last_only=True) if last_only else model(feed, cache, position)
            position += feed.size(1)
        else:
            logits = model(seq)
        nxt = select(logits, step).reshape(1, 1).to(device)
        if use_cache:
            feed = nxt
        else:
            seq = torch.cat((seq, nxt), dim=-1)
        yield int(nxt.item())


class ReplyText:
    """Incremental detokenisation of a growing reply: the whole reply is decoded after every token
    and only the new tail is handed out, because a single token need not be valid text on its own
    (ohara/chat_engine.py:407-412)."""

    def __init__(self, tokenizer):
        self.tokenizer = tokenizer
        self.ids: list[int] = []
        self.text = ""

    def push(self, token_id: int) -> str:
        self.ids.append(token_id)
        text = self.tokenizer.decode(self.ids, skip_special_tokens=True)
        if len(text) <= len(self.text):
            return ""
        new, self.text = text[len(self.text):], text
        return new
