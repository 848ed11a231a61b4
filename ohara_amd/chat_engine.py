"""``ChatEngine`` with the reference's call surface (ohara/chat_engine.py:248-422): render a
conversation, prefill, then stream decoded text deltas while the model decodes and samples on the
device.  With the kernel-backed dense ``Llama`` a reply is produced by the device-resident loop of
``ohara_amd.generation.DeviceLoop`` (one graph replay per token, ids read back in chunks); other
models are stepped one forward at a time.

Prompt rendering and the chat special tokens belong to the reference's ``ohara.chat``
(host-side string work, not part of the decode path); the engine takes them as
``renderer`` / ``stop_ids`` arguments and falls back to a minimal rendering of the same
turn markers when none is given.
"""

from __future__ import annotations

from typing import Any, Iterator, Mapping, Sequence

import torch

from .generation import DeviceLoop, ReplyText, stepwise_tokens, supports_device_loop
from .sampling import SamplingConfig, sample_next_token

USER_START, USER_END = "<|user_start|>", "<|user_end|>"
ASSISTANT_START, ASSISTANT_END = "<|assistant_start|>", "<|assistant_end|>"


def default_renderer(tokenizer, messages, max_tokens: int = 2048) -> list[int]:
    """The reference's turn layout (ohara/chat.py:154-246) for plain string messages:
    boundary token, <|user_start|>text<|user_end|> / <|assistant_start|>text<|assistant_end|>
    per turn, a trailing assistant turn dropped, then <|assistant_start|>."""
    vocab = tokenizer.get_vocab()
    turns = [dict(m) for m in messages]
    if turns and turns[-1].get("role") == "assistant":
        turns.pop()
    if not turns:
        raise ValueError("conversation has no prompt messages")
    ids: list[int] = []
    boundary = getattr(tokenizer, "bos_token_id", None)
    if boundary is None:
        boundary = tokenizer.eos_token_id
    if boundary is not None:
        ids.append(boundary)
    for m in turns:
        if not isinstance(m.get("content"), str):
            raise ValueError("the built-in renderer handles string messages only; pass renderer=")
        start, end = (USER_START, USER_END) if m["role"] == "user" else (ASSISTANT_START, ASSISTANT_END)
        ids.append(vocab[start])
        ids.extend(tokenizer.encode(m["content"], add_special_tokens=False))
        ids.append(vocab[end])
    ids = ids[:max_tokens]
    ids.append(vocab[ASSISTANT_START])
    return ids


def _window_starts(n_turns: int):
    """Which leading turns to drop, in order, when a conversation does not fit: whole user/assistant
    pairs from the front, and at the very end the last remaining turn before the final one
    (ohara/chat_engine.py:352-366)."""
    start = 0
    while n_turns - start > 0:
        yield start
        start += 2 if n_turns - start > 2 else 1


class ChatEngine:
    """A model plus its tokenizer answering conversations (ohara/chat_engine.py:248-422).

    Additions to the reference's signature, all keyword-only and optional: ``renderer`` (the prompt
    renderer, by default the turn layout of ohara/chat.py), ``stop_ids`` (by default the
    assistant-end marker and the tokenizer's eos), ``sampler_fn`` (a replacement for
    ``sample_next_token``; giving one selects the stepwise path)."""

    def __init__(self, model, tokenizer, *, device=None, dtype=None, renderer=None, stop_ids=None,
                 sampler_fn=None):
        on_gpu = torch.cuda.is_available()
        self.device = torch.device(device if device is not None else ("cuda" if on_gpu else "cpu"))
        self.dtype = dtype if dtype is not None else (torch.bfloat16 if self.device.type == "cuda" else torch.float32)
        # a kernel-backed model accepts only its own device and bfloat16 here and raises otherwise,
        # so self.dtype never misreports what runs
        self.model = model.to(device=self.device, dtype=self.dtype).eval()
        self.tokenizer = tokenizer
        self.renderer = renderer or default_renderer
        vocab = tokenizer.get_vocab() if hasattr(tokenizer, "get_vocab") else {}
        self.assistant_end_id = vocab.get(ASSISTANT_END)
        self.eos_token_id = tokenizer.eos_token_id
        wanted = stop_ids if stop_ids is not None else (self.assistant_end_id, self.eos_token_id)
        self.stop_ids = {int(t) for t in wanted if t is not None}
        # ids at or above the tokenizer's size only pad the vocabulary projection: never sampled
        self.tokenizer_vocab_size = len(tokenizer)
        self.max_sequence_length = model.config.max_sequence_length
        self._sample = sampler_fn
        self._loop = None
        if sampler_fn is None and supports_device_loop(self.model):
            padded = self.model.config.vocab_size > self.tokenizer_vocab_size
            self._loop = DeviceLoop(self.model, self.tokenizer_vocab_size if padded else 0)

    @classmethod
    def from_checkpoint(cls, checkpoint_path, tokenizer, *, device=None, dtype=None, moe_experts_per_tok: int = 2,
                        moe_gate_fn: str = "softmax", moe_normalize_weights: bool = True, renderer=None,
                        stop_ids=None):
        """ohara/chat_engine.py:275-329: architecture from the tensor shapes (or the exported
        ``config.json``), weights into the kernel-backed model.  The tokenizer is passed in (the
        reference rebuilds it from a directory or a hub name, which is outside this path); a
        checkpoint narrower than the tokenizer is rejected as there."""
        from .checkpoint import build_model, load_checkpoint

        config, state = load_checkpoint(checkpoint_path, moe_experts_per_tok=moe_experts_per_tok,
                                        moe_gate_fn=moe_gate_fn, moe_normalize_weights=moe_normalize_weights)
        if config.vocab_size < len(tokenizer):
            raise ValueError(
                f"checkpoint vocabulary ({config.vocab_size:,}) is smaller than the "
                f"tokenizer ({len(tokenizer):,}). Point --tokenizer-dir at the "
                "directory saved next to the checkpoint."
            )
        if device is None:
            device = "cuda"
        model = build_model(config, state, device=device)
        return cls(model, tokenizer, device=device, dtype=dtype, renderer=renderer, stop_ids=stop_ids)

    def metadata(self, checkpoint_path=None) -> dict[str, Any]:
        """The model facts of ohara/chat_engine.py:331-350 (the SFT sidecar file is not read)."""
        cfg = self.model.config
        n_params = 0
        for p in self.model.parameters():
            n_params += p.numel()
        return dict(parameters=n_params, layers=cfg.num_hidden_layers, hidden_size=cfg.hidden_size,
                    heads=cfg.num_attention_heads, context_length=self.max_sequence_length,
                    vocab_size=cfg.vocab_size, device=str(self.device), dtype=str(self.dtype).removeprefix("torch."))

    def render_prompt(self, messages: Sequence[Mapping[str, Any]]) -> list[int]:
        """The rendered conversation, with as many leading turns dropped as it takes to leave room
        for at least one reply token (never part of a turn)."""
        window = self.max_sequence_length
        turns = list(messages)
        for start in _window_starts(len(turns)):
            ids = self.renderer(self.tokenizer, turns[start:], max_tokens=window)
            if len(ids) < window:
                return ids
        raise ValueError("the latest message alone does not fit in the context window")

    def _reply_tokens(self, prompt_ids, budget: int, config: SamplingConfig, seed, u) -> Iterator[int]:
        generator = None if seed is None else torch.Generator(device=self.device).manual_seed(seed)
        if self._loop is not None:
            return self._loop.tokens(prompt_ids, budget, config, u=u, generator=generator)
        sample = self._sample if self._sample is not None else sample_next_token
        limit = self.tokenizer_vocab_size

        def select(logits, step):
            extra = {}
            if logits.size(-1) > limit:  # chat_engine.py:398-399
                if sample is sample_next_token:
                    extra["valid_vocab"] = limit  # masked inside the kernel
                else:
                    logits[..., limit:] = float("-inf")
            if u is not None:
                extra["u"] = u[step: step + 1]
            return sample(logits, config, generator, **extra)

        cache = self.model.build_kv_cache(batch_size=1)
        return stepwise_tokens(self.model, prompt_ids, budget, select, self.device, cache=cache)

    @torch.no_grad()
    def generate_stream(self, messages, config: SamplingConfig | None = None, *, seed: int | None = None,
                        u: torch.Tensor | None = None) -> Iterator[str]:
        """Text deltas of the assistant's reply (ohara/chat_engine.py:368-412).  ``u`` (one uniform
        draw per new token) optionally fixes the sampler's randomness (the parity path); otherwise
        the draws come from a generator seeded with ``seed``, or from the global one."""
        config = config or SamplingConfig()
        prompt_ids = self.render_prompt(messages)
        budget = min(config.max_new_tokens, self.max_sequence_length - len(prompt_ids))
        if budget < 1:
            raise ValueError("no room left in the context window for a reply")
        reply = ReplyText(self.tokenizer)
        for token_id in self._reply_tokens(prompt_ids, budget, config, seed, u):
            if token_id in self.stop_ids:
                return
            piece = reply.push(token_id)
            if piece:
                yield piece

    def generate(self, messages, config: SamplingConfig | None = None, *, seed: int | None = None,
                 u: torch.Tensor | None = None) -> str:
        return "".join(self.generate_stream(messages, config, seed=seed, u=u))
