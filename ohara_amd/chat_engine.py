"""``ChatEngine`` with the reference's call surface (ohara/chat_engine.py:248-422): render a
conversation, prefill, then stream decoded text deltas while sampling on the device.

Prompt rendering and the chat special tokens belong to the reference's ``ohara.chat``
(host-side string work, not part of the decode path); the engine takes them as
``renderer`` / ``stop_ids`` arguments and falls back to a minimal rendering of the same
turn markers when none is given.
"""

from __future__ import annotations

from typing import Any, Iterator, Mapping, Sequence

import torch

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


class ChatEngine:
    def __init__(self, model, tokenizer, *, device=None, dtype=None, renderer=None, stop_ids=None,
                 sampler_fn=None):
        # ohara/chat_engine.py:251-273
        if device is None:
            device = "cuda" if torch.cuda.is_available() else "cpu"
        self.device = torch.device(device)
        if dtype is None:
            dtype = torch.bfloat16 if self.device.type == "cuda" else torch.float32
        self.dtype = dtype
        self.model = model.to(device=self.device, dtype=self.dtype).eval()
        self.tokenizer = tokenizer
        self.renderer = renderer or default_renderer
        vocab = tokenizer.get_vocab() if hasattr(tokenizer, "get_vocab") else {}
        self.assistant_end_id = vocab.get(ASSISTANT_END)
        self.eos_token_id = tokenizer.eos_token_id
        self.stop_ids = set(stop_ids) if stop_ids is not None else {self.assistant_end_id, self.eos_token_id}
        self.stop_ids.discard(None)
        # ids at or above this only pad the vocabulary projection; never sampled
        self.tokenizer_vocab_size = len(tokenizer)
        self.max_sequence_length = model.config.max_sequence_length
        self._sample = sampler_fn if sampler_fn is not None else sample_next_token

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
        # ohara/chat_engine.py:331-350 (without the checkpoint sidecar file)
        cfg = self.model.config
        return {
            "parameters": sum(p.numel() for p in self.model.parameters()),
            "layers": cfg.num_hidden_layers,
            "hidden_size": cfg.hidden_size,
            "heads": cfg.num_attention_heads,
            "context_length": self.max_sequence_length,
            "vocab_size": cfg.vocab_size,
            "device": str(self.device),
            "dtype": str(self.dtype).removeprefix("torch."),
        }

    def render_prompt(self, messages: Sequence[Mapping[str, Any]]) -> list[int]:
        # ohara/chat_engine.py:352-366: drop whole leading turns until the prompt fits
        budget = self.max_sequence_length
        turns = list(messages)
        while turns:
            ids = self.renderer(self.tokenizer, turns, max_tokens=budget)
            if len(ids) < budget:
                return ids
            turns = turns[2:] if len(turns) > 2 else turns[1:]
        raise ValueError("the latest message alone does not fit in the context window")

    def _forward(self, inputs, cache, pos):
        if getattr(self.model, "supports_last_only", False):
            return self.model(inputs, cache, pos, last_only=True)
        return self.model(inputs, cache, pos)

    @torch.no_grad()
    def generate_stream(self, messages, config: SamplingConfig | None = None, *, seed: int | None = None,
                        u: torch.Tensor | None = None) -> Iterator[str]:
        """ohara/chat_engine.py:368-412.  ``u`` (max_new_tokens,) optionally supplies the
        uniform draws (the parity path); otherwise they come from a generator seeded with
        ``seed`` (or the global RNG)."""
        config = config or SamplingConfig()
        prompt_ids = self.render_prompt(messages)
        room = self.max_sequence_length - len(prompt_ids)
        if room < 1:
            raise ValueError("no room left in the context window for a reply")
        max_new_tokens = min(config.max_new_tokens, room)

        generator = None
        if seed is not None:
            generator = torch.Generator(device=self.device).manual_seed(seed)

        kv_cache = self.model.build_kv_cache(batch_size=1)
        tokens = torch.tensor(prompt_ids, dtype=torch.long, device=self.device).view(1, -1)
        model_input = tokens
        position = 0
        produced: list[int] = []
        emitted = ""
        vocab_limit = self.tokenizer_vocab_size

        for step in range(max_new_tokens):
            logits = self._forward(model_input, kv_cache, position)
            position += model_input.size(1)
            kwargs = {}
            if logits.size(-1) > vocab_limit:
                if self._sample is sample_next_token:
                    kwargs["valid_vocab"] = vocab_limit  # masked inside the kernel
                else:
                    logits[..., vocab_limit:] = float("-inf")
            if u is not None:
                kwargs["u"] = u[step : step + 1]
            next_token = self._sample(logits, config, generator, **kwargs)
            token_id = int(next_token.item())
            if token_id in self.stop_ids:
                break
            produced.append(token_id)
            model_input = next_token.to(self.device)

            text = self.tokenizer.decode(produced, skip_special_tokens=True)
            if len(text) > len(emitted):
                yield text[len(emitted):]
                emitted = text

    def generate(self, messages, config: SamplingConfig | None = None, *, seed: int | None = None,
                 u: torch.Tensor | None = None) -> str:
        return "".join(self.generate_stream(messages, config, seed=seed, u=u))
