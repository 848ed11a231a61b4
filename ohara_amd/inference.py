"""``Inference`` with the reference's call surface (ohara/inference.py:10-127): complete a text
prompt token by token.  With the kernel-backed dense ``Llama`` and the KV cache the continuation comes
from the device-resident loop (``ohara_amd.generation.DeviceLoop``: one graph replay per token);
otherwise every token is one forward of the model (with the cache: the prompt once, then single
tokens; without: the growing sequence) and one call of the sampler."""

from __future__ import annotations

import time
from types import SimpleNamespace

import torch

from . import sampling
from .generation import DeviceLoop, stepwise_tokens, supports_device_loop


def _sampler_rule(temperature, top_p):
    """Inference.sampler's selection rule (ohara/inference.py:37-65) as sampler-kernel parameters:
    None = arg-max (temperature <= 0, or the defaults temperature 1 / top_p <= 0); else nucleus
    sampling at ``temperature`` with the whole distribution when top_p is not inside (0, 1)."""
    if temperature <= 0 or (temperature == 1 and top_p <= 0):
        return None
    return SimpleNamespace(temperature=float(temperature), top_k=0, top_p=float(top_p) if 0 < top_p < 1 else 1.0)


class Inference:
    def __init__(self, model, tokenizer, device=None, temperature: float = 1.0, top_p: float = 0.0,
                 max_new_tokens: int = 500, use_kv_cache: bool = True, sampler_fn=None):
        """``sampler_fn``: optional replacement for the HIP sampler with the signature
        ``(logits, temperature=, top_p=) -> (B, 1) ids``; giving one selects the stepwise path."""
        if device is None:
            device = "cuda" if torch.cuda.is_available() else "cpu"
        self.device = torch.device(device)
        self.model = model.to(self.device).eval()
        self.tokenizer = tokenizer
        self.default_temperature, self.default_top_p = temperature, top_p
        self.max_new_tokens = max_new_tokens
        self.use_kv_cache = use_kv_cache
        self._sampler = sampler_fn
        self._has_cache = use_kv_cache and hasattr(self.model, "build_kv_cache")
        self._loop = None
        if sampler_fn is None and self._has_cache and supports_device_loop(self.model):
            self._loop = DeviceLoop(self.model)  # owns its caches; self.kv_cache shows them after a run
        self.kv_cache = self.model.build_kv_cache() if (self._has_cache and self._loop is None) else None

    @staticmethod
    def sampler(logits, temperature=1, top_p=0.0) -> torch.Tensor:
        """ohara/inference.py:37-65 on the fused HIP sampler."""
        return sampling.inference_sampler(logits, temperature=temperature, top_p=top_p)

    def _continuation(self, prompt_ids, budget, temperature, top_p):
        if self._loop is not None:
            return self._loop.tokens(prompt_ids, budget, _sampler_rule(temperature, top_p))
        pick = self._sampler if self._sampler is not None else sampling.inference_sampler

        def select(logits, _step):
            return pick(logits, temperature=temperature, top_p=top_p)

        # Only models that advertise it are asked for the last row of logits alone.
        return stepwise_tokens(self.model, prompt_ids, budget, select, self.device, cache=self.kv_cache,
                               use_cache=self.use_kv_cache)

    @torch.no_grad()
    def generate(self, prompt: str, temperature=None, top_p=None, max_new_tokens=None, stream: bool = True):
        """ohara/inference.py:67-127: the prompt plus up to ``max_new_tokens`` sampled tokens, decoded.
        The budget is clamped to what the model's context window leaves after the prompt; an eos
        token ends the text and is not part of it.  ``stream`` prints the text as it grows."""
        temperature = self.default_temperature if temperature is None else temperature
        top_p = self.default_top_p if top_p is None else top_p
        budget = self.max_new_tokens if max_new_tokens is None else max_new_tokens
        if budget < 0:
            raise ValueError("max_new_tokens cannot be negative")
        if self._loop is None:
            self.kv_cache = self.model.build_kv_cache() if self._has_cache else None
        ids = list(self.tokenizer.encode(prompt))
        if not ids:
            raise ValueError("prompt must encode to at least one token")
        window = getattr(getattr(self.model, "config", None), "max_sequence_length", None)
        if window is not None:
            if len(ids) > window:
                raise ValueError("prompt exceeds model max_sequence_length")
            budget = min(budget, window - len(ids))
        t_start = time.time()
        if stream:
            print(self.tokenizer.decode(ids), end="")
        eos = self.tokenizer.eos_token_id
        for token_id in self._continuation(tuple(ids), budget, temperature, top_p):
            if token_id == eos:
                break
            ids.append(token_id)
            if stream:
                print(self.tokenizer.decode([token_id]), end="", flush=True)
        if self._loop is not None and self._loop.session is not None:
            self.kv_cache = self._loop.session.cache
        if stream:
            print(f"\nTime: {time.time() - t_start}s")
        return self.tokenizer.decode(ids)
