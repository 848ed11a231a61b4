"""``Inference`` with the reference's call surface (ohara/inference.py:10-127): prefill the
prompt, then one token per call through the KV cache, sampling on the device."""

from __future__ import annotations

import time

import torch

from . import sampling


class Inference:
    def __init__(self, model, tokenizer, device=None, temperature: float = 1.0, top_p: float = 0.0,
                 max_new_tokens: int = 500, use_kv_cache: bool = True, sampler_fn=None):
        # ohara/inference.py:11-35
        if device is None:
            device = torch.device("cuda" if torch.cuda.is_available() else "cpu")
        elif not isinstance(device, torch.device):
            device = torch.device(device)
        self.device = device
        self.model = model.to(self.device).eval()
        self.tokenizer = tokenizer
        self.default_temperature = temperature
        self.default_top_p = top_p
        self.max_new_tokens = max_new_tokens
        self.use_kv_cache = use_kv_cache
        # the sampler is the HIP kernel; a caller may inject another callable with the same
        # signature (logits, temperature=, top_p=) -> (B, 1) ids
        self._sampler = sampler_fn if sampler_fn is not None else sampling.inference_sampler
        if self.use_kv_cache and hasattr(self.model, "build_kv_cache"):
            self.kv_cache = self.model.build_kv_cache()
        else:
            self.kv_cache = None

    @staticmethod
    def sampler(logits, temperature=1, top_p=0.0) -> torch.Tensor:
        """ohara/inference.py:37-65 on the fused HIP sampler."""
        return sampling.inference_sampler(logits, temperature=temperature, top_p=top_p)

    def _forward(self, inputs, cache, pos):
        if getattr(self.model, "supports_last_only", False):
            return self.model(inputs, cache, pos, last_only=True)
        return self.model(inputs, cache, pos)

    def generate(self, prompt: str, temperature=None, top_p=None, max_new_tokens=None, stream: bool = True):
        """ohara/inference.py:67-127: same validation order, context clamp, call pattern
        (prefill at position 0, then single tokens), eos handling and return value."""
        if temperature is None:
            temperature = self.default_temperature
        if top_p is None:
            top_p = self.default_top_p
        if max_new_tokens is None:
            max_new_tokens = self.max_new_tokens
        if max_new_tokens < 0:
            raise ValueError("max_new_tokens cannot be negative")
        if self.use_kv_cache and hasattr(self.model, "build_kv_cache"):
            self.kv_cache = self.model.build_kv_cache()
        else:
            self.kv_cache = None
        token_ids = self.tokenizer.encode(prompt)
        if not token_ids:
            raise ValueError("prompt must encode to at least one token")
        inputs = torch.tensor(token_ids, dtype=torch.long, device=self.device).reshape(1, -1)
        model_config = getattr(self.model, "config", None)
        max_sequence_length = getattr(model_config, "max_sequence_length", None)
        if max_sequence_length is not None:
            if inputs.size(1) > max_sequence_length:
                raise ValueError("prompt exceeds model max_sequence_length")
            max_new_tokens = min(max_new_tokens, max(0, max_sequence_length - inputs.size(1)))

        generated = inputs
        model_inputs = inputs
        input_pos = 0
        start_time = time.time()
        with torch.no_grad():
            if stream:
                print(self.tokenizer.decode(generated.tolist()[0]), end="")
            for _ in range(max_new_tokens):
                if self.use_kv_cache:
                    logits = self._forward(model_inputs, self.kv_cache, input_pos)
                else:
                    logits = self.model(generated)
                next_token = self._sampler(logits, temperature=temperature, top_p=top_p)
                next_token = next_token.to(generated.device)
                if next_token.item() == self.tokenizer.eos_token_id:
                    break
                generated = torch.cat((generated, next_token), dim=-1)
                if self.use_kv_cache:
                    input_pos += model_inputs.size(1)
                    model_inputs = next_token
                if stream:
                    print(self.tokenizer.decode([next_token.item()]), end="", flush=True)
            end_time = time.time()
        if stream:
            print(f"\nTime: {end_time - start_time}s")
        return self.tokenizer.decode(generated.squeeze(0).tolist())
