"""Token sampling with the reference's call surface (ohara/chat_engine.py:33-82,
ohara/inference.py:37-65) over the fused HIP sampler.

``torch.multinomial`` cannot be reproduced from a seed by another implementation, so
the stochastic step is inverse-CDF sampling driven by one uniform draw per row: either
supplied by the caller (``u=``, the parity path) or drawn from ``generator`` / the
global RNG with ``torch.rand`` (so a seeded generator still gives reproducible tokens).
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from . import ops


@dataclass
class SamplingConfig:
    """ohara/chat_engine.py:33-48, same defaults and validation."""

    temperature: float = 0.8
    top_p: float = 0.95
    top_k: int = 0
    max_new_tokens: int = 512

    def __post_init__(self) -> None:
        if self.temperature < 0:
            raise ValueError("temperature cannot be negative")
        if not 0.0 <= self.top_p <= 1.0:
            raise ValueError("top_p must be in [0, 1]")
        if self.top_k < 0:
            raise ValueError("top_k cannot be negative")
        if self.max_new_tokens < 1:
            raise ValueError("max_new_tokens must be at least 1")


def _device_logits(logits: torch.Tensor) -> torch.Tensor:
    last = logits[:, -1]
    if not last.is_cuda:
        if not torch.cuda.is_available():
            raise RuntimeError("ohara_amd samples on the GPU only (no CPU fallback)")
        last = last.cuda()
    if last.dtype not in (torch.bfloat16, torch.float32):
        last = last.float()
    return last.contiguous()


def _draw(batch: int, device, u, generator) -> torch.Tensor:
    if u is not None:
        return u.to(device=device, dtype=torch.float32).reshape(batch).contiguous()
    gdev = generator.device if generator is not None else device
    return torch.rand(batch, generator=generator, device=gdev, dtype=torch.float32).to(device)


def sample_next_token(logits: torch.Tensor, config: SamplingConfig, generator: torch.Generator | None = None,
                      *, u: torch.Tensor | None = None, valid_vocab: int | None = None) -> torch.Tensor:
    """ohara/chat_engine.py:51-82: logits (B, S, V) -> token ids (B, 1) int64 on the
    logits' device.  ``temperature == 0`` is greedy (first index of the maximum)."""
    src_device = logits.device
    last = _device_logits(logits)
    if config.temperature == 0:
        out = greedy(last, valid_vocab)
    else:
        uu = _draw(last.shape[0], last.device, u, generator)
        out = ops.sample_topk_topp(last, config.temperature, config.top_k, config.top_p, uu, valid_vocab)
    return out.view(-1, 1).to(src_device)


def _greedy_fp32(last: torch.Tensor, valid_vocab) -> torch.Tensor:
    u = torch.zeros(last.shape[0], dtype=torch.float32, device=last.device)
    # temperature 1, top-k 1: candidates = all ids tied at the maximum; vocabulary-order
    # inverse CDF at u = 0 returns the lowest such id = torch.argmax's answer.
    return ops.sample_topk_topp(last, 1.0, 1, 1.0, u, valid_vocab)


def greedy(logits_last: torch.Tensor, valid_vocab: int | None = None) -> torch.Tensor:
    if logits_last.dtype == torch.bfloat16:
        return ops.argmax(logits_last, valid_vocab)
    return _greedy_fp32(logits_last, valid_vocab)


def inference_sampler(logits: torch.Tensor, temperature=1, top_p=0.0, *, u=None) -> torch.Tensor:
    """Inference.sampler (ohara/inference.py:37-65): nucleus only; greedy both for
    ``temperature <= 0`` and for the default ``temperature == 1 and top_p <= 0``."""
    src_device = logits.device
    last = _device_logits(logits)
    if temperature <= 0 or (temperature == 1 and top_p <= 0):
        out = greedy(last)
    else:
        uu = _draw(last.shape[0], last.device, u, None)
        p = top_p if 0 < top_p < 1 else 1.0
        out = ops.sample_topk_topp(last, float(temperature), 0, p, uu)
    return out.view(-1, 1).to(src_device)
