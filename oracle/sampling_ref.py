"""CPU restatement of the reference's token samplers and generate loops.
TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

``torch.multinomial`` cannot be reproduced from a uniform draw, so for parity
both the oracle and the fused kernel consume a caller-supplied ``u`` in [0,1) by
inverse CDF over the distribution the reference hands to ``multinomial``:
the filtered, renormalised, descending-sorted probabilities when nucleus
filtering is active (chat_engine.py:72-81), the vocabulary-ordered probabilities
otherwise (chat_engine.py:82).  ``torch.sort`` leaves the order of equal
probabilities unspecified; oracle and kernel both order ties lowest id first.
"""

from __future__ import annotations

import torch


def _inverse_cdf(p: torch.Tensor, u: torch.Tensor):
    """p: (B, n) non-negative, sums to ~1 per row; u: (B,) in [0,1).
    Returns (choice (B,), margin (B,)) - choice = first j with cdf[j] > u
    (clamped to the last entry with p > 0); margin = distance from u to the
    nearest CDF boundary, which tells a test how fragile the draw is against
    last-ulp differences in the summation order.  CDF in fp64.
    """
    cdf = torch.cumsum(p.double(), dim=-1)
    total = cdf[:, -1:]
    cdf = cdf / total
    ud = u.double().unsqueeze(-1)
    choice = (cdf <= ud).sum(dim=-1)
    last = (p > 0).long().cumsum(-1).argmax(-1)  # last index with p > 0
    choice = torch.minimum(choice, last)
    margin = (cdf - ud).abs().min(dim=-1).values
    return choice, margin


def sample_next_token_ref(logits, temperature=0.8, top_p=0.95, top_k=0, u=None, generator=None,
                          valid_vocab=None, return_margin=False):
    """chat_engine.py:51-82 (+ the padded-vocabulary mask of :398-399 when
    ``valid_vocab`` is given).  logits: (B, S, V).  Returns (B, 1) int64.
    """
    x = logits[:, -1].float()
    if valid_vocab is not None and valid_vocab < x.size(-1):
        x = x.clone()
        x[:, valid_vocab:] = float("-inf")
    if temperature == 0:
        out = x.argmax(dim=-1, keepdim=True)
        return (out, torch.full((x.size(0),), float("inf"))) if return_margin else out
    x = x / temperature
    if top_k > 0:
        k = min(top_k, x.size(-1))
        thr = torch.sort(x, dim=-1, descending=True).values[:, k - 1 : k]
        x = x.masked_fill(x < thr, float("-inf"))  # ties at the threshold survive
    probs = torch.softmax(x, dim=-1)
    if 0.0 < top_p < 1.0:
        sp, si = torch.sort(probs, dim=-1, descending=True, stable=True)
        cum = torch.cumsum(sp, dim=-1)
        drop = cum - sp > top_p
        sp = sp.masked_fill(drop, 0.0)
        sp = sp / sp.sum(dim=-1, keepdim=True)
        if u is None:
            choice = torch.multinomial(sp, 1, generator=generator)
            margin = torch.full((x.size(0),), float("inf"))
        else:
            choice, margin = _inverse_cdf(sp, u)
            choice = choice.unsqueeze(-1)
        out = torch.gather(si, -1, choice)
    elif u is None:
        out = torch.multinomial(probs, 1, generator=generator)
        margin = torch.full((x.size(0),), float("inf"))
    else:
        choice, margin = _inverse_cdf(probs, u)
        out = choice.unsqueeze(-1)
    return (out, margin) if return_margin else out


def candidate_cdf_ref(logits, temperature, top_p, top_k, valid_vocab=None):
    """Ids in the order the draw walks them and their cumulative distribution (fp64, ends
    at 1): the sorted, filtered, renormalised prefix when nucleus filtering is active
    (chat_engine.py:72-81), the vocabulary-ordered probabilities otherwise (:82).
    logits: (B, S, V).  Returns (ids (B, n), cdf (B, n)); dropped entries have cdf 1."""
    x = logits[:, -1].float()
    if valid_vocab is not None and valid_vocab < x.size(-1):
        x = x.clone()
        x[:, valid_vocab:] = float("-inf")
    x = x / temperature
    if top_k > 0:
        k = min(top_k, x.size(-1))
        thr = torch.sort(x, dim=-1, descending=True).values[:, k - 1 : k]
        x = x.masked_fill(x < thr, float("-inf"))
    probs = torch.softmax(x, dim=-1)
    if 0.0 < top_p < 1.0:
        sp, si = torch.sort(probs, dim=-1, descending=True, stable=True)
        cum = torch.cumsum(sp, dim=-1)
        sp = sp.masked_fill(cum - sp > top_p, 0.0)
    else:
        sp, si = probs, torch.arange(probs.size(-1)).expand_as(probs)
    cdf = torch.cumsum(sp.double(), dim=-1)
    return si, cdf / cdf[:, -1:]


def kept_set_ref(logits_row: torch.Tensor, temperature, top_p, top_k):
    """The candidate ids and renormalised probabilities the reference would hand
    to multinomial for one row, in fp64, by direct loops (small V only).  A second,
    independent statement of chat_engine.py:65-81 used to pin the vectorised one.
    """
    V = logits_row.numel()
    x = [float(v) / temperature for v in logits_row.float().tolist()]
    if top_k > 0:
        k = min(top_k, V)
        thr = sorted(x, reverse=True)[k - 1]
        x = [v if v >= thr else float("-inf") for v in x]
    m = max(x)
    import math

    e = [math.exp(v - m) if v != float("-inf") else 0.0 for v in x]
    z = sum(e)
    p = [v / z for v in e]
    order = sorted(range(V), key=lambda i: (-p[i], i))
    kept, cum = [], 0.0
    if 0.0 < top_p < 1.0:
        for i in order:
            if cum > top_p:  # cumulative mass *before* this token already exceeds p
                break
            kept.append(i)
            cum += p[i]
    else:
        kept = [i for i in range(V) if p[i] > 0]
    z2 = sum(p[i] for i in kept)
    return kept, [p[i] / z2 for i in kept]


def inference_sampler_ref(logits, temperature=1, top_p=0.0, u=None):
    """inference.py:37-65: nucleus only, no fp32 upcast, greedy both for
    ``temperature <= 0`` and for the default ``temperature == 1 and top_p <= 0``."""
    x = logits[:, -1]
    if temperature <= 0 or (temperature == 1 and top_p <= 0):
        return torch.argmax(x, dim=-1, keepdim=True)
    x = x / temperature
    probs = torch.softmax(x, dim=-1)
    if top_p <= 0 or top_p >= 1:
        if u is None:
            return torch.multinomial(probs.float(), 1)
        return _inverse_cdf(probs.float(), u)[0].unsqueeze(-1)
    sp, si = torch.sort(probs, dim=-1, descending=True, stable=True)
    cum = torch.cumsum(sp, dim=-1)
    sp = sp.masked_fill(cum - sp > top_p, 0.0)
    sp = sp / sp.sum(dim=-1, keepdim=True)
    if u is None:
        choice = torch.multinomial(sp.float(), 1)
    else:
        choice = _inverse_cdf(sp.float(), u)[0].unsqueeze(-1)
    return torch.gather(si, -1, choice)


def greedy_decode_ref(model, prompt_ids: torch.Tensor, steps: int, return_logits: bool = False):
    """Prefill once at position 0, then one token per step with a scalar position
    (chat_engine.py:388-405; inference.py:102-121).  prompt_ids: (B, P) int64.
    Returns generated ids (B, steps) and, optionally, the last-position logits of
    every call (steps, B, V)."""
    B = prompt_ids.size(0)
    cache = model.build_kv_cache(B)
    inp, pos = prompt_ids, 0
    toks, logs = [], []
    for _ in range(steps):
        logits = model(inp, cache, pos)
        pos += inp.size(1)
        nxt = logits[:, -1].float().argmax(dim=-1, keepdim=True)
        toks.append(nxt)
        if return_logits:
            logs.append(logits[:, -1].clone())
        inp = nxt
    out = torch.cat(toks, dim=1)
    return (out, torch.stack(logs)) if return_logits else out


def inference_generate_ref(model, tokenizer, prompt, temperature=1.0, top_p=0.0, max_new_tokens=500,
                           use_kv_cache=True):
    """inference.py:67-127 without the printing: validation order, context clamp,
    prefill-then-one-token call pattern, eos stop (the eos token is not appended)."""
    if max_new_tokens < 0:
        raise ValueError("max_new_tokens cannot be negative")
    cache = model.build_kv_cache() if (use_kv_cache and hasattr(model, "build_kv_cache")) else None
    ids = tokenizer.encode(prompt)
    if not ids:
        raise ValueError("prompt must encode to at least one token")
    inputs = torch.tensor(ids, dtype=torch.long).reshape(1, -1)
    msl = getattr(getattr(model, "config", None), "max_sequence_length", None)
    if msl is not None:
        if inputs.size(1) > msl:
            raise ValueError("prompt exceeds model max_sequence_length")
        max_new_tokens = min(max_new_tokens, max(0, msl - inputs.size(1)))
    generated, model_inputs, pos = inputs, inputs, 0
    for _ in range(max_new_tokens):
        logits = model(model_inputs, cache, pos) if use_kv_cache else model(generated)
        nxt = inference_sampler_ref(logits, temperature=temperature, top_p=top_p)
        if nxt.item() == tokenizer.eos_token_id:
            break
        generated = torch.cat((generated, nxt), dim=-1)
        if use_kv_cache:
            pos += model_inputs.size(1)
            model_inputs = nxt
    return tokenizer.decode(generated.squeeze(0).tolist())
