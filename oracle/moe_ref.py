"""CPU restatement of the reference's grouped mixture-of-experts feed-forward
(eval mode).  TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

Follows ohara/modules/moe_grouped.py:122-228 (routing, per-expert loop dispatch,
shared expert); ohara/modules/moe.py:65-127 states the same routing for the loop
variant.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F


def _linear(x, w, f32_cache=None):
    from .llama_ref import linear

    return linear(x, w, f32_cache)


def topk_lowest_index_first(scores: torch.Tensor, k: int) -> torch.Tensor:
    """Indices of the k largest entries per row, descending; equal values are
    ordered lowest index first (torch.topk leaves tie order unspecified; both the
    oracle and the kernels fix it this way)."""
    order = torch.sort(scores, dim=-1, descending=True, stable=True).indices
    return order[..., :k]


def moe_route(flat_x, router_w, router_bias, k: int, gate_fn: str = "softmax",
              normalize_weights: bool = True, quantile_balancing: bool = True, f32_cache=None):
    """moe_grouped.py:122-147.

    Router logits are a Linear in the model dtype, upcast to fp32 (:126).  With
    quantile balancing the experts are the first k of top-(k+1) of
    ``logits + router_bias`` (:129-133); the weights come from the *unbiased*
    logits of the selected experts (:140): softmax over the k selected, or
    sigmoid (optionally normalised, :144-146).
    Returns (expert_indices (N,k) int64, weights (N,k) fp32, logits (N,E) fp32).
    """
    logits = _linear(flat_x, router_w, f32_cache).float()
    if quantile_balancing:
        biased = logits + router_bias
        idx = topk_lowest_index_first(biased, k + 1)[:, :k]
    else:
        idx = topk_lowest_index_first(logits, k)
    selected = logits.gather(-1, idx)
    if gate_fn == "softmax":
        weights = selected.softmax(dim=-1)
    else:
        weights = torch.sigmoid(selected)
        if normalize_weights:
            weights = weights / weights.sum(dim=-1, keepdim=True).clamp_min(1e-9)
    return idx, weights, logits


def moe_dispatch(flat_x, idx, weights, w_gate, w_up, w_down, f32_cache=None):
    """Per-expert loop, moe_grouped.py:187-204.

    Expert weights are stored (E, in, out) - applied as ``x @ w[e]`` (no transpose).
    Each expert's output is multiplied by the routing weight *after* the down
    projection, in the activation dtype (:199-201), and scatter-added into the
    output in the activation dtype in ascending expert order (:203).
    """
    N, dim = flat_x.shape
    k = idx.shape[1]
    out = torch.zeros_like(flat_x)
    flat_idx = idx.reshape(-1)
    flat_w = weights.to(flat_x.dtype).reshape(-1)  # cast before use, moe_grouped.py:217
    rows = torch.arange(N * k) // k
    for e in range(w_gate.shape[0]):
        m = flat_idx == e
        if not bool(m.any()):
            continue
        tr = rows[m]
        xe = flat_x[tr]
        g = _linear(xe, w_gate[e].t(), f32_cache)
        u = _linear(xe, w_up[e].t(), f32_cache)
        hidden = F.silu(g) * u
        ye = _linear(hidden, w_down[e].t(), f32_cache) * flat_w[m].unsqueeze(-1)
        out.index_add_(0, tr, ye)
    return out


def moe_forward(x, router_w, router_bias, w_gate, w_up, w_down, k, gate_fn="softmax",
                normalize_weights=True, quantile_balancing=True, shared=None, f32_cache=None):
    """GroupedMoE.forward in eval mode - moe_grouped.py:209-228."""
    B, S, dim = x.shape
    flat_x = x.reshape(B * S, dim)
    idx, weights, _ = moe_route(flat_x, router_w, router_bias, k, gate_fn, normalize_weights,
                                quantile_balancing, f32_cache)
    out = moe_dispatch(flat_x, idx, weights, w_gate, w_up, w_down, f32_cache)
    if shared is not None:
        sg, su, sd = shared
        # moe_grouped.py:206-207,219-220
        out = out + _linear(F.silu(_linear(flat_x, sg, f32_cache)) * _linear(flat_x, su, f32_cache), sd, f32_cache)
    return out.view(B, S, dim)
