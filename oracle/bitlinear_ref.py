"""CPU restatement of BitNet-b1.58 BitLinear with real integer arithmetic.
TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

The reference (experiments/bitnet/bitnet.py:29-59) is float fake-quantisation:

    x_hat = RMSNorm_in(x)                                   (:49,53)
    s     = 127 / clamp(max|x_hat|, 1e-5)   per token       (:31)
    x_q   = clamp(round(x_hat * s), -128, 127) / s          (:32)
    g     = 1 / clamp(mean|W|, 1e-5)        per tensor      (:38)
    W_q   = clamp(round(W * g), -1, 1) / g                  (:39)
    y     = linear(x_q, W_q / max|W_q|) * max|W_q|          (:41-43,58-59), bias dropped

Its effective integer semantics, which this file states directly:

    T   = clamp(round(W * g), -1, 1)           in {-1,0,1}
    q   = clamp(round(x_hat * s), -128, 127)   int8
    acc = sum_k q[k] * T[n,k]                  int32   <- bit-exact contract
    y   = (float(acc) / s) * gamma,  gamma = clamp(mean|W|, 1e-5)

``torch.round`` rounds half to even; quantisation multiplies by the reciprocal.
Scales are computed in fp32 from the (model-dtype) normalised activations.

Packed weight format ("row-major 2-bit"): code = T + 1 in {0,1,2}; byte j of row n
holds columns 4j..4j+3, column 4j+i in bits [2i, 2i+2).
"""

from __future__ import annotations

import numpy as np
import torch

from .llama_ref import rms_norm


def weight_ternarize(w: torch.Tensor):
    """bitnet.py:37-43 -> (T int8 (N,K), gamma fp32 scalar)."""
    wf = w.float()
    gamma = wf.abs().mean().clamp(min=1e-5)
    g = 1.0 / gamma
    t = (wf * g).round().clamp(-1, 1).to(torch.int8)
    return t, gamma


def activation_quant(x_hat: torch.Tensor):
    """bitnet.py:30-33 -> (q int8 (..., K), s fp32 (..., 1))."""
    xf = x_hat.float()
    s = 127.0 / xf.abs().amax(dim=-1, keepdim=True).clamp(min=1e-5)
    q = (xf * s).round().clamp(-128, 127).to(torch.int8)
    return q, s


def pack_ternary(t: torch.Tensor) -> torch.Tensor:
    """(N,K) int8 in {-1,0,1}, K % 4 == 0 -> (N, K/4) uint8, format in the header."""
    code = (t.to(torch.int16) + 1).to(torch.uint8).numpy()
    n, k = code.shape
    assert k % 4 == 0
    c = code.reshape(n, k // 4, 4)
    packed = c[..., 0] | (c[..., 1] << 2) | (c[..., 2] << 4) | (c[..., 3] << 6)
    return torch.from_numpy(packed.astype(np.uint8))


def unpack_ternary(packed: torch.Tensor) -> torch.Tensor:
    p = packed.numpy()
    n, kb = p.shape
    out = np.empty((n, kb, 4), dtype=np.int8)
    for i in range(4):
        out[..., i] = ((p >> (2 * i)) & 3).astype(np.int8) - 1
    return torch.from_numpy(out.reshape(n, kb * 4))


def int_accumulate(q: torch.Tensor, t: torch.Tensor, force_int: bool = False) -> torch.Tensor:
    """(M,K) int8 x (N,K) int8 -> (M,N) int32, exact.

    For ternary ``t`` every partial sum is an integer of magnitude <= 128 * K; below 2**24 such
    integers and their sums are exact in fp32 whatever the order of the additions, so the fp32
    BLAS product gives the int32 result bit for bit (and is ~50x faster on a CPU).  Larger K, or
    ``force_int``, uses the int32 product; tests/test_oracle.py checks the two against each other."""
    k = q.shape[-1]
    if not force_int and 128 * k < (1 << 24) and int(t.abs().max()) <= 1:
        return (q.float() @ t.float().t()).to(torch.int32)
    return (q.to(torch.int32) @ t.to(torch.int32).t()).to(torch.int32)


def bitlinear_forward(x: torch.Tensor, norm_w: torch.Tensor, t: torch.Tensor, gamma, return_acc=False):
    """BitLinear.forward (bitnet.py:51-59) on pre-ternarised weights.
    x: (M, K) in the model dtype.  Returns y (M, N) in x's dtype (and acc int32)."""
    x_hat = rms_norm(x, norm_w)
    q, s = activation_quant(x_hat)
    acc = int_accumulate(q, t)
    y = ((acc.float() / s) * float(gamma)).to(x.dtype)
    return (y, acc, q, s) if return_acc else y


def fake_quant_forward(x: torch.Tensor, norm_w: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """The reference's float formulation, restated line by line in fp32
    (bitnet.py:29-59), used to pin the integer formulation against it."""
    xf = rms_norm(x.float(), norm_w.float())
    s = 127.0 / xf.abs().amax(dim=-1, keepdim=True).clamp(min=1e-5)
    xq = (xf * s).round().clamp(-128, 127) / s
    g = 1.0 / w.float().abs().mean().clamp(min=1e-5)
    wq = (w.float() * g).round().clamp(-1, 1) / g
    sc = wq.abs().max()
    return (xq @ (wq / sc).t()) * sc


BIT_TARGETS = ("attn.key", "attn.query", "attn.value", "attn.proj", "ff.gate", "ff.up", "ff.down")


def init_ternary_weights(cfg, seed: int = 2, dtype=torch.bfloat16, gamma: float = 0.02) -> dict:
    """Weights of a ternary Llama: the seven per-layer Linears hold T ~ uniform{-1,0,1}
    (int8) with a per-tensor fp32 scale and a unit BitLinear RMSNorm weight; embedding,
    norms and LM head stay in ``dtype`` (the reference's target list names only the
    per-layer projections, experiments/bitnet/train_bitnet.py:240)."""
    from .llama_ref import init_weights, weight_names

    w = init_weights(cfg, seed=seed, dtype=dtype)
    g = torch.Generator().manual_seed(seed + 1000)
    for name, shape, _ in weight_names(cfg):
        base = name[: -len(".weight")] if name.endswith(".weight") else None
        if base is None or not any(base.endswith(t) for t in BIT_TARGETS):
            continue
        del w[name]
        w[base + ".ternary"] = torch.randint(-1, 2, shape, generator=g, dtype=torch.int8)
        w[base + ".gamma"] = torch.tensor(gamma, dtype=torch.float32)
        w[base + ".rms_norm.weight"] = torch.ones(shape[1], dtype=dtype)
    return w
