"""Loader of the committed golden fixtures (tests/golden/*.pt): plain tensors, read with
``weights_only=True``; a value ``"=<key>"`` stands for the tensor stored under that key."""

import os

import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load_fixture(name: str) -> dict:
    fx = torch.load(os.path.join(GOLDEN, name), weights_only=True)
    for k, v in list(fx.items()):
        if isinstance(v, str) and v.startswith("="):
            fx[k] = fx[v[1:]]
    return fx


def weight_checksum(w: dict) -> torch.Tensor:
    """The fingerprint tests/golden/make_llama_bf16_golden.py stores for seeded weights."""
    names = sorted(k for k in w if not k.startswith("freq_"))
    return torch.tensor([[w[k].double().sum().item(), w[k].double().pow(2).sum().item()] for k in names],
                        dtype=torch.float64).sum(0)


def identical_fraction(a: torch.Tensor, b: torch.Tensor) -> float:
    """Share of bit-identical elements of two bf16 tensors."""
    assert a.shape == b.shape and a.dtype == b.dtype == torch.bfloat16
    return (a.contiguous().view(torch.int16) == b.contiguous().view(torch.int16)).float().mean().item()


def bf16_ulps(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """|a - b| in units of the bf16 spacing at max(|a|, |b|)."""
    af, bf = a.float(), b.float()
    mag = torch.maximum(af.abs(), bf.abs()).clamp_min(2.0 ** -120)
    ulp = torch.exp2(torch.floor(torch.log2(mag)) - 7)
    return (af - bf).abs() / ulp


def reference_self_distance(fx: dict) -> float:
    """How far the reference reproduces ITSELF on this fixture's model: the largest per-row mean
    |logit difference| (over the row's max |logit|) between its run with all threads and its repeats
    (one thread; the library's other matrix kernels), over every stored row."""
    worst = 0.0
    for tag in ("one_thread", "other_kernels"):
        if "logits_at_columns" in fx:  # the greedy d12 run: (steps, columns), scale stored per step
            pairs = [(fx["logits_at_columns"], fx[f"logits_at_columns_{tag}"], fx["logit_absmax"].float())]
        else:
            pairs = [(fx[k], fx[f"{k}_{tag}"], None) for k in fx
                     if k.startswith("logits_") and not k.endswith(("one_thread", "other_kernels")) and f"{k}_{tag}" in fx]
        for a, b, scale in pairs:
            a, b = a.float(), b.float()
            if scale is None:
                scale = a.abs().amax(-1)
            worst = max(worst, ((a - b).abs().mean(-1) / scale).max().item())
    return worst
