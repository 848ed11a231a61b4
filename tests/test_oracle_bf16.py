"""Pins of the oracle's bf16 arithmetic: the reference model cast to bf16 as ChatEngine casts it
(ohara/chat_engine.py:262-265), run on the CPU (fixtures tests/golden/llama_bf16_*.pt, written by
tests/golden/make_llama_bf16_golden.py), and the library routine its attention calls
(F.scaled_dot_product_attention, ohara/models/llama.py:116-123), called here directly.

Two kinds of statement are made.  Operator by operator, on the reference's own operands, the oracle
returns the reference's bits (a Linear: all but a few elements in ten thousand, where the library sums
in another order).  Through a whole model those few flipped bits travel: the logits of two runs of the
REFERENCE ITSELF - with all threads, with one, with the library's other matrix kernels - share only
15 % of their bit patterns at the d12 widths and lie 2.1-3.1e-3 of the logit scale apart on average.
The fixtures hold these runs, and the oracle is asked to lie as close to the reference as the
reference lies to itself (1.25 x the largest distance between two of its own runs).
"""

import dataclasses
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import llama_ref as R

from _fixtures import bf16_ulps, identical_fraction, load_fixture, reference_self_distance, weight_checksum

BF = torch.bfloat16


def _cfg(d):
    fields = {f.name for f in dataclasses.fields(R.RefConfig)}
    return R.RefConfig(**{k: v for k, v in d.items() if k in fields})


def _rel(a, b):
    d = (a.float() - b.float()).abs()
    scale = b.float().abs().max().item()
    return d.max().item() / scale, d.mean().item() / scale


# ---- the exponential and the attention kernel of the library ------------------------------------


def test_fexp_u20_is_the_library_kernels_exponential():
    # (a) it is an exponential, to the accuracy its authors state
    x = torch.linspace(-20.0, 0.0, 200001)
    err = ((R.fexp_u20(x).double() - torch.exp(x.double())).abs() / torch.exp(x.double())).max().item()
    assert err < 1.2e-4
    assert R.fexp_u20(torch.tensor([-200.0, float("-inf")])).tolist() == [0.0, 0.0]
    # (b) it is THAT exponential: with V = identity the library's output is bf16(bf16(p_j) / l), which
    # exposes every weight's bits.  The exact exponential matches 99.3 % of them, this one all.
    g = torch.Generator().manual_seed(0)
    H, L = 16, 256
    q = torch.randn(1, H, 1, L, generator=g).to(BF)
    k = torch.randn(1, H, L, L, generator=g).to(BF)
    v = torch.eye(L).to(BF)[None, None].expand(1, H, L, L).contiguous()
    lib = F.scaled_dot_product_attention(q, k, v, attn_mask=torch.ones(1, L, dtype=torch.bool))
    s = (q.float() @ k.float().transpose(-1, -2)) * torch.tensor(1 / math.sqrt(L))
    m = s.amax(-1, keepdim=True)

    def weights_as_output(ex):
        p = ex(s - m)
        return (p.to(BF).float() * (1.0 / p.sum(-1, keepdim=True))).to(BF)

    assert identical_fraction(weights_as_output(R.fexp_u20), lib) == 1.0
    assert identical_fraction(weights_as_output(torch.exp), lib) < 0.999


@pytest.mark.parametrize("B,H,Hkv,S,L,D", [
    (2, 4, 2, 1, 40, 64),      # one cached step, GQA
    (1, 6, 6, 1, 1100, 128),   # d12 head shape, three key blocks
    (2, 6, 6, 1, 4000, 128),   # the full cache
    (1, 8, 2, 300, 1300, 64),  # many queries over a longer cache
    (2, 4, 4, 5, 5, 16),       # tiny prefill
    (1, 2, 1, 700, 700, 64),   # prefill across a key-block boundary
])
def test_attention_bf16_reproduces_the_library_routine(B, H, Hkv, S, L, D):
    g = torch.Generator().manual_seed(L + S)
    q = torch.randn(B, S, H, D, generator=g).to(BF)
    k = torch.randn(B, L, Hkv, D, generator=g).to(BF)
    v = torch.randn(B, L, Hkv, D, generator=g).to(BF)
    start = L - S
    got = R.attention_core(q, k, v, start)
    grp = H // Hkv
    mask = torch.arange(L)[None, :] <= (start + torch.arange(S))[:, None]  # llama.py:109-113
    kk, vv = (t.transpose(1, 2).repeat_interleave(grp, 1) for t in (k, v))  # llama.py:101-107
    lib = F.scaled_dot_product_attention(q.transpose(1, 2), kk, vv, attn_mask=mask, is_causal=False)
    lib = lib.transpose(1, 2).reshape(B, S, H * D)
    assert identical_fraction(got, lib) >= 0.97
    # where they differ: by a flipped weight or two, far below one bf16 step of the output's scale
    assert (got.float() - lib.float()).abs().max().item() <= lib.float().abs().max().item() * 2.0 ** -8
    if S == L:  # the uncached call of the same model (is_causal=True, llama.py:122)
        lib2 = F.scaled_dot_product_attention(q.transpose(1, 2), kk, vv, is_causal=True)
        assert identical_fraction(R.attention_core(q, k, v, None), lib2.transpose(1, 2).reshape(B, S, H * D)) >= 0.97
    # a restatement that keeps the weights in fp32 (one rounding at the end) is NOT that routine
    qf, kf, vf = (t.float().permute(0, 2, 1, 3) for t in (q, k, v))
    sc = (qf @ kf.repeat_interleave(grp, 1).transpose(-1, -2)) / math.sqrt(D)
    naive = (torch.softmax(sc.masked_fill(~mask, float("-inf")), -1) @ vf.repeat_interleave(grp, 1)).to(BF)
    assert identical_fraction(naive.permute(0, 2, 1, 3).reshape(B, S, H * D), lib) < 0.95


# ---- operator by operator on the reference's operands ------------------------------------------------


@pytest.mark.parametrize("name", ["mid_gqa", "mid_bias"])
def test_every_operator_on_the_references_own_operands(name):
    fx = load_fixture(f"llama_bf16_{name}.pt")
    cfg = _cfg(fx["config"])
    w = R.init_weights(cfg, seed=fx["seed"], dtype=BF, norm_jitter=fx["norm_jitter"])
    assert torch.allclose(weight_checksum(w), fx["weight_checksum"], rtol=1e-12)
    prompt = fx["ids"].size(1) - 3
    worst_linear = 1.0
    attn_same = []
    for call, pos, S in (("ops_step0", prompt, 1), ("ops_prefill", prompt - 4, 4)):
        def io(name):
            return fx[f"{call}/{name}/in"], fx[f"{call}/{name}/out"]

        x, y = io("token_emb")
        assert torch.equal(w["token_emb.weight"][x], y)
        for i in range(cfg.num_hidden_layers):
            p = f"layers.{i}."
            for n in ("norm1", "norm2"):
                x, y = io(p + n)
                assert torch.equal(R.rms_norm(x, w[p + n + ".weight"]), y), (call, p + n)
            for n in ("attn.key", "attn.query", "attn.value", "attn.proj", "ff.up", "ff.gate", "ff.down"):
                x, y = io(p + n)
                got = R.linear(x, w[p + n + ".weight"], bias=w.get(p + n + ".bias"))
                if cfg.bias:  # llama.py:60-63, mlp.py:146-148: the bias is there, and dropping it is seen
                    assert identical_fraction(R.linear(x, w[p + n + ".weight"]), y) < 0.5
                worst_linear = min(worst_linear, identical_fraction(got, y))
                # one bf16 step where the fp32 sums straddle a rounding boundary (more only where a sum
                # cancels to next to nothing)
                off = (bf16_ulps(got, y) > 1.0) & ((got.float() - y.float()).abs() > 2.0 ** -16 * y.float().abs().max())
                assert not off.any(), (call, p + n)
            # SwiGLU's elementwise part (mlp.py:152) and the two residual adds (llama.py:199-200)
            assert torch.equal(F.silu(io(p + "ff.gate")[1]) * io(p + "ff.up")[1], io(p + "ff.down")[0])
            xb, yb = io(p[:-1])
            h1 = xb + io(p + "attn")[1]
            assert torch.equal(h1, io(p + "norm2")[0])
            assert torch.equal(h1 + io(p + "ff")[1], yb)
            if call == "ops_step0":
                # rotary + append + attention of the cached step, from the reference's projections
                B = xb.size(0)
                ql = io(p + "attn.query")[1].view(B, S, cfg.num_attention_heads, cfg.head_dim)
                kl = io(p + "attn.key")[1].view(B, S, cfg.kv_heads, cfg.head_dim)
                cos, sin = w["freq_cos"][pos : pos + S], w["freq_sin"][pos : pos + S]
                qr, kr = R.apply_rope(ql, kl, cos, sin)
                kc, vc = fx[f"{call}/cache{i}_key"], fx[f"{call}/cache{i}_value"]
                assert torch.equal(kr, kc[:, pos : pos + S])  # rotary.py:55-93, kv_cache.py:104-105
                assert torch.equal(io(p + "attn.value")[1].view_as(kr), vc[:, pos : pos + S])
                att = R.attention_core(qr, kc, vc, pos)
                want = io(p + "attn.proj")[0]
                attn_same.append(identical_fraction(att, want))
                assert attn_same[-1] >= 0.97, (p, attn_same[-1])  # (one flipped weight moves a few of a row's 64 outputs)
                assert (att.float() - want.float()).abs().max().item() <= want.float().abs().max().item() * 2.0 ** -8
        x, y = io("norm")
        assert torch.equal(R.rms_norm(x, w["norm.weight"]), y)
        x, y = io("vocab_proj")
        assert identical_fraction(R.linear(x, w["vocab_proj.weight"]), y) >= 0.999
    assert worst_linear >= 0.998, worst_linear
    assert sum(attn_same) / len(attn_same) >= 0.985, attn_same


# ---- whole models ------------------------------------------------------------------------------------


@pytest.mark.parametrize("name", ["dense", "gqa", "moe"])
def test_tiny_models_in_bf16(name):
    fx = load_fixture(f"llama_bf16_tiny_{name}.pt")
    src = load_fixture(f"llama_tiny_{name}.pt")
    m = R.RefLlama(_cfg(src["config"]), {k: v.to(BF) for k, v in src["state"].items()})
    ids = fx["ids"]
    taps = []
    orig = R.attention_core

    def tapped(q, k, v, s):
        out = orig(q, k, v, s)
        taps.append(out)
        return out

    R.attention_core = tapped
    try:
        full = m(ids)
        cache = m.build_kv_cache(ids.size(0))
        taps.clear()
        calls = [("prefill", m(ids[:, :5], cache, 0)), ("step0", m(ids[:, 5:6], cache, 5)),
                 ("step1", m(ids[:, 6:7], cache, 6))]
        layers = m.config.num_hidden_layers
        attn0 = [taps[i * layers] for i in range(3)]
    finally:
        R.attention_core = orig
    # layer 0's attention sees inputs that no earlier attention has touched: its bits are the reference's
    for (tag, _), got in zip(calls, attn0):
        assert identical_fraction(got, fx[f"attn0_{tag}"]) >= 0.99, (tag, identical_fraction(got, fx[f"attn0_{tag}"]))
    assert identical_fraction(cache[0].value[:, :7], fx["cache0_value"]) >= 0.999
    for tag, got in calls + [("full", full)]:
        mx, mean = _rel(got, fx[f"logits_{tag}"])
        assert mx <= 2e-2 and mean <= 2e-3, (tag, mx, mean)


@pytest.mark.parametrize("name", ["mid_gqa", "mid_bias", "d12w"])
def test_seeded_models_lie_as_close_to_the_reference_as_it_lies_to_itself(name):
    fx = load_fixture(f"llama_bf16_{name}.pt")
    cfg = _cfg(fx["config"])
    w = R.init_weights(cfg, seed=fx["seed"], dtype=BF, norm_jitter=fx["norm_jitter"])
    assert torch.allclose(weight_checksum(w), fx["weight_checksum"], rtol=1e-12)
    m = R.RefLlama(cfg, w)
    ids = fx["ids"]
    steps = 3
    prompt = ids.size(1) - steps
    cache = m.build_kv_cache(ids.size(0))
    got = {"prefill": m(ids[:, :prompt], cache, 0)[:, -8:]}
    for s in range(steps):
        got[f"step{s}"] = m(ids[:, prompt + s : prompt + s + 1], cache, prompt + s)
    assert identical_fraction(cache[0].key[:, prompt + steps - 16 : prompt + steps], fx["cache0_key"]) >= 0.998
    self_mean = reference_self_distance(fx)  # the reference against its own repeats, worst row
    for tag, mine in got.items():
        ref = fx[f"logits_{tag}"].float()
        d = (mine.float() - ref).abs()
        scale = ref.abs().amax(-1)
        assert (d.amax(-1) / scale).max().item() <= 2e-2, tag
        assert (d.mean(-1) / scale).max().item() <= max(2e-3, 1.25 * self_mean), (tag, self_mean)
