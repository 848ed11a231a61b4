"""Pins of the CPU oracle (oracle/): golden fixtures written from the reference, the
reference tests' known answers, closed forms, invariants and fp64 brute force.  Each check
is chosen so that a plausible slip (dropped norm weight, wrong rotary pairing, wrong GQA
head mapping, bias leaking into the gate weights, wrong rounding mode) fails it.
"""

import dataclasses
import math
import os

import numpy as np
import pytest
import torch

from oracle import bitlinear_ref as BL
from oracle import llama_ref as R
from oracle import moe_ref as M
from oracle import sampling_ref as S

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def _cfg(d):
    fields = {f.name for f in dataclasses.fields(R.RefConfig)}
    return R.RefConfig(**{k: v for k, v in d.items() if k in fields})


# ---- composition: the reference's own outputs -------------------------------------------


@pytest.mark.parametrize("name", ["dense", "gqa", "moe"])
def test_llama_forward_matches_reference_fixture(name):
    g = torch.load(os.path.join(GOLD, f"llama_tiny_{name}.pt"), weights_only=True)
    m = R.RefLlama(_cfg(g["config"]), g["state"])
    ids = g["ids"]
    torch.testing.assert_close(m(ids), g["logits_full"], atol=2e-6, rtol=1e-5)
    c = m.build_kv_cache(2)
    torch.testing.assert_close(m(ids[:, :5], c, 0), g["logits_prefill5"], atol=2e-6, rtol=1e-5)
    torch.testing.assert_close(m(ids[:, 5:6], c, 5), g["logits_step5"], atol=2e-6, rtol=1e-5)
    torch.testing.assert_close(m(ids[:, 6:7], c, torch.tensor(6)), g["logits_step6"], atol=2e-6, rtol=1e-5)
    torch.testing.assert_close(c[0].key, g["cache0_key"], atol=1e-6, rtol=1e-5)
    torch.testing.assert_close(c[0].value, g["cache0_value"], atol=1e-6, rtol=1e-5)
    assert c[0].length == 7


def test_cached_equals_uncached_with_gqa():
    # tests/test_training_stack.py:105-136 pattern: prefill 3 + two single steps == full forward
    cfg = R.RefConfig(vocab_size=50, hidden_size=32, intermediate_size=48, num_attention_heads=4,
                      num_key_value_heads=2, num_hidden_layers=2, max_sequence_length=8)
    m = R.RefLlama(cfg, R.init_weights(cfg, 3, norm_jitter=0.2))
    ids = torch.randint(0, 50, (2, 5), generator=torch.Generator().manual_seed(0))
    full = m(ids)
    c = m.build_kv_cache(2)
    parts = [m(ids[:, :3], c, 0), m(ids[:, 3:4], c, 3), m(ids[:, 4:5], c, 4)]
    torch.testing.assert_close(torch.cat(parts, 1), full, atol=1e-5, rtol=1e-4)
    # uncached path reduces to the library routine with is_causal=True
    q = torch.randn(2, 5, 4, 8)
    k = torch.randn(2, 5, 2, 8)
    v = torch.randn(2, 5, 2, 8)
    lib = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(1, 2), k.repeat_interleave(2, 2).transpose(1, 2), v.repeat_interleave(2, 2).transpose(1, 2),
        is_causal=True).transpose(1, 2).reshape(2, 5, 32)
    torch.testing.assert_close(R.attention_core(q, k, v, None), lib, atol=1e-6, rtol=1e-5)


def test_forward_and_cache_errors():
    cfg = R.RefConfig(vocab_size=20, hidden_size=16, intermediate_size=16, num_attention_heads=2,
                      num_hidden_layers=2, max_sequence_length=6)
    m = R.RefLlama(cfg, R.init_weights(cfg, 0))
    ids = torch.zeros(1, 3, dtype=torch.long)
    for call, msg in (
        (lambda: m(ids[0]), "shape"),
        (lambda: m(ids, m.build_kv_cache(1)[:1], 0), "one entry per model layer"),
        (lambda: m(ids, m.build_kv_cache(1), None), "non-negative position_ids"),
        (lambda: m(ids, None, 2), "only valid when using a KV cache"),
        (lambda: m(ids[:, :0]), "cannot be empty"),
        (lambda: m(torch.zeros(1, 7, dtype=torch.long)), "exceeds max_sequence_length"),
        (lambda: m.build_kv_cache(0), "at least 1"),
    ):
        with pytest.raises(ValueError, match=msg):
            call()
    # tests/test_modules.py:46-79
    c = R.KVCacheRef((2, 6, 2, 4), 6)
    k = torch.randn(2, 3, 2, 4)
    ck, cv = c.forward(k, k + 1, 0)
    assert ck.shape == (2, 3, 2, 4) and c.length == 3 and torch.equal(cv, k + 1)
    with pytest.raises(ValueError, match="sequential"):
        c.forward(k, k, 5)
    with pytest.raises(ValueError, match="max_sequence_length"):
        c.forward(torch.randn(2, 4, 2, 4), torch.randn(2, 4, 2, 4), 3)
    with pytest.raises(ValueError, match="matching shapes"):
        c.forward(k, k[:, :2], 3)
    with pytest.raises(ValueError, match="cannot change"):
        c.forward(k[:1], k[:1], 3)


# ---- parts ---------------------------------------------------------------------------------


def test_rms_norm_closed_form_and_unit_rms():
    x = torch.randn(5, 64, dtype=torch.float64) * 3
    w = torch.rand(64, dtype=torch.float64) + 0.5
    want = x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-5) * w
    torch.testing.assert_close(R.rms_norm(x.float(), w.float()).double(), want, atol=1e-5, rtol=1e-5)
    out = R.rms_norm(torch.randn(4, 256), torch.ones(256))
    assert torch.allclose(out.pow(2).mean(-1).sqrt(), torch.ones(4), atol=1e-3)  # tests/test_modules.py:168-172
    # bf16: rounds once before the weight multiply (norm.py:20-21)
    xb = torch.randn(3, 128).to(torch.bfloat16)
    wb = (torch.rand(128) + 0.5).to(torch.bfloat16)
    inner = (xb.float() * torch.rsqrt(xb.float().pow(2).mean(-1, keepdim=True) + 1e-5)).to(torch.bfloat16)
    assert torch.equal(R.rms_norm(xb, wb), inner * wb)


def test_rope_table_and_rotation():
    cos, sin = R.rope_table(16, 32, 10000.0)
    t, i = 7, 3
    ang = t * 10000.0 ** (-2 * i / 16)
    assert abs(cos[t, i].item() - math.cos(ang)) < 1e-5 and abs(sin[t, i].item() - math.sin(ang)) < 1e-5
    assert not torch.equal(R.rope_table(16, 32, 500.0)[0], cos)  # theta is honoured
    q = torch.randn(2, 5, 3, 16)
    k = torch.randn(2, 5, 3, 16)
    qr, kr = R.apply_rope(q, k, cos[4:9], sin[4:9])
    # complex multiply on adjacent pairs (library routine)
    zc = torch.view_as_complex(q.reshape(2, 5, 3, 8, 2).contiguous())
    rot = torch.polar(torch.ones(5, 8), torch.outer(torch.arange(4, 9).float(),
                                                    1.0 / 10000.0 ** (torch.arange(0, 16, 2).float() / 16)))
    want = torch.view_as_real(zc * rot[None, :, None, :]).reshape(2, 5, 3, 16)
    torch.testing.assert_close(qr, want, atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(qr.norm(dim=-1), q.norm(dim=-1), atol=1e-5, rtol=1e-5)  # tests/test_modules.py:106-122
    q0, _ = R.apply_rope(q[:, :1], k[:, :1], cos[:1], sin[:1])
    torch.testing.assert_close(q0, q[:, :1], atol=1e-6, rtol=0)  # position 0 is the identity
    # NOT the half-split layout: element 0 mixes with element 1, not with element 8
    e = torch.zeros(1, 1, 1, 16)
    e[..., 0] = 1.0
    r, _ = R.apply_rope(e, e, cos[5:6], sin[5:6])
    assert abs(r[0, 0, 0, 1].item() - sin[5, 0].item()) < 1e-6 and r[0, 0, 0, 8].item() == 0.0


def test_attention_brute_force_gqa_and_mask():
    B, S, H, Hkv, D, L, start = 2, 3, 4, 2, 8, 7, 4
    q = torch.randn(B, S, H, D, dtype=torch.float64)
    k = torch.randn(B, L, Hkv, D, dtype=torch.float64)
    v = torch.randn(B, L, Hkv, D, dtype=torch.float64)
    got = R.attention_core(q.float(), k.float(), v.float(), start).double()
    want = torch.zeros(B, S, H * D, dtype=torch.float64)
    for b in range(B):
        for s in range(S):
            for h in range(H):
                kv = h // (H // Hkv)  # repeat_interleave semantics, llama.py:101-103
                sc = [float(q[b, s, h] @ k[b, t, kv]) / math.sqrt(D) if t <= start + s else -math.inf for t in range(L)]
                mx = max(sc)
                e = [math.exp(x - mx) for x in sc]
                z = sum(e)
                for t in range(L):
                    want[b, s, h * D:(h + 1) * D] += e[t] / z * v[b, t, kv]
    torch.testing.assert_close(got, want, atol=1e-5, rtol=1e-5)


def test_swiglu_and_linear():
    x = torch.randn(3, 8)
    wg, wu, wd = torch.randn(12, 8), torch.randn(12, 8), torch.randn(8, 12)
    want = (torch.nn.functional.silu(x @ wg.T) * (x @ wu.T)) @ wd.T
    torch.testing.assert_close(R.swiglu(x, wg, wu, wd), want, atol=1e-5, rtol=1e-5)


# ---- mixture of experts ------------------------------------------------------------------------


def test_moe_routing_and_dispatch_hand_loop():
    # tests/test_moe_grouped.py:45-60,89-124 and tests/test_modules.py:192-210
    torch.manual_seed(0)
    N, d, E, hdim, k = 9, 16, 6, 8, 2
    x = torch.randn(N, d)
    rw, bias = torch.randn(E, d), torch.randn(E) * 2
    wg, wu, wdn = torch.randn(E, d, hdim), torch.randn(E, d, hdim), torch.randn(E, hdim, d)
    idx, w, logits = M.moe_route(x, rw, bias, k)
    assert all(len(set(r.tolist())) == k for r in idx)
    torch.testing.assert_close(w.sum(-1), torch.ones(N), atol=1e-5, rtol=0)
    # selection uses logits + bias (top k of top k+1), weights use the unbiased logits
    want_idx = torch.topk(logits + bias, k + 1, dim=-1).indices[:, :k]
    assert torch.equal(idx, want_idx)
    torch.testing.assert_close(w, logits.gather(-1, idx).softmax(-1))
    idx0, w0, _ = M.moe_route(x, rw, torch.zeros(E), k)
    assert not torch.equal(idx0, idx)  # the bias moves the selection
    out = M.moe_dispatch(x, idx, w, wg, wu, wdn)
    want = torch.zeros_like(x)
    for n in range(N):
        for j in range(k):
            e = int(idx[n, j])
            h = torch.nn.functional.silu(x[n] @ wg[e]) * (x[n] @ wu[e])
            want[n] += w[n, j] * (h @ wdn[e])
    torch.testing.assert_close(out, want, atol=1e-4, rtol=1e-4)
    sig = M.moe_route(x, rw, bias, k, gate_fn="sigmoid")[1]
    torch.testing.assert_close(sig.sum(-1), torch.ones(N), atol=1e-5, rtol=0)
    # ties in the router logits resolve to the lowest expert id
    tie = M.topk_lowest_index_first(torch.tensor([[1.0, 3.0, 3.0, 0.0, 3.0]]), 2)
    assert tie.tolist() == [[1, 2]]


# ---- samplers ----------------------------------------------------------------------------------


def test_sampler_known_answers_and_kept_set():
    # tests/test_inference.py:45-48, tests/test_chat.py:355-373
    assert S.inference_sampler_ref(torch.tensor([[[0.1, 0.2, 0.9]]]), temperature=0.0).item() == 2
    assert S.sample_next_token_ref(torch.tensor([[[0.1, 5.0, 0.2, 0.3]]]), temperature=0.0).item() == 1
    logits = torch.tensor([[[10.0, 9.0, -50.0, -60.0]]])
    seen = {int(S.sample_next_token_ref(logits, 1.0, 1.0, 2).item()) for _ in range(200)}
    assert seen <= {0, 1}
    seen = {int(S.sample_next_token_ref(torch.tensor([[[20.0, 0.0, 0.0, 0.0]]]), 1.0, 0.01, 0).item())
            for _ in range(50)}
    assert seen == {0}
    a = S.sample_next_token_ref(torch.randn(1, 1, 32, generator=torch.Generator().manual_seed(1)), 1.0, 0.9, 0,
                                generator=torch.Generator().manual_seed(7))
    b = S.sample_next_token_ref(torch.randn(1, 1, 32, generator=torch.Generator().manual_seed(1)), 1.0, 0.9, 0,
                                generator=torch.Generator().manual_seed(7))
    assert a.item() == b.item()
    # the vectorised filter equals the direct fp64 loops; the u-walk hits every kept id in order
    g = torch.Generator().manual_seed(5)
    for T, p, k in ((0.8, 0.9, 5), (1.0, 0.5, 0), (1.3, 0.0, 3), (0.7, 0.999, 0)):
        row = torch.randn(12, generator=g) * 2
        kept, probs = S.kept_set_ref(row, T, p, k)
        ids, cdf = S.candidate_cdf_ref(row.view(1, 1, -1), T, p, k)
        live = [int(i) for i, c, c0 in zip(ids[0], cdf[0], [0.0] + cdf[0].tolist()[:-1]) if c > c0]
        assert sorted(live) == sorted(kept)
        acc = 0.0
        for i, pr in zip(kept, probs) if 0 < p < 1 else ():
            u = torch.tensor([acc + pr / 2])
            assert S.sample_next_token_ref(row.view(1, 1, -1), T, p, k, u=u).item() == i
            acc += pr
    # top-k keeps ties at the threshold; nucleus keeps the boundary-crossing token
    row = torch.tensor([2.0, 2.0, 2.0, 1.0])
    assert S.kept_set_ref(row, 1.0, 0.0, 2)[0] == [0, 1, 2]
    assert S.kept_set_ref(torch.tensor([math.log(0.5), math.log(0.3), math.log(0.2)]), 1.0, 0.6, 0)[0] == [0, 1]


def test_generate_loop_literals():
    # tests/test_inference.py:50-79
    class Tok:
        eos_token_id = 99

        def encode(self, _):
            return [1, 2, 3]

        def decode(self, t):
            return " ".join(str(x) for x in t)

    class Dummy:
        class config:
            max_sequence_length = 6

        def __init__(self):
            self.calls = []

        def build_kv_cache(self):
            return object()

        def __call__(self, x, cache=None, position=0):
            self.calls.append((x.shape[1], cache is not None, position))
            out = torch.zeros(x.shape[0], x.shape[1], 128)
            out[:, :, 5] = 1.0
            return out

    m = Dummy()
    assert S.inference_generate_ref(m, Tok(), "hello", temperature=0.0, max_new_tokens=10) == "1 2 3 5 5 5"
    assert [c[0] for c in m.calls] == [3, 1, 1] and [c[2] for c in m.calls] == [0, 3, 4]
    with pytest.raises(ValueError):
        S.inference_generate_ref(m, Tok(), "hello", max_new_tokens=-1)


# ---- BitLinear ---------------------------------------------------------------------------------


def test_bitlinear_integer_semantics():
    g = torch.Generator().manual_seed(2)
    # W = c * T reproduces T, gamma = c * fraction non-zero
    T = torch.randint(-1, 2, (24, 40), generator=g).float()
    c = 0.037
    t, gamma = BL.weight_ternarize(c * T)
    assert torch.equal(t.float(), T)
    assert abs(float(gamma) - c * T.abs().mean().item()) < 1e-7
    # equal activations quantise to +-127; round is half-to-even (2.5 -> 2, 3.5 -> 4)
    q, s = BL.activation_quant(torch.tensor([[0.5, -0.5, 0.5, -0.5]]))
    assert q.tolist() == [[127, -127, 127, -127]]
    q, _ = BL.activation_quant(torch.tensor([[127.0, 2.5, 3.5, -2.5]]))
    assert q.tolist() == [[127, 2, 4, -2]]
    # int32 accumulation is exact: compare with python integers
    qq = torch.randint(-128, 128, (3, 40), generator=g, dtype=torch.int8)
    acc = BL.int_accumulate(qq, t)
    for m in range(3):
        for n in (0, 7, 23):
            assert int(acc[m, n]) == sum(int(a) * int(b) for a, b in zip(qq[m].tolist(), t[n].tolist()))
    # the fp32-BLAS route of int_accumulate (used below 128*K < 2**24) equals the int32 product, also
    # at the largest K of the ternary model (5632) with worst-case magnitudes
    for K in (40, 2048, 5632):
        q8 = torch.randint(-128, 128, (9, K), generator=g, dtype=torch.int8)
        t8 = torch.randint(-1, 2, (33, K), generator=g, dtype=torch.int8)
        q8[0], t8[0] = -128, -1  # |sum| = 128 * K, the bound of the exactness argument
        assert torch.equal(BL.int_accumulate(q8, t8), BL.int_accumulate(q8, t8, force_int=True))
        assert int(BL.int_accumulate(q8, t8)[0, 0]) == 128 * K
    # packing round trip and bit layout
    packed = BL.pack_ternary(t)
    assert packed.shape == (24, 10) and torch.equal(BL.unpack_ternary(packed), t)
    assert int(packed[0, 0]) == sum((int(t[0, i]) + 1) << (2 * i) for i in range(4))
    # integer formulation == the reference's float fake-quant formulation (bitnet.py:29-59)
    x = torch.randn(5, 40, generator=g)
    w = torch.randn(24, 40, generator=g) * 0.05
    nw = torch.rand(40, generator=g) + 0.5
    tt, gm = BL.weight_ternarize(w)
    y = BL.bitlinear_forward(x, nw, tt, gm)
    torch.testing.assert_close(y, BL.fake_quant_forward(x, nw, w), atol=2e-5, rtol=1e-4)


# --- int8 KV cache (kv_cache.py:15-33, 94-118) ---------------------------------------------


def _rne(q, bits: int):
    """An exact rational rounded to `bits` significant bits, ties to even (normal range only)."""
    from fractions import Fraction

    if q == 0:
        return Fraction(0)
    sign, q = (-1 if q < 0 else 1), abs(q)
    e = q.numerator.bit_length() - q.denominator.bit_length()
    if Fraction(2) ** e > q:
        e -= 1
    ulp = Fraction(2) ** (e - bits + 1)
    n, rem = divmod(q, ulp)
    if rem * 2 > ulp or (rem * 2 == ulp and n % 2 == 1):
        n += 1
    return sign * n * ulp


def _bf16_op(q):
    """A bf16 tensor op: the exact result rounded to fp32 (the arithmetic runs in fp32), then to bf16."""
    return _rne(_rne(q, 24), 8)


def _quant_row_bf16_by_hand(row: np.ndarray):
    """One bf16 row through the int8 quantiser in exact rational arithmetic with the roundings of
    every op written out (kv_cache.py:20-27 on a bf16 tensor)."""
    from fractions import Fraction

    vals = [Fraction(float(x)) for x in row]
    lo, hi = min(vals), max(vals)
    scale = max(_bf16_op(_bf16_op(hi - lo) / 255), _bf16_op(Fraction(1e-8)))
    codes = []
    for x in vals:
        t = _bf16_op(_bf16_op(_bf16_op(x - lo) / scale) - 128)
        n = math.floor(t)  # round half to even
        r = t - n
        n += 1 if (r > Fraction(1, 2) or (r == Fraction(1, 2) and n % 2 == 1)) else 0
        codes.append(min(127, max(-128, n)))
    return np.array(codes, np.int8), np.float32(float(scale)), np.float32(float(lo))


def test_int8_quantiser_closed_forms():
    # an exact 256-level ramp maps onto the codes -128..127 and inverts exactly
    lo, step = -3.0, 0.03125
    ramp = (lo + step * torch.arange(256, dtype=torch.float32)).view(1, 256)
    q, scale, mn = R.quantize_int8(ramp)
    assert q.dtype == torch.int8 and scale.shape == mn.shape == (1, 1)
    assert torch.equal(q.view(-1).int(), torch.arange(256, dtype=torch.int32) - 128)
    assert float(scale) == step and float(mn) == lo
    assert torch.equal(R.dequantize_int8(q, scale, mn), ramp)
    # a constant row: the scale floors at 1e-8, all codes -128, the value comes back
    const = torch.full((2, 8), 0.75)
    q, scale, mn = R.quantize_int8(const)
    assert torch.all(q == -128) and torch.all(scale == 1e-8) and torch.equal(R.dequantize_int8(q, scale, mn), const)
    # extremes hit the end codes; the error never exceeds half a level (+ fp32 rounding)
    g = torch.Generator().manual_seed(3)
    x = torch.randn(64, 48, generator=g) * 3
    q, scale, mn = R.quantize_int8(x)
    assert torch.all(q.amin(-1) == -128) and torch.all(q.amax(-1) == 127)
    err = (R.dequantize_int8(q, scale, mn) - x).abs()
    assert torch.all(err <= scale * 0.5 + 1e-5)
    # other reduction axes quantise along that axis
    qt, st, mt = R.quantize_int8(x.t().contiguous(), dim=0)
    assert torch.equal(qt.t(), q) and torch.equal(st.view(-1), scale.view(-1))
    # the reference's own tolerance for the round trip (tests/test_modules.py:94-100)
    t = torch.randn(4, 16, generator=g)
    torch.testing.assert_close(R.dequantize_int8(*R.quantize_int8(t)), t, rtol=0.05, atol=0.05)


def test_int8_quantiser_bf16_rounding_points_by_hand():
    g = torch.Generator().manual_seed(11)
    x = (torch.randn(6, 32, generator=g) * 2).to(torch.bfloat16)
    x[5] = 1.5  # constant row
    q, scale, mn = R.quantize_int8(x)
    assert scale.dtype == torch.bfloat16
    for i in range(x.shape[0]):
        hq, hs, hm = _quant_row_bf16_by_hand(x[i].float().numpy())
        assert float(scale[i]) == float(hs) and float(mn[i]) == float(hm)
        assert np.array_equal(q[i].numpy(), hq), i
    # dequantisation is fp32: product rounds once, sum rounds once
    d = R.dequantize_int8(q, scale.float(), mn.float())
    assert d.dtype == torch.float32
    by_hand = (np.float32(1) * (q.numpy().astype(np.float32) + 128) * scale.float().numpy()).astype(np.float32) \
        + mn.float().numpy()
    assert np.array_equal(d.numpy(), by_hand.astype(np.float32))


def test_int8_cache_reads_dequantised_values():
    """tests/test_modules.py:82-91 on the restated cache, plus sequential appends."""
    g = torch.Generator().manual_seed(5)
    cache = R.KVCacheRef((2, 8, 2, 4), 8, dtype=torch.float32, int8=True)
    entry = torch.randn(1, 4, 2, 4, generator=g)
    keys, values = cache.forward(entry, entry.clone(), 0)
    assert keys.dtype == torch.float32 and cache.key.dtype == torch.int8
    torch.testing.assert_close(keys, entry, rtol=0.05, atol=0.05)
    torch.testing.assert_close(values, entry, rtol=0.05, atol=0.05)
    nxt = torch.randn(1, 1, 2, 4, generator=g)
    k2, v2 = cache.forward(nxt, -nxt, 4)
    assert k2.shape == (1, 5, 2, 4) and torch.equal(k2[:, :4], keys)
    torch.testing.assert_close(v2[:, 4:], -nxt, rtol=0.05, atol=0.05)
    assert cache.key_scale.shape == (2, 8, 2, 1) and torch.all(cache.key_scale[0, :5] > 0)
    assert torch.all(cache.key_scale[1] == 0) and torch.all(cache.key_scale[0, 5:] == 0)
    with pytest.raises(ValueError, match="sequential"):
        cache.forward(nxt, nxt, 3)


def test_int8_cache_model_stays_close_to_the_exact_cache():
    cfg = R.RefConfig(vocab_size=97, max_sequence_length=32, hidden_size=64, intermediate_size=128,
                      num_attention_heads=4, num_key_value_heads=2, num_hidden_layers=2)
    model = R.RefLlama(cfg, R.init_weights(cfg, 2, norm_jitter=0.2))
    ids = torch.randint(0, 97, (2, 9), generator=torch.Generator().manual_seed(1))
    exact = model(ids, model.build_kv_cache(2), 0)
    quant = model(ids, model.build_kv_cache(2, int8=True), 0)
    assert 0 < (exact - quant).abs().max() < 0.05 * exact.abs().max()
