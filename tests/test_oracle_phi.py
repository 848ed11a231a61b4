"""Pins the Phi oracle (oracle/phi_ref.py): closed forms, library routines, fp64 brute force,
the reference RoPE module's vectors, and the invariant of the reference's own Phi test."""

import math
import os

import pytest
import torch
import torch.nn.functional as F

from oracle import phi_ref as P

HERE = os.path.dirname(os.path.abspath(__file__))


def test_rope_partial_matches_the_reference_module_vectors():
    cases = torch.load(os.path.join(HERE, "golden", "phi_rope.pt"), weights_only=True)
    assert len(cases) == 5
    for c in cases:
        got = P.rope_partial(c["x"], c["dims"], offset=c["offset"])
        torch.testing.assert_close(got, c["y"], rtol=0, atol=0)


def test_rope_partial_closed_form_fp64():
    """Feature i < dims/2 and its partner i + dims/2 rotate as the complex number x1 + i*x2 by the
    angle t * base^(-i / (dims/2)); a swapped pair, a wrong sign or an adjacent-pair layout fails."""
    g = torch.Generator().manual_seed(0)
    dims, D, T, off = 6, 10, 5, 4
    x = torch.randn(2, T, D, generator=g)
    got = P.rope_partial(x, dims, offset=off).double()
    half = dims // 2
    for t in range(T):
        for i in range(half):
            ang = (off + t) * 10000.0 ** (-i / half)
            z = complex(x[0, t, i].item(), x[0, t, i + half].item()) * complex(math.cos(ang), math.sin(ang))
            assert abs(got[0, t, i].item() - z.real) < 1e-5 and abs(got[0, t, i + half].item() - z.imag) < 1e-5
    assert torch.equal(got[..., dims:].float(), x[..., dims:])  # the tail passes through
    assert torch.allclose(P.rope_partial(x[:, :1], dims, offset=0), x[:, :1])  # position 0 is the identity
    # rotation preserves the norm of the rotated part
    assert torch.allclose(got[..., :dims].norm(dim=-1).float(), x[..., :dims].norm(dim=-1), atol=1e-5)


def test_new_gelu_is_the_tanh_gelu():
    x = torch.linspace(-6, 6, 1001)
    torch.testing.assert_close(P.new_gelu(x), F.gelu(x, approximate="tanh"), rtol=1e-5, atol=1e-6)
    assert P.new_gelu(torch.tensor([0.0])).item() == 0.0
    # bf16: every op rounds; the coarsest step is 1 + tanh(.) (ulp 2^-8 near -1), scaled by 0.5 * x
    xb = x.to(torch.bfloat16)
    ref = F.gelu(xb.float(), approximate="tanh")
    assert ((P.new_gelu(xb).float() - ref).abs() <= 2 ** -7 * xb.float().abs() + 1e-3).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_layer_norm_is_the_library_routine(dtype):
    g = torch.Generator().manual_seed(1)
    x = (torch.randn(5, 48, generator=g) * 3 + 1).to(dtype)
    w = (1 + 0.1 * torch.randn(48, generator=g)).to(dtype)
    b = (0.1 * torch.randn(48, generator=g)).to(dtype)
    got = P.layer_norm(x, w, b, 1e-5)
    want = F.layer_norm(x, (48,), w, b, 1e-5)
    if dtype == torch.float32:
        torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-6)
    else:  # one rounding of the same fp32 value: at most one bf16 ulp apart
        assert ((got.float() - want.float()).abs() <= 2 ** -7 * want.float().abs().clamp_min(2 ** -7)).all()
    y = P.layer_norm(x.float(), torch.ones(48), torch.zeros(48), 0.0)
    assert y.mean(-1).abs().max() < 1e-5 and (y.var(-1, unbiased=False) - 1).abs().max() < 1e-4


def test_linear_bias_is_addmm():
    g = torch.Generator().manual_seed(2)
    x, w, b = torch.randn(3, 16, generator=g), torch.randn(8, 16, generator=g), torch.randn(8, generator=g)
    torch.testing.assert_close(P.linear_bias(x, w, b), F.linear(x, w, b))


def test_attention_brute_force_fp64():
    g = torch.Generator().manual_seed(3)
    B, S, L0, H, D, rot = 2, 2, 3, 2, 8, 4
    q = torch.randn(B, S, H, D, generator=g)
    k = torch.randn(B, L0 + S, H, D, generator=g)
    v = torch.randn(B, L0 + S, H, D, generator=g)
    got = P.attention(q, k, v, L0, rot, torch.float32)
    half = rot // 2

    def rotate(vec, pos):
        out = [float(e) for e in vec]
        for i in range(half):
            ang = pos * 10000.0 ** (-i / half)
            a, b_ = float(vec[i]), float(vec[i + half])
            out[i] = a * math.cos(ang) - b_ * math.sin(ang)
            out[i + half] = a * math.sin(ang) + b_ * math.cos(ang)
        return out

    for b in range(B):
        for h in range(H):
            for s in range(S):
                qr = rotate(q[b, s, h], L0 + s)
                sc = []
                for t in range(L0 + s + 1):  # keys beyond the query's position are masked
                    kr = rotate(k[b, t, h], t)
                    sc.append(sum(a * c for a, c in zip(qr, kr)) / math.sqrt(D))
                m = max(sc)
                e = [math.exp(z - m) for z in sc]
                for dd in range(D):
                    want = sum(e[t] * float(v[b, t, h, dd]) for t in range(len(sc))) / sum(e)
                    assert abs(got[b, s, h, dd].item() - want) < 1e-5


def _tiny(dtype=torch.float32, **kw):
    base = dict(vocab_size=64, max_sequence_length=16, hidden_size=64, num_attention_heads=4, num_hidden_layers=2,
                multiple_of=4, rotary_dim=0.4)
    base.update(kw)
    cfg = P.RefPhiConfig(**base)
    return cfg, P.RefPhi(cfg, P.init_weights(cfg, seed=5, dtype=dtype, std=0.08, bias_std=0.05))


def test_cached_decode_matches_full_forward():
    """The reference's own Phi test (tests/test_models.py:133-149), same tolerances."""
    cfg, model = _tiny()
    ids = torch.randint(0, 64, (1, 8), generator=torch.Generator().manual_seed(0))
    full = model(ids)
    cache = model.build_kv_cache()
    prefill = model(ids[:, :4], cache, 0)
    step = model(ids[:, 4:5], cache, 4)
    torch.testing.assert_close(prefill[:, -1], full[:, 3], rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(step[:, -1], full[:, 4], rtol=1e-4, atol=1e-4)
    # the cache holds the un-rotated key projection (phi.py:95 precedes the rotation at :103-104)
    h = P.layer_norm(model.w["wte.weight"][ids[:, :5]], model.w["layers.0.ln.weight"], model.w["layers.0.ln.bias"], cfg.eps)
    k = P.linear_bias(h, model.w["layers.0.mixer.k_proj.weight"], model.w["layers.0.mixer.k_proj.bias"])
    torch.testing.assert_close(cache[0].key[:1, :5].reshape(1, 5, -1), k)
    with pytest.raises(ValueError, match="position_ids is required"):
        model(ids[:, :1], model.build_kv_cache(), None)
    with pytest.raises(ValueError, match="one entry per model layer"):
        model(ids[:, :1], cache[:1], 0)
    with pytest.raises(ValueError, match="at least 1"):
        model.build_kv_cache(0)


def test_block_by_hand_fp64():
    """One block, one sequence, written out with python floats: parallel attention + MLP off the same
    LayerNorm output, summed with the block input (phi.py:147-151)."""
    cfg, model = _tiny(hidden_size=8, num_attention_heads=2, num_hidden_layers=1, vocab_size=16, multiple_of=2,
                       rotary_dim=0.5)
    w = {k: v.double() for k, v in model.w.items()}
    ids = torch.tensor([[3, 7, 1]])
    x = w["wte.weight"][ids][0]  # (3, 8)
    mean = x.mean(-1, keepdim=True)
    var = ((x - mean) ** 2).mean(-1, keepdim=True)
    h = (x - mean) / torch.sqrt(var + cfg.eps) * w["layers.0.ln.weight"] + w["layers.0.ln.bias"]
    lin = lambda t, n: t @ w[f"layers.0.{n}.weight"].t() + w[f"layers.0.{n}.bias"]
    q, k, v = (lin(h, f"mixer.{n}").view(3, 2, 4) for n in ("q_proj", "k_proj", "v_proj"))
    rot = cfg.rotary_width
    assert rot == 2
    out = torch.zeros(3, 2, 4, dtype=torch.float64)

    def rotate(vec, pos):
        o = vec.clone()
        for i in range(rot // 2):
            ang = pos * 10000.0 ** (-i / (rot // 2))
            o[i] = vec[i] * math.cos(ang) - vec[i + rot // 2] * math.sin(ang)
            o[i + rot // 2] = vec[i] * math.sin(ang) + vec[i + rot // 2] * math.cos(ang)
        return o

    for hd in range(2):
        for s in range(3):
            sc = torch.stack([(rotate(q[s, hd], s) * rotate(k[t, hd], t)).sum() / 2.0 for t in range(s + 1)])
            p = torch.softmax(sc, 0)
            out[s, hd] = sum(p[t] * v[t, hd] for t in range(s + 1))
    mixer = lin(out.view(3, 8), "mixer.dense")
    z = lin(h, "mlp.fc1")
    gel = 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))
    y = mixer + lin(gel, "mlp.fc2") + x
    mean = y.mean(-1, keepdim=True)
    var = ((y - mean) ** 2).mean(-1, keepdim=True)
    yn = (y - mean) / torch.sqrt(var + cfg.eps) * w["ln.weight"] + w["ln.bias"]
    want = yn @ w["lm_head.weight"].t() + w["lm_head.bias"]
    got = model(ids)[0]
    torch.testing.assert_close(got.double(), want, rtol=1e-4, atol=1e-5)
