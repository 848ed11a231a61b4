"""Parity of each HIP entry point against the CPU oracle on identical seeded inputs.

All calls go through the C ABI (ohara_amd.ops -> libohara_decode.so).  Tolerances:
element-wise kernels must reproduce the oracle's bf16 values exactly except where an
fp32 reduction order differs (then <= 1 bf16 ulp on a small fraction of elements);
GEMM-like kernels are compared in units of the output scale.
"""

import math

import pytest
import torch

from oracle import llama_ref as R

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


def _ulp_close(a, b, max_ulp=1, frac=0.02):
    """bf16 tensors equal up to `max_ulp` units in the last place on at most `frac` of elements."""
    a16 = a.cpu().view(torch.int16).to(torch.int32)
    b16 = b.cpu().view(torch.int16).to(torch.int32)
    diff = (a16 - b16).abs()
    assert int(diff.max()) <= max_ulp, f"max ulp diff {int(diff.max())}"
    assert float((diff > 0).float().mean()) <= frac, f"fraction differing {float((diff > 0).float().mean())}"


def test_embed(cuda):
    from ohara_amd import ops

    g = torch.Generator().manual_seed(0)
    table = torch.randn(100, 48, generator=g).to(BF)
    ids = torch.randint(0, 100, (3, 5), generator=g)
    out = ops.embed(ids.to(cuda), table.to(cuda))
    assert torch.equal(out.cpu(), table[ids.reshape(-1)])


@pytest.mark.parametrize("d", [32, 768, 2048, 100])
def test_rmsnorm(cuda, d):
    from ohara_amd import ops

    g = torch.Generator().manual_seed(d)
    x = (torch.randn(7, d, generator=g) * 3).to(BF)
    w = (1 + 0.2 * torch.randn(d, generator=g)).to(BF)
    ref = R.rms_norm(x, w)
    out = ops.rmsnorm(x.to(cuda), w.to(cuda))
    _ulp_close(out, ref)


@pytest.mark.parametrize("B,N,K", [(1, 768, 768), (3, 64, 32), (8, 3072, 768), (16, 768, 3072), (17, 100, 96),
                                   (32, 2304, 768), (64, 768, 3072), (5, 65, 40),
                                   # >= 1024 strips: the kernel that keeps the activations in LDS
                                   (1, 16384, 768), (17, 16390, 776), (33, 20000, 96), (64, 16384, 768),
                                   (48, 16400, 1000),
                                   # the same kernel with more than 128 KB of rows in LDS, and close to the 160 KB it may take
                                   (64, 16384, 1024), (64, 16400, 1216)])
@pytest.mark.parametrize("norm", [False, True])
def test_gemm_skinny_store(cuda, B, N, K, norm):
    from ohara_amd import ops

    g = torch.Generator().manual_seed(B * 1000 + N + K)
    x = torch.randn(B, K, generator=g).to(BF)
    w = (torch.randn(N, K, generator=g) * 0.05).to(BF)
    nw = (1 + 0.2 * torch.randn(K, generator=g)).to(BF)
    xin = R.rms_norm(x, nw) if norm else x
    ref = R.linear(xin, w)
    wp = ops.pack_linear(w.to(cuda))
    out = ops.gemm_skinny(x.to(cuda), wp, norm_w=nw.to(cuda) if norm else None)
    scale = ref.float().abs().max().item()
    err = (out.cpu().float() - ref.float()).abs().max().item()
    assert err <= 2 ** -7 * scale, (err, scale)  # one bf16 ulp at the output scale
    # and nearly everything identical
    assert (out.cpu() != ref).float().mean().item() < 0.05


def test_gemm_skinny_residual(cuda):
    from ohara_amd import ops

    g = torch.Generator().manual_seed(5)
    B, N, K = 4, 768, 3072
    x = torch.randn(B, K, generator=g).to(BF)
    w = (torch.randn(N, K, generator=g) * 0.02).to(BF)
    res = torch.randn(B, N, generator=g).to(BF)
    ref = res + R.linear(x, w)
    out = ops.gemm_skinny(x.to(cuda), ops.pack_linear(w.to(cuda)), residual=res.to(cuda))
    _ulp_close(out, ref, max_ulp=2, frac=0.05)


@pytest.mark.parametrize("B,F,K", [(1, 3072, 768), (8, 64, 32), (33, 520, 64), (2, 12, 32)])
def test_gemm_skinny_swiglu(cuda, B, F, K):
    from ohara_amd import ops

    g = torch.Generator().manual_seed(F)
    x = torch.randn(B, K, generator=g).to(BF)
    wg = (torch.randn(F, K, generator=g) * 0.1).to(BF)
    wu = (torch.randn(F, K, generator=g) * 0.1).to(BF)
    nw = (1 + 0.2 * torch.randn(K, generator=g)).to(BF)
    h = R.rms_norm(x, nw)
    ref = torch.nn.functional.silu(R.linear(h, wg)) * R.linear(h, wu)
    wp = ops.pack_gate_up(wg.to(cuda), wu.to(cuda))
    out = ops.gemm_skinny(x.to(cuda), wp, norm_w=nw.to(cuda))
    scale = ref.float().abs().max().item()
    err = (out.cpu().float() - ref.float()).abs().max().item()
    assert err <= 2 ** -6 * scale, (err, scale)
    assert (out.cpu() != ref).float().mean().item() < 0.08


@pytest.mark.parametrize("B,H,Hkv,D,K", [(1, 6, 6, 128, 768), (3, 4, 2, 16, 64), (16, 32, 8, 128, 256), (2, 4, 4, 8, 32)])
def test_qkv_rope_append(cuda, B, H, Hkv, D, K):
    from ohara_amd import ops

    g = torch.Generator().manual_seed(H * D)
    Tmax, pos = 32, 11
    x = torch.randn(B, K, generator=g).to(BF)
    wq = (torch.randn(H * D, K, generator=g) * 0.05).to(BF)
    wk = (torch.randn(Hkv * D, K, generator=g) * 0.05).to(BF)
    wv = (torch.randn(Hkv * D, K, generator=g) * 0.05).to(BF)
    nw = (1 + 0.2 * torch.randn(K, generator=g)).to(BF)
    cos, sin = R.rope_table(D, 2 * Tmax, 10000.0)
    cos, sin = cos.to(BF), sin.to(BF)
    h = R.rms_norm(x, nw)
    q = R.linear(h, wq).view(B, 1, H, D)
    k = R.linear(h, wk).view(B, 1, Hkv, D)
    v = R.linear(h, wv).view(B, 1, Hkv, D)
    qr, kr = R.apply_rope(q, k, cos[pos : pos + 1], sin[pos : pos + 1])
    kc = torch.zeros(B + 1, Tmax, Hkv, D, dtype=BF, device=cuda)
    vc = torch.zeros_like(kc)
    wp = ops.pack_qkv(wq.to(cuda), wk.to(cuda), wv.to(cuda))
    qo = ops.qkv_rope_append(x.to(cuda), wp, nw.to(cuda), 1e-5, H, Hkv, D, cos.to(cuda), sin.to(cuda), pos, kc, vc)
    for got, ref in ((qo.view(B, H, D), qr[:, 0]), (kc[:B, pos], kr[:, 0]), (vc[:B, pos], v[:, 0])):
        scale = ref.float().abs().max().item()
        err = (got.cpu().float() - ref.float()).abs().max().item()
        assert err <= 2 ** -6 * scale, (err, scale)
        assert (got.cpu() != ref).float().mean().item() < 0.08
    # nothing else in the cache was touched
    kc[:B, pos] = 0
    vc[:B, pos] = 0
    assert not kc.any() and not vc.any()


def _attn_ref64(q, k, v, L):
    """fp64 brute force: q (B,H,D), k/v (B,T,Hkv,D) -> (B,H,D)."""
    B, H, D = q.shape
    Hkv = k.shape[2]
    G = H // Hkv
    qd, kd, vd = q.double(), k[:, :L].double(), v[:, :L].double()
    out = torch.empty(B, H, D, dtype=torch.float64)
    for h in range(H):
        s = torch.einsum("bd,btd->bt", qd[:, h], kd[:, :, h // G]) / math.sqrt(D)
        p = torch.softmax(s, dim=-1)
        out[:, h] = torch.einsum("bt,btd->bd", p, vd[:, :, h // G])
    return out


@pytest.mark.parametrize("B,H,Hkv,D,L,ns", [(1, 6, 6, 128, 1153, 16), (2, 32, 8, 128, 700, 8), (3, 16, 16, 64, 64, 4),
                                            (2, 4, 2, 16, 37, 3), (1, 4, 4, 8, 5, 1), (4, 8, 4, 128, 1, 4),
                                            (2, 16, 2, 64, 300, 5)])
def test_attn_decode(cuda, B, H, Hkv, D, L, ns):
    from ohara_amd import ops

    g = torch.Generator().manual_seed(L)
    Tmax = L + 9
    q = torch.randn(B, H, D, generator=g).to(BF)
    k = torch.randn(B, Tmax, Hkv, D, generator=g).to(BF)
    v = torch.randn(B, Tmax, Hkv, D, generator=g).to(BF)
    ref = _attn_ref64(q, k, v, L)
    ws = ops.attn_workspace(B, H, Hkv, D, ns, cuda)
    kd, vd, qd = k.to(cuda), v.to(cuda), q.to(cuda).view(B, H * D)
    for _ in range(2):  # second call checks that the counters were left at zero
        out = ops.attn_decode(qd, kd, vd, H, Hkv, D, L, ns, ws)
        err = (out.cpu().double().view(B, H, D) - ref).abs().max().item()
        assert err <= 2e-2 * max(1.0, ref.abs().max().item()), err
    # device-side length
    pos_dev = torch.tensor([L - 1], dtype=torch.int32, device=cuda)
    out2 = ops.attn_decode(qd, kd, vd, H, Hkv, D, 0, ns, ws, pos_dev=pos_dev)
    assert torch.equal(out2, out)


def test_argmax(cuda):
    from ohara_amd import ops

    g = torch.Generator().manual_seed(3)
    logits = torch.randn(5, 65536, generator=g).to(BF)
    logits[1, 77] = logits[1, 9000] = 50.0  # tie -> lowest index
    logits[2, 65000] = 60.0
    ref = logits.float().argmax(-1)
    assert ref[1] == 77
    out = ops.argmax(logits.to(cuda))
    assert torch.equal(out.cpu(), ref)
    out = ops.argmax(logits.to(cuda), valid_vocab=60000)
    assert torch.equal(out.cpu(), logits[:, :60000].float().argmax(-1))


# ---- tiled MFMA GEMM (many rows) -------------------------------------------------------------

@pytest.mark.parametrize("M,N,K", [(128, 128, 64), (1, 16, 32), (65, 768, 768), (300, 2304, 768), (257, 100, 96),
                                   (1024, 768, 3072), (130, 65, 40), (2048, 640, 136)])
def test_gemm_tiled_store(cuda, M, N, K):
    from ohara_amd import ops

    g = torch.Generator().manual_seed(M * 7 + N + K)
    x = torch.randn(M, K, generator=g).to(BF)
    w = (torch.randn(N, K, generator=g) * 0.05).to(BF)
    ref = R.linear(x, w)
    out = ops.gemm(x.to(cuda), ops.pack_linear(w.to(cuda)))
    scale = ref.float().abs().max().item()
    err = (out.cpu().float() - ref.float()).abs().max().item()
    assert err <= 2 ** -7 * scale, (err, scale)
    assert (out.cpu() != ref).float().mean().item() < 0.05


def test_gemm_tiled_strided_rows_and_residual_in_place(cuda):
    from ohara_amd import ops

    g = torch.Generator().manual_seed(77)
    M, N, K = 200, 768, 3072
    xw = torch.randn(M, K + 64, generator=g).to(BF)  # a view with a row stride larger than K
    w = (torch.randn(N, K, generator=g) * 0.02).to(BF)
    res = torch.randn(M, N, generator=g).to(BF)
    ref = res + R.linear(xw[:, :K], w)
    buf = res.to(cuda).clone()
    out = ops.gemm(xw.to(cuda)[:, :K], ops.pack_linear(w.to(cuda)), residual=buf, out=buf)
    assert out.data_ptr() == buf.data_ptr()
    _ulp_close(out, ref, max_ulp=2, frac=0.05)


@pytest.mark.parametrize("M,F,K", [(256, 3072, 768), (100, 520, 64), (70, 12, 32)])
def test_gemm_tiled_swiglu(cuda, M, F, K):
    from ohara_amd import ops

    g = torch.Generator().manual_seed(F + M)
    x = torch.randn(M, K, generator=g).to(BF)
    wg = (torch.randn(F, K, generator=g) * 0.1).to(BF)
    wu = (torch.randn(F, K, generator=g) * 0.1).to(BF)
    ref = torch.nn.functional.silu(R.linear(x, wg)) * R.linear(x, wu)
    out = ops.gemm(x.to(cuda), ops.pack_gate_up(wg.to(cuda), wu.to(cuda)))
    scale = ref.float().abs().max().item()
    err = (out.cpu().float() - ref.float()).abs().max().item()
    assert err <= 2 ** -6 * scale, (err, scale)
    assert (out.cpu() != ref).float().mean().item() < 0.08


def test_gemm_tiled_matches_skinny_bitwise_on_shared_rows(cuda):
    """Both kernels accumulate a 32-column k-step per MFMA in the same lane order; with K = 32
    there is a single MFMA per output, so the two must agree bit for bit."""
    from ohara_amd import ops

    g = torch.Generator().manual_seed(3)
    x = torch.randn(64, 32, generator=g).to(BF).to(cuda)
    w = torch.randn(256, 32, generator=g).to(BF).to(cuda)
    wp = ops.pack_linear(w)
    assert torch.equal(ops.gemm(x, wp), ops.gemm_skinny(x, wp))


@pytest.mark.parametrize("B,S,H,Hkv,D,K", [(2, 100, 6, 6, 128, 768), (3, 40, 4, 2, 16, 64)])
def test_qkv_rope_append_many_rows(cuda, B, S, H, Hkv, D, K):
    """More than 64 rows without a fused norm: the tiled kernel with the rotary/append epilogue."""
    from ohara_amd import ops

    g = torch.Generator().manual_seed(S)
    Tmax, pos = 128, 5
    x = torch.randn(B * S, K, generator=g).to(BF)
    wq = (torch.randn(H * D, K, generator=g) * 0.05).to(BF)
    wk = (torch.randn(Hkv * D, K, generator=g) * 0.05).to(BF)
    wv = (torch.randn(Hkv * D, K, generator=g) * 0.05).to(BF)
    cos, sin = R.rope_table(D, 2 * Tmax, 10000.0)
    cos, sin = cos.to(BF), sin.to(BF)
    q = R.linear(x, wq).view(B, S, H, D)
    k = R.linear(x, wk).view(B, S, Hkv, D)
    v = R.linear(x, wv).view(B, S, Hkv, D)
    qr, kr = R.apply_rope(q, k, cos[pos : pos + S], sin[pos : pos + S])
    kc = torch.zeros(B, Tmax, Hkv, D, dtype=BF, device=cuda)
    vc = torch.zeros_like(kc)
    wp = ops.pack_qkv(wq.to(cuda), wk.to(cuda), wv.to(cuda))
    qo = ops.qkv_rope_append(x.to(cuda), wp, None, 1e-5, H, Hkv, D, cos.to(cuda), sin.to(cuda), pos, kc, vc, seq_len=S)
    for got, ref in ((qo.view(B, S, H, D), qr), (kc[:, pos : pos + S], kr), (vc[:, pos : pos + S], v)):
        scale = ref.float().abs().max().item()
        err = (got.cpu().float() - ref.float()).abs().max().item()
        assert err <= 2 ** -6 * scale, (err, scale)
        assert (got.cpu() != ref).float().mean().item() < 0.08
    assert kc[:, :pos].abs().sum().item() == 0 and kc[:, pos + S :].abs().sum().item() == 0


# ---- causal prefill attention on MFMA ----------------------------------------------------------

@pytest.mark.parametrize("B,S,H,Hkv,D,pos", [(2, 128, 6, 6, 128, 0), (1, 300, 4, 2, 128, 0), (3, 77, 8, 8, 64, 0),
                                             (2, 130, 8, 2, 64, 45), (1, 16, 2, 1, 128, 200), (1, 1024, 2, 2, 128, 0)])
def test_attn_prefill(cuda, B, S, H, Hkv, D, pos):
    from ohara_amd import ops

    g = torch.Generator().manual_seed(S + pos)
    Tmax = pos + S + 5
    q = torch.randn(B, S, H, D, generator=g).to(BF)
    k = torch.randn(B, Tmax, Hkv, D, generator=g).to(BF)
    v = torch.randn(B, Tmax, Hkv, D, generator=g).to(BF)
    # positions past the fed tokens hold junk the kernel must not read into the result
    k[:, pos + S :] = 1e4
    v[:, pos + S :] = -1e4
    ref = R.attention_core(q, k[:, : pos + S], v[:, : pos + S], pos).float()  # fp32 softmax, one rounding
    out = ops.attn_prefill(q.to(cuda).view(B * S, H * D), k.to(cuda), v.to(cuda), H, Hkv, D, pos, S)
    got = out.cpu().float().view(B, S, H * D)
    scale = ref.abs().max().item()
    assert (got - ref).abs().max().item() <= 2e-2 * max(1.0, scale)
    assert (got - ref).abs().mean().item() <= 2e-3 * max(1.0, scale)
    # the one-query-per-row decode kernel computes the same function
    ws = ops.attn_workspace(B * S, H, Hkv, D, 1, cuda)
    dec = ops.attn_cached(q.to(cuda).view(B * S, H * D), k.to(cuda), v.to(cuda), H, Hkv, D, pos, 1, ws, seq_len=S)
    assert (dec.cpu().float().view(B, S, H * D) - got).abs().max().item() <= 2e-2 * max(1.0, scale)


@pytest.mark.parametrize("B,H,Hkv,D,L", [(2, 6, 6, 128, 1500), (3, 8, 2, 64, 700), (1, 4, 1, 128, 4000)])
def test_attention_does_not_depend_on_how_the_context_is_cut(cuda, B, H, Hkv, D, L):
    """The softmax weights are rounded to bf16 relative to an INTEGER power of two above the running
    maximum, so cutting the context into 1, 2, ... 16 chunks (or walking it with the many-query kernel)
    changes only the order of fp32 sums: the outputs agree bit for bit almost everywhere and are never
    further apart than the last bf16 place at the output's scale."""
    from ohara_amd import ops

    g = torch.Generator().manual_seed(L)
    q = torch.randn(B, H * D, generator=g).to(BF).to(cuda)
    k = torch.randn(B, L + 3, Hkv, D, generator=g).to(BF).to(cuda)
    v = torch.randn(B, L + 3, Hkv, D, generator=g).to(BF).to(cuda)
    outs = {}
    for ns in (1, 2, 4, 7, 16):
        ws = ops.attn_workspace(B, H, Hkv, D, ns, cuda)
        outs[ns] = ops.attn_cached(q, k, v, H, Hkv, D, L - 1, ns, ws).clone()
    base = outs[1]
    scale = base.float().abs().max().item()
    for ns, o in outs.items():
        same = (o == base).float().mean().item()
        assert same >= 0.995, (ns, same)
        assert (o.float() - base.float()).abs().max().item() <= scale * 2.0 ** -8, ns
    # against the oracle (the library kernel's own cut: 512-key blocks around the true running maximum)
    ref = R.attention_core(q.cpu().view(B, 1, H, D), k.cpu()[:, :L], v.cpu()[:, :L], L - 1).view(B, H * D)
    assert (base.cpu().float() - ref.float()).abs().max().item() <= scale * 2.0 ** -7
    assert (base.cpu().float() - ref.float()).abs().mean().item() <= scale * 2.0 ** -10
