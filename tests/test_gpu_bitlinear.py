"""BitLinear integer kernels (C ABI: ohara_bitlinear_pack_ternary / ohara_act_quant_int8 /
ohara_gemv_ternary_i8 / ohara_bitlinear_bf16) against the CPU oracle.

Contract: the int32 accumulators are BIT-EXACT against a CPU int32 matmul of the same int8
activations and ternary weights.  The float parts (RMSNorm before quantisation, the final
scale) follow the bf16 tolerance of the other kernels.
"""

import pytest
import torch

from oracle import bitlinear_ref as BL
from oracle import llama_ref as R

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


@pytest.mark.parametrize("rows,N,K", [(1, 2048, 2048), (8, 5632, 2048), (3, 2048, 5632), (17, 48, 96), (70, 100, 520),
                                      (2, 16, 32)])
def test_ternary_gemv_accumulators_bit_exact(cuda, rows, N, K):
    from ohara_amd import ops

    g = torch.Generator().manual_seed(rows + N + K)
    t = torch.randint(-1, 2, (N, K), generator=g, dtype=torch.int8)
    q = torch.randint(-128, 128, (rows, K), generator=g, dtype=torch.int8)
    s = (torch.rand(rows, generator=g) * 50 + 1).float()
    gamma = 0.0213
    want_acc = BL.int_accumulate(q, t)
    ldq = (K + 15) // 16 * 16
    qd = torch.zeros(rows, ldq, dtype=torch.int8)
    qd[:, :K] = q
    sumq = q.to(torch.int32).sum(-1).to(torch.int32)
    w = ops.pack_ternary(t.to(cuda), gamma)
    res = torch.randn(rows, N, generator=g).to(BF)
    out, acc = ops.gemv_ternary(qd.to(cuda), s.to(cuda), sumq.to(cuda), w, residual=res.to(cuda), want_acc=True)
    assert torch.equal(acc.cpu(), want_acc), "int32 accumulators must be bit-exact"
    want = res + ((want_acc.float() / s[:, None]) * gamma).to(BF)
    assert torch.equal(out.cpu(), want)


def test_act_quant_matches_oracle(cuda):
    from ohara_amd import ops

    g = torch.Generator().manual_seed(0)
    for rows, K in ((5, 2048), (3, 5632), (4, 104)):
        x = (torch.randn(rows, K, generator=g) * 2).to(BF)
        nw = (1 + 0.2 * torch.randn(K, generator=g)).to(BF)
        q_ref, s_ref = BL.activation_quant(R.rms_norm(x, nw))
        q, s, sq = ops.act_quant(x.to(cuda), nw.to(cuda))
        q = q.cpu()[:, :K]
        # the norm's fp32 reduction order can flip a bf16 rounding of x_hat, i.e. move a q by one
        diff = (q.int() - q_ref.int()).abs()
        assert int(diff.max()) <= 1 and float((diff > 0).float().mean()) < 5e-3
        torch.testing.assert_close(s.cpu(), s_ref[:, 0], rtol=1e-2, atol=0)
        assert torch.equal(sq.cpu(), q.int().sum(-1).to(torch.int32))
    # closed forms: equal magnitudes quantise to +-127; half-way cases round to even
    x = torch.tensor([[0.5, -0.5, 0.5, -0.5] * 8]).to(BF)
    q, s, _ = ops.act_quant(x.to(cuda), torch.ones(32, dtype=BF, device=cuda))
    assert q.cpu()[0, :4].tolist() == [127, -127, 127, -127]


@pytest.mark.parametrize("rows,N,K", [(1, 2048, 2048), (8, 2048, 5632), (33, 64, 128)])
def test_fused_bitlinear(cuda, rows, N, K):
    from ohara_amd import ops

    g = torch.Generator().manual_seed(N + K)
    x = torch.randn(rows, K, generator=g).to(BF)
    nw = (1 + 0.1 * torch.randn(K, generator=g)).to(BF)
    wfloat = torch.randn(N, K, generator=g) * 0.03
    t, gamma = BL.weight_ternarize(wfloat)
    w = ops.pack_ternary(t.to(cuda), float(gamma))
    out, acc = ops.bitlinear(x.to(cuda), nw.to(cuda), w, want_acc=True)
    # accumulators: exact against the kernel's own quantised activations
    q, s, sq = ops.act_quant(x.to(cuda), nw.to(cuda))
    assert torch.equal(acc.cpu(), BL.int_accumulate(q.cpu()[:, :K], t))
    # end to end against the oracle (which quantises on its own): bf16-level agreement
    want = BL.bitlinear_forward(x, nw, t, gamma)
    scale = want.float().abs().max().item()
    d = (out.cpu().float() - want.float()).abs()
    assert d.max().item() <= 3e-2 * scale and d.mean().item() <= 3e-3 * scale
    # and against the reference's float fake-quant formulation (bitnet.py:29-59)
    fq = BL.fake_quant_forward(x.float(), nw.float(), wfloat)
    assert (out.cpu().float() - fq).abs().mean().item() <= 1e-2 * scale


def test_fused_bitlinear_with_block_norm(cuda):
    """pre_norm_w folds the block-level RMSNorm (llama.py:199-200) into the quantisation pass: same
    result as normalising first with the stand-alone kernel."""
    from ohara_amd import ops

    g = torch.Generator().manual_seed(9)
    rows, N, K = 5, 2048, 2048
    x = (torch.randn(rows, K, generator=g) * 3).to(BF).to(cuda)
    pre = (1 + 0.2 * torch.randn(K, generator=g)).to(BF).to(cuda)
    nw = (1 + 0.1 * torch.randn(K, generator=g)).to(BF).to(cuda)
    t = torch.randint(-1, 2, (N, K), generator=g, dtype=torch.int8)
    w = ops.pack_ternary(t.to(cuda), 0.04)
    fused, acc_f = ops.bitlinear(x, nw, w, want_acc=True, pre_norm_w=pre)
    two, acc_t = ops.bitlinear(ops.rmsnorm(x, pre), nw, w, want_acc=True)
    # the two norms' fp32 reduction orders can flip single bf16 roundings: nearly all accumulators
    # identical, the rest off by a few units
    d = (acc_f - acc_t).abs()
    assert float((d > 0).float().mean()) < 0.2 and int(d.max()) <= 4 * 127
    want = BL.bitlinear_forward(R.rms_norm(x.cpu(), pre.cpu()), nw.cpu(), t, 0.04)
    scale = want.float().abs().max().item()
    e = (fused.cpu().float() - want.float()).abs()
    assert e.max().item() <= 3e-2 * scale and e.mean().item() <= 3e-3 * scale


def test_ternarize_matches_oracle(cuda):
    from ohara_amd.bitnet import ternarize

    w = torch.randn(64, 96, generator=torch.Generator().manual_seed(1)) * 0.04
    t, gamma = ternarize(w)
    t2, g2 = BL.weight_ternarize(w)
    assert torch.equal(t, t2) and abs(gamma - float(g2)) < 1e-9


def test_bitnet_llama_parity(cuda):
    """A small ternary Llama (d 256, 3 layers, 2 heads x 128, GQA off): prefill + cached steps
    against the oracle; greedy tokens up to a near-tie."""
    from ohara_amd.bitnet import BitLlama
    from ohara_amd.llama import Config

    kw = dict(vocab_size=320, hidden_size=256, intermediate_size=512, num_attention_heads=2,
              num_key_value_heads=0, num_hidden_layers=3, max_sequence_length=64, rope_theta=10000.0)
    rcfg = R.RefConfig(**kw)
    w = BL.init_ternary_weights(rcfg, seed=2, dtype=BF, gamma=0.05)
    ref = R.RefLlama(rcfg, w)
    model = BitLlama(Config(**kw), w, device=cuda)
    ids = torch.randint(0, 320, (2, 9), generator=torch.Generator().manual_seed(0))
    rc, cache = ref.build_kv_cache(2), model.build_kv_cache(2)
    want = ref(ids, rc, 0)
    got = model(ids.to(cuda), cache, 0)
    scale = want.float().abs().max().item()

    def close(a, b):
        d = (a.float().cpu() - b.float()).abs()
        # int8 activation quantisation turns a one-ulp bf16 flip into a full quantisation step,
        # so the ternary model's noise floor is several times the bf16 model's
        assert d.max().item() <= 8e-2 * scale and d.mean().item() <= 1e-2 * scale, (d.max().item(), d.mean().item(), scale)

    close(got, want)
    nxt = want[:, -1].float().argmax(-1, keepdim=True)
    for step in range(3):
        want = ref(nxt, rc, 9 + step)
        got = model(nxt.to(cuda), cache, 9 + step)
        close(got, want)
        nxt = want[:, -1].float().argmax(-1, keepdim=True)
    assert cache[0].length == 12
    toks = model.generate_greedy(ids.to(cuda), 6).cpu()
    assert toks.shape == (2, 6)


def test_fused_groups_match_the_separate_calls(cuda):
    """One launch for q/k/v + rotary + append and one for gate/up + SwiGLU: the same arithmetic as
    the separate BitLinear, rope_append and silu_mul calls, so bit-identical results."""
    from ohara_amd import ops

    g = torch.Generator().manual_seed(21)
    B, S, H, Hkv, D, K, F, Tmax, pos = 3, 2, 4, 2, 64, 256, 384, 16, 5
    rows = B * S
    x = (torch.randn(rows, K, generator=g) * 2).to(BF).to(cuda)
    pre = (1 + 0.2 * torch.randn(K, generator=g)).to(BF).to(cuda)

    def proj(n):
        t = torch.randint(-1, 2, (n, K), generator=g, dtype=torch.int8)
        return (1 + 0.1 * torch.randn(K, generator=g)).to(BF).to(cuda), ops.pack_ternary(t.to(cuda), 0.03 + 0.01 * n / 256)

    pq, pk, pv, pg, pu = proj(H * D), proj(Hkv * D), proj(Hkv * D), proj(F), proj(F)
    cos, sin = R.rope_table(D, 2 * Tmax, 10000.0)
    cos, sin = cos.to(BF).to(cuda), sin.to(BF).to(cuda)
    kc1 = torch.zeros(B, Tmax, Hkv, D, dtype=BF, device=cuda)
    vc1, kc2, vc2 = torch.zeros_like(kc1), torch.zeros_like(kc1), torch.zeros_like(kc1)
    q1 = ops.bitlinear(x, pq[0], pq[1], pre_norm_w=pre)
    k1 = ops.bitlinear(x, pk[0], pk[1], pre_norm_w=pre)
    v1 = ops.bitlinear(x, pv[0], pv[1], pre_norm_w=pre)
    ops.rope_append(q1, k1, v1, B, S, H, Hkv, D, cos, sin, pos, kc1, vc1)
    q2 = ops.bitlinear_qkv_rope_append(x, pre, [pq, pk, pv], 1e-5, H, Hkv, D, cos, sin, pos, kc2, vc2, seq_len=S)
    assert torch.equal(q1, q2) and torch.equal(kc1, kc2) and torch.equal(vc1, vc2)
    assert kc2[:, pos : pos + S].abs().sum().item() > 0 and kc2[:, :pos].abs().sum().item() == 0
    a1 = ops.silu_mul(ops.bitlinear(x, pg[0], pg[1], pre_norm_w=pre), ops.bitlinear(x, pu[0], pu[1], pre_norm_w=pre))
    a2 = ops.bitlinear_gate_up(x, pre, pg, pu)
    assert torch.equal(a1, a2)


@pytest.mark.parametrize("B", [9, 20, 70])
def test_bitnet_decode_at_larger_batches(cuda, B):
    """The ternary model with more than 8, more than 16 and more than 64 sequences (the last takes
    the unfused projection path for single-token calls too): prefill and cached steps against the
    oracle."""
    from ohara_amd.bitnet import BitLlama
    from ohara_amd.llama import Config

    kw = dict(vocab_size=320, hidden_size=256, intermediate_size=512, num_attention_heads=2,
              num_key_value_heads=0, num_hidden_layers=2, max_sequence_length=32, rope_theta=10000.0)
    rcfg = R.RefConfig(**kw)
    w = BL.init_ternary_weights(rcfg, seed=5, dtype=BF, gamma=0.05)
    ref, model = R.RefLlama(rcfg, w), BitLlama(Config(**kw), w, device=cuda)
    ids = torch.randint(0, 320, (B, 8), generator=torch.Generator().manual_seed(B))
    rc, cache = ref.build_kv_cache(B), model.build_kv_cache(B)

    def close(a, b):
        scale = b.float().abs().max().item()
        d = (a.float().cpu() - b.float()).abs()
        assert d.max().item() <= 8e-2 * scale and d.mean().item() <= 1e-2 * scale, (B, d.max().item(), d.mean().item(), scale)

    close(model(ids[:, :5].to(cuda), cache, 0), ref(ids[:, :5], rc, 0))
    for t in (5, 6, 7):
        close(model(ids[:, t:t + 1].to(cuda), cache, t), ref(ids[:, t:t + 1], rc, t))


PERSISTENT_SHAPES = [
    # d, heads, d_ff, vocab, layers, batch
    (256, 2, 512, 320, 3, 1),     # head_dim 128, one 256-column chunk per row
    (256, 2, 512, 320, 3, 5),
    (512, 8, 1536, 333, 2, 1),    # head_dim 64, several chunks, vocabulary not a multiple of 16
    (512, 8, 1536, 333, 2, 8),
    (320, 5, 528, 300, 2, 3),     # widths that are not multiples of 256 (zero-padded code rows)
    (256, 2, 2304, 320, 4, 6),    # a hidden width beyond 2048 (rows parked in LDS at batch > 1), four layers
    (256, 2, 2304, 320, 4, 1),
    (256, 2, 512, 320, 3, 2),     # code rows of 272 bytes: the sets of a layer's code mailbox start between cache lines
    (512, 8, 1536, 333, 2, 7),
]


@pytest.mark.parametrize("d,heads,ff,vocab,layers,B", PERSISTENT_SHAPES)
def test_bitnet_persistent_step_matches_the_kernel_chain(cuda, d, heads, ff, vocab, layers, B):
    """The single-launch ternary decode step against the chain of BitLinear kernels and the oracle:
    the rows appended to layer 0's cache (no attention in front of them) bit for bit, nearly all
    logits bit for bit, tokens from the captured graph equal to the eager launches."""
    from ohara_amd.bitnet import BitLlama
    from ohara_amd.llama import Config

    kw = dict(vocab_size=vocab, hidden_size=d, intermediate_size=ff, num_attention_heads=heads,
              num_key_value_heads=0, num_hidden_layers=layers, max_sequence_length=64, rope_theta=10000.0)
    rcfg = R.RefConfig(**kw)
    w = BL.init_ternary_weights(rcfg, seed=7, dtype=BF, gamma=0.05)
    ref, model = R.RefLlama(rcfg, w), BitLlama(Config(**kw), w, device=cuda)
    assert model.supports_persistent(B)
    P, steps = 9, 12
    ids = torch.randint(0, vocab, (B, P), generator=torch.Generator().manual_seed(B + d))

    sess = model.session(B, steps, persistent=True)
    sess.prefill(ids.to(cuda))
    first = sess.ids.clone()
    # chain: same prompt, same first token, one cached step
    cache = model.build_kv_cache(B)
    model(ids.to(cuda), cache, 0, last_only=True)
    chain_logits = model(first.view(B, 1), cache, P, last_only=True)[:, 0]
    sess.step()
    torch.cuda.synchronize()
    sess.check_error()
    assert torch.equal(sess.cache[0].key[:, P], cache[0].key[:, P])
    assert torch.equal(sess.cache[0].value[:, P], cache[0].value[:, P])
    # oracle
    rc = ref.build_kv_cache(B)
    ref(ids, rc, 0)
    want = ref(first.cpu().view(B, 1), rc, P)[:, -1].float()
    scale = want.abs().max().item()
    # at these small widths one int8 step of a code is a large relative change: the oracle distance of
    # either path is the model's noise (the two paths are at the same distance from it).  The kernels'
    # attention rounds its softmax weights to bf16 as the oracle's does, but relative to a power of two
    # instead of the maximum itself: one output in four is a bf16 step off, which the absmax quantisers
    # of the layers behind it amplify
    for got, name in ((sess.logits, "persistent"), (chain_logits, "chain")):
        e = (got.float().cpu() - want).abs()
        assert e.max().item() <= 1e-1 * scale and e.mean().item() <= 2e-2 * scale, (name, e.max().item(), e.mean().item(), scale)
    # against the chain: same codes, same integer sums, same rounding points; only the order of the
    # fp32 sums inside attention differs, which can flip single bf16 roundings
    same = (sess.logits == chain_logits).float().mean().item()
    e = (sess.logits.float() - chain_logits.float()).abs()
    assert same >= 0.98 and e.max().item() <= 2e-2 * scale, (same, e.max().item(), scale)
    assert torch.equal(sess.ids, ops_argmax(sess.logits))
    # the rest of the tokens from the graph; then the same tokens again from eager launches
    sess.run(steps - 2)
    toks = sess.tokens()
    assert toks.shape == (B, steps)
    again = model.generate_greedy(ids.to(cuda), steps, persistent=True, use_graph=False)
    assert torch.equal(toks, again)
    assert int(toks.min()) >= 0 and int(toks.max()) < vocab
    chain = model.generate_greedy(ids.to(cuda), steps, persistent=False)
    assert (toks == chain).float().mean().item() >= 0.9


def ops_argmax(logits):
    from ohara_amd import ops

    return ops.argmax(logits.contiguous())
