"""The headline configurations at their full sizes, checked through properties that do not need a
CPU oracle of that size: batch invariance (a sequence decodes the same alone and inside a batch of
32), softmax normalisation (constant values come back unchanged) and agreement with a plain fp32
torch evaluation of sub-sampled (sequence, head) pairs on the device.
"""

import math

import pytest
import torch

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


@pytest.mark.parametrize("B,L", [(b, l) for b in (1, 16, 64) for l in (1024, 4096, 16384, 32768)])
def test_decode_attention_microbench_shape(cuda, B, L):
    """32 query / 8 KV heads x 128, one query per sequence over L cached positions: every (batch,
    context) point the benchmark times, with the benchmark's chunk count (64 x 32768 is 4.3 GB per
    tensor)."""
    from ohara_amd import ops

    H, Hkv, D = 32, 8, 128
    G = H // Hkv
    ns = max(1, min(1024 // (B * Hkv), L // 128, 64))  # bench.py:bench_attention_microbench
    g = torch.Generator(device=cuda).manual_seed(1)
    q = torch.randn(B, H * D, device=cuda, generator=g).to(BF)
    k = torch.randn(B, L, Hkv, D, device=cuda, generator=g).to(BF)
    v = torch.randn(B, L, Hkv, D, device=cuda, generator=g).to(BF)
    ws = ops.attn_workspace(B, H, Hkv, D, ns, cuda)
    out = ops.attn_decode(q, k, v, H, Hkv, D, L, ns, ws).view(B, H, D)
    # sub-sampled (sequence, head) pairs against fp32 torch on the device
    for b, h in ((0, 0), (B // 2, 13), (B - 1, H - 1), (min(3, B - 1), 6)):
        kk, vv = k[b, :, h // G].float(), v[b, :, h // G].float()
        s = (kk @ q[b].view(H, D)[h].float()) / math.sqrt(D)
        want = torch.softmax(s, 0) @ vv
        err = (out[b, h].float() - want).abs().max().item()
        assert err <= 2e-2 * max(1.0, want.abs().max().item()), (b, h, err)
    # the weights of every head sum to one: constant values come back unchanged (to bf16 rounding)
    v.fill_(0.75)
    out = ops.attn_decode(q, k, v, H, Hkv, D, L, ns, ws)
    assert (out.float() - 0.75).abs().max().item() <= 2 ** -8
    # a context of identical keys is a plain average of the values
    k.copy_(k[:, :1].expand_as(k))
    v.copy_(torch.randn(B, L, Hkv, D, device=cuda, generator=g).to(BF))
    out = ops.attn_decode(q, k, v, H, Hkv, D, L, ns, ws).view(B, Hkv, G, D)
    want = v.float().mean(1)  # (B, Hkv, D)
    assert (out.float() - want[:, :, None, :]).abs().max().item() <= 2e-3


@pytest.mark.parametrize("B,L", [(16, 16384), (64, 4096), (1, 32768)])
def test_decode_attention_microbench_shape_int8_cache(cuda, B, L):
    """The same shape over the int8 cache, as the benchmark times it: the kernel must return what bf16
    attention returns over the dequantised cache (same values, same rounding points; the tiles are cut
    differently, so single bf16 roundings may differ), and sub-sampled pairs must match fp32 torch."""
    from ohara_amd import ops
    from ohara_amd.llama import KVCache

    H, Hkv, D = 32, 8, 128
    G = H // Hkv
    ns = max(1, min(1024 // (B * Hkv), L // 128, 64))
    g = torch.Generator(device=cuda).manual_seed(1)
    q = torch.randn(B, H * D, device=cuda, generator=g).to(BF)
    k = torch.randn(B, L, Hkv, D, device=cuda, generator=g).to(BF)
    v = torch.randn(B, L, Hkv, D, device=cuda, generator=g).to(BF)
    cache = KVCache((B, L, Hkv, D), L, device=cuda, dtype=BF, int8=True)
    step = max(1, 4096 // B)
    for p0 in range(0, L, step):
        ops.kv_quant_append(k[:, p0:p0 + step].contiguous(), v[:, p0:p0 + step].contiguous(), cache, p0)
    ws = ops.attn_workspace(B, H, Hkv, D, ns, cuda)
    out = ops.attn_cached_int8(q, cache, H, Hkv, D, L - 1, ns, ws).clone()
    kd, vd = ops.kv_dequant(cache, "key", B, L), ops.kv_dequant(cache, "value", B, L)
    assert (kd.float() - k.float()).abs().max().item() <= 0.05  # tests/test_modules.py:82-100 of the reference
    same = ops.attn_decode(q, kd, vd, H, Hkv, D, L, ns, ws)
    scale = same.float().abs().max().item()
    assert (out.float() - same.float()).abs().max().item() <= 2.0 ** -7 * scale  # one bf16 ulp of the largest output
    assert (out == same).float().mean().item() >= 0.99
    o3 = out.view(B, H, D)
    for b, h in ((0, 0), (B // 2, 13), (B - 1, H - 1)):
        kk, vv = kd[b, :, h // G].float(), vd[b, :, h // G].float()
        s_ = (kk @ q[b].view(H, D)[h].float()) / math.sqrt(D)
        want = torch.softmax(s_, 0) @ vv
        assert (o3[b, h].float() - want).abs().max().item() <= 2e-2 * max(1.0, want.abs().max().item()), (b, h)


def test_d12_sampled_session_at_the_full_vocabulary(cuda):
    """The sampled mode of the headline configuration end to end: d12 (vocabulary 65536), temperature
    0.8 / top-k 50 / top-p 0.9, uniform draws fixed in advance and shared with the oracle sampler;
    batch 1 on the single-launch kernel and batch 8, prompts of 1024 tokens.  At every step the oracle
    sampler, applied to the session's own logits of that step, must place the session's token in the
    CDF interval that holds the step's draw."""
    import bench
    from oracle.sampling_ref import candidate_cdf_ref
    from ohara_amd.llama import Llama
    from ohara_amd.sampling import SamplingConfig

    cfg, st = bench.d12_state(cuda)
    model = Llama(cfg, st, device=cuda)
    scfg = SamplingConfig(temperature=0.8, top_k=50, top_p=0.9)
    for B, N in ((1, 24), (8, 10)):
        g = torch.Generator().manual_seed(B)
        prompt = torch.randint(0, cfg.vocab_size, (B, 1024), generator=g)
        u = torch.rand(N, B, generator=g)
        sess = model.session(B, N, sampling=scfg, u=u.to(cuda))
        sess.prefill(prompt.to(cuda))
        own = [sess.logits.clone().cpu()]
        for _ in range(N - 1):
            sess.step()
            own.append(sess.logits.clone().cpu())
        toks = sess.tokens().cpu()
        assert toks.shape == (B, N)
        for t in range(N):
            ids, cdf = candidate_cdf_ref(own[t].view(B, 1, -1).float(), scfg.temperature, scfg.top_p, scfg.top_k)
            for b in range(B):
                hit = (ids[b] == int(toks[b, t])).nonzero()
                assert hit.numel(), (B, t, b, "token outside the candidate order")
                j = int(hit[0])
                lo = float(cdf[b, j - 1]) if j > 0 else 0.0
                assert lo - 5e-5 <= float(u[t, b]) <= float(cdf[b, j]) + 5e-5, (B, t, b, lo, float(cdf[b, j]), float(u[t, b]))
        # the captured graph replays the same tokens
        sess2 = model.session(B, N, sampling=scfg, u=u.to(cuda))
        sess2.prefill(prompt.to(cuda))
        sess2.run(N - 1)
        assert torch.equal(sess2.tokens().cpu(), toks)


def test_d12_batch32_prompt1024_matches_single_sequence_runs(cuda):
    """Headline decode configuration: 32 sequences, prompts of 1024 tokens, cache capacity 4096.
    Rows of the batched run equal the same sequences decoded alone, to bf16 accumulation noise
    (the kernels that serve 1 row and 32 rows differ, so this is not a bit-for-bit identity)."""
    import bench
    from ohara_amd.llama import Llama

    cfg, st = bench.d12_state(cuda)
    model = Llama(cfg, st, device=cuda)
    B, P, steps = 32, 1024, 6
    prompt = torch.randint(0, cfg.vocab_size, (B, P), generator=torch.Generator().manual_seed(0)).to(cuda)
    cache = model.build_kv_cache(B)
    logits = [model(prompt, cache, 0, last_only=True)[:, 0]]
    toks = [logits[0].float().argmax(-1)]
    for t in range(steps):
        logits.append(model(toks[-1].view(B, 1), cache, P + t)[:, 0])
        toks.append(logits[-1].float().argmax(-1))
    assert cache[0].length == P + steps
    for b in (0, 17, 31):
        c1 = model.build_kv_cache(1)
        l1 = model(prompt[b:b + 1], c1, 0, last_only=True)[:, 0]
        for t in range(steps + 1):
            scale = l1.float().abs().max().item()
            d = (logits[t][b].float() - l1[0].float()).abs()
            assert d.max().item() <= 2e-2 * scale and d.mean().item() <= 3e-3 * scale, (b, t, d.max().item(), scale)
            if t < steps:
                l1 = model(toks[t][b].view(1, 1), c1, P + t)[:, 0]  # teacher-forced on the batch's tokens
    # the device-resident loop reproduces the step-by-step tokens
    got = model.generate_greedy(prompt, steps + 1)
    agree = (got == torch.stack(toks, 1)).float().mean().item()
    assert agree >= 0.97, agree


@pytest.mark.parametrize("B", [1, 8])
def test_d12_single_launch_decode_over_the_int8_cache(cuda, B):
    """d12 size, prompts of 1088 tokens (chunks of more than 64 positions: a wave's second tile, and the appended
    position in it), cache capacity 4096, int8 KV cache: the single-launch kernel - which reads codes and statistics
    and quantises the appended row itself - against the kernel chain on the same caches, teacher-forced on the chain's
    tokens: logits to a bf16 ulp, the first layer's appended codes and statistics bit for bit, deeper layers' rows through
    the values their codes stand for, nothing written behind the last position."""
    import bench
    from ohara_amd.llama import Llama

    cfg, st = bench.d12_state(cuda)
    model = Llama(cfg, st, device=cuda)
    P, steps = 1088, 6
    prompt = torch.randint(0, cfg.vocab_size, (B, P), generator=torch.Generator().manual_seed(B + 40)).to(cuda)
    chain_cache = model.build_kv_cache(B, int8=True)
    chain = model.session(B, steps + 1, kv_cache=chain_cache, persistent=False)
    chain.prefill(prompt)
    want, fed = [chain.logits.float().cpu()], []
    for _ in range(steps):
        fed.append(want[-1].argmax(-1))
        chain.feed(fed[-1].to(cuda))
        chain.step()
        want.append(chain.logits.float().cpu())
    cache = model.build_kv_cache(B, int8=True)
    sess = model.session(B, steps + 1, kv_cache=cache, persistent=True)
    assert sess.persistent
    sess.prefill(prompt)
    for t in range(steps):
        sess.feed(fed[t].to(cuda))
        sess.step()
        got = sess.logits.float().cpu()
        scale = want[t + 1].abs().max().item()
        d = (got - want[t + 1]).abs()
        assert d.max().item() <= 1.5e-2 * scale and d.mean().item() <= 2.5e-3 * scale, (B, t, d.max().item(), d.mean().item(), scale)
    sess.check_error()
    from ohara_amd import ops
    for l in (0, 5, 11):
        for name in ("key", "value"):
            a = getattr(cache[l], name)[:B, P:P + steps].int()
            b = getattr(chain_cache[l], name)[:B, P:P + steps].int()
            if l == 0:  # the first layer's rows depend on the fed tokens only
                assert torch.equal(a, b), name
            # deeper layers: through the values the codes stand for (a last bit of a row's minimum or maximum moves
            # every code of the row)
            va = ops.kv_dequant(cache[l], name, B, P + steps)[:, P:].float()
            vb = ops.kv_dequant(chain_cache[l], name, B, P + steps)[:, P:].float()
            scale = vb.abs().max().item()
            assert (va - vb).abs().max().item() <= 3e-2 * scale and (va - vb).abs().mean().item() <= 4e-3 * scale, (l, name)
        if l == 0:
            assert torch.equal(cache[l].stats[:B, :, P:P + steps], chain_cache[l].stats[:B, :, P:P + steps])
        assert not cache[l].key[:B, P + steps:].any() and not cache[l].stats[:B, :, P + steps:].any()


def test_phi2_width_prefill_and_decode_against_the_oracle(cuda):
    """Phi-2's real widths (d 2560, 32 heads of 80 with 32 rotated features, MLP 10240, vocabulary
    51200) on four layers: a 70-token prefill (the tiled kernel's epilogues), cached decode steps of
    3 sequences (8- and 16-wave strip kernels, context chunks in attention) and the uncached forward,
    against the CPU oracle on the same bf16 weights."""
    from ohara_amd.phi import Phi, PhiConfig
    from oracle import phi_ref as P

    kw = dict(num_hidden_layers=4, max_sequence_length=256)
    rcfg = P.RefPhiConfig(**kw)
    w = P.init_weights(rcfg, seed=11, dtype=torch.bfloat16, std=0.02, bias_std=0.02)
    ref, model = P.RefPhi(rcfg, w), Phi(PhiConfig(**kw), w, device=cuda)
    g = torch.Generator().manual_seed(0)
    B, S0 = 3, 70
    ids = torch.randint(0, rcfg.vocab_size, (B, S0 + 2), generator=g)
    rc, cache = ref.build_kv_cache(B), model.build_kv_cache(B)

    def close(got, want):
        got, want = got.float().cpu(), want.float()
        scale = want.abs().max().item()
        d = (got - want).abs()
        assert d.max().item() <= 4e-2 * scale and d.mean().item() <= 4e-3 * scale, (d.max().item(), d.mean().item(), scale)

    close(model(ids[:, :S0].to(cuda), cache, 0, last_only=True)[:, 0], ref(ids[:, :S0], rc, 0)[:, -1])
    for t in (S0, S0 + 1):
        close(model(ids[:, t:t + 1].to(cuda), cache, t), ref(ids[:, t:t + 1], rc, t))
    close(cache[-1].key[:B, :S0 + 2], rc[-1].key[:B, :S0 + 2])
    toks = model.generate_greedy(ids[:, :S0].to(cuda), 4)
    assert toks.shape == (B, 4) and int(toks.min()) >= 0 and int(toks.max()) < rcfg.vocab_size


def _near_tie(logits_row, a, b, ulps=2):
    la, lb = float(logits_row[a]), float(logits_row[b])
    ulp = 2.0 ** (math.floor(math.log2(max(abs(la), abs(lb), 1e-30))) - 7)
    return abs(la - lb) <= ulps * ulp


def test_bitnet_c4_model_full_size(cuda):
    """The BitNet-b1.58 ternary Llama at its full size (d 2048, 24 layers, 16 heads x 128, FFN 5632,
    vocabulary 32000, cache capacity 2048):
    (a) the int32 accumulators of layer 0's q / k / v / gate / up projections, computed by the kernels
        from the model's own embedding rows, equal a CPU integer product of the kernels' own int8
        codes with the ternary weights, bit for bit;
    (b) a 64-token prefill and three cached decode steps against the CPU oracle (whole model);
    (c) at context 2047 -> 2048 (the last cache row), a decode step of 8 sequences equals the same
        sequences decoded alone; a captured graph replays to the eager result bit for bit;
    (d) the single-launch decode step on the same caches against the kernel chain (batch 8 and one
        sequence), and 128 greedy tokens from its captured graph against its eager launches."""
    import bench
    from ohara_amd import ops
    from ohara_amd.bitnet import BitLlama
    from oracle import bitlinear_ref as BL
    from oracle import llama_ref as R

    cfg, st = bench.bitnet_c4_state(cuda)
    model = BitLlama(cfg, st, device=cuda)
    g = torch.Generator().manual_seed(5)
    V = cfg.vocab_size

    # (a) layer 0, rows = embedding rows of 8 tokens
    ids8 = torch.randint(0, V, (8,), generator=g)
    h = ops.embed(ids8.to(cuda), model.token_emb)
    L0 = model.layers[0]
    for name in ("attn.query", "attn.key", "attn.value", "ff.gate", "ff.up"):
        packed, nw = L0[name]
        pre = L0["norm1"] if name.startswith("attn") else L0["norm2"]
        q, s, sq = ops.act_quant(ops.rmsnorm(h, pre, model.eps), nw, model.eps)
        _, acc = ops.gemv_ternary(q, s, sq, packed, want_acc=True)
        want = BL.int_accumulate(q.cpu()[:, : packed.k], st[f"layers.0.{name}.ternary"].cpu(), force_int=True)
        assert torch.equal(acc.cpu(), want), name
        # the fused kernel (block norm + BitLinear norm + codes in one pass) reduces the norms in another
        # fp32 order, which flips single bf16 roundings: nearly all accumulators identical
        _, acc_f = ops.bitlinear(h, nw, packed, model.eps, want_acc=True, pre_norm_w=pre)
        d = (acc_f - acc).abs()
        assert float((d > 0).float().mean()) < 0.2 and int(d.max()) <= 4 * 127, name

    # (b) the whole model against the oracle: prefill 64, then 3 decode steps (2 sequences)
    cpu_state = {k: v.cpu() for k, v in st.items()}
    del st
    rcfg = R.RefConfig(**{f: getattr(cfg, f) for f in ("vocab_size", "hidden_size", "intermediate_size",
                                                      "num_attention_heads", "num_key_value_heads",
                                                      "num_hidden_layers", "max_sequence_length", "rope_theta")})
    cos, sin = R.rope_table(rcfg.head_dim, rcfg.max_sequence_length * 2, rcfg.rope_theta)
    cpu_state["freq_cos"], cpu_state["freq_sin"] = cos.to(BF), sin.to(BF)
    ref = R.RefLlama(rcfg, cpu_state)
    ids = torch.randint(0, V, (2, 64), generator=g)

    # (b1) one layer, operator by operator, each fed the ORACLE's inputs: identical inputs give
    # bit-identical outputs on nearly every row.  (The per-row absmax scale makes the quantiser
    # discontinuous: when a bf16 rounding flips the largest element of a row, every code of the row
    # is re-rounded; such rows differ at the 1e-3 level, all others not at all.)
    import torch.nn.functional as F

    S1 = 8
    w = cpu_state

    def bl(name, inp, pre=None):
        if pre is not None:
            inp = R.rms_norm(inp, w[f"layers.0.{pre}.weight"])
        return BL.bitlinear_forward(inp, w[f"layers.0.{name}.rms_norm.weight"], w[f"layers.0.{name}.ternary"],
                                    w[f"layers.0.{name}.gamma"])

    def same_rows(got, want, what, min_identical=0.75, elements=False):
        got, want = got.float().cpu().reshape(2 * S1, -1), want.float().reshape(2 * S1, -1)
        d = (got - want).abs()
        # share of identical rows; for attention of identical ELEMENTS (its softmax weights are rounded to
        # bf16 relative to a power of two here and to the maximum itself in the oracle: single elements
        # of nearly every row are a bf16 step off)
        ident = float((d == 0).float().mean()) if elements else float((d.max(-1).values == 0).float().mean())
        assert ident >= min_identical and d.mean().item() <= 2e-3 * want.abs().max().item(), (what, ident, d.mean().item())
        return ident

    x1 = ids[:, :S1]
    h0 = w["token_emb.weight"][x1].reshape(2 * S1, -1)
    q, k, v = (bl(n, h0, "norm1").view(2, S1, 16, 128) for n in ("attn.query", "attn.key", "attn.value"))
    qr, kr = R.apply_rope(q, k, w["freq_cos"][:S1], w["freq_sin"][:S1])
    att = R.attention_core(qr, kr, v, 0).reshape(2 * S1, -1)
    h1 = h0 + bl("attn.proj", att)
    act = F.silu(bl("ff.gate", h1, "norm2")) * bl("ff.up", h1, "norm2")
    h2 = h1 + bl("ff.down", act)
    c0 = model.build_kv_cache(2)[0]
    eps = model.eps
    qd = ops.bitlinear_qkv_rope_append(h0.to(cuda), L0["norm1"],
                                       [(L0[n][1], L0[n][0]) for n in ("attn.query", "attn.key", "attn.value")], eps,
                                       16, 16, 128, model.cos, model.sin, 0, c0.key, c0.value, seq_len=S1)
    idents = {"q": same_rows(qd, qr, "q"), "k": same_rows(c0.key[:, :S1], kr, "k"),
              "v": same_rows(c0.value[:, :S1], v, "v")}
    c0.key[:, :S1].copy_(kr.to(cuda))
    c0.value[:, :S1].copy_(v.to(cuda))
    ws = ops.attn_workspace(2, 16, 16, 128, 1, cuda)
    idents["attention"] = same_rows(ops.attn_auto(qr.reshape(2 * S1, -1).contiguous().to(cuda), c0.key, c0.value, 16, 16,
                                                  128, 0, 1, ws, S1), att, "attention", min_identical=0.6, elements=True)
    idents["proj"] = same_rows(ops.bitlinear(att.to(cuda), L0["attn.proj"][1], L0["attn.proj"][0], eps,
                                             residual=h0.to(cuda)), h1, "proj")
    idents["gate_up"] = same_rows(ops.bitlinear_gate_up(h1.to(cuda), L0["norm2"], (L0["ff.gate"][1], L0["ff.gate"][0]),
                                                        (L0["ff.up"][1], L0["ff.up"][0]), eps), act, "gate_up")
    idents["down"] = same_rows(ops.bitlinear(act.to(cuda), L0["ff.down"][1], L0["ff.down"][0], eps, residual=h1.to(cuda)),
                               h2, "down")
    del c0

    # (b2) the 24-layer model.  Its tolerance comes from the model's own sensitivity: the distance
    # between the oracle and a variant of it that is an equally valid implementation (softmax weights
    # rounded to bf16 before they meet the values, as fused attention kernels do, and the norm statistics
    # in fp64).  Through 24 absmax quantisers such last-bit differences grow to the percent level.
    rc, cache = ref.build_kv_cache(2), model.build_kv_cache(2)
    want_all = ref(ids, rc, 0)
    want = want_all[:, -1]
    orig_attn, orig_norm, orig_norm_bl = R.attention_core, R.rms_norm, BL.rms_norm

    def attn_bf16_weights(q, k, v, start_pos):
        B_, S_, H_, D_ = q.shape
        sc = q.float().permute(0, 2, 1, 3) @ k.float().permute(0, 2, 3, 1) / math.sqrt(D_)
        vis = torch.arange(k.shape[1])[None, :] <= (start_pos + torch.arange(S_))[:, None]
        p_ = torch.softmax(sc.masked_fill(~vis[None, None], float("-inf")), -1).to(BF).float()
        return (p_ @ v.float().permute(0, 2, 1, 3)).to(q.dtype).permute(0, 2, 1, 3).reshape(B_, S_, H_ * D_)

    def norm_fp64(x, weight, eps=1e-5):
        xf = x.double()
        return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)).to(x.dtype) * weight

    try:
        R.attention_core, R.rms_norm, BL.rms_norm = attn_bf16_weights, norm_fp64, norm_fp64
        other = R.RefLlama(rcfg, cpu_state)(ids, ref.build_kv_cache(2), 0)[:, -1]
    finally:
        R.attention_core, R.rms_norm, BL.rms_norm = orig_attn, orig_norm, orig_norm_bl
    fd = (other.float() - want.float()).abs()
    fscale = want.float().abs().max().item()
    floor_max, floor_mean = fd.max().item() / fscale, fd.mean().item() / fscale
    tol_max, tol_mean = max(8e-2, 2 * floor_max), max(1e-2, 2 * floor_mean)

    def close(got, want, what):
        got, want = got.float().cpu(), want.float()
        scale = want.abs().max().item()
        d = (got - want).abs()
        assert d.max().item() <= tol_max * scale and d.mean().item() <= tol_mean * scale, (what, d.max().item(), d.mean().item(), scale)
        return round(d.max().item() / scale, 5), round(d.mean().item() / scale, 5)

    got = model(ids.to(cuda), cache, 0, last_only=True)[:, 0]
    errs = {"prefill": close(got, want, "prefill")}
    nxt = want.float().argmax(-1, keepdim=True)
    for t in range(3):
        want = ref(nxt, rc, 64 + t)[:, -1]
        got = model(nxt.to(cuda), cache, 64 + t)[:, 0]
        errs[f"step{t}"] = close(got, want, f"step {t}")
        nxt = want.float().argmax(-1, keepdim=True)
    report = {"config": "BitNet ternary Llama d2048 x 24 layers, 2 sequences, prefill 64 + 3 steps",
              "layer0_rows_bit_identical_per_operator": idents, "model_vs_oracle_max_mean": errs,
              "oracle_vs_equally_valid_oracle_max_mean": (round(floor_max, 5), round(floor_mean, 5)),
              "tolerance_used_max_mean": (tol_max, tol_mean)}
    try:
        import json
        import os

        out_dir = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "gpurun_out")
        os.makedirs(out_dir, exist_ok=True)
        with open(os.path.join(out_dir, "parity_bitnet_c4.json"), "w") as f:
            json.dump(report, f, indent=1)
    except OSError:
        pass
    print(report)
    del ref, rc, cpu_state, cache, w

    # (c) batch 8 at the end of the context: rows equal the sequences decoded alone; graph == eager
    B, Lc = 8, cfg.max_sequence_length - 1
    cache = model.build_kv_cache(B)
    gd = torch.Generator(device=cuda).manual_seed(6)
    for c in cache:
        c.key[:, :Lc].copy_(torch.randn(B, Lc, model.kv_heads, model.head_dim, device=cuda, generator=gd).to(BF))
        c.value[:, :Lc].copy_(torch.randn(B, Lc, model.kv_heads, model.head_dim, device=cuda, generator=gd).to(BF))
        c.length, c.batch_size = Lc, B
    tok = torch.randint(0, V, (B, 1), generator=g).to(cuda)
    lb = model(tok, cache, Lc, last_only=True)[:, 0].clone()
    assert cache[0].length == Lc + 1
    for b in (0, 3, 7):
        c1 = model.build_kv_cache(1)
        for cs, cb in zip(c1, cache):
            cs.key[0, :Lc].copy_(cb.key[b, :Lc])
            cs.value[0, :Lc].copy_(cb.value[b, :Lc])
            cs.length, cs.batch_size = Lc, 1
        l1 = model(tok[b:b + 1], c1, Lc, last_only=True)[0, 0]
        scale = l1.float().abs().max().item()
        d = (lb[b].float() - l1.float()).abs()
        # the kernels serving 1 row and 8 rows reduce the norms in different orders: two equally valid
        # implementations, so the model's own sensitivity measured in (b2) is the yardstick here too
        assert d.max().item() <= tol_max * scale and d.mean().item() <= tol_mean * scale, (b, d.max().item(), d.mean().item())
        del c1

    def step():
        for c in cache:
            c.length, c.batch_size = Lc, B
        return model(tok, cache, Lc, last_only=True)

    eager = step()[:, 0].clone()
    assert torch.equal(eager, lb)
    gr = torch.cuda.CUDAGraph()
    with torch.cuda.graph(gr):
        out = step()
    for _ in range(3):
        out.zero_()
        gr.replay()
        torch.cuda.synchronize()
        assert torch.equal(out[:, 0], eager)

    # (d) the single-launch step on the same caches at the last cache row: the same codes and integer
    # sums as the kernel chain, so nearly every logit is the chain's bit for bit (attention sums its
    # context in another order, which flips single bf16 roundings that the quantisers then amplify)
    def persistent_logits(Bp, rows):
        cp = model.build_kv_cache(Bp)
        sess = model.session(Bp, 4, kv_cache=cp, persistent=True)
        sess.prefill(tok[rows, :1])  # one token: builds the workspace; the caches are then replaced
        for cs, cb in zip(cp, cache):
            cs.key[:, :Lc].copy_(cb.key[rows, :Lc])
            cs.value[:, :Lc].copy_(cb.value[rows, :Lc])
            cs.length, cs.batch_size = Lc, Bp
        sess.ids.copy_(tok[rows, 0])
        sess.step_state.copy_(torch.tensor([Lc, 1, 0, 0], dtype=torch.int32))
        sess.pos, sess.produced = Lc, 1
        sess.step()
        torch.cuda.synchronize()
        sess.check_error()
        assert torch.equal(sess.ids, ops.argmax(sess.logits))
        return sess.logits.clone()

    all_rows = torch.arange(B, device=cuda)
    for Bp, rows in ((B, all_rows), (1, all_rows[3:4])):
        got = persistent_logits(Bp, rows)
        want = lb[rows]
        scale = want.float().abs().max().item()
        dlt = (got.float() - want.float()).abs()
        same = (got == want).float().mean().item()
        report[f"persistent_vs_chain_batch{Bp}"] = {"identical_fraction": round(same, 4),
                                                    "max_over_scale": round(dlt.max().item() / scale, 5)}
        if Bp == B:
            assert same >= 0.5 and dlt.max().item() <= tol_max * scale and dlt.mean().item() <= tol_mean * scale, (Bp, same)
        else:  # one sequence against the row of the batch of eight: two reduction orders, as in (c)
            assert dlt.max().item() <= tol_max * scale and dlt.mean().item() <= tol_mean * scale, (Bp, same)
    print(report)
    del cache
    torch.cuda.empty_cache()
    # 128 greedy tokens after a 64-token prompt: the captured graph equals the eager launches
    prompt = torch.randint(0, V, (1, 64), generator=g).to(cuda)
    t_graph = model.generate_greedy(prompt, 128, persistent=True)
    t_eager = model.generate_greedy(prompt, 128, persistent=True, use_graph=False)
    assert torch.equal(t_graph, t_eager) and t_graph.shape == (1, 128)
    t_chain = model.generate_greedy(prompt, 128, persistent=False)
    first_diff = int((t_graph != t_chain).float().argmax()) if not torch.equal(t_graph, t_chain) else 128
    print({"persistent_vs_chain_first_differing_token": first_diff})
    assert first_diff >= 8


def test_moe_c5_model_full_size(cuda):
    """The MoE Llama at its full size (16 layers, d 1024, 16 heads x 64, 64 routed SwiGLU experts of
    hidden 512, top-8, one shared expert, softmax router):
    (a) a short prompt (2 x 12 tokens) and two cached steps against the CPU oracle of the whole model;
    (b) one decode step of 64 sequences at context 2047 -> 2048: every layer's routing indices equal
        the oracle's selection rule applied to the kernels' own router logits, 8 distinct experts per
        token with weights that sum to one; three rows equal the same sequences decoded alone."""
    import bench
    from ohara_amd.moe import MoeLlama
    from oracle import llama_ref as R
    from oracle import moe_ref as MR

    cfg, st = bench.moe_c5_state(cuda)
    model = MoeLlama(cfg, st, device=cuda)
    g = torch.Generator().manual_seed(7)
    V, k = cfg.vocab_size, cfg.moe_experts_per_tok

    def close(got, want, what, mx=3e-2, mn=4e-3):
        got, want = got.float().cpu(), want.float().cpu()
        scale = want.abs().max().item()
        d = (got - want).abs()
        assert d.max().item() <= mx * scale and d.mean().item() <= mn * scale, (what, d.max().item(), d.mean().item(), scale)
        return d.max().item() / scale, d.mean().item() / scale

    # (a) against the oracle
    fields = ("vocab_size", "hidden_size", "intermediate_size", "num_attention_heads", "num_key_value_heads",
              "num_hidden_layers", "max_sequence_length", "rope_theta", "moe_num_experts", "moe_experts_per_tok",
              "moe_layer_interval", "moe_gate_fn", "moe_quantile_balancing", "moe_grouped", "moe_num_shared_experts",
              "moe_normalize_weights")
    rcfg = R.RefConfig(**{f: getattr(cfg, f) for f in fields})
    cpu_state = {kk: v.cpu() for kk, v in st.items()}
    cos, sin = R.rope_table(rcfg.head_dim, rcfg.max_sequence_length * 2, rcfg.rope_theta)
    cpu_state["freq_cos"], cpu_state["freq_sin"] = cos.to(BF), sin.to(BF)
    ref = R.RefLlama(rcfg, cpu_state)
    del cpu_state
    del st
    ids = torch.randint(0, V, (2, 12), generator=g)
    rc, cache = ref.build_kv_cache(2), model.build_kv_cache(2)
    want = ref(ids, rc, 0)[:, -1]
    errs = [close(model(ids.to(cuda), cache, 0, last_only=True)[:, 0], want, "prefill")]
    nxt = want.float().argmax(-1, keepdim=True)
    for t in range(2):
        want = ref(nxt, rc, 12 + t)[:, -1]
        errs.append(close(model(nxt.to(cuda), cache, 12 + t)[:, 0], want, f"step {t}"))
        nxt = want.float().argmax(-1, keepdim=True)
    print("moe C5 vs oracle (max, mean error / logit scale):", errs)
    del ref, rc, cache

    # (b) 64 sequences at the end of the context
    B, Lc = 64, cfg.max_sequence_length - 1
    cache = model.build_kv_cache(B)
    gd = torch.Generator(device=cuda).manual_seed(8)
    for c in cache:
        c.key[:, :Lc].copy_(torch.randn(B, Lc, model.kv_heads, model.head_dim, device=cuda, generator=gd).to(BF))
        c.value[:, :Lc].copy_(torch.randn(B, Lc, model.kv_heads, model.head_dim, device=cuda, generator=gd).to(BF))
        c.length, c.batch_size = Lc, B
    tok = torch.randint(0, V, (B, 1), generator=g).to(cuda)
    trace = []
    for L in model.layers:
        L["moe"].trace = trace
    lb = model(tok, cache, Lc, last_only=True)[:, 0].clone()
    for L in model.layers:
        L["moe"].trace = None
    assert len(trace) == cfg.num_hidden_layers
    for li, (logits, idx, w) in enumerate(trace):
        lg = logits.float().cpu()
        assert lg.shape == (B, cfg.moe_num_experts)
        want_idx = MR.topk_lowest_index_first(lg + model.layers[li]["moe"].router_bias.float().cpu(), k + 1)[:, :k]
        assert torch.equal(idx.cpu().long(), want_idx), li
        assert all(len(set(r)) == k for r in idx.cpu().tolist())
        want_w = lg.gather(-1, want_idx).softmax(-1)
        assert (w.float().cpu() - want_w).abs().max().item() <= 2 ** -8
        assert (w.float().sum(-1) - 1).abs().max().item() <= 2e-2
    # Rows of the batch against the same sequences decoded alone (other kernels serve 1 row: bf16-level
    # differences).  Top-k routing is discontinuous, so a row whose router logits hold a near-tie at the
    # selection boundary may pick another expert when decoded alone; such a flip must BE a near-tie, and
    # only rows routed identically in every layer are held to the bf16 tolerance.
    outcomes = {}
    for b in (0, 13, 31, 47, 63):
        c1 = model.build_kv_cache(1)
        for cs, cb in zip(c1, cache):
            cs.key[0, :Lc].copy_(cb.key[b, :Lc])
            cs.value[0, :Lc].copy_(cb.value[b, :Lc])
            cs.length, cs.batch_size = Lc, 1
        t1 = []
        for L in model.layers:
            L["moe"].trace = t1
        l1 = model(tok[b:b + 1], c1, Lc, last_only=True)[0, 0]
        for L in model.layers:
            L["moe"].trace = None
        flipped = None
        for li, ((lg64, idx64, _), (lg1, idx1, _)) in enumerate(zip(trace, t1)):
            a, bb = set(idx64[b].tolist()), set(idx1[0].tolist())
            if a != bb:
                flipped = li
                row = lg1[0].float().cpu()
                lo, hi = min(float(row[e]) for e in a ^ bb), max(float(row[e]) for e in a ^ bb)
                assert hi - lo <= 2.0 ** -5 * max(abs(hi), abs(lo), 0.25), (b, li, lo, hi)
                break
        if flipped is None:
            outcomes[b] = ("routed identically", close(lb[b], l1, f"row {b} alone", mx=4e-2, mn=6e-3))
        else:
            outcomes[b] = (f"near-tie flip at layer {flipped}", close(lb[b], l1, f"row {b} alone", mx=0.3, mn=0.05))
        del c1
    print("moe C5 rows of the batch of 64 vs alone:", outcomes)
    assert sum(1 for v in outcomes.values() if v[0] == "routed identically") >= 2
