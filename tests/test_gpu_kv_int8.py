"""The int8 KV cache (ohara/modules/kv_cache.py:15-33, 94-118) on the GPU against the CPU oracle.

Integer results (codes) and the stored statistics must match the oracle bit for bit when both
quantise the same bf16 rows; dequantised reads likewise.  Attention over the int8 cache is
compared with an fp64 brute force over the oracle's dequantised cache, and whole-model logits
with the oracle run on int8 caches, at the tolerances of the bf16 cache tests.
"""

import dataclasses
import math

import pytest
import torch

from oracle import llama_ref as R

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


def _rows(B, S, Hkv, D, seed):
    g = torch.Generator().manual_seed(seed)
    k = (torch.randn(B, S, Hkv, D, generator=g) * 1.7).to(BF)
    v = (torch.randn(B, S, Hkv, D, generator=g) * 0.3 + 0.5).to(BF)
    k[0, 0, 0] = 0.625        # constant row: scale floors at 1e-8
    v[0, 0, 0] = 0.0
    if S > 1:
        k[-1, -1, -1] *= 300  # wide range
        v[-1, -1, -1, 1:] = v[-1, -1, -1, 0]  # all but... one distinct element
        v[-1, -1, -1, 0] += 1
    return k, v


@pytest.mark.parametrize("B,S,Hkv,D,pos", [(2, 5, 2, 128, 3), (1, 1, 6, 128, 0), (3, 40, 4, 64, 7), (2, 3, 2, 16, 1),
                                           (1, 2, 1, 8, 0), (2, 2, 3, 256, 4)])
def test_quantise_append_and_dequantise_bit_exact(cuda, B, S, Hkv, D, pos):
    from ohara_amd import ops
    from ohara_amd.llama import KVCache

    Tmax = pos + S + 3
    k, v = _rows(B, S, Hkv, D, seed=B * 100 + S)
    cache = KVCache((B + 1, Tmax, Hkv, D), Tmax, device=cuda, dtype=BF, int8=True)
    ops.kv_quant_append(k.to(cuda), v.to(cuda), cache, pos)
    for src, codes, scale, mn in ((k, cache.key, cache.key_scale, cache.key_min),
                                  (v, cache.value, cache.value_scale, cache.value_min)):
        rq, rs, rm = R.quantize_int8(src)
        assert torch.equal(codes[:B, pos:pos + S].cpu(), rq)
        assert torch.equal(scale[:B, pos:pos + S].cpu(), rs.float())
        assert torch.equal(mn[:B, pos:pos + S].cpu(), rm.float())
        # nothing outside the window was written
        codes = codes.clone()
        codes[:B, pos:pos + S] = 0
        assert not codes.any()
    scale = cache.key_scale.clone()
    scale[:B, pos:pos + S] = 0
    assert not scale.any()
    # reads: fp32 (code + 128) * scale + min, one rounding to bf16 (kv_cache.py:31-33, :118)
    for which, src in (("key", k), ("value", v)):
        rq, rs, rm = R.quantize_int8(src)
        want = R.dequantize_int8(rq, rs.float(), rm.float()).to(BF)
        full = ops.kv_dequant(cache, which, B, pos + S)
        assert full.shape == (B, pos + S, Hkv, D)
        assert torch.equal(full[:, pos:].cpu(), want)
        assert not full[:, :pos].any()  # code 0 rows with zero statistics read as (0 + 128) * 0 + 0
    # position read on the device
    cache2 = KVCache((B + 1, Tmax, Hkv, D), Tmax, device=cuda, dtype=BF, int8=True)
    if S == 1:
        pos_dev = torch.tensor([pos], dtype=torch.int32, device=cuda)
        ops.kv_quant_append(k.to(cuda), v.to(cuda), cache2, 0, pos_dev=pos_dev)
        assert torch.equal(cache2.key, cache.key) and torch.equal(cache2.value_scale, cache.value_scale)


def test_cache_forward_matches_the_oracle_cache(cuda):
    """KVCache(int8=True).forward: the reference's semantics (tests/test_modules.py:82-91) and
    messages, results equal to the restated cache fed the same bf16 rows."""
    from ohara_amd.llama import KVCache

    B, Hkv, D, Tmax = 2, 2, 64, 12
    cache = KVCache((B, Tmax, Hkv, D), Tmax, device=cuda, dtype=BF, int8=True)
    ref = R.KVCacheRef((B, Tmax, Hkv, D), Tmax, dtype=BF, int8=True)
    start = 0
    for S, seed in ((4, 1), (1, 2), (1, 3), (3, 4)):
        k, v = _rows(B, S, Hkv, D, seed)
        gk, gv = cache.forward(k.to(cuda), v.to(cuda), start)
        rk, rv = ref.forward(k, v, start)
        assert gk.dtype == BF and gk.shape == rk.shape
        assert torch.equal(gk.cpu(), rk) and torch.equal(gv.cpu(), rv)
        torch.testing.assert_close(gk[:, start:].cpu().float(), k.float(), rtol=0.05, atol=0.05 * float(k.abs().max()))
        start += S
    assert cache.length == ref.length == 9 and cache.batch_size == 2
    assert torch.equal(cache.key.cpu(), ref.key) and torch.equal(cache.value_min.cpu(), ref.value_min)
    with pytest.raises(ValueError, match="sequential"):
        cache.forward(k.to(cuda), v.to(cuda), 4)
    with pytest.raises(ValueError, match="exceeds max_sequence_length"):
        cache.forward(torch.zeros(B, 4, Hkv, D, dtype=BF, device=cuda), torch.zeros(B, 4, Hkv, D, dtype=BF, device=cuda), 9)
    with pytest.raises(ValueError, match="bfloat16"):
        KVCache((1, 4, 1, 8), 4, device=cuda, dtype=BF, int8=True).forward(
            torch.zeros(1, 1, 1, 8, device=cuda), torch.zeros(1, 1, 1, 8, device=cuda), 0)


def _attn_ref64(q, k, v, pos):
    """q (B,S,H,D); k, v (B,T,Hkv,D) dequantised bf16; query s sees positions <= pos + s."""
    B, S, H, D = q.shape
    G = H // k.shape[2]
    out = torch.empty(B, S, H, D, dtype=torch.float64)
    for s in range(S):
        L = pos + s + 1
        for h in range(H):
            sc = torch.einsum("bd,btd->bt", q[:, s, h].double(), k[:, :L, h // G].double()) / math.sqrt(D)
            out[:, s, h] = torch.einsum("bt,btd->bd", torch.softmax(sc, -1), v[:, :L, h // G].double())
    return out


@pytest.mark.parametrize("B,S,H,Hkv,D,L,ns", [(1, 1, 6, 6, 128, 1153, 16), (2, 1, 32, 8, 128, 700, 8),
                                              (3, 1, 16, 16, 64, 64, 4), (2, 1, 4, 2, 16, 37, 3), (4, 1, 8, 4, 128, 1, 4),
                                              (2, 5, 8, 2, 128, 200, 1), (1, 3, 4, 4, 8, 9, 1)])
def test_attention_over_the_int8_cache(cuda, B, S, H, Hkv, D, L, ns):
    """L = positions the last query sees."""
    from ohara_amd import ops
    from ohara_amd.llama import KVCache

    g = torch.Generator().manual_seed(L + S)
    Tmax = L + 6
    k = torch.randn(B, L, Hkv, D, generator=g).to(BF)
    v = torch.randn(B, L, Hkv, D, generator=g).to(BF)
    q = torch.randn(B, S, H, D, generator=g).to(BF)
    cache = KVCache((B, Tmax, Hkv, D), Tmax, device=cuda, dtype=BF, int8=True)
    gk, gv = cache.forward(k.to(cuda), v.to(cuda), 0)
    ref = R.KVCacheRef((B, Tmax, Hkv, D), Tmax, dtype=BF, int8=True)
    rk, rv = ref.forward(k, v, 0)
    assert torch.equal(gk.cpu(), rk) and torch.equal(gv.cpu(), rv)
    pos = L - S
    want = _attn_ref64(q, rk, rv, pos)
    ws = ops.attn_workspace(B, H, Hkv, D, ns, cuda)
    qd = q.to(cuda).view(B * S, H * D)
    for _ in range(2):
        out = ops.attn_cached_int8(qd, cache, H, Hkv, D, pos, ns, ws, seq_len=S)
        err = (out.cpu().double().view(B, S, H, D) - want).abs().max().item()
        assert err <= 2e-2 * max(1.0, want.abs().max().item()), err
    # the same numbers as bf16 attention over the dequantised tensors, up to the merge order
    padk = torch.zeros(B, Tmax, Hkv, D, dtype=BF, device=cuda)
    padv = torch.zeros_like(padk)
    padk[:, :L], padv[:, :L] = gk, gv
    same = ops.attn_cached(qd, padk, padv, H, Hkv, D, pos, ns, ws, seq_len=S)
    assert (out.float() - same.float()).abs().max().item() <= 2 ** -7 * max(1.0, want.abs().max().item())
    if S == 1:
        pos_dev = torch.tensor([pos], dtype=torch.int32, device=cuda)
        out2 = ops.attn_cached_int8(qd, cache, H, Hkv, D, 0, ns, ws, pos_dev=pos_dev)
        assert torch.equal(out2, out)


def test_projection_to_row_buffers_equals_the_cache_append(cuda):
    from ohara_amd import ops

    B, S, H, Hkv, D, K, Tmax, pos = 2, 3, 4, 2, 64, 128, 16, 5
    g = torch.Generator().manual_seed(9)
    x = torch.randn(B * S, K, generator=g).to(BF).to(cuda)
    wq, wk, wv = ((torch.randn(n * D, K, generator=g) * 0.05).to(BF).to(cuda) for n in (H, Hkv, Hkv))
    nw = (1 + 0.2 * torch.randn(K, generator=g)).to(BF).to(cuda)
    cos, sin = (t.to(BF).to(cuda) for t in R.rope_table(D, 2 * Tmax, 10000.0))
    wp = ops.pack_qkv(wq, wk, wv)
    kc = torch.zeros(B, Tmax, Hkv, D, dtype=BF, device=cuda)
    vc = torch.zeros_like(kc)
    qa = ops.qkv_rope_append(x, wp, nw, 1e-5, H, Hkv, D, cos, sin, pos, kc, vc, seq_len=S)
    q, k, v = ops.qkv_rope(x, wp, nw, 1e-5, H, Hkv, D, cos, sin, pos, Tmax, seq_len=S)
    assert torch.equal(q, qa)
    assert torch.equal(k.view(B, S, Hkv, D), kc[:, pos:pos + S]) and torch.equal(v.view(B, S, Hkv, D), vc[:, pos:pos + S])


def _cfg_pair(**kw):
    from ohara_amd.llama import Config

    fields = {f.name for f in dataclasses.fields(R.RefConfig)}
    kw = {k: v for k, v in kw.items() if k in fields}
    return R.RefConfig(**kw), Config(**kw)


def _close(got, ref, max_rel, mean_rel):
    got, ref = got.float().cpu(), ref.float()
    scale = ref.abs().max().item()
    d = (got - ref).abs()
    assert d.max().item() <= max_rel * scale, (d.max().item(), scale)
    assert d.mean().item() <= mean_rel * scale, (d.mean().item(), scale)


@pytest.mark.parametrize("heads,kv_heads,hidden,P", [(4, 2, 256, 5), (4, 2, 256, 40), (2, 2, 256, 21)])
def test_model_with_int8_caches(cuda, heads, kv_heads, hidden, P):
    """Prefill (short prompts attend straight over the codes, long ones over a dequantised copy)
    and decode steps against the oracle on int8 caches; then the device-resident greedy loop
    against step-by-step forward calls."""
    from ohara_amd.llama import Llama

    rcfg, cfg = _cfg_pair(vocab_size=512, hidden_size=hidden, intermediate_size=512, num_attention_heads=heads,
                          num_key_value_heads=kv_heads, num_hidden_layers=3, max_sequence_length=128,
                          rope_theta=10000.0)
    w = R.init_weights(rcfg, seed=4, dtype=BF, std=0.06, norm_jitter=0.1)
    ref, model = R.RefLlama(rcfg, w), Llama(cfg, w, device=cuda)
    B = 2
    prompt = torch.randint(0, 512, (B, P), generator=torch.Generator().manual_seed(P))
    rc, cache = ref.build_kv_cache(B, int8=True), model.build_kv_cache(B, int8=True)
    assert cache[0].key.dtype == torch.int8
    want = ref(prompt, rc, 0)
    got = model(prompt.to(cuda), cache, 0)
    _close(got, want, 4e-2, 4e-3)
    # the caches hold the oracle's rows up to the bf16 noise of the projections feeding them (a flipped
    # last bit of a row's minimum or maximum moves every code of the row, so codes are compared
    # through the values they stand for)
    from ohara_amd import ops
    for l in (0, 2):
        gk = ops.kv_dequant(cache[l], "key", B, P).cpu().float()
        rk = R.dequantize_int8(rc[l].key[:B, :P], rc[l].key_scale[:B, :P], rc[l].key_min[:B, :P])
        assert (gk - rk).abs().max().item() <= 3e-2 * rk.abs().max().item()
        assert (gk - rk).abs().mean().item() <= 4e-3 * rk.abs().max().item()
        torch.testing.assert_close(cache[l].value_scale[:, :P].cpu(), rc[l].value_scale[:, :P], rtol=0.05, atol=1e-6)
    assert cache[0].length == P
    nxt = want[:, -1].float().argmax(-1, keepdim=True)
    for step in range(3):
        want = ref(nxt, rc, P + step)
        got = model(nxt.to(cuda), cache, P + step)
        _close(got, want, 4e-2, 4e-3)
        nxt = want[:, -1].float().argmax(-1, keepdim=True)
    # int8 and bf16 caches give different (close) logits: the mode is really in effect
    exact = model(prompt.to(cuda), model.build_kv_cache(B), 0)
    quant = model(prompt.to(cuda), model.build_kv_cache(B, int8=True), 0)
    assert 0 < (exact.float() - quant.float()).abs().max().item() < 0.1 * exact.float().abs().max().item()

    # device-resident loop (graph replay and eager) == forward calls, token for token
    steps = 12
    c2 = model.build_kv_cache(B, int8=True)
    lg = model(prompt.to(cuda), c2, 0, last_only=True)
    toks = [lg[:, -1].float().argmax(-1)]
    for t in range(steps - 1):
        lg = model(toks[-1].view(B, 1), c2, P + t)
        toks.append(lg[:, -1].float().argmax(-1))
    stepwise = torch.stack(toks, 1).cpu()
    for use_graph in (True, False):
        got = model.generate_greedy(prompt.to(cuda), steps, use_graph=use_graph,
                                    kv_cache=model.build_kv_cache(B, int8=True)).cpu()
        assert torch.equal(got, stepwise), use_graph


def test_int8_cache_mode_errors(cuda):
    from ohara_amd.llama import Llama

    rcfg, cfg = _cfg_pair(vocab_size=64, hidden_size=64, intermediate_size=64, num_attention_heads=2,
                          num_hidden_layers=2, max_sequence_length=16)
    w = R.init_weights(rcfg, seed=1, dtype=BF)
    model = Llama(cfg, w, device=cuda)
    mixed = [model.build_kv_cache(1, int8=True)[0], model.build_kv_cache(1)[1]]
    with pytest.raises(ValueError, match="same KV cache mode"):
        model(torch.zeros(1, 2, dtype=torch.int64), mixed, 0)
    sess = model.session(1, 4, kv_cache=model.build_kv_cache(1, int8=True), persistent=None)
    assert sess.persistent is False


@pytest.mark.parametrize("B", [9, 33, 70])
def test_int8_cache_decode_at_larger_batches(cuda, B):
    """int8 caches with more than 16 and more than 64 sequences: prefill and cached steps against the
    oracle's int8 caches."""
    from ohara_amd.llama import Llama

    rcfg, cfg = _cfg_pair(vocab_size=512, hidden_size=256, intermediate_size=512, num_attention_heads=4,
                          num_key_value_heads=2, num_hidden_layers=2, max_sequence_length=64, rope_theta=10000.0)
    w = R.init_weights(rcfg, seed=8, dtype=BF, std=0.06, norm_jitter=0.1)
    ref, model = R.RefLlama(rcfg, w), Llama(cfg, w, device=cuda)
    ids = torch.randint(0, 512, (B, 8), generator=torch.Generator().manual_seed(B))
    rc, cache = ref.build_kv_cache(B, int8=True), model.build_kv_cache(B, int8=True)
    _close(model(ids[:, :5].to(cuda), cache, 0), ref(ids[:, :5], rc, 0), 4e-2, 4e-3)
    for t in (5, 6, 7):
        _close(model(ids[:, t:t + 1].to(cuda), cache, t), ref(ids[:, t:t + 1], rc, t), 4e-2, 4e-3)


@pytest.mark.parametrize("P", [5, 24])
def test_moe_model_with_int8_caches(cuda, P):
    """The MoE model on int8 caches (short prompts attend straight over the codes, prompts of 16 and
    more tokens over a dequantised copy of the live prefix), prefill and cached steps against the
    oracle on its own int8 caches.  A router near-tie that bf16 noise decides the other way moves a
    row's logits, so rows are judged one by one and a few may differ."""
    from ohara_amd.llama import Llama
    from ohara_amd.moe import MoeLlama

    kw = dict(vocab_size=256, hidden_size=128, intermediate_size=64, num_attention_heads=2, num_key_value_heads=0,
              num_hidden_layers=3, max_sequence_length=48, dropout=0.0, moe_num_experts=8, moe_experts_per_tok=2,
              moe_layer_interval=2, moe_grouped=True, moe_num_shared_experts=1, moe_gate_fn="softmax")
    rcfg, cfg = _cfg_pair(**kw)
    w = R.init_weights(rcfg, seed=21, dtype=BF, std=0.06, norm_jitter=0.1)
    ref, model = R.RefLlama(rcfg, w), Llama(cfg, w, device=cuda)
    assert isinstance(model, MoeLlama)
    B = 3
    ids = torch.randint(0, 256, (B, P + 3), generator=torch.Generator().manual_seed(P))
    rc, cache = ref.build_kv_cache(B, int8=True), model.build_kv_cache(B, int8=True)
    assert cache[0].key.dtype == torch.int8

    def close(got, want):
        got, want = got.float().cpu().reshape(-1, 256), want.float().reshape(-1, 256)
        scale = want.abs().max().item()
        good = (got - want).abs().amax(-1) <= 4e-2 * scale
        assert good.float().mean().item() >= 0.9, good.float().mean().item()
        assert (got - want).abs()[good].mean().item() <= 6e-3 * scale

    close(model(ids[:, :P].to(cuda), cache, 0), ref(ids[:, :P], rc, 0))
    for t in range(P, P + 3):
        close(model(ids[:, t:t + 1].to(cuda), cache, t), ref(ids[:, t:t + 1], rc, t))
    # the codes written are the oracle's wherever the rows going in agree; at least the cache is in use
    assert cache[0].length == P + 3
    mixed = [model.build_kv_cache(1, int8=True)[0]] + model.build_kv_cache(1)[1:]
    with pytest.raises(ValueError, match="same KV cache mode"):
        model(ids[:1, :2].to(cuda), mixed, 0)


@pytest.mark.parametrize("heads,kv_heads,hidden,B,P", [(2, 2, 256, 1, 21), (4, 2, 256, 3, 40), (8, 2, 512, 8, 70),
                                                       (4, 1, 512, 2, 130), (2, 1, 256, 5, 63), (4, 4, 256, 2, 33),
                                                       (6, 6, 768, 1, 1200)])
def test_persistent_kernel_on_int8_caches(cuda, heads, kv_heads, hidden, B, P):
    """The single-launch decode step over int8 caches (its polled builds, up to eight sequences): the attention
    phase reads codes and statistics and quantises the appended row itself.  Teacher-forced logits against the
    oracle on int8 caches, for the single launch and for the kernel chain; the rows the single launch appended
    against the oracle's through the values they stand for; and its quantiser bit for bit: the first layer's
    appended rows depend on the fed tokens only, so a bf16-cache session of the same kernel holds exactly the
    rows that were quantised, and the oracle's codes and statistics of those rows must be the cache's."""
    from ohara_amd import ops
    from ohara_amd.llama import Llama

    T = 2048 if P > 1000 else 256
    rcfg, cfg = _cfg_pair(vocab_size=512, hidden_size=hidden, intermediate_size=512, num_attention_heads=heads,
                          num_key_value_heads=kv_heads, num_hidden_layers=2, max_sequence_length=T, rope_theta=10000.0)
    w = R.init_weights(rcfg, seed=heads + B, dtype=BF, std=0.06, norm_jitter=0.1)
    ref, model = R.RefLlama(rcfg, w), Llama(cfg, w, device=cuda)
    prompt = torch.randint(0, 512, (B, P), generator=torch.Generator().manual_seed(P))
    steps = 5
    rc = ref.build_kv_cache(B, int8=True)
    want = [ref(prompt, rc, 0)[:, -1]]
    fed = []
    for s in range(steps):
        fed.append(want[-1].float().argmax(-1))
        want.append(ref(fed[-1].view(B, 1), rc, P + s)[:, -1])
    caches, logits = {}, {}
    for persistent in (True, False):
        cache = model.build_kv_cache(B, int8=True)
        sess = model.session(B, steps + 1, kv_cache=cache, persistent=persistent)
        assert sess.persistent is persistent
        sess.prefill(prompt.to(cuda))
        _close(sess.logits, want[0], 4e-2, 6e-3)
        logits[persistent] = []
        for s in range(steps):
            sess.feed(fed[s].to(cuda))
            sess.step()
            # (the quantisation noise of these small random models: the mean is 3e-3 to 5e-3 of the scale for both paths)
            _close(sess.logits, want[s + 1], 4e-2, 6e-3)
            logits[persistent].append(sess.logits.float().cpu())
        sess.check_error()
        caches[persistent] = cache
    cache = caches[True]
    # the two device paths against each other: the same rows quantised the same way, up to the bf16 noise of the
    # projections that feed the second layer (a code off by one here and there)
    for s in range(steps):
        _close(logits[True][s], logits[False][s], 1e-2, 2.5e-3)  # (a bf16 ulp of a logit is 2e-3 to 4e-3 of the scale)
    for l in range(2):
        for name in ("key", "value"):
            a, b = getattr(cache[l], name)[:B, P:P + steps].int(), getattr(caches[False][l], name)[:B, P:P + steps].int()
            assert (a - b).abs().max().item() <= (0 if l == 0 else 1), (l, name)
            assert (a != b).float().mean().item() <= 0.03, (l, name)
    for l in range(2):
        for which in ("key", "value"):
            got = ops.kv_dequant(cache[l], which, B, P + steps).cpu().float()[:, P:]
            rq, rs, rm = ((rc[l].key, rc[l].key_scale, rc[l].key_min) if which == "key"
                          else (rc[l].value, rc[l].value_scale, rc[l].value_min))
            exp = R.dequantize_int8(rq[:B, P:P + steps], rs[:B, P:P + steps], rm[:B, P:P + steps])
            assert (got - exp).abs().max().item() <= 3e-2 * exp.abs().max().item(), (l, which)
            assert (got - exp).abs().mean().item() <= 4e-3 * exp.abs().max().item(), (l, which)
    # nothing behind the last appended position was touched
    assert not cache[0].key[:, P + steps:].any() and not cache[1].stats[:, :, P + steps:].any()
    # the in-kernel quantiser, bit for bit
    plain = model.build_kv_cache(B)
    sess = model.session(B, steps + 1, kv_cache=plain, persistent=True)
    sess.prefill(prompt.to(cuda))
    for s in range(steps):
        sess.feed(fed[s].to(cuda))
        sess.step()
    sess.check_error()
    for rows, codes, scale, mn in ((plain[0].key, cache[0].key, cache[0].key_scale, cache[0].key_min),
                                   (plain[0].value, cache[0].value, cache[0].value_scale, cache[0].value_min)):
        rq, rs, rm = R.quantize_int8(rows[:B, P:P + steps].cpu())
        assert torch.equal(codes[:B, P:P + steps].cpu(), rq)
        assert torch.equal(scale[:B, P:P + steps].cpu(), rs.float())
        assert torch.equal(mn[:B, P:P + steps].cpu(), rm.float())


@pytest.mark.parametrize("P", [6, 20])
def test_bitnet_model_with_int8_caches(cuda, P):
    """The ternary (BitNet) Llama on int8 caches through the kernel chain: prefill (short prompts attend over
    the codes, prompts of 16 and more tokens over a dequantised copy of the live prefix) and cached steps
    against the oracle on its own int8 caches, at the ternary model's tolerance; layer 0's codes and
    statistics (no attention in front of them) against the oracle's quantiser applied to the bf16 session's
    rows; the decode session falls back to the kernel chain for such caches."""
    from oracle import bitlinear_ref as BL
    from ohara_amd.bitnet import BitLlama
    from ohara_amd.llama import Config

    kw = dict(vocab_size=320, hidden_size=256, intermediate_size=512, num_attention_heads=2,
              num_key_value_heads=0, num_hidden_layers=3, max_sequence_length=64, rope_theta=10000.0)
    rcfg = R.RefConfig(**kw)
    w = BL.init_ternary_weights(rcfg, seed=2, dtype=BF, gamma=0.05)
    ref, model = R.RefLlama(rcfg, w), BitLlama(Config(**kw), w, device=cuda)
    B = 2
    ids = torch.randint(0, 320, (B, P + 3), generator=torch.Generator().manual_seed(P))
    rc, cache = ref.build_kv_cache(B, int8=True), model.build_kv_cache(B, int8=True)
    assert cache[0].key.dtype == torch.int8

    def close(got, want):
        d = (got.float().cpu() - want.float()).abs()
        scale = want.float().abs().max().item()
        assert d.max().item() <= 1e-1 * scale and d.mean().item() <= 1.5e-2 * scale, (d.max().item(), d.mean().item(), scale)

    close(model(ids[:, :P].to(cuda), cache, 0), ref(ids[:, :P], rc, 0))
    for t in range(P, P + 3):
        close(model(ids[:, t:t + 1].to(cuda), cache, t), ref(ids[:, t:t + 1], rc, t))
    assert cache[0].length == P + 3
    # layer 0: the rows that went in are those of a bf16-cache run of the same model (bit for bit: nothing in front of
    # them depends on the cache), so its codes are the oracle quantiser's codes of those rows
    plain = model.build_kv_cache(B)
    model(ids[:, :P].to(cuda), plain, 0)
    kq, ks, km = R.quantize_int8(plain[0].key[:, :P].cpu())
    assert torch.equal(cache[0].key[:, :P].cpu(), kq)
    vq, _, _ = R.quantize_int8(plain[0].value[:, :P].cpu())
    assert torch.equal(cache[0].value[:, :P].cpu(), vq)
    # sessions: int8 caches run the kernel chain
    sess = model.session(B, 4, kv_cache=model.build_kv_cache(B, int8=True))
    assert sess.persistent is False
    sess.prefill(ids[:, :P].to(cuda))
    sess.run(3)
    assert sess.tokens().shape == (B, 4)
    with pytest.raises(ValueError, match="int8 caches run the kernel chain"):
        model.session(B, 4, kv_cache=model.build_kv_cache(B, int8=True), persistent=True)
    mixed = [model.build_kv_cache(1, int8=True)[0]] + model.build_kv_cache(1)[1:]
    with pytest.raises(ValueError, match="same KV cache mode"):
        model(ids[:1, :2].to(cuda), mixed, 0)
