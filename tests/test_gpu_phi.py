"""Phi's cached decode path on the GPU (ohara/models/phi.py) against the CPU oracle
(oracle/phi_ref.py) on the same seeded inputs, through the C ABI."""

import dataclasses

import pytest
import torch
import torch.nn.functional as F

from oracle import phi_ref as P

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


def _ulp_close(got, want32, ulps=1.0, floor=2.0 ** -9):
    """|got - want| within `ulps` bf16 ulps of the fp32 value (an ulp is at most 2^-7 of the value)."""
    got, want32 = got.float().cpu(), want32.float().cpu()
    bound = ulps * 2.0 ** -7 * want32.abs().clamp_min(floor) + 1e-6
    bad = (got - want32).abs() > bound
    assert not bad.any(), ((got - want32).abs().max().item(), int(bad.sum()))


def test_layernorm_matches_the_library_routine(cuda):
    from ohara_amd import ops

    g = torch.Generator().manual_seed(0)
    for rows, d in ((1, 64), (5, 2560), (33, 320), (3, 4104)):
        x = (torch.randn(rows, d, generator=g) * 2 + 0.5).to(BF)
        w = (1 + 0.1 * torch.randn(d, generator=g)).to(BF)
        b = (0.1 * torch.randn(d, generator=g)).to(BF)
        got = ops.layernorm(x.to(cuda), w.to(cuda), b.to(cuda), 1e-5)
        want32 = F.layer_norm(x.float(), (d,), w.float(), b.float(), 1e-5)
        _ulp_close(got, want32, ulps=0.51)  # one rounding of the fp32 value
        ref = P.layer_norm(x, w, b, 1e-5)
        assert (got.cpu() != ref).float().mean() < 2e-3  # round-to-nearest ties of fp32 noise only


def test_linear_bias_epilogues(cuda):
    from ohara_amd import ops

    g = torch.Generator().manual_seed(1)
    for rows, n, k in ((1, 64, 64), (7, 320, 1280), (64, 1280, 320), (70, 96, 64), (3, 64, 2560), (20, 160, 10240),
                       (128, 96, 320), (130, 96, 64), (200, 320, 1280)):
        x = torch.randn(rows, k, generator=g).to(BF)
        w = (torch.randn(n, k, generator=g) / k ** 0.5).to(BF)
        b = (0.2 * torch.randn(n, generator=g)).to(BF)
        a1 = torch.randn(rows, n, generator=g).to(BF)
        a2 = torch.randn(rows, n, generator=g).to(BF)
        pw = ops.pack_linear(w.to(cuda))
        y = ops.linear_bias(x.to(cuda), pw, b.to(cuda))
        y32 = x.float() @ w.float().t() + b.float()
        _ulp_close(y, y32, ulps=0.6)
        # the fused epilogues continue from the same rounded y: compare with the oracle's op-by-op
        # bf16 arithmetic applied to the kernel's own y
        gel = ops.linear_bias(x.to(cuda), pw, b.to(cuda), "gelu")
        want = P.new_gelu(y.cpu())
        diff = (gel.cpu().float() - want.float()).abs()
        assert (diff > 0).float().mean() < 5e-3, (diff > 0).float().mean()  # tanhf vs the host's tanh, last fp32 ulp
        # where they differ, tanh's bf16 rounding moved by one ulp (2^-8 near +-1), scaled by 0.5 * y
        assert (diff <= 2.0 ** -8 * y.cpu().float().abs() + 2.0 ** -7 * want.float().abs() + 1e-6).all()
        out = ops.linear_bias(x.to(cuda), pw, b.to(cuda), "add2", add1=a1.to(cuda), add2=a2.to(cuda))
        assert torch.equal(out.cpu(), (a1 + y.cpu()) + a2)
    # strided input rows (a column slice of a wider buffer)
    wide = torch.randn(5, 3 * 64, generator=g).to(BF).to(cuda)
    w = (torch.randn(32, 64, generator=g) / 8).to(BF).to(cuda)
    b = torch.zeros(32, dtype=BF, device=cuda)
    got = ops.linear_bias(wide[:, 64:128], ops.pack_linear(w), b)
    _ulp_close(got, wide[:, 64:128].float() @ w.float().t(), ulps=0.6)
    with pytest.raises(ValueError):
        ops.linear_bias(wide[:, :64], ops.pack_linear(w), torch.zeros(16, dtype=BF, device=cuda))


def test_kv_append_and_attention_against_the_oracle(cuda):
    from ohara_amd import ops
    from ohara_amd.phi import rope_cos_sin

    g = torch.Generator().manual_seed(2)
    for B, S, L0, H, D, rot, Tmax in ((2, 1, 9, 4, 16, 6, 32), (1, 5, 0, 2, 80, 32, 16), (3, 2, 30, 2, 128, 128, 40),
                                      (1, 1, 0, 1, 8, 2, 4), (2, 1, 299, 2, 64, 24, 300),
                                      # many (sequence, head) pairs: workgroup counts that are multiples of 8 are
                                      # handed to the XCDs in a re-read order
                                      (4, 1, 300, 32, 80, 32, 320), (16, 1, 37, 8, 64, 64, 48), (2, 1, 0, 64, 16, 16, 4),
                                      (5, 1, 130, 40, 24, 16, 131),
                                      # 16 tokens and more: query tiles of 64 against key tiles of 32
                                      (2, 40, 0, 2, 80, 32, 64), (1, 100, 29, 2, 128, 128, 160), (3, 16, 5, 4, 16, 6, 32),
                                      (1, 65, 0, 1, 64, 24, 80), (2, 33, 0, 2, 32, 16, 40), (1, 200, 0, 3, 80, 32, 200),
                                      (1, 20, 3, 2, 48, 16, 32)):  # width 48: the one-query-per-workgroup kernel
        hd = H * D
        kc = torch.zeros(B, Tmax, H, D, dtype=BF)
        vc = torch.zeros(B, Tmax, H, D, dtype=BF)
        kc[:, :L0] = torch.randn(B, L0, H, D, generator=g).to(BF)
        vc[:, :L0] = torch.randn(B, L0, H, D, generator=g).to(BF)
        qkv = torch.randn(B * S, 3 * hd, generator=g).to(BF)
        kcd, vcd, qkvd = kc.to(cuda), vc.to(cuda), qkv.to(cuda)
        ops.kv_append(qkvd[:, hd:2 * hd], qkvd[:, 2 * hd:], kcd, vcd, B, S, H, D, L0)
        kc[:, L0:L0 + S] = qkv[:, hd:2 * hd].view(B, S, H, D)
        vc[:, L0:L0 + S] = qkv[:, 2 * hd:].view(B, S, H, D)
        assert torch.equal(kcd.cpu(), kc) and torch.equal(vcd.cpu(), vc)
        cos, sin = rope_cos_sin(Tmax, rot)
        ref_cos, ref_sin = P.rope_cos_sin(Tmax, rot)
        assert torch.equal(cos, ref_cos) and torch.equal(sin, ref_sin)
        got = ops.phi_attn(qkvd[:, :hd], kcd, vcd, cos.to(cuda), sin.to(cuda), rot, B, S, H, D, L0)
        want = P.attention(qkv[:, :hd].view(B, S, H, D), kc[:, :L0 + S], vc[:, :L0 + S], L0, rot, torch.float32)
        _ulp_close(got.view(B, S, H, D), want, ulps=0.6, floor=2.0 ** -6)
        if S == 1:  # position read on the device; context spread over several workgroups
            pd = torch.tensor([L0], dtype=torch.int32, device=cuda)
            got2 = ops.phi_attn(qkvd[:, :hd], kcd, vcd, cos.to(cuda), sin.to(cuda), rot, B, S, H, D, 0, pos_dev=pd)
            assert torch.equal(got2, got)
            for ns in (2, 5, 16, 64):
                ws = ops.phi_attn_workspace(B, H, D, ns, cuda)
                got3 = ops.phi_attn(qkvd[:, :hd], kcd, vcd, cos.to(cuda), sin.to(cuda), rot, B, S, H, D, L0, n_split=ns,
                                    workspace=ws)
                _ulp_close(got3.view(B, S, H, D), want, ulps=0.6, floor=2.0 ** -6)


def _pair(cuda, dtype=BF, seed=5, **kw):
    from ohara_amd.phi import Phi, PhiConfig

    base = dict(vocab_size=64, max_sequence_length=16, hidden_size=64, num_attention_heads=4, num_hidden_layers=2,
                multiple_of=4, rotary_dim=0.4)
    base.update(kw)
    rcfg = P.RefPhiConfig(**base)
    w = P.init_weights(rcfg, seed=seed, dtype=dtype, std=0.08, bias_std=0.05)
    return P.RefPhi(rcfg, w), Phi(PhiConfig(**base), w, device=cuda)


def _close(got, ref, max_rel=4e-2, mean_rel=4e-3):
    got, ref = got.float().cpu(), ref.float()
    scale = ref.abs().max().item()
    d = (got - ref).abs()
    assert d.max().item() <= max_rel * scale, (d.max().item(), scale)
    assert d.mean().item() <= mean_rel * scale, (d.mean().item(), scale)


@pytest.mark.parametrize("kw", [
    dict(),                                                                      # head_dim 16, 6 rotated features
    dict(vocab_size=80, max_sequence_length=12, num_attention_heads=2, num_hidden_layers=3, multiple_of=2,
         rotary_dim=0.5),                                                        # head_dim 32, 16 rotated
    dict(vocab_size=512, max_sequence_length=96, hidden_size=320, num_attention_heads=4, num_hidden_layers=3),  # 80 / 32
])
def test_model_prefill_and_cached_steps_against_the_oracle(cuda, kw):
    ref, model = _pair(cuda, **kw)
    c = ref.cfg
    g = torch.Generator().manual_seed(0)
    B, S0 = 2, 7
    ids = torch.randint(0, c.vocab_size, (B, S0 + 3), generator=g)
    rc, cache = ref.build_kv_cache(B), model.build_kv_cache(B)
    _close(model(ids[:, :S0].to(cuda), cache, 0), ref(ids[:, :S0], rc, 0))
    for t in range(S0, S0 + 3):
        _close(model(ids[:, t:t + 1].to(cuda), cache, t), ref(ids[:, t:t + 1], rc, t))
    assert cache[0].length == S0 + 3
    # the cache holds what the oracle's holds: the un-rotated key projection
    _close(cache[-1].key[:B, :S0 + 3], rc[-1].key[:B, :S0 + 3])
    # no cache: the plain causal forward
    _close(model(ids.to(cuda)), ref(ids))
    # last_only computes just the last row
    c2 = model.build_kv_cache(B)
    full = model(ids[:, :S0].to(cuda), c2, 0)
    c3 = model.build_kv_cache(B)
    last = model(ids[:, :S0].to(cuda), c3, 0, last_only=True)
    assert torch.equal(last[:, 0], full[:, -1])


def test_cached_decode_matches_full_forward_on_the_gpu(cuda):
    """The reference's own Phi test (tests/test_models.py:133-149) run on the HIP path; bf16
    tolerances instead of its fp32 1e-4."""
    _, model = _pair(cuda, vocab_size=128, max_sequence_length=32, hidden_size=128, num_attention_heads=4)
    ids = torch.randint(0, 128, (1, 9), generator=torch.Generator().manual_seed(1)).to(cuda)
    full = model(ids)
    cache = model.build_kv_cache()
    prefill = model(ids[:, :4], cache, 0)
    step = model(ids[:, 4:5], cache, 4)
    _close(prefill[:, -1], full[:, 3].cpu(), 2e-2, 2e-3)
    _close(step[:, -1], full[:, 4].cpu(), 2e-2, 2e-3)


def test_graph_replayed_decode_reads_the_position_on_the_device(cuda):
    from ohara_amd import ops

    ref, model = _pair(cuda, vocab_size=128, max_sequence_length=32, hidden_size=128, num_attention_heads=4)
    ids = torch.randint(0, 128, (2, 6), generator=torch.Generator().manual_seed(2))
    rc, cache = ref.build_kv_cache(2), model.build_kv_cache(2)
    want = ref(ids, rc, 0)
    model(ids.to(cuda), cache, 0)
    tok = want[:, -1].float().argmax(-1).view(2, 1)
    pos_dev = torch.tensor([6], dtype=torch.int32, device=cuda)
    for t in range(6, 10):  # eager launches, position from the device scalar
        got = model(tok.to(cuda), cache, t, pos_dev=pos_dev)
        want = ref(tok, rc, t)
        _close(got, want)
        ops.advance_positions(pos_dev)
        tok = want[:, -1].float().argmax(-1).view(2, 1)
    assert int(pos_dev.item()) == 10


def test_error_surface(cuda):
    _, model = _pair(cuda)
    ids = torch.zeros(1, 1, dtype=torch.int64, device=cuda)
    cache = model.build_kv_cache()
    with pytest.raises(ValueError, match="position_ids is required"):
        model(ids, cache, None)
    with pytest.raises(ValueError, match="one entry per model layer"):
        model(ids, cache[:1], 0)
    with pytest.raises(ValueError, match="at least 1"):
        model.build_kv_cache(0)
    with pytest.raises(ValueError, match="sequential"):
        model(ids, cache, 3)
    model(ids, cache, 0)
    with pytest.raises(ValueError, match="exceeds max_sequence_length"):
        model(torch.zeros(1, 16, dtype=torch.int64, device=cuda), cache, 1)


@pytest.mark.parametrize("use_graph", [True, False])
def test_greedy_generation_matches_the_oracle_teacher_forced(cuda, use_graph):
    """Every generated token is the oracle's arg-max for the same history (or a near-tie of its own
    logits); the oracle is teacher-forced on the tokens produced."""
    ref, model = _pair(cuda, vocab_size=256, max_sequence_length=48, hidden_size=128, num_attention_heads=4,
                       num_hidden_layers=2)
    prompt = torch.randint(0, 256, (2, 9), generator=torch.Generator().manual_seed(3))
    steps = 12
    toks = model.generate_greedy(prompt.to(cuda), steps, use_graph=use_graph).cpu()
    assert toks.shape == (2, steps)
    rc = ref.build_kv_cache(2)
    logits = ref(prompt, rc, 0)[:, -1]
    for t in range(steps):
        for b in range(2):
            best, tok = int(logits[b].float().argmax()), int(toks[b, t])
            if tok != best:
                la, lb = logits[b, tok].float().item(), logits[b, best].float().item()
                assert abs(la - lb) <= 2.0 ** -6 * max(abs(la), abs(lb)), (t, b, tok, best)
        if t + 1 < steps:
            logits = ref(toks[:, t:t + 1], rc, 9 + t)[:, -1]


def test_block_head_matches_the_separate_kernels(cuda):
    """LayerNorm + [q; k; v; fc1] + append + new_gelu in one launch against the same steps as
    separate kernels (its variance comes from the sums of x and x^2, so a normalised value may
    round the other way now and then)."""
    from ohara_amd import ops

    g = torch.Generator().manual_seed(4)
    for B, S, d, ff, H, pos in ((2, 3, 64, 256, 4, 5), (1, 1, 320, 1280, 4, 0), (3, 1, 2560, 10240, 32, 7),
                                (70, 1, 64, 128, 2, 2), (2, 1, 2048, 128, 16, 1), (130, 1, 64, 128, 2, 2),
                                (10, 10, 128, 512, 4, 2)):
        rows, D, Tmax = B * S, d // H, 16
        x = (torch.randn(rows, d, generator=g) + 0.3).to(BF).to(cuda)
        lw = (1 + 0.1 * torch.randn(d, generator=g)).to(BF).to(cuda)
        lb = (0.1 * torch.randn(d, generator=g)).to(BF).to(cuda)
        w = (torch.randn(3 * d + ff, d, generator=g) / d ** 0.5).to(BF).to(cuda)
        b = (0.2 * torch.randn(3 * d + ff, generator=g)).to(BF).to(cuda)
        pw = ops.pack_linear(w)
        kc = torch.zeros(B, Tmax, H, D, dtype=BF, device=cuda)
        vc = torch.zeros_like(kc)
        q = torch.empty(rows, d, dtype=BF, device=cuda)
        act = torch.empty(rows, ff, dtype=BF, device=cuda)
        ops.phi_block_in(x, lw, lb, 1e-5, pw, b, d, ff, B, S, pos, kc, vc, q, act)
        h = ops.layernorm(x, lw, lb, 1e-5)
        y = ops.linear_bias(h, pw, b)
        kc2, vc2 = torch.zeros_like(kc), torch.zeros_like(vc)
        ops.kv_append(y[:, d:2 * d], y[:, 2 * d:3 * d], kc2, vc2, B, S, H, D, pos)
        want_act = P.new_gelu(y[:, 3 * d:].cpu())
        # without the prologue (normalised rows handed in) the results are those of the separate kernels
        kc3, vc3, q3, act3 = torch.zeros_like(kc), torch.zeros_like(vc), torch.empty_like(q), torch.empty_like(act)
        ops.phi_block_in(h, None, None, 1e-5, pw, b, d, ff, B, S, pos, kc3, vc3, q3, act3)
        assert torch.equal(q3, y[:, :d]) and torch.equal(kc3, kc2) and torch.equal(vc3, vc2)
        assert (act3.cpu() != want_act).float().mean().item() < 5e-3
        for name, got, want in (("q", q, y[:, :d]), ("k", kc, kc2), ("v", vc, vc2), ("act", act.cpu(), want_act)):
            got, want = got.float().cpu(), want.float().cpu()
            diff = (got - want).abs()
            scale = want.abs().max().item()
            assert diff.max().item() <= 2.0 ** -6 * scale, (name, B, d, diff.max().item(), scale)
            assert (diff > 0).float().mean().item() < 0.02, (name, B, d, (diff > 0).float().mean().item())
        assert torch.equal(kc[:, :pos], torch.zeros_like(kc[:, :pos])) and torch.equal(kc[:, pos + S:], torch.zeros_like(kc[:, pos + S:]))


@pytest.mark.parametrize("B", [5, 20, 70, 130])
def test_decode_batches_of_several_row_groups(cuda, B):
    """More than 16 rows (several row groups per weight strip), more than 64 (two passes of the
    weight-streaming kernel) and more than 128 (the tiled kernel also serves single-token calls):
    prefill and cached steps against the oracle."""
    ref, model = _pair(cuda, vocab_size=256, max_sequence_length=32, hidden_size=128, num_attention_heads=4,
                       num_hidden_layers=2)
    ids = torch.randint(0, 256, (B, 7), generator=torch.Generator().manual_seed(B))
    rc, cache = ref.build_kv_cache(B), model.build_kv_cache(B)
    _close(model(ids[:, :4].to(cuda), cache, 0), ref(ids[:, :4], rc, 0))
    for t in (4, 5, 6):
        _close(model(ids[:, t:t + 1].to(cuda), cache, t), ref(ids[:, t:t + 1], rc, t))
    _close(cache[0].value[:B, :7], rc[0].value[:B, :7])


def test_model_from_local_checkpoint_shards(cuda, tmp_path):
    """Phi.from_local_checkpoint: safetensors shards under microsoft/phi-2's tensor names
    (ohara/models/phi.py:208-256) -> the same logits as the model built from the state dict."""
    from safetensors.torch import save_file

    from ohara_amd.phi import Phi, PhiConfig, huggingface_state_dict_map

    kw = dict(vocab_size=64, max_sequence_length=16, hidden_size=64, num_attention_heads=4, num_hidden_layers=2)
    w = P.init_weights(P.RefPhiConfig(**kw), seed=6, dtype=BF, std=0.08, bias_std=0.05)
    mapping = huggingface_state_dict_map(2)
    save_file({mapping[k]: v.contiguous() for k, v in w.items()}, str(tmp_path / "model.safetensors"))
    a = Phi.from_local_checkpoint(str(tmp_path), PhiConfig(**kw), device=cuda)
    b = Phi(PhiConfig(**kw), w, device=cuda)
    ids = torch.randint(0, 64, (2, 6), generator=torch.Generator().manual_seed(0)).to(cuda)
    assert torch.equal(a(ids), b(ids))


@pytest.mark.parametrize("kw", [
    dict(vocab_size=80, max_sequence_length=24, num_attention_heads=2, num_hidden_layers=3, multiple_of=2, rotary_dim=0.5),
    dict(vocab_size=512, max_sequence_length=96, hidden_size=320, num_attention_heads=4, num_hidden_layers=3),  # 80 / 32
])
def test_model_on_int8_caches_against_the_oracle(cuda, kw):
    """Phi on the int8 caches of ohara/modules/kv_cache.py:15-32: the un-rotated rows are quantised on write and attention
    reads the dequantised prefix; prefill and cached steps against the oracle on its own int8 caches, and layer 0's
    codes (no attention in front of them) against the oracle quantiser applied to a bf16-cache run's rows."""
    from oracle import llama_ref as R

    ref, model = _pair(cuda, **kw)
    c = ref.cfg
    g = torch.Generator().manual_seed(3)
    B, S0 = 2, 9
    ids = torch.randint(0, c.vocab_size, (B, S0 + 3), generator=g)
    rc, cache = ref.build_kv_cache(B, int8=True), model.build_kv_cache(B, int8=True)
    assert cache[0].key.dtype == torch.int8
    _close(model(ids[:, :S0].to(cuda), cache, 0), ref(ids[:, :S0], rc, 0), 4e-2, 6e-3)
    for t in range(S0, S0 + 3):
        _close(model(ids[:, t:t + 1].to(cuda), cache, t), ref(ids[:, t:t + 1], rc, t), 4e-2, 6e-3)
    assert cache[0].length == S0 + 3
    plain = model.build_kv_cache(B)
    model(ids[:, :S0].to(cuda), plain, 0)
    kq, _, _ = R.quantize_int8(plain[0].key[:, :S0].cpu())
    vq, _, _ = R.quantize_int8(plain[0].value[:, :S0].cpu())
    assert torch.equal(cache[0].key[:, :S0].cpu(), kq) and torch.equal(cache[0].value[:, :S0].cpu(), vq)
    mixed = [model.build_kv_cache(1, int8=True)[0]] + model.build_kv_cache(1)[1:]
    with pytest.raises(ValueError, match="same KV cache mode"):
        model(ids[:1, :2].to(cuda), mixed, 0)


def test_greedy_generation_on_int8_caches_with_the_position_on_the_device(cuda):
    """generate_greedy(int8=True): the captured step (position read on the device, the dequantised working copy
    spanning the cache's capacity) produces the tokens of eager single-token forwards over int8 caches."""
    ref, model = _pair(cuda, vocab_size=512, max_sequence_length=96, hidden_size=320, num_attention_heads=4,
                       num_hidden_layers=3)  # head width 80, 32 rotated
    c = ref.cfg
    B, P, steps = 2, 7, 8
    ids = torch.randint(0, c.vocab_size, (B, P), generator=torch.Generator().manual_seed(8)).to(cuda)
    cache = model.build_kv_cache(B, int8=True)
    tok = model(ids, cache, 0, last_only=True).view(B, -1).float().argmax(-1)
    want = [tok]
    for t in range(P, P + steps - 1):
        tok = model(tok.view(B, 1), cache, t).view(B, -1).float().argmax(-1)
        want.append(tok)
    want = torch.stack(want, 1).cpu()
    for use_graph in (False, True):
        got = model.generate_greedy(ids, steps, use_graph=use_graph, int8=True).cpu()
        assert torch.equal(got, want), (use_graph, got, want)
