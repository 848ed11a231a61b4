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


@pytest.mark.parametrize("B,L", [(16, 32768), (64, 4096)])
def test_decode_attention_microbench_shape(cuda, B, L):
    """32 query / 8 KV heads x 128, one query per sequence over L cached positions."""
    from ohara_amd import ops

    H, Hkv, D = 32, 8, 128
    G = H // Hkv
    ns = max(1, min(1024 // (B * Hkv), L // 128, 64))
    g = torch.Generator(device=cuda).manual_seed(1)
    q = torch.randn(B, H * D, device=cuda, generator=g).to(BF)
    k = torch.randn(B, L, Hkv, D, device=cuda, generator=g).to(BF)
    v = torch.randn(B, L, Hkv, D, device=cuda, generator=g).to(BF)
    ws = ops.attn_workspace(B, H, Hkv, D, ns, cuda)
    out = ops.attn_decode(q, k, v, H, Hkv, D, L, ns, ws).view(B, H, D)
    # sub-sampled (sequence, head) pairs against fp32 torch on the device
    for b, h in ((0, 0), (B // 2, 13), (B - 1, H - 1), (3, 6)):
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
