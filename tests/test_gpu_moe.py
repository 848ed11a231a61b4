"""Grouped MoE kernels (C ABI: ohara_moe_*) against the CPU oracle and the reference fixture."""

import dataclasses
import os

import pytest
import torch

from oracle import llama_ref as R
from oracle import moe_ref as M

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


def _make(N, d, E, hidden, k, shared, seed, std=0.05):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: (torch.randn(*s, generator=g) * std).to(BF)
    w = dict(w_gate=r(E, d, hidden), w_up=r(E, d, hidden), w_down=r(E, hidden, d),
             router=(torch.randn(E, d, generator=g) * d ** -0.5).to(BF),
             bias=(torch.randn(E, generator=g) * 0.3).to(BF))
    sh = (r(hidden * shared, d), r(hidden * shared, d), r(d, hidden * shared)) if shared else None
    x = torch.randn(N, d, generator=g).to(BF)
    return w, sh, x


@pytest.mark.parametrize("N,d,E,hidden,k,shared,gate", [(64, 1024, 64, 512, 8, 1, "softmax"), (9, 64, 6, 24, 2, 0, "softmax"),
                                                       (40, 128, 16, 32, 4, 2, "sigmoid"), (5, 32, 8, 16, 2, 1, "softmax")])
def test_grouped_moe_matches_oracle(cuda, N, d, E, hidden, k, shared, gate):
    from ohara_amd.moe import GroupedMoE

    w, sh, x = _make(N, d, E, hidden, k, shared, seed=N + E)
    moe = GroupedMoE(w["w_gate"], w["w_up"], w["w_down"], w["router"], w["bias"], k, sh, gate_fn=gate, device=cuda)
    idx_ref, wt_ref, logits = M.moe_route(x, w["router"], w["bias"], k, gate_fn=gate)
    idx, wt = moe.route(x.to(cuda))
    # selection: identical except where the router's own bf16 rounding noise swaps near-equal logits
    same = (idx.cpu().long() == idx_ref).all(-1)
    assert same.float().mean().item() >= 0.9
    for n in (~same).nonzero().flatten().tolist():
        biased = logits[n] + w["bias"].float()
        a, b = set(idx.cpu()[n].tolist()), set(idx_ref[n].tolist())
        gap = max(abs(float(biased[i]) - float(biased[j])) for i in a ^ b for j in a ^ b)
        assert gap <= 2 ** -6 * max(1.0, float(biased.abs().max())), (n, gap)
    ok = same.nonzero().flatten()
    torch.testing.assert_close(wt.cpu().float()[ok], wt_ref.to(BF).float()[ok], atol=2e-3, rtol=2e-2)
    # weights of every token sum to 1 (tests/test_moe_grouped.py:89-110)
    assert (wt.float().sum(-1).cpu() - 1).abs().max().item() < 2e-2
    want = M.moe_forward(x.view(1, N, d), w["router"], w["bias"], w["w_gate"], w["w_up"], w["w_down"], k, gate_fn=gate,
                         shared=sh)[0]
    got = moe.forward(x.view(1, N, d).to(cuda))[0].cpu()
    scale = want.float().abs().max().item()
    dd = (got.float() - want.float())[ok].abs()
    assert dd.max().item() <= 3e-2 * scale and dd.mean().item() <= 3e-3 * scale, (dd.max().item(), dd.mean().item(), scale)


def test_moe_sort_is_stable(cuda):
    from ohara_amd._lib import check, lib

    idx = torch.randint(0, 7, (50, 3), generator=torch.Generator().manual_seed(0), dtype=torch.int32)
    offs = torch.empty(8, dtype=torch.int32, device=cuda)
    pair_of = torch.empty(150, dtype=torch.int32, device=cuda)
    pos_of = torch.empty(150, dtype=torch.int32, device=cuda)
    check(lib().ohara_moe_sort_pairs(idx.to(cuda).data_ptr(), 150, 7, offs.data_ptr(), pair_of.data_ptr(),
                                     pos_of.data_ptr(), 0), "sort")
    torch.cuda.synchronize()
    flat = idx.reshape(-1).long()
    order = torch.argsort(flat, stable=True)  # ohara/modules/moe_grouped.py:165
    assert torch.equal(pair_of.cpu().long(), order)
    assert torch.equal(offs.cpu().long()[1:], torch.bincount(flat, minlength=7).cumsum(0))
    assert torch.equal(pos_of.cpu().long()[order], torch.arange(150))


def test_moe_llama_matches_reference_fixture(cuda):
    """The tiny grouped-MoE Llama whose logits were written from the reference."""
    from ohara_amd.llama import Config
    from ohara_amd.moe import MoeLlama

    g = torch.load(os.path.join(os.path.dirname(__file__), "golden", "llama_tiny_moe.pt"), weights_only=True)
    fields = {f.name for f in dataclasses.fields(R.RefConfig)}
    kw = {k: v for k, v in g["config"].items() if k in fields}
    state = {k: (v.to(BF) if v.is_floating_point() else v) for k, v in g["state"].items()}
    ref = R.RefLlama(R.RefConfig(**kw), state)
    from ohara_amd.llama import Llama

    model = Llama(Config(**kw), state, device=cuda)  # a config with routed experts: Llama hands out the MoE model
    assert isinstance(model, MoeLlama)
    ids = g["ids"]
    want = ref(ids)
    got = model(ids.to(cuda)).cpu()
    scale = want.float().abs().max().item()
    d = (got.float() - want.float()).abs()
    assert d.max().item() <= 4e-2 * scale and d.mean().item() <= 5e-3 * scale, (d.max().item(), d.mean().item())
    d = (got.float() - g["logits_full"]).abs()
    assert d.mean().item() <= 1.5e-2 * scale
    cache = model.build_kv_cache(2)
    a = model(ids[:, :5].to(cuda), cache, 0)
    b = model(ids[:, 5:6].to(cuda), cache, 5)
    assert (torch.cat([a, b], 1).cpu().float() - got[:, :6].float()).abs().max().item() <= 4e-2 * scale


@pytest.mark.parametrize("B", [20, 70])
def test_moe_llama_decode_at_larger_batches(cuda, B):
    """MoE and dense layers alternating (16 experts, top-4, one shared expert), prefill and cached
    steps of more than 16 and more than 64 sequences against the oracle.  A router near-tie that bf16
    noise decides the other way sends a token to another expert and moves that row's logits, so rows
    are judged one by one and a few may differ."""
    from ohara_amd.llama import Config
    from ohara_amd.moe import MoeLlama

    kw = dict(vocab_size=256, hidden_size=128, intermediate_size=64, num_attention_heads=2, num_key_value_heads=0,
              num_hidden_layers=3, max_sequence_length=32, dropout=0.0, moe_num_experts=16, moe_experts_per_tok=4,
              moe_layer_interval=2, moe_grouped=True, moe_num_shared_experts=1, moe_gate_fn="softmax")
    rcfg = R.RefConfig(**kw)
    w = R.init_weights(rcfg, seed=9, dtype=BF, std=0.06, norm_jitter=0.1)
    ref, model = R.RefLlama(rcfg, w), MoeLlama(Config(**kw), w, device=cuda)
    ids = torch.randint(0, 256, (B, 7), generator=torch.Generator().manual_seed(B))
    rc, cache = ref.build_kv_cache(B), model.build_kv_cache(B)

    def close(got, want):
        got, want = got.float().cpu().reshape(-1, 256), want.float().reshape(-1, 256)
        scale = want.abs().max().item()
        row_err = (got - want).abs().amax(-1)
        good = row_err <= 4e-2 * scale
        assert good.float().mean().item() >= 0.9, (B, good.float().mean().item())
        assert (got - want).abs()[good].mean().item() <= 5e-3 * scale

    close(model(ids[:, :4].to(cuda), cache, 0), ref(ids[:, :4], rc, 0))
    for t in (4, 5, 6):
        close(model(ids[:, t:t + 1].to(cuda), cache, t), ref(ids[:, t:t + 1], rc, t))


def test_loop_form_moe_config_is_served(cuda):
    """``Llama(Config(moe_grouped=False, ...))`` - the per-expert loop of ohara/models/llama.py:171-178,
    state dict in the layout of ohara/modules/moe.py:51-52 (``ff.experts.N.{gate,up,down}``, router
    ``ff.gate``) - against the oracle's grouped form without shared expert and with sigmoid weights left
    unnormalised (the function the loop form computes), and bit for bit against the grouped-form model
    built from the same weights."""
    from ohara_amd.llama import Config, Llama
    from ohara_amd.moe import MoeLlama

    kw = dict(vocab_size=256, hidden_size=128, intermediate_size=64, num_attention_heads=2, num_key_value_heads=0,
              num_hidden_layers=2, max_sequence_length=32, dropout=0.0, moe_num_experts=8, moe_experts_per_tok=2,
              moe_layer_interval=1, moe_num_shared_experts=0, moe_gate_fn="sigmoid", moe_normalize_weights=False)
    rcfg = R.RefConfig(**kw, moe_grouped=True)
    w = R.init_weights(rcfg, seed=11, dtype=BF, std=0.06, norm_jitter=0.1)
    loop = {k: v for k, v in w.items() if ".ff.w_" not in k and ".ff.router.weight" not in k}
    for l in range(2):
        p = f"layers.{l}.ff."
        for e in range(8):
            loop[f"{p}experts.{e}.gate.weight"] = w[p + "w_gate"][e].t().contiguous()
            loop[f"{p}experts.{e}.up.weight"] = w[p + "w_up"][e].t().contiguous()
            loop[f"{p}experts.{e}.down.weight"] = w[p + "w_down"][e].t().contiguous()
        loop[p + "gate.weight"] = w[p + "router.weight"]
    # the loop form knows no normalisation flag: the default (True) of the config must not leak in
    model = Llama(Config(**{**kw, "moe_normalize_weights": True}, moe_grouped=False), loop, device=cuda)
    assert isinstance(model, MoeLlama)
    twin = MoeLlama(Config(**kw, moe_grouped=True), w, device=cuda)
    ref = R.RefLlama(rcfg, w)
    ids = torch.randint(0, 256, (3, 6), generator=torch.Generator().manual_seed(4))
    c1, c2, rc = model.build_kv_cache(3), twin.build_kv_cache(3), ref.build_kv_cache(3)
    for t0, t1 in ((0, 4), (4, 5), (5, 6)):
        got = model(ids[:, t0:t1].to(cuda), c1, t0)
        assert torch.equal(got, twin(ids[:, t0:t1].to(cuda), c2, t0))
        want = ref(ids[:, t0:t1], rc, t0).float()
        scale = want.abs().max().item()
        row_err = (got.float().cpu() - want).abs().amax(-1).reshape(-1)
        assert (row_err <= 4e-2 * scale).float().mean().item() >= 0.9


@pytest.mark.parametrize("N,d,E,hidden,k,shared,gate", [(64, 1024, 64, 512, 8, 1, "softmax"), (9, 64, 6, 24, 2, 0, "softmax"),
                                                       (40, 128, 16, 32, 4, 2, "sigmoid"), (5, 32, 8, 16, 2, 1, "softmax"),
                                                       (33, 256, 40, 64, 3, 1, "softmax")])
def test_moe_block_in_four_launches(cuda, N, d, E, hidden, k, shared, gate):
    """h + moe(rmsnorm(h)) as norm + router + selection + sort in one launch, the experts' two launches with the
    shared expert as one more row of their grids, and the combine - against the launch-per-step form of the same
    block: the selection from the launch's own router outputs exactly (ties to the lowest id), the sort against a
    stable host sort, rows whose selection is the same in both forms at bf16 tolerance, twice in a row (the arrival
    counter must be left at zero)."""
    from ohara_amd import ops
    from ohara_amd.moe import GroupedMoE

    w, sh, x = _make(N, d, E, hidden, k, shared, seed=3 * N + E)
    moe = GroupedMoE(w["w_gate"], w["w_up"], w["w_down"], w["router"], w["bias"], k, sh, gate_fn=gate, device=cuda)
    assert moe.fused_ok(N)
    g = torch.Generator().manual_seed(N)
    h = (torch.randn(N, d, generator=g) * 1.5).to(BF).to(cuda)
    nw = (1 + 0.1 * torch.randn(d, generator=g)).to(BF).to(cuda)
    moe.trace = []
    want = moe.forward_rows(ops.rmsnorm(h, nw, 1e-5), residual=h)
    _, idx_sep, _ = moe.trace[0]
    for rep in range(2):
        moe.trace = []
        got = moe.forward_block(h, nw, 1e-5)
        logits, idx, wt = moe.trace[0]
        offs, pair_of, pos_of = moe.last_sort
        assert int(moe._counter.item()) == 0
        lg = logits.float().cpu()
        sel = lg + w["bias"].float() if moe.biased else lg
        want_idx = M.topk_lowest_index_first(sel, k + 1)[:, :k] if moe.biased else M.topk_lowest_index_first(sel, k)
        assert torch.equal(idx.cpu().long(), want_idx), rep
        flat = idx.cpu().long().flatten()
        order = torch.sort(flat, stable=True).indices
        assert torch.equal(pair_of.cpu().long(), order)
        assert torch.equal(offs.cpu().long()[1:], torch.bincount(flat, minlength=E).cumsum(0))
        assert torch.equal(pos_of.cpu().long()[order], torch.arange(N * k))
        same = (idx.cpu().sort(-1).values == idx_sep.cpu().sort(-1).values).all(-1)
        assert same.float().mean().item() >= 0.9
        scale = want.float().abs().max().item()
        dd = (got.float() - want.float()).cpu()[same].abs()
        assert dd.max().item() <= 2e-2 * scale and dd.mean().item() <= 2e-3 * scale, (dd.max().item(), dd.mean().item(), scale)
    moe.trace = None
