"""One cache position per sequence (ragged batches) and continuous batching.

The reference has a single scalar position for the whole batch (ohara/models/llama.py:287-299),
so its answer for a ragged batch is what it computes for every sequence on its own: the checks
compare the batched kernels with per-sequence calls (bit for bit at kernel level) and with the
CPU oracle run sequence by sequence (bf16 tolerances of the model tests).
"""

import dataclasses

import pytest
import torch

from oracle import llama_ref as R

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


def test_rotary_append_and_attention_per_sequence_positions(cuda):
    from ohara_amd import ops

    B, S, H, Hkv, D, K, Tmax = 3, 2, 4, 2, 64, 128, 40
    pos = [7, 0, 31]
    g = torch.Generator().manual_seed(3)
    x = torch.randn(B * S, K, generator=g).to(BF).to(cuda)
    wq, wk, wv = ((torch.randn(n * D, K, generator=g) * 0.05).to(BF).to(cuda) for n in (H, Hkv, Hkv))
    nw = (1 + 0.2 * torch.randn(K, generator=g)).to(BF).to(cuda)
    cos, sin = (t.to(BF).to(cuda) for t in R.rope_table(D, 2 * Tmax, 10000.0))
    wp = ops.pack_qkv(wq, wk, wv)
    base = torch.randn(B, Tmax, Hkv, D, generator=g).to(BF).to(cuda)
    kc, vc = base.clone(), (base * 0.5).to(BF)
    kc1, vc1 = kc.clone(), vc.clone()
    seq_pos = torch.tensor(pos, dtype=torch.int32, device=cuda)
    q = ops.qkv_rope_append(x, wp, nw, 1e-5, H, Hkv, D, cos, sin, 0, kc, vc, seq_len=S, seq_pos=seq_pos)
    for b in range(B):  # the same rows through the scalar-position entry point, one sequence at a time
        qb = ops.qkv_rope_append(x[b * S:(b + 1) * S], wp, nw, 1e-5, H, Hkv, D, cos, sin, pos[b], kc1[b:b + 1],
                                 vc1[b:b + 1], seq_len=S)
        assert torch.equal(qb, q[b * S:(b + 1) * S])
    assert torch.equal(kc, kc1) and torch.equal(vc, vc1)
    for ns in (1, 3):
        ws = ops.attn_workspace(B * S, H, Hkv, D, ns, cuda)
        out = ops.attn_cached(q, kc, vc, H, Hkv, D, 0, ns, ws, seq_len=S, seq_pos=seq_pos)
        for b in range(B):
            ob = ops.attn_cached(q[b * S:(b + 1) * S], kc[b:b + 1], vc[b:b + 1], H, Hkv, D, pos[b], ns, ws, seq_len=S)
            assert torch.equal(ob, out[b * S:(b + 1) * S]), (ns, b)
    # advancing on the device
    act = torch.tensor([1, 0, 1], dtype=torch.uint8, device=cuda)
    ops.advance_positions(seq_pos, act, 2)
    assert seq_pos.tolist() == [9, 0, 33]
    ops.advance_positions(seq_pos)
    assert seq_pos.tolist() == [10, 1, 34]


def _cfg_pair(**kw):
    from ohara_amd.llama import Config

    fields = {f.name for f in dataclasses.fields(R.RefConfig)}
    kw = {k: v for k, v in kw.items() if k in fields}
    return R.RefConfig(**kw), Config(**kw)


def _close(got, ref, max_rel=4e-2, mean_rel=4e-3):
    got, ref = got.float().cpu(), ref.float()
    scale = ref.abs().max().item()
    d = (got - ref).abs()
    assert d.max().item() <= max_rel * scale, (d.max().item(), scale)
    assert d.mean().item() <= mean_rel * scale, (d.mean().item(), scale)


def _small_model(cuda):
    from ohara_amd.llama import Llama

    rcfg, cfg = _cfg_pair(vocab_size=512, hidden_size=256, intermediate_size=512, num_attention_heads=4,
                          num_key_value_heads=2, num_hidden_layers=3, max_sequence_length=96, rope_theta=10000.0)
    w = R.init_weights(rcfg, seed=6, dtype=BF, std=0.06, norm_jitter=0.1)
    return R.RefLlama(rcfg, w), Llama(cfg, w, device=cuda)


def test_model_forward_with_one_position_per_sequence(cuda):
    ref, model = _small_model(cuda)
    lens = [5, 23, 1]
    B = len(lens)
    g = torch.Generator().manual_seed(0)
    prompts = [torch.randint(0, 512, (1, n), generator=g) for n in lens]
    cache = model.build_kv_cache(B)
    for c in cache:
        c._commit_ragged(B, [0] * B)
    rcaches = [ref.build_kv_cache(1) for _ in range(B)]
    want_last = []
    for b, p in enumerate(prompts):  # every prompt alone into its own rows of the shared caches
        views = [c._row_view(b) for c in cache]
        got = model(p.to(cuda), views, 0)
        want = ref(p, rcaches[b], 0)
        _close(got, want)
        want_last.append(want[:, -1])
        for c in cache:
            c.lengths[b] = lens[b]
            c.length = max(c.lengths)
    pos = list(lens)
    nxt = torch.stack([w.float().argmax(-1) for w in want_last]).view(B, 1)
    for step in range(4):  # batched decode, every sequence at its own position
        got = model(nxt.to(cuda), cache, pos)
        want = torch.cat([ref(nxt[b:b + 1], rcaches[b], pos[b]) for b in range(B)])
        _close(got, want)
        pos = [p + 1 for p in pos]
        nxt = want[:, -1].float().argmax(-1).view(B, 1)
    assert cache[0].lengths == pos and cache[0].length == max(pos)
    # two tokens per sequence in one ragged call, positions as a tensor
    two = torch.randint(0, 512, (B, 2), generator=g)
    got = model(two.to(cuda), cache, torch.tensor(pos))
    want = torch.cat([ref(two[b:b + 1], rcaches[b], pos[b]) for b in range(B)])
    _close(got, want)
    # bookkeeping and messages
    with pytest.raises(ValueError, match="sequential"):
        model(nxt.to(cuda), cache, pos)  # stale positions
    with pytest.raises(ValueError, match="different lengths"):
        model(nxt.to(cuda), cache, 7)
    with pytest.raises(ValueError, match="one position per sequence"):
        model(nxt.to(cuda), cache, [1, 2])
    with pytest.raises(ValueError, match="exceeds max_sequence_length"):
        model(nxt.to(cuda), cache, [95, 96, 3])


@pytest.mark.parametrize("use_graph,chunked", [(True, False), (False, False), (True, True)])
def test_continuous_batching_matches_sequences_run_alone(cuda, use_graph, chunked):
    """Sequences join and leave at different times; every token a slot produces is the oracle's
    greedy choice for that sequence alone (or a near-tie of the oracle's own logits).  ``chunked``: several
    steps per read-back (``ContinuousBatcher.steps``)."""
    from ohara_amd.batching import ContinuousBatcher

    ref, model = _small_model(cuda)
    g = torch.Generator().manual_seed(5)
    prompts = {name: torch.randint(0, 512, (n,), generator=g) for name, n in (("a", 9), ("b", 30), ("c", 3), ("d", 17))}
    bat = ContinuousBatcher(model, slots=3)
    out = {k: [] for k in prompts}
    slot_of = {}

    def add(name):
        slot, tok = bat.add(prompts[name])
        slot_of[name] = slot
        out[name].append(tok)

    def steps(n):
        if chunked:
            got = bat.steps(n, use_graph=use_graph)
            for name, slot in slot_of.items():
                assert len(got[slot]) == n
                out[name].extend(got[slot])
            return
        for _ in range(n):
            toks = bat.step(use_graph=use_graph)
            for name, slot in slot_of.items():
                out[name].append(toks[slot])

    add("a")
    steps(3)
    add("b")
    add("c")
    assert bat.free_slots() == []
    with pytest.raises(RuntimeError, match="no free slot"):
        bat.add(prompts["d"])
    steps(5)
    bat.remove(slot_of.pop("a"))  # a leaves, d takes its slot and cache rows
    add("d")
    steps(6)
    bat.remove(slot_of.pop("c"))
    steps(4)
    assert bat.lengths[slot_of["b"]] == 30 + 15 and bat.lengths[slot_of["d"]] == 17 + 10
    assert [len(out[k]) for k in "abcd"] == [9, 16, 12, 11]

    for name, toks in out.items():  # oracle, teacher-forced on the tokens the batcher produced
        rc = ref.build_kv_cache(1)
        logits = ref(prompts[name].view(1, -1), rc, 0)[:, -1]
        pos = prompts[name].numel()
        for t, tok in enumerate(toks):
            best = int(logits.float().argmax(-1))
            if tok != best:
                la, lb = logits[0, tok].float().item(), logits[0, best].float().item()
                ulp = 2.0 ** (torch.tensor(max(abs(la), abs(lb), 1e-30)).log2().floor().item() - 7)
                assert abs(la - lb) <= 2 * ulp, (name, t, tok, best)
            logits = ref(torch.tensor([[tok]]), rc, pos)[:, -1]
            pos += 1


def test_continuous_batching_with_sampling_runs(cuda):
    from ohara_amd.batching import ContinuousBatcher
    from ohara_amd.sampling import SamplingConfig

    _, model = _small_model(cuda)
    gen = torch.Generator(device=cuda).manual_seed(0)
    bat = ContinuousBatcher(model, slots=2, sampling=SamplingConfig(temperature=0.8, top_k=20, top_p=0.9), valid_vocab=500,
                            generator=gen)
    s0, t0 = bat.add([1, 2, 3])
    s1, t1 = bat.add(list(range(40)))
    seen = [t0, t1]
    for _ in range(5):
        seen.extend(bat.step().values())
    assert all(0 <= t < 500 for t in seen) and bat.lengths == [8, 45]


@pytest.mark.parametrize("B", [20, 70])
def test_ragged_decode_at_larger_batches(cuda, B):
    """One position per sequence with more than 16 and more than 64 sequences: every sequence is
    prefilled alone to its own length, then the whole batch decodes together; the oracle runs sequence
    by sequence."""
    ref, model = _small_model(cuda)
    g = torch.Generator().manual_seed(B)
    lens = torch.randint(1, 40, (B,), generator=g).tolist()
    prompts = [torch.randint(0, 512, (1, n), generator=g) for n in lens]
    cache = model.build_kv_cache(B)
    for c in cache:
        c._commit_ragged(B, [0] * B)
    rcaches = [ref.build_kv_cache(1) for _ in range(B)]
    last = []
    for b, p in enumerate(prompts):
        model(p.to(cuda), [c._row_view(b) for c in cache], 0)
        last.append(ref(p, rcaches[b], 0)[:, -1])
        for c in cache:
            c.lengths[b] = lens[b]
            c.length = max(c.lengths)
    pos = list(lens)
    nxt = torch.stack([w.float().argmax(-1) for w in last]).view(B, 1)
    for step in range(3):
        got = model(nxt.to(cuda), cache, pos)
        want = torch.cat([ref(nxt[b:b + 1], rcaches[b], pos[b]) for b in range(B)])
        _close(got, want)
        pos = [p + 1 for p in pos]
        nxt = want[:, -1].float().argmax(-1).view(B, 1)


def test_int8_append_and_attention_per_sequence_positions(cuda):
    """The int8 cache's append and the attention over its codes with one position per sequence: bit for bit what
    the scalar-position entry points give sequence by sequence."""
    from ohara_amd import ops
    from ohara_amd.llama import KVCache

    B, S, H, Hkv, D, Tmax = 3, 2, 4, 2, 64, 40
    pos = [7, 0, 31]
    g = torch.Generator().manual_seed(11)
    shape = (B, Tmax, Hkv, D)
    ca, cb = (KVCache(shape, Tmax, 0, device=cuda, dtype=BF, int8=True) for _ in range(2))
    # a common prefix in both caches (positions 0 .. 31 of every sequence), appended with the scalar entry point
    pk = (torch.randn(B, 32, Hkv, D, generator=g) * 1.3).to(BF).to(cuda)
    pv = (torch.randn(B, 32, Hkv, D, generator=g) * 0.4).to(BF).to(cuda)
    for c in (ca, cb):
        ops.kv_quant_append(pk, pv, c, 0)
    k = (torch.randn(B, S, Hkv, D, generator=g) * 1.3).to(BF).to(cuda)
    v = (torch.randn(B, S, Hkv, D, generator=g) * 0.4).to(BF).to(cuda)
    q = torch.randn(B * S, H * D, generator=g).to(BF).to(cuda)
    seq_pos = torch.tensor(pos, dtype=torch.int32, device=cuda)
    ops.kv_quant_append(k, v, ca, 0, seq_pos=seq_pos)
    for b in range(B):
        ops.kv_quant_append(k[b:b + 1], v[b:b + 1], cb._row_view(b), pos[b])
    assert torch.equal(ca.key, cb.key) and torch.equal(ca.value, cb.value) and torch.equal(ca.stats, cb.stats)
    for ns in (1, 3):
        ws = ops.attn_workspace(B * S, H, Hkv, D, ns, cuda)
        out = ops.attn_cached_int8(q, ca, H, Hkv, D, 0, ns, ws, seq_len=S, seq_pos=seq_pos)
        for b in range(B):
            ob = ops.attn_cached_int8(q[b * S:(b + 1) * S], cb._row_view(b), H, Hkv, D, pos[b], ns, ws, seq_len=S)
            assert torch.equal(ob, out[b * S:(b + 1) * S]), (ns, b)


def test_model_forward_with_one_position_per_sequence_on_int8_caches(cuda):
    """Ragged batches over int8 caches against the oracle run sequence by sequence on its own int8 caches."""
    ref, model = _small_model(cuda)
    lens = [5, 23, 1]
    B = len(lens)
    g = torch.Generator().manual_seed(1)
    prompts = [torch.randint(0, 512, (1, n), generator=g) for n in lens]
    cache = model.build_kv_cache(B, int8=True)
    for c in cache:
        c._commit_ragged(B, [0] * B)
    rcaches = [ref.build_kv_cache(1, int8=True) for _ in range(B)]
    want_last = []
    for b, p in enumerate(prompts):
        views = [c._row_view(b) for c in cache]
        got = model(p.to(cuda), views, 0)
        want = ref(p, rcaches[b], 0)
        _close(got, want, 4e-2, 6e-3)
        want_last.append(want[:, -1])
        for c in cache:
            c.lengths[b] = lens[b]
            c.length = max(c.lengths)
    pos = list(lens)
    nxt = torch.stack([w.float().argmax(-1) for w in want_last]).view(B, 1)
    for step in range(4):
        got = model(nxt.to(cuda), cache, pos)
        want = torch.cat([ref(nxt[b:b + 1], rcaches[b], pos[b]) for b in range(B)])
        _close(got, want, 4e-2, 6e-3)
        pos = [p + 1 for p in pos]
        nxt = want[:, -1].float().argmax(-1).view(B, 1)
    two = torch.randint(0, 512, (B, 2), generator=g)
    got = model(two.to(cuda), cache, torch.tensor(pos))
    want = torch.cat([ref(two[b:b + 1], rcaches[b], pos[b]) for b in range(B)])
    _close(got, want, 4e-2, 6e-3)
    # layer 0's codes are the oracle's wherever its rows agree bit for bit with the oracle's: at least the first
    # position of every sequence (an embedding row through norm, projection and rotary at position 0)
    assert cache[0].lengths == [p + 2 for p in pos]


def test_continuous_batching_on_int8_caches(cuda):
    """The batcher over int8 caches: the tokens of every slot are those of the same sequence decoded alone by a
    session on int8 caches (the kernel chain both times; greedy), up to near-ties of the oracle's logits."""
    from ohara_amd.batching import ContinuousBatcher

    ref, model = _small_model(cuda)
    g = torch.Generator().manual_seed(9)
    prompts = {name: torch.randint(0, 512, (n,), generator=g) for name, n in (("a", 9), ("b", 30), ("c", 3))}
    bat = ContinuousBatcher(model, slots=3, int8=True)
    assert bat.cache[0].int8
    out, slot_of = {k: [] for k in prompts}, {}
    for name in "ab":
        slot_of[name], tok = bat.add(prompts[name])
        out[name].append(tok)
    for _ in range(4):
        toks = bat.step()
        for name, slot in slot_of.items():
            out[name].append(toks[slot])
    slot_of["c"], tok = bat.add(prompts["c"])
    out["c"].append(tok)
    for _ in range(5):
        toks = bat.step()
        for name, slot in slot_of.items():
            out[name].append(toks[slot])
    for name, toks in out.items():  # oracle on int8 caches, teacher-forced on the tokens the batcher produced
        rc = ref.build_kv_cache(1, int8=True)
        logits = ref(prompts[name].view(1, -1), rc, 0)[:, -1]
        pos = prompts[name].numel()
        for t, tok in enumerate(toks):
            best = int(logits.float().argmax(-1))
            if tok != best:
                la, lb = logits[0, tok].float().item(), logits[0, best].float().item()
                ulp = 2.0 ** (torch.tensor(max(abs(la), abs(lb), 1e-30)).log2().floor().item() - 7)
                assert abs(la - lb) <= 3 * ulp, (name, t, tok, best)
            logits = ref(torch.tensor([[tok]]), rc, pos)[:, -1]
            pos += 1
