"""End-to-end parity of the HIP Llama (C ABI: ohara_llama_forward) against the CPU oracle
and the golden fixtures written from the reference.

Tolerances (from the build's targets): bf16 logits max-abs <= 2e-2 and mean-abs <= 2e-3,
both relative to the logit scale (max |logit| of the oracle); greedy tokens identical to
the oracle's, except that a first divergence is accepted only where the oracle's own
top-2 logits are within 2 bf16 ulps of each other (bf16 accumulation order is unpinned
by the reference, so such near-ties are decided by rounding noise on either side).

At the d12 size the mean bound is the target or 1.25 x the distance at which the REFERENCE
reproduces itself, whichever is larger: tests/golden/llama_bf16_d12_greedy.pt holds two runs of the
reference's own bf16 model on the CPU and two repeats (one thread; the library's other matrix kernels:
its products then sum in another order), 64 steps each; they lie up to 2.5e-3 of the logit scale apart
in the mean (41 of 64 steps above 2e-3) and pick different greedy tokens at step 60.  tests/test_gpu_reference_bf16.py compares the HIP path with that run itself.
"""

import dataclasses

import pytest
import torch

from oracle import llama_ref as R
from oracle.sampling_ref import greedy_decode_ref

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


def _cfg_pair(**kw):
    from ohara_amd.llama import Config

    fields = {f.name for f in dataclasses.fields(R.RefConfig)}
    kw = {k: v for k, v in kw.items() if k in fields}
    return R.RefConfig(**kw), Config(**kw)


def _assert_logits_close(got, ref, max_rel=2e-2, mean_rel=2e-3):
    got, ref = got.float().cpu(), ref.float()
    scale = ref.abs().max().item()
    d = (got - ref).abs()
    assert d.max().item() <= max_rel * scale, (d.max().item(), scale)
    assert d.mean().item() <= mean_rel * scale, (d.mean().item(), scale)


def _rel_errors(got, ref):
    got, ref = got.float().cpu(), ref.float()
    scale = ref.abs().max().item()
    d = (got - ref).abs()
    return d.max().item() / scale, d.mean().item() / scale


def _report(name, payload):
    """Measured parity figures of the headline model, written where a GPU run's outputs are collected
    (best effort: the assertions do not depend on it)."""
    import json
    import os

    try:
        root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
        out = os.path.join(root, "gpurun_out")
        os.makedirs(out, exist_ok=True)
        with open(os.path.join(out, f"parity_{name}.json"), "w") as f:
            json.dump(payload, f, indent=1)
    except OSError:
        pass
    print(name, payload)


def _golden(name):
    import os

    g = torch.load(os.path.join(os.path.dirname(__file__), "golden", f"llama_tiny_{name}.pt"), weights_only=True)
    state = {k: (v.to(BF) if v.is_floating_point() else v) for k, v in g["state"].items()}
    return g, state


@pytest.mark.parametrize("name", ["dense", "gqa"])
def test_golden_tiny_models(cuda, name):
    """bf16 HIP path vs (a) the bf16 oracle on the same bf16 weights, (b) the reference's
    own fp32 logits from the fixture (looser: bf16 vs fp32 arithmetic)."""
    from ohara_amd.llama import Llama

    g, state = _golden(name)
    rcfg, cfg = _cfg_pair(**g["config"])
    ref = R.RefLlama(rcfg, state)
    model = Llama(cfg, state, device=cuda)
    ids = g["ids"]
    full_ref = ref(ids)
    full = model(ids.to(cuda))
    assert full.shape == full_ref.shape and full.dtype == BF
    _assert_logits_close(full, full_ref)
    _assert_logits_close(full, g["logits_full"], max_rel=6e-2, mean_rel=1e-2)
    # prefill 5 + two cached single-token steps (tests/test_training_stack.py:105-136 pattern)
    cache = model.build_kv_cache(2)
    rc = ref.build_kv_cache(2)
    a = model(ids[:, :5].to(cuda), cache, 0)
    b = model(ids[:, 5:6].to(cuda), cache, 5)
    c = model(ids[:, 6:7].to(cuda), cache, torch.tensor(6))
    ra, rb, rcc = ref(ids[:, :5], rc, 0), ref(ids[:, 5:6], rc, 5), ref(ids[:, 6:7], rc, 6)
    for got, want, gold in ((a, ra, "logits_prefill5"), (b, rb, "logits_step5"), (c, rcc, "logits_step6")):
        _assert_logits_close(got, want)
        _assert_logits_close(got, g[gold], max_rel=6e-2, mean_rel=1e-2)
    assert cache[0].length == 7 and cache[0].batch_size == 2
    # cache contents: post-rotary keys and values, reference layout (B, T, Hkv, D)
    _assert_logits_close(cache[0].key[:, :7], rc[0].key[:, :7], max_rel=2e-2, mean_rel=2e-3)
    _assert_logits_close(cache[1].value[:, :7], rc[1].value[:, :7], max_rel=2e-2, mean_rel=2e-3)
    assert not cache[0].key[:, 7:].any()
    # cached == uncached on the HIP path itself (tests/test_models.py:133-149)
    _assert_logits_close(torch.cat([a, b, c], 1), full.cpu(), max_rel=1.6e-2, mean_rel=2e-3)


def test_forward_validation_messages(cuda):
    """Same ValueErrors as the reference (llama.py:285-308, kv_cache.py:78-90)."""
    from ohara_amd.llama import Llama

    g, state = _golden("dense")
    _, cfg = _cfg_pair(**g["config"])
    m = Llama(cfg, state, device=cuda)
    ids = g["ids"].to(cuda)
    with pytest.raises(ValueError, match="shape \\(batch, sequence\\)"):
        m(ids[0])
    with pytest.raises(ValueError, match="one entry per model layer"):
        m(ids, m.build_kv_cache(2)[:1], 0)
    with pytest.raises(ValueError, match="non-negative position_ids"):
        m(ids, m.build_kv_cache(2), None)
    with pytest.raises(ValueError, match="only valid when using a KV cache"):
        m(ids, None, 3)
    with pytest.raises(ValueError, match="cannot be empty"):
        m(ids[:, :0])
    with pytest.raises(ValueError, match="exceeds max_sequence_length"):
        m(torch.zeros(1, 17, dtype=torch.long, device=cuda))
    cache = m.build_kv_cache(2)
    m(ids[:, :3], cache, 0)
    with pytest.raises(ValueError, match="sequential"):
        m(ids[:, 3:4], cache, 5)
    with pytest.raises(ValueError, match="batch size cannot change"):
        m(ids[:1, 3:4], cache, 3)
    with pytest.raises(ValueError, match="smaller than the input batch"):
        m(ids.repeat(2, 1)[:, :1], m.build_kv_cache(2), 0)
    with pytest.raises(ValueError, match="at least 1"):
        m.build_kv_cache(0)
    # a failed call must not have advanced the cache
    assert cache[0].length == 3
    m(ids[:, 3:4], cache, 3)
    assert cache[0].length == 4


def _near_tie(logits_row, a, b, ulps=2):
    la, lb = logits_row[a].float().item(), logits_row[b].float().item()
    ulp = 2.0 ** (torch.tensor(max(abs(la), abs(lb), 1e-30)).log2().floor().item() - 7)
    return abs(la - lb) <= ulps * ulp


def _reference_self_distance():
    """Worst per-step mean |logit difference| (of the logit scale) between the reference's own bf16 runs
    of the d12 model stored in the fixture (all threads against one thread and against the library's
    other matrix kernels, 64 decode steps each)."""
    from _fixtures import load_fixture, reference_self_distance

    return reference_self_distance(load_fixture("llama_bf16_d12_greedy.pt"))


def _check_greedy(model, ref, prompt, steps, cuda, max_rel=2e-2, mean_rel=2e-3, stats_out=None, tie_ulps=2):
    """(1) free-running device loop vs the oracle's greedy tokens: identical, or first
    divergence at a near-tie of the oracle's logits; (2) teacher-forced on the oracle's
    tokens so that every one of the `steps` positions is checked: logits within tolerance
    and the argmax identical or a near-tie."""
    want, want_logits = greedy_decode_ref(ref, prompt, steps, return_logits=True)
    got = model.generate_greedy(prompt.to(cuda), steps).cpu()
    assert got.shape == want.shape
    n_diverged = 0
    for b in range(prompt.size(0)):
        neq = (got[b] != want[b]).nonzero()
        if neq.numel() == 0:
            continue
        t = int(neq[0])
        assert _near_tie(want_logits[t, b], int(got[b, t]), int(want[b, t]), tie_ulps), (
            f"sequence {b} diverged at step {t}: got {int(got[b, t])}, oracle {int(want[b, t])} and not a near-tie: "
            f"{want_logits[t, b, int(got[b, t])].item()} against {want_logits[t, b, int(want[b, t])].item()}"
        )
        n_diverged += 1
    B, P = prompt.shape
    cache = model.build_kv_cache(B)
    inp, pos, same = prompt.to(cuda), 0, 0
    stats = {"free_running_identical": bool(torch.equal(got, want)), "sequences_diverged_at_a_near_tie": n_diverged,
             "first_divergence_step": [int((got[b] != want[b]).nonzero()[0]) if (got[b] != want[b]).any() else None
                                       for b in range(B)],
             "max_err": 0.0, "mean_err_worst_step": 0.0, "mean_err_avg": 0.0}
    if stats_out is not None:
        stats_out.update(stats)
        stats = stats_out
    stats["steps_within_strict_mean_2e-3"] = 0
    for t in range(steps):
        logits = model(inp, cache, pos, last_only=True)[:, 0]
        pos += inp.size(1)
        _assert_logits_close(logits, want_logits[t], max_rel, mean_rel)
        mx, mn = _rel_errors(logits, want_logits[t])
        stats["steps_within_strict_mean_2e-3"] += int(mn <= 2e-3)
        stats["max_err"] = max(stats["max_err"], mx)
        stats["mean_err_worst_step"] = max(stats["mean_err_worst_step"], mn)
        stats["mean_err_avg"] += mn / steps
        mine = logits.float().argmax(-1).cpu()
        for b in range(B):
            if int(mine[b]) == int(want[b, t]):
                same += 1
            else:
                assert _near_tie(want_logits[t, b], int(mine[b]), int(want[b, t]), tie_ulps), (t, b)
        inp = want[:, t : t + 1].to(cuda)
    assert same >= 0.9 * steps * B, f"only {same}/{steps * B} teacher-forced argmaxes identical"
    stats["teacher_forced_argmax_identical"] = f"{same}/{steps * B}"
    return got, want, n_diverged


def test_greedy_small_model(cuda):
    """A 4-layer GQA model with a small vocabulary: 64 greedy tokens, graph replay == eager.
    Weights N(0, 0.08) give this model a per-layer gain above 1, which lifts the bf16 noise
    floor (the bf16 oracle itself sits 4e-3 mean / 2e-2 max from an fp32 run of the same
    weights), hence the wider tolerance here; the d12 tests state theirs."""
    from ohara_amd.llama import Llama

    rcfg, cfg = _cfg_pair(vocab_size=512, hidden_size=256, intermediate_size=512, num_attention_heads=4,
                          num_key_value_heads=2, num_hidden_layers=4, max_sequence_length=256, rope_theta=10000.0)
    w = R.init_weights(rcfg, seed=0, dtype=BF, std=0.08, norm_jitter=0.1)
    ref = R.RefLlama(rcfg, w)
    model = Llama(cfg, w, device=cuda)
    prompt = torch.randint(0, 512, (3, 17), generator=torch.Generator().manual_seed(1))
    # (twice the maximum and three times the mean tolerance - measured: worst step 4.1e-3 -, twice the
    # near-tie width: 4 bf16 steps between the oracle's two candidates)
    got, want, nd = _check_greedy(model, ref, prompt, 64, cuda, max_rel=4e-2, mean_rel=6e-3, tie_ulps=4)
    eager = model.generate_greedy(prompt.to(cuda), 64, use_graph=False).cpu()
    assert torch.equal(eager, got), "graph replay and eager launches must agree bit for bit"
    # the kernel-per-op chain and the single persistent launch both satisfy the oracle
    assert model.supports_persistent(3)
    chain = model.generate_greedy(prompt.to(cuda), 64, persistent=False).cpu()
    chain_eager = model.generate_greedy(prompt.to(cuda), 64, persistent=False, use_graph=False).cpu()
    assert torch.equal(chain, chain_eager)
    for b in range(3):
        neq = (chain[b] != want[b]).nonzero()
        if neq.numel():
            t = int(neq[0])
            wl = greedy_decode_ref(ref, prompt, t + 1, return_logits=True)[1]
            assert _near_tie(wl[t, b], int(chain[b, t]), int(want[b, t]), 4)


def test_d12_decode_parity(cuda):
    """The d12 Llama of the headline config (d 768, 12 layers, 6 heads x 128, FFN 3072,
    vocab 65536, bf16, N(0,0.02) seed 0) at a prompt the CPU oracle finishes in seconds:
    logits of the prefill and of decode steps, then 64 greedy tokens, two sequences.

    Target: max-abs 2e-2, mean-abs 2e-3 of the logit scale.  Asserted: max-abs 2e-2 and a mean of
    max(2e-3, 1.25 x the reference's distance from itself) at every step (see the module docstring);
    whether the strict target holds at every step is recorded."""
    from ohara_amd.llama import Llama

    rcfg, cfg = _cfg_pair(vocab_size=65536, hidden_size=768, intermediate_size=3072, num_attention_heads=6,
                          num_key_value_heads=0, num_hidden_layers=12, max_sequence_length=4096, dropout=0.0)
    w = R.init_weights(rcfg, seed=0, dtype=BF)
    ref = R.RefLlama(rcfg, w)
    model = Llama(cfg, w, device=cuda)
    prompt = torch.randint(0, 65536, (2, 96), generator=torch.Generator().manual_seed(0))
    self_mean = _reference_self_distance()
    mean_tol = max(2e-3, 1.25 * self_mean)
    print(f"reference against itself: mean {self_mean:.2e}; mean tolerance {mean_tol:.2e}")
    rc, cache = ref.build_kv_cache(2), model.build_kv_cache(2)
    want = ref(prompt, rc, 0)[:, -1:]
    got = model(prompt.to(cuda), cache, 0, last_only=True)
    _assert_logits_close(got, want, 2e-2, mean_tol)
    nxt = want[:, -1].float().argmax(-1, keepdim=True)
    for step in range(3):
        want = ref(nxt, rc, 96 + step)
        got = model(nxt.to(cuda), cache, 96 + step)
        _assert_logits_close(got, want, 2e-2, mean_tol)
        nxt = want[:, -1].float().argmax(-1, keepdim=True)
    stats = {}
    _check_greedy(model, ref, prompt, 64, cuda, 2e-2, mean_tol, stats_out=stats)
    stats.update(config="d12 bf16, 2 sequences, prompt 96, 64 greedy tokens, against the CPU oracle",
                 reference_vs_itself_mean=self_mean, mean_tolerance_used=mean_tol,
                 strict_mean_2em3_holds=stats["mean_err_worst_step"] <= 2e-3,
                 strict_max_2em2_holds=stats["max_err"] <= 2e-2,
                 strict_identical_64_holds=stats["free_running_identical"])
    _report("d12_prompt96_batch2", stats)


def test_d12_prompt1024_batch1_first_64_tokens(cuda):
    """The headline configuration as stated: batch 1, a 1024-token prompt, cache capacity 4096, the
    first 64 greedy tokens against the CPU oracle (the same run against the reference's own tokens and
    logits: tests/test_gpu_reference_bf16.py).  Asserted with the same criteria as above; whether the
    strict criteria (mean-abs 2e-3, 64 identical tokens) hold is recorded without asserting it."""
    from ohara_amd.llama import Llama

    rcfg, cfg = _cfg_pair(vocab_size=65536, hidden_size=768, intermediate_size=3072, num_attention_heads=6,
                          num_key_value_heads=0, num_hidden_layers=12, max_sequence_length=4096, dropout=0.0)
    w = R.init_weights(rcfg, seed=0, dtype=BF)
    ref = R.RefLlama(rcfg, w)
    model = Llama(cfg, w, device=cuda)
    prompt = torch.randint(0, 65536, (1, 1024), generator=torch.Generator().manual_seed(0))
    self_mean = _reference_self_distance()
    mean_tol = max(2e-3, 1.25 * self_mean)
    stats = {}
    _check_greedy(model, ref, prompt, 64, cuda, 2e-2, mean_tol, stats_out=stats)
    stats.update(config="d12 bf16, batch 1, prompt 1024, 64 greedy tokens, against the CPU oracle",
                 reference_vs_itself_mean=self_mean, mean_tolerance_used=mean_tol,
                 strict_mean_2em3_holds=stats["mean_err_worst_step"] <= 2e-3,
                 strict_max_2em2_holds=stats["max_err"] <= 2e-2,
                 strict_identical_64_holds=stats["free_running_identical"])
    _report("d12_prompt1024_batch1", stats)


@pytest.mark.parametrize("batch", [8])
def test_d12_persistent_kernel_batch8_prompt1024(cuda, batch):
    """The single-launch kernel at the d12 size with eight sequences (the largest batch it serves by
    default) after 1024-token prompts: four steps, teacher-forced on the oracle's tokens, logits against
    the CPU oracle; and the same steps through the kernel chain on the same inputs."""
    from ohara_amd.llama import Llama

    rcfg, cfg = _cfg_pair(vocab_size=65536, hidden_size=768, intermediate_size=3072, num_attention_heads=6,
                          num_key_value_heads=0, num_hidden_layers=12, max_sequence_length=4096, dropout=0.0)
    w = R.init_weights(rcfg, seed=0, dtype=BF)
    ref = R.RefLlama(rcfg, w)
    model = Llama(cfg, w, device=cuda)
    P, steps = 1024, 4
    prompt = torch.randint(0, 65536, (batch, P), generator=torch.Generator().manual_seed(8))
    mean_tol = max(2e-3, 1.25 * _reference_self_distance())
    rc = ref.build_kv_cache(batch)
    # (last position only: the oracle's vocabulary projection of all 8192 prompt rows would be 2 GB)
    want = [R.linear(ref(prompt, rc, 0, return_hidden=True)[:, -1], w["vocab_proj.weight"])]
    fed = []
    for s in range(steps):
        fed.append(want[-1].float().argmax(-1))
        want.append(ref(fed[-1].view(batch, 1), rc, P + s)[:, -1])
    for persistent in (True, False):
        sess = model.session(batch, steps + 1, persistent=persistent)
        sess.prefill(prompt.to(cuda))
        _assert_logits_close(sess.logits, want[0], 2e-2, mean_tol)
        for s in range(steps):
            sess.feed(fed[s])
            sess.step()
            _assert_logits_close(sess.logits, want[s + 1], 2e-2, mean_tol)
        sess.check_error()


@pytest.mark.parametrize("persistent", [True, False])
def test_sampled_decode_session(cuda, persistent):
    """Temperature 0.8 / top-k 50 / top-p 0.9 decode driven by a pre-drawn uniform tensor, with no
    host round trip per token (forward + sampler replayed from one graph).  Checked teacher-forced:
    at every step the oracle, fed the session's own tokens, must place the session's choice in the
    CDF interval that contains that step's draw (the logits differ at the bf16 level, so the
    interval is widened by what that can move a boundary)."""
    from oracle.sampling_ref import candidate_cdf_ref
    from ohara_amd.llama import Config, Llama
    from ohara_amd.sampling import SamplingConfig

    kw = dict(vocab_size=1024, hidden_size=256, intermediate_size=512, num_attention_heads=2,
              num_key_value_heads=0, num_hidden_layers=3, max_sequence_length=128, rope_theta=10000.0)
    rcfg = R.RefConfig(**kw)
    w = R.init_weights(rcfg, seed=4, dtype=BF, std=0.08)
    ref = R.RefLlama(rcfg, w)
    model = Llama(Config(**kw), w, device=cuda)
    B, P, N = 2, 9, 24
    g = torch.Generator().manual_seed(11)
    prompt = torch.randint(0, 1024, (B, P), generator=g)
    u = torch.rand(N, B, generator=g)
    cfg = SamplingConfig(temperature=0.8, top_k=50, top_p=0.9)
    sess = model.session(B, N, persistent=persistent, sampling=cfg, u=u.to(cuda))
    sess.prefill(prompt.to(cuda))
    sess.run(N - 1)
    toks = sess.tokens().cpu()  # (B, N)
    assert toks.shape == (B, N)
    # a second session with the same draws reproduces the tokens bit for bit, eagerly too
    sess2 = model.session(B, N, persistent=persistent, sampling=cfg, u=u.to(cuda))
    sess2.prefill(prompt.to(cuda))
    sess2.run(N - 1, use_graph=False)
    assert torch.equal(sess2.tokens().cpu(), toks)
    # teacher-forced: the oracle model (loose: its logits differ from the kernels' at the bf16 level,
    # which moves CDF boundaries by a few percent on this high-gain model) and the oracle sampler on
    # the session's own logits of every step (tight: pins the wiring of draws, steps and bookkeeping)
    sess3 = model.session(B, N, persistent=persistent, sampling=cfg, u=u.to(cuda))
    sess3.prefill(prompt.to(cuda))
    own = [sess3.logits.clone().cpu()]
    for _ in range(N - 1):
        sess3.step()
        own.append(sess3.logits.clone().cpu())
    assert torch.equal(sess3.tokens().cpu(), toks)
    cache = ref.build_kv_cache(B)
    inp, pos = prompt, 0
    for t in range(N):
        logits = ref(inp, cache, pos)
        pos += inp.shape[1]
        for lg, tol in ((logits[:, -1:], 6e-2), (own[t].view(B, 1, -1), 5e-3)):
            ids, cdf = candidate_cdf_ref(lg.float(), cfg.temperature, cfg.top_p, cfg.top_k)
            for b in range(B):
                hit = (ids[b] == int(toks[b, t])).nonzero()
                assert hit.numel(), (t, b, "token outside the candidate order")
                j = int(hit[0])
                lo = float(cdf[b, j - 1]) if j > 0 else 0.0
                hi = float(cdf[b, j])
                assert lo - tol <= float(u[t, b]) <= hi + tol, (t, b, tol, int(toks[b, t]), lo, hi, float(u[t, b]))
        inp = toks[:, t : t + 1]


@pytest.mark.parametrize("persistent", [True, False])
def test_decode_to_the_last_cache_position(cuda, persistent):
    """Maximum size: the prompt plus the generated tokens fill the cache exactly (the last decode
    step appends at position T_max - 1); one more step is refused on the host.  Tokens equal the
    oracle's up to near-ties, as in the other greedy tests."""
    from ohara_amd.llama import Llama

    rcfg, cfg = _cfg_pair(vocab_size=256, hidden_size=128, intermediate_size=256, num_attention_heads=2,
                          num_key_value_heads=1, num_hidden_layers=2, max_sequence_length=48, rope_theta=10000.0)
    w = R.init_weights(rcfg, seed=9, dtype=BF, std=0.08, norm_jitter=0.1)
    ref, model = R.RefLlama(rcfg, w), Llama(cfg, w, device=cuda)
    P = 29
    prompt = torch.randint(0, 256, (2, P), generator=torch.Generator().manual_seed(2))
    steps = 48 - P + 1  # the first token comes from the prefill, the last step feeds position 47
    sess = model.session(2, steps + 1, persistent=persistent)
    sess.prefill(prompt.to(cuda))
    sess.run(steps - 1)
    got = sess.tokens().cpu()
    assert got.shape == (2, steps) and sess.cache[0].length == 48
    with pytest.raises(ValueError, match="exceeds max_sequence_length"):
        sess.run(1)
    want, want_logits = greedy_decode_ref(ref, prompt, steps, return_logits=True)
    for b in range(2):
        neq = (got[b] != want[b]).nonzero()
        if neq.numel():
            t = int(neq[0])
            assert _near_tie(want_logits[t, b], int(got[b, t]), int(want[b, t])), (b, t)
    # a single-token prompt and a prompt that fills the cache by itself
    one = model(prompt[:, :1].to(cuda), model.build_kv_cache(2), 0)
    _assert_logits_close(one, ref(prompt[:, :1], ref.build_kv_cache(2), 0), 4e-2, 4e-3)
    full = torch.randint(0, 256, (1, 48), generator=torch.Generator().manual_seed(3))
    _assert_logits_close(model(full.to(cuda)), ref(full), 4e-2, 4e-3)


def test_expired_barrier_wait_is_reported_and_does_not_hang(cuda):
    """Failure handling of the persistent kernel, forced from the host: with a spin limit of one
    every barrier wait expires, the kernel still runs to its end, the sticky error word is set and
    the session reports it; after re-initialising the workspace the same session synchronises
    normally again and a fresh session produces the tokens of an undisturbed run."""
    from ohara_amd.llama import Config, Llama

    kw = dict(vocab_size=512, hidden_size=256, intermediate_size=512, num_attention_heads=4, num_key_value_heads=2,
              num_hidden_layers=3, max_sequence_length=96, rope_theta=10000.0)
    w = R.init_weights(R.RefConfig(**kw), seed=3, dtype=torch.bfloat16, std=0.06, norm_jitter=0.1)
    model = Llama(Config(**kw), w, device=cuda)
    if not model.supports_persistent(2):
        pytest.skip("shape not covered by the persistent kernel")
    prompt = torch.randint(0, 512, (2, 12), generator=torch.Generator().manual_seed(0)).to(cuda)
    good = model.generate_greedy(prompt, 10, persistent=True).cpu()

    sess = model.session(2, 16, persistent=True)
    sess.prefill(prompt)
    sess.spin_limit = 1
    for _ in range(3):
        sess.step()
    torch.cuda.synchronize()
    with pytest.raises(RuntimeError, match="barrier wait expired"):
        sess.check_error()
    sess.spin_limit = 0
    sess.reset_error()
    sess.step()
    torch.cuda.synchronize()
    sess.check_error()
    again = model.generate_greedy(prompt, 10, persistent=True).cpu()
    assert torch.equal(again, good)


def test_device_loop_reports_an_expired_wait_with_the_chunk_and_refuses_reentry(cuda):
    """The engines' token source: (a) an expired barrier wait is raised with the chunk of ids that
    carries it, also for a consumer that stops early (a stop id) and never drains the generator, and
    the session is usable afterwards; (b) a second generation on the same loop while the first one's
    generator is still open is refused (one session, one cache)."""
    from ohara_amd.generation import DeviceLoop
    from ohara_amd.llama import Config, Llama

    kw = dict(vocab_size=512, hidden_size=256, intermediate_size=512, num_attention_heads=4, num_key_value_heads=2,
              num_hidden_layers=3, max_sequence_length=96, rope_theta=10000.0)
    w = R.init_weights(R.RefConfig(**kw), seed=3, dtype=torch.bfloat16, std=0.06, norm_jitter=0.1)
    model = Llama(Config(**kw), w, device=cuda)
    if not model.supports_persistent(1):
        pytest.skip("shape not covered by the persistent kernel")
    prompt = torch.randint(0, 512, (12,), generator=torch.Generator().manual_seed(0)).tolist()
    good = list(DeviceLoop(model).tokens(prompt, 24))
    assert len(good) == 24

    loop = DeviceLoop(model)
    sess = loop._get_session(None)
    assert sess.persistent
    sess.spin_limit = 1  # every barrier wait of the steps launched from here on expires
    with pytest.raises(RuntimeError, match="barrier wait expired"):
        for i, _ in enumerate(loop.tokens(prompt, 24)):
            if i == 6:  # a consumer that stops early
                break
    torch.cuda.synchronize()
    assert not loop._busy
    # the launches captured with that limit are dropped; the same session then decodes normally
    sess.spin_limit = 0
    sess.graph = sess.graph_multi = None
    assert list(loop.tokens(prompt, 24)) == good

    first = loop.tokens(prompt, 24)
    assert next(first) == good[0]
    second = loop.tokens(prompt, 24)
    with pytest.raises(RuntimeError, match="still generating"):
        next(second)
    first.close()
    assert list(loop.tokens(prompt, 8)) == good[:8]


@pytest.mark.parametrize("batch", [1, 3, 6, 7])
def test_persistent_workspace_need_not_be_zeroed(cuda, batch):
    """A C-ABI caller hands the single-launch kernel any device memory as its workspace: filled with
    0xFF bytes (NaN patterns in every fp32 slot) the tokens must equal those of a zeroed one - also at
    chunk counts that are not a power of two (batch 6 / 7), where the merge's loads reach slots that no
    workgroup writes."""
    from ohara_amd.llama import Config, Llama

    kw = dict(vocab_size=512, hidden_size=256, intermediate_size=512, num_attention_heads=4, num_key_value_heads=2,
              num_hidden_layers=3, max_sequence_length=160, rope_theta=10000.0)
    w = R.init_weights(R.RefConfig(**kw), seed=5, dtype=torch.bfloat16, std=0.06, norm_jitter=0.1)
    model = Llama(Config(**kw), w, device=cuda)
    prompt = torch.randint(0, 512, (batch, 70), generator=torch.Generator().manual_seed(batch)).to(cuda)
    good = model.generate_greedy(prompt, 12, persistent=True).cpu()
    sess = model.session(batch, 12, persistent=True)
    sess._pws = torch.full((64 << 20,), 0xFF, dtype=torch.uint8, device=cuda)  # larger than any workspace here
    sess.prefill(prompt)
    sess.run(11, use_graph=False)
    dirty = sess.tokens().cpu()
    assert torch.isfinite(sess.logits.float()).all()
    assert torch.equal(dirty, good)


def test_persistent_launch_refuses_more_workgroups_than_can_be_resident(cuda):
    """The grid barrier needs every workgroup resident at once: a launch with more workgroups than
    the device holds of this kernel (one per CU) is refused with OHARA_ESIZE before anything runs,
    instead of running into the barrier's spin limit."""
    import ctypes as C

    from ohara_amd._lib import lib
    from ohara_amd.llama import Config, Llama

    kw = dict(vocab_size=512, hidden_size=256, intermediate_size=512, num_attention_heads=4, num_key_value_heads=2,
              num_hidden_layers=2, max_sequence_length=64, rope_theta=10000.0)
    w = R.init_weights(R.RefConfig(**kw), seed=5, dtype=torch.bfloat16, std=0.06, norm_jitter=0.1)
    model = Llama(Config(**kw), w, device=cuda)
    if not model.supports_persistent(1):
        pytest.skip("shape not covered by the persistent kernel")
    sess = model.session(1, 8, persistent=True)
    sess.prefill(torch.randint(0, 512, (1, 6), generator=torch.Generator().manual_seed(0)).to(cuda))
    too_many = sess._nwg + 1
    need = lib().ohara_persistent_workspace_bytes(C.byref(model._c_model), 1, sess.PERSISTENT_SPLITS, too_many)
    ws = torch.zeros(max(need, 1), dtype=torch.uint8, device=cuda)
    stream = torch.cuda.current_stream().cuda_stream
    assert lib().ohara_llama_decode_persistent(C.byref(model._c_model), C.byref(sess._dst), ws.data_ptr(), too_many, 1, 1,
                                               0, stream) == 0  # workspace set-up alone launches nothing
    rc = lib().ohara_llama_decode_persistent(C.byref(model._c_model), C.byref(sess._dst), ws.data_ptr(), too_many, 0, 1,
                                             0, stream)
    assert rc == -3, rc
    torch.cuda.synchronize()
    sess.step()  # the session itself is untouched
    torch.cuda.synchronize()
    sess.check_error()


@pytest.mark.parametrize("B", [9, 17, 33, 70, 130])
def test_decode_batches_between_and_beyond_the_tuned_sizes(cuda, B):
    """Batches that are not multiples of 16, and more rows than one strip-kernel launch takes (64):
    prefill and three cached steps against the oracle on the same weights."""
    from ohara_amd.llama import Llama

    rcfg, cfg = _cfg_pair(vocab_size=512, hidden_size=256, intermediate_size=512, num_attention_heads=4,
                          num_key_value_heads=2, num_hidden_layers=2, max_sequence_length=64, rope_theta=10000.0)
    w = R.init_weights(rcfg, seed=2, dtype=BF, std=0.06, norm_jitter=0.1)
    ref, model = R.RefLlama(rcfg, w), Llama(cfg, w, device=cuda)
    g = torch.Generator().manual_seed(B)
    ids = torch.randint(0, 512, (B, 8), generator=g)
    rc, cache = ref.build_kv_cache(B), model.build_kv_cache(B)

    def close(got, want):
        got, want = got.float().cpu(), want.float()
        scale = want.abs().max().item()
        d = (got - want).abs()
        assert d.max().item() <= 4e-2 * scale and d.mean().item() <= 4e-3 * scale, (B, d.max().item(), d.mean().item(), scale)

    close(model(ids[:, :5].to(cuda), cache, 0), ref(ids[:, :5], rc, 0))
    for t in (5, 6, 7):
        close(model(ids[:, t:t + 1].to(cuda), cache, t), ref(ids[:, t:t + 1], rc, t))
    toks = model.generate_greedy(ids[:, :5].to(cuda), 3).cpu()
    want = greedy_decode_ref(ref, ids[:, :5], 3)
    # a near-tie of this random model flips a token now and then, and the sequence then differs from there on
    assert (toks == want).float().mean().item() >= 0.9


@pytest.mark.parametrize("heads,kv_heads,hidden", [(4, 4, 256), (8, 2, 512), (4, 2, 512), (4, 1, 512), (2, 2, 256)])
def test_every_persistent_kernel_variant_against_the_oracle(cuda, heads, kv_heads, hidden):
    """Head widths 64 / 128 with 1, 2 and 4 query heads per KV head: the single-launch decode step
    (free-running greedy tokens, then teacher-forced logits through the chain) against the oracle,
    and the single launch against the kernel chain token for token up to a near-tie."""
    from ohara_amd.llama import Llama

    rcfg, cfg = _cfg_pair(vocab_size=512, hidden_size=hidden, intermediate_size=512, num_attention_heads=heads,
                          num_key_value_heads=kv_heads, num_hidden_layers=3, max_sequence_length=128, rope_theta=10000.0)
    w = R.init_weights(rcfg, seed=heads * 10 + kv_heads, dtype=BF, std=0.05, norm_jitter=0.1)
    ref, model = R.RefLlama(rcfg, w), Llama(cfg, w, device=cuda)
    assert model.supports_persistent(3) and model.head_dim in (64, 128)
    prompt = torch.randint(0, 512, (3, 21), generator=torch.Generator().manual_seed(heads))
    want, want_logits = greedy_decode_ref(ref, prompt, 24, return_logits=True)
    for persistent in (True, False):
        got = model.generate_greedy(prompt.to(cuda), 24, persistent=persistent).cpu()
        for b in range(3):
            neq = (got[b] != want[b]).nonzero()
            if neq.numel():
                t = int(neq[0])
                assert _near_tie(want_logits[t, b], int(got[b, t]), int(want[b, t])), (persistent, b, t)


@pytest.mark.parametrize("B", [6, 7])
def test_persistent_kernel_with_chunk_counts_that_are_not_powers_of_two(cuda, B):
    """36 and 42 (sequence, KV head) pairs on 256 workgroups: the context of a pair is cut into 7 and 6
    chunks, which the merge takes as the next power of two with the rest weighing nothing.  Greedy tokens
    against the oracle (first divergence only at a near-tie) and against the kernel chain."""
    from ohara_amd.llama import Llama

    rcfg, cfg = _cfg_pair(vocab_size=512, hidden_size=384, intermediate_size=512, num_attention_heads=6,
                          num_key_value_heads=6, num_hidden_layers=2, max_sequence_length=160, rope_theta=10000.0)
    w = R.init_weights(rcfg, seed=13, dtype=BF, std=0.05, norm_jitter=0.1)
    ref, model = R.RefLlama(rcfg, w), Llama(cfg, w, device=cuda)
    assert model.supports_persistent(B)
    prompt = torch.randint(0, 512, (B, 100), generator=torch.Generator().manual_seed(B))
    want, want_logits = greedy_decode_ref(ref, prompt, 12, return_logits=True)
    got = model.generate_greedy(prompt.to(cuda), 12, persistent=True).cpu()
    chain = model.generate_greedy(prompt.to(cuda), 12, persistent=False).cpu()
    for other in (want, chain):
        for b in range(B):
            neq = (got[b] != other[b]).nonzero()
            if neq.numel():
                t = int(neq[0])
                assert _near_tie(want_logits[t, b], int(got[b, t]), int(other[b, t])), (b, t)


@pytest.mark.parametrize("B", [5, 12, 16])
def test_persistent_kernel_at_batches_up_to_its_limit(cuda, B):
    """The single launch is the default up to 8 sequences and can be asked for up to 16: greedy
    tokens against the oracle (first divergence only at a near-tie)."""
    from ohara_amd.llama import Llama

    rcfg, cfg = _cfg_pair(vocab_size=512, hidden_size=256, intermediate_size=512, num_attention_heads=4,
                          num_key_value_heads=2, num_hidden_layers=2, max_sequence_length=96, rope_theta=10000.0)
    w = R.init_weights(rcfg, seed=12, dtype=BF, std=0.05, norm_jitter=0.1)
    ref, model = R.RefLlama(rcfg, w), Llama(cfg, w, device=cuda)
    assert model.supports_persistent(B) and not model.supports_persistent(17)
    prompt = torch.randint(0, 512, (B, 30), generator=torch.Generator().manual_seed(B))
    want, want_logits = greedy_decode_ref(ref, prompt, 16, return_logits=True)
    got = model.generate_greedy(prompt.to(cuda), 16, persistent=True).cpu()
    for b in range(B):
        neq = (got[b] != want[b]).nonzero()
        if neq.numel():
            t = int(neq[0])
            assert _near_tie(want_logits[t, b], int(got[b, t]), int(want[b, t])), (b, t)
