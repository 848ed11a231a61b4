"""Fused sampler (C ABI: ohara_sample_topk_topp / ohara_argmax_bf16) against the CPU oracle
and the known answers of the reference's own tests (tests/test_inference.py:45-48,
tests/test_chat.py:355-390).

Stochastic parity: both sides consume the same uniform draw u by inverse CDF over the same
distribution.  The kernel sums the sorted probabilities sequentially in fp32 (as
torch.cumsum does), the oracle's reference CDF is fp64, so the check is: u lies inside the
CDF interval of the token the kernel returned, widened by 5e-5 (fp32 summation error over
up to 65536 terms, which also moves the nucleus boundary by a few tail tokens), and the token is identical to the oracle's wherever u is further than
that from an interval boundary.
"""

import pytest
import torch

from oracle.sampling_ref import candidate_cdf_ref, inference_sampler_ref, kept_set_ref, sample_next_token_ref

pytestmark = pytest.mark.gpu


def test_reference_known_answers(cuda):
    from ohara_amd.sampling import SamplingConfig, inference_sampler, sample_next_token

    t = sample_next_token(torch.tensor([[[0.1, 5.0, 0.2, 0.3]]]).to(cuda), SamplingConfig(temperature=0.0))
    assert int(t.item()) == 1 and t.shape == (1, 1) and t.dtype == torch.int64
    t = inference_sampler(torch.tensor([[[0.1, 0.2, 0.9]]]).to(cuda), temperature=0.0)
    assert int(t.item()) == 2
    # default Inference sampler (temperature 1, top_p 0) is greedy
    assert int(inference_sampler(torch.tensor([[[0.1, 0.2, 0.9]]]).to(cuda)).item()) == 2
    # top-k = 2 never leaks outside {0, 1}
    logits = torch.tensor([[[10.0, 9.0, -50.0, -60.0]]]).to(cuda)
    cfg = SamplingConfig(temperature=1.0, top_p=1.0, top_k=2)
    seen = {int(sample_next_token(logits, cfg).item()) for _ in range(200)}
    assert seen <= {0, 1} and len(seen) == 2
    # a tiny top_p still keeps the most likely token
    logits = torch.tensor([[[20.0, 0.0, 0.0, 0.0]]]).to(cuda)
    cfg = SamplingConfig(temperature=1.0, top_p=0.01)
    assert {int(sample_next_token(logits, cfg).item()) for _ in range(50)} == {0}
    # seeded sampling is reproducible
    logits = torch.randn(1, 1, 32).to(cuda)
    cfg = SamplingConfig(temperature=1.0, top_p=0.9)
    a = sample_next_token(logits, cfg, torch.Generator(device=cuda).manual_seed(7))
    b = sample_next_token(logits, cfg, torch.Generator(device=cuda).manual_seed(7))
    assert int(a.item()) == int(b.item())
    # CPU logits and a CPU generator are accepted too (the result comes back on the CPU)
    c = sample_next_token(logits.cpu(), cfg, torch.Generator().manual_seed(7))
    assert c.device.type == "cpu"
    for kw in ({"temperature": -1.0}, {"top_p": 1.5}, {"top_k": -1}, {"max_new_tokens": 0}):
        with pytest.raises(ValueError):
            SamplingConfig(**kw)


CASES = [
    # V, B, temperature, top_k, top_p, logit std, dtype
    (32, 8, 1.0, 0, 0.9, 1.0, torch.float32),
    (1000, 16, 0.8, 50, 0.9, 2.0, torch.bfloat16),
    (1000, 16, 1.3, 0, 1.0, 2.0, torch.float32),
    (1000, 16, 0.7, 7, 0.0, 2.0, torch.bfloat16),
    (65536, 8, 0.8, 50, 0.9, 0.55, torch.bfloat16),    # the headline sampling setting
    (65536, 4, 1.0, 0, 0.95, 3.0, torch.bfloat16),     # peaked, nucleus only
    (65536, 6, 0.8, 0, 0.95, 8.0, torch.bfloat16),     # the reference's chat defaults on a sharp row: a few candidates
    (65536, 6, 1.0, 0, 0.5, 5.0, torch.bfloat16),      # nucleus closes inside the sorted candidates
    (32000, 6, 0.7, 0, 0.9, 6.0, torch.bfloat16),
    (65536, 4, 1.0, 0, 0.999, 8.0, torch.bfloat16),    # candidates run out: falls back to the general path
    (65536, 3, 1.0, 0, 0.9, 0.5, torch.bfloat16),      # flat: tens of thousands kept (multi-round path)
    (65536, 3, 1.0, 5000, 0.5, 0.5, torch.float32),
    (65536, 3, 1.0, 5000, 0.5, 0.5, torch.bfloat16),   # top-k beyond the sorted block + nucleus: the count table
    (65536, 3, 0.9, 3000, 1.0, 1.0, torch.bfloat16),   # the same without a nucleus: vocabulary-order draw above a threshold
    (40000, 3, 1.2, 2000, 0.0, 2.0, torch.bfloat16),
    (32000, 4, 0.8, 0, 0.0, 1.0, torch.bfloat16),      # vocabulary-order draw
    (50, 5, 1.0, 100, 0.3, 1.0, torch.float32),        # top_k larger than the vocabulary
]


@pytest.mark.parametrize("V,B,T,k,p,std,dtype", CASES)
def test_sampler_matches_oracle(cuda, V, B, T, k, p, std, dtype):
    from ohara_amd import ops

    g = torch.Generator().manual_seed(V + B + k)
    logits = (torch.randn(B, V, generator=g) * std).to(dtype)
    tol = 5e-5
    for trial in range(4):
        u = torch.rand(B, generator=g)
        if trial == 0:
            u[0] = 0.0
            u[-1] = 0.999999
        want, margin = sample_next_token_ref(logits.unsqueeze(1), T, p, k, u=u, return_margin=True)
        ids, cdf = candidate_cdf_ref(logits.unsqueeze(1), T, p, k)
        got = ops.sample_topk_topp(logits.to(cuda), T, k, p, u.to(cuda)).cpu()
        for b in range(B):
            j = int((ids[b] == int(got[b])).nonzero()[0])
            lo = float(cdf[b, j - 1]) if j > 0 else 0.0
            hi = float(cdf[b, j])
            assert hi > lo, (b, "sampled a token outside the kept set")
            assert lo - tol <= float(u[b]) <= hi + tol, (b, int(got[b]), lo, hi, float(u[b]))
            if float(margin[b]) > tol:
                assert int(got[b]) == int(want[b, 0]), (b, int(got[b]), int(want[b, 0]), float(margin[b]))


def test_sampler_valid_vocab_and_ties(cuda):
    from ohara_amd import ops

    g = torch.Generator().manual_seed(9)
    V, B = 4096, 6
    logits = torch.randn(B, V, generator=g).to(torch.bfloat16)  # bf16: many exactly equal values
    logits[:, 3000:] += 8.0                                     # the padded region would dominate
    u = torch.rand(B, generator=g)
    want = sample_next_token_ref(logits.unsqueeze(1), 0.9, 0.92, 40, u=u, valid_vocab=3000)
    got = ops.sample_topk_topp(logits.to(cuda), 0.9, 40, 0.92, u.to(cuda), valid_vocab=3000).cpu()
    assert torch.equal(got, want[:, 0]) and int(got.max()) < 3000
    # the kept set of the direct fp64 restatement contains every sampled id
    for b in range(B):
        kept, _ = kept_set_ref(logits[b, :3000], 0.9, 0.92, 40)
        assert int(got[b]) in kept
    # exact ties: four equal maxima, top_k = 1 keeps all four; u picks among them in id order
    row = torch.full((1, 64), -3.0)
    row[0, [5, 17, 33, 60]] = 2.0
    for uu, expect in ((0.0, 5), (0.26, 17), (0.51, 33), (0.99, 60)):
        got = ops.sample_topk_topp(row.to(cuda), 1.0, 1, 1.0, torch.tensor([uu], device=cuda))
        assert int(got.item()) == expect
        got = ops.sample_topk_topp(row.to(cuda), 1.0, 1, 0.999, torch.tensor([uu], device=cuda))
        assert int(got.item()) == expect


def test_inference_sampler_matches_oracle(cuda):
    from ohara_amd.sampling import inference_sampler

    g = torch.Generator().manual_seed(4)
    logits = torch.randn(5, 3, 777, generator=g) * 2
    u = torch.rand(5, generator=g)
    want = inference_sampler_ref(logits, temperature=0.7, top_p=0.8, u=u)
    got = inference_sampler(logits.to(cuda), temperature=0.7, top_p=0.8, u=u).cpu()
    assert torch.equal(got, want)
    want = inference_sampler_ref(logits, temperature=0.7, top_p=0.0, u=u)
    got = inference_sampler(logits.to(cuda), temperature=0.7, top_p=0.0, u=u).cpu()
    assert torch.equal(got, want)


def test_nucleus_alone_on_rows_with_many_ties(cuda):
    """Top-p without top-k on bf16 rows built from a handful of levels (whole blocks of equal
    probabilities), with and without a padded vocabulary tail: ties are taken lowest id first, the
    nucleus may end inside a block of ties, and the candidate route and the general route must agree
    with the oracle."""
    from ohara_amd import ops

    g = torch.Generator().manual_seed(21)
    V, B = 65536, 6
    levels = torch.tensor([0.0, 2.0, 4.0, 9.0, 12.0])
    pick = torch.multinomial(torch.tensor([0.9, 0.07, 0.02, 0.009, 0.001]), B * V, replacement=True, generator=g)
    logits = levels[pick].view(B, V).to(torch.bfloat16)
    tol = 5e-5
    for T, p, valid in ((1.0, 0.6, None), (0.8, 0.95, None), (1.0, 0.3, 60000), (1.3, 0.05, None)):
        for trial in range(3):
            u = torch.rand(B, generator=g)
            want, margin = sample_next_token_ref(logits.unsqueeze(1), T, p, 0, u=u, valid_vocab=valid, return_margin=True)
            got = ops.sample_topk_topp(logits.to(cuda), T, 0, p, u.to(cuda), valid_vocab=valid).cpu()
            for b in range(B):
                if float(margin[b]) > tol:
                    assert int(got[b]) == int(want[b, 0]), (T, p, valid, b, int(got[b]), int(want[b, 0]), float(margin[b]))
                if valid is not None:
                    assert int(got[b]) < valid


def test_rows_of_one_single_value(cuda):
    """Every id has the same logit (the one case in which a 16-bit count of the table-based sampler
    could overflow): uniform probabilities, the nucleus keeps the first floor(top_p * V) + 1 ids, ties
    are taken lowest id first, so the draw u lands on id floor(u * kept)."""
    from ohara_amd import ops

    for V in (65536, 50000):
        row = torch.full((2, V), 1.5, dtype=torch.bfloat16, device=cuda)
        u = torch.tensor([0.25, 0.9], device=cuda)
        got = ops.sample_topk_topp(row, 0.8, 0, 0.5, u).cpu()
        kept = int(0.5 * V) + 1
        for b in range(2):
            assert abs(int(got[b]) - int(float(u[b]) * kept)) <= 2, (V, b, int(got[b]))
        got = ops.sample_topk_topp(row, 1.0, 0, 1.0, u).cpu()  # plain multinomial: vocabulary order
        for b in range(2):
            assert abs(int(got[b]) - int(float(u[b]) * V)) <= 2, (V, b, int(got[b]))
        got = ops.sample_topk_topp(row, 1.0, 2000, 1.0, u).cpu()  # top-k keeps every tie
        for b in range(2):
            assert abs(int(got[b]) - int(float(u[b]) * V)) <= 2, (V, b, int(got[b]))


@pytest.mark.parametrize("V,B,T,k,p,std", [(65536, 8, 0.8, 50, 0.9, 0.55), (65536, 3, 1.0, 1, 1.0, 1.0),
                                           (32000, 5, 0.7, 64, 0.0, 2.0), (50000, 2, 1.2, 40, 0.95, 6.0)])
def test_small_top_k_over_several_workgroups(cuda, V, B, T, k, p, std):
    """ohara_sample_topk_topp_exclusive spreads a small top-k on a long bf16 row over one workgroup per
    8192 ids: the same token as the single-workgroup kernel for the same draw, on calls in a row (the
    arrival counters return to zero), with a masked vocabulary tail, and inside the oracle's CDF interval."""
    from ohara_amd import ops

    g = torch.Generator().manual_seed(V + B + k)
    logits = (torch.randn(B, V, generator=g) * std).to(torch.bfloat16)
    dl = logits.to(cuda)
    tol = 5e-5
    for trial in range(5):
        u = torch.rand(B, generator=g)
        if trial == 0:
            u[0] = 0.0
            u[-1] = 0.999999
        valid = None if trial < 3 else V - 5000
        one = ops.sample_topk_topp(dl, T, k, p, u.to(cuda), valid).cpu()
        many = ops.sample_topk_topp(dl, T, k, p, u.to(cuda), valid, exclusive=True).cpu()
        assert torch.equal(one, many), (trial, one, many)
        if valid is None:
            ids, cdf = candidate_cdf_ref(logits.unsqueeze(1), T, p, k)
            for b in range(B):
                j = int((ids[b] == int(many[b])).nonzero()[0])
                lo = float(cdf[b, j - 1]) if j > 0 else 0.0
                assert lo - tol <= float(u[b]) <= float(cdf[b, j]) + tol
    # ties: rows of few distinct values (more than 128 candidates in a part: the last workgroup walks the
    # whole row itself), and a row whose largest values all sit in one part
    tied = (torch.randint(0, 3, (B, V), generator=g).float() * 2).to(torch.bfloat16)
    one_part = logits.clone()
    one_part[:, 9000:9100] += 12.0
    for rows in (tied, one_part):
        u = torch.rand(B, generator=g)
        one = ops.sample_topk_topp(rows.to(cuda), T, k, p, u.to(cuda)).cpu()
        many = ops.sample_topk_topp(rows.to(cuda), T, k, p, u.to(cuda), exclusive=True).cpu()
        assert torch.equal(one, many)
    # the device-side bookkeeping (history, step counter, draws indexed by step)
    steps = 3
    us = torch.rand(steps, B, generator=g).to(cuda)
    for excl in (False, True):
        state = torch.tensor([7, 0, 0, 0], dtype=torch.int32, device=cuda)
        hist = torch.zeros(steps, B, dtype=torch.int64, device=cuda)
        out = torch.zeros(B, dtype=torch.int64, device=cuda)
        for _ in range(steps):
            ops.sample_topk_topp(dl, T, k, p, us, out=out, history=hist, step_state=state, u_per_step=True, exclusive=excl)
        if excl:
            assert torch.equal(hist, first_hist) and state.tolist() == [7 + steps, steps, 0, 0]
        first_hist = hist.clone()


def test_sampler_with_the_callers_workspace(cuda):
    """ohara_sample_topk_topp_ws: the spread selection meeting in a caller-owned workspace gives the
    single-workgroup kernel's tokens, on calls in a row and on two streams that each bring their own
    workspace (what two sampling decode sessions do); a short or misaligned workspace is refused."""
    from ohara_amd import ops

    V, B, T, k, p = 65536, 8, 0.8, 50, 0.9
    g = torch.Generator().manual_seed(17)
    rows = [(torch.randn(B, V, generator=g) * 0.55).to(torch.bfloat16).to(cuda) for _ in range(2)]
    us = [torch.rand(6, B, generator=g).to(cuda) for _ in range(2)]
    want = [[ops.sample_topk_topp(rows[i], T, k, p, us[i][j]).cpu() for j in range(6)] for i in range(2)]
    ws = [ops.sample_workspace(cuda) for _ in range(2)]
    for j in range(3):  # one stream, calls in a row: the counters return to zero
        assert torch.equal(ops.sample_topk_topp(rows[0], T, k, p, us[0][j], workspace=ws[0]).cpu(), want[0][j])
    streams = [torch.cuda.Stream() for _ in range(2)]
    outs = [[torch.empty(B, dtype=torch.int64, device=cuda) for _ in range(6)] for _ in range(2)]
    torch.cuda.synchronize()
    for j in range(6):
        for i in range(2):
            with torch.cuda.stream(streams[i]):
                ops.sample_topk_topp(rows[i], T, k, p, us[i][j], out=outs[i][j], workspace=ws[i])
    torch.cuda.synchronize()
    for i in range(2):
        for j in range(6):
            assert torch.equal(outs[i][j].cpu(), want[i][j]), (i, j)
    with pytest.raises(Exception):
        ops.sample_topk_topp(rows[0], T, k, p, us[0][0], workspace=ws[0][: ws[0].numel() // 2])
    with pytest.raises(Exception):
        ops.sample_topk_topp(rows[0], T, k, p, us[0][0], workspace=torch.zeros(ws[0].numel() + 64, dtype=torch.uint8, device=cuda)[8:])
