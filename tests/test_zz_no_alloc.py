"""ohara_attn_cached_bf16_noalloc (the entry point for callers that cannot allocate device memory)
against ohara_attn_cached_bf16, through the C ABI.  Both run the same kernels over the same chunking,
so the outputs must be bit-identical.  Two calls in a row share the library's device array; the
second is smaller, so stale partials and counters of the first lie where it does not write."""

import pytest
import torch

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


def _case(cuda, seed, B, L, H, Hkv, D, T, ns):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, H * D, generator=g).to(BF).to(cuda)
    k = torch.randn(B, T, Hkv, D, generator=g).to(BF).to(cuda)
    v = torch.randn(B, T, Hkv, D, generator=g).to(BF).to(cuda)
    return q, k, v, (B, L, H, Hkv, D, T, ns)


def _both(q, k, v, shape):
    from ohara_amd import ops
    from ohara_amd._lib import check, lib

    B, L, H, Hkv, D, T, ns = shape
    ws = ops.attn_workspace(B, H, Hkv, D, ns, q.device)
    want = torch.empty(B, H * D, dtype=BF, device=q.device)
    got = torch.full_like(want, float("nan"))
    st = torch.cuda.current_stream().cuda_stream
    check(lib().ohara_attn_cached_bf16(q.data_ptr(), k.data_ptr(), v.data_ptr(), B, 1, H, Hkv, D, T, L - 1, 0, ns,
                                       ws.data_ptr(), want.data_ptr(), st), "attn_cached")
    check(lib().ohara_attn_cached_bf16_noalloc(q.data_ptr(), k.data_ptr(), v.data_ptr(), B, 1, H, Hkv, D, T, L - 1, 0,
                                               ns, got.data_ptr(), st), "attn_cached_noalloc")
    torch.cuda.synchronize()
    return got, want


def test_noalloc_attention_matches_workspace_version_twice(cuda):
    from ohara_amd._lib import ESIZE, lib

    big = _case(cuda, 1, 4, 3000, 8, 2, 128, 3072, 8)
    small = _case(cuda, 2, 2, 700, 8, 2, 128, 1024, 4)
    for q, k, v, shape in (big, small, big):
        before = torch.cuda.memory_allocated()
        got, want = _both(q, k, v, shape)
        assert torch.isfinite(want.float()).all()
        assert torch.equal(got, want), shape
        del got, want
        assert torch.cuda.memory_allocated() <= before + (1 << 26)  # only this test's own tensors
    # one chunk (no partials) and a head width served by the generic kernel
    for shape in ((3, 200, 4, 4, 64, 256, 1), (2, 500, 6, 3, 80, 512, 4)):
        q, k, v, shape = _case(cuda, 3, *shape)
        got, want = _both(q, k, v, shape)
        assert torch.equal(got, want), shape
    # beyond the array: rejected before anything is launched
    q, k, v, _ = small
    assert lib().ohara_attn_cached_bf16_noalloc(q.data_ptr(), k.data_ptr(), v.data_ptr(), 64, 1, 32, 8, 128, 1024,
                                                10, 0, 64, q.data_ptr(), 0) == ESIZE
    assert lib().ohara_attn_cached_bf16_noalloc(q.data_ptr(), k.data_ptr(), v.data_ptr(), 20000, 1, 1, 1, 128, 1024,
                                                10, 0, 1, q.data_ptr(), 0) == ESIZE
