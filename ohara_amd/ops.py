"""Tensor-level wrappers over the C ABI (one Python function per entry point).

PyTorch is used for device memory and the current stream only; every function here
hands raw pointers to libohara_decode.so.
"""

from __future__ import annotations

import ctypes as C

import torch

from . import _lib
from ._lib import check, lib

BF16 = torch.bfloat16


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ptr(t):
    return 0 if t is None else t.data_ptr()


def _need(t: torch.Tensor, dtype, name: str):
    if not t.is_cuda:
        raise ValueError(f"{name} must be a device tensor")
    if t.dtype != dtype:
        raise ValueError(f"{name} must be {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")


class PackedLinear:
    """A Linear weight (N, K) in the kernels' strip/kstep/lane tile order."""

    __slots__ = ("data", "n", "k", "kind")

    def __init__(self, data, n, k, kind="rows"):
        self.data, self.n, self.k, self.kind = data, n, k, kind


def pack_rows(w: torch.Tensor, perm: torch.Tensor | None = None, n_padded: int | None = None) -> torch.Tensor:
    """Pack a (N, K) bf16 matrix; ``perm`` (int32, device) maps packed row -> source row."""
    _need(w, BF16, "w")
    n, k = w.shape
    if n_padded is None:
        n_padded = (n + 15) // 16 * 16
    nbytes = C.c_int64(0)
    check(lib().ohara_pack_rows_bf16(0, n, k, k, 0, n_padded, 0, C.byref(nbytes), 0), "pack size")
    dst = torch.empty(nbytes.value // 2, dtype=BF16, device=w.device)
    check(lib().ohara_pack_rows_bf16(_ptr(w), n, k, k, _ptr(perm), n_padded, _ptr(dst), None, _stream()), "pack")
    return dst


def pack_linear(w: torch.Tensor) -> PackedLinear:
    return PackedLinear(pack_rows(w), w.shape[0], w.shape[1])


def swiglu_perm(f: int, device) -> torch.Tensor:
    fp = (f + 7) // 8 * 8
    buf = (C.c_int32 * (2 * fp))()
    check(lib().ohara_swiglu_perm(f, buf), "swiglu_perm")
    return torch.tensor(list(buf), dtype=torch.int32, device=device)


def pack_gate_up(w_gate: torch.Tensor, w_up: torch.Tensor) -> PackedLinear:
    """Interleave gate/up rows so the SwiGLU epilogue finds a gate/up pair in one lane."""
    f, k = w_gate.shape
    cat = torch.cat([w_gate, w_up], dim=0).contiguous()
    perm = swiglu_perm(f, w_gate.device)
    return PackedLinear(pack_rows(cat, perm, perm.numel()), f, k, kind="swiglu")


def pack_qkv(wq, wk, wv) -> PackedLinear:
    cat = torch.cat([wq, wk, wv], dim=0).contiguous()
    return PackedLinear(pack_rows(cat), cat.shape[0], cat.shape[1], kind="qkv")


def embed(ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    _need(table, BF16, "table")
    ids = ids.reshape(-1).contiguous()
    n, d = ids.numel(), table.shape[1]
    if out is None:
        out = torch.empty(n, d, dtype=BF16, device=table.device)
    check(lib().ohara_embed_bf16(_ptr(ids), _ptr(table), _ptr(out), n, d, table.shape[0], _stream()), "embed")
    return out


def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float = 1e-5, out=None) -> torch.Tensor:
    _need(x, BF16, "x")
    d = x.shape[-1]
    rows = x.numel() // d
    if out is None:
        out = torch.empty_like(x)
    check(lib().ohara_rmsnorm_bf16(_ptr(x), _ptr(w), _ptr(out), rows, d, eps, _stream()), "rmsnorm")
    return out


def gemm_skinny(x, w: PackedLinear, norm_w=None, eps=1e-5, residual=None, out=None) -> torch.Tensor:
    """y = [rmsnorm(x)] @ W^T (+ residual / SwiGLU epilogue by the packing kind). x: (B, K)."""
    _need(x, BF16, "x")
    b, k = x.shape
    if k != w.k:
        raise ValueError(f"x has {k} columns, weight expects {w.k}")
    if out is None:
        out = torch.empty(b, w.n, dtype=BF16, device=x.device)
    if w.kind == "swiglu":
        epi = _lib.EPI_SWIGLU
    elif residual is not None:
        epi = _lib.EPI_RESIDUAL
    else:
        epi = _lib.EPI_STORE
    check(
        lib().ohara_gemm_skinny_bf16(
            _ptr(x), x.stride(0), _ptr(w.data), w.n, w.k, _ptr(norm_w), eps, b, epi,
            _ptr(residual), 0 if residual is None else residual.stride(0), _ptr(out), out.stride(0), _stream(),
        ),
        "gemm_skinny",
    )
    return out


def gemm(x, w: PackedLinear, residual=None, out=None) -> torch.Tensor:
    """y = x @ W^T (+ residual / SwiGLU epilogue by the packing kind) on the tiled MFMA kernel,
    for any number of rows.  x: (rows, K), rows may be strided (a column slice of a wider buffer)."""
    if not x.is_cuda or x.dtype != BF16 or x.ndim != 2 or x.stride(1) != 1:
        raise ValueError("x must be a 2-D bfloat16 device tensor with unit column stride")
    rows, k = x.shape
    if k != w.k:
        raise ValueError(f"x has {k} columns, weight expects {w.k}")
    if out is None:
        out = torch.empty(rows, w.n, dtype=BF16, device=x.device)
    epi = _lib.EPI_SWIGLU if w.kind == "swiglu" else (_lib.EPI_RESIDUAL if residual is not None else _lib.EPI_STORE)
    check(
        lib().ohara_gemm_bf16(
            _ptr(x), x.stride(0), _ptr(w.data), w.n, w.k, rows, epi,
            _ptr(residual), 0 if residual is None else residual.stride(0), _ptr(out), out.stride(0), _stream(),
        ),
        "gemm",
    )
    return out


def qkv_rope_append(x, wqkv: PackedLinear, norm_w, eps, h, h_kv, dh, cos, sin, pos, kcache, vcache,
                    q_out=None, pos_dev=None, seq_len=1, seq_pos=None):
    """x: (batch*seq_len, K) rows ordered (sequence, position).  ``seq_pos`` (int32, one entry per
    sequence, on the device) gives every sequence its own cache position instead of ``pos``."""
    _need(x, BF16, "x")
    rows = x.shape[0]
    b = rows // seq_len
    if q_out is None:
        q_out = torch.empty(rows, h * dh, dtype=BF16, device=x.device)
    t_max = kcache.shape[1]
    if seq_pos is not None:
        _need(seq_pos, torch.int32, "seq_pos")
        check(
            lib().ohara_qkv_rope_append_ragged_bf16(
                _ptr(x), x.stride(0), _ptr(wqkv.data), wqkv.k, _ptr(norm_w), eps, b, seq_len, h, h_kv, dh, _ptr(cos),
                _ptr(sin), _ptr(seq_pos), _ptr(q_out), _ptr(kcache), _ptr(vcache), t_max, _stream(),
            ),
            "qkv_rope_append_ragged",
        )
        return q_out
    check(
        lib().ohara_qkv_rope_append_bf16(
            _ptr(x), x.stride(0), _ptr(wqkv.data), wqkv.k, _ptr(norm_w), eps, b, seq_len, h, h_kv, dh, _ptr(cos), _ptr(sin),
            int(pos), _ptr(pos_dev), _ptr(q_out), _ptr(kcache), _ptr(vcache), t_max, _stream(),
        ),
        "qkv_rope_append",
    )
    return q_out


def qkv_rope(x, wqkv: PackedLinear, norm_w, eps, h, h_kv, dh, cos, sin, pos, t_max, pos_dev=None, seq_len=1):
    """As ``qkv_rope_append`` with the rotated keys and the values returned as (rows, h_kv*dh) row
    buffers instead of written into a cache -> (q, k, v)."""
    _need(x, BF16, "x")
    rows = x.shape[0]
    q = torch.empty(rows, h * dh, dtype=BF16, device=x.device)
    k = torch.empty(rows, h_kv * dh, dtype=BF16, device=x.device)
    v = torch.empty(rows, h_kv * dh, dtype=BF16, device=x.device)
    check(
        lib().ohara_qkv_rope_bf16(
            _ptr(x), x.stride(0), _ptr(wqkv.data), wqkv.k, _ptr(norm_w), eps, rows // seq_len, seq_len, h, h_kv, dh,
            _ptr(cos), _ptr(sin), int(pos), _ptr(pos_dev), t_max, _ptr(q), _ptr(k), _ptr(v), _stream(),
        ),
        "qkv_rope",
    )
    return q, k, v


def attn_workspace(batch, h, h_kv, dh, n_split, device) -> torch.Tensor:
    n = lib().ohara_attn_workspace_bytes(batch, h, h_kv, dh, n_split)
    if n < 0:
        raise ValueError("bad attention workspace shape")
    return torch.zeros(n, dtype=torch.uint8, device=device)


def attn_cached(q, kcache, vcache, h, h_kv, dh, pos, n_split, workspace, out=None, pos_dev=None, seq_len=1,
                seq_pos=None):
    """q: (batch*seq_len, h*dh); query s of a sequence sits at cache position pos + s (or at
    seq_pos[sequence] + s when the int32 device tensor ``seq_pos`` is given)."""
    rows = q.shape[0]
    if out is None:
        out = torch.empty(rows, h * dh, dtype=BF16, device=q.device)
    if seq_pos is not None:
        _need(seq_pos, torch.int32, "seq_pos")
        check(
            lib().ohara_attn_cached_ragged_bf16(
                _ptr(q), _ptr(kcache), _ptr(vcache), rows // seq_len, seq_len, h, h_kv, dh, kcache.shape[1],
                _ptr(seq_pos), n_split, _ptr(workspace), _ptr(out), _stream(),
            ),
            "attn_cached_ragged",
        )
        return out
    check(
        lib().ohara_attn_cached_bf16(
            _ptr(q), _ptr(kcache), _ptr(vcache), rows // seq_len, seq_len, h, h_kv, dh, kcache.shape[1], int(pos),
            _ptr(pos_dev), n_split, _ptr(workspace), _ptr(out), _stream(),
        ),
        "attn_cached",
    )
    return out


def attn_prefill(q, kcache, vcache, h, h_kv, dh, pos, seq_len, out=None):
    """q: (batch*seq_len, h*dh); causal attention of seq_len queries per sequence over cache
    positions [0, pos + s] on the MFMA prefill kernel."""
    _need(q, BF16, "q")
    rows = q.shape[0]
    if out is None:
        out = torch.empty(rows, h * dh, dtype=BF16, device=q.device)
    check(
        lib().ohara_attn_prefill_bf16(
            _ptr(q), _ptr(kcache), _ptr(vcache), rows // seq_len, seq_len, h, h_kv, dh, kcache.shape[1], int(pos),
            _ptr(out), _stream(),
        ),
        "attn_prefill",
    )
    return out


def attn_auto(q, kcache, vcache, h, h_kv, dh, pos, n_split, workspace, seq_len, out=None):
    """The MFMA prefill kernel for calls with many positions per sequence, else the decode kernel."""
    if seq_len >= 16 and dh in (64, 128):
        return attn_prefill(q, kcache, vcache, h, h_kv, dh, pos, seq_len, out)
    return attn_cached(q, kcache, vcache, h, h_kv, dh, pos, n_split if seq_len == 1 else 1, workspace, out, None, seq_len)


def kv_quant_append(keys, values, cache, pos, pos_dev=None, seq_pos=None):
    """keys / values (B, S, Hkv, D) bf16 -> quantised into an int8 ``KVCache`` at positions pos + s
    (``seq_pos``: one position per sequence, an int32 device tensor)."""
    _need(keys, BF16, "keys")
    _need(values, BF16, "values")
    b, s_len, hkv, d = keys.shape
    if seq_pos is not None:
        _need(seq_pos, torch.int32, "seq_pos")
        check(lib().ohara_kv_quant_append_ragged_int8(
            _ptr(keys), _ptr(values), b, s_len, hkv, d, _ptr(seq_pos), _ptr(cache.key), _ptr(cache.value), _ptr(cache.stats),
            cache.key.shape[1], _stream()), "kv_quant_append_ragged")
        return
    check(lib().ohara_kv_quant_append_int8(
        _ptr(keys), _ptr(values), b, s_len, hkv, d, int(pos), _ptr(pos_dev), _ptr(cache.key), _ptr(cache.value),
        _ptr(cache.stats), cache.key.shape[1], _stream()), "kv_quant_append")


def kv_dequant(cache, which: str, batch: int, length: int, out=None) -> torch.Tensor:
    """The first `length` positions of the int8 cache's key or value tensor as bf16 (B, length, Hkv, D)."""
    q = cache.key if which == "key" else cache.value
    _, t_max, hkv, d = q.shape
    if out is None:
        out = torch.empty(batch, length, hkv, d, dtype=BF16, device=q.device)
    check(lib().ohara_kv_dequant_int8(_ptr(q), _ptr(cache.stats), 0 if which == "key" else 1, batch, length, hkv, d, t_max,
                                      _ptr(out), _stream()), "kv_dequant")
    return out


def attn_cached_int8(q, cache, h, h_kv, dh, pos, n_split, workspace, out=None, pos_dev=None, seq_len=1, seq_pos=None):
    """attn_cached over an int8 ``KVCache`` (``seq_pos``: one position per sequence, an int32 device tensor)."""
    rows = q.shape[0]
    if out is None:
        out = torch.empty(rows, h * dh, dtype=BF16, device=q.device)
    if seq_pos is not None:
        _need(seq_pos, torch.int32, "seq_pos")
        check(lib().ohara_attn_cached_ragged_int8(
            _ptr(q), _ptr(cache.key), _ptr(cache.value), _ptr(cache.stats), rows // seq_len, seq_len, h, h_kv, dh,
            cache.key.shape[1], _ptr(seq_pos), n_split, _ptr(workspace), _ptr(out), _stream()), "attn_cached_ragged_int8")
        return out
    check(lib().ohara_attn_cached_int8(
        _ptr(q), _ptr(cache.key), _ptr(cache.value), _ptr(cache.stats), rows // seq_len, seq_len, h, h_kv, dh,
        cache.key.shape[1], int(pos), _ptr(pos_dev), n_split, _ptr(workspace), _ptr(out), _stream()), "attn_cached_int8")
    return out


def attn_decode(q, kcache, vcache, h, h_kv, dh, length, n_split, workspace, out=None, pos_dev=None):
    """Decode case: one query per sequence seeing `length` cached positions."""
    return attn_cached(q, kcache, vcache, h, h_kv, dh, length - 1, n_split, workspace, out, pos_dev, 1)


def advance_positions(seq_pos: torch.Tensor, active: torch.Tensor | None = None, by: int = 1) -> None:
    """seq_pos[b] += by where active[b] (uint8) is non-zero; all entries when ``active`` is None."""
    _need(seq_pos, torch.int32, "seq_pos")
    if active is not None:
        _need(active, torch.uint8, "active")
    check(lib().ohara_advance_positions(_ptr(seq_pos), _ptr(active), seq_pos.numel(), by, _stream()), "advance_positions")


def advance_ragged(seq_pos: torch.Tensor, active: torch.Tensor | None, new_ids: torch.Tensor, next_ids: torch.Tensor,
                   by: int = 1) -> None:
    """``advance_positions`` and, in the same launch, next_ids[b] = new_ids[b] where active[b], else 0."""
    _need(seq_pos, torch.int32, "seq_pos")
    _need(new_ids, torch.int64, "new_ids")
    _need(next_ids, torch.int64, "next_ids")
    if active is not None:
        _need(active, torch.uint8, "active")
    if new_ids.numel() != seq_pos.numel() or next_ids.numel() != seq_pos.numel():
        raise ValueError("one id per sequence is required")
    check(lib().ohara_advance_ragged(_ptr(seq_pos), _ptr(active), _ptr(new_ids), _ptr(next_ids), seq_pos.numel(), by,
                                     _stream()), "advance_ragged")


def argmax(logits: torch.Tensor, valid_vocab: int | None = None, next_ids=None, history=None, step_state=None):
    _need(logits, BF16, "logits")
    b, v = logits.shape
    if next_ids is None:
        next_ids = torch.empty(b, dtype=torch.int64, device=logits.device)
    check(
        lib().ohara_argmax_bf16(
            _ptr(logits), logits.stride(0), b, v, v if valid_vocab is None else valid_vocab, _ptr(next_ids),
            _ptr(history), 0 if history is None else history.shape[0], _ptr(step_state), _stream(),
        ),
        "argmax",
    )
    return next_ids


def sample_topk_topp(logits: torch.Tensor, temperature: float, top_k: int, top_p: float, u: torch.Tensor,
                     valid_vocab: int | None = None, out=None, history=None, step_state=None,
                     u_per_step: bool = False, exclusive: bool = False, workspace=None) -> torch.Tensor:
    """logits (B, V) bf16 or fp32 on the device, u (B,) fp32 uniform draws -> ids (B,) int64.
    With ``u_per_step`` (needs step_state) u is (steps, B) and row ``step`` is read on the device.
    ``exclusive``: the caller's sampler calls on this GPU do not overlap in time (a decode loop on one
    stream), which lets a small top-k on a long row run on several workgroups (same results).
    ``workspace`` (``sample_workspace``): the same with the workgroups meeting in the caller's buffer instead of
    the library's, so that callers with a workspace each may overlap (one per decode session)."""
    if logits.dtype not in (BF16, torch.float32):
        raise ValueError("logits must be bfloat16 or float32")
    _need(logits, logits.dtype, "logits")
    _need(u, torch.float32, "u")
    b, v = logits.shape
    if u_per_step:
        if step_state is None or u.ndim != 2 or u.shape[1] != b:
            raise ValueError("u_per_step needs step_state and a (steps, batch) tensor of draws")
    elif u.numel() != b:
        raise ValueError("one uniform draw per row is required")
    if out is None:
        out = torch.empty(b, dtype=torch.int64, device=logits.device)
    args = (_ptr(logits), 1 if logits.dtype == torch.float32 else 0, logits.stride(0), b, v,
            v if valid_vocab is None else valid_vocab, float(temperature), int(top_k), float(top_p), _ptr(u),
            b if u_per_step else 0, _ptr(out), _ptr(history), 0 if history is None else history.shape[0], _ptr(step_state))
    if workspace is not None:
        _need(workspace, torch.uint8, "workspace")
        check(lib().ohara_sample_topk_topp_ws(*args, _ptr(workspace), workspace.numel(), _stream()), "sample_topk_topp")
        return out
    check((lib().ohara_sample_topk_topp_exclusive if exclusive else lib().ohara_sample_topk_topp)(*args, _stream()),
          "sample_topk_topp")
    return out


def sample_workspace(device) -> torch.Tensor:
    """A zeroed workspace for ``sample_topk_topp(..., workspace=)``: one per caller whose calls may overlap others'."""
    return torch.zeros(lib().ohara_sample_workspace_bytes(), dtype=torch.uint8, device=device)


# ---- BitLinear ---------------------------------------------------------------------------------


class PackedTernary:
    """Ternary weight (N, K) in the kernels' 2-bit layout with its per-tensor scale."""

    __slots__ = ("data", "n", "k", "gamma")

    def __init__(self, data, n, k, gamma):
        self.data, self.n, self.k, self.gamma = data, n, k, float(gamma)


def pack_ternary(t: torch.Tensor, gamma: float) -> PackedTernary:
    _need(t, torch.int8, "t")
    n, k = t.shape
    nbytes = C.c_int64(0)
    check(lib().ohara_bitlinear_pack_ternary(0, n, k, k, 0, C.byref(nbytes), 0), "pack_ternary size")
    dst = torch.empty(nbytes.value // 4, dtype=torch.int32, device=t.device)
    check(lib().ohara_bitlinear_pack_ternary(_ptr(t), n, k, k, _ptr(dst), None, _stream()), "pack_ternary")
    return PackedTernary(dst, n, k, gamma)


def act_quant(x: torch.Tensor, norm_w: torch.Tensor, eps: float = 1e-5):
    """(rows, K) bf16 -> q int8 (rows, K padded to 16), s fp32 (rows,), sum q int32 (rows,)."""
    _need(x, BF16, "x")
    rows, k = x.shape
    ldq = (k + 15) // 16 * 16
    q = torch.zeros(rows, ldq, dtype=torch.int8, device=x.device)
    s = torch.empty(rows, dtype=torch.float32, device=x.device)
    sq = torch.empty(rows, dtype=torch.int32, device=x.device)
    check(lib().ohara_act_quant_int8(_ptr(x), x.stride(0), _ptr(norm_w), eps, rows, k, _ptr(q), ldq, _ptr(s), _ptr(sq),
                                     _stream()), "act_quant")
    return q, s, sq


def gemv_ternary(q, s, sumq, w: PackedTernary, residual=None, out=None, want_acc=False):
    rows = q.shape[0]
    if out is None:
        out = torch.empty(rows, w.n, dtype=BF16, device=q.device)
    acc = torch.empty(rows, w.n, dtype=torch.int32, device=q.device) if want_acc else None
    check(lib().ohara_gemv_ternary_i8(_ptr(q), q.stride(0), _ptr(s), _ptr(sumq), _ptr(w.data), w.n, w.k, w.gamma, rows,
                                      _ptr(residual), 0 if residual is None else residual.stride(0), _ptr(out),
                                      out.stride(0), _ptr(acc), w.n, _stream()), "gemv_ternary")
    return (out, acc) if want_acc else out


def bitlinear(x, norm_w, w: PackedTernary, eps=1e-5, residual=None, out=None, want_acc=False, pre_norm_w=None):
    """Fused BitLinear.forward on rows of x (rows, K) bf16; ``pre_norm_w`` applies a block-level
    RMSNorm to x first, in the same pass."""
    _need(x, BF16, "x")
    rows, k = x.shape
    if k != w.k:
        raise ValueError(f"x has {k} columns, weight expects {w.k}")
    if out is None:
        out = torch.empty(rows, w.n, dtype=BF16, device=x.device)
    acc = torch.empty(rows, w.n, dtype=torch.int32, device=x.device) if want_acc else None
    check(lib().ohara_bitlinear_bf16(_ptr(x), x.stride(0), _ptr(pre_norm_w), _ptr(norm_w), eps, _ptr(w.data), w.n, w.k, w.gamma, rows,
                                     _ptr(residual), 0 if residual is None else residual.stride(0), _ptr(out),
                                     out.stride(0), _ptr(acc), w.n, _stream()), "bitlinear")
    return (out, acc) if want_acc else out


def bitlinear_qkv_rope_append(x, pre_norm_w, projs, eps, h, h_kv, dh, cos, sin, pos, kcache, vcache, q_out=None,
                              pos_dev=None, seq_len=1):
    """The query / key / value BitLinears of one layer on rows of x (rows <= 64) in one launch, with
    rotary + cache append.  ``projs``: three (norm_w, PackedTernary) pairs.  Returns q (rows, h*dh)."""
    _need(x, BF16, "x")
    rows, k = x.shape
    if q_out is None:
        q_out = torch.empty(rows, h * dh, dtype=BF16, device=x.device)
    nw = (C.c_void_p * 3)(*[p[0].data_ptr() for p in projs])
    wp = (C.c_void_p * 3)(*[p[1].data.data_ptr() for p in projs])
    gm = (C.c_float * 3)(*[p[1].gamma for p in projs])
    check(lib().ohara_bitlinear_qkv_rope_append_bf16(
        _ptr(x), x.stride(0), _ptr(pre_norm_w), eps, k, nw, wp, gm, rows // seq_len, seq_len, h, h_kv, dh, _ptr(cos),
        _ptr(sin), int(pos), _ptr(pos_dev), _ptr(q_out), _ptr(kcache), _ptr(vcache), kcache.shape[1], _stream()),
        "bitlinear_qkv_rope_append")
    return q_out


def bitlinear_gate_up(x, pre_norm_w, gate, up, eps=1e-5, out=None):
    """silu(gate(x)) * up(x) for two BitLinears ((norm_w, PackedTernary) pairs) on rows of x (<= 64)."""
    _need(x, BF16, "x")
    rows, k = x.shape
    f = gate[1].n
    if out is None:
        out = torch.empty(rows, f, dtype=BF16, device=x.device)
    check(lib().ohara_bitlinear_gate_up_bf16(
        _ptr(x), x.stride(0), _ptr(pre_norm_w), eps, k, f, _ptr(gate[0]), _ptr(gate[1].data), gate[1].gamma,
        _ptr(up[0]), _ptr(up[1].data), up[1].gamma, rows, _ptr(out), out.stride(0), _stream()), "bitlinear_gate_up")
    return out


def silu_mul(gate, up, out=None):
    _need(gate, BF16, "gate")
    _need(up, BF16, "up")
    if out is None:
        out = torch.empty_like(gate)
    check(lib().ohara_silu_mul_bf16(_ptr(gate), _ptr(up), _ptr(out), gate.numel(), _stream()), "silu_mul")
    return out


def rope_append(q, k, v, batch, seq_len, h, h_kv, dh, cos, sin, pos, kcache, vcache, pos_dev=None):
    """In-place rotary on q (rows, h*dh); rotated k and v appended to the cache."""
    check(lib().ohara_rope_append_bf16(_ptr(q), _ptr(k), _ptr(v), batch, seq_len, h, h_kv, dh, _ptr(cos), _ptr(sin),
                                       int(pos), _ptr(pos_dev), _ptr(kcache), _ptr(vcache), kcache.shape[1], _stream()),
          "rope_append")
    return q


def rope_rows(q, k, v, batch, seq_len, h, h_kv, dh, cos, sin, pos, pos_dev=None):
    """In-place rotary on q; returns the rotated k and v as (batch, seq_len, h_kv, dh) tensors (what an int8
    cache's append quantises)."""
    kr, vr = torch.empty_like(k), torch.empty_like(v)
    check(lib().ohara_rope_append_bf16(_ptr(q), _ptr(k), _ptr(v), batch, seq_len, h, h_kv, dh, _ptr(cos), _ptr(sin),
                                       int(pos), _ptr(pos_dev), _ptr(kr), _ptr(vr), 0, _stream()), "rope_rows")
    return kr.view(batch, seq_len, h_kv, dh), vr.view(batch, seq_len, h_kv, dh)


# ---- Phi (ohara/models/phi.py) ----------------------------------------------------------------

_LIN_EPI = {"bias": 0, "gelu": 1, "add2": 2}


def linear_bias(x, w: PackedLinear, bias, epilogue: str = "bias", add1=None, add2=None, out=None) -> torch.Tensor:
    """nn.Linear with bias on a packed weight; ``epilogue``: "bias", "gelu" (new_gelu of the result,
    phi.py:37-40) or "add2" (bf16(bf16(add1 + y) + add2), phi.py:151).  x: (rows, K), any row stride."""
    if x.dtype != BF16 or not x.is_cuda or x.stride(1) != 1:
        raise ValueError("x must be a bf16 device matrix with unit column stride")
    _need(bias, BF16, "bias")
    rows, k = x.shape
    if k != w.k or bias.numel() != w.n:
        raise ValueError(f"x has {k} columns / bias {bias.numel()} entries, weight is {w.n} x {w.k}")
    if out is None:
        out = torch.empty(rows, w.n, dtype=BF16, device=x.device)
    for t in (add1, add2):
        if t is not None and (t.dtype != BF16 or t.stride(1) != 1):
            raise ValueError("addends must be bf16 with unit column stride")
    check(
        lib().ohara_linear_bias_bf16(
            _ptr(x), x.stride(0), _ptr(w.data), w.n, w.k, _ptr(bias), rows, _LIN_EPI[epilogue],
            _ptr(add1), 0 if add1 is None else add1.stride(0), _ptr(add2), 0 if add2 is None else add2.stride(0),
            _ptr(out), out.stride(0), _stream(),
        ),
        "linear_bias",
    )
    return out


def phi_block_in(x, ln_w, ln_b, eps, w: PackedLinear, bias, d, ff, batch, seq_len, pos, kcache, vcache, q, act,
                 pos_dev=None) -> None:
    """LayerNorm + [q; k; v; fc1] projection with bias + cache append + new_gelu in one launch
    (phi.py:150, :81-87, :95, :50-51).  x: (rows, d); q: (rows, d); act: (rows, ff)."""
    _need(x, BF16, "x")
    if w.n != 3 * d + ff or w.k != d or bias.numel() != w.n:
        raise ValueError("packed weight / bias do not match [q; k; v; fc1]")
    check(lib().ohara_phi_block_in_bf16(_ptr(x), x.stride(0), _ptr(ln_w), _ptr(ln_b), eps, _ptr(w.data), _ptr(bias), d, ff,
                                        batch, seq_len, pos, _ptr(pos_dev), _ptr(q), q.stride(0), _ptr(kcache), _ptr(vcache),
                                        kcache.shape[1], _ptr(act), act.stride(0), _stream()), "phi_block_in")


def layernorm(x, weight, bias, eps: float = 1e-5, out=None) -> torch.Tensor:
    """nn.LayerNorm over the last dimension of a (rows, d) bf16 matrix (phi.py:132, :160)."""
    _need(x, BF16, "x")
    rows, d = x.shape
    if out is None:
        out = torch.empty_like(x)
    check(lib().ohara_layernorm_bf16(_ptr(x), x.stride(0), _ptr(weight), _ptr(bias), _ptr(out), out.stride(0), rows, d, eps,
                                     _stream()), "layernorm")
    return out


def kv_append(k, v, kcache, vcache, batch, seq_len, h, dh, pos, pos_dev=None) -> None:
    """Rows (b, s) of k / v (views with a common row stride) -> cache[b, pos + s] as they are
    (phi.py:95)."""
    if k.stride(0) != v.stride(0) or k.stride(1) != 1 or v.stride(1) != 1:
        raise ValueError("k and v must share a row stride and have unit column stride")
    check(lib().ohara_kv_append_bf16(_ptr(k), _ptr(v), k.stride(0), batch, seq_len, h, dh, pos, _ptr(pos_dev), _ptr(kcache),
                                     _ptr(vcache), kcache.shape[1], _stream()), "kv_append")


def phi_attn_workspace(batch, h, dh, n_split, device) -> torch.Tensor:
    nbytes = lib().ohara_phi_attn_workspace_bytes(batch, h, dh, n_split)
    if nbytes < 0:
        raise ValueError("phi_attn_workspace: invalid sizes")
    return torch.zeros(nbytes, dtype=torch.uint8, device=device)  # the chunk counters start at zero


def phi_attn(q, kcache, vcache, cos, sin, rot, batch, seq_len, h, dh, pos, pos_dev=None, out=None, n_split=1,
             workspace=None) -> torch.Tensor:
    """PhiMHA's attention core over the cache (phi.py:98-117); q: (rows, h*dh) view with any row
    stride; cos / sin: fp32 (t_max, rot/2).  ``n_split`` > 1 (single-token calls) spreads the context
    over that many workgroups per (sequence, head); ``workspace`` from ``phi_attn_workspace``."""
    if q.stride(1) != 1:
        raise ValueError("q must have unit column stride")
    if cos.dtype != torch.float32 or sin.dtype != torch.float32:
        raise ValueError("cos / sin must be fp32")
    if out is None:
        out = torch.empty(batch * seq_len, h * dh, dtype=BF16, device=q.device)
    check(lib().ohara_phi_attn_bf16(_ptr(q), q.stride(0), _ptr(kcache), _ptr(vcache), _ptr(cos), _ptr(sin), rot, batch,
                                    seq_len, h, dh, kcache.shape[1], pos, _ptr(pos_dev), n_split, _ptr(workspace), _ptr(out),
                                    _stream()), "phi_attn")
    return out
