"""CPU restatement of the reference's Llama forward with a KV cache.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).  Citations are into the
reference tree (``ohara/...``).

The model is a flat dict of tensors keyed by the reference's state-dict names
(``token_emb.weight``, ``layers.N.attn.{key,query,value,proj}.weight``,
``layers.N.ff.{up,gate,down}.weight``, ``layers.N.norm{1,2}.weight``, ``norm.weight``,
``vocab_proj.weight``, ``freq_cos``, ``freq_sin``; MoE layers:
``layers.N.ff.{w_gate,w_up,w_down,router.weight,router_bias,shared_gate.weight,
shared_up.weight,shared_down.weight}``).

Rounding points follow the reference when the model is cast to bf16: every
elementwise torch op rounds to the tensor dtype; a Linear is an fp32-accumulated
product rounded once to the model dtype.
"""

from __future__ import annotations

import math
from dataclasses import dataclass

import torch
import torch.nn.functional as F

from . import moe_ref


@dataclass
class RefConfig:
    """Same fields and defaults as ``Config`` (ohara/models/llama.py:16-45)."""

    vocab_size: int = 65
    max_sequence_length: int = 64
    hidden_size: int = 128
    intermediate_size: int = 256
    num_attention_heads: int = 4
    num_key_value_heads: int = 0
    num_hidden_layers: int = 4
    dropout: float = 0.2
    multiple_of: int = 4
    bias: bool = False
    weight_tying: bool = False
    rope_theta: float = 100000
    init_style: str = "standard"
    moe_num_experts: int = 0
    moe_experts_per_tok: int = 2
    moe_layer_interval: int = 1
    moe_gate_fn: str = "softmax"
    moe_quantile_balancing: bool = True
    moe_grouped: bool = False
    moe_num_shared_experts: int = 0
    moe_normalize_weights: bool = True

    @property
    def head_dim(self) -> int:
        return self.hidden_size // self.num_attention_heads

    @property
    def kv_heads(self) -> int:
        # llama.py:54-56 - 0 means "same as the query heads".
        return self.num_attention_heads if self.num_key_value_heads == 0 else self.num_key_value_heads

    def layer_is_moe(self, idx: int) -> bool:
        # llama.py:147-151
        return self.moe_num_experts >= 1 and idx % self.moe_layer_interval == 0


# ---------------------------------------------------------------------------
# parts
# ---------------------------------------------------------------------------


def rope_table(head_dim: int, end: int, theta: float = 10000.0):
    """cos/sin(t * theta^(-2i/D)), t in [0,end), i in [0,D/2) - rotary.py:24-38.

    Computed in fp32 exactly as the reference does (fp32 exponent, fp32 outer
    product), so that the table, once rounded to bf16 with the model
    (chat_engine.py:265 casts registered buffers), carries the same values.
    """
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2)[: head_dim // 2].float() / head_dim))
    t = torch.arange(end)
    ang = torch.outer(t, inv).float()
    return torch.cos(ang), torch.sin(ang)


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-5) -> torch.Tensor:
    """norm.py:16-21 - fp32 normalise, round to x's dtype, then times the weight."""
    xf = x.float()
    normed = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)).type_as(x)
    return normed * weight


def linear(x: torch.Tensor, w: torch.Tensor, f32_cache: dict | None = None,
           bias: torch.Tensor | None = None) -> torch.Tensor:
    """``x @ w.T (+ bias)`` (nn.Linear, llama.py:60-63,252; mlp.py:146-148; ``bias`` with Config.bias=True).

    fp32 accumulation over the dtype-rounded operands, the bias added to the fp32 sum, one rounding
    to x's dtype.
    """
    if w.dtype == torch.float32:
        wf = w
    elif f32_cache is not None:
        key = (w.data_ptr(), tuple(w.shape), tuple(w.stride()))
        wf = f32_cache.get(key)
        if wf is None:
            wf = w.float()
            f32_cache[key] = wf
    else:
        wf = w.float()
    y = x.float() @ wf.t()
    if bias is not None:
        y = y + bias.float()
    return y.to(x.dtype)


def apply_rope(q: torch.Tensor, k: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor):
    """Adjacent-pair rotation - rotary.py:55-93.

    q, k: (B, S, heads, D); cos, sin: (S, D/2) rows for the positions being
    processed (already sliced, llama.py:311-314).  Maths in fp32 on the (possibly
    bf16-rounded) operands, result rounded to q's dtype.
    """

    def rot(x):
        xf = x.float()
        even, odd = xf[..., 0::2], xf[..., 1::2]
        c = cos.float()[None, :, None, :]
        s = sin.float()[None, :, None, :]
        out = torch.empty_like(xf)
        out[..., 0::2] = even * c - odd * s
        out[..., 1::2] = even * s + odd * c
        return out.to(q.dtype)

    return rot(q), rot(k)


def quantize_int8(tensor, dim: int = -1):
    """Affine int8 codes along ``dim`` - kv_cache.py:15-28.

    Every step is a separate elementwise op in the tensor's dtype (so each rounds to bf16 when the
    rows are bf16): range = max - min; scale = max(range / 255, 1e-8); code = clamp(round((x - min)
    / scale - 128), -128, 127).  ``round`` is to nearest even.  Returns (codes int8, scale, min).
    """
    lo, hi = tensor.amin(dim, keepdim=True), tensor.amax(dim, keepdim=True)
    scale = ((hi - lo) / 255).clamp(min=1e-8)
    codes = ((tensor - lo) / scale - 128).round().clamp(-128, 127).to(torch.int8)
    return codes, scale, lo


def dequantize_int8(codes, scale, lo):
    """(code + 128) * scale + min in fp32 - kv_cache.py:31-33 (the stored statistics are fp32,
    kv_cache.py:69-74, so the product and the sum each round once to fp32)."""
    return (codes.float() + 128) * scale + lo


class KVCacheRef:
    """Fixed-size sequential-append cache - kv_cache.py:35-118.

    Storage (B, T_max, H_kv, D) for keys and values; holds post-rotary keys.  With ``int8`` the
    entries are int8 codes with one fp32 (scale, min) pair per (batch, position, head) row and reads
    return the dequantised values cast to the dtype of the appended rows (kv_cache.py:94-118).
    """

    def __init__(self, shape, max_seq_length, idx=None, dtype=torch.float32, int8=False):
        self.idx = idx
        self.int8 = int8
        self.max_seq_length = max_seq_length
        self.length = 0
        self.batch_size = None
        self.dtype = dtype
        self.key = torch.zeros(shape, dtype=torch.int8 if int8 else dtype)
        self.value = torch.zeros(shape, dtype=torch.int8 if int8 else dtype)
        if int8:
            stats = (*shape[:-1], 1)
            self.key_scale = torch.zeros(stats, dtype=torch.float32)
            self.key_min = torch.zeros(stats, dtype=torch.float32)
            self.value_scale = torch.zeros(stats, dtype=torch.float32)
            self.value_min = torch.zeros(stats, dtype=torch.float32)

    def forward(self, keys, values, start_pos):
        bsz, seq_len = keys.shape[0], keys.shape[1]
        # kv_cache.py:78-90, in the reference's order.
        if values.shape != keys.shape:
            raise ValueError("KV cache keys and values must have matching shapes")
        if bsz > self.key.size(0):
            raise ValueError("KV cache batch size is smaller than the input batch")
        if self.batch_size is not None and bsz != self.batch_size:
            raise ValueError("KV cache batch size cannot change during decoding")
        if start_pos != self.length:
            raise ValueError(
                f"KV cache writes must be sequential: expected position {self.length}, got {start_pos}"
            )
        if start_pos < 0 or start_pos + seq_len > self.max_seq_length:
            raise ValueError("KV cache position exceeds max_sequence_length")
        end = start_pos + seq_len
        if self.int8:
            kq, ks, km = quantize_int8(keys)
            vq, vs, vm = quantize_int8(values)
            self.key[:bsz, start_pos:end] = kq
            self.value[:bsz, start_pos:end] = vq
            self.key_scale[:bsz, start_pos:end] = ks
            self.key_min[:bsz, start_pos:end] = km
            self.value_scale[:bsz, start_pos:end] = vs
            self.value_min[:bsz, start_pos:end] = vm
        else:
            self.key[:bsz, start_pos:end] = keys
            self.value[:bsz, start_pos:end] = values
        self.length = end
        self.batch_size = bsz
        if not self.int8:
            return self.key[:bsz, :end], self.value[:bsz, :end]
        k = dequantize_int8(self.key[:bsz, :end], self.key_scale[:bsz, :end], self.key_min[:bsz, :end])
        v = dequantize_int8(self.value[:bsz, :end], self.value_scale[:bsz, :end], self.value_min[:bsz, :end])
        return k.to(keys.dtype), v.to(keys.dtype)


_LOG2E_F32 = torch.tensor([0x3FB8AA3B], dtype=torch.int32).view(torch.float32)[0]
_LN_FLT_MIN = torch.tensor([0xC2AEAC50 - (1 << 32)], dtype=torch.int32).view(torch.float32)[0]


def _fma32(a, b, c):
    """One fused multiply-add in fp32: the product of two fp32 values is exact in fp64."""
    return (a.double() * b.double() + c.double()).float()


def fexp_u20(x: torch.Tensor) -> torch.Tensor:
    """The exponential of torch's CPU flash-attention kernel for bf16 / fp16 inputs (torch 2.10.0,
    pinned by the reference's pyproject.toml:49-52; ``Vectorized<float>::fexp_u20``), restated from its
    published algorithm (Malossi, Ineichen, Bekas, Curioni: Fast Exponential Computation on SIMD
    Architectures): ``2**(x log2 e)`` with the fractional part corrected by a cubic, assembled
    directly in the exponent and mantissa fields.  Relative error up to 1.1e-4 - what it returns,
    not exp(x), is what the reference's bf16 attention rounds to bf16.  Arguments are <= 0 here.
    """
    c0, c1, c2, c3 = (torch.tensor(c, dtype=torch.float32) for c in
                      (0.00010703434948458272, 0.30354260500649682, -0.22433836478672356, -0.079204240219773236))
    src = x * _LOG2E_F32
    frac = src - torch.floor(src)
    r = _fma32(frac, c3, c2)
    r = _fma32(frac, r, c1)
    r = _fma32(frac, r, c0)
    src = src - r
    bits = _fma32(torch.tensor(float(2 ** 23)), src, torch.tensor(float(2 ** 23) * 127.0))
    out = bits.clamp(min=0).to(torch.int32).view(torch.float32)  # truncating conversion
    return torch.where(x < _LN_FLT_MIN, torch.zeros_like(out), out)


SDPA_KV_BLOCK = 512  # keys per block of torch's CPU flash-attention kernel
SDPA_VEC = 16         # fp32 lanes of its vector loop (AVX-512, the build the fixtures were made with)


def _attention_reduced(q, k, v, visible):
    """``F.scaled_dot_product_attention`` as torch 2.10.0 computes it on the CPU for bf16 / fp16
    tensors (the dtype ChatEngine casts the model to, chat_engine.py:262-265; call site
    llama.py:116-123), with every rounding point of that kernel:

    keys are taken in blocks of 512; per block the scores are an fp32-accumulated product times
    1/sqrt(D) (fp32), masked with -inf; the running maximum m and sum l are fp32; the weights
    ``p = fexp_u20(s - m_new)`` (the block's last ``len % 16`` keys, which the vector loop leaves to a
    scalar tail: ``exp``) enter the sum unrounded and are ROUNDED TO THE INPUT DTYPE before
    the fp32-accumulated product with V; earlier blocks' sum and accumulator are rescaled by
    ``exp(m_old - m_new)``; the result is ``acc * (1 / l)`` rounded once.

    q: (B,H,S,D), k, v: (B,H,L,D), visible: (S,L) bool.  Pinned against the library routine itself
    in tests/test_oracle.py (>= 97 % of the elements bit-identical at every size tried, the rest
    one ulp: the fp32 summation order inside the library's products is not restated).
    """
    B, H, S, D = q.shape
    L = k.shape[2]
    qf, kf, vf = q.float(), k.float(), v.float()
    scale = torch.tensor(1.0 / math.sqrt(D), dtype=torch.float32)
    m = torch.full((B, H, S), float("-inf"))
    l = torch.zeros(B, H, S)
    acc = torch.zeros(B, H, S, D)
    for n in range(0, L, SDPA_KV_BLOCK):
        e = min(L, n + SDPA_KV_BLOCK)
        s = (qf @ kf[:, :, n:e].transpose(-1, -2)) * scale
        s = s.masked_fill(~visible[None, None, :, n:e], float("-inf"))
        m_new = torch.maximum(m, s.amax(-1))
        d = s - m_new[..., None]
        nv = (e - n) // SDPA_VEC * SDPA_VEC  # full vectors of the block: fast exponential; the tail: exp
        p = torch.cat([fexp_u20(d[..., :nv]), torch.exp(d[..., nv:])], dim=-1)
        corr = torch.exp(m - m_new)
        corr = torch.where(torch.isnan(corr), torch.zeros_like(corr), corr)  # -inf - -inf: nothing seen yet
        l = l * corr + p.sum(-1)
        acc = acc * corr[..., None] + p.to(q.dtype).float() @ vf[:, :, n:e]
        m = m_new
    return (acc * (1.0 / l)[..., None]).to(q.dtype)


def attention_core(q, k, v, start_pos: int | None):
    """softmax(q k^T / sqrt(D) + mask) v with GQA - llama.py:100-135.

    q: (B, S, H, D); k, v: (B, L, H_kv, D).  ``start_pos`` None = uncached causal
    (is_causal=True, llama.py:122); otherwise the cache mask
    ``key_pos <= start_pos + q_idx`` over all L cached positions (llama.py:109-113).
    GQA: query head h reads kv head h // (H/H_kv) (repeat_interleave, llama.py:101-103).
    fp32 tensors: fp32 scores / softmax / accumulation, one rounding.  bf16 / fp16 tensors: the
    rounding points of the library kernel the reference calls (``_attention_reduced``).
    Returns (B, S, H*D).
    """
    B, S, H, D = q.shape
    L, Hkv = k.shape[1], k.shape[2]
    group = H // Hkv
    base = 0 if start_pos is None else start_pos
    qpos = base + torch.arange(S)
    kpos = torch.arange(L)
    visible = kpos[None, :] <= qpos[:, None]
    if q.dtype != torch.float32 and q.dtype != torch.float64:
        qh, kh, vh = q.permute(0, 2, 1, 3), k.permute(0, 2, 1, 3), v.permute(0, 2, 1, 3)
        if group > 1:
            kh = kh.repeat_interleave(group, dim=1)
            vh = vh.repeat_interleave(group, dim=1)
        out = _attention_reduced(qh, kh, vh, visible)
        return out.permute(0, 2, 1, 3).reshape(B, S, H * D)
    qf = q.float().permute(0, 2, 1, 3)  # (B,H,S,D)
    kf = k.float().permute(0, 2, 1, 3)  # (B,Hkv,L,D)
    vf = v.float().permute(0, 2, 1, 3)
    if group > 1:
        kf = kf.repeat_interleave(group, dim=1)
        vf = vf.repeat_interleave(group, dim=1)
    scores = qf @ kf.transpose(-1, -2) / math.sqrt(D)  # (B,H,S,L)
    scores = scores.masked_fill(~visible[None, None], float("-inf"))
    p = torch.softmax(scores, dim=-1)
    out = (p @ vf).to(q.dtype)  # (B,H,S,D)
    return out.permute(0, 2, 1, 3).reshape(B, S, H * D)


def swiglu(x, w_gate, w_up, w_down, f32_cache=None):
    """down(silu(gate(x)) * up(x)) - mlp.py:152."""
    g = linear(x, w_gate, f32_cache)
    u = linear(x, w_up, f32_cache)
    return linear(F.silu(g) * u, w_down, f32_cache)


# ---------------------------------------------------------------------------
# model
# ---------------------------------------------------------------------------


def weight_names(cfg: RefConfig):
    """(name, shape, kind) in a fixed order; kind in {'normal','ones','zeros'}."""
    d, F_, V = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    D, H, Hkv = cfg.head_dim, cfg.num_attention_heads, cfg.kv_heads
    out = [("token_emb.weight", (V, d), "normal")]
    for i in range(cfg.num_hidden_layers):
        p = f"layers.{i}."
        out += [
            (p + "attn.key.weight", (Hkv * D, d), "normal"),
            (p + "attn.query.weight", (H * D, d), "normal"),
            (p + "attn.value.weight", (Hkv * D, d), "normal"),
            (p + "attn.proj.weight", (d, H * D), "normal"),
        ]
        if cfg.layer_is_moe(i):
            E = cfg.moe_num_experts
            out += [
                (p + "ff.w_gate", (E, d, F_), "normal"),
                (p + "ff.w_up", (E, d, F_), "normal"),
                (p + "ff.w_down", (E, F_, d), "normal"),
                (p + "ff.router.weight", (E, d), "normal"),
                (p + "ff.router_bias", (E,), "zeros"),
            ]
            if cfg.moe_num_shared_experts > 0:
                sh = F_ * cfg.moe_num_shared_experts
                out += [
                    (p + "ff.shared_gate.weight", (sh, d), "normal"),
                    (p + "ff.shared_up.weight", (sh, d), "normal"),
                    (p + "ff.shared_down.weight", (d, sh), "normal"),
                ]
        else:
            out += [
                (p + "ff.up.weight", (F_, d), "normal"),
                (p + "ff.down.weight", (d, F_), "normal"),
                (p + "ff.gate.weight", (F_, d), "normal"),
            ]
        out += [(p + "norm1.weight", (d,), "ones"), (p + "norm2.weight", (d,), "ones")]
    out += [("norm.weight", (d,), "ones"), ("vocab_proj.weight", (V, d), "normal")]
    if cfg.bias:
        # llama.py:60-63 and :185 (mlp.py:146-148): a bias on every attention projection and on a dense
        # feed-forward's three Linears, never on vocab_proj (llama.py:252).  Drawn after all the matrices,
        # so that a config's matrices do not depend on the flag; the reference starts them at zero
        # (llama.py:429-430), here they are drawn like the matrices so that a dropped bias shows.
        for i in range(cfg.num_hidden_layers):
            p = f"layers.{i}."
            out += [(p + "attn.key.bias", (Hkv * D,), "normal"), (p + "attn.query.bias", (H * D,), "normal"),
                    (p + "attn.value.bias", (Hkv * D,), "normal"), (p + "attn.proj.bias", (d,), "normal")]
            if not cfg.layer_is_moe(i):
                out += [(p + "ff.up.bias", (F_,), "normal"), (p + "ff.down.bias", (d,), "normal"),
                        (p + "ff.gate.bias", (F_,), "normal")]
    return out


def init_weights(cfg: RefConfig, seed: int = 0, dtype=torch.float32, std: float = 0.02,
                 norm_jitter: float = 0.0) -> dict:
    """Oracle-owned seeded weights: N(0, std) matrices, unit norm weights
    (llama.py:426-439 draws the same distributions; the exact RNG stream of the
    reference's module construction is not reproduced - parity is kernel-vs-oracle
    on identical tensors).  ``norm_jitter`` > 0 perturbs the norm weights so tests
    notice a dropped norm weight.
    """
    g = torch.Generator().manual_seed(seed)
    w = {}
    for name, shape, kind in weight_names(cfg):
        if kind == "normal":
            t = torch.empty(shape).normal_(0.0, std, generator=g)
        elif kind == "ones":
            t = torch.ones(shape)
            if norm_jitter:
                t = t + norm_jitter * torch.empty(shape).uniform_(-1, 1, generator=g)
        else:
            t = torch.zeros(shape)
        # router_bias stays fp32 in the reference only until .to(dtype) casts the
        # buffer with the module; it is added to fp32 logits (moe_grouped.py:131).
        w[name] = t.to(dtype)
    if cfg.weight_tying:
        w["token_emb.weight"] = w["vocab_proj.weight"]  # llama.py:254-255
    cos, sin = rope_table(cfg.head_dim, cfg.max_sequence_length * 2, cfg.rope_theta)  # llama.py:257-263
    w["freq_cos"] = cos.to(dtype)
    w["freq_sin"] = sin.to(dtype)
    return w


class RefLlama:
    """Functional restatement of ``Llama`` (llama.py:204-348) over a weight dict."""

    def __init__(self, cfg: RefConfig, weights: dict):
        self.config = cfg
        self.w = weights
        self.dtype = weights["token_emb.weight"].dtype
        self._f32 = {}

    # llama.py:325-348
    def build_kv_cache(self, batch_size: int = 1, int8: bool = False):
        if batch_size < 1:
            raise ValueError("batch_size must be at least 1")
        c = self.config
        shape = (batch_size, c.max_sequence_length, c.kv_heads, c.head_dim)
        return [KVCacheRef(shape, c.max_sequence_length, i, dtype=self.dtype, int8=int8)
                for i in range(c.num_hidden_layers)]

    def _lin(self, name, x):
        """A Linear, or - when the weight dict holds ``name.ternary`` - a BitLinear
        (experiments/bitnet/bitnet.py:46-59 installed by apply_bitlinear :70-95) on
        pre-ternarised weights ``name.ternary`` (int8), ``name.gamma`` and its own
        ``name.rms_norm.weight``."""
        w = self.w
        if name + ".ternary" in w:
            from .bitlinear_ref import bitlinear_forward

            shp = x.shape
            y = bitlinear_forward(x.reshape(-1, shp[-1]), w[name + ".rms_norm.weight"],
                                  w[name + ".ternary"], w[name + ".gamma"])
            return y.view(*shp[:-1], -1)
        return linear(x, w[name + ".weight"], self._f32, w.get(name + ".bias"))

    def _attn(self, i, h, cos, sin, cache, start_pos):
        c, w = self.config, self.w
        p = f"layers.{i}.attn."
        B, S, _ = h.shape
        k = self._lin(p + "key", h).view(B, S, c.kv_heads, c.head_dim)
        q = self._lin(p + "query", h).view(B, S, c.num_attention_heads, c.head_dim)
        v = self._lin(p + "value", h).view(B, S, c.kv_heads, c.head_dim)
        q, k = apply_rope(q, k, cos, sin)  # llama.py:93
        if cache is not None:
            k, v = cache.forward(k, v, start_pos)  # llama.py:96-98
        o = attention_core(q, k, v, start_pos if cache is not None else None)
        return self._lin(p + "proj", o)  # llama.py:142

    def _ff(self, i, h):
        c, w = self.config, self.w
        p = f"layers.{i}.ff."
        if c.layer_is_moe(i):
            return moe_ref.moe_forward(
                h,
                router_w=w[p + "router.weight"],
                router_bias=w[p + "router_bias"],
                w_gate=w[p + "w_gate"],
                w_up=w[p + "w_up"],
                w_down=w[p + "w_down"],
                k=c.moe_experts_per_tok,
                gate_fn=c.moe_gate_fn,
                normalize_weights=c.moe_normalize_weights,
                quantile_balancing=c.moe_quantile_balancing,
                shared=(
                    (w[p + "shared_gate.weight"], w[p + "shared_up.weight"], w[p + "shared_down.weight"])
                    if c.moe_num_shared_experts > 0
                    else None
                ),
                f32_cache=self._f32,
            )
        # mlp.py:152
        return self._lin(p + "down", F.silu(self._lin(p + "gate", h)) * self._lin(p + "up", h))

    # llama.py:279-323
    def forward(self, x, kv_cache=None, position_ids=None, return_hidden: bool = False):
        c, w = self.config, self.w
        if x.ndim != 2:
            raise ValueError("input token IDs must have shape (batch, sequence)")
        if isinstance(position_ids, torch.Tensor):
            if position_ids.numel() != 1:
                raise ValueError("position_ids must be a scalar cache position")
            position_ids = int(position_ids.item())
        start_pos = 0
        if kv_cache is not None:
            if len(kv_cache) != c.num_hidden_layers:
                raise ValueError("KV cache must contain one entry per model layer")
            if position_ids is None or position_ids < 0:
                raise ValueError("a non-negative position_ids is required with KV cache")
            start_pos = position_ids
        elif position_ids is not None:
            raise ValueError("position_ids is only valid when using a KV cache")
        S = x.size(1)
        if S < 1:
            raise ValueError("input sequence cannot be empty")
        if start_pos + S > c.max_sequence_length:
            raise ValueError("input exceeds max_sequence_length")

        h = w["token_emb.weight"][x]
        cos = w["freq_cos"][start_pos : start_pos + S]
        sin = w["freq_sin"][start_pos : start_pos + S]
        for i in range(c.num_hidden_layers):
            cache = kv_cache[i] if kv_cache is not None else None
            pre = f"layers.{i}."
            # Block.forward, llama.py:199-200
            h = h + self._attn(i, rms_norm(h, w[pre + "norm1.weight"]), cos, sin, cache, start_pos)
            h = h + self._ff(i, rms_norm(h, w[pre + "norm2.weight"]))
        h = rms_norm(h, w["norm.weight"])
        if return_hidden:
            return h
        return linear(h, w["vocab_proj.weight"], self._f32)

    __call__ = forward
