"""CPU restatement of the reference's Phi forward with a KV cache (ohara/models/phi.py).

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).  Citations are into the reference tree.

The model is a flat dict of tensors keyed by the reference's state-dict names
(``wte.weight``, ``layers.N.ln.{weight,bias}``, ``layers.N.mixer.{q_proj,k_proj,v_proj,dense}.
{weight,bias}``, ``layers.N.mlp.{fc1,fc2}.{weight,bias}``, ``ln.{weight,bias}``,
``lm_head.{weight,bias}``).

Rounding points follow the reference when the model is cast to a 16-bit dtype: every
elementwise torch op rounds to the tensor dtype; a Linear is an fp32-accumulated product plus the
bias, rounded once; LayerNorm is the library routine (fp32 statistics, one rounding); the
attention core runs in fp32 from the cached 16-bit rows and rounds its output once
(phi.py:91-117).

Pinning status (tests/test_oracle_phi.py):
  rope_partial        fp64 closed form (complex rotation of half-split pairs), the reference's
                      own RoPE module on seeded inputs (tests/golden/phi_rope.pt), identity at
                      position 0, pass-through of the un-rotated tail
  new_gelu            F.gelu(approximate="tanh") (library routine)
  layer_norm          F.layer_norm (library routine), zero mean / unit variance closed form
  attention           fp64 brute-force loops on tiny inputs
  phi_forward         PARITY UNPINNED as a composition: ohara/models/phi.py cannot be imported here
                      (it pulls ohara.utils, which needs the absent `lightning` package), so no
                      golden logits exist.  What holds it: the reference test's invariant
                      (prefill + cached step == uncached forward, tests/test_models.py:133-149)
                      and hand-written fp64 loops over one tiny block.
"""

from __future__ import annotations

import math
from dataclasses import dataclass

import torch
import torch.nn.functional as F

from .llama_ref import KVCacheRef


@dataclass
class RefPhiConfig:
    """Same fields and defaults as ``PhiConfig`` (ohara/models/phi.py:23-34)."""

    vocab_size: int = 51200
    max_sequence_length: int = 2048
    hidden_size: int = 2560
    num_attention_heads: int = 32
    num_hidden_layers: int = 32
    dropout: float = 0.2
    multiple_of: int = 4
    bias: bool = True
    eps: float = 1e-5
    rotary_dim: float = 0.4

    @property
    def head_dim(self) -> int:
        return self.hidden_size // self.num_attention_heads

    @property
    def rotary_width(self) -> int:
        # phi.py:69 - int(rotary_dim * head_dim) leading features of every head are rotated
        return int(self.rotary_dim * self.head_dim)


def rope_cos_sin(num_positions: int, dims: int, offset: int = 0, base: float = 10000.0):
    """rotary.py:166-184 - cos/sin(t * exp(-i * log(base) / (dims/2))), t in [offset, num_positions),
    i in [0, dims/2), all in fp32 as the reference computes them for fp32 inputs."""
    half = dims // 2
    positions = torch.arange(offset, num_positions, dtype=torch.float32)
    freqs = torch.exp(-torch.arange(0.0, half, dtype=torch.float32) * (math.log(base) / half))
    theta = positions.reshape(-1, 1) * freqs.reshape(1, -1)
    return torch.cos(theta), torch.sin(theta)


def rope_partial(x: torch.Tensor, dims: int, offset: int = 0) -> torch.Tensor:
    """RoPE(dims, traditional=False) on (..., T, D) - rotary.py:131-164: feature i < dims/2 is
    paired with feature i + dims/2, features from ``dims`` on pass through; row t sits at position
    offset + t."""
    T = x.shape[-2]
    cos, sin = rope_cos_sin(T + offset, dims, offset)
    cos, sin = cos.to(x.dtype), sin.to(x.dtype)
    half = dims // 2
    x1, x2 = x[..., :half], x[..., half:dims]
    r1 = x1 * cos - x2 * sin
    r2 = x1 * sin + x2 * cos
    return torch.cat([r1, r2, x[..., dims:]], dim=-1)


def new_gelu(x: torch.Tensor) -> torch.Tensor:
    """phi.py:37-40, op by op (every op rounds to x's dtype)."""
    return 0.5 * x * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * torch.pow(x, 3.0))))


def layer_norm(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float) -> torch.Tensor:
    """nn.LayerNorm (phi.py:132,160): fp32 mean and biased variance over the last dimension,
    ((x - mean) * rstd) * weight + bias in fp32, one rounding to x's dtype."""
    xf = x.float()
    mean = xf.mean(-1, keepdim=True)
    var = (xf - mean).pow(2).mean(-1, keepdim=True)
    y = (xf - mean) * torch.rsqrt(var + eps) * weight.float() + bias.float()
    return y.to(x.dtype)


def linear_bias(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, f32_cache: dict | None = None) -> torch.Tensor:
    """nn.Linear with bias (phi.py:46-47,63-66,161): fp32 accumulation over the dtype-rounded
    operands plus the bias, one rounding to x's dtype."""
    if w.dtype == torch.float32:
        wf = w
    elif f32_cache is not None:
        key = (w.data_ptr(), tuple(w.shape))
        wf = f32_cache.get(key)
        if wf is None:
            wf = w.float()
            f32_cache[key] = wf
    else:
        wf = w.float()
    return (x.float() @ wf.t() + b.float()).to(x.dtype)


def attention(q, k_all, v_all, start_pos: int, rot: int, out_dtype):
    """phi.py:91-117.  q: (B, S, H, D) new queries; k_all / v_all: (B, L, H, D) every cached row
    (un-rotated keys).  fp32 throughout; queries rotate from ``start_pos``, keys from 0; key t is
    visible to query s when t <= start_pos + s."""
    q = q.transpose(1, 2).to(torch.float32)
    k = k_all.transpose(1, 2).to(torch.float32)
    v = v_all.transpose(1, 2).to(torch.float32)
    q = rope_partial(q, rot, offset=start_pos)
    k = rope_partial(k, rot)
    scores = (q @ k.transpose(-1, -2)) * math.sqrt(1 / q.shape[-1])
    S, L = q.shape[2], k.shape[2]
    allowed = torch.arange(L).unsqueeze(0) <= (start_pos + torch.arange(S)).unsqueeze(1)
    scores = scores.masked_fill(~allowed, float("-inf"))
    out = (torch.softmax(scores, dim=-1) @ v).to(out_dtype)
    return out.transpose(1, 2)  # (B, S, H, D)


def weight_names(cfg: RefPhiConfig):
    d, f = cfg.hidden_size, cfg.multiple_of * cfg.hidden_size
    names = {"wte.weight": (cfg.vocab_size, d), "ln.weight": (d,), "ln.bias": (d,),
             "lm_head.weight": (cfg.vocab_size, d), "lm_head.bias": (cfg.vocab_size,)}
    for i in range(cfg.num_hidden_layers):
        p = f"layers.{i}."
        names[p + "ln.weight"] = (d,)
        names[p + "ln.bias"] = (d,)
        for n in ("q_proj", "k_proj", "v_proj", "dense"):
            names[p + f"mixer.{n}.weight"] = (d, d)
            names[p + f"mixer.{n}.bias"] = (d,)
        names[p + "mlp.fc1.weight"] = (f, d)
        names[p + "mlp.fc1.bias"] = (f,)
        names[p + "mlp.fc2.weight"] = (d, f)
        names[p + "mlp.fc2.bias"] = (d,)
    return names


def init_weights(cfg: RefPhiConfig, seed: int = 0, dtype=torch.float32, std: float = 0.02, bias_std: float = 0.02):
    """Seeded random weights under the reference's names (LayerNorm weights near one)."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in weight_names(cfg).items():
        if name.endswith("ln.weight"):
            t = 1.0 + 0.1 * torch.randn(shape, generator=g)
        elif name.endswith("bias"):
            t = bias_std * torch.randn(shape, generator=g)
        else:
            t = std * torch.randn(shape, generator=g)
        out[name] = t.to(dtype)
    return out


class RefPhi:
    """Functional Phi (phi.py:155-205) over a flat weight dict."""

    def __init__(self, cfg: RefPhiConfig, weights: dict):
        self.cfg = cfg
        self.w = weights
        self.dtype = weights["wte.weight"].dtype
        self._f32: dict = {}

    def build_kv_cache(self, batch_size: int = 1, int8: bool = False):
        """phi.py:189-202; ``int8``: the caches' int8 mode (kv_cache.py:15-32, 94-118: a property of the cache class
        the model constructs, which quantises the un-rotated rows on write and returns dequantised tensors on read)."""
        if batch_size < 1:
            raise ValueError("batch_size must be at least 1")  # phi.py:190-191
        c = self.cfg
        shape = (batch_size, c.max_sequence_length, c.num_attention_heads, c.head_dim)
        return [KVCacheRef(shape, c.max_sequence_length, i, dtype=self.dtype, int8=int8) for i in range(c.num_hidden_layers)]

    def block(self, i: int, x, cache, position_ids):
        c, w, p = self.cfg, self.w, f"layers.{i}."
        B, S, _ = x.shape
        H, D = c.num_attention_heads, c.head_dim
        h = layer_norm(x, w[p + "ln.weight"], w[p + "ln.bias"], c.eps)  # phi.py:150
        lin = lambda t, n: linear_bias(t, w[p + n + ".weight"], w[p + n + ".bias"], self._f32)
        k = lin(h, "mixer.k_proj").view(B, S, H, D)  # phi.py:81-87
        q = lin(h, "mixer.q_proj").view(B, S, H, D)
        v = lin(h, "mixer.v_proj").view(B, S, H, D)
        start = 0
        if cache is not None:
            if position_ids is None:
                raise ValueError("position_ids is required when using a KV cache")  # phi.py:92-93
            start = int(position_ids)
            k, v = cache.forward(k, v, start)  # the un-rotated rows go into the cache (phi.py:95)
        a = attention(q, k, v, start, c.rotary_width, x.dtype).reshape(B, S, c.hidden_size)
        mixer = lin(a, "mixer.dense")  # phi.py:120
        mlp = lin(new_gelu(lin(h, "mlp.fc1")), "mlp.fc2")  # phi.py:49-52
        return mixer + mlp + x  # phi.py:151

    def forward(self, ids, kv_cache=None, position_ids=None):
        c, w = self.cfg, self.w
        if kv_cache is not None and len(kv_cache) != c.num_hidden_layers:
            raise ValueError("KV cache must contain one entry per model layer")  # phi.py:176-177
        x = w["wte.weight"][ids]
        for i in range(c.num_hidden_layers):
            x = self.block(i, x, kv_cache[i] if kv_cache is not None else None, position_ids)
        x = layer_norm(x, w["ln.weight"], w["ln.bias"], c.eps)
        return linear_bias(x, w["lm_head.weight"], w["lm_head.bias"], self._f32)

    __call__ = forward
