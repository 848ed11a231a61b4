"""BitNet-b1.58 Llama decode path: the Llama of ohara/models/llama.py whose seven per-layer
projections were swapped for BitLinear by ``apply_bitlinear`` (experiments/bitnet/bitnet.py:70-95;
target list of experiments/bitnet/train_bitnet.py:240), served with real 2-bit/int8 integer
kernels.  Embedding, norms and the vocabulary projection stay bf16.

State dict keys per BitLinear ``<name>``: either the float ``<name>.weight`` (ternarised here
with weight_quant's rule, bitnet.py:37-43) or pre-ternarised ``<name>.ternary`` (int8) and
``<name>.gamma``; plus ``<name>.rms_norm.weight``.
"""

from __future__ import annotations

import torch

from . import ops
from .llama import BF16, Config, KVCache, _validate_config, rope_tables

BIT_TARGETS = ("attn.key", "attn.query", "attn.value", "attn.proj", "ff.gate", "ff.up", "ff.down")


def ternarize(w: torch.Tensor):
    """weight_quant (bitnet.py:37-43): gamma = max(mean|W|, 1e-5), T = clamp(round(W / gamma), -1, 1)."""
    wf = w.float()
    gamma = wf.abs().mean().clamp(min=1e-5)
    t = (wf * (1.0 / gamma)).round().clamp(-1, 1).to(torch.int8)
    return t, float(gamma)


class BitLlama:
    supports_last_only = True

    def __init__(self, config: Config, state: dict, device="cuda"):
        _validate_config(config)
        ops.lib()
        self.config, self.device = config, torch.device(device)
        c = config
        self.head_dim = c.hidden_size // c.num_attention_heads
        self.kv_heads = c.num_attention_heads if c.num_key_value_heads == 0 else c.num_key_value_heads
        self.eps = 1e-5

        def dev(t):
            return t.detach().to(device=self.device, dtype=BF16).contiguous()

        def bit(name):
            if name + ".ternary" in state:
                t, gamma = state[name + ".ternary"], float(state[name + ".gamma"])
            else:
                t, gamma = ternarize(state[name + ".weight"])
            w = ops.pack_ternary(t.to(self.device).contiguous(), gamma)
            return w, dev(state[name + ".rms_norm.weight"])

        self.token_emb = dev(state["token_emb.weight"])
        self.final_norm = dev(state["norm.weight"])
        self.w_vocab = ops.pack_linear(dev(state["token_emb.weight"] if c.weight_tying else state["vocab_proj.weight"]))
        if "freq_cos" in state:
            cos, sin = state["freq_cos"], state["freq_sin"]
        else:
            cos, sin = rope_tables(self.head_dim, c.max_sequence_length * 2, c.rope_theta)
        self.cos, self.sin = dev(cos), dev(sin)
        self.layers = []
        for i in range(c.num_hidden_layers):
            p = f"layers.{i}."
            L = {nm: bit(p + nm) for nm in BIT_TARGETS}
            L["norm1"], L["norm2"] = dev(state[p + "norm1.weight"]), dev(state[p + "norm2.weight"])
            self.layers.append(L)
        self._ws = {}

    def eval(self):
        return self

    def to(self, *a, **k):
        return self

    def build_kv_cache(self, batch_size: int = 1):
        if batch_size < 1:
            raise ValueError("batch_size must be at least 1")
        c = self.config
        shape = (batch_size, c.max_sequence_length, self.kv_heads, self.head_dim)
        return [KVCache(shape, c.max_sequence_length, i, device=self.device, dtype=BF16)
                for i in range(c.num_hidden_layers)]

    def packed_weight_bytes(self) -> int:
        return sum(L[nm][0].data.numel() * 4 for L in self.layers for nm in BIT_TARGETS)

    @torch.no_grad()
    def forward(self, x, kv_cache=None, position_ids=None, *, last_only: bool = False):
        """Llama.forward (ohara/models/llama.py:279-323) with BitLinear projections."""
        c = self.config
        if x.ndim != 2:
            raise ValueError("input token IDs must have shape (batch, sequence)")
        if isinstance(position_ids, torch.Tensor):
            if position_ids.numel() != 1:
                raise ValueError("position_ids must be a scalar cache position")
            position_ids = int(position_ids.item())
        start = 0
        if kv_cache is not None:
            if len(kv_cache) != c.num_hidden_layers:
                raise ValueError("KV cache must contain one entry per model layer")
            if position_ids is None or position_ids < 0:
                raise ValueError("a non-negative position_ids is required with KV cache")
            start = position_ids
        elif position_ids is not None:
            raise ValueError("position_ids is only valid when using a KV cache")
        B, S = x.shape
        if S < 1:
            raise ValueError("input sequence cannot be empty")
        if start + S > c.max_sequence_length:
            raise ValueError("input exceeds max_sequence_length")
        if kv_cache is None:
            kv_cache = self.build_kv_cache(B)
        if any(cc.int8 for cc in kv_cache):
            raise NotImplementedError("ohara_amd: int8 KV caches are served by the dense Llama only")
        ends = [cc._reserve(B, S, start) for cc in kv_cache]
        H, Hkv, D = c.num_attention_heads, self.kv_heads, self.head_dim
        rows = B * S
        n_split = 1 if S > 1 else max(1, min(1024 // max(1, B * Hkv), c.max_sequence_length // 128, 64))
        key = (B, n_split)
        ws = self._ws.get(key)
        if ws is None:
            ws = self._ws[key] = ops.attn_workspace(B, H, Hkv, D, n_split, self.device)
        h = ops.embed(x.to(self.device), self.token_emb)
        for L, cache in zip(self.layers, kv_cache):
            # the block norm (norm1 / norm2) is applied inside each projection's quantisation pass
            if rows <= 64:  # decode: one launch for q/k/v + rotary + append, one for gate/up + SwiGLU
                q = ops.bitlinear_qkv_rope_append(
                    h, L["norm1"], [(L[n][1], L[n][0]) for n in ("attn.query", "attn.key", "attn.value")], self.eps,
                    H, Hkv, D, self.cos, self.sin, start, cache.key, cache.value, seq_len=S)
            else:
                q = ops.bitlinear(h, L["attn.query"][1], L["attn.query"][0], self.eps, pre_norm_w=L["norm1"])
                k = ops.bitlinear(h, L["attn.key"][1], L["attn.key"][0], self.eps, pre_norm_w=L["norm1"])
                v = ops.bitlinear(h, L["attn.value"][1], L["attn.value"][0], self.eps, pre_norm_w=L["norm1"])
                ops.rope_append(q, k, v, B, S, H, Hkv, D, self.cos, self.sin, start, cache.key, cache.value)
            att = ops.attn_auto(q, cache.key, cache.value, H, Hkv, D, start, n_split, ws, S)
            h = ops.bitlinear(att, L["attn.proj"][1], L["attn.proj"][0], self.eps, residual=h)
            if rows <= 64:
                act = ops.bitlinear_gate_up(h, L["norm2"], (L["ff.gate"][1], L["ff.gate"][0]),
                                            (L["ff.up"][1], L["ff.up"][0]), self.eps)
            else:
                g = ops.bitlinear(h, L["ff.gate"][1], L["ff.gate"][0], self.eps, pre_norm_w=L["norm2"])
                u = ops.bitlinear(h, L["ff.up"][1], L["ff.up"][0], self.eps, pre_norm_w=L["norm2"])
                act = ops.silu_mul(g, u)
            h = ops.bitlinear(act, L["ff.down"][1], L["ff.down"][0], self.eps, residual=h)
        if last_only:
            h = h.view(B, S, -1)[:, -1].contiguous()
        logits = ops.gemm_skinny(h, self.w_vocab, norm_w=self.final_norm, eps=self.eps)
        for cc, end in zip(kv_cache, ends):
            cc._commit(B, end)
        return logits.view(B, 1 if last_only else S, c.vocab_size)

    __call__ = forward

    @torch.no_grad()
    def generate_greedy(self, prompt_ids: torch.Tensor, steps: int) -> torch.Tensor:
        B, P = prompt_ids.shape
        cache = self.build_kv_cache(B)
        inp, pos, out = prompt_ids.to(self.device), 0, []
        for _ in range(steps):
            logits = self.forward(inp, cache, pos, last_only=True)
            pos += inp.shape[1]
            inp = ops.argmax(logits[:, 0].contiguous()).view(B, 1)
            out.append(inp)
        return torch.cat(out, dim=1)
