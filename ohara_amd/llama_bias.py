"""Llama built with ``Config.bias=True``: every attention projection and the SwiGLU's three Linears carry a
bias (ohara/models/llama.py:60-63, :180-186; ohara/modules/mlp.py:146-148; the vocabulary projection never
does, llama.py:252).  The forward runs through the KV cache over the library's Linear-with-bias kernel, one
launch per Linear; the fused projections, the persistent kernel and the decode session serve the default
``bias=False`` only."""

from __future__ import annotations

import torch

from . import ops
from ._lib import lib
from .llama import BF16, Config, KVCache, _validate_config, rope_tables

_ATTN = ("attn.query", "attn.key", "attn.value", "attn.proj")
_FF = ("ff.gate", "ff.up", "ff.down")


class BiasLlama:
    """The reference's ``Llama`` call surface (llama.py:204-348) for a dense config with ``bias=True``."""

    supports_last_only = True

    def __init__(self, config: Config, state: dict, device="cuda"):
        _validate_config(config, allow_bias=True)
        if not config.bias:
            raise ValueError("BiasLlama serves configs with bias=True")
        if config.moe_num_experts > 0:
            raise ValueError("ohara_amd: Linear biases are served for dense feed-forwards only")
        lib()
        self.config, self.device = config, torch.device(device)
        c = config
        self.head_dim = c.hidden_size // c.num_attention_heads
        self.kv_heads = c.num_attention_heads if c.num_key_value_heads == 0 else c.num_key_value_heads
        self.eps = 1e-5

        def dev(t):
            return t.detach().to(device=self.device, dtype=BF16).contiguous()

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
            L = {n: (ops.pack_linear(dev(state[p + n + ".weight"])), dev(state[p + n + ".bias"])) for n in _ATTN + _FF}
            L["norm1"], L["norm2"] = dev(state[p + "norm1.weight"]), dev(state[p + "norm2.weight"])
            self.layers.append(L)
        self._ws = {}

    def eval(self):
        return self

    def to(self, *a, **k):
        return self

    def build_kv_cache(self, batch_size: int = 1, int8: bool = False):
        """ohara/models/llama.py:325-348; ``int8=True`` builds the int8 caches of kv_cache.py:15-32."""
        if batch_size < 1:
            raise ValueError("batch_size must be at least 1")
        c = self.config
        shape = (batch_size, c.max_sequence_length, self.kv_heads, self.head_dim)
        return [KVCache(shape, c.max_sequence_length, i, device=self.device, dtype=BF16, int8=int8)
                for i in range(c.num_hidden_layers)]

    @torch.no_grad()
    def forward(self, x, kv_cache=None, position_ids=None, *, last_only: bool = False):
        """Llama.forward (llama.py:279-323); every Linear's result is rounded to bf16 after its bias, the residual
        sums once more, as the eager modules round."""
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
        if len({cc.int8 for cc in kv_cache}) > 1:
            raise ValueError("all layers must use the same KV cache mode")
        int8 = kv_cache[0].int8
        ends = [cc._reserve(B, S, start) for cc in kv_cache]
        H, Hkv, D = c.num_attention_heads, self.kv_heads, self.head_dim
        n_split = 1 if S > 1 else max(1, min(1024 // max(1, B * Hkv), c.max_sequence_length // 128, 64))
        ws = self._ws.get((B, n_split))
        if ws is None:
            ws = self._ws[(B, n_split)] = ops.attn_workspace(B, H, Hkv, D, n_split, self.device)
        h = ops.embed(x.to(self.device), self.token_emb)
        for L, cache in zip(self.layers, kv_cache):
            hn = ops.rmsnorm(h, L["norm1"], self.eps)
            q, k, v = (ops.linear_bias(hn, *L[n]) for n in _ATTN[:3])
            if int8:
                # kv_cache.py:94-118 with quantisation: the new rows go in as codes, attention reads the
                # dequantised prefix (the new rows included)
                kr, vr = ops.rope_rows(q, k, v, B, S, H, Hkv, D, self.cos, self.sin, start)
                ops.kv_quant_append(kr, vr, cache, start)
                if S >= 16 and D in (64, 128):
                    att = ops.attn_prefill(q, ops.kv_dequant(cache, "key", B, start + S),
                                           ops.kv_dequant(cache, "value", B, start + S), H, Hkv, D, start, S)
                else:
                    att = ops.attn_cached_int8(q, cache, H, Hkv, D, start, n_split, ws, seq_len=S)
            else:
                ops.rope_append(q, k, v, B, S, H, Hkv, D, self.cos, self.sin, start, cache.key, cache.value)
                att = ops.attn_auto(q, cache.key, cache.value, H, Hkv, D, start, n_split, ws, S)
            h = h + ops.linear_bias(att, *L["attn.proj"])
            hn = ops.rmsnorm(h, L["norm2"], self.eps)
            act = ops.silu_mul(ops.linear_bias(hn, *L["ff.gate"]), ops.linear_bias(hn, *L["ff.up"]))
            h = h + ops.linear_bias(act, *L["ff.down"])
        if last_only:
            h = h.view(B, S, -1)[:, -1].contiguous()
        logits = ops.gemm_skinny(h, self.w_vocab, norm_w=self.final_norm, eps=self.eps)
        for cc, end in zip(kv_cache, ends):
            cc._commit(B, end)
        return logits.view(B, 1 if last_only else S, c.vocab_size)

    __call__ = forward
