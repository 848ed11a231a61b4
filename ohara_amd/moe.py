"""Grouped mixture-of-experts decode path: ``GroupedMoE`` (ohara/modules/moe_grouped.py) in eval
mode and the Llama whose feed-forwards are GroupedMoE layers (ohara/models/llama.py:154-201 with
``moe_grouped=True``), over the HIP kernels of libohara_decode.so."""

from __future__ import annotations

import torch

from . import ops
from ._lib import check, lib
from .llama import BF16, Config, KVCache, _validate_config, rope_tables


def _ptr(t):
    return 0 if t is None else t.data_ptr()


class GroupedMoE:
    """Eval-mode GroupedMoE.forward (moe_grouped.py:209-228).  Weights use the reference's
    names and layouts: w_gate/w_up (E, dim, hidden), w_down (E, hidden, dim), router.weight
    (E, dim), router_bias (E,), shared_{gate,up,down}.weight."""

    def __init__(self, w_gate, w_up, w_down, router_w, router_bias, num_experts_per_tok: int,
                 shared=None, gate_fn: str = "softmax", normalize_weights: bool = True,
                 quantile_balancing: bool = True, device="cuda"):
        dev = torch.device(device)

        def d(t):
            return t.detach().to(device=dev, dtype=BF16).contiguous()

        E, dim, hidden = w_gate.shape
        if not 1 <= num_experts_per_tok <= E:
            raise ValueError("num_experts_per_tok must be in [1, num_experts]")
        if quantile_balancing and num_experts_per_tok >= E:
            raise ValueError("quantile balancing needs num_experts_per_tok < num_experts")
        if gate_fn not in ("softmax", "sigmoid"):
            raise ValueError("gate_fn must be 'softmax' or 'sigmoid'")
        self.E, self.dim, self.hidden, self.k = E, dim, hidden, num_experts_per_tok
        self.gate_fn, self.normalize, self.biased = gate_fn, normalize_weights, quantile_balancing
        self.device = dev
        perm = ops.swiglu_perm(hidden, dev)
        gu, dn = [], []
        for e in range(E):
            cat = torch.cat([d(w_gate[e]).t(), d(w_up[e]).t()], dim=0).contiguous()  # rows = output features
            gu.append(ops.pack_rows(cat, perm, perm.numel()))
            dn.append(ops.pack_rows(d(w_down[e]).t().contiguous()))
        self.wp_gu = torch.stack(gu).contiguous()
        self.wp_dn = torch.stack(dn).contiguous()
        self.router = ops.pack_linear(d(router_w))
        self.router_bias = d(router_bias)
        self.trace = None  # a list: route() appends (router logits, expert ids, weights) to it
        self.shared = None
        if shared is not None:
            sg, su, sd = shared
            self.shared = (ops.pack_gate_up(d(sg), d(su)), ops.pack_linear(d(sd)))
        self._counter = torch.zeros(1, dtype=torch.int32, device=dev)  # the fused route launch's arrival counter

    def route(self, flat_x: torch.Tensor):
        """-> (expert ids (N, k) int32, weights (N, k) bf16)"""
        n = flat_x.shape[0]
        logits = ops.gemm_skinny(flat_x, self.router)
        idx = torch.empty(n, self.k, dtype=torch.int32, device=self.device)
        w = torch.empty(n, self.k, dtype=BF16, device=self.device)
        check(lib().ohara_moe_route_topk(_ptr(logits), logits.stride(0), _ptr(self.router_bias), n, self.E, self.k,
                                         int(self.biased), int(self.gate_fn == "sigmoid"), int(self.normalize),
                                         _ptr(idx), _ptr(w), ops._stream()), "moe_route")
        if self.trace is not None:
            self.trace.append((logits, idx, w))
        return idx, w

    def forward_rows(self, flat_x: torch.Tensor, residual: torch.Tensor | None = None) -> torch.Tensor:
        """flat_x (N, dim) bf16 -> moe(flat_x) [+ residual]."""
        n, k, E = flat_x.shape[0], self.k, self.E
        st = ops._stream()
        idx, w = self.route(flat_x)
        offs = torch.empty(E + 1, dtype=torch.int32, device=self.device)
        pair_of = torch.empty(n * k, dtype=torch.int32, device=self.device)
        pos_of = torch.empty(n * k, dtype=torch.int32, device=self.device)
        check(lib().ohara_moe_sort_pairs(_ptr(idx), n * k, E, _ptr(offs), _ptr(pair_of), _ptr(pos_of), st), "moe_sort")
        act = torch.empty(n * k, self.hidden, dtype=BF16, device=self.device)
        check(lib().ohara_moe_experts_gate_up(_ptr(flat_x), flat_x.stride(0), _ptr(self.wp_gu),
                                              self.wp_gu.stride(0) * 2, E, self.hidden, self.dim, k, _ptr(offs),
                                              _ptr(pair_of), _ptr(act), self.hidden, st), "moe_gate_up")
        y = torch.empty(n * k, self.dim, dtype=BF16, device=self.device)
        check(lib().ohara_moe_experts_down(_ptr(act), self.hidden, _ptr(self.wp_dn), self.wp_dn.stride(0) * 2, E,
                                           self.dim, self.hidden, k, _ptr(offs), _ptr(pair_of), _ptr(w), _ptr(y),
                                           self.dim, st), "moe_down")
        sh = None
        if self.shared is not None:
            sh = ops.gemm_skinny(ops.gemm_skinny(flat_x, self.shared[0]), self.shared[1])
        out = torch.empty(n, self.dim, dtype=BF16, device=self.device)
        check(lib().ohara_moe_combine(_ptr(y), self.dim, _ptr(idx), _ptr(pos_of), n, k, _ptr(sh), self.dim,
                                      _ptr(residual), 0 if residual is None else residual.stride(0), _ptr(out), self.dim,
                                      self.dim, st), "moe_combine")
        return out

    def fused_ok(self, n: int) -> bool:
        """The four-launch form serves at most 64 experts and 1024 (token, expert) pairs: decode steps."""
        return (self.E <= 64 and n * self.k <= 1024 and self.dim % 8 == 0 and self.dim <= 4096 and self.hidden % 8 == 0
                and (self.shared is None or self.shared[0].n % 8 == 0))

    def forward_block(self, h: torch.Tensor, norm_w: torch.Tensor, eps: float) -> torch.Tensor:
        """h (N, dim) bf16 -> h + moe(rmsnorm(h)) (ohara/models/llama.py:200) in four launches: norm + router +
        selection + sort, gate/up of the experts and the shared expert, their down projections, the combine."""
        n, k, E = h.shape[0], self.k, self.E
        if not self.fused_ok(n):
            return self.forward_rows(ops.rmsnorm(h, norm_w, eps), residual=h)
        st, dev = ops._stream(), self.device
        xn = torch.empty(n, self.dim, dtype=BF16, device=dev)
        idx = torch.empty(n, k, dtype=torch.int32, device=dev)
        w = torch.empty(n, k, dtype=BF16, device=dev)
        meta = torch.empty(E + 1 + 2 * n * k, dtype=torch.int32, device=dev)
        offs, pair_of, pos_of = meta[: E + 1], meta[E + 1: E + 1 + n * k], meta[E + 1 + n * k:]
        logits = torch.empty(n, E, dtype=BF16, device=dev) if self.trace is not None else None
        check(lib().ohara_moe_route_fused(_ptr(h), h.stride(0), _ptr(norm_w), float(eps), _ptr(self.router.data),
                                          _ptr(self.router_bias), n, self.dim, E, k, int(self.biased),
                                          int(self.gate_fn == "sigmoid"), int(self.normalize), _ptr(xn), self.dim,
                                          _ptr(logits), E, _ptr(idx), _ptr(w), _ptr(offs), _ptr(pair_of), _ptr(pos_of),
                                          _ptr(self._counter), st), "moe_route_fused")
        if self.trace is not None:
            self.trace.append((logits, idx, w))
            self.last_sort = (offs, pair_of, pos_of)
        sh_gu, sh_dn = self.shared if self.shared is not None else (None, None)
        sh_hidden = sh_gu.n if sh_gu is not None else 0
        act = torch.empty(n * k, self.hidden, dtype=BF16, device=dev)
        act_sh = torch.empty(n, sh_hidden, dtype=BF16, device=dev) if sh_gu is not None else None
        check(lib().ohara_moe_experts_gate_up_shared(_ptr(xn), self.dim, _ptr(self.wp_gu), self.wp_gu.stride(0) * 2, E,
                                                     self.hidden, self.dim, k, _ptr(offs), _ptr(pair_of), _ptr(act),
                                                     self.hidden, _ptr(sh_gu.data) if sh_gu is not None else 0, sh_hidden,
                                                     n, _ptr(act_sh), sh_hidden, st), "moe_gate_up")
        y = torch.empty(n * k + (n if sh_gu is not None else 0), self.dim, dtype=BF16, device=dev)
        y_sh = y[n * k:] if sh_gu is not None else None
        check(lib().ohara_moe_experts_down_shared(_ptr(act), self.hidden, _ptr(self.wp_dn), self.wp_dn.stride(0) * 2, E,
                                                  self.dim, self.hidden, k, _ptr(offs), _ptr(pair_of), _ptr(w), _ptr(y),
                                                  self.dim, _ptr(sh_dn.data) if sh_dn is not None else 0, sh_hidden, n,
                                                  _ptr(act_sh), sh_hidden, _ptr(y_sh), self.dim, st), "moe_down")
        out = torch.empty(n, self.dim, dtype=BF16, device=dev)
        check(lib().ohara_moe_combine(_ptr(y), self.dim, _ptr(idx), _ptr(pos_of), n, k, _ptr(y_sh), self.dim, _ptr(h),
                                      h.stride(0), _ptr(out), self.dim, self.dim, st), "moe_combine")
        return out

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        b, s, dim = x.shape
        return self.forward_rows(x.reshape(b * s, dim).contiguous()).view(b, s, dim)

    __call__ = forward

    def expert_bytes(self) -> int:
        return (self.wp_gu.numel() + self.wp_dn.numel()) * 2


class MoeLlama:
    """Llama with GroupedMoE feed-forwards (every ``moe_layer_interval``-th layer; the others
    dense SwiGLU), forward through the KV cache."""

    supports_last_only = True
    # decode attention: the context of a (sequence, KV head) pair is cut into chunks of at least 192 positions
    # until about this many workgroups run (64 sequences x 16 heads at context 2048: 8 chunks of 256 positions,
    # 2.97 ms per step against 3.11 ms with one workgroup per pair)
    ATTN_WORKGROUPS = 8192

    def __init__(self, config: Config, state: dict, device="cuda"):
        _validate_config(config)
        if config.moe_num_experts < 1 or not config.moe_grouped:
            raise ValueError("MoeLlama serves configs with moe_grouped=True and moe_num_experts > 0")
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
            L = dict(
                wqkv=ops.pack_qkv(dev(state[p + "attn.query.weight"]), dev(state[p + "attn.key.weight"]),
                                  dev(state[p + "attn.value.weight"])),
                wo=ops.pack_linear(dev(state[p + "attn.proj.weight"])),
                norm1=dev(state[p + "norm1.weight"]), norm2=dev(state[p + "norm2.weight"]),
            )
            if c.moe_num_experts >= 1 and i % c.moe_layer_interval == 0:
                shared = None
                if c.moe_num_shared_experts > 0:
                    shared = (state[p + "ff.shared_gate.weight"], state[p + "ff.shared_up.weight"],
                              state[p + "ff.shared_down.weight"])
                L["moe"] = GroupedMoE(state[p + "ff.w_gate"], state[p + "ff.w_up"], state[p + "ff.w_down"],
                                      state[p + "ff.router.weight"], state[p + "ff.router_bias"],
                                      c.moe_experts_per_tok, shared, c.moe_gate_fn, c.moe_normalize_weights,
                                      c.moe_quantile_balancing, device=self.device)
            else:
                L["wgu"] = ops.pack_gate_up(dev(state[p + "ff.gate.weight"]), dev(state[p + "ff.up.weight"]))
                L["wdown"] = ops.pack_linear(dev(state[p + "ff.down.weight"]))
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
        n_split = 1 if S > 1 else max(1, min(self.ATTN_WORKGROUPS // max(1, B * Hkv), (start + 1) // 192, 64))
        ws = self._ws.get((B, n_split))
        if ws is None:
            ws = self._ws[(B, n_split)] = ops.attn_workspace(B, H, Hkv, D, n_split, self.device)
        h = ops.embed(x.to(self.device), self.token_emb)
        for L, cache in zip(self.layers, kv_cache):
            if int8:
                # kv_cache.py:94-118 with quantisation: the new rows go in as codes, attention reads what
                # the reference's cache read returns (the dequantised prefix, the new rows included);
                # many new positions per sequence attend over a dequantised copy of the live prefix
                q, k, v = ops.qkv_rope(h, L["wqkv"], L["norm1"], self.eps, H, Hkv, D, self.cos, self.sin, start,
                                       c.max_sequence_length, seq_len=S)
                ops.kv_quant_append(k.view(B, S, Hkv, D), v.view(B, S, Hkv, D), cache, start)
                if S >= 16 and D in (64, 128):
                    att = ops.attn_prefill(q, ops.kv_dequant(cache, "key", B, start + S),
                                           ops.kv_dequant(cache, "value", B, start + S), H, Hkv, D, start, S)
                else:
                    att = ops.attn_cached_int8(q, cache, H, Hkv, D, start, n_split, ws, seq_len=S)
            else:
                q = ops.qkv_rope_append(h, L["wqkv"], L["norm1"], self.eps, H, Hkv, D, self.cos, self.sin, start,
                                        cache.key, cache.value, seq_len=S)
                att = ops.attn_auto(q, cache.key, cache.value, H, Hkv, D, start, n_split, ws, S)
            h = ops.gemm_skinny(att, L["wo"], residual=h)
            if "moe" in L:
                h = L["moe"].forward_block(h, L["norm2"], self.eps)
            else:
                act = ops.gemm_skinny(h, L["wgu"], norm_w=L["norm2"], eps=self.eps)
                h = ops.gemm_skinny(act, L["wdown"], residual=h)
        if last_only:
            h = h.view(B, S, -1)[:, -1].contiguous()
        logits = ops.gemm_skinny(h, self.w_vocab, norm_w=self.final_norm, eps=self.eps)
        for cc, end in zip(kv_cache, ends):
            cc._commit(B, end)
        return logits.view(B, 1 if last_only else S, c.vocab_size)

    __call__ = forward
