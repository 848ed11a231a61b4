"""BitNet-b1.58 Llama decode path: the Llama of ohara/models/llama.py whose seven per-layer
projections were swapped for BitLinear by ``apply_bitlinear`` (experiments/bitnet/bitnet.py:70-95;
target list of experiments/bitnet/train_bitnet.py:240), served with real 2-bit/int8 integer
kernels.  Embedding, norms and the vocabulary projection stay bf16.

State dict keys per BitLinear ``<name>``: either the float ``<name>.weight`` (ternarised here
with weight_quant's rule, bitnet.py:37-43) or pre-ternarised ``<name>.ternary`` (int8) and
``<name>.gamma``; plus ``<name>.rms_norm.weight``.
"""

from __future__ import annotations

import ctypes as C

import torch

from . import _lib, ops
from ._lib import OharaBitLayer, OharaBitModel, OharaDecodeState, check, lib
from .llama import BF16, Config, KVCache, _check_ids_on_host, _validate_config, rope_tables

BIT_TARGETS = ("attn.key", "attn.query", "attn.value", "attn.proj", "ff.gate", "ff.up", "ff.down")
# order of OharaBitLayer's arrays (OHARA_BIT_QUERY ... OHARA_BIT_DOWN)
BIT_ORDER = ("attn.query", "attn.key", "attn.value", "attn.proj", "ff.gate", "ff.up", "ff.down")


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
        torch.cuda.synchronize(self.device)
        # host-side description of the model for the single-launch decode step
        self._c_layers = (OharaBitLayer * c.num_hidden_layers)()
        for i, L in enumerate(self.layers):
            cl = self._c_layers[i]
            for j, nm in enumerate(BIT_ORDER):
                w, nw = L[nm]
                cl.w[j], cl.norm_w[j], cl.gamma[j] = w.data.data_ptr(), nw.data_ptr(), w.gamma
            cl.norm1, cl.norm2 = L["norm1"].data_ptr(), L["norm2"].data_ptr()
        m = OharaBitModel()
        m.n_layers, m.d_model, m.n_heads, m.n_kv_heads = c.num_hidden_layers, c.hidden_size, c.num_attention_heads, self.kv_heads
        m.head_dim, m.d_ff, m.vocab, m.t_max = self.head_dim, c.intermediate_size, c.vocab_size, c.max_sequence_length
        m.eps = self.eps
        m.token_emb, m.final_norm, m.w_vocab = self.token_emb.data_ptr(), self.final_norm.data_ptr(), self.w_vocab.data.data_ptr()
        m.cos, m.sin = self.cos.data_ptr(), self.sin.data_ptr()
        m.layers = C.cast(self._c_layers, C.POINTER(OharaBitLayer))
        self._c_model = m

    def eval(self):
        return self

    def to(self, *a, **k):
        return self

    def build_kv_cache(self, batch_size: int = 1, int8: bool = False):
        if batch_size < 1:
            raise ValueError("batch_size must be at least 1")
        c = self.config
        shape = (batch_size, c.max_sequence_length, self.kv_heads, self.head_dim)
        return [KVCache(shape, c.max_sequence_length, i, device=self.device, dtype=BF16, int8=int8)
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
        if len({cc.int8 for cc in kv_cache}) > 1:
            raise ValueError("all layers must use the same KV cache mode")
        int8 = kv_cache[0].int8
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
            if int8:
                # kv_cache.py:94-118 with quantisation: the new rows go in as codes and attention reads what the
                # reference's cache read returns (the dequantised prefix, the new rows included); many new
                # positions per sequence attend over a dequantised copy of the live prefix
                q = ops.bitlinear(h, L["attn.query"][1], L["attn.query"][0], self.eps, pre_norm_w=L["norm1"])
                k = ops.bitlinear(h, L["attn.key"][1], L["attn.key"][0], self.eps, pre_norm_w=L["norm1"])
                v = ops.bitlinear(h, L["attn.value"][1], L["attn.value"][0], self.eps, pre_norm_w=L["norm1"])
                kr, vr = ops.rope_rows(q, k, v, B, S, H, Hkv, D, self.cos, self.sin, start)
                ops.kv_quant_append(kr, vr, cache, start)
            elif rows <= 64:  # decode: one launch for q/k/v + rotary + append, one for gate/up + SwiGLU
                q = ops.bitlinear_qkv_rope_append(
                    h, L["norm1"], [(L[n][1], L[n][0]) for n in ("attn.query", "attn.key", "attn.value")], self.eps,
                    H, Hkv, D, self.cos, self.sin, start, cache.key, cache.value, seq_len=S)
            else:
                q = ops.bitlinear(h, L["attn.query"][1], L["attn.query"][0], self.eps, pre_norm_w=L["norm1"])
                k = ops.bitlinear(h, L["attn.key"][1], L["attn.key"][0], self.eps, pre_norm_w=L["norm1"])
                v = ops.bitlinear(h, L["attn.value"][1], L["attn.value"][0], self.eps, pre_norm_w=L["norm1"])
                ops.rope_append(q, k, v, B, S, H, Hkv, D, self.cos, self.sin, start, cache.key, cache.value)
            if not int8:
                att = ops.attn_auto(q, cache.key, cache.value, H, Hkv, D, start, n_split, ws, S)
            elif S >= 16 and D in (64, 128):
                att = ops.attn_prefill(q, ops.kv_dequant(cache, "key", B, start + S),
                                       ops.kv_dequant(cache, "value", B, start + S), H, Hkv, D, start, S)
            else:
                att = ops.attn_cached_int8(q, cache, H, Hkv, D, start, n_split, ws, seq_len=S)
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

    # -- device-resident loop ---------------------------------------------------------

    def supports_persistent(self, batch: int) -> bool:
        """Shapes the single-launch ternary decode kernel covers."""
        c = self.config
        return (batch <= 8 and self.head_dim in (64, 128) and self.kv_heads == c.num_attention_heads
                and c.hidden_size % 16 == 0 and c.intermediate_size % 16 == 0 and c.hidden_size <= 2048
                and c.intermediate_size <= 6144)

    def session(self, batch: int, max_new_tokens: int, valid_vocab: int = 0, kv_cache: list | None = None,
                persistent: bool | None = None, sampling=None, u=None):
        return BitDecodeSession(self, batch, max_new_tokens, valid_vocab, kv_cache, persistent, sampling, u)

    @torch.no_grad()
    def generate_greedy(self, prompt_ids: torch.Tensor, steps: int, *, persistent: bool | None = None,
                        use_graph: bool = True, valid_vocab: int = 0) -> torch.Tensor:
        """Prefill the prompt, then ``steps`` greedy tokens (the loop of ohara/chat_engine.py:395-405
        for a batch of equal-length prompts).  Returns the generated ids (B, steps)."""
        B, P = prompt_ids.shape
        if steps < 1:
            return torch.zeros(B, 0, dtype=torch.int64, device=self.device)
        sess = self.session(B, steps, valid_vocab, persistent=persistent)
        sess.prefill(prompt_ids)
        sess.run(steps - 1, use_graph=use_graph)
        return sess.tokens()


class BitDecodeSession:
    """One batch of equal-length sequences decoded on the device by the BitNet model: the prompt
    goes through ``BitLlama.forward`` once, then every token is one launch of the single-launch
    ternary decode kernel (selection included; with sampling the fused sampler follows it), replayed
    from a HIP graph.  Where that kernel does not cover the shape, every token is one eager
    ``forward`` of the kernel chain.  Same surface as ``ohara_amd.llama.DecodeSession``."""

    PERSISTENT_SPLITS = 16

    def __init__(self, model: BitLlama, batch: int, max_new_tokens: int, valid_vocab: int = 0, kv_cache=None,
                 persistent: bool | None = None, sampling=None, u=None):
        self.model, self.batch = model, batch
        self.sampling = sampling if (sampling is not None and sampling.temperature > 0) else None
        self.u = None
        rows = max(max_new_tokens, 1)
        if self.sampling is not None:
            if u is None:
                u = torch.rand(rows, batch, device=model.device, dtype=torch.float32)
            if u.shape != (rows, batch):
                raise ValueError("u must have shape (max_new_tokens, batch)")
            self.u = u.to(device=model.device, dtype=torch.float32).contiguous()
            self._sample_ws = ops.sample_workspace(model.device)  # this session's own: sessions may overlap
        self.cache = kv_cache if kv_cache is not None else model.build_kv_cache(batch)
        int8 = any(cc.int8 for cc in self.cache)  # int8 caches are served by the kernel chain
        if persistent is None:
            persistent = model.supports_persistent(batch) and not int8
        elif persistent and (int8 or not model.supports_persistent(batch)):
            raise ValueError("the persistent decode kernel does not cover this shape" if not int8 else
                             "the single-launch ternary decode kernel reads bfloat16 caches; int8 caches run the kernel chain")
        self.persistent = persistent
        self.spin_limit = 0
        self.valid_vocab = valid_vocab
        dev = model.device
        self.history = torch.zeros(rows, batch, dtype=torch.int64, device=dev)
        self.logits = torch.empty(batch, model.config.vocab_size, dtype=BF16, device=dev)
        self.ids = torch.zeros(batch, dtype=torch.int64, device=dev)
        self.step_state = torch.zeros(4, dtype=torch.int32, device=dev)
        self.produced = 0
        self.pos = 0
        self.graph = None
        self.graph_multi = None
        self._dst = None
        self._pws = None

    def _select(self, logits: torch.Tensor, row: int) -> torch.Tensor:
        if self.sampling is None:
            return ops.argmax(logits, self.valid_vocab or None)
        return ops.sample_topk_topp(logits, self.sampling.temperature, self.sampling.top_k, self.sampling.top_p,
                                    self.u[row], self.valid_vocab or None)

    def prefill(self, prompt_ids: torch.Tensor) -> None:
        m, B = self.model, self.batch
        if prompt_ids.ndim != 2 or prompt_ids.shape[0] != B:
            raise ValueError("input token IDs must have shape (batch, sequence)")
        P = prompt_ids.shape[1]
        _check_ids_on_host(prompt_ids, m.config.vocab_size)
        logits = m.forward(prompt_ids, self.cache, 0, last_only=True)  # validates the rest
        first = self._select(logits[:, 0].contiguous(), 0).view(B)
        self.ids.copy_(first)
        self.history[0].copy_(first)
        self.step_state.copy_(torch.tensor([P, 1, 0, 0], dtype=torch.int32))
        self.pos, self.produced = P, 1
        if self._dst is not None or not self.persistent:
            return
        st = OharaDecodeState()
        st.batch, st.rows_cap, st.n_split = B, B, self.PERSISTENT_SPLITS
        st.valid_vocab, st.hist_cap, st.prof_kernel = self.valid_vocab, self.history.shape[0], -1
        st.ids, st.logits = self.ids.data_ptr(), self.logits.data_ptr()
        st.step_state, st.history = self.step_state.data_ptr(), self.history.data_ptr()
        n = len(self.cache)
        self._kptrs = (C.c_void_p * n)(*[cc.key.data_ptr() for cc in self.cache])
        self._vptrs = (C.c_void_p * n)(*[cc.value.data_ptr() for cc in self.cache])
        st.kcache = C.cast(self._kptrs, C.POINTER(C.c_void_p))
        st.vcache = C.cast(self._vptrs, C.POINTER(C.c_void_p))
        self._dst = st
        self._nwg = torch.cuda.get_device_properties(m.device).multi_processor_count
        nbytes = lib().ohara_bitnet_persistent_workspace_bytes(C.byref(m._c_model), B, self._nwg)
        if nbytes < 0:
            raise RuntimeError("persistent workspace query failed")
        self._pws = torch.zeros(nbytes, dtype=torch.uint8, device=m.device)
        self._err_off = lib().ohara_bitnet_persistent_error_offset(C.byref(m._c_model), B, self._nwg)
        self._prof_off = lib().ohara_bitnet_persistent_profile_offset(C.byref(m._c_model), B, self._nwg)
        self._init_workspace()

    def _init_workspace(self) -> None:
        torch.cuda.current_stream().synchronize()
        check(lib().ohara_bitnet_decode_persistent(C.byref(self.model._c_model), C.byref(self._dst), self._pws.data_ptr(),
                                                   self._nwg, 1, 1, 0, torch.cuda.current_stream().cuda_stream),
              "persistent init")

    def restart(self, u: torch.Tensor | None = None) -> None:
        """Forget the sequences decoded so far; caches, workspace and the captured graph are kept."""
        for cc in self.cache:
            cc.length, cc.batch_size, cc.lengths = 0, None, None
        self.pos = 0
        self.produced = 0
        if u is not None:
            if self.u is None:
                raise ValueError("this session selects greedily: it takes no uniform draws")
            if u.ndim != 2 or u.shape[1] != self.batch or u.shape[0] > self.u.shape[0]:
                raise ValueError("u must have shape (rows <= max_new_tokens, batch)")
            self.u[: u.shape[0]].copy_(u)

    def _launch_step(self) -> None:
        stream = torch.cuda.current_stream().cuda_stream
        greedy = 0 if self.sampling else 1
        check(lib().ohara_bitnet_decode_persistent(C.byref(self.model._c_model), C.byref(self._dst), self._pws.data_ptr(),
                                                   self._nwg, 0, greedy, int(self.spin_limit), stream),
              "persistent decode step")
        if self.sampling:
            ops.sample_topk_topp(self.logits, self.sampling.temperature, self.sampling.top_k, self.sampling.top_p,
                                 self.u, self.valid_vocab or None, out=self.ids, history=self.history,
                                 step_state=self.step_state, u_per_step=True, workspace=self._sample_ws)

    def check_error(self) -> None:
        """Raise if a barrier wait of the persistent kernel expired (synchronises)."""
        if self.persistent and self._pws is not None:
            word = self._pws[self._err_off : self._err_off + 4].view(torch.int32).cpu()
            if int(word[0]) != 0:
                raise RuntimeError("persistent decode kernel: a grid barrier wait expired")

    def reset_error(self) -> None:
        if self.persistent and self._pws is not None:
            self._init_workspace()

    def phase_clocks(self) -> torch.Tensor:
        """Shader-clock samples of workgroup 0 at the barriers of the last step launched while
        ``self._dst.prof_kernel`` was -2 (measurement aid)."""
        return self._pws[self._prof_off : self._prof_off + 8192].view(torch.int64).cpu()

    def _room(self, n: int) -> None:
        if self.produced < 1:
            raise RuntimeError("prefill first")
        if self.pos + n > self.model.config.max_sequence_length:
            raise ValueError("input exceeds max_sequence_length")
        if self.produced + n > self.history.shape[0]:
            raise ValueError("max_new_tokens exceeded")

    def _advance(self, n: int) -> None:
        self.pos += n
        self.produced += n
        for cc in self.cache:
            cc._commit(self.batch, self.pos)

    def step(self) -> None:
        """One eager decode step (enqueue only)."""
        self._room(1)
        if self.persistent:
            self._launch_step()
            self._advance(1)
            return
        m, B = self.model, self.batch
        logits = m.forward(self.ids.view(B, 1), self.cache, self.pos, last_only=True)  # commits the caches
        self.logits.copy_(logits[:, 0])
        nxt = self._select(self.logits, self.produced).view(B)
        self.ids.copy_(nxt)
        self.history[self.produced].copy_(nxt)
        self.pos += 1
        self.produced += 1

    GRAPH_STEPS = 8  # steps in the second captured graph

    def capture(self) -> None:
        """One step in one HIP graph, GRAPH_STEPS steps in a second (one host launch per eight tokens)."""
        if self.graph is not None:
            return
        self.step()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            self._launch_step()
        self.graph = g
        gm = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gm):
            for _ in range(self.GRAPH_STEPS):
                self._launch_step()
        self.graph_multi = gm

    def run(self, n: int, use_graph: bool = True) -> None:
        """Enqueue n more decode steps."""
        if n <= 0:
            return
        if not (use_graph and self.persistent):
            for _ in range(n):
                self.step()
            return
        if self.graph is None:
            self.capture()
            n -= 1
        self._room(n)
        many, rest = divmod(n, self.GRAPH_STEPS)
        for _ in range(many):
            self.graph_multi.replay()
        for _ in range(rest):
            self.graph.replay()
        self._advance(n)

    def tokens(self) -> torch.Tensor:
        """(B, produced) generated ids (synchronises)."""
        out = self.history[: self.produced].t().contiguous()
        self.check_error()
        return out
