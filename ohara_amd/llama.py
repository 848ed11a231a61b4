"""Host-side mirror of ohara's Llama + KVCache for the KV-cache decode path.

Same call surface as the reference (ohara/models/llama.py:16-45,204-348 and
ohara/modules/kv_cache.py:35-118):

    model = Llama(config, state_dict)              # reference state-dict keys
    cache = model.build_kv_cache(batch_size)
    logits = model(tokens, cache, position)        # (B, S, V)

but every tensor operation runs in the HIP kernels of libohara_decode.so.  All
argument validation happens on the host before any kernel is launched and raises the
reference's ValueErrors (same messages).
"""

from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

import torch

from . import _lib, ops
from ._lib import OharaDecodeState, OharaLayer, OharaModel, check, lib

BF16 = torch.bfloat16


@dataclass
class Config:
    """Field-for-field the reference's ``Config`` (ohara/models/llama.py:16-45)."""

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


def _validate_config(cfg: Config, allow_bias: bool = False) -> None:
    # ohara/models/llama.py:208-241
    if cfg.vocab_size < 2:
        raise ValueError("vocab_size must be at least 2")
    if cfg.hidden_size < 1 or cfg.num_hidden_layers < 1:
        raise ValueError("hidden_size and num_hidden_layers must be positive")
    if cfg.intermediate_size < 1:
        raise ValueError("intermediate_size must be positive")
    if cfg.num_attention_heads < 1 or cfg.hidden_size % cfg.num_attention_heads != 0:
        raise ValueError("hidden_size must be divisible by num_attention_heads")
    if (cfg.hidden_size // cfg.num_attention_heads) % 2 != 0:
        raise ValueError("attention head dimension must be even for rotary embeddings")
    if cfg.max_sequence_length < 2:
        raise ValueError("max_sequence_length must be at least 2")
    kv = cfg.num_attention_heads if cfg.num_key_value_heads == 0 else cfg.num_key_value_heads
    if kv < 1 or cfg.num_attention_heads % kv != 0:
        raise ValueError("num_key_value_heads must divide num_attention_heads")
    if cfg.bias and not allow_bias:
        raise ValueError("ohara_amd: Linear biases are served for dense feed-forwards only, by BiasLlama")


class KVCache:
    """ohara/modules/kv_cache.py:35-118 (bf16 storage): (batch, T_max, H_kv, D) key and
    value tensors written sequentially.  ``forward`` keeps the reference's semantics
    and error messages for external callers; the model's own path appends inside the
    fused projection kernel and only does the bookkeeping here (``_reserve``)."""

    def __init__(self, shape, max_seq_length, idx=None, device=None, dtype=None, int8=False):
        self.idx = idx
        self.int8 = bool(int8)
        self.max_seq_length = max_seq_length
        self.length = 0
        self.batch_size = None
        self.lengths = None  # per-sequence lengths, once sequences have advanced by different amounts
        self.dtype = dtype
        storage = torch.int8 if self.int8 else dtype
        self.key = torch.zeros(shape, device=device, dtype=storage)
        self.value = torch.zeros(shape, device=device, dtype=storage)
        if self.int8:
            # One scale / minimum per quantised row, i.e. per (batch, position, head): kv_cache.py:67-73.
            # Stored as one 16-byte record (key scale, key min, value scale, value min) per row with the
            # positions of a head contiguous - (B, H_kv, T, 4), the order decode attention reads them in;
            # the reference's four (B, T, H_kv, 1) tensors are strided views of it.
            B_, T_, H_ = shape[0], shape[1], shape[2]
            self.stats = torch.zeros((B_, H_, T_, 4), device=device, dtype=torch.float32)
            self.key_scale, self.key_min, self.value_scale, self.value_min = (
                self.stats[..., i:i + 1].permute(0, 2, 1, 3) for i in range(4))

    def _reserve(self, bsz: int, seq_len: int, start_pos: int) -> int:
        # ohara/modules/kv_cache.py:80-90, same order
        if bsz > self.key.size(0):
            raise ValueError("KV cache batch size is smaller than the input batch")
        if self.batch_size is not None and bsz != self.batch_size:
            raise ValueError("KV cache batch size cannot change during decoding")
        if self.lengths is not None and any(n != self.lengths[0] for n in self.lengths[:bsz]):
            raise ValueError("KV cache writes must be sequential: the sequences have different lengths, "
                             "pass one position per sequence")
        if start_pos != self.length:
            raise ValueError(
                f"KV cache writes must be sequential: expected position {self.length}, got {start_pos}"
            )
        if start_pos < 0 or start_pos + seq_len > self.max_seq_length:
            raise ValueError("KV cache position exceeds max_sequence_length")
        return start_pos + seq_len

    def _commit(self, bsz: int, end: int) -> None:
        self.length = end
        self.batch_size = bsz
        self.lengths = None

    # One position per sequence (no counterpart in the reference, whose cache has a single length):
    # the same checks as above, sequence by sequence.
    def _reserve_ragged(self, bsz: int, seq_len: int, starts) -> list:
        if bsz > self.key.size(0):
            raise ValueError("KV cache batch size is smaller than the input batch")
        if self.batch_size is not None and bsz != self.batch_size:
            raise ValueError("KV cache batch size cannot change during decoding")
        have = self.lengths if self.lengths is not None else [self.length] * bsz
        for b, (start, n) in enumerate(zip(starts, have)):
            if start != n:
                raise ValueError(f"KV cache writes must be sequential: expected position {n}, got {start} "
                                 f"(sequence {b})")
            if start < 0 or start + seq_len > self.max_seq_length:
                raise ValueError("KV cache position exceeds max_sequence_length")
        return [start + seq_len for start in starts]

    def _commit_ragged(self, bsz: int, ends) -> None:
        self.lengths = list(ends)
        self.length = max(ends)
        self.batch_size = bsz

    def _row_view(self, b: int) -> "KVCache":
        """The cache of sequence b alone, sharing storage."""
        v = KVCache.__new__(KVCache)
        v.idx, v.int8, v.max_seq_length, v.dtype = self.idx, self.int8, self.max_seq_length, self.dtype
        v.key, v.value = self.key[b:b + 1], self.value[b:b + 1]
        if self.int8:
            v.stats = self.stats[b:b + 1]
            v.key_scale, v.key_min, v.value_scale, v.value_min = (
                v.stats[..., i:i + 1].permute(0, 2, 1, 3) for i in range(4))
        v.length = (self.lengths[b] if self.lengths is not None else self.length)
        v.batch_size, v.lengths = None, None
        return v

    def forward(self, keys, values, start_pos):
        bsz, seq_len = keys.shape[0], keys.shape[1]
        if values.shape != keys.shape:
            raise ValueError("KV cache keys and values must have matching shapes")
        end = self._reserve(bsz, seq_len, start_pos)
        if self.int8:
            # kv_cache.py:94-102 and :116-118: quantise on write, hand back dequantised values
            if keys.dtype != BF16:
                raise ValueError("ohara_amd: the int8 KV cache quantises bfloat16 keys and values")
            ops.kv_quant_append(keys.contiguous(), values.contiguous(), self, start_pos)
            self._commit(bsz, end)
            return ops.kv_dequant(self, "key", bsz, end), ops.kv_dequant(self, "value", bsz, end)
        self.key[:bsz, start_pos:end] = keys
        self.value[:bsz, start_pos:end] = values
        self._commit(bsz, end)
        return self.key[:bsz, :end], self.value[:bsz, :end]


def rope_tables(head_dim: int, end: int, theta: float):
    """precompute_freqs_cis (ohara/embeddings_pos/rotary.py:24-38): fp32 on the host,
    exactly the reference's operation order, so the bf16-rounded tables match."""
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2)[: head_dim // 2].float() / head_dim))
    ang = torch.outer(torch.arange(end), inv).float()
    return torch.cos(ang), torch.sin(ang)


def _check_ids_on_host(x: torch.Tensor, vocab: int) -> None:
    """nn.Embedding raises on an id outside the table (llama.py:310).  Ids that arrive in host memory
    are checked here; ids already on the device are not read back (that would cost a synchronisation
    per call) - the kernels map an id outside [0, vocab) to row 0 instead of reading out of bounds."""
    if not x.is_cuda and x.numel() and (int(x.min()) < 0 or int(x.max()) >= vocab):
        raise IndexError("index out of range in self")


class _Buffers:
    """Activation buffers and the C state struct for up to `rows` rows."""

    def __init__(self, model: "Llama", batch: int, rows: int, n_split: int):
        c, dev = model.config, model.device
        hd = c.num_attention_heads * model.head_dim
        self.batch, self.rows, self.n_split = batch, rows, n_split
        self.ids = torch.zeros(rows, dtype=torch.int64, device=dev)
        self.x = torch.empty(rows, c.hidden_size, dtype=BF16, device=dev)
        self.q = torch.empty(rows, hd, dtype=BF16, device=dev)
        self.attn = torch.empty(rows, hd, dtype=BF16, device=dev)
        self.act = torch.empty(rows, model.act_width, dtype=BF16, device=dev)
        self.xn = torch.empty(rows, c.hidden_size, dtype=BF16, device=dev) if rows > 64 else None
        self.attn_ws = ops.attn_workspace(batch, c.num_attention_heads, model.kv_heads, model.head_dim, n_split, dev)
        self.step_state = torch.zeros(4, dtype=torch.int32, device=dev)
        self.logits = None
        self.history = None
        self.kstage = self.vstage = self.kdeq = self.vdeq = None  # int8 cache mode only


class Llama:
    """The reference's ``Llama`` call surface (ohara/models/llama.py:204-348) over HIP kernels.

    ``state`` uses the reference's state-dict keys; tensors may live anywhere, they are
    cast to bf16, moved to ``device`` and repacked once.
    """

    def __new__(cls, config: Config, state: dict | None = None, device="cuda", dtype=BF16):
        # A config with routed experts builds Blocks with a GroupedMoE feed-forward in the reference
        # (llama.py:154-170); here those layers live in ``MoeLlama``, which this constructor hands out.
        if cls is Llama and getattr(config, "moe_num_experts", 0) > 0:
            if dtype != BF16:
                raise ValueError("ohara_amd runs the decode path in bfloat16 only")
            from .moe import MoeLlama

            if not config.moe_grouped:
                # the per-expert loop of llama.py:171-178 (ohara/modules/moe.py) computes the function of the
                # grouped form without shared experts: its weights are restacked and served by the same kernels
                from .checkpoint import loop_moe_config, loop_moe_to_grouped

                return MoeLlama(loop_moe_config(config), loop_moe_to_grouped(state or {}), device=device)
            return MoeLlama(config, state, device=device)
        if cls is Llama and getattr(config, "bias", False):
            # Linears with a bias (llama.py:60-63, :185): one launch per Linear, in ``BiasLlama``
            if dtype != BF16:
                raise ValueError("ohara_amd runs the decode path in bfloat16 only")
            from .llama_bias import BiasLlama

            return BiasLlama(config, state or {}, device=device)
        return super().__new__(cls)

    def __init__(self, config: Config, state: dict, device="cuda", dtype=BF16):
        _validate_config(config)
        if dtype != BF16:
            raise ValueError("ohara_amd runs the decode path in bfloat16 only")
        lib()  # fail loudly now if the HIP library is missing
        self.config = config
        self.device = torch.device(device)
        self.dtype = dtype
        c = config
        self.head_dim = c.hidden_size // c.num_attention_heads
        self.kv_heads = c.num_attention_heads if c.num_key_value_heads == 0 else c.num_key_value_heads
        self.act_width = c.intermediate_size
        self.eps = 1e-5

        def dev(t):
            return t.detach().to(device=self.device, dtype=BF16).contiguous()

        self.token_emb = dev(state["token_emb.weight"])
        self.final_norm = dev(state["norm.weight"])
        vocab_w = state["token_emb.weight"] if c.weight_tying else state["vocab_proj.weight"]
        self.w_vocab = ops.pack_linear(dev(vocab_w))
        if "freq_cos" in state:
            cos, sin = state["freq_cos"], state["freq_sin"]
        else:
            cos, sin = rope_tables(self.head_dim, c.max_sequence_length * 2, c.rope_theta)
        self.cos, self.sin = dev(cos), dev(sin)
        self.layers = []
        for i in range(c.num_hidden_layers):
            p = f"layers.{i}."
            self.layers.append(
                dict(
                    wqkv=ops.pack_qkv(dev(state[p + "attn.query.weight"]), dev(state[p + "attn.key.weight"]),
                                      dev(state[p + "attn.value.weight"])),
                    wo=ops.pack_linear(dev(state[p + "attn.proj.weight"])),
                    wgu=ops.pack_gate_up(dev(state[p + "ff.gate.weight"]), dev(state[p + "ff.up.weight"])),
                    wdown=ops.pack_linear(dev(state[p + "ff.down.weight"])),
                    norm1=dev(state[p + "norm1.weight"]),
                    norm2=dev(state[p + "norm2.weight"]),
                )
            )
        torch.cuda.synchronize(self.device)
        self._c_layers = (OharaLayer * c.num_hidden_layers)()
        for i, L in enumerate(self.layers):
            cl = self._c_layers[i]
            cl.wqkv, cl.wo, cl.wgu, cl.wdown = (L[k].data.data_ptr() for k in ("wqkv", "wo", "wgu", "wdown"))
            cl.norm1, cl.norm2 = L["norm1"].data_ptr(), L["norm2"].data_ptr()
        m = OharaModel()
        m.n_layers, m.d_model, m.n_heads, m.n_kv_heads = c.num_hidden_layers, c.hidden_size, c.num_attention_heads, self.kv_heads
        m.head_dim, m.d_ff, m.vocab, m.t_max = self.head_dim, c.intermediate_size, c.vocab_size, c.max_sequence_length
        m.eps = self.eps
        m.token_emb, m.final_norm, m.w_vocab = self.token_emb.data_ptr(), self.final_norm.data_ptr(), self.w_vocab.data.data_ptr()
        m.cos, m.sin = self.cos.data_ptr(), self.sin.data_ptr()
        m.layers = C.cast(self._c_layers, C.POINTER(OharaLayer))
        self._c_model = m
        self._buffers: dict = {}

    # -- reference surface -------------------------------------------------------

    supports_last_only = True  # forward(..., last_only=True) computes the last row of logits only

    def eval(self):
        return self

    def to(self, *args, **kwargs):
        """nn.Module.to for a model whose weights are already packed on its device in bf16: a request
        for that device / dtype is a no-op, anything else raises (the kernels run bf16 only)."""
        dtype = kwargs.get("dtype")
        device = kwargs.get("device")
        for a in args:
            if isinstance(a, torch.dtype):
                dtype = a
            elif a is not None:
                device = a
        if dtype is not None and dtype != BF16:
            raise ValueError(f"ohara_amd runs the decode path in bfloat16 only (got {dtype})")
        if device is not None:
            want = torch.device(device)
            if want.type != self.device.type or (want.index is not None and want.index != (self.device.index or 0)):
                raise ValueError(f"ohara_amd: the model lives on {self.device}; build it on {want} instead of moving it")
        return self

    def parameters(self):
        yield self.token_emb
        yield self.final_norm
        yield self.w_vocab.data
        for L in self.layers:
            for k in ("wqkv", "wo", "wgu", "wdown"):
                yield L[k].data
            yield L["norm1"]
            yield L["norm2"]

    def build_kv_cache(self, batch_size: int = 1, int8: bool = False) -> list[KVCache]:
        """ohara/models/llama.py:325-348; ``int8=True`` builds the int8 caches of
        ohara/modules/kv_cache.py:47-73 (the reference leaves that choice to whoever constructs the
        caches)."""
        if batch_size < 1:
            raise ValueError("batch_size must be at least 1")
        c = self.config
        shape = (batch_size, c.max_sequence_length, self.kv_heads, self.head_dim)
        return [KVCache(shape, c.max_sequence_length, i, device=self.device, dtype=BF16, int8=int8)
                for i in range(c.num_hidden_layers)]

    def default_n_split(self, batch: int) -> int:
        """Context chunks per (sequence, KV head) so that decode attention launches about
        four workgroups per CU (measured on d12, 6 KV heads, at batch 16 / 32 / 64: 6, 6 and 2-4
        chunks are the fastest, twice as many are slower); a chunk is never shorter than 128
        positions."""
        want = max(1, 1024 // max(1, batch * self.kv_heads))
        return max(1, min(want, self.config.max_sequence_length // 128, 64))

    def _get_buffers(self, batch: int, rows: int) -> _Buffers:
        key = (batch, rows)
        buf = self._buffers.get(key)
        if buf is None:
            # keep at most one prefill-sized set alive
            for k in [k for k in self._buffers if k[1] > k[0] and k != key]:
                del self._buffers[k]
            buf = _Buffers(self, batch, rows, self.default_n_split(batch))
            self._buffers[key] = buf
        return buf

    def _state_struct(self, buf: _Buffers, kv_cache, logits, history=None, valid_vocab=0,
                      seq_pos=None) -> OharaDecodeState:
        n = self.config.num_hidden_layers
        kc = (C.c_void_p * n)(*[c.key.data_ptr() for c in kv_cache])
        vc = (C.c_void_p * n)(*[c.value.data_ptr() for c in kv_cache])
        s = OharaDecodeState()
        s.batch, s.rows_cap, s.n_split, s.valid_vocab = buf.batch, buf.rows, buf.n_split, valid_vocab
        s.hist_cap = 0 if history is None else history.shape[0]
        s.prof_kernel = -1
        s.ids, s.x, s.q, s.attn, s.act = (t.data_ptr() for t in (buf.ids, buf.x, buf.q, buf.attn, buf.act))
        s.xn = 0 if buf.xn is None else buf.xn.data_ptr()
        s.logits = 0 if logits is None else logits.data_ptr()
        s.attn_ws, s.step_state = buf.attn_ws.data_ptr(), buf.step_state.data_ptr()
        s.history = 0 if history is None else history.data_ptr()
        s.kcache, s.vcache = C.cast(kc, C.POINTER(C.c_void_p)), C.cast(vc, C.POINTER(C.c_void_p))
        s._keep = (kc, vc)
        if len({c.int8 for c in kv_cache}) > 1:
            raise ValueError("all layers must use the same KV cache mode")
        if seq_pos is not None:
            s.seq_pos = seq_pos.data_ptr()
            s._keep = (kc, vc, seq_pos)
        if kv_cache[0].int8:
            stats = [(C.c_void_p * n)(*[c.stats.data_ptr() for c in kv_cache])]
            s.kv_int8 = 1
            s.kvstats = C.cast(stats[0], C.POINTER(C.c_void_p))
            kvw = self.kv_heads * self.head_dim
            if buf.kstage is None:
                buf.kstage = torch.empty(buf.rows, kvw, dtype=BF16, device=self.device)
                buf.vstage = torch.empty(buf.rows, kvw, dtype=BF16, device=self.device)
            s.kstage, s.vstage = buf.kstage.data_ptr(), buf.vstage.data_ptr()
            if buf.rows >= 16 * buf.batch:  # calls with many positions attend over a dequantised copy
                shape = (kv_cache[0].key.shape[0], self.config.max_sequence_length, self.kv_heads, self.head_dim)
                if buf.kdeq is None or tuple(buf.kdeq.shape) != shape:
                    buf.kdeq = torch.empty(shape, dtype=BF16, device=self.device)
                    buf.vdeq = torch.empty(shape, dtype=BF16, device=self.device)
                s.kdeq, s.vdeq = buf.kdeq.data_ptr(), buf.vdeq.data_ptr()
            s._keep = (kc, vc, *stats) if seq_pos is None else (kc, vc, seq_pos, *stats)
        return s

    def forward(self, x: torch.Tensor, kv_cache: list | None = None, position_ids=None, *, last_only: bool = False,
                seq_pos: torch.Tensor | None = None):
        """ohara/models/llama.py:279-323.  Returns logits (B, S, V) in bf16, or (B, 1, V)
        with ``last_only=True`` (an extension: the generate loops read only the last row).

        A second extension: ``position_ids`` may hold one cache position per sequence (a list, or a
        1-D tensor with more than one element) - the reference has a single scalar for the whole
        batch (llama.py:287-299), which forces equal lengths.  ``seq_pos`` optionally supplies the same
        positions as an int32 device tensor that the caller keeps up to date (no upload per call)."""
        c = self.config
        if x.ndim != 2:
            raise ValueError("input token IDs must have shape (batch, sequence)")
        ragged = None
        if isinstance(position_ids, (list, tuple)):
            ragged = [int(p) for p in position_ids]
        elif isinstance(position_ids, torch.Tensor):
            if position_ids.ndim == 1 and position_ids.numel() > 1:
                ragged = [int(p) for p in position_ids.tolist()]
            elif position_ids.numel() != 1:
                raise ValueError("position_ids must be a scalar cache position")
            else:
                position_ids = int(position_ids.item())
        B, S = x.shape
        if ragged is not None:
            if kv_cache is None:
                raise ValueError("position_ids is only valid when using a KV cache")
            if len(kv_cache) != c.num_hidden_layers:
                raise ValueError("KV cache must contain one entry per model layer")
            if len(ragged) != B:
                raise ValueError("one position per sequence is required")
            if min(ragged) < 0:
                raise ValueError("a non-negative position_ids is required with KV cache")
            if S < 1:
                raise ValueError("input sequence cannot be empty")
            if max(ragged) + S > c.max_sequence_length:
                raise ValueError("input exceeds max_sequence_length")
            ends = [cache._reserve_ragged(B, S, ragged) for cache in kv_cache]
            if seq_pos is None:
                seq_pos = torch.tensor(ragged, dtype=torch.int32).to(self.device)
        else:
            start_pos = 0
            if kv_cache is not None:
                if len(kv_cache) != c.num_hidden_layers:
                    raise ValueError("KV cache must contain one entry per model layer")
                if position_ids is None or position_ids < 0:
                    raise ValueError("a non-negative position_ids is required with KV cache")
                start_pos = position_ids
            elif position_ids is not None:
                raise ValueError("position_ids is only valid when using a KV cache")
            if S < 1:
                raise ValueError("input sequence cannot be empty")
            if start_pos + S > c.max_sequence_length:
                raise ValueError("input exceeds max_sequence_length")
            if kv_cache is None:
                # Uncached causal forward == a fresh cache filled from position 0.
                kv_cache = self.build_kv_cache(B)
            ends = [cache._reserve(B, S, start_pos) for cache in kv_cache]
            seq_pos = None

        _check_ids_on_host(x, c.vocab_size)
        rows = B * S
        buf = self._get_buffers(B, rows)
        buf.ids.copy_(x.reshape(-1).to(device=self.device, dtype=torch.int64))
        out_rows = B if last_only else rows
        logits = torch.empty(out_rows, c.vocab_size, dtype=BF16, device=self.device)
        st = self._state_struct(buf, kv_cache, logits, seq_pos=seq_pos)
        mode = _lib.OHARA_LOGITS_LAST if last_only else _lib.OHARA_LOGITS_ALL
        check(lib().ohara_llama_forward(C.byref(self._c_model), C.byref(st), S, 0 if ragged is not None else start_pos, 0,
                                        mode, 0, torch.cuda.current_stream().cuda_stream), "llama_forward")
        for cache, end in zip(kv_cache, ends):
            if ragged is not None:
                cache._commit_ragged(B, end)
            else:
                cache._commit(B, end)
        return logits.view(B, 1 if last_only else S, c.vocab_size)

    __call__ = forward

    # -- device-resident greedy loop --------------------------------------------------

    def session(self, batch: int, max_new_tokens: int, valid_vocab: int = 0, kv_cache: list | None = None,
                persistent: bool | None = None, sampling=None, u=None):
        return DecodeSession(self, batch, max_new_tokens, valid_vocab, kv_cache, persistent, sampling, u)

    def supports_persistent(self, batch: int) -> bool:
        """Shapes the single-launch decode kernel covers."""
        c = self.config
        g = c.num_attention_heads // self.kv_heads
        return (batch <= 16 and self.head_dim in (64, 128) and g in (1, 2, 4) and c.hidden_size <= 1024
                and c.hidden_size % 8 == 0 and c.intermediate_size % 8 == 0)

    @torch.no_grad()
    def generate_greedy(self, prompt_ids: torch.Tensor, steps: int, *, use_graph: bool = True,
                        valid_vocab: int = 0, kv_cache: list | None = None,
                        persistent: bool | None = None) -> torch.Tensor:
        """Prefill the prompt, then ``steps`` greedy tokens with no host round trip per
        token (the loop of ohara/chat_engine.py:395-405 for a batch of equal-length
        prompts).  Returns the generated ids (B, steps)."""
        B, P = prompt_ids.shape
        if steps < 1:
            return torch.zeros(B, 0, dtype=torch.int64, device=self.device)
        sess = self.session(B, steps, valid_vocab, kv_cache, persistent)
        sess.prefill(prompt_ids)
        sess.run(steps - 1, use_graph=use_graph)
        return sess.tokens()


class DecodeSession:
    """One batch of equal-length sequences decoded greedily on the device: prefill once,
    then one ``ohara_llama_forward`` (S = 1, device-side position, fused selection) per
    token, replayed from a HIP graph.  The host reads tokens only when it asks for them."""

    PERSISTENT_SPLITS = 16

    def __init__(self, model: Llama, batch: int, max_new_tokens: int, valid_vocab: int = 0, kv_cache=None,
                 persistent: bool | None = None, sampling=None, u=None):
        """``sampling``: an object with temperature / top_k / top_p (a ``SamplingConfig``); None or
        temperature 0 selects greedily.  ``u``: (max_new_tokens, batch) fp32 uniform draws in [0, 1),
        row t for the t-th generated token (ohara/chat_engine.py:51-82 with multinomial replaced by
        inverse-CDF sampling); drawn from torch's generator when omitted."""
        self.model, self.batch = model, batch
        self.sampling = sampling if (sampling is not None and sampling.temperature > 0) else None
        self.u = None
        if self.sampling is not None:
            rows = max(max_new_tokens, 1)
            if u is None:
                u = torch.rand(rows, batch, device=model.device, dtype=torch.float32)
            if u.shape != (rows, batch):
                raise ValueError("u must have shape (max_new_tokens, batch)")
            self.u = u.to(device=model.device, dtype=torch.float32).contiguous()
            # the sampler's workgroups meet in a buffer of this session's own: sessions on other streams may overlap
            self._sample_ws = ops.sample_workspace(model.device)
        if persistent is None:
            # measured on d12: the single launch wins up to eight sequences (0.40 ms against 0.48 ms
            # per step at 4, 0.49 against 0.49 at 8); beyond that the kernel chain is faster (0.52
            # against 0.64 ms at 12)
            persistent = model.supports_persistent(batch) and batch <= 8
        elif persistent and not model.supports_persistent(batch):
            raise ValueError("the persistent decode kernel does not cover this shape")
        self._pws = None
        self.spin_limit = 0  # bound of the persistent kernel's barrier waits (0 = the library's default)
        self.cache = kv_cache if kv_cache is not None else model.build_kv_cache(batch)
        self._nwg = torch.cuda.get_device_properties(model.device).multi_processor_count
        if persistent and self.cache[0].int8:
            # the int8 cache is read (and the appended row quantised) by the polled builds of the kernel only
            persistent = lib().ohara_persistent_polled(C.byref(model._c_model), batch, self._nwg) > 0
        self.persistent = persistent
        self.valid_vocab = valid_vocab
        self.history = torch.zeros(max(max_new_tokens, 1), batch, dtype=torch.int64, device=model.device)
        self.logits = torch.empty(batch, model.config.vocab_size, dtype=BF16, device=model.device)
        self.produced = 0
        self.pos = 0
        self.graph = None
        self.graph_multi = None
        self._dst = None
        self._dbuf = None

    def prefill(self, prompt_ids: torch.Tensor) -> None:
        m, B = self.model, self.batch
        if prompt_ids.ndim != 2 or prompt_ids.shape[0] != B:
            raise ValueError("input token IDs must have shape (batch, sequence)")
        P = prompt_ids.shape[1]
        if P < 1:
            raise ValueError("input sequence cannot be empty")
        if P > m.config.max_sequence_length:
            raise ValueError("input exceeds max_sequence_length")
        _check_ids_on_host(prompt_ids, m.config.vocab_size)
        for cc in self.cache:
            cc._reserve(B, P, 0)
        pbuf = m._get_buffers(B, B * P)
        pbuf.ids.copy_(prompt_ids.reshape(-1).to(device=m.device, dtype=torch.int64))
        st = m._state_struct(pbuf, self.cache, self.logits, valid_vocab=self.valid_vocab)
        st.step_state = 0
        check(lib().ohara_llama_forward(C.byref(m._c_model), C.byref(st), P, 0, 0, _lib.OHARA_LOGITS_LAST,
                                        0 if self.sampling else 1, torch.cuda.current_stream().cuda_stream), "prefill")
        if self.sampling:
            ops.sample_topk_topp(self.logits, self.sampling.temperature, self.sampling.top_k, self.sampling.top_p,
                                 self.u[0], self.valid_vocab or None, out=pbuf.ids[:B])
        for cc in self.cache:
            cc._commit(B, P)
        self.pos = P
        # the decode buffers (fed ids, step state, activations) belong to this session alone: their
        # addresses are baked into the captured graph, so neither another session of the same batch
        # nor an eager model(...) call may share them
        dbuf = self._dbuf
        if dbuf is None:
            dbuf = _Buffers(m, B, B, m.default_n_split(B))
        self.history[0].copy_(pbuf.ids[:B])
        dbuf.ids.copy_(pbuf.ids[:B])
        dbuf.step_state.copy_(torch.tensor([P, 1, 0, 0], dtype=torch.int32))
        self.produced = 1
        if self._dst is not None:
            return  # a restarted session: buffers, workspace and the captured graph stay as they are
        self._dbuf = dbuf
        self._dst = m._state_struct(dbuf, self.cache, self.logits, history=self.history, valid_vocab=self.valid_vocab)
        self.graph = None
        if self.persistent:
            self._dst.n_split = self.PERSISTENT_SPLITS
            nbytes = lib().ohara_persistent_workspace_bytes(C.byref(m._c_model), B, self.PERSISTENT_SPLITS, self._nwg)
            if nbytes < 0:
                raise RuntimeError("persistent workspace query failed")
            if self._pws is None or self._pws.numel() < nbytes:
                self._pws = torch.zeros(nbytes, dtype=torch.uint8, device=m.device)
            self._err_off = lib().ohara_persistent_error_offset(C.byref(m._c_model), B, self.PERSISTENT_SPLITS,
                                                                self._nwg)
            self._prof_off = lib().ohara_persistent_profile_offset(C.byref(m._c_model), B, self.PERSISTENT_SPLITS,
                                                                   self._nwg)
            torch.cuda.current_stream().synchronize()
            check(lib().ohara_llama_decode_persistent(C.byref(m._c_model), C.byref(self._dst), self._pws.data_ptr(),
                                                      self._nwg, 1, 1, 0, torch.cuda.current_stream().cuda_stream),
                  "persistent init")

    def restart(self, u: torch.Tensor | None = None) -> None:
        """Forget the sequences decoded so far and make the session ready for another ``prefill``:
        the caches, buffers, workspace and the captured graph are kept (the graph reads the position
        and the fed ids from device memory, so it serves any later run), only the bookkeeping is
        reset.  Positions beyond a sequence's length are never read, so the caches need no clearing.
        ``u``: new uniform draws for a sampling session, (rows <= max_new_tokens, batch)."""
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

    def feed(self, ids: torch.Tensor) -> None:
        """Replace the ids the next step consumes (one per sequence) - teacher forcing: the step then
        continues the sequences with these tokens instead of the ones the last step selected.  The
        history keeps what was selected."""
        if self._dbuf is None:
            raise RuntimeError("prefill first")
        ids = ids.reshape(-1)
        if ids.numel() != self.batch:
            raise ValueError("one id per sequence is required")
        _check_ids_on_host(ids.view(1, -1), self.model.config.vocab_size)
        self._dbuf.ids[: self.batch].copy_(ids.to(device=self.model.device, dtype=torch.int64))

    def _launch_step(self) -> None:
        m = self.model
        stream = torch.cuda.current_stream().cuda_stream
        greedy = 0 if self.sampling else 1
        if self.persistent:
            check(lib().ohara_llama_decode_persistent(C.byref(m._c_model), C.byref(self._dst), self._pws.data_ptr(),
                                                      self._nwg, 0, greedy, int(self.spin_limit), stream), "persistent decode step")
        else:
            check(lib().ohara_llama_forward(C.byref(m._c_model), C.byref(self._dst), 1, 0, 1, _lib.OHARA_LOGITS_LAST,
                                            greedy, stream), "decode step")
        if self.sampling:
            # the sampler does the selection kernel's bookkeeping (next ids, history, position)
            ops.sample_topk_topp(self.logits, self.sampling.temperature, self.sampling.top_k, self.sampling.top_p,
                                 self.u, self.valid_vocab or None, out=self._dbuf.ids[: self.batch],
                                 history=self.history, step_state=self._dbuf.step_state, u_per_step=True, workspace=self._sample_ws)

    def error_word(self):
        """The persistent kernel's sticky error word as a one-element int32 device view (None for the
        kernel chain, which has no barrier waits): non-zero once a barrier wait has expired."""
        if self.persistent and self._pws is not None:
            return self._pws[self._err_off : self._err_off + 4].view(torch.int32)
        return None

    def check_error(self) -> None:
        """Raise if a barrier wait of the persistent kernel expired (synchronises)."""
        if self.persistent and self._pws is not None:
            word = self._pws[self._err_off : self._err_off + 4].view(torch.int32).cpu()
            if int(word[0]) != 0:
                raise RuntimeError("persistent decode kernel: a grid barrier wait expired")

    def reset_error(self) -> None:
        """Recover from an expired barrier wait: re-initialise the workspace (barrier counters, launch
        count and the sticky error word).  A workgroup whose wait expired runs ahead, so arrivals of
        different barriers mix in the counters and later barriers would never release; the counters
        cannot be kept.  Synchronises."""
        if self.persistent and self._pws is not None:
            torch.cuda.current_stream().synchronize()
            check(lib().ohara_llama_decode_persistent(C.byref(self.model._c_model), C.byref(self._dst), self._pws.data_ptr(),
                                                      self._nwg, 1, 1, 0, torch.cuda.current_stream().cuda_stream),
                  "persistent init")

    def phase_clocks(self, workgroup: int | None = 0) -> torch.Tensor:
        """Clock samples (constant 100 MHz counter) that thread 0 of ``workgroup`` took at the phase
        boundaries of the last step run with ``step(prof_kernel=-2)`` (measurement aid); ``None``: one
        row per workgroup."""
        if workgroup is None:
            off = self._prof_off
            return self._pws[off : off + 8192 * self._nwg].view(torch.int64).cpu().view(self._nwg, 1024)
        off = self._prof_off + workgroup * 8192
        return self._pws[off : off + 8192].view(torch.int64).cpu()

    def _room(self, n: int) -> None:
        if self._dst is None:
            raise RuntimeError("prefill first")
        if self.pos + n > self.model.config.max_sequence_length:
            raise ValueError("input exceeds max_sequence_length")
        if self.produced + n > self.history.shape[0]:
            raise ValueError("max_new_tokens exceeded")

    def step(self, prof_kernel: int = -1, prof_start=None, prof_stop=None) -> None:
        """One eager decode step (enqueue only)."""
        self._room(1)
        stream = torch.cuda.current_stream().cuda_stream
        if self.persistent:
            # a single launch: bracket it directly
            if prof_start is not None:
                check(lib().ohara_event_record(prof_start, stream), "event record")
            self._dst.prof_kernel = -2 if prof_kernel == -2 else -1
            self._launch_step()
            self._dst.prof_kernel = -1
            if prof_stop is not None:
                check(lib().ohara_event_record(prof_stop, stream), "event record")
        else:
            self._dst.prof_kernel = prof_kernel
            self._dst.prof_start, self._dst.prof_stop = prof_start, prof_stop
            self._launch_step()
            self._dst.prof_kernel = -1
        self._advance(1)

    def _advance(self, n: int) -> None:
        self.pos += n
        self.produced += n
        for cc in self.cache:
            cc._commit(self.batch, self.pos)

    GRAPH_STEPS = 8  # steps in the second captured graph: one graph launch then covers eight tokens

    def capture(self) -> None:
        """Record one decode step into a HIP graph (after one eager warm-up step), and GRAPH_STEPS
        steps into a second one: a step reads its position, fed ids and step index from device memory,
        so the same launches serve any later token, and a replay of the longer graph pays the host's
        launch of a graph once for eight tokens (measured at batch 1: 12 us per replay)."""
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
        if not use_graph:
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
