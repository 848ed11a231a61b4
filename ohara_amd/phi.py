"""Phi-2 (ohara/models/phi.py) on the HIP kernels: the reference's ``Phi`` call surface for the
cached decode path.

What differs from Llama, all of it as the reference has it: attention and the MLP run in parallel
off one LayerNorm (phi.py:147-151), every Linear has a bias, the MLP is fc1 -> new_gelu -> fc2
(phi.py:37-52), only ``int(rotary_dim * head_dim)`` features of a head rotate, in the half-split
layout, and the cache holds the UN-rotated keys: the rotation is applied to all cached keys at
every step, in fp32, inside the attention kernel (phi.py:95-104).

bf16 only (the reference's ``from_pretrained`` builds an fp16 model, phi.py:229-231; its tests run
fp32).  The Hub download of ``from_pretrained`` (phi.py:239) is not provided; a checkpoint already on
disk loads through ``Phi.from_local_checkpoint`` (same name mapping, same errors).
"""

from __future__ import annotations

import math
from dataclasses import dataclass

import torch

from . import ops
from ._lib import lib
from .llama import KVCache

BF16 = torch.bfloat16


@dataclass
class PhiConfig:
    """ohara/models/phi.py:23-34, same fields and defaults."""

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


def rope_cos_sin(num_positions: int, dims: int, base: float = 10000.0):
    """RoPE.create_cos_sin_theta (ohara/embeddings_pos/rotary.py:166-184) for fp32 inputs, positions
    0 .. num_positions-1: the same fp32 operations on the host, so the tables carry the same values."""
    half = dims // 2
    positions = torch.arange(0, num_positions, dtype=torch.float32)
    freqs = torch.exp(-torch.arange(0.0, half, dtype=torch.float32) * (math.log(base) / half))
    theta = positions.reshape(-1, 1) * freqs.reshape(1, -1)
    return torch.cos(theta), torch.sin(theta)


def huggingface_state_dict_map(num_hidden_layers: int) -> dict:
    """Reference parameter name -> microsoft/phi-2 checkpoint name
    (``Phi._huggingface_state_dict_map``, ohara/models/phi.py:208-233)."""
    mapping = {
        "wte.weight": "model.embed_tokens.weight",
        "ln.weight": "model.final_layernorm.weight",
        "ln.bias": "model.final_layernorm.bias",
        "lm_head.weight": "lm_head.weight",
        "lm_head.bias": "lm_head.bias",
    }
    for idx in range(num_hidden_layers):
        for suffix in ("weight", "bias"):
            mapping[f"layers.{idx}.ln.{suffix}"] = f"model.layers.{idx}.input_layernorm.{suffix}"
            for name in ("fc1", "fc2"):
                mapping[f"layers.{idx}.mlp.{name}.{suffix}"] = f"model.layers.{idx}.mlp.{name}.{suffix}"
            for name in ("q_proj", "k_proj", "v_proj", "dense"):
                mapping[f"layers.{idx}.mixer.{name}.{suffix}"] = f"model.layers.{idx}.self_attn.{name}.{suffix}"
    return mapping


def load_huggingface_state_dict(path: str, num_hidden_layers: int) -> dict:
    """Read the ``*.safetensors`` shards of a microsoft/phi-2 style checkpoint in the local directory
    ``path`` and return a state dict under the reference's names: what ``Phi.from_pretrained`` does
    after its download (ohara/models/phi.py:239-256), with the same error for an empty directory and
    for missing tensors.  Nothing is fetched from the network."""
    from pathlib import Path

    from safetensors import safe_open

    weights = {}
    for shard in sorted(Path(path).glob("*.safetensors")):
        with safe_open(str(shard), framework="pt", device="cpu") as reader:
            for key in reader.keys():
                weights[key] = reader.get_tensor(key)
    if not weights:
        raise FileNotFoundError(f"no safetensors shards found in {path}")
    mapping = huggingface_state_dict_map(num_hidden_layers)
    missing = sorted(set(mapping.values()) - set(weights))
    if missing:
        raise KeyError(f"checkpoint is missing expected tensors: {missing[:5]}")
    return {ours: weights[theirs] for ours, theirs in mapping.items()}


class Phi:
    """``Phi`` (ohara/models/phi.py:155-205): ``forward(x, kv_cache, position_ids)`` and
    ``build_kv_cache``.  ``state`` uses the reference's state-dict names."""

    attn_target_wgs = 512  # decode attention: workgroups aimed at when choosing the context chunks (measured: batch 2-16)

    def __init__(self, config: PhiConfig, state: dict, device="cuda", dtype=BF16):
        if dtype != BF16:
            raise ValueError("ohara_amd runs the decode path in bfloat16 only")
        c = config
        if c.hidden_size % c.num_attention_heads:
            raise ValueError("hidden_size must be divisible by num_attention_heads")
        self.head_dim = c.hidden_size // c.num_attention_heads
        self.rot = int(c.rotary_dim * self.head_dim)  # phi.py:69
        if self.rot < 2 or self.rot % 2:
            raise ValueError(f"RoPE dims must be a positive even number, got {self.rot}")  # rotary.py:118-121
        if self.head_dim % 8 or self.head_dim > 128 or c.hidden_size % 8:
            raise NotImplementedError("ohara_amd Phi: head_dim must be a multiple of 8 up to 128")
        if not c.bias:
            raise NotImplementedError("ohara_amd Phi: bias=False is not a configuration the reference builds")
        lib()  # fail loudly now if the HIP library is missing
        self.config, self.device, self.dtype = c, torch.device(device), dtype
        self.ff = c.multiple_of * c.hidden_size  # phi.py:138

        def dev(t):
            return t.detach().to(device=self.device, dtype=BF16).contiguous()

        self.wte = dev(state["wte.weight"])
        self.ln_w, self.ln_b = dev(state["ln.weight"]), dev(state["ln.bias"])
        self.lm_head = ops.pack_linear(dev(state["lm_head.weight"]))
        self.lm_bias = dev(state["lm_head.bias"])
        cos, sin = rope_cos_sin(c.max_sequence_length, self.rot)
        self.cos, self.sin = cos.to(self.device).contiguous(), sin.to(self.device).contiguous()
        self.layers = []
        for i in range(c.num_hidden_layers):
            p = f"layers.{i}."
            # one packed [q; k; v; fc1] weight: the four projections read the same normalised rows
            # (phi.py:81-83, :50), so they are one launch
            names = ("mixer.q_proj", "mixer.k_proj", "mixer.v_proj", "mlp.fc1")
            w_in = torch.cat([dev(state[p + n + ".weight"]) for n in names])
            b_in = torch.cat([dev(state[p + n + ".bias"]) for n in names])
            self.layers.append(dict(
                ln_w=dev(state[p + "ln.weight"]), ln_b=dev(state[p + "ln.bias"]),
                w_in=ops.pack_linear(w_in), b_in=b_in.contiguous(),
                dense=ops.pack_linear(dev(state[p + "mixer.dense.weight"])), dense_b=dev(state[p + "mixer.dense.bias"]),
                fc2=ops.pack_linear(dev(state[p + "mlp.fc2.weight"])), fc2_b=dev(state[p + "mlp.fc2.bias"]),
            ))
            del w_in
        torch.cuda.synchronize(self.device)
        self._bufs: dict = {}

    supports_last_only = True  # forward(..., last_only=True) computes the last row of logits only

    def eval(self):
        return self

    def to(self, *args, **kwargs):
        return self

    @classmethod
    def from_local_checkpoint(cls, path: str, config: PhiConfig | None = None, device="cuda") -> "Phi":
        """``Phi.from_pretrained`` (ohara/models/phi.py:235-256) for a checkpoint that is already on
        disk: the safetensors shards in ``path`` under microsoft/phi-2's tensor names, cast to bf16
        (the reference builds an fp16 model)."""
        config = config or PhiConfig()
        return cls(config, load_huggingface_state_dict(path, config.num_hidden_layers), device=device)

    def build_kv_cache(self, batch_size: int = 1, int8: bool = False) -> list[KVCache]:
        """phi.py:189-202; ``int8=True`` builds the int8 caches of ohara/modules/kv_cache.py:15-32."""
        if batch_size < 1:
            raise ValueError("batch_size must be at least 1")  # phi.py:190-191
        c = self.config
        shape = (batch_size, c.max_sequence_length, c.num_attention_heads, self.head_dim)
        return [KVCache(shape, c.max_sequence_length, i, device=self.device, dtype=BF16, int8=int8)
                for i in range(c.num_hidden_layers)]

    def _buffers(self, rows: int):
        b = self._bufs.get(rows)
        if b is None:
            if len(self._bufs) > 4:
                self._bufs.clear()
            d = self.config.hidden_size
            new = lambda n: torch.empty(rows, n, dtype=BF16, device=self.device)
            b = dict(x=[new(d), new(d)], h=new(d), q=new(d), attn=new(d), mixer=new(d), act=new(self.ff))
            # single-token calls: the context of a (sequence, head) is spread over up to 16 workgroups,
            # aiming at about 512 workgroups of at least 64 positions
            heads = rows * self.config.num_attention_heads
            b["ns"] = max(1, min(16, self.config.max_sequence_length // 64, -(-self.attn_target_wgs // heads)))
            b["ws"] = ops.phi_attn_workspace(rows, self.config.num_attention_heads, self.head_dim, b["ns"], self.device)
            self._bufs[rows] = b
        return b

    @torch.no_grad()
    def forward(self, x: torch.Tensor, kv_cache: list | None = None, position_ids=None, *, pos_dev=None,
                last_only: bool = False) -> torch.Tensor:
        """Logits (B, S, vocab) for the tokens not cached yet (phi.py:170-186).  Without a cache the
        tokens run through a scratch cache from position 0, which is the causal forward.  ``pos_dev``
        (int32 device scalar, S == 1) lets the kernels read the position on the device, for graph
        replay; the caller advances it.  ``last_only`` computes the last row of logits only."""
        c = self.config
        if kv_cache is not None and len(kv_cache) != c.num_hidden_layers:
            raise ValueError("KV cache must contain one entry per model layer")
        if x.dim() != 2:
            raise ValueError("x must be (batch, seq_len) token ids")
        B, S = x.shape
        if kv_cache is None:
            if S > c.max_sequence_length:
                raise ValueError("input exceeds max_sequence_length")
            kv_cache, start = self.build_kv_cache(B), 0
        else:
            if position_ids is None:
                raise ValueError("position_ids is required when using a KV cache")  # phi.py:92-93
            start = int(position_ids)
        if len({bool(getattr(cache, "int8", False)) for cache in kv_cache}) > 1:
            raise ValueError("all layers must use the same KV cache mode")
        ends = [cache._reserve(B, S, start) for cache in kv_cache]
        logits = self._run(x.reshape(-1).to(device=self.device, dtype=torch.int64), B, S, kv_cache, start, pos_dev, last_only)
        for cache, end in zip(kv_cache, ends):
            cache._commit(B, end)
        return logits.view(B, 1 if last_only else S, c.vocab_size)

    def _run(self, ids, B, S, kv_cache, start, pos_dev, last_only):
        """The launches of one forward call; no host-side state, so it can be captured in a graph."""
        c = self.config
        rows, d, H, D = B * S, c.hidden_size, c.num_attention_heads, self.head_dim
        buf = self._buffers(rows)
        cur, nxt = buf["x"]
        ops.embed(ids, self.wte, out=cur)
        int8 = kv_cache[0].int8
        for L, cache in zip(self.layers, kv_cache):
            ops.layernorm(cur, L["ln_w"], L["ln_b"], c.eps, out=buf["h"])
            if int8:
                # kv_cache.py:94-118 with quantisation: the new (un-rotated) rows are quantised into the cache and
                # attention runs over what the reference's cache read returns - the dequantised prefix, the new rows
                # included - as a bf16 working copy (the rotary attention kernel reads bf16 rows)
                sk = torch.empty(B, S, H, D, dtype=BF16, device=self.device)
                sv = torch.empty_like(sk)
                ops.phi_block_in(buf["h"], None, None, c.eps, L["w_in"], L["b_in"], d, self.ff, B, S, 0, sk, sv, buf["q"],
                                 buf["act"])
                ops.kv_quant_append(sk, sv, cache, start, pos_dev=pos_dev)
                # (with the position on the device - a captured step - the copy covers the cache's whole capacity:
                # rows past the live prefix are never read)
                live = c.max_sequence_length if pos_dev is not None else start + S
                kd = ops.kv_dequant(cache, "key", B, live)
                vd = ops.kv_dequant(cache, "value", B, live)
                ops.phi_attn(buf["q"], kd, vd, self.cos, self.sin, self.rot, B, S, H, D, start, pos_dev, out=buf["attn"],
                             n_split=buf["ns"] if S == 1 else 1, workspace=buf["ws"])
            else:
                ops.phi_block_in(buf["h"], None, None, c.eps, L["w_in"], L["b_in"], d, self.ff, B, S, start, cache.key,
                                 cache.value, buf["q"], buf["act"], pos_dev)
                ops.phi_attn(buf["q"], cache.key, cache.value, self.cos, self.sin, self.rot, B, S, H, D, start, pos_dev,
                             out=buf["attn"], n_split=buf["ns"] if S == 1 else 1, workspace=buf["ws"])
            ops.linear_bias(buf["attn"], L["dense"], L["dense_b"], out=buf["mixer"])
            ops.linear_bias(buf["act"], L["fc2"], L["fc2_b"], "add2", add1=buf["mixer"], add2=cur, out=nxt)
            cur, nxt = nxt, cur
        src = cur.view(B, S, d)[:, -1].contiguous() if (last_only and S > 1) else cur
        hn = ops.layernorm(src, self.ln_w, self.ln_b, c.eps)
        return ops.linear_bias(hn, self.lm_head, self.lm_bias)

    __call__ = forward

    @torch.no_grad()
    def generate_greedy(self, prompt_ids: torch.Tensor, steps: int, *, use_graph: bool = True,
                        int8: bool = False) -> torch.Tensor:
        """Prefill the prompt, then ``steps`` greedy tokens with no host round trip per token: the
        cache position lives on the device and one decode step (all launches of ``_run`` plus the
        arg-max that feeds the next step) is captured once and replayed.  Returns (B, steps) ids.
        ``int8``: over the int8 caches of ohara/modules/kv_cache.py:15-32."""
        B, P = prompt_ids.shape
        c = self.config
        if steps < 1:
            return torch.zeros(B, 0, dtype=torch.int64, device=self.device)
        if P + steps - 1 > c.max_sequence_length:
            raise ValueError("input exceeds max_sequence_length")
        cache = self.build_kv_cache(B, int8=int8)
        logits = self.forward(prompt_ids, cache, 0, last_only=True).view(B, c.vocab_size)
        ids = ops.argmax(logits)
        history = torch.zeros(steps, B, dtype=torch.int64, device=self.device)
        history[0].copy_(ids)
        state = torch.tensor([P, 1, 0, 0], dtype=torch.int32, device=self.device)  # {pos, step, done, pad}

        def step():
            lg = self._run(ids, B, 1, cache, 0, state, False)
            ops.argmax(lg, next_ids=ids, history=history, step_state=state)  # also advances pos and step

        todo = steps - 1
        if use_graph and todo > 2:
            step()  # warm up outside the capture (allocations, lazy module loading)
            todo -= 1
            torch.cuda.synchronize(self.device)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                step()
            # the captured step is recorded, not run
            for _ in range(todo):
                graph.replay()
        else:
            for _ in range(todo):
                step()
        for cc in cache:
            cc._commit(B, P + steps - 1)
        return history.t().contiguous()
