"""Checkpoint loading for the decode path: recover the architecture from a bare state dict and
build the matching model.

Mirrors ``config_from_state_dict`` / ``ChatEngine.from_checkpoint`` of the reference
(ohara/chat_engine.py:84-245, 275-329) and reads the safetensors + ``config.json`` layout written
by examples/export_safetensors.py:60-117.  Files are opened with loaders that execute nothing
from them (``torch.load(weights_only=True)``, safetensors, JSON); the reference's
``weights_only=False`` is deliberately not reproduced.
"""

from __future__ import annotations

import json
from dataclasses import fields
from pathlib import Path
from typing import Mapping

import torch

from .llama import Config

# DDP adds "module.", torch.compile adds "_orig_mod.", in either order (chat_engine.py:84-88).
_WRAPPER_PREFIXES = ("module.", "_orig_mod.")


def strip_wrapper_prefixes(key: str) -> str:
    """chat_engine.py:91-99."""
    changed = True
    while changed:
        changed = False
        for prefix in _WRAPPER_PREFIXES:
            if key.startswith(prefix):
                key = key[len(prefix):]
                changed = True
    return key


def clean_state_dict(state: Mapping[str, torch.Tensor]) -> dict[str, torch.Tensor]:
    """chat_engine.py:102-103."""
    return {strip_wrapper_prefixes(k): v for k, v in state.items()}


def _freq_cos(state):
    freq_cos = state.get("freq_cos")
    if freq_cos is None:
        raise ValueError("checkpoint has no rotary buffer; cannot infer head dimension")
    return freq_cos


def _head_count(state, projection: str) -> int:
    """chat_engine.py:115-121: heads = projection width / (2 * rotary table width)."""
    head_dim = int(_freq_cos(state).shape[-1]) * 2
    return int(state[f"layers.0.attn.{projection}.weight"].shape[0]) // head_dim


def _moe_layer_interval(moe_layers: list[int], num_layers: int) -> int:
    """chat_engine.py:124-126."""
    return moe_layers[1] - moe_layers[0] if len(moe_layers) > 1 else num_layers


def _tied(state) -> bool:
    return state["vocab_proj.weight"].data_ptr() == state["token_emb.weight"].data_ptr()


def config_from_state_dict(state: Mapping[str, torch.Tensor], *, moe_experts_per_tok: int = 2,
                           moe_gate_fn: str = "softmax", moe_normalize_weights: bool = True) -> Config:
    """chat_engine.py:129-245: every field from a tensor shape, except the head dimension (rotary
    buffer) and the routing choices top-k / gate function / weight normalisation, which leave no
    trace in the weights and must be supplied by the caller."""
    vocab_size, hidden_size = state["token_emb.weight"].shape
    num_layers = 1 + max(int(k.split(".")[1]) for k in state if k.startswith("layers."))
    max_len = int(_freq_cos(state).shape[0]) // 2
    heads, kv_heads = _head_count(state, "query"), _head_count(state, "key")
    common = dict(vocab_size=int(vocab_size), hidden_size=int(hidden_size), max_sequence_length=max_len,
                  num_hidden_layers=num_layers, num_attention_heads=heads,
                  num_key_value_heads=0 if kv_heads == heads else kv_heads, dropout=0.0, weight_tying=_tied(state))

    grouped = sorted({int(k.split(".")[1]) for k in state if k.startswith("layers.") and k.endswith(".ff.w_gate")})
    if grouped:
        first = grouped[0]
        num_experts, _, inter = state[f"layers.{first}.ff.w_gate"].shape  # (experts, dim, hidden)
        shared = state.get(f"layers.{first}.ff.shared_gate.weight")
        return Config(**common, intermediate_size=int(inter), moe_num_experts=int(num_experts),
                      moe_experts_per_tok=moe_experts_per_tok,
                      moe_layer_interval=_moe_layer_interval(grouped, num_layers), moe_grouped=True,
                      moe_num_shared_experts=int(shared.shape[0] // inter) if shared is not None else 0,
                      moe_gate_fn=moe_gate_fn, moe_normalize_weights=moe_normalize_weights)

    loop = sorted({int(k.split(".")[1]) for k in state if k.startswith("layers.") and ".ff.experts." in k})
    if loop:
        num_experts = 1 + max(int(k.split(".")[4]) for k in state if k.startswith(f"layers.{loop[0]}.ff.experts."))
        inter = state[f"layers.{loop[0]}.ff.experts.0.up.weight"].shape[0]
        interval = _moe_layer_interval(loop, num_layers)
    else:
        num_experts, inter, interval = 0, state["layers.0.ff.up.weight"].shape[0], 1
    return Config(**common, intermediate_size=int(inter), moe_num_experts=num_experts,
                  moe_experts_per_tok=moe_experts_per_tok if num_experts else 2, moe_layer_interval=interval,
                  moe_gate_fn=moe_gate_fn if num_experts else "softmax")


def loop_moe_to_grouped(state: Mapping[str, torch.Tensor]) -> dict[str, torch.Tensor]:
    """The per-expert module layout of ohara/modules/moe.py:51-52 (``ff.experts.N.{up,gate,down}``,
    router ``ff.gate``) restacked into the grouped layout of ohara/modules/moe_grouped.py
    (``ff.w_gate`` / ``ff.w_up`` (E, dim, hidden), ``ff.w_down`` (E, hidden, dim), ``ff.router``):
    both compute the same function, the kernels serve the grouped one."""
    out = {k: v for k, v in state.items() if ".ff.experts." not in k}
    layers = sorted({int(k.split(".")[1]) for k in state if ".ff.experts." in k})
    for l in layers:
        p = f"layers.{l}.ff."
        n = 1 + max(int(k.split(".")[4]) for k in state if k.startswith(p + "experts."))
        out[p + "w_gate"] = torch.stack([state[f"{p}experts.{e}.gate.weight"].t() for e in range(n)])
        out[p + "w_up"] = torch.stack([state[f"{p}experts.{e}.up.weight"].t() for e in range(n)])
        out[p + "w_down"] = torch.stack([state[f"{p}experts.{e}.down.weight"].t() for e in range(n)])
        out[p + "router.weight"] = out.pop(p + "gate.weight")
    return out


def loop_moe_config(config: Config) -> Config:
    """The grouped-form config that computes what ``MoE`` (ohara/modules/moe.py:65-98) computes for a
    config with ``moe_grouped=False``: no shared expert and sigmoid weights left as they are (the loop
    form has neither, llama.py:171-178 passes neither)."""
    from dataclasses import replace

    return replace(config, moe_grouped=True, moe_num_shared_experts=0, moe_normalize_weights=False)


def load_checkpoint(path, *, moe_experts_per_tok: int = 2, moe_gate_fn: str = "softmax",
                    moe_normalize_weights: bool = True):
    """-> (Config, state dict).  ``path`` is a ``.pt`` file holding a state dict (bare or under
    ``"model"``, chat_engine.py:307-308), a ``.safetensors`` file, or a directory with
    ``model.safetensors`` + ``config.json`` (export_safetensors.py:95-111)."""
    path = Path(path)
    if not path.exists():
        raise FileNotFoundError(f"checkpoint not found: {path}")
    cfg_json = None
    if path.is_dir():
        cfg_json = path / "config.json"
        path = path / "model.safetensors"
    elif path.suffix == ".safetensors" and (path.parent / "config.json").exists():
        cfg_json = path.parent / "config.json"
    if path.suffix == ".safetensors":
        from safetensors.torch import load_file

        state = clean_state_dict(load_file(str(path)))
    else:
        blob = torch.load(path, map_location="cpu", weights_only=True)
        state = clean_state_dict(blob.get("model", blob))
    if cfg_json is not None and cfg_json.exists():
        payload = json.loads(cfg_json.read_text(encoding="utf-8"))
        names = {f.name for f in fields(Config)}
        config = Config(**{k: v for k, v in payload.items() if k in names})
        if "vocab_proj.weight" not in state and config.weight_tying:  # the export drops aliases
            state["vocab_proj.weight"] = state["token_emb.weight"]
    else:
        config = config_from_state_dict(state, moe_experts_per_tok=moe_experts_per_tok, moe_gate_fn=moe_gate_fn,
                                        moe_normalize_weights=moe_normalize_weights)
    return config, state


def build_model(config: Config, state: Mapping[str, torch.Tensor], device="cuda"):
    """The kernel-backed model for a config: dense ``Llama`` or ``MoeLlama``."""
    if config.moe_num_experts > 0:
        from .moe import MoeLlama

        if not config.moe_grouped:
            state, config = loop_moe_to_grouped(state), loop_moe_config(config)
        return MoeLlama(config, state, device=device)
    from .llama import Llama

    return Llama(config, state, device=device)
