"""Checkpoint loading (host logic, no GPU): the architecture recovered from tensor shapes follows
ohara/chat_engine.py:129-245; the cases mirror tests/test_chat.py:419-430 and
tests/test_moe_grouped.py:365-472 of the reference, with state dicts of the reference's key names
and shapes built by the oracle's weight table."""

import json

import pytest
import torch

from oracle import llama_ref as R
from ohara_amd.checkpoint import (clean_state_dict, config_from_state_dict, load_checkpoint, loop_moe_to_grouped,
                                  strip_wrapper_prefixes)
from ohara_amd.llama import Config, rope_tables


def _state(cfg: Config, with_rotary=True):
    rcfg = R.RefConfig(**{k: getattr(cfg, k) for k in R.RefConfig.__dataclass_fields__ if hasattr(cfg, k)})
    st = {name: torch.zeros(shape) for name, shape, _ in R.weight_names(rcfg)}
    if cfg.weight_tying:
        st["vocab_proj.weight"] = st["token_emb.weight"]
    if with_rotary:
        d = cfg.hidden_size // cfg.num_attention_heads
        st["freq_cos"], st["freq_sin"] = rope_tables(d, 2 * cfg.max_sequence_length, cfg.rope_theta)
    return st


def _moe_cfg(**over):
    kw = dict(vocab_size=320, hidden_size=64, intermediate_size=28, max_sequence_length=64, num_hidden_layers=4,
              num_attention_heads=2, dropout=0.0, moe_num_experts=64, moe_experts_per_tok=4, moe_grouped=True,
              moe_num_shared_experts=1, moe_gate_fn="sigmoid")
    kw.update(over)
    return Config(**kw)


@pytest.mark.parametrize("name", ["dense", "gqa", "moe"])
def test_reference_made_state_dicts(tmp_path, name):
    """State dicts the reference's own Llama produced (tests/golden/llama_tiny_*.pt, with the Config each
    was built from): the architecture is recovered from the tensor shapes alone, through the raw dict
    and through both on-disk formats.  What leaves no trace in the weights (top-k, gate function, rope
    theta - which the reference does not recover either, chat_engine.py:129-245) is passed in."""
    from _fixtures import load_fixture

    fx = load_fixture(f"llama_tiny_{name}.pt")
    want = Config(**{k: v for k, v in fx["config"].items() if k in Config.__dataclass_fields__})
    hints = dict(moe_experts_per_tok=want.moe_experts_per_tok, moe_gate_fn=want.moe_gate_fn) if name == "moe" else {}
    got = config_from_state_dict(fx["state"], **hints)
    for f in Config.__dataclass_fields__:
        if f not in ("rope_theta", "dropout", "init_style"):
            assert getattr(got, f) == getattr(want, f), f
    wrapped = {"model": {"module._orig_mod." + k: v for k, v in fx["state"].items()}, "idx": 7}
    path = tmp_path / "ckpt.pt"
    torch.save(wrapped, path)
    cfg2, state2 = load_checkpoint(str(path), **hints)
    assert cfg2 == got and set(state2) == set(clean_state_dict(fx["state"]))
    for k, v in state2.items():
        assert torch.equal(v, fx["state"][k]), k


def test_dense_config_round_trips():
    cfg = Config(vocab_size=300, hidden_size=64, intermediate_size=128, max_sequence_length=96, num_hidden_layers=3,
                 num_attention_heads=2, dropout=0.0)
    assert config_from_state_dict(_state(cfg)) == cfg
    gqa = Config(vocab_size=300, hidden_size=64, intermediate_size=128, max_sequence_length=32, num_hidden_layers=2,
                 num_attention_heads=4, num_key_value_heads=2, dropout=0.0, weight_tying=True)
    assert config_from_state_dict(_state(gqa)) == gqa


def test_grouped_moe_config_round_trips():
    cfg = _moe_cfg()
    assert config_from_state_dict(_state(cfg), moe_experts_per_tok=4, moe_gate_fn="sigmoid") == cfg
    cfg = _moe_cfg(moe_normalize_weights=False)
    got = config_from_state_dict(_state(cfg), moe_experts_per_tok=4, moe_gate_fn="sigmoid", moe_normalize_weights=False)
    assert got == cfg
    for shared in (0, 1, 2):
        got = config_from_state_dict(_state(_moe_cfg(moe_num_shared_experts=shared)), moe_experts_per_tok=4)
        assert got.moe_num_shared_experts == shared
    # top-k leaves no trace in the weights: the default comes back, not the 4 it was built with
    assert config_from_state_dict(_state(_moe_cfg())).moe_experts_per_tok == 2
    cfg = _moe_cfg(moe_layer_interval=4)
    got = config_from_state_dict(_state(cfg), moe_experts_per_tok=4, moe_gate_fn="sigmoid")
    assert got.moe_layer_interval == 4 and got == cfg


def _loop_state(num_experts=8, layers=2, d=64, f=32):
    cfg = Config(vocab_size=320, hidden_size=d, intermediate_size=f, max_sequence_length=64, num_hidden_layers=layers,
                 num_attention_heads=2, dropout=0.0)
    st = {k: v for k, v in _state(cfg).items() if ".ff." not in k}
    g = torch.Generator().manual_seed(0)
    for l in range(layers):
        p = f"layers.{l}.ff."
        for e in range(num_experts):
            for nm, shape in (("up", (f, d)), ("gate", (f, d)), ("down", (d, f))):
                st[f"{p}experts.{e}.{nm}.weight"] = torch.randn(*shape, generator=g)
        st[p + "gate.weight"] = torch.randn(num_experts, d, generator=g)
        st[p + "router_bias"] = torch.zeros(num_experts)
    return st


def test_loop_moe_detected_and_restacked():
    st = _loop_state()
    got = config_from_state_dict(st, moe_gate_fn="sigmoid")
    assert got.moe_num_experts == 8 and not got.moe_grouped and got.moe_gate_fn == "sigmoid"
    assert got.intermediate_size == 32 and got.moe_layer_interval == 1
    grouped = loop_moe_to_grouped(st)
    assert grouped["layers.1.ff.w_gate"].shape == (8, 64, 32) and grouped["layers.1.ff.w_down"].shape == (8, 32, 64)
    assert torch.equal(grouped["layers.0.ff.w_up"][3], st["layers.0.ff.experts.3.up.weight"].t())
    assert torch.equal(grouped["layers.0.ff.router.weight"], st["layers.0.ff.gate.weight"])
    assert not any(".ff.experts." in k or k.endswith(".ff.gate.weight") for k in grouped)
    # the restacked layout is what the grouped branch recovers
    assert config_from_state_dict(grouped).moe_grouped


def test_wrapper_prefixes_and_missing_rotary():
    assert strip_wrapper_prefixes("module._orig_mod.layers.0.norm1.weight") == "layers.0.norm1.weight"
    assert strip_wrapper_prefixes("_orig_mod.module.module.norm.weight") == "norm.weight"
    cfg = Config(vocab_size=50, hidden_size=32, intermediate_size=64, max_sequence_length=16, num_hidden_layers=1,
                 num_attention_heads=2, dropout=0.0)
    wrapped = {"module._orig_mod." + k: v for k, v in _state(cfg).items()}
    assert config_from_state_dict(clean_state_dict(wrapped)) == cfg
    with pytest.raises(ValueError, match="no rotary buffer"):
        config_from_state_dict(_state(cfg, with_rotary=False))


def test_load_checkpoint_formats(tmp_path):
    from safetensors.torch import save_file

    cfg = Config(vocab_size=50, hidden_size=32, intermediate_size=64, max_sequence_length=16, num_hidden_layers=2,
                 num_attention_heads=2, dropout=0.0)
    st = {k: torch.randn_like(v) if v.is_floating_point() else v for k, v in _state(cfg).items()}
    torch.save({"model": {"module." + k: v for k, v in st.items()}, "idx": 7}, tmp_path / "a.pt")
    got_cfg, got = load_checkpoint(tmp_path / "a.pt")
    assert got_cfg == cfg and torch.equal(got["norm.weight"], st["norm.weight"])
    torch.save(st, tmp_path / "bare.pt")
    assert load_checkpoint(tmp_path / "bare.pt")[0] == cfg
    # exported layout: safetensors without the derived rotary buffers + config.json
    out = tmp_path / "export"
    out.mkdir()
    save_file({k: v.contiguous() for k, v in st.items() if not k.startswith("freq_")}, str(out / "model.safetensors"))
    from dataclasses import asdict

    (out / "config.json").write_text(json.dumps({"architecture": "ohara.models.llama.Llama", "iteration": 7, **asdict(cfg)}))
    got_cfg, got = load_checkpoint(out)
    assert got_cfg == cfg and "freq_cos" not in got and torch.equal(got["token_emb.weight"], st["token_emb.weight"])
    with pytest.raises(FileNotFoundError):
        load_checkpoint(tmp_path / "missing.pt")
