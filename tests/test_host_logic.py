"""Host-side logic of the drop-in surface (no GPU): the generate loops of Inference and
ChatEngine, SamplingConfig, Config validation and the KVCache bookkeeping.  The loops are
exercised with dummy models; the token selection is injected (the oracle's samplers), since
the product's own samplers run on the GPU only.  Expected values are the literals of the
reference's tests (tests/test_inference.py:50-95, tests/test_chat.py:382-482,
tests/test_modules.py:46-79).
"""

import pytest
import torch

from oracle import sampling_ref as S


class DummyTokenizer:
    eos_token_id = 99

    def encode(self, _):
        return [1, 2, 3]

    def decode(self, tokens):
        return " ".join(str(t) for t in tokens)


class DummyModel:
    def to(self, *a, **k):
        return self

    def eval(self):
        return self

    def __call__(self, x, *args, **kwargs):
        logits = torch.zeros(x.shape[0], x.shape[1], 128)
        logits[:, :, 5] = 1.0
        return logits


class CachedDummyModel(DummyModel):
    class config:
        max_sequence_length = 6

    def __init__(self):
        self.calls = []

    def build_kv_cache(self):
        return object()

    def __call__(self, x, cache=None, position=0):
        self.calls.append((x.tolist(), cache is not None, position))
        return super().__call__(x)


def _ref_sampler(logits, temperature=1, top_p=0.0):
    return S.inference_sampler_ref(logits, temperature=temperature, top_p=top_p)


def test_inference_generate_call_pattern():
    from ohara_amd.inference import Inference

    inf = Inference(DummyModel(), DummyTokenizer(), device="cpu", max_new_tokens=3, use_kv_cache=False,
                    sampler_fn=_ref_sampler)
    assert inf.generate("hello", stream=False, temperature=0.0) == "1 2 3 5 5 5"
    model = CachedDummyModel()
    inf = Inference(model, DummyTokenizer(), device="cpu", max_new_tokens=10, use_kv_cache=True,
                    sampler_fn=_ref_sampler)
    # the context length (6) limits the three-token prompt to three generated tokens
    assert inf.generate("hello", stream=False, temperature=0.0) == "1 2 3 5 5 5"
    assert [len(c[0][0]) for c in model.calls] == [3, 1, 1]
    assert [c[2] for c in model.calls] == [0, 3, 4]
    assert all(c[1] for c in model.calls)


def test_inference_generate_validation_and_eos():
    from ohara_amd.inference import Inference

    class Empty(DummyTokenizer):
        def encode(self, _):
            return []

    with pytest.raises(ValueError, match="at least one token"):
        Inference(DummyModel(), Empty(), device="cpu", sampler_fn=_ref_sampler).generate("", stream=False)
    with pytest.raises(ValueError, match="cannot be negative"):
        Inference(DummyModel(), DummyTokenizer(), device="cpu", sampler_fn=_ref_sampler).generate(
            "hello", max_new_tokens=-1, stream=False)

    class Long(DummyTokenizer):
        def encode(self, _):
            return list(range(9))

    with pytest.raises(ValueError, match="exceeds model max_sequence_length"):
        Inference(CachedDummyModel(), Long(), device="cpu", sampler_fn=_ref_sampler).generate("x", stream=False)

    class EosTok(DummyTokenizer):
        eos_token_id = 5

    inf = Inference(DummyModel(), EosTok(), device="cpu", max_new_tokens=4, use_kv_cache=False,
                    sampler_fn=_ref_sampler)
    assert inf.generate("hello", stream=False, temperature=0.0) == "1 2 3"  # eos is not appended


# ---- ChatEngine -------------------------------------------------------------------------------


class CharTokenizer:
    """Char-level tokenizer with the chat markers, like the reference tests' FakeTokenizer."""

    SPECIALS = ["<|bos|>", "<|user_start|>", "<|user_end|>", "<|assistant_start|>", "<|assistant_end|>"]

    def __init__(self):
        chars = [chr(c) for c in range(32, 127)]
        self.vocab = {t: i for i, t in enumerate(self.SPECIALS + chars)}
        self.inv = {i: t for t, i in self.vocab.items()}
        self.bos_token_id = 0
        self.eos_token_id = 0

    def __len__(self):
        return len(self.vocab)

    def get_vocab(self):
        return dict(self.vocab)

    def encode(self, text, add_special_tokens=False):
        return [self.vocab[c] for c in text]

    def decode(self, ids, skip_special_tokens=True):
        return "".join(self.inv[i] for i in ids if not (skip_special_tokens and i < len(self.SPECIALS)))


class ForcedModel:
    """Emits one fixed token whatever the input; records the call pattern."""

    def __init__(self, vocab, forced, max_sequence_length=128, pad_to=None):
        class config:
            pass

        self.config = config
        config.max_sequence_length = max_sequence_length
        config.vocab_size = pad_to or vocab
        config.num_hidden_layers, config.hidden_size, config.num_attention_heads = 2, 32, 2
        self.forced = forced
        self.calls = []

    def to(self, *a, **k):
        return self

    def eval(self):
        return self

    def parameters(self):
        return [torch.zeros(10)]

    def build_kv_cache(self, batch_size=1):
        return ["cache"]

    def __call__(self, x, cache, position):
        self.calls.append((x.shape[1], position))
        logits = torch.zeros(x.shape[0], x.shape[1], self.config.vocab_size)
        logits[..., self.forced] = 5.0
        if self.config.vocab_size > 100:
            logits[..., -1] = 50.0  # a padded id that must never be sampled
        return logits


def _ref_chat_sampler(logits, config, generator=None, **kw):
    return S.sample_next_token_ref(logits, config.temperature, config.top_p, config.top_k, generator=generator)


def test_chat_engine_generate_loop():
    from ohara_amd.chat_engine import ChatEngine
    from ohara_amd.sampling import SamplingConfig

    tok = CharTokenizer()
    msgs = [{"role": "user", "content": "hi"}]
    # stop on <|assistant_end|> without emitting it (tests/test_chat.py:432-440)
    eng = ChatEngine(ForcedModel(len(tok), tok.vocab["<|assistant_end|>"]), tok, device="cpu", dtype=torch.float32,
                     sampler_fn=_ref_chat_sampler)
    assert list(eng.generate_stream(msgs, SamplingConfig(temperature=0.0, max_new_tokens=32))) == []
    # max_new_tokens (tests/test_chat.py:442-449) and the prefill-then-single-token pattern
    model = ForcedModel(len(tok), tok.vocab["x"])
    eng = ChatEngine(model, tok, device="cpu", dtype=torch.float32, sampler_fn=_ref_chat_sampler)
    assert eng.generate(msgs, SamplingConfig(temperature=0.0, max_new_tokens=5)) == "xxxxx"
    prompt_len = len(eng.render_prompt(msgs))
    assert [c[0] for c in model.calls] == [prompt_len, 1, 1, 1, 1]
    assert [c[1] for c in model.calls] == [0, prompt_len, prompt_len + 1, prompt_len + 2, prompt_len + 3]
    # streaming and batch generation agree (tests/test_chat.py:451-457)
    cfg = SamplingConfig(temperature=0.0, max_new_tokens=6)
    assert "".join(eng.generate_stream(msgs, cfg)) == eng.generate(msgs, cfg)
    # padded vocabulary ids are masked before sampling (chat_engine.py:398-399)
    eng = ChatEngine(ForcedModel(len(tok), tok.vocab["q"], pad_to=128), tok, device="cpu", dtype=torch.float32,
                     sampler_fn=_ref_chat_sampler)
    assert eng.generate(msgs, SamplingConfig(temperature=0.0, max_new_tokens=3)) == "qqq"
    info = eng.metadata()
    assert info["layers"] == 2 and info["hidden_size"] == 32 and info["context_length"] == 128
    assert info["vocab_size"] == 128 and info["parameters"] > 0


def test_chat_engine_prompt_window():
    from ohara_amd.chat_engine import ChatEngine

    tok = CharTokenizer()
    eng = ChatEngine(ForcedModel(len(tok), 7, max_sequence_length=64), tok, device="cpu", dtype=torch.float32,
                     sampler_fn=_ref_chat_sampler)
    messages = []
    for i in range(20):
        messages.append({"role": "user", "content": "u" * 20})
        messages.append({"role": "assistant", "content": f"a{i}" * 5})
    messages.append({"role": "user", "content": "final question"})
    ids = eng.render_prompt(messages)  # tests/test_chat.py:459-469
    assert len(ids) < 64 and ids[-1] == tok.vocab["<|assistant_start|>"]
    small = ChatEngine(ForcedModel(len(tok), 7, max_sequence_length=32), tok, device="cpu", dtype=torch.float32,
                       sampler_fn=_ref_chat_sampler)
    with pytest.raises(ValueError):
        small.render_prompt([{"role": "user", "content": "z" * 500}])


def test_sampling_config_validation():
    from ohara_amd.sampling import SamplingConfig

    assert SamplingConfig() == SamplingConfig(temperature=0.8, top_p=0.95, top_k=0, max_new_tokens=512)
    for kw in ({"temperature": -1.0}, {"top_p": 1.5}, {"top_k": -1}, {"max_new_tokens": 0}):
        with pytest.raises(ValueError):
            SamplingConfig(**kw)


def test_config_and_kv_cache_bookkeeping():
    from ohara_amd.llama import Config, KVCache, _validate_config

    assert Config().rope_theta == 100000 and Config().num_key_value_heads == 0
    for kw in ({"vocab_size": 1}, {"hidden_size": 30, "num_attention_heads": 4}, {"max_sequence_length": 1},
               {"num_attention_heads": 4, "num_key_value_heads": 3}, {"hidden_size": 12, "num_attention_heads": 4}):
        with pytest.raises(ValueError):
            _validate_config(Config(**kw))
    # what the kernels do not cover is refused when the model is built, before anything touches a GPU
    from ohara_amd.llama import Llama

    with pytest.raises(ValueError, match="biases"):
        Llama(Config(bias=True, moe_num_experts=4, moe_grouped=True), {})  # biases: dense feed-forwards only
    # a loop-form MoE config (llama.py:171-178) is served by the grouped kernels: no shared expert, sigmoid
    # weights as they are, expert weights restacked as (E, dim, hidden) / (E, hidden, dim)
    from ohara_amd.checkpoint import loop_moe_config, loop_moe_to_grouped

    lc = loop_moe_config(Config(moe_num_experts=4, moe_grouped=False, moe_num_shared_experts=2))
    assert lc.moe_grouped and lc.moe_num_shared_experts == 0 and not lc.moe_normalize_weights
    st = {f"layers.0.ff.experts.{e}.{n}.weight": torch.full((3, 2) if n != "down" else (2, 3), float(e))
          for e in range(4) for n in ("gate", "up", "down")}
    st["layers.0.ff.gate.weight"] = torch.zeros(4, 2)
    g = loop_moe_to_grouped(st)
    assert g["layers.0.ff.w_gate"].shape == (4, 2, 3) and g["layers.0.ff.w_down"].shape == (4, 3, 2)
    assert g["layers.0.ff.w_up"][2].eq(2.0).all() and "layers.0.ff.router.weight" in g and "layers.0.ff.gate.weight" not in g
    with pytest.raises(ValueError, match="bfloat16"):
        Llama(Config(), {}, dtype=torch.float16)
    c = KVCache((2, 8, 2, 4), 8, dtype=torch.float32)
    k = torch.randn(2, 3, 2, 4)
    ck, cv = c.forward(k, k * 2, 0)  # tests/test_modules.py:46-58
    assert torch.equal(ck, k) and torch.equal(cv, k * 2) and c.length == 3 and c.batch_size == 2
    ck, _ = c.forward(k[:, :1], k[:, :1], 3)
    assert ck.shape == (2, 4, 2, 4) and c.length == 4
    with pytest.raises(ValueError, match="sequential"):
        c.forward(k[:, :1], k[:, :1], 7)
    with pytest.raises(ValueError, match="max_sequence_length"):
        c.forward(torch.randn(2, 5, 2, 4), torch.randn(2, 5, 2, 4), 4)
    with pytest.raises(ValueError, match="matching shapes"):
        c.forward(k[:, :1], k[:, :2], 4)
    with pytest.raises(ValueError, match="cannot change"):
        c.forward(k[:1, :1], k[:1, :1], 4)
    with pytest.raises(ValueError, match="smaller than the input batch"):
        KVCache((1, 8, 2, 4), 8, dtype=torch.float32).forward(k, k, 0)
    q = KVCache((1, 8, 2, 4), 8, dtype=torch.float32, int8=True)  # kv_cache.py:64-74
    assert q.key.dtype == torch.int8 and q.value.dtype == torch.int8
    assert q.key_scale.shape == (1, 8, 2, 1) and q.value_min.dtype == torch.float32
    with pytest.raises(ValueError, match="sequential"):
        q.forward(k[:1, :1], k[:1, :1], 2)


def test_product_has_no_cpu_fallback():
    """Without a GPU the product refuses to sample instead of computing on the CPU."""
    from ohara_amd.sampling import SamplingConfig, sample_next_token

    if torch.cuda.is_available():
        pytest.skip("needs a machine without a GPU")
    with pytest.raises(RuntimeError, match="GPU only"):
        sample_next_token(torch.zeros(1, 1, 8), SamplingConfig(temperature=0.0))


def test_kv_cache_per_sequence_bookkeeping():
    """One length per sequence: the reference's checks (kv_cache.py:78-90), sequence by sequence."""
    from ohara_amd.llama import KVCache

    c = KVCache((3, 16, 2, 4), 16, dtype=torch.float32)
    ends = c._reserve_ragged(3, 2, [0, 0, 0])
    c._commit_ragged(3, ends)
    assert c.lengths == [2, 2, 2] and c.length == 2 and c.batch_size == 3
    c._commit_ragged(3, c._reserve_ragged(3, 1, [2, 2, 2]))
    c.lengths[1] = 7
    with pytest.raises(ValueError, match=r"expected position 7, got 3 \(sequence 1\)"):
        c._reserve_ragged(3, 1, [3, 3, 3])
    with pytest.raises(ValueError, match="different lengths"):
        c._reserve(3, 1, 3)
    with pytest.raises(ValueError, match="exceeds max_sequence_length"):
        c._reserve_ragged(3, 10, [3, 7, 3])
    with pytest.raises(ValueError, match="cannot change"):
        c._reserve_ragged(2, 1, [3, 7])
    c._commit_ragged(3, c._reserve_ragged(3, 1, [3, 7, 3]))
    assert c.lengths == [4, 8, 4] and c.length == 8
    v = c._row_view(1)
    assert v.length == 8 and v.key.shape == (1, 16, 2, 4) and v.key.data_ptr() == c.key[1].data_ptr()
    # equal lengths again: the scalar interface works and clears the per-sequence state
    c.lengths = [8, 8, 8]
    c._commit(3, c._reserve(3, 1, 8))
    assert c.lengths is None and c.length == 9


def test_phi_host_side_tables_and_validation():
    """Phi's host logic needs no GPU: the angle tables are the oracle's (ohara/embeddings_pos/
    rotary.py:166-184) and a configuration the kernels do not cover is refused before any device work."""
    import torch

    from ohara_amd.phi import Phi, PhiConfig, rope_cos_sin
    from oracle import phi_ref as P

    for n, dims in ((16, 6), (2048, 32), (5, 2)):
        cos, sin = rope_cos_sin(n, dims)
        rc, rs = P.rope_cos_sin(n, dims)
        assert cos.dtype == torch.float32 and cos.shape == (n, dims // 2)
        assert torch.equal(cos, rc) and torch.equal(sin, rs)
    assert PhiConfig() == PhiConfig(vocab_size=51200, max_sequence_length=2048, hidden_size=2560, num_attention_heads=32,
                                    num_hidden_layers=32, dropout=0.2, multiple_of=4, bias=True, eps=1e-5, rotary_dim=0.4)
    with pytest.raises(ValueError, match="divisible"):
        Phi(PhiConfig(hidden_size=62, num_attention_heads=4), {}, device="cpu")
    with pytest.raises(ValueError, match="positive even number"):  # int(0.1 * 16) = 1 rotated feature
        Phi(PhiConfig(hidden_size=64, num_attention_heads=4, rotary_dim=0.1), {}, device="cpu")
    with pytest.raises(NotImplementedError, match="multiple of 8"):
        Phi(PhiConfig(hidden_size=48, num_attention_heads=4), {}, device="cpu")
    with pytest.raises(ValueError, match="bfloat16"):
        Phi(PhiConfig(), {}, device="cpu", dtype=torch.float16)


def test_phi_checkpoint_name_mapping_and_local_shards(tmp_path):
    """The microsoft/phi-2 name mapping of the reference (ohara/models/phi.py:208-233) and the loader of
    local safetensors shards: every reference name is produced, tensors come back under the right
    names, an empty directory and a missing tensor raise the reference's errors."""
    import torch
    from safetensors.torch import save_file

    from ohara_amd.phi import huggingface_state_dict_map, load_huggingface_state_dict
    from oracle import phi_ref as P

    cfg = P.RefPhiConfig(vocab_size=32, hidden_size=16, num_attention_heads=2, num_hidden_layers=2, max_sequence_length=8)
    mapping = huggingface_state_dict_map(2)
    assert set(mapping) == set(P.weight_names(cfg))
    assert mapping["layers.1.mixer.dense.bias"] == "model.layers.1.self_attn.dense.bias"
    assert mapping["layers.0.ln.weight"] == "model.layers.0.input_layernorm.weight"
    assert mapping["wte.weight"] == "model.embed_tokens.weight" and mapping["ln.bias"] == "model.final_layernorm.bias"
    assert len(set(mapping.values())) == len(mapping)

    w = P.init_weights(cfg, seed=1)
    hf = {mapping[k]: v.contiguous() for k, v in w.items()}
    names = sorted(hf)
    save_file({k: hf[k] for k in names[::2]}, str(tmp_path / "model-00001-of-00002.safetensors"))
    save_file({k: hf[k] for k in names[1::2]}, str(tmp_path / "model-00002-of-00002.safetensors"))
    back = load_huggingface_state_dict(str(tmp_path), 2)
    assert set(back) == set(w) and all(torch.equal(back[k], w[k]) for k in w)
    empty = tmp_path / "empty"
    empty.mkdir()
    with pytest.raises(FileNotFoundError, match="no safetensors shards"):
        load_huggingface_state_dict(str(empty), 2)
    with pytest.raises(KeyError, match="missing expected tensors"):
        load_huggingface_state_dict(str(tmp_path), 3)
