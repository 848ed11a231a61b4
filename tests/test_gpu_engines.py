"""Inference / ChatEngine over the real HIP Llama and the fused sampler (GPU)."""

import pytest
import torch

from oracle import llama_ref as R
from oracle.sampling_ref import sample_next_token_ref
from tests.test_host_logic import CharTokenizer

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


def _tiny(tok, cuda, forced=None, max_sequence_length=128):
    from ohara_amd.llama import Config, Llama

    kw = dict(vocab_size=len(tok), hidden_size=32, intermediate_size=64, max_sequence_length=max_sequence_length,
              num_hidden_layers=2, num_attention_heads=2, dropout=0.0)
    rcfg = R.RefConfig(**kw)
    w = R.init_weights(rcfg, seed=0, dtype=BF, std=0.1)
    if forced is not None:  # tests/test_chat.py:393-416: drive the head to one token
        w["vocab_proj.weight"] = torch.zeros_like(w["vocab_proj.weight"])
        w["vocab_proj.weight"][forced] = 5.0
        w["token_emb.weight"] = torch.ones_like(w["token_emb.weight"])
    return Llama(Config(**kw), w, device=cuda), R.RefLlama(rcfg, w)


def test_chat_engine_on_gpu(cuda):
    from ohara_amd.chat_engine import ChatEngine
    from ohara_amd.sampling import SamplingConfig

    tok = CharTokenizer()
    msgs = [{"role": "user", "content": "hi"}]
    model, _ = _tiny(tok, cuda, forced=tok.vocab["<|assistant_end|>"])
    eng = ChatEngine(model, tok)
    assert eng.device.type == "cuda" and eng.dtype == BF
    assert list(eng.generate_stream(msgs, SamplingConfig(temperature=0.0, max_new_tokens=32))) == []
    model, _ = _tiny(tok, cuda, forced=tok.vocab["x"])
    eng = ChatEngine(model, tok)
    assert eng.generate(msgs, SamplingConfig(temperature=0.0, max_new_tokens=5)) == "xxxxx"
    cfg = SamplingConfig(temperature=0.0, max_new_tokens=6)
    assert "".join(eng.generate_stream(msgs, cfg)) == eng.generate(msgs, cfg)
    assert eng.metadata()["layers"] == 2
    # sampled generation with shared uniform draws == the oracle model + oracle sampler
    model, ref = _tiny(tok, cuda)
    eng = ChatEngine(model, tok)
    cfg = SamplingConfig(temperature=0.8, top_p=0.9, top_k=20, max_new_tokens=12)
    u = torch.rand(12, generator=torch.Generator().manual_seed(3))
    text = eng.generate(msgs, cfg, u=u)
    ids = torch.tensor(eng.render_prompt(msgs)).view(1, -1)
    cache, pos, inp, out = ref.build_kv_cache(1), 0, ids, []
    for step in range(12):
        logits = ref(inp, cache, pos)
        pos += inp.size(1)
        nxt = sample_next_token_ref(logits, 0.8, 0.9, 20, u=u[step:step + 1], valid_vocab=len(tok))
        if int(nxt) in eng.stop_ids:
            break
        out.append(int(nxt))
        inp = nxt
    want = tok.decode(out)
    # identical unless bf16 noise moved a probability across the uniform draw; require a common prefix
    n = min(len(text), len(want))
    assert n >= 1 and text[:4] == want[:4], (text, want)
    # same seed, same text
    assert eng.generate(msgs, cfg, seed=11) == eng.generate(msgs, cfg, seed=11)


def test_inference_on_gpu(cuda):
    from ohara_amd.inference import Inference

    tok = CharTokenizer()

    class Tok:
        eos_token_id = 0

        def encode(self, text):
            return tok.encode(text)

        def decode(self, ids):
            return tok.decode(ids, skip_special_tokens=False)

    model, ref = _tiny(tok, cuda, forced=tok.vocab["y"], max_sequence_length=16)
    inf = Inference(model, Tok(), max_new_tokens=50)
    out = inf.generate("hello", stream=False, temperature=0.0)
    assert out == "hello" + "y" * 11  # clamped to the context window: 16 - 5 prompt tokens
    assert Inference.sampler(torch.tensor([[[0.1, 0.2, 0.9]]]).to(cuda), temperature=0.0).item() == 2


def test_chat_engine_from_checkpoint(cuda, tmp_path):
    """A state dict saved the way the reference's training scripts do (bare, DDP/compile prefixes,
    rotary buffers included) comes back as the same model: same config, bit-identical logits."""
    from ohara_amd.chat_engine import ChatEngine
    from ohara_amd.llama import Config, Llama, rope_tables
    from ohara_amd.sampling import SamplingConfig

    tok = CharTokenizer()
    kw = dict(vocab_size=len(tok) + 13, hidden_size=64, intermediate_size=96, max_sequence_length=48,
              num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, dropout=0.0)
    rcfg = R.RefConfig(**kw)
    w = R.init_weights(rcfg, seed=5, dtype=BF, std=0.1)
    cos, sin = rope_tables(16, 96, rcfg.rope_theta)
    saved = {"module._orig_mod." + k: v for k, v in {**w, "freq_cos": cos, "freq_sin": sin}.items()}
    torch.save({"model": saved, "idx": 3}, tmp_path / "sft.pt")
    eng = ChatEngine.from_checkpoint(tmp_path / "sft.pt", tok)
    assert eng.model.config == Config(**kw)
    direct = Llama(Config(**kw), w, device=cuda)
    ids = torch.randint(0, len(tok), (2, 7), generator=torch.Generator().manual_seed(0)).to(cuda)
    assert torch.equal(eng.model(ids), direct(ids))
    # the 13 padded vocabulary rows are never produced
    msgs = [{"role": "user", "content": "hello"}]
    text = eng.generate(msgs, SamplingConfig(temperature=1.5, top_p=1.0, max_new_tokens=16), seed=1)
    assert isinstance(text, str)
    # a tokenizer wider than the checkpoint is rejected with the reference's message
    small = {k: v for k, v in saved.items()}
    small["module._orig_mod.token_emb.weight"] = saved["module._orig_mod.token_emb.weight"][:10].clone()
    small["module._orig_mod.vocab_proj.weight"] = saved["module._orig_mod.vocab_proj.weight"][:10].clone()
    torch.save(small, tmp_path / "small.pt")
    with pytest.raises(ValueError, match="smaller than the"):
        ChatEngine.from_checkpoint(tmp_path / "small.pt", tok)


def test_inference_drives_phi_as_the_reference_example_does(cuda):
    """examples/phi_inference.py: Inference(model, tokenizer, device, use_kv_cache) over Phi, with and
    without the cache; greedy text equals the oracle's greedy continuation."""
    from ohara_amd.inference import Inference
    from ohara_amd.phi import Phi, PhiConfig
    from oracle import phi_ref as P

    tok = CharTokenizer()

    class Tok:
        eos_token_id = 0

        def encode(self, text):
            return tok.encode(text)

        def decode(self, ids):
            return tok.decode(ids, skip_special_tokens=False)

    V = (len(tok) + 3) // 4 * 4  # the vocabulary projection wants a multiple of four rows
    kw = dict(vocab_size=V, max_sequence_length=32, hidden_size=64, num_attention_heads=4, num_hidden_layers=2)
    rcfg = P.RefPhiConfig(**kw)
    w = P.init_weights(rcfg, seed=3, dtype=BF, std=0.1, bias_std=0.05)
    w["lm_head.bias"][len(tok):] = -30.0  # padded ids are never chosen
    for name, i in tok.vocab.items():     # nor the special tokens (end of text among them): the run fills
        if len(name) > 1 or i == 0:       # its token budget with one character per token
            w["lm_head.bias"][i] = -30.0
    ref, model = P.RefPhi(rcfg, w), Phi(PhiConfig(**kw), w, device=cuda)
    ids = torch.tensor([tok.encode("hello")])
    rc, pos, inp, out = ref.build_kv_cache(1), 0, ids, []
    logits_seen = []
    for _ in range(8):
        lg = ref(inp, rc, pos)[:, -1]
        pos += inp.size(1)
        logits_seen.append(lg[0])
        inp = lg.float().argmax(-1, keepdim=True)
        out.append(int(inp))
    for use_cache in (True, False):
        inf = Inference(model, Tok(), cuda, use_kv_cache=use_cache)
        text = inf.generate("hello", temperature=0.0, max_new_tokens=8, stream=False)
        assert text.startswith("hello") and len(text) == 5 + 8
        got = tok.encode(text)[5:]
        for t, (g_, w_) in enumerate(zip(got, out)):
            if g_ != w_:  # first divergence only at a near-tie of the oracle's own logits
                la, lb = logits_seen[t][g_].float().item(), logits_seen[t][w_].float().item()
                assert abs(la - lb) <= 2.0 ** -6 * max(abs(la), abs(lb), 1e-3), (use_cache, t)
                break


def test_engines_run_on_the_device_loop(cuda):
    """ChatEngine / Inference over the dense Llama decode through the device-resident loop (persistent
    step + selection replayed from a graph), reuse one session across requests, and give what the
    stepwise path (one eager forward + one sampler call per token) gives."""
    from ohara_amd.chat_engine import ChatEngine
    from ohara_amd.inference import Inference
    from ohara_amd.sampling import SamplingConfig, sample_next_token

    tok = CharTokenizer()
    msgs = [{"role": "user", "content": "tell me"}]
    model, ref = _tiny(tok, cuda)
    eng = ChatEngine(model, tok, stop_ids=())
    assert eng._loop is not None
    greedy = SamplingConfig(temperature=0.0, max_new_tokens=70)  # several chunks of the loop
    text = eng.generate(msgs, greedy)
    sess = eng._loop.session
    assert sess.graph is not None and len(text) > 0  # (head width 16: the kernel chain, not the persistent kernel)
    assert eng.generate(msgs, greedy) == text and eng._loop.session is sess  # restarted, not rebuilt
    # the stepwise path over the same model: same greedy reply up to a near-tie of bf16 logits
    step = ChatEngine(model, tok, stop_ids=(), sampler_fn=sample_next_token)
    assert step._loop is None
    want = step.generate(msgs, greedy)
    n = next((i for i, (a, b) in enumerate(zip(text, want)) if a != b), min(len(text), len(want)))
    assert n >= 8, (text, want)
    # sampled: the loop walks the caller's uniforms on the device; same draws, same text as stepwise
    cfg = SamplingConfig(temperature=0.8, top_p=0.95, max_new_tokens=40)
    u = torch.rand(40, generator=torch.Generator().manual_seed(5))
    a, b = eng.generate(msgs, cfg, u=u), step.generate(msgs, cfg, u=u)
    n = next((i for i, (x, y) in enumerate(zip(a, b)) if x != y), min(len(a), len(b)))
    assert n >= 6, (a, b)
    assert eng.generate(msgs, cfg, u=u) == a
    assert eng.generate(msgs, cfg, seed=3) == eng.generate(msgs, cfg, seed=3)
    # a stop id ends the reply although later tokens were already launched
    first = tok.encode(text[:1])[0]
    assert ChatEngine(model, tok, stop_ids=(first,)).generate(msgs, greedy) == ""
    second_stop = ChatEngine(model, tok, stop_ids=(tok.encode(text[5:6])[0],)).generate(msgs, greedy)
    assert text.startswith(second_stop) and len(second_stop) <= 5
    # Inference on the loop
    class Tok:
        eos_token_id = None

        def encode(self, t):
            return tok.encode(t)

        def decode(self, ids):
            return tok.decode(ids, skip_special_tokens=False)

    inf = Inference(model, Tok(), max_new_tokens=20)
    assert inf._loop is not None
    out = inf.generate("hello", temperature=0.0, stream=False)
    assert out.startswith("hello") and len(tok.encode(out)) == 25 and inf.kv_cache[0].length == 24
    ids = torch.tensor([tok.encode("hello")])
    want_ids = []
    rc, pos, inp = ref.build_kv_cache(1), 0, ids
    for _ in range(6):
        lg = ref(inp, rc, pos)[:, -1]
        pos += inp.size(1)
        inp = lg.float().argmax(-1, keepdim=True)
        want_ids.append(int(inp))
    assert tok.encode(out)[5:8] == want_ids[:3]


def test_sessions_do_not_share_decode_buffers(cuda):
    """Two sessions of the same batch size and an eager forward in between: each session's fed ids,
    position and captured graph are its own, so interleaving them changes nothing."""
    tok = CharTokenizer()
    model, _ = _tiny(tok, cuda)
    g = torch.Generator().manual_seed(2)
    p1, p2 = torch.randint(5, len(tok), (1, 9), generator=g), torch.randint(5, len(tok), (1, 13), generator=g)
    alone1 = model.generate_greedy(p1.to(cuda), 24).cpu()
    alone2 = model.generate_greedy(p2.to(cuda), 24).cpu()
    s1, s2 = model.session(1, 24), model.session(1, 24)
    s1.prefill(p1.to(cuda))
    s2.prefill(p2.to(cuda))
    for i in range(23):
        s1.run(1)
        if i % 3 == 0:  # an eager single-token forward of the same batch size between the steps
            model(p2[:, :1].to(cuda), model.build_kv_cache(1), 0)
        s2.run(1)
    assert torch.equal(s1.tokens().cpu(), alone1) and torch.equal(s2.tokens().cpu(), alone2)


def test_dtype_and_id_validation(cuda):
    from ohara_amd.chat_engine import ChatEngine

    tok = CharTokenizer()
    model, _ = _tiny(tok, cuda)
    assert model.to(cuda) is model and model.to(device="cuda", dtype=BF) is model
    with pytest.raises(ValueError, match="bfloat16 only"):
        model.to(torch.float32)
    with pytest.raises(ValueError, match="bfloat16 only"):
        ChatEngine(model, tok, dtype=torch.float32)
    with pytest.raises(ValueError, match="lives on"):
        model.to("cpu")
    with pytest.raises(IndexError):
        model(torch.tensor([[1, len(tok) + 5]]))
    with pytest.raises(IndexError):
        model(torch.tensor([[-1, 2]]))
