#!/usr/bin/env python3
"""Decode benchmark of the MI355X KV-cache decode path.

One "step" = one decode step (one new token for every sequence of the batch) of the d12
Llama (d_model 768, 12 layers, 6 heads x 128, SwiGLU 3072, vocab 65536, bf16, random-init
N(0, 0.02) seed 0) after a 1024-token prompt, through the KV cache (capacity 4096).
Inputs (weights, prompt, cache) are resident in HBM before the timed region.

    python bench.py [--gpus 1] [--steps 256] [--warmup 16]

prints ONE JSON line: decode tokens/s at batch 1 (the configuration the >= 70 %-of-HBM
target is quoted on) with the same measurement at batch 8/32/64 under "also", the
roofline of the dominant kernel measured with HIP events inside real decode steps, and the
CPU oracle timed on this host's cores.
"""

from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

import torch

HBM_PEAK_GBS = 8000.0

# HBM bytes per launch of the persistent decode kernel at batch 1, prompt 1024, from two
# rocprofv3 --pmc runs of this script (FETCH_SIZE, then WRITE_SIZE), each scaled by what the same
# counter reads for a 1 GiB copy (--pmc-calibration): 375.6 MB read + 1.3 MB written.  Counters
# cannot be read from inside this process, so the figure is carried here; the runs and the
# arithmetic are in profiles/decode_mega_kernel_d12_batch1_pmc.txt.
PMC_TRAFFIC_BYTES = {("persistent", 1, 1024): 377.2e6}

D12 = dict(vocab_size=65536, hidden_size=768, intermediate_size=3072, num_attention_heads=6,
           num_key_value_heads=0, num_hidden_layers=12, max_sequence_length=4096, dropout=0.0)


def d12_state(device, seed=0):
    """Random-init weights of the reference's shapes, N(0, 0.02), unit norm weights."""
    from ohara_amd.llama import Config

    cfg = Config(**D12)
    g = torch.Generator(device=device).manual_seed(seed)
    d, f, v = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size

    def n(*shape):
        return (torch.randn(*shape, generator=g, device=device) * 0.02).to(torch.bfloat16)

    st = {"token_emb.weight": n(v, d), "vocab_proj.weight": n(v, d),
          "norm.weight": torch.ones(d, dtype=torch.bfloat16, device=device)}
    for i in range(cfg.num_hidden_layers):
        p = f"layers.{i}."
        for nm in ("key", "query", "value", "proj"):
            st[p + f"attn.{nm}.weight"] = n(d, d)
        st[p + "ff.up.weight"] = n(f, d)
        st[p + "ff.gate.weight"] = n(f, d)
        st[p + "ff.down.weight"] = n(d, f)
        st[p + "norm1.weight"] = torch.ones(d, dtype=torch.bfloat16, device=device)
        st[p + "norm2.weight"] = torch.ones(d, dtype=torch.bfloat16, device=device)
    return cfg, st


def step_bytes(cfg, batch, length, int8=False):
    """Algorithmic HBM bytes of one decode step at cached length `length` (after append); int8: the caches hold one
    byte per value plus an fp32 (scale, minimum) pair per head row."""
    d, f, v, nl = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size, cfg.num_hidden_layers
    params = nl * (4 * d * d + 3 * d * f) + v * d + (2 * nl + 1) * d
    kv_row = nl * 2 * d * 2
    if int8:
        kv_row = nl * 2 * (d + 8 * (cfg.num_key_value_heads or cfg.num_attention_heads))
    return 2 * params + batch * (kv_row * length + kv_row + 2 * d + 2 * v)


def lm_head_bytes(cfg, batch):
    d, v = cfg.hidden_size, cfg.vocab_size
    return 2 * (v * d + d) + batch * 2 * (d + v)


def time_decode(model, batch, prompt_len, warmup, steps, seed=0, persistent=None, sampling=None, int8=False):
    g = torch.Generator().manual_seed(seed)
    prompt = torch.randint(0, model.config.vocab_size, (batch, prompt_len), generator=g).to(model.device)
    u = None
    if sampling is not None:  # one fixed, seeded tensor of uniform draws for the whole run
        u = torch.rand(warmup + steps + 8, batch, generator=g).to(model.device)
    sess = model.session(batch, warmup + steps + 8, persistent=persistent, sampling=sampling, u=u,
                         kv_cache=model.build_kv_cache(batch, int8=True) if int8 else None)
    sess.prefill(prompt)
    sess.capture()
    sess.run(max(0, warmup - 1))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    sess.run(steps)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    sess.check_error()
    l_mean = prompt_len + warmup + (steps + 1) / 2.0
    return dt, l_mean, sess


def time_kernel_in_situ(sess, kernel_index, steps):
    """Average duration of launch `kernel_index` inside real (eager) decode steps, from HIP
    events recorded on the launch stream right before and after that launch."""
    from ohara_amd._lib import check, lib

    L = lib()
    evs = []
    for _ in range(steps):
        a, b = C.c_void_p(), C.c_void_p()
        check(L.ohara_event_create(C.byref(a)), "event")
        check(L.ohara_event_create(C.byref(b)), "event")
        evs.append((a, b))
    for a, b in evs:
        sess.step(prof_kernel=kernel_index, prof_start=a, prof_stop=b)
    torch.cuda.synchronize()
    tot = 0.0
    for a, b in evs:
        ms = C.c_float()
        check(L.ohara_event_elapsed_ms(a, b, C.byref(ms)), "elapsed")
        tot += ms.value
        L.ohara_event_destroy(a)
        L.ohara_event_destroy(b)
    return tot / steps * 1e-3


def cpu_baseline(budget_s=20.0):
    """The CPU oracle (a PyTorch restatement of the reference's eager path) on this host:
    d12 Llama in fp32, batch 1, 128-token prompt, greedy decode through the KV cache."""
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    from oracle import llama_ref as R

    cores = torch.get_num_threads()
    rcfg = R.RefConfig(**D12)
    w = R.init_weights(rcfg, seed=0, dtype=torch.float32)
    ref = R.RefLlama(rcfg, w)
    prompt = torch.randint(0, rcfg.vocab_size, (1, 128), generator=torch.Generator().manual_seed(0))
    cache = ref.build_kv_cache(1)
    t0 = time.perf_counter()
    logits = ref(prompt, cache, 0)
    prefill_s = time.perf_counter() - t0
    nxt = logits[:, -1].argmax(-1, keepdim=True)
    pos, n = 128, 0
    for _ in range(4):  # warm-up
        nxt = ref(nxt, cache, pos)[:, -1].argmax(-1, keepdim=True)
        pos += 1
    t0 = time.perf_counter()
    while n < 512 and time.perf_counter() - t0 < budget_s:  # about 14 s on 16 cores
        nxt = ref(nxt, cache, pos)[:, -1].argmax(-1, keepdim=True)
        pos += 1
        n += 1
    dt = time.perf_counter() - t0
    return {
        "value": round(n / dt, 2), "unit": "tokens/s", "cores": cores, "kind": "port",
        "sample": f"d12 Llama fp32, batch 1, prompt 128 (prefill {prefill_s:.2f}s), {n} greedy decode steps "
                  f"through the KV cache, torch {torch.__version__} CPU, {os.cpu_count()} logical CPUs visible",
    }


# ---------------------------------------------------------------------------------------------
# Per-kernel figures of the other configurations (attention microbench, prefill on MFMA, BitNet
# ternary decode, MoE decode).  Each is timed as a HIP graph replay, so host launch cost is out.
# ---------------------------------------------------------------------------------------------
MFMA_BF16_PEAK_TFLOPS = 2500.0


def graph_time(fn, iters=10):
    """Seconds per call of fn(), captured once into a HIP graph and replayed `iters` times."""
    fn()
    fn()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        fn()
    g.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        g.replay()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters * 1e-3


def bench_attention_microbench(dev):
    """GQA decode attention, 32 query / 8 KV heads x 128, one query per sequence over L cached
    positions.  Algorithmic bytes: K + V (4*Hkv*D*B*L) + Q and O (4*H*D*B)."""
    from ohara_amd import ops
    from ohara_amd.llama import KVCache

    H, Hkv, D = 32, 8, 128
    out = []
    for B, L in ((b, l) for b in (1, 16, 64) for l in (1024, 4096, 16384, 32768)):
        ns = max(1, min(1024 // (B * Hkv), L // 128, 64))
        g = torch.Generator(device=dev).manual_seed(1)
        q = torch.randn(B, H * D, device=dev, generator=g).to(torch.bfloat16)
        k = torch.randn(B, L, Hkv, D, device=dev, generator=g).to(torch.bfloat16)
        v = torch.randn(B, L, Hkv, D, device=dev, generator=g).to(torch.bfloat16)
        ws = ops.attn_workspace(B, H, Hkv, D, ns, dev)
        o = torch.empty(B, H * D, device=dev, dtype=torch.bfloat16)
        t = graph_time(lambda: ops.attn_decode(q, k, v, H, Hkv, D, L, ns, ws, o))
        by = 4.0 * Hkv * D * B * L + 4.0 * H * D * B
        row = {"batch": B, "context": L, "n_split": ns, "us": round(t * 1e6, 1), "GBs": round(by / t / 1e9, 1),
               "frac_of_hbm_peak": round(by / t / 1e9 / HBM_PEAK_GBS, 4)}
        # the same rows through the int8 cache: codes (1 byte) + an fp32 scale and minimum per row
        cache = KVCache((B, L, Hkv, D), L, device=dev, dtype=torch.bfloat16, int8=True)
        step = max(1, 4096 // B)
        for p0 in range(0, L, step):
            ops.kv_quant_append(k[:, p0:p0 + step].contiguous(), v[:, p0:p0 + step].contiguous(), cache, p0)
        t8 = graph_time(lambda: ops.attn_cached_int8(q, cache, H, Hkv, D, L - 1, ns, ws, o))
        by8 = 2.0 * Hkv * (D + 8) * B * L + 4.0 * H * D * B
        row["int8_cache"] = {"us": round(t8 * 1e6, 1), "GBs": round(by8 / t8 / 1e9, 1),
                             "frac_of_hbm_peak": round(by8 / t8 / 1e9 / HBM_PEAK_GBS, 4)}
        out.append(row)
        del q, k, v, ws, o, cache
        torch.cuda.empty_cache()
    return out


def bench_continuous(model, cfg, dev, slots=32, steps=128):
    """Continuous batching: `slots` sequences of different lengths (prompts of 256..1279 tokens)
    decode in one batch, every slot at its own cache position; one graph replay per step."""
    from ohara_amd.batching import ContinuousBatcher

    g = torch.Generator().manual_seed(4)
    lens = torch.randint(256, 1280, (slots,), generator=g).tolist()
    bat = ContinuousBatcher(model, slots)
    for n in lens:
        bat.add(torch.randint(0, cfg.vocab_size, (n,), generator=g))
    for _ in range(8):
        bat.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        bat.step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    mean_len = sum(lens) / slots + 8 + steps / 2
    by = step_bytes(cfg, slots, mean_len)
    return {"slots": slots, "prompt_lengths": "uniform 256..1279", "mean_context": round(mean_len, 1),
            "ms_per_step": round(dt * 1e3, 4), "tokens_per_s": round(slots / dt, 1),
            "frac_of_hbm_peak": round(by / dt / 1e9 / HBM_PEAK_GBS, 4),
            "note": "host reads the new ids every step (one synchronisation per step)"}


def bench_chat_engine(model, cfg, dev, prompt_len=1024, new_tokens=256, warmup=16):
    """The reference's caller-facing API on the same workload: ChatEngine.generate (render, prefill,
    device-resident sampled decode, stop check and incremental detokenisation on the host) with the
    reference's chat defaults (temperature 0.8, top-p 0.95, no top-k), against a bare decode session
    with the same sampler.  Tokens/s of the API leg count the whole call, prompt prefill included."""
    from ohara_amd.chat_engine import ChatEngine
    from ohara_amd.sampling import SamplingConfig

    class Tok:  # one printable character per id
        eos_token_id = None
        bos_token_id = None

        def __len__(self):
            return cfg.vocab_size

        def get_vocab(self):
            return {}

        def decode(self, ids, skip_special_tokens=True):
            return "".join(chr(0x4E00 + (i % 0x5000)) for i in ids)

    g = torch.Generator().manual_seed(9)
    prompt = torch.randint(0, cfg.vocab_size, (prompt_len,), generator=g).tolist()
    eng = ChatEngine(model, Tok(), renderer=lambda tok, turns, max_tokens: prompt, stop_ids=())
    sc = SamplingConfig(temperature=0.8, top_p=0.95, max_new_tokens=new_tokens)
    msgs = [{"role": "user", "content": "x"}]
    eng.generate(msgs, sc, seed=0)  # builds the session and captures the graph
    torch.cuda.synchronize()
    best = None
    for rep in range(3):
        t0 = time.perf_counter()
        text = eng.generate(msgs, sc, seed=1 + rep)
        dt = time.perf_counter() - t0
        assert len(text) == new_tokens
        best = dt if best is None else min(best, dt)
    dts, _, sess = time_decode(model, 1, prompt_len, warmup, new_tokens, sampling=sc)
    del sess
    api, bare = new_tokens / best, new_tokens / dts
    return {"tokens_per_s": round(api, 1), "ms_per_token": round(best / new_tokens * 1e3, 4),
            "new_tokens": new_tokens, "prompt_len": prompt_len,
            "sampling": "temperature 0.8, top-p 0.95 (ohara/chat_engine.py:35-37 defaults)",
            "bare_session_tokens_per_s": round(bare, 1), "api_over_session": round(api / bare, 3),
            "note": "ChatEngine.generate end to end (prefill of the prompt, chunked read-back, stop check, "
                    "whole-reply detokenisation per token); the session figure is decode steps only"}


def bench_prefill(model, cfg, dev):
    """Batched prefill of the d12 model (1024 tokens per sequence) and its MFMA kernels alone."""
    from ohara_amd import ops

    res = {}
    B, S = 8, 1024
    prompt = torch.randint(0, cfg.vocab_size, (B, S), device=dev)
    for _ in range(2):
        cache = model.build_kv_cache(B)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        model(prompt, cache, 0, last_only=True)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
    d, f = cfg.hidden_size, cfg.intermediate_size
    flops = 2.0 * B * S * cfg.num_hidden_layers * (4 * d * d + 3 * d * f) + 4.0 * B * d * S * (S + 1) / 2 * cfg.num_hidden_layers
    res["d12_prefill"] = {"batch": B, "prompt": S, "ms": round(dt * 1e3, 3), "tokens_per_s": round(B * S / dt, 1),
                          "TFLOPs": round(flops / dt / 1e12, 1)}
    del cache
    M = B * S
    x = torch.randn(M, f, device=dev).to(torch.bfloat16)
    kern = []
    for name, n, k, kind in (("qkv 2304x768", 3 * d, d, "store"), ("wo 768x768", d, d, "store"),
                             ("gate/up 2x3072x768 + SwiGLU", f, d, "swiglu"), ("down 768x3072", d, f, "store")):
        if kind == "swiglu":
            wp = ops.pack_gate_up((torch.randn(n, k, device=dev) * 0.02).to(torch.bfloat16),
                                  (torch.randn(n, k, device=dev) * 0.02).to(torch.bfloat16))
            fl = 2.0 * M * 2 * n * k
        else:
            wp = ops.pack_linear((torch.randn(n, k, device=dev) * 0.02).to(torch.bfloat16))
            fl = 2.0 * M * n * k
        o = torch.empty(M, n, device=dev, dtype=torch.bfloat16)
        xin = x[:, :k]
        t = graph_time(lambda: ops.gemm(xin, wp, out=o), iters=50)
        kern.append({"kernel": "gemm_tile_kernel " + name, "rows": M, "us": round(t * 1e6, 1),
                     "TFLOPs": round(fl / t / 1e12, 1), "mfma_util": round(fl / t / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)})
    H, D = cfg.num_attention_heads, d // cfg.num_attention_heads
    q = torch.randn(M, d, device=dev).to(torch.bfloat16)
    kk = torch.randn(B, S, H, D, device=dev).to(torch.bfloat16)
    vv = torch.randn(B, S, H, D, device=dev).to(torch.bfloat16)
    o = torch.empty_like(q)
    t = graph_time(lambda: ops.attn_prefill(q, kk, vv, H, H, D, 0, S, o))
    fl = 4.0 * B * H * D * S * (S + 1) / 2
    kern.append({"kernel": "attn_prefill_kernel<128> causal", "rows": M, "us": round(t * 1e6, 1),
                 "TFLOPs": round(fl / t / 1e12, 1), "mfma_util": round(fl / t / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)})
    res["mfma_kernels"] = kern
    return res


def _fill_cache(cache, length, batch):
    for c in cache:
        c.key.normal_()
        c.value.normal_()
        c.length, c.batch_size = length, batch


def bitnet_c4_state(dev, n_layers=24, t_max=2048):
    """Config and state dict of the BitNet-b1.58 ternary Llama (d 2048, 16 x 128 heads, FFN 5632,
    vocab 32000): ternary weights uniform over {-1, 0, 1} (seed 2) with a per-tensor scale, unit norms."""
    from ohara_amd.bitnet import BIT_TARGETS
    from ohara_amd.llama import Config

    cfg = Config(vocab_size=32000, hidden_size=2048, intermediate_size=5632, num_attention_heads=16,
                 num_key_value_heads=0, num_hidden_layers=n_layers, max_sequence_length=t_max, dropout=0.0)
    g = torch.Generator(device=dev).manual_seed(2)
    d, f, v = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    shapes = {"attn.key": (d, d), "attn.query": (d, d), "attn.value": (d, d), "attn.proj": (d, d),
              "ff.gate": (f, d), "ff.up": (f, d), "ff.down": (d, f)}
    st = {"token_emb.weight": (torch.randn(v, d, device=dev, generator=g) * 0.02).to(torch.bfloat16),
          "vocab_proj.weight": (torch.randn(v, d, device=dev, generator=g) * 0.02).to(torch.bfloat16),
          "norm.weight": torch.ones(d, device=dev, dtype=torch.bfloat16)}
    for i in range(cfg.num_hidden_layers):
        p = f"layers.{i}."
        for nm in BIT_TARGETS:
            n, k = shapes[nm]
            st[p + nm + ".ternary"] = torch.randint(-1, 2, (n, k), device=dev, generator=g, dtype=torch.int8)
            st[p + nm + ".gamma"] = torch.tensor(0.02)
            st[p + nm + ".rms_norm.weight"] = torch.ones(k, device=dev, dtype=torch.bfloat16)
        st[p + "norm1.weight"] = torch.ones(d, device=dev, dtype=torch.bfloat16)
        st[p + "norm2.weight"] = torch.ones(d, device=dev, dtype=torch.bfloat16)
    return cfg, st


def bench_bitnet(dev, batches=(1, 8)):
    """BitNet-b1.58 ternary Llama (d 2048, 24 layers, 16 x 128 heads, FFN 5632, vocab 32000):
    one decode step at context 2048, batch 1 and 8."""
    from ohara_amd.bitnet import BitLlama

    cfg, st = bitnet_c4_state(dev)
    d, v = cfg.hidden_size, cfg.vocab_size
    model = BitLlama(cfg, st, device=dev)
    del st
    out = []
    L = cfg.max_sequence_length
    for B in batches:
        cache = model.build_kv_cache(B)
        ids = torch.randint(0, v, (B, 1), device=dev)

        def step():
            _fill_len(cache, L - 1, B)
            return model(ids, cache, L - 1, last_only=True)

        _fill_cache(cache, L - 1, B)
        t = graph_time(step)
        by = model.packed_weight_bytes() + 2.0 * v * d + 2.0 * 2 * d * cfg.num_hidden_layers * B * L
        row = {"batch": B, "context": L, "launch": "chain of 5 kernels per layer", "ms_per_step": round(t * 1e3, 4),
               "tokens_per_s": round(B / t, 1), "step_bytes": int(by), "GBs": round(by / t / 1e9, 1),
               "frac_of_hbm_peak": round(by / t / 1e9 / HBM_PEAK_GBS, 4)}
        out.append(row)
        if model.supports_persistent(B):
            # the single-launch step on the same caches: every replay starts from position L - 1 again
            sess = model.session(B, 4, kv_cache=cache, persistent=True)
            _fill_len(cache, 0, B)
            sess.prefill(ids)
            _fill_cache(cache, L - 1, B)
            start = torch.tensor([L - 1, 1, 0, 0], dtype=torch.int32, device=dev)

            def pstep():
                sess.step_state.copy_(start)
                sess._launch_step()

            tp = graph_time(pstep)
            sess.check_error()
            out.append(dict(row, launch="one persistent kernel per step", ms_per_step=round(tp * 1e3, 4),
                            tokens_per_s=round(B / tp, 1), GBs=round(by / tp / 1e9, 1),
                            frac_of_hbm_peak=round(by / tp / 1e9 / HBM_PEAK_GBS, 4)))
            del sess
        del cache
        torch.cuda.empty_cache()
    return out


def _fill_len(cache, length, batch):
    for c in cache:
        c.length, c.batch_size = length, batch


def moe_c5_state(dev, n_layers=16, t_max=2048):
    """Config and state dict of the MoE Llama (d 1024, 16 x 64 heads, 64 routed SwiGLU experts of
    hidden 512, top-8, one shared expert, softmax router): bf16 N(0, 0.02) seed 3, router rows
    N(0, 1/d) so that the router logits spread like N(0, 1)."""
    from ohara_amd.llama import Config

    cfg = Config(vocab_size=32000, hidden_size=1024, intermediate_size=512, num_attention_heads=16,
                 num_key_value_heads=0, num_hidden_layers=n_layers, max_sequence_length=t_max, dropout=0.0,
                 moe_num_experts=64, moe_experts_per_tok=8, moe_grouped=True, moe_num_shared_experts=1)
    g = torch.Generator(device=dev).manual_seed(3)
    d, f, v, E = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size, cfg.moe_num_experts

    def n(*shape):
        return (torch.randn(*shape, device=dev, generator=g) * 0.02).to(torch.bfloat16)

    one = lambda: torch.ones(d, device=dev, dtype=torch.bfloat16)  # noqa: E731
    st = {"token_emb.weight": n(v, d), "vocab_proj.weight": n(v, d), "norm.weight": one()}
    for i in range(cfg.num_hidden_layers):
        p = f"layers.{i}."
        for nm in ("key", "query", "value", "proj"):
            st[p + f"attn.{nm}.weight"] = n(d, d)
        st[p + "ff.w_gate"], st[p + "ff.w_up"], st[p + "ff.w_down"] = n(E, d, f), n(E, d, f), n(E, f, d)
        st[p + "ff.router.weight"] = (torch.randn(E, d, device=dev, generator=g) / d ** 0.5).to(torch.bfloat16)
        st[p + "ff.router_bias"] = torch.zeros(E, device=dev, dtype=torch.bfloat16)
        st[p + "ff.shared_gate.weight"], st[p + "ff.shared_up.weight"] = n(f, d), n(f, d)
        st[p + "ff.shared_down.weight"] = n(d, f)
        st[p + "norm1.weight"], st[p + "norm2.weight"] = one(), one()
    return cfg, st


def bench_moe(dev):
    """MoE decode (16 layers, d 1024, 16 x 64 heads, 64 routed SwiGLU experts of hidden 512, top-8,
    one shared expert): one step of 64 sequences at context 2048."""
    from ohara_amd.moe import MoeLlama

    cfg, st = moe_c5_state(dev)
    d, f, v, E = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size, cfg.moe_num_experts
    model = MoeLlama(cfg, st, device=dev)
    del st
    B, L = 64, cfg.max_sequence_length
    cache = model.build_kv_cache(B)
    _fill_cache(cache, L - 1, B)
    ids = torch.randint(0, v, (B, 1), device=dev)

    def step():
        _fill_len(cache, L - 1, B)
        return model(ids, cache, L - 1, last_only=True)

    t = graph_time(step, iters=5)
    nl = cfg.num_hidden_layers
    expert_b = nl * 3.0 * E * d * f * 2
    by = expert_b + nl * (3.0 * d * f + 4.0 * d * d + E * d) * 2 + 2.0 * v * d + 2.0 * 2 * d * nl * B * L
    flops = nl * 2.0 * 3 * (B * cfg.moe_experts_per_tok) * d * f
    return {"batch": B, "context": L, "ms_per_step": round(t * 1e3, 4), "tokens_per_s": round(B / t, 1),
            "step_bytes": int(by), "GBs": round(by / t / 1e9, 1), "frac_of_hbm_peak": round(by / t / 1e9 / HBM_PEAK_GBS, 4),
            "expert_ffn_TFLOPs_if_all_time": round(flops / t / 1e12, 2),
            "bound": "hbm (about 8 rows per expert: ~8 flop/byte)"}


def phi2_model(dev):
    """Phi-2 shape (32 layers, d 2560, 32 x 80 heads, 32 rotated features, MLP 10240, vocab 51200)
    with random bf16 weights."""
    from ohara_amd.phi import Phi, PhiConfig

    cfg = PhiConfig()
    g = torch.Generator(device=dev).manual_seed(4)
    d, f, v = cfg.hidden_size, cfg.multiple_of * cfg.hidden_size, cfg.vocab_size

    def n(*shape):
        return (torch.randn(*shape, device=dev, generator=g) * 0.02).to(torch.bfloat16)

    st = {"wte.weight": n(v, d), "lm_head.weight": n(v, d), "lm_head.bias": n(v), "ln.weight": torch.ones(d, device=dev),
          "ln.bias": n(d)}
    for i in range(cfg.num_hidden_layers):
        p = f"layers.{i}."
        st[p + "ln.weight"], st[p + "ln.bias"] = torch.ones(d, device=dev), n(d)
        for nm in ("q_proj", "k_proj", "v_proj", "dense"):
            st[p + f"mixer.{nm}.weight"], st[p + f"mixer.{nm}.bias"] = n(d, d), n(d)
        st[p + "mlp.fc1.weight"], st[p + "mlp.fc1.bias"] = n(f, d), n(f)
        st[p + "mlp.fc2.weight"], st[p + "mlp.fc2.bias"] = n(d, f), n(d)
    model = Phi(cfg, st, device=dev)
    del st
    torch.cuda.empty_cache()
    return cfg, model


def phi_decode_only(dev, batch, steps=12, context=1024):
    """Eager Phi-2 decode steps over a randomly filled cache and nothing else: the workload of the
    per-kernel profiles (`--phi-decode-only B`)."""
    from ohara_amd import ops

    cfg, model = phi2_model(dev)
    cache = model.build_kv_cache(batch)
    for c in cache:
        c.key.normal_()
        c.value.normal_()
    ids = torch.randint(0, cfg.vocab_size, (batch,), device=dev)
    state = torch.tensor([context, 0, 0, 0], dtype=torch.int32, device=dev)
    for _ in range(steps):
        lg = model._run(ids, batch, 1, cache, 0, state, False)
        ops.argmax(lg, next_ids=ids, step_state=state)
    torch.cuda.synchronize()
    return {"batch": batch, "steps": steps, "context_end": int(state[0])}


def bench_phi(dev):
    """Phi-2 shape, random bf16 weights: greedy decode at batch 1 and 8 after a 1024-token context, one
    graph replay per step (5 launches per layer)."""
    cfg, model = phi2_model(dev)
    d, f, v = cfg.hidden_size, cfg.multiple_of * cfg.hidden_size, cfg.vocab_size
    nl, ctx, steps = cfg.num_hidden_layers, 1024, 64
    weight_b = 2.0 * (nl * (4 * d * d + 2 * d * f) + v * d)
    out = []
    for B in (1, 8):
        prompt = torch.randint(0, v, (B, ctx), device=dev)
        model.generate_greedy(prompt[:, :16], 8)  # warm up kernels and buffers
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        model.generate_greedy(prompt, 1)
        torch.cuda.synchronize()
        t_prefill = time.perf_counter() - t0
        t0 = time.perf_counter()
        model.generate_greedy(prompt, steps + 1)
        torch.cuda.synchronize()
        t = (time.perf_counter() - t0 - t_prefill) / steps  # decode steps only (graph capture included)
        by = weight_b + 2.0 * 2 * d * nl * B * (ctx + steps / 2)
        out.append({"batch": B, "context": ctx, "ms_per_step": round(t * 1e3, 4), "tokens_per_s": round(B / t, 1),
                    "prefill_ms": round(t_prefill * 1e3, 1), "step_bytes": int(by), "GBs": round(by / t / 1e9, 1),
                    "frac_of_hbm_peak": round(by / t / 1e9 / HBM_PEAK_GBS, 4)})
    return out


# Shader-clock samples that thread 0 of every workgroup of the batch-1 persistent kernel takes per layer,
# in order (csrc/mega.hip: the stamps in the layer loop, and two inside every gemm_phase).  The kernel has
# no grid barrier inside the layers: a phase's units sit on their own stretch of workgroups and every
# hand-off is polled for, so a step's critical path runs from role to role.
_GEMM = ["activations in LDS -> MFMAs issued", "cross-wave sum"]
PHASE_STAMPS = (
    ["P1 staged"] + ["P1 " + x for x in _GEMM] + ["P1 epilogue", "P2 chunk announced", "P2 requests issued", "P3 merged"]
    + ["P3 " + x for x in _GEMM] + ["P3 epilogue", "P4 staged"] + ["P4 " + x for x in _GEMM]
    + ["P4 epilogue", "P4 requests issued", "P5 staged"] + ["P5 " + x for x in _GEMM] + ["P5 epilogue", "P5 requests issued"]
)
PHASE_TAIL = 13  # samples after the layers: three around the final norm, vocabulary projection (2), its end, selection (6), the end


def _batch1_roles(cfg, nwg, batch=1):
    """Which workgroups take which phase of the batch-1 kernel (mirrors the assignment in csrc/mega.hip)."""
    d, F = cfg.hidden_size, cfg.intermediate_size
    H = cfg.num_attention_heads
    Hkv = cfg.num_key_value_heads or H
    D = d // H
    n_qkv, n_wo, n_dn = (H + 2 * Hkv) * D // 16, d // 16, d // 16
    n_gu = (2 * ((F + 7) // 8 * 8) // 16 + 1) // 2
    ns = max(1, min(16, nwg // (batch * Hkv)))
    p2 = 1 << (ns.bit_length() - 1)
    if not (2 * ns >= 3 * p2 and ns <= 8):
        ns = p2
    dn0 = n_wo if n_wo + n_dn <= nwg else nwg - n_dn
    return {"qkv": range(nwg - n_qkv, nwg), "attention": range(0, batch * Hkv * ns), "wo": range(0, n_wo),
            "gate/up": range(0, n_gu), "down": range(dn0, dn0 + n_dn)}


def phase_timeline(dev, prompt_len, steps=32, batch=1, int8=False):
    """The critical path of a layer of the batch-1 persistent kernel: for every hand-off, when the last
    workgroup of the producing role had issued its stores and when the last workgroup of the consuming
    role had the data staged, from the kernel's own clock samples (a 100 MHz counter common to all
    workgroups), averaged over `steps` real decode steps and over the layers after the first."""
    from ohara_amd.llama import Llama

    cfg, st = d12_state(dev)
    model = Llama(cfg, st, device=dev)
    sess = model.session(batch, steps + 24, persistent=True, kv_cache=model.build_kv_cache(batch, int8=True) if int8 else None)
    sess.prefill(torch.randint(0, cfg.vocab_size, (batch, prompt_len)).to(dev))
    for _ in range(8):
        sess.step()
    nl = cfg.num_hidden_layers
    per = len(PHASE_STAMPS)
    roles = _batch1_roles(cfg, sess._nwg, batch)
    acc, total_ms = None, 0.0
    for _ in range(steps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        sess.step(prof_kernel=-2)
        e1.record()
        torch.cuda.synchronize()
        total_ms += e0.elapsed_time(e1)
        c = sess.phase_clocks(None).double()
        c = c - c[:, 0].min()
        acc = c if acc is None else acc + c
    acc = acc / steps / 100.0  # us
    kernel_us = total_ms / steps * 1e3
    idx = {name: j + 1 for j, name in enumerate(PHASE_STAMPS)}  # sample 0 precedes the first layer

    def last(role, name, layer):
        return float(acc[list(roles[role]), layer * per + idx[name]].max())

    chain = [("qkv", "P1 staged", "stream polled for, norm1 in LDS"), ("qkv", "P1 epilogue", "q/k/v product, rotary, q and new k/v rows stored"),
             ("attention", "P2 chunk announced", "q polled for, chunk, partials stored and announced"),
             ("wo", "P3 merged", "chunks polled for, partials fetched and merged"), ("wo", "P3 epilogue", "output projection + residual stored"),
             ("gate/up", "P4 staged", "stream polled for, norm2 in LDS"), ("gate/up", "P4 epilogue", "gate/up product, SwiGLU stored"),
             ("down", "P5 staged", "activations polled for, in LDS"), ("down", "P5 epilogue", "down projection + residual stored")]
    seg = torch.zeros(len(chain) + 1, dtype=torch.float64)
    layers = range(1, nl - 1)
    for l in layers:
        t = [last(r, n, l) for r, n, _ in chain] + [last("qkv", "P1 staged", l + 1)]
        prev = last("down", "P5 epilogue", l - 1)
        seg += torch.tensor([t[0] - prev] + [t[i] - t[i - 1] for i in range(1, len(chain))] + [t[-1] - t[0]])
    seg /= len(layers)
    out = {"kernel_us_hip_events (stamps on)": round(kernel_us, 2), "layers": nl, "workgroups": sess._nwg,
           "roles (workgroups)": {k: [v.start, v.stop - 1] for k, v in roles.items()},
           "per_layer_us": round(float(seg[-1]), 3),
           "before_first_layer_us": round(float(acc[list(roles["qkv"]), idx["P1 staged"]].max()), 2),
           "after_last_layer_us (final norm + vocabulary projection + selection)":
               round(float(acc[:, nl * per + PHASE_TAIL].max()) - last("down", "P5 epilogue", nl - 1), 2),
           "critical_path_us (last workgroup of the role, from the previous entry)":
               {f"{r}: {what}": round(float(seg[i]), 3) for i, (r, _, what) in enumerate(chain)}}
    return out


def bitnet_phase_timeline(dev, batch=1, steps=16):
    """Per-phase timeline of the single-launch BitNet decode step (C4 size, context 2047 -> 2048):
    workgroup 0's shader-clock samples at every grid barrier (six per barrier: phase work issued, own
    stores complete, workgroup barrier passed, arrival issued, prefetch issued, barrier passed),
    averaged over `steps` launches and over the layers after the first."""
    from ohara_amd.bitnet import BitLlama

    cfg, st = bitnet_c4_state(dev)
    model = BitLlama(cfg, st, device=dev)
    del st
    L, nl = cfg.max_sequence_length, cfg.num_hidden_layers
    cache = model.build_kv_cache(batch)
    sess = model.session(batch, 8, kv_cache=cache, persistent=True)
    sess.prefill(torch.randint(0, cfg.vocab_size, (batch, 1), device=dev))
    _fill_cache(cache, L - 1, batch)
    start = torch.tensor([L - 1, 1, 0, 0], dtype=torch.int32, device=dev)
    acc, total_ms = None, 0.0
    for it in range(steps + 4):
        sess.step_state.copy_(start)
        sess._dst.prof_kernel = -2
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        sess._launch_step()
        e1.record()
        torch.cuda.synchronize()
        if it >= 4:
            c = sess.phase_clocks().double()
            acc = c if acc is None else acc + c
            total_ms += e0.elapsed_time(e1)
    sess.check_error()
    c = acc / steps
    kernel_us = total_ms / steps * 1e3
    per = c[: nl * 30].view(nl, 30)
    n_tail = 8  # after the last barrier of the layers: vocabulary projection (2), selection arrive (4) / wait (2)
    ticks_per_us = float(c[nl * 30 + n_tail - 1] - c[0]) / kernel_us  # within a few us of the whole launch
    names = ["P1 q/k/v + rotary + append", "P2 attention partials", "P3 merge + attn.proj + residual",
             "P4 gate/up + SwiGLU", "P5 down (K split in 2)"]
    out = {"batch": batch, "kernel_us_hip_events": round(kernel_us, 1), "layers": nl,
           "clock_ticks_per_us": round(ticks_per_us, 1),
           "per_layer_us": round(float((per[1:, 29] - per[:-1, 29]).mean()) / ticks_per_us, 2),
           "after_last_layer_us (final norm + vocabulary projection + selection)":
               round(float(c[nl * 30 + n_tail - 1] - per[-1, 29]) / ticks_per_us, 1), "phases": {}}
    for i, nm in enumerate(names):
        b = per[1:, i * 6: i * 6 + 6]
        began = per[:-1, 29] if i == 0 else per[1:, i * 6 - 1]
        out["phases"][nm] = {
            "work_us": round(float((b[:, 0] - began).mean()) / ticks_per_us, 2),
            "own_stores_complete_us": round(float((b[:, 1] - b[:, 0]).mean()) / ticks_per_us, 2),
            "workgroup_barrier_us": round(float((b[:, 2] - b[:, 1]).mean()) / ticks_per_us, 2),
            "arrival_us": round(float((b[:, 3] - b[:, 2]).mean()) / ticks_per_us, 2),
            "prefetch_issue_us": round(float((b[:, 4] - b[:, 3]).mean()) / ticks_per_us, 2),
            "wait_for_release_us": round(float((b[:, 5] - b[:, 4]).mean()) / ticks_per_us, 2)}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--prompt", type=int, default=1024)
    ap.add_argument("--batches", type=str, default="1,8,32,64")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extended", action="store_true",
                    help="skip the per-kernel figures of the other configurations (attention microbench, "
                         "prefill on MFMA, BitNet and MoE decode)")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="also run three 1 GiB device-to-device copies (a kernel of known traffic to scale "
                         "FETCH_SIZE / WRITE_SIZE counters against)")
    ap.add_argument("--timeline-batch", type=int, default=1, help="sequences of the --phase-timeline run (1 to 8)")
    ap.add_argument("--timeline-int8", action="store_true", help="the --phase-timeline run over an int8 KV cache")
    ap.add_argument("--phase-timeline", action="store_true",
                    help="print the per-phase timeline of the persistent decode kernel at batch 1 and exit")
    ap.add_argument("--bitnet-phase-timeline", type=int, default=0, metavar="B",
                    help="print the per-phase timeline of the single-launch BitNet decode step at batch B and exit")
    ap.add_argument("--bitnet-only", type=str, default="", metavar="BATCHES",
                    help="run the BitNet ternary decode figures alone at these batch sizes (e.g. 1,8) and exit "
                         "(profiling workload)")
    ap.add_argument("--moe-only", action="store_true",
                    help="run the MoE decode figure alone and exit (profiling workload)")
    ap.add_argument("--prefill-only", action="store_true",
                    help="run the d12 prefill figures (tiled MFMA GEMMs, prefill attention) alone and exit")
    ap.add_argument("--attention-only", action="store_true",
                    help="run the GQA decode-attention figures (bf16 and int8 cache) alone and exit")
    ap.add_argument("--phi-decode-only", type=int, default=0, metavar="B",
                    help="run 12 eager Phi-2 decode steps of B sequences at context 1024 and exit (profiling workload)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE MI355X (no sharding, no collectives); --gpus must be 1",
              file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)

    from ohara_amd.llama import Llama

    dev = torch.device("cuda:0")
    if args.pmc_calibration:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if args.phi_decode_only:
        print(json.dumps(phi_decode_only(dev, args.phi_decode_only)))
        return
    if args.bitnet_phase_timeline:
        print(json.dumps(bitnet_phase_timeline(dev, args.bitnet_phase_timeline), indent=1))
        return
    if args.moe_only:
        print(json.dumps(bench_moe(dev), indent=1))
        return
    if args.attention_only:
        print(json.dumps(bench_attention_microbench(dev), indent=1))
        return
    if args.bitnet_only:
        print(json.dumps(bench_bitnet(dev, tuple(int(b) for b in args.bitnet_only.split(","))), indent=1))
        return
    if args.phase_timeline:
        print(json.dumps(phase_timeline(dev, args.prompt, batch=args.timeline_batch, int8=args.timeline_int8), indent=1))
        return
    cfg, st = d12_state(dev)
    model = Llama(cfg, st, device=dev)
    del st
    if args.prefill_only:
        print(json.dumps(bench_prefill(model, cfg, dev), indent=1))
        return
    batches = [int(b) for b in args.batches.split(",") if b]
    if 1 not in batches:
        batches = [1] + batches
    results = {}
    roof = None
    lm_index = 1 + 5 * cfg.num_hidden_layers
    for b in batches:
        dt, l_mean, sess = time_decode(model, b, args.prompt, args.warmup, args.steps)
        ms = dt / args.steps * 1e3
        by = step_bytes(cfg, b, l_mean)
        results[b] = {"tokens_per_s": round(b * args.steps / dt, 1), "ms_per_step": round(ms, 4),
                      "step_bytes": int(by), "step_GBs": round(by / (dt / args.steps) / 1e9, 1),
                      "step_frac_of_hbm_peak": round(by / (dt / args.steps) / 1e9 / HBM_PEAK_GBS, 4)}
        results[b]["launch"] = "one persistent kernel per step" if sess.persistent else "63 kernels per step"
        if b == 1:
            # the dominant kernel, timed with HIP events on the launch stream inside real
            # decode steps of a fresh session that continues from the same prompt length
            n_prof = 64
            sess2 = model.session(1, args.warmup + n_prof + 8)
            sess2.prefill(torch.randint(0, cfg.vocab_size, (1, args.prompt)).to(dev))
            for _ in range(args.warmup):
                sess2.step()
            torch.cuda.synchronize()
            t_k = time_kernel_in_situ(sess2, lm_index, n_prof)
            sess2.check_error()
            if sess2.persistent:
                kb = step_bytes(cfg, 1, args.prompt + args.warmup + (n_prof + 1) / 2.0)
                kname = "decode_mega_kernel<128,1,1,false,false> (batch-1 polled build; whole decode step: 12 layers + vocabulary projection + selection)"
            else:
                kb = lm_head_bytes(cfg, 1)
                kname = "wide_kernel<1,true,STORE> (final norm + vocabulary projection 65536x768)"
            roof = {"kernel": kname, "bound": "hbm", "achieved": round(kb / t_k / 1e9, 1), "peak": HBM_PEAK_GBS,
                    "unit": "GB/s", "frac": round(kb / t_k / 1e9 / HBM_PEAK_GBS, 4),
                    "traffic": PMC_TRAFFIC_BYTES.get(("persistent" if sess2.persistent else "chain", 1, args.prompt)),
                    "traffic_source": "constant carried in bench.py from two rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE) "
                                      "summarised in profiles/decode_mega_kernel_d12_batch1_pmc.txt; not measured by this run",
                    "bytes_per_launch": int(kb), "avg_launch_us": round(t_k * 1e6, 2)}
        del sess
        torch.cuda.empty_cache()

    # the same decode at batch 1 with temperature 0.8 / top-k 50 / top-p 0.9 sampling from a
    # pre-drawn uniform tensor (forward + fused sampler per step, replayed from one graph)
    from ohara_amd.sampling import SamplingConfig

    dt, _, sess = time_decode(model, 1, args.prompt, args.warmup, args.steps,
                              sampling=SamplingConfig(temperature=0.8, top_k=50, top_p=0.9))
    results["1_sampled"] = {"tokens_per_s": round(args.steps / dt, 1), "ms_per_step": round(dt / args.steps * 1e3, 4),
                            "sampling": "temperature 0.8, top-k 50, top-p 0.9, seeded uniform draws",
                            "launch": "persistent kernel + sampler kernel per step"}
    del sess
    torch.cuda.empty_cache()
    # the int8 KV cache (codes + a scale and a minimum per head row) through the same single launch
    for b in (1, 8):
        dt, l_mean, sess = time_decode(model, b, args.prompt, args.warmup, args.steps, int8=True)
        by = step_bytes(cfg, b, l_mean, int8=True)
        results[f"{b}_int8_cache"] = {
            "tokens_per_s": round(b * args.steps / dt, 1), "ms_per_step": round(dt / args.steps * 1e3, 4),
            "step_bytes": int(by), "step_frac_of_hbm_peak": round(by / (dt / args.steps) / 1e9 / HBM_PEAK_GBS, 4),
            "launch": "one persistent kernel per step" if sess.persistent else "kernel chain"}
        del sess
        torch.cuda.empty_cache()
    r1 = results[1]
    out = {
        "metric": "decode tokens/s at batch 1 & 32 (d12 Llama, 4k ctx) + % of HBM roofline",
        "value": r1["tokens_per_s"], "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": r1["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"d12 Llama bf16 greedy decode, batch 1, prompt {args.prompt}, KV cache 4096 "
                               f"(the configuration the metric is quoted on)", "batch": 1, "prompt_len": args.prompt,
                   "context_capacity": 4096, "launch": r1["launch"] + ", HIP graph replay"},
        "also": {f"batch{b}": r for b, r in results.items()},
        "roofline": roof,
    }
    out["also"]["chat_engine_batch1"] = bench_chat_engine(model, cfg, dev, args.prompt, args.steps, args.warmup)
    if not args.no_extended:
        out["also"]["continuous_batch32"] = bench_continuous(model, cfg, dev)
        out["kernels"] = {"prefill_d12": bench_prefill(model, cfg, dev)}
        del model
        torch.cuda.empty_cache()
        out["kernels"]["decode_attention_gqa_32q_8kv_128"] = bench_attention_microbench(dev)
        out["kernels"]["bitnet_decode"] = bench_bitnet(dev)
        out["kernels"]["moe_decode"] = bench_moe(dev)
        out["kernels"]["phi2_decode"] = bench_phi(dev)
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
