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
# counter reads for a 1 GiB copy (--pmc-calibration): 379.7 MB read + 1.5 MB written.  Counters
# cannot be read from inside this process, so the figure is carried here; the runs and the
# arithmetic are in profiles/decode_mega_kernel_d12_batch1_pmc.txt.
PMC_TRAFFIC_BYTES = {("persistent", 1, 1024): 381.3e6}

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


def step_bytes(cfg, batch, length):
    """Algorithmic HBM bytes of one decode step at cached length `length` (after append)."""
    d, f, v, nl = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size, cfg.num_hidden_layers
    params = nl * (4 * d * d + 3 * d * f) + v * d + (2 * nl + 1) * d
    kv_row = nl * 2 * d * 2
    return 2 * params + batch * (kv_row * length + kv_row + 2 * d + 2 * v)


def lm_head_bytes(cfg, batch):
    d, v = cfg.hidden_size, cfg.vocab_size
    return 2 * (v * d + d) + batch * 2 * (d + v)


def time_decode(model, batch, prompt_len, warmup, steps, seed=0, persistent=None):
    g = torch.Generator().manual_seed(seed)
    prompt = torch.randint(0, model.config.vocab_size, (batch, prompt_len), generator=g).to(model.device)
    sess = model.session(batch, warmup + steps + 8, persistent=persistent)
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
    while n < 128 and time.perf_counter() - t0 < budget_s:
        nxt = ref(nxt, cache, pos)[:, -1].argmax(-1, keepdim=True)
        pos += 1
        n += 1
    dt = time.perf_counter() - t0
    return {
        "value": round(n / dt, 2), "unit": "tokens/s", "cores": cores, "kind": "port",
        "sample": f"d12 Llama fp32, batch 1, prompt 128 (prefill {prefill_s:.2f}s), {n} greedy decode steps "
                  f"through the KV cache, torch {torch.__version__} CPU, {os.cpu_count()} logical CPUs visible",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--prompt", type=int, default=1024)
    ap.add_argument("--batches", type=str, default="1,8,32,64")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="also run three 1 GiB device-to-device copies (a kernel of known traffic to scale "
                         "FETCH_SIZE / WRITE_SIZE counters against)")
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
    cfg, st = d12_state(dev)
    model = Llama(cfg, st, device=dev)
    del st
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
                kname = "decode_mega_kernel<128,1> (whole decode step: 12 layers + vocabulary projection + selection)"
            else:
                kb = lm_head_bytes(cfg, 1)
                kname = "skinny_kernel<1,true,STORE> (final norm + vocabulary projection 65536x768)"
            roof = {"kernel": kname, "bound": "hbm", "achieved": round(kb / t_k / 1e9, 1), "peak": HBM_PEAK_GBS,
                    "unit": "GB/s", "frac": round(kb / t_k / 1e9 / HBM_PEAK_GBS, 4),
                    "traffic": PMC_TRAFFIC_BYTES.get(("persistent" if sess2.persistent else "chain", 1, args.prompt)),
                    "bytes_per_launch": int(kb), "avg_launch_us": round(t_k * 1e6, 2)}
        del sess
        torch.cuda.empty_cache()

    r1 = results[1]
    out = {
        "metric": "decode tokens/s at batch 1 & 32 (d12 Llama, 4k ctx) + % of HBM roofline",
        "value": r1["tokens_per_s"], "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": r1["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"d12 Llama bf16 greedy decode, batch 1, prompt {args.prompt}, KV cache 4096 "
                               f"(BASELINE configs[1])", "batch": 1, "prompt_len": args.prompt,
                   "context_capacity": 4096, "launch": r1["launch"] + ", HIP graph replay"},
        "also": {f"batch{b}": r for b, r in results.items()},
        "roofline": roof,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
