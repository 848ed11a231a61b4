"""Writes tests/golden/llama_bf16_*.pt - run ONCE, in the build container, where the reference
tree is mounted at /root/reference.

What these fixtures pin is the reference's bf16 arithmetic: ``Llama(cfg).eval().to(torch.bfloat16)``
exactly as ``ChatEngine.__init__`` casts it (ohara/chat_engine.py:262-265: parameters AND the rotary
buffers), run on the CPU through the KV cache.  Every file holds plain tensors
(``torch.load(..., weights_only=True)``):

  tiny_dense / tiny_gqa / tiny_moe   the state dicts of tests/golden/llama_tiny_*.pt cast to bf16; the
                     logits of a prefill of 5 tokens + two cached steps, the uncached logits, layer 0's
                     attention output (the input of ``attn.proj``) of every call
  mid_gqa            hidden 256, 4 layers, 4 query / 2 KV heads of width 64, 40-token prompt + 3 steps,
                     batch 2; also input and output of every module (``ops_prefill/<module>/in|out`` for the
                     last 4 prompt positions, ``ops_step0/...`` for the first cached step, with every
                     layer's cache as that step read it): each operator can be checked on the reference's
                     own operands, where one flipped bit does not travel through the layers behind it
  mid_bias           ``Config.bias=True`` (llama.py:60-63, :185): hidden 256, 3 layers, 4 query / 2 KV heads of
                     width 64, 24-token prompt + 3 steps, batch 2, with the same module inputs and outputs; the
                     biases are drawn like the matrices (the reference starts them at zero)
  d12w               the d12 widths (hidden 768, 12 layers, 6 heads x 128, FFN 3072) with a 4096-entry
                     vocabulary: 600-token prompt (two key blocks of the library's attention kernel) + 3 steps
  d12_greedy         the full d12 model of the benchmark (vocabulary 65536, cache 4096), batch 1,
                     1024-token prompt, 64 greedy tokens: the tokens, and per step the logits at 2048
                     fixed vocabulary columns plus the 32 largest logits with their ids

mid_gqa, mid_bias, d12w and d12_greedy are run three times: with all threads, with one (``*_one_thread``) and with
the library's other set of CPU matrix kernels (oneDNN switched off, ``*_other_kernels``); d12_greedy's
repeats are fed the first run's tokens.  Same code, same inputs, another summation order inside the
library's products.  The distances between the runs are how far the reference reproduces itself.

The larger cases do not store their weights: they are ``oracle.llama_ref.init_weights(cfg, seed,
torch.bfloat16)`` (a seeded CPU generator, loaded into the reference model with
``load_state_dict``); a checksum of the weights is stored so that a drifting generator is noticed.

Usage: python tests/golden/make_llama_bf16_golden.py [case ...]
"""

import dataclasses
import os
import sys
import time

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, "/root/reference")

from ohara.models.llama import Config, Llama  # noqa: E402

from oracle import llama_ref as R  # noqa: E402  (seeded weights only)

SEEDED = {
    "mid_gqa": dict(cfg=dict(vocab_size=512, hidden_size=256, intermediate_size=704, num_attention_heads=4,
                             num_key_value_heads=2, num_hidden_layers=4, max_sequence_length=64, dropout=0.0),
                    seed=11, batch=2, prompt=40, steps=3, ops=True),
    "mid_bias": dict(cfg=dict(vocab_size=512, hidden_size=256, intermediate_size=704, num_attention_heads=4,
                              num_key_value_heads=2, num_hidden_layers=3, max_sequence_length=64, dropout=0.0,
                              bias=True),
                     seed=13, batch=2, prompt=24, steps=3, ops=True),
    "d12w": dict(cfg=dict(vocab_size=4096, hidden_size=768, intermediate_size=3072, num_attention_heads=6,
                          num_key_value_heads=0, num_hidden_layers=12, max_sequence_length=1024, dropout=0.0),
                 seed=12, batch=1, prompt=600, steps=3),
}
D12 = dict(vocab_size=65536, hidden_size=768, intermediate_size=3072, num_attention_heads=6,
           num_key_value_heads=0, num_hidden_layers=12, max_sequence_length=4096, dropout=0.0)


def weight_checksum(w: dict) -> torch.Tensor:
    """Order-independent fingerprint of a weight dict: per tensor the fp64 sum and sum of squares."""
    names = sorted(k for k in w if not k.startswith("freq_"))
    return torch.tensor([[w[k].double().sum().item(), w[k].double().pow(2).sum().item()] for k in names],
                        dtype=torch.float64).sum(0)


class AttnTap:
    """Records the input of layer 0's output projection: the attention core's result."""

    def __init__(self, model):
        self.rows = []
        model.layers[0].attn.proj.register_forward_pre_hook(lambda mod, args: self.rows.append(args[0].clone()))


class OpTap:
    """Records input and output of every Linear / norm / block of the model for one call (the last one
    made), so that each operator can be checked by itself on the reference's own operands."""

    def __init__(self, model):
        self.rec = {}
        for name, mod in model.named_modules():
            if name and "dropout" not in name and name.count(".") >= 0 and not name == "layers":
                mod.register_forward_hook(self._hook(name))

    def _hook(self, name):
        def fn(mod, args, out):
            if torch.is_tensor(out) and torch.is_tensor(args[0]):
                self.rec[name] = (args[0].detach().clone(), out.detach().clone())
        return fn

    def flat(self, prefix, rows=None):
        out = {}
        for name, (x, y) in self.rec.items():
            if rows is not None and x.ndim == 3:
                x, y = x[:, -rows:], y[:, -rows:]
            out[f"{prefix}/{name}/in"] = x.clone()
            out[f"{prefix}/{name}/out"] = y.clone()
        return out


def bf16_model(cfg, state):
    model = Llama(cfg).eval()
    model.load_state_dict(state)
    return model.to(dtype=torch.bfloat16)  # chat_engine.py:265


def run_cached(model, ids, prompt, steps, ops=None):
    tap = AttnTap(model)
    cache = model.build_kv_cache(batch_size=ids.size(0))
    out = {"logits_prefill": model(ids[:, :prompt], cache, 0)}
    if ops is not None:
        out.update(ops.flat("ops_prefill", rows=4))
    for s in range(steps):
        out[f"logits_step{s}"] = model(ids[:, prompt + s : prompt + s + 1], cache, prompt + s)
        if ops is not None and s == 0:
            out.update(ops.flat("ops_step0"))
            for i, c in enumerate(cache):  # what the attention of that step read
                out[f"ops_step0/cache{i}_key"] = c.key[:, : prompt + 1].clone()
                out[f"ops_step0/cache{i}_value"] = c.value[:, : prompt + 1].clone()
    out["attn0_prefill"] = tap.rows[0]
    for s in range(steps):
        out[f"attn0_step{s}"] = tap.rows[1 + s]
    out["cache0_key"] = cache[0].key[:, : prompt + steps].clone()
    out["cache0_value"] = cache[0].value[:, : prompt + steps].clone()
    return out


@torch.no_grad()
def tiny(name):
    src = torch.load(os.path.join(HERE, f"llama_tiny_{name}.pt"), weights_only=True)
    cfg = Config(**src["config"])
    model = bf16_model(cfg, src["state"])
    ids = src["ids"]
    out = {"ids": ids, "logits_full": model(ids)}
    out.update(run_cached(model, ids, 5, 2))
    return out


@torch.no_grad()
def seeded(name):
    spec = SEEDED[name]
    cfg = Config(**spec["cfg"])
    rc = R.RefConfig(**spec["cfg"])
    w = R.init_weights(rc, seed=spec["seed"], dtype=torch.bfloat16, norm_jitter=0.1)
    model = bf16_model(cfg, {k: v.float() for k, v in w.items()})
    g = torch.Generator().manual_seed(spec["seed"])
    ids = torch.randint(0, cfg.vocab_size, (spec["batch"], spec["prompt"] + spec["steps"]), generator=g)
    out = {"config": dataclasses.asdict(cfg), "seed": spec["seed"], "norm_jitter": 0.1, "ids": ids,
           "weight_checksum": weight_checksum(w)}
    res = run_cached(model, ids, spec["prompt"], spec["steps"], ops=OpTap(model) if spec.get("ops") else None)
    # The same model, the same inputs, one thread instead of all: the library's products then sum in
    # another order.  The distance between the two runs is the reference's own reproducibility.
    n = torch.get_num_threads()
    torch.set_num_threads(1)
    one = run_cached(model, ids, spec["prompt"], spec["steps"])
    torch.set_num_threads(n)
    # ... and with the library's other set of CPU matrix kernels (oneDNN switched off)
    with torch.backends.mkldnn.flags(enabled=False):
        other = run_cached(model, ids, spec["prompt"], spec["steps"])
    out["threads"] = torch.tensor([n, 1])
    for tag, res2 in (("one_thread", one), ("other_kernels", other)):
        out[f"logits_prefill_{tag}"] = res2["logits_prefill"][:, -8:].clone()
        for s in range(spec["steps"]):
            out[f"logits_step{s}_{tag}"] = res2[f"logits_step{s}"]
    # keep the files small: the last 8 prompt positions of the prefill are enough to pin it
    res["logits_prefill"] = res["logits_prefill"][:, -8:].clone()
    res["attn0_prefill"] = res["attn0_prefill"][:, -8:].clone()
    res["cache0_key"] = res["cache0_key"][:, -16:].clone()
    res["cache0_value"] = res["cache0_value"][:, -16:].clone()
    out.update(res)
    return out


@torch.no_grad()
def d12_greedy(prompt=1024, steps=64, seed=0):
    cfg = Config(**D12)
    w = R.init_weights(R.RefConfig(**D12), seed=seed, dtype=torch.bfloat16)
    model = bf16_model(cfg, {k: v.float() for k, v in w.items()})
    g = torch.Generator().manual_seed(seed)
    ids = torch.randint(0, cfg.vocab_size, (1, prompt), generator=g)
    cols = torch.randperm(cfg.vocab_size, generator=g)[:2048].sort().values

    def run(forced):
        """Greedy decode; with ``forced`` the model is fed those tokens instead of its own choices."""
        cache = model.build_kv_cache(batch_size=1)
        t0 = time.time()
        logits = model(ids, cache, 0)[:, -1]
        print(f"  prefill {time.time() - t0:.1f} s")
        choice, sampled, top_v, top_i, scale = [], [], [], [], []
        pos = prompt
        for s in range(steps):
            row = logits[0].float()
            tv, ti = row.topk(32)
            choice.append(int(row.argmax()))
            sampled.append(logits[0, cols].clone())
            top_v.append(logits[0, ti].clone())
            top_i.append(ti)
            scale.append(row.abs().max())
            nxt = choice[-1] if forced is None else int(forced[s])
            logits = model(torch.tensor([[nxt]]), cache, pos)[:, -1]
            pos += 1
        print(f"  {steps} steps {time.time() - t0:.1f} s")
        return {"tokens": torch.tensor(choice), "logits_at_columns": torch.stack(sampled),
                "top32_values": torch.stack(top_v), "top32_ids": torch.stack(top_i),
                "logit_absmax": torch.stack(scale)}

    out = {"config": dataclasses.asdict(cfg), "seed": seed, "prompt_ids": ids, "columns": cols,
           "weight_checksum": weight_checksum(w)}
    out.update(run(None))
    n = torch.get_num_threads()
    torch.set_num_threads(1)
    one = run(out["tokens"])
    torch.set_num_threads(n)
    with torch.backends.mkldnn.flags(enabled=False):
        other = run(out["tokens"])
    out["threads"] = torch.tensor([n, 1])
    for tag, res in (("one_thread", one), ("other_kernels", other)):
        out[f"tokens_{tag}"] = res["tokens"]  # its own arg-max at every step, fed the first run's tokens
        out[f"logits_at_columns_{tag}"] = res["logits_at_columns"]
    return out


def alias_duplicates(out: dict) -> dict:
    """A module's input is usually another module's output: store such a tensor once and the string
    ``"=<key>"`` in its other places (tests/_fixtures.py:load_fixture resolves them)."""
    seen, res = {}, {}
    for k, v in out.items():
        if torch.is_tensor(v) and v.numel() > 64:
            sig = (v.dtype, tuple(v.shape), v.contiguous().view(-1).view(torch.uint8).numpy().tobytes())
            if sig in seen:
                res[k] = "=" + seen[sig]
                continue
            seen[sig] = k
        res[k] = v
    return res


def main(argv):
    cases = argv or ["tiny_dense", "tiny_gqa", "tiny_moe", "mid_gqa", "mid_bias", "d12w", "d12_greedy"]
    torch.manual_seed(0)
    for name in cases:
        if name.startswith("tiny_"):
            out = tiny(name[5:])
        elif name == "d12_greedy":
            out = d12_greedy()
        else:
            out = seeded(name)
        path = os.path.join(HERE, f"llama_bf16_{name}.pt")
        torch.save(alias_duplicates(out), path)
        print(name, "->", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main(sys.argv[1:])
