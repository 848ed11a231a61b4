"""Writes tests/golden/llama_tiny_{dense,gqa,moe}.pt - run ONCE, in the build
container, where the reference tree is mounted at /root/reference.

The fixtures pin the one thing no closed form or invariant pins: the *composition*
of the reference's Llama.forward (block order, residual placement, which norm feeds
what, cache positions, MoE routing inside a block).  Each file holds plain tensors:
the reference model's state dict, seeded token ids, its uncached logits and the
logits of a prefill + two cached single-token steps.  Loaded with
``torch.load(..., weights_only=True)``.

Usage: python tests/golden/make_llama_golden.py
"""

import dataclasses
import os
import sys

import torch

sys.path.insert(0, "/root/reference")

from ohara.models.llama import Config, Llama  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))

CASES = {
    "dense": dict(vocab_size=64, hidden_size=32, intermediate_size=64, num_attention_heads=4,
                  num_key_value_heads=0, num_hidden_layers=2, max_sequence_length=16, dropout=0.0,
                  rope_theta=10000.0),
    "gqa": dict(vocab_size=96, hidden_size=64, intermediate_size=96, num_attention_heads=4,
                num_key_value_heads=2, num_hidden_layers=3, max_sequence_length=16, dropout=0.0),
    "moe": dict(vocab_size=64, hidden_size=32, intermediate_size=16, num_attention_heads=2,
                num_key_value_heads=0, num_hidden_layers=2, max_sequence_length=16, dropout=0.0,
                moe_num_experts=8, moe_experts_per_tok=2, moe_grouped=True, moe_num_shared_experts=1,
                moe_gate_fn="softmax"),
}


def main():
    for name, kw in CASES.items():
        torch.manual_seed(1234)
        cfg = Config(**kw)
        model = Llama(cfg).eval()
        with torch.no_grad():
            # Non-trivial norm weights and router bias, so a dropped weight shows.
            for k, p in model.state_dict().items():
                if k.endswith("norm1.weight") or k.endswith("norm2.weight") or k == "norm.weight":
                    p.add_(0.1 * torch.randn_like(p))
                if k.endswith("router_bias"):
                    p.add_(0.05 * torch.randn_like(p))
            ids = torch.randint(0, cfg.vocab_size, (2, 7))
            full = model(ids)
            cache = model.build_kv_cache(batch_size=2)
            a = model(ids[:, :5], cache, 0)
            b = model(ids[:, 5:6], cache, 5)
            c = model(ids[:, 6:7], cache, torch.tensor(6))
        out = {
            "config": {k: v for k, v in dataclasses.asdict(cfg).items()},
            "state": {k: v.clone() for k, v in model.state_dict().items()},
            "ids": ids,
            "logits_full": full,
            "logits_prefill5": a,
            "logits_step5": b,
            "logits_step6": c,
            "cache0_key": cache[0].key.clone(),
            "cache0_value": cache[0].value.clone(),
        }
        path = os.path.join(HERE, f"llama_tiny_{name}.pt")
        torch.save(out, path)
        print(name, "->", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
