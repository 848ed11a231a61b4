"""Writes tests/golden/phi_rope.pt - run ONCE, in the build container, where the reference tree is
mounted at /root/reference.

Seeded inputs and the outputs of the reference's RoPE module (ohara/embeddings_pos/rotary.py:96-184,
the half-split partial rotation Phi uses) for a few (rotated width, head width, offset) cases.  Plain
tensors, loaded with ``torch.load(..., weights_only=True)``.  Phi itself cannot be imported here
(ohara/models/phi.py pulls ohara.utils, which needs the absent `lightning` package), so only this
part of its attention has reference-made vectors.

Usage: python tests/golden/make_phi_rope_golden.py
"""

import os
import sys

import torch

sys.path.insert(0, "/root/reference")

from ohara.embeddings_pos.rotary import RoPE  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
CASES = [(6, 16, 0), (6, 16, 3), (32, 80, 11), (16, 16, 5), (2, 8, 1)]  # (dims, head width, offset)


def main():
    g = torch.Generator().manual_seed(99)
    out = []
    for dims, width, offset in CASES:
        x = torch.randn(2, 3, 7, width, generator=g)
        with torch.no_grad():
            y = RoPE(dims, traditional=False)(x, offset=offset)
        out.append({"dims": dims, "offset": offset, "x": x, "y": y})
    path = os.path.join(HERE, "phi_rope.pt")
    torch.save(out, path)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
