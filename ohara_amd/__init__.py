"""MI355X-native implementation of ohara's KV-cache decode path.

Host code is Python on PyTorch-ROCm (device memory and streams only); all compute
runs in hand-written gfx950 HIP kernels behind the C ABI of libohara_decode.so.
"""

__all__ = ["ops"]
