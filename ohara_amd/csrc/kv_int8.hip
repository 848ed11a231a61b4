// int8 KV cache mode (ohara/modules/kv_cache.py:15-32, 94-102, 116-118): every (sequence, position,
// head) row of D values is stored affine-quantised with its own fp32 scale and minimum,
//   scale = max((max - min) / 255, 1e-8),  q = clamp(round((x - min) / scale - 128), -128, 127),
//   x~ = (q + 128) * scale + min  (fp32, then rounded to the model dtype on read).
// The reference computes the quantisation with tensor ops in the cache dtype (bf16), i.e. every
// intermediate is rounded to bf16; the kernels round at the same points, so codes, scales and
// minima are bit-identical to it.
//
// Statistics layout: one 16-byte record (key scale, key minimum, value scale, value minimum) per
// (sequence, head, position), (Bcap, Hkv, Tmax, 4) fp32 - consecutive positions of a head are contiguous,
// which is how decode attention walks them.  The reference's four (B, T, Hkv, 1) tensors are strided views
// of it on the host side.
#include "common.h"

namespace {

// one wave per (row, head): D <= 512, D % 2 == 0
__global__ __launch_bounds__(256) void kv_quant_append_kernel(const bf16_t* k, const bf16_t* v, int rows, int S, int Hkv,
                                                              int D, int pos0, const int32_t* pos_dev, int pos_stride,
                                                              int8_t* kq, int8_t* vq, float* stats, int Tmax) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int item = blockIdx.x * 4 + wave;  // (tensor, row, head)
  if (item >= 2 * rows * Hkv) return;
  const int which = item / (rows * Hkv);
  const int rh = item - which * rows * Hkv;
  const int row = rh / Hkv, h = rh - row * Hkv;
  const int seq = row / S;
  const int pos = (pos_dev ? pos_dev[(size_t)seq * pos_stride] : pos0) + (row - seq * S);  // stride 1: one position per sequence
  if (pos < 0 || pos >= Tmax) return;
  const bf16_t* src = (which ? v : k) + ((size_t)row * Hkv + h) * D;
  const size_t slot = ((size_t)seq * Tmax + pos) * Hkv + h;
  int8_t* dst = (which ? vq : kq) + slot * D;
  float x[8];
  float mn = INFINITY, mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int d = lane + 64 * i;
    x[i] = d < D ? bf2f(src[d]) : 0.f;
    if (d < D) {
      mn = fminf(mn, x[i]);
      mx = fmaxf(mx, x[i]);
    }
  }
  mn = lanes_min<32, 1>(mn);
  mx = lanes_max<32, 1>(mx);
  // kv_cache.py:23-24 in the cache dtype: (max - min) -> bf16, / 255 -> bf16, clamp at bf16(1e-8)
  const float scale = fmaxf(rbf(rbf(mx - mn) / 255.0f), rbf(1e-8f));
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int d = lane + 64 * i;
    if (d < D) {
      // kv_cache.py:26: ((x - min) / scale - 128).round().clamp(-128, 127), each op rounded to bf16
      const float t = rbf(rbf(rbf(x[i] - mn) / scale) - 128.0f);
      dst[d] = (int8_t)(int)fminf(fmaxf(rintf(t), -128.f), 127.f);
    }
  }
  if (lane == 0) {
    float* rec = stats + (((size_t)seq * Hkv + h) * Tmax + pos) * 4 + 2 * which;
    *reinterpret_cast<float2*>(rec) = make_float2(scale, mn);
  }
}

// (B, len) leading positions of an int8 cache -> bf16 (B, len, Hkv, D) contiguous (kv_cache.py:116-118)
__global__ void kv_dequant_kernel(const int8_t* q, const float* stats, int which, int len, int Hkv, int D, int Tmax,
                                  bf16_t* out, size_t total) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;  // over (b, t, h, d/4)
  if (i >= total) return;
  const int d4 = D >> 2;
  const size_t rowi = i / d4;
  const int c = (int)(i - rowi * d4);
  const int h = (int)(rowi % Hkv);
  const size_t bt = rowi / Hkv;
  const int t = (int)(bt % len);
  const size_t b = bt / len;
  const size_t slot = (b * Tmax + t) * Hkv + h;
  const uint32_t w = *reinterpret_cast<const uint32_t*>(q + slot * D + 4 * c) ^ 0x80808080u;  // q + 128 as bytes
  const float2 sm = *reinterpret_cast<const float2*>(stats + ((b * Hkv + h) * (size_t)Tmax + t) * 4 + 2 * which);
  const float s = sm.x, m = sm.y;
  float f[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) f[j] = __fadd_rn(__fmul_rn((float)((w >> (8 * j)) & 0xffu), s), m);
  *reinterpret_cast<uint2*>(out + rowi * D + 4 * c) = make_uint2(pack_bf(f[0], f[1]), pack_bf(f[2], f[3]));
}

}  // namespace

extern "C" {

int ohara_kv_quant_append_int8(const uint16_t* k, const uint16_t* v, int batch, int seq_len, int h_kv, int dh, int pos,
                               const int32_t* pos_dev, int8_t* kq, int8_t* vq, float* stats, int t_max, void* stream) {
  if (!k || !v || !kq || !vq || !stats) return OHARA_EINVAL;
  if (batch < 1 || seq_len < 1 || h_kv < 1 || dh < 2 || (dh & 3) || dh > 512 || t_max < 1) return OHARA_EINVAL;
  if (!pos_dev && (pos < 0 || pos + seq_len > t_max)) return OHARA_EINVAL;
  const int64_t items = (int64_t)2 * batch * seq_len * h_kv;
  if (items > INT32_MAX) return OHARA_ESIZE;
  hipLaunchKernelGGL(kv_quant_append_kernel, dim3((unsigned)((items + 3) / 4)), dim3(256), 0, (hipStream_t)stream, k, v,
                     batch * seq_len, seq_len, h_kv, dh, pos, pos_dev, 0, kq, vq, stats, t_max);
  return ohara_launch_status();
}

int ohara_kv_quant_append_ragged_int8(const uint16_t* k, const uint16_t* v, int batch, int seq_len, int h_kv, int dh,
                                      const int32_t* seq_pos, int8_t* kq, int8_t* vq, float* stats, int t_max,
                                      void* stream) {
  if (!k || !v || !kq || !vq || !stats || !seq_pos) return OHARA_EINVAL;
  if (batch < 1 || seq_len < 1 || h_kv < 1 || dh < 2 || (dh & 3) || dh > 512 || t_max < 1) return OHARA_EINVAL;
  const int64_t items = (int64_t)2 * batch * seq_len * h_kv;
  if (items > INT32_MAX) return OHARA_ESIZE;
  hipLaunchKernelGGL(kv_quant_append_kernel, dim3((unsigned)((items + 3) / 4)), dim3(256), 0, (hipStream_t)stream, k, v,
                     batch * seq_len, seq_len, h_kv, dh, 0, seq_pos, 1, kq, vq, stats, t_max);
  return ohara_launch_status();
}

int ohara_kv_dequant_int8(const int8_t* q, const float* stats, int which, int batch, int len, int h_kv, int dh,
                          int t_max, uint16_t* out, void* stream) {
  if (!q || !stats || which < 0 || which > 1 || !out || batch < 1 || len < 1 || len > t_max || h_kv < 1 || dh < 4 || (dh & 3)) return OHARA_EINVAL;
  const size_t total = (size_t)batch * len * h_kv * (dh / 4);
  hipLaunchKernelGGL(kv_dequant_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream, q, stats,
                     which, len, h_kv, dh, t_max, out, total);
  return ohara_launch_status();
}

}  // extern "C"
