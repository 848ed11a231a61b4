// BitNet-b1.58 BitLinear with real integer arithmetic: 2-bit packed ternary weights x int8
// per-token activations, int32 accumulation on v_mfma_i32_16x16x64_i8.
//
// The reference (experiments/bitnet/bitnet.py:29-59) is float fake-quantisation recomputed on
// every forward; its effective semantics, which these kernels implement exactly, are
//   x_hat = RMSNorm_in(x)                                  (:49,53; own norm weight, eps 1e-5)
//   s     = 127 / max(max|x_hat|, 1e-5)      per token     (:31)
//   q     = clamp(rint(x_hat * s), -128, 127)              (:32; torch.round = half to even)
//   T     = clamp(rint(W / mean|W|), -1, 1),  gamma = max(mean|W|, 1e-5)   (:37-43)
//   acc   = sum_k q[k] * T[n,k]              int32, exact  <- the bit-exact contract
//   y     = (float(acc) / s) * gamma         (bias dropped, :58)
//
// Packed weight layout: strips of 16 rows, chunks of 256 columns; the tile (strip, chunk) is
// 64 lanes x 16 bytes; lane 16*g + m holds row 16*strip + m; its dword j serves the j-th MFMA of
// the chunk and carries, at bit 8*t + 2*r, the code T+1 of column 256*chunk + 64*j + 16*g + 4*r + t,
// so "(dword >> 2r) & 0x03030303" is register r of the MFMA operand.  Codes are 0..2, hence
// acc = sum q*code - sum q, the second term being one number per token.
#include "common.h"

namespace {

constexpr int BL_EPL = 96;  // K <= 6144 (LDS: int8 rows + four staged bf16 rows)

__device__ __forceinline__ float sumsq8_bits(uint4 v) {
  float s = 0.f;
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float a = lo_bf(w[i]), b = hi_bf(w[i]);
    s += a * a + b * b;
  }
  return s;
}

struct QuantOut {
  float s;      // 127 / max|x_hat|
  int sumq;     // sum of the quantised row
};

// One wave normalises and quantises one row.  The row is walked three or four times (sum of
// squares [, block norm], BitLinear norm + max, quantise); between the walks it lives in `stage`
// (LDS, K bf16 values - every intermediate is a bf16 value, so nothing is lost), which keeps the
// register footprint independent of K.  Lane l owns the 8-value pieces l, l + 64, ...
// pre_w (optional) is the weight of a block-level RMSNorm applied first (ohara/models/llama.py:
// 199-200 norm1 / norm2), nw the BitLinear's own norm weight.  xq: int8 destination (LDS or
// global).  Returns (s, sum q) in every lane.  K % 8 == 0.
__device__ __forceinline__ QuantOut wave_quant_row(const bf16_t* x, const bf16_t* pre_w, const bf16_t* nw, int K,
                                                   float eps, int8_t* xq, bf16_t* stage) {
  const int lane = threadIdx.x & 63;
  const int pieces = K >> 3;
  float ss = 0.f;
  for (int p = lane; p < pieces; p += 64) {
    const uint4 u = ldg16(x + (size_t)p * 8);
    *reinterpret_cast<uint4*>(stage + p * 8) = u;
    ss += sumsq8_bits(u);
  }
  if (pre_w) {
    ss = wave_sum(ss);
    const float rinv0 = 1.0f / sqrtf(ss / (float)K + eps);
    ss = 0.f;
    for (int p = lane; p < pieces; p += 64) {
      const uint4 u = *reinterpret_cast<const uint4*>(stage + p * 8);
      const uint4 w = ldg16(pre_w + (size_t)p * 8);
      const uint32_t uu[4] = {u.x, u.y, u.z, u.w}, ww[4] = {w.x, w.y, w.z, w.w};
      uint32_t o[4];
#pragma unroll
      for (int j = 0; j < 4; ++j)
        o[j] = pack_bf(rbf(lo_bf(uu[j]) * rinv0) * lo_bf(ww[j]), rbf(hi_bf(uu[j]) * rinv0) * hi_bf(ww[j]));
      const uint4 v = make_uint4(o[0], o[1], o[2], o[3]);
      *reinterpret_cast<uint4*>(stage + p * 8) = v;
      ss += sumsq8_bits(v);
    }
  }
  ss = wave_sum(ss);
  const float rinv = 1.0f / sqrtf(ss / (float)K + eps);
  float mx = 0.f;
  for (int p = lane; p < pieces; p += 64) {
    const uint4 u = *reinterpret_cast<const uint4*>(stage + p * 8);
    const uint4 w = ldg16(nw + (size_t)p * 8);
    const uint32_t uu[4] = {u.x, u.y, u.z, u.w}, ww[4] = {w.x, w.y, w.z, w.w};
    uint32_t o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float a0 = rbf(rbf(lo_bf(uu[j]) * rinv) * lo_bf(ww[j]));  // RMSNorm output in the model dtype
      const float a1 = rbf(rbf(hi_bf(uu[j]) * rinv) * hi_bf(ww[j]));
      mx = fmaxf(mx, fmaxf(fabsf(a0), fabsf(a1)));
      o[j] = pack_bf(a0, a1);
    }
    *reinterpret_cast<uint4*>(stage + p * 8) = make_uint4(o[0], o[1], o[2], o[3]);
  }
  mx = wave_max(mx);
  const float s = 127.0f / fmaxf(mx, 1e-5f);
  int sq = 0;
  for (int p = lane; p < pieces; p += 64) {
    const uint4 u = *reinterpret_cast<const uint4*>(stage + p * 8);
    const uint32_t uu[4] = {u.x, u.y, u.z, u.w};
    uint32_t pk[2] = {0u, 0u};
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float v = (j & 1) ? hi_bf(uu[j >> 1]) : lo_bf(uu[j >> 1]);
      const int qi = (int)fminf(fmaxf(rintf(v * s), -128.f), 127.f);
      sq += qi;
      pk[j >> 2] |= ((uint32_t)qi & 0xffu) << (8 * (j & 3));
    }
    *reinterpret_cast<uint2*>(xq + (size_t)p * 8) = make_uint2(pk[0], pk[1]);
  }
  sq = lanes_sum<32, 1>(sq);
  return QuantOut{s, sq};
}

// The same for a single row with the whole workgroup (four waves) on it: a decode step at batch 1
// has one row per projection, and one wave walking 2048-5632 values four times is most of such a
// kernel's critical path.  Thread t owns the pieces t, t + 256, ...; the three reductions go through
// `red` (four floats of LDS).  Every thread of the workgroup must call it.
__device__ __forceinline__ QuantOut block_quant_row(const bf16_t* x, const bf16_t* pre_w, const bf16_t* nw, int K,
                                                    float eps, int8_t* xq, bf16_t* stage, float* red) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int pieces = K >> 3;
  auto bsum = [&](float v) {
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    return ((red[0] + red[1]) + red[2]) + red[3];
  };
  float ss = 0.f;
  for (int p = tid; p < pieces; p += 256) {
    const uint4 u = ldg16(x + (size_t)p * 8);
    *reinterpret_cast<uint4*>(stage + p * 8) = u;
    ss += sumsq8_bits(u);
  }
  if (pre_w) {
    const float rinv0 = 1.0f / sqrtf(bsum(ss) / (float)K + eps);
    ss = 0.f;
    for (int p = tid; p < pieces; p += 256) {
      const uint4 u = *reinterpret_cast<const uint4*>(stage + p * 8);
      const uint4 w = ldg16(pre_w + (size_t)p * 8);
      const uint32_t uu[4] = {u.x, u.y, u.z, u.w}, ww[4] = {w.x, w.y, w.z, w.w};
      uint32_t o[4];
#pragma unroll
      for (int j = 0; j < 4; ++j)
        o[j] = pack_bf(rbf(lo_bf(uu[j]) * rinv0) * lo_bf(ww[j]), rbf(hi_bf(uu[j]) * rinv0) * hi_bf(ww[j]));
      const uint4 v = make_uint4(o[0], o[1], o[2], o[3]);
      *reinterpret_cast<uint4*>(stage + p * 8) = v;
      ss += sumsq8_bits(v);
    }
  }
  const float rinv = 1.0f / sqrtf(bsum(ss) / (float)K + eps);
  float mx = 0.f;
  for (int p = tid; p < pieces; p += 256) {
    const uint4 u = *reinterpret_cast<const uint4*>(stage + p * 8);
    const uint4 w = ldg16(nw + (size_t)p * 8);
    const uint32_t uu[4] = {u.x, u.y, u.z, u.w}, ww[4] = {w.x, w.y, w.z, w.w};
    uint32_t o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float a0 = rbf(rbf(lo_bf(uu[j]) * rinv) * lo_bf(ww[j]));
      const float a1 = rbf(rbf(hi_bf(uu[j]) * rinv) * hi_bf(ww[j]));
      mx = fmaxf(mx, fmaxf(fabsf(a0), fabsf(a1)));
      o[j] = pack_bf(a0, a1);
    }
    *reinterpret_cast<uint4*>(stage + p * 8) = make_uint4(o[0], o[1], o[2], o[3]);
  }
  mx = wave_max(mx);
  __syncthreads();
  if (lane == 0) red[wave] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  const float s = 127.0f / fmaxf(mx, 1e-5f);
  int sq = 0;
  for (int p = tid; p < pieces; p += 256) {
    const uint4 u = *reinterpret_cast<const uint4*>(stage + p * 8);
    const uint32_t uu[4] = {u.x, u.y, u.z, u.w};
    uint32_t pk[2] = {0u, 0u};
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float v = (j & 1) ? hi_bf(uu[j >> 1]) : lo_bf(uu[j >> 1]);
      const int qi = (int)fminf(fmaxf(rintf(v * s), -128.f), 127.f);
      sq += qi;
      pk[j >> 2] |= ((uint32_t)qi & 0xffu) << (8 * (j & 3));
    }
    *reinterpret_cast<uint2*>(xq + (size_t)p * 8) = make_uint2(pk[0], pk[1]);
  }
  sq = lanes_sum<32, 1>(sq);
  int* redi = reinterpret_cast<int*>(red);
  __syncthreads();
  if (lane == 0) redi[wave] = sq;
  __syncthreads();
  return QuantOut{s, redi[0] + redi[1] + redi[2] + redi[3]};
}

__global__ __launch_bounds__(256) void act_quant_kernel(const bf16_t* x, int ldx, const bf16_t* nw, int rows, int K,
                                                        float eps, int8_t* q, int ldq, float* s_out, int* sumq_out) {
  extern __shared__ __align__(16) unsigned char qsm[];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (rows == 1) {  // the whole workgroup on the one row (the order of sums the fused kernels use for it)
    const QuantOut o = block_quant_row(x, nullptr, nw, K, eps, q, reinterpret_cast<bf16_t*>(qsm),
                                       reinterpret_cast<float*>(qsm + (size_t)K * 2));
    if (threadIdx.x == 0) {
      s_out[0] = o.s;
      sumq_out[0] = o.sumq;
    }
    return;
  }
  const int r = blockIdx.x * 4 + wave;
  if (r >= rows) return;
  const QuantOut o = wave_quant_row(x + (size_t)r * ldx, nullptr, nw, K, eps, q + (size_t)r * ldq,
                                    reinterpret_cast<bf16_t*>(qsm) + (size_t)wave * K);
  if (lane == 0) {
    s_out[r] = o.s;
    sumq_out[r] = o.sumq;
  }
}

struct BitArgs {
  const uint4* wp;       // packed ternary
  float gamma;
  const bf16_t* x;       // FUSED: (B, K) bf16 activations
  int ldx;
  const bf16_t* nw;      // FUSED: BitLinear's RMSNorm weight
  const bf16_t* pre_w;   // FUSED, optional: weight of a block-level RMSNorm applied before it
  float eps;
  const int8_t* q;       // !FUSED: (B, ldq) int8
  int ldq;
  const float* s;        // !FUSED
  const int* sumq;       // !FUSED
  int B, N, K;
  bf16_t* out;
  int ldo;
  const bf16_t* resid;
  int ldr;
  int32_t* acc_out;      // optional (B, N) raw accumulators
  int ldacc;
};

// One workgroup, one 16-row strip of one BitLinear: quantise the activation rows into LDS (FUSED)
// or copy them in, stream the strip's packed weights, leave the int32 accumulators (codes T+1, so
// sum q still to subtract) of the strip in wave 0.  Returns false in waves 1..3.  Every thread of
// the workgroup must call it; LDS is reusable after the call's last barrier.
template <int BT, bool FUSED>
__device__ __forceinline__ bool bitlinear_strip(const BitArgs& a, int strip, unsigned char* smem, i32x4* acc,
                                                float** s_s_out, int** s_sum_out) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m = lane & 15, g = lane >> 4;
  const int KC = (a.K + 255) >> 8;      // 256-column chunks
  const int Kp = KC << 8;
  const int ldq = Kp + 16;              // LDS row stride in bytes (16-byte skew against bank conflicts)
  int8_t* xq = reinterpret_cast<int8_t*>(smem);
  float* s_s = reinterpret_cast<float*>(smem + (((size_t)BT * 16 * ldq + 255) & ~(size_t)255));
  int* s_sum = reinterpret_cast<int*>(s_s + BT * 16);
  int* red = s_sum + BT * 16;           // [3][BT][64][4]
  bf16_t* stage = reinterpret_cast<bf16_t*>(red + 3 * BT * 64 * 4);  // [4][Kp] rows being quantised (FUSED)

  // the first weights of this wave are requested before the activations are prepared
  const int per = (KC + 3) >> 2;
  const int c0 = wave * per, c1 = min(KC, c0 + per);
  const uint4* wrow = a.wp + (size_t)strip * KC * 64 + lane;
  constexpr int CH = 6;
  uint4 wpre[CH];
#pragma unroll
  for (int c = 0; c < CH; ++c) wpre[c] = (c0 + c < c1) ? ldg16_nt(wrow + (size_t)(c0 + c) * 64) : make_uint4(0, 0, 0, 0);

  // ---- activations -> int8 rows in LDS ---------------------------------------------------
  // rows beyond B and columns beyond K must read as zero; rows < B are overwritten up to K below
  {
    const int p16 = ldq / 16;
    const int kfull = a.K >> 4;  // 16-byte pieces wholly below K
    for (int i = tid; i < BT * 16 * p16; i += 256) {
      const int r = i / p16, c = i - r * p16;
      if (r >= a.B || c >= kfull) reinterpret_cast<uint4*>(xq)[i] = make_uint4(0, 0, 0, 0);
    }
  }
  __syncthreads();
  if (FUSED && a.B == 1) {
    const QuantOut o = block_quant_row(a.x, a.pre_w, a.nw, a.K, a.eps, xq, stage, reinterpret_cast<float*>(red));
    if (tid == 0) {
      s_s[0] = o.s;
      s_sum[0] = o.sumq;
    }
  } else if (FUSED) {
    for (int b = wave; b < a.B; b += 4) {
      const QuantOut o = wave_quant_row(a.x + (size_t)b * a.ldx, a.pre_w, a.nw, a.K, a.eps, xq + (size_t)b * ldq,
                                        stage + (size_t)wave * Kp);
      if (lane == 0) {
        s_s[b] = o.s;
        s_sum[b] = o.sumq;
      }
    }
  } else {
    const int n16 = (a.K + 15) >> 4;
    for (int i = tid; i < a.B * n16; i += 256) {
      const int b = i / n16, c = i - b * n16;
      reinterpret_cast<uint4*>(xq + (size_t)b * ldq)[c] = ldg16(a.q + (size_t)b * a.ldq + c * 16);
    }
    for (int b = tid; b < a.B; b += 256) {
      s_s[b] = a.s[b];
      s_sum[b] = a.sumq[b];
    }
  }
  __syncthreads();

  // ---- weight stream -----------------------------------------------------------------------
#pragma unroll
  for (int t = 0; t < BT; ++t) acc[t] = (i32x4){0, 0, 0, 0};
  for (int cb = c0; cb < c1; cb += CH) {
    uint4 wv[CH];
    if (cb == c0) {
#pragma unroll
      for (int c = 0; c < CH; ++c) wv[c] = wpre[c];
    } else {
#pragma unroll
      for (int c = 0; c < CH; ++c) wv[c] = (cb + c < c1) ? ldg16_nt(wrow + (size_t)(cb + c) * 64) : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      if (cb + c >= c1) continue;
      const uint32_t dw[4] = {wv[c].x, wv[c].y, wv[c].z, wv[c].w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        i32x4 av;
        av[0] = (int)(dw[j] & 0x03030303u);
        av[1] = (int)((dw[j] >> 2) & 0x03030303u);
        av[2] = (int)((dw[j] >> 4) & 0x03030303u);
        av[3] = (int)((dw[j] >> 6) & 0x03030303u);
        const int k0 = ((cb + c) << 8) + 64 * j + 16 * g;
#pragma unroll
        for (int t = 0; t < BT; ++t) {
          const uint4 xv = *reinterpret_cast<const uint4*>(xq + (size_t)(m + 16 * t) * ldq + k0);
          i32x4 bv;
          bv[0] = (int)xv.x; bv[1] = (int)xv.y; bv[2] = (int)xv.z; bv[3] = (int)xv.w;
          acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, bv, acc[t], 0, 0, 0);
        }
      }
    }
  }
  if (wave > 0) {
#pragma unroll
    for (int t = 0; t < BT; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) red[(((wave - 1) * BT + t) * 64 + lane) * 4 + i] = acc[t][i];
  }
  __syncthreads();
  *s_s_out = s_s;
  *s_sum_out = s_sum;
  if (wave != 0) return false;
#pragma unroll
  for (int t = 0; t < BT; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i)
      acc[t][i] += red[((0 * BT + t) * 64 + lane) * 4 + i] + red[((1 * BT + t) * 64 + lane) * 4 + i] +
                   red[((2 * BT + t) * 64 + lane) * 4 + i];
  return true;
}

// y = bf16((float(acc - sum q) / s) * gamma): the four outputs of one MFMA fragment (bitnet.py:58-59)
__device__ __forceinline__ void bit_scale4(const i32x4& acc, int sq, float s, float gamma, int* ai, float* y) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    ai[i] = acc[i] - sq;  // codes are T+1
    y[i] = rbf(__fmul_rn(__fdiv_rn((float)ai[i], s), gamma));
  }
}

template <int BT, bool FUSED>
__global__ __launch_bounds__(256) void bitlinear_kernel(BitArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int strip = blockIdx.x;
  const int lane = threadIdx.x & 63;
  const int m = lane & 15, g = lane >> 4;
  i32x4 acc[BT];
  float* s_s;
  int* s_sum;
  if (!bitlinear_strip<BT, FUSED>(a, strip, smem, acc, &s_s, &s_sum)) return;
  const int r0 = strip * 16 + 4 * g;
#pragma unroll
  for (int t = 0; t < BT; ++t) {
    const int b = m + 16 * t;
    if (b >= a.B) continue;
    int ai[4];
    float y[4];
    bit_scale4(acc[t], s_sum[b], s_s[b], a.gamma, ai, y);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = r0 + i;
      if (n >= a.N) continue;
      if (a.acc_out) a.acc_out[(size_t)b * a.ldacc + n] = ai[i];
      float v = y[i];
      if (a.resid) v = bf2f(a.resid[(size_t)b * a.ldr + n]) + v;
      a.out[(size_t)b * a.ldo + n] = f2bf(v);
    }
  }
}

// ---- fused groups of BitLinears that share their input row ---------------------------------------
// Q/K/V (bitnet.py:70-95 swaps attn.query/key/value; each keeps its own norm weight and scale, so
// each strip quantises the row with its projection's norm): one launch over the strips of all three,
// with rotary + cache append as the epilogue (rotary.py:55-93, kv_cache.py:104-105).
struct BitQkvArgs {
  BitArgs p[3];          // query, key, value: wp, gamma, nw, N; x / pre_w / K / B shared
  int strips[3];
  int H, Hkv, Dh, Tmax, S, pos;
  const int32_t* pos_dev;
  const bf16_t* cos;
  const bf16_t* sin;
  bf16_t* q_out;         // (B*S, H*Dh)
  bf16_t* kcache;
  bf16_t* vcache;
};

template <int BT>
__global__ __launch_bounds__(256) void bitlinear_qkv_kernel(BitQkvArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  int strip = blockIdx.x, which = 0;
  if (strip >= a.strips[0]) { strip -= a.strips[0]; which = 1; }
  if (which == 1 && strip >= a.strips[1]) { strip -= a.strips[1]; which = 2; }
  BitArgs pa = a.p[0];  // the three differ in weights, scale, norm weight and width only (no dynamic
                        // indexing of the argument block: that would copy it to scratch memory)
  if (which == 1) { pa.wp = a.p[1].wp; pa.gamma = a.p[1].gamma; pa.nw = a.p[1].nw; pa.N = a.p[1].N; }
  if (which == 2) { pa.wp = a.p[2].wp; pa.gamma = a.p[2].gamma; pa.nw = a.p[2].nw; pa.N = a.p[2].N; }
  const int lane = threadIdx.x & 63;
  const int m = lane & 15, g = lane >> 4;
  i32x4 acc[BT];
  float* s_s;
  int* s_sum;
  if (!bitlinear_strip<BT, true>(pa, strip, smem, acc, &s_s, &s_sum)) return;
  const int r0 = strip * 16 + 4 * g;
  if (r0 >= pa.N) return;
#pragma unroll
  for (int t = 0; t < BT; ++t) {
    const int b = m + 16 * t;  // row = sequence * S + s
    if (b >= pa.B) continue;
    int ai[4];
    float v[4];
    bit_scale4(acc[t], s_sum[b], s_s[b], pa.gamma, ai, v);
    const int seq = b / a.S;
    const int pos = (a.pos_dev ? *a.pos_dev : a.pos) + (b - seq * a.S);
    if (pos < 0 || pos >= a.Tmax) continue;
    bf16_t* o;
    if (which < 2) {
      const int d = r0 % a.Dh;
      const bf16_t* cs = a.cos + (size_t)pos * (a.Dh >> 1) + (d >> 1);
      const bf16_t* sn = a.sin + (size_t)pos * (a.Dh >> 1) + (d >> 1);
#pragma unroll
      for (int pr = 0; pr < 2; ++pr) {
        const float c = bf2f(cs[pr]), sv = bf2f(sn[pr]);
        const float e = v[2 * pr], od = v[2 * pr + 1];
        v[2 * pr] = __fsub_rn(__fmul_rn(e, c), __fmul_rn(od, sv));
        v[2 * pr + 1] = __fadd_rn(__fmul_rn(e, sv), __fmul_rn(od, c));
      }
      o = which == 0 ? a.q_out + (size_t)b * a.H * a.Dh + r0
                     : a.kcache + (((size_t)seq * a.Tmax + pos) * a.Hkv) * a.Dh + r0;
    } else {
      o = a.vcache + (((size_t)seq * a.Tmax + pos) * a.Hkv) * a.Dh + r0;
    }
    *reinterpret_cast<uint2*>(o) = make_uint2(pack_bf(v[0], v[1]), pack_bf(v[2], v[3]));
  }
}

// gate and up (ff.gate / ff.up) for the same strip of hidden columns in one workgroup, SwiGLU as the
// epilogue: out = bf16(bf16(silu(gate)) * up) (ohara/modules/mlp.py:152).
struct BitGateUpArgs {
  BitArgs gate, up;      // out/ldo of `gate` receive the product
};

template <int BT>
__global__ __launch_bounds__(256) void bitlinear_gate_up_kernel(BitGateUpArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int strip = blockIdx.x;
  const int lane = threadIdx.x & 63;
  const int m = lane & 15, g = lane >> 4;
  i32x4 acc_g[BT], acc_u[BT];
  float yg[BT][4];
  float* s_s;
  int* s_sum;
  const bool w0 = bitlinear_strip<BT, true>(a.gate, strip, smem, acc_g, &s_s, &s_sum);
  if (w0) {
#pragma unroll
    for (int t = 0; t < BT; ++t) {
      const int b = m + 16 * t;
      int ai[4];
      if (b < a.gate.B) bit_scale4(acc_g[t], s_sum[b], s_s[b], a.gate.gamma, ai, yg[t]);
    }
  }
  __syncthreads();  // the row statistics in LDS are about to be overwritten
  if (!bitlinear_strip<BT, true>(a.up, strip, smem, acc_u, &s_s, &s_sum)) return;
  const int r0 = strip * 16 + 4 * g;
#pragma unroll
  for (int t = 0; t < BT; ++t) {
    const int b = m + 16 * t;
    if (b >= a.up.B) continue;
    int ai[4];
    float yu[4];
    bit_scale4(acc_u[t], s_sum[b], s_s[b], a.up.gamma, ai, yu);
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (r0 + i < a.gate.N) a.gate.out[(size_t)b * a.gate.ldo + r0 + i] = f2bf(rbf(silu_f(yg[t][i])) * yu[i]);
  }
}

// T (N, K) int8 in {-1,0,1} row-major -> packed layout
__global__ void pack_ternary_kernel(const int8_t* t, int n, int k, int ldt, int KC, size_t total, uint4* dst) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const int lane = idx & 63;
  const size_t sc = idx >> 6;
  const int chunk = (int)(sc % KC);
  const int strip = (int)(sc / KC);
  const int m = lane & 15, g = lane >> 4;
  const int row = strip * 16 + m;
  uint32_t dw[4];
  for (int j = 0; j < 4; ++j) {
    uint32_t w = 0;
    for (int r = 0; r < 4; ++r)
      for (int b = 0; b < 4; ++b) {
        const int col = chunk * 256 + 64 * j + 16 * g + 4 * r + b;
        int code = 1;  // zero weight
        if (row < n && col < k) code = (int)t[(size_t)row * ldt + col] + 1;
        w |= (uint32_t)(code & 3) << (8 * b + 2 * r);
      }
    dw[j] = w;
  }
  dst[idx] = make_uint4(dw[0], dw[1], dw[2], dw[3]);
}

// silu(gate) * up with the reference's rounding (ohara/modules/mlp.py:152)
__global__ void silu_mul_kernel(const bf16_t* gate, const bf16_t* up, bf16_t* out, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = f2bf(rbf(silu_f(bf2f(gate[i]))) * bf2f(up[i]));
}

// Rotary on q and k rows + append of k, v to the cache (ohara/embeddings_pos/rotary.py:55-93,
// ohara/modules/kv_cache.py:104-105); one workgroup per (sequence, position) row.
__global__ __launch_bounds__(256) void rope_append_kernel(bf16_t* q, const bf16_t* k, const bf16_t* v, int S, int H,
                                                          int Hkv, int D, const bf16_t* cos, const bf16_t* sin, int pos0,
                                                          const int32_t* pos_dev, bf16_t* kc, bf16_t* vc, int Tmax) {
  const int row = blockIdx.x;
  const int seq = row / S;
  const int pos = (pos_dev ? *pos_dev : pos0) + (row - seq * S);
  if (pos < 0 || (Tmax > 0 && pos >= Tmax)) return;
  const int half = D >> 1;
  const bf16_t* cs = cos + (size_t)pos * half;
  const bf16_t* sn = sin + (size_t)pos * half;
  for (int i = threadIdx.x; i < H * half; i += 256) {
    const int h = i / half, p = i - h * half;
    bf16_t* x = q + (size_t)row * H * D + (size_t)h * D + 2 * p;
    const float e = bf2f(x[0]), o = bf2f(x[1]), c = bf2f(cs[p]), s = bf2f(sn[p]);
    x[0] = f2bf(__fsub_rn(__fmul_rn(e, c), __fmul_rn(o, s)));
    x[1] = f2bf(__fadd_rn(__fmul_rn(e, s), __fmul_rn(o, c)));
  }
  // Tmax == 0: kc / vc are row buffers like k / v (the rows an int8 cache's append quantises)
  const size_t dst_row = Tmax > 0 ? (size_t)seq * Tmax + pos : (size_t)row;
  bf16_t* kd = kc + dst_row * Hkv * D;
  bf16_t* vd = vc + dst_row * Hkv * D;
  for (int i = threadIdx.x; i < Hkv * half; i += 256) {
    const int h = i / half, p = i - h * half;
    const bf16_t* x = k + (size_t)row * Hkv * D + (size_t)h * D + 2 * p;
    const float e = bf2f(x[0]), o = bf2f(x[1]), c = bf2f(cs[p]), s = bf2f(sn[p]);
    kd[h * D + 2 * p] = f2bf(__fsub_rn(__fmul_rn(e, c), __fmul_rn(o, s)));
    kd[h * D + 2 * p + 1] = f2bf(__fadd_rn(__fmul_rn(e, s), __fmul_rn(o, c)));
  }
  for (int i = threadIdx.x; i < Hkv * D; i += 256) vd[i] = v[(size_t)row * Hkv * D + i];
}

template <bool FUSED>
int launch_bit(const BitArgs& a0, hipStream_t st) {
  const int strips = (a0.N + 15) / 16;
  const int KC = (a0.K + 255) >> 8;
  const int ldq = (KC << 8) + 16;
  // rows per pass: as many 16-row tiles (4, 2 or 1) as fit the LDS with this K
  auto smem_of = [&](int btt) {
    return (((size_t)btt * 16 * ldq + 255) & ~(size_t)255) + (size_t)btt * 16 * 8 +
           (size_t)3 * btt * 64 * 4 * sizeof(int) + (FUSED ? (size_t)4 * (KC << 8) * 2 : 0);
  };
  int cap = 64;
  while (cap > 16 && smem_of(cap / 16) > 160 * 1024) cap >>= 1;
  for (int r = 0; r < a0.B; r += cap) {
    BitArgs a = a0;
    a.B = a0.B - r < cap ? a0.B - r : cap;
    if (FUSED) a.x = a0.x + (size_t)r * a0.ldx;
    else {
      a.q = a0.q + (size_t)r * a0.ldq;
      a.s = a0.s + r;
      a.sumq = a0.sumq + r;
    }
    a.out = a0.out + (size_t)r * a0.ldo;
    if (a0.resid) a.resid = a0.resid + (size_t)r * a0.ldr;
    if (a0.acc_out) a.acc_out = a0.acc_out + (size_t)r * a0.ldacc;
    const int bt = (a.B + 15) / 16;
    const int btt = bt == 3 ? 4 : bt;
    const size_t smem = smem_of(btt);
    if (smem > 160 * 1024) return OHARA_ESIZE;
    dim3 grid(strips), block(256);
#define OHARA_BIT(BTV)                                                                                   \
  do {                                                                                                   \
    if (smem > 64 * 1024)                                                                                \
      (void)hipFuncSetAttribute((const void*)bitlinear_kernel<BTV, FUSED>,                               \
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);                  \
    hipLaunchKernelGGL((bitlinear_kernel<BTV, FUSED>), grid, block, smem, st, a);                        \
  } while (0)
    if (btt == 1) OHARA_BIT(1);
    else if (btt == 2) OHARA_BIT(2);
    else OHARA_BIT(4);
#undef OHARA_BIT
    const int rc = ohara_launch_status();
    if (rc) return rc;
  }
  return OHARA_OK;
}

}  // namespace

extern "C" {

int ohara_bitlinear_pack_ternary(const int8_t* t, int n, int k, int ldt, uint32_t* dst, int64_t* bytes, void* stream) {
  if (n < 1 || k < 1) return OHARA_EINVAL;
  const int KC = (k + 255) / 256;
  const size_t total = (size_t)((n + 15) / 16) * KC * 64;
  if (bytes) *bytes = (int64_t)total * 16;
  if (!dst) return OHARA_OK;
  if (!t || ldt < k) return OHARA_EINVAL;
  hipLaunchKernelGGL(pack_ternary_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream, t, n,
                     k, ldt, KC, total, reinterpret_cast<uint4*>(dst));
  return ohara_launch_status();
}

int ohara_act_quant_int8(const uint16_t* x, int ldx, const uint16_t* norm_w, float eps, int rows, int k, int8_t* q,
                         int ldq, float* s, int32_t* sumq, void* stream) {
  if (!x || !norm_w || !q || !s || !sumq || rows < 1 || k < 1 || ldx < k || ldq < k) return OHARA_EINVAL;
  if ((k & 7) || (ldx & 7) || (ldq & 7)) return OHARA_EINVAL;  // 16-byte loads, 8-byte stores
  if (k > BL_EPL * 64) return OHARA_ESIZE;
  hipLaunchKernelGGL(act_quant_kernel, dim3((rows + 3) / 4), dim3(256), (size_t)4 * k * 2, (hipStream_t)stream, x, ldx, norm_w, rows, k,
                     eps, q, ldq, s, sumq);
  return ohara_launch_status();
}

int ohara_gemv_ternary_i8(const int8_t* q, int ldq, const float* s, const int32_t* sumq, const uint32_t* wp, int n,
                          int k, float gamma, int rows, const uint16_t* resid, int ldr, uint16_t* out, int ldo,
                          int32_t* acc_out, int ldacc, void* stream) {
  if (!q || !s || !sumq || !wp || !out || n < 1 || k < 1 || rows < 1) return OHARA_EINVAL;
  if ((ldq & 15) || ldq < k || ldo < n || (resid && ldr < n) || (acc_out && ldacc < n)) return OHARA_EINVAL;
  BitArgs a{};
  a.wp = reinterpret_cast<const uint4*>(wp); a.gamma = gamma;
  a.q = q; a.ldq = ldq; a.s = s; a.sumq = sumq;
  a.B = rows; a.N = n; a.K = k; a.out = out; a.ldo = ldo; a.resid = resid; a.ldr = ldr;
  a.acc_out = acc_out; a.ldacc = ldacc;
  return launch_bit<false>(a, (hipStream_t)stream);
}

int ohara_bitlinear_bf16(const uint16_t* x, int ldx, const uint16_t* pre_norm_w, const uint16_t* norm_w, float eps,
                         const uint32_t* wp, int n, int k, float gamma, int rows, const uint16_t* resid, int ldr,
                         uint16_t* out, int ldo, int32_t* acc_out, int ldacc, void* stream) {
  if (!x || !norm_w || !wp || !out || n < 1 || k < 1 || rows < 1) return OHARA_EINVAL;
  if (ldx < k || ldo < n || (resid && ldr < n) || (acc_out && ldacc < n)) return OHARA_EINVAL;
  if ((k & 7) || (ldx & 7)) return OHARA_EINVAL;  // 16-byte activation loads
  if (k > BL_EPL * 64) return OHARA_ESIZE;
  BitArgs a{};
  a.wp = reinterpret_cast<const uint4*>(wp); a.gamma = gamma;
  a.x = x; a.ldx = ldx; a.nw = norm_w; a.pre_w = pre_norm_w; a.eps = eps;
  a.B = rows; a.N = n; a.K = k; a.out = out; a.ldo = ldo; a.resid = resid; a.ldr = ldr;
  a.acc_out = acc_out; a.ldacc = ldacc;
  return launch_bit<true>(a, (hipStream_t)stream);
}

static size_t bit_smem(int rows, int k, int* btt_out) {
  const int KC = (k + 255) >> 8;
  const int ldq = (KC << 8) + 16;
  const int bt = (rows + 15) / 16;
  const int btt = bt == 3 ? 4 : bt;
  *btt_out = btt;
  return (((size_t)btt * 16 * ldq + 255) & ~(size_t)255) + (size_t)btt * 16 * 8 + (size_t)3 * btt * 64 * 4 * sizeof(int) +
         (size_t)4 * (KC << 8) * 2;
}

int ohara_bitlinear_qkv_rope_append_bf16(const uint16_t* x, int ldx, const uint16_t* pre_norm_w, float eps, int k,
                                         const uint16_t* const* norm_w, const uint32_t* const* wp, const float* gamma,
                                         int batch, int seq_len, int h, int h_kv, int dh, const uint16_t* cos,
                                         const uint16_t* sin, int pos, const int32_t* pos_dev, uint16_t* q_out,
                                         uint16_t* kcache, uint16_t* vcache, int t_max, void* stream) {
  if (!x || !norm_w || !wp || !gamma || !cos || !sin || !q_out || !kcache || !vcache) return OHARA_EINVAL;
  if (batch < 1 || seq_len < 1 || h < 1 || h_kv < 1 || h % h_kv || dh < 4 || (dh & 3) || t_max < 1) return OHARA_EINVAL;
  if ((k & 7) || (ldx & 7) || ldx < k) return OHARA_EINVAL;
  if (!pos_dev && (pos < 0 || pos + seq_len > t_max)) return OHARA_EINVAL;
  const int rows = batch * seq_len;
  if (rows > 64 || k > BL_EPL * 64) return OHARA_ESIZE;
  BitQkvArgs a{};
  const int n[3] = {h * dh, h_kv * dh, h_kv * dh};
  int total = 0;
  for (int i = 0; i < 3; ++i) {
    if (!norm_w[i] || !wp[i]) return OHARA_EINVAL;
    BitArgs& p = a.p[i];
    p.wp = reinterpret_cast<const uint4*>(wp[i]); p.gamma = gamma[i];
    p.x = x; p.ldx = ldx; p.nw = norm_w[i]; p.pre_w = pre_norm_w; p.eps = eps;
    p.B = rows; p.N = n[i]; p.K = k;
    a.strips[i] = (n[i] + 15) / 16;
    total += a.strips[i];
  }
  a.H = h; a.Hkv = h_kv; a.Dh = dh; a.Tmax = t_max; a.S = seq_len; a.pos = pos; a.pos_dev = pos_dev;
  a.cos = cos; a.sin = sin; a.q_out = q_out; a.kcache = kcache; a.vcache = vcache;
  int btt;
  const size_t smem = bit_smem(rows, k, &btt);
  if (smem > 160 * 1024) return OHARA_ESIZE;
  hipStream_t st = (hipStream_t)stream;
#define OHARA_BITQ(BTV)                                                                                     \
  do {                                                                                                      \
    if (smem > 64 * 1024)                                                                                   \
      (void)hipFuncSetAttribute((const void*)bitlinear_qkv_kernel<BTV>, hipFuncAttributeMaxDynamicSharedMemorySize, \
                                (int)smem);                                                                 \
    hipLaunchKernelGGL((bitlinear_qkv_kernel<BTV>), dim3(total), dim3(256), smem, st, a);                   \
  } while (0)
  if (btt == 1) OHARA_BITQ(1);
  else if (btt == 2) OHARA_BITQ(2);
  else OHARA_BITQ(4);
#undef OHARA_BITQ
  return ohara_launch_status();
}

int ohara_bitlinear_gate_up_bf16(const uint16_t* x, int ldx, const uint16_t* pre_norm_w, float eps, int k, int f,
                                 const uint16_t* gate_norm_w, const uint32_t* gate_wp, float gate_gamma,
                                 const uint16_t* up_norm_w, const uint32_t* up_wp, float up_gamma, int rows,
                                 uint16_t* out, int ldo, void* stream) {
  if (!x || !gate_norm_w || !gate_wp || !up_norm_w || !up_wp || !out || rows < 1 || k < 1 || f < 1) return OHARA_EINVAL;
  if ((k & 7) || (ldx & 7) || ldx < k || ldo < f) return OHARA_EINVAL;
  if (rows > 64 || k > BL_EPL * 64) return OHARA_ESIZE;
  BitGateUpArgs a{};
  BitArgs* ps[2] = {&a.gate, &a.up};
  for (int i = 0; i < 2; ++i) {
    BitArgs& p = *ps[i];
    p.wp = reinterpret_cast<const uint4*>(i ? up_wp : gate_wp); p.gamma = i ? up_gamma : gate_gamma;
    p.x = x; p.ldx = ldx; p.nw = i ? up_norm_w : gate_norm_w; p.pre_w = pre_norm_w; p.eps = eps;
    p.B = rows; p.N = f; p.K = k; p.out = out; p.ldo = ldo;
  }
  int btt;
  const size_t smem = bit_smem(rows, k, &btt);
  if (smem > 160 * 1024) return OHARA_ESIZE;
  hipStream_t st = (hipStream_t)stream;
  const int strips = (f + 15) / 16;
#define OHARA_BITG(BTV)                                                                                     \
  do {                                                                                                      \
    if (smem > 64 * 1024)                                                                                   \
      (void)hipFuncSetAttribute((const void*)bitlinear_gate_up_kernel<BTV>,                                 \
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);                     \
    hipLaunchKernelGGL((bitlinear_gate_up_kernel<BTV>), dim3(strips), dim3(256), smem, st, a);              \
  } while (0)
  if (btt == 1) OHARA_BITG(1);
  else if (btt == 2) OHARA_BITG(2);
  else OHARA_BITG(4);
#undef OHARA_BITG
  return ohara_launch_status();
}

int ohara_silu_mul_bf16(const uint16_t* gate, const uint16_t* up, uint16_t* out, int64_t n, void* stream) {
  if (!gate || !up || !out || n < 1) return OHARA_EINVAL;
  hipLaunchKernelGGL(silu_mul_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, gate, up, out,
                     (size_t)n);
  return ohara_launch_status();
}

int ohara_rope_append_bf16(uint16_t* q, const uint16_t* k, const uint16_t* v, int batch, int seq_len, int h, int h_kv,
                           int dh, const uint16_t* cos, const uint16_t* sin, int pos, const int32_t* pos_dev,
                           uint16_t* kcache, uint16_t* vcache, int t_max, void* stream) {
  if (!q || !k || !v || !cos || !sin || !kcache || !vcache) return OHARA_EINVAL;
  if (batch < 1 || seq_len < 1 || h < 1 || h_kv < 1 || dh < 2 || (dh & 1) || t_max < 0) return OHARA_EINVAL;
  if (!pos_dev && (pos < 0 || (t_max > 0 && pos + seq_len > t_max))) return OHARA_EINVAL;
  hipLaunchKernelGGL(rope_append_kernel, dim3(batch * seq_len), dim3(256), 0, (hipStream_t)stream, q, k, v, seq_len, h,
                     h_kv, dh, cos, sin, pos, pos_dev, kcache, vcache, t_max);
  return ohara_launch_status();
}

}  // extern "C"
