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

constexpr int BL_EPL = 96;  // values per lane when a wave holds one activation row: K <= 6144

struct QuantOut {
  float s;      // 127 / max|x_hat|
  int sumq;     // sum of the quantised row
};

// One wave normalises and quantises one row held in registers (16-byte loads: lane l owns the
// 8-value pieces l, l + 64, ...).  pre_w (optional) is the weight of a block-level RMSNorm applied
// first (ohara/models/llama.py:199-200 norm1 / norm2), nw the BitLinear's own norm weight.
// xq: int8 destination (LDS or global).  Returns (s, sum q) in every lane.  K % 8 == 0.
template <int EPL>
__device__ __forceinline__ QuantOut wave_quant_row(const bf16_t* x, const bf16_t* pre_w, const bf16_t* nw, int K,
                                                   float eps, int8_t* xq) {
  constexpr int NP = EPL / 8;  // pieces per lane
  const int lane = threadIdx.x & 63;
  const int pieces = K >> 3;
  float v[NP][8];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    const int p = i * 64 + lane;
    const uint4 u = p < pieces ? ldg16(x + (size_t)p * 8) : make_uint4(0, 0, 0, 0);
    const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      v[i][2 * j] = lo_bf(w[j]);
      v[i][2 * j + 1] = hi_bf(w[j]);
      ss += v[i][2 * j] * v[i][2 * j] + v[i][2 * j + 1] * v[i][2 * j + 1];
    }
  }
  if (pre_w) {
    ss = wave_sum(ss);
    const float rinv0 = 1.0f / sqrtf(ss / (float)K + eps);
    ss = 0.f;
#pragma unroll
    for (int i = 0; i < NP; ++i) {
      const int p = i * 64 + lane;
      if (p < pieces) {
        const uint4 u = ldg16(pre_w + (size_t)p * 8);
        const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          v[i][2 * j] = rbf(rbf(v[i][2 * j] * rinv0) * lo_bf(w[j]));
          v[i][2 * j + 1] = rbf(rbf(v[i][2 * j + 1] * rinv0) * hi_bf(w[j]));
          ss += v[i][2 * j] * v[i][2 * j] + v[i][2 * j + 1] * v[i][2 * j + 1];
        }
      }
    }
  }
  ss = wave_sum(ss);
  const float rinv = 1.0f / sqrtf(ss / (float)K + eps);
  float mx = 0.f;
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    const int p = i * 64 + lane;
    if (p < pieces) {
      const uint4 u = ldg16(nw + (size_t)p * 8);
      const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v[i][2 * j] = rbf(rbf(v[i][2 * j] * rinv) * lo_bf(w[j]));  // RMSNorm output in the model dtype
        v[i][2 * j + 1] = rbf(rbf(v[i][2 * j + 1] * rinv) * hi_bf(w[j]));
        mx = fmaxf(mx, fmaxf(fabsf(v[i][2 * j]), fabsf(v[i][2 * j + 1])));
      }
    }
  }
  mx = wave_max(mx);
  const float s = 127.0f / fmaxf(mx, 1e-5f);
  int sq = 0;
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    const int p = i * 64 + lane;
    if (p < pieces) {
      uint32_t pk[2] = {0u, 0u};
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int qi = (int)fminf(fmaxf(rintf(v[i][j] * s), -128.f), 127.f);
        sq += qi;
        pk[j >> 2] |= ((uint32_t)qi & 0xffu) << (8 * (j & 3));
      }
      *reinterpret_cast<uint2*>(xq + (size_t)p * 8) = make_uint2(pk[0], pk[1]);
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) sq += __shfl_xor(sq, o, WAVE);
  return QuantOut{s, sq};
}

__global__ __launch_bounds__(256) void act_quant_kernel(const bf16_t* x, int ldx, const bf16_t* nw, int rows, int K,
                                                        float eps, int8_t* q, int ldq, float* s_out, int* sumq_out) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = blockIdx.x * 4 + wave;
  if (r >= rows) return;
  const QuantOut o = wave_quant_row<BL_EPL>(x + (size_t)r * ldx, nullptr, nw, K, eps, q + (size_t)r * ldq);
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

template <int BT, bool FUSED>
__global__ __launch_bounds__(256) void bitlinear_kernel(BitArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int strip = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m = lane & 15, g = lane >> 4;
  const int KC = (a.K + 255) >> 8;      // 256-column chunks
  const int Kp = KC << 8;
  const int ldq = Kp + 16;              // LDS row stride in bytes (16-byte skew against bank conflicts)
  int8_t* xq = reinterpret_cast<int8_t*>(smem);
  float* s_s = reinterpret_cast<float*>(smem + (((size_t)BT * 16 * ldq + 255) & ~(size_t)255));
  int* s_sum = reinterpret_cast<int*>(s_s + BT * 16);
  int* red = s_sum + BT * 16;           // [3][BT][64][4]

  // the first weights of this wave are requested before the activations are prepared
  const int per = (KC + 3) >> 2;
  const int c0 = wave * per, c1 = min(KC, c0 + per);
  const uint4* wrow = a.wp + (size_t)strip * KC * 64 + lane;
  constexpr int CH = 6;
  uint4 wpre[CH];
#pragma unroll
  for (int c = 0; c < CH; ++c) wpre[c] = (c0 + c < c1) ? ldg16_nt(wrow + (size_t)(c0 + c) * 64) : make_uint4(0, 0, 0, 0);

  // ---- activations -> int8 rows in LDS ---------------------------------------------------
  for (int i = tid; i < BT * 16 * (ldq / 16); i += 256) reinterpret_cast<uint4*>(xq)[i] = make_uint4(0, 0, 0, 0);
  __syncthreads();
  if (FUSED) {
    for (int b = wave; b < a.B; b += 4) {
      const QuantOut o = wave_quant_row<BL_EPL>(a.x + (size_t)b * a.ldx, a.pre_w, a.nw, a.K, a.eps, xq + (size_t)b * ldq);
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
  i32x4 acc[BT];
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
  if (wave != 0) return;
#pragma unroll
  for (int t = 0; t < BT; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i)
      acc[t][i] += red[((0 * BT + t) * 64 + lane) * 4 + i] + red[((1 * BT + t) * 64 + lane) * 4 + i] +
                   red[((2 * BT + t) * 64 + lane) * 4 + i];

  const int r0 = strip * 16 + 4 * g;
#pragma unroll
  for (int t = 0; t < BT; ++t) {
    const int b = m + 16 * t;
    if (b >= a.B) continue;
    const float s = s_s[b];
    const int sq = s_sum[b];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = r0 + i;
      if (n >= a.N) continue;
      const int ai = acc[t][i] - sq;  // codes are T+1
      if (a.acc_out) a.acc_out[(size_t)b * a.ldacc + n] = ai;
      float y = rbf(__fmul_rn(__fdiv_rn((float)ai, s), a.gamma));
      if (a.resid) y = bf2f(a.resid[(size_t)b * a.ldr + n]) + y;
      a.out[(size_t)b * a.ldo + n] = f2bf(y);
    }
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
  if (pos < 0 || pos >= Tmax) return;
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
  bf16_t* kd = kc + (((size_t)seq * Tmax + pos) * Hkv) * D;
  bf16_t* vd = vc + (((size_t)seq * Tmax + pos) * Hkv) * D;
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
  for (int r = 0; r < a0.B; r += 64) {
    BitArgs a = a0;
    a.B = a0.B - r < 64 ? a0.B - r : 64;
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
    const size_t smem = (((size_t)btt * 16 * ldq + 255) & ~(size_t)255) + (size_t)btt * 16 * 8 +
                        (size_t)3 * btt * 64 * 4 * sizeof(int);
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
  hipLaunchKernelGGL(act_quant_kernel, dim3((rows + 3) / 4), dim3(256), 0, (hipStream_t)stream, x, ldx, norm_w, rows, k,
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
  if (batch < 1 || seq_len < 1 || h < 1 || h_kv < 1 || dh < 2 || (dh & 1) || t_max < 1) return OHARA_EINVAL;
  if (!pos_dev && (pos < 0 || pos + seq_len > t_max)) return OHARA_EINVAL;
  hipLaunchKernelGGL(rope_append_kernel, dim3(batch * seq_len), dim3(256), 0, (hipStream_t)stream, q, k, v, seq_len, h,
                     h_kv, dh, cos, sin, pos, pos_dev, kcache, vcache, t_max);
  return ohara_launch_status();
}

}  // extern "C"
