// Weight-streaming skinny GEMM for the decode projections (batch <= 64).
//
// y[b, n] = sum_k x[b, k] * W[n, k].  W is read exactly once, in a packed tile
// order whose every wave-load is one contiguous 1 KiB (64 lanes x 16 B), straight
// into the A operand of v_mfma_f32_16x16x32_bf16; the activations are the B
// operand (16 batch columns per MFMA), so batch 1..16 costs the same weight
// stream.  One workgroup (4 waves) owns one 16-row strip; the waves split K and
// their fp32 partial tiles are summed in a fixed order through LDS, so results do
// not depend on scheduling.
//
// Fusions (rounding points follow the reference's bf16 eager path):
//   prologue  RMSNorm           ohara/modules/norm.py:16-21
//   epilogue  residual add      ohara/models/llama.py:199-200
//             SwiGLU            ohara/modules/mlp.py:152
//             rotary + KV append ohara/embeddings_pos/rotary.py:55-93,
//                               ohara/modules/kv_cache.py:104-105
#include "gemm_epilogue.h"

namespace {

__device__ __forceinline__ float sumsq8(uint4 v) {
  float s = 0.f;
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    float a = lo_bf(w[i]), b = hi_bf(w[i]);
    s += a * a + b * b;
  }
  return s;
}

// bf16(bf16(x * rinv) * w) on 8 packed values.
__device__ __forceinline__ uint4 norm8(uint4 xv, uint4 wv, float rinv) {
  const uint32_t xs[4] = {xv.x, xv.y, xv.z, xv.w};
  const uint32_t ws[4] = {wv.x, wv.y, wv.z, wv.w};
  uint32_t o[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    float a = rbf(lo_bf(xs[i]) * rinv) * lo_bf(ws[i]);
    float b = rbf(hi_bf(xs[i]) * rinv) * hi_bf(ws[i]);
    o[i] = pack_bf(a, b);
  }
  return make_uint4(o[0], o[1], o[2], o[3]);
}

// LayerNorm on 8 packed values: bf16((x - mean) * rstd * w + b), one rounding (nn.LayerNorm).
__device__ __forceinline__ uint4 lnorm8(uint4 xv, uint4 wv, uint4 bv, float mean, float rstd) {
  const uint32_t xs[4] = {xv.x, xv.y, xv.z, xv.w};
  const uint32_t ws[4] = {wv.x, wv.y, wv.z, wv.w};
  const uint32_t bs[4] = {bv.x, bv.y, bv.z, bv.w};
  uint32_t o[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
    o[i] = pack_bf((lo_bf(xs[i]) - mean) * rstd * lo_bf(ws[i]) + lo_bf(bs[i]),
                   (hi_bf(xs[i]) - mean) * rstd * hi_bf(ws[i]) + hi_bf(bs[i]));
  return make_uint4(o[0], o[1], o[2], o[3]);
}

__device__ __forceinline__ float sum8(uint4 v) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) s += lo_bf(w[i]) + hi_bf(w[i]);
  return s;
}

// NORM: 0 none, 1 RMSNorm (norm.py:16-21), 2 LayerNorm with bias (phi.py:132).
// NW waves per workgroup split K.  A workgroup keeps NW * CH KiB of weight loads in flight, so when
// there are too few strips to put several workgroups on every CU (few output rows, long K) 16 waves
// instead of 4 are what fills the memory pipeline.
template <int BT, int NORM, int EPI, int NW = 4>
__global__ __launch_bounds__(NW * 64) void skinny_kernel(GemmArgs a) {
  // k-steps whose loads are issued back to back (the many-wave variants have no norm operands to hold)
  constexpr int CH = (NORM == 0 && NW > 4) ? 10 : (BT <= 2 ? 6 : 4);
  // workgroup id -> (strip, chunk of 16*BT rows).  Ids go round-robin over the 8 XCDs; the chunks of
  // one strip get ids 8 apart, so they run on the same XCD and share its L2 copy of the weights.
  const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
  const int strip = (local / a.ny) * 8 + xcd;
  const int rbase = (local % a.ny) * 16 * BT;
  if (strip >= a.nstrips) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m = lane & 15, g = lane >> 4;
  const int KS = (a.K + 31) >> 5;
  const int per_wave = (KS + NW - 1) / NW;
  const int j0 = wave * per_wave;
  const int j1 = min(KS, j0 + per_wave);

  __shared__ float red[NW - 1][BT][64][4];
  __shared__ float ssq[NW][BT * 16];
  __shared__ float ssum[NORM == 2 ? NW : 1][BT * 16];

  // A launch of this kernel is a chain of memory round trips - the rows for the norm, the weights, what the epilogue
  // adds or rotates with - and lasts about as long as their sum (6-9 us for 1-9 MB at 32 rows).  What does not depend
  // on anything computed here is therefore requested first: the epilogue's operands (wave 0 finishes the fragments),
  // and, where a wave's share of K is at most SP k-steps (K <= 1024 with four waves), the rows, the norm weights and
  // the weights of the whole share in one go - the rows arrive first (loads return in order), the norm's sums run
  // while the weights are still on their way, and the rows are not fetched a second time.
  constexpr int SP = 8;
  const bool pre_ok = ((a.N | a.ldo | a.ldr | a.ldr2) & 3) == 0 && EPI != EPI_STORE && EPI != EPI_SWIGLU;
  EpiPre ep[BT];
  if (wave == 0 && pre_ok) {
#pragma unroll
    for (int t = 0; t < BT; ++t) gemm_epilogue_fetch<EPI>(a, rbase + m + 16 * t, strip, g, ep[t]);
  }
  const uint4* wrow = a.wp + (size_t)strip * KS * 64 + lane;
  f32x4 acc[BT];
#pragma unroll
  for (int t = 0; t < BT; ++t) acc[t] = (f32x4){0.f, 0.f, 0.f, 0.f};

  float rinv[BT], mean[BT];
  if (NORM == 1 && BT == 1 && per_wave <= SP) {
    uint4 xv[SP], nw[SP], wv[SP];
    const int b = rbase + m;
#pragma unroll
    for (int c = 0; c < SP; ++c) {
      const int k0 = 32 * (j0 + c) + 8 * g;
      const bool in = j0 + c < j1 && b < a.B && k0 < a.K;
      xv[c] = ldg16(a.x + (in ? (size_t)b * a.ldx + k0 : (size_t)0));
    }
#pragma unroll
    for (int c = 0; c < SP; ++c) {
      const int k0 = 32 * (j0 + c) + 8 * g;
      nw[c] = ldg16(a.norm_w + (j0 + c < j1 && k0 < a.K ? k0 : 0));
    }
#pragma unroll
    for (int c = 0; c < SP; ++c) wv[c] = ldg16_nt(wrow + (size_t)min(j0 + c, KS - 1) * 64);
    __builtin_amdgcn_sched_barrier(0);
    float part = 0.f;
#pragma unroll
    for (int c = 0; c < SP; ++c) {
      const int k0 = 32 * (j0 + c) + 8 * g;
      if (j0 + c < j1 && b < a.B && k0 < a.K) part += sumsq8(xv[c]);
    }
    part = lanes_sum<16, 16>(part);
    part = lanes_sum<32, 32>(part);
    if (g == 0) ssq[wave][m] = part;
    __syncthreads();
    float tot = ssq[0][m];
#pragma unroll
    for (int w = 1; w < NW; ++w) tot += ssq[w][m];
    rinv[0] = 1.0f / sqrtf(tot / (float)a.K + a.eps);
    mean[0] = 0.f;
#pragma unroll
    for (int c = 0; c < SP; ++c) {
      const int k0 = 32 * (j0 + c) + 8 * g;
      const bool in = j0 + c < j1 && b < a.B && k0 < a.K;
      const bool inw = j0 + c < j1;
      const uint4 xn = in ? norm8(xv[c], (k0 < a.K) ? nw[c] : make_uint4(0, 0, 0, 0), rinv[0]) : make_uint4(0, 0, 0, 0);
      if (inw)
        acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wv[c]), __builtin_bit_cast(bf16x8, xn),
                                                         acc[0], 0, 0, 0);
    }
  } else {
  if (NORM) {
    float part[BT], psum[BT];
#pragma unroll
    for (int t = 0; t < BT; ++t) part[t] = psum[t] = 0.f;
    // CH k-steps per round, all loads of a round issued before the first is used (one round trip
    // per round instead of one per k-step); pieces outside the matrix read element 0 and are not added
    for (int j = j0; j < j1; j += CH) {
      uint4 xv[CH][BT];
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        const int k0 = 32 * (j + c) + 8 * g;
#pragma unroll
        for (int t = 0; t < BT; ++t) {
          const int b = rbase + m + 16 * t;
          const bool in = j + c < j1 && b < a.B && k0 < a.K;
          xv[c][t] = ldg16(a.x + (in ? (size_t)b * a.ldx + k0 : (size_t)0));
        }
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        const int k0 = 32 * (j + c) + 8 * g;
#pragma unroll
        for (int t = 0; t < BT; ++t) {
          const int b = rbase + m + 16 * t;
          if (j + c < j1 && b < a.B && k0 < a.K) {
            part[t] += sumsq8(xv[c][t]);
            if (NORM == 2) psum[t] += sum8(xv[c][t]);
          }
        }
      }
    }
#pragma unroll
    for (int t = 0; t < BT; ++t) {
      float p = part[t];
      p = lanes_sum<16, 16>(p);
      p = lanes_sum<32, 32>(p);
      if (g == 0) ssq[wave][16 * t + m] = p;
      if (NORM == 2) {
        float q = psum[t];
        q = lanes_sum<16, 16>(q);
        q = lanes_sum<32, 32>(q);
        if (g == 0) ssum[wave][16 * t + m] = q;
      }
    }
    __syncthreads();
#pragma unroll
    for (int t = 0; t < BT; ++t) {
      float tot = ssq[0][16 * t + m];
#pragma unroll
      for (int w = 1; w < NW; ++w) tot += ssq[w][16 * t + m];
      if (NORM == 2) {
        // mean and biased variance from the sums of x and x^2 (fp32; rows are O(1) activations)
        float sm = ssum[0][16 * t + m];
#pragma unroll
        for (int w = 1; w < NW; ++w) sm += ssum[w][16 * t + m];
        mean[t] = sm / (float)a.K;
        rinv[t] = 1.0f / sqrtf(fmaxf(tot / (float)a.K - mean[t] * mean[t], 0.f) + a.eps);
      } else {
        mean[t] = 0.f;
        rinv[t] = 1.0f / sqrtf(tot / (float)a.K + a.eps);
      }
    }
  }

  // A group of CH k-steps: all loads of the group (weights, norm weights, the activations of
  // every 16-row block) are issued before the first product, so their latencies overlap.
  auto group = [&](int j, int n) {  // k-steps j .. j+n-1, n <= CH
    uint4 wv[CH], nw[CH], nb[NORM == 2 ? CH : 1], xv[CH][BT];
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int k0 = 32 * (j + c) + 8 * g;
      const bool in = c < n;
      wv[c] = in ? ldg16_nt(wrow + (size_t)(j + c) * 64) : make_uint4(0, 0, 0, 0);
      nw[c] = (NORM && in && k0 < a.K) ? ldg16(a.norm_w + k0) : make_uint4(0, 0, 0, 0);
      if (NORM == 2) nb[c] = (in && k0 < a.K) ? ldg16(a.norm_b + k0) : make_uint4(0, 0, 0, 0);
#pragma unroll
      for (int t = 0; t < BT; ++t) {
        const int b = rbase + m + 16 * t;
        xv[c][t] = (in && b < a.B && k0 < a.K) ? ldg16(a.x + (size_t)b * a.ldx + k0) : make_uint4(0, 0, 0, 0);
      }
    }
#pragma unroll
    for (int c = 0; c < CH; ++c) {
#pragma unroll
      for (int t = 0; t < BT; ++t) {
        uint4 xn = xv[c][t];
        if (NORM == 1) xn = norm8(xn, nw[c], rinv[t]);
        if (NORM == 2) {
          // rows beyond the batch and columns beyond K must stay zero (the bias would leak in)
          const bool live = rbase + m + 16 * t < a.B && 32 * (j + c) + 8 * g < a.K && c < n;
          xn = live ? lnorm8(xn, nw[c], nb[c], mean[t], rinv[t]) : make_uint4(0, 0, 0, 0);
        }
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wv[c]),
                                                         __builtin_bit_cast(bf16x8, xn), acc[t], 0, 0, 0);
      }
    }
  };

  int j = j0;
  for (; j + CH <= j1; j += CH) group(j, CH);
  if (j < j1) group(j, j1 - j);
  }

  // Fixed-order cross-wave sum: ((w0 + w1) + w2) + w3 ...
  if (wave > 0) {
#pragma unroll
    for (int t = 0; t < BT; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) red[wave - 1][t][lane][i] = acc[t][i];
  }
  __syncthreads();
  if (wave != 0) return;
#pragma unroll
  for (int t = 0; t < BT; ++t)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int w = 0; w < NW - 1; ++w) acc[t][i] += red[w][t][lane][i];
    }

#pragma unroll
  for (int t = 0; t < BT; ++t) {
    const int b = rbase + m + 16 * t;
    if (b < a.B) {
      if (pre_ok) gemm_epilogue<EPI, true>(a, b, strip, g, acc[t], ep[t]);
      else gemm_epilogue<EPI>(a, b, strip, g, acc[t]);
    }
  }
}

// Many strips (the vocabulary projection): the activations are the stationary operand.  Every
// workgroup normalises all rows once into LDS (up to 64 rows, zero-padded to
// 16*BT rows and 32*KS columns), then each of its 8 waves walks whole strips - full K, no
// cross-wave sum - reading the MFMA B operands from LDS, so the weights are read exactly once
// whatever the row count and the norm is computed once per workgroup, not once per strip.
constexpr int WIDE_WAVES = 8;
constexpr int WIDE_CH = 12;

template <int BT, bool NORM, int EPI>
__global__ __launch_bounds__(WIDE_WAVES * 64) void wide_kernel(GemmArgs a) {
  extern __shared__ __align__(16) unsigned char wide_smem[];
  bf16_t* xs = reinterpret_cast<bf16_t*>(wide_smem);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m = lane & 15, g = lane >> 4;
  const int KS = (a.K + 31) >> 5;
  const int ldxs = KS * 32 + 8;
  const int stride = gridDim.x * WIDE_WAVES;
  int strip = blockIdx.x * WIDE_WAVES + wave;
  // two register buffers of WIDE_CH k-steps; the first strip's are requested before the
  // activations are staged, so the weight stream starts with the kernel
  uint4 wa[WIDE_CH], wb[WIDE_CH];
  // No branch around a load and nothing that touches the value: k-steps and strips outside the
  // matrix read a valid tile instead and are never multiplied (mul() skips k-steps >= KS, the strip
  // loop ends before a strip >= nstrips is used).  The compiler can then count the loads in flight
  // and wait for one buffer while the other fills.
  auto load = [&](uint4* w, int st, int j) {
    const uint4* wrow = a.wp + (size_t)(st < a.nstrips ? st : 0) * KS * 64 + lane;
#pragma unroll
    for (int c = 0; c < WIDE_CH; ++c) w[c] = ldg16_nt(wrow + (size_t)min(j + c, KS - 1) * 64);
  };
  load(wa, strip, 0);
  load(wb, strip, WIDE_CH);

  if (a.K <= 1024) {
    // every row of this wave is requested before any is used (K <= 1024: two 16-byte pieces per lane)
    constexpr int RPW = 16 * BT / WIDE_WAVES;
    uint4 v[RPW][2], nwv[2];
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      const int k = lane * 8 + 512 * c;
      nwv[c] = (NORM && k < a.K) ? ldg16(a.norm_w + k) : make_uint4(0, 0, 0, 0);
#pragma unroll
      for (int r = 0; r < RPW; ++r) {
        const int b = wave + WIDE_WAVES * r;
        v[r][c] = (b < a.B && k < a.K) ? ldg16(a.x + (size_t)b * a.ldx + k) : make_uint4(0, 0, 0, 0);
      }
    }
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
      const int b = wave + WIDE_WAVES * r;
      float rinv = 1.f;
      if (NORM) rinv = 1.0f / sqrtf(wave_sum(sumsq8(v[r][0]) + sumsq8(v[r][1])) / (float)a.K + a.eps);
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        const int k = lane * 8 + 512 * c;
        if (k < KS * 32)
          *reinterpret_cast<uint4*>(xs + (size_t)b * ldxs + k) = NORM ? norm8(v[r][c], nwv[c], rinv) : v[r][c];
      }
    }
  } else {
    for (int b = wave; b < 16 * BT; b += WIDE_WAVES) {
      float rinv = 1.f;
      if (NORM && b < a.B) {
        float ss = 0.f;
        for (int k = lane * 8; k < a.K; k += 512) ss += sumsq8(ldg16(a.x + (size_t)b * a.ldx + k));
        rinv = 1.0f / sqrtf(wave_sum(ss) / (float)a.K + a.eps);
      }
      for (int k = lane * 8; k < KS * 32; k += 512) {
        uint4 v = make_uint4(0, 0, 0, 0);
        if (b < a.B && k < a.K) {
          v = ldg16(a.x + (size_t)b * a.ldx + k);
          if (NORM) v = norm8(v, ldg16(a.norm_w + k), rinv);
        }
        *reinterpret_cast<uint4*>(xs + (size_t)b * ldxs + k) = v;
      }
    }
  }
  __syncthreads();

  const bf16_t* xrow = xs + (size_t)m * ldxs + 8 * g;
  for (; strip < a.nstrips; strip += stride) {
    f32x4 acc[BT];
#pragma unroll
    for (int t = 0; t < BT; ++t) acc[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
    auto mul = [&](const uint4* w, int j) {
#pragma unroll
      for (int c = 0; c < WIDE_CH; ++c) {
        if (j + c < KS) {
#pragma unroll
          for (int t = 0; t < BT; ++t) {
            const uint4 xv = *reinterpret_cast<const uint4*>(xrow + (size_t)(16 * t) * ldxs + 32 * (j + c));
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, w[c]),
                                                             __builtin_bit_cast(bf16x8, xv), acc[t], 0, 0, 0);
          }
        }
      }
    };
    // wa / wb hold k-steps [j, j + CH) and [j + CH, j + 2 CH) of this strip; each buffer is refilled
    // (from this strip, or from the start of the wave's next one) as soon as it has been multiplied
    for (int j = 0; j < KS; j += 2 * WIDE_CH) {
      const bool more = j + 2 * WIDE_CH < KS;
      mul(wa, j);
      if (more) load(wa, strip, j + 2 * WIDE_CH);
      else load(wa, strip + stride, 0);
      mul(wb, j + WIDE_CH);
      if (more) load(wb, strip, j + 3 * WIDE_CH);
      else load(wb, strip + stride, WIDE_CH);
    }
#pragma unroll
    for (int t = 0; t < BT; ++t) {
      const int b = m + 16 * t;
      if (b < a.B) gemm_epilogue<EPI>(a, b, strip, g, acc[t]);
    }
  }
}

template <int BT>
int launch_wide_bt(const GemmArgs& a, int epi, hipStream_t st) {
  const int KS = (a.K + 31) >> 5;
  const size_t smem = (size_t)16 * BT * (KS * 32 + 8) * sizeof(bf16_t);
  const int grid = (a.nstrips + WIDE_WAVES - 1) / WIDE_WAVES < 256 ? (a.nstrips + WIDE_WAVES - 1) / WIDE_WAVES : 256;
#define OHARA_WIDE(NORM_, EPI_)                                                                                   \
  do {                                                                                                            \
    if (smem > 64 * 1024)                                                                                         \
      (void)hipFuncSetAttribute((const void*)wide_kernel<BT, NORM_, EPI_>, hipFuncAttributeMaxDynamicSharedMemorySize, \
                                (int)smem);                                                                       \
    hipLaunchKernelGGL((wide_kernel<BT, NORM_, EPI_>), dim3(grid), dim3(WIDE_WAVES * 64), smem, st, a);           \
  } while (0)
  if (epi == EPI_STORE) {
    if (a.norm_w) OHARA_WIDE(true, EPI_STORE);
    else OHARA_WIDE(false, EPI_STORE);
  } else {
    return OHARA_EINVAL;
  }
#undef OHARA_WIDE
  return ohara_launch_status();
}

// The wide kernel serves plain stores of many strips whose rows fit LDS.
bool wide_applies(const GemmArgs& a, int epi, int strips) {
  const int KS = (a.K + 31) >> 5;
  const int bt = (a.B + 15) / 16;
  return epi == EPI_STORE && strips >= 1024 && a.B <= 64 && (size_t)16 * bt * (KS * 32 + 8) * 2 <= 160 * 1024;
}

int launch_wide(const GemmArgs& a0, int epi, int strips, hipStream_t st) {
  GemmArgs a = a0;
  a.nstrips = strips;
  switch ((a.B + 15) / 16) {
    case 1: return launch_wide_bt<1>(a, epi, st);
    case 2: return launch_wide_bt<2>(a, epi, st);
    case 3: return launch_wide_bt<3>(a, epi, st);
    default: return launch_wide_bt<4>(a, epi, st);
  }
}

template <int BT, bool NORM>
int launch_epi(const GemmArgs& a, int epi, int strips, hipStream_t st) {
  dim3 grid((unsigned)((strips + 7) / 8 * 8 * a.ny)), block(256);
  // Linear-with-bias calls with a long K (2048 and up): 16 waves per workgroup.  (For the d12 Llama
  // projections, K 768 / 2048 with 48 - 256 strips, 16 waves measured no faster than 4.)
  if (!NORM && epi >= EPI_BIAS && a.K >= 2048) {
    if (strips * a.ny >= 400) {  // enough workgroups for four per CU: 8 waves each measured 5-9 % faster
      dim3 mid(512);
      switch (epi) {
        case EPI_BIAS: hipLaunchKernelGGL((skinny_kernel<BT, false, EPI_BIAS, 8>), grid, mid, 0, st, a); break;
        case EPI_BIAS_GELU: hipLaunchKernelGGL((skinny_kernel<BT, false, EPI_BIAS_GELU, 8>), grid, mid, 0, st, a); break;
        case EPI_BIAS_ADD2: hipLaunchKernelGGL((skinny_kernel<BT, false, EPI_BIAS_ADD2, 8>), grid, mid, 0, st, a); break;
        default: return OHARA_EINVAL;
      }
      return ohara_launch_status();
    }
    dim3 big(1024);
    switch (epi) {
      case EPI_BIAS: hipLaunchKernelGGL((skinny_kernel<BT, false, EPI_BIAS, 16>), grid, big, 0, st, a); break;
      case EPI_BIAS_GELU: hipLaunchKernelGGL((skinny_kernel<BT, false, EPI_BIAS_GELU, 16>), grid, big, 0, st, a); break;
      case EPI_BIAS_ADD2: hipLaunchKernelGGL((skinny_kernel<BT, false, EPI_BIAS_ADD2, 16>), grid, big, 0, st, a); break;
      default: return OHARA_EINVAL;
    }
    return ohara_launch_status();
  }
  switch (epi) {
    case EPI_STORE: hipLaunchKernelGGL((skinny_kernel<BT, NORM, EPI_STORE>), grid, block, 0, st, a); break;
    case EPI_RESIDUAL: hipLaunchKernelGGL((skinny_kernel<BT, NORM, EPI_RESIDUAL>), grid, block, 0, st, a); break;
    case EPI_SWIGLU: hipLaunchKernelGGL((skinny_kernel<BT, NORM, EPI_SWIGLU>), grid, block, 0, st, a); break;
    case EPI_ROPE: hipLaunchKernelGGL((skinny_kernel<BT, NORM, EPI_ROPE>), grid, block, 0, st, a); break;
    case EPI_BIAS: hipLaunchKernelGGL((skinny_kernel<BT, NORM, EPI_BIAS>), grid, block, 0, st, a); break;
    case EPI_BIAS_GELU: hipLaunchKernelGGL((skinny_kernel<BT, NORM, EPI_BIAS_GELU>), grid, block, 0, st, a); break;
    case EPI_BIAS_ADD2: hipLaunchKernelGGL((skinny_kernel<BT, NORM, EPI_BIAS_ADD2>), grid, block, 0, st, a); break;
    default: return OHARA_EINVAL;
  }
  return ohara_launch_status();
}

// Up to 64 rows: every workgroup multiplies one strip by 16 rows; more rows are more workgroups
// per strip (the strip is then read once from HBM and again from L2), which keeps the per-wave
// register footprint and the norm work of a workgroup at the 16-row level.
int launch_chunk(const GemmArgs& a0, int epi, int strips, hipStream_t st) {
  GemmArgs a = a0;
  a.ny = (a.B + 15) / 16;
  a.nstrips = strips;
  if (a.ny > 4) return OHARA_ESIZE;
  if (epi == EPI_PHI_IN) {
    // optional LayerNorm prologue; wave count as for the Linear-with-bias calls
    dim3 grid((unsigned)((strips + 7) / 8 * 8 * a.ny));
#define OHARA_PHI_IN(NORM_)                                                                                              \
  do {                                                                                                                   \
    if (a.K < 2048) hipLaunchKernelGGL((skinny_kernel<1, NORM_, EPI_PHI_IN, 4>), grid, dim3(256), 0, st, a);             \
    else if (strips * a.ny >= 400) hipLaunchKernelGGL((skinny_kernel<1, NORM_, EPI_PHI_IN, 8>), grid, dim3(512), 0, st, a); \
    else hipLaunchKernelGGL((skinny_kernel<1, NORM_, EPI_PHI_IN, 16>), grid, dim3(1024), 0, st, a);                      \
  } while (0)
    if (a.norm_w) OHARA_PHI_IN(2);
    else OHARA_PHI_IN(0);
#undef OHARA_PHI_IN
    return ohara_launch_status();
  }
  return a.norm_w ? launch_epi<1, true>(a, epi, strips, st) : launch_epi<1, false>(a, epi, strips, st);
}

// Rows beyond 64 are processed in chunks of 64 (each chunk streams the weights once).
int launch_skinny(const GemmArgs& a0, int epi, int packed_rows, hipStream_t st) {
  const int strips = packed_rows / 16;
  const int rows = a0.B;
  if (wide_applies(a0, epi, strips)) return launch_wide(a0, epi, strips, st);
  for (int r = 0; r < rows; r += 64) {
    GemmArgs a = a0;
    a.B = rows - r < 64 ? rows - r : 64;
    a.x = a0.x + (size_t)r * a0.ldx;
    if (epi == EPI_ROPE || epi == EPI_PHI_IN) {
      a.row0 = r;
    } else {
      a.out = a0.out + (size_t)r * a0.ldo;
      if (a0.resid) a.resid = a0.resid + (size_t)r * a0.ldr;
      if (a0.resid2) a.resid2 = a0.resid2 + (size_t)r * a0.ldr2;
    }
    const int rc = launch_chunk(a, epi, strips, st);
    if (rc) return rc;
  }
  return OHARA_OK;
}

__global__ void pack_rows_kernel(const bf16_t* w, int n, int k, int ldw, const int32_t* perm, int n_padded,
                                 int KS, uint4* dst) {
  // one thread per (strip, kstep, lane)
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t total = (size_t)(n_padded / 16) * KS * 64;
  if (idx >= total) return;
  const int lane = idx & 63;
  const size_t sj = idx >> 6;
  const int j = (int)(sj % KS);
  const int s = (int)(sj / KS);
  const int m = lane & 15, g = lane >> 4;
  const int prow = 16 * s + m;
  const int src = perm ? perm[prow] : (prow < n ? prow : -1);
  const int k0 = 32 * j + 8 * g;
  uint16_t v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = (src >= 0 && src < n && k0 + i < k) ? w[(size_t)src * ldw + k0 + i] : 0;
  dst[idx] = make_uint4(v[0] | (v[1] << 16), v[2] | (v[3] << 16), v[4] | (v[5] << 16), v[6] | (v[7] << 16));
}

}  // namespace

extern "C" {

int ohara_pack_rows_bf16(const uint16_t* w, int n, int k, int ldw, const int32_t* perm, int n_padded,
                         uint16_t* dst, int64_t* bytes, void* stream) {
  if (n < 1 || k < 1 || (n_padded < n && perm == nullptr)) return OHARA_EINVAL;
  if (n_padded % 16) return OHARA_EINVAL;
  const int KS = (k + 31) / 32;
  const int64_t total = (int64_t)(n_padded / 16) * KS * 64;
  if (bytes) *bytes = total * 16;
  if (!dst) return OHARA_OK;
  if (!w || ldw < k) return OHARA_EINVAL;
  const int threads = 256;
  const int64_t blocks = (total + threads - 1) / threads;
  hipLaunchKernelGGL(pack_rows_kernel, dim3((unsigned)blocks), dim3(threads), 0, (hipStream_t)stream, w, n, k, ldw,
                     perm, n_padded, KS, reinterpret_cast<uint4*>(dst));
  return ohara_launch_status();
}

int ohara_swiglu_perm(int f, int32_t* perm_host) {
  if (f < 1 || !perm_host) return OHARA_EINVAL;
  const int fp = (f + 7) / 8 * 8;
  for (int s = 0; s < fp / 8; ++s)
    for (int g = 0; g < 4; ++g)
      for (int i = 0; i < 4; ++i) {
        const int fcol = 8 * s + 2 * g + (i & 1);
        const int src = (i < 2) ? fcol : f + fcol;
        perm_host[16 * s + 4 * g + i] = fcol < f ? src : -1;
      }
  return OHARA_OK;
}

int ohara_linear_bias_bf16(const uint16_t* x, int ldx, const uint16_t* wp, int n, int k, const uint16_t* bias, int rows,
                           int epilogue, const uint16_t* add1, int ld1, const uint16_t* add2, int ld2, uint16_t* out,
                           int ldo, void* stream) {
  if (!x || !wp || !bias || !out || n < 1 || k < 1 || rows < 1) return OHARA_EINVAL;
  if ((k & 7) || (ldx & 7) || ldx < k) return OHARA_EINVAL;  // 16-byte activation loads
  if ((n & 3) || (ldo & 3) || ldo < n) return OHARA_EINVAL;   // 8-byte bias loads and stores
  int epi;
  switch (epilogue) {
    case OHARA_LIN_BIAS: epi = EPI_BIAS; break;
    case OHARA_LIN_BIAS_GELU: epi = EPI_BIAS_GELU; break;
    case OHARA_LIN_BIAS_ADD2: epi = EPI_BIAS_ADD2; break;
    default: return OHARA_EINVAL;
  }
  if (epi == EPI_BIAS_ADD2 && (!add1 || !add2 || (ld1 & 3) || (ld2 & 3) || ld1 < n || ld2 < n)) return OHARA_EINVAL;
  GemmArgs a{};
  a.wp = reinterpret_cast<const uint4*>(wp);
  a.x = x; a.ldx = ldx;
  a.B = rows; a.N = n; a.K = k;
  a.out = out; a.ldo = ldo; a.bias = bias;
  a.resid = add1; a.ldr = ld1; a.resid2 = add2; a.ldr2 = ld2;
  // Many rows (prefill) go to the tiled kernel.  Up to 128 rows it would run N / 128 workgroups only;
  // two passes of the weight-streaming kernel over 64 rows each measured faster there (Phi-2 widths,
  // 128 rows: fc2 89 against 171 us, dense 26 against 49 us).
  if (rows > 128) return ohara_launch_gemm_tile(a, epi, (n + 15) / 16 * 16, (hipStream_t)stream);
  return launch_skinny(a, epi, (n + 15) / 16 * 16, (hipStream_t)stream);
}

int ohara_phi_block_in_bf16(const uint16_t* x, int ldx, const uint16_t* ln_w, const uint16_t* ln_b, float eps,
                            const uint16_t* wp, const uint16_t* bias, int d, int ff, int batch, int seq_len, int pos,
                            const int32_t* pos_dev, uint16_t* q, int ldq, uint16_t* kcache, uint16_t* vcache, int t_max,
                            uint16_t* act, int ldact, void* stream) {
  if (!x || !wp || !bias || !q || !kcache || !vcache || !act || (ln_w && !ln_b)) return OHARA_EINVAL;
  if (d < 8 || ff < 4 || batch < 1 || seq_len < 1 || t_max < 1) return OHARA_EINVAL;
  if ((d & 15) || (ff & 3) || (ldx & 7) || ldx < d || (ldq & 3) || ldq < d || (ldact & 3) || ldact < ff) return OHARA_EINVAL;
  if (!pos_dev && (pos < 0 || pos + seq_len > t_max)) return OHARA_EINVAL;
  if (pos_dev && seq_len != 1) return OHARA_EINVAL;
  if ((int64_t)batch * seq_len > INT32_MAX) return OHARA_ESIZE;
  GemmArgs a{};
  a.wp = reinterpret_cast<const uint4*>(wp);
  a.x = x; a.ldx = ldx; a.norm_w = ln_w; a.norm_b = ln_b; a.eps = eps;
  a.B = batch * seq_len; a.N = 3 * d + ff; a.K = d;
  a.out = q; a.ldo = ldq; a.out2 = act; a.ldo2 = ldact; a.split_n = 3 * d; a.bias = bias;
  a.S = seq_len; a.Tmax = t_max; a.pos = pos; a.pos_dev = pos_dev; a.kcache = kcache; a.vcache = vcache;
  if (a.B > 128 && !ln_w) return ohara_launch_gemm_tile(a, EPI_PHI_IN, (a.N + 15) / 16 * 16, (hipStream_t)stream);  // prefill
  return launch_skinny(a, EPI_PHI_IN, (a.N + 15) / 16 * 16, (hipStream_t)stream);
}

int ohara_gemm_skinny_bf16(const uint16_t* x, int ldx, const uint16_t* wp, int n, int k, const uint16_t* norm_w,
                           float eps, int batch, int epilogue, const uint16_t* resid, int ldr, uint16_t* out,
                           int ldo, void* stream) {
  if (!x || !wp || !out || n < 1 || k < 1 || batch < 1) return OHARA_EINVAL;
  if ((k & 7) || (ldx & 7) || ldx < k) return OHARA_EINVAL;  // 16-byte activation loads
  if (epilogue == OHARA_EPI_RESIDUAL && (!resid || ldr < n)) return OHARA_EINVAL;
  if (epilogue < OHARA_EPI_STORE || epilogue > OHARA_EPI_SWIGLU) return OHARA_EINVAL;
  if (ldo < n) return OHARA_EINVAL;
  GemmArgs a{};
  a.wp = reinterpret_cast<const uint4*>(wp);
  a.x = x; a.ldx = ldx; a.norm_w = norm_w; a.eps = eps;
  a.B = batch; a.N = n; a.K = k;
  a.out = out; a.ldo = ldo; a.resid = resid; a.ldr = ldr;
  int packed_rows;
  if (epilogue == OHARA_EPI_SWIGLU) packed_rows = 2 * ((n + 7) / 8 * 8);
  else packed_rows = (n + 15) / 16 * 16;
  if (batch > 64 && !norm_w) return ohara_launch_gemm_tile(a, epilogue, packed_rows, (hipStream_t)stream);
  return launch_skinny(a, epilogue, packed_rows, (hipStream_t)stream);
}

static int qkv_rope_impl(const uint16_t* x, int ldx, const uint16_t* wp, int k, const uint16_t* norm_w,
                         float eps, int batch, int seq_len, int h, int h_kv, int dh, const uint16_t* cos,
                         const uint16_t* sin, int pos, const int32_t* pos_dev, int pos_stride, uint16_t* q_out,
                         uint16_t* kcache, uint16_t* vcache, int t_max, int stage, void* stream) {
  if (!x || !wp || !cos || !sin || !q_out || !kcache || !vcache) return OHARA_EINVAL;
  if (batch < 1 || seq_len < 1 || h < 1 || h_kv < 1 || h % h_kv || dh < 4 || (dh & 3) || t_max < 1)
    return OHARA_EINVAL;
  if ((k & 7) || (ldx & 7) || ldx < k) return OHARA_EINVAL;
  if (!pos_dev && (pos < 0 || pos + seq_len > t_max)) return OHARA_EINVAL;
  if ((int64_t)batch * seq_len > INT32_MAX) return OHARA_ESIZE;
  GemmArgs a{};
  a.wp = reinterpret_cast<const uint4*>(wp);
  a.x = x; a.ldx = ldx; a.norm_w = norm_w; a.eps = eps;
  a.B = batch * seq_len; a.N = (h + 2 * h_kv) * dh; a.K = k;
  a.S = seq_len; a.row0 = 0;
  a.out = q_out; a.ldo = h * dh;
  a.H = h; a.Hkv = h_kv; a.Dh = dh; a.Tmax = t_max; a.pos = pos; a.pos_dev = pos_dev; a.pos_stride = pos_stride;
  a.cos = cos; a.sin = sin; a.kcache = kcache; a.vcache = vcache; a.stage = stage;
  if (a.B > 64 && !norm_w) return ohara_launch_gemm_tile(a, EPI_ROPE, (a.N + 15) / 16 * 16, (hipStream_t)stream);
  return launch_skinny(a, EPI_ROPE, (a.N + 15) / 16 * 16, (hipStream_t)stream);
}

int ohara_qkv_rope_append_bf16(const uint16_t* x, int ldx, const uint16_t* wp, int k, const uint16_t* norm_w,
                               float eps, int batch, int seq_len, int h, int h_kv, int dh, const uint16_t* cos,
                               const uint16_t* sin, int pos, const int32_t* pos_dev, uint16_t* q_out,
                               uint16_t* kcache, uint16_t* vcache, int t_max, void* stream) {
  return qkv_rope_impl(x, ldx, wp, k, norm_w, eps, batch, seq_len, h, h_kv, dh, cos, sin, pos, pos_dev, 0, q_out, kcache,
                       vcache, t_max, 0, stream);
}

int ohara_qkv_rope_append_ragged_bf16(const uint16_t* x, int ldx, const uint16_t* wp, int k, const uint16_t* norm_w,
                                      float eps, int batch, int seq_len, int h, int h_kv, int dh, const uint16_t* cos,
                                      const uint16_t* sin, const int32_t* seq_pos, uint16_t* q_out, uint16_t* kcache,
                                      uint16_t* vcache, int t_max, void* stream) {
  if (!seq_pos) return OHARA_EINVAL;
  return qkv_rope_impl(x, ldx, wp, k, norm_w, eps, batch, seq_len, h, h_kv, dh, cos, sin, 0, seq_pos, 1, q_out, kcache,
                       vcache, t_max, 0, stream);
}

int ohara_qkv_rope_bf16(const uint16_t* x, int ldx, const uint16_t* wp, int k, const uint16_t* norm_w, float eps,
                        int batch, int seq_len, int h, int h_kv, int dh, const uint16_t* cos, const uint16_t* sin,
                        int pos, const int32_t* pos_dev, int t_max, uint16_t* q_out, uint16_t* k_out, uint16_t* v_out,
                        void* stream) {
  return qkv_rope_impl(x, ldx, wp, k, norm_w, eps, batch, seq_len, h, h_kv, dh, cos, sin, pos, pos_dev, 0, q_out, k_out,
                       v_out, t_max, 1, stream);
}

int ohara_qkv_rope_ragged_bf16(const uint16_t* x, int ldx, const uint16_t* wp, int k, const uint16_t* norm_w, float eps,
                               int batch, int seq_len, int h, int h_kv, int dh, const uint16_t* cos, const uint16_t* sin,
                               const int32_t* seq_pos, int t_max, uint16_t* q_out, uint16_t* k_out, uint16_t* v_out,
                               void* stream) {
  if (!seq_pos) return OHARA_EINVAL;
  return qkv_rope_impl(x, ldx, wp, k, norm_w, eps, batch, seq_len, h, h_kv, dh, cos, sin, 0, seq_pos, 1, q_out, k_out,
                       v_out, t_max, 1, stream);
}

}  // extern "C"
