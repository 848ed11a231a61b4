// Persistent decode kernel of the BitNet-b1.58 Llama: one launch computes a whole decode step (one
// new token per sequence, batch <= 8) of the Llama of ohara/models/llama.py:279-323 whose seven
// per-layer projections are BitLinears (experiments/bitnet/bitnet.py:29-95).
//
// Same skeleton as the bf16 persistent kernel (one resident workgroup per CU, grid-wide barriers
// between phases, write-once mailboxes written with device-scope stores), with integer GEMM phases:
//   P1  [embedding] + norm1 + per-projection BitLinear norm / int8 codes + Q, K, V on
//       v_mfma_i32_16x16x64_i8 + rotary + cache append
//   P2  attention over the cache, split along the context (the bf16 kernel's phase as it is)
//   P3  merge of the partials + codes + attn.proj + residual
//   P4  norm2 + codes for ff.gate and ff.up + both products + SwiGLU
//   P5  codes + ff.down, K split over two groups of workgroups; the int32 partial sums are exact, so
//       whoever needs the residual stream next adds them, scales and rounds as one BitLinear would
// then final norm + vocabulary projection (bf16, the bf16 kernel's phase) and the arg-max.
// Every workgroup derives the codes of the rows it multiplies itself (a row is 2-11 KB; the three
// passes over it cost about as much as one hand-off), with the reduction orders of the stand-alone
// BitLinear kernels, so the integer accumulators are those kernels' accumulators.
#include <vector>

#include "persistent.h"

namespace {

#define OHARA_BIT_DOWN_SPLIT 2

struct BitLayerDev {  // one layer's device pointers and scales, as the kernel keeps them in LDS
  const uint4* w[7];      // packed ternary: query, key, value, proj, gate, up, down
  const bf16_t* nw[7];    // the BitLinears' own norm weights
  const bf16_t* norm1;
  const bf16_t* norm2;
  bf16_t* kc;
  bf16_t* vc;
  float gamma[7];
  float pad;
};
enum { BQ = 0, BK = 1, BV = 2, BO = 3, BG = 4, BU = 5, BD = 6 };

struct BitMegaArgs {
  OharaBitModel m;
  const BitLayerDev* layers_dev;
  int B, valid_vocab, hist_cap, select, ns, blk_x, blk_a;
  int64_t* ids;
  char* xm;        // NL x-mailboxes: the residual stream after each layer's attention block (bf16, strip-blocked)
  char* qm;        // NL q-mailboxes
  char* am;        // NL act-mailboxes
  float* pm;       // NL attention-partial mailboxes
  int32_t* dm;     // NL mailboxes of the down projection's int32 partial sums [part][strip][row][16]
  float* ds;       // NL x 16 floats: the activation scale s of every row of the down projection
  size_t xm_stride, qm_stride, am_stride, pm_stride, dm_stride;
  float* cand_val;
  int* cand_idx;
  bf16_t* logits;
  int32_t* step_state;
  int64_t* history;
  unsigned int* bar;
  unsigned long long* prof;
  unsigned int spin_limit;
};

// ---- the residual stream entering a layer ------------------------------------------------------
// x[b][n] = bf16(x_mid[b][n] + bf16((float(p0 + p1) / s_b) * gamma))   (llama.py:200 with a BitLinear
// ff.down, bitnet.py:58-59), or an embedding row, or x_mid as it is.
struct BitX {
  const char* xmid;
  int blk;
  const int32_t* parts;  // nullptr: x_mid is the stream
  const float* ds;       // scales of the rows that went into the down projection
  float gamma;
  const int64_t* ids;    // non-null: rows of the embedding table instead
  const bf16_t* table;
  int vocab;
  int B, N;
};

__device__ __forceinline__ const int32_t* iparts_addr(const int32_t* base, int nstrips, int B, int q, int b, int n) {
  return reinterpret_cast<const int32_t*>(reinterpret_cast<const char*>(base) +
                                          (size_t)(q * nstrips + (n >> 4)) * pm_blk(B) + b * 64) + (n & 15);
}

template <int NW>  // NW columns (4 or 8) starting at n, n % NW == 0 -> NW / 2 packed bf16 pairs
__device__ __forceinline__ void bitx_load(const BitX& x, int b, int n, uint32_t (&out)[NW / 2]) {
  if (x.ids) {
    int64_t id = ldg_i64(x.ids + b);
    if (id < 0 || id >= x.vocab) id = 0;
    const bf16_t* src = x.table + (size_t)id * x.N + n;
    if (NW == 8) {
      const uint4 v = ldg16(src);
      out[0] = v.x; out[1] = v.y; out[NW / 2 - 2] = v.z; out[NW / 2 - 1] = v.w;
    } else {
      const uint2 v = ldg8(src);
      out[0] = v.x; out[1] = v.y;
    }
    return;
  }
  uint32_t xm[NW / 2];
  if (NW == 8) {
    const uint4 v = ldg16(xm_addr(x.xmid, x.blk, b, n));
    xm[0] = v.x; xm[1] = v.y; xm[NW / 2 - 2] = v.z; xm[NW / 2 - 1] = v.w;
  } else {
    const uint2 v = ldg8(xm_addr(x.xmid, x.blk, b, n));
    xm[0] = v.x; xm[1] = v.y;
  }
  if (!x.parts) {
#pragma unroll
    for (int i = 0; i < NW / 2; ++i) out[i] = xm[i];
    return;
  }
  const int nstrips = (x.N + 15) >> 4;
  uint4 pv[OHARA_BIT_DOWN_SPLIT][NW / 4];
#pragma unroll
  for (int q = 0; q < OHARA_BIT_DOWN_SPLIT; ++q)
#pragma unroll
    for (int i = 0; i < NW / 4; ++i) pv[q][i] = ldg16(iparts_addr(x.parts, nstrips, x.B, q, b, n + 4 * i));
  const float s = __uint_as_float(ldg4(x.ds + b));
#pragma unroll
  for (int i = 0; i < NW / 4; ++i) {
    const int a[4] = {(int)pv[0][i].x + (int)pv[1][i].x, (int)pv[0][i].y + (int)pv[1][i].y,
                      (int)pv[0][i].z + (int)pv[1][i].z, (int)pv[0][i].w + (int)pv[1][i].w};
    float y[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) y[e] = rbf(__fmul_rn(__fdiv_rn((float)a[e], s), x.gamma));
    out[2 * i] = pack_bf(lo_bf(xm[2 * i]) + y[0], hi_bf(xm[2 * i]) + y[1]);
    out[2 * i + 1] = pack_bf(lo_bf(xm[2 * i + 1]) + y[2], hi_bf(xm[2 * i + 1]) + y[3]);
  }
}

__device__ __forceinline__ float bit_sumsq8(uint4 v) {
  float s = 0.f;
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float a = lo_bf(w[i]), b = hi_bf(w[i]);
    s += a * a + b * b;
  }
  return s;
}

// ---- a row in LDS -> its int8 codes ------------------------------------------------------------
// BitLinear's activation side (bitnet.py:29-33, 49-53) on a row of K bf16 values that already sits in
// LDS (`row`, overwritten): [block RMSNorm with pre_w,] the BitLinear's RMSNorm with nw, s = 127 /
// max|x_hat|, q = clamp(rint(x_hat * s), -128, 127).  The passes and the order of every reduction are
// those of the stand-alone kernels (csrc/bitlinear.hip), so the codes are the same codes.
struct RowQ {
  float s;
  int sumq;
};

// one wave on the row; lane l owns the 8-value pieces l, l + 64, ...
__device__ __forceinline__ RowQ wave_quant_lds(bf16_t* row, const bf16_t* pre_w, const bf16_t* nw, int K, float eps,
                                               int8_t* xq) {
  const int lane = threadIdx.x & 63;
  const int pieces = K >> 3;
  float ss = 0.f;
  for (int p = lane; p < pieces; p += 64) ss += bit_sumsq8(lds16(row + p * 8));
  if (pre_w) {
    ss = wave_sum(ss);
    const float rinv0 = 1.0f / sqrtf(ss / (float)K + eps);
    ss = 0.f;
    for (int p = lane; p < pieces; p += 64) {
      const uint4 u = lds16(row + p * 8);
      const uint4 w = ldg16(pre_w + (size_t)p * 8);
      const uint32_t uu[4] = {u.x, u.y, u.z, u.w}, ww[4] = {w.x, w.y, w.z, w.w};
      uint32_t o[4];
#pragma unroll
      for (int j = 0; j < 4; ++j)
        o[j] = pack_bf(rbf(lo_bf(uu[j]) * rinv0) * lo_bf(ww[j]), rbf(hi_bf(uu[j]) * rinv0) * hi_bf(ww[j]));
      const uint4 v = make_uint4(o[0], o[1], o[2], o[3]);
      sts16(row + p * 8, v);
      ss += bit_sumsq8(v);
    }
  }
  ss = wave_sum(ss);
  const float rinv = 1.0f / sqrtf(ss / (float)K + eps);
  float mx = 0.f;
  for (int p = lane; p < pieces; p += 64) {
    const uint4 u = lds16(row + p * 8);
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
    sts16(row + p * 8, make_uint4(o[0], o[1], o[2], o[3]));
  }
  mx = wave_max(mx);
  const float s = 127.0f / fmaxf(mx, 1e-5f);
  int sq = 0;
  for (int p = lane; p < pieces; p += 64) {
    const uint4 u = lds16(row + p * 8);
    const uint32_t uu[4] = {u.x, u.y, u.z, u.w};
    uint32_t pk[2] = {0u, 0u};
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float v = (j & 1) ? hi_bf(uu[j >> 1]) : lo_bf(uu[j >> 1]);
      const int qi = (int)fminf(fmaxf(rintf(v * s), -128.f), 127.f);
      sq += qi;
      pk[j >> 2] |= ((uint32_t)qi & 0xffu) << (8 * (j & 3));
    }
    sts8(xq + (size_t)p * 8, make_uint2(pk[0], pk[1]));
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) sq += __shfl_xor(sq, o, WAVE);
  return RowQ{s, sq};
}

// the whole workgroup on one row (batch 1): thread t owns the pieces t, t + 256, ...; every thread calls
__device__ __forceinline__ RowQ block_quant_lds(bf16_t* row, const bf16_t* pre_w, const bf16_t* nw, int K, float eps,
                                                int8_t* xq, float* red) {
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
  for (int p = tid; p < pieces; p += 256) ss += bit_sumsq8(lds16(row + p * 8));
  if (pre_w) {
    const float rinv0 = 1.0f / sqrtf(bsum(ss) / (float)K + eps);
    ss = 0.f;
    for (int p = tid; p < pieces; p += 256) {
      const uint4 u = lds16(row + p * 8);
      const uint4 w = ldg16(pre_w + (size_t)p * 8);
      const uint32_t uu[4] = {u.x, u.y, u.z, u.w}, ww[4] = {w.x, w.y, w.z, w.w};
      uint32_t o[4];
#pragma unroll
      for (int j = 0; j < 4; ++j)
        o[j] = pack_bf(rbf(lo_bf(uu[j]) * rinv0) * lo_bf(ww[j]), rbf(hi_bf(uu[j]) * rinv0) * hi_bf(ww[j]));
      const uint4 v = make_uint4(o[0], o[1], o[2], o[3]);
      sts16(row + p * 8, v);
      ss += bit_sumsq8(v);
    }
  }
  const float rinv = 1.0f / sqrtf(bsum(ss) / (float)K + eps);
  float mx = 0.f;
  for (int p = tid; p < pieces; p += 256) {
    const uint4 u = lds16(row + p * 8);
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
    sts16(row + p * 8, make_uint4(o[0], o[1], o[2], o[3]));
  }
  mx = wave_max(mx);
  __syncthreads();
  if (lane == 0) red[wave] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  const float s = 127.0f / fmaxf(mx, 1e-5f);
  int sq = 0;
  for (int p = tid; p < pieces; p += 256) {
    const uint4 u = lds16(row + p * 8);
    const uint32_t uu[4] = {u.x, u.y, u.z, u.w};
    uint32_t pk[2] = {0u, 0u};
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float v = (j & 1) ? hi_bf(uu[j >> 1]) : lo_bf(uu[j >> 1]);
      const int qi = (int)fminf(fmaxf(rintf(v * s), -128.f), 127.f);
      sq += qi;
      pk[j >> 2] |= ((uint32_t)qi & 0xffu) << (8 * (j & 3));
    }
    sts8(xq + (size_t)p * 8, make_uint2(pk[0], pk[1]));
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) sq += __shfl_xor(sq, o, WAVE);
  int* redi = reinterpret_cast<int*>(red);
  __syncthreads();
  if (lane == 0) redi[wave] = sq;
  __syncthreads();
  return RowQ{s, redi[0] + redi[1] + redi[2] + redi[3]};
}

// LDS of the kernel.  `codes`: up to two code sets (gate and up) of B rows x ldq bytes; `stage`: bf16
// rows being turned into codes - B rows of the model width (attention output, all rows at once) or
// four rows of the largest K (one per wave); row stride ldst elements.
struct BitLds {
  int8_t* codes;
  int ldq;          // bytes per code row of the current phase (K padded to 256, + 16 against bank conflicts)
  size_t set;       // bytes between the two code sets of the current phase
  bf16_t* stage;
  int ldst;         // elements between the rows being quantised (one per wave)
  int ldm;          // elements between the rows of the merged attention output
  __device__ __forceinline__ void shape(int B, int K) {
    ldq = (((K + 255) >> 8) << 8) + 16;
    set = (size_t)B * ldq;
  }
  float* s_s;       // [2][16] activation scales
  int* s_sum;       // [2][16] sums of the codes
  float* red;       // 4 KiB: cross-wave sums
};

// Rows from `load(b, piece) -> uint4` into codes of set `set` (every thread of the workgroup calls).
// pre_w: block norm weight or null.  The tail of every code row up to the padded K reads as zero.
template <typename Load>
__device__ __forceinline__ void bit_stage_codes(const BitLds& L, int set, int B, int K, const bf16_t* pre_w,
                                                const bf16_t* nw, float eps, Load load) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int pieces = K >> 3;
  int8_t* xq = L.codes + (size_t)set * L.set;
  __syncthreads();  // whoever still reads the previous codes, scales or staged rows is done
  // zero the padding columns [K, ldq) of the rows in use (K is a multiple of 8, ldq of 16)
  {
    const int pad8 = (L.ldq - K) >> 3;
    for (int i = tid; i < B * pad8; i += 256) {
      const int b = i / pad8, c = i - b * pad8;
      sts8(xq + (size_t)b * L.ldq + K + c * 8, make_uint2(0, 0));
    }
  }
  if (B == 1) {
    for (int p = tid; p < pieces; p += 256) sts16(L.stage + p * 8, load(0, p));
    __syncthreads();
    const RowQ o = block_quant_lds(L.stage, pre_w, nw, K, eps, xq, L.red);
    if (tid == 0) {
      L.s_s[set * 16] = o.s;
      L.s_sum[set * 16] = o.sumq;
    }
  } else {
    bf16_t* row = L.stage + (size_t)wave * L.ldst;
    for (int b = wave; b < B; b += 4) {
      for (int p = lane; p < pieces; p += 64) sts16(row + p * 8, load(b, p));
      const RowQ o = wave_quant_lds(row, pre_w, nw, K, eps, xq + (size_t)b * L.ldq);
      if (lane == 0) {
        L.s_s[set * 16 + b] = o.s;
        L.s_sum[set * 16 + b] = o.sumq;
      }
    }
  }
  __syncthreads();
}

// The same when the rows already sit in `stage` (row b at b * ldst): the merged attention output.
__device__ __forceinline__ void bit_codes_from_stage(const BitLds& L, int set, int B, int K, const bf16_t* nw, float eps) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int8_t* xq = L.codes + (size_t)set * L.set;
  __syncthreads();  // the merged rows are complete; the previous codes and scales are no longer read
  {
    const int pad8 = (L.ldq - K) >> 3;
    for (int i = tid; i < B * pad8; i += 256) {
      const int b = i / pad8, c = i - b * pad8;
      sts8(xq + (size_t)b * L.ldq + K + c * 8, make_uint2(0, 0));
    }
  }
  if (B == 1) {
    const RowQ o = block_quant_lds(L.stage, nullptr, nw, K, eps, xq, L.red);
    if (tid == 0) {
      L.s_s[set * 16] = o.s;
      L.s_sum[set * 16] = o.sumq;
    }
  } else {
    for (int b = wave; b < B; b += 4) {
      const RowQ o = wave_quant_lds(L.stage + (size_t)b * L.ldm, nullptr, nw, K, eps, xq + (size_t)b * L.ldq);
      if (lane == 0) {
        L.s_s[set * 16 + b] = o.s;
        L.s_sum[set * 16 + b] = o.sumq;
      }
    }
  }
  __syncthreads();
}

// ---- one strip of a ternary weight x the code rows ---------------------------------------------
// Chunks [cb, ce) of 256 columns, split over the four waves; the sum over the waves lands in wave 0
// (returns true there).  `wpre`: the first BIT_PF chunks of this wave, fetched ahead.  Rows beyond B
// read row B - 1 (their results are never looked at).  Every thread of the workgroup calls.
#define BIT_PF 6
struct BitPre {
  uint4 w[BIT_PF];
};
__device__ __forceinline__ void bit_wave_chunks(int cb, int ce, int& c0, int& c1) {
  const int wave = threadIdx.x >> 6;
  const int per = (ce - cb + 3) >> 2;
  c0 = cb + wave * per;
  c1 = min(ce, c0 + per);
}
__device__ __forceinline__ void bit_prefetch(const uint4* wp, int KC, int strip, int cb, int ce, bool live, BitPre& pre) {
  int c0, c1;
  bit_wave_chunks(cb, ce, c0, c1);
  const uint4* wrow = wp + (size_t)strip * KC * 64 + (threadIdx.x & 63);
#pragma unroll
  for (int c = 0; c < BIT_PF; ++c)
    pre.w[c] = (live && c0 + c < c1) ? ldg16_nt(wrow + (size_t)(c0 + c) * 64) : make_uint4(0, 0, 0, 0);
}
__device__ __forceinline__ bool bit_strip(const uint4* wp, int KC, int strip, int cb, int ce, bool live,
                                          const BitPre* pre, const int8_t* xq, int ldq, int B, int* red, i32x4& acc) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int m = lane & 15, g = lane >> 4;
  int c0, c1;
  bit_wave_chunks(cb, ce, c0, c1);
  const uint4* wrow = wp + (size_t)strip * KC * 64 + lane;
  const int8_t* xrow = xq + (size_t)min(m, B - 1) * ldq + 16 * g;
  acc = (i32x4){0, 0, 0, 0};
  if (live) {
    for (int cbk = c0; cbk < c1; cbk += BIT_PF) {
      uint4 wv[BIT_PF];
      if (pre && cbk == c0) {
#pragma unroll
        for (int c = 0; c < BIT_PF; ++c) wv[c] = pre->w[c];
      } else {
#pragma unroll
        for (int c = 0; c < BIT_PF; ++c)
          wv[c] = (cbk + c < c1) ? ldg16_nt(wrow + (size_t)(cbk + c) * 64) : make_uint4(0, 0, 0, 0);
      }
#pragma unroll
      for (int c = 0; c < BIT_PF; ++c) {
        if (cbk + c >= c1) continue;
        const uint32_t dw[4] = {wv[c].x, wv[c].y, wv[c].z, wv[c].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          i32x4 av;
          av[0] = (int)(dw[j] & 0x03030303u);
          av[1] = (int)((dw[j] >> 2) & 0x03030303u);
          av[2] = (int)((dw[j] >> 4) & 0x03030303u);
          av[3] = (int)((dw[j] >> 6) & 0x03030303u);
          const uint4 xv = lds16(xrow + ((cbk + c) << 8) + 64 * j);
          i32x4 bv;
          bv[0] = (int)xv.x; bv[1] = (int)xv.y; bv[2] = (int)xv.z; bv[3] = (int)xv.w;
          acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, bv, acc, 0, 0, 0);
        }
      }
    }
  }
  if (wave > 0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) red[((wave - 1) * 64 + lane) * 4 + i] = acc[i];
  }
  __syncthreads();
  if (wave == 0) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      acc[i] += red[(0 * 64 + lane) * 4 + i] + red[(1 * 64 + lane) * 4 + i] + red[(2 * 64 + lane) * 4 + i];
  }
  __syncthreads();  // red is free again
  return wave == 0;
}

// y = bf16((float(acc - sum q) / s) * gamma)   (bitnet.py:58-59; the packed codes are T + 1)
__device__ __forceinline__ void bit_scale(const i32x4& acc, int sq, float s, float gamma, float* y) {
#pragma unroll
  for (int i = 0; i < 4; ++i) y[i] = rbf(__fmul_rn(__fdiv_rn((float)(acc[i] - sq), s), gamma));
}

// final RMSNorm of the stream into bf16 rows in LDS (norm.py:16-21), one wave per row
template <int NLD>
__device__ void bit_stage_final_norm(bf16_t* xs, int ldxs, const BitX& x, const bf16_t* nw, float eps, int B, int K) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int b = wave; b < B; b += 4) {
    uint4 v[NLD], g[NLD];
#pragma unroll
    for (int c = 0; c < NLD; ++c) {
      const int k = (c * 64 + lane) * 8;
      v[c] = make_uint4(0, 0, 0, 0);
      g[c] = make_uint4(0, 0, 0, 0);
      if (k < K) {
        uint32_t w[4];
        bitx_load<8>(x, b, k, w);
        v[c] = make_uint4(w[0], w[1], w[2], w[3]);
        g[c] = ldg16(nw + k);
      }
    }
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < NLD; ++c) ss += bit_sumsq8(v[c]);
    ss = wave_sum(ss);
    const float rinv = 1.0f / sqrtf(ss / (float)K + eps);
#pragma unroll
    for (int c = 0; c < NLD; ++c) {
      const int k = (c * 64 + lane) * 8;
      if (k < K) {
        const uint32_t xv[4] = {v[c].x, v[c].y, v[c].z, v[c].w};
        const uint32_t gv[4] = {g[c].x, g[c].y, g[c].z, g[c].w};
        uint32_t o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
          o[i] = pack_bf(rbf(lo_bf(xv[i]) * rinv) * lo_bf(gv[i]), rbf(hi_bf(xv[i]) * rinv) * hi_bf(gv[i]));
        sts16(xs + (size_t)b * ldxs + k, make_uint4(o[0], o[1], o[2], o[3]));
      }
    }
  }
}

// ---------------------------------------------------------------------------------------
// the kernel
// ---------------------------------------------------------------------------------------
template <int D, int G>
__global__ __launch_bounds__(256) void bitnet_mega_kernel(BitMegaArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const OharaBitModel& m = a.m;
  const int d = m.d_model, H = m.n_heads, Hkv = m.n_kv_heads, F = m.d_ff, V = m.vocab, B = a.B;
  const int nwg = gridDim.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int mm = lane & 15, gg = lane >> 4;
  const int HD = H * D;
  const int kmax = max(max(d, HD), F);
  const int Kp = ((kmax + 255) >> 8) << 8;
  // ---- LDS carve-up (the host computes the same sizes) ----
  BitLds L;
  const int dmax = max(d, HD);
  const int Kpd1 = ((d + 255) >> 8) << 8;
  const size_t codes_bytes = max((size_t)B * (Kp + 16), (size_t)2 * B * (Kpd1 + 16));
  L.codes = reinterpret_cast<int8_t*>(smem);
  L.shape(B, d);
  size_t off = (codes_bytes + 255) & ~(size_t)255;
  const size_t stage_bytes = max((size_t)(B == 1 ? 1 : 4) * Kp * 2, (size_t)B * (dmax + 8) * 2);
  L.stage = reinterpret_cast<bf16_t*>(smem + off);
  L.ldst = Kp;
  L.ldm = dmax + 8;
  off += (stage_bytes + 255) & ~(size_t)255;
  L.red = reinterpret_cast<float*>(smem + off); off += 4096;
  L.s_s = reinterpret_cast<float*>(smem + off); off += 128;
  L.s_sum = reinterpret_cast<int*>(smem + off); off += 128;
  float* att = reinterpret_cast<float*>(smem + off); off += (size_t)(8 + 4 * D) * G * sizeof(float);
  float* mrg_w = reinterpret_cast<float*>(smem + off); off += (size_t)((B * H * a.ns + 1) & ~1) * sizeof(float);
  float* mrg_l = reinterpret_cast<float*>(smem + off); off += (size_t)((B * H * a.ns + 1) & ~1) * sizeof(float);
  off = (off + 15) & ~(size_t)15;
  BitLayerDev* ltab = reinterpret_cast<BitLayerDev*>(smem + off);
  // the layer table -> LDS, so that no phase starts with a chain of dependent global loads
  {
    const uint32_t* src = reinterpret_cast<const uint32_t*>(a.layers_dev);
    uint32_t* dst = reinterpret_cast<uint32_t*>(ltab);
    const int n = m.n_layers * (int)(sizeof(BitLayerDev) / 4);
    for (int i = tid; i < n; i += 256) dst[i] = src[i];
  }
  __syncthreads();
  auto gptr = [&](const void* p) {  // a pointer read from LDS, made wave-uniform and global
    const unsigned long long v = reinterpret_cast<unsigned long long>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return ((unsigned long long)hi << 32) | lo;
  };

  GridSync gs;
  gs.init(a.bar, nwg, a.spin_limit);
  const int pos = a.step_state[0];
  const int step = a.step_state[1];
  const int Lc = min(pos + 1, m.t_max);
  float best_v = -INFINITY;
  int best_i = 0x7fffffff;
  Prof pf{(blockIdx.x == 0 && tid == 0) ? a.prof : nullptr, 0};

  const int KCd = (d + 255) >> 8, KCo = (HD + 255) >> 8, KCf = (F + 255) >> 8;
  const int ns_q = HD / 16, ns_kv = (Hkv * D) / 16, ns_d = (d + 15) / 16, ns_f = (F + 15) / 16;
  const bool ok_pos = pos >= 0 && pos < m.t_max;

  GemmP lm{};
  lm.N = V; lm.K = d; lm.nstrips = (V + 15) / 16; lm.out = reinterpret_cast<char*>(a.logits); lm.ldo = V;
  lm.valid = a.valid_vocab > 0 ? min(a.valid_vocab, V) : V;
  lm.wp = reinterpret_cast<const uint4*>(m.w_vocab);
  GemmPre lpre;
  AttnPre<D> apre;
  BitPre wpre;

  for (int l = 0; l < m.n_layers; ++l) {
    const BitLayerDev& LY = ltab[l];
    bf16_t* kc = reinterpret_cast<bf16_t*>(gptr(LY.kc));
    bf16_t* vc = reinterpret_cast<bf16_t*>(gptr(LY.vc));
    char* x_mid = a.xm + (size_t)l * a.xm_stride;
    char* q_l = a.qm + (size_t)l * a.qm_stride;
    char* a_l = a.am + (size_t)l * a.am_stride;
    float* p_l = a.pm + (size_t)l * a.pm_stride;
    int32_t* d_l = a.dm + (size_t)l * a.dm_stride;
    // the stream entering this layer
    BitX xin{};
    xin.B = B; xin.N = d; xin.blk = a.blk_x;
    if (l == 0) {
      xin.ids = a.ids; xin.table = m.token_emb; xin.vocab = V;
    } else {
      xin.xmid = a.xm + (size_t)(l - 1) * a.xm_stride;
      xin.parts = a.dm + (size_t)(l - 1) * a.dm_stride;
      xin.ds = a.ds + (size_t)(l - 1) * 16;
      xin.gamma = ltab[l - 1].gamma[BD];
    }
    const bf16_t* norm1 = reinterpret_cast<const bf16_t*>(gptr(LY.norm1));
    const bf16_t* norm2 = reinterpret_cast<const bf16_t*>(gptr(LY.norm2));

    // ---- P1: Q, K, V.  Units [0, ns_q) query strips, then key strips, then value strips. ----
    {
      const int nunits = ns_q + 2 * ns_kv;
      L.shape(B, d);
      int have = -1;  // projection whose codes are staged
      for (int unit = blockIdx.x; unit < nunits; unit += nwg) {
        const int which = unit < ns_q ? BQ : (unit < ns_q + ns_kv ? BK : BV);
        const int strip = unit - (which == BQ ? 0 : (which == BK ? ns_q : ns_q + ns_kv));
        const uint4* wp = reinterpret_cast<const uint4*>(gptr(LY.w[which]));
        bit_prefetch(wp, KCd, strip, 0, KCd, true, wpre);
        if (have != which) {
          const bf16_t* nw = reinterpret_cast<const bf16_t*>(gptr(LY.nw[which]));
          bit_stage_codes(L, 0, B, d, norm1, nw, m.eps, [&](int b, int p) {
            uint32_t w[4];
            bitx_load<8>(xin, b, p * 8, w);
            return make_uint4(w[0], w[1], w[2], w[3]);
          });
          have = which;
        }
        i32x4 acc;
        if (bit_strip(wp, KCd, strip, 0, KCd, true, &wpre, L.codes, L.ldq, B, reinterpret_cast<int*>(L.red), acc) &&
            mm < B && ok_pos) {
          const int b = mm;
          const int r0 = strip * 16 + 4 * gg;
          float v[4];
          bit_scale(acc, L.s_sum[b], L.s_s[b], LY.gamma[which], v);
          char* o;
          if (which != BV) {
            const int dd = r0 % D;
            const uint32_t cs = ldg4(m.cos + (size_t)pos * (D >> 1) + (dd >> 1));
            const uint32_t sn = ldg4(m.sin + (size_t)pos * (D >> 1) + (dd >> 1));
            const float c2[2] = {lo_bf(cs), hi_bf(cs)}, s2[2] = {lo_bf(sn), hi_bf(sn)};
#pragma unroll
            for (int pr = 0; pr < 2; ++pr) {
              const float e = v[2 * pr], od = v[2 * pr + 1];
              v[2 * pr] = __fsub_rn(__fmul_rn(e, c2[pr]), __fmul_rn(od, s2[pr]));
              v[2 * pr + 1] = __fadd_rn(__fmul_rn(e, s2[pr]), __fmul_rn(od, c2[pr]));
            }
            o = which == BQ ? const_cast<char*>(xm_addr(q_l, a.blk_x, b, r0))
                            : reinterpret_cast<char*>(kc + (((size_t)b * m.t_max + pos) * Hkv) * D + r0);
          } else {
            o = reinterpret_cast<char*>(vc + (((size_t)b * m.t_max + pos) * Hkv) * D + r0);
          }
          st_coh8(o, make_uint2(pack_bf(v[0], v[1]), pack_bf(v[2], v[3])));
        }
      }
    }
    gs.arrive(pf);
    attn_prefetch<D>(B, Hkv, m.t_max, a.ns, kc, vc, Lc, apre);
    gs.wait(pf);
    // ---- P2: attention partials ----
    attn_phase<D, G>(B, H, Hkv, m.t_max, a.blk_x, a.ns, apre, q_l, p_l, kc, vc, Lc, att);
    gs.arrive(pf);
    const uint4* wo = reinterpret_cast<const uint4*>(gptr(LY.w[BO]));
    bit_prefetch(wo, KCo, blockIdx.x, 0, KCo, (int)blockIdx.x < ns_d, wpre);
    gs.wait(pf);
    // ---- P3: merge + attn.proj + residual ----
    L.shape(B, HD);
    for (int strip = blockIdx.x; strip < ns_d; strip += nwg) {
      const bool first = strip == (int)blockIdx.x;
      if (first) {
        bf16_t* xs = L.stage;
        const int ldxs = L.ldm;
        if (a.ns == OHARA_MEGA_NS && B * HD <= 4 * 256) stage_attn_merge_small(xs, ldxs, p_l, B, H, D);
        else if (a.ns == 16) stage_attn_merge<16>(xs, ldxs, p_l, B, H, D, mrg_w, mrg_l);
        else if (a.ns == 8) stage_attn_merge<8>(xs, ldxs, p_l, B, H, D, mrg_w, mrg_l);
        else if (a.ns == 4) stage_attn_merge<4>(xs, ldxs, p_l, B, H, D, mrg_w, mrg_l);
        else if (a.ns == 2) stage_attn_merge<2>(xs, ldxs, p_l, B, H, D, mrg_w, mrg_l);
        else stage_attn_merge<1>(xs, ldxs, p_l, B, H, D, mrg_w, mrg_l);
        __syncthreads();
        bit_codes_from_stage(L, 0, B, HD, reinterpret_cast<const bf16_t*>(gptr(LY.nw[BO])), m.eps);
      }
      i32x4 acc;
      if (bit_strip(wo, KCo, strip, 0, KCo, true, first ? &wpre : nullptr, L.codes, L.ldq, B,
                    reinterpret_cast<int*>(L.red), acc) && mm < B) {
        const int b = mm;
        const int r0 = strip * 16 + 4 * gg;
        if (r0 < d) {
          float y[4];
          bit_scale(acc, L.s_sum[b], L.s_s[b], LY.gamma[BO], y);
          uint32_t r[2];
          bitx_load<4>(xin, b, r0, r);
          st_coh8(const_cast<char*>(xm_addr(x_mid, a.blk_x, b, r0)),
                  make_uint2(pack_bf(lo_bf(r[0]) + y[0], hi_bf(r[0]) + y[1]), pack_bf(lo_bf(r[1]) + y[2], hi_bf(r[1]) + y[3])));
        }
      }
    }
    gs.arrive(pf);
    const uint4* wg = reinterpret_cast<const uint4*>(gptr(LY.w[BG]));
    const uint4* wu = reinterpret_cast<const uint4*>(gptr(LY.w[BU]));
    bit_prefetch(wg, KCd, blockIdx.x, 0, KCd, (int)blockIdx.x < ns_f, wpre);
    gs.wait(pf);
    // ---- P4: norm2 + ff.gate, ff.up + SwiGLU ----
    L.shape(B, d);
    if ((int)blockIdx.x < ns_f) {
      BitX xmid{};
      xmid.B = B; xmid.N = d; xmid.blk = a.blk_x; xmid.xmid = x_mid;
      auto load_mid = [&](int b, int p) {
        uint32_t w[4];
        bitx_load<8>(xmid, b, p * 8, w);
        return make_uint4(w[0], w[1], w[2], w[3]);
      };
      bit_stage_codes(L, 0, B, d, norm2, reinterpret_cast<const bf16_t*>(gptr(LY.nw[BG])), m.eps, load_mid);
      bit_stage_codes(L, 1, B, d, norm2, reinterpret_cast<const bf16_t*>(gptr(LY.nw[BU])), m.eps, load_mid);
      for (int strip = blockIdx.x; strip < ns_f; strip += nwg) {
        const bool first = strip == (int)blockIdx.x;
        i32x4 ag, au;
        const bool w0g = bit_strip(wg, KCd, strip, 0, KCd, true, first ? &wpre : nullptr, L.codes, L.ldq, B,
                                   reinterpret_cast<int*>(L.red), ag);
        const bool w0u = bit_strip(wu, KCd, strip, 0, KCd, true, nullptr, L.codes + L.set, L.ldq, B,
                                   reinterpret_cast<int*>(L.red), au);
        if (w0g && w0u && mm < B) {
          const int b = mm;
          const int f0 = strip * 16 + 4 * gg;
          if (f0 < F) {
            float yg[4], yu[4];
            bit_scale(ag, L.s_sum[b], L.s_s[b], LY.gamma[BG], yg);
            bit_scale(au, L.s_sum[16 + b], L.s_s[16 + b], LY.gamma[BU], yu);
            const uint32_t lo = pack_bf(rbf(silu_f(yg[0])) * yu[0], rbf(silu_f(yg[1])) * yu[1]);
            const uint32_t hi = pack_bf(rbf(silu_f(yg[2])) * yu[2], rbf(silu_f(yg[3])) * yu[3]);
            st_coh8(const_cast<char*>(am_addr(a_l, a.blk_a, b, f0)), make_uint2(lo, hi));
          }
        }
      }
    }
    gs.arrive(pf);
    const uint4* wd = reinterpret_cast<const uint4*>(gptr(LY.w[BD]));
    const int per_part = (KCf + OHARA_BIT_DOWN_SPLIT - 1) / OHARA_BIT_DOWN_SPLIT;
    {
      const int unit = blockIdx.x, part = unit / ns_d, strip = unit - part * ns_d;
      bit_prefetch(wd, KCf, strip, part * per_part, min(KCf, (part + 1) * per_part), unit < ns_d * OHARA_BIT_DOWN_SPLIT, wpre);
    }
    gs.wait(pf);
    // ---- P5: ff.down, K split over OHARA_BIT_DOWN_SPLIT groups of workgroups ----
    {
      const int nunits = ns_d * OHARA_BIT_DOWN_SPLIT;
      L.shape(B, F);
      bool staged = false;
      for (int unit = blockIdx.x; unit < nunits; unit += nwg) {
        const bool first = unit == (int)blockIdx.x;
        const int part = unit / ns_d, strip = unit - part * ns_d;
        if (!staged) {
          bit_stage_codes(L, 0, B, F, nullptr, reinterpret_cast<const bf16_t*>(gptr(LY.nw[BD])), m.eps, [&](int b, int p) {
            return ldg16(am_addr(a_l, a.blk_a, b, p * 8));
          });
          staged = true;
        }
        i32x4 acc;
        if (bit_strip(wd, KCf, strip, part * per_part, min(KCf, (part + 1) * per_part), true, first ? &wpre : nullptr,
                      L.codes, L.ldq, B, reinterpret_cast<int*>(L.red), acc) && mm < B) {
          const int b = mm;
          const int r0 = strip * 16 + 4 * gg;
          if (r0 < d) {
            const int sq = part == 0 ? L.s_sum[b] : 0;  // the codes are T + 1: the first part takes the correction
            int32_t* o = const_cast<int32_t*>(iparts_addr(d_l, ns_d, B, part, b, r0));
            st_coh8(o, make_uint2((uint32_t)(acc[0] - sq), (uint32_t)(acc[1] - sq)));
            st_coh8(o + 2, make_uint2((uint32_t)(acc[2] - sq), (uint32_t)(acc[3] - sq)));
          }
          if (unit == 0 && gg == 0) st_coh4(a.ds + (size_t)l * 16 + b, __float_as_uint(L.s_s[b]));
        }
      }
    }
    gs.arrive(pf);
    if (l + 1 == m.n_layers) gemm_prefetch<1, 24, E_LOGITS>(lm, lpre, B);
    gs.wait(pf);
  }
  // ---- final norm + vocabulary projection (bf16), running arg-max per lane ----
  {
    BitX xf{};
    xf.B = B; xf.N = d; xf.blk = a.blk_x;
    xf.xmid = a.xm + (size_t)(m.n_layers - 1) * a.xm_stride;
    xf.parts = a.dm + (size_t)(m.n_layers - 1) * a.dm_stride;
    xf.ds = a.ds + (size_t)(m.n_layers - 1) * 16;
    xf.gamma = ltab[m.n_layers - 1].gamma[BD];
    bf16_t* xs = L.stage;
    const int ldxs = d + 8;
    bit_stage_final_norm<8>(xs, ldxs, xf, m.final_norm, m.eps, B, d);
    __syncthreads();
    gemm_phase<1, 24, E_LOGITS>(lm, lpre, xs, ldxs, B, L.red, best_v, best_i, pf);
  }
  if (a.select) {
#pragma unroll
    for (int o = 16; o < 64; o <<= 1) {
      const float ov = __shfl_xor(best_v, o, WAVE);
      const int oi = __shfl_xor(best_i, o, WAVE);
      if (ov > best_v || (ov == best_v && oi < best_i)) {
        best_v = ov;
        best_i = oi;
      }
    }
    __syncthreads();
    float* cv = L.red;
    int* ci = reinterpret_cast<int*>(L.red + 64);
    if (lane < 16) {
      cv[wave * 16 + lane] = best_v;
      ci[wave * 16 + lane] = best_i;
    }
    __syncthreads();
    if (tid < B) {
      float bv = cv[tid];
      int bi = ci[tid];
      for (int w = 1; w < 4; ++w) {
        const float ov = cv[w * 16 + tid];
        const int oi = ci[w * 16 + tid];
        if (ov > bv || (ov == bv && oi < bi)) {
          bv = ov;
          bi = oi;
        }
      }
      st_coh4(a.cand_val + (size_t)blockIdx.x * B + tid, __float_as_uint(bv));
      st_coh4(a.cand_idx + (size_t)blockIdx.x * B + tid, (uint32_t)bi);
    }
    gs.arrive(pf);
    gs.wait(pf);
    if (blockIdx.x == 0) {
      for (int b = wave; b < B; b += 4) {
        float bv = -INFINITY;
        int bi = 0x7fffffff;
        for (int w = lane; w < nwg; w += 64) {
          const float ov = __uint_as_float(ld_coh4(a.cand_val + (size_t)w * B + b));
          const int oi = (int)ld_coh4(a.cand_idx + (size_t)w * B + b);
          if (ov > bv || (ov == bv && oi < bi)) {
            bv = ov;
            bi = oi;
          }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
          const float ov = __shfl_xor(bv, o, WAVE);
          const int oi = __shfl_xor(bi, o, WAVE);
          if (ov > bv || (ov == bv && oi < bi)) {
            bv = ov;
            bi = oi;
          }
        }
        if (lane == 0) {
          if (bi == 0x7fffffff) bi = 0;
          a.ids[b] = bi;
          if (a.history && step < a.hist_cap) a.history[(size_t)step * B + b] = bi;
        }
      }
    }
  }
  if (blockIdx.x == 0 && tid == 0) {
    *gs.done = gs.k - 1;
    if (a.select) {
      a.step_state[0] = pos + 1;
      a.step_state[1] = step + 1;
    }
  }
}

// ---- workspace layout ------------------------------------------------------------------
#define OHARA_BIT_BAR_WORDS(nwg) ((((nwg) + OHARA_BAR_GROUP - 1) / OHARA_BAR_GROUP + 4) * 64)

size_t bit_al(size_t v) { return (v + 255) & ~(size_t)255; }

struct BitLayout {
  size_t layers, xm, qm, am, pm, dm, ds, candv, candi, prof, bar, total;
  size_t xm_stride, qm_stride, am_stride, pm_stride, dm_stride;
  int blk_x, blk_a;
};

BitLayout bit_layout(const OharaBitModel* m, int B, int nwg) {
  BitLayout L{};
  const int NL = m->n_layers, D = m->head_dim;
  L.blk_x = (B * 32 + 127) / 128 * 128;
  L.blk_a = (B * 16 + 127) / 128 * 128;
  const int hd = m->n_heads * D;
  L.xm_stride = bit_al((size_t)((m->d_model + 15) / 16) * L.blk_x);
  L.qm_stride = bit_al((size_t)((hd + 15) / 16) * L.blk_x);
  L.am_stride = bit_al((size_t)((m->d_ff + 7) / 8) * L.blk_a);
  L.pm_stride = bit_al((size_t)B * m->n_heads * OHARA_MEGA_NS * (D + 32) * sizeof(float)) / sizeof(float);
  L.dm_stride = bit_al((size_t)OHARA_BIT_DOWN_SPLIT * ((m->d_model + 15) / 16) * ((B * 64 + 127) / 128 * 128)) / sizeof(int32_t);
  size_t o = 0;
  L.layers = o; o += bit_al(sizeof(BitLayerDev) * NL);
  L.xm = o; o += L.xm_stride * NL;
  L.qm = o; o += L.qm_stride * NL;
  L.am = o; o += L.am_stride * NL;
  L.pm = o; o += L.pm_stride * sizeof(float) * NL;
  L.dm = o; o += L.dm_stride * sizeof(int32_t) * NL;
  L.ds = o; o += bit_al((size_t)NL * 16 * sizeof(float));
  L.candv = o; o += bit_al((size_t)nwg * B * sizeof(float));
  L.candi = o; o += bit_al((size_t)nwg * B * sizeof(int));
  L.prof = o; o += bit_al(1024 * sizeof(unsigned long long));
  L.bar = o; o += bit_al(OHARA_BIT_BAR_WORDS(nwg) * sizeof(unsigned int));
  L.total = o;
  return L;
}

size_t bit_smem_bytes(const OharaBitModel* m, int B, int ns) {
  const int D = m->head_dim, G = m->n_heads / m->n_kv_heads, HD = m->n_heads * D;
  const int dmax = m->d_model > HD ? m->d_model : HD;
  const int kmax = dmax > m->d_ff ? dmax : m->d_ff;
  const int Kp = ((kmax + 255) >> 8) << 8, Kpd = ((dmax + 255) >> 8) << 8;
  size_t codes = (size_t)B * (Kp + 16);
  if ((size_t)2 * B * (Kpd + 16) > codes) codes = (size_t)2 * B * (Kpd + 16);
  size_t stage = (size_t)(B == 1 ? 1 : 4) * Kp * 2;
  if ((size_t)B * (dmax + 8) * 2 > stage) stage = (size_t)B * (dmax + 8) * 2;
  size_t o = ((codes + 255) & ~(size_t)255) + ((stage + 255) & ~(size_t)255) + 4096 + 256;
  o += (size_t)(8 + 4 * D) * G * sizeof(float);
  o += (size_t)2 * ((B * m->n_heads * ns + 1) & ~1) * sizeof(float);
  o = (o + 15) & ~(size_t)15;
  o += sizeof(BitLayerDev) * m->n_layers;
  return o;
}

}  // namespace

extern "C" {

int64_t ohara_bitnet_persistent_workspace_bytes(const OharaBitModel* m, int batch, int n_workgroups) {
  if (!m || batch < 1 || n_workgroups < 1) return OHARA_EINVAL;
  return (int64_t)bit_layout(m, batch, n_workgroups).total;
}

int64_t ohara_bitnet_persistent_error_offset(const OharaBitModel* m, int batch, int n_workgroups) {
  if (!m || batch < 1 || n_workgroups < 1) return OHARA_EINVAL;
  const int ng = (n_workgroups + OHARA_BAR_GROUP - 1) / OHARA_BAR_GROUP;
  return (int64_t)bit_layout(m, batch, n_workgroups).bar + (int64_t)(ng + 2) * 64 * 4;
}

int ohara_bitnet_decode_persistent(const OharaBitModel* m, const OharaDecodeState* s, void* workspace, int n_workgroups,
                                   int init_workspace, int select_greedy, unsigned int spin_limit, void* stream) {
  if (!m || !s || !workspace || !m->layers || !s->kcache || !s->vcache || !s->step_state) return OHARA_EINVAL;
  if (s->batch < 1 || s->batch > 8) return OHARA_ESIZE;
  if (n_workgroups < 1 || n_workgroups > 1024) return OHARA_EINVAL;
  if (s->n_split != OHARA_MEGA_NS) return OHARA_EINVAL;
  const int D = m->head_dim;
  if (m->n_kv_heads < 1 || m->n_heads % m->n_kv_heads) return OHARA_EINVAL;
  const int G = m->n_heads / m->n_kv_heads;
  if (!(D == 128 || D == 64) || G != 1) return OHARA_ESIZE;
  if ((m->d_model & 15) || (m->d_ff & 15) || m->d_model > 4096 || m->d_ff > 6144) return OHARA_ESIZE;
  hipStream_t st = (hipStream_t)stream;
  char* ws = reinterpret_cast<char*>(workspace);
  const BitLayout L = bit_layout(m, s->batch, n_workgroups);
  BitMegaArgs a{};
  a.m = *m;
  a.layers_dev = reinterpret_cast<const BitLayerDev*>(ws + L.layers);
  if (init_workspace) {
    // small synchronous copies: done once per (model, cache) binding, outside any capture
    std::vector<BitLayerDev> tab(m->n_layers);
    for (int l = 0; l < m->n_layers; ++l) {
      const OharaBitLayer& src = m->layers[l];
      BitLayerDev& t = tab[l];
      for (int i = 0; i < 7; ++i) {
        t.w[i] = reinterpret_cast<const uint4*>(src.w[i]);
        t.nw[i] = src.norm_w[i];
        t.gamma[i] = src.gamma[i];
        if (!src.w[i] || !src.norm_w[i]) return OHARA_EINVAL;
      }
      t.norm1 = src.norm1; t.norm2 = src.norm2;
      t.kc = s->kcache[l]; t.vc = s->vcache[l];
      t.pad = 0.f;
    }
    if (hipMemcpyAsync((void*)a.layers_dev, tab.data(), sizeof(BitLayerDev) * m->n_layers, hipMemcpyHostToDevice, st) !=
            hipSuccess ||
        hipMemsetAsync((void*)(ws + L.bar), 0, L.total - L.bar, st) != hipSuccess ||
        hipStreamSynchronize(st) != hipSuccess)
      return OHARA_ELAUNCH;
    return OHARA_OK;
  }
  a.xm = ws + L.xm; a.qm = ws + L.qm; a.am = ws + L.am; a.pm = reinterpret_cast<float*>(ws + L.pm);
  a.dm = reinterpret_cast<int32_t*>(ws + L.dm); a.ds = reinterpret_cast<float*>(ws + L.ds);
  a.xm_stride = L.xm_stride; a.qm_stride = L.qm_stride; a.am_stride = L.am_stride; a.pm_stride = L.pm_stride;
  a.dm_stride = L.dm_stride;
  a.blk_x = L.blk_x; a.blk_a = L.blk_a;
  a.cand_val = reinterpret_cast<float*>(ws + L.candv);
  a.cand_idx = reinterpret_cast<int*>(ws + L.candi);
  a.bar = reinterpret_cast<unsigned int*>(ws + L.bar);
  a.B = s->batch; a.valid_vocab = s->valid_vocab; a.hist_cap = s->hist_cap;
  a.select = select_greedy;
  a.ids = s->ids; a.logits = s->logits;
  a.step_state = s->step_state; a.history = s->history;
  a.prof = nullptr;
  a.spin_limit = spin_limit ? spin_limit : (1u << 19);
  int ns = n_workgroups / (s->batch * m->n_kv_heads);
  ns = ns < 1 ? 1 : (ns > OHARA_MEGA_NS ? OHARA_MEGA_NS : ns);
  while (ns & (ns - 1)) ns &= ns - 1;
  a.ns = ns;
  const size_t smem = bit_smem_bytes(m, s->batch, ns);
  if (smem > 160 * 1024) return OHARA_ESIZE;
  dim3 grid(n_workgroups), block(256);
#define OHARA_BITMEGA(DD)                                                                                    \
  do {                                                                                                       \
    if (smem > 64 * 1024)                                                                                    \
      (void)hipFuncSetAttribute((const void*)bitnet_mega_kernel<DD, 1>,                                      \
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);                      \
    hipLaunchKernelGGL((bitnet_mega_kernel<DD, 1>), grid, block, smem, st, a);                               \
  } while (0)
  if (D == 128) OHARA_BITMEGA(128);
  else OHARA_BITMEGA(64);
#undef OHARA_BITMEGA
  return ohara_launch_status();
}

}  // extern "C"
