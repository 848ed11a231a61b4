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
// A single sequence: every workgroup derives the codes of the row it multiplies itself (a row is 2-11 KB;
// the three passes over it, spread over the workgroup, cost about as much as one hand-off).  Two to eight
// sequences: each (BitLinear, row) pair is quantised once, by one workgroup, and handed to the others
// through a code mailbox and one more grid barrier per GEMM phase.  Either way the reduction orders are
// those of the stand-alone BitLinear kernels, so the integer accumulators are those kernels' accumulators.
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
  int8_t* cq;      // NL code mailboxes (batch > 1): the code rows of the seven BitLinears, each quantised by one workgroup
  float* cs;       // NL x [7][16] {s, sum q} pairs of those rows (eight used)
  size_t cq_stride;
  float* ds;       // NL x 32 floats (a 128-byte line per layer: one writer, written before it is read):
                   // the activation scale s of every row of the down projection
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

// ---- a row -> its int8 codes -------------------------------------------------------------------
// BitLinear's activation side (bitnet.py:29-33, 49-53) on a row of K bf16 values: [block RMSNorm with
// pre_w,] the BitLinear's RMSNorm with nw, s = 127 / max|x_hat|, q = clamp(rint(x_hat * s), -128, 127).
// Which thread owns which 8-value piece and the order of every reduction are those of the stand-alone
// kernels (block_quant_row / wave_quant_row in csrc/bitlinear.hip), so the codes are the same codes.

// LDS of the kernel.  `codes`: up to two code sets (gate and up) of B rows x ldq bytes; `stage`: B bf16
// rows of the model width (the merged attention output, the normalised final stream).
struct BitLds {
  int8_t* codes;
  int ldq;          // bytes per code row of the current phase (K padded to 256, + 16 against bank conflicts)
  size_t set;       // bytes between the two code sets of the current phase
  bf16_t* stage;
  int ldm;          // elements between the rows of the merged attention output
  __device__ __forceinline__ void shape(int B, int K) {
    ldq = (((K + 255) >> 8) << 8) + 16;
    set = (size_t)B * ldq;
  }
  float* s_s;       // [2][16] activation scales
  int* s_sum;       // [2][16] sums of the codes
  float* red;       // 4 KiB: cross-wave sums
  int* sumw;        // [2][4] per-wave shares of the sums of the codes (and of the maximum, when a row is quantised once)
};

// The arithmetic of a row's codes, two values at a time.  x_hat = bf16(bf16(h * rinv) * nw) is formed once and
// kept as packed bf16 pairs; its largest magnitude is taken on the 15-bit patterns (for bf16 values the
// order of the magnitudes is the order of the patterns); q = rint(x_hat * s) is read from the low mantissa
// bits of x_hat * s + 1.5 * 2^23 (that addition rounds to the nearest integer, ties to even, as rintf does;
// |x_hat * s| <= 127 * (1 + 2^-22), so the clamp of bitnet.py:33 never acts and the low byte is the code).
typedef unsigned short u16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t bit_xhat2(uint32_t h, uint32_t w, float rinv) {
  return pack_bf(rbf(lo_bf(h) * rinv) * lo_bf(w), rbf(hi_bf(h) * rinv) * hi_bf(w));
}
__device__ __forceinline__ uint4 bit_xhat8(uint4 h, uint4 w, float rinv) {
  return make_uint4(bit_xhat2(h.x, w.x, rinv), bit_xhat2(h.y, w.y, rinv), bit_xhat2(h.z, w.z, rinv), bit_xhat2(h.w, w.w, rinv));
}
__device__ __forceinline__ uint32_t bit_mag_max2(uint32_t m, uint32_t xh) {
  return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(u16x2_t, m),
                                                                 __builtin_bit_cast(u16x2_t, xh & 0x7fff7fffu)));
}
__device__ __forceinline__ uint32_t bit_mag_max8(uint32_t m, uint4 xh) {
  return bit_mag_max2(bit_mag_max2(bit_mag_max2(bit_mag_max2(m, xh.x), xh.y), xh.z), xh.w);
}
__device__ __forceinline__ float bit_mag_float(uint32_t m) { return __uint_as_float(max(m & 0xffffu, m >> 16) << 16); }
#define BIT_RINT_MAGIC 12582912.0f      // 1.5 * 2^23
#define BIT_RINT_MAGIC_BITS 0x4B400000u
// eight packed x_hat values -> their eight code bytes; the raw words (code + BIT_RINT_MAGIC_BITS) are added to `sq`
__device__ __forceinline__ uint2 bit_codes8(uint4 xh, float s, uint32_t& sq) {
  const uint32_t u[4] = {xh.x, xh.y, xh.z, xh.w};
  uint32_t c[8];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    float p0 = lo_bf(u[j]) * s, p1 = hi_bf(u[j]) * s;
    // the products are rounded before the addition, as rintf's argument is: the empty statement keeps the compiler from
    // fusing the two into one multiply-add (it does so even for __fadd_rn(__fmul_rn(..))), which rounds once and sends
    // the frequent tie x_hat = max / 2 -> 63.5 to either side
    asm("" : "+v"(p0), "+v"(p1));
    c[2 * j] = __float_as_uint(p0 + BIT_RINT_MAGIC);
    c[2 * j + 1] = __float_as_uint(p1 + BIT_RINT_MAGIC);
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) sq += c[j];
  // byte 0 of four words -> one word (v_perm_b32: selector bytes 0-3 take from the second operand, 4-7 from the first, 0x0c is zero)
  const uint32_t lo = __builtin_amdgcn_perm(c[1], c[0], 0x0c0c0400u) | __builtin_amdgcn_perm(c[3], c[2], 0x04000c0cu);
  const uint32_t hi = __builtin_amdgcn_perm(c[5], c[4], 0x0c0c0400u) | __builtin_amdgcn_perm(c[7], c[6], 0x04000c0cu);
  return make_uint2(lo, hi);
}
// the sum of the codes from the sum of `n` raw words
__device__ __forceinline__ int bit_code_sum(uint32_t sq, int n) { return (int)(sq - (uint32_t)n * BIT_RINT_MAGIC_BITS); }

// ---- batch 1: the row in registers -------------------------------------------------------------
// Thread t owns the 8-value pieces t, t + 256, ... (NP of them; pieces beyond the row are zero and
// change no sum or maximum); the row never goes through LDS, all loads (row, norm weights) are
// in flight together, and the sum of the codes - needed only after the product - is left as four
// per-wave partial sums.
template <int NP, typename F>
__device__ __forceinline__ void row1_load(uint4 (&r)[NP], int pieces, F f) {
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    const int p = (int)threadIdx.x + 256 * i;
    r[i] = p < pieces ? f(p) : make_uint4(0, 0, 0, 0);
  }
}
__device__ __forceinline__ float row1_sum(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return ((red[0] + red[1]) + red[2]) + red[3];
}
// block-level RMSNorm (norm.py:16-21) of the row, in place
template <int NP>
__device__ __forceinline__ void row1_block_norm(uint4 (&v)[NP], const uint4 (&w)[NP], int K, float eps, float* red) {
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < NP; ++i) ss += bit_sumsq8(v[i]);
  const float rinv0 = 1.0f / sqrtf(row1_sum(ss, red) / (float)K + eps);
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    const uint32_t uu[4] = {v[i].x, v[i].y, v[i].z, v[i].w}, ww[4] = {w[i].x, w[i].y, w[i].z, w[i].w};
    uint32_t o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
      o[j] = pack_bf(rbf(lo_bf(uu[j]) * rinv0) * lo_bf(ww[j]), rbf(hi_bf(uu[j]) * rinv0) * hi_bf(ww[j]));
    v[i] = make_uint4(o[0], o[1], o[2], o[3]);
  }
}
// the BitLinear's own norm, scale and codes of the row h (bitnet.py:29-33, 49-53) -> xq (LDS);
// thread 0 leaves the scale in *s_out, every wave its share of the sum of the codes in sumw[wave]
template <int NP>
__device__ __forceinline__ void row1_codes(const uint4 (&h)[NP], const uint4 (&nw)[NP], int pieces, int K, float eps,
                                           int8_t* xq, float* red, float* s_out, int* sumw) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < NP; ++i) ss += bit_sumsq8(h[i]);
  const float rinv = 1.0f / sqrtf(row1_sum(ss, red) / (float)K + eps);
  uint4 xh[NP];
  uint32_t mg = 0u;
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    xh[i] = bit_xhat8(h[i], nw[i], rinv);
    mg = bit_mag_max8(mg, xh[i]);
  }
  float mx = wave_max(bit_mag_float(mg));
  __syncthreads();
  if (lane == 0) red[wave] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  const float s = 127.0f / fmaxf(mx, 1e-5f);
  uint32_t sqw = 0u;
#pragma unroll
  for (int i = 0; i < NP; ++i) {
    const uint2 pk = bit_codes8(xh[i], s, sqw);
    const int p = tid + 256 * i;
    if (p < pieces) sts8(xq + (size_t)p * 8, pk);
  }
  int sq = bit_code_sum(sqw, NP * 8);
  sq = lanes_sum<32, 1>(sq);
  if (lane == 0) sumw[wave] = sq;
  if (tid == 0) *s_out = s;
}

// Batch 1: one row from `load(piece) -> uint4` into one or two code sets (two BitLinears that share
// the input and the block norm: ff.gate and ff.up).  Every thread of the workgroup calls.
template <int NP, typename Load>
__device__ __forceinline__ void bit_stage_row1(const BitLds& L, int nsets, int K, const bf16_t* pre_w, const bf16_t* nw0,
                                               const bf16_t* nw1, float eps, Load load) {
  const int tid = threadIdx.x;
  const int pieces = K >> 3;
  uint4 x[NP], pw[NP], n0[NP], n1[NP];
  row1_load(x, pieces, load);
  if (pre_w) row1_load(pw, pieces, [&](int p) { return ldg16(pre_w + (size_t)p * 8); });
  row1_load(n0, pieces, [&](int p) { return ldg16(nw0 + (size_t)p * 8); });
  if (nsets == 2) row1_load(n1, pieces, [&](int p) { return ldg16(nw1 + (size_t)p * 8); });
  __syncthreads();  // whoever still reads the previous codes or scales is done
  {
    const int pad8 = (L.ldq - K) >> 3;
    for (int i = tid; i < nsets * pad8; i += 256) {
      const int st = i / pad8, c = i - st * pad8;
      sts8(L.codes + (size_t)st * L.set + K + c * 8, make_uint2(0, 0));
    }
  }
  if (pre_w) row1_block_norm(x, pw, K, eps, L.red);
  row1_codes(x, n0, pieces, K, eps, L.codes, L.red, L.s_s, L.sumw);
  if (nsets == 2) row1_codes(x, n1, pieces, K, eps, L.codes + L.set, L.red, L.s_s + 16, L.sumw + 4);
  __syncthreads();
  if (tid < nsets) L.s_sum[tid * 16] = (L.sumw[tid * 4] + L.sumw[tid * 4 + 1]) + (L.sumw[tid * 4 + 2] + L.sumw[tid * 4 + 3]);
  // the product that follows passes a workgroup barrier before anyone reads s_sum
}
// The norm weights of a row's staging (block norm `pre_w`, the BitLinears' own norms `nw0` / `nw1`) do not
// depend on the phase before it: row1_norm_fetch issues their loads - in the barrier window, next to the
// phase's weight prefetch, where a cold HBM read costs nothing - and bit_stage_row1_pre takes them from
// registers.  Pieces past the row read the last piece and multiply values that are zero.
template <int NP>
__device__ __forceinline__ void row1_norm_fetch(uint4 (&r)[NP], int pieces, const bf16_t* w) {
#pragma unroll
  for (int i = 0; i < NP; ++i) r[i] = ldg16(w + (size_t)min((int)threadIdx.x + 256 * i, pieces - 1) * 8);
}
template <int NP, typename Load>
__device__ __forceinline__ void bit_stage_row1_pre(const BitLds& L, int nsets, int K, bool block_norm, const uint4 (&pw)[NP],
                                                   const uint4 (&n0)[NP], const uint4 (&n1)[NP], float eps, Load load) {
  const int tid = threadIdx.x;
  const int pieces = K >> 3;
  uint4 x[NP];
  row1_load(x, pieces, load);
  __syncthreads();  // whoever still reads the previous codes or scales is done
  {
    const int pad8 = (L.ldq - K) >> 3;
    for (int i = tid; i < nsets * pad8; i += 256) {
      const int st = i / pad8, c = i - st * pad8;
      sts8(L.codes + (size_t)st * L.set + K + c * 8, make_uint2(0, 0));
    }
  }
  if (block_norm) row1_block_norm(x, pw, K, eps, L.red);
  row1_codes(x, n0, pieces, K, eps, L.codes, L.red, L.s_s, L.sumw);
  if (nsets == 2) row1_codes(x, n1, pieces, K, eps, L.codes + L.set, L.red, L.s_s + 16, L.sumw + 4);
  __syncthreads();
  if (tid < nsets) L.s_sum[tid * 16] = (L.sumw[tid * 4] + L.sumw[tid * 4 + 1]) + (L.sumw[tid * 4 + 2] + L.sumw[tid * 4 + 3]);
  // the product that follows passes a workgroup barrier before anyone reads s_sum
}

// ---- batch > 1: every (BitLinear, row) pair is quantised once ---------------------------------
// With B rows a workgroup that derived all the codes itself would spend 8 - 17 us per phase on them at eight rows
// (the three passes are instruction-bound with one wave per SIMD), 256 times over.  Instead ONE workgroup
// per (BitLinear, row) pair derives the row's codes with all its threads (thread t owns the pieces t, t + 256, ...),
// stores them and {s, sum q} in a per-layer mailbox, a grid barrier follows, and every workgroup copies the code
// rows it multiplies into its LDS.  The sums of squares keep the order of the stand-alone kernels' wave-owned
// rows (wave_quant_row in csrc/bitlinear.hip: lane l adds the pieces l, l + 64, ... in turn, then the wave's
// butterfly): the per-piece sums go through LDS and the first wave adds them in that order; the maximum and the
// sum of the codes are exact in any order.  So the codes are still those kernels' codes.
__host__ __device__ inline size_t bit_cq_al(size_t v) { return (v + 255) & ~(size_t)255; }
template <int NP1, typename Load>
__device__ __forceinline__ void bit_quant_once(const BitLds& L, int K, const bf16_t* pre_w, const bf16_t* nw, float eps,
                                               Load load, int8_t* cq_row, int ldq, float* stat) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int pieces = K >> 3;
  uint4 x[NP1], pw[NP1], n0[NP1];
  row1_load(x, pieces, load);
  if (pre_w) row1_norm_fetch<NP1>(pw, pieces, pre_w);
  row1_norm_fetch<NP1>(n0, pieces, nw);
  float* psum = L.red;  // one sum of squares per piece (at most 768), the result at [1000]
  auto rinv_of = [&](const uint4 (&v)[NP1]) {
    __syncthreads();
#pragma unroll
    for (int i = 0; i < NP1; ++i) {
      const int p = tid + 256 * i;
      if (p < pieces) psum[p] = bit_sumsq8(v[i]);
    }
    __syncthreads();
    if (wave == 0) {
      float ss = 0.f;
#pragma unroll
      for (int i = 0; i < 4 * NP1; ++i) {
        const int p = lane + 64 * i;
        ss += p < pieces ? psum[p] : 0.f;
      }
      ss = wave_sum(ss);
      if (lane == 0) psum[1000] = 1.0f / sqrtf(ss / (float)K + eps);
    }
    __syncthreads();
    return psum[1000];
  };
  if (pre_w) {  // block-level RMSNorm (norm.py:16-21)
    const float r0 = rinv_of(x);
#pragma unroll
    for (int i = 0; i < NP1; ++i) x[i] = bit_xhat8(x[i], pw[i], r0);
  }
  const float rinv = rinv_of(x);
  uint4 xh[NP1];
  uint32_t mg = 0u;
#pragma unroll
  for (int i = 0; i < NP1; ++i) {
    xh[i] = bit_xhat8(x[i], n0[i], rinv);
    mg = bit_mag_max8(mg, xh[i]);
  }
  float mx = wave_max(bit_mag_float(mg));
  int* iw = L.sumw;
  if (lane == 0) iw[wave] = __float_as_int(mx);
  __syncthreads();
  mx = fmaxf(fmaxf(__int_as_float(iw[0]), __int_as_float(iw[1])), fmaxf(__int_as_float(iw[2]), __int_as_float(iw[3])));
  const float s = 127.0f / fmaxf(mx, 1e-5f);
  uint32_t sqw = 0u;
#pragma unroll
  for (int i = 0; i < NP1; ++i) {
    const uint2 pk = bit_codes8(xh[i], s, sqw);
    const int p = tid + 256 * i;
    if (p < pieces) st_coh8(cq_row + (size_t)p * 8, pk);
  }
  for (int c = K + tid * 8; c < ldq; c += 2048) st_coh8(cq_row + c, make_uint2(0, 0));  // the columns up to the chunk's end
  const int sq = lanes_sum<32, 1>(bit_code_sum(sqw, NP1 * 8));
  if (lane == 0) iw[4 + wave] = sq;
  __syncthreads();
  if (tid == 0) st_coh8(stat, make_uint2(__float_as_uint(s), (uint32_t)((iw[4] + iw[5]) + (iw[6] + iw[7]))));
}
// Unit u of `units` goes to workgroup u * (nwg / units) (spread over the grid; with fewer workgroups than units they loop).
template <typename F>
__device__ __forceinline__ void bit_for_units(int units, int nwg, F fn) {
  const int stride = max(1, nwg / units);
  const int nq = (nwg + stride - 1) / stride;
  if ((int)blockIdx.x % stride == 0)
    for (int u = (int)blockIdx.x / stride; u < units; u += nq) fn(u);
}
// The code rows of `nsets` consecutive BitLinears (B rows each; the mailbox has the row and set strides of the LDS
// copy) and their scales -> LDS.  Whole rows are one flat copy; a K partition [c0, c1) of 256-column chunks (at most
// 16 of them) is copied row by row.  Every thread of the workgroup calls.
__device__ __forceinline__ void bit_codes_fetch(const BitLds& L, int nsets, int B, const int8_t* cq, const float* st, int c0,
                                                int c1, bool whole) {
  const int tid = threadIdx.x;
  __syncthreads();  // whoever still reads the previous codes or scales is done
  if (whole) {
    const int n16 = (int)((size_t)nsets * B * L.ldq) >> 4;
    for (int i0 = 0; i0 < n16; i0 += 256 * 6) {
      uint4 v[6];
#pragma unroll
      for (int u = 0; u < 6; ++u) v[u] = ldg16(cq + (size_t)min(i0 + u * 256 + tid, n16 - 1) * 16);
#pragma unroll
      for (int u = 0; u < 6; ++u)
        if (i0 + u * 256 + tid < n16) sts16(L.codes + (size_t)(i0 + u * 256 + tid) * 16, v[u]);
    }
  } else {
    const int segs = (c1 - c0) * 16;  // 16-byte pieces per row: at most 256
    uint4 v[8];
#pragma unroll
    for (int b = 0; b < 8; ++b)
      v[b] = ldg16(cq + (size_t)min(b, B - 1) * L.ldq + (size_t)c0 * 256 + (size_t)min(tid, segs - 1) * 16);
#pragma unroll
    for (int b = 0; b < 8; ++b)
      if (b < B && tid < segs) sts16(L.codes + (size_t)b * L.ldq + (size_t)c0 * 256 + (size_t)tid * 16, v[b]);
  }
  if (tid < nsets * B) {
    const int set = tid / B, b = tid - set * B;
    const uint2 v = ldg8(st + set * 32 + b * 2);
    L.s_s[set * 16 + b] = __uint_as_float(v.x);
    L.s_sum[set * 16 + b] = (int)v.y;
  }
  __syncthreads();
}

// ---- one strip of a ternary weight x the code rows ---------------------------------------------
// Chunks [cb, ce) of 256 columns, split over KP waves (a workgroup works on 4 / KP strips at a time,
// wave w on the strip of its group w / KP); the integer sum over the KP waves lands in the group's
// first wave (returns true there).  `wpre`: the first BIT_PF chunks of this wave, fetched ahead.  Rows beyond B
// read row B - 1 (their results are never looked at).  Every thread of the workgroup calls.
#define BIT_PF 6
struct BitPre {
  uint4 w[BIT_PF];
};
template <int KP>
__device__ __forceinline__ void bit_wave_chunks(int cb, int ce, int& c0, int& c1) {
  const int kpart = (threadIdx.x >> 6) % KP;
  const int per = (ce - cb + KP - 1) / KP;
  c0 = cb + kpart * per;
  c1 = min(ce, c0 + per);
}
template <int KP>
__device__ __forceinline__ void bit_prefetch(const uint4* wp, int KC, int strip, int cb, int ce, bool live, BitPre& pre) {
  int c0, c1;
  bit_wave_chunks<KP>(cb, ce, c0, c1);
  const uint4* wrow = wp + (size_t)strip * KC * 64 + (threadIdx.x & 63);
#pragma unroll
  for (int c = 0; c < BIT_PF; ++c)
    pre.w[c] = (live && c0 + c < c1) ? ldg16_nt(wrow + (size_t)(c0 + c) * 64) : make_uint4(0, 0, 0, 0);
}
template <int KP>
__device__ __forceinline__ bool bit_strip(const uint4* wp, int KC, int strip, int cb, int ce, bool live,
                                          const BitPre& pre, bool use_pre, const int8_t* xq, int ldq, int B, int* red,
                                          i32x4& acc) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int kpart = wave % KP;
  const int m = lane & 15, g = lane >> 4;
  int c0, c1;
  bit_wave_chunks<KP>(cb, ce, c0, c1);
  const uint4* wrow = wp + (size_t)strip * KC * 64 + lane;
  const int8_t* xrow = xq + (size_t)min(m, B - 1) * ldq + 16 * g;
  acc = (i32x4){0, 0, 0, 0};
  if (live) {
    for (int cbk = c0; cbk < c1; cbk += BIT_PF) {
      uint4 wv[BIT_PF];
      if (use_pre && cbk == c0) {
#pragma unroll
        for (int c = 0; c < BIT_PF; ++c) wv[c] = pre.w[c];
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
  if (KP > 1) {
    if (kpart > 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i) red[(wave * 64 + lane) * 4 + i] = acc[i];
    }
    __syncthreads();
    if (kpart == 0) {
#pragma unroll
      for (int w = 1; w < KP; ++w)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] += red[((wave + w) * 64 + lane) * 4 + i];
    }
    __syncthreads();  // red is free again
  }
  return kpart == 0 && live;
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
// ONE: a single sequence.  The staging of the workgroup's own row is then the only one compiled in, the
// quantise-once sub-phases and the code fetch otherwise, which keeps either kernel's layer loop much smaller
// than one that holds both.
// PROFILE: with the phase stamps (measurement builds of the head-dim-128 kernels only).
template <int D, int G, bool ONE, bool PROFILE = false>
__global__ __launch_bounds__(256) void bitnet_mega_kernel(BitMegaArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const OharaBitModel& m = a.m;
  const int d = m.d_model, H = m.n_heads, Hkv = m.n_kv_heads, F = m.d_ff, V = m.vocab, B = ONE ? 1 : a.B;
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
  const size_t stage_bytes = (size_t)B * (dmax + 8) * 2;
  L.stage = reinterpret_cast<bf16_t*>(smem + off);
  L.ldm = dmax + 8;
  off += (stage_bytes + 255) & ~(size_t)255;
  L.red = reinterpret_cast<float*>(smem + off); off += 4096;
  L.s_s = reinterpret_cast<float*>(smem + off); off += 128;
  L.s_sum = reinterpret_cast<int*>(smem + off); off += 128;
  L.sumw = reinterpret_cast<int*>(smem + off); off += 64;
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
  ProfT<PROFILE> pf((blockIdx.x == 0 && tid == 0) ? a.prof : nullptr);

  const int KCd = (d + 255) >> 8, KCo = (HD + 255) >> 8, KCf = (F + 255) >> 8;
  const int ns_q = HD / 16, ns_kv = (Hkv * D) / 16, ns_d = (d + 15) / 16, ns_f = (F + 15) / 16;
  const bool ok_pos = pos >= 0 && pos < m.t_max;
  // batch > 1: where the code rows of the seven BitLinears start in a layer's code mailbox (B rows each)
  const int ldq_d = (KCd << 8) + 16, ldq_o = (KCo << 8) + 16, ldq_f = (KCf << 8) + 16;
  // (a group of sets that one sub-phase writes starts on its own 256 bytes: a cache line that an earlier phase's readers
  // fetched while part of it was still unwritten would be found stale by the later phase's plain loads)
  const size_t cq_o = bit_cq_al((size_t)3 * B * ldq_d), cq_g = bit_cq_al(cq_o + (size_t)B * ldq_o);
  const size_t cq_dn = bit_cq_al(cq_g + (size_t)2 * B * ldq_d);
  ProfT<false> nopf(nullptr);  // the barrier after a quantising sub-phase is not stamped

  GemmP lm{};
  lm.N = V; lm.K = d; lm.nstrips = (V + 15) / 16; lm.out = reinterpret_cast<char*>(a.logits); lm.ldo = V;
  lm.valid = a.valid_vocab > 0 ? min(a.valid_vocab, V) : V;
  lm.wp = reinterpret_cast<const uint4*>(m.w_vocab);
  AttnPre<D> apre;
  BitPre wpre, wpre2;

  // P1: the workgroups are split into three groups, one per projection, in proportion to the
  // projections' strips, so that a workgroup derives the codes of one BitLinear only; it works on
  // two strips at a time (two waves each)
  const int sub2 = wave >> 1;
  const int p1_units = ns_q + 2 * ns_kv;
  const int gq = max(1, (int)((long long)nwg * ns_q / p1_units));
  const int gk = max(1, (nwg - gq) / 2);
  const int p1_which = (int)blockIdx.x < gq ? BQ : ((int)blockIdx.x < gq + gk ? BK : BV);
  const int p1_gi = (int)blockIdx.x - (p1_which == BQ ? 0 : (p1_which == BK ? gq : gq + gk));
  const int p1_gsz = p1_which == BQ ? gq : (p1_which == BK ? gk : nwg - gq - gk);
  const int p1_nstr = p1_which == BQ ? ns_q : ns_kv;
  const int p1_strip0 = 2 * p1_gi + sub2;
  // the rotation of this lane's outputs in its first strip: the same in every layer
  uint32_t rope_c = 0, rope_s = 0;
  if (p1_which != BV && p1_strip0 < p1_nstr && ok_pos) {
    const int dd = (p1_strip0 * 16 + 4 * gg) % D;
    rope_c = ldg4(m.cos + (size_t)pos * (D >> 1) + (dd >> 1));
    rope_s = ldg4(m.sin + (size_t)pos * (D >> 1) + (dd >> 1));
  }
  bit_prefetch<2>(reinterpret_cast<const uint4*>(gptr(ltab[0].w[p1_which])), KCd, p1_strip0, 0, KCd, p1_strip0 < p1_nstr, wpre);
  // batch-1 build: the norm weights of the next phase's staging, fetched in the barrier windows
  uint4 npw[1], nn0[3], nn1[1];
  npw[0] = nn0[0] = nn0[1] = nn0[2] = nn1[0] = make_uint4(0, 0, 0, 0);
  if (ONE && 2 * p1_gi < p1_nstr) {
    row1_norm_fetch<1>(npw, d >> 3, reinterpret_cast<const bf16_t*>(gptr(ltab[0].norm1)));
    row1_norm_fetch<1>(reinterpret_cast<uint4(&)[1]>(nn0), d >> 3, reinterpret_cast<const bf16_t*>(gptr(ltab[0].nw[p1_which])));
  }

  for (int l = 0; l < m.n_layers; ++l) {
    const BitLayerDev& LY = ltab[l];
    bf16_t* kc = reinterpret_cast<bf16_t*>(gptr(LY.kc));
    bf16_t* vc = reinterpret_cast<bf16_t*>(gptr(LY.vc));
    char* x_mid = a.xm + (size_t)l * a.xm_stride;
    char* q_l = a.qm + (size_t)l * a.qm_stride;
    char* a_l = a.am + (size_t)l * a.am_stride;
    float* p_l = a.pm + (size_t)l * a.pm_stride;
    int32_t* d_l = a.dm + (size_t)l * a.dm_stride;
    int8_t* cq_l = a.cq + (size_t)l * a.cq_stride;
    float* cs_l = a.cs + (size_t)l * 256;  // {s, sum q} of row b of set i at (i * 32 + b * 2): a 128-byte line per set
    // the stream entering this layer
    BitX xin{};
    xin.B = B; xin.N = d; xin.blk = a.blk_x;
    if (l == 0) {
      xin.ids = a.ids; xin.table = m.token_emb; xin.vocab = V;
    } else {
      xin.xmid = a.xm + (size_t)(l - 1) * a.xm_stride;
      xin.parts = a.dm + (size_t)(l - 1) * a.dm_stride;
      xin.ds = a.ds + (size_t)(l - 1) * 32;
      xin.gamma = ltab[l - 1].gamma[BD];
    }
    const bf16_t* norm1 = reinterpret_cast<const bf16_t*>(gptr(LY.norm1));
    const bf16_t* norm2 = reinterpret_cast<const bf16_t*>(gptr(LY.norm2));

    // ---- P1: Q, K, V + rotary + append ----
    L.shape(B, d);
    auto load_in = [&](int b, int p) {
      uint32_t w[4];
      bitx_load<8>(xin, b, p * 8, w);
      return make_uint4(w[0], w[1], w[2], w[3]);
    };
    if (!ONE) {
      bit_for_units(3 * B, nwg, [&](int u) {
        const int which = u / B, b = u - which * B;
        bit_quant_once<1>(L, d, norm1, reinterpret_cast<const bf16_t*>(gptr(LY.nw[which])), m.eps,
                          [&](int p) { return load_in(b, p); }, cq_l + (size_t)u * ldq_d, ldq_d, cs_l + which * 32 + b * 2);
      });
      gs.arrive(nopf);
      gs.wait(nopf);
    }
    if (2 * p1_gi < p1_nstr) {
      const int which = p1_which;
      const uint4* wp = reinterpret_cast<const uint4*>(gptr(LY.w[which]));
      if (ONE) {
        auto load0 = [&](int p) { return load_in(0, p); };
        bit_stage_row1_pre<1>(L, 1, d, true, npw, reinterpret_cast<const uint4(&)[1]>(nn0), nn1, m.eps, load0);
      } else {
        bit_codes_fetch(L, 1, B, cq_l + (size_t)which * B * ldq_d, cs_l + which * 32, 0, KCd, true);
      }
      for (int s0 = 2 * p1_gi; s0 < p1_nstr; s0 += 2 * p1_gsz) {
        const bool first = s0 == 2 * p1_gi;
        const int strip = s0 + sub2;
        i32x4 acc;
        if (bit_strip<2>(wp, KCd, strip, 0, KCd, strip < p1_nstr, wpre, first, L.codes, L.ldq, B,
                         reinterpret_cast<int*>(L.red), acc) &&
            mm < B && ok_pos) {
          const int b = mm;
          const int r0 = strip * 16 + 4 * gg;
          float v[4];
          bit_scale(acc, L.s_sum[b], L.s_s[b], LY.gamma[which], v);
          char* o;
          if (which != BV) {
            uint32_t cs = rope_c, sn = rope_s;
            if (!first) {
              const int dd = r0 % D;
              cs = ldg4(m.cos + (size_t)pos * (D >> 1) + (dd >> 1));
              sn = ldg4(m.sin + (size_t)pos * (D >> 1) + (dd >> 1));
            }
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
    bit_prefetch<4>(wo, KCo, blockIdx.x, 0, KCo, (int)blockIdx.x < ns_d, wpre);
    if (ONE && (int)blockIdx.x < ns_d)
      row1_norm_fetch<1>(reinterpret_cast<uint4(&)[1]>(nn0), HD >> 3, reinterpret_cast<const bf16_t*>(gptr(LY.nw[BO])));
    // the residual of this lane's outputs in the first strip: known since the previous layer
    uint32_t rpre[2] = {0u, 0u};
    if ((int)blockIdx.x < ns_d && wave == 0 && mm < B && (int)blockIdx.x * 16 + 4 * gg < d)
      bitx_load<4>(xin, mm, (int)blockIdx.x * 16 + 4 * gg, rpre);
    gs.wait(pf);
    // ---- P3: merge + attn.proj + residual ----
    L.shape(B, HD);
    if (!ONE) {  // one workgroup per row merges the row's chunks and derives its codes
      bit_for_units(B, nwg, [&](int b) {
        bf16_t* xs = L.stage;
        __syncthreads();
        stage_attn_merge_any<false>(a.ns, xs, L.ldm, p_l + (size_t)b * H * OHARA_MEGA_NS * (D + 32), 1, H, D, mrg_w, mrg_l);
        __syncthreads();
        bit_quant_once<1>(L, HD, nullptr, reinterpret_cast<const bf16_t*>(gptr(LY.nw[BO])), m.eps,
                          [&](int p) { return lds16(xs + p * 8); }, cq_l + cq_o + (size_t)b * ldq_o, ldq_o, cs_l + BO * 32 + b * 2);
      });
      gs.arrive(nopf);
      gs.wait(nopf);
    }
    for (int strip = blockIdx.x; strip < ns_d; strip += nwg) {
      const bool first = strip == (int)blockIdx.x;
      if (first) {
        if (ONE) {
          bf16_t* xs = L.stage;
          const int ldxs = L.ldm;
          // a single sequence always runs with 16 chunks unless there are more than 16 KV heads: that
          // merge is part of the kernel (a call would wait for the weights already in flight)
          if (a.ns == 16 && B * HD > 4 * 256) stage_attn_merge<16>(xs, ldxs, p_l, B, H, D, mrg_w, mrg_l);
          else stage_attn_merge_any<false>(a.ns, xs, ldxs, p_l, B, H, D, mrg_w, mrg_l);
          __syncthreads();
          auto load0 = [&](int p) { return lds16(xs + p * 8); };
          bit_stage_row1_pre<1>(L, 1, HD, false, npw, reinterpret_cast<const uint4(&)[1]>(nn0), nn1, m.eps, load0);
        } else {
          bit_codes_fetch(L, 1, B, cq_l + cq_o, cs_l + BO * 32, 0, KCo, true);
        }
      }
      i32x4 acc;
      if (bit_strip<4>(wo, KCo, strip, 0, KCo, true, wpre, first, L.codes, L.ldq, B,
                       reinterpret_cast<int*>(L.red), acc) && mm < B) {
        const int b = mm;
        const int r0 = strip * 16 + 4 * gg;
        if (r0 < d) {
          float y[4];
          bit_scale(acc, L.s_sum[b], L.s_s[b], LY.gamma[BO], y);
          uint32_t r[2] = {rpre[0], rpre[1]};
          if (!first) bitx_load<4>(xin, b, r0, r);
          st_coh8(const_cast<char*>(xm_addr(x_mid, a.blk_x, b, r0)),
                  make_uint2(pack_bf(lo_bf(r[0]) + y[0], hi_bf(r[0]) + y[1]), pack_bf(lo_bf(r[1]) + y[2], hi_bf(r[1]) + y[3])));
        }
      }
    }
    gs.arrive(pf);
    const uint4* wg = reinterpret_cast<const uint4*>(gptr(LY.w[BG]));
    const uint4* wu = reinterpret_cast<const uint4*>(gptr(LY.w[BU]));
    {
      const int strip = 2 * (int)blockIdx.x + sub2;
      bit_prefetch<2>(wg, KCd, strip, 0, KCd, strip < ns_f, wpre);
      bit_prefetch<2>(wu, KCd, strip, 0, KCd, strip < ns_f, wpre2);
    }
    if (ONE && 2 * (int)blockIdx.x < ns_f) {
      row1_norm_fetch<1>(npw, d >> 3, norm2);
      row1_norm_fetch<1>(reinterpret_cast<uint4(&)[1]>(nn0), d >> 3, reinterpret_cast<const bf16_t*>(gptr(LY.nw[BG])));
      row1_norm_fetch<1>(nn1, d >> 3, reinterpret_cast<const bf16_t*>(gptr(LY.nw[BU])));
    }
    gs.wait(pf);
    // ---- P4: norm2 + ff.gate, ff.up + SwiGLU; two strips at a time, two waves each ----
    L.shape(B, d);
    BitX xmid{};
    xmid.B = B; xmid.N = d; xmid.blk = a.blk_x; xmid.xmid = x_mid;
    auto load_mid = [&](int b, int p) {
      uint32_t w[4];
      bitx_load<8>(xmid, b, p * 8, w);
      return make_uint4(w[0], w[1], w[2], w[3]);
    };
    if (!ONE) {
      bit_for_units(2 * B, nwg, [&](int u) {
        const int set = u / B, b = u - set * B;
        bit_quant_once<1>(L, d, norm2, reinterpret_cast<const bf16_t*>(gptr(LY.nw[BG + set])), m.eps,
                          [&](int p) { return load_mid(b, p); }, cq_l + cq_g + (size_t)u * ldq_d, ldq_d,
                          cs_l + (BG + set) * 32 + b * 2);
      });
      gs.arrive(nopf);
      gs.wait(nopf);
    }
    if (2 * (int)blockIdx.x < ns_f) {
      if (ONE) {
        auto load0 = [&](int p) { return load_mid(0, p); };
        bit_stage_row1_pre<1>(L, 2, d, true, npw, reinterpret_cast<const uint4(&)[1]>(nn0), nn1, m.eps, load0);
      } else {
        bit_codes_fetch(L, 2, B, cq_l + cq_g, cs_l + BG * 32, 0, KCd, true);
      }
      for (int s0 = 2 * (int)blockIdx.x; s0 < ns_f; s0 += 2 * nwg) {
        const bool first = s0 == 2 * (int)blockIdx.x;
        const int strip = s0 + sub2;
        i32x4 ag, au;
        const bool w0g = bit_strip<2>(wg, KCd, strip, 0, KCd, strip < ns_f, wpre, first, L.codes, L.ldq, B,
                                      reinterpret_cast<int*>(L.red), ag);
        const bool w0u = bit_strip<2>(wu, KCd, strip, 0, KCd, strip < ns_f, wpre2, first, L.codes + L.set, L.ldq,
                                      B, reinterpret_cast<int*>(L.red), au);
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
      bit_prefetch<4>(wd, KCf, strip, part * per_part, min(KCf, (part + 1) * per_part), unit < ns_d * OHARA_BIT_DOWN_SPLIT, wpre);
      if (ONE && unit < ns_d * OHARA_BIT_DOWN_SPLIT) {
        const bf16_t* nwd = reinterpret_cast<const bf16_t*>(gptr(LY.nw[BD]));
        if (F <= 2048) row1_norm_fetch<1>(reinterpret_cast<uint4(&)[1]>(nn0), F >> 3, nwd);
        else row1_norm_fetch<3>(nn0, F >> 3, nwd);
      }
    }
    gs.wait(pf);
    // ---- P5: ff.down, K split over OHARA_BIT_DOWN_SPLIT groups of workgroups ----
    {
      const int nunits = ns_d * OHARA_BIT_DOWN_SPLIT;
      L.shape(B, F);
      if (!ONE) {
        const bf16_t* nwd = reinterpret_cast<const bf16_t*>(gptr(LY.nw[BD]));
        bit_for_units(B, nwg, [&](int b) {
          auto loadq = [&](int p) { return ldg16(am_addr(a_l, a.blk_a, b, p * 8)); };
          if (F <= 2048) bit_quant_once<1>(L, F, nullptr, nwd, m.eps, loadq, cq_l + cq_dn + (size_t)b * ldq_f, ldq_f, cs_l + BD * 32 + b * 2);
          else bit_quant_once<3>(L, F, nullptr, nwd, m.eps, loadq, cq_l + cq_dn + (size_t)b * ldq_f, ldq_f, cs_l + BD * 32 + b * 2);
        });
        gs.arrive(nopf);
        gs.wait(nopf);
      }
      bool staged = false;
      for (int unit = blockIdx.x; unit < nunits; unit += nwg) {
        const bool first = unit == (int)blockIdx.x;
        const int part = unit / ns_d, strip = unit - part * ns_d;
        if (!staged) {
          if (ONE) {
            auto load0 = [&](int p) { return ldg16(am_addr(a_l, a.blk_a, 0, p * 8)); };
            if (F <= 2048) bit_stage_row1_pre<1>(L, 1, F, false, npw, reinterpret_cast<const uint4(&)[1]>(nn0), nn1, m.eps, load0);
            else bit_stage_row1_pre<3>(L, 1, F, false, nn0, nn0, nn0, m.eps, load0);
          } else {  // the codes of this workgroup's K partition (its units all lie in one partition or take whole rows)
            const bool one_part = (int)blockIdx.x + nwg >= nunits;
            if (one_part) bit_codes_fetch(L, 1, B, cq_l + cq_dn, cs_l + BD * 32, part * per_part, min(KCf, (part + 1) * per_part), false);
            else bit_codes_fetch(L, 1, B, cq_l + cq_dn, cs_l + BD * 32, 0, KCf, true);
          }
          staged = true;
        }
        i32x4 acc;
        if (bit_strip<4>(wd, KCf, strip, part * per_part, min(KCf, (part + 1) * per_part), true, wpre, first,
                         L.codes, L.ldq, B, reinterpret_cast<int*>(L.red), acc) && mm < B) {
          const int b = mm;
          const int r0 = strip * 16 + 4 * gg;
          if (r0 < d) {
            const int sq = part == 0 ? L.s_sum[b] : 0;  // the codes are T + 1: the first part takes the correction
            int32_t* o = const_cast<int32_t*>(iparts_addr(d_l, ns_d, B, part, b, r0));
            st_coh8(o, make_uint2((uint32_t)(acc[0] - sq), (uint32_t)(acc[1] - sq)));
            st_coh8(o + 2, make_uint2((uint32_t)(acc[2] - sq), (uint32_t)(acc[3] - sq)));
          }
          if (unit == 0 && gg == 0) st_coh4(a.ds + (size_t)l * 32 + b, __float_as_uint(L.s_s[b]));
        }
      }
    }
    gs.arrive(pf);
    if (l + 1 == m.n_layers) break;  // the last barrier's wait follows the loop, behind another prefetch
    bit_prefetch<2>(reinterpret_cast<const uint4*>(gptr(ltab[l + 1].w[p1_which])), KCd, p1_strip0, 0, KCd,
                    p1_strip0 < p1_nstr, wpre);
    if (ONE && 2 * p1_gi < p1_nstr) {
      row1_norm_fetch<1>(npw, d >> 3, reinterpret_cast<const bf16_t*>(gptr(ltab[l + 1].norm1)));
      row1_norm_fetch<1>(reinterpret_cast<uint4(&)[1]>(nn0), d >> 3, reinterpret_cast<const bf16_t*>(gptr(ltab[l + 1].nw[p1_which])));
    }
    gs.wait(pf);
  }
  GemmPre lpre;
  gemm_prefetch<1, 24, E_LOGITS>(lm, lpre, B);
  gs.wait(pf);
  // ---- final norm + vocabulary projection (bf16), running arg-max per lane ----
  {
    BitX xf{};
    xf.B = B; xf.N = d; xf.blk = a.blk_x;
    xf.xmid = a.xm + (size_t)(m.n_layers - 1) * a.xm_stride;
    xf.parts = a.dm + (size_t)(m.n_layers - 1) * a.dm_stride;
    xf.ds = a.ds + (size_t)(m.n_layers - 1) * 32;
    xf.gamma = ltab[m.n_layers - 1].gamma[BD];
    bf16_t* xs = L.stage;
    const int ldxs = d + 8;
    bit_stage_final_norm<4>(xs, ldxs, xf, m.final_norm, m.eps, B, d);
    __syncthreads();
    lm_phase(lm, lpre, xs, ldxs, B, best_v, best_i, pf);
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
#define OHARA_BIT_BAR_WORDS(nwg) ((((nwg) + OHARA_BAR_GROUP - 1) / OHARA_BAR_GROUP + 12) * 64)

size_t bit_al(size_t v) { return (v + 255) & ~(size_t)255; }

struct BitLayout {
  size_t layers, xm, qm, am, pm, dm, ds, cq, cs, candv, candi, prof, bar, total;
  size_t xm_stride, qm_stride, am_stride, pm_stride, dm_stride, cq_stride;
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
  L.ds = o; o += bit_al((size_t)NL * 32 * sizeof(float));
  {  // batch > 1: code rows of the seven BitLinears (K padded to 256 columns + 16), B rows each; {s, sum q} pairs
    const int ldq_d = (((m->d_model + 255) >> 8) << 8) + 16, ldq_o = (((hd + 255) >> 8) << 8) + 16;
    const int ldq_f = (((m->d_ff + 255) >> 8) << 8) + 16;
    const size_t o_ = bit_cq_al((size_t)3 * B * ldq_d), g_ = bit_cq_al(o_ + (size_t)B * ldq_o), dn_ = bit_cq_al(g_ + (size_t)2 * B * ldq_d);
    L.cq_stride = B > 1 ? bit_cq_al(dn_ + (size_t)B * ldq_f) : 0;
  }
  L.cq = o; o += L.cq_stride * NL;
  L.cs = o; o += bit_al((size_t)NL * 256 * sizeof(float));
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
  const size_t stage = (size_t)B * (dmax + 8) * 2;
  size_t o = ((codes + 255) & ~(size_t)255) + ((stage + 255) & ~(size_t)255) + 4096 + 256 + 64;
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

int64_t ohara_bitnet_persistent_profile_offset(const OharaBitModel* m, int batch, int n_workgroups) {
  if (!m || batch < 1 || n_workgroups < 1) return OHARA_EINVAL;
  return (int64_t)bit_layout(m, batch, n_workgroups).prof;
}

int ohara_bitnet_decode_persistent(const OharaBitModel* m, const OharaDecodeState* s, void* workspace, int n_workgroups,
                                   int init_workspace, int select_greedy, unsigned int spin_limit, void* stream) {
  if (!m || !s || !workspace || !m->layers || !s->kcache || !s->vcache || !s->step_state) return OHARA_EINVAL;
  if (s->batch < 1 || s->batch > 8) return OHARA_ESIZE;
  if (n_workgroups < 4 || n_workgroups > 1024) return OHARA_EINVAL;
  if (s->n_split != OHARA_MEGA_NS) return OHARA_EINVAL;
  const int D = m->head_dim;
  if (m->n_kv_heads < 1 || m->n_heads % m->n_kv_heads) return OHARA_EINVAL;
  const int G = m->n_heads / m->n_kv_heads;
  if (!(D == 128 || D == 64) || G != 1) return OHARA_ESIZE;
  if ((m->d_model & 15) || (m->d_ff & 15) || m->d_model > 2048 || m->n_heads * D > 2048 || m->d_ff > 6144) return OHARA_ESIZE;
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
  a.cq = reinterpret_cast<int8_t*>(ws + L.cq); a.cs = reinterpret_cast<float*>(ws + L.cs); a.cq_stride = L.cq_stride;
  a.blk_x = L.blk_x; a.blk_a = L.blk_a;
  a.cand_val = reinterpret_cast<float*>(ws + L.candv);
  a.cand_idx = reinterpret_cast<int*>(ws + L.candi);
  a.bar = reinterpret_cast<unsigned int*>(ws + L.bar);
  a.B = s->batch; a.valid_vocab = s->valid_vocab; a.hist_cap = s->hist_cap;
  a.select = select_greedy;
  a.ids = s->ids; a.logits = s->logits;
  a.step_state = s->step_state; a.history = s->history;
  a.prof = (s->prof_kernel == -2 && 30 * m->n_layers + 16 <= 1024) ? reinterpret_cast<unsigned long long*>(ws + L.prof) : nullptr;
  a.spin_limit = spin_limit ? spin_limit : (1u << 19);
  int ns = n_workgroups / (s->batch * m->n_kv_heads);
  ns = ns < 1 ? 1 : (ns > OHARA_MEGA_NS ? OHARA_MEGA_NS : ns);
  while (ns & (ns - 1)) ns &= ns - 1;
  a.ns = ns;
  const size_t smem = bit_smem_bytes(m, s->batch, ns);
  if (smem > 160 * 1024) return OHARA_ESIZE;
  dim3 grid(n_workgroups), block(256);
#define OHARA_BITMEGA_B(DD, ONE_)                                                                            \
  do {                                                                                                       \
    if (smem > 64 * 1024)                                                                                    \
      (void)hipFuncSetAttribute((const void*)bitnet_mega_kernel<DD, 1, ONE_>,                                \
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);                      \
    static ResidencySlot slot;                                                                               \
    if (!ohara_grid_fits(slot, (const void*)bitnet_mega_kernel<DD, 1, ONE_>, smem, n_workgroups))            \
      return OHARA_ESIZE; /* the workgroups could not all be resident: the grid barrier would expire */      \
    hipLaunchKernelGGL((bitnet_mega_kernel<DD, 1, ONE_>), grid, block, smem, st, a);                         \
  } while (0)
#define OHARA_BITMEGA(DD)                                                                                    \
  do {                                                                                                       \
    if (s->batch == 1) OHARA_BITMEGA_B(DD, true);                                                            \
    else OHARA_BITMEGA_B(DD, false);                                                                         \
  } while (0)
#define OHARA_BITMEGA_PROF(ONE_)                                                                             \
  do {                                                                                                       \
    if (smem > 64 * 1024)                                                                                    \
      (void)hipFuncSetAttribute((const void*)bitnet_mega_kernel<128, 1, ONE_, true>,                         \
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);                      \
    static ResidencySlot slot;                                                                               \
    if (!ohara_grid_fits(slot, (const void*)bitnet_mega_kernel<128, 1, ONE_, true>, smem, n_workgroups))     \
      return OHARA_ESIZE;                                                                                    \
    hipLaunchKernelGGL((bitnet_mega_kernel<128, 1, ONE_, true>), grid, block, smem, st, a);                  \
  } while (0)
  if (a.prof && D == 128) {  // the stamps exist in these two instantiations only
    if (s->batch == 1) OHARA_BITMEGA_PROF(true);
    else OHARA_BITMEGA_PROF(false);
  } else if (D == 128) OHARA_BITMEGA(128);
  else OHARA_BITMEGA(64);
#undef OHARA_BITMEGA
#undef OHARA_BITMEGA_B
#undef OHARA_BITMEGA_PROF
  return ohara_launch_status();
}

}  // extern "C"
