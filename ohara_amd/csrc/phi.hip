// Phi's side of the KV-cache decode path (ohara/models/phi.py): what differs from Llama.
//   LayerNorm with bias                     phi.py:132, :160 (nn.LayerNorm: fp32 statistics, one rounding)
//   append of the UN-rotated key / value    phi.py:95 (kv_cache.py:104-105)
//   attention in fp32 with the partial half-split rotation applied after the cache read
//                                           phi.py:98-117, rotary.py:131-184
// The projections with bias, new_gelu and the parallel-block sum are epilogues of the skinny
// GEMM (gemm_epilogue.h).
#include "common.h"

namespace {

// ---- LayerNorm: one workgroup per row ---------------------------------------------------
__global__ __launch_bounds__(256) void layernorm_kernel(const bf16_t* x, int ldx, const bf16_t* w, const bf16_t* b,
                                                        bf16_t* out, int ldo, int d, float eps) {
  __shared__ float red[2][4];
  const int row = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const bf16_t* xr = x + (size_t)row * ldx;
  // pass 1: mean
  float s = 0.f;
  for (int k = tid * 8; k < d; k += 256 * 8) {
    const uint4 v = ldg16(xr + k);
    const uint32_t u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) s += lo_bf(u[i]) + hi_bf(u[i]);
  }
  s = wave_sum(s);
  if (lane == 0) red[0][wave] = s;
  __syncthreads();
  const float mean = (((red[0][0] + red[0][1]) + red[0][2]) + red[0][3]) / (float)d;
  // pass 2: biased variance around the mean (the row is re-read from cache)
  float q = 0.f;
  for (int k = tid * 8; k < d; k += 256 * 8) {
    const uint4 v = ldg16(xr + k);
    const uint32_t u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float a0 = lo_bf(u[i]) - mean, a1 = hi_bf(u[i]) - mean;
      q += a0 * a0 + a1 * a1;
    }
  }
  q = wave_sum(q);
  if (lane == 0) red[1][wave] = q;
  __syncthreads();
  const float var = (((red[1][0] + red[1][1]) + red[1][2]) + red[1][3]) / (float)d;
  const float rstd = 1.0f / sqrtf(var + eps);
  for (int k = tid * 8; k < d; k += 256 * 8) {
    const uint4 v = ldg16(xr + k), g = ldg16(w + k), c = ldg16(b + k);
    const uint32_t u[4] = {v.x, v.y, v.z, v.w}, gu[4] = {g.x, g.y, g.z, g.w}, cu[4] = {c.x, c.y, c.z, c.w};
    uint32_t o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
      o[i] = pack_bf((lo_bf(u[i]) - mean) * rstd * lo_bf(gu[i]) + lo_bf(cu[i]),
                     (hi_bf(u[i]) - mean) * rstd * hi_bf(gu[i]) + hi_bf(cu[i]));
    *reinterpret_cast<uint4*>(out + (size_t)row * ldo + k) = make_uint4(o[0], o[1], o[2], o[3]);
  }
}

// ---- append: rows (seq, s) of k and v -> cache position pos + s ------------------------------
__global__ void kv_append_kernel(const bf16_t* k, const bf16_t* v, int ld, int rows, int S, int hd, int t_max, int pos,
                                 const int32_t* pos_dev, bf16_t* kc, bf16_t* vc) {
  const int n8 = hd >> 3;
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= rows * n8) return;
  const int row = idx / n8, c = (idx - row * n8) * 8;
  const int seq = row / S, t = (pos_dev ? *pos_dev : pos) + (row - seq * S);
  if (t < 0 || t >= t_max) return;
  const size_t dst = ((size_t)seq * t_max + t) * hd + c;
  *reinterpret_cast<uint4*>(kc + dst) = ldg16(k + (size_t)row * ld + c);
  *reinterpret_cast<uint4*>(vc + dst) = ldg16(v + (size_t)row * ld + c);
}

// ---- attention ---------------------------------------------------------------------------
// One workgroup per (sequence, head, new token) and context chunk.  Sixteen lanes own one cached
// position at a time (lane l the eight features 8l .. 8l+7) and fetch two positions per round before
// using either (four measured slower: 178 registers halve the occupancy), so a workgroup walks 32
// positions per round with an online softmax per 16-lane group;
// the groups are merged through LDS at the end.  With several chunks (decode: few queries, long
// context) every chunk leaves {weighted sum, max, sum} and the workgroup that finishes last combines
// them in chunk order.
//
// The reference rotates every cached key again at each step (phi.py:104).  With the rotated query
// qr and c, s the cosine / sine of key position t the score is
//   sum_i (k1_i c_i - k2_i s_i) qr1_i + (k1_i s_i + k2_i c_i) qr2_i + sum_rest k_j q_j
//     = sum_i k1_i (c_i qr1_i + s_i qr2_i) + k2_i (c_i qr2_i - s_i qr1_i) + sum_rest k_j q_j,
// i.e. a dot product of the raw key row with a per-position weight vector built from two per-lane
// constants A, B: w_j = c A_j + s B_j.  All of it in fp32, as the reference (phi.py:98-100).
struct PhiAttnArgs {
  const bf16_t* q;
  int ldq;
  const bf16_t* kc;
  const bf16_t* vc;
  const float* cos;  // (t_max, rot/2) fp32
  const float* sin;
  bf16_t* out;       // (rows, H*D)
  int S, H, D, rot, t_max, pos;
  const int32_t* pos_dev;
  int ns;         // context chunks (decode): chunk c of a (sequence, head) is blockIdx.y
  float* ws;      // ns > 1: per (row, head, chunk) D + 2 floats {weighted sum[D], max, sum}
  int* counters;  // ns > 1: per (row, head) chunks finished; zero between calls
};

#ifndef PHI_ATTN_R
#define PHI_ATTN_R 2
#endif
__global__ __launch_bounds__(256) void phi_attn_kernel(PhiAttnArgs a) {
  __shared__ float qr[128];
  __shared__ float gm[16], gl[16];
  __shared__ float gacc[16][128];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int grp = wave * 4 + (lane >> 4), l = lane & 15;
  const int D = a.D, half = a.rot >> 1;
  // The cache is position-major: the heads of one position lie side by side, 2 * D bytes each, so the rows of
  // neighbouring heads share 128-byte lines.  Workgroups are handed to the eight XCDs in turn, each with an L2 of
  // its own: taken as launched, neighbouring heads would land on different XCDs and every L2 would fetch the
  // shared lines again.  So the launch order is re-read: XCD x works through the x-th eighth of the (chunk,
  // sequence, head) list, heads fastest.  (Any bijection is correct; this one needs a workgroup count that is a
  // multiple of 8, otherwise the order stays as launched.)
  int bx = blockIdx.x, by = blockIdx.y;
  {
    const int n = gridDim.x * gridDim.y;
    if ((n & 7) == 0) {
      const int id = by * gridDim.x + bx;
      const int lid = (id & 7) * (n >> 3) + (id >> 3);
      bx = lid % gridDim.x;
      by = lid / gridDim.x;
    }
  }
  int w = bx;
  const int s = w % a.S; w /= a.S;
  const int h = w % a.H;
  const int seq = w / a.H;
  const int row = seq * a.S + s;
  const int pq = (a.pos_dev ? *a.pos_dev : a.pos) + s;  // position of this query; keys 0 .. pq are visible
  if (pq < 0 || pq >= a.t_max) return;

  if (tid < D) {
    const bf16_t* qrow = a.q + (size_t)row * a.ldq + h * D;
    float v = bf2f(qrow[tid]);
    if (tid < half) {
      const float c = a.cos[(size_t)pq * half + tid], sn = a.sin[(size_t)pq * half + tid];
      v = v * c - bf2f(qrow[tid + half]) * sn;
    } else if (tid < a.rot) {
      const int i = tid - half;
      const float c = a.cos[(size_t)pq * half + i], sn = a.sin[(size_t)pq * half + i];
      v = bf2f(qrow[i]) * sn + v * c;
    }
    qr[tid] = v;
  }
  __syncthreads();

  const int e0 = 8 * l;
  const bool own = e0 < D;
  float A[8], Bc[8];
  int f[8];
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    const int j = e0 + u;
    A[u] = own ? qr[j] : 0.f;
    Bc[u] = 0.f;
    f[u] = -1;
    if (own && j < half) {
      Bc[u] = qr[j + half];
      f[u] = j;
    } else if (own && j < a.rot) {
      Bc[u] = -qr[j - half];
      f[u] = j - half;
    }
  }
  const bool rotates = own && e0 < a.rot;
  const bool vec8 = (half & 7) == 0;  // then rot % 16 == 0 and a lane's features are all rotated or all not
  const uint4 one4 = make_uint4(0x3f800000u, 0x3f800000u, 0x3f800000u, 0x3f800000u), zero4 = make_uint4(0, 0, 0, 0);
  const float scale = sqrtf(1.0f / (float)D);

  float m = -INFINITY, lsum = 0.f, acc[8];
#pragma unroll
  for (int u = 0; u < 8; ++u) acc[u] = 0.f;
  const size_t hd = (size_t)a.H * D;
  // Lanes beyond the head (own == false) read the head's first features instead: their weights A / Bc are
  // zero, so what they read only has to be mapped memory.
  const int e0c = own ? e0 : 0;
  const bf16_t* kb = a.kc + (size_t)seq * a.t_max * hd + (size_t)h * D + e0c;
  const bf16_t* vb = a.vc + (size_t)seq * a.t_max * hd + (size_t)h * D + e0c;
  // this workgroup's positions [t_lo, t_hi]
  int t_lo = 0, t_hi = pq;
  if (a.ns > 1) {
    const int per = ((pq + a.ns) / a.ns + 15) & ~15;  // ceil((pq + 1) / ns) rounded up to whole rounds
    t_lo = by * per;
    t_hi = min(pq, t_lo + per - 1);
  }
  constexpr int R = PHI_ATTN_R;  // positions a lane group has in flight per round
  const int fc = rotates ? f[0] : 0;
  for (int t = t_lo + grp; t <= t_hi; t += 16 * R) {
    // every load of the round is issued whatever its position (clamped to the chunk's last one): one run
    // of loads without branches; a position past the end is skipped when the round is consumed
    uint4 kv[R], vv[R];
    float cs[R][8], sn[R][8];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int tt = min(t + 16 * r, t_hi);
      kv[r] = ldg16(kb + (size_t)tt * hd);
      vv[r] = ldg16(vb + (size_t)tt * hd);
      if (vec8) {
        // the lane's eight features lie in one half: their angles are eight adjacent table entries
        const float* cp = a.cos + (size_t)tt * half + fc;
        const float* sp = a.sin + (size_t)tt * half + fc;
        const uint4 c0 = ldg16(cp), c1 = ldg16(cp + 4), s0 = ldg16(sp), s1 = ldg16(sp + 4);
        const uint32_t cu[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
        const uint32_t su[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          cs[r][u] = __uint_as_float(cu[u]);
          sn[r][u] = __uint_as_float(su[u]);
        }
      } else {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const bool rot_u = rotates && f[u] >= 0;
          cs[r][u] = rot_u ? a.cos[(size_t)tt * half + f[u]] : 1.0f;
          sn[r][u] = rot_u ? a.sin[(size_t)tt * half + f[u]] : 0.0f;
        }
      }
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      if (t + 16 * r > t_hi) break;  // uniform within the 16-lane group
      const uint32_t ku[4] = {kv[r].x, kv[r].y, kv[r].z, kv[r].w};
      float part = 0.f;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float c0 = (vec8 && !rotates) ? 1.0f : cs[r][2 * i], s0 = (vec8 && !rotates) ? 0.0f : sn[r][2 * i];
        const float c1 = (vec8 && !rotates) ? 1.0f : cs[r][2 * i + 1], s1 = (vec8 && !rotates) ? 0.0f : sn[r][2 * i + 1];
        part += lo_bf(ku[i]) * (c0 * A[2 * i] + s0 * Bc[2 * i]);
        part += hi_bf(ku[i]) * (c1 * A[2 * i + 1] + s1 * Bc[2 * i + 1]);
      }
      part = lane_xor_sum<8>(lane_xor_sum<4>(lane_xor_sum<2>(lane_xor_sum<1>(part))));
      const float sc = part * scale;
      const float mn = fmaxf(m, sc);
      // hardware exponential: its error (about 1e-6 relative) is far below the bf16 rounding of the output
      const float corr = __expf(m - mn), p = __expf(sc - mn);  // m = -inf on the first round: corr = 0
      lsum = lsum * corr + p;
      const uint32_t vu[4] = {vv[r].x, vv[r].y, vv[r].z, vv[r].w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc[2 * i] = acc[2 * i] * corr + p * lo_bf(vu[i]);
        acc[2 * i + 1] = acc[2 * i + 1] * corr + p * hi_bf(vu[i]);
      }
      m = mn;
    }
  }
  if (l == 0) {
    gm[grp] = m;
    gl[grp] = lsum;
  }
  if (own) {
#pragma unroll
    for (int u = 0; u < 8; ++u) gacc[grp][e0 + u] = acc[u];
  }
  __syncthreads();
  if (tid < D) {
    float M = -INFINITY;
#pragma unroll
    for (int g = 0; g < 16; ++g) M = fmaxf(M, gm[g]);
    float num = 0.f, den = 0.f;
#pragma unroll
    for (int g = 0; g < 16; ++g) {
      if (gm[g] == -INFINITY) continue;  // a group that saw no position
      const float wg = expf(gm[g] - M);
      num += wg * gacc[g][tid];
      den += wg * gl[g];
    }
    if (a.ns > 1) {
      // write-through stores: the workgroup that merges may sit on another XCD
      float* o = a.ws + (((size_t)row * a.H + h) * a.ns + by) * (D + 2);
      st_coh4(o + tid, __float_as_uint(num));
      if (tid == 0) {
        st_coh4(o + D, __float_as_uint(M));  // -inf: this chunk lies beyond the query's position
        st_coh4(o + D + 1, __float_as_uint(den));
      }
    } else {
      a.out[(size_t)row * hd + (size_t)h * D + tid] = f2bf(num / den);
    }
  }
  if (a.ns == 1) return;

  // The workgroup that finishes last merges the chunks of its (row, head), in chunk order.  Every
  // wave waits for its own write-through stores before the workgroup barrier; the counter is a
  // relaxed device-scope atomic; the merge reads with cache-bypassing loads.
  __shared__ int is_last;
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  wait_own_stores();
  __syncthreads();
  int* counter = a.counters + (size_t)row * a.H + h;
  if (tid == 0) {
    const int old = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    is_last = old == a.ns - 1;
    if (is_last) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next call
  }
  __syncthreads();
  if (!is_last) return;
  const float* p = a.ws + ((size_t)row * a.H + h) * a.ns * (D + 2);
  if (tid < a.ns) {  // ns <= 64: one round of loads for all (max, sum) pairs
    // qr and gacc are free again: chunk maxima and sums go there
    qr[tid] = __uint_as_float(ld_coh4(p + (size_t)tid * (D + 2) + D));
    gacc[0][tid] = __uint_as_float(ld_coh4(p + (size_t)tid * (D + 2) + D + 1));
  }
  __syncthreads();
  if (tid < D) {
    float M = -INFINITY;
    for (int c = 0; c < a.ns; ++c) M = fmaxf(M, qr[c]);
    float num = 0.f, den = 0.f;
    for (int c0 = 0; c0 < a.ns; c0 += 16) {  // sixteen chunks' values in flight, every load unconditional
      float av[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) av[i] = __uint_as_float(ld_coh4(p + (size_t)min(c0 + i, a.ns - 1) * (D + 2) + tid));
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        if (c0 + i >= a.ns || qr[c0 + i] == -INFINITY) continue;
        const float wg = expf(qr[c0 + i] - M);
        num += wg * av[i];
        den += wg * gacc[0][c0 + i];
      }
    }
    a.out[(size_t)row * hd + (size_t)h * D + tid] = f2bf(num / den);
  }
}

// ---- attention over many new tokens (prefill) -----------------------------------------------
// One workgroup per (sequence, head, 64 queries); each of its four waves owns 16 queries.  Keys
// and values go through LDS in tiles of 32 positions, as fp32, the keys rotated there once per
// tile; scores and the weighted sum are fp32 matrix products (v_mfma_f32_16x16x4_f32), the same
// arithmetic type the reference uses (phi.py:98-117).  Both products are formed transposed,
//   S^T (position x query) = K . Q^T        O^T (feature x query) = V^T . P^T,
// so that a lane's four score registers are rows 4g .. 4g+3 of one query column: the softmax
// runs down registers plus two cross-group shuffles, and register r is already the B operand of
// the second product's k-step r (the A operand then reads value row 4g + r).
constexpr int PF_Q = 64, PF_T = 32;

template <int DT>  // head width / 16
__global__ __launch_bounds__(256) void phi_attn_prefill_kernel(PhiAttnArgs a) {
  constexpr int D = 16 * DT, LD = D + 4, NV = (PF_T * (D / 8) + 255) / 256;
  __shared__ float sm[2 * PF_T * LD];  // keys | values of a tile; the rotated queries before the loop
  float* ks = sm;
  float* vs = sm + PF_T * LD;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l16 = lane & 15, g = lane >> 4;
  const int half = a.rot >> 1;
  const int h = blockIdx.y, seq = blockIdx.z;
  const int s0 = ((int)gridDim.x - 1 - (int)blockIdx.x) * PF_Q;  // long contexts first
  const size_t hd = (size_t)a.H * D;
  const int pos0 = a.pos;

  // rotated queries -> LDS -> registers (phi.py:103; rows beyond the call's tokens are zero)
  for (int idx = tid; idx < PF_Q * D; idx += 256) {
    const int qi = idx / D, j = idx - qi * D;
    const int sq = s0 + qi;
    float v = 0.f;
    if (sq < a.S) {
      const bf16_t* qrow = a.q + ((size_t)seq * a.S + sq) * a.ldq + h * D;
      const size_t cb = (size_t)(pos0 + sq) * half;
      v = bf2f(qrow[j]);
      if (j < half) v = v * a.cos[cb + j] - bf2f(qrow[j + half]) * a.sin[cb + j];
      else if (j < a.rot) v = bf2f(qrow[j - half]) * a.sin[cb + j - half] + v * a.cos[cb + j - half];
    }
    sm[qi * LD + j] = v;
  }
  __syncthreads();
  float qreg[D / 4];
#pragma unroll
  for (int kk = 0; kk < D / 4; ++kk) qreg[kk] = sm[(16 * wave + l16) * LD + 4 * kk + g];
  __syncthreads();

  // this lane's query column; columns beyond the call's tokens repeat the last one and are not stored
  const int sq = min(s0 + 16 * wave + l16, a.S - 1);
  const int pq = pos0 + sq;
  const int wave_hi = pos0 + min(s0 + 16 * wave + 15, a.S - 1);  // last position any query of the wave sees
  const int t_end = pos0 + min(s0 + PF_Q - 1, a.S - 1);
  const float scale = sqrtf(1.0f / (float)D);
  const bf16_t* kb = a.kc + (size_t)seq * a.t_max * hd + (size_t)h * D;
  const bf16_t* vb = a.vc + (size_t)seq * a.t_max * hd + (size_t)h * D;

  f32x4 o[DT];
#pragma unroll
  for (int t = 0; t < DT; ++t) o[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, lsum = 0.f;

  uint4 kr[NV], vr[NV];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int idx = tid + 256 * i;
      const int p = idx / (D / 8), c = idx - p * (D / 8);
      const bool in = idx < PF_T * (D / 8) && t0 + p <= t_end;
      kr[i] = in ? ldg16(kb + (size_t)(t0 + p) * hd + 8 * c) : make_uint4(0, 0, 0, 0);
      vr[i] = in ? ldg16(vb + (size_t)(t0 + p) * hd + 8 * c) : make_uint4(0, 0, 0, 0);
    }
  };
  auto put8 = [](float* dst, uint4 v) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      dst[2 * i] = lo_bf(w[i]);
      dst[2 * i + 1] = hi_bf(w[i]);
    }
  };

  fetch(0);
  for (int t0 = 0; t0 <= t_end; t0 += PF_T) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int idx = tid + 256 * i;
      if (idx < PF_T * (D / 8)) {
        const int p = idx / (D / 8), c = idx - p * (D / 8);
        put8(ks + p * LD + 8 * c, kr[i]);
        put8(vs + p * LD + 8 * c, vr[i]);
      }
    }
    __syncthreads();
    if (t0 + PF_T <= t_end) fetch(t0 + PF_T);  // in flight during this tile's products
    // rotate the tile's keys in place (phi.py:104): pair (i, i + half) of every position
    for (int idx = tid; idx < PF_T * half; idx += 256) {
      const int p = idx / half, i = idx - p * half;
      if (t0 + p <= t_end) {
        const float c = a.cos[(size_t)(t0 + p) * half + i], sn = a.sin[(size_t)(t0 + p) * half + i];
        const float k1 = ks[p * LD + i], k2 = ks[p * LD + i + half];
        ks[p * LD + i] = k1 * c - k2 * sn;
        ks[p * LD + i + half] = k1 * sn + k2 * c;
      }
    }
    __syncthreads();
#pragma unroll
    for (int blk = 0; blk < PF_T / 16; ++blk) {
      const int tb = t0 + 16 * blk;
      if (tb > wave_hi) break;  // wave-uniform: nothing in this block is visible to the wave's queries
      f32x4 sc = (f32x4){0.f, 0.f, 0.f, 0.f};
      const float* krow = ks + (16 * blk + l16) * LD + g;
#pragma unroll
      for (int kk = 0; kk < D / 4; ++kk) sc = __builtin_amdgcn_mfma_f32_16x16x4f32(krow[4 * kk], qreg[kk], sc, 0, 0, 0);
      float mx = -INFINITY;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        sc[r] = tb + 4 * g + r <= pq ? sc[r] * scale : -INFINITY;
        mx = fmaxf(mx, sc[r]);
      }
      mx = lane_xor_max<32>(lane_xor_max<16>(mx));
      const float mn = fmaxf(m, mx);  // finite: position 0 is in the first block and visible to every query
      const float corr = __expf(m - mn);
      float ps = 0.f;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        sc[r] = __expf(sc[r] - mn);
        ps += sc[r];
      }
      lsum = lsum * corr + ps;
      m = mn;
#pragma unroll
      for (int t = 0; t < DT; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) o[t][r] *= corr;
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        const float* vrow = vs + (16 * blk + 4 * g + kk) * LD + l16;
#pragma unroll
        for (int t = 0; t < DT; ++t) o[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(vrow[16 * t], sc[kk], o[t], 0, 0, 0);
      }
    }
    __syncthreads();
  }
  lsum = lane_xor_sum<32>(lane_xor_sum<16>(lsum));
  if (s0 + 16 * wave + l16 < a.S) {
    const float inv = 1.0f / lsum;
    bf16_t* orow = a.out + ((size_t)seq * a.S + sq) * hd + (size_t)h * D + 4 * g;
#pragma unroll
    for (int t = 0; t < DT; ++t)
      *reinterpret_cast<uint2*>(orow + 16 * t) =
          make_uint2(pack_bf(o[t][0] * inv, o[t][1] * inv), pack_bf(o[t][2] * inv, o[t][3] * inv));
  }
}

}  // namespace

extern "C" {

int ohara_layernorm_bf16(const uint16_t* x, int ldx, const uint16_t* weight, const uint16_t* bias, uint16_t* out, int ldo,
                         int rows, int d, float eps, void* stream) {
  if (!x || !weight || !bias || !out || rows < 1 || d < 8) return OHARA_EINVAL;
  if ((d & 7) || (ldx & 7) || (ldo & 7) || ldx < d || ldo < d) return OHARA_EINVAL;
  hipLaunchKernelGGL(layernorm_kernel, dim3(rows), dim3(256), 0, (hipStream_t)stream, x, ldx, weight, bias, out, ldo, d,
                     eps);
  return ohara_launch_status();
}

int ohara_kv_append_bf16(const uint16_t* k, const uint16_t* v, int ld, int batch, int seq_len, int h, int dh, int pos,
                         const int32_t* pos_dev, uint16_t* kcache, uint16_t* vcache, int t_max, void* stream) {
  if (!k || !v || !kcache || !vcache || batch < 1 || seq_len < 1 || h < 1 || dh < 1 || t_max < 1) return OHARA_EINVAL;
  const int64_t hd = (int64_t)h * dh;
  if ((hd & 7) || (ld & 7) || ld < hd) return OHARA_EINVAL;
  if (!pos_dev && (pos < 0 || pos + seq_len > t_max)) return OHARA_EINVAL;
  if (pos_dev && seq_len != 1) return OHARA_EINVAL;
  const int64_t total = (int64_t)batch * seq_len * (hd >> 3);
  if (total > INT32_MAX) return OHARA_ESIZE;
  hipLaunchKernelGGL(kv_append_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, (hipStream_t)stream, k, v, ld,
                     batch * seq_len, seq_len, (int)hd, t_max, pos, pos_dev, kcache, vcache);
  return ohara_launch_status();
}

int64_t ohara_phi_attn_workspace_bytes(int batch, int h, int dh, int n_split) {
  if (batch < 1 || h < 1 || dh < 1 || n_split < 1) return OHARA_EINVAL;
  const int64_t counters = (((int64_t)batch * h * (int64_t)sizeof(int)) + 255) & ~(int64_t)255;
  return counters + (int64_t)batch * h * n_split * (dh + 2) * (int64_t)sizeof(float);
}

int ohara_phi_attn_bf16(const uint16_t* q, int ldq, const uint16_t* kcache, const uint16_t* vcache, const float* cos,
                        const float* sin, int rot, int batch, int seq_len, int h, int dh, int t_max, int pos,
                        const int32_t* pos_dev, int n_split, void* workspace, uint16_t* out, void* stream) {
  if (!q || !kcache || !vcache || !cos || !sin || !out) return OHARA_EINVAL;
  if (batch < 1 || seq_len < 1 || h < 1 || t_max < 1) return OHARA_EINVAL;
  if (dh < 8 || dh > 128 || (dh & 7)) return OHARA_ESIZE;
  if (rot < 2 || (rot & 1) || rot > dh) return OHARA_EINVAL;  // rotary.py:118-121
  if (ldq < h * dh) return OHARA_EINVAL;
  if (!pos_dev && (pos < 0 || pos + seq_len > t_max)) return OHARA_EINVAL;
  if (pos_dev && seq_len != 1) return OHARA_EINVAL;
  if (n_split < 1 || n_split > 64 || (n_split > 1 && (!workspace || seq_len != 1))) return OHARA_EINVAL;
  const int64_t grid = (int64_t)batch * seq_len * h;
  if (grid > INT32_MAX) return OHARA_ESIZE;
  const size_t counters = (((size_t)batch * h * sizeof(int)) + 255) & ~(size_t)255;
  PhiAttnArgs a{q, ldq, kcache, vcache, cos, sin, out, seq_len, h, dh, rot, t_max, pos, pos_dev, n_split,
                reinterpret_cast<float*>(reinterpret_cast<char*>(workspace) + counters), reinterpret_cast<int*>(workspace)};
  if (seq_len >= 16 && !pos_dev && (dh == 16 || dh == 32 || dh == 64 || dh == 80 || dh == 128) && h <= 65535 &&
      batch <= 65535) {
    // many new tokens: queries in tiles of 64 against key / value tiles in LDS, fp32 matrix products
    const dim3 pgrid((unsigned)((seq_len + PF_Q - 1) / PF_Q), (unsigned)h, (unsigned)batch);
    switch (dh / 16) {
      case 1: hipLaunchKernelGGL((phi_attn_prefill_kernel<1>), pgrid, dim3(256), 0, (hipStream_t)stream, a); break;
      case 2: hipLaunchKernelGGL((phi_attn_prefill_kernel<2>), pgrid, dim3(256), 0, (hipStream_t)stream, a); break;
      case 4: hipLaunchKernelGGL((phi_attn_prefill_kernel<4>), pgrid, dim3(256), 0, (hipStream_t)stream, a); break;
      case 5: hipLaunchKernelGGL((phi_attn_prefill_kernel<5>), pgrid, dim3(256), 0, (hipStream_t)stream, a); break;
      default: hipLaunchKernelGGL((phi_attn_prefill_kernel<8>), pgrid, dim3(256), 0, (hipStream_t)stream, a); break;
    }
    return ohara_launch_status();
  }
  hipLaunchKernelGGL(phi_attn_kernel, dim3((unsigned)grid, (unsigned)n_split), dim3(256), 0, (hipStream_t)stream, a);
  return ohara_launch_status();
}

}  // extern "C"
