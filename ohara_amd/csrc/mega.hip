// Persistent decode kernel: one launch computes a whole decode step (one new token per
// sequence, batch <= 16) of the Llama of ohara/models/llama.py:279-323.
//
// Why: at batch 1 a layer streams only ~19 MB, so a chain of five kernels per layer
// spends its time in launch and drain latency, not in HBM.  Here the whole chip stays
// resident (one workgroup per CU) and walks the same five phases per layer, separated by
// a grid-wide barrier (a device-scope counter), each phase spreading its work over all
// workgroups:
//   P1  [embedding] + norm1 + QKV projection + rotary + cache append
//   P2  attention over the cache, split along the context, partial (max,sum,acc) triples
//   P3  merge of the partials + output projection + residual
//   P4  norm2 + gate/up projection + SwiGLU
//   P5  down projection + residual
// then final norm + vocabulary projection with a running arg-max per workgroup, and the
// selection of the next token.  Rounding points are those of the unfused kernels.
//
// Every barrier wait is bounded: a workgroup that spins longer than the limit raises the
// error flag and moves on, so the grid always drains.
#include "common.h"

namespace {

struct MegaArgs {
  OharaModel m;                 // by value; the layer table is read from layers_dev
  const OharaLayer* layers_dev;
  uint16_t* const* kcache_dev;  // device arrays [n_layers]
  uint16_t* const* vcache_dev;
  int B, nsplit, valid_vocab, hist_cap, select;
  int64_t* ids;
  bf16_t* x;       // (B, d) residual stream                    } "mailbox" buffers: written by
  bf16_t* q;       // (B, H*Dh)                                 } one phase, read by a later one
  bf16_t* act;     // (B, F)                                    } on other CUs/XCDs; accessed
  float* part_ml;  // (B, H, nsplit, 2)                         } only through the coherent
  float* part_acc; // (B, H, nsplit, Dh)                        } helpers below
  float* cand_val; // (nwg, B)
  int* cand_idx;   // (nwg, B)
  bf16_t* logits;  // (B, V)
  int32_t* step_state;  // {pos, step, done, pad}
  int64_t* history;
  unsigned int* bar;    // barrier words, see GridSync
  unsigned long long* prof;  // optional: clock of workgroup 0 at every phase boundary
  unsigned int spin_limit;
};

// ---------------------------------------------------------------------------------------
// Cross-workgroup data goes through device-scope (sc1) loads and stores: each access is
// coherent across the XCDs' L2s by itself, so the barrier needs no L2 write-back or
// invalidate (those cost ~1.7 us each on this chip, more than the barrier).  A producer
// waits for its stores to complete (workgroup release = s_waitcnt vmcnt(0)) before it
// arrives at the barrier.
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ uint2 ld_coh8(const void* p) {
  const unsigned long long v =
      __hip_atomic_load(reinterpret_cast<const unsigned long long*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return make_uint2((uint32_t)v, (uint32_t)(v >> 32));
}
__device__ __forceinline__ void st_coh8(void* p, uint2 v) {
  __hip_atomic_store(reinterpret_cast<unsigned long long*>(p), ((unsigned long long)v.y << 32) | v.x,
                     __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t ld_coh4(const void* p) {
  return __hip_atomic_load(reinterpret_cast<const uint32_t*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_coh4(void* p, uint32_t v) {
  __hip_atomic_store(reinterpret_cast<uint32_t*>(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float ld_cohf(const float* p) { return __uint_as_float(ld_coh4(p)); }
__device__ __forceinline__ void st_cohf(float* p, float v) { st_coh4(p, __float_as_uint(v)); }
__device__ __forceinline__ uint4 ld_coh16(const void* p) {
  const uint2 a = ld_coh8(p), b = ld_coh8(reinterpret_cast<const char*>(p) + 8);
  return make_uint4(a.x, a.y, b.x, b.y);
}

// ---------------------------------------------------------------------------------------
// Grid barrier.  Two levels of monotonic counters (groups of 16 workgroups, each counter on
// its own 256-byte line, then one counter over the groups) and a release word everyone
// polls; a flat counter serialises 256 read-modify-writes on one address (~11 us here),
// this takes ~1.6 us.  Words (uint32, stride 64 per counter): [g*64] group g, [ng*64] top,
// [(ng+1)*64] release, [(ng+2)*64] sticky error, [(ng+3)*64] barriers completed by earlier
// launches.  Every wait is bounded; an expired wait raises the error word, after which all
// waits return at once and the grid drains.
// ---------------------------------------------------------------------------------------
#define OHARA_BAR_GROUP 16
struct GridSync {
  unsigned int* gc;
  unsigned int* top;
  unsigned int* rel;
  unsigned int* err;
  unsigned int* done;
  unsigned int k;      // index of the next barrier (1-based, across launches)
  unsigned int gsize;  // workgroups in my group
  unsigned int ng;
  unsigned int limit;
  __device__ void init(unsigned int* bar, unsigned int nwg, unsigned int lim) {
    ng = (nwg + OHARA_BAR_GROUP - 1) / OHARA_BAR_GROUP;
    const unsigned int g = blockIdx.x / OHARA_BAR_GROUP;
    gsize = min((unsigned int)OHARA_BAR_GROUP, nwg - g * OHARA_BAR_GROUP);
    gc = bar + g * 64;
    top = bar + ng * 64;
    rel = bar + (ng + 1) * 64;
    err = bar + (ng + 2) * 64;
    done = bar + (ng + 3) * 64;
    limit = lim;
    k = *done + 1;  // written by the previous launch (or the host): plain load
  }
  __device__ void sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");  // my coherent stores have completed
    __syncthreads();
    if (threadIdx.x == 0) {
      const unsigned int a = __hip_atomic_fetch_add(gc, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1;
      if (a == k * gsize) {
        const unsigned int t = __hip_atomic_fetch_add(top, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1;
        if (t == k * ng) __hip_atomic_store(rel, k, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      unsigned int spins = 0;
      while ((int)(__hip_atomic_load(rel, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - k) < 0) {
        ++spins;
        if (spins > limit) {
          __hip_atomic_store(err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          break;
        }
        if ((spins & 63u) == 0 && __hip_atomic_load(err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) break;
        __builtin_amdgcn_s_sleep(1);
      }
    }
    __syncthreads();
    ++k;
  }
};

__device__ __forceinline__ float dot8m(uint4 a, uint4 b, float s) {
  s = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a.x), __builtin_bit_cast(bf16x2, b.x), s, false);
  s = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a.y), __builtin_bit_cast(bf16x2, b.y), s, false);
  s = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a.z), __builtin_bit_cast(bf16x2, b.z), s, false);
  s = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a.w), __builtin_bit_cast(bf16x2, b.w), s, false);
  return s;
}

// ---------------------------------------------------------------------------------------
// staging of the GEMM activations in LDS: xs[b][ldxs] bf16
// ---------------------------------------------------------------------------------------

// norm.py:16-21 on rows of the residual stream (mailbox `src`, (B, K)), or - for the first
// layer - on rows gathered from the embedding table (llama.py:310), which workgroup 0 also
// publishes as the residual stream.  One wave per row; all loads of a row are issued
// before any is consumed.  K <= 8 * 64 * NLD elements.
template <int NLD>
__device__ void stage_norm(bf16_t* xs, int ldxs, const bf16_t* src, const int64_t* ids, const bf16_t* table,
                           int vocab, bf16_t* x_out, const bf16_t* nw, float eps, int B, int K) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int b = wave; b < B; b += 4) {
    uint2 v[NLD * 2], g[NLD * 2];
    if (ids) {
      int64_t id = ids[b];
      if (id < 0 || id >= vocab) id = 0;
      const bf16_t* row = table + (size_t)id * K;
#pragma unroll
      for (int c = 0; c < NLD * 2; ++c) {
        const int k = (c * 64 + lane) * 4;
        v[c] = k < K ? *reinterpret_cast<const uint2*>(row + k) : make_uint2(0, 0);
      }
    } else {
      const bf16_t* row = src + (size_t)b * K;
#pragma unroll
      for (int c = 0; c < NLD * 2; ++c) {
        const int k = (c * 64 + lane) * 4;
        v[c] = k < K ? ld_coh8(row + k) : make_uint2(0, 0);
      }
    }
#pragma unroll
    for (int c = 0; c < NLD * 2; ++c) {
      const int k = (c * 64 + lane) * 4;
      g[c] = k < K ? *reinterpret_cast<const uint2*>(nw + k) : make_uint2(0, 0);
    }
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < NLD * 2; ++c) {
      const float a0 = lo_bf(v[c].x), a1 = hi_bf(v[c].x), a2 = lo_bf(v[c].y), a3 = hi_bf(v[c].y);
      ss += (a0 * a0 + a1 * a1) + (a2 * a2 + a3 * a3);
    }
    ss = wave_sum(ss);
    const float rinv = 1.0f / sqrtf(ss / (float)K + eps);
#pragma unroll
    for (int c = 0; c < NLD * 2; ++c) {
      const int k = (c * 64 + lane) * 4;
      if (k < K) {
        const uint2 o = make_uint2(
            pack_bf(rbf(lo_bf(v[c].x) * rinv) * lo_bf(g[c].x), rbf(hi_bf(v[c].x) * rinv) * hi_bf(g[c].x)),
            pack_bf(rbf(lo_bf(v[c].y) * rinv) * lo_bf(g[c].y), rbf(hi_bf(v[c].y) * rinv) * hi_bf(g[c].y)));
        *reinterpret_cast<uint2*>(xs + (size_t)b * ldxs + k) = o;
        if (ids && x_out && blockIdx.x == 0) st_coh8(x_out + (size_t)b * K + k, v[c]);
      }
    }
  }
}

// Plain copy of a mailbox matrix (B, K) into LDS.
__device__ void stage_copy(bf16_t* xs, int ldxs, const bf16_t* src, int B, int K) {
  const int n4 = K >> 2;
  for (int i = threadIdx.x; i < B * n4; i += blockDim.x) {
    const int b = i / n4, k = (i - b * n4) << 2;
    *reinterpret_cast<uint2*>(xs + (size_t)b * ldxs + k) = ld_coh8(src + (size_t)b * K + k);
  }
}

// Merge of the attention partials of all chunks, in chunk order (llama.py:116-123 output,
// rounded to bf16 as SDPA's result is) -> xs[b][h*Dh + d].  A thread owns two adjacent
// columns; the (max, sum) pairs and the accumulators of all NS chunks are loaded before any
// is used.
template <int NS>
__device__ void stage_attn_merge(bf16_t* xs, int ldxs, const MegaArgs& a) {
  const int H = a.m.n_heads, Dh = a.m.head_dim;
  const int HD = H * Dh;
  for (int e = threadIdx.x * 2; e < a.B * HD; e += blockDim.x * 2) {
    const int b = e / HD, hd = e - b * HD;
    const int h = hd / Dh, d = hd - h * Dh;
    const float* ml = a.part_ml + ((size_t)(b * H + h) * NS) * 2;
    const float* pa = a.part_acc + ((size_t)(b * H + h) * NS) * Dh + d;
    uint2 mlv[NS], av[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      mlv[s] = ld_coh8(ml + 2 * s);
      av[s] = ld_coh8(pa + (size_t)s * Dh);
    }
    float M = -INFINITY;
#pragma unroll
    for (int s = 0; s < NS; ++s) M = fmaxf(M, __uint_as_float(mlv[s].x));
    float Ls = 0.f, o0 = 0.f, o1 = 0.f;
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      const float ms = __uint_as_float(mlv[s].x);
      const float w = (ms == -INFINITY) ? 0.f : __expf(ms - M);
      Ls += __uint_as_float(mlv[s].y) * w;
      o0 += __uint_as_float(av[s].x) * w;
      o1 += __uint_as_float(av[s].y) * w;
    }
    *reinterpret_cast<uint32_t*>(xs + (size_t)b * ldxs + hd) = pack_bf(o0 / Ls, o1 / Ls);
  }
}

// ---------------------------------------------------------------------------------------
// GEMM phase: strips of 16 packed rows, KP waves per strip, activations from LDS.  The
// weights of a workgroup's first strip(s) are fetched into registers BEFORE the barrier
// that precedes the phase (they do not depend on the activations), so the HBM stream runs
// under the barrier latency.
// ---------------------------------------------------------------------------------------
enum { E_RESID = 1, E_SWIGLU = 2, E_ROPE = 3, E_LOGITS = 4 };

struct GemmP {
  const uint4* wp;
  int N, K;        // logical rows (for E_SWIGLU: hidden width F) and columns
  int nstrips;
  bf16_t* out;     // mailbox output (E_ROPE: q; E_RESID: residual stream, read-modify-write)
  int ldo;
  int H, Hkv, Dh, Tmax, pos;
  const bf16_t* cos;
  const bf16_t* sin;
  bf16_t* kc;
  bf16_t* vc;
  int valid;       // E_LOGITS: ids >= valid never win
};

#define OHARA_MAX_PF 24
struct GemmPre {  // one register buffer, reused by every phase (only one prefetch is live at a time)
  uint4 w[OHARA_MAX_PF];
};

template <int KP, int PF>
__device__ __forceinline__ void gemm_prefetch(const GemmP& p, GemmPre& pre) {
  constexpr int SPW = 4 / KP;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int sub = wave / KP, kpart = wave % KP;
  const int KS = (p.K + 31) >> 5;
  const int per = (KS + KP - 1) / KP;
  const int j0 = kpart * per, j1 = min(KS, j0 + per);
  const int strip = (int)blockIdx.x * SPW + sub;
  const uint4* wrow = p.wp + (size_t)strip * KS * 64 + lane;
#pragma unroll
  for (int c = 0; c < PF; ++c)
    pre.w[c] = (strip < p.nstrips && j0 + c < j1) ? ldg16_nt(wrow + (size_t)(j0 + c) * 64) : make_uint4(0, 0, 0, 0);
}

template <int KP, int PF, int EPI>
__device__ __forceinline__ void gemm_phase(const GemmP& p, const GemmPre& pre, const bf16_t* xs, int ldxs, int B, float* red,
                           float& best_v, int& best_i) {
  constexpr int SPW = 4 / KP;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m = lane & 15, g = lane >> 4;
  const int sub = wave / KP, kpart = wave % KP;
  const int KS = (p.K + 31) >> 5;
  const int per = (KS + KP - 1) / KP;
  const int j0 = kpart * per, j1 = min(KS, j0 + per);
  const int nwg = gridDim.x;
  const int iters = (p.nstrips + nwg * SPW - 1) / (nwg * SPW);
  const bool mine = m < B;
  const bf16_t* xrow = xs + (size_t)m * ldxs + 8 * g;

#pragma unroll 1
  for (int it = 0; it < iters; ++it) {
    const int strip = (it * nwg + blockIdx.x) * SPW + sub;
    const bool live = strip < p.nstrips;
    f32x4 acc = (f32x4){0.f, 0.f, 0.f, 0.f};
    if (live) {
      const uint4* wrow = p.wp + (size_t)strip * KS * 64 + lane;
#pragma unroll 1
      for (int jc = j0; jc < j1; jc += PF) {
        uint4 wv[PF];
        if (it == 0 && jc == j0) {
#pragma unroll
          for (int c = 0; c < PF; ++c) wv[c] = pre.w[c];
        } else {
#pragma unroll
          for (int c = 0; c < PF; ++c)
            wv[c] = (jc + c < j1) ? ldg16_nt(wrow + (size_t)(jc + c) * 64) : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int c = 0; c < PF; ++c) {
          uint4 xv = make_uint4(0, 0, 0, 0);
          if (mine && jc + c < j1 && 32 * (jc + c) + 8 * g < p.K)
            xv = *reinterpret_cast<const uint4*>(xrow + 32 * (jc + c));
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wv[c]),
                                                        __builtin_bit_cast(bf16x8, xv), acc, 0, 0, 0);
        }
      }
    }
    if (KP > 1) {
      if (kpart > 0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) red[((wave * 64) + lane) * 4 + i] = acc[i];
      }
      __syncthreads();
      if (kpart == 0) {
#pragma unroll
        for (int w = 1; w < KP; ++w)
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[i] += red[(((wave + w) * 64) + lane) * 4 + i];
      }
    }
    if (live && kpart == 0 && mine) {
      const int b = m;
      const int r0 = strip * 16 + 4 * g;
      const float y0 = rbf(acc[0]), y1 = rbf(acc[1]), y2 = rbf(acc[2]), y3 = rbf(acc[3]);
      if (EPI == E_RESID) {  // N % 4 == 0 is required by the entry point
        if (r0 < p.N) {
          bf16_t* o = p.out + (size_t)b * p.ldo + r0;
          const uint2 r = ld_coh8(o);
          st_coh8(o, make_uint2(pack_bf(lo_bf(r.x) + y0, hi_bf(r.x) + y1), pack_bf(lo_bf(r.y) + y2, hi_bf(r.y) + y3)));
        }
      } else if (EPI == E_LOGITS) {
        const float v[4] = {y0, y1, y2, y3};
        bf16_t* o = p.out + (size_t)b * p.ldo + r0;
        if (r0 + 3 < p.N && ((p.ldo & 3) == 0)) {
          *reinterpret_cast<uint2*>(o) = make_uint2(pack_bf(v[0], v[1]), pack_bf(v[2], v[3]));
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (r0 + i < p.N) o[i] = f2bf(v[i]);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int id = r0 + i;
          if (id < p.valid && (v[i] > best_v || (v[i] == best_v && id < best_i))) {
            best_v = v[i];
            best_i = id;
          }
        }
      } else if (EPI == E_SWIGLU) {  // F % 8 == 0 is required by the entry point
        const int f = strip * 8 + 2 * g;
        if (f < p.N) {
          const float s0 = rbf(silu_f(y0)), s1 = rbf(silu_f(y1));
          st_coh4(p.out + (size_t)b * p.ldo + f, pack_bf(s0 * y2, s1 * y3));
        }
      } else {  // E_ROPE
        const int nq = p.H * p.Dh, nk = p.Hkv * p.Dh;
        if (r0 < nq + 2 * nk && p.pos >= 0 && p.pos < p.Tmax) {
          float v[4] = {y0, y1, y2, y3};
          bf16_t* o;
          if (r0 < nq + nk) {
            const int d = (r0 < nq ? r0 : r0 - nq) % p.Dh;
            const uint32_t cs = *reinterpret_cast<const uint32_t*>(p.cos + (size_t)p.pos * (p.Dh >> 1) + (d >> 1));
            const uint32_t sn = *reinterpret_cast<const uint32_t*>(p.sin + (size_t)p.pos * (p.Dh >> 1) + (d >> 1));
            const float c2[2] = {lo_bf(cs), hi_bf(cs)}, s2[2] = {lo_bf(sn), hi_bf(sn)};
#pragma unroll
            for (int pr = 0; pr < 2; ++pr) {
              const float e = v[2 * pr], od = v[2 * pr + 1];
              v[2 * pr] = __fsub_rn(__fmul_rn(e, c2[pr]), __fmul_rn(od, s2[pr]));
              v[2 * pr + 1] = __fadd_rn(__fmul_rn(e, s2[pr]), __fmul_rn(od, c2[pr]));
            }
            o = (r0 < nq) ? p.out + (size_t)b * p.ldo + r0
                          : p.kc + (((size_t)b * p.Tmax + p.pos) * p.Hkv) * p.Dh + (r0 - nq);
          } else {
            o = p.vc + (((size_t)b * p.Tmax + p.pos) * p.Hkv) * p.Dh + (r0 - nq - nk);
          }
          st_coh8(o, make_uint2(pack_bf(v[0], v[1]), pack_bf(v[2], v[3])));
        }
      }
    }
    if (KP > 1) __syncthreads();
  }
}

// ---------------------------------------------------------------------------------------
// attention phase: items (sequence, kv head, chunk); writes partial triples
// ---------------------------------------------------------------------------------------
template <int D, int G>
__device__ void attn_phase(const MegaArgs& a, const bf16_t* kc, const bf16_t* vc, int L, float* lds) {
  constexpr int NC = D / 32, DC = D / 8, PP = 64 / DC, NV = 16 / PP;
  const int H = a.m.n_heads, Hkv = a.m.n_kv_heads, Tmax = a.m.t_max, ns = a.nsplit;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int p = lane & 15, dq = lane >> 4;
  const int pp = lane / DC, dc = lane % DC;
  const float scale = 1.0f / sqrtf((float)D);
  float* s_m = lds;                 // [4][G]
  float* s_l = lds + 4 * G;         // [4][G]
  float* s_acc = lds + 8 * G;       // [4][G][D]
  const int chunk = (((L + ns - 1) / ns) + 15) & ~15;
  const int nitems = a.B * Hkv * ns;
  const size_t row = (size_t)Hkv * D;
  for (int item = blockIdx.x; item < nitems; item += gridDim.x) {
    const int split = item % ns;
    const int kvh = (item / ns) % Hkv;
    const int b = item / (ns * Hkv);
    const int t0 = split * chunk, t1 = min(L, t0 + chunk);
    const bf16_t* kb = kc + (size_t)b * Tmax * row + (size_t)kvh * D;
    const bf16_t* vb = vc + (size_t)b * Tmax * row + (size_t)kvh * D;
    float m_run[G], l_run[G], acc[G][8];
#pragma unroll
    for (int hh = 0; hh < G; ++hh) {
      m_run[hh] = -INFINITY;
      l_run[hh] = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[hh][i] = 0.f;
    }
    if (t0 + wave * 16 < t1) {
      uint4 qv[G][NC];
#pragma unroll
      for (int hh = 0; hh < G; ++hh)
#pragma unroll
        for (int c = 0; c < NC; ++c)
          qv[hh][c] = ld_coh16(a.q + (size_t)b * H * D + (size_t)(kvh * G + hh) * D + (4 * c + dq) * 8);
      for (int tb = t0 + wave * 16; tb < t1; tb += 64) {
        const int pos = tb + p;
        const bool valid = pos < t1;
        uint4 kv[NC], vv[NV];
#pragma unroll
        for (int c = 0; c < NC; ++c)
          kv[c] = valid ? ldg16_nt(kb + (size_t)pos * row + (4 * c + dq) * 8) : make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int c = 0; c < NV; ++c) {
          const int vp = tb + c * PP + pp;
          vv[c] = vp < t1 ? ldg16_nt(vb + (size_t)vp * row + dc * 8) : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int hh = 0; hh < G; ++hh) {
          float s = 0.f;
#pragma unroll
          for (int c = 0; c < NC; ++c) s = dot8m(kv[c], qv[hh][c], s);
          s += __shfl_xor(s, 16, WAVE);
          s += __shfl_xor(s, 32, WAVE);
          s = valid ? s * scale : -INFINITY;
          float tm = s;
#pragma unroll
          for (int o = 8; o > 0; o >>= 1) tm = fmaxf(tm, __shfl_xor(tm, o, WAVE));
          const float mn = fmaxf(m_run[hh], tm);
          const float corr = __expf(m_run[hh] - mn);
          const float pv = __expf(s - mn);
          float ts = pv;
#pragma unroll
          for (int o = 8; o > 0; o >>= 1) ts += __shfl_xor(ts, o, WAVE);
          l_run[hh] = l_run[hh] * corr + ts;
          m_run[hh] = mn;
#pragma unroll
          for (int i = 0; i < 8; ++i) acc[hh][i] *= corr;
#pragma unroll
          for (int c = 0; c < NV; ++c) {
            const float pw = __shfl(pv, c * PP + pp, WAVE);
            const uint32_t w4[4] = {vv[c].x, vv[c].y, vv[c].z, vv[c].w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              acc[hh][2 * i] += pw * lo_bf(w4[i]);
              acc[hh][2 * i + 1] += pw * hi_bf(w4[i]);
            }
          }
        }
      }
    }
#pragma unroll
    for (int hh = 0; hh < G; ++hh) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        float v = acc[hh][i];
#pragma unroll
        for (int o = DC; o < 64; o <<= 1) v += __shfl_xor(v, o, WAVE);
        acc[hh][i] = v;
      }
      if (lane < DC) {
#pragma unroll
        for (int i = 0; i < 8; ++i) s_acc[(wave * G + hh) * D + dc * 8 + i] = acc[hh][i];
      }
      if (lane == 0) {
        s_m[wave * G + hh] = m_run[hh];
        s_l[wave * G + hh] = l_run[hh];
      }
    }
    __syncthreads();
    for (int idx = tid * 2; idx < G * D; idx += 512) {
      const int hh = idx / D, d = idx - hh * D;
      const int h = kvh * G + hh;
      const float M = fmaxf(fmaxf(s_m[hh], s_m[G + hh]), fmaxf(s_m[2 * G + hh], s_m[3 * G + hh]));
      float Ls = 0.f, o0 = 0.f, o1 = 0.f;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const float mw = s_m[w * G + hh];
        const float sc = (mw == -INFINITY) ? 0.f : __expf(mw - M);
        Ls += s_l[w * G + hh] * sc;
        o0 += s_acc[(w * G + hh) * D + d] * sc;
        o1 += s_acc[(w * G + hh) * D + d + 1] * sc;
      }
      const size_t pi = (size_t)(b * H + h) * ns + split;
      st_coh8(a.part_acc + pi * D + d, make_uint2(__float_as_uint(o0), __float_as_uint(o1)));
      if (d == 0) st_coh8(a.part_ml + pi * 2, make_uint2(__float_as_uint(M), __float_as_uint(Ls)));
    }
    __syncthreads();
  }
}

// ---------------------------------------------------------------------------------------
// the kernel
// ---------------------------------------------------------------------------------------
#define OHARA_MEGA_NS 16  // context chunks per (sequence, kv head)

template <int D, int G>
__global__ __launch_bounds__(256) void decode_mega_kernel(MegaArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const OharaModel& m = a.m;
  const int d = m.d_model, H = m.n_heads, Hkv = m.n_kv_heads, F = m.d_ff, V = m.vocab, B = a.B;
  const int kmax = max(d, max(F, H * D));
  const int ldxs = kmax + 8;
  bf16_t* xs = reinterpret_cast<bf16_t*>(smem);
  float* red = reinterpret_cast<float*>(smem + (((size_t)B * ldxs * 2 + 255) & ~(size_t)255));  // 4 KiB
  float* att = red + 1024;                                                                      // (8 + 4*D)*G floats

  GridSync gs;
  gs.init(a.bar, gridDim.x, a.spin_limit);
  const int pos = a.step_state[0];
  const int step = a.step_state[1];
  const int L = min(pos + 1, m.t_max);
  float best_v = -INFINITY;
  int best_i = 0x7fffffff;
  int nprof = 0;
  auto stamp = [&]() {
    if (a.prof && blockIdx.x == 0 && threadIdx.x == 0) a.prof[nprof] = __builtin_readcyclecounter();
    ++nprof;
  };

  GemmP qkv{}, prj{}, gu{}, dn{}, lm{};
  qkv.H = H; qkv.Hkv = Hkv; qkv.Dh = D; qkv.Tmax = m.t_max; qkv.pos = pos; qkv.cos = m.cos; qkv.sin = m.sin;
  qkv.N = (H + 2 * Hkv) * D; qkv.K = d; qkv.nstrips = (qkv.N + 15) / 16; qkv.out = a.q; qkv.ldo = H * D;
  prj.N = d; prj.K = H * D; prj.nstrips = (d + 15) / 16; prj.out = a.x; prj.ldo = d;
  gu.N = F; gu.K = d; gu.nstrips = 2 * ((F + 7) / 8 * 8) / 16; gu.out = a.act; gu.ldo = F;
  dn.N = d; dn.K = F; dn.nstrips = (d + 15) / 16; dn.out = a.x; dn.ldo = d;
  lm.N = V; lm.K = d; lm.nstrips = (V + 15) / 16; lm.out = a.logits; lm.ldo = V;
  lm.valid = a.valid_vocab > 0 ? min(a.valid_vocab, V) : V;
  lm.wp = reinterpret_cast<const uint4*>(m.w_vocab);

  GemmPre pre;

  {
    const OharaLayer& L0 = a.layers_dev[0];
    qkv.wp = reinterpret_cast<const uint4*>(L0.wqkv);
    gemm_prefetch<4, 6>(qkv, pre);
  }
  stamp();
  for (int l = 0; l < m.n_layers; ++l) {
    const OharaLayer& Lw = a.layers_dev[l];
    bf16_t* kc = a.kcache_dev[l];
    bf16_t* vc = a.vcache_dev[l];
    // P1: [embedding] + norm1 + QKV + rotary + append
    qkv.kc = kc; qkv.vc = vc;
    if ((int)blockIdx.x < qkv.nstrips) {
      if (l == 0) stage_norm<2>(xs, ldxs, nullptr, a.ids, m.token_emb, V, a.x, Lw.norm1, m.eps, B, d);
      else stage_norm<2>(xs, ldxs, a.x, nullptr, nullptr, 0, nullptr, Lw.norm1, m.eps, B, d);
    }
    __syncthreads();
    stamp();
    gemm_phase<4, 6, E_ROPE>(qkv, pre, xs, ldxs, B, red, best_v, best_i);
    stamp();
    prj.wp = reinterpret_cast<const uint4*>(Lw.wo);
    gemm_prefetch<4, 6>(prj, pre);
    gs.sync();
    stamp();
    // P2: attention partials
    attn_phase<D, G>(a, kc, vc, L, att);
    gs.sync();
    stamp();
    // P3: merge + output projection + residual
    if ((int)blockIdx.x < prj.nstrips) stage_attn_merge<OHARA_MEGA_NS>(xs, ldxs, a);
    __syncthreads();
    stamp();
    gemm_phase<4, 6, E_RESID>(prj, pre, xs, ldxs, B, red, best_v, best_i);
    stamp();
    gu.wp = reinterpret_cast<const uint4*>(Lw.wgu);
    gemm_prefetch<2, 12>(gu, pre);
    gs.sync();
    stamp();
    // P4: norm2 + gate/up + SwiGLU
    if ((int)blockIdx.x * 2 < gu.nstrips) stage_norm<2>(xs, ldxs, a.x, nullptr, nullptr, 0, nullptr, Lw.norm2, m.eps, B, d);
    __syncthreads();
    gemm_phase<2, 12, E_SWIGLU>(gu, pre, xs, ldxs, B, red, best_v, best_i);
    dn.wp = reinterpret_cast<const uint4*>(Lw.wdown);
    gemm_prefetch<4, 24>(dn, pre);
    gs.sync();
    stamp();
    // P5: down projection + residual
    if ((int)blockIdx.x < dn.nstrips) stage_copy(xs, ldxs, a.act, B, F);
    __syncthreads();
    gemm_phase<4, 24, E_RESID>(dn, pre, xs, ldxs, B, red, best_v, best_i);
    if (l + 1 < m.n_layers) {
      qkv.wp = reinterpret_cast<const uint4*>(a.layers_dev[l + 1].wqkv);
      gemm_prefetch<4, 6>(qkv, pre);
    } else {
      gemm_prefetch<1, 24>(lm, pre);
    }
    gs.sync();
    stamp();
  }
  // final norm + vocabulary projection, running arg-max per lane
  stage_norm<2>(xs, ldxs, a.x, nullptr, nullptr, 0, nullptr, m.final_norm, m.eps, B, d);
  __syncthreads();
  gemm_phase<1, 24, E_LOGITS>(lm, pre, xs, ldxs, B, red, best_v, best_i);
  stamp();
  if (a.select) {
    // lanes with the same batch column (lane & 15) fold their candidates; then the waves
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
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
    float* cv = red;
    int* ci = reinterpret_cast<int*>(red + 64);
    if (lane < 16) {
      cv[wave * 16 + lane] = best_v;
      ci[wave * 16 + lane] = best_i;
    }
    __syncthreads();
    if (threadIdx.x < B) {
      float bv = cv[threadIdx.x];
      int bi = ci[threadIdx.x];
      for (int w = 1; w < 4; ++w) {
        const float ov = cv[w * 16 + threadIdx.x];
        const int oi = ci[w * 16 + threadIdx.x];
        if (ov > bv || (ov == bv && oi < bi)) {
          bv = ov;
          bi = oi;
        }
      }
      st_cohf(a.cand_val + (size_t)blockIdx.x * B + threadIdx.x, bv);
      st_coh4(a.cand_idx + (size_t)blockIdx.x * B + threadIdx.x, (uint32_t)bi);
    }
    gs.sync();
    if (blockIdx.x == 0) {
      // one wave per sequence (round robin): reduce the per-workgroup candidates
      for (int b = wave; b < B; b += 4) {
        float bv = -INFINITY;
        int bi = 0x7fffffff;
        for (int w = lane; w < (int)gridDim.x; w += 64) {
          const float ov = ld_cohf(a.cand_val + (size_t)w * B + b);
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
  stamp();
  // bookkeeping by workgroup 0: everyone is past the last barrier, nobody reads these again
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    *gs.done = gs.k - 1;
    if (a.select) {
      a.step_state[0] = pos + 1;
      a.step_state[1] = step + 1;
    }
  }
}

}  // namespace

extern "C" {

#define OHARA_BAR_WORDS(nwg) ((((nwg) + OHARA_BAR_GROUP - 1) / OHARA_BAR_GROUP + 4) * 64)
#define OHARA_PROF_SLOTS 512

static size_t mega_al(size_t v) { return (v + 255) & ~(size_t)255; }

// Bytes of the device scratch block ohara_llama_decode_persistent needs.
int64_t ohara_persistent_workspace_bytes(const OharaModel* m, int batch, int n_split, int n_workgroups) {
  if (!m || batch < 1 || n_split < 1 || n_workgroups < 1) return OHARA_EINVAL;
  size_t tot = 0;
  tot += mega_al(sizeof(OharaLayer) * m->n_layers);
  tot += 2 * mega_al(sizeof(void*) * m->n_layers);
  tot += mega_al((size_t)batch * m->n_heads * n_split * 2 * sizeof(float));
  tot += mega_al((size_t)batch * m->n_heads * n_split * m->head_dim * sizeof(float));
  tot += 2 * mega_al((size_t)n_workgroups * batch * sizeof(float));
  tot += mega_al(OHARA_PROF_SLOTS * sizeof(unsigned long long));
  tot += mega_al(OHARA_BAR_WORDS(n_workgroups) * sizeof(unsigned int));
  return (int64_t)tot;
}

int64_t ohara_persistent_barrier_offset(const OharaModel* m, int batch, int n_split, int n_workgroups) {
  const int64_t tot = ohara_persistent_workspace_bytes(m, batch, n_split, n_workgroups);
  return tot < 0 ? tot : tot - (int64_t)mega_al(OHARA_BAR_WORDS(n_workgroups) * sizeof(unsigned int));
}

int ohara_llama_decode_persistent(const OharaModel* m, const OharaDecodeState* s, void* workspace, int n_workgroups,
                                  int init_workspace, int select_greedy, unsigned int spin_limit, void* stream) {
  if (!m || !s || !workspace || !m->layers || !s->kcache || !s->vcache || !s->step_state) return OHARA_EINVAL;
  if (s->batch < 1 || s->batch > 16) return OHARA_ESIZE;
  if (n_workgroups < 1 || n_workgroups > 1024) return OHARA_EINVAL;
  if (s->n_split != OHARA_MEGA_NS) return OHARA_EINVAL;
  const int D = m->head_dim, G = m->n_heads / m->n_kv_heads;
  if (!(D == 128 || D == 64) || !(G == 1 || G == 2 || G == 4) || m->n_heads % m->n_kv_heads) return OHARA_ESIZE;
  if ((m->d_model & 7) || (m->d_ff & 7) || m->d_model > 1024) return OHARA_ESIZE;
  hipStream_t st = (hipStream_t)stream;
  char* ws = reinterpret_cast<char*>(workspace);
  MegaArgs a{};
  a.m = *m;
  a.layers_dev = reinterpret_cast<const OharaLayer*>(ws);
  ws += mega_al(sizeof(OharaLayer) * m->n_layers);
  a.kcache_dev = reinterpret_cast<uint16_t* const*>(ws);
  ws += mega_al(sizeof(void*) * m->n_layers);
  a.vcache_dev = reinterpret_cast<uint16_t* const*>(ws);
  ws += mega_al(sizeof(void*) * m->n_layers);
  a.part_ml = reinterpret_cast<float*>(ws);
  ws += mega_al((size_t)s->batch * m->n_heads * s->n_split * 2 * sizeof(float));
  a.part_acc = reinterpret_cast<float*>(ws);
  ws += mega_al((size_t)s->batch * m->n_heads * s->n_split * D * sizeof(float));
  a.cand_val = reinterpret_cast<float*>(ws);
  ws += mega_al((size_t)n_workgroups * s->batch * sizeof(float));
  a.cand_idx = reinterpret_cast<int*>(ws);
  ws += mega_al((size_t)n_workgroups * s->batch * sizeof(float));
  unsigned long long* prof = reinterpret_cast<unsigned long long*>(ws);
  ws += mega_al(OHARA_PROF_SLOTS * sizeof(unsigned long long));
  a.bar = reinterpret_cast<unsigned int*>(ws);
  if (init_workspace) {
    // small synchronous copies: done once per (model, cache) binding, outside any capture
    const size_t barb = mega_al(OHARA_BAR_WORDS(n_workgroups) * sizeof(unsigned int));
    if (hipMemcpyAsync((void*)a.layers_dev, m->layers, sizeof(OharaLayer) * m->n_layers, hipMemcpyHostToDevice, st) !=
            hipSuccess ||
        hipMemcpyAsync((void*)a.kcache_dev, s->kcache, sizeof(void*) * m->n_layers, hipMemcpyHostToDevice, st) !=
            hipSuccess ||
        hipMemcpyAsync((void*)a.vcache_dev, s->vcache, sizeof(void*) * m->n_layers, hipMemcpyHostToDevice, st) !=
            hipSuccess ||
        hipMemsetAsync((void*)a.bar, 0, barb, st) != hipSuccess || hipStreamSynchronize(st) != hipSuccess)
      return OHARA_ELAUNCH;
    return OHARA_OK;
  }
  a.B = s->batch; a.nsplit = s->n_split; a.valid_vocab = s->valid_vocab; a.hist_cap = s->hist_cap;
  a.select = select_greedy;
  a.ids = s->ids; a.x = s->x; a.q = s->q; a.act = s->act; a.logits = s->logits;
  a.step_state = s->step_state; a.history = s->history;
  a.prof = s->prof_kernel == -2 ? prof : nullptr;  // -2: record per-phase clocks of workgroup 0
  a.spin_limit = spin_limit ? spin_limit : (1u << 19);
  const int kmax = m->d_model > m->d_ff ? m->d_model : m->d_ff;
  const int kmax2 = kmax > m->n_heads * D ? kmax : m->n_heads * D;
  const size_t xs_bytes = ((size_t)s->batch * (kmax2 + 8) * 2 + 255) & ~(size_t)255;
  const size_t smem = xs_bytes + 4096 + (size_t)(8 + 4 * D) * G * sizeof(float);
  if (smem > 160 * 1024) return OHARA_ESIZE;
  if (9 * m->n_layers + 4 > OHARA_PROF_SLOTS) a.prof = nullptr;
  dim3 grid(n_workgroups), block(256);
#define OHARA_MEGA(DD, GG)                                                                                  \
  do {                                                                                                      \
    if (smem > 64 * 1024)                                                                                   \
      (void)hipFuncSetAttribute((const void*)decode_mega_kernel<DD, GG>,                                    \
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);                     \
    hipLaunchKernelGGL((decode_mega_kernel<DD, GG>), grid, block, smem, st, a);                             \
  } while (0)
  if (D == 128 && G == 1) OHARA_MEGA(128, 1);
  else if (D == 128 && G == 2) OHARA_MEGA(128, 2);
  else if (D == 128 && G == 4) OHARA_MEGA(128, 4);
  else if (D == 64 && G == 1) OHARA_MEGA(64, 1);
  else if (D == 64 && G == 2) OHARA_MEGA(64, 2);
  else OHARA_MEGA(64, 4);
#undef OHARA_MEGA
  return ohara_launch_status();
}

// Byte offset of the sticky barrier-error word (uint32) inside the workspace.
int64_t ohara_persistent_error_offset(const OharaModel* m, int batch, int n_split, int n_workgroups) {
  const int64_t b = ohara_persistent_barrier_offset(m, batch, n_split, n_workgroups);
  const int ng = (n_workgroups + OHARA_BAR_GROUP - 1) / OHARA_BAR_GROUP;
  return b < 0 ? b : b + (int64_t)(ng + 2) * 64 * 4;
}

// Byte offset of the per-phase clock samples (uint64 x 256) inside the workspace.
int64_t ohara_persistent_profile_offset(const OharaModel* m, int batch, int n_split, int n_workgroups) {
  const int64_t b = ohara_persistent_barrier_offset(m, batch, n_split, n_workgroups);
  return b < 0 ? b : b - (int64_t)mega_al(OHARA_PROF_SLOTS * sizeof(unsigned long long));
}

}  // extern "C"
