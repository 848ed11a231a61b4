// Device-side building blocks of the persistent (whole-step, one launch) decode kernels: the grid
// barrier, the strip-blocked mailboxes, activation staging, the bf16 GEMM phase over packed weight
// strips, and the split-context attention phase.  Included by the kernels that are built from them
// (the bf16 Llama step and the BitNet ternary step); everything here is file-local to its includer.
#pragma once
#include "common.h"

// Host side: can `n_workgroups` workgroups of `kernel` (256 threads, `smem` bytes of dynamic LDS) be
// resident on the current device at the same time?  The grid barrier of the persistent kernels needs
// that: a workgroup that is not dispatched until another one exits would be waited for until the
// spin limit expires.  The answer per (kernel, smem) is cached in `slot` (one per launch site).
struct ResidencySlot {
  const void* kernel = nullptr;
  size_t smem = 0;
  int max_workgroups = 0;
};
inline bool ohara_grid_fits(ResidencySlot& slot, const void* kernel, size_t smem, int n_workgroups) {
  if (slot.kernel != kernel || slot.smem != smem) {
    int dev = 0, cus = 0, per_cu = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, 256, smem) != hipSuccess)
      return false;
    slot.kernel = kernel;
    slot.smem = smem;
    slot.max_workgroups = cus * per_cu;
  }
  return n_workgroups <= slot.max_workgroups;
}

namespace {


#define OHARA_MEGA_NS 16  // context chunks per (sequence, kv head)
#define OHARA_MAX_PF 24   // weight tiles (16 B per lane) a wave holds fetched ahead of its phases
#define OHARA_LDS_PF 24   // weight tiles a wave can park in LDS (E_XNEXT: the down projection of the batch-1 kernels)
#define OHARA_DOWN_SPLIT 4  // K partitions of the down projection (static_assert below: x_load sums four)

// Optional fine-grained timeline: thread 0 of every workgroup records the constant 100 MHz clock
// (the same counter on every XCD, so that workgroups can be compared).  The stamps are
// compiled in only for kernels instantiated with ON (dozens of clock reads and guarded stores per
// layer are several KB of code the ordinary kernel does not have to fetch).
template <bool ON>
struct ProfT;
template <>
struct ProfT<true> {
  unsigned long long* p;
  int n;
  __device__ __forceinline__ explicit ProfT(unsigned long long* q) : p(q), n(0) {}
  __device__ __forceinline__ void stamp() {
    if (p) p[n] = __builtin_amdgcn_s_memrealtime();
    ++n;
  }
};
template <>
struct ProfT<false> {
  __device__ __forceinline__ explicit ProfT(unsigned long long*) {}
  __device__ __forceinline__ void stamp() {}
};

// ---------------------------------------------------------------------------------------
// Grid barrier.  Arrivals are fire-and-forget atomics on monotonic group counters (groups of 16
// workgroups, each counter on its own 256-byte line: same-address atomics serialise at ~11 ns
// each); ONE master workgroup - the last of the grid, which has the least work in most phases -
// polls all group counters with one load per lane and publishes the barrier index in eight release
// words (one per XCD's workgroups, each on its own line: 32 pollers per word instead of 256 measured
// 0.14 us faster per barrier).  The chain after the last arrival is: atomic reaches memory, the
// master's next poll sees it (a device-scope load takes 0.13 us), release store seen by the
// pollers (0.58 us) - about 1.5 us per barrier in a stand-alone loop against 2.0 us for two levels
// of atomics WITH return (each 0.39 us) in front of the same release.  The master polls before it
// issues its own prefetch for the next phase (its polls would otherwise return behind those loads)
// and moves on as soon as it has seen every arrival, which is before anyone else sees the release.
// Words (uint32, stride 64 per counter): [g*64] group g, [ng*64] and [(ng+1)*64] unused,
// [(ng+2)*64] sticky error, [(ng+3)*64] barriers completed by earlier launches, [(ng+4+x)*64]
// release word x (workgroups with blockIdx % 8 == x poll it).  arrive() and
// wait() are split so that a workgroup can issue the loads of its next phase (weights, cache
// tiles: nothing that depends on this phase) in between and have them in flight while it waits.
// (Measured and dropped: a flat counter (serialises 256 read-modify-writes); the workgroup that
// completes a group publishing a flag that one wave per workgroup polls (0.352 against 0.339 ms per
// step); everyone polling a counter that is still receiving atomics (twice as slow); flags gathered
// by one wave or by group leaders.)
// ---------------------------------------------------------------------------------------
#define OHARA_BAR_GROUP 16
struct GridSync {
  unsigned int* bar;
  unsigned int* gc;
  unsigned int* rel;
  unsigned int* err;
  unsigned int* done;
  unsigned int k;      // index of the next barrier (1-based, across launches)
  unsigned int nwg;
  unsigned int ng;
  unsigned int limit;
  bool master;
  __device__ void init(unsigned int* b, unsigned int n, unsigned int lim) {
    bar = b;
    nwg = n;
    ng = (nwg + OHARA_BAR_GROUP - 1) / OHARA_BAR_GROUP;
    gc = bar + (blockIdx.x / OHARA_BAR_GROUP) * 64;
    rel = bar + (ng + 4 + (blockIdx.x & 7)) * 64;
    err = bar + (ng + 2) * 64;
    done = bar + (ng + 3) * 64;
    limit = lim;
    master = blockIdx.x == nwg - 1;
    k = *done + 1;  // written by the previous launch (or the host): plain load
  }
  template <class PROF>
  __device__ __forceinline__ void arrive(PROF& pf) {
    pf.stamp();  // phase work issued
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");  // orders my LDS and global accesses within the workgroup
    wait_own_stores();  // every wave: its sc1 stores have reached memory before the barrier below
    pf.stamp();  // stores complete
    __builtin_amdgcn_s_barrier();
    pf.stamp();  // workgroup barrier passed
    // The arrival happens here, before the caller's prefetch: nobody's arrival waits behind loads.
    if (threadIdx.x == 0) (void)__hip_atomic_fetch_add(gc, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (master && threadIdx.x < 64) {
      // lane l watches group l: k * (its size) arrivals since the workspace was cleared
      const unsigned int lane = threadIdx.x;
      const unsigned int gsize = lane < ng ? min((unsigned int)OHARA_BAR_GROUP, nwg - lane * OHARA_BAR_GROUP) : 0u;
      const unsigned int want = k * gsize;
      unsigned int spins = 0;
      bool ok = true;
      for (;;) {
        const unsigned int v = lane < ng ? __hip_atomic_load(bar + lane * 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : want;
        if (__all((int)(v - want) >= 0)) break;
        if (++spins > limit) { ok = false; break; }
        if ((spins & 63u) == 0 && __hip_atomic_load(err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) { ok = false; break; }
      }
      if (ok && lane < 8) __hip_atomic_store(bar + (ng + 4 + lane) * 64, k, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (!ok && lane == 0) __hip_atomic_store(err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    asm volatile("" ::: "memory");  // compiler only: keep the caller's prefetch loads after this point
    pf.stamp();  // arrival issued
  }
  template <class PROF>
  __device__ __forceinline__ void wait(PROF& pf) {
    pf.stamp();  // prefetch issued
    if (threadIdx.x == 0 && !master) {
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
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): nothing of mine is still on its way to LDS
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");  // compiler only: mailbox loads of the next phase stay below the barrier
    pf.stamp();  // barrier passed
    ++k;
  }
};

// A pointer from the workgroup's LDS copy of the layer table, made wave-uniform.
template <typename T>
__device__ __forceinline__ T* lds_ptr(const unsigned long long* tab, int i) {
  const unsigned long long v = tab[i];
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return reinterpret_cast<T*>(((unsigned long long)hi << 32) | lo);
}

__device__ __forceinline__ float dot8m(uint4 a, uint4 b, float s) {
  s = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a.x), __builtin_bit_cast(bf16x2, b.x), s, false);
  s = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a.y), __builtin_bit_cast(bf16x2, b.y), s, false);
  s = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a.z), __builtin_bit_cast(bf16x2, b.z), s, false);
  s = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a.w), __builtin_bit_cast(bf16x2, b.w), s, false);
  return s;
}

// ---------------------------------------------------------------------------------------
// Polled mailboxes: hand-offs of a single row (batch 1) WITHOUT a grid barrier.  A mailbox is the plain
// bf16 row, two values to a 32-bit word, and a word that has not been written yet holds 0xFFFFFFFF - two
// NaNs of a payload that arithmetic does not produce (the producer turns a pair that happens to look
// like it into two other NaNs).  There are two sets of mailboxes: launch n writes and reads set n & 1,
// and whoever stores a word there resets the same word of the other set, which every consumer finished
// with a launch ago and which the next launch finds unwritten again; the entry point fills both sets
// with 0xFF when it clears the workspace.  Each word is written once per launch with a device-scope
// store and consumers poll the words they need with 16-byte device-scope loads, all of them every
// round: what a hand-off costs is the round trips to memory and the number of load instructions per
// round (a 1 KB row polled by one instruction per lane is seen ~0.7 us after its stores were issued, a
// 4 KB row polled by four ~1.7 us; one round that only watched a flag first would add a trip), not
// the number of pollers.  That is against ~1.6 us for a grid barrier plus the producers' wait for
// their stores before it plus fetching the data cold.  Every poll loop is bounded like the barrier's
// spins.  Only worth it where a consumer needs little (a row, a head's 128 values).
// The attention partials (fp32, 48 KB per consumer) go another way: see stage_attn_merge.
// ---------------------------------------------------------------------------------------
#define OHARA_UNWRITTEN 0xFFFFFFFFu
struct Poll {
  uint32_t tag;   // the number of this launch since the workspace was cleared
  unsigned int limit;
  unsigned int* err;
};
__device__ __forceinline__ bool poll_expired(const Poll& pc, unsigned int& spins) {
  if (++spins > pc.limit) {
    __hip_atomic_store(pc.err, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return true;
  }
  return (spins & 63u) == 0 && __hip_atomic_load(pc.err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0;
}
__device__ __forceinline__ uint32_t mb_word(uint32_t v) { return v == OHARA_UNWRITTEN ? 0xFFFEFFFFu : v; }
// four values starting at column `col` (a multiple of 4); `other`: from this set's mailbox to the other set's
__device__ __forceinline__ void mb_st8(char* base, ptrdiff_t other, int col, uint32_t lo, uint32_t hi) {
  char* q = base + (size_t)col * 2;
  st_coh8(q, make_uint2(mb_word(lo), mb_word(hi)));
  st_coh8(q + other, make_uint2(OHARA_UNWRITTEN, OHARA_UNWRITTEN));
}
// two values starting at column `col` (a multiple of 2)
__device__ __forceinline__ void mb_st4(char* base, ptrdiff_t other, int col, uint32_t v) {
  char* q = base + (size_t)col * 2;
  st_coh4(q, mb_word(v));
  st_coh4(q + other, OHARA_UNWRITTEN);
}
// The load side: a buffer descriptor over the mailbox (the 16-byte device-scope load is a buffer load with sc1).
typedef __amdgpu_buffer_rsrc_t MbRsrc;
__device__ __forceinline__ MbRsrc mb_rsrc(const void* base) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, 0x7FFFFFFF, 0x00020000);
}
// eight values starting at column `col` (a multiple of 8); true when all of them have been written
__device__ __forceinline__ bool mb_ld16(MbRsrc r, int col, uint4& out) {
  const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(r, (uint32_t)col * 2u, 0, 16);
  out = make_uint4(v.x, v.y, v.z, v.w);
  return v.x != OHARA_UNWRITTEN && v.y != OHARA_UNWRITTEN && v.z != OHARA_UNWRITTEN && v.w != OHARA_UNWRITTEN;
}

// two values starting at column `col` (even); true when they have been written
__device__ __forceinline__ bool mb_ld4(MbRsrc r, int col, uint32_t& out) {
  out = __builtin_amdgcn_raw_buffer_load_b32(r, (uint32_t)col * 2u, 0, 16);
  return out != OHARA_UNWRITTEN;
}

// Strip-blocked mailbox of a (B, N) bf16 matrix: the 16 columns [16s, 16s+16) of all rows
// form block s of `blk` bytes (a multiple of 128), row b at byte b*32 inside it.
__device__ __forceinline__ const char* xm_addr(const char* base, int blk, int b, int n) {
  return base + (size_t)(n >> 4) * blk + b * 32 + (n & 15) * 2;
}
// act mailbox: 8 columns per block, row b at byte b*16.
__device__ __forceinline__ const char* am_addr(const char* base, int blk, int b, int f) {
  return base + (size_t)(f >> 3) * blk + b * 16 + (f & 7) * 2;
}

// The down projection is split along K over OHARA_DOWN_SPLIT groups of workgroups (a 16-row strip
// of it is too much for one CU to stream); each group leaves fp32 partial sums and whoever needs
// the residual stream after the block forms it on the fly, in a fixed order:
//   x[b][n] = bf16(x_mid[b][n] + bf16(((p0 + p1) + p2) + p3))        (llama.py:200)
// The sums are strip-blocked like the x mailbox, one block of `blk` bytes (a multiple of 128) per
// (part, strip) with row b at byte b*64, so that every 128-byte line has a single writer.
struct XParts {
  const char* xmid;   // x mailbox holding the stream before the feed-forward block
  const float* parts; // partial sums; nullptr: `xmid` already is the stream that is wanted
  int blk, B, N;
};
__device__ __forceinline__ int pm_blk(int B) { return (B * 64 + 127) & ~127; }
__device__ __forceinline__ const float* parts_addr(const float* base, int nstrips, int B, int q, int b, int n) {
  return reinterpret_cast<const float*>(reinterpret_cast<const char*>(base) +
                                        (size_t)(q * nstrips + (n >> 4)) * pm_blk(B) + b * 64) + (n & 15);
}

// PARTS says at compile time whether xp.parts is set: a branch on the pointer would keep the
// compiler from issuing the loads of several calls together.  The loads (x_fetch) and the sums
// (x_combine) are separate so that a caller can issue the loads of several pieces back to back.
template <int NW, bool PARTS>  // NW columns (4 or 8) starting at n, n % NW == 0
struct XRaw {
  uint4 xm;  // NW == 4: .x, .y only
  uint4 pv[PARTS ? OHARA_DOWN_SPLIT : 1][NW / 4];
};
template <int NW, bool PARTS>
__device__ __forceinline__ void x_fetch(const XParts& xp, int b, int n, XRaw<NW, PARTS>& r) {
  if (NW == 8) {
    r.xm = ldg16(xm_addr(xp.xmid, xp.blk, b, n));
  } else {
    const uint2 v = ldg8(xm_addr(xp.xmid, xp.blk, b, n));
    r.xm = make_uint4(v.x, v.y, 0, 0);
  }
  if (PARTS) {
#pragma unroll
    for (int q = 0; q < OHARA_DOWN_SPLIT; ++q)
#pragma unroll
      for (int i = 0; i < NW / 4; ++i) r.pv[q][i] = ldg16(parts_addr(xp.parts, (xp.N + 15) >> 4, xp.B, q, b, n + 4 * i));
  }
}
template <int NW, bool PARTS>
__device__ __forceinline__ void x_combine(const XRaw<NW, PARTS>& r, uint32_t (&out)[NW / 2]) {
  uint32_t xm[NW / 2];
  xm[0] = r.xm.x; xm[1] = r.xm.y;
  if (NW == 8) { xm[NW / 2 - 2] = r.xm.z; xm[NW / 2 - 1] = r.xm.w; }
  if (!PARTS) {
#pragma unroll
    for (int i = 0; i < NW / 2; ++i) out[i] = xm[i];
    return;
  }
  static_assert(OHARA_DOWN_SPLIT == 4, "x_combine sums four partitions");
#pragma unroll
  for (int i = 0; i < NW / 4; ++i) {
    float y[4];
    const uint4 p0 = r.pv[0][i], p1 = r.pv[PARTS ? 1 : 0][i], p2 = r.pv[PARTS ? 2 : 0][i], p3 = r.pv[PARTS ? 3 : 0][i];
    const uint32_t w[OHARA_DOWN_SPLIT][4] = {{p0.x, p0.y, p0.z, p0.w}, {p1.x, p1.y, p1.z, p1.w},
                                             {p2.x, p2.y, p2.z, p2.w}, {p3.x, p3.y, p3.z, p3.w}};
#pragma unroll
    for (int e = 0; e < 4; ++e)
      y[e] = rbf(((__uint_as_float(w[0][e]) + __uint_as_float(w[1][e])) + __uint_as_float(w[2][e])) +
                 __uint_as_float(w[3][e]));
    out[2 * i] = pack_bf(lo_bf(xm[2 * i]) + y[0], hi_bf(xm[2 * i]) + y[1]);
    out[2 * i + 1] = pack_bf(lo_bf(xm[2 * i + 1]) + y[2], hi_bf(xm[2 * i + 1]) + y[3]);
  }
}
template <int NW, bool PARTS>
__device__ __forceinline__ void x_load(const XParts& xp, int b, int n, uint32_t (&out)[NW / 2]) {
  XRaw<NW, PARTS> r;
  x_fetch<NW, PARTS>(xp, b, n, r);
  x_combine<NW, PARTS>(r, out);
}

// ---------------------------------------------------------------------------------------
// staging of the GEMM activations in LDS: xs[b][ldxs] bf16
// ---------------------------------------------------------------------------------------

// norm.py:16-21 on rows of the residual stream (x-mailbox `src`), or - for the first layer
// - on rows gathered from the embedding table (llama.py:310).  One wave per row; all loads
// of a row are issued before any is consumed.  K <= 8 * 64 * NLD elements.
// PRE: the lane's norm-weight pieces were fetched ahead (gemm_prefetch) and are in gpre[0 .. NLD).
// PARTS: `parts` is set (the rows are x-mailbox rows plus down-projection sums).
// The embedding rows of a wave (rows wave and wave + 4 of at most eight), requested ahead of everything else a
// workgroup fetches at the start of a launch: the ids first, the rows as soon as the ids are there.
template <int NLD>
struct EmbedPre {
  int64_t id[2];
  uint4 v[2][NLD];
};
template <int NLD>
__device__ __forceinline__ void embed_request_ids(const int64_t* ids, int B, EmbedPre<NLD>& e) {
  const int wave = threadIdx.x >> 6;
#pragma unroll
  for (int r = 0; r < 2; ++r) e.id[r] = ldg_i64(ids + min(wave + 4 * r, B - 1));
}
template <int NLD>
__device__ __forceinline__ void embed_request_rows(const bf16_t* table, int vocab, int K, EmbedPre<NLD>& e) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int r = 0; r < 2; ++r) {
    int64_t id = e.id[r];
    if (id < 0 || id >= vocab) id = 0;
#pragma unroll
    for (int c = 0; c < NLD; ++c) {
      const int k = (c * 64 + lane) * 8;
      e.v[r][c] = ldg16(table + (size_t)id * K + (k < K ? k : 0));
    }
  }
}

// EPRE (with EMBED): the rows were requested ahead (embed_request_rows; B <= 8) and are in epre
template <int NLD, bool EMBED, bool PRE, bool PARTS, bool EPRE = false>
__device__ __forceinline__ void stage_norm(bf16_t* xs, int ldxs, const char* src, int blk, const float* parts,
                                           const int64_t* ids, const bf16_t* table, int vocab, const bf16_t* nw, float eps,
                                           int B, int K, const uint4 (&gpre)[NLD], const EmbedPre<NLD>& epre = EmbedPre<NLD>()) {
  const XParts xp{src, parts, blk, B, K};
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int b = wave; b < B; b += 4) {
    uint4 v[NLD], g[NLD];
    size_t row_off = 0;
    if (EMBED && !EPRE) {
      int64_t id = ldg_i64(ids + b);
      if (id < 0 || id >= vocab) id = 0;
      row_off = (size_t)id * K;
    }
    // Every piece is loaded without a branch (pieces beyond K read column 0 and are zeroed below):
    // behind a branch per piece the compiler waits for one piece's loads before it issues the
    // next piece's, one cold round trip after the other.
    XRaw<8, PARTS> raw[NLD];
#pragma unroll
    for (int c = 0; c < NLD; ++c) {
      const int k = (c * 64 + lane) * 8;
      const int kc = k < K ? k : 0;
      if (EMBED && EPRE) v[c] = epre.v[b >= 4 ? 1 : 0][c];
      else if (EMBED) v[c] = ldg16(table + row_off + kc);
      else x_fetch<8, PARTS>(xp, b, kc, raw[c]);
      g[c] = PRE ? gpre[c] : ldg16(nw + kc);
    }
    __builtin_amdgcn_sched_barrier(0);  // all loads above, all sums below
#pragma unroll
    for (int c = 0; c < NLD; ++c) {
      if (!EMBED) {
        uint32_t w[4];
        x_combine<8, PARTS>(raw[c], w);
        v[c] = make_uint4(w[0], w[1], w[2], w[3]);
      }
      if ((c * 64 + lane) * 8 >= K) {
        v[c] = make_uint4(0, 0, 0, 0);
        g[c] = make_uint4(0, 0, 0, 0);
      }
    }
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < NLD; ++c) {
      const uint32_t w[4] = {v[c].x, v[c].y, v[c].z, v[c].w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float a0 = lo_bf(w[i]), a1 = hi_bf(w[i]);
        ss += a0 * a0 + a1 * a1;
      }
    }
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

// act mailbox (B, F) -> LDS
// act mailbox (B, F), columns [f0, f1) (multiples of 8) -> LDS
__device__ __forceinline__ void stage_act(bf16_t* xs, int ldxs, const char* src, int blk, int B, int f0, int f1) {
  const int n8 = (f1 - f0) >> 3;
  for (int i = threadIdx.x; i < B * n8; i += blockDim.x) {
    const int b = i / n8, c = (f0 >> 3) + i - b * n8;
    sts16(xs + (size_t)b * ldxs + c * 8, ldg16(am_addr(src, blk, b, c * 8)));
  }
}

// The row of a polled mailbox (batch 1) -> norm.py:16-21 -> LDS, by wave 0: stage_norm on a row that is
// polled for instead of fetched after a barrier.  The norm weights were fetched ahead (gpre).
template <int NLD>
__device__ __forceinline__ void stage_norm_tagged(bf16_t* xs, const char* xt, const Poll& pc, float eps, int K,
                                                  const uint4 (&gpre)[NLD], int B = 1, int ldxs = 0, int row_bytes = 0) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // one wave per row, rows wave and wave + 4 together (up to eight sequences): both are polled for in the same rounds
  if (wave >= B) return;
  if (B == 1) {  // a single sequence, spelled out (the general form below costs it 0.1 - 0.2 us per call)
    uint4 v[NLD];
    unsigned int spins = 0;
    const MbRsrc rs = mb_rsrc(xt);
    for (;;) {
      bool ok = true;
#pragma unroll
      for (int c = 0; c < NLD; ++c) {
        const int k = (c * 64 + lane) * 8;
        ok = mb_ld16(rs, k < K ? k : 0, v[c]) && ok;
      }
      if (__all(ok) || poll_expired(pc, spins)) break;
    }
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < NLD; ++c) {
      if ((c * 64 + lane) * 8 >= K) v[c] = make_uint4(0, 0, 0, 0);
      const uint32_t w[4] = {v[c].x, v[c].y, v[c].z, v[c].w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float a0 = lo_bf(w[i]), a1 = hi_bf(w[i]);
        ss += a0 * a0 + a1 * a1;
      }
    }
    ss = wave_sum(ss);
    const float rinv = 1.0f / sqrtf(ss / (float)K + eps);
#pragma unroll
    for (int c = 0; c < NLD; ++c) {
      const int k = (c * 64 + lane) * 8;
      if (k < K) {
        const uint32_t xv[4] = {v[c].x, v[c].y, v[c].z, v[c].w};
        const uint32_t gv[4] = {gpre[c].x, gpre[c].y, gpre[c].z, gpre[c].w};
        uint32_t o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
          o[i] = pack_bf(rbf(lo_bf(xv[i]) * rinv) * lo_bf(gv[i]), rbf(hi_bf(xv[i]) * rinv) * hi_bf(gv[i]));
        sts16(xs + k, make_uint4(o[0], o[1], o[2], o[3]));
      }
    }
    return;
  }
  const bool two = wave + 4 < B;
  uint4 v[2][NLD];
  unsigned int spins = 0;
  const MbRsrc rs0 = mb_rsrc(xt + (size_t)wave * row_bytes);
  const MbRsrc rs1 = mb_rsrc(xt + (size_t)(two ? wave + 4 : wave) * row_bytes);
  // every round fetches the whole row (1.5 KB at K = 768) and looks at every word
  for (;;) {
    bool ok = true;
#pragma unroll
    for (int c = 0; c < NLD; ++c) {
      const int k = (c * 64 + lane) * 8;
      ok = mb_ld16(rs0, k < K ? k : 0, v[0][c]) && ok;
    }
    if (two) {
#pragma unroll
      for (int c = 0; c < NLD; ++c) {
        const int k = (c * 64 + lane) * 8;
        ok = mb_ld16(rs1, k < K ? k : 0, v[1][c]) && ok;
      }
    }
    if (__all(ok) || poll_expired(pc, spins)) break;
  }
  for (int r = 0; r < (two ? 2 : 1); ++r) {
    const int b = wave + 4 * r;
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < NLD; ++c) {
      if ((c * 64 + lane) * 8 >= K) v[r][c] = make_uint4(0, 0, 0, 0);
      const uint32_t w[4] = {v[r][c].x, v[r][c].y, v[r][c].z, v[r][c].w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float a0 = lo_bf(w[i]), a1 = hi_bf(w[i]);
        ss += a0 * a0 + a1 * a1;
      }
    }
    ss = wave_sum(ss);
    const float rinv = 1.0f / sqrtf(ss / (float)K + eps);
#pragma unroll
    for (int c = 0; c < NLD; ++c) {
      const int k = (c * 64 + lane) * 8;
      if (k < K) {
        const uint32_t xv[4] = {v[r][c].x, v[r][c].y, v[r][c].z, v[r][c].w};
        const uint32_t gv[4] = {gpre[c].x, gpre[c].y, gpre[c].z, gpre[c].w};
        uint32_t o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
          o[i] = pack_bf(rbf(lo_bf(xv[i]) * rinv) * lo_bf(gv[i]), rbf(hi_bf(xv[i]) * rinv) * hi_bf(gv[i]));
        sts16(xs + (size_t)b * ldxs + k, make_uint4(o[0], o[1], o[2], o[3]));
      }
    }
  }
}

// Columns [f0, f1) (multiples of 8) of the polled act mailbox -> LDS.  Pieces of 8 columns, all rows in one
// index space; a thread polls FLY of its pieces in the same rounds, without a test per piece (past the end:
// the last piece again, not stored).  One row after the other, each with rounds of its own, was 6.7 us for
// eight rows of 3072; a test per piece made every load wait for the one before.
template <int FLY>
__device__ __forceinline__ void stage_act_fly(bf16_t* xs, const char* at, const Poll& pc, int f0, int n8, int total, int ldxs,
                                              int row_bytes) {
  const MbRsrc rs = mb_rsrc(at);
  for (int i0 = threadIdx.x; i0 < total; i0 += (int)blockDim.x * FLY) {
    uint4 v[FLY];
    int col[FLY], row[FLY];
#pragma unroll
    for (int j = 0; j < FLY; ++j) {
      const int i = min(i0 + j * (int)blockDim.x, total - 1);
      row[j] = i / n8;
      col[j] = ((f0 >> 3) + (i - row[j] * n8)) * 8;
    }
    unsigned int spins = 0;
    for (;;) {
      bool ok = true;
#pragma unroll
      for (int j = 0; j < FLY; ++j) ok = mb_ld16(rs, row[j] * (row_bytes >> 1) + col[j], v[j]) && ok;
      if (ok || poll_expired(pc, spins)) break;
    }
#pragma unroll
    for (int j = 0; j < FLY; ++j)
      if (i0 + j * (int)blockDim.x < total) sts16(xs + (size_t)row[j] * ldxs + col[j], v[j]);
  }
}
__device__ __forceinline__ void stage_act_tagged(bf16_t* xs, const char* at, const Poll& pc, int f0, int f1, int B = 1,
                                                 int ldxs = 0, int row_bytes = 0) {
  const int n8 = (f1 - f0) >> 3, total = B * n8;
  if (total <= 2 * (int)blockDim.x) stage_act_fly<2>(xs, at, pc, f0, n8, total, ldxs, row_bytes);
  else stage_act_fly<6>(xs, at, pc, f0, n8, total, ldxs, row_bytes);
}

// Merge of the attention partials of all chunks, in chunk order (llama.py:116-123 output,
// rounded to bf16 as SDPA's result is) -> xs[b][h*Dh + d].  NS (a power of two) chunks are in use.
// The (max, sum) pairs of every (sequence, head, chunk) are fetched in one round into LDS and
// turned into chunk weights exp(m_s - M) and the sum L there; a thread then owns four adjacent
// columns per pass and issues the accumulator loads of 16 / NS passes - 16 loads - before it uses
// any, so the number of dependent load rounds does not grow with the chunk count times the batch.
// `mw`: B*H*NS floats, `ml`: B*H floats of LDS.
// TAGGED (batch-1 kernels without a barrier ahead of the merge): a chunk's maximum and sum are stored as
// {max, tag, sum, tag} - each value in one 8-byte word with the tag of the launch - once the chunk's accumulators
// have reached memory; they are polled for, one lane per chunk, and the accumulators are fetched only after
// every chunk of the workgroup has been seen.
template <int NS, bool TAGGED = false>  // NS: a power of two; `used` <= NS chunks hold partials (the others weigh nothing)
__device__ __forceinline__ void stage_attn_merge(bf16_t* xs, int ldxs, const float* pm, int B, int H, int Dh, float* mw_, float* ml_,
                                                 int used = NS, const Poll pc = Poll{0, 0, nullptr}) {
  constexpr int NSM = OHARA_MEGA_NS, PR = 16 / NS;
  const int HD = H * Dh, PS = Dh + 32;
  const int nbh = B * H, total = B * HD;
  const int pass = (int)blockDim.x * 4;
  OHARA_LDS float* mw = (OHARA_LDS float*)mw_;
  OHARA_LDS float* ml = (OHARA_LDS float*)ml_;
  uint4 av[PR][NS];
  auto load = [&](int e0) {
#pragma unroll
    for (int r = 0; r < PR; ++r) {
      const int e = min(e0 + r * pass, total - 4);  // columns past the end read the last group again (not used):
      const int b = e / HD, hd = e - b * HD;        // no load behind a branch
      const float* base = pm + (size_t)(b * H + hd / Dh) * NSM * PS + (hd % Dh);
#pragma unroll
      for (int sp = 0; sp < NS; ++sp)  // slots past `used` are never written: read the last used one (weight 0)
        av[r][sp] = ldg16(base + (size_t)min(sp, used - 1) * PS);
    }
  };
  // the accumulator loads of the first round go out first: they do not depend on the chunk
  // weights, which are formed while they are in flight
  if (!TAGGED) load((int)threadIdx.x * 4);
  // NS lanes per (sequence, head): lane sp holds chunk sp's (max, sum); max and weighted sum by
  // shuffles inside the group
  for (int i0 = 0; i0 < nbh * NS; i0 += blockDim.x) {
    const int i = i0 + threadIdx.x;
    const int bh = i / NS, sp = i % NS;
    const bool in = bh < nbh && sp < used;
    float ms = -INFINITY, ls = 0.f;
    if (in) {
      if (TAGGED) {
        uint4 v;
        unsigned int spins = 0;
        do v = ld_coh16(pm + ((size_t)bh * NSM + sp) * PS + Dh);  // {max, tag}, {sum, tag}: two 8-byte loads
        while ((v.y != pc.tag || v.w != pc.tag) && !poll_expired(pc, spins));
        ms = __uint_as_float(v.x);
        ls = __uint_as_float(v.z);
      } else {
        const uint2 v = ldg8(pm + ((size_t)bh * NSM + sp) * PS + Dh);
        ms = __uint_as_float(v.x);
        ls = __uint_as_float(v.y);
      }
    }
    float M = ms;
    if (NS > 8) M = lane_xor_max<8>(M);
    if (NS > 4) M = lane_xor_max<4>(M);
    if (NS > 2) M = lane_xor_max<2>(M);
    if (NS > 1) M = lane_xor_max<1>(M);
    const float w = (ms == -INFINITY) ? 0.f : pow2_neg_int(ms - M);  // maxima are integers (log2 units): exact
    float Ls = ls * w;
    if (NS > 8) Ls = lane_xor_sum<8>(Ls);
    if (NS > 4) Ls = lane_xor_sum<4>(Ls);
    if (NS > 2) Ls = lane_xor_sum<2>(Ls);
    if (NS > 1) Ls = lane_xor_sum<1>(Ls);
    if (bh < nbh) mw[bh * NS + sp] = w;  // 0 for chunks that are not in use
    if (in && sp == 0) ml[bh] = Ls;
  }
  __syncthreads();
  asm volatile("" ::: "memory");  // compiler only (TAGGED): the accumulator loads stay behind the polls
  for (int e0 = threadIdx.x * 4; e0 < total; e0 += pass * PR) {
    if (TAGGED || e0 != (int)threadIdx.x * 4) load(e0);
#pragma unroll
    for (int r = 0; r < PR; ++r) {
      const int e = e0 + r * pass;
      if (e < total) {
        const int b = e / HD, hd = e - b * HD;
        const int bh = b * H + hd / Dh;
        float o[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int sp = 0; sp < NS; ++sp) {
          const float w = mw[bh * NS + sp];
          o[0] += __uint_as_float(av[r][sp].x) * w;
          o[1] += __uint_as_float(av[r][sp].y) * w;
          o[2] += __uint_as_float(av[r][sp].z) * w;
          o[3] += __uint_as_float(av[r][sp].w) * w;
        }
        const float inv = 1.0f / ml[bh];
        sts8(xs + (size_t)b * ldxs + hd, make_uint2(pack_bf(o[0] * inv, o[1] * inv), pack_bf(o[2] * inv, o[3] * inv)));
      }
    }
  }
}

// One pass for the small case (all OHARA_MEGA_NS chunks in use, one group of four columns per
// thread): every thread fetches the (max, sum) pairs itself, so there is a single round of loads
// and no workgroup barrier.
__device__ __forceinline__ void stage_attn_merge_small(bf16_t* xs, int ldxs, const float* pm, int B, int H, int Dh) {
  constexpr int NS = OHARA_MEGA_NS;
  const int HD = H * Dh, PS = Dh + 32;
  const int e = threadIdx.x * 4;
  if (e >= B * HD) return;
  const int b = e / HD, hd = e - b * HD;
  const int h = hd / Dh, d = hd - h * Dh;
  const float* base = pm + (size_t)(b * H + h) * NS * PS;
  uint2 mlv[NS];
  uint4 av[NS];
#pragma unroll
  for (int s = 0; s < NS; ++s) {
    mlv[s] = ldg8(base + (size_t)s * PS + Dh);
    av[s] = ldg16(base + (size_t)s * PS + d);
  }
  float M = -INFINITY;
#pragma unroll
  for (int s = 0; s < NS; ++s) M = fmaxf(M, __uint_as_float(mlv[s].x));
  float Ls = 0.f, o[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int s = 0; s < NS; ++s) {
    const float ms = __uint_as_float(mlv[s].x);
    const float w = (ms == -INFINITY) ? 0.f : pow2_neg_int(ms - M);  // maxima are integers (log2 units): exact
    Ls += __uint_as_float(mlv[s].y) * w;
    o[0] += __uint_as_float(av[s].x) * w;
    o[1] += __uint_as_float(av[s].y) * w;
    o[2] += __uint_as_float(av[s].z) * w;
    o[3] += __uint_as_float(av[s].w) * w;
  }
  const float inv = 1.0f / Ls;
  sts8(xs + (size_t)b * ldxs + hd, make_uint2(pack_bf(o[0] * inv, o[1] * inv), pack_bf(o[2] * inv, o[3] * inv)));
}

// Out-of-line copies of the merge, for kernels that want to keep their own code compact.
template <int NS, bool TAGGED = false>
__device__ __noinline__ void stage_attn_merge_call(bf16_t* xs, int ldxs, const float* pm, int B, int H, int Dh, float* mw,
                                                   float* ml, int used, uint32_t tag = 0, unsigned int limit = 0, unsigned int* err = nullptr) {
  stage_attn_merge<NS, TAGGED>(xs, ldxs, pm, B, H, Dh, mw, ml, used, Poll{tag, limit, err});  // (a struct would travel through memory)
}

// The power of two that the merge of `ns` chunks is specialised for (the chunk weights in LDS are laid
// out with this stride).
__host__ __device__ inline int attn_merge_width(int ns) {
  int w = 1;
  while (w < ns) w <<= 1;
  return w;
}

// The merge for `ns` chunks (any count up to OHARA_MEGA_NS: the specialisation for the next power of two
// runs with the chunks past `ns` weighing nothing).  INLINE: the five specialisations become part of the
// caller (no call in the layer loop: a call makes the caller wait for every load it has in flight, the
// weights fetched ahead included); otherwise they stay outside it, which keeps a kernel whose usual case
// is the small merge within the instruction cache.
template <bool INLINE, bool TAGGED = false>
__device__ __forceinline__ void stage_attn_merge_any(int ns, bf16_t* xs, int ldxs, const float* pm, int B, int H, int Dh,
                                                     float* mw, float* ml, const Poll pc = Poll{0, 0, nullptr}) {
  const int w = attn_merge_width(ns);
  if (!TAGGED && ns == OHARA_MEGA_NS && B * H * Dh <= 4 * 256) {  // (TAGGED: one lane polls one chunk's pair)
    stage_attn_merge_small(xs, ldxs, pm, B, H, Dh);
  } else if (TAGGED && w == 16) {
    // the usual width at batch 1, inline: a call would park the caller's prefetched weights in scratch memory
    stage_attn_merge<16, TAGGED>(xs, ldxs, pm, B, H, Dh, mw, ml, ns, pc);
  } else if (INLINE) {
    if (w == 16) stage_attn_merge<16, TAGGED>(xs, ldxs, pm, B, H, Dh, mw, ml, ns, pc);
    else if (w == 8) stage_attn_merge<8, TAGGED>(xs, ldxs, pm, B, H, Dh, mw, ml, ns, pc);
    else if (w == 4) stage_attn_merge<4, TAGGED>(xs, ldxs, pm, B, H, Dh, mw, ml, ns, pc);
    else if (w == 2) stage_attn_merge<2, TAGGED>(xs, ldxs, pm, B, H, Dh, mw, ml, ns, pc);
    else stage_attn_merge<1, TAGGED>(xs, ldxs, pm, B, H, Dh, mw, ml, ns, pc);
  } else {
    if (w == 16) stage_attn_merge_call<16, TAGGED>(xs, ldxs, pm, B, H, Dh, mw, ml, ns, pc.tag, pc.limit, pc.err);
    else if (w == 8) stage_attn_merge_call<8, TAGGED>(xs, ldxs, pm, B, H, Dh, mw, ml, ns, pc.tag, pc.limit, pc.err);
    else if (w == 4) stage_attn_merge_call<4, TAGGED>(xs, ldxs, pm, B, H, Dh, mw, ml, ns, pc.tag, pc.limit, pc.err);
    else if (w == 2) stage_attn_merge_call<2, TAGGED>(xs, ldxs, pm, B, H, Dh, mw, ml, ns, pc.tag, pc.limit, pc.err);
    else stage_attn_merge_call<1, TAGGED>(xs, ldxs, pm, B, H, Dh, mw, ml, ns, pc.tag, pc.limit, pc.err);
  }
}

// ---------------------------------------------------------------------------------------
// GEMM phase: strips of 16 packed rows, KP waves per strip, activations from LDS.  The
// weights of a workgroup's first strip(s) - and the residual it will add - are fetched
// into registers between arrive() and wait() of the barrier that precedes the phase.
// ---------------------------------------------------------------------------------------
enum { E_RESID = 1, E_SWIGLU = 2, E_ROPE = 3, E_LOGITS = 4, E_PART = 5, E_XNEXT = 6 };  // E_XNEXT: the whole down projection + residual (batch-1 kernels)

struct GemmP {
  const uint4* wp;
  int N, K;        // logical rows (for E_SWIGLU: hidden width F) and columns
  int nstrips;
  char* out;       // output mailbox (E_ROPE: q; E_RESID: x; E_SWIGLU: act) or logits
  int blk;         // its block size
  const char* resid;      // E_RESID: x mailbox to add ...
  const float* resid_parts;  // ... plus, when set, the partial sums of the previous block's down projection
  int resid_embed;        // E_RESID: add the embedding rows instead (first half layer)
  float* pout;            // E_PART: partial sums [part][b][n] (fp32, not rounded); K is split over
                          // OHARA_DOWN_SPLIT groups of workgroups, unit = part * nstrips + strip
  const int64_t* ids;     // E_RESID with resid == nullptr
  const bf16_t* table;
  int vocab;
  int H, Hkv, Dh, Tmax, pos;
  const bf16_t* cos;
  const bf16_t* sin;
  bf16_t* kc;
  bf16_t* vc;
  int valid;       // E_LOGITS: ids >= valid never win
  int ldo;         // E_LOGITS: row stride of the logits
  const bf16_t* norm_w;  // weights of the norm staged ahead of this phase (fetched with the weights when set)
  // batch-1 kernels with tagged hand-offs (TAG): where the epilogue leaves its row for the consumers that poll
  char* tout;      // E_RESID: the residual stream (besides `out`); E_SWIGLU: the activations; E_ROPE: the q rows
  char* tkv;       // E_ROPE: the new key row, then the new value row (besides the cache)
  const char* tresid;  // E_RESID (unless resid_embed), E_XNEXT: the tagged row that is added to the product
  uint32_t wlds_addr;  // E_XNEXT: LDS byte address of the workgroup's parked tiles, OHARA_LDS_PF per wave (gemm_prefetch_lds)
  Poll poll;
  ptrdiff_t tother;  // from a mailbox of this launch's set to the same mailbox of the other set
  int trow, tkv_row, tres_row;  // bytes between the rows (sequences) of the mailboxes tout, tkv and tresid
  int kv_i8;       // E_ROPE with polled hand-offs: the caches hold int8 codes (the new rows travel by mailbox only)
  int wg0;         // the workgroup that takes the phase's first unit (units go to wg0, wg0 + 1, ... round the grid)
};
// A workgroup's position in a phase whose units start at workgroup p.wg0.
__device__ __forceinline__ int phase_block(const GemmP& p) {
  const int v = (int)blockIdx.x - p.wg0;
  return v < 0 ? v + (int)gridDim.x : v;
}

struct GemmPre {  // one register buffer, reused by every phase (only one prefetch is live at a time)
  uint4 w[OHARA_MAX_PF];
  uint4 g[2];     // the lane's pieces of the weights of the norm staged ahead of the phase (GemmP::norm_w)
  uint2 r;        // E_RESID with embedding rows: the four residual values of this lane (first strip); E_ROPE: its cos / sin pairs
  // E_RESID (which fetches six weight tiles): w[OHARA_PRE_RESID .. +4] hold the residual's pieces as loaded -
  // the stream before the block and the four partial sums of the down projection - and the epilogue adds them
  // up (adding them here would make the prefetch wait for them before it goes on)
};
#define OHARA_PRE_RESID 18

// Work unit -> strip and this wave's k-steps [j0, j1).  E_PART: the units of K partition q follow
// those of partition q - 1, so the partitions of a strip land on different workgroups.
template <int KP, int EPI>
__device__ __forceinline__ bool gemm_unit(const GemmP& p, int unit, int kpart, int KS, int& strip, int& j0, int& j1) {
  int kq = 0, KSq = KS;
  strip = unit;
  bool live = unit < p.nstrips;
  if (EPI == E_PART) {
    kq = unit / p.nstrips;
    strip = unit - kq * p.nstrips;
    KSq = (KS + OHARA_DOWN_SPLIT - 1) / OHARA_DOWN_SPLIT;
    live = kq < OHARA_DOWN_SPLIT;
  }
  const int per = (KSq + KP - 1) / KP;
  const int kend = min(KS, (kq + 1) * KSq);
  j0 = kq * KSq + kpart * per;
  j1 = min(kend, j0 + per);
  return live;
}

// PO: first slot of pre.w this phase's tiles go to (several phases' weights can be held at once)
// (g, r: where the norm weights and the rotary pair / embedding residual go - pre.g and pre.r unless the caller keeps
// those of several phases at once)
// PAIR = false: E_ROPE without the rotary pair (it is the same for every layer: a caller that keeps it fetches it once)
template <int KP, int PF, int EPI, int PO = 0, bool PAIR = true>
__device__ __forceinline__ void gemm_prefetch(const GemmP& p, GemmPre& pre, int B, uint4 (&g_out)[2], uint2& r_out) {
  static_assert(PO + PF <= OHARA_MAX_PF, "prefetch buffer");
  constexpr int SPW = 4 / KP;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int sub = wave / KP, kpart = wave % KP;
  const int KS = (p.K + 31) >> 5;
  int strip, j0, j1;
  const bool live = gemm_unit<KP, EPI>(p, phase_block(p) * SPW + sub, kpart, KS, strip, j0, j1);
  // Everything else the phase reads that does not depend on the phase before it is requested here
  // too: cold reads from HBM behind the barrier would sit on the critical path of the phase.
  if (EPI == E_ROPE || EPI == E_SWIGLU || EPI == E_LOGITS) {
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      const int k = (c * 64 + lane) * 8;
      g_out[c] = (p.norm_w && wave < B && k < p.K) ? ldg16(p.norm_w + k) : make_uint4(0, 0, 0, 0);
    }
  }
  if (EPI == E_ROPE && PAIR) {
    const int m = lane & 15, g = lane >> 4;
    const int r0 = strip * 16 + 4 * g;
    const int nq = p.H * p.Dh, nk = p.Hkv * p.Dh;
    r_out = make_uint2(0, 0);
    if (live && kpart == 0 && m < B && r0 < nq + nk && p.pos >= 0 && p.pos < p.Tmax) {
      const int d = (r0 < nq ? r0 : r0 - nq) % p.Dh;
      r_out = make_uint2(ldg4(p.cos + (size_t)p.pos * (p.Dh >> 1) + (d >> 1)),
                         ldg4(p.sin + (size_t)p.pos * (p.Dh >> 1) + (d >> 1)));
    }
  }
  if (EPI == E_RESID) {
    const int m = lane & 15, g = lane >> 4;
    const int r0 = strip * 16 + 4 * g;
    r_out = make_uint2(0, 0);
    if (live && kpart == 0 && m < B && r0 < p.N && !p.tout) {  // (tagged mode: the residual is fetched by the phase itself)
      if (!p.resid_embed) {
        static_assert(EPI != E_RESID || PF <= OHARA_PRE_RESID, "the residual's pieces share the weight buffer");
        XRaw<4, true> t;
        x_fetch<4, true>(XParts{p.resid, p.resid_parts, p.blk, B, p.N}, m, r0, t);
        pre.w[OHARA_PRE_RESID] = t.xm;
#pragma unroll
        for (int q = 0; q < OHARA_DOWN_SPLIT; ++q) pre.w[OHARA_PRE_RESID + 1 + q] = t.pv[q][0];
      } else {
        int64_t id = ldg_i64(p.ids + m);
        if (id < 0 || id >= p.vocab) id = 0;
        r_out = ldg8(p.table + (size_t)id * p.N + r0);
      }
    }
  }
  // the weights last: the small loads above are then issued with nothing of this prefetch in flight
  // (placed behind the weight loads, the compiler made each of them wait for all of those first)
  // One running address, no test per tile: a tile past the wave's last k-step is that last tile again (finite
  // values that meet activations of zero), and a wave without a unit fetches nothing and never looks at its
  // slots.  (With an address and a branch per tile the compiler kept all of them - they do not change from
  // layer to layer - in scratch memory and waited for every earlier load before each reload.)
  if (live && j0 < j1) {
    const uint4* ptr = p.wp + ((size_t)strip * KS + j0) * 64 + lane;
    asm volatile("" : "+v"(ptr));  // formed here, not ahead of a loop around the caller (and kept until here)
    const int left = j1 - j0 - 1;
#pragma unroll
    for (int c = 0; c < PF; ++c) {
      pre.w[PO + c] = ldg16_nt(ptr);
      ptr += c < left ? 64 : 0;
    }
  }
}

template <int KP, int PF, int EPI, int PO = 0>
__device__ __forceinline__ void gemm_prefetch(const GemmP& p, GemmPre& pre, int B) {
  gemm_prefetch<KP, PF, EPI, PO>(p, pre, B, pre.g, pre.r);
}

// The weights of a workgroup's first unit straight into LDS (global_load_lds: 16 bytes per lane, a wave's
// load lands as one contiguous 1 KB tile; no registers are held while they travel): wave w's tile c at
// wl + (w * OHARA_LDS_PF + c) KB.  The wave that issued them waits for its own (vmcnt) before it reads.
template <int KP, int EPI>
__device__ __forceinline__ void gemm_prefetch_lds(const GemmP& p, char* wl) {
  constexpr int SPW = 4 / KP;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int sub = wave / KP, kpart = wave % KP;
  const int KS = (p.K + 31) >> 5;
  int strip, j0, j1;
  const bool live = gemm_unit<KP, EPI>(p, phase_block(p) * SPW + sub, kpart, KS, strip, j0, j1);
  if (!live) return;
  // a rolled loop with a running address: unrolled, the compiler computed all 24 addresses first, spilled
  // them, and waited for every earlier load before each reload
  const uint4* src = p.wp + ((size_t)strip * KS + j0) * 64 + lane;
  char* dst = wl + (size_t)wave * OHARA_LDS_PF * 1024;
  const int n = min(j1 - j0, OHARA_LDS_PF);
#pragma unroll 1
  for (int c = 0; c < n; ++c) {
    __builtin_amdgcn_global_load_lds((const OHARA_GLOBAL void*)src, (OHARA_LDS void*)dst, 16, 0, 0);
    src += 64;
    dst += 1024;
  }
}

template <int KP, int PF, int EPI, class PROF, int PO = 0, bool TAG = false>
__device__ __forceinline__ void gemm_phase(const GemmP& p, const GemmPre& pre, const bf16_t* xs, int ldxs, int B,
                                           float* red, float& best_v, int& best_i, PROF& pf) {
  constexpr int SPW = 4 / KP;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m = lane & 15, g = lane >> 4;
  const int sub = wave / KP, kpart = wave % KP;
  const int KS = (p.K + 31) >> 5;
  const int nwg = gridDim.x;
  const int nunits = EPI == E_PART ? p.nstrips * OHARA_DOWN_SPLIT : p.nstrips;
  const int iters = (nunits + nwg * SPW - 1) / (nwg * SPW);
  const bool mine = m < B;
  const bf16_t* xrow = xs + (size_t)m * ldxs + 8 * g;

#pragma unroll 1
  for (int it = 0; it < iters; ++it) {
    const int unit = (it * nwg + phase_block(p)) * SPW + sub;
    int strip, j0, j1;
    const bool live = gemm_unit<KP, EPI>(p, unit, kpart, KS, strip, j0, j1);
    f32x4 acc = (f32x4){0.f, 0.f, 0.f, 0.f};
    // TAG: the four residual values of this lane (two entries of a tagged row that has been visible for a
    // while), requested ahead of the products and checked in the epilogue
    const bool tres = TAG && (EPI == E_XNEXT || (EPI == E_RESID && !p.resid_embed)) && live && kpart == 0 && mine &&
                      strip * 16 + 4 * g < p.N;
    uint2 rx = make_uint2(0, 0);
    if (tres) rx = ld_coh8(p.tresid + (size_t)(B == 1 ? 0 : m) * p.tres_row + (size_t)(strip * 16 + 4 * g) * 2);
    if (live) {
      const uint4* wrow = p.wp + (size_t)strip * KS * 64 + lane;
#pragma unroll 1
      for (int jc = j0; jc < j1; jc += PF) {
        uint4 wv[PF];
        uint4 xv[PF];
        // The usual case - all PF k-steps of the chunk exist and lie inside K - runs without a predicate per
        // k-step: one wave per SIMD issues an instruction every few cycles, so a phase costs what its
        // instruction count costs, and a predicated k-step is fifteen instructions where three do (weight
        // tile from LDS / nothing for a register tile, activations from LDS, product).  Lanes of batch
        // columns that do not exist read row 0: their products land in output columns nobody stores.
        const bool full = jc + PF <= j1 && 32 * (jc + PF) <= p.K;
        if (full) {
          const uint32_t xa = (uint32_t)(uintptr_t)(const OHARA_LDS bf16_t*)(xs + (size_t)(mine ? m : 0) * ldxs + 8 * g) + 64u * jc;
          if (EPI == E_XNEXT && it == 0 && jc - j0 + PF <= OHARA_LDS_PF) {  // parked in LDS by gemm_prefetch_lds
            if (jc == j0) wait_own_stores();  // this wave's own loads into LDS have landed
            const uint32_t wa = p.wlds_addr + ((uint32_t)(wave * OHARA_LDS_PF + (jc - j0)) * 64 + lane) * 16;
#pragma unroll
            for (int c = 0; c < PF; ++c) wv[c] = lds16_at(wa + c * 1024);
          } else if (EPI != E_XNEXT && it == 0 && jc == j0) {
#pragma unroll
            for (int c = 0; c < PF; ++c) wv[c] = pre.w[PO + c];
          } else {
#pragma unroll
            for (int c = 0; c < PF; ++c) wv[c] = ldg16_nt(wrow + (size_t)(jc + c) * 64);
          }
#pragma unroll
          for (int c = 0; c < PF; ++c) xv[c] = lds16_at(xa + 64u * c);
        } else {
          if (EPI == E_XNEXT && it == 0 && jc - j0 + PF <= OHARA_LDS_PF) {
            if (jc == j0) wait_own_stores();
#pragma unroll
            for (int c = 0; c < PF; ++c)
              wv[c] = (jc + c < j1) ? lds16_at(p.wlds_addr + ((uint32_t)(wave * OHARA_LDS_PF + (jc - j0) + c) * 64 + lane) * 16)
                                    : make_uint4(0, 0, 0, 0);
          } else if (EPI != E_XNEXT && it == 0 && jc == j0) {
#pragma unroll
            for (int c = 0; c < PF; ++c) wv[c] = pre.w[PO + c];
          } else {
#pragma unroll
            for (int c = 0; c < PF; ++c)
              wv[c] = (jc + c < j1) ? ldg16_nt(wrow + (size_t)(jc + c) * 64) : make_uint4(0, 0, 0, 0);
          }
          // The activations of all PF k-steps are read from LDS before the first product: they do not
          // depend on the weights, and left next to their products every read's latency is exposed
          // (read, wait, product, PF times) on the critical path of the phase.
#pragma unroll
          for (int c = 0; c < PF; ++c) {
            xv[c] = make_uint4(0, 0, 0, 0);
            if (mine && jc + c < j1 && 32 * (jc + c) + 8 * g < p.K)
              xv[c] = *reinterpret_cast<const uint4*>(xrow + 32 * (jc + c));
          }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int c = 0; c < PF; ++c)
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wv[c]),
                                                        __builtin_bit_cast(bf16x8, xv[c]), acc, 0, 0, 0);
      }
    }
    if (it == 0) pf.stamp();  // MFMAs issued
    if (KP > 1) {
      if (kpart > 0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) red[((wave * 64) + lane) * 4 + i] = acc[i];
      }
      __syncthreads();
      if (kpart == 0) {
        // all partial tiles are read before the first add (same order of adds; the reads overlap)
        f32x4 part[KP > 1 ? KP - 1 : 1];
#pragma unroll
        for (int w = 1; w < KP; ++w) part[w - 1] = *reinterpret_cast<const f32x4*>(red + (((wave + w) * 64) + lane) * 4);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int w = 1; w < KP; ++w)
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[i] += part[w - 1][i];
      }
    }
    if (it == 0) pf.stamp();  // cross-wave sum done
    if (live && kpart == 0 && mine) {
      const int b = B == 1 ? 0 : m;  // (a single sequence: the row offsets below fold away)
      const int r0 = strip * 16 + 4 * g;
      const float y0 = rbf(acc[0]), y1 = rbf(acc[1]), y2 = rbf(acc[2]), y3 = rbf(acc[3]);
      if (EPI == E_XNEXT || (TAG && EPI == E_RESID)) {  // batch 1: the row goes to the tagged mailbox only
        if (r0 < p.N) {
          uint2 r = make_uint2(0, 0);
          if (tres) {
            unsigned int spins = 0;
            while (rx.x == OHARA_UNWRITTEN || rx.y == OHARA_UNWRITTEN) {
              if (poll_expired(p.poll, spins)) break;
              rx = ld_coh8(p.tresid + (size_t)b * p.tres_row + (size_t)r0 * 2);
            }
            r = rx;
          } else {  // the first half layer: the embedding row (llama.py:310)
            int64_t id = ldg_i64(p.ids + b);
            if (id < 0 || id >= p.vocab) id = 0;
            r = ldg8(p.table + (size_t)id * p.N + r0);
          }
          mb_st8(p.tout + (size_t)b * p.trow, p.tother, r0, pack_bf(lo_bf(r.x) + y0, hi_bf(r.x) + y1),
                 pack_bf(lo_bf(r.y) + y2, hi_bf(r.y) + y3));
        }
      } else if (EPI == E_RESID) {  // N % 4 == 0 is required by the entry point
        if (r0 < p.N) {
          uint2 r = pre.r;
          if (it == 0 && !p.resid_embed) {
            XRaw<4, true> t;
            t.xm = pre.w[OHARA_PRE_RESID];
#pragma unroll
            for (int q = 0; q < OHARA_DOWN_SPLIT; ++q) t.pv[q][0] = pre.w[OHARA_PRE_RESID + 1 + q];
            uint32_t w[2];
            x_combine<4, true>(t, w);
            r = make_uint2(w[0], w[1]);
          }
          if (it > 0) {
            if (!p.resid_embed) {
              uint32_t w[2];
              x_load<4, true>(XParts{p.resid, p.resid_parts, p.blk, B, p.N}, b, r0, w);
              r = make_uint2(w[0], w[1]);
            } else {
              int64_t id = ldg_i64(p.ids + b);
              if (id < 0 || id >= p.vocab) id = 0;
              r = ldg8(p.table + (size_t)id * p.N + r0);
            }
          }
          const uint2 xo = make_uint2(pack_bf(lo_bf(r.x) + y0, hi_bf(r.x) + y1), pack_bf(lo_bf(r.y) + y2, hi_bf(r.y) + y3));
          st_coh8(const_cast<char*>(xm_addr(p.out, p.blk, b, r0)), xo);
        }
      } else if (EPI == E_PART) {  // the raw fp32 sums of this K partition
        if (r0 < p.N) {
          float* o = const_cast<float*>(parts_addr(p.pout, p.nstrips, B, unit / p.nstrips, b, r0));
          st_coh8(o, make_uint2(__float_as_uint(acc[0]), __float_as_uint(acc[1])));
          st_coh8(o + 2, make_uint2(__float_as_uint(acc[2]), __float_as_uint(acc[3])));
        }
      } else if (EPI == E_LOGITS) {
        const float v[4] = {y0, y1, y2, y3};
        bf16_t* o = reinterpret_cast<bf16_t*>(p.out) + (size_t)b * p.ldo + r0;
        if (r0 + 3 < p.N && ((p.ldo & 3) == 0)) {
          stg8(o, make_uint2(pack_bf(v[0], v[1]), pack_bf(v[2], v[3])));
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
          if (TAG) mb_st4(p.tout + (size_t)b * p.trow, p.tother, f, pack_bf(s0 * y2, s1 * y3));
          else st_coh4(const_cast<char*>(am_addr(p.out, p.blk, b, f)), pack_bf(s0 * y2, s1 * y3));
        }
      } else {  // E_ROPE
        const int nq = p.H * p.Dh, nk = p.Hkv * p.Dh;
        if (r0 < nq + 2 * nk && p.pos >= 0 && p.pos < p.Tmax) {
          float v[4] = {y0, y1, y2, y3};
          char* o;
          if (r0 < nq + nk) {
            const int d = (r0 < nq ? r0 : r0 - nq) % p.Dh;
            const uint32_t cs = it == 0 ? pre.r.x : ldg4(p.cos + (size_t)p.pos * (p.Dh >> 1) + (d >> 1));
            const uint32_t sn = it == 0 ? pre.r.y : ldg4(p.sin + (size_t)p.pos * (p.Dh >> 1) + (d >> 1));
            const float c2[2] = {lo_bf(cs), hi_bf(cs)}, s2[2] = {lo_bf(sn), hi_bf(sn)};
#pragma unroll
            for (int pr = 0; pr < 2; ++pr) {
              const float e = v[2 * pr], od = v[2 * pr + 1];
              v[2 * pr] = __fsub_rn(__fmul_rn(e, c2[pr]), __fmul_rn(od, s2[pr]));
              v[2 * pr + 1] = __fadd_rn(__fmul_rn(e, s2[pr]), __fmul_rn(od, c2[pr]));
            }
            o = (r0 < nq) ? const_cast<char*>(xm_addr(p.out, p.blk, b, r0))
                          : reinterpret_cast<char*>(p.kc + (((size_t)b * p.Tmax + p.pos) * p.Hkv) * p.Dh + (r0 - nq));
          } else {
            o = reinterpret_cast<char*>(p.vc + (((size_t)b * p.Tmax + p.pos) * p.Hkv) * p.Dh + (r0 - nq - nk));
          }
          const uint2 ro = make_uint2(pack_bf(v[0], v[1]), pack_bf(v[2], v[3]));
          if (TAG) {  // attention polls for the q row and for the new key / value rows; the cache rows are for later steps
            if (r0 < nq) mb_st8(p.tout + (size_t)b * p.trow, p.tother, r0, ro.x, ro.y);
            else mb_st8(p.tkv + (size_t)b * p.tkv_row, p.tother, r0 - nq, ro.x, ro.y);
          }
          if (!TAG || (r0 >= nq && !p.kv_i8)) st_coh8(o, ro);  // (an int8 cache gets the row from the attention phase)
        }
      }
    }
    if (KP > 1) __syncthreads();
  }
}

// ---------------------------------------------------------------------------------------
// Vocabulary projection (one wave per strip, the whole K in that wave, running arg-max): the
// phase that is bound by HBM bandwidth, so it must never run out of loads in flight.  The
// (strip, 12-k-step chunk) pairs of a wave form one sequence; two register buffers of twelve
// tiles take turns along it: while one is multiplied, the other is on its way, and each is
// requested again the moment its products are issued.  No load sits behind a branch or is
// touched before use (chunks past the end read a valid tile that is never multiplied), so the
// compiler waits for exactly the buffer it needs.  Same products in the same order as
// gemm_phase<1, 24, E_LOGITS>, whose prefetch (the first strip's first 24 k-steps) it takes over.
// ---------------------------------------------------------------------------------------
// `staged` (a byte address in LDS, 0 = nothing): the tiles of this wave's SECOND strip were parked there
// ahead of the phase (tile c at staged + c KB; strips of at most 24 k-steps); they are multiplied while the
// first loads from memory are on their way.  `extra`: the first chunk (HC tiles) of the THIRD strip follows
// them there (strips of exactly two chunks).
template <class PROF>
__device__ __forceinline__ void lm_phase(const GemmP& p, const GemmPre& pre, const bf16_t* xs, int ldxs, int B,
                                         float& best_v, int& best_i, PROF& pf, uint32_t staged = 0, bool extra = false) {
  constexpr int HC = 12;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m = lane & 15, g = lane >> 4;
  const int KS = (p.K + 31) >> 5;
  const int nwg = gridDim.x;
  const int iters = (p.nstrips + nwg * 4 - 1) / (nwg * 4);
  const int ncps = (KS + HC - 1) / HC;  // chunks per strip
  const int total = iters * ncps;
  const bool mine = m < B;
  const bf16_t* xrow = xs + (size_t)m * ldxs + 8 * g;
  auto strip_of = [&](int it) { return (it * nwg + (int)blockIdx.x) * 4 + wave; };
  auto load = [&](uint4 (&w)[HC], int q) {
    const int it = q / ncps, c = q - it * ncps;
    const int st = strip_of(it);
    const uint4* wrow = p.wp + (size_t)(st < p.nstrips ? st : 0) * KS * 64 + lane;
#pragma unroll
    for (int cc = 0; cc < HC; ++cc) w[cc] = ldg16_nt(wrow + (size_t)min(c * HC + cc, KS - 1) * 64);
  };
  uint4 wa[HC], wb[HC];
#pragma unroll
  for (int cc = 0; cc < HC; ++cc) wa[cc] = pre.w[cc];
  if (ncps >= 2) {
#pragma unroll
    for (int cc = 0; cc < HC; ++cc) wb[cc] = pre.w[HC + cc];
  } else {
    load(wb, staged ? 2 : 1);
  }
  f32x4 acc = (f32x4){0.f, 0.f, 0.f, 0.f};
  auto process = [&](const uint4 (&w)[HC], int q) {
    const int it = q / ncps, c = q - it * ncps;
    const int strip = strip_of(it);
    if (c == 0) acc = (f32x4){0.f, 0.f, 0.f, 0.f};
    if (strip >= p.nstrips) return;
    uint4 xv[HC];
#pragma unroll
    for (int cc = 0; cc < HC; ++cc) {
      const int j = c * HC + cc;
      xv[cc] = make_uint4(0, 0, 0, 0);  // k-steps past K multiply zeros
      if (mine && j < KS && 32 * j + 8 * g < p.K) xv[cc] = *reinterpret_cast<const uint4*>(xrow + 32 * j);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int cc = 0; cc < HC; ++cc)
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, w[cc]), __builtin_bit_cast(bf16x8, xv[cc]),
                                                    acc, 0, 0, 0);
    if (c != ncps - 1 || !mine) return;
    const int b = m;
    const int r0 = strip * 16 + 4 * g;
    const float v[4] = {rbf(acc[0]), rbf(acc[1]), rbf(acc[2]), rbf(acc[3])};
    bf16_t* o = reinterpret_cast<bf16_t*>(p.out) + (size_t)b * p.ldo + r0;
    if (r0 + 3 < p.N && ((p.ldo & 3) == 0)) {
      stg8(o, make_uint2(pack_bf(v[0], v[1]), pack_bf(v[2], v[3])));
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
  };
  // chunks that come from memory, in order: all of them but the staged ones (chunks ncps .. 2 ncps - 1, and chunk
  // 2 ncps with `extra`)
  const int nskip = staged ? ncps + (extra ? 1 : 0) : 0;
  auto gq = [&](int k) { return (staged && k >= ncps) ? k + nskip : k; };
  const int nglob = total - nskip;
  for (int k = 0; k < nglob; k += 2) {
    process(wa, gq(k));
    load(wa, gq(k + 2));
    if (k == 0) {
      pf.stamp();  // first products issued
      pf.stamp();
    }
    if (k + 1 < nglob) {
      process(wb, gq(k + 1));
      load(wb, gq(k + 3));
    }
    if (k == 0 && staged) {
      wait_own_stores();  // this wave's own loads into LDS have landed (requested layers ago)
      for (int c = 0; c < ncps; ++c) {
        uint4 wc[HC];
#pragma unroll
        for (int cc = 0; cc < HC; ++cc) wc[cc] = lds16_at(staged + ((uint32_t)min(c * HC + cc, KS - 1) * 64 + lane) * 16);
        process(wc, ncps + c);
      }
      if (extra) {  // the third strip's first chunk: its second one is the next chunk from memory
        uint4 wc[HC];
#pragma unroll
        for (int cc = 0; cc < HC; ++cc) wc[cc] = lds16_at(staged + ((uint32_t)(KS + cc) * 64 + lane) * 16);
        process(wc, 2 * ncps);
      }
    }
  }
}

// ---------------------------------------------------------------------------------------
// attention phase: items (sequence, kv head, chunk); writes partial triples.  The K/V
// tiles of a wave's first 16 positions are fetched before the barrier.
// ---------------------------------------------------------------------------------------
template <int D>
struct AttnPre {
  uint4 k[D / 32];
  uint4 v[D / 32];  // NV = 16 / (64 / (D / 8)) = D / 32
};

// One 16-position tile: positions >= t1 load nothing; position `coh_pos` (the row appended in
// this step, or -1) is read with device-scope loads.
template <int D>
__device__ __forceinline__ void attn_tile_load(const bf16_t* kb, const bf16_t* vb, size_t row, int tb, int t1,
                                               int coh_pos, uint4* kv, uint4* vv) {
  constexpr int NC = D / 32, DC = D / 8, PP = 64 / DC, NV = 16 / PP;
  const int lane = threadIdx.x & 63;
  const int p = lane & 15, dq = lane >> 4;
  const int pp = lane / DC, dc = lane % DC;
  const int pos = tb + p;
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const bf16_t* src = kb + (size_t)pos * row + (4 * c + dq) * 8;
    kv[c] = pos < t1 ? (pos == coh_pos ? ld_coh16(src) : ldg16_nt(src)) : make_uint4(0, 0, 0, 0);
  }
#pragma unroll
  for (int c = 0; c < NV; ++c) {
    const int vp = tb + c * PP + pp;
    const bf16_t* src = vb + (size_t)vp * row + dc * 8;
    vv[c] = vp < t1 ? (vp == coh_pos ? ld_coh16(src) : ldg16_nt(src)) : make_uint4(0, 0, 0, 0);
  }
}

// The same tile inside the loop over a chunk: every load issued without a branch (positions past
// the chunk repeat its last row; their scores are masked and their weights are zero), so that the
// compiler can count the loads in flight and wait for the current tile only while the next one is
// on its way.  The row appended in this step is then fetched again with device-scope loads by the
// lanes that hold it (a branch the whole wave takes or skips).
// `last`: the last position these loads may touch (t1 - 1; one less where the row appended in this step
// is not in the cache yet and will be patched in from its tagged mailbox).
template <int D>
__device__ __forceinline__ void attn_tile_load_u(const bf16_t* kb, const bf16_t* vb, size_t row, int tb, int t1,
                                                 int coh_pos, uint4* kv, uint4* vv, int last) {
  constexpr int NC = D / 32, DC = D / 8, PP = 64 / DC, NV = 16 / PP;
  const int lane = threadIdx.x & 63;
  const int p = lane & 15, dq = lane >> 4;
  const int pp = lane / DC, dc = lane % DC;
  const int pos = min(tb + p, last);
#pragma unroll
  for (int c = 0; c < NC; ++c) kv[c] = ldg16_nt(kb + (size_t)pos * row + (4 * c + dq) * 8);
#pragma unroll
  for (int c = 0; c < NV; ++c) {
    const int vp = min(tb + c * PP + pp, last);
    vv[c] = ldg16_nt(vb + (size_t)vp * row + dc * 8);
  }
  if (coh_pos >= tb && coh_pos < tb + 16) {  // wave-uniform: this tile holds the appended row
    if (pos == coh_pos) {
#pragma unroll
      for (int c = 0; c < NC; ++c) kv[c] = ld_coh16(kb + (size_t)pos * row + (4 * c + dq) * 8);
    }
#pragma unroll
    for (int c = 0; c < NV; ++c) {
      const int vp = min(tb + c * PP + pp, t1 - 1);
      if (vp == coh_pos) vv[c] = ld_coh16(vb + (size_t)vp * row + dc * 8);
    }
  }
}

__device__ __forceinline__ void attn_item_range(int item, int ns, int Hkv, int L, int& b, int& kvh, int& split, int& t0,
                                                int& t1) {
  const int chunk = (((L + ns - 1) / ns) + 15) & ~15;
  split = item % ns;
  kvh = (item / ns) % Hkv;
  b = item / (ns * Hkv);
  t0 = split * chunk;
  t1 = min(L, t0 + chunk);
}

// The first tile of each wave's first item, if it lies wholly below the row being appended.
template <int D>
__device__ __forceinline__ bool attn_first_tile_prefetchable(int t0, int t1, int L) {
  const int tb = t0 + (threadIdx.x >> 6) * 16;
  return tb + 16 <= min(t1, L - 1);
}

template <int D>
__device__ __forceinline__ void attn_prefetch(int B, int Hkv, int Tmax, int ns, const bf16_t* kc, const bf16_t* vc,
                                              int L, AttnPre<D>& pre) {
  const int wave = threadIdx.x >> 6;
  const size_t row = (size_t)Hkv * D;
  int b, kvh, split, t0, t1;
  attn_item_range(blockIdx.x, ns, Hkv, L, b, kvh, split, t0, t1);
  const bool has = (int)blockIdx.x < B * Hkv * ns && attn_first_tile_prefetchable<D>(t0, t1, L);
  const bf16_t* kb = kc + (size_t)b * Tmax * row + (size_t)kvh * D;
  const bf16_t* vb = vc + (size_t)b * Tmax * row + (size_t)kvh * D;
  attn_tile_load<D>(kb, vb, row, t0 + wave * 16, has ? t1 : 0, -1, pre.k, pre.v);
}

// The row appended in this step, as the wave staged it in its LDS ([... | new key row | new value row], see
// attn_phase): the lanes of the tile at `tb` that hold position `pos_new` take their pieces.
template <int D>
__device__ __forceinline__ void attn_new_row_staged(const char* krow, int tb, int t1, int pos_new, uint4* kv, uint4* vv) {
  constexpr int NC = D / 32, DC = D / 8, PP = 64 / DC, NV = 16 / PP;
  const int lane = threadIdx.x & 63;
  const int p = lane & 15, dq = lane >> 4;
  const int pp = lane / DC, dc = lane % DC;
  if (min(tb + p, t1 - 1) == pos_new) {
#pragma unroll
    for (int c = 0; c < NC; ++c) kv[c] = lds16(krow + (4 * c + dq) * 16);
  }
#pragma unroll
  for (int c = 0; c < NV; ++c)
    if (min(tb + c * PP + pp, t1 - 1) == pos_new) vv[c] = lds16(krow + (DC + dc) * 16);
}

// ---- the int8 cache in the polled builds (ohara/modules/kv_cache.py:15-32, 94-102, 116-118) -------------------
// A tile as loaded: the codes of this lane's K pieces and V rows and the rows' (scale, minimum) pairs - half the
// registers of a bf16 tile; they become the bf16 values the reference's read returns (common.h: dequant4)
// where the bf16 path copies the next tile over the current one.
template <int D>
struct AttnRaw {
  uint2 k[D / 32];    // piece 4 c + dq (8 codes) of row tb + p
  uint2 kst;          // (key scale, key minimum) of that row
  uint2 v[D / 32];    // columns 8 dc .. of row tb + c * PP + pp
  uint2 vst[D / 32];  // (value scale, value minimum) of those rows
};
// st: the statistics records of this (sequence, KV head): 4 floats per position
template <int D>
__device__ __forceinline__ void attn_tile_load_i8(const int8_t* kb, const int8_t* vb, const float* st, size_t row, int tb,
                                                  int last, AttnRaw<D>& r) {
  constexpr int NC = D / 32, DC = D / 8, PP = 64 / DC, NV = 16 / PP;
  const int lane = threadIdx.x & 63;
  const int p = lane & 15, dq = lane >> 4;
  const int pp = lane / DC, dc = lane % DC;
  const int pos = min(tb + p, last);
  r.kst = ldg8(st + (size_t)pos * 4);
#pragma unroll
  for (int c = 0; c < NC; ++c) r.k[c] = ldg8(kb + (size_t)pos * row + (4 * c + dq) * 8);
#pragma unroll
  for (int c = 0; c < NV; ++c) {
    const int vp = min(tb + c * PP + pp, last);
    r.v[c] = ldg8(vb + (size_t)vp * row + dc * 8);
    r.vst[c] = ldg8(st + (size_t)vp * 4 + 2);
  }
}
template <int D>
__device__ __forceinline__ void attn_tile_dequant(const AttnRaw<D>& r, uint4* kv, uint4* vv) {
  constexpr int NC = D / 32, NV = D / 32;
  const float ks = __uint_as_float(r.kst.x), km = __uint_as_float(r.kst.y);
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const uint2 lo = dequant4(r.k[c].x ^ 0x80808080u, ks, km), hi = dequant4(r.k[c].y ^ 0x80808080u, ks, km);
    kv[c] = make_uint4(lo.x, lo.y, hi.x, hi.y);
  }
#pragma unroll
  for (int c = 0; c < NV; ++c) {
    const float vs = __uint_as_float(r.vst[c].x), vm = __uint_as_float(r.vst[c].y);
    const uint2 lo = dequant4(r.v[c].x ^ 0x80808080u, vs, vm), hi = dequant4(r.v[c].y ^ 0x80808080u, vs, vm);
    vv[c] = make_uint4(lo.x, lo.y, hi.x, hi.y);
  }
}
// The row appended in this step, int8 cache.  The wave whose tile holds position `pos_new` has the head's new key and
// value rows from the mailbox with every lane holding one bf16 pair of them (w[j]: pair lane + 64 j of [key row | value
// row], D / 64 pairs a lane), and quantises them as the cache's append does - minimum and maximum over the head's row,
// scale = max(bf16(bf16(max - min) / 255), bf16(1e-8)), code = clamp(round(bf16(bf16(bf16(x - min) / scale) - 128))),
// every op rounded to bf16 as the reference's tensor ops in the cache dtype round (kv_cache.py:23-26; csrc/kv_int8.hip)
// - writes codes and statistics to the cache, and hands the values a read of those codes returns to the lanes of the
// tile that hold the position through `stage` (2 D bf16 of LDS that only this wave touches).  Spread over the wave
// the divisions cost a fifth of a microsecond; done by the four lanes that hold the key row they cost two.
template <int D>
__device__ __forceinline__ void attn_new_row_i8(const uint32_t* w, int8_t* kq, int8_t* vq, float* st, size_t row, int tb,
                                                int t1, int pos_new, uint4* kv, uint4* vv, float* stage) {
  constexpr int NC = D / 32, DC = D / 8, PP = 64 / DC, NV = 16 / PP;
  constexpr int W = D / 2;    // pairs per row
  constexpr int NW = D / 64;  // pairs per lane
  const int lane = threadIdx.x & 63;
  uint32_t* stw = reinterpret_cast<uint32_t*>(stage);
#pragma unroll
  for (int j = 0; j < NW; ++j) {
    const int i = lane + 64 * j;
    const bool is_v = i >= W;
    const int ir = is_v ? i - W : i;
    const float x0 = lo_bf(w[j]), x1 = hi_bf(w[j]);
    // over the W lanes that share the row (the whole wave, or its half)
    const float mn = lanes_min<(W < 64 ? W : 64) / 2, 1>(fminf(x0, x1));
    const float mx = lanes_max<(W < 64 ? W : 64) / 2, 1>(fmaxf(x0, x1));
    const float scale = fmaxf(rbf(rbf(mx - mn) / 255.0f), rbf(1e-8f));
    const float t0 = rbf(rbf(rbf(x0 - mn) / scale) - 128.0f), t1q = rbf(rbf(rbf(x1 - mn) / scale) - 128.0f);
    const int q0 = (int)fminf(fmaxf(rintf(t0), -128.f), 127.f), q1 = (int)fminf(fmaxf(rintf(t1q), -128.f), 127.f);
    int8_t* dst = (is_v ? vq : kq) + (size_t)pos_new * row + 2 * ir;
    *reinterpret_cast<uint16_t*>(dst) = (uint16_t)(((uint32_t)q0 & 0xffu) | (((uint32_t)q1 & 0xffu) << 8));
    if (ir == 0) stg8(st + (size_t)pos_new * 4 + (is_v ? 2 : 0), make_uint2(__float_as_uint(scale), __float_as_uint(mn)));
    stw[i] = pack_bf(__fmaf_rn((float)(q0 + 128), scale, mn), __fmaf_rn((float)(q1 + 128), scale, mn));
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  // the lanes of the tile that hold the position (and those past the chunk's end that repeat it, which weigh nothing)
  const int p = lane & 15, dq = lane >> 4;
  const int pp = lane / DC, dc = lane % DC;
  const uint4* sv = reinterpret_cast<const uint4*>(stage);
  if (min(tb + p, t1 - 1) == pos_new) {
#pragma unroll
    for (int c = 0; c < NC; ++c) kv[c] = sv[4 * c + dq];
  }
#pragma unroll
  for (int c = 0; c < NV; ++c)
    if (min(tb + c * PP + pp, t1 - 1) == pos_new) vv[c] = sv[W / 4 + dc];
}

// TAG (batch 1): the q row and the row appended in this step come from tagged mailboxes (qt, kvt) that
// are polled for - there is no barrier between the projection that writes them and this phase.
// I8 (with TAG only): kc / vc are the int8 caches, `stats` their (sequence, KV head, position) records.
// AHEAD (with TAG only): a wave's second tile is requested before the poll for q (the single-sequence build: with more
// sequences a chunk is many tiles and the registers the request holds across the poll are spilled).
template <int D, int G, bool TAG = false, bool I8 = false, bool AHEAD = false>
__device__ __forceinline__ void attn_phase(int B, int H, int Hkv, int Tmax, int blk_x, int ns, const AttnPre<D>& pre,
                                           const char* qm, float* pm, const bf16_t* kc, const bf16_t* vc, int L,
                                           float* lds, const char* qt = nullptr, const char* kvt = nullptr,
                                           const Poll pc = Poll{0, 0, nullptr}, bool announce = false, int q_row = 0,
                                           int kv_row = 0,  // q_row, kv_row: bytes between the sequences' rows of qt, kvt
                                           float* stats = nullptr,
                                           float* wave_lds = nullptr) {  // TAG: 1 KB of LDS per wave, free during this phase
  static_assert(!I8 || TAG, "the int8 cache is served by the polled builds");
  constexpr int NC = D / 32, DC = D / 8, PP = 64 / DC, NV = 16 / PP;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int p = lane & 15;
  const int dq = lane >> 4;
  const int pp = lane / DC, dc = lane % DC;
  const float scale = (1.0f / sqrtf((float)D)) * OHARA_LOG2E;  // scores in log2 units (common.h: softmax bookkeeping)
  float* s_m = lds;                 // [4][G]
  float* s_l = lds + 4 * G;         // [4][G]
  float* s_acc = lds + 8 * G;       // [4][G][D]
  const int nitems = B * Hkv * ns;
  const size_t row = (size_t)Hkv * D;
  const int PS = D + 32;
  bool first = true;
  for (int item = blockIdx.x; item < nitems; item += gridDim.x) {
    int b, kvh, split, t0, t1;
    attn_item_range(item, ns, Hkv, L, b, kvh, split, t0, t1);
    if (B == 1) b = 0;  // (a single sequence: the row offsets below fold away)
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
      // the tile after the current one is in flight while the current one is consumed
      const bool use_pre = !I8 && first && attn_first_tile_prefetchable<D>(t0, t1, L);
      uint4 ka[NC], va[NV], kn[NC], vn[NV];
      int tb = t0 + wave * 16;
      const int coh = TAG ? -1 : L - 1;  // TAG: the appended row is patched in from the tagged mailbox below ...
      const int last = TAG ? max(min(t1, L - 1) - 1, 0) : t1 - 1;  // ... and its cache row is not touched
      // int8 cache: the codes of (sequence b, KV head kvh) and their records
      int8_t* kq8 = reinterpret_cast<int8_t*>(const_cast<bf16_t*>(kc)) + (size_t)b * Tmax * row + (size_t)kvh * D;
      int8_t* vq8 = reinterpret_cast<int8_t*>(const_cast<bf16_t*>(vc)) + (size_t)b * Tmax * row + (size_t)kvh * D;
      float* stb = stats + ((size_t)b * Hkv + kvh) * Tmax * 4;
      AttnRaw<D> raw;
      if (I8) {
        attn_tile_load_i8<D>(kq8, vq8, stb, row, tb, last, raw);
      } else if (use_pre) {
#pragma unroll
        for (int c = 0; c < NC; ++c) ka[c] = pre.k[c];
#pragma unroll
        for (int c = 0; c < NV; ++c) va[c] = pre.v[c];
      } else {
        attn_tile_load_u<D>(kb, vb, row, tb, t1, coh, ka, va, last);
      }
      // (int8: the first tile's codes become values before q is polled for - a wave's loads return in order anyway)
      if constexpr (I8) attn_tile_dequant<D>(raw, ka, va);
      // Polled builds: what the wave needs from the mailboxes - the group's q rows, and the row appended in this step if
      // one of the wave's tiles holds its position - is polled for as ONE 16-byte piece per lane (two with four heads
      // per KV head) and handed round through the wave's own LDS.  A round costs by its load instructions: four for q
      // (lanes sharing addresses) and a second poll of up to nine for the new key / value rows after it were 0.8 us a
      // layer more.  staging area: [q rows of the group | new key row | new value row], bf16.
      constexpr int NPQ = G * D / 8, NPK = D / 8, NP = NPQ + 2 * NPK, NPL = (NP + 63) / 64;
      char* stage = reinterpret_cast<char*>(G * D * 4 >= NP * 16 ? s_acc + wave * G * D : wave_lds + wave * 256);
      const int pn = L - 1;
      // (the appended position sits at the end of the last chunk; a wave's tiles are every fourth one of the chunk)
      const bool need_new = TAG && pn >= t0 && pn < t1 && (((pn - t0) >> 4) & 3) == wave;
      uint32_t nw[D / 64];  // int8 cache: this lane's pairs of the new rows
      auto patch = [&](int tbx, uint4* kx, uint4* vx) {  // the appended row into the tile at tbx, if that holds its position
        if (need_new && pn >= tbx && pn < tbx + 16) {
          if constexpr (I8) attn_new_row_i8<D>(nw, kq8, vq8, stb, row, tbx, t1, pn, kx, vx, reinterpret_cast<float*>(stage));
          else attn_new_row_staged<D>(stage + NPQ * 16, tbx, t1, pn, kx, vx);
        }
      };
      // the wave's second tile, requested ahead of the poll (a workgroup waits for q for microseconds; what is requested
      // behind the poll is a memory latency late)
      bool ahead = false;
      if (AHEAD && tb + 64 < t1) {
        if constexpr (I8) attn_tile_load_i8<D>(kq8, vq8, stb, row, tb + 64, last, raw);
        else attn_tile_load_u<D>(kb, vb, row, tb + 64, t1, coh, kn, vn, last);
        ahead = true;
      }
      if (TAG) {
        unsigned int spins = 0;
        const char* qrow = qt + (size_t)b * q_row;
        const MbRsrc rs = mb_rsrc(qrow);
        const uint32_t kv_off = (uint32_t)((kvt + (size_t)b * kv_row) - qrow);  // (the mailboxes of a layer are one block)
        uint32_t off[NPL];
#pragma unroll
        for (int l = 0; l < NPL; ++l) {
          const int i = lane + 64 * l;
          const uint32_t oq = (uint32_t)(kvh * G * D + (i < NPQ ? i : 0) * 8) * 2u;
          const int j = i - NPQ;  // piece of [key row | value row]
          const uint32_t ok_ = kv_off + (uint32_t)((j < NPK ? kvh * D + j * 8 : Hkv * D + kvh * D + (j - NPK) * 8)) * 2u;
          off[l] = (need_new && i >= NPQ && i < NP) ? ok_ : oq;
        }
        uint4 piece[NPL];
        for (;;) {
          bool ok = true;
#pragma unroll
          for (int l = 0; l < NPL; ++l) {
            const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rs, off[l], 0, 16);
            piece[l] = make_uint4(v.x, v.y, v.z, v.w);
            ok = ok && v.x != OHARA_UNWRITTEN && v.y != OHARA_UNWRITTEN && v.z != OHARA_UNWRITTEN && v.w != OHARA_UNWRITTEN;
          }
          if (__all(ok) || poll_expired(pc, spins)) break;
        }
#pragma unroll
        for (int l = 0; l < NPL; ++l)
          if (lane + 64 * l < NP) sts16(stage + (lane + 64 * l) * 16, piece[l]);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int hh = 0; hh < G; ++hh)
#pragma unroll
          for (int c = 0; c < NC; ++c) qv[hh][c] = lds16(stage + (hh * (D / 8) + 4 * c + dq) * 16);
        if constexpr (I8) {
          if (need_new) {
#pragma unroll
            for (int j = 0; j < D / 64; ++j) nw[j] = reinterpret_cast<const uint32_t*>(stage + NPQ * 16)[lane + 64 * j];
          }
        }
        if (!use_pre) patch(tb, ka, va);
      } else {
#pragma unroll
        for (int hh = 0; hh < G; ++hh)
#pragma unroll
          for (int c = 0; c < NC; ++c)
            qv[hh][c] = ldg16(xm_addr(qm, blk_x, b, (kvh * G + hh) * D + (4 * c + dq) * 8));
      }
      auto consume = [&](int tb, const uint4* kv, const uint4* vv) {
        const bool valid = tb + p < t1;
        // The heads of the group advance in lock step (their cross-lane exchanges overlap); l_run is
        // this lane's share of the sum, folded over the 16 positions after the loop; the running
        // maximum is re-derived only for tiles in which some score exceeds it.
        float sc[G], pv[G], pvr[G];  // pvr: the weight rounded to bf16, as it enters the value product
#pragma unroll
        for (int hh = 0; hh < G; ++hh) {
          float s = 0.f;
#pragma unroll
          for (int c = 0; c < NC; ++c) s = dot8m(kv[c], qv[hh][c], s);
          sc[hh] = s;
        }
#pragma unroll
        for (int hh = 0; hh < G; ++hh) sc[hh] = lane_xor_sum<16>(sc[hh]);
#pragma unroll
        for (int hh = 0; hh < G; ++hh) sc[hh] = lane_xor_sum<32>(sc[hh]);
        bool raise = false;
#pragma unroll
        for (int hh = 0; hh < G; ++hh) {
          sc[hh] = valid ? sc[hh] * scale : -INFINITY;
          raise = raise || sc[hh] > m_run[hh];
        }
        if (__any(raise)) {
          float tm[G];
#pragma unroll
          for (int hh = 0; hh < G; ++hh) tm[hh] = sc[hh];
#pragma unroll
          for (int hh = 0; hh < G; ++hh) tm[hh] = lane_xor_max<8>(tm[hh]);
#pragma unroll
          for (int hh = 0; hh < G; ++hh) tm[hh] = lane_xor_max<4>(tm[hh]);
#pragma unroll
          for (int hh = 0; hh < G; ++hh) tm[hh] = lane_xor_max<2>(tm[hh]);
#pragma unroll
          for (int hh = 0; hh < G; ++hh) tm[hh] = lane_xor_max<1>(tm[hh]);
#pragma unroll
          for (int hh = 0; hh < G; ++hh) {
            const float mn = fmaxf(m_run[hh], ceilf(tm[hh]));
            const float corr = pow2_neg_int(m_run[hh] - mn);
            m_run[hh] = mn;
            l_run[hh] *= corr;
#pragma unroll
            for (int i = 0; i < 8; ++i) acc[hh][i] *= corr;
          }
        }
#pragma unroll
        for (int hh = 0; hh < G; ++hh) {
          pv[hh] = __builtin_amdgcn_exp2f(sc[hh] - m_run[hh]);
          l_run[hh] += pv[hh];
          pvr[hh] = rbf(pv[hh]);
        }
        // all weight exchanges first (they are independent), then the products
        float pw[NV][G];
#pragma unroll
        for (int c = 0; c < NV; ++c)
#pragma unroll
          for (int hh = 0; hh < G; ++hh) pw[c][hh] = __shfl(pvr[hh], c * PP + pp, WAVE);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int c = 0; c < NV; ++c) {
          const uint32_t w4[4] = {vv[c].x, vv[c].y, vv[c].z, vv[c].w};
#pragma unroll
          for (int hh = 0; hh < G; ++hh)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              acc[hh][2 * i] += pw[c][hh] * lo_bf(w4[i]);
              acc[hh][2 * i + 1] += pw[c][hh] * hi_bf(w4[i]);
            }
        }
      };
      // (a chunk is one or two tiles per wave here: the next tile goes through a second register set
      // and is copied over, which costs a wait but far fewer registers than two sets taking turns; the polled builds
      // have requested the wave's second tile before the poll for q)
      for (; tb + 64 < t1; tb += 64) {
        if constexpr (I8) {  // the next tile's codes travel while the current tile is consumed, and become values after it
          if (!AHEAD || !ahead) attn_tile_load_i8<D>(kq8, vq8, stb, row, tb + 64, last, raw);
          ahead = false;
          consume(tb, ka, va);
          attn_tile_dequant<D>(raw, ka, va);
        } else {
          if (!AHEAD || !ahead) attn_tile_load_u<D>(kb, vb, row, tb + 64, t1, coh, kn, vn, last);
          ahead = false;
          consume(tb, ka, va);
#pragma unroll
          for (int c = 0; c < NC; ++c) ka[c] = kn[c];
#pragma unroll
          for (int c = 0; c < NV; ++c) va[c] = vn[c];
        }
        if (TAG) patch(tb + 64, ka, va);
      }
      consume(tb, ka, va);
    }
    first = false;
#pragma unroll
    for (int hh = 0; hh < G; ++hh)
      l_run[hh] = lane_xor_sum<1>(lane_xor_sum<2>(lane_xor_sum<4>(lane_xor_sum<8>(l_run[hh]))));
#pragma unroll
    for (int hh = 0; hh < G; ++hh) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        float v = acc[hh][i];
        if (DC == 8) v = lane_xor_sum<8>(v);
        v = lane_xor_sum<16>(v);
        acc[hh][i] = lane_xor_sum<32>(v);
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
    float* ann = nullptr;  // the thread that holds a head's maximum and sum: where they go
    float ann_m = 0.f, ann_l = 0.f;
    for (int idx = tid * 2; idx < G * D; idx += 512) {
      const int hh = idx / D, d = idx - hh * D;
      const int h = kvh * G + hh;
      const float M = fmaxf(fmaxf(s_m[hh], s_m[G + hh]), fmaxf(s_m[2 * G + hh], s_m[3 * G + hh]));
      float Ls = 0.f, o0 = 0.f, o1 = 0.f;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const float mw = s_m[w * G + hh];
        const float sc = (mw == -INFINITY) ? 0.f : pow2_neg_int(mw - M);
        Ls += s_l[w * G + hh] * sc;
        o0 += s_acc[(w * G + hh) * D + d] * sc;
        o1 += s_acc[(w * G + hh) * D + d + 1] * sc;
      }
      float* dst = pm + ((size_t)(b * H + h) * OHARA_MEGA_NS + split) * PS;
      st_coh8(dst + d, make_uint2(__float_as_uint(o0), __float_as_uint(o1)));
      if (d == 0) {
        if (TAG && announce) {
          ann = dst + D;
          ann_m = M;
          ann_l = Ls;
        } else {
          st_coh8(dst + D, make_uint2(__float_as_uint(M), __float_as_uint(Ls)));
        }
      }
    }
    // `announce`: the merge polls for the head's maximum and sum, which are stored - each in an 8-byte word of its own
    // together with the launch's tag, {max, tag, sum, tag} - once the item's accumulators have reached memory
    if (TAG && announce) wait_own_stores();
    __syncthreads();
    if (TAG && announce && ann) {
      st_coh8(ann, make_uint2(__float_as_uint(ann_m), pc.tag));
      st_coh8(ann + 2, make_uint2(__float_as_uint(ann_l), pc.tag));
    }
  }
}

}  // namespace
