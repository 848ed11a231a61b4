// Split-context GQA decode attention: one query position per sequence, every cached
// position visible (ohara/models/llama.py:100-135 with S = 1; mask :109-113 is all
// true; scale 1/sqrt(Dh) :116-125; GQA head mapping of repeat_interleave :101-103
// done by indexing, the expanded K/V are never materialised).
//
// Grid (query rows, H_kv, n_split).  A workgroup streams its chunk of the context for one
// KV head once and serves all G = H/H_kv query heads from it.  Per 16-position tile
// a wave holds one position per quad of lanes (the four lanes hold the four quarters of its K
// row), so q.k needs two adds inside the quad (DPP, no LDS round trip); the running max/sum of
// the online softmax are wavefront shuffle reductions.  Partial (max, sum, acc) triples of the chunks are
// merged by whichever workgroup of the (sequence, KV head) finishes last, in chunk
// order, so the result does not depend on scheduling.
#include <mutex>

#include "common.h"

namespace {

struct AttnArgs {
  const bf16_t* q;   // (B, H*D)
  const bf16_t* k;   // (Bcap, Tmax, Hkv, D); int8 mode: the same shape in int8
  const bf16_t* v;
  const float* stats;   // int8 mode (ohara/modules/kv_cache.py:67-73): (Bcap, Hkv, Tmax, 4) = key scale, key
                        // minimum, value scale, value minimum of every (sequence, head, position) row
  bf16_t* out;       // (B, H*D)
  int B, S, H, Hkv, D, Tmax, start;  // query s of sequence b sees positions [0, start + s]
  const int32_t* pos_dev;            // when set: start = *pos_dev, or pos_dev[sequence] with pos_stride 1
  int pos_stride;
  int nsplit;
  int* counters;     // (B*Hkv)
  float* part_ml;    // (B, H, nsplit, 2)
  float* part_acc;   // (B, H, nsplit, D)
  float scale;
};

__device__ __forceinline__ float dot8(uint4 a, uint4 b, float s) {
  s = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a.x), __builtin_bit_cast(bf16x2, b.x), s, false);
  s = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a.y), __builtin_bit_cast(bf16x2, b.y), s, false);
  s = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a.z), __builtin_bit_cast(bf16x2, b.z), s, false);
  s = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a.w), __builtin_bit_cast(bf16x2, b.w), s, false);
  return s;
}

// Sum over the four lanes of a quad (lanes 4i .. 4i+3) with two DPP adds: no LDS round trip, unlike a
// shuffle across rows.  quad_perm [1,0,3,2] = 0xB1 (lane ^ 1), [2,3,0,1] = 0x4E (lane ^ 2).
__device__ __forceinline__ float quad_sum(float v) {
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xF, 0xF, true));
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xF, 0xF, true));
  return v;
}

__device__ __forceinline__ float ldf_coh(const float* p) { return __uint_as_float(ld_coh4(p)); }
__device__ __forceinline__ void stf_coh(float* p, float v) { st_coh4(p, __float_as_uint(v)); }

// Merge the chunk partials of the G heads of (b, kvh) and write bf16 output.  Called by all
// 256 threads of the last workgroup to finish.  A chain of dependent device-coherent loads
// costs about a microsecond per link on this chip, so the (max, sum) pairs of all chunks are
// fetched in one round into LDS, the chunk weights exp(m_s - M) are formed there, and the
// accumulator columns are then summed in chunk order with the loads of up to 32 chunks issued together.
// Needs G * n_split <= OHARA_MERGE_CAP.
#define OHARA_MERGE_CAP 2048
template <int MAXD>
__device__ void merge_partials(const AttnArgs& a, int b /* query row */, int kvh, int G) {
  __shared__ float s_w[OHARA_MERGE_CAP];   // max, then weight, of (head, chunk)
  __shared__ float s_ls[OHARA_MERGE_CAP];  // sum of (head, chunk)
  __shared__ float s_tot[64];              // per head: normaliser
  const int D = a.D, ns = a.nsplit;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const float* ml0 = a.part_ml + ((size_t)(b * a.H + kvh * G) * ns) * 2;  // heads of a group are adjacent
  for (int i = tid; i < G * ns; i += blockDim.x) {
    const uint2 v = ld_coh8(ml0 + 2 * (size_t)i);
    s_w[i] = __uint_as_float(v.x);
    s_ls[i] = __uint_as_float(v.y);
  }
  __syncthreads();
  for (int hh = wave; hh < G; hh += 4) {
    float M = -INFINITY;
    for (int s0 = lane; s0 < ns; s0 += 64) M = fmaxf(M, s_w[hh * ns + s0]);
    M = wave_max(M);
    float L = 0.f;
    for (int s0 = lane; s0 < ns; s0 += 64) {
      const float ms = s_w[hh * ns + s0];
      const float w = (ms == -INFINITY) ? 0.f : pow2_neg_int(ms - M);  // maxima are integers (log2 units): exact
      s_w[hh * ns + s0] = w;
      L += s_ls[hh * ns + s0] * w;
    }
    L = wave_sum(L);
    if (lane == 0) s_tot[hh] = L;
  }
  __syncthreads();
  for (int idx = tid; idx < G * D; idx += blockDim.x) {
    const int hh = idx / D, d = idx - hh * D;
    const int h = kvh * G + hh;
    const float* pa = a.part_acc + ((size_t)(b * a.H + h) * ns) * D + d;
    const float* w = s_w + hh * ns;
    float o = 0.f;
    // Up to 32 chunks' values are in flight at once, every load unconditional (chunks past the last
    // read the last one again and are not added): with eight at a time behind a test each, 32 chunks
    // were four dependent round trips and more than half of a batch-1 launch.
    for (int s0 = 0; s0 < ns; s0 += 32) {
      float av[32];
#pragma unroll
      for (int i = 0; i < 32; ++i) av[i] = ldf_coh(pa + (size_t)min(s0 + i, ns - 1) * D);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < 32; ++i)
        if (s0 + i < ns) o += av[i] * w[s0 + i];
    }
    a.out[(size_t)b * a.H * D + h * D + d] = f2bf(o * (1.0f / s_tot[hh]));
  }
}

// Counts this workgroup's chunk as done and returns true in the workgroup that observes all
// n_split chunks done (every thread gets the same answer).  The partials were written with
// write-through stores; every wave waits for the completion of its own before the workgroup
// barrier, the counter is a relaxed device-scope atomic and the merge reads with
// cache-bypassing loads: no L2 write-back or invalidate.
__device__ bool last_chunk_done(int* counter, int nsplit) {
  __shared__ int is_last;
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  wait_own_stores();
  __syncthreads();
  if (threadIdx.x == 0) {
    const int old = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    is_last = (old == nsplit - 1);
    if (is_last) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next call
  }
  __syncthreads();
  return is_last != 0;
}

template <int D, int G>
__global__ __launch_bounds__(256) void attn_decode_kernel(AttnArgs a) {
  constexpr int NC = D / 32;        // 16-byte K loads per lane per tile
  constexpr int DC = D / 8;         // lanes covering one V row with 16-byte loads
  static_assert(DC == 8 || DC == 16, "head_dim 64 or 128");
  constexpr int PP = 64 / DC;       // V rows fetched per load instruction
  constexpr int NV = 16 / PP;       // V load instructions per 16-position tile
  const int split = blockIdx.z, kvh = blockIdx.y, b = blockIdx.x;  // b: query row = seq * S + s
  const int seq = b / a.S;
  const int L = min((a.pos_dev ? a.pos_dev[(size_t)seq * a.pos_stride] : a.start) + (b - seq * a.S) + 1, a.Tmax);
  const int chunk = (((L + a.nsplit - 1) / a.nsplit) + 63) & ~63;
  const int t0 = split * chunk;
  const int t1 = min(L, t0 + chunk);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int p = lane >> 2, dq = lane & 3;  // position of the tile, quarter of its K row: a quad holds one row
  const int pp = lane / DC, dc = lane % DC;
  const float scale_l2 = a.scale * OHARA_LOG2E;  // scores in log2 units (common.h: softmax bookkeeping)

  __shared__ float s_m[4][G], s_l[4][G];
  __shared__ float s_acc[4][G][D];

  // q for this lane's quarter-row: columns (4c + dq)*8 .. +7
  uint4 qv[G][NC];
#pragma unroll
  for (int hh = 0; hh < G; ++hh)
#pragma unroll
    for (int c = 0; c < NC; ++c)
      qv[hh][c] = ldg16(a.q + (size_t)b * a.H * D + (size_t)(kvh * G + hh) * D + (4 * c + dq) * 8);

  float m_run[G], l_run[G], acc[G][8];
#pragma unroll
  for (int hh = 0; hh < G; ++hh) {
    m_run[hh] = -INFINITY;
    l_run[hh] = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[hh][i] = 0.f;
  }

  const size_t row = (size_t)a.Hkv * D;
  const bf16_t* kb = a.k + (size_t)seq * a.Tmax * row + (size_t)kvh * D;
  const bf16_t* vb = a.v + (size_t)seq * a.Tmax * row + (size_t)kvh * D;

  struct Tile {
    uint4 k[NC];
    uint4 v[NV];
  };
  // Every load of a tile is issued without a branch (positions past the chunk read its last row;
  // their scores are masked and their weights are zero): with the loads behind per-lane conditions
  // the compiler cannot count how many are outstanding and waits for ALL of them - the next tile's
  // included - before it touches the current tile, which undoes the double buffering.
  auto load_tile = [&](int tb, Tile& t) {
    const int pos = min(tb + p, t1 - 1);
#pragma unroll
    for (int c = 0; c < NC; ++c) t.k[c] = ldg16_nt(kb + (size_t)pos * row + (4 * c + dq) * 8);
#pragma unroll
    for (int c = 0; c < NV; ++c) {
      const int vp = min(tb + c * PP + pp, t1 - 1);
      t.v[c] = ldg16_nt(vb + (size_t)vp * row + dc * 8);
    }
  };
  auto expand = [&](const Tile& t, uint4* kv, uint4* vv) {
#pragma unroll
    for (int c = 0; c < NC; ++c) kv[c] = t.k[c];
#pragma unroll
    for (int c = 0; c < NV; ++c) vv[c] = t.v[c];
  };
  // 16-position tiles, wave w takes tiles w, w+4, ...; the loads of the next tile are in
  // flight while the current one is consumed (a second tile in flight costs more in occupancy
  // than it gains: measured)
  Tile cur, nxt;
  auto consume = [&](int tb, const Tile& tile) {
    const bool valid = tb + p < t1;
    uint4 kv[NC], vv[NV];
    expand(tile, kv, vv);
    // The heads of the group advance together, one step at a time, so that their cross-lane
    // exchanges overlap instead of forming G dependent chains.  l_run is this lane's share of the
    // sum (its own position only; folded over the 16 positions after the loop), and the running
    // maximum is re-derived only for tiles in which some score exceeds it - for every other tile
    // the usual update would multiply by exp(0).
    float sc[G], pv[G], pvr[G];  // pvr: the weight as the value product sees it (bf16, as the library kernel rounds it)
#pragma unroll
    for (int hh = 0; hh < G; ++hh) {
      float s = 0.f;
#pragma unroll
      for (int c = 0; c < NC; ++c) s = dot8(kv[c], qv[hh][c], s);
      sc[hh] = s;
    }
#pragma unroll
    for (int hh = 0; hh < G; ++hh) sc[hh] = quad_sum(sc[hh]);
    bool raise = false;
#pragma unroll
    for (int hh = 0; hh < G; ++hh) {
      sc[hh] = valid ? sc[hh] * scale_l2 : -INFINITY;  // log2 units
      raise = raise || sc[hh] > m_run[hh];
    }
    if (__any(raise)) {
      float tm[G];
#pragma unroll
      for (int hh = 0; hh < G; ++hh) tm[hh] = sc[hh];
#pragma unroll
      for (int hh = 0; hh < G; ++hh) tm[hh] = lanes_max<32, 4>(tm[hh]);
#pragma unroll
      for (int hh = 0; hh < G; ++hh) {
        const float mn = fmaxf(m_run[hh], ceilf(tm[hh]));  // finite: the tile holds at least one position
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
    // all weight exchanges first (they are independent), then the products: next to their products
    // every exchange is waited for by itself
    float pw[NV][G];
#pragma unroll
    for (int c = 0; c < NV; ++c)
#pragma unroll
      for (int hh = 0; hh < G; ++hh) pw[c][hh] = __shfl(pvr[hh], 4 * (c * PP + pp), WAVE);
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
  int tb = t0 + wave * 16;
  if (tb < t1) {
    // two register tiles take turns (no copy between iterations: a copy would wait for the tile
    // that has just been requested)
    load_tile(tb, cur);
    if constexpr (G >= 4) {  // four heads' accumulators leave no room for a second resident tile
      for (; tb + 64 < t1; tb += 64) {
        load_tile(tb + 64, nxt);
        consume(tb, cur);
        cur = nxt;
      }
      consume(tb, cur);
    } else {
      for (;;) {
        if (tb + 64 >= t1) { consume(tb, cur); break; }
        load_tile(tb + 64, nxt);
        consume(tb, cur);
        tb += 64;
        if (tb + 64 >= t1) { consume(tb, nxt); break; }
        load_tile(tb + 64, cur);
        consume(tb, nxt);
        tb += 64;
      }
    }
  }

  // fold the sums over the 16 positions of a tile (every lane of a quarter holds the same share),
  // the PP row-groups of the wave, then the four waves
#pragma unroll
  for (int hh = 0; hh < G; ++hh) l_run[hh] = lanes_sum<32, 4>(l_run[hh]);
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
      for (int i = 0; i < 8; ++i) s_acc[wave][hh][dc * 8 + i] = acc[hh][i];
    }
    if (lane == 0) {
      s_m[wave][hh] = m_run[hh];
      s_l[wave][hh] = l_run[hh];
    }
  }
  __syncthreads();
  for (int idx = tid; idx < G * D; idx += 256) {
    const int hh = idx / D, d = idx - hh * D;
    const int h = kvh * G + hh;
    float M = fmaxf(fmaxf(s_m[0][hh], s_m[1][hh]), fmaxf(s_m[2][hh], s_m[3][hh]));
    float Ls = 0.f, o = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float mw = s_m[w][hh];
      const float sc = (mw == -INFINITY) ? 0.f : pow2_neg_int(mw - M);
      Ls += s_l[w][hh] * sc;
      o += s_acc[w][hh][d] * sc;
    }
    if (a.nsplit == 1) {  // whole context in this workgroup: no partials
      a.out[(size_t)b * a.H * D + h * D + d] = f2bf(o * (1.0f / Ls));
      continue;
    }
    const size_t pi = (size_t)(b * a.H + h) * a.nsplit + split;
    stf_coh(a.part_acc + pi * D + d, o);
    if (d == 0) {
      stf_coh(a.part_ml + pi * 2, M);
      stf_coh(a.part_ml + pi * 2 + 1, Ls);
    }
  }
  if (a.nsplit == 1) return;
  if (last_chunk_done(a.counters + b * a.Hkv + kvh, a.nsplit)) merge_partials<D>(a, b, kvh, G);
}


// The same attention over the int8 cache (ohara/modules/kv_cache.py:15-32, 116-118).  A row of codes is
// half the bytes of a bf16 row, and what bounds this kernel is the bytes a wave has in flight, so a tile
// here is 32 positions (two sub-tiles of 16 with the lane roles of the bf16 kernel): the same bytes in
// flight, twice the positions per round trip.  The four statistics of a position are one 16-byte record
// ((Bcap, Hkv, Tmax, 4) fp32: consecutive positions are contiguous, nothing is fetched that is not used);
// the lane that owns a position loads its record, the value rows get their scale and minimum from that
// lane by a shuffle.  Codes become the bf16 values the reference's read returns - bf16((code + 128) *
// scale + min) - right before use, so the results are those of bf16 attention over the dequantised cache.
// Turning the codes into those values is most of what a position costs (2.5 vector instructions per
// element), so the score product runs on the matrix cores: A = the group's q rows (row m = head m, the
// other rows zero), B = the sixteen dequantised key rows of a sub-tile (lane (position n, quarter kg)
// holds the 8 elements of its quarter that step c contracts - the k index of the product is a
// permutation of the head dimension, the same one on both sides), NC products of 16x16x32 per sub-tile;
// lanes 0..15 end up with the scores of position n for every head.  The value product stays on the
// vector units (its operand would have to be transposed).
template <int D, int G>
__global__ __launch_bounds__(256, (G == 1 ? 3 : 2)) void attn_decode_i8_kernel(AttnArgs a) {
  constexpr int NC = D / 32;        // bf16 uint4 of a K quarter-row after expansion
  constexpr int NCB = (NC + 1) / 2; // uint4 of codes per K quarter-row (NC = 2: one 16-byte load)
  constexpr int DC = D / 8;         // lanes covering one V row with 8-byte loads
  static_assert(DC == 8 || DC == 16, "head_dim 64 or 128");
  constexpr int PP = 64 / DC;       // V rows fetched per load instruction
  constexpr int NV = 32 / PP;       // V load instructions per 32-position tile
  static_assert(NC >= 2, "head width 64 or 128");
  const int split = blockIdx.z, kvh = blockIdx.y, b = blockIdx.x;  // b: query row = seq * S + s
  const int seq = b / a.S;
  const int L = min((a.pos_dev ? a.pos_dev[(size_t)seq * a.pos_stride] : a.start) + (b - seq * a.S) + 1, a.Tmax);
  const int chunk = (((L + a.nsplit - 1) / a.nsplit) + 127) & ~127;
  const int t0 = split * chunk;
  const int t1 = min(L, t0 + chunk);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int p = lane & 15, dq = lane >> 4;  // position of the sub-tile, quarter of its K row (the B operand's column and k group)
  const int pp = lane / DC, dc = lane % DC;
  const float scale_l2 = a.scale * OHARA_LOG2E;  // scores in log2 units (common.h: softmax bookkeeping)

  __shared__ float s_m[4][G], s_l[4][G];
  __shared__ float s_acc[4][G][D];

  uint4 qa[NC];  // A operand: row (lane & 15) = head of the group (rows past the group are zero), this lane's quarter dq
#pragma unroll
  for (int c = 0; c < NC; ++c)
    qa[c] = p < G ? ldg16(a.q + (size_t)b * a.H * D + (size_t)(kvh * G + p) * D + (dq * NC + c) * 8) : make_uint4(0, 0, 0, 0);

  float m_run[G], l_run[G], acc[G][8];
#pragma unroll
  for (int hh = 0; hh < G; ++hh) {
    m_run[hh] = -INFINITY;
    l_run[hh] = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[hh][i] = 0.f;
  }

  const size_t row = (size_t)a.Hkv * D;
  const int8_t* kb8 = reinterpret_cast<const int8_t*>(a.k) + (size_t)seq * a.Tmax * row + (size_t)kvh * D;
  const int8_t* vb8 = reinterpret_cast<const int8_t*>(a.v) + (size_t)seq * a.Tmax * row + (size_t)kvh * D;
  const float* stb = a.stats + ((size_t)seq * a.Hkv + kvh) * a.Tmax * 4;

  struct Tile {
    uint4 k[2][NCB];  // sub-tile s: codes of this lane's quarter of row tb + 16 s + p
    uint2 v[NV];      // eight codes of row tb + c * PP + pp
    uint4 st[2];      // (key scale, key min, value scale, value min) of position tb + 16 s + p
  };
  // Loads without branches, as in the bf16 kernel: positions past the chunk read its last row (their
  // scores are masked, their weights zero), so that the compiler can count the loads in flight and
  // wait for the current tile only.
  auto load_tile = [&](int tb, Tile& t) {
#pragma unroll
    for (int sb = 0; sb < 2; ++sb) {
      const int pos = min(tb + 16 * sb + p, t1 - 1);
      t.st[sb] = ldg16(stb + (size_t)pos * 4);
#pragma unroll
      for (int c = 0; c < NCB; ++c) t.k[sb][c] = ldg16_nt(kb8 + (size_t)pos * row + dq * (D / 4) + 16 * c);
    }
#pragma unroll
    for (int c = 0; c < NV; ++c) {
      const int vp = min(tb + c * PP + pp, t1 - 1);
      const u32x2 w = __builtin_nontemporal_load((const OHARA_GLOBAL u32x2*)(vb8 + (size_t)vp * row + dc * 8));
      t.v[c] = make_uint2(w.x, w.y);
    }
  };
  Tile cur, nxt;
  auto consume = [&](int tb, const Tile& cur) {
    // One sub-tile of 16 positions at a time (both at once would need the registers of two expanded K
    // tiles); within it the heads of the group advance together, as in the bf16 kernel.
#pragma unroll
    for (int sb = 0; sb < 2; ++sb) {
      float sc[G], pv[G], pvr[G];  // pvr: the weight as the value product sees it (bf16, as the library kernel rounds it)
      {
        const float ks = __uint_as_float(cur.st[sb].x), km = __uint_as_float(cur.st[sb].y);
        uint4 kv[NC];
#pragma unroll
        for (int c = 0; c < NC; ++c) {
          const uint32_t* w = reinterpret_cast<const uint32_t*>(&cur.k[sb][c >> 1]) + 2 * (c & 1);
          const uint2 lo = dequant4(w[0] ^ 0x80808080u, ks, km), hi = dequant4(w[1] ^ 0x80808080u, ks, km);
          kv[c] = make_uint4(lo.x, lo.y, hi.x, hi.y);
        }
        f32x4 sacc = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < NC; ++c)
          sacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, qa[c]), __builtin_bit_cast(bf16x8, kv[c]),
                                                         sacc, 0, 0, 0);
#pragma unroll
        for (int hh = 0; hh < G; ++hh) sc[hh] = sacc[hh];  // lanes 0..15: head hh against position p (rows 4.. of the product are zero)
      }
      const bool valid = lane < 16 && tb + 16 * sb + p < t1;
      bool raise = false;
#pragma unroll
      for (int hh = 0; hh < G; ++hh) {
        sc[hh] = valid ? sc[hh] * scale_l2 : -INFINITY;  // log2 units
        raise = raise || sc[hh] > m_run[hh];
      }
      if (__any(raise)) {
        float tm[G];
#pragma unroll
        for (int hh = 0; hh < G; ++hh) tm[hh] = sc[hh];
#pragma unroll
        for (int hh = 0; hh < G; ++hh) tm[hh] = lanes_max<32, 1>(tm[hh]);
#pragma unroll
        for (int hh = 0; hh < G; ++hh) {
          const float mn = fmaxf(m_run[hh], ceilf(tm[hh]));  // finite here: some position of the sub-tile raised it
          const float corr = pow2_neg_int(m_run[hh] - mn);
          m_run[hh] = mn;
          l_run[hh] *= corr;
#pragma unroll
          for (int i = 0; i < 8; ++i) acc[hh][i] *= corr;
        }
      }
#pragma unroll
      for (int hh = 0; hh < G; ++hh) {
        pv[hh] = __builtin_amdgcn_exp2f(sc[hh] - m_run[hh]);  // (a sub-tile past the end: 2^(-inf - m) = 0; m is finite by then)
        l_run[hh] += pv[hh];
        pvr[hh] = rbf(pv[hh]);
      }
      // the exchanges of a few rows first (scale, minimum and weight of the row whose codes this lane
      // holds: independent of each other), then their products; next to its products every exchange
      // would be waited for by itself
      constexpr int XB = G >= 4 ? 1 : (G == 2 ? 2 : NV / 2);  // rows per round: what the registers allow
#pragma unroll
      for (int c0 = 0; c0 < NV / 2; c0 += XB) {
        float vs[XB], vm[XB], pw[XB][G];
#pragma unroll
        for (int cc = 0; cc < XB; ++cc) {
          const int c = sb * (NV / 2) + c0 + cc;
          const int src = (c * PP + pp) & 15;  // the lane that holds the weight (and a record) of the row I hold eight codes of
          vs[cc] = __shfl(__uint_as_float(cur.st[sb].z), src, WAVE);
          vm[cc] = __shfl(__uint_as_float(cur.st[sb].w), src, WAVE);
#pragma unroll
          for (int hh = 0; hh < G; ++hh) pw[cc][hh] = __shfl(pvr[hh], src, WAVE);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int cc = 0; cc < XB; ++cc) {
          const int c = sb * (NV / 2) + c0 + cc;
          const uint2 lo = dequant4(cur.v[c].x ^ 0x80808080u, vs[cc], vm[cc]),
                      hi = dequant4(cur.v[c].y ^ 0x80808080u, vs[cc], vm[cc]);
          const uint32_t w4[4] = {lo.x, lo.y, hi.x, hi.y};
#pragma unroll
          for (int hh = 0; hh < G; ++hh)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              acc[hh][2 * i] += pw[cc][hh] * lo_bf(w4[i]);
              acc[hh][2 * i + 1] += pw[cc][hh] * hi_bf(w4[i]);
            }
        }
      }
    }
  };
  int tb = t0 + wave * 32;
  if (tb < t1) {
    load_tile(tb, cur);
    if constexpr (G >= 4) {  // two tiles taking turns do not fit the registers of four heads
      for (; tb + 128 < t1; tb += 128) {
        load_tile(tb + 128, nxt);
        consume(tb, cur);
        cur = nxt;
      }
      consume(tb, cur);
    } else {
      for (;;) {
        if (tb + 128 >= t1) { consume(tb, cur); break; }
        load_tile(tb + 128, nxt);
        consume(tb, cur);
        tb += 128;
        if (tb + 128 >= t1) { consume(tb, nxt); break; }
        load_tile(tb + 128, cur);
        consume(tb, nxt);
        tb += 128;
      }
    }
  }

  // fold the sums over the 16 positions of a sub-tile, the PP row-groups of the wave, then the four waves
#pragma unroll
  for (int hh = 0; hh < G; ++hh) l_run[hh] = lanes_sum<32, 1>(l_run[hh]);  // (lanes 16.. hold zeros)
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
      for (int i = 0; i < 8; ++i) s_acc[wave][hh][dc * 8 + i] = acc[hh][i];
    }
    if (lane == 0) {
      s_m[wave][hh] = m_run[hh];
      s_l[wave][hh] = l_run[hh];
    }
  }
  __syncthreads();
  for (int idx = tid; idx < G * D; idx += 256) {
    const int hh = idx / D, d = idx - hh * D;
    const int h = kvh * G + hh;
    float M = fmaxf(fmaxf(s_m[0][hh], s_m[1][hh]), fmaxf(s_m[2][hh], s_m[3][hh]));
    float Ls = 0.f, o = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float mw = s_m[w][hh];
      const float scw = (mw == -INFINITY) ? 0.f : pow2_neg_int(mw - M);
      Ls += s_l[w][hh] * scw;
      o += s_acc[w][hh][d] * scw;
    }
    if (a.nsplit == 1) {  // whole context in this workgroup: no partials
      a.out[(size_t)b * a.H * D + h * D + d] = f2bf(o * (1.0f / Ls));
      continue;
    }
    const size_t pi = (size_t)(b * a.H + h) * a.nsplit + split;
    stf_coh(a.part_acc + pi * D + d, o);
    if (d == 0) {
      stf_coh(a.part_ml + pi * 2, M);
      stf_coh(a.part_ml + pi * 2 + 1, Ls);
    }
  }
  if (a.nsplit == 1) return;
  if (last_chunk_done(a.counters + b * a.Hkv + kvh, a.nsplit)) merge_partials<D>(a, b, kvh, G);
}

// Head width 128 over the int8 cache with BOTH products on the matrix cores.  What a position costs in the
// kernel above is vector instructions - 2.5 per element to turn codes into the reference's bf16 values,
// and again as many multiply-adds per head for the value product - so at four heads per group it stays well
// below the memory's speed.  Here a wave walks tiles of 32 positions:
//   S^T = K Q^T    v_mfma_f32_16x16x32_bf16 per sub-tile of 16 positions: A = the dequantised key rows (lane
//                  (position, quarter) holds the 8 elements of its quarter that step c contracts), B = the
//                  group's q rows (column n = head n, the other columns zero).  Lane (head n, rg) ends up with
//                  the scores of positions 4 rg .. 4 rg + 3 of the sub-tile for ONE head: its running maximum,
//                  sum and rescale are per-lane scalars and the row maximum needs two cross-lane steps.
//   O^T += V^T P   the weights go from the score accumulators straight into the B operand: k-slot j of lane
//                  (n, rg) is position 4 rg + j of the first sub-tile for j < 4 and of the second for j >= 4.
//                  A lane dequantises 8 consecutive positions x 8 columns of V, transposes them in registers
//                  and parks them in the wave's own LDS as V^T (column-major), from where the A operand of a
//                  16-column block is two 8-byte reads that follow the same slot mapping.
// A lane then holds O[head n][16 blk + 4 rg + i]: no cross-lane sums at the end.  The weights are rounded
// to bf16 by the operand format, the sum is taken from the unrounded ones, scores are in log2 units with an
// integer running maximum: the rounding points of the kernels above.
template <int G>
__global__ __launch_bounds__(256, 2) void attn_decode_i8_mfma_kernel(AttnArgs a) {
  constexpr int D = 128, NC = 4, NB = 8;
  constexpr int LDV = 36;  // V^T row stride in elements (72 bytes: 8-byte reads and writes stay aligned)
  const int split = blockIdx.z, kvh = blockIdx.y, b = blockIdx.x;
  const int seq = b / a.S;
  const int L = min((a.pos_dev ? a.pos_dev[(size_t)seq * a.pos_stride] : a.start) + (b - seq * a.S) + 1, a.Tmax);
  const int chunk = (((L + a.nsplit - 1) / a.nsplit) + 127) & ~127;
  const int t0 = split * chunk;
  const int t1 = min(L, t0 + chunk);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n = lane & 15, rg = lane >> 4;  // K side: position n of a sub-tile, quarter rg; scores: head n, position group rg
  const float scale_l2 = a.scale * OHARA_LOG2E;

  __shared__ float s_m[4][G], s_l[4][G];
  __shared__ float s_acc[4][G][D];
  __shared__ __align__(16) bf16_t s_vt[4][D][LDV];

  uint4 qa[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c)
    qa[c] = n < G ? ldg16(a.q + (size_t)b * a.H * D + (size_t)(kvh * G + n) * D + (rg * NC + c) * 8) : make_uint4(0, 0, 0, 0);

  float m_run = -INFINITY, l_run = 0.f;
  f32x4 acc[NB];
#pragma unroll
  for (int i = 0; i < NB; ++i) acc[i] = (f32x4){0.f, 0.f, 0.f, 0.f};

  const size_t row = (size_t)a.Hkv * D;
  const int8_t* kb8 = reinterpret_cast<const int8_t*>(a.k) + (size_t)seq * a.Tmax * row + (size_t)kvh * D;
  const int8_t* vb8 = reinterpret_cast<const int8_t*>(a.v) + (size_t)seq * a.Tmax * row + (size_t)kvh * D;
  const float* stb = a.stats + ((size_t)seq * a.Hkv + kvh) * a.Tmax * 4;

  struct Tile {
    uint4 k[2][2];  // sub-tile s: the 32 codes of quarter rg of row tb + 16 s + n
    uint2 ks[2];    // (key scale, key minimum) of that row
    uint2 v[8];     // eight codes (columns 8 dc ..) of row tb + 8 pp + c
    uint2 vs[8];    // (value scale, value minimum) of that row
  };
  // Loads without branches: positions past the chunk read its last row (their scores are masked).
  auto load_tile = [&](int tb, Tile& t) {
#pragma unroll
    for (int sb = 0; sb < 2; ++sb) {
      const int pos = min(tb + 16 * sb + n, t1 - 1);
      t.ks[sb] = ldg8(stb + (size_t)pos * 4);
#pragma unroll
      for (int c = 0; c < 2; ++c) t.k[sb][c] = ldg16_nt(kb8 + (size_t)pos * row + rg * 32 + 16 * c);
    }
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      const int vp = min(tb + 8 * rg + c, t1 - 1);  // (V side: lane (pp = rg, dc = n))
      const u32x2 w = __builtin_nontemporal_load((const OHARA_GLOBAL u32x2*)(vb8 + (size_t)vp * row + n * 8));
      t.v[c] = make_uint2(w.x, w.y);
      t.vs[c] = ldg8(stb + (size_t)vp * 4 + 2);
    }
  };
  bf16_t* vt = &s_vt[wave][0][0];
  auto consume = [&](int tb, const Tile& cur) {
    // ---- V: dequantise 8 positions x 8 columns, transpose, park as V^T ---------------------------------
    {
      uint32_t w[8][4];  // row c: four dwords = columns (0,1) (2,3) (4,5) (6,7) as bf16 pairs
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        const float vs = __uint_as_float(cur.vs[c].x), vm = __uint_as_float(cur.vs[c].y);
        const uint2 lo = dequant4(cur.v[c].x ^ 0x80808080u, vs, vm), hi = dequant4(cur.v[c].y ^ 0x80808080u, vs, vm);
        w[c][0] = lo.x; w[c][1] = lo.y; w[c][2] = hi.x; w[c][3] = hi.y;
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {  // column pair (2e, 2e + 1) of this lane's eight columns
        uint32_t ev[4], od[4];       // positions (0,1) (2,3) (4,5) (6,7) of the even / the odd column
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          ev[q] = (w[2 * q][e] & 0xffffu) | (w[2 * q + 1][e] << 16);
          od[q] = (w[2 * q][e] >> 16) | (w[2 * q + 1][e] & 0xffff0000u);
        }
        bf16_t* c0 = vt + (size_t)(n * 8 + 2 * e) * LDV + 8 * rg;
        *reinterpret_cast<uint2*>(c0) = make_uint2(ev[0], ev[1]);
        *reinterpret_cast<uint2*>(c0 + 4) = make_uint2(ev[2], ev[3]);
        *reinterpret_cast<uint2*>(c0 + LDV) = make_uint2(od[0], od[1]);
        *reinterpret_cast<uint2*>(c0 + LDV + 4) = make_uint2(od[2], od[3]);
      }
    }
    // ---- scores of both sub-tiles ---------------------------------------------------------------------------
    float sc[8];
#pragma unroll
    for (int sb = 0; sb < 2; ++sb) {
      const float ks = __uint_as_float(cur.ks[sb].x), km = __uint_as_float(cur.ks[sb].y);
      f32x4 sacc = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const uint32_t* w = reinterpret_cast<const uint32_t*>(&cur.k[sb][c >> 1]) + 2 * (c & 1);
        const uint2 lo = dequant4(w[0] ^ 0x80808080u, ks, km), hi = dequant4(w[1] ^ 0x80808080u, ks, km);
        const uint4 kv = make_uint4(lo.x, lo.y, hi.x, hi.y);
        sacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kv), __builtin_bit_cast(bf16x8, qa[c]), sacc,
                                                       0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
        sc[4 * sb + i] = (n < G && tb + 16 * sb + 4 * rg + i < t1) ? sacc[i] * scale_l2 : -INFINITY;
    }
    float tm = sc[0];
#pragma unroll
    for (int i = 1; i < 8; ++i) tm = fmaxf(tm, sc[i]);
    tm = lane_xor_max<32>(lane_xor_max<16>(tm));  // over the four position groups of this head
    if (__any(tm > m_run)) {
      const float mn = fmaxf(m_run, ceilf(tm));
      const float corr = pow2_neg_int(m_run - mn);  // (both -inf, a head past the group: 2^-126 times zeros)
      m_run = mn;
      l_run *= corr;
#pragma unroll
      for (int blk = 0; blk < NB; ++blk)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[blk][i] *= corr;
    }
    float pw[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      pw[i] = sc[i] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(sc[i] - m_run);
      l_run += pw[i];
    }
    const uint4 pb = make_uint4(pack_bf(pw[0], pw[1]), pack_bf(pw[2], pw[3]), pack_bf(pw[4], pw[5]), pack_bf(pw[6], pw[7]));
    // ---- O^T += V^T P: the A operand of block blk is column 16 blk + n, positions 4 rg .. and 16 + 4 rg .. --------
    // (the wave reads what its own lanes wrote above: LDS accesses of a wave complete in order)
    uint4 va[NB];
#pragma unroll
    for (int blk = 0; blk < NB; ++blk) {
      const bf16_t* col = vt + (size_t)(16 * blk + n) * LDV + 4 * rg;
      const uint2 lo = *reinterpret_cast<const uint2*>(col);
      const uint2 hi = *reinterpret_cast<const uint2*>(col + 16);
      va[blk] = make_uint4(lo.x, lo.y, hi.x, hi.y);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int blk = 0; blk < NB; ++blk)
      acc[blk] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, va[blk]), __builtin_bit_cast(bf16x8, pb),
                                                         acc[blk], 0, 0, 0);
  };
  Tile cur, nxt;
  int tb = t0 + wave * 32;
  if (tb < t1) {
    load_tile(tb, cur);
    for (;;) {
      if (tb + 128 >= t1) { consume(tb, cur); break; }
      load_tile(tb + 128, nxt);
      consume(tb, cur);
      tb += 128;
      if (tb + 128 >= t1) { consume(tb, nxt); break; }
      load_tile(tb + 128, cur);
      consume(tb, nxt);
      tb += 128;
    }
  }
  // the sum over the four position groups; a lane holds O[head n][16 blk + 4 rg + i]
  l_run = lane_xor_sum<32>(lane_xor_sum<16>(l_run));
  if (n < G) {
#pragma unroll
    for (int blk = 0; blk < NB; ++blk)
#pragma unroll
      for (int i = 0; i < 4; ++i) s_acc[wave][n][16 * blk + 4 * rg + i] = acc[blk][i];
    if (rg == 0) {
      s_m[wave][n] = m_run;
      s_l[wave][n] = l_run;
    }
  }
  __syncthreads();
  for (int idx = tid; idx < G * D; idx += 256) {
    const int hh = idx / D, d = idx - hh * D;
    const int h = kvh * G + hh;
    float M = fmaxf(fmaxf(s_m[0][hh], s_m[1][hh]), fmaxf(s_m[2][hh], s_m[3][hh]));
    float Ls = 0.f, o = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float mw = s_m[w][hh];
      const float scw = (mw == -INFINITY) ? 0.f : pow2_neg_int(mw - M);
      Ls += s_l[w][hh] * scw;
      o += s_acc[w][hh][d] * scw;
    }
    if (a.nsplit == 1) {  // whole context in this workgroup: no partials
      a.out[(size_t)b * a.H * D + h * D + d] = f2bf(o * (1.0f / Ls));
      continue;
    }
    const size_t pi = (size_t)(b * a.H + h) * a.nsplit + split;
    stf_coh(a.part_acc + pi * D + d, o);
    if (d == 0) {
      stf_coh(a.part_ml + pi * 2, M);
      stf_coh(a.part_ml + pi * 2 + 1, Ls);
    }
  }
  if (a.nsplit == 1) return;
  if (last_chunk_done(a.counters + b * a.Hkv + kvh, a.nsplit)) merge_partials<D>(a, b, kvh, G);
}

// Any even head width up to 256, any group size: one thread per position for q.k,
// one thread per column for p.V.  Slow path for shapes the tuned kernel skips.
template <bool I8>
__global__ __launch_bounds__(256) void attn_decode_generic(AttnArgs a) {
  const int split = blockIdx.z, kvh = blockIdx.y, b = blockIdx.x;
  const int seq = b / a.S;
  const int G = a.H / a.Hkv, D = a.D;
  const int L = min((a.pos_dev ? a.pos_dev[(size_t)seq * a.pos_stride] : a.start) + (b - seq * a.S) + 1, a.Tmax);
  const int chunk = (((L + a.nsplit - 1) / a.nsplit) + 63) & ~63;
  const int t0 = split * chunk;
  const int t1 = min(L, t0 + chunk);
  const int tid = threadIdx.x;
  __shared__ float s_p[256];
  __shared__ float s_red[4];
  __shared__ float s_q[256];
  const size_t row = (size_t)a.Hkv * D;
  const bf16_t* kb = a.k + (size_t)seq * a.Tmax * row + (size_t)kvh * D;
  const bf16_t* vb = a.v + (size_t)seq * a.Tmax * row + (size_t)kvh * D;
  // int8 mode: element (pos, d) is code * scale + min of its (pos, head) row, rounded to bf16
  const int8_t* kb8 = reinterpret_cast<const int8_t*>(a.k) + (size_t)seq * a.Tmax * row + (size_t)kvh * D;
  const int8_t* vb8 = reinterpret_cast<const int8_t*>(a.v) + (size_t)seq * a.Tmax * row + (size_t)kvh * D;
  const float* stb = I8 ? a.stats + ((size_t)seq * a.Hkv + kvh) * a.Tmax * 4 : nullptr;  // records of my (sequence, head)
  auto deq = [](int8_t c, float sc, float mn) {
    return bf2f(f2bf(__fadd_rn(__fmul_rn((float)((int)c + 128), sc), mn)));
  };
  for (int hh = 0; hh < G; ++hh) {
    const int h = kvh * G + hh;
    __syncthreads();
    if (tid < D) s_q[tid] = bf2f(a.q[(size_t)b * a.H * D + (size_t)h * D + tid]);
    __syncthreads();
    float m_run = -INFINITY, l_run = 0.f, acc = 0.f;
    for (int tb = t0; tb < t1; tb += 256) {
      const int pos = tb + tid;
      float s = -INFINITY;
      if (pos < t1) {
        float d_ = 0.f;
        if (I8) {
          const float sc = stb[(size_t)pos * 4], mn = stb[(size_t)pos * 4 + 1];
          for (int d = 0; d < D; ++d) d_ += s_q[d] * deq(kb8[(size_t)pos * row + d], sc, mn);
        } else {
          for (int d = 0; d < D; ++d) d_ += s_q[d] * bf2f(kb[(size_t)pos * row + d]);
        }
        s = d_ * (a.scale * OHARA_LOG2E);  // log2 units
      }
      float tm = wave_max(s);
      if ((tid & 63) == 0) s_red[tid >> 6] = tm;
      __syncthreads();
      tm = fmaxf(fmaxf(s_red[0], s_red[1]), fmaxf(s_red[2], s_red[3]));
      __syncthreads();
      const float mn = fmaxf(m_run, ceilf(tm));
      const float corr = pow2_neg_int(m_run - mn);
      const float pv = (pos < t1) ? __builtin_amdgcn_exp2f(s - mn) : 0.f;
      s_p[tid] = rbf(pv);  // the weights enter the value product rounded to bf16, the sum unrounded
      float ts = wave_sum(pv);
      if ((tid & 63) == 0) s_red[tid >> 6] = ts;
      __syncthreads();
      ts = ((s_red[0] + s_red[1]) + s_red[2]) + s_red[3];
      l_run = l_run * corr + ts;
      m_run = mn;
      acc *= corr;
      if (tid < D) {
        const int n = min(256, t1 - tb);
        if (I8) {
          for (int i = 0; i < n; ++i) {
            const float* rec = stb + (size_t)(tb + i) * 4;
            acc += s_p[i] * deq(vb8[(size_t)(tb + i) * row + tid], rec[2], rec[3]);
          }
        } else {
          for (int i = 0; i < n; ++i) acc += s_p[i] * bf2f(vb[(size_t)(tb + i) * row + tid]);
        }
      }
      __syncthreads();
    }
    if (a.nsplit == 1) {
      if (tid < D) a.out[(size_t)b * a.H * D + h * D + tid] = f2bf(acc * (1.0f / l_run));
      continue;
    }
    const size_t pi = (size_t)(b * a.H + h) * a.nsplit + split;
    if (tid < D) stf_coh(a.part_acc + pi * D + tid, acc);
    if (tid == 0) {
      stf_coh(a.part_ml + pi * 2, m_run);
      stf_coh(a.part_ml + pi * 2 + 1, l_run);
    }
  }
  if (a.nsplit == 1) return;
  if (last_chunk_done(a.counters + b * a.Hkv + kvh, a.nsplit)) merge_partials<256>(a, b, kvh, G);
}

template <int D, bool I8>
int launch_fast(const AttnArgs& a, int G, dim3 grid, hipStream_t st) {
  if (I8) {
    if (D == 128 && G > 1) {  // several heads share the dequantised rows: both products on the matrix cores
      if (G == 2) hipLaunchKernelGGL((attn_decode_i8_mfma_kernel<2>), grid, dim3(256), 0, st, a);
      else if (G == 4) hipLaunchKernelGGL((attn_decode_i8_mfma_kernel<4>), grid, dim3(256), 0, st, a);
      else return 1;
      return 0;
    }
    switch (G) {
      case 1: hipLaunchKernelGGL((attn_decode_i8_kernel<D, 1>), grid, dim3(256), 0, st, a); break;
      case 2: hipLaunchKernelGGL((attn_decode_i8_kernel<D, 2>), grid, dim3(256), 0, st, a); break;
      case 4: hipLaunchKernelGGL((attn_decode_i8_kernel<D, 4>), grid, dim3(256), 0, st, a); break;
      default: return 1;
    }
    return 0;
  }
  switch (G) {
    case 1: hipLaunchKernelGGL((attn_decode_kernel<D, 1>), grid, dim3(256), 0, st, a); break;
    case 2: hipLaunchKernelGGL((attn_decode_kernel<D, 2>), grid, dim3(256), 0, st, a); break;
    case 4: hipLaunchKernelGGL((attn_decode_kernel<D, 4>), grid, dim3(256), 0, st, a); break;
    default: return 1;
  }
  return 0;
}

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

}  // namespace

extern "C" {

int64_t ohara_attn_workspace_bytes(int batch, int h, int h_kv, int dh, int n_split) {
  if (batch < 1 || h < 1 || h_kv < 1 || dh < 1 || n_split < 1) return OHARA_EINVAL;
  size_t c = align256((size_t)batch * h_kv * sizeof(int));
  size_t ml = align256((size_t)batch * h * n_split * 2 * sizeof(float));
  size_t acc = align256((size_t)batch * h * n_split * dh * sizeof(float));
  return (int64_t)(c + ml + acc);
}

// `fixed_counter_bytes` > 0: the workspace keeps its counters in a region of that fixed size (the
// layout of the allocation-free entry point, whose array is shared by calls of different shapes).
static int attn_cached_impl(const uint16_t* q, const void* kcache, const void* vcache, const float* stats, bool i8,
                            int batch, int seq_len,
                            int h, int h_kv, int dh, int t_max, int pos, const int32_t* pos_dev, int pos_stride, int n_split,
                            void* workspace, uint16_t* out, void* stream, size_t fixed_counter_bytes = 0) {
  if (!q || !kcache || !vcache || !out) return OHARA_EINVAL;
  if (i8 && !stats) return OHARA_EINVAL;
  if (batch < 1 || seq_len < 1 || h < 1 || h_kv < 1 || h % h_kv || dh < 2 || (dh & 1) || dh > 256)
    return OHARA_EINVAL;
  if (t_max < 1 || n_split < 1 || n_split > 1024) return OHARA_EINVAL;
  if (n_split > 1 && ((h / h_kv) * n_split > OHARA_MERGE_CAP || h / h_kv > 64)) return OHARA_ESIZE;
  if (n_split > 1 && !workspace) return OHARA_EINVAL;
  if (!pos_dev && (pos < 0 || pos + seq_len > t_max)) return OHARA_EINVAL;
  if ((int64_t)batch * seq_len > INT32_MAX / 2 || h_kv > 65535) return OHARA_ESIZE;
  AttnArgs a{};
  a.q = q; a.k = reinterpret_cast<const bf16_t*>(kcache); a.v = reinterpret_cast<const bf16_t*>(vcache); a.out = out;
  a.stats = stats;
  a.B = batch; a.S = seq_len; a.H = h; a.Hkv = h_kv; a.D = dh; a.Tmax = t_max; a.start = pos; a.pos_dev = pos_dev;
  a.pos_stride = pos_stride;
  a.nsplit = n_split;
  batch *= seq_len;  // one workspace slot per query row
  char* ws = reinterpret_cast<char*>(workspace);
  a.counters = reinterpret_cast<int*>(ws);
  ws += fixed_counter_bytes ? fixed_counter_bytes : align256((size_t)batch * h_kv * sizeof(int));
  a.part_ml = reinterpret_cast<float*>(ws);
  ws += align256((size_t)batch * h * n_split * 2 * sizeof(float));
  a.part_acc = reinterpret_cast<float*>(ws);
  a.scale = 1.0f / sqrtf((float)dh);
  dim3 grid(batch, h_kv, n_split);
  hipStream_t st = (hipStream_t)stream;
  const int G = h / h_kv;
  int miss = 1;
  if (i8) {
    if (dh == 128) miss = launch_fast<128, true>(a, G, grid, st);
    else if (dh == 64) miss = launch_fast<64, true>(a, G, grid, st);
    if (miss) hipLaunchKernelGGL(attn_decode_generic<true>, grid, dim3(256), 0, st, a);
    return ohara_launch_status();
  }
  if (dh == 128) miss = launch_fast<128, false>(a, G, grid, st);
  else if (dh == 64) miss = launch_fast<64, false>(a, G, grid, st);
  if (miss) hipLaunchKernelGGL(attn_decode_generic<false>, grid, dim3(256), 0, st, a);
  return ohara_launch_status();
}

int ohara_attn_cached_bf16(const uint16_t* q, const uint16_t* kcache, const uint16_t* vcache, int batch,
                           int seq_len, int h, int h_kv, int dh, int t_max, int pos, const int32_t* pos_dev,
                           int n_split, void* workspace, uint16_t* out, void* stream) {
  return attn_cached_impl(q, kcache, vcache, nullptr, false, batch, seq_len, h, h_kv, dh, t_max, pos, pos_dev, 0,
                          n_split, workspace, out, stream);
}

int ohara_attn_cached_ragged_bf16(const uint16_t* q, const uint16_t* kcache, const uint16_t* vcache, int batch,
                                  int seq_len, int h, int h_kv, int dh, int t_max, const int32_t* seq_pos, int n_split,
                                  void* workspace, uint16_t* out, void* stream) {
  if (!seq_pos) return OHARA_EINVAL;
  return attn_cached_impl(q, kcache, vcache, nullptr, false, batch, seq_len, h, h_kv, dh, t_max, 0, seq_pos, 1,
                          n_split, workspace, out, stream);
}

int ohara_attn_cached_int8(const uint16_t* q, const int8_t* kcache, const int8_t* vcache, const float* stats, int batch,
                           int seq_len, int h, int h_kv, int dh, int t_max, int pos, const int32_t* pos_dev, int n_split,
                           void* workspace, uint16_t* out, void* stream) {
  return attn_cached_impl(q, kcache, vcache, stats, true, batch, seq_len, h, h_kv, dh, t_max, pos, pos_dev, 0, n_split,
                          workspace, out, stream);
}

int ohara_attn_cached_ragged_int8(const uint16_t* q, const int8_t* kcache, const int8_t* vcache, const float* stats,
                                  int batch, int seq_len, int h, int h_kv, int dh, int t_max, const int32_t* seq_pos,
                                  int n_split, void* workspace, uint16_t* out, void* stream) {
  if (!seq_pos) return OHARA_EINVAL;
  return attn_cached_impl(q, kcache, vcache, stats, true, batch, seq_len, h, h_kv, dh, t_max, 0, seq_pos, 1, n_split,
                          workspace, out, stream);
}

// ---- the same attention for callers that cannot allocate -------------------------------------
// The chunk partials and counters live in a file-scope device array instead of a caller-supplied
// workspace.  Layout: OHARA_SCRATCH_COUNTER_BYTES of counters (one int per (query row, kv head)),
// then the (max, sum) pairs, then the accumulators, as in ohara_attn_workspace_bytes.  Every GPU
// holds its own copy of the array; its address is looked up once per device.
#define OHARA_SCRATCH_COUNTER_BYTES (64 * 1024)
#define OHARA_SCRATCH_BYTES (OHARA_SCRATCH_COUNTER_BYTES + 8 * 1024 * 1024)
#define OHARA_SCRATCH_MAX_DEVICES 64
static __device__ __align__(256) unsigned char scratch[OHARA_SCRATCH_BYTES];

static __global__ void scratch_clear_kernel(int* p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

// Device address of `scratch` on the current device (nullptr on failure).  The array's name is only
// a host-side handle; kernels and fills must be given this address.
static unsigned char* scratch_device_ptr() {
  static unsigned char* ptrs[OHARA_SCRATCH_MAX_DEVICES];
  static std::mutex mu;
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= OHARA_SCRATCH_MAX_DEVICES) return nullptr;
  std::lock_guard<std::mutex> lock(mu);
  if (!ptrs[dev]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess) return nullptr;
    ptrs[dev] = reinterpret_cast<unsigned char*>(p);
  }
  return ptrs[dev];
}

int ohara_attn_cached_bf16_noalloc(const uint16_t* q, const uint16_t* kcache, const uint16_t* vcache, int batch,
                                   int seq_len, int h, int h_kv, int dh, int t_max, int pos, const int32_t* pos_dev,
                                   int n_split, uint16_t* out, void* stream) {
  if (batch < 1 || seq_len < 1 || h < 1 || h_kv < 1 || dh < 1 || n_split < 1) return OHARA_EINVAL;
  const size_t rows = (size_t)batch * seq_len;
  const size_t counters = rows * h_kv * sizeof(int);
  const size_t need = OHARA_SCRATCH_COUNTER_BYTES + align256(rows * h * n_split * 2 * sizeof(float)) +
                      align256(rows * h * n_split * dh * sizeof(float));
  if (counters > OHARA_SCRATCH_COUNTER_BYTES || need > OHARA_SCRATCH_BYTES) return OHARA_ESIZE;
  unsigned char* ws = scratch_device_ptr();
  if (!ws) return OHARA_ELAUNCH;
  if (n_split > 1) {
    // the counters must start at zero whatever an earlier call (of any shape) left behind; a fill
    // kernel rather than a memset node, so that the call can be recorded into a graph
    const int n = (int)(rows * h_kv);
    hipLaunchKernelGGL(scratch_clear_kernel, dim3((n + 255) / 256), dim3(256), 0, (hipStream_t)stream,
                       reinterpret_cast<int*>(ws), n);
    if (ohara_launch_status() != OHARA_OK) return OHARA_ELAUNCH;
  }
  return attn_cached_impl(q, kcache, vcache, nullptr, false, batch, seq_len, h, h_kv, dh, t_max, pos, pos_dev, 0,
                          n_split, ws, out, stream, OHARA_SCRATCH_COUNTER_BYTES);
}

}  // extern "C"
