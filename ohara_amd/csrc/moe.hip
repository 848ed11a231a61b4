// Grouped mixture-of-experts feed-forward for decode (eval mode of GroupedMoE,
// ohara/modules/moe_grouped.py:122-228; same routing as the loop variant ohara/modules/moe.py:65-127).
//
//   route    logits = float(bf16 router Linear) (:126); experts = first k of top-(k+1) of
//            logits + router_bias (:129-133) or plain top-k (:135), ties to the lowest id;
//            weights = softmax over the k selected UNBIASED logits (:140-142) or sigmoid,
//            optionally normalised (:144-146); cast to bf16 (:217)
//   sort     (token, slot) pairs grouped by expert, token order kept inside an expert (the
//            stable argsort + bincount + cumsum of :165-168), as a counting sort in LDS
//   experts  per expert e and its pairs: hidden = bf16(silu(bf16(x W_gate[e]))) * bf16(x W_up[e]),
//            y = bf16(bf16(hidden W_down[e]) * weight) (:175-181) - the expert weights are
//            streamed once per 16-token column tile through the same packed MFMA tiles as the
//            dense projections (at ~8 tokens per expert this is a weight stream, not a GEMM)
//   combine  out[token] = sum over its experts in ascending expert id, each add rounded to bf16
//            (index_add_ in the activation dtype, :184), + shared expert (:206-207,219-220),
//            + residual (ohara/models/llama.py:200)
#include "common.h"

namespace {

// ---- routing ---------------------------------------------------------------------------------
// The selection and the weights of one token by one wave: lane l holds experts l, l + 64, ... (raw: the unbiased
// logits, sel: what the top-k looks at, -inf past E); lanes below k end up with one selected expert and its weight.
template <int MAXPL>
__device__ __forceinline__ void route_core(float (&sel)[MAXPL], const float (&raw)[MAXPL], int E, int k, int sigmoid,
                                           int normalize, int lane, int& my_id, float& wt) {
  // Winner j is kept by lane j; the arg-max butterfly runs on DPP moves and row swaps.
  float my_raw = 0.f;
  my_id = 0;
  for (int j = 0; j < k; ++j) {
    // lane-local best (lowest id on ties), then across the wave
    float bv = -INFINITY;
    int bi = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < MAXPL; ++i) {
      const int e = i * 64 + lane;
      if (e < E && (sel[i] > bv || (sel[i] == bv && e < bi))) {
        bv = sel[i];
        bi = e;
      }
    }
    lane_xor_argmax<32>(bv, bi);
    lane_xor_argmax<16>(bv, bi);
    lane_xor_argmax<8>(bv, bi);
    lane_xor_argmax<4>(bv, bi);
    lane_xor_argmax<2>(bv, bi);
    lane_xor_argmax<1>(bv, bi);
    // fetch the unbiased logit of the winner and retire it
    float r = 0.f;
#pragma unroll
    for (int i = 0; i < MAXPL; ++i)
      if (i * 64 + lane == bi) {
        r = raw[i];
        sel[i] = -INFINITY;
      }
    r = __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(r), bi & 63));
    if (lane == j) {
      my_raw = r;
      my_id = bi;
    }
  }
  // weights: every lane below k holds one; the sums run in slot order, as a loop over the slots would
  const bool has = lane < k;
  if (!sigmoid) {
    const float m = wave_max(has ? my_raw : -INFINITY);
    const float e = has ? expf(my_raw - m) : 0.f;
    float z = 0.f;
    for (int j = 0; j < k; ++j) z += __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(e), j));
    wt = e / z;
  } else {
    const float sg = has ? 1.0f / (1.0f + expf(-my_raw)) : 0.f;
    float z = 0.f;
    for (int j = 0; j < k; ++j) z += __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(sg), j));
    wt = normalize ? sg / fmaxf(z, 1e-9f) : sg;
  }
}

// one wave per token; E <= 64 * MAXPL experts (MAXPL experts per lane), k <= 16
template <int MAXPL>
__global__ __launch_bounds__(256) void moe_route_kernel(const bf16_t* logits, int ldl, const bf16_t* bias, int N, int E,
                                                        int k, int biased, int sigmoid, int normalize, int32_t* idx,
                                                        bf16_t* w) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n = blockIdx.x * 4 + wave;
  if (n >= N) return;
  float sel[MAXPL], raw[MAXPL];
#pragma unroll
  for (int i = 0; i < MAXPL; ++i) {
    const int e = i * 64 + lane;
    if (e < E) {
      raw[i] = bf2f(logits[(size_t)n * ldl + e]);
      sel[i] = biased ? raw[i] + bf2f(bias[e]) : raw[i];
    } else {
      raw[i] = 0.f;
      sel[i] = -INFINITY;
    }
  }
  int my_id;
  float wt;
  route_core<MAXPL>(sel, raw, E, k, sigmoid, normalize, lane, my_id, wt);
  if (lane < k) {
    idx[(size_t)n * k + lane] = my_id;
    w[(size_t)n * k + lane] = f2bf(wt);
  }
}

// ---- counting sort of the (token, slot) pairs by expert -----------------------------------------
// offs[e] .. offs[e+1]: pairs of expert e, in token order; pair_of[sorted position] = n*k + j;
// pos_of[n*k + j] = sorted position.  One workgroup; N*k <= 65536, E <= 1024.
__global__ __launch_bounds__(1024) void moe_sort_kernel(const int32_t* idx, int NK, int E, int32_t* offs, int32_t* pair_of,
                                                        int32_t* pos_of) {
  __shared__ int cnt[1025];   // histogram, then the next free sorted position of every expert
  __shared__ __align__(16) int sidx[1024];  // expert ids of the current block of 1024 pairs
  const int tid = threadIdx.x;
  for (int e = tid; e <= E; e += 1024) cnt[e] = 0;
  __syncthreads();
  for (int p = tid; p < NK; p += 1024) atomicAdd(&cnt[idx[p]], 1);
  __syncthreads();
  if (tid == 0) {
    int run = 0;
    for (int e = 0; e < E; ++e) {
      const int c = cnt[e];
      cnt[e] = run;
      offs[e] = run;
      run += c;
    }
    offs[E] = run;
  }
  __syncthreads();
  // stable placement, 1024 pairs at a time: a pair's position is its expert's next free slot
  // plus the number of earlier pairs of the block with the same expert (LDS broadcast reads)
  for (int p0 = 0; p0 < NK; p0 += 1024) {
    const int p = p0 + tid;
    const int e = p < NK ? idx[p] : -1;
    sidx[tid] = e;
    __syncthreads();
    // only earlier pairs count: a wave scans the entries below its last lane, and a wave without a
    // valid pair scans nothing (entries past the end hold -1 and never match)
    const int wave_first = tid & ~63;
    const int n4 = p0 + wave_first < NK ? (min(wave_first + 64, NK - p0) + 3) >> 2 : 0;
    int rank = 0;
    const int4* s4 = reinterpret_cast<const int4*>(sidx);
#pragma unroll 4
    for (int t4 = 0; t4 < n4; ++t4) {
      const int4 v = s4[t4];
      const int t = 4 * t4;
      rank += (t < tid && v.x == e) + (t + 1 < tid && v.y == e) + (t + 2 < tid && v.z == e) + (t + 3 < tid && v.w == e);
    }
    if (e >= 0) {
      const int o = cnt[e] + rank;
      pair_of[o] = p;
      pos_of[p] = o;
    }
    __syncthreads();
    if (e >= 0) atomicAdd(&cnt[e], 1);
    __syncthreads();
  }
}

// The same sort for at most 64 experts and 1024 pairs (decode): a pair's rank among the earlier pairs of
// its expert is a ballot match inside its wave (six ballots for the six bits of an expert id) plus the
// counts of the waves before it, instead of a scan over all earlier pairs; the offsets are one wave's scan.
__global__ __launch_bounds__(1024) void moe_sort_small_kernel(const int32_t* idx, int NK, int E, int32_t* offs,
                                                              int32_t* pair_of, int32_t* pos_of) {
  __shared__ int wcnt[16][64];   // pairs of expert e in wave w, then the first sorted position of that wave's pairs of e
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  wcnt[wave][lane] = 0;
  const int e = tid < NK ? idx[tid] : -1;
  unsigned long long same = __ballot(e >= 0);
#pragma unroll
  for (int bit = 0; bit < 6; ++bit) {
    const unsigned long long b = __ballot((e >> bit) & 1);
    same &= ((e >> bit) & 1) ? b : ~b;
  }
  const int rank = __popcll(same & ((1ull << lane) - 1ull));
  __syncthreads();
  if (e >= 0 && (same >> lane) == 1ull) wcnt[wave][e] = __popcll(same);  // the last lane of the wave with this expert
  __syncthreads();
  if (wave == 0) {
    int tot = 0, c[16];
#pragma unroll
    for (int w = 0; w < 16; ++w) {
      c[w] = wcnt[w][lane];
      tot += c[w];
    }
    const int incl = wave_incl_scan_i(lane < E ? tot : 0);
    int run = incl - (lane < E ? tot : 0);
    if (lane < E) offs[lane] = run;
    if (lane == 63) offs[E] = incl;  // lanes at and past E added nothing
#pragma unroll
    for (int w = 0; w < 16; ++w) {
      wcnt[w][lane] = run;
      run += c[w];
    }
  }
  __syncthreads();
  if (e >= 0) {
    const int o = wcnt[wave][e] + rank;
    pair_of[o] = tid;
    pos_of[tid] = o;
  }
}

// ---- norm + router + selection + sort in one launch (decode: at most 64 experts and 1024 pairs) -------
// What precedes the experts is four small steps on the same rows - RMSNorm (ohara/modules/norm.py:16-21), the router
// Linear, the selection, the sort of the pairs - and as four launches they cost four launch latencies for a few
// microseconds of work.  Here a workgroup takes four tokens, one per wave: the wave norms its row (into LDS for the
// router product and out to memory for the experts), wave s multiplies the four rows with strip s of the router's
// packed weights (16 experts, the whole contraction in one wave; the products are rounded to bf16 as the Linear's
// output is), every wave selects for its token, and the workgroup that finishes last sorts the pairs of all tokens.
struct RouteFusedArgs {
  const bf16_t* x;        // (N, d) rows before the norm
  int ldx;
  const bf16_t* norm_w;
  float eps;
  const uint4* wp;        // the router's packed rows: [strip][KS][64]
  const bf16_t* bias;
  int N, d, E, k, biased, sigmoid, normalize;
  bf16_t* xn;             // (N, d) normalised rows
  int ldxn;
  bf16_t* logits;         // optional (N, E) router outputs
  int ldl;
  int32_t* idx;           // (N, k)
  bf16_t* w;              // (N, k)
  int32_t* offs;
  int32_t* pair_of;
  int32_t* pos_of;
  int* counter;           // one word, zero between calls
};

// moe_sort_small_kernel's sort by 256 threads: a thread takes pairs tid + 256 r; a "wave" of that kernel is a run of 64
// consecutive pairs, four of which a wave here handles one after the other.  idx is read past the caches (other
// workgroups wrote it in this launch).
__device__ __forceinline__ void sort_small_256(const int32_t* idx, int NK, int E, int32_t* offs, int32_t* pair_of,
                                               int32_t* pos_of, int (*wcnt)[64]) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int e[4], rank[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) wcnt[wave + 4 * r][lane] = 0;
  __syncthreads();
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int p = tid + 256 * r;
    e[r] = p < NK ? (int)ld_coh4(idx + p) : -1;
    unsigned long long same = __ballot(e[r] >= 0);
#pragma unroll
    for (int bit = 0; bit < 6; ++bit) {
      const unsigned long long b = __ballot((e[r] >> bit) & 1);
      same &= ((e[r] >> bit) & 1) ? b : ~b;
    }
    rank[r] = __popcll(same & ((1ull << lane) - 1ull));
    if (e[r] >= 0 && (same >> lane) == 1ull) wcnt[wave + 4 * r][e[r]] = __popcll(same);  // the run's last pair of this expert
  }
  __syncthreads();
  if (wave == 0) {
    int tot = 0, c[16];
#pragma unroll
    for (int w = 0; w < 16; ++w) {
      c[w] = wcnt[w][lane];
      tot += c[w];
    }
    const int incl = wave_incl_scan_i(lane < E ? tot : 0);
    int run = incl - (lane < E ? tot : 0);
    if (lane < E) offs[lane] = run;
    if (lane == 63) offs[E] = incl;  // lanes at and past E added nothing
#pragma unroll
    for (int w = 0; w < 16; ++w) {
      wcnt[w][lane] = run;
      run += c[w];
    }
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < 4; ++r)
    if (e[r] >= 0) {
      const int p = tid + 256 * r;
      const int o = wcnt[wave + 4 * r][e[r]] + rank[r];
      pair_of[o] = p;
      pos_of[p] = o;
    }
}

__global__ __launch_bounds__(256) void moe_route_fused_kernel(RouteFusedArgs a) {
  extern __shared__ __align__(16) unsigned char route_smem[];
  __shared__ float slog[4][64];
  __shared__ int wcnt[16][64];
  __shared__ int is_last;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int KS = (a.d + 31) >> 5;
  const int ldxs = KS * 32 + 8;
  bf16_t* xs = reinterpret_cast<bf16_t*>(route_smem);  // four normalised rows
  const int t0 = blockIdx.x * 4;
  // 1. RMSNorm, a row per wave (the row stays in registers between the sum and the scaling):
  //    y = bf16(bf16(x * rinv) * w), rinv = 1 / sqrt(mean(x^2) + eps)
  {
    const int n = t0 + wave;
    const bf16_t* xr = a.x + (size_t)min(n, a.N - 1) * a.ldx;
    uint4 xv[8], gv[8];  // (d <= 4096)
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      const int i = (c * 64 + lane) * 8;
      xv[c] = i < a.d ? ldg16(xr + i) : make_uint4(0, 0, 0, 0);
      gv[c] = i < a.d ? ldg16(a.norm_w + i) : make_uint4(0, 0, 0, 0);
    }
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      const uint32_t u[4] = {xv[c].x, xv[c].y, xv[c].z, xv[c].w};
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float lo = lo_bf(u[q]), hi = hi_bf(u[q]);
        ss += lo * lo + hi * hi;
      }
    }
    ss = wave_sum(ss);
    const float rinv = 1.0f / sqrtf(ss / (float)a.d + a.eps);
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      const int i = (c * 64 + lane) * 8;
      if (i < KS * 32) {  // (the columns between d and the next multiple of 32 are zero for the product)
        const uint32_t u[4] = {xv[c].x, xv[c].y, xv[c].z, xv[c].w}, gw[4] = {gv[c].x, gv[c].y, gv[c].z, gv[c].w};
        uint32_t y[4];
#pragma unroll
        for (int q = 0; q < 4; ++q)
          y[q] = pack_bf(rbf(lo_bf(u[q]) * rinv) * lo_bf(gw[q]), rbf(hi_bf(u[q]) * rinv) * hi_bf(gw[q]));
        const uint4 o = make_uint4(y[0], y[1], y[2], y[3]);
        if (n < a.N && i < a.d) *reinterpret_cast<uint4*>(a.xn + (size_t)n * a.ldxn + i) = o;
        *reinterpret_cast<uint4*>(xs + (size_t)wave * ldxs + i) = o;
      }
    }
  }
  __syncthreads();
  // 2. the router product: wave s takes strip s (experts 16 s ..) over the whole contraction, the four tokens in
  //    columns 0..3 (the other columns repeat them and are dropped), sixteen k-steps of weights in flight
  {
    const int m = lane & 15, g = lane >> 4;
    const int strips = (a.E + 15) >> 4;
    if (wave < strips) {
      const uint4* wrow = a.wp + (size_t)wave * KS * 64 + lane;
      const bf16_t* xrow = xs + (size_t)(m & 3) * ldxs + 8 * g;
      f32x4 acc = (f32x4){0.f, 0.f, 0.f, 0.f};
      for (int jb = 0; jb < KS; jb += 16) {
        uint4 wv[16];
#pragma unroll
        for (int c = 0; c < 16; ++c) wv[c] = ldg16_nt(wrow + (size_t)min(jb + c, KS - 1) * 64);
#pragma unroll
        for (int c = 0; c < 16; ++c) {
          if (jb + c < KS) {
            const uint4 xv = *reinterpret_cast<const uint4*>(xrow + 32 * (jb + c));
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wv[c]), __builtin_bit_cast(bf16x8, xv),
                                                          acc, 0, 0, 0);
          }
        }
      }
      if (m < 4) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int e = 16 * wave + 4 * g + i;
          const float y = rbf(acc[i]);
          slog[m][e] = y;
          if (a.logits && e < a.E && t0 + m < a.N) a.logits[(size_t)(t0 + m) * a.ldl + e] = f2bf(y);
        }
      }
    }
  }
  __syncthreads();
  // 3. the selection: a token per wave, lane = expert
  {
    const int n = t0 + wave;
    if (n < a.N) {  // (wave-uniform)
      float raw[1], sel[1];
      raw[0] = lane < a.E ? slog[wave][lane] : 0.f;
      sel[0] = lane < a.E ? (a.biased ? raw[0] + bf2f(a.bias[lane]) : raw[0]) : -INFINITY;
      int my_id;
      float wt;
      route_core<1>(sel, raw, a.E, a.k, a.sigmoid, a.normalize, lane, my_id, wt);
      if (lane < a.k) {
        st_coh4(a.idx + (size_t)n * a.k + lane, (uint32_t)my_id);  // (read by the workgroup that sorts)
        a.w[(size_t)n * a.k + lane] = f2bf(wt);
      }
    }
  }
  // 4. the workgroup that finishes last sorts all pairs
  wait_own_stores();
  __syncthreads();
  if (tid == 0) {
    const int old = __hip_atomic_fetch_add(a.counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    is_last = old == (int)gridDim.x - 1;
    if (is_last) __hip_atomic_store(a.counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next call
  }
  __syncthreads();
  if (is_last) sort_small_256(a.idx, a.N * a.k, a.E, a.offs, a.pair_of, a.pos_of, wcnt);
}

// ---- expert projections --------------------------------------------------------------------------
enum { X_SWIGLU = 0, X_DOWN = 1 };

struct ExpertArgs {
  const uint4* wp;        // [E][strips][KS][64] packed rows of every expert
  size_t expert_stride;   // uint4 per expert
  const bf16_t* x;        // X_SWIGLU: (N, K) activations, gathered by token; X_DOWN: (NK, K) by sorted position
  int ldx;
  const int32_t* offs;    // (E+1)
  const int32_t* pair_of; // (NK)
  const bf16_t* w;        // (NK) routing weights, pair order (X_DOWN)
  int k;                  // experts per token
  int N_out, K;           // output width (X_SWIGLU: hidden F; X_DOWN: d) and contraction length
  bf16_t* out;            // (NK, N_out) by sorted position
  int ldo;
  // The shared expert (moe_grouped.py:206-207, 219-220) as more rows of the grid, blockIdx.y >= E, 16 tokens a row:
  // every token is its "pair" (row n of x_sh -> row n of out_sh), its weights have their own widths, and its output
  // is not scaled.
  int E, N_sh;            // experts; tokens of the shared expert (0: none)
  const uint4* wp_sh;
  const bf16_t* x_sh;     // X_SWIGLU: (N, K) the tokens' rows; X_DOWN: (N, K_sh) the shared expert's activations
  int ldx_sh;
  int N_out_sh, K_sh;
  bf16_t* out_sh;
  int ldo_sh;
};

// CH: k-steps a wave has in flight at once (the host takes 4 when a wave's share of K is that short).
// Every load of a batch is issued whatever its index - clamped into the strip and the row, zeroed
// afterwards where it lies beyond the wave's share - so the batch is one run of loads without branches.
template <int EPI, int CH>
__global__ __launch_bounds__(256) void moe_expert_kernel(ExpertArgs a) {
  const int strip = blockIdx.x, e = blockIdx.y;
  const bool sh = e >= a.E;  // (workgroup-uniform) a row of the shared expert: 16 tokens each
  const int p0 = sh ? (e - a.E) * 16 : a.offs[e], p1 = sh ? min(a.N_sh, p0 + 16) : a.offs[e + 1];
  if (p0 >= p1) return;
  const int N_out = sh ? a.N_out_sh : a.N_out, K = sh ? a.K_sh : a.K;
  if (strip * 16 >= (EPI == X_SWIGLU ? 2 * ((N_out + 7) / 8 * 8) : N_out)) return;  // (the grid is as wide as the widest)
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m = lane & 15, g = lane >> 4;
  const int KS = (K + 31) >> 5;
  const int per = (KS + 3) >> 2;
  const int j0 = wave * per, j1 = min(KS, j0 + per);
  __shared__ float red[3][64][4];
  const uint4* wrow = (sh ? a.wp_sh : a.wp + (size_t)e * a.expert_stride) + (size_t)strip * KS * 64 + lane;
  bf16_t* const outp = sh ? a.out_sh : a.out;
  const int ldo = sh ? a.ldo_sh : a.ldo;
  for (int pt = p0; pt < p1; pt += 16) {  // 16-token column tiles of this expert
    const int pos = pt + m;
    const bool has = pos < p1;
    const int posc = min(pos, p1 - 1);  // a token of this expert: lanes past the end compute a column nobody stores
    const int pair = sh ? 0 : a.pair_of[posc];
    const bf16_t* xrow = sh ? a.x_sh + (size_t)posc * a.ldx_sh
                            : a.x + (size_t)((EPI == X_SWIGLU) ? pair / a.k : posc) * a.ldx;
    float wt = 1.0f;  // (the shared expert's output is not scaled: a bf16 value times one is itself)
    if (EPI == X_DOWN && !sh) wt = bf2f(a.w[pair]);  // asked for here, used in the epilogue
    f32x4 acc = (f32x4){0.f, 0.f, 0.f, 0.f};
    for (int jb = j0; jb < j1; jb += CH) {
      uint4 wv[CH], xv[CH];
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        const int j = min(jb + c, j1 - 1);
        wv[c] = ldg16_nt(wrow + (size_t)j * 64);
        xv[c] = ldg16(xrow + min(32 * j + 8 * g, K - 8));
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        const bool live = jb + c < j1 && 32 * (jb + c) + 8 * g < K;
        if (!live) xv[c] = make_uint4(0, 0, 0, 0);  // the packed weights are zero beyond K; the row's values are not
        if (jb + c >= j1) wv[c] = make_uint4(0, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wv[c]), __builtin_bit_cast(bf16x8, xv[c]),
                                                      acc, 0, 0, 0);
      }
    }
    if (wave > 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i) red[wave - 1][lane][i] = acc[i];
    }
    __syncthreads();
    if (wave == 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] = ((acc[i] + red[0][lane][i]) + red[1][lane][i]) + red[2][lane][i];
      if (has) {
        const float y0 = rbf(acc[0]), y1 = rbf(acc[1]), y2 = rbf(acc[2]), y3 = rbf(acc[3]);
        if (EPI == X_SWIGLU) {
          const int f = strip * 8 + 2 * g;
          bf16_t* o = outp + (size_t)pos * ldo + f;
          if (f < N_out) o[0] = f2bf(rbf(silu_f(y0)) * y2);
          if (f + 1 < N_out) o[1] = f2bf(rbf(silu_f(y1)) * y3);
        } else {
          const int r0 = strip * 16 + 4 * g;
          const float v[4] = {y0 * wt, y1 * wt, y2 * wt, y3 * wt};
          bf16_t* o = outp + (size_t)pos * ldo + r0;
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (r0 + i < N_out) o[i] = f2bf(v[i]);
        }
      }
    }
    __syncthreads();
  }
}

// ---- combine ---------------------------------------------------------------------------------------
// out[n] = resid[n] + ( (sum over the token's experts, ascending id, bf16 adds) + shared[n] )
__global__ __launch_bounds__(256) void moe_combine_kernel(const bf16_t* y, int ldy, const int32_t* idx, const int32_t* pos_of,
                                                          int k, const bf16_t* shared, int lds_, const bf16_t* resid, int ldr,
                                                          bf16_t* out, int ldo, int d) {
  const int n = blockIdx.x;
  __shared__ int order[16];
  if (threadIdx.x < 64) {
    // slots of this token in ascending expert id (k <= 16 distinct experts): lane j ranks its own slot
    const int lane = threadIdx.x;
    const int mine = lane < k ? idx[(size_t)n * k + lane] : 0x7fffffff;
    const int pos = lane < k ? pos_of[(size_t)n * k + lane] : 0;
    int rank = 0;
    for (int j = 0; j < k; ++j) {
      const int other = __shfl(mine, j, WAVE);
      rank += (other < mine || (other == mine && j < lane)) ? 1 : 0;
    }
    if (lane < k) order[rank] = pos;
  }
  __syncthreads();
  const bool vec = ((d | ldy | ldo | lds_ | ldr) & 3) == 0;
  if (vec) {  // four columns per thread, 8-byte loads; the adds stay one bf16 add per expert, in order
    for (int c = threadIdx.x * 4; c < d; c += 1024) {
      uint2 yv[16];
#pragma unroll
      for (int j = 0; j < 16; ++j) yv[j] = j < k ? ldg8(y + (size_t)order[j] * ldy + c) : make_uint2(0, 0);
      const uint2 sv = shared ? ldg8(shared + (size_t)n * lds_ + c) : make_uint2(0, 0);
      const uint2 rv = resid ? ldg8(resid + (size_t)n * ldr + c) : make_uint2(0, 0);
      float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < 16; ++j)
        if (j < k) {
          acc[0] = rbf(acc[0] + lo_bf(yv[j].x)); acc[1] = rbf(acc[1] + hi_bf(yv[j].x));
          acc[2] = rbf(acc[2] + lo_bf(yv[j].y)); acc[3] = rbf(acc[3] + hi_bf(yv[j].y));
        }
      if (shared) {
        acc[0] = rbf(acc[0] + lo_bf(sv.x)); acc[1] = rbf(acc[1] + hi_bf(sv.x));
        acc[2] = rbf(acc[2] + lo_bf(sv.y)); acc[3] = rbf(acc[3] + hi_bf(sv.y));
      }
      if (resid) {
        acc[0] = rbf(lo_bf(rv.x) + acc[0]); acc[1] = rbf(hi_bf(rv.x) + acc[1]);
        acc[2] = rbf(lo_bf(rv.y) + acc[2]); acc[3] = rbf(hi_bf(rv.y) + acc[3]);
      }
      stg8(out + (size_t)n * ldo + c, make_uint2(pack_bf(acc[0], acc[1]), pack_bf(acc[2], acc[3])));
    }
    return;
  }
  for (int c = threadIdx.x; c < d; c += 256) {
    float acc = 0.f;
    for (int j = 0; j < k; ++j) acc = rbf(acc + bf2f(y[(size_t)order[j] * ldy + c]));
    if (shared) acc = rbf(acc + bf2f(shared[(size_t)n * lds_ + c]));
    if (resid) acc = rbf(bf2f(resid[(size_t)n * ldr + c]) + acc);
    out[(size_t)n * ldo + c] = f2bf(acc);
  }
}

}  // namespace

extern "C" {

int ohara_moe_route_topk(const uint16_t* router_logits, int ldl, const uint16_t* router_bias, int n_tokens, int n_experts,
                         int k, int biased_topk, int gate_sigmoid, int normalize, int32_t* expert_idx,
                         uint16_t* expert_w, void* stream) {
  if (!router_logits || !expert_idx || !expert_w || n_tokens < 1 || n_experts < 1 || k < 1) return OHARA_EINVAL;
  if (k > 16 || n_experts > 1024 || k > n_experts || ldl < n_experts) return OHARA_ESIZE;
  if (biased_topk && !router_bias) return OHARA_EINVAL;
  const dim3 grid((n_tokens + 3) / 4), block(256);
#define OHARA_ROUTE(PL_)                                                                                            \
  hipLaunchKernelGGL(moe_route_kernel<PL_>, grid, block, 0, (hipStream_t)stream, router_logits, ldl, router_bias, \
                     n_tokens, n_experts, k, biased_topk, gate_sigmoid, normalize, expert_idx, expert_w)
  if (n_experts <= 64) OHARA_ROUTE(1);
  else if (n_experts <= 256) OHARA_ROUTE(4);
  else OHARA_ROUTE(16);
#undef OHARA_ROUTE
  return ohara_launch_status();
}

int ohara_moe_route_fused(const uint16_t* x, int ldx, const uint16_t* norm_w, float eps, const uint16_t* router_wp,
                          const uint16_t* router_bias, int n_tokens, int d, int n_experts, int k, int biased_topk,
                          int gate_sigmoid, int normalize, uint16_t* x_norm, int ld_x_norm, uint16_t* router_logits, int ldl,
                          int32_t* expert_idx, uint16_t* expert_w, int32_t* offsets, int32_t* pair_of, int32_t* pos_of,
                          int32_t* counter, void* stream) {
  if (!x || !norm_w || !router_wp || !x_norm || !expert_idx || !expert_w || !offsets || !pair_of || !pos_of || !counter)
    return OHARA_EINVAL;
  if (n_tokens < 1 || d < 8 || (d & 7) || (ldx & 7) || (ld_x_norm & 7) || k < 1 || n_experts < 1) return OHARA_EINVAL;
  if (n_experts > 64 || k > 16 || k > n_experts || (int64_t)n_tokens * k > 1024 || d > 4096) return OHARA_ESIZE;
  if (biased_topk && !router_bias) return OHARA_EINVAL;
  if (router_logits && ldl < n_experts) return OHARA_EINVAL;
  RouteFusedArgs a{};
  a.x = x; a.ldx = ldx; a.norm_w = norm_w; a.eps = eps; a.wp = reinterpret_cast<const uint4*>(router_wp); a.bias = router_bias;
  a.N = n_tokens; a.d = d; a.E = n_experts; a.k = k; a.biased = biased_topk; a.sigmoid = gate_sigmoid; a.normalize = normalize;
  a.xn = x_norm; a.ldxn = ld_x_norm; a.logits = router_logits; a.ldl = ldl; a.idx = expert_idx; a.w = expert_w;
  a.offs = offsets; a.pair_of = pair_of; a.pos_of = pos_of; a.counter = counter;
  const size_t smem = (size_t)4 * (((d + 31) / 32) * 32 + 8) * sizeof(bf16_t);
  hipLaunchKernelGGL(moe_route_fused_kernel, dim3((n_tokens + 3) / 4), dim3(256), smem, (hipStream_t)stream, a);
  return ohara_launch_status();
}

int ohara_moe_sort_pairs(const int32_t* expert_idx, int n_pairs, int n_experts, int32_t* offsets, int32_t* pair_of,
                         int32_t* pos_of, void* stream) {
  if (!expert_idx || !offsets || !pair_of || !pos_of || n_pairs < 1 || n_experts < 1) return OHARA_EINVAL;
  if (n_pairs > 65536 || n_experts > 1024) return OHARA_ESIZE;
  if (n_experts <= 64 && n_pairs <= 1024)
    hipLaunchKernelGGL(moe_sort_small_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, expert_idx, n_pairs, n_experts,
                       offsets, pair_of, pos_of);
  else
    hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, expert_idx, n_pairs, n_experts, offsets,
                       pair_of, pos_of);
  return ohara_launch_status();
}

int ohara_moe_experts_gate_up_shared(const uint16_t* x, int ldx, const uint16_t* wp_gate_up, int64_t expert_stride_bytes,
                                     int n_experts, int hidden, int d, int k, const int32_t* offsets,
                                     const int32_t* pair_of, uint16_t* act, int ld_act, const uint16_t* wp_shared,
                                     int shared_hidden, int n_tokens, uint16_t* act_shared, int ld_act_shared,
                                     void* stream) {
  if (!x || !wp_gate_up || !offsets || !pair_of || !act || hidden < 1 || d < 1 || (d & 7) || (ldx & 7)) return OHARA_EINVAL;
  ExpertArgs a{};
  a.wp = reinterpret_cast<const uint4*>(wp_gate_up); a.expert_stride = (size_t)expert_stride_bytes / 16;
  a.x = x; a.ldx = ldx; a.offs = offsets; a.pair_of = pair_of; a.k = k; a.N_out = hidden; a.K = d;
  a.out = act; a.ldo = ld_act; a.E = n_experts;
  int strips = 2 * ((hidden + 7) / 8 * 8) / 16;
  int rows = n_experts;
  if (wp_shared) {  // the shared expert: a row of the grid per 16 tokens
    if (!act_shared || n_tokens < 1 || shared_hidden < 1 || ld_act_shared < shared_hidden) return OHARA_EINVAL;
    a.N_sh = n_tokens; a.wp_sh = reinterpret_cast<const uint4*>(wp_shared); a.x_sh = x; a.ldx_sh = ldx;
    a.N_out_sh = shared_hidden; a.K_sh = d; a.out_sh = act_shared; a.ldo_sh = ld_act_shared;
    const int s2 = 2 * ((shared_hidden + 7) / 8 * 8) / 16;
    strips = strips > s2 ? strips : s2;
    rows += (n_tokens + 15) / 16;
  }
  if ((d + 31) / 32 <= 16)
    hipLaunchKernelGGL((moe_expert_kernel<X_SWIGLU, 4>), dim3(strips, rows), dim3(256), 0, (hipStream_t)stream, a);
  else
    hipLaunchKernelGGL((moe_expert_kernel<X_SWIGLU, 8>), dim3(strips, rows), dim3(256), 0, (hipStream_t)stream, a);
  return ohara_launch_status();
}

int ohara_moe_experts_gate_up(const uint16_t* x, int ldx, const uint16_t* wp_gate_up, int64_t expert_stride_bytes,
                              int n_experts, int hidden, int d, int k, const int32_t* offsets, const int32_t* pair_of,
                              uint16_t* act, int ld_act, void* stream) {
  return ohara_moe_experts_gate_up_shared(x, ldx, wp_gate_up, expert_stride_bytes, n_experts, hidden, d, k, offsets, pair_of,
                                          act, ld_act, nullptr, 0, 0, nullptr, 0, stream);
}

int ohara_moe_experts_down_shared(const uint16_t* act, int ld_act, const uint16_t* wp_down, int64_t expert_stride_bytes,
                                  int n_experts, int d, int hidden, int k, const int32_t* offsets, const int32_t* pair_of,
                                  const uint16_t* expert_w, uint16_t* y, int ldy, const uint16_t* wp_shared,
                                  int shared_hidden, int n_tokens, const uint16_t* act_shared, int ld_act_shared,
                                  uint16_t* y_shared, int ldy_shared, void* stream) {
  if (!act || !wp_down || !offsets || !pair_of || !expert_w || !y || hidden < 1 || d < 1 || (hidden & 7) || (ld_act & 7))
    return OHARA_EINVAL;
  ExpertArgs a{};
  a.wp = reinterpret_cast<const uint4*>(wp_down); a.expert_stride = (size_t)expert_stride_bytes / 16;
  a.x = act; a.ldx = ld_act; a.offs = offsets; a.pair_of = pair_of; a.w = expert_w; a.k = k; a.N_out = d; a.K = hidden;
  a.out = y; a.ldo = ldy; a.E = n_experts;
  int rows = n_experts, ks = (hidden + 31) / 32;
  if (wp_shared) {  // the shared expert: a row of the grid per 16 tokens
    if (!act_shared || !y_shared || n_tokens < 1 || shared_hidden < 1 || (shared_hidden & 7) || (ld_act_shared & 7))
      return OHARA_EINVAL;
    a.N_sh = n_tokens; a.wp_sh = reinterpret_cast<const uint4*>(wp_shared); a.x_sh = act_shared; a.ldx_sh = ld_act_shared;
    a.N_out_sh = d; a.K_sh = shared_hidden; a.out_sh = y_shared; a.ldo_sh = ldy_shared;
    const int ks2 = (shared_hidden + 31) / 32;
    ks = ks > ks2 ? ks : ks2;
    rows += (n_tokens + 15) / 16;
  }
  if (ks <= 16)
    hipLaunchKernelGGL((moe_expert_kernel<X_DOWN, 4>), dim3((d + 15) / 16, rows), dim3(256), 0, (hipStream_t)stream, a);
  else
    hipLaunchKernelGGL((moe_expert_kernel<X_DOWN, 8>), dim3((d + 15) / 16, rows), dim3(256), 0, (hipStream_t)stream, a);
  return ohara_launch_status();
}

int ohara_moe_experts_down(const uint16_t* act, int ld_act, const uint16_t* wp_down, int64_t expert_stride_bytes,
                           int n_experts, int d, int hidden, int k, const int32_t* offsets, const int32_t* pair_of,
                           const uint16_t* expert_w, uint16_t* y, int ldy, void* stream) {
  return ohara_moe_experts_down_shared(act, ld_act, wp_down, expert_stride_bytes, n_experts, d, hidden, k, offsets, pair_of,
                                       expert_w, y, ldy, nullptr, 0, 0, nullptr, 0, nullptr, 0, stream);
}

int ohara_moe_combine(const uint16_t* y, int ldy, const int32_t* expert_idx, const int32_t* pos_of, int n_tokens, int k,
                      const uint16_t* shared, int ld_shared, const uint16_t* resid, int ldr, uint16_t* out, int ldo, int d,
                      void* stream) {
  if (!y || !expert_idx || !pos_of || !out || n_tokens < 1 || k < 1 || k > 16 || d < 1) return OHARA_EINVAL;
  hipLaunchKernelGGL(moe_combine_kernel, dim3(n_tokens), dim3(256), 0, (hipStream_t)stream, y, ldy, expert_idx, pos_of, k,
                     shared, ld_shared, resid, ldr, out, ldo, d);
  return ohara_launch_status();
}

}  // extern "C"
