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
  // Winner j is kept by lane j; the arg-max butterfly runs on DPP moves and row swaps.
  float my_raw = 0.f;
  int my_id = 0;
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
  float wt;
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
  if (has) {
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
};

// CH: k-steps a wave has in flight at once (the host takes 4 when a wave's share of K is that short).
// Every load of a batch is issued whatever its index - clamped into the strip and the row, zeroed
// afterwards where it lies beyond the wave's share - so the batch is one run of loads without branches.
template <int EPI, int CH>
__global__ __launch_bounds__(256) void moe_expert_kernel(ExpertArgs a) {
  const int strip = blockIdx.x, e = blockIdx.y;
  const int p0 = a.offs[e], p1 = a.offs[e + 1];
  if (p0 >= p1) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m = lane & 15, g = lane >> 4;
  const int KS = (a.K + 31) >> 5;
  const int per = (KS + 3) >> 2;
  const int j0 = wave * per, j1 = min(KS, j0 + per);
  __shared__ float red[3][64][4];
  const uint4* wrow = a.wp + (size_t)e * a.expert_stride + (size_t)strip * KS * 64 + lane;
  for (int pt = p0; pt < p1; pt += 16) {  // 16-token column tiles of this expert
    const int pos = pt + m;
    const bool has = pos < p1;
    const int posc = min(pos, p1 - 1);  // a token of this expert: lanes past the end compute a column nobody stores
    const int pair = a.pair_of[posc];
    const bf16_t* xrow = a.x + (size_t)((EPI == X_SWIGLU) ? pair / a.k : posc) * a.ldx;
    float wt = 0.f;
    if (EPI == X_DOWN) wt = bf2f(a.w[pair]);  // asked for here, used in the epilogue
    f32x4 acc = (f32x4){0.f, 0.f, 0.f, 0.f};
    for (int jb = j0; jb < j1; jb += CH) {
      uint4 wv[CH], xv[CH];
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        const int j = min(jb + c, j1 - 1);
        wv[c] = ldg16_nt(wrow + (size_t)j * 64);
        xv[c] = ldg16(xrow + min(32 * j + 8 * g, a.K - 8));
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        const bool live = jb + c < j1 && 32 * (jb + c) + 8 * g < a.K;
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
          bf16_t* o = a.out + (size_t)pos * a.ldo + f;
          if (f < a.N_out) o[0] = f2bf(rbf(silu_f(y0)) * y2);
          if (f + 1 < a.N_out) o[1] = f2bf(rbf(silu_f(y1)) * y3);
        } else {
          const int r0 = strip * 16 + 4 * g;
          const float v[4] = {y0 * wt, y1 * wt, y2 * wt, y3 * wt};
          bf16_t* o = a.out + (size_t)pos * a.ldo + r0;
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (r0 + i < a.N_out) o[i] = f2bf(v[i]);
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

int ohara_moe_experts_gate_up(const uint16_t* x, int ldx, const uint16_t* wp_gate_up, int64_t expert_stride_bytes,
                              int n_experts, int hidden, int d, int k, const int32_t* offsets, const int32_t* pair_of,
                              uint16_t* act, int ld_act, void* stream) {
  if (!x || !wp_gate_up || !offsets || !pair_of || !act || hidden < 1 || d < 1 || (d & 7) || (ldx & 7)) return OHARA_EINVAL;
  ExpertArgs a{};
  a.wp = reinterpret_cast<const uint4*>(wp_gate_up); a.expert_stride = (size_t)expert_stride_bytes / 16;
  a.x = x; a.ldx = ldx; a.offs = offsets; a.pair_of = pair_of; a.k = k; a.N_out = hidden; a.K = d;
  a.out = act; a.ldo = ld_act;
  const int strips = 2 * ((hidden + 7) / 8 * 8) / 16;
  if ((d + 31) / 32 <= 16)
    hipLaunchKernelGGL((moe_expert_kernel<X_SWIGLU, 4>), dim3(strips, n_experts), dim3(256), 0, (hipStream_t)stream, a);
  else
    hipLaunchKernelGGL((moe_expert_kernel<X_SWIGLU, 8>), dim3(strips, n_experts), dim3(256), 0, (hipStream_t)stream, a);
  return ohara_launch_status();
}

int ohara_moe_experts_down(const uint16_t* act, int ld_act, const uint16_t* wp_down, int64_t expert_stride_bytes,
                           int n_experts, int d, int hidden, int k, const int32_t* offsets, const int32_t* pair_of,
                           const uint16_t* expert_w, uint16_t* y, int ldy, void* stream) {
  if (!act || !wp_down || !offsets || !pair_of || !expert_w || !y || hidden < 1 || d < 1 || (hidden & 7) || (ld_act & 7))
    return OHARA_EINVAL;
  ExpertArgs a{};
  a.wp = reinterpret_cast<const uint4*>(wp_down); a.expert_stride = (size_t)expert_stride_bytes / 16;
  a.x = act; a.ldx = ld_act; a.offs = offsets; a.pair_of = pair_of; a.w = expert_w; a.k = k; a.N_out = d; a.K = hidden;
  a.out = y; a.ldo = ldy;
  if ((hidden + 31) / 32 <= 16)
    hipLaunchKernelGGL((moe_expert_kernel<X_DOWN, 4>), dim3((d + 15) / 16, n_experts), dim3(256), 0, (hipStream_t)stream, a);
  else
    hipLaunchKernelGGL((moe_expert_kernel<X_DOWN, 8>), dim3((d + 15) / 16, n_experts), dim3(256), 0, (hipStream_t)stream, a);
  return ohara_launch_status();
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
