// Fused temperature / top-k / top-p sampler: one workgroup per row of logits.
//
// Follows sample_next_token (ohara/chat_engine.py:51-82) and Inference.sampler
// (ohara/inference.py:37-65):
//   x = float(logits) / T ; ids >= valid_vocab are -inf          (:61,65; :398-399)
//   top-k: thr = k-th largest x ; x < thr -> -inf (ties at thr survive)   (:66-69)
//   p = softmax(x)                                                        (:71)
//   0 < top_p < 1: sort p descending, cum = cumsum, drop where cum - p > top_p,
//                  renormalise, draw from the sorted distribution         (:72-81)
//   else: draw from p in vocabulary order                                 (:82)
// torch.multinomial is replaced by inverse-CDF sampling with a caller-supplied uniform
// u in [0,1) per row; equal probabilities are ordered lowest id first (torch.sort leaves
// that order open).  Every reduction runs in a fixed order, so the result is a pure
// function of (logits, parameters, u).
//
// A thread owns EPT consecutive vocabulary entries in registers; the 1024 threads cover up to
// 1024*EPT ids.  Three routes from there:
//   * top-p alone on bf16 rows (the reference's chat default, chat_engine.py:35-37): every id at or
//     above the 256-th largest per-thread maximum is a candidate; if the candidates' share of the
//     whole-row softmax exceeds top_p they are sorted and scanned like the survivors of a small
//     top-k below, otherwise the third route runs;
//   * top-k <= 1024: the survivors (everything at or above the k-th largest; a lower bound of it
//     comes from the per-thread maxima) are compacted into LDS, sorted once (bitonic, descending,
//     ties lowest id first), soft-maxed and scanned sequentially in fp32 by one thread - the
//     order the reference's cumsum walks;
//   * otherwise the nucleus is found without sorting: the smallest probability that is still
//     kept, and then the probability the draw lands on, by bisection over the probability bits
//     with block-wide mass sums in a fixed order (cost independent of how many tokens are kept).
#include <mutex>

#include "common.h"

namespace {

constexpr int NT = 1024;
constexpr int NW = NT / 64;  // waves per workgroup
constexpr int CAP = 1024;  // candidates sorted per round

struct SampleArgs {
  const void* logits;
  int ldl, V, valid;
  float temperature, top_p;
  int top_k;
  const float* u;
  int u_step_stride;     // with step_state: the draw of row b is u[step * u_step_stride + b]
  int64_t* out;
  int64_t* history;      // optional (hist_cap, B)
  int32_t* step_state;   // optional {pos, step, done, pad}
  int hist_cap, B;
};

__device__ __forceinline__ uint32_t fkey(float f) {  // order-preserving: larger float -> larger key
  const uint32_t b = __float_as_uint(f);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

struct Smem {
  int hist[256];
  int hist2[3][256];  // further counting tables of select16_block
  float wred[16];
  int wredi[16];
  uint32_t skey[CAP];
  int sid[CAP];
  int misc[8];
  float fmisc[8];
};

__device__ __forceinline__ float block_max(float v, Smem& s) {
  v = wave_max(v);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) s.wred[w] = v;
  __syncthreads();
  float r = s.wred[0];
#pragma unroll
  for (int i = 1; i < NW; ++i) r = fmaxf(r, s.wred[i]);
  return r;
}

// Sum in a fixed order: butterfly inside each wave, then the wave sums left to right.
__device__ __forceinline__ float block_sum(float v, Smem& s) {
  v = wave_sum(v);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) s.wred[w] = v;
  __syncthreads();
  float r = s.wred[0];
#pragma unroll
  for (int i = 1; i < NW; ++i) r += s.wred[i];
  return r;
}

__device__ __forceinline__ int block_sum_i(int v, Smem& s) {
  v = lanes_sum<32, 1>(v);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) s.wredi[w] = v;
  __syncthreads();
  int r = 0;
#pragma unroll
  for (int i = 0; i < NW; ++i) r += s.wredi[i];
  return r;
}

// Exclusive prefix sum of one int per thread, in thread order.  Returns the total.
// Wave-level DPP scan, then the wave totals.
__device__ __forceinline__ int block_excl_scan_i(int v, int& excl, Smem& s) {
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int incl = wave_incl_scan_i(v);
  __syncthreads();
  if (lane == 63) s.wredi[w] = incl;
  __syncthreads();
  int before = 0, total = 0;
#pragma unroll
  for (int i = 0; i < NW; ++i) {
    const int t = s.wredi[i];
    if (i < w) before += t;
    total += t;
  }
  excl = before + incl - v;
  return total;
}

// Prefix sums of one float per thread, in thread order, in a fixed association (shuffle scan
// inside each wave, then the wave totals left to right): thread t gets lo = sum over threads
// before it and hi = lo of thread t + 1 (bit-identical), so the intervals [lo, hi) tile
// [0, total) without gaps.  Returns the total.
__device__ __forceinline__ float block_scan_f(float v, float& lo, float& hi, Smem& s) {
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  float incl = v;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const float t = __shfl_up(incl, o, WAVE);
    if (lane >= o) incl += t;
  }
  const float prev = __shfl_up(incl, 1, WAVE);
  __syncthreads();
  if (lane == 63) s.wred[w] = incl;
  __syncthreads();
  float before = 0.f, total = 0.f;
#pragma unroll
  for (int i = 0; i < NW; ++i) {
    if (i == w) before = total;
    total += s.wred[i];
  }
  lo = lane == 0 ? before : before + prev;
  hi = lane == 63 ? before + s.wred[w] : before + incl;
  return total;
}

// The `want`-th largest key (1-based) among the keys for which live(i) holds; returns the
// key and the number of live keys strictly greater than it.
// Keys use the low TOP + 8 bits (TOP = 24: 32-bit keys, TOP = 8: 16-bit keys in two passes).
template <int EPT, int TOP = 24, typename LiveFn, typename KeyFn>
__device__ __forceinline__ uint32_t radix_select(int want, int& n_greater, Smem& s, LiveFn live, KeyFn key) {
  uint32_t prefix = 0, mask = 0;
  int above = 0;
  for (int shift = TOP; shift >= 0; shift -= 8) {
    __syncthreads();
    if (threadIdx.x < 256) s.hist[threadIdx.x] = 0;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < EPT; ++i) {
      if (live(i)) {
        const uint32_t k = key(i);
        if ((k & mask) == prefix) atomicAdd(&s.hist[(k >> shift) & 255], 1);
      }
    }
    __syncthreads();
    // the digit whose bin holds the want-th largest: suffix sums of the 256 bins by four waves
    {
      const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
      int h = 0, incl = 0;
      if (threadIdx.x < 256) {
        h = s.hist[threadIdx.x];
        incl = h;  // inclusive sum over bins >= mine within the wave
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
          const int t = __shfl_down(incl, o, WAVE);
          if (lane + o < 64) incl += t;
        }
        if (lane == 0) s.wredi[w] = incl;
      }
      __syncthreads();
      if (threadIdx.x < 256) {
        for (int i = w + 1; i < 4; ++i) incl += s.wredi[i];
        const int gt = above + incl - h;  // elements in bins above mine (and in earlier digits' higher bins)
        if (gt < want && (threadIdx.x == 0 || want <= gt + h)) {
          s.misc[0] = threadIdx.x;
          s.misc[1] = gt;
        }
      }
    }
    __syncthreads();
    const int d = s.misc[0];
    above = s.misc[1];
    prefix |= (uint32_t)d << shift;
    mask |= 255u << shift;
  }
  n_greater = above;
  return prefix;
}

// The same selection for want <= 1024, without a histogram pass over every element (tens of
// thousands of LDS atomics on the handful of bins that share the leading key bits): the want-th
// largest of the 1024 per-thread maxima is a lower bound of the answer (at least `want` elements
// are >= it), so only the elements at or above that bound - usually a few times `want` - take part
// in the exact radix select.
template <int EPT, typename LiveFn, typename KeyFn>
__device__ __forceinline__ uint32_t select_small(int want, int& n_greater, Smem& s, LiveFn live, KeyFn key) {
  uint32_t tmax = 0;  // keys of live elements are > 0
#pragma unroll
  for (int i = 0; i < EPT; ++i)
    if (live(i)) tmax = max(tmax, key(i));
  const int have = block_sum_i(tmax > 0 ? 1 : 0, s);
  uint32_t bound = 0;
  if (have >= want) {
    int dummy;
    bound = radix_select<1>(want, dummy, s, [&](int) { return tmax > 0; }, [&](int) { return tmax; });
  }
  return radix_select<EPT>(want, n_greater, s, [&](int i) { return live(i) && key(i) >= bound; }, key);
}

// The `want`-th largest (1-based) of one 16-bit key per thread (0: the thread holds none), two counting
// passes of 8 bits like radix_select<1, 8>, with fewer stops: the two tables `t1`, `t2` were cleared by
// the caller (select16_clear, behind a workgroup barrier), and one wave finds the digit of a pass (a
// lane adds up four bins, highest first, a DPP scan across the lanes), so that a pass is two
// workgroup barriers.  Fewer than `want` keys: digit 0, as there.
__device__ __forceinline__ void select16_clear(Smem& s) {  // all four tables; a workgroup barrier must follow
  const int tid = threadIdx.x;
  if (tid < 256) s.hist[tid] = 0;
  else s.hist2[(tid >> 8) - 1][tid & 255] = 0;
}
__device__ __forceinline__ uint32_t select16_block(int want, uint32_t key, Smem& s, int* t1, int* t2) {
  const int tid = threadIdx.x, lane = tid & 63;
  auto find = [&](const int* h, int want_) {  // by wave 0: the bin that holds the want_-th largest, and the count above it
    const int b0 = 255 - 4 * lane;            // lane l owns bins 255 - 4l .. 252 - 4l
    const int c0 = h[b0], c1 = h[b0 - 1], c2 = h[b0 - 2], c3 = h[b0 - 3];
    const int tot = c0 + c1 + c2 + c3;
    const int incl = wave_incl_scan_i(tot);
    const int excl = incl - tot;
    if (excl < want_ && want_ <= incl) {
      int above = excl, d = b0;
      if (want_ > above + c0) {
        above += c0;
        d = b0 - 1;
        if (want_ > above + c1) {
          above += c1;
          d = b0 - 2;
          if (want_ > above + c2) {
            above += c2;
            d = b0 - 3;
          }
        }
      }
      s.misc[0] = d;
      s.misc[1] = above;
    } else if (lane == 63 && want_ > incl) {
      s.misc[0] = 0;
      s.misc[1] = incl - c3;
    }
  };
  if (key) atomicAdd(&t1[key >> 8], 1);
  __syncthreads();
  if (tid < 64) find(t1, want);
  __syncthreads();
  const uint32_t d1 = (uint32_t)s.misc[0];
  const int above = s.misc[1];
  if (key && (key >> 8) == d1) atomicAdd(&t2[key & 255u], 1);
  __syncthreads();
  if (tid < 64) find(t2, want - above);
  __syncthreads();
  return (d1 << 8) | (uint32_t)s.misc[0];
}

template <typename T>
__device__ __forceinline__ float load_logit(const void* base, size_t i);
template <>
__device__ __forceinline__ float load_logit<bf16_t>(const void* base, size_t i) {
  return bf2f(reinterpret_cast<const bf16_t*>(base)[i]);
}
template <>
__device__ __forceinline__ float load_logit<float>(const void* base, size_t i) {
  return reinterpret_cast<const float*>(base)[i];
}

__device__ __forceinline__ float unfkey(uint32_t k) {  // inverse of fkey
  return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

// Bitonic sort of the first n2 (power of two) entries of (skey, sid): descending by key,
// ascending by id among equal keys.
__device__ __forceinline__ void sort_candidates(Smem& s, int n2) {
  const int tid = threadIdx.x;
  for (int k2 = 2; k2 <= n2; k2 <<= 1) {
    for (int j = k2 >> 1; j > 0; j >>= 1) {
      for (int t = tid; t < n2; t += NT) {
        const int ixj = t ^ j;
        if (ixj > t) {
          const uint32_t ka = s.skey[t], kb = s.skey[ixj];
          const int ia = s.sid[t], ib = s.sid[ixj];
          const bool a_first = ka > kb || (ka == kb && ia < ib);  // a precedes b in the target order
          const bool up = (t & k2) == 0;
          if (up ? !a_first : a_first) {
            s.skey[t] = kb; s.skey[ixj] = ka;
            s.sid[t] = ib; s.sid[ixj] = ia;
          }
        }
      }
      __syncthreads();
    }
  }
}

// The same by ascending id only (vocabulary order), carrying the keys.
__device__ __forceinline__ void sort_by_id(Smem& s, int n2) {
  const int tid = threadIdx.x;
  for (int k2 = 2; k2 <= n2; k2 <<= 1) {
    for (int j = k2 >> 1; j > 0; j >>= 1) {
      for (int t = tid; t < n2; t += NT) {
        const int ixj = t ^ j;
        if (ixj > t) {
          const int ia = s.sid[t], ib = s.sid[ixj];
          const bool up = (t & k2) == 0;
          if (up ? ia > ib : ia < ib) {
            const uint32_t ka = s.skey[t], kb = s.skey[ixj];
            s.skey[t] = kb; s.skey[ixj] = ka;
            s.sid[t] = ib; s.sid[ixj] = ia;
          }
        }
      }
      __syncthreads();
    }
  }
}

template <typename T, int EPT>
__device__ __forceinline__ void load_row_scalar(const SampleArgs& a, int b, int base, int nvalid, float temp, float* x) {
#pragma unroll
  for (int i = 0; i < EPT; ++i) {
    const int id = base + i;
    x[i] = id < nvalid ? load_logit<T>(a.logits, (size_t)b * a.ldl + id) / temp : -INFINITY;
  }
}

// The draw from a block of n_c candidates in (skey = fkey(x), sid = id) that holds at least the k
// largest valid ids of the row with all ties of the k-th: sort (descending key, ascending id among equal
// keys), cut at the k-th key, softmax over the kept entries, nucleus or vocabulary-order inverse CDF
// (chat_engine.py:66-82).  Every thread of the workgroup calls; returns the token in every thread.
__device__ __forceinline__ int draw_from_block(const SampleArgs& a, Smem& s, int n_c, int k, float u) {
  const int tid = threadIdx.x;
  int n2 = 64;
  while (n2 < n_c) n2 <<= 1;
  __syncthreads();
  for (int i = n_c + tid; i < n2; i += NT) {
    s.skey[i] = 0;  // padding sorts last
    s.sid[i] = 0x7fffffff;
  }
  __syncthreads();
  sort_candidates(s, n2);
  // kept: everything >= the k-th largest key (ties at the threshold survive, chat_engine.py:66-69)
  const uint32_t tk = s.skey[min(k, n_c) - 1];
  int n_kept = block_sum_i((tid < n_c && s.skey[tid] >= tk) ? 1 : 0, s);
  // softmax over the kept entries (the rest of the vocabulary is -inf): entry 0 is the maximum
  const float m0 = unfkey(s.skey[0]);
  const float e = tid < n_kept ? expf(unfkey(s.skey[tid]) - m0) : 0.f;
  const float Z = block_sum(e, s);
  __syncthreads();
  if (tid < n_kept) s.skey[tid] = __float_as_uint(e / Z);  // probabilities, still in sorted order
  __syncthreads();
  const bool nucleus = a.top_p > 0.f && a.top_p < 1.f;
  if (!nucleus) {  // vocabulary-order draw (chat_engine.py:82): order the kept entries by id
    int m2 = 64;
    while (m2 < n_kept) m2 <<= 1;
    for (int i = n_kept + tid; i < m2; i += NT) {
      s.skey[i] = 0;
      s.sid[i] = 0x7fffffff;
    }
    __syncthreads();
    sort_by_id(s, m2);
  }
  if (tid == 0) {
    // sequential fp32 sums in the order the reference's cumsum walks
    int tok = -1, last = -1;
    if (nucleus) {
      float kept = 0.f, run = 0.f;
      int n_in = 0;
      for (int j = 0; j < n_kept; ++j) {  // kept prefix: mass before the token <= top_p
        if (run > a.top_p) break;
        const float p = __uint_as_float(s.skey[j]);
        kept += p;
        run += p;
        ++n_in;
      }
      const float target = u * kept;
      run = 0.f;
      for (int j = 0; j < n_in; ++j) {
        run += __uint_as_float(s.skey[j]);
        last = s.sid[j];
        if (run > target) {
          tok = s.sid[j];
          break;
        }
      }
    } else {
      float total = 0.f;
      for (int j = 0; j < n_kept; ++j) total += __uint_as_float(s.skey[j]);
      const float target = u * total;
      float run = 0.f;
      for (int j = 0; j < n_kept; ++j) {
        const float p = __uint_as_float(s.skey[j]);
        run += p;
        if (p > 0.f) last = s.sid[j];
        if (p > 0.f && run > target) {
          tok = s.sid[j];
          break;
        }
      }
    }
    s.misc[3] = tok >= 0 ? tok : max(last, 0);  // rounding pushed the target past the end: last kept id
  }
  __syncthreads();
  return s.misc[3];
}

// ---- the same draw by ONE wave -------------------------------------------------------------------
// For at most 128 candidates the whole draw fits one wave's registers (lane l holds entries l and
// l + 64): the bitonic sorts exchange through DPP moves and row swaps instead of LDS and a
// workgroup barrier per stage (28 stages for 128 entries, 16 waves waiting at each), counts are
// ballots, and the sequential sums of the reference's order read the probabilities lane by lane
// with v_readlane.  Every comparison, sum and its order are those of draw_from_block: the sorts
// use the same strict total orders, Z adds the butterfly sum of entries 0..63 and that of entries
// 64..127 exactly as block_sum adds its first two wave sums (the other fourteen are zero).
template <int J>
__device__ __forceinline__ uint32_t wave_partner(uint32_t v, int lane) {  // v of lane ^ J
  if constexpr (J < 16) {
    return lane_xor_u32<J>(v);
  } else {
    const u32x2 r = J == 16 ? __builtin_amdgcn_permlane16_swap(v, v, false, false)
                            : __builtin_amdgcn_permlane32_swap(v, v, false, false);
    return (lane & J) ? r[0] : r[1];
  }
}
// one compare-exchange stage of the bitonic network on entries t = lane (k0, i0) and lane + 64 (k1, i1);
// BY_ID: ascending ids; otherwise descending keys, ties by ascending id
template <int J, bool BY_ID>
__device__ __forceinline__ void wave_sort_stage(uint32_t& k0, int& i0, uint32_t& k1, int& i1, int k2, int lane) {
  auto first = [](uint32_t ka, int ia, uint32_t kb, int ib) {  // a precedes b in the target order
    return BY_ID ? ia < ib : (ka > kb || (ka == kb && ia < ib));
  };
  if constexpr (J == 64) {
    const bool up = (lane & k2) == 0;  // k2 == 128 here: always up
    const bool a_first = first(k0, i0, k1, i1);
    if (up ? !a_first : a_first) {
      const uint32_t tk = k0; k0 = k1; k1 = tk;
      const int ti = i0; i0 = i1; i1 = ti;
    }
  } else {
    const bool lower = (lane & J) == 0;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      uint32_t& km = h ? k1 : k0;
      int& im = h ? i1 : i0;
      const uint32_t kp = wave_partner<J>(km, lane);
      const int ip = (int)wave_partner<J>((uint32_t)im, lane);
      const int t = lane + 64 * h;
      const bool up = (t & k2) == 0;
      // the pair in position order (a = lower index): keep as is when a already precedes b (up) / follows b (down)
      const bool a_first = lower ? first(km, im, kp, ip) : first(kp, ip, km, im);
      const bool swap = up ? !a_first : a_first;
      if (swap) { km = kp; im = ip; }
    }
  }
}
template <bool BY_ID>
__device__ __forceinline__ void wave_sort128(uint32_t& k0, int& i0, uint32_t& k1, int& i1, int lane) {
#define OHARA_WS(J, K2) wave_sort_stage<J, BY_ID>(k0, i0, k1, i1, K2, lane)
  OHARA_WS(1, 2);
  OHARA_WS(2, 4); OHARA_WS(1, 4);
  OHARA_WS(4, 8); OHARA_WS(2, 8); OHARA_WS(1, 8);
  OHARA_WS(8, 16); OHARA_WS(4, 16); OHARA_WS(2, 16); OHARA_WS(1, 16);
  OHARA_WS(16, 32); OHARA_WS(8, 32); OHARA_WS(4, 32); OHARA_WS(2, 32); OHARA_WS(1, 32);
  OHARA_WS(32, 64); OHARA_WS(16, 64); OHARA_WS(8, 64); OHARA_WS(4, 64); OHARA_WS(2, 64); OHARA_WS(1, 64);
  OHARA_WS(64, 128); OHARA_WS(32, 128); OHARA_WS(16, 128); OHARA_WS(8, 128); OHARA_WS(4, 128); OHARA_WS(2, 128);
  OHARA_WS(1, 128);
#undef OHARA_WS
}
// n_c <= 128 candidates in (s.skey, s.sid); every thread of the workgroup calls, wave 0 draws
__device__ __forceinline__ int draw_from_wave(const SampleArgs& a, Smem& s, int n_c, int k, float u) {
  const int tid = threadIdx.x;
  __syncthreads();  // the candidates are in place
  if (tid < 64) {
    const int lane = tid;
    uint32_t k0 = lane < n_c ? s.skey[lane] : 0u, k1 = lane + 64 < n_c ? s.skey[lane + 64] : 0u;  // padding sorts last
    int i0 = lane < n_c ? s.sid[lane] : 0x7fffffff, i1 = lane + 64 < n_c ? s.sid[lane + 64] : 0x7fffffff;
    wave_sort128<false>(k0, i0, k1, i1, lane);
    const int kth = min(k, n_c) - 1;
    const uint32_t tk = kth < 64 ? (uint32_t)__builtin_amdgcn_readlane((int)k0, kth) : (uint32_t)__builtin_amdgcn_readlane((int)k1, kth - 64);
    const int n_kept = __popcll(__ballot(lane < n_c && k0 >= tk)) + __popcll(__ballot(lane + 64 < n_c && k1 >= tk));
    const float m0 = unfkey((uint32_t)__builtin_amdgcn_readlane((int)k0, 0));
    const float e0 = lane < n_kept ? expf(unfkey(k0) - m0) : 0.f;
    const float e1 = lane + 64 < n_kept ? expf(unfkey(k1) - m0) : 0.f;
    const float Z = wave_sum(e0) + wave_sum(e1);
    uint32_t p0 = lane < n_kept ? __float_as_uint(e0 / Z) : k0;       // probabilities, still in sorted order
    uint32_t p1 = lane + 64 < n_kept ? __float_as_uint(e1 / Z) : k1;  // (entries past n_kept are never read)
    const bool nucleus = a.top_p > 0.f && a.top_p < 1.f;
    if (!nucleus) {  // vocabulary-order draw: the kept entries by id, the rest as padding
      if (lane >= n_kept) { p0 = 0u; i0 = 0x7fffffff; }
      if (lane + 64 >= n_kept) { p1 = 0u; i1 = 0x7fffffff; }
      wave_sort128<true>(p0, i0, p1, i1, lane);
    }
    auto prob = [&](int j) {
      return __uint_as_float(j < 64 ? (uint32_t)__builtin_amdgcn_readlane((int)p0, j) : (uint32_t)__builtin_amdgcn_readlane((int)p1, j - 64));
    };
    auto ident = [&](int j) { return j < 64 ? __builtin_amdgcn_readlane(i0, j) : __builtin_amdgcn_readlane(i1, j - 64); };
    // sequential fp32 sums in the order the reference's cumsum walks (all lanes run them: the loops are uniform)
    int tok = -1, last = -1;
    if (nucleus) {
      float kept = 0.f, run = 0.f;
      int n_in = 0;
      for (int j = 0; j < n_kept; ++j) {  // kept prefix: mass before the token <= top_p
        if (run > a.top_p) break;
        const float p = prob(j);
        kept += p;
        run += p;
        ++n_in;
      }
      const float target = u * kept;
      run = 0.f;
      for (int j = 0; j < n_in; ++j) {
        run += prob(j);
        last = ident(j);
        if (run > target) {
          tok = last;
          break;
        }
      }
    } else {
      float total = 0.f;
      for (int j = 0; j < n_kept; ++j) total += prob(j);
      const float target = u * total;
      float run = 0.f;
      for (int j = 0; j < n_kept; ++j) {
        const float p = prob(j);
        run += p;
        if (p > 0.f) last = ident(j);
        if (p > 0.f && run > target) {
          tok = ident(j);
          break;
        }
      }
    }
    if (lane == 0) s.misc[3] = tok >= 0 ? tok : max(last, 0);  // rounding pushed the target past the end: last kept id
  }
  __syncthreads();
  return s.misc[3];
}

// ---- the draw by one wave from packed candidates (bf16 rows, ids below 65536) -----------------------
// A candidate is ONE sortable word: the order-preserving 16-bit key of its bf16 logit above, 0xffff - id
// below, so that descending words are descending logits with ties in ascending id order, and a stage
// of the bitonic network is an exchange, a max and a min.  For the vocabulary-order draw the kept
// entries are sorted again as ~(id << 8 | position) and fetch their probability from that position.
// The sequential fp32 sums of the reference's cumsum are one chain: run_j = run_(j-1) + p_j
// for every kept entry, lane j keeps run_(j-1) and run_j; the prefix
// under top_p, the total and the first entry past the target are then ballots.  The values, their
// order and every sum are those of draw_from_block.
template <int J>
__device__ __forceinline__ uint32_t packed_stage(uint32_t v, bool take_max) {
  uint32_t mx, mn;
  if constexpr (J < 16) {
    const uint32_t o = lane_xor_u32<J>(v);
    mx = max(v, o);
    mn = min(v, o);
  } else {
    const u32x2 r = J == 16 ? __builtin_amdgcn_permlane16_swap(v, v, false, false)
                            : __builtin_amdgcn_permlane32_swap(v, v, false, false);
    mx = max(r[0], r[1]);
    mn = min(r[0], r[1]);
  }
  return take_max ? mx : mn;
}
// descending sort of 64 (TWO == false: w0 only) or 128 words (entry t = lane: w0, t = lane + 64: w1)
template <bool TWO>
__device__ __forceinline__ void packed_sort(uint32_t& w0, uint32_t& w1, int lane) {
#define OHARA_PS(J, K2)                                                                       \
  {                                                                                           \
    const bool lower = (lane & J) == 0;                                                       \
    w0 = packed_stage<J>(w0, lower == ((lane & K2) == 0));                                    \
    if (TWO) w1 = packed_stage<J>(w1, lower == (((lane + 64) & K2) == 0));                    \
  }
  OHARA_PS(1, 2);
  OHARA_PS(2, 4); OHARA_PS(1, 4);
  OHARA_PS(4, 8); OHARA_PS(2, 8); OHARA_PS(1, 8);
  OHARA_PS(8, 16); OHARA_PS(4, 16); OHARA_PS(2, 16); OHARA_PS(1, 16);
  OHARA_PS(16, 32); OHARA_PS(8, 32); OHARA_PS(4, 32); OHARA_PS(2, 32); OHARA_PS(1, 32);
  OHARA_PS(32, 64); OHARA_PS(16, 64); OHARA_PS(8, 64); OHARA_PS(4, 64); OHARA_PS(2, 64); OHARA_PS(1, 64);
  if (TWO) {
    const uint32_t mx = max(w0, w1), mn = min(w0, w1);  // entries t and t + 64, block of 128: descending
    w0 = mx;
    w1 = mn;
    OHARA_PS(32, 128); OHARA_PS(16, 128); OHARA_PS(8, 128); OHARA_PS(4, 128); OHARA_PS(2, 128); OHARA_PS(1, 128);
  }
#undef OHARA_PS
}
// run_(j-1) and run_j of the sequential sum over the first n entries of q (uniform chain, lane j keeps
// its two values).  Eight steps per trip: a trip of one step is half loop overhead, and 64 unrolled
// steps are 40 cache lines of straight-line code that runs once per launch from a cold instruction cache.
__device__ __forceinline__ float seq_sums(uint32_t q, float run, int n, int lane, float& before, float& after) {
  for (int j0 = 0; j0 < n; j0 += 8) {  // entries past n hold +0: the steps of the last trip that overshoot change nothing
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int j = j0 + i;
      const float prev = run;
      run += __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)q, j));
      before = lane == j ? prev : before;
      after = lane == j ? run : after;
    }
  }
  return run;
}
__device__ __forceinline__ float logit_of_key16(uint32_t key, float temperature) {
  const uint32_t bits = (key & 0x8000u) ? (key ^ 0x8000u) : (~key & 0xffffu);
  return __uint_as_float(bits << 16) / temperature;
}
// n_c <= 128 packed candidates in s.skey[0 .. n_c); every thread of the workgroup calls, wave 0 draws
__device__ __forceinline__ int draw_from_wave_packed(const SampleArgs& a, Smem& s, int n_c, int k, float u) {
  const int tid = threadIdx.x;
  __syncthreads();  // the candidates are in place
  if (tid < 64) {
    const int lane = tid;
    const bool two = n_c > 64;
    uint32_t w0 = lane < n_c ? s.skey[lane] : 0u, w1 = lane + 64 < n_c ? s.skey[lane + 64] : 0u;  // padding sorts last
    if (two) packed_sort<true>(w0, w1, lane);
    else packed_sort<false>(w0, w1, lane);
    const int kth = min(k, n_c) - 1;
    const uint32_t tk = (kth < 64 ? (uint32_t)__builtin_amdgcn_readlane((int)w0, kth)
                                  : (uint32_t)__builtin_amdgcn_readlane((int)w1, kth - 64)) >> 16;
    const int n_kept = __popcll(__ballot(lane < n_c && (w0 >> 16) >= tk)) +
                       __popcll(__ballot(lane + 64 < n_c && (w1 >> 16) >= tk));
    const float m0 = logit_of_key16((uint32_t)__builtin_amdgcn_readlane((int)w0, 0) >> 16, a.temperature);
    const float e0 = lane < n_kept ? expf(logit_of_key16(w0 >> 16, a.temperature) - m0) : 0.f;
    float e1 = 0.f, z1 = 0.f;  // entries 64 .. 127: none in the usual case, and their sum is the +0 it would be
    if (n_kept > 64) {
      e1 = lane + 64 < n_kept ? expf(logit_of_key16(w1 >> 16, a.temperature) - m0) : 0.f;
      z1 = wave_sum(e1);
    }
    const float Z = wave_sum(e0) + z1;
    uint32_t p0 = lane < n_kept ? __float_as_uint(e0 / Z) : 0u;  // probabilities in sorted order, +0 past the kept ones
    uint32_t p1 = lane + 64 < n_kept ? __float_as_uint(e1 / Z) : 0u;
    int i0 = 0xffff - (int)(w0 & 0xffffu), i1 = 0xffff - (int)(w1 & 0xffffu);
    const bool nucleus = a.top_p > 0.f && a.top_p < 1.f;
    if (!nucleus) {  // vocabulary-order draw: the kept entries by ascending id
      uint32_t c0 = lane < n_kept ? ~(((uint32_t)i0 << 8) | (uint32_t)lane) : 0u;
      uint32_t c1 = lane + 64 < n_kept ? ~(((uint32_t)i1 << 8) | (uint32_t)(lane + 64)) : 0u;
      if (two) packed_sort<true>(c0, c1, lane);
      else packed_sort<false>(c0, c1, lane);
      const uint32_t s0 = ~c0, s1 = ~c1;
      const int f0 = (int)(s0 & 0xffu), f1 = (int)(s1 & 0xffu);  // where the entry stood in logit order
      const uint32_t a0 = __shfl(p0, f0 & 63, WAVE), b0 = __shfl(p1, f0 & 63, WAVE);
      const uint32_t a1 = __shfl(p0, f1 & 63, WAVE), b1 = __shfl(p1, f1 & 63, WAVE);
      p0 = lane < n_kept ? (f0 < 64 ? a0 : b0) : 0u;
      p1 = lane + 64 < n_kept ? (f1 < 64 ? a1 : b1) : 0u;
      i0 = (int)(s0 >> 8);
      i1 = (int)(s1 >> 8);
    }
    float bf0 = 0.f, af0 = 0.f, bf1 = 0.f, af1 = 0.f;
    float run = seq_sums(p0, 0.f, min(n_kept, 64), lane, bf0, af0);
    if (n_kept > 64) run = seq_sums(p1, run, n_kept - 64, lane, bf1, af1);
    auto after_at = [&](int j) { return j < 64 ? __builtin_amdgcn_readlane(__float_as_int(af0), j) : __builtin_amdgcn_readlane(__float_as_int(af1), j - 64); };
    auto ident = [&](int j) { return j < 64 ? __builtin_amdgcn_readlane(i0, j) : __builtin_amdgcn_readlane(i1, j - 64); };
    int tok = -1, last = -1;
    unsigned long long h0, h1;
    if (nucleus) {
      // the kept prefix: entries whose mass before them is <= top_p (the sums never decrease)
      const unsigned long long in0 = __ballot(lane < n_kept && !(bf0 > a.top_p));
      const unsigned long long in1 = __ballot(lane + 64 < n_kept && !(bf1 > a.top_p));
      const int n_in = __popcll(in0) + __popcll(in1);
      if (n_in > 0) {
        const float target = u * __int_as_float(after_at(n_in - 1));
        last = ident(n_in - 1);
        h0 = __ballot(lane < n_in && af0 > target);
        h1 = __ballot(lane + 64 < n_in && af1 > target);
      } else {
        h0 = h1 = 0;
      }
    } else {
      const float target = u * run;
      const unsigned long long pos0 = __ballot(lane < n_kept && __uint_as_float(p0) > 0.f);
      const unsigned long long pos1 = __ballot(lane + 64 < n_kept && __uint_as_float(p1) > 0.f);
      if (pos1) last = ident(64 + 63 - __clzll(pos1));
      else if (pos0) last = ident(63 - __clzll(pos0));
      h0 = __ballot(lane < n_kept && __uint_as_float(p0) > 0.f && af0 > target);
      h1 = __ballot(lane + 64 < n_kept && __uint_as_float(p1) > 0.f && af1 > target);
    }
    if (h0) tok = ident(__ffsll(h0) - 1);
    else if (h1) tok = ident(64 + __ffsll(h1) - 1);
    if (lane == 0) s.misc[3] = tok >= 0 ? tok : max(last, 0);  // rounding pushed the target past the end: last kept id
  }
  __syncthreads();
  return s.misc[3];
}

// The selected id of a row goes out, with the loop bookkeeping when the caller keeps a step state.
__device__ __forceinline__ void finish_row(const SampleArgs& a, int b, int token) {
  a.out[b] = token;
  if (a.step_state) {
    const int step = a.step_state[1];
    if (a.history && step < a.hist_cap) a.history[(size_t)step * a.B + b] = token;
    // only the counter is shared between workgroups: no fence, the ids are read by later kernels
    const int old = __hip_atomic_fetch_add(&a.step_state[2], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (old == a.B - 1) {
      a.step_state[2] = 0;
      a.step_state[0] += 1;
      a.step_state[1] = step + 1;
    }
  }
}

// One workgroup on the whole row b: returns the token in every thread.
template <typename T, int EPT>
__device__ __forceinline__ int sample_row(const SampleArgs& a, int b, Smem& s) {
  const int tid = threadIdx.x;
  const int V = a.V, nvalid = min(a.valid, V);
  const int base = tid * EPT;
  float x[EPT];
  const float temp = a.temperature;
  const float u = a.u[(a.step_state && a.u_step_stride > 0 ? (size_t)a.step_state[1] * a.u_step_stride : 0) + b];
  const bool packed_row = sizeof(T) == 2 && EPT % 8 == 0 && (a.ldl & 7) == 0 &&
                          ((reinterpret_cast<uintptr_t>(a.logits) & 15) == 0);
  // x = logits / temperature for this thread's ids (ids past the valid vocabulary: -inf)
  auto load_x = [&]() {
    if (packed_row) {
      // bf16 rows: eight values per 16-byte load
      const bf16_t* row = reinterpret_cast<const bf16_t*>(a.logits) + (size_t)b * a.ldl + base;
#pragma unroll
      for (int c = 0; c < EPT / 8; ++c) {
        const uint4 v = base + 8 * c < V ? ldg16(row + 8 * c) : make_uint4(0, 0, 0, 0);
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int id = base + 8 * c + 2 * j;
          x[8 * c + 2 * j] = id < nvalid ? lo_bf(w[j]) / temp : -INFINITY;
          x[8 * c + 2 * j + 1] = id + 1 < nvalid ? hi_bf(w[j]) / temp : -INFINITY;
        }
      }
    } else {
      load_row_scalar<T, EPT>(a, b, base, nvalid, temp, x);
    }
  };
  int token = -1;
  bool compact = false;
  bool have_x = false;
  // ---- nucleus only (the reference's chat default: temperature 0.8, top_p 0.95, no top-k,
  // chat_engine.py:35-37), bf16 rows ---------------------------------------------------------------
  // For a peaked distribution the nucleus is a few tokens out of tens of thousands.  The candidates
  // are every id at or above the 256-th largest of the per-thread maxima - a complete upper set of
  // the row, usually a few hundred ids; they are sorted and walked exactly as the reference's sort +
  // cumsum does, with probabilities from the softmax of the WHOLE row.  When their mass does not
  // reach top_p (flat rows) the general path below takes over.
  if (a.top_k == 0 && a.top_p > 0.f && a.top_p < 1.f && packed_row && EPT % 8 == 0 && nvalid > 0) {
    uint32_t raw[EPT / 2];
    const bf16_t* row = reinterpret_cast<const bf16_t*>(a.logits) + (size_t)b * a.ldl + base;
#pragma unroll
    for (int c = 0; c < EPT / 8; ++c) {
      const uint4 v = base + 8 * c < V ? ldg16(row + 8 * c) : make_uint4(0, 0, 0, 0);
      raw[4 * c] = v.x; raw[4 * c + 1] = v.y; raw[4 * c + 2] = v.z; raw[4 * c + 3] = v.w;
    }
    auto bits16 = [&](int i) -> uint32_t { return (i & 1) ? (raw[i >> 1] >> 16) : (raw[i >> 1] & 0xffffu); };
    auto key16 = [&](int i) -> uint32_t {  // order-preserving 16-bit key of element i, 0 when masked
      const uint32_t bits = bits16(i);
      const uint32_t kk = (bits & 0x8000u) ? (~bits & 0xffffu) : (bits | 0x8000u);
      return base + i < nvalid ? kk : 0u;
    };
    uint32_t tmax = 0;
#pragma unroll
    for (int i = 0; i < EPT; ++i) tmax = max(tmax, key16(i));
    // softmax statistics of the whole row, formed as the general path forms them: dividing by the
    // temperature is monotone, so the maximum of the quotients is the quotient of the maximum
    const uint32_t mbits = (tmax & 0x8000u) ? (tmax & 0x7fffu) : (~tmax & 0xffffu);
    const float m = block_max(tmax > 0 ? __uint_as_float(mbits << 16) / temp : -INFINITY, s);
    const int have = block_sum_i(tmax > 0 ? 1 : 0, s);
    uint32_t bound = 1;  // fewer than 256 threads hold a valid id: every valid id is a candidate
    if (have >= 256) {
      int dummy;
      bound = radix_select<1, 8>(256, dummy, s, [&](int) { return tmax > 0; }, [&](int) { return tmax; });
    }
    // One CU walks the whole row, so every instruction per element costs about half a microsecond:
    // this pass only has to decide whether the candidates hold the nucleus, and uses the hardware
    // exponential and a multiplication by 1 / temperature (exact arithmetic follows for the
    // candidates only).  Candidates claim their slot with an LDS counter; the order they land in
    // does not matter, the sort below is total (key, then id).
    __syncthreads();
    if (tid == 0) s.misc[0] = 0;
    __syncthreads();
    float zs = 0.f, zc = 0.f;
    const float rtemp = 1.0f / temp;
#pragma unroll
    for (int i = 0; i < EPT; ++i) {
      const uint32_t kk = key16(i);
      const float e = kk == 0 ? 0.f : __expf(__uint_as_float(bits16(i) << 16) * rtemp - m);  // exp(-inf) = 0
      zs += e;
      if (kk >= bound) {
        zc += e;
        const int slot = atomicAdd(&s.misc[0], 1);
        if (slot < CAP) {
          s.skey[slot] = fkey(__uint_as_float(bits16(i) << 16) / temp);
          s.sid[slot] = base + i;
        }
      }
    }
    const float Zq = block_sum(zs, s);
    const float Zc = block_sum(zc, s);  // (the syncs inside also publish the counter and the slots)
    const int n_c = s.misc[0];
    // the nucleus closes inside the candidates when their mass exceeds top_p (with a margin for the
    // different summation orders), or when the candidates are all there is
    if (n_c <= CAP && (Zc / Zq > a.top_p + 1e-3f || bound == 1)) {
      int n2 = 64;
      while (n2 < n_c) n2 <<= 1;
      __syncthreads();
      for (int i = n_c + tid; i < n2; i += NT) {
        s.skey[i] = 0;  // padding sorts last
        s.sid[i] = 0x7fffffff;
      }
      __syncthreads();
      sort_candidates(s, n2);
      if (tid < n_c) {
        const float xi = unfkey(s.skey[tid]);
        s.skey[tid] = __float_as_uint(xi == -INFINITY ? 0.f : expf(xi - m) / Zq);  // probabilities, sorted order
      }
      __syncthreads();
      if (tid == 0) {
        // sequential fp32 sums in the order the reference's cumsum walks (chat_engine.py:71-79)
        float kept = 0.f, run = 0.f;
        int n_in = 0;
        bool closed = bound == 1;
        for (int j = 0; j < n_c; ++j) {  // kept prefix: mass before the token <= top_p
          if (run > a.top_p) {
            closed = true;
            break;
          }
          const float pj = __uint_as_float(s.skey[j]);
          kept += pj;
          run += pj;
          ++n_in;
        }
        int tok = -2;  // -2: the candidates ran out before the nucleus closed
        if (closed || run > a.top_p) {
          const float target = u * kept;
          int last = -1;
          tok = -1;
          run = 0.f;
          for (int j = 0; j < n_in; ++j) {
            const float pj = __uint_as_float(s.skey[j]);
            run += pj;
            if (pj > 0.f) last = s.sid[j];
            if (pj > 0.f && run > target) {
              tok = s.sid[j];
              break;
            }
          }
          if (tok < 0) tok = max(last, 0);  // rounding pushed the target past the end: last kept id
        }
        s.misc[3] = tok;
      }
      __syncthreads();
      if (s.misc[3] >= 0) {
        token = s.misc[3];
        compact = true;
      }
      __syncthreads();
    }
  }
  // ---- small top-k: the survivors fit one sorted block, everything after works on that block -----
  if (a.top_k > 0 && min(a.top_k, V) <= CAP) {
    const int k = min(a.top_k, V);
    int n_c = 0;
    if (packed_row && EPT % 8 == 0) {
      // The selection runs on the raw bf16 logits, two per register: dividing by the temperature
      // is monotone and keeps distinct bf16 values distinct in fp32, so the survivors - and the
      // ties among them - are those of the divided values, and only the survivors are divided.
      // (Half the registers of the fp32 row: nothing spills.)  key 0 = masked id.
      uint32_t raw[EPT / 2];
      const bf16_t* row = reinterpret_cast<const bf16_t*>(a.logits) + (size_t)b * a.ldl + base;
#pragma unroll
      for (int c = 0; c < EPT / 8; ++c) {
        const uint4 v = base + 8 * c < V ? ldg16(row + 8 * c) : make_uint4(0, 0, 0, 0);
        raw[4 * c] = v.x; raw[4 * c + 1] = v.y; raw[4 * c + 2] = v.z; raw[4 * c + 3] = v.w;
      }
      auto key16 = [&](int i) -> uint32_t {  // order-preserving 16-bit key of element i, 0 when masked
        const uint32_t bits = (i & 1) ? (raw[i >> 1] >> 16) : (raw[i >> 1] & 0xffffu);
        const uint32_t kk = (bits & 0x8000u) ? (~bits & 0xffffu) : (bits | 0x8000u);
        return base + i < nvalid ? kk : 0u;
      };
      uint32_t tmax = 0;
#pragma unroll
      for (int i = 0; i < EPT; ++i) tmax = max(tmax, key16(i));
      // ids in [nvalid, V) take part in the reference's top-k as -inf; they can only matter when fewer
      // than k ids are valid, which the general path below handles
      const int have = block_sum_i(tmax > 0 ? 1 : 0, s);
      uint32_t bound = 1;
      if (have >= k) {
        int dummy;
        bound = radix_select<1, 8>(k, dummy, s, [&](int) { return tmax > 0; }, [&](int) { return tmax; });
      }
      int c = 0;
#pragma unroll
      for (int i = 0; i < EPT; ++i) c += key16(i) >= bound ? 1 : 0;
      int off;
      n_c = block_excl_scan_i(c, off, s);
      if (n_c <= CAP && n_c >= min(k, nvalid) && nvalid >= k) {
        compact = true;
        __syncthreads();
        if (c > 0) {
#pragma unroll
          for (int i = 0; i < EPT; ++i)
            if (key16(i) >= bound) {
              const uint32_t bits = (i & 1) ? (raw[i >> 1] >> 16) : (raw[i >> 1] & 0xffffu);
              s.skey[off] = fkey(__uint_as_float(bits << 16) / temp);
              s.sid[off] = base + i;
              ++off;
            }
        }
      }
    }
    if (!compact) {
      load_x();
      have_x = true;
      auto in_vocab = [&](int i) { return base + i < V; };
      auto xkey = [&](int i) { return fkey(x[i]); };  // > 0 for every float but -NaN
      // lower bound of the k-th largest: the k-th largest of the per-thread maxima
      uint32_t tmax = 0;
#pragma unroll
      for (int i = 0; i < EPT; ++i)
        if (in_vocab(i)) tmax = max(tmax, xkey(i));
      const int have = block_sum_i(tmax > 0 ? 1 : 0, s);
      uint32_t bound = 0;
      if (have >= k) {
        int dummy;
        bound = radix_select<1>(k, dummy, s, [&](int) { return tmax > 0; }, [&](int) { return tmax; });
      }
      int c = 0;
#pragma unroll
      for (int i = 0; i < EPT; ++i) c += (in_vocab(i) && xkey(i) >= bound) ? 1 : 0;
      int off;
      n_c = block_excl_scan_i(c, off, s);
      if (n_c <= CAP) {  // (else: many ties at the bound - the general path below handles it)
        compact = true;
        __syncthreads();
        if (c > 0) {
#pragma unroll
          for (int i = 0; i < EPT; ++i)
            if (in_vocab(i) && xkey(i) >= bound) {
              s.skey[off] = xkey(i);
              s.sid[off] = base + i;
              ++off;
            }
        }
      }
    }
    if (compact) token = n_c <= 128 ? draw_from_wave(a, s, n_c, k, u) : draw_from_block(a, s, n_c, k, u);
  }
  if (!compact && !have_x) load_x();
  // ---- top-k: keep x >= k-th largest ---------------------------------------------
  if (!compact && a.top_k > 0) {
    const int k = min(a.top_k, V);
    int ngt;
    auto in_vocab = [&](int i) { return base + i < V; };
    auto xkey = [&](int i) { return fkey(x[i]); };  // > 0 for every float but -NaN
    const uint32_t tk = k <= 1024 ? select_small<EPT>(k, ngt, s, in_vocab, xkey) : radix_select<EPT>(k, ngt, s, in_vocab, xkey);
#pragma unroll
    for (int i = 0; i < EPT; ++i)
      if (fkey(x[i]) < tk) x[i] = -INFINITY;
  }
  if (!compact) {
  // ---- softmax ---------------------------------------------------------------------
  float m = -INFINITY;
#pragma unroll
  for (int i = 0; i < EPT; ++i) m = fmaxf(m, x[i]);
  m = block_max(m, s);
  float zs = 0.f;
#pragma unroll
  for (int i = 0; i < EPT; ++i) {
    x[i] = (x[i] == -INFINITY) ? 0.f : expf(x[i] - m);
    zs += x[i];
  }
  const float Z = block_sum(zs, s);
#pragma unroll
  for (int i = 0; i < EPT; ++i) x[i] = x[i] / Z;  // probabilities; 0 marks a filtered id

  if (!(a.top_p > 0.f && a.top_p < 1.f)) {
    // ---- inverse CDF in vocabulary order ------------------------------------------
    float ts = 0.f;
#pragma unroll
    for (int i = 0; i < EPT; ++i) ts += x[i];
    // prefix sums of the per-thread masses, in thread order: thread t owns [lo, hi)
    float lo, hi;
    const float total = block_scan_f(ts, lo, hi, s);
    const float target = u * total;
    // last id with p > 0 (fallback when rounding pushes target past the end)
    int lastpos = -1;
#pragma unroll
    for (int i = 0; i < EPT; ++i)
      if (x[i] > 0.f) lastpos = base + i;
    int mx = lastpos;
    mx = lanes_max<32, 1>(mx);
    __syncthreads();
    if ((tid & 63) == 0) s.wredi[tid >> 6] = mx;
    if (tid == 0) s.misc[2] = 0x7fffffff;
    __syncthreads();
    int last_id = -1;
#pragma unroll
    for (int i = 0; i < NW; ++i) last_id = max(last_id, s.wredi[i]);
    if (target >= lo && target < hi) {  // exactly one thread
      float run = lo;
      int found = lastpos;  // the running sum inside the thread may round short of hi
      bool hit = false;
#pragma unroll
      for (int i = 0; i < EPT; ++i) {
        run += x[i];
        if (x[i] > 0.f && run > target && !hit) {
          found = base + i;
          hit = true;
        }
      }
      s.misc[2] = found;
    }
    __syncthreads();
    token = s.misc[2] == 0x7fffffff ? max(last_id, 0) : s.misc[2];
  } else {
    // ---- nucleus without sorting: thresholds on the probability bits by bisection --------------
    // In descending order (ties lowest id first) a token is kept iff the mass before it is <= top_p.
    // With G(t) = mass of the keys above t, that is: every key above Tk, plus the first
    // floor((top_p - G(T)) / p_T) + 1 ties at T, where T is the smallest key with G(T) <= top_p.  T is
    // found bit by bit (31 block sums in a fixed order), and so is the key the draw u * S lands on;
    // the sums are over registers, so the cost does not depend on how many tokens are kept.
    auto pkey = [&](int i) { return __float_as_uint(x[i]); };  // p > 0: bits are monotone; 0 = filtered
    auto mass_ge = [&](uint32_t c) {
      float t = 0.f;
#pragma unroll
      for (int i = 0; i < EPT; ++i) t += (pkey(i) >= c) ? x[i] : 0.f;
      return block_sum(t, s);
    };
    auto count_eq = [&](uint32_t c) {
      int n = 0;
#pragma unroll
      for (int i = 0; i < EPT; ++i) n += (pkey(i) == c) ? 1 : 0;
      return block_sum_i(n, s);
    };
    // smallest key Tk >= 1 with mass(keys > Tk) <= limit; needs mass(keys >= 1) > limit
    auto threshold = [&](float limit) {
      uint32_t tf = 0;  // largest t with mass(keys >= t + 1) > limit
      for (int bit = 30; bit >= 0; --bit) {
        const uint32_t c = tf | (1u << bit);
        if (mass_ge(c + 1) > limit) tf = c;
      }
      return tf + 1;
    };
    const float total = mass_ge(1u);
    uint32_t Tk = 1;  // everything with p > 0 when top_p is not below the total mass
    float G = 0.f, S = total;
    int n_keep = 0x7fffffff;
    if (total > a.top_p) {
      Tk = threshold(a.top_p);
      G = mass_ge(Tk + 1);
      const float pT = __uint_as_float(Tk);
      n_keep = min(count_eq(Tk), (int)floorf((a.top_p - G) / pT) + 1);
      S = G + (float)n_keep * pT;
    }
    const float target = u * S;
    uint32_t Td = threshold(target);  // target < S <= mass(keys >= Tk): the key found is >= Tk
    if (Td < Tk) Td = Tk;               // (rounding guard)
    const float Gd = mass_ge(Td + 1);
    const int ties = count_eq(Td);
    int r = (int)floorf((target - Gd) / __uint_as_float(Td));
    r = max(0, min(r, min(ties, Td == Tk ? n_keep : ties) - 1));
    // the r-th token in id order among the ties at Td
    int c = 0;
#pragma unroll
    for (int i = 0; i < EPT; ++i) c += (pkey(i) == Td) ? 1 : 0;
    int off;
    block_excl_scan_i(c, off, s);
    if (tid == 0) s.misc[3] = -1;
    __syncthreads();
    if (c > 0 && off <= r && r < off + c) {
      int seen = off;
#pragma unroll
      for (int i = 0; i < EPT; ++i)
        if (pkey(i) == Td) {
          if (seen == r) s.misc[3] = base + i;
          ++seen;
        }
    }
    __syncthreads();
    token = max(s.misc[3], 0);
  }
  }  // !compact
  return token;
}

template <typename T, int EPT>
__global__ __launch_bounds__(NT) void sample_kernel(SampleArgs a) {
  __shared__ Smem s;
  const int token = sample_row<T, EPT>(a, blockIdx.x, s);
  if (threadIdx.x == 0) finish_row(a, blockIdx.x, token);
}


// Out-of-line copies of the two rarely taken routes of sample_parts_kernel (a part that gave up; more
// than 128 survivors): inlined, the whole-row algorithm is nine tenths of that kernel's code and its
// register demand spills values of the route that is always taken.
__device__ __attribute__((noinline)) int sample_row_bf16_call(SampleArgs a, int b, Smem& s) {  // by value: a reference would put the caller's copy in scratch
  return sample_row<bf16_t, 64>(a, b, s);
}
__device__ __attribute__((noinline)) int draw_from_block_call(SampleArgs a, Smem& s, int n_c, int k, float u) {
  return draw_from_block(a, s, n_c, k, u);
}

// ---------------------------------------------------------------------------------------------
// Small top-k over several workgroups.  With top-k the draw depends on the k largest logits of the
// row only (ties of the k-th included), and one CU walking 65536 ids is what the single-workgroup
// kernel spends its time on.  Here a row is cut into parts of 8192 ids, one workgroup each (eight ids
// per thread, one 16-byte load): a part hands over every id at or above the k-th largest of its
// per-thread maxima - a lower bound of the part's k-th largest, so the union of the parts' candidates
// holds the row's k largest with all their ties - as (id << 16 | bf16 bits) words; the workgroup that
// finishes last gathers at most 8 x 128 candidates and draws from them exactly as the single-workgroup
// kernel draws from its own (draw_from_block).  Candidates travel as write-through stores, the
// arrival counter is a relaxed device-scope atomic behind a wait for the own stores, the gather uses
// cache-bypassing loads (the hand-off of the split attention kernels).  A part with more than 128
// candidates (a row of mostly equal values) makes the last workgroup run the single-workgroup
// algorithm on the whole row instead.
// Scratch: a static device array, [row] counters one 128-byte line apart, then per (row, part) one
// line with the count and 512 bytes of candidates.  Calls that overlap in time on one GPU would share
// it: the host takes this route only for callers that said their sampler calls do not overlap.
// ---------------------------------------------------------------------------------------------
constexpr int PART_IDS = NT * 8;   // ids per part
constexpr int PART_CAP = 128;      // candidates a part may hand over
constexpr int PART_MAX = 8;        // parts per row (65536 ids)
constexpr int PART_ROWS = 64;      // rows per call
constexpr int PART_REC = 32 + PART_CAP;  // dwords per (row, part) record
constexpr size_t PART_SCRATCH_DWORDS = (size_t)PART_ROWS * 32 + (size_t)PART_ROWS * PART_MAX * PART_REC;

__global__ __launch_bounds__(NT) void sample_parts_kernel(SampleArgs a, uint32_t* scratch, int nparts) {
  __shared__ Smem s;
  const int part = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
  const int V = a.V, nvalid = min(a.valid, V);
  const int k = min(a.top_k, V);
  const int base = part * PART_IDS + tid * 8;
  const bf16_t* row = reinterpret_cast<const bf16_t*>(a.logits) + (size_t)b * a.ldl + base;
  const uint4 v = base < V ? ldg16(row) : make_uint4(0, 0, 0, 0);
  static_assert(NT == 1024, "select16_clear: one thread per table entry");
  select16_clear(s);  // the counting tables of both selections, while the load is in flight
  __syncthreads();
  const uint32_t raw[4] = {v.x, v.y, v.z, v.w};
  auto bits16 = [&](int i) -> uint32_t { return (i & 1) ? (raw[i >> 1] >> 16) : (raw[i >> 1] & 0xffffu); };
  auto key16 = [&](int i) -> uint32_t {  // order-preserving 16-bit key of element i, 0 when masked
    const uint32_t bits = bits16(i);
    const uint32_t kk = (bits & 0x8000u) ? (~bits & 0xffffu) : (bits | 0x8000u);
    return base + i < nvalid ? kk : 0u;
  };
  uint32_t tmax = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) tmax = max(tmax, key16(i));
  // threads that hold a valid id: all of them when the part lies below the valid ids' end and k is
  // small (then a thread whose eight values are all NaN patterns cannot take the count below k)
  const bool whole = (part + 1) * PART_IDS <= nvalid && k <= NT / 2;
  const int have = whole ? NT : block_sum_i(tmax > 0 ? 1 : 0, s);
  uint32_t bound = 1;  // fewer than k threads hold a valid id: every valid id of the part is a candidate
  if (have >= k) {
    bound = select16_block(k, tmax, s, s.hist, s.hist2[0]);
  }
  int c = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) c += key16(i) >= bound ? 1 : 0;
  int off;
  const int n_part = block_excl_scan_i(c, off, s);
  uint32_t* rec = scratch + (size_t)PART_ROWS * 32 + ((size_t)b * PART_MAX + part) * PART_REC;
  if (n_part <= PART_CAP && c > 0) {
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (key16(i) >= bound) st_coh4(rec + 32 + off++, ((uint32_t)(base + i) << 16) | bits16(i));
  }
  if (tid == 0) st_coh4(rec, n_part <= PART_CAP ? (uint32_t)n_part : 0xffffffffu);
  // ---- hand-off: the workgroup that arrives last draws -------------------------------------------
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  wait_own_stores();
  __syncthreads();
  if (tid == 0) {
    int* counter = reinterpret_cast<int*>(scratch) + b * 32;
    const int old = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const int last = old == nparts - 1;
    if (last) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next call
    s.misc[7] = last;
  }
  __syncthreads();
  if (!s.misc[7]) return;
  // One round of loads: thread t looks at slot t % 128 of part t / 128 (8 parts x 128 slots are the
  // 1024 threads) and at that part's count; lane l of every wave reads the count of part l as well, so
  // that each wave knows by itself whether some part gave up.
  const uint32_t* rec0 = scratch + (size_t)PART_ROWS * 32 + (size_t)b * PART_MAX * PART_REC;
  static_assert(PART_MAX * PART_CAP == NT, "one thread per candidate slot");
  const int my_part = tid / PART_CAP, my_slot = tid % PART_CAP;
  const int lane = tid & 63;
  uint32_t n_mine = 0, w = 0, n_lane = 0;
  if (my_part < nparts) {
    n_mine = ld_coh4(rec0 + (size_t)my_part * PART_REC);
    w = ld_coh4(rec0 + (size_t)my_part * PART_REC + 32 + my_slot);
  }
  if (lane < nparts) n_lane = ld_coh4(rec0 + (size_t)lane * PART_REC);
  const bool overflow = __ballot(n_lane == 0xffffffffu) != 0;
  int token;
  if (overflow) {
    token = sample_row_bf16_call(a, b, s);
  } else {
    // the k-th largest of the gathered candidates first (16-bit keys, two counting passes), so that the
    // block that is sorted holds the k survivors and their ties, not eight times as many
    uint32_t k16 = 0;
    if (my_slot < (int)n_mine) {
      const uint32_t bits = w & 0xffffu;
      k16 = (bits & 0x8000u) ? (~bits & 0xffffu) : (bits | 0x8000u);
    }
    const uint32_t tk16 = select16_block(k, k16, s, s.hist2[1], s.hist2[2]);
    const int keep = (k16 > 0 && k16 >= tk16) ? 1 : 0;
    int slot;
    const int n_keep = block_excl_scan_i(keep, slot, s);
    const float u = a.u[(a.step_state && a.u_step_stride > 0 ? (size_t)a.step_state[1] * a.u_step_stride : 0) + b];
    __syncthreads();
    if (n_keep <= 128) {
      if (keep) s.skey[slot] = (k16 << 16) | (0xffffu - (w >> 16));
      token = draw_from_wave_packed(a, s, n_keep, k, u);
    } else {
      if (keep) {
        s.skey[slot] = fkey(__uint_as_float((w & 0xffffu) << 16) / a.temperature);
        s.sid[slot] = (int)(w >> 16);
      }
      token = draw_from_block_call(a, s, n_keep, k, u);
    }
  }
  if (tid == 0) finish_row(a, b, token);
}

static __device__ __align__(256) uint32_t sampler_scratch[PART_SCRATCH_DWORDS];

// Device address of sampler_scratch on the current device (nullptr on failure): the array's name is a
// host-side handle only.
uint32_t* sampler_scratch_ptr() {
  static uint32_t* ptrs[16];
  static std::mutex mu;
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return nullptr;
  std::lock_guard<std::mutex> lock(mu);
  if (!ptrs[dev]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(sampler_scratch)) != hipSuccess) return nullptr;
    ptrs[dev] = reinterpret_cast<uint32_t*>(p);
  }
  return ptrs[dev];
}

// ---------------------------------------------------------------------------------------------
// bf16 rows of at most 65536 ids: selection on the histogram of the 16-bit keys.
//
// A bf16 logit has one of 65536 bit patterns, dividing by the temperature and the softmax are
// monotone, so every id with the same pattern has the same probability and the whole distribution is
// the table (pattern -> count).  One pass counts the patterns into LDS (two 16-bit counts per dword,
// 128 KB); everything the sampler has to find is then a walk over that table in descending key order,
// 64 keys per thread with block-wide prefix sums in a fixed order:
//   * top-k: the key at which the cumulative count reaches k (ties at it survive, chat_engine.py:66-69);
//   * softmax normaliser: sum of count * exp(x(key) - max) over the surviving keys;
//   * nucleus: in descending order (ties lowest id first) a token is kept iff the mass before it is
//     <= top_p (chat_engine.py:72-79); the j-th tie of a key has run + j * p(key) before it, so the last
//     kept key and the number of its ties that are kept follow in closed form;
//   * the draw: the key the target u * (kept mass) falls into and the index r of the tie inside it;
// and one last pass over the row picks the r-th id (in id order) with that key.  Without a nucleus the
// draw walks the ids in vocabulary order (chat_engine.py:82) and the table only supplies the top-k
// threshold.  No sort, no bisection, nothing spills, and the time does not depend on what the row looks like.
// ---------------------------------------------------------------------------------------------
constexpr int HB = 32768;      // dwords of the count table
constexpr int ENT_CAP = 4096;  // entries of the compacted (key, count) list

__device__ __forceinline__ int block_max_i(int v, Smem& s) {
  v = lanes_max<32, 1>(v);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) s.wredi[w] = v;
  __syncthreads();
  int r = s.wredi[0];
#pragma unroll
  for (int i = 1; i < NW; ++i) r = max(r, s.wredi[i]);
  return r;
}

__device__ __forceinline__ float key16_value(uint32_t key) {  // the bf16 value an order-preserving key stands for
  const uint32_t bits = (key & 0x8000u) ? (key & 0x7fffu) : (~key & 0xffffu);
  return __uint_as_float(bits << 16);
}

// max of a, max of b and sum of c over the workgroup in one exchange (two barriers instead of six)
__device__ __forceinline__ void block_max_max_sum_i(int& a, int& b, int& c, Smem& s) {
  a = lanes_max<32, 1>(a);
  b = lanes_max<32, 1>(b);
  c = lanes_sum<32, 1>(c);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) {
    s.wredi[w] = a;
    s.hist[w] = b;
    s.hist[NW + w] = c;
  }
  __syncthreads();
  int ra = s.wredi[0], rb = s.hist[0], rc = s.hist[NW];
#pragma unroll
  for (int i = 1; i < NW; ++i) {
    ra = max(ra, s.wredi[i]);
    rb = max(rb, s.hist[i]);
    rc += s.hist[NW + i];
  }
  a = ra;
  b = rb;
  c = rc;
}

template <int EPT>
__global__ __launch_bounds__(NT) void sample_hist_kernel(SampleArgs a) {
  extern __shared__ uint32_t hist[];  // HB dwords: key k counted in half (k & 1) of dword k >> 1; then the list
  __shared__ Smem s;
  const int b = blockIdx.x, tid = threadIdx.x;
  const int V = a.V, nvalid = min(a.valid, V);
  const int base = tid * EPT;
  const float temp = a.temperature;
  const float u = a.u[(a.step_state && a.u_step_stride > 0 ? (size_t)a.step_state[1] * a.u_step_stride : 0) + b];
  const bf16_t* row = reinterpret_cast<const bf16_t*>(a.logits) + (size_t)b * a.ldl + base;
  // One CU walks the whole row, so every instruction per id costs about half a microsecond.  The row
  // is not kept in registers between the passes: each pass re-reads its 16 bytes per eight ids from
  // the L2 and turns the two bf16 patterns of a register into order-preserving
  // 16-bit keys with four integer instructions.  fn(id, key) is called for the thread's valid ids in
  // id order; key 0 cannot occur for a number (it is the pattern of one NaN) and is skipped.
  // All loads of a pass go out before the first is used (addresses past the valid ids fall back on the
  // chunk of the last valid id, whose values are not looked at): one round trip to the L2 per pass.
  const bf16_t* row0 = reinterpret_cast<const bf16_t*>(a.logits) + (size_t)b * a.ldl;
  const int last_chunk = nvalid > 0 ? ((nvalid - 1) & ~7) : 0;
  auto for_each_key = [&](auto&& fn) {
    uint4 vv[EPT / 8];
#pragma unroll
    for (int c = 0; c < EPT / 8; ++c) vv[c] = ldg16(row0 + min(base + 8 * c, last_chunk));
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int c = 0; c < EPT / 8; ++c) {
      const int id0 = base + 8 * c;
      if (id0 < nvalid) {
        const uint4 v = vv[c];
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
        const bool whole = id0 + 8 <= nvalid;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t neg = ((w[j] >> 15) & 0x00010001u) * 0xffffu;  // 0xffff in the halves that hold a negative value
          const uint32_t kk = w[j] ^ (neg | 0x80008000u);                // negative: all bits flipped; else the sign bit set
          const uint32_t klo = kk & 0xffffu, khi = kk >> 16;
          if (klo && (whole || id0 + 2 * j < nvalid)) fn(id0 + 2 * j, klo);
          if (khi && (whole || id0 + 2 * j + 1 < nvalid)) fn(id0 + 2 * j + 1, khi);
        }
      }
    }
  };
  auto xval = [&](uint32_t key) { return key16_value(key) / temp; };
  const bool nucleus = a.top_p > 0.f && a.top_p < 1.f;
  const bool want_table = a.top_k > 0 || nucleus;
  if (want_table) {
    uint4* h4 = reinterpret_cast<uint4*>(hist);
    for (int i = tid; i < HB / 4; i += NT) h4[i] = make_uint4(0, 0, 0, 0);
    __syncthreads();
  }
  int tmax = 0, tmin = 0x10000, live = 0;
  for_each_key([&](int, uint32_t kk) {
    tmax = max(tmax, (int)kk);
    tmin = min(tmin, (int)kk);
    ++live;
    if (want_table) atomicAdd(&hist[kk >> 1], (kk & 1u) ? 0x10000u : 1u);
  });
  int kmax = tmax, nkmin = -tmin, n_live = live;
  block_max_max_sum_i(kmax, nkmin, n_live, s);  // (the barriers inside also complete the table)
  const int kmin = -nkmin;
  int token = 0;
  if (kmax > 0) {
    const float m = xval((uint32_t)kmax);
    const int k = min(a.top_k, V);
    const bool use_topk = a.top_k > 0 && k < n_live;  // k >= the number of valid ids: everything survives
    // a row of one single value is the only way a 16-bit count can overflow: its table is not looked at
    const bool one_value = kmax == kmin;
    const bool need_table = (use_topk || nucleus) && !one_value;
    // The keys that occur, with their counts, compacted into a list in descending key order (a flat
    // row of N(0,1)-like logits has about 1500 distinct patterns out of 65536): every later walk then
    // touches one or two entries per thread instead of 64 table slots.
    uint32_t* ent = hist + HB;  // entry = key << 16 | count (count < 65536: more than one value occurs)
    int n_ent = 1;
    if (need_table) {
      const uint4* seg = reinterpret_cast<const uint4*>(hist + HB - 32 * (tid + 1));  // my 64 keys, ascending
      uint4 sv[8];
#pragma unroll
      for (int q = 0; q < 8; ++q) sv[q] = seg[q];
      int nz = 0;
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        const uint32_t w[4] = {sv[q].x, sv[q].y, sv[q].z, sv[q].w};
#pragma unroll
        for (int i = 0; i < 4; ++i) nz += ((w[i] >> 16) ? 1 : 0) + ((w[i] & 0xffffu) ? 1 : 0);
      }
      int off;
      n_ent = block_excl_scan_i(nz, off, s);
      if (n_ent <= ENT_CAP && nz) {
        const int kbase = 65536 - 64 * (tid + 1);  // key of the low half of seg[0].x
#pragma unroll
        for (int q = 7; q >= 0; --q) {
          const uint32_t w[4] = {sv[q].x, sv[q].y, sv[q].z, sv[q].w};
#pragma unroll
          for (int i = 3; i >= 0; --i) {
            const int key = kbase + 8 * q + 2 * i;
            if (w[i] >> 16) ent[off++] = ((uint32_t)(key + 1) << 16) | (w[i] >> 16);
            if (w[i] & 0xffffu) ent[off++] = ((uint32_t)key << 16) | (w[i] & 0xffffu);
          }
        }
      }
      __syncthreads();
    }
    const bool listed = n_ent <= ENT_CAP;
    const int per = (n_ent + NT - 1) / NT;
    // fn(key, count) for this thread's share of the keys that occur, in descending key order (thread 0
    // holds the largest keys); fn returns true to stop
    auto walk = [&](auto&& fn) {
      if (one_value) {
        if (tid == 0) fn((uint32_t)kmax, (uint32_t)n_live);
        return;
      }
      if (listed) {
        const int e1 = min(n_ent, (tid + 1) * per);
#pragma unroll 1
        for (int e = tid * per; e < e1; ++e) {
          const uint32_t w = ent[e];
          if (fn(w >> 16, w & 0xffffu)) return;
        }
        return;
      }
      const int ktop = 65535 - 64 * tid;  // more distinct patterns than the list holds: the table itself
#pragma unroll 1
      for (int j = 0; j < 64; ++j) {
        const int key = ktop - j;
        const uint32_t c = key ? (hist[key >> 1] >> ((key & 1) << 4)) & 0xffffu : 0u;
        if (c && fn((uint32_t)key, c)) return;
      }
    };
    // ---- top-k threshold: the key at which the cumulative count reaches k ----------------------
    uint32_t Tk = 1;
    if (use_topk) {
      int cnt = 0;
      walk([&](uint32_t, uint32_t c) { cnt += (int)c; return false; });
      int before;
      block_excl_scan_i(cnt, before, s);
      if (before < k && k <= before + cnt) {
        int run = before;
        walk([&](uint32_t key, uint32_t c) {
          run += (int)c;
          if (run >= k) {
            s.misc[4] = (int)key;
            return true;
          }
          return false;
        });
      }
      __syncthreads();
      Tk = (uint32_t)s.misc[4];
    }
    auto prob = [&](uint32_t key) {  // exp(x - max): the unnormalised probability of one id with this key
      const float xv = xval(key);
      return xv == -INFINITY ? 0.f : expf(xv - m);
    };
    if (nucleus) {
      // ---- masses in descending key order: thread t owns [lo, hi) of the total Z -------------------
      float mass = 0.f;
      walk([&](uint32_t key, uint32_t c) {
        if (key < Tk) return true;
        mass += (float)c * prob(key);
        return false;
      });
      float lo, hi;
      const float Z = block_scan_f(mass, lo, hi, s);
      const float limit = a.top_p * Z;
      if (tid == 0) {  // defaults: everything kept
        s.misc[5] = (int)Tk;
        s.misc[6] = -1;  // all ties of the boundary key
        s.fmisc[0] = Z;
      }
      __syncthreads();
      if (lo <= limit && limit < hi) {
        // the last kept key, how many of its ties are kept, and the kept mass S
        float run = lo, S = hi;
        uint32_t Tn = 0, nk = 0, lastk = 0, lastc = 0;
        bool found = false;
        walk([&](uint32_t key, uint32_t c) {
          if (key < Tk) return true;
          const float e = prob(key);
          if (e == 0.f) return false;
          lastk = key;
          lastc = c;
          const float room = floorf((limit - run) / e) + 1.f;  // ties whose preceding mass is <= limit
          if (room < (float)c) {
            Tn = key; nk = (uint32_t)room; S = run + room * e; found = true;
            return true;
          }
          run += (float)c * e;
          if (run > limit) {  // the next token already has more than top_p before it
            Tn = key; nk = c; S = run; found = true;
            return true;
          }
          return false;
        });
        if (!found) { Tn = lastk; nk = lastc; S = run; }
        if (Tn) {
          s.misc[5] = (int)Tn;
          s.misc[6] = (int)nk;
          s.fmisc[0] = S;
        }
      }
      __syncthreads();
      const uint32_t Tn = (uint32_t)s.misc[5];
      const int nk = s.misc[6];
      const float target = u * s.fmisc[0];
      __syncthreads();
      if (tid == 0) {
        s.misc[7] = kmax;  // fallback: the first id of the largest key
        s.misc[3] = 0;
      }
      __syncthreads();
      if (lo <= target && target < hi) {
        float run = lo;
        uint32_t lastk = 0, lastc = 0;
        bool found = false;
        walk([&](uint32_t key, uint32_t c) {
          if (key < Tn) return true;
          const float e = prob(key);
          if (e == 0.f) return false;
          const uint32_t cc = (key == Tn && nk >= 0) ? (uint32_t)nk : c;
          if (cc == 0) return true;
          lastk = key;
          lastc = cc;
          const float end = run + (float)cc * e;
          if (target < end) {
            int r = (int)floorf((target - run) / e);
            r = max(0, min(r, (int)cc - 1));
            s.misc[7] = (int)key;
            s.misc[3] = r;
            found = true;
            return true;
          }
          run = end;
          return false;
        });
        if (!found && lastk) {  // rounding pushed the target past the last kept tie
          s.misc[7] = (int)lastk;
          s.misc[3] = (int)lastc - 1;
        }
      }
      __syncthreads();
      const uint32_t Td = (uint32_t)s.misc[7];
      const int r = s.misc[3];
      // the r-th id, in id order, among the ids with key Td: one pass notes where in the thread's ids
      // the key occurs (the bf16 pattern behind the key is compared as loaded: two instructions an id,
      // on a CU that spends 0.44 us on every instruction per id), the thread that owns the r-th
      // occurrence picks it from its own notes
      unsigned long long where = 0;
      {
        const uint32_t pat = (Td & 0x8000u) ? (Td & 0x7fffu) : (~Td & 0xffffu);  // key -> bf16 bits
        const uint32_t pat2 = pat | (pat << 16);
        uint4 vv[EPT / 8];
#pragma unroll
        for (int c = 0; c < EPT / 8; ++c) vv[c] = ldg16(row0 + min(base + 8 * c, last_chunk));
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int c = 0; c < EPT / 8; ++c) {
          const uint32_t w[4] = {vv[c].x, vv[c].y, vv[c].z, vv[c].w};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const uint32_t x = w[j] ^ pat2;
            if ((x & 0xffffu) == 0) where |= 1ull << (8 * c + 2 * j);
            if ((x >> 16) == 0) where |= 1ull << (8 * c + 2 * j + 1);
          }
        }
        // ids at or past the end of the valid ones (and the chunks that stood in for them) do not count
        const int nv = nvalid - base;
        where = nv >= EPT ? where : (nv <= 0 ? 0ull : where & ((1ull << nv) - 1ull));
      }
      static_assert(EPT <= 64, "one bit per id of the thread");
      const int c = __popcll(where);
      int off;
      block_excl_scan_i(c, off, s);
      if (tid == 0) s.misc[2] = -1;
      __syncthreads();
      if (c > 0 && off <= r && r < off + c) {
        for (int skip = r - off; skip > 0; --skip) where &= where - 1;  // drop the occurrences before the r-th
        s.misc[2] = base + __ffsll((long long)where) - 1;
      }
      __syncthreads();
      token = max(s.misc[2], 0);
    } else {
      // ---- inverse CDF in vocabulary order over the surviving ids (chat_engine.py:82) ---------------
      // This pass touches every id: a multiplication by 1 / temperature and the hardware exponential
      // 2^((x - max) * log2 e), a handful of instructions instead of forty; the relative error (about
      // 1e-6 for x - max > -30) is far inside what the fp32 sums over 65536 terms carry anyway.
      const float rtemp = 1.0f / temp;
      auto pe = [&](uint32_t kk) {
        const float xv = key16_value(kk) * rtemp;
        return (kk >= Tk && xv != -INFINITY) ? __expf(xv - m) : 0.f;
      };
      float ts = 0.f;
      int lastpos = -1;
      for_each_key([&](int id, uint32_t kk) {
        const float e = pe(kk);
        ts += e;
        if (e > 0.f) lastpos = id;
      });
      float lo, hi;
      const float total = block_scan_f(ts, lo, hi, s);
      const float target = u * total;
      const int last_id = block_max_i(lastpos, s);
      if (tid == 0) s.misc[2] = 0x7fffffff;
      __syncthreads();
      if (target >= lo && target < hi) {  // exactly one thread
        float run = lo;
        int found = lastpos;  // the running sum inside the thread may round short of hi
        bool hit = false;
        for_each_key([&](int id, uint32_t kk) {
          const float e = pe(kk);
          run += e;
          if (e > 0.f && run > target && !hit) {
            found = id;
            hit = true;
          }
        });
        s.misc[2] = found;
      }
      __syncthreads();
      token = s.misc[2] == 0x7fffffff ? max(last_id, 0) : s.misc[2];
    }
  }
  if (tid == 0) {
    a.out[b] = token;
    if (a.step_state) {
      const int step = a.step_state[1];
      if (a.history && step < a.hist_cap) a.history[(size_t)step * a.B + b] = token;
      // only the counter is shared between workgroups: no fence, the ids are read by later kernels
      const int old = __hip_atomic_fetch_add(&a.step_state[2], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (old == a.B - 1) {
        a.step_state[2] = 0;
        a.step_state[0] += 1;
        a.step_state[1] = step + 1;
      }
    }
  }
}

template <int EPT>
int launch_hist(const SampleArgs& a, hipStream_t st) {
  static bool configured = false;  // (benign if two threads both set it)
  const int smem = (HB + ENT_CAP) * (int)sizeof(uint32_t);
  if (!configured) {
    if (hipFuncSetAttribute((const void*)sample_hist_kernel<EPT>, hipFuncAttributeMaxDynamicSharedMemorySize, smem) !=
        hipSuccess)
      return OHARA_ELAUNCH;
    configured = true;
  }
  hipLaunchKernelGGL((sample_hist_kernel<EPT>), dim3(a.B), dim3(NT), smem, st, a);
  return ohara_launch_status();
}

template <typename T>
int launch_sample(const SampleArgs& a, hipStream_t st) {
  dim3 grid(a.B), block(NT);
  if (a.V <= NT * 4) hipLaunchKernelGGL((sample_kernel<T, 4>), grid, block, 0, st, a);
  else if (a.V <= NT * 32) hipLaunchKernelGGL((sample_kernel<T, 32>), grid, block, 0, st, a);
  else if (a.V <= NT * 64) hipLaunchKernelGGL((sample_kernel<T, 64>), grid, block, 0, st, a);
  else if (a.V <= NT * 128) hipLaunchKernelGGL((sample_kernel<T, 128>), grid, block, 0, st, a);
  else return OHARA_ESIZE;
  return ohara_launch_status();
}


int sample_dispatch(const void* logits, int logits_are_fp32, int ldl, int batch, int vocab, int valid_vocab,
                    float temperature, int top_k, float top_p, const float* u, int u_step_stride, int64_t* out_ids,
                    int64_t* history, int hist_cap, int32_t* step_state, void* stream, bool exclusive,
                    uint32_t* workspace = nullptr) {
  if (!logits || !u || !out_ids || batch < 1 || vocab < 1 || ldl < vocab) return OHARA_EINVAL;
  if (!(temperature > 0.f) || top_k < 0 || !(top_p >= 0.f && top_p <= 1.f) || u_step_stride < 0) return OHARA_EINVAL;
  SampleArgs a{};
  a.logits = logits; a.ldl = ldl; a.V = vocab; a.valid = valid_vocab > 0 ? valid_vocab : vocab;
  a.temperature = temperature; a.top_p = top_p; a.top_k = top_k; a.u = u; a.u_step_stride = u_step_stride; a.out = out_ids;
  a.history = history; a.hist_cap = hist_cap; a.step_state = step_state; a.B = batch;
  hipStream_t st = (hipStream_t)stream;
  const bool aligned = (ldl & 7) == 0 && (reinterpret_cast<uintptr_t>(logits) & 15) == 0;
  // a small top-k on a long bf16 row, for a caller whose sampler calls do not overlap: the row spread
  // over one workgroup per 8192 ids (measured at 65536 ids, top-k 50 + top-p 0.9: see the header)
  if (exclusive && !logits_are_fp32 && aligned && top_k > 0 && top_k <= 64 && vocab > PART_IDS &&
      vocab <= PART_IDS * PART_MAX && batch <= PART_ROWS && (a.valid < vocab ? a.valid : vocab) >= top_k) {
    uint32_t* scratch = workspace ? workspace : sampler_scratch_ptr();  // the caller's own, or the library's
    if (!scratch) return OHARA_ELAUNCH;
    const int nparts = (vocab + PART_IDS - 1) / PART_IDS;
    hipLaunchKernelGGL(sample_parts_kernel, dim3(nparts, batch), dim3(NT), 0, st, a, scratch, nparts);
    return ohara_launch_status();
  }
  // bf16 rows: selection on the histogram of the 16-bit patterns, except for a small top-k, where sorting
  // the few survivors is quicker (measured at 65536 ids: top-k 50 + top-p 0.9: 27 us sorted, 37 us by the
  // table; top-p alone: 37 us (sharp row) to 139 us (flat row) with candidates / bisection, 37-38 us by
  // the table whatever the row; plain multinomial 33 us either way)
  const bool small_k = top_k > 0 && top_k <= CAP;
  if (!logits_are_fp32 && !small_k && vocab <= 65536 && (ldl & 7) == 0 &&
      (reinterpret_cast<uintptr_t>(logits) & 15) == 0) {
    if (vocab <= NT * 8) return launch_hist<8>(a, st);
    if (vocab <= NT * 32) return launch_hist<32>(a, st);
    return launch_hist<64>(a, st);
  }
  return logits_are_fp32 ? launch_sample<float>(a, st) : launch_sample<bf16_t>(a, st);
}

}  // namespace

extern "C" {

int ohara_sample_topk_topp(const void* logits, int logits_are_fp32, int ldl, int batch, int vocab, int valid_vocab,
                           float temperature, int top_k, float top_p, const float* u, int u_step_stride,
                           int64_t* out_ids, int64_t* history, int hist_cap, int32_t* step_state, void* stream) {
  return sample_dispatch(logits, logits_are_fp32, ldl, batch, vocab, valid_vocab, temperature, top_k, top_p, u,
                         u_step_stride, out_ids, history, hist_cap, step_state, stream, false);
}

int ohara_sample_topk_topp_exclusive(const void* logits, int logits_are_fp32, int ldl, int batch, int vocab,
                                     int valid_vocab, float temperature, int top_k, float top_p, const float* u,
                                     int u_step_stride, int64_t* out_ids, int64_t* history, int hist_cap,
                                     int32_t* step_state, void* stream) {
  return sample_dispatch(logits, logits_are_fp32, ldl, batch, vocab, valid_vocab, temperature, top_k, top_p, u,
                         u_step_stride, out_ids, history, hist_cap, step_state, stream, true);
}

int64_t ohara_sample_workspace_bytes(void) { return (int64_t)(PART_SCRATCH_DWORDS * sizeof(uint32_t)); }

int ohara_sample_topk_topp_ws(const void* logits, int logits_are_fp32, int ldl, int batch, int vocab, int valid_vocab,
                              float temperature, int top_k, float top_p, const float* u, int u_step_stride,
                              int64_t* out_ids, int64_t* history, int hist_cap, int32_t* step_state, void* workspace,
                              int64_t workspace_bytes, void* stream) {
  if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 255) ||
      workspace_bytes < (int64_t)(PART_SCRATCH_DWORDS * sizeof(uint32_t)))
    return OHARA_EINVAL;
  return sample_dispatch(logits, logits_are_fp32, ldl, batch, vocab, valid_vocab, temperature, top_k, top_p, u,
                         u_step_stride, out_ids, history, hist_cap, step_state, stream, true,
                         static_cast<uint32_t*>(workspace));
}

}  // extern "C"
