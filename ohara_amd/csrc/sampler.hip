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
// A thread owns EPT consecutive vocabulary entries in registers; the 1024 threads cover up
// to 1024*EPT ids.  The sorted prefix is built 1024 candidates at a time (radix select on
// the probability bits, ordered compaction, bitonic sort in LDS) and scanned sequentially
// in fp32, the order torch.cumsum uses; a peaked distribution or any top-k <= 1024 needs a
// single round.
#include "common.h"

namespace {

constexpr int NT = 1024;
constexpr int CAP = 1024;  // candidates sorted per round

struct SampleArgs {
  const void* logits;
  int ldl, V, valid;
  float temperature, top_p;
  int top_k;
  const float* u;
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
  float wred[16];
  int wredi[16];
  float fscan[NT];
  int iscan[NT];
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
  for (int i = 1; i < 16; ++i) r = fmaxf(r, s.wred[i]);
  return r;
}

// Sum in a fixed order: butterfly inside each wave, then the 16 wave sums left to right.
__device__ __forceinline__ float block_sum(float v, Smem& s) {
  v = wave_sum(v);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) s.wred[w] = v;
  __syncthreads();
  float r = s.wred[0];
#pragma unroll
  for (int i = 1; i < 16; ++i) r += s.wred[i];
  return r;
}

__device__ __forceinline__ int block_sum_i(int v, Smem& s) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) s.wredi[w] = v;
  __syncthreads();
  int r = 0;
#pragma unroll
  for (int i = 0; i < 16; ++i) r += s.wredi[i];
  return r;
}

// Exclusive prefix sum of one int per thread, in thread order.  Returns the total.
// Wave-level shuffle scan, then the 16 wave totals.
__device__ __forceinline__ int block_excl_scan_i(int v, int& excl, Smem& s) {
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  int incl = v;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int t = __shfl_up(incl, o, WAVE);
    if (lane >= o) incl += t;
  }
  __syncthreads();
  if (lane == 63) s.wredi[w] = incl;
  __syncthreads();
  int before = 0, total = 0;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int t = s.wredi[i];
    if (i < w) before += t;
    total += t;
  }
  excl = before + incl - v;
  return total;
}

// The `want`-th largest key (1-based) among the keys for which live(i) holds; returns the
// key and the number of live keys strictly greater than it.
template <int EPT, typename LiveFn, typename KeyFn>
__device__ uint32_t radix_select(int want, int& n_greater, Smem& s, LiveFn live, KeyFn key) {
  uint32_t prefix = 0, mask = 0;
  int above = 0;
  for (int shift = 24; shift >= 0; shift -= 8) {
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
__device__ uint32_t select_small(int want, int& n_greater, Smem& s, LiveFn live, KeyFn key) {
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

template <typename T, int EPT>
__global__ __launch_bounds__(NT) void sample_kernel(SampleArgs a) {
  __shared__ Smem s;
  const int b = blockIdx.x, tid = threadIdx.x;
  const int V = a.V, nvalid = min(a.valid, V);
  const int base = tid * EPT;
  float x[EPT];
  const float temp = a.temperature;
#pragma unroll
  for (int i = 0; i < EPT; ++i) {
    const int id = base + i;
    x[i] = id < nvalid ? load_logit<T>(a.logits, (size_t)b * a.ldl + id) / temp : -INFINITY;
  }
  // ---- top-k: keep x >= k-th largest ---------------------------------------------
  if (a.top_k > 0) {
    const int k = min(a.top_k, V);
    int ngt;
    auto in_vocab = [&](int i) { return base + i < V; };
    auto xkey = [&](int i) { return fkey(x[i]); };  // > 0 for every float but -NaN
    const uint32_t tk = k <= 1024 ? select_small<EPT>(k, ngt, s, in_vocab, xkey) : radix_select<EPT>(k, ngt, s, in_vocab, xkey);
#pragma unroll
    for (int i = 0; i < EPT; ++i)
      if (fkey(x[i]) < tk) x[i] = -INFINITY;
  }
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
  const float u = a.u[b];
  int token = -1;

  if (!(a.top_p > 0.f && a.top_p < 1.f)) {
    // ---- inverse CDF in vocabulary order ------------------------------------------
    float ts = 0.f;
#pragma unroll
    for (int i = 0; i < EPT; ++i) ts += x[i];
    // exclusive scan of the per-thread sums, in thread order
    __syncthreads();
    s.fscan[tid] = ts;
    __syncthreads();
    if (tid == 0) {
      float run = 0.f;
      for (int t = 0; t < NT; ++t) {
        const float v = s.fscan[t];
        s.fscan[t] = run;
        run += v;
      }
      s.fmisc[0] = run;
    }
    __syncthreads();
    const float total = s.fmisc[0];
    const float target = u * total;
    const float lo = s.fscan[tid];
    // last id with p > 0 (fallback when rounding pushes target past the end)
    int lastpos = -1;
#pragma unroll
    for (int i = 0; i < EPT; ++i)
      if (x[i] > 0.f) lastpos = base + i;
    int mx = lastpos;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = max(mx, __shfl_xor(mx, o, WAVE));
    __syncthreads();
    if ((tid & 63) == 0) s.wredi[tid >> 6] = mx;
    __syncthreads();
    int last_id = -1;
#pragma unroll
    for (int i = 0; i < 16; ++i) last_id = max(last_id, s.wredi[i]);
    if (tid == 0) s.misc[2] = 0x7fffffff;
    __syncthreads();
    int found = 0x7fffffff;
    if (target >= lo && ts > 0.f) {
      float run = lo;
#pragma unroll
      for (int i = 0; i < EPT; ++i) {
        run += x[i];
        if (x[i] > 0.f && run > target && found == 0x7fffffff) found = base + i;
      }
    }
    if (found != 0x7fffffff) atomicMin(&s.misc[2], found);
    __syncthreads();
    token = s.misc[2] == 0x7fffffff ? max(last_id, 0) : s.misc[2];
  } else {
    // ---- nucleus: sorted prefix, CAP candidates per round --------------------------
    // live(i): probability > 0 and not yet extracted
    uint32_t taken[(EPT + 31) / 32];
#pragma unroll
    for (int w = 0; w < (EPT + 31) / 32; ++w) taken[w] = 0;
    if (tid == 0) s.misc[4] = -1;
    int my_live = 0;
#pragma unroll
    for (int i = 0; i < EPT; ++i) my_live += x[i] > 0.f ? 1 : 0;
    const int C = block_sum_i(my_live, s);
    // pass 0 finds the kept mass S; pass 1 finds the token at u * S
    float S = 0.f;
    for (int pass = 0; pass < 2 && token < 0; ++pass) {
#pragma unroll
      for (int w = 0; w < (EPT + 31) / 32; ++w) taken[w] = 0;
      int remaining = C;
      float cum = 0.f;       // mass before the current round, as the sequential fp32 sum
      bool done = false;
      while (!done && remaining > 0) {
        const int take = min(remaining, CAP);
        auto live = [&](int i) { return x[i] > 0.f && !((taken[i >> 5] >> (i & 31)) & 1u); };
        auto key = [&](int i) { return __float_as_uint(x[i]); };  // p > 0: bits are monotone
        int ngt = 0;
        uint32_t tk = 0;
        if (take < remaining) tk = select_small<EPT>(take, ngt, s, live, key);
        // ordered compaction: all keys > tk, then ties at tk in id order until `take`
        int c_gt = 0, c_eq = 0;
#pragma unroll
        for (int i = 0; i < EPT; ++i)
          if (live(i)) {
            const uint32_t k = key(i);
            if (take == remaining || k > tk) ++c_gt;
            else if (k == tk) ++c_eq;
          }
        int off_gt, off_eq;
        const int tot_gt = block_excl_scan_i(c_gt, off_gt, s);
        block_excl_scan_i(c_eq, off_eq, s);
        const int room_eq = take - tot_gt;
#pragma unroll
        for (int i = 0; i < EPT; ++i)
          if (live(i)) {
            const uint32_t k = key(i);
            int slot = -1;
            if (take == remaining || k > tk) slot = off_gt++;
            else if (k == tk) {
              if (off_eq < room_eq) slot = tot_gt + off_eq;
              ++off_eq;
            }
            if (slot >= 0) {
              s.skey[slot] = k;
              s.sid[slot] = base + i;
              taken[i >> 5] |= 1u << (i & 31);
            }
          }
        __syncthreads();
        int n2 = 64;  // sort length: the power of two that holds this round's candidates
        while (n2 < take) n2 <<= 1;
        for (int i = take + tid; i < n2; i += NT) {
          s.skey[i] = 0;  // padding sorts last
          s.sid[i] = 0x7fffffff;
        }
        __syncthreads();
        // bitonic sort, descending by key, ascending by id among equal keys
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
        // sequential fp32 scan of the sorted block
        if (tid == 0) {
          float run = cum;
          int stop = 0, tok = -1;
          if (pass == 0) {
            float kept = S;
            for (int j = 0; j < take; ++j) {
              const float p = __uint_as_float(s.skey[j]);
              if (run > a.top_p) {  // mass before this token already exceeds top_p: dropped, and all after
                stop = 1;
                break;
              }
              kept += p;
              run += p;
            }
            S = kept;
            s.fmisc[1] = S;
            if (cum == 0.f && (stop || remaining == take)) {
              // the whole kept set sits in this sorted block: draw from it now, no second pass
              const float target = u * S;
              float r2 = 0.f;
              int last = -1;
              for (int j = 0; j < take; ++j) {
                const float p = __uint_as_float(s.skey[j]);
                if (r2 > a.top_p) break;
                r2 += p;
                last = s.sid[j];
                if (r2 > target) {
                  tok = s.sid[j];
                  break;
                }
              }
              if (tok < 0) tok = max(last, 0);  // rounding pushed the target past the end: last kept id
              stop = 1;
            }
          } else {
            const float target = u * S;
            int last = -1;
            for (int j = 0; j < take; ++j) {
              const float p = __uint_as_float(s.skey[j]);
              if (run > a.top_p) {
                stop = 1;
                break;
              }
              run += p;
              last = s.sid[j];
              if (run > target) {
                tok = s.sid[j];
                stop = 1;
                break;
              }
            }
            if (tok < 0 && (stop || remaining - take == 0) && last >= 0) tok = last;  // rounding: last kept id
            if (tok < 0 && stop) tok = s.misc[4];                                    // boundary fell between rounds
            if (last >= 0) s.misc[4] = last;
          }
          s.fmisc[0] = run;
          s.misc[2] = stop;
          s.misc[3] = tok;
        }
        __syncthreads();
        cum = s.fmisc[0];
        S = s.fmisc[1];
        done = s.misc[2] != 0;
        if (s.misc[3] >= 0) token = s.misc[3];
        remaining -= take;
        __syncthreads();
      }
      if (pass == 1 && token < 0) token = max(s.misc[4], 0);
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

}  // namespace

extern "C" int ohara_sample_topk_topp(const void* logits, int logits_are_fp32, int ldl, int batch, int vocab,
                                      int valid_vocab, float temperature, int top_k, float top_p, const float* u,
                                      int64_t* out_ids, int64_t* history, int hist_cap, int32_t* step_state,
                                      void* stream) {
  if (!logits || !u || !out_ids || batch < 1 || vocab < 1 || ldl < vocab) return OHARA_EINVAL;
  if (!(temperature > 0.f) || top_k < 0 || !(top_p >= 0.f && top_p <= 1.f)) return OHARA_EINVAL;
  SampleArgs a{};
  a.logits = logits; a.ldl = ldl; a.V = vocab; a.valid = valid_vocab > 0 ? valid_vocab : vocab;
  a.temperature = temperature; a.top_p = top_p; a.top_k = top_k; a.u = u; a.out = out_ids;
  a.history = history; a.hist_cap = hist_cap; a.step_state = step_state; a.B = batch;
  return logits_are_fp32 ? launch_sample<float>(a, (hipStream_t)stream) : launch_sample<bf16_t>(a, (hipStream_t)stream);
}
