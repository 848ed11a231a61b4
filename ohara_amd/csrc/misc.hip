// Small memory-bound kernels of the decode step: embedding gather, standalone
// RMSNorm, greedy token selection and the device-side step bookkeeping.
#include "common.h"

namespace {

// out[t, :] = table[ids[t], :]   (nn.Embedding, ohara/models/llama.py:245,310)
__global__ __launch_bounds__(256) void embed_kernel(const int64_t* ids, const bf16_t* table, bf16_t* out, int d,
                                                    int vocab) {
  const int t = blockIdx.x;
  int64_t id = ids[t];
  if (id < 0 || id >= vocab) id = 0;  // the host validates ids; never read out of bounds
  const bf16_t* src = table + (size_t)id * d;
  bf16_t* dst = out + (size_t)t * d;
  if ((d & 7) == 0) {
    for (int i = threadIdx.x; i < d / 8; i += blockDim.x)
      reinterpret_cast<uint4*>(dst)[i] = reinterpret_cast<const uint4*>(src)[i];
  } else {
    for (int i = threadIdx.x; i < d; i += blockDim.x) dst[i] = src[i];
  }
}

// ohara/modules/norm.py:16-21, one workgroup per row.
__global__ __launch_bounds__(256) void rmsnorm_kernel(const bf16_t* x, const bf16_t* w, bf16_t* out, int d,
                                                      float eps) {
  const size_t r = blockIdx.x;
  const bf16_t* xr = x + r * d;
  __shared__ float red[4];
  float s = 0.f;
  for (int i = threadIdx.x; i < d; i += 256) {
    const float v = bf2f(xr[i]);
    s += v * v;
  }
  s = wave_sum(s);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
  __syncthreads();
  const float tot = ((red[0] + red[1]) + red[2]) + red[3];
  const float rinv = 1.0f / sqrtf(tot / (float)d + eps);
  for (int i = threadIdx.x; i < d; i += 256) out[r * d + i] = f2bf(rbf(bf2f(xr[i]) * rinv) * bf2f(w[i]));
}

struct StepState {  // device-resident bookkeeping of a decode loop
  int32_t pos;      // cache position of the token being fed
  int32_t step;     // index of the token being produced
  int32_t done;     // workgroups of the selection kernel that have finished
  int32_t pad;
};

// Greedy selection: first index of the row maximum over the valid vocabulary
// (argmax of the last position, ohara/chat_engine.py:61-63, ohara/inference.py:40-45;
// padded ids masked as in chat_engine.py:398-399).  One workgroup per row.
// Writes next_ids[b] (fed back to the embedding) and, when `history` is given,
// history[step * B + b].  The last workgroup to finish advances pos and step.
__global__ __launch_bounds__(1024) void argmax_kernel(const bf16_t* logits, int ldl, int vocab, int valid,
                                                      int64_t* next_ids, int64_t* history, int hist_cap,
                                                      StepState* st, int B) {
  const int b = blockIdx.x;
  const bf16_t* row = logits + (size_t)b * ldl;
  const int n = min(valid, vocab);
  float best = -INFINITY;
  int bi = 0x7fffffff;
  auto take = [&](float v, int i) {
    if (v > best || (v == best && i < bi)) {
      best = v;
      bi = i;
    }
  };
  if (((ldl & 7) == 0) && ((reinterpret_cast<uintptr_t>(logits) & 15) == 0)) {
    // 16-byte loads, four in flight per thread
    const int n8 = n >> 3;
    for (int c0 = threadIdx.x; c0 < n8; c0 += 4 * 1024) {
      uint4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int c = c0 + u * 1024;
        v[u] = c < n8 ? ldg16(row + (size_t)c * 8) : make_uint4(0xff80ff80u, 0xff80ff80u, 0xff80ff80u, 0xff80ff80u);  // -inf
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int i0 = (c0 + u * 1024) * 8;
        const uint32_t w[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          take(lo_bf(w[j]), i0 + 2 * j);
          take(hi_bf(w[j]), i0 + 2 * j + 1);
        }
      }
    }
    for (int i = (n8 << 3) + threadIdx.x; i < n; i += 1024) take(bf2f(row[i]), i);
  } else {
    for (int i = threadIdx.x; i < n; i += 1024) take(bf2f(row[i]), i);
  }
  // NaN-free comparison network; ties resolve to the lowest index
  lane_xor_argmax<32>(best, bi);
  lane_xor_argmax<16>(best, bi);
  lane_xor_argmax<8>(best, bi);
  lane_xor_argmax<4>(best, bi);
  lane_xor_argmax<2>(best, bi);
  lane_xor_argmax<1>(best, bi);
  __shared__ float sv[16];
  __shared__ int si[16];
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) {
    sv[wave] = best;
    si[wave] = bi;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 16; ++w)
      if (sv[w] > best || (sv[w] == best && si[w] < bi)) {
        best = sv[w];
        bi = si[w];
      }
    if (bi == 0x7fffffff) bi = 0;  // all -inf / NaN row
    next_ids[b] = bi;
    if (st) {
      const int step = st->step;
      if (history && step < hist_cap) history[(size_t)step * B + b] = bi;
      // only the counter is shared between workgroups: no fence, the ids are read by later kernels
      const int old = __hip_atomic_fetch_add(&st->done, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (old == B - 1) {
        st->done = 0;
        st->pos += 1;
        st->step = step + 1;
      }
    }
  }
}

}  // namespace

namespace {
__global__ void advance_positions_kernel(int32_t* seq_pos, const uint8_t* active, int batch, int by) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b < batch && (!active || active[b])) seq_pos[b] += by;
}
// the same, and the ids the next step feeds: what the step selected for an active sequence, 0 for an idle slot
__global__ void advance_ragged_kernel(int32_t* seq_pos, const uint8_t* active, const int64_t* new_ids, int64_t* next_ids,
                                      int batch, int by) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= batch) return;
  const bool on = !active || active[b];
  if (on) seq_pos[b] += by;
  next_ids[b] = on ? new_ids[b] : 0;
}
}  // namespace

extern "C" {

int ohara_abi_version(void) { return 1; }

int ohara_embed_bf16(const int64_t* ids, const uint16_t* table, uint16_t* out, int n_tokens, int d, int vocab,
                     void* stream) {
  if (!ids || !table || !out || n_tokens < 1 || d < 1 || vocab < 1) return OHARA_EINVAL;
  hipLaunchKernelGGL(embed_kernel, dim3(n_tokens), dim3(256), 0, (hipStream_t)stream, ids, table, out, d, vocab);
  return ohara_launch_status();
}

int ohara_rmsnorm_bf16(const uint16_t* x, const uint16_t* w, uint16_t* out, int rows, int d, float eps,
                       void* stream) {
  if (!x || !w || !out || rows < 1 || d < 1) return OHARA_EINVAL;
  hipLaunchKernelGGL(rmsnorm_kernel, dim3(rows), dim3(256), 0, (hipStream_t)stream, x, w, out, d, eps);
  return ohara_launch_status();
}

int ohara_argmax_bf16(const uint16_t* logits, int ldl, int batch, int vocab, int valid_vocab, int64_t* next_ids,
                      int64_t* history, int hist_cap, int32_t* step_state, void* stream) {
  if (!logits || !next_ids || batch < 1 || vocab < 1 || valid_vocab < 1 || ldl < vocab) return OHARA_EINVAL;
  hipLaunchKernelGGL(argmax_kernel, dim3(batch), dim3(1024), 0, (hipStream_t)stream, logits, ldl, vocab,
                     valid_vocab, next_ids, history, hist_cap, reinterpret_cast<StepState*>(step_state), batch);
  return ohara_launch_status();
}

}  // extern "C"

extern "C" int ohara_advance_positions(int32_t* seq_pos, const uint8_t* active, int batch, int by, void* stream) {
  if (!seq_pos || batch < 1) return OHARA_EINVAL;
  hipLaunchKernelGGL(advance_positions_kernel, dim3((batch + 255) / 256), dim3(256), 0, (hipStream_t)stream, seq_pos,
                     active, batch, by);
  return ohara_launch_status();
}

extern "C" int ohara_advance_ragged(int32_t* seq_pos, const uint8_t* active, const int64_t* new_ids, int64_t* next_ids,
                                    int batch, int by, void* stream) {
  if (!seq_pos || !new_ids || !next_ids || batch < 1) return OHARA_EINVAL;
  hipLaunchKernelGGL(advance_ragged_kernel, dim3((batch + 255) / 256), dim3(256), 0, (hipStream_t)stream, seq_pos,
                     active, new_ids, next_ids, batch, by);
  return ohara_launch_status();
}
