// Shared by the skinny (decode) and tiled (prefill) GEMM kernels: argument block and the
// fused epilogues.  Rounding points follow the reference's bf16 eager path:
//   residual add       ohara/models/llama.py:199-200
//   SwiGLU             ohara/modules/mlp.py:152
//   rotary + KV append ohara/embeddings_pos/rotary.py:55-93, ohara/modules/kv_cache.py:104-105
//   bias / new_gelu / parallel-block sum of Phi   ohara/models/phi.py:37-52, :147-151
#pragma once
#include "common.h"

enum { EPI_STORE = 0, EPI_RESIDUAL = 1, EPI_SWIGLU = 2, EPI_ROPE = 3, EPI_BIAS = 4, EPI_BIAS_GELU = 5, EPI_BIAS_ADD2 = 6, EPI_PHI_IN = 7 };

struct GemmArgs {
  const uint4* wp;
  const bf16_t* x;
  int ldx;
  const bf16_t* norm_w;
  float eps;
  int B, N, K;  // rows, logical output width (EPI_SWIGLU: hidden width F) and depth
  bf16_t* out;
  int ldo;
  const bf16_t* resid;
  int ldr;
  // rotary + append
  int H, Hkv, Dh, Tmax, pos;
  int S, row0;  // rows are (sequence, position) pairs: row = seq * S + s, position = pos + s
  int ny, nstrips;  // skinny kernel: 16-row chunks per strip (workgroups of a strip share an XCD) and strips
  const int32_t* pos_dev;
  int pos_stride;  // 0: *pos_dev is the position of every sequence; 1: pos_dev[seq] (ragged batches)
  const bf16_t* cos;
  const bf16_t* sin;
  bf16_t* kcache;
  bf16_t* vcache;
  int stage;  // rotary epilogue: k / v rows go to (rows, Hkv*Dh) buffers at the row index instead of into a cache
  // nn.Linear with bias (EPI_BIAS*): y = bf16(acc + bias[n]); EPI_BIAS_ADD2: bf16(bf16(resid + y) + resid2)
  const bf16_t* bias;
  const bf16_t* resid2;
  int ldr2;
  // LayerNorm prologue (NORM == 2): norm_w / norm_b
  const bf16_t* norm_b;
  // EPI_PHI_IN: packed rows [q; k; v; fc1] off one normalised input (phi.py:81-83, :50): rows below
  // split_n are the QKV projection (q -> out, k / v rows -> cache position pos + s, un-rotated), the
  // rest go through new_gelu into out2
  int split_n;
  bf16_t* out2;
  int ldo2;
};

// gemm_tile.hip: the tiled kernel for calls with many rows (a.B rows, no fused norm).
int ohara_launch_gemm_tile(const GemmArgs& a, int epi, int packed_rows, hipStream_t st);

namespace {

// What an epilogue reads besides the accumulators, fetched ahead: a kernel that finishes many fragments
// per thread (the tiled GEMM: sixteen) issues the loads of all of them before the first is used instead of
// one dependent round trip per fragment.  gemm_epilogue_fetch requires N, ldo, ldr, ldr2 to be multiples
// of 4 (the caller checks once); fragments and rows outside the matrix read clamped addresses and are
// never finished.
struct EpiPre {
  uint2 r1, r2, bv;  // residual rows, bias
  uint32_t c, s;     // two cos and two sin values of the rotary table
  int pos;
};
template <int EPI>
__device__ __forceinline__ void gemm_epilogue_fetch(const GemmArgs& a, int b, int strip, int g, EpiPre& p) {
  const int r0 = min(strip * 16 + 4 * g, a.N - 4);
  const int bc = min(b, a.B - 1);
  if (EPI == EPI_RESIDUAL) p.r1 = *reinterpret_cast<const uint2*>(a.resid + (size_t)bc * a.ldr + r0);
  if (EPI == EPI_BIAS || EPI == EPI_BIAS_GELU || EPI == EPI_BIAS_ADD2 || EPI == EPI_PHI_IN)
    p.bv = *reinterpret_cast<const uint2*>(a.bias + r0);
  if (EPI == EPI_BIAS_ADD2) {
    p.r1 = *reinterpret_cast<const uint2*>(a.resid + (size_t)bc * a.ldr + r0);
    p.r2 = *reinterpret_cast<const uint2*>(a.resid2 + (size_t)bc * a.ldr2 + r0);
  }
  if (EPI == EPI_ROPE) {
    const int grow = a.row0 + bc;
    const int seq = grow / a.S;
    p.pos = (a.pos_dev ? a.pos_dev[(size_t)seq * a.pos_stride] : a.pos) + (grow - seq * a.S);
    const int nq = a.H * a.Dh;
    const int rr = strip * 16 + 4 * g;
    const int d = (rr < nq ? rr : rr - nq) % a.Dh;
    const int pc = min(max(p.pos, 0), a.Tmax - 1);
    p.c = *reinterpret_cast<const uint32_t*>(a.cos + (size_t)pc * (a.Dh >> 1) + (d >> 1));
    p.s = *reinterpret_cast<const uint32_t*>(a.sin + (size_t)pc * (a.Dh >> 1) + (d >> 1));
  }
}

// One MFMA output fragment: the four consecutive packed rows 16*strip + 4*g .. +3 of activation
// row b (relative to a.out / a.resid; global row a.row0 + b for the rotary epilogue).
template <int EPI, bool PRE = false>  // PRE: the operands were fetched ahead into `p`
__device__ __forceinline__ void gemm_epilogue(const GemmArgs& a, int b, int strip, int g, f32x4 acc, const EpiPre& p = EpiPre{}) {
  const int r0 = strip * 16 + 4 * g;
  const float y0 = rbf(acc[0]), y1 = rbf(acc[1]), y2 = rbf(acc[2]), y3 = rbf(acc[3]);
  if (EPI == EPI_STORE || EPI == EPI_RESIDUAL) {
    float v[4] = {y0, y1, y2, y3};
    bf16_t* o = a.out + (size_t)b * a.ldo + r0;
    if (EPI == EPI_RESIDUAL) {
      const bf16_t* r = a.resid + (size_t)b * a.ldr + r0;
      if (r0 + 3 < a.N && ((a.ldr & 3) == 0)) {
        const uint2 rv = PRE ? p.r1 : *reinterpret_cast<const uint2*>(r);
        v[0] = lo_bf(rv.x) + v[0]; v[1] = hi_bf(rv.x) + v[1]; v[2] = lo_bf(rv.y) + v[2]; v[3] = hi_bf(rv.y) + v[3];
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (r0 + i < a.N) v[i] = bf2f(r[i]) + v[i];
      }
    }
    if (r0 + 3 < a.N && ((a.ldo & 3) == 0)) {
      *reinterpret_cast<uint2*>(o) = make_uint2(pack_bf(v[0], v[1]), pack_bf(v[2], v[3]));
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (r0 + i < a.N) o[i] = f2bf(v[i]);
    }
  } else if (EPI == EPI_BIAS || EPI == EPI_BIAS_GELU || EPI == EPI_BIAS_ADD2) {
    // N % 4 == 0 and 4-element aligned leading dimensions are required by the entry point
    if (r0 >= a.N) return;
    const uint2 bv = PRE ? p.bv : *reinterpret_cast<const uint2*>(a.bias + r0);
    float v[4] = {rbf(acc[0] + lo_bf(bv.x)), rbf(acc[1] + hi_bf(bv.x)), rbf(acc[2] + lo_bf(bv.y)),
                  rbf(acc[3] + hi_bf(bv.y))};
    if (EPI == EPI_BIAS_GELU) {
      // phi.py:37-40 op by op, every result rounded as the eager bf16 ops round; torch.pow(x, 3.0)
      // on bf16 is (x * x) * x with both products rounded
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float x = v[i];
        const float t2 = rbf(x + rbf(0.044715f * rbf(rbf(x * x) * x)));
        const float t5 = rbf(1.0f + rbf(tanhf(rbf(0.7978845608028654f * t2))));
        v[i] = rbf(0.5f * x) * t5;
      }
    } else if (EPI == EPI_BIAS_ADD2) {
      const uint2 r1 = PRE ? p.r1 : *reinterpret_cast<const uint2*>(a.resid + (size_t)b * a.ldr + r0);
      const uint2 r2 = PRE ? p.r2 : *reinterpret_cast<const uint2*>(a.resid2 + (size_t)b * a.ldr2 + r0);
      v[0] = rbf(lo_bf(r1.x) + v[0]) + lo_bf(r2.x);
      v[1] = rbf(hi_bf(r1.x) + v[1]) + hi_bf(r2.x);
      v[2] = rbf(lo_bf(r1.y) + v[2]) + lo_bf(r2.y);
      v[3] = rbf(hi_bf(r1.y) + v[3]) + hi_bf(r2.y);
    }
    *reinterpret_cast<uint2*>(a.out + (size_t)b * a.ldo + r0) = make_uint2(pack_bf(v[0], v[1]), pack_bf(v[2], v[3]));
  } else if (EPI == EPI_PHI_IN) {
    if (r0 >= a.N) return;
    const uint2 bv = PRE ? p.bv : *reinterpret_cast<const uint2*>(a.bias + r0);
    float v[4] = {rbf(acc[0] + lo_bf(bv.x)), rbf(acc[1] + hi_bf(bv.x)), rbf(acc[2] + lo_bf(bv.y)),
                  rbf(acc[3] + hi_bf(bv.y))};
    const int grow = a.row0 + b;
    bf16_t* o;
    if (r0 >= a.split_n) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {  // new_gelu as in EPI_BIAS_GELU
        const float x = v[i];
        const float t2 = rbf(x + rbf(0.044715f * rbf(rbf(x * x) * x)));
        const float t5 = rbf(1.0f + rbf(tanhf(rbf(0.7978845608028654f * t2))));
        v[i] = rbf(0.5f * x) * t5;
      }
      o = a.out2 + (size_t)grow * a.ldo2 + (r0 - a.split_n);
    } else {
      const int dm = a.split_n / 3;
      if (r0 < dm) {
        o = a.out + (size_t)grow * a.ldo + r0;
      } else {
        const int seq = grow / a.S;
        const int pos = (a.pos_dev ? *a.pos_dev : a.pos) + (grow - seq * a.S);
        if (pos < 0 || pos >= a.Tmax) return;
        const bool isk = r0 < 2 * dm;
        o = (isk ? a.kcache : a.vcache) + ((size_t)seq * a.Tmax + pos) * dm + (r0 - (isk ? dm : 2 * dm));
      }
    }
    *reinterpret_cast<uint2*>(o) = make_uint2(pack_bf(v[0], v[1]), pack_bf(v[2], v[3]));
  } else if (EPI == EPI_SWIGLU) {
    // rows: gate f, gate f+1, up f, up f+1 with f = 8*strip + 2*g; N = hidden width F
    const int f = strip * 8 + 2 * g;
    const float s0 = rbf(silu_f(y0)), s1 = rbf(silu_f(y1));
    bf16_t* o = a.out + (size_t)b * a.ldo + f;
    if (f + 1 < a.N && ((a.ldo & 1) == 0)) {
      *reinterpret_cast<uint32_t*>(o) = pack_bf(s0 * y2, s1 * y3);
    } else {
      if (f < a.N) o[0] = f2bf(s0 * y2);
      if (f + 1 < a.N) o[1] = f2bf(s1 * y3);
    }
  } else {  // EPI_ROPE: rows [q (H*Dh); k (Hkv*Dh); v (Hkv*Dh)], one position per sequence
    const int grow = a.row0 + b;
    const int seq = grow / a.S;
    const int pos = PRE ? p.pos : (a.pos_dev ? a.pos_dev[(size_t)seq * a.pos_stride] : a.pos) + (grow - seq * a.S);
    const int nq = a.H * a.Dh, nk = a.Hkv * a.Dh;
    if (r0 >= nq + 2 * nk || pos < 0 || pos >= a.Tmax) return;
    float v[4] = {y0, y1, y2, y3};
    bf16_t* o;
    if (r0 < nq + nk) {
      const int d = (r0 < nq ? r0 : r0 - nq) % a.Dh;
      const bf16_t* cs = a.cos + (size_t)pos * (a.Dh >> 1) + (d >> 1);
      const bf16_t* sn = a.sin + (size_t)pos * (a.Dh >> 1) + (d >> 1);
#pragma unroll
      for (int pr = 0; pr < 2; ++pr) {
        const float c = PRE ? (pr ? hi_bf(p.c) : lo_bf(p.c)) : bf2f(cs[pr]), s = PRE ? (pr ? hi_bf(p.s) : lo_bf(p.s)) : bf2f(sn[pr]);
        const float e = v[2 * pr], od = v[2 * pr + 1];
        // separate fp32 multiplies and add/sub, as the reference's eager ops round
        v[2 * pr] = __fsub_rn(__fmul_rn(e, c), __fmul_rn(od, s));
        v[2 * pr + 1] = __fadd_rn(__fmul_rn(e, s), __fmul_rn(od, c));
      }
      if (r0 < nq) {
        o = a.out + (size_t)grow * a.ldo + r0;
      } else {
        o = a.stage ? a.kcache + (size_t)grow * nk + (r0 - nq)
                    : a.kcache + (((size_t)seq * a.Tmax + pos) * a.Hkv) * a.Dh + (r0 - nq);
      }
    } else {
      o = a.stage ? a.vcache + (size_t)grow * nk + (r0 - nq - nk)
                  : a.vcache + (((size_t)seq * a.Tmax + pos) * a.Hkv) * a.Dh + (r0 - nq - nk);
    }
    *reinterpret_cast<uint2*>(o) = make_uint2(pack_bf(v[0], v[1]), pack_bf(v[2], v[3]));
  }
}

}  // namespace
