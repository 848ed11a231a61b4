// Tiled MFMA GEMM for the batched (prefill) projections: y = epi(x W^T) with many rows.
//
// A workgroup (4 waves) owns a tile of 128 activation rows x 128 packed weight rows.  Each wave
// owns two 16-row weight strips for all 128 activation rows: 16 accumulators of
// v_mfma_f32_16x16x32_bf16 (weights = A operand, activations = B operand, exactly as in the
// skinny kernel, so the epilogues are shared).  Per 64-deep k-step
//   * the weights of a wave's strips come straight from the packed layout into registers
//     (one contiguous 1 KiB per wave-load, no duplication between waves, prefetched one
//     step ahead),
//   * the 128 x 64 activation tile is loaded once per workgroup with 128-byte row segments,
//     staged in LDS (rows padded to 144 B: conflict-free 16-byte reads) and double-buffered,
//     so one barrier per step suffices.
// Workgroup ids are remapped so that all weight tiles of one activation tile run on the same
// XCD (ids round-robin over the 8 XCDs): the activation tile is then fetched into one L2 only,
// while the weights (a few MB) live in every L2.
//
// Replaces the F.linear calls of ohara/models/llama.py:84-86,142,322 and
// ohara/modules/mlp.py:152 when the call carries more than 64 rows.
#include "gemm_epilogue.h"

namespace {

constexpr int TM = 128;        // activation rows per tile
constexpr int TS = 8;          // weight strips per tile (128 packed rows)
constexpr int KB = 64;         // k per step
constexpr int LDX = KB + 8;    // LDS row stride in elements (144 B)

template <int EPI>
__global__ __launch_bounds__(256, 2) void gemm_tile_kernel(GemmArgs a, int MT, int NT, int nstrips) {
  __shared__ __align__(16) bf16_t xs[2][TM][LDX];
  const int id = blockIdx.x;
  const int xcd = id & 7, q = id >> 3;
  const int tn = q % NT;
  const int tm = (q / NT) * 8 + xcd;
  if (tm >= MT) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m = lane & 15, g = lane >> 4;
  const int row0 = tm * TM;
  const int strip0 = tn * TS + wave * 2;
  const int KS = (a.K + 31) >> 5;
  const int nsteps = (KS + 1) >> 1;

  // activation tile loader: 8 threads x 16 B per row, 32 rows per pass, 4 passes
  const int lr = tid >> 3, lc = (tid & 7) * 8;
  auto load_x = [&](int step, uint4* xr) {
    const int k = step * KB + lc;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const int r = row0 + p * 32 + lr;
      xr[p] = (r < a.B && k < a.K) ? ldg16(a.x + (size_t)r * a.ldx + k) : make_uint4(0, 0, 0, 0);
    }
  };
  auto store_x = [&](int buf, const uint4* xr) {
#pragma unroll
    for (int p = 0; p < 4; ++p) *reinterpret_cast<uint4*>(&xs[buf][p * 32 + lr][lc]) = xr[p];
  };
  const uint4* w0 = a.wp + (size_t)strip0 * KS * 64 + lane;
  const uint4* w1 = w0 + (size_t)KS * 64;
  const bool live0 = strip0 < nstrips, live1 = strip0 + 1 < nstrips;
  auto load_w = [&](int step, uint4* wv) {
    const int j = step * 2;
    wv[0] = (live0 && j < KS) ? ldg16(w0 + (size_t)j * 64) : make_uint4(0, 0, 0, 0);
    wv[1] = (live0 && j + 1 < KS) ? ldg16(w0 + (size_t)(j + 1) * 64) : make_uint4(0, 0, 0, 0);
    wv[2] = (live1 && j < KS) ? ldg16(w1 + (size_t)j * 64) : make_uint4(0, 0, 0, 0);
    wv[3] = (live1 && j + 1 < KS) ? ldg16(w1 + (size_t)(j + 1) * 64) : make_uint4(0, 0, 0, 0);
  };

  f32x4 acc[2][8];
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int t = 0; t < 8; ++t) acc[u][t] = (f32x4){0.f, 0.f, 0.f, 0.f};

  uint4 xr[4], wv[4], wn[4];
  load_x(0, xr);
  load_w(0, wv);
  store_x(0, xr);
  __syncthreads();
  for (int s = 0; s < nsteps; ++s) {
    const int buf = s & 1;
    const bool more = s + 1 < nsteps;
    if (more) {
      load_x(s + 1, xr);
      load_w(s + 1, wn);
    }
    // The eight B operands of a half step are read from LDS into registers of their own before its
    // products.  (Left to itself the compiler reuses one register quad: read, wait, two products,
    // sixteen times per step, every LDS latency exposed.  All sixteen up front would take the
    // kernel from three workgroups per CU to two, which costs more than it gains.)
#pragma unroll
    for (int jj = 0; jj < 2; ++jj) {
      uint4 bv[8];
#pragma unroll
      for (int t = 0; t < 8; ++t) bv[t] = *reinterpret_cast<const uint4*>(&xs[buf][t * 16 + m][jj * 32 + 8 * g]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        acc[0][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wv[jj]),
                                                            __builtin_bit_cast(bf16x8, bv[t]), acc[0][t], 0, 0, 0);
        acc[1][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wv[2 + jj]),
                                                            __builtin_bit_cast(bf16x8, bv[t]), acc[1][t], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if (more) {
      store_x(buf ^ 1, xr);
#pragma unroll
      for (int i = 0; i < 4; ++i) wv[i] = wn[i];
    }
    __syncthreads();
  }

  // A thread finishes sixteen fragments.  What their epilogues read (residual rows, biases, rotary
  // values) is fetched for eight of them before the first is used, instead of one dependent round trip
  // per fragment.
  // Rotary epilogue: position, sequence and cache row depend on the activation row alone (eight per
  // thread, and rows of a tile are consecutive: no division per row when a sequence is at least a tile
  // long), the region (q / k / v) and the feature index inside the head on the strip alone (uniform
  // over the wave).  Worked out per fragment they were 40 % of this kernel's instructions.
  if (EPI == EPI_ROPE && a.S >= TM && ((a.ldo | a.Dh) & 15) == 0 && ((a.H * a.Dh) & 15) == 0 && !a.stage) {
    const int nq = a.H * a.Dh, nk = a.Hkv * a.Dh;
    const int base = a.row0 + row0;                            // global row of the tile's first row
    const int seq0 = base / a.S, rem0 = base - seq0 * a.S;     // uniform over the workgroup
    int pos_t[8];
    size_t qoff_t[8], coff_t[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      const int x = rem0 + t * 16 + m;
      const bool wrap = x >= a.S;
      const int seq = seq0 + (wrap ? 1 : 0), sidx = x - (wrap ? a.S : 0);
      const int grow = base + t * 16 + m;
      pos_t[t] = (a.pos_dev ? a.pos_dev[(size_t)seq * a.pos_stride] : a.pos) + sidx;
      qoff_t[t] = (size_t)grow * a.ldo;
      coff_t[t] = (((size_t)seq * a.Tmax + pos_t[t]) * a.Hkv) * a.Dh;
    }
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int strip = strip0 + u;
      if (strip >= nstrips) continue;
      const int rr = strip * 16;  // uniform: the whole strip lies in one region and one head
      if (rr >= nq + 2 * nk) continue;
      const int region = rr < nq ? 0 : (rr < nq + nk ? 1 : 2);
      const int rloc = rr - (region == 0 ? 0 : (region == 1 ? nq : nq + nk)) + 4 * g;  // column inside q, k or v
      const int d = (rr - (region == 0 ? 0 : nq)) % a.Dh + 4 * g;
      uint32_t cv[8], sv[8];
      if (region < 2) {
#pragma unroll
        for (int t = 0; t < 8; ++t) {
          const int pc = min(max(pos_t[t], 0), a.Tmax - 1);
          cv[t] = *reinterpret_cast<const uint32_t*>(a.cos + (size_t)pc * (a.Dh >> 1) + (d >> 1));
          sv[t] = *reinterpret_cast<const uint32_t*>(a.sin + (size_t)pc * (a.Dh >> 1) + (d >> 1));
        }
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const int b = row0 + t * 16 + m;
        if (b >= a.B || pos_t[t] < 0 || pos_t[t] >= a.Tmax) continue;
        float v[4] = {rbf(acc[u][t][0]), rbf(acc[u][t][1]), rbf(acc[u][t][2]), rbf(acc[u][t][3])};
        if (region < 2) {
#pragma unroll
          for (int pr = 0; pr < 2; ++pr) {
            const float c = pr ? hi_bf(cv[t]) : lo_bf(cv[t]), sn = pr ? hi_bf(sv[t]) : lo_bf(sv[t]);
            const float e = v[2 * pr], od = v[2 * pr + 1];
            // separate fp32 multiplies and add/sub, as the reference's eager ops round
            v[2 * pr] = __fsub_rn(__fmul_rn(e, c), __fmul_rn(od, sn));
            v[2 * pr + 1] = __fadd_rn(__fmul_rn(e, sn), __fmul_rn(od, c));
          }
        }
        bf16_t* o = region == 0 ? a.out + qoff_t[t] + rloc : (region == 1 ? a.kcache : a.vcache) + coff_t[t] + rloc;
        *reinterpret_cast<uint2*>(o) = make_uint2(pack_bf(v[0], v[1]), pack_bf(v[2], v[3]));
      }
    }
    return;
  }
  constexpr bool READS = EPI == EPI_RESIDUAL || EPI == EPI_ROPE || EPI == EPI_BIAS || EPI == EPI_BIAS_GELU ||
                         EPI == EPI_BIAS_ADD2 || EPI == EPI_PHI_IN;
  if (READS && a.N >= 4 && ((a.N | a.ldo | a.ldr | (EPI == EPI_BIAS_ADD2 ? a.ldr2 : 0)) & 3) == 0) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {  // eight fragments at a time: sixteen sets of operands cost a resident workgroup
      EpiPre pre[8];
#pragma unroll
      for (int t = 0; t < 8; ++t) gemm_epilogue_fetch<EPI>(a, row0 + t * 16 + m, min(strip0 + u, nstrips - 1), g, pre[t]);
      __builtin_amdgcn_sched_barrier(0);
      if (strip0 + u >= nstrips) continue;
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const int b = row0 + t * 16 + m;
        if (b < a.B) gemm_epilogue<EPI, true>(a, b, strip0 + u, g, acc[u][t], pre[t]);
      }
    }
    return;
  }
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    if (strip0 + u >= nstrips) continue;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      const int b = row0 + t * 16 + m;
      if (b < a.B) gemm_epilogue<EPI>(a, b, strip0 + u, g, acc[u][t]);
    }
  }
}

}  // namespace

// Launcher shared with the skinny entry points (declared there).
int ohara_launch_gemm_tile(const GemmArgs& a, int epi, int packed_rows, hipStream_t st) {
  const int nstrips = packed_rows / 16;
  const int NT = (nstrips + TS - 1) / TS;
  const int MT = (a.B + TM - 1) / TM;
  const int64_t blocks = (int64_t)((MT + 7) / 8) * 8 * NT;
  if (blocks > INT32_MAX) return OHARA_ESIZE;
  dim3 grid((unsigned)blocks), block(256);
  switch (epi) {
    case EPI_STORE: hipLaunchKernelGGL((gemm_tile_kernel<EPI_STORE>), grid, block, 0, st, a, MT, NT, nstrips); break;
    case EPI_RESIDUAL: hipLaunchKernelGGL((gemm_tile_kernel<EPI_RESIDUAL>), grid, block, 0, st, a, MT, NT, nstrips); break;
    case EPI_SWIGLU: hipLaunchKernelGGL((gemm_tile_kernel<EPI_SWIGLU>), grid, block, 0, st, a, MT, NT, nstrips); break;
    case EPI_ROPE: hipLaunchKernelGGL((gemm_tile_kernel<EPI_ROPE>), grid, block, 0, st, a, MT, NT, nstrips); break;
    case EPI_BIAS: hipLaunchKernelGGL((gemm_tile_kernel<EPI_BIAS>), grid, block, 0, st, a, MT, NT, nstrips); break;
    case EPI_BIAS_GELU: hipLaunchKernelGGL((gemm_tile_kernel<EPI_BIAS_GELU>), grid, block, 0, st, a, MT, NT, nstrips); break;
    case EPI_BIAS_ADD2: hipLaunchKernelGGL((gemm_tile_kernel<EPI_BIAS_ADD2>), grid, block, 0, st, a, MT, NT, nstrips); break;
    case EPI_PHI_IN: hipLaunchKernelGGL((gemm_tile_kernel<EPI_PHI_IN>), grid, block, 0, st, a, MT, NT, nstrips); break;
    default: return OHARA_EINVAL;
  }
  return ohara_launch_status();
}

extern "C" int ohara_gemm_bf16(const uint16_t* x, int ldx, const uint16_t* wp, int n, int k, int rows, int epilogue,
                               const uint16_t* resid, int ldr, uint16_t* out, int ldo, void* stream) {
  if (!x || !wp || !out || n < 1 || k < 1 || rows < 1) return OHARA_EINVAL;
  if ((k & 7) || (ldx & 7) || ldx < k) return OHARA_EINVAL;  // 16-byte activation loads
  if (epilogue == OHARA_EPI_RESIDUAL && (!resid || ldr < n)) return OHARA_EINVAL;
  if (epilogue < OHARA_EPI_STORE || epilogue > OHARA_EPI_SWIGLU) return OHARA_EINVAL;
  if (ldo < n) return OHARA_EINVAL;
  GemmArgs a{};
  a.wp = reinterpret_cast<const uint4*>(wp);
  a.x = x; a.ldx = ldx;
  a.B = rows; a.N = n; a.K = k;
  a.out = out; a.ldo = ldo; a.resid = resid; a.ldr = ldr;
  const int packed_rows = epilogue == OHARA_EPI_SWIGLU ? 2 * ((n + 7) / 8 * 8) : (n + 15) / 16 * 16;
  return ohara_launch_gemm_tile(a, epilogue, packed_rows, (hipStream_t)stream);
}
