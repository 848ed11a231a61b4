// Causal attention over the KV cache for many query positions per sequence (prefill), on MFMA.
//
// Query s of sequence b sits at cache position pos + s and sees positions [0, pos + s]
// (ohara/models/llama.py:100-135: the cache mask key_pos <= start_pos + q_idx :109-113, GQA head
// mapping of repeat_interleave :101-103 by indexing, scale 1/sqrt(Dh), softmax in fp32).
//
// A workgroup (4 waves) owns 128 consecutive queries of one (sequence, head); a wave owns 32 of
// them (two 16-query blocks).  Keys/values are walked in tiles of 64 positions:
//   S^T = K Q^T   v_mfma_f32_16x16x32_bf16, A = K tile rows from LDS, B = Q rows held in
//                 registers for the whole walk; a lane ends up with 16 scores of ONE query
//                 (its column), so the row max/sum need two cross-lane steps only;
//   O^T += V^T P  the probabilities go from the score accumulators straight into the B operand
//                 (the k-slot -> position mapping is chosen so that no lane exchange is needed);
//                 V is transposed on its way into LDS so that the A operand (8 positions of one
//                 column) is two 8-byte reads.
// The running max / sum / rescale are the usual online softmax; probabilities are rounded to
// bf16 for the second product, sums are kept in fp32.
#include "common.h"

namespace {

struct PrefillArgs {
  const bf16_t* q;   // (B*S, H*D)
  const bf16_t* k;   // (Bcap, Tmax, Hkv, D)
  const bf16_t* v;
  bf16_t* out;       // (B*S, H*D)
  int B, S, H, Hkv, Tmax, pos;
  int nqb;           // query blocks (of 128 or 64) per sequence
  float scale_log2e;
};

template <int D, int QW>  // QW: blocks of 16 queries per wave (2: 128 queries per workgroup, 1: 64)
__global__ __launch_bounds__(256, 2) void attn_prefill_kernel(PrefillArgs a) {
  constexpr int QB = 64 * QW, KT = 64;
  constexpr int NK = D / 32;   // k-steps of the score product
  constexpr int ND = D / 16;   // 16-column blocks of the output
  constexpr int LDK = D + 8;   // K tile row stride (elements): 16-byte reads without bank conflicts
  constexpr int LDV = KT + 4;  // V^T row stride (elements)
  constexpr int RPT = KT * D / 8 / 256;  // 16-byte pieces of a tile per thread (K and V each)
  constexpr int GP = RPT >= 4 ? 4 : 2;   // positions a thread transposes together
  __shared__ __align__(16) bf16_t Ks[KT][LDK];
  __shared__ __align__(16) bf16_t Vt[D][LDV];
  // A column's 64 positions are rotated by four positions per group of eight columns (GP == 4): the sixteen
  // threads that transpose one position group write columns eight apart, which would land on two banks.
  auto vt_off = [](int col, int p) { return GP == 4 ? ((p + 4 * (col >> 3)) & (KT - 1)) : p; };

  // heavy (late) query blocks first
  const int qblk = a.nqb - 1 - (int)blockIdx.x;
  const int h = blockIdx.y, b = blockIdx.z;
  const int kvh = h / (a.H / a.Hkv);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int m = lane & 15, g = lane >> 4;
  const int q0 = qblk * QB;                       // first query of the workgroup
  const int wq0 = q0 + wave * 16 * QW;            // first query of the wave
  const size_t row = (size_t)a.Hkv * D;
  const bf16_t* kb = a.k + (size_t)b * a.Tmax * row + (size_t)kvh * D;
  const bf16_t* vb = a.v + (size_t)b * a.Tmax * row + (size_t)kvh * D;
  const int Lall = a.pos + a.S;                   // cached positions that exist
  const int kv_end = min(a.pos + q0 + QB, Lall);  // positions any query of the workgroup sees

  // Q fragments: lane (n = query within block, g) holds Q[q][32 j + 8 g .. +7]
  uint4 qf[QW][NK];
  int qpos[QW];
#pragma unroll
  for (int qb = 0; qb < QW; ++qb) {
    const int qi = wq0 + qb * 16 + m;
    qpos[qb] = qi < a.S ? a.pos + qi : 0x3fffffff;  // rows past the end: never masked, never stored
#pragma unroll
    for (int j = 0; j < NK; ++j)
      qf[qb][j] = qi < a.S ? ldg16(a.q + ((size_t)b * a.S + qi) * a.H * D + (size_t)h * D + 32 * j + 8 * g)
                           : make_uint4(0, 0, 0, 0);
  }
  const int wave_last = min(a.pos + wq0 + 16 * QW - 1, Lall - 1);  // last position any query of the wave sees

  f32x4 o[QW][ND];
  float m_run[QW], l_run[QW];
#pragma unroll
  for (int qb = 0; qb < QW; ++qb) {
    m_run[qb] = -INFINITY;
    l_run[qb] = 0.f;
#pragma unroll
    for (int db = 0; db < ND; ++db) o[qb][db] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }

  // tile loaders.  K: thread (r = tid / (D/8) + i * (256 / (D/8)), c = tid % (D/8)) one 16-byte
  // piece.  V: thread (kq = tid / (D/8), c) takes rows 4 kq' .. with kq' = kq + i * (256/(D/8))
  constexpr int CPR = D / 8;         // 16-byte pieces per row
  constexpr int RPP = 256 / CPR;     // rows per pass
  const int lr = tid / CPR, lc = tid % CPR;
  uint4 kr[RPT], vr[RPT];
  auto load_tile = [&](int t0) {
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      const int p = t0 + lr + i * RPP;
      kr[i] = p < Lall ? ldg16(kb + (size_t)p * row + lc * 8) : make_uint4(0, 0, 0, 0);
    }
    // V: GP consecutive positions per thread and group, so that the transposed write is wide
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
      const int p = t0 + GP * (lr + (i / GP) * RPP) + (i % GP);
      vr[i] = p < Lall ? ldg16(vb + (size_t)p * row + lc * 8) : make_uint4(0, 0, 0, 0);
    }
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int i = 0; i < RPT; ++i) *reinterpret_cast<uint4*>(&Ks[lr + i * RPP][lc * 8]) = kr[i];
    // transpose GP positions x 8 columns: per column one write of GP positions
#pragma unroll
    for (int grp = 0; grp < RPT / GP; ++grp) {
      const int p0 = GP * (lr + grp * RPP);
      uint32_t w[GP][4];
#pragma unroll
      for (int r = 0; r < GP; ++r) {
        w[r][0] = vr[GP * grp + r].x; w[r][1] = vr[GP * grp + r].y;
        w[r][2] = vr[GP * grp + r].z; w[r][3] = vr[GP * grp + r].w;
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {  // column pair 2e, 2e+1 of this thread's 8 columns
        const uint32_t lo01 = (w[0][e] & 0xffffu) | (w[1][e] << 16);
        const uint32_t hi01 = (w[0][e] >> 16) | (w[1][e] & 0xffff0000u);
        if (GP == 4) {
          const uint32_t lo23 = (w[GP - 2][e] & 0xffffu) | (w[GP - 1][e] << 16);
          const uint32_t hi23 = (w[GP - 2][e] >> 16) | (w[GP - 1][e] & 0xffff0000u);
          *reinterpret_cast<uint2*>(&Vt[lc * 8 + 2 * e][vt_off(lc * 8 + 2 * e, p0)]) = make_uint2(lo01, lo23);
          *reinterpret_cast<uint2*>(&Vt[lc * 8 + 2 * e + 1][vt_off(lc * 8 + 2 * e + 1, p0)]) = make_uint2(hi01, hi23);
        } else {
          *reinterpret_cast<uint32_t*>(&Vt[lc * 8 + 2 * e][p0]) = lo01;
          *reinterpret_cast<uint32_t*>(&Vt[lc * 8 + 2 * e + 1][p0]) = hi01;
        }
      }
    }
  };

  load_tile(0);
  for (int t0 = 0; t0 < kv_end; t0 += KT) {
    __syncthreads();  // everyone is done reading the previous tile
    store_tile();
    __syncthreads();
    if (t0 + KT < kv_end) load_tile(t0 + KT);  // in flight during the products below
    if (t0 > wave_last) continue;               // wholly masked for this wave (barriers stay uniform)

    // scores: s[kb][qb] = D[16 positions x 16 queries]
    // The K fragments of two 16-position blocks are read from LDS into registers of their own before
    // their products (left to itself the compiler reuses one register quad: read, wait, product,
    // sixteen times per tile, every LDS latency exposed - a quarter of a tile's time).
    constexpr int KBB = QW == 1 ? 1 : 2;  // 16-position blocks whose fragments are read together (registers: three workgroups per CU with QW == 1)
    f32x4 s[4][QW];
#pragma unroll
    for (int kb2 = 0; kb2 < 4; kb2 += KBB) {
      uint4 kf[KBB][NK];
#pragma unroll
      for (int kk = 0; kk < KBB; ++kk)
#pragma unroll
        for (int j = 0; j < NK; ++j) kf[kk][j] = *reinterpret_cast<const uint4*>(&Ks[(kb2 + kk) * 16 + m][32 * j + 8 * g]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int kk = 0; kk < KBB; ++kk) {
        const int kbk = kb2 + kk;
#pragma unroll
        for (int qb = 0; qb < QW; ++qb) s[kbk][qb] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < NK; ++j)
#pragma unroll
          for (int qb = 0; qb < QW; ++qb)
            s[kbk][qb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kf[kk][j]),
                                                                 __builtin_bit_cast(bf16x8, qf[qb][j]), s[kbk][qb], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    // online softmax per query (= per lane column)
    uint4 pf[QW][2];  // [qb][32-position window]: B operand of the second product
#pragma unroll
    for (int qb = 0; qb < QW; ++qb) {
      float tmax = -INFINITY;
      float mul = 1.0f;  // what the stored scores still have to be multiplied with
      if (t0 + KT - 1 > a.pos + wq0) {  // (wave-uniform) the tile reaches past the wave's first query: mask
#pragma unroll
        for (int kbk = 0; kbk < 4; ++kbk)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            float v = s[kbk][qb][i] * a.scale_log2e;
            if (t0 + kbk * 16 + 4 * g + i > qpos[qb]) v = -INFINITY;
            s[kbk][qb][i] = v;
            tmax = fmaxf(tmax, v);
          }
      } else {
#pragma unroll
        for (int kbk = 0; kbk < 4; ++kbk)
#pragma unroll
          for (int i = 0; i < 4; ++i) tmax = fmaxf(tmax, s[kbk][qb][i]);
        tmax *= a.scale_log2e;  // the scale is positive: the maximum of the products is the product of the maximum
        mul = a.scale_log2e;    // and the scaling itself rides in the fused multiply-add of the exponent below
      }
      tmax = lane_xor_max<32>(lane_xor_max<16>(tmax));
      // the running maximum is kept as an integer (log2 units): every rescale is then an exact power of
      // two and the bf16 weights do not depend on which tile raised it (common.h: softmax bookkeeping)
      const float mn = fmaxf(m_run[qb], ceilf(tmax));  // finite: position 0 is visible to every query
      const float corr = pow2_neg_int(m_run[qb] - mn);
      m_run[qb] = mn;
      float ts = 0.f;
      float p[4][4];
#pragma unroll
      for (int kbk = 0; kbk < 4; ++kbk)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          p[kbk][i] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kbk][qb][i], mul, -mn));
          ts += p[kbk][i];
        }
      l_run[qb] = l_run[qb] * corr + ts;  // this lane's share; lanes g = 0..3 are added at the end
      if (__any(corr != 1.0f)) {  // most tiles leave the running maximum of every query of the wave alone
#pragma unroll
        for (int db = 0; db < ND; ++db)
#pragma unroll
          for (int i = 0; i < 4; ++i) o[qb][db][i] *= corr;
      }
      // k-slot 8 g + i of window w  <->  position 32 w + 4 g + i (i < 4), 32 w + 16 + 4 g + i - 4
#pragma unroll
      for (int w = 0; w < 2; ++w)
        pf[qb][w] = make_uint4(pack_bf(p[2 * w][0], p[2 * w][1]), pack_bf(p[2 * w][2], p[2 * w][3]),
                               pack_bf(p[2 * w + 1][0], p[2 * w + 1][1]), pack_bf(p[2 * w + 1][2], p[2 * w + 1][3]));
    }
    // O^T[16 columns x 16 queries] += V^T[16 columns x 32 slots] P[32 slots x 16 queries]
    constexpr int DBB = QW == 1 ? 4 : ND;  // 16-column blocks of V^T whose fragments are read together
#pragma unroll
    for (int w = 0; w < 2; ++w)
#pragma unroll
      for (int d0 = 0; d0 < ND; d0 += DBB) {
        uint2 v0[DBB], v1[DBB];  // all read before the first product, as above
#pragma unroll
        for (int i = 0; i < DBB; ++i) {
          const int db = d0 + i;
          v0[i] = *reinterpret_cast<const uint2*>(&Vt[db * 16 + m][vt_off(db * 16 + m, 32 * w + 4 * g)]);
          v1[i] = *reinterpret_cast<const uint2*>(&Vt[db * 16 + m][vt_off(db * 16 + m, 32 * w + 16 + 4 * g)]);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < DBB; ++i) {
          const uint4 vf = make_uint4(v0[i].x, v0[i].y, v1[i].x, v1[i].y);
#pragma unroll
          for (int qb = 0; qb < QW; ++qb)
            o[qb][d0 + i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, vf),
                                                                    __builtin_bit_cast(bf16x8, pf[qb][w]), o[qb][d0 + i], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
  }

#pragma unroll
  for (int qb = 0; qb < QW; ++qb) {
    const int qi = wq0 + qb * 16 + m;
    float l = l_run[qb];
    l = lane_xor_sum<32>(lane_xor_sum<16>(l));
    if (qi >= a.S) continue;
    const float inv = 1.0f / l;
    bf16_t* dst = a.out + ((size_t)b * a.S + qi) * a.H * D + (size_t)h * D + 4 * g;
#pragma unroll
    for (int db = 0; db < ND; ++db)
      *reinterpret_cast<uint2*>(dst + db * 16) = make_uint2(pack_bf(o[qb][db][0] * inv, o[qb][db][1] * inv),
                                                            pack_bf(o[qb][db][2] * inv, o[qb][db][3] * inv));
  }
}

}  // namespace

extern "C" int ohara_attn_prefill_bf16(const uint16_t* q, const uint16_t* kcache, const uint16_t* vcache, int batch,
                                       int seq_len, int h, int h_kv, int dh, int t_max, int pos, uint16_t* out,
                                       void* stream) {
  if (!q || !kcache || !vcache || !out) return OHARA_EINVAL;
  if (batch < 1 || seq_len < 1 || h < 1 || h_kv < 1 || h % h_kv || t_max < 1) return OHARA_EINVAL;
  if (pos < 0 || pos + seq_len > t_max) return OHARA_EINVAL;
  if (dh != 64 && dh != 128) return OHARA_ESIZE;
  if (batch > 65535 || h > 65535) return OHARA_ESIZE;
  PrefillArgs a{};
  a.q = q; a.k = kcache; a.v = vcache; a.out = out;
  a.B = batch; a.S = seq_len; a.H = h; a.Hkv = h_kv; a.Tmax = t_max; a.pos = pos;
  a.scale_log2e = (1.0f / sqrtf((float)dh)) * OHARA_LOG2E;  // the same constant as the decode kernels'
  // A causal launch lasts as long as its last query block (sixteen tiles at 1024 tokens, twice the
  // average), whatever the other workgroups do.  With fewer than two blocks of 128 queries per CU,
  // blocks of 64 fit three workgroups on a CU and all of them are resident at once (8 x 1024 tokens,
  // 6 heads: 56.1 -> 54.5 us; the tile of the last block, about 2.9 us, stays what bounds the launch).
  static int cus = 0;
  if (!cus) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
      cus = 256;
  }
  const bool small = (int64_t)((seq_len + 127) / 128) * h * batch < 2 * (int64_t)cus;
  a.nqb = small ? (seq_len + 63) / 64 : (seq_len + 127) / 128;
  dim3 grid(a.nqb, h, batch), block(256);
  if (dh == 128) {
    if (small) hipLaunchKernelGGL((attn_prefill_kernel<128, 1>), grid, block, 0, (hipStream_t)stream, a);
    else hipLaunchKernelGGL((attn_prefill_kernel<128, 2>), grid, block, 0, (hipStream_t)stream, a);
  } else {
    if (small) hipLaunchKernelGGL((attn_prefill_kernel<64, 1>), grid, block, 0, (hipStream_t)stream, a);
    else hipLaunchKernelGGL((attn_prefill_kernel<64, 2>), grid, block, 0, (hipStream_t)stream, a);
  }
  return ohara_launch_status();
}
