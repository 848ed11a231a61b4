// Persistent decode kernel: one launch computes a whole decode step (one new token per
// sequence, batch <= 16) of the Llama of ohara/models/llama.py:279-323.
//
// Why: at batch 1 a layer streams only ~19 MB, so a chain of five kernels per layer
// spends its time in launch and drain latency, not in HBM.  Here the whole chip stays
// resident (one workgroup per CU) and walks the same five phases per layer, separated by
// a grid-wide barrier, each phase spreading its work over all workgroups:
//   P1  [embedding] + norm1 + QKV projection + rotary + cache append
//   P2  attention over the cache, split along the context, partial (max,sum,acc) triples
//   P3  merge of the partials + output projection + residual
//   P4  norm2 + gate/up projection + SwiGLU
//   P5  down projection, split along K over four groups of workgroups (fp32 partial sums; the
//       residual add happens where the stream is read next)
// then final norm + vocabulary projection with a running arg-max per workgroup, and the
// selection of the next token.  Rounding points are those of the unfused kernels.
//
// Cross-workgroup data ("mailboxes").  The eight XCDs have private L2s, so a phase's
// outputs must reach memory before the barrier and must not be served from a stale cache
// line after it.  An L2 write-back / invalidate per barrier costs ~1.7 us each on this
// chip - more than the barrier - so instead:
//   * producers write with device-scope (sc1, write-through) stores and wait for their
//     completion before arriving at the barrier;
//   * every mailbox is written ONCE per launch and read only after the barrier that
//     follows it (one buffer per layer and phase), so no cache anywhere can hold an older
//     copy of it within the launch, and consumers use ordinary cached loads - an XCD
//     fetches a line once and its 32 CUs share it;
//   * every 128-byte line of a mailbox is written by exactly one workgroup (strip-blocked
//     layout), so a partially written line is never completed from memory too early.
// The one exception is the KV-cache row appended in this step (its lines are shared by
// several writers): attention reads that single row with device-scope loads.
//
// Batch 1 (the ONE builds): three of the five hand-offs of a layer carry one short row - the q row and
// the new key / value rows (P1 -> P2), the residual stream (P3 -> P4), the activations (P4 -> P5) - and
// go through TAGGED mailboxes that the consumers poll for (persistent.h) instead of a barrier; two grid
// barriers per layer remain (after the attention partials, after the down projection's sums).  The
// weights of P4 and P5 are requested around the first of them, where a workgroup is idle anyway, so that
// no weight load is in flight ahead of a poll (a wave's loads return in order).
//
// Every barrier wait is bounded: a workgroup that spins longer than the limit raises a
// sticky error word and moves on, all later waits return at once, and the grid drains.
#pragma once
#include "persistent.h"

#define OHARA_PROF_SLOTS 1024  // clock samples per workgroup (measurement builds)

namespace ohara_mega {

struct MegaArgs {
  OharaModel m;                 // by value; the layer table is read from layers_dev
  const OharaLayer* layers_dev;
  uint16_t* const* kcache_dev;  // device arrays [n_layers]
  uint16_t* const* vcache_dev;
  float* const* kvstats_dev;    // int8 cache: the layers' statistics records (device array [n_layers]), else null
  int B, valid_vocab, hist_cap, select;
  int ns;                       // context chunks per (sequence, kv head) in this launch, <= OHARA_MEGA_NS
  int blk_x, blk_a;             // bytes per strip block of the x/q and act mailboxes
  int64_t* ids;
  char* xm;        // NL x-mailboxes of xm_stride bytes: the residual stream after each layer's attention block
  char* qm;        // NL q-mailboxes of qm_stride bytes
  char* am;        // NL act-mailboxes of am_stride bytes
  float* pm;       // NL partial mailboxes of pm_stride floats: [b*H + h][chunk][Dh + 32]
  float* dm;       // NL mailboxes of dm_stride floats: partial sums of the down projection (see XParts)
  size_t xm_stride, qm_stride, am_stride, pm_stride, dm_stride;
  float* cand_val; // (nwg, B)
  int* cand_idx;   // (nwg, B)
  bf16_t* logits;  // (B, V)
  int32_t* step_state;  // {pos, step, done, pad}
  int64_t* history;
  char* tg;             // batch 1: two sets of NL blocks of polled mailboxes, tg_stride bytes a block, tg_set bytes a set
  size_t tg_stride, tg_set;
  int tg_n, tg_q, tg_kv, tg_a;  // byte offsets inside a layer's block: stream after the layer | q | new k, v | activations
  int tg_rx, tg_rq, tg_rkv, tg_ra;  // bytes between the sequences' rows of those mailboxes
  unsigned int* bar;    // barrier words, see GridSync
  unsigned long long* prof;  // optional: clock of every workgroup's thread 0 at every phase boundary (OHARA_PROF_SLOTS each)
  int lm_park;  // polled builds: KB of LDS per wave in which a workgroup without a down-projection strip parks vocabulary tiles
  unsigned int spin_limit;
};


// ---------------------------------------------------------------------------------------
// the kernel
// ---------------------------------------------------------------------------------------
// MODE 0: any batch up to 16, a grid barrier between the phases.  MODE 1 and 2: the polled builds (no barrier inside the
// layers) - 1: the batch is a single sequence (the row loops and row masks fold away at compile time), 2: up to eight.
// I8 (polled builds only): the caches hold int8 codes (a.kvstats_dev their statistics records); the attention phase turns
// the tiles it reads into bf16 values and quantises the appended row itself.
// PROFILE: with the phase stamps (measurement builds of the head-dim-128, no-GQA kernels only).
template <int D, int G, int MODE, bool I8 = false, bool PROFILE = false>
__global__ __launch_bounds__(256) void decode_mega_kernel(MegaArgs a) {
  constexpr bool ONE = MODE == 1, POLLED = MODE != 0;
  static_assert(!I8 || POLLED, "the int8 cache is served by the polled builds");
  extern __shared__ __align__(16) unsigned char smem[];
  const OharaModel& m = a.m;
  const int d = m.d_model, H = m.n_heads, Hkv = m.n_kv_heads, F = m.d_ff, V = m.vocab, B = ONE ? 1 : a.B;
  const int kmax = max(d, max(F, H * D));
  const int ldxs = kmax + 8;
  bf16_t* xs = reinterpret_cast<bf16_t*>(smem);
  float* red = reinterpret_cast<float*>(smem + (((size_t)B * ldxs * 2 + 255) & ~(size_t)255));  // 4 KiB
  float* att = red + 1024;                                                                      // (8 + 4*D)*G floats
  // per-layer pointers (6 weights/norms + K and V cache), copied once to LDS so that no phase
  // starts with a chain of dependent global loads
  float* mrg_w = att + (8 + 4 * D) * G;       // B*H*ns chunk weights
  float* mrg_l = mrg_w + ((B * H * attn_merge_width(a.ns) + 1) & ~1);  // B*H*(merge width) chunk weights before it
  unsigned long long* ptab = reinterpret_cast<unsigned long long*>(mrg_l + ((B * H * attn_merge_width(a.ns) + 1) & ~1));
  // (polled builds: the ids of the rows this wave embeds are the first thing requested - their rows are what the first
  // layer's q/k/v workgroups wait for, and a wave's loads return in the order they were issued)
  // (the single-sequence build only: with more rows the registers this holds across the prefetches are spilled)
  EmbedPre<2> emb;
  if constexpr (ONE) embed_request_ids<2>(a.ids, B, emb);
  for (int i = threadIdx.x; i < m.n_layers * 8; i += blockDim.x) {
    const int l = i >> 3, j = i & 7;
    unsigned long long v;
    if (j < 6) v = reinterpret_cast<const unsigned long long*>(a.layers_dev + l)[j];
    else v = reinterpret_cast<const unsigned long long*>(j == 6 ? a.kcache_dev : a.vcache_dev)[l];
    ptab[i] = v;
  }
  unsigned long long* stab = ptab + m.n_layers * 8;  // int8 cache: the layers' statistics records
  if (I8)
    for (int i = threadIdx.x; i < m.n_layers; i += blockDim.x)
      stab[i] = reinterpret_cast<const unsigned long long*>(a.kvstats_dev)[i];
  __syncthreads();

  GridSync gs;
  gs.init(a.bar, gridDim.x, a.spin_limit);
  // batch 1: the number of this launch since the workspace was cleared, the tag of its hand-offs (read once, here: the
  // last workgroup out advances it)
  unsigned int* launches = a.bar + (gs.ng + 12) * 64;
  const unsigned int nth = POLLED ? *launches + 1u : 0u;
  const int pos = a.step_state[0];
  const int step = a.step_state[1];
  const int L = min(pos + 1, m.t_max);
  float best_v = -INFINITY;
  int best_i = 0x7fffffff;
  ProfT<PROFILE> pf((a.prof && threadIdx.x == 0) ? a.prof + (size_t)blockIdx.x * OHARA_PROF_SLOTS : nullptr);

  GemmP qkv{}, prj{}, gu{}, dn{}, lm{};
  qkv.H = H; qkv.Hkv = Hkv; qkv.Dh = D; qkv.Tmax = m.t_max; qkv.pos = pos; qkv.cos = m.cos; qkv.sin = m.sin;
  qkv.N = (H + 2 * Hkv) * D; qkv.K = d; qkv.nstrips = (qkv.N + 15) / 16; qkv.blk = a.blk_x;
  prj.N = d; prj.K = H * D; prj.nstrips = (d + 15) / 16; prj.blk = a.blk_x;
  prj.ids = a.ids; prj.table = m.token_emb; prj.vocab = V;
  gu.N = F; gu.K = d; gu.nstrips = 2 * ((F + 7) / 8 * 8) / 16; gu.blk = a.blk_a;
  dn.N = d; dn.K = F; dn.nstrips = (d + 15) / 16;
  lm.N = V; lm.K = d; lm.nstrips = (V + 15) / 16; lm.out = reinterpret_cast<char*>(a.logits); lm.ldo = V;
  lm.valid = a.valid_vocab > 0 ? min(a.valid_vocab, V) : V;
  lm.wp = reinterpret_cast<const uint4*>(m.w_vocab);
  lm.norm_w = m.final_norm;

  GemmPre pre;
  AttnPre<D> apre;
  qkv.wp = lds_ptr<const uint4>(ptab, 0);
  qkv.norm_w = lds_ptr<const bf16_t>(ptab, 4);
  // The polled builds (batch 1, and up to eight sequences); the host launches them only on a grid wide enough for
  // gate/up and the down projection (and the output projection and the down projection) to sit on different
  // workgroups, and the general build otherwise.
  uint32_t lm_staged_addr = 0;  // batch 1: where this wave's second vocabulary strip is parked in LDS (0: nowhere)
  bool lm_extra = false;        // ... followed by the first half of its third strip
  if constexpr (POLLED) {
   {
    // ---- polled hand-offs, no grid barrier inside the layers ------------------------------------------
    const Poll pc{nth, a.spin_limit, gs.err};
    const int nwg = (int)gridDim.x;
    // this launch's set of mailboxes, and the way from there to the other set
    char* const tgs = a.tg + (size_t)(nth & 1u) * a.tg_set;
    qkv.tother = prj.tother = gu.tother = dn.tother = (nth & 1u) ? -(ptrdiff_t)a.tg_set : (ptrdiff_t)a.tg_set;
    qkv.poll = prj.poll = gu.poll = dn.poll = pc;
    // Who does what.  Every phase is a handful of units, and what a unit costs is the fetch of its weights
    // (a CU takes in ~55 GB/s) - so the phases are spread over the grid such that a workgroup's next
    // weights can be on their way while it has nothing else to do, long before the poll that precedes
    // their use (a wave's loads return in order: a poll issued behind a batch of weights comes back after
    // it).  Attention chunks, the output projection and gate/up start at workgroup 0; q/k/v sits at the far
    // end; the down projection (whole K per strip: 24 k-step tiles per wave from LDS, no partial sums)
    // follows the output projection, clear of the workgroups that the next layer starts on.
    dn.nstrips = (d + 15) / 16;
    qkv.wg0 = max(0, nwg - qkv.nstrips);
    dn.wg0 = prj.nstrips + dn.nstrips <= nwg ? prj.nstrips : max(0, nwg - dn.nstrips);
    const int n_chunks = B * Hkv * a.ns;
    const bool has_attn = (int)blockIdx.x < n_chunks;
    const bool has_dn = phase_block(dn) < dn.nstrips;
    const bool has_qkv = phase_block(qkv) < qkv.nstrips;
    qkv.kv_i8 = I8;  // (the attention phase quantises the appended row itself)
    // ahead of the first layer: gate/up and output projection weights, the first K/V tile, q/k/v weights
    // (q/k/v last: its prefetch leaves norm1's weights in pre.g and the rotary pair in pre.r)
    prj.tout = tgs;  // (marks the polled mode for the prefetch: the residual is fetched by the phase itself)
    gu.wp = lds_ptr<const uint4>(ptab, 2); gu.norm_w = lds_ptr<const bf16_t>(ptab, 5);
    uint4 g1[2], g2[2];  // norm1's and norm2's weights, the rotary pair: each prefetch writes its own
    uint2 r1, r_unused;
    if constexpr (ONE) {
      if (has_qkv) embed_request_rows<2>(m.token_emb, V, d, emb);  // (ahead of the weights: see above)
    }
    gemm_prefetch<2, 12, E_SWIGLU, 6>(gu, pre, B, g2, r_unused);
    prj.wp = lds_ptr<const uint4>(ptab, 1);
    gemm_prefetch<4, 6, E_RESID, 18>(prj, pre, B, g2, r_unused);
    gemm_prefetch<4, 6, E_ROPE>(qkv, pre, B, g1, r1);
    char* wl = reinterpret_cast<char*>(((uintptr_t)(stab + m.n_layers) + 255) & ~(uintptr_t)255);  // 4 x OHARA_LDS_PF KB
    dn.wlds_addr = (uint32_t)(uintptr_t)(OHARA_LDS char*)wl;
    pf.stamp();
    // The vocabulary projection is the one long stream of the step (100 MB at d12) and the layers leave the memory
    // system idle: a workgroup without a down-projection strip parks the tiles of each wave's second vocabulary strip
    // in the LDS that the down projection's workgroups use for their weights, a few tiles per layer, requested where
    // the workgroup has nothing to wait for soon.
    const int KSL = (lm.K + 31) >> 5;
    const int lm_strip1 = (nwg + (int)blockIdx.x) * 4 + (int)(threadIdx.x >> 6);
    const bool lm_staged = !has_dn && KSL <= OHARA_LDS_PF && lm_strip1 < lm.nstrips && 2 * nwg * 4 <= lm.nstrips;
    // (where the LDS allows it, the first half of the wave's third strip follows the second strip)
    const int lm_strip2 = lm_strip1 + nwg * 4;
    if constexpr (ONE && !I8 && !PROFILE) lm_extra = lm_staged && KSL == 24 && a.lm_park >= KSL + 12 && 3 * nwg * 4 <= lm.nstrips;
    const int lm_tiles = KSL + (lm_extra ? 12 : 0);
    const int lm_per = (lm_tiles + m.n_layers - 1) / m.n_layers;
    const int lm_park = ONE ? a.lm_park : OHARA_LDS_PF;
    if (lm_staged) lm_staged_addr = dn.wlds_addr + (uint32_t)(threadIdx.x >> 6) * (uint32_t)lm_park * 1024;
    for (int l = 0; l < m.n_layers; ++l) {
      auto lm_stage = [&]() {
        if (!lm_staged) return;
        const int c0 = l * lm_per, c1 = min(lm_tiles, c0 + lm_per);
        char* dst = wl + ((size_t)(threadIdx.x >> 6) * lm_park + c0) * 1024;
#pragma unroll 1
        for (int c = c0; c < c1; ++c) {  // tile c of the second strip, then (a single sequence) tile c - KSL of the third
          const bool third = ONE && !I8 && !PROFILE && c >= KSL;
          const uint4* src = lm.wp + ((size_t)(third ? lm_strip2 : lm_strip1) * KSL + (third ? c - KSL : c)) * 64 + (threadIdx.x & 63);
          __builtin_amdgcn_global_load_lds((const OHARA_GLOBAL void*)src, (OHARA_LDS void*)dst, 16, 0, 0);
          dst += 1024;
        }
      };
      const unsigned long long* pl = ptab + l * 8;
      bf16_t* kc = lds_ptr<bf16_t>(pl, 6);
      bf16_t* vc = lds_ptr<bf16_t>(pl, 7);
      float* p_l = a.pm + (size_t)l * a.pm_stride;
      char* xt = tgs + (size_t)l * a.tg_stride;    // the stream after the attention block
      char* xn = xt + a.tg_n;                       // the stream after the layer
      char* qt = xt + a.tg_q;
      char* kvt = xt + a.tg_kv;
      char* at = xt + a.tg_a;
      const char* xn_prev = xn - a.tg_stride;       // (l > 0)
      const bool more = l + 1 < m.n_layers;
      // the first K/V tile of this workgroup's attention chunk (the attention workgroups have no q/k/v strip: nothing
      // of theirs is polled for until q is)
      if (has_attn && !I8) attn_prefetch<D>(B, Hkv, m.t_max, a.ns, kc, vc, L, apre);
      // P1: [embedding | poll for the stream] + norm1 + QKV + rotary + append; q and the new k / v rows are left tagged
      qkv.kc = kc; qkv.vc = vc; qkv.out = nullptr; qkv.tout = qt; qkv.tkv = kvt; qkv.trow = a.tg_rq; qkv.tkv_row = a.tg_rkv;
      if (has_qkv) {
        if (l == 0) stage_norm<2, true, true, false, ONE>(xs, ldxs, a.xm, 0, nullptr, a.ids, m.token_emb, V, lds_ptr<const bf16_t>(pl, 4), m.eps, B, d, g1, emb);
        else stage_norm_tagged<2>(xs, xn_prev, pc, m.eps, d, g1, B, ldxs, a.tg_rx);
      }
      __syncthreads();
      pf.stamp();  // 1: row polled for + norm1 in LDS
      pre.r = r1;
      gemm_phase<4, 6, E_ROPE, ProfT<PROFILE>, 0, true>(qkv, pre, xs, ldxs, B, red, best_v, best_i, pf);  // 2 stamps
      pf.stamp();  // 4: rotary epilogue, tagged stores issued
      // P2: attention partials (polls for q; the chunk that holds the new position polls for its k / v rows); each chunk
      // leaves the launch's tag behind its (max, sum) pair
      attn_phase<D, G, true, I8, ONE>(B, H, Hkv, m.t_max, a.blk_x, a.ns, apre, nullptr, p_l, kc, vc, L, att, qt, kvt, pc, true,
                                 a.tg_rq, a.tg_rkv, I8 ? lds_ptr<float>(stab, l) : nullptr, red);
      pf.stamp();  // 5: partials stored, flag raised
      // the next layer's q/k/v weights (+ norm1's, the rotary pair): their registers are free again (behind the attention
      // phase, which needs many: a workgroup without a chunk - at the usual sizes those with q/k/v strips - is here at once)
      if (has_qkv && more) {
        qkv.wp = lds_ptr<const uint4>(pl, 8);
        qkv.norm_w = lds_ptr<const bf16_t>(pl, 12);
        gemm_prefetch<4, 6, E_ROPE, 0, false>(qkv, pre, B, g1, r1);  // (the rotary pair is the same in every layer)
      }
      if (has_qkv) lm_stage();  // (the next thing a q/k/v workgroup polls for is a phase or more away)
      // the down projection's weights (98 KB a workgroup) into LDS: on their way from here, used after P4
      dn.wp = lds_ptr<const uint4>(pl, 3); dn.tout = xn; dn.tresid = xt; dn.trow = dn.tres_row = a.tg_rx;
      if (has_dn) {
        // (not before the chunk's flag has reached memory: behind the other waves' 72 KB of requests it was seen 1.5 us late)
        if (has_attn) {
          wait_own_stores();
          __syncthreads();
        }
        gemm_prefetch_lds<4, E_XNEXT>(dn, wl);
      }
      pf.stamp();  // 6: requests issued
      // P3: polls for every chunk's tag; merge + output projection + residual
      prj.tout = xt; prj.tresid = l > 0 ? xn_prev : nullptr; prj.resid_embed = l == 0; prj.trow = prj.tres_row = a.tg_rx;
      if ((int)blockIdx.x < prj.nstrips) stage_attn_merge_any<!ONE, true>(a.ns, xs, ldxs, p_l, B, H, D, mrg_w, mrg_l, pc);
      __syncthreads();
      pf.stamp();  // 7: merge in LDS
      gemm_phase<4, 6, E_RESID, ProfT<PROFILE>, 18, true>(prj, pre, xs, ldxs, B, red, best_v, best_i, pf);  // 2 stamps
      pf.stamp();  // 10: residual epilogue
      // P4: polls for the stream, norm2 + gate/up + SwiGLU; the activations are left tagged
      gu.out = nullptr; gu.tout = at; gu.trow = a.tg_ra;
      if (phase_block(gu) * 2 < gu.nstrips) stage_norm_tagged<2>(xs, xt, pc, m.eps, d, g2, B, ldxs, a.tg_rx);
      __syncthreads();
      pf.stamp();  // 11: stream polled for + norm2 in LDS
      gemm_phase<2, 12, E_SWIGLU, ProfT<PROFILE>, 6, true>(gu, pre, xs, ldxs, B, red, best_v, best_i, pf);  // 2 stamps
      // What the next layer needs of this workgroup besides q/k/v is requested now, a phase and a half before its use:
      // output projection and gate/up weights (+ norm2's); after the last layer, the vocabulary projection's first tiles.
      // (the workgroups of the down projection do this after it: the wait for their LDS tiles would wait for these too)
      auto next_weights = [&]() {
        if (more) {
          gu.wp = lds_ptr<const uint4>(pl, 10); gu.norm_w = lds_ptr<const bf16_t>(pl, 13);
          gemm_prefetch<2, 12, E_SWIGLU, 6>(gu, pre, B, g2, r_unused);
          prj.wp = lds_ptr<const uint4>(pl, 9);
          gemm_prefetch<4, 6, E_RESID, 18>(prj, pre, B, g2, r_unused);
        } else {
          gemm_prefetch<1, 24, E_LOGITS>(lm, pre, B);  // (+ the final norm's weights)
        }
      };
      pf.stamp();  // SwiGLU epilogue
      if (!has_dn) next_weights();
      pf.stamp();  // next layer's weights requested
      // P5: polls for the activations, down projection + residual; the stream is left tagged
      if (has_dn) stage_act_tagged(xs, at, pc, 0, F, B, ldxs, a.tg_ra);
      __syncthreads();
      pf.stamp();  // 15: activations polled for, in LDS
      gemm_phase<4, 12, E_XNEXT, ProfT<PROFILE>, 0, true>(dn, pre, xs, ldxs, B, red, best_v, best_i, pf);  // 2 stamps
      pf.stamp();  // x_next stored
      if (has_dn) next_weights();
      if (!has_qkv) lm_stage();
      pf.stamp();  // next layer's weights requested
    }
    // final norm + vocabulary projection: the stream of the last layer is polled for like any other
    pf.stamp();
    stage_norm_tagged<2>(xs, tgs + (size_t)(m.n_layers - 1) * a.tg_stride + a.tg_n, pc, m.eps, d, pre.g, B, ldxs, a.tg_rx);
    __syncthreads();
    pf.stamp();
    pf.stamp();
   }
  }
  if constexpr (!POLLED) {
  gemm_prefetch<4, 6, E_ROPE>(qkv, pre, B);
  pf.stamp();
  for (int l = 0; l < m.n_layers; ++l) {
    const unsigned long long* pl = ptab + l * 8;
    bf16_t* kc = lds_ptr<bf16_t>(pl, 6);
    bf16_t* vc = lds_ptr<bf16_t>(pl, 7);
    char* x_mid = a.xm + (size_t)l * a.xm_stride;                  // after attention
    // the stream entering layer l > 0 is x_mid of layer l - 1 plus that layer's down-projection sums
    const char* x_prev = a.xm + (size_t)(l > 0 ? l - 1 : 0) * a.xm_stride;
    const float* d_prev = l > 0 ? a.dm + (size_t)(l - 1) * a.dm_stride : nullptr;
    float* d_l = a.dm + (size_t)l * a.dm_stride;
    char* q_l = a.qm + (size_t)l * a.qm_stride;
    char* a_l = a.am + (size_t)l * a.am_stride;
    float* p_l = a.pm + (size_t)l * a.pm_stride;
    // P1: [embedding] + norm1 + QKV + rotary + append
    qkv.kc = kc; qkv.vc = vc; qkv.out = q_l;
    if ((int)blockIdx.x < qkv.nstrips) {
      if (l == 0) stage_norm<2, true, true, false>(xs, ldxs, a.xm, 0, nullptr, a.ids, m.token_emb, V, lds_ptr<const bf16_t>(pl, 4), m.eps, B, d, pre.g);
      else stage_norm<2, false, true, true>(xs, ldxs, x_prev, a.blk_x, d_prev, a.ids, m.token_emb, V, lds_ptr<const bf16_t>(pl, 4), m.eps, B, d, pre.g);
    }
    __syncthreads();
    pf.stamp();
    gemm_phase<4, 6, E_ROPE>(qkv, pre, xs, ldxs, B, red, best_v, best_i, pf);
    pf.stamp();
    gs.arrive(pf);
    attn_prefetch<D>(B, Hkv, m.t_max, a.ns, kc, vc, L, apre);
    gs.wait(pf);
    pf.stamp();
    // P2: attention partials
    attn_phase<D, G>(B, H, Hkv, m.t_max, a.blk_x, a.ns, apre, q_l, p_l, kc, vc, L, att);
    gs.arrive(pf);
    prj.wp = lds_ptr<const uint4>(pl, 1); prj.out = x_mid; prj.resid = x_prev; prj.resid_parts = d_prev;
    prj.resid_embed = l == 0;
    gemm_prefetch<4, 6, E_RESID>(prj, pre, B);
    gs.wait(pf);
    pf.stamp();
    // P3: merge + output projection + residual
    if ((int)blockIdx.x < prj.nstrips) {
      stage_attn_merge_any<true>(a.ns, xs, ldxs, p_l, B, H, D, mrg_w, mrg_l);
    }
    __syncthreads();
    pf.stamp();
    gemm_phase<4, 6, E_RESID>(prj, pre, xs, ldxs, B, red, best_v, best_i, pf);
    pf.stamp();
    gs.arrive(pf);
    gu.wp = lds_ptr<const uint4>(pl, 2); gu.out = a_l; gu.norm_w = lds_ptr<const bf16_t>(pl, 5);
    gemm_prefetch<2, 12, E_SWIGLU>(gu, pre, B);
    gs.wait(pf);
    pf.stamp();
    // P4: norm2 + gate/up + SwiGLU
    if ((int)blockIdx.x * 2 < gu.nstrips) stage_norm<2, false, true, false>(xs, ldxs, x_mid, a.blk_x, nullptr, a.ids, m.token_emb, V, lds_ptr<const bf16_t>(pl, 5), m.eps, B, d, pre.g);
    __syncthreads();
    gemm_phase<2, 12, E_SWIGLU>(gu, pre, xs, ldxs, B, red, best_v, best_i, pf);
    gs.arrive(pf);
    dn.wp = lds_ptr<const uint4>(pl, 3); dn.pout = d_l;
    gemm_prefetch<4, 6, E_PART>(dn, pre, B);
    gs.wait(pf);
    pf.stamp();
    // P5: down projection, K split over OHARA_DOWN_SPLIT groups of workgroups; a workgroup stages
    // only the columns of its partition (all of them when it will take more than one unit)
    {
      const int nunits = dn.nstrips * OHARA_DOWN_SPLIT;
      if ((int)blockIdx.x < nunits) {
        const int KSq = (((F + 31) >> 5) + OHARA_DOWN_SPLIT - 1) / OHARA_DOWN_SPLIT;
        const int kq = (int)blockIdx.x / dn.nstrips;
        const bool whole = nunits > (int)gridDim.x;
        stage_act(xs, ldxs, a_l, a.blk_a, B, whole ? 0 : min(F, kq * KSq * 32), whole ? F : min(F, (kq + 1) * KSq * 32));
      }
    }
    __syncthreads();
    gemm_phase<4, 6, E_PART>(dn, pre, xs, ldxs, B, red, best_v, best_i, pf);
    gs.arrive(pf);
    // (the last layer leaves the loop here: with both prefetches behind one if / else the compiler
    // waited for the vocabulary projection's 24 tiles at the join, before the barrier wait)
    if (l + 1 == m.n_layers) break;
    qkv.wp = lds_ptr<const uint4>(pl, 8);
    qkv.norm_w = lds_ptr<const bf16_t>(pl, 12);
    gemm_prefetch<4, 6, E_ROPE>(qkv, pre, B);
    gs.wait(pf);
    pf.stamp();
  }
  gemm_prefetch<1, 24, E_LOGITS>(lm, pre, B);
  gs.wait(pf);
  pf.stamp();
  // final norm + vocabulary projection, running arg-max per lane
  stage_norm<2, false, true, true>(xs, ldxs, a.xm + (size_t)(m.n_layers - 1) * a.xm_stride, a.blk_x,
                             a.dm + (size_t)(m.n_layers - 1) * a.dm_stride, a.ids, m.token_emb, V, m.final_norm, m.eps, B, d,
                             pre.g);
  __syncthreads();
  }
  lm_phase(lm, pre, xs, ldxs, B, best_v, best_i, pf, lm_staged_addr, ONE && !I8 && !PROFILE && lm_extra);
  pf.stamp();
  if (a.select) {
    // lanes with the same batch column (lane & 15) fold their candidates; then the waves
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int o = 16; o < 64; o <<= 1) {
      const float ov = __shfl_xor(best_v, o, WAVE);
      const int oi = __shfl_xor(best_i, o, WAVE);
      if (ov > best_v || (ov == best_v && oi < best_i)) {
        best_v = ov;
        best_i = oi;
      }
    }
    __syncthreads();
    float* cv = red;
    int* ci = reinterpret_cast<int*>(red + 64);
    if (lane < 16) {
      cv[wave * 16 + lane] = best_v;
      ci[wave * 16 + lane] = best_i;
    }
    __syncthreads();
    if (threadIdx.x < B) {
      float bv = cv[threadIdx.x];
      int bi = ci[threadIdx.x];
      for (int w = 1; w < 4; ++w) {
        const float ov = cv[w * 16 + threadIdx.x];
        const int oi = ci[w * 16 + threadIdx.x];
        if (ov > bv || (ov == bv && oi < bi)) {
          bv = ov;
          bi = oi;
        }
      }
      st_coh4(a.cand_val + (size_t)blockIdx.x * B + threadIdx.x, __float_as_uint(bv));
      st_coh4(a.cand_idx + (size_t)blockIdx.x * B + threadIdx.x, (uint32_t)bi);
    }
    gs.arrive(pf);
    gs.wait(pf);
    if (blockIdx.x == 0) {
      // one wave per sequence (round robin): reduce the per-workgroup candidates
      for (int b = wave; b < B; b += 4) {
        float bv = -INFINITY;
        int bi = 0x7fffffff;
        for (int w = lane; w < (int)gridDim.x; w += 64) {
          const float ov = __uint_as_float(ld_coh4(a.cand_val + (size_t)w * B + b));
          const int oi = (int)ld_coh4(a.cand_idx + (size_t)w * B + b);
          if (ov > bv || (ov == bv && oi < bi)) {
            bv = ov;
            bi = oi;
          }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
          const float ov = __shfl_xor(bv, o, WAVE);
          const int oi = __shfl_xor(bi, o, WAVE);
          if (ov > bv || (ov == bv && oi < bi)) {
            bv = ov;
            bi = oi;
          }
        }
        if (lane == 0) {
          if (bi == 0x7fffffff) bi = 0;
          a.ids[b] = bi;
          if (a.history && step < a.hist_cap) a.history[(size_t)step * B + b] = bi;
        }
      }
    }
  }
  pf.stamp();
  if constexpr (POLLED) {
    // bookkeeping by the last workgroup out (the batch-1 layers have no barrier that everyone has passed, and without the
    // selection there is none at all): nobody reads these again in this launch
    if (threadIdx.x == 0) {
      const unsigned int out = __hip_atomic_fetch_add(a.bar + (gs.ng + 13) * 64, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (out + 1u == nth * gs.nwg) {
        *launches = nth;
        *gs.done = gs.k - 1;
        if (a.select) {
          a.step_state[0] = pos + 1;
          a.step_state[1] = step + 1;
        }
      }
    }
  } else {
  // bookkeeping by workgroup 0: everyone is past the last barrier, nobody reads these again
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    *gs.done = gs.k - 1;
    if (a.select) {
      a.step_state[0] = pos + 1;
      a.step_state[1] = step + 1;
    }
  }
  }
}

// One launch of an instantiation: raises the LDS limit where needed, refuses a grid whose workgroups cannot all be
// resident (a hand-off would never arrive), launches.
template <typename K>
int mega_launch(K kernel, ResidencySlot& slot, const MegaArgs& a, size_t smem, int n_workgroups, hipStream_t st) {
  if (smem > 64 * 1024)
    (void)hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
  if (!ohara_grid_fits(slot, (const void*)kernel, smem, n_workgroups)) return OHARA_ESIZE;
  hipLaunchKernelGGL(kernel, dim3(n_workgroups), dim3(256), smem, st, a);
  return OHARA_OK;
}

// the polled builds over an int8 cache (mega_i8.hip); mode 1 or 2
int mega_launch_i8(const MegaArgs& a, int D, int G, int mode, size_t smem, int n_workgroups, hipStream_t st);

}  // namespace ohara_mega
