// The persistent decode kernel's host side: workspace layout, launch planning, the C entry points (the kernel itself:
// mega_kernel.h; its builds over an int8 cache are compiled in mega_i8.hip).
#include "mega_kernel.h"

using namespace ohara_mega;

namespace {

// ---- workspace layout ------------------------------------------------------------------
// (two words behind GridSync's: the launches since the workspace was cleared - the tag of the batch-1 hand-offs - and the
// workgroups that have finished, which tells the last one out that it is the one to advance the launch count)
#define OHARA_BAR_WORDS(nwg) ((((nwg) + OHARA_BAR_GROUP - 1) / OHARA_BAR_GROUP + 14) * 64)

size_t mega_al(size_t v) { return (v + 255) & ~(size_t)255; }

struct MegaLayout {
  size_t layers, kptr, vptr, sptr, xm, qm, am, pm, dm, candv, candi, prof, bar, tg, total;
  size_t xm_stride, qm_stride, am_stride, pm_stride, dm_stride, tg_stride, tg_set;
  int blk_x, blk_a, tg_n, tg_q, tg_kv, tg_a, tg_rx, tg_rq, tg_rkv, tg_ra;
};

MegaLayout mega_layout(const OharaModel* m, int B, int nwg) {
  MegaLayout L{};
  const int NL = m->n_layers, D = m->head_dim;
  L.blk_x = (B * 32 + 127) / 128 * 128;
  L.blk_a = (B * 16 + 127) / 128 * 128;
  const int nq_rows = (m->n_heads + 2 * m->n_kv_heads) * D;
  L.xm_stride = mega_al((size_t)((m->d_model + 15) / 16) * L.blk_x);
  L.qm_stride = mega_al((size_t)((nq_rows + 15) / 16) * L.blk_x);
  L.am_stride = mega_al((size_t)((m->d_ff + 7) / 8) * L.blk_a);
  L.pm_stride = mega_al((size_t)B * m->n_heads * OHARA_MEGA_NS * (D + 32) * sizeof(float)) / sizeof(float);
  size_t o = 0;
  L.layers = o; o += mega_al(sizeof(OharaLayer) * NL);
  L.kptr = o; o += mega_al(sizeof(void*) * NL);
  L.vptr = o; o += mega_al(sizeof(void*) * NL);
  L.sptr = o; o += mega_al(sizeof(void*) * NL);
  L.xm = o; o += L.xm_stride * NL;
  L.qm = o; o += L.qm_stride * NL;
  L.am = o; o += L.am_stride * NL;
  L.dm_stride = mega_al((size_t)OHARA_DOWN_SPLIT * ((m->d_model + 15) / 16) * ((B * 64 + 127) / 128 * 128)) / sizeof(float);
  L.dm = o; o += L.dm_stride * sizeof(float) * NL;
  L.candv = o; o += mega_al((size_t)nwg * B * sizeof(float));
  L.candi = o; o += mega_al((size_t)nwg * B * sizeof(int));
  L.prof = o; o += mega_al((size_t)nwg * OHARA_PROF_SLOTS * sizeof(unsigned long long));
  L.bar = o; o += mega_al(OHARA_BAR_WORDS(nwg) * sizeof(unsigned int));
  // behind the barrier words, cleared with them: the attention partials (batch 1: a tag follows each (max, sum) pair);
  // then the two sets of polled mailboxes (batch 1), filled with 0xFF ("not written yet")
  L.pm = o; o += L.pm_stride * sizeof(float) * NL;
  L.tg_rx = (int)mega_al((size_t)m->d_model * 2);
  L.tg_rq = (int)mega_al((size_t)m->n_heads * D * 2);
  L.tg_rkv = (int)mega_al((size_t)2 * m->n_kv_heads * D * 2);
  L.tg_ra = (int)mega_al((size_t)((m->d_ff + 7) / 8 * 8) * 2);
  const int PB = B <= 8 ? B : 1;  // (the polled builds serve up to eight sequences)
  L.tg_n = PB * L.tg_rx;
  L.tg_q = 2 * L.tg_n;
  L.tg_kv = L.tg_q + PB * L.tg_rq;
  L.tg_a = L.tg_kv + PB * L.tg_rkv;
  L.tg_stride = L.tg_a + (size_t)PB * L.tg_ra;
  L.tg_set = L.tg_stride * NL;
  L.tg = o; o += 2 * L.tg_set;
  L.total = o;
  return L;
}

// What a launch looks like for (model, batch, grid): chunks per (sequence, KV head), which build, its LDS bytes.
struct MegaPlan {
  int ns, mode;
  size_t smem;
  int lm_park;  // KB of LDS per wave for parked vocabulary tiles (polled builds)
};

MegaPlan mega_plan(const OharaModel* m, int batch, int n_workgroups) {
  const int D = m->head_dim, G = m->n_heads / m->n_kv_heads;
  const int kmax = m->d_model > m->d_ff ? m->d_model : m->d_ff;
  const int kmax2 = kmax > m->n_heads * D ? kmax : m->n_heads * D;
  const size_t xs_bytes = ((size_t)batch * (kmax2 + 8) * 2 + 255) & ~(size_t)255;
  // one attention item per workgroup where the batch allows it
  int ns = n_workgroups / (batch * m->n_kv_heads);
  ns = ns < 1 ? 1 : (ns > OHARA_MEGA_NS ? OHARA_MEGA_NS : ns);
  // A power of two unless the exact count keeps at least half as many workgroups again busy and its
  // merge stays narrow (the merge reads the next power of two of chunk slots): 7 chunks of 36 pairs
  // instead of 4 took batch 6 from 0.397 to 0.379 ms per step, 5 instead of 4 at batch 8 lost what the
  // attention phase gained to the wider merge.
  int p2 = ns;
  while (p2 & (p2 - 1)) p2 &= p2 - 1;
  if (!(2 * ns >= 3 * p2 && attn_merge_width(ns) <= 8)) ns = p2;
  const size_t mrg = (size_t)2 * ((batch * m->n_heads * attn_merge_width(ns) + 1) & ~1) * sizeof(float);
  // The polled builds (batch 1; up to eight sequences) park the down projection's tiles in LDS (4 waves x
  // OHARA_LDS_PF KB) and want gate/up, the output projection and the down projection on workgroups of their own.
  const int n_dn = (m->d_model + 15) / 16, n_gu = (2 * ((m->d_ff + 7) / 8 * 8) / 16 + 1) / 2;
  const size_t smem0 = xs_bytes + 4096 + (size_t)(8 + 4 * D) * G * sizeof(float) + mrg + (size_t)m->n_layers * 72;
  const size_t smem_polled = smem0 + 256 + (size_t)4 * OHARA_LDS_PF * 1024;
  const bool roles = n_gu + n_dn <= n_workgroups && 2 * n_dn <= n_workgroups;
  const int mode = !roles ? 0 : (batch == 1 ? 1 : (batch <= 8 && smem_polled <= 160 * 1024 ? 2 : 0));
  // A single sequence leaves LDS free: the workgroups that park their waves' second vocabulary strip add half of the
  // third (12 more tiles per wave) where that fits.
  const size_t smem_more = smem0 + 256 + (size_t)4 * (OHARA_LDS_PF + 12) * 1024;
  if (mode == 1 && smem_more <= 160 * 1024) return MegaPlan{ns, 1, smem_more, OHARA_LDS_PF + 12};
  return MegaPlan{ns, mode, mode ? smem_polled : smem0, OHARA_LDS_PF};
}

}  // namespace

extern "C" {

int64_t ohara_persistent_workspace_bytes(const OharaModel* m, int batch, int n_split, int n_workgroups) {
  if (!m || batch < 1 || n_split != OHARA_MEGA_NS || n_workgroups < 1) return OHARA_EINVAL;
  return (int64_t)mega_layout(m, batch, n_workgroups).total;
}

int64_t ohara_persistent_barrier_offset(const OharaModel* m, int batch, int n_split, int n_workgroups) {
  if (!m || batch < 1 || n_split != OHARA_MEGA_NS || n_workgroups < 1) return OHARA_EINVAL;
  return (int64_t)mega_layout(m, batch, n_workgroups).bar;
}

int64_t ohara_persistent_error_offset(const OharaModel* m, int batch, int n_split, int n_workgroups) {
  const int64_t b = ohara_persistent_barrier_offset(m, batch, n_split, n_workgroups);
  const int ng = (n_workgroups + OHARA_BAR_GROUP - 1) / OHARA_BAR_GROUP;
  return b < 0 ? b : b + (int64_t)(ng + 2) * 64 * 4;
}

int64_t ohara_persistent_profile_offset(const OharaModel* m, int batch, int n_split, int n_workgroups) {
  if (!m || batch < 1 || n_split != OHARA_MEGA_NS || n_workgroups < 1) return OHARA_EINVAL;
  return (int64_t)mega_layout(m, batch, n_workgroups).prof;
}

int ohara_persistent_polled(const OharaModel* m, int batch, int n_workgroups) {
  if (!m || batch < 1 || batch > 16 || n_workgroups < 1 || m->n_kv_heads < 1 || m->n_heads % m->n_kv_heads) return OHARA_EINVAL;
  return mega_plan(m, batch, n_workgroups).mode;
}

int ohara_llama_decode_persistent(const OharaModel* m, const OharaDecodeState* s, void* workspace, int n_workgroups,
                                  int init_workspace, int select_greedy, unsigned int spin_limit, void* stream) {
  if (!m || !s || !workspace || !m->layers || !s->kcache || !s->vcache || !s->step_state) return OHARA_EINVAL;
  if (s->batch < 1 || s->batch > 16) return OHARA_ESIZE;
  if (n_workgroups < 1 || n_workgroups > 1024) return OHARA_EINVAL;
  if (s->n_split != OHARA_MEGA_NS) return OHARA_EINVAL;
  const int D = m->head_dim, G = m->n_heads / m->n_kv_heads;
  if (!(D == 128 || D == 64) || !(G == 1 || G == 2 || G == 4) || m->n_heads % m->n_kv_heads) return OHARA_ESIZE;
  if ((m->d_model & 7) || (m->d_ff & 7) || m->d_model > 1024) return OHARA_ESIZE;
  hipStream_t st = (hipStream_t)stream;
  char* ws = reinterpret_cast<char*>(workspace);
  const MegaLayout L = mega_layout(m, s->batch, n_workgroups);
  MegaArgs a{};
  a.m = *m;
  a.layers_dev = reinterpret_cast<const OharaLayer*>(ws + L.layers);
  a.kcache_dev = reinterpret_cast<uint16_t* const*>(ws + L.kptr);
  a.vcache_dev = reinterpret_cast<uint16_t* const*>(ws + L.vptr);
  if (s->kv_int8 && !s->kvstats) return OHARA_EINVAL;
  a.kvstats_dev = s->kv_int8 ? reinterpret_cast<float* const*>(ws + L.sptr) : nullptr;
  a.xm = ws + L.xm; a.qm = ws + L.qm; a.am = ws + L.am; a.pm = reinterpret_cast<float*>(ws + L.pm);
  a.xm_stride = L.xm_stride; a.qm_stride = L.qm_stride; a.am_stride = L.am_stride; a.pm_stride = L.pm_stride;
  a.dm = reinterpret_cast<float*>(ws + L.dm); a.dm_stride = L.dm_stride;
  a.blk_x = L.blk_x; a.blk_a = L.blk_a;
  a.cand_val = reinterpret_cast<float*>(ws + L.candv);
  a.cand_idx = reinterpret_cast<int*>(ws + L.candi);
  a.bar = reinterpret_cast<unsigned int*>(ws + L.bar);
  a.tg = ws + L.tg; a.tg_stride = L.tg_stride; a.tg_set = L.tg_set; a.tg_n = L.tg_n; a.tg_q = L.tg_q; a.tg_kv = L.tg_kv; a.tg_a = L.tg_a;
  a.tg_rx = L.tg_rx; a.tg_rq = L.tg_rq; a.tg_rkv = L.tg_rkv; a.tg_ra = L.tg_ra;
  if (init_workspace) {
    // small synchronous copies: done once per (model, cache) binding, outside any capture
    if (hipMemcpyAsync((void*)a.layers_dev, m->layers, sizeof(OharaLayer) * m->n_layers, hipMemcpyHostToDevice, st) !=
            hipSuccess ||
        hipMemcpyAsync((void*)a.kcache_dev, s->kcache, sizeof(void*) * m->n_layers, hipMemcpyHostToDevice, st) !=
            hipSuccess ||
        hipMemcpyAsync((void*)a.vcache_dev, s->vcache, sizeof(void*) * m->n_layers, hipMemcpyHostToDevice, st) !=
            hipSuccess ||
        (s->kv_int8 && hipMemcpyAsync((void*)a.kvstats_dev, s->kvstats, sizeof(void*) * m->n_layers,
                                      hipMemcpyHostToDevice, st) != hipSuccess) ||
        hipMemsetAsync((void*)a.bar, 0, L.tg - L.bar, st) != hipSuccess ||
        hipMemsetAsync((void*)a.tg, 0xFF, L.total - L.tg, st) != hipSuccess || hipStreamSynchronize(st) != hipSuccess)
      return OHARA_ELAUNCH;
    return OHARA_OK;
  }
  a.B = s->batch; a.valid_vocab = s->valid_vocab; a.hist_cap = s->hist_cap;
  a.select = select_greedy;
  a.ids = s->ids; a.logits = s->logits;
  a.step_state = s->step_state; a.history = s->history;
  a.prof = s->prof_kernel == -2 ? reinterpret_cast<unsigned long long*>(ws + L.prof) : nullptr;
  if (48 * m->n_layers + 16 > OHARA_PROF_SLOTS) a.prof = nullptr;
  a.spin_limit = spin_limit ? spin_limit : (1u << 19);
  const MegaPlan P = mega_plan(m, s->batch, n_workgroups);
  const int mode = P.mode;
  const size_t smem = P.smem;
  a.lm_park = P.lm_park;
  a.ns = P.ns;
  if (s->kv_int8 && !mode) return OHARA_ESIZE;  // the int8 cache is served by the polled builds only
  if (smem > 160 * 1024) return OHARA_ESIZE;
  int rc;
#define OHARA_MEGA_ONE(...)                                                         \
  do {                                                                              \
    static ResidencySlot slot;                                                      \
    rc = mega_launch(decode_mega_kernel<__VA_ARGS__>, slot, a, smem, n_workgroups, st); \
  } while (0)
#define OHARA_MEGA(DD, GG)                                \
  do {                                                    \
    if (mode == 1) OHARA_MEGA_ONE(DD, GG, 1);             \
    else if (mode == 2) OHARA_MEGA_ONE(DD, GG, 2);        \
    else OHARA_MEGA_ONE(DD, GG, 0);                       \
  } while (0)
  if (s->kv_int8) rc = mega_launch_i8(a, D, G, mode, smem, n_workgroups, st);
  else if (a.prof && D == 128 && G == 1) {  // the stamps exist in these three instantiations only
    if (mode == 1) OHARA_MEGA_ONE(128, 1, 1, false, true);
    else if (mode == 2) OHARA_MEGA_ONE(128, 1, 2, false, true);
    else OHARA_MEGA_ONE(128, 1, 0, false, true);
  } else if (D == 128 && G == 1) OHARA_MEGA(128, 1);
  else if (D == 128 && G == 2) OHARA_MEGA(128, 2);
  else if (D == 128 && G == 4) OHARA_MEGA(128, 4);
  else if (D == 64 && G == 1) OHARA_MEGA(64, 1);
  else if (D == 64 && G == 2) OHARA_MEGA(64, 2);
  else OHARA_MEGA(64, 4);
#undef OHARA_MEGA
#undef OHARA_MEGA_ONE
  if (rc != OHARA_OK) return rc;
  return ohara_launch_status();
}

}  // extern "C"
