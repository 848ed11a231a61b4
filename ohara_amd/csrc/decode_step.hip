// Llama.forward through the KV cache (ohara/models/llama.py:279-323) as a fixed chain
// of five kernels per layer:
//   norm1 + QKV projection + rotary + cache append     (Block :199, Attention :84-98)
//   attention over the cache                           (:100-135)
//   output projection + residual                       (:142, :199)
//   norm2 + gate/up projection + SwiGLU                (:200, mlp.py:152)
//   down projection + residual                         (:200)
// then final norm + vocabulary projection (:321-322) and, optionally, greedy
// selection feeding the next step.  No host synchronisation, no allocation: the
// chain can be captured once into a HIP graph and replayed per token.
#include "common.h"

extern "C" int ohara_llama_forward(const OharaModel* m, const OharaDecodeState* s, int seq_len, int pos,
                                   int use_pos_dev, int logits_mode, int select_greedy, void* stream) {
  if (!m || !s || !m->layers || !s->kcache || !s->vcache) return OHARA_EINVAL;
  if (s->kv_int8 && (!s->kvstats || !s->kstage || !s->vstage)) return OHARA_EINVAL;
  if (s->batch < 1 || seq_len < 1) return OHARA_EINVAL;
  const int64_t rows64 = (int64_t)s->batch * seq_len;
  if (rows64 > s->rows_cap) return OHARA_ESIZE;
  const bool ragged = s->seq_pos != nullptr;
  if (!ragged && use_pos_dev && (!s->step_state || seq_len != 1)) return OHARA_EINVAL;
  if (!ragged && !use_pos_dev && (pos < 0 || pos + seq_len > m->t_max)) return OHARA_EINVAL;
  if (logits_mode < OHARA_LOGITS_NONE || logits_mode > OHARA_LOGITS_ALL) return OHARA_EINVAL;
  if (select_greedy && !(logits_mode == OHARA_LOGITS_LAST || (logits_mode == OHARA_LOGITS_ALL && seq_len == 1)))
    return OHARA_EINVAL;
  const int B = s->batch, R = (int)rows64;
  const int d = m->d_model, H = m->n_heads, Hkv = m->n_kv_heads, Dh = m->head_dim;
  const int32_t* pos_dev = use_pos_dev ? s->step_state : nullptr;  // first field is pos
  const int n_split = seq_len == 1 ? s->n_split : 1;
  hipStream_t hs = (hipStream_t)stream;
  int launch = 0;
  // Brackets launch number s->prof_kernel with the caller's events.
#define OHARA_RUN(call)                                                                     \
  do {                                                                                      \
    const bool prof_ = (launch == s->prof_kernel) && s->prof_start && s->prof_stop;         \
    if (prof_) (void)hipEventRecord((hipEvent_t)s->prof_start, hs);                         \
    rc = (call);                                                                            \
    if (prof_) (void)hipEventRecord((hipEvent_t)s->prof_stop, hs);                          \
    ++launch;                                                                               \
    if (rc) return rc;                                                                      \
  } while (0)
  int rc = 0;
  const bool tiled = R > 64 && s->xn != nullptr;
  OHARA_RUN(ohara_embed_bf16(s->ids, m->token_emb, s->x, R, d, m->vocab, stream));
  for (int l = 0; l < m->n_layers; ++l) {
    const OharaLayer& L = m->layers[l];
    if (tiled) {  // many rows: normalise once, then the tiled MFMA kernel (launches are not numbered)
      rc = ohara_rmsnorm_bf16(s->x, L.norm1, s->xn, R, d, m->eps, stream);
      if (rc) return rc;
    }
    if (ragged && s->kv_int8) {
      // one position per sequence over the int8 cache: rows to staging, quantise into the cache at each sequence's
      // own position, attention straight over the codes (the extra launch is not numbered)
      int8_t* kq = reinterpret_cast<int8_t*>(s->kcache[l]);
      int8_t* vq = reinterpret_cast<int8_t*>(s->vcache[l]);
      OHARA_RUN(ohara_qkv_rope_ragged_bf16(tiled ? s->xn : s->x, d, L.wqkv, d, tiled ? nullptr : L.norm1, m->eps, B,
                                           seq_len, H, Hkv, Dh, m->cos, m->sin, s->seq_pos, m->t_max, s->q, s->kstage,
                                           s->vstage, stream));
      rc = ohara_kv_quant_append_ragged_int8(s->kstage, s->vstage, B, seq_len, Hkv, Dh, s->seq_pos, kq, vq, s->kvstats[l],
                                             m->t_max, stream);
      if (rc) return rc;
      OHARA_RUN(ohara_attn_cached_ragged_int8(s->q, kq, vq, s->kvstats[l], B, seq_len, H, Hkv, Dh, m->t_max, s->seq_pos,
                                              n_split, s->attn_ws, s->attn, stream));
    } else if (ragged) {
      // one position per sequence; attention of any length through the split-context kernel
      OHARA_RUN(ohara_qkv_rope_append_ragged_bf16(tiled ? s->xn : s->x, d, L.wqkv, d, tiled ? nullptr : L.norm1, m->eps,
                                                  B, seq_len, H, Hkv, Dh, m->cos, m->sin, s->seq_pos, s->q, s->kcache[l],
                                                  s->vcache[l], m->t_max, stream));
      OHARA_RUN(ohara_attn_cached_ragged_bf16(s->q, s->kcache[l], s->vcache[l], B, seq_len, H, Hkv, Dh, m->t_max,
                                              s->seq_pos, n_split, s->attn_ws, s->attn, stream));
    } else if (!s->kv_int8) {
      OHARA_RUN(ohara_qkv_rope_append_bf16(tiled ? s->xn : s->x, d, L.wqkv, d, tiled ? nullptr : L.norm1, m->eps, B,
                                           seq_len, H, Hkv, Dh, m->cos, m->sin, pos, pos_dev, s->q, s->kcache[l],
                                           s->vcache[l], m->t_max, stream));
      if (seq_len >= 16 && (Dh == 64 || Dh == 128))
        OHARA_RUN(ohara_attn_prefill_bf16(s->q, s->kcache[l], s->vcache[l], B, seq_len, H, Hkv, Dh, m->t_max, pos,
                                          s->attn, stream));
      else
        OHARA_RUN(ohara_attn_cached_bf16(s->q, s->kcache[l], s->vcache[l], B, seq_len, H, Hkv, Dh, m->t_max, pos,
                                         pos_dev, n_split, s->attn_ws, s->attn, stream));
    } else {
      // int8 cache (kv_cache.py:94-102): rows to staging, quantise into the cache, attention on the
      // dequantised values (the extra launches are not numbered)
      int8_t* kq = reinterpret_cast<int8_t*>(s->kcache[l]);
      int8_t* vq = reinterpret_cast<int8_t*>(s->vcache[l]);
      OHARA_RUN(ohara_qkv_rope_bf16(tiled ? s->xn : s->x, d, L.wqkv, d, tiled ? nullptr : L.norm1, m->eps, B, seq_len, H,
                                    Hkv, Dh, m->cos, m->sin, pos, pos_dev, m->t_max, s->q, s->kstage, s->vstage, stream));
      rc = ohara_kv_quant_append_int8(s->kstage, s->vstage, B, seq_len, Hkv, Dh, pos, pos_dev, kq, vq, s->kvstats[l],
                                      m->t_max, stream);
      if (rc) return rc;
      if (seq_len >= 16 && (Dh == 64 || Dh == 128) && s->kdeq && s->vdeq) {
        const int len = pos + seq_len;
        rc = ohara_kv_dequant_int8(kq, s->kvstats[l], 0, B, len, Hkv, Dh, m->t_max, s->kdeq, stream);
        if (!rc) rc = ohara_kv_dequant_int8(vq, s->kvstats[l], 1, B, len, Hkv, Dh, m->t_max, s->vdeq, stream);
        if (rc) return rc;
        OHARA_RUN(ohara_attn_prefill_bf16(s->q, s->kdeq, s->vdeq, B, seq_len, H, Hkv, Dh, len, pos, s->attn, stream));
      } else {
        OHARA_RUN(ohara_attn_cached_int8(s->q, kq, vq, s->kvstats[l], B, seq_len, H, Hkv, Dh, m->t_max, pos, pos_dev,
                                         n_split, s->attn_ws, s->attn, stream));
      }
    }
    OHARA_RUN(ohara_gemm_skinny_bf16(s->attn, H * Dh, L.wo, d, H * Dh, nullptr, m->eps, R, OHARA_EPI_RESIDUAL, s->x, d,
                                s->x, d, stream));
    if (tiled) {
      rc = ohara_rmsnorm_bf16(s->x, L.norm2, s->xn, R, d, m->eps, stream);
      if (rc) return rc;
    }
    OHARA_RUN(ohara_gemm_skinny_bf16(tiled ? s->xn : s->x, d, L.wgu, m->d_ff, d, tiled ? nullptr : L.norm2, m->eps, R,
                                     OHARA_EPI_SWIGLU, nullptr, 0, s->act, m->d_ff, stream));
    OHARA_RUN(ohara_gemm_skinny_bf16(s->act, m->d_ff, L.wdown, d, m->d_ff, nullptr, m->eps, R, OHARA_EPI_RESIDUAL, s->x, d,
                                s->x, d, stream));
  }
  if (logits_mode == OHARA_LOGITS_ALL) {
    if (tiled) {
      rc = ohara_rmsnorm_bf16(s->x, m->final_norm, s->xn, R, d, m->eps, stream);
      if (rc) return rc;
    }
    OHARA_RUN(ohara_gemm_skinny_bf16(tiled ? s->xn : s->x, d, m->w_vocab, m->vocab, d, tiled ? nullptr : m->final_norm,
                                     m->eps, R, OHARA_EPI_STORE, nullptr, 0, s->logits, m->vocab, stream));
  } else if (logits_mode == OHARA_LOGITS_LAST) {
    // row b*seq_len + seq_len-1 of x for every sequence: a strided view, no gather
    OHARA_RUN(ohara_gemm_skinny_bf16(s->x + (size_t)(seq_len - 1) * d, seq_len * d, m->w_vocab, m->vocab, d,
                                     m->final_norm, m->eps, B, OHARA_EPI_STORE, nullptr, 0, s->logits, m->vocab,
                                     stream));
  }
  if (select_greedy)
    OHARA_RUN(ohara_argmax_bf16(s->logits, m->vocab, B, m->vocab, s->valid_vocab > 0 ? s->valid_vocab : m->vocab,
                                s->ids, s->history, s->hist_cap, s->step_state, stream));
#undef OHARA_RUN
  return OHARA_OK;
}

extern "C" int ohara_event_create(void** event) {
  if (!event) return OHARA_EINVAL;
  hipEvent_t e;
  if (hipEventCreate(&e) != hipSuccess) return OHARA_ELAUNCH;
  *event = e;
  return OHARA_OK;
}
extern "C" int ohara_event_destroy(void* event) {
  return hipEventDestroy((hipEvent_t)event) == hipSuccess ? OHARA_OK : OHARA_ELAUNCH;
}
extern "C" int ohara_event_record(void* event, void* stream) {
  return hipEventRecord((hipEvent_t)event, (hipStream_t)stream) == hipSuccess ? OHARA_OK : OHARA_ELAUNCH;
}
extern "C" int ohara_event_elapsed_ms(void* start, void* stop, float* ms) {
  if (!ms) return OHARA_EINVAL;
  return hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop) == hipSuccess ? OHARA_OK : OHARA_ELAUNCH;
}
