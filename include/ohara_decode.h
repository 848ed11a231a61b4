/*
 * ohara_decode.h - C ABI of libohara_decode.so, the MI355X (gfx950) kernels behind
 * ohara's KV-cache decode path.
 *
 * The reference (joey00072/ohara) is pure Python/PyTorch and has no FFI of its own;
 * each entry point below names the reference code it replaces (file:line in the
 * reference tree).  Conventions shared by every function:
 *
 *   - plain C: raw device pointers, sizes, a hipStream_t passed as void*;
 *   - returns OHARA_OK (0) or a negative OHARA_E* code; never throws, never exits,
 *     never allocates or frees device memory, and does not synchronise the host (the one
 *     exception is the one-time workspace set-up ohara_llama_decode_persistent(init_workspace=1));
 *   - all work is enqueued on `stream` and is stream-ordered, so every call can be
 *     recorded into a HIP graph;
 *   - bf16 tensors are passed as uint16_t* (raw bfloat16 bits), row-major;
 *   - `pos_dev` arguments: when non-NULL the kernel reads the cache position of the
 *     token being fed from that device int32 instead of the host argument (the
 *     visible length is then *pos_dev + 1), so a captured graph can be replayed
 *     while the position advances on the device.
 *
 * Weight matrices of Linear layers are consumed in a packed tile order produced by
 * ohara_pack_rows_bf16 (see below); everything else is in the reference's layout.
 */
#ifndef OHARA_DECODE_H
#define OHARA_DECODE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define OHARA_OK 0
#define OHARA_EINVAL (-1)   /* an argument violates the documented constraints */
#define OHARA_ELAUNCH (-2)  /* the HIP runtime rejected a launch */
#define OHARA_ESIZE (-3)    /* a size exceeds what the entry point supports */

/* Library version and a self-description string (build flags, arch). */
int ohara_abi_version(void);

/* ---- weight packing -------------------------------------------------------
 * Packed layout "strip/kstep/lane": the (N, K) row-major bf16 matrix of a Linear
 * (nn.Linear.weight, ohara/models/llama.py:60-63,252; ohara/modules/mlp.py:146-148)
 * is cut into strips of 16 rows and k-steps of 32 columns; the tile (strip s,
 * k-step j) is stored as 64 lanes x 8 bf16, lane = 16*g + m holding row
 * perm[16*s + m], columns 32*j + 8*g .. +7.  N is padded to a multiple of 16 and
 * K to a multiple of 32 with zeros.  `perm` (length padded N, int32, source row or
 * -1 for a zero row) may be NULL for the identity.
 * Returns the packed size in bytes through *bytes when `dst` is NULL. */
int ohara_pack_rows_bf16(const uint16_t* w, int n, int k, int ldw, const int32_t* perm, int n_padded,
                         uint16_t* dst, int64_t* bytes, void* stream);

/* ---- embedding ------------------------------------------------------------
 * out[t, :] = table[ids[t], :]            (nn.Embedding, llama.py:245,310) */
int ohara_embed_bf16(const int64_t* ids, const uint16_t* table, uint16_t* out, int n_tokens, int d, int vocab,
                     void* stream);

/* ---- RMSNorm --------------------------------------------------------------
 * out = bf16(x * rsqrt(mean(x^2) + eps)) * w      (ohara/modules/norm.py:16-21) */
int ohara_rmsnorm_bf16(const uint16_t* x, const uint16_t* w, uint16_t* out, int rows, int d, float eps,
                       void* stream);

/* ---- skinny GEMM (decode projections) ------------------------------------------
 * y = [rmsnorm(x; norm_w, eps)] @ W^T  with one of three epilogues.  `wp` is W in
 * the packed layout; n / k are the logical sizes of W.  norm_w may be NULL.
 * `batch` rows of x.  More than 64 rows without a fused norm go to the tiled MFMA
 * kernel of ohara_gemm_bf16; with a fused norm they are processed 64 at a time, each
 * chunk streaming W once.
 *
 * OHARA_EPI_STORE      out[b, n] = bf16(y)                      (any Linear)
 * OHARA_EPI_RESIDUAL   out[b, n] = bf16(resid[b, n] + bf16(y))  (llama.py:199-200)
 * OHARA_EPI_SWIGLU     W packed with gate/up rows interleaved (ohara_swiglu_perm);
 *                      out[b, f] = bf16(bf16(silu(bf16(gate))) * bf16(up))
 *                                                               (mlp.py:152)
 * The fused QKV + rotary + cache append is a separate entry point below. */
#define OHARA_EPI_STORE 0
#define OHARA_EPI_RESIDUAL 1
#define OHARA_EPI_SWIGLU 2
int ohara_gemm_skinny_bf16(const uint16_t* x, int ldx, const uint16_t* wp, int n, int k, const uint16_t* norm_w,
                           float eps, int batch, int epilogue, const uint16_t* resid, int ldr, uint16_t* out,
                           int ldo, void* stream);

/* Row permutation that interleaves gate and up rows for OHARA_EPI_SWIGLU: packed
 * row 16*s + 4*g + i is gate row 8*s + 2*g + i (i < 2) or up row 8*s + 2*g + i - 2.
 * Source rows index the vertical concatenation [gate; up] of two (f, k) matrices.
 * perm has 2 * f_padded entries, f_padded = f rounded up to a multiple of 8. */
int ohara_swiglu_perm(int f, int32_t* perm_host);

/* ---- tiled MFMA GEMM (batched prefill projections) ---------------------------
 * out = epi(x @ W^T) for any number of rows: 128 x 128 output tiles, K in steps of 64,
 * activations staged through LDS, packed weights streamed straight into the MFMA A operand.
 * Same packed `wp`, same epilogues and the same rounding points as ohara_gemm_skinny_bf16
 * (llama.py:84-86,142,322, mlp.py:152 with more than one position per call).  No fused norm. */
int ohara_gemm_bf16(const uint16_t* x, int ldx, const uint16_t* wp, int n, int k, int rows, int epilogue,
                    const uint16_t* resid, int ldr, uint16_t* out, int ldo, void* stream);

/* Fused q/k/v projection + rotary + KV-cache append: replaces Attention.forward's
 * three Linears, apply_rope and KVCache.forward (llama.py:84-98;
 * ohara/embeddings_pos/rotary.py:55-93; ohara/modules/kv_cache.py:75-118).
 * x holds batch*seq_len rows, row b*seq_len + s being position pos + s of sequence b
 * (seq_len = 1 at decode).  `wp` packs the rows [W_q; W_k; W_v].
 *   q_out  (batch*seq_len, h*dh) bf16, rotated
 *   kcache/vcache (batch_cap, t_max, h_kv, dh) bf16; rows pos..pos+seq_len-1 of
 *   sequence b are written with the rotated keys / the values.
 * cos/sin: (>= pos+seq_len, dh/2) bf16 tables (precompute_freqs_cis, rotary.py:24-38). */
int ohara_qkv_rope_append_bf16(const uint16_t* x, int ldx, const uint16_t* wp, int k, const uint16_t* norm_w,
                               float eps, int batch, int seq_len, int h, int h_kv, int dh, const uint16_t* cos,
                               const uint16_t* sin, int pos, const int32_t* pos_dev, uint16_t* q_out,
                               uint16_t* kcache, uint16_t* vcache, int t_max, void* stream);

/* The same projection + rotary, with the rotated k and the v rows written to (batch*seq_len,
 * h_kv*dh) buffers instead of into a cache (the int8 cache quantises them in a second step).
 * t_max only bounds the positions. */
/* ohara_qkv_rope_append_bf16 with one cache position per sequence: token s of sequence b is
 * rotated for, and appended at, position seq_pos[b] + s (device array, `batch` entries). */
int ohara_qkv_rope_append_ragged_bf16(const uint16_t* x, int ldx, const uint16_t* wp, int k, const uint16_t* norm_w,
                                      float eps, int batch, int seq_len, int h, int h_kv, int dh, const uint16_t* cos,
                                      const uint16_t* sin, const int32_t* seq_pos, uint16_t* q_out, uint16_t* kcache,
                                      uint16_t* vcache, int t_max, void* stream);
int ohara_qkv_rope_bf16(const uint16_t* x, int ldx, const uint16_t* wp, int k, const uint16_t* norm_w, float eps,
                        int batch, int seq_len, int h, int h_kv, int dh, const uint16_t* cos, const uint16_t* sin,
                        int pos, const int32_t* pos_dev, int t_max, uint16_t* q_out, uint16_t* k_out, uint16_t* v_out,
                        void* stream);

/* ohara_qkv_rope_bf16 with one position per sequence (seq_pos as in ohara_qkv_rope_append_ragged_bf16). */
int ohara_qkv_rope_ragged_bf16(const uint16_t* x, int ldx, const uint16_t* wp, int k, const uint16_t* norm_w, float eps,
                               int batch, int seq_len, int h, int h_kv, int dh, const uint16_t* cos, const uint16_t* sin,
                               const int32_t* seq_pos, int t_max, uint16_t* q_out, uint16_t* k_out, uint16_t* v_out,
                               void* stream);

/* ---- attention over the KV cache ------------------------------------------------
 * Query s (0 <= s < seq_len) of sequence b sits at cache position pos + s and sees
 * positions [0, pos + s] (the cache mask key_pos <= start_pos + q_idx, llama.py:109-113):
 *   out[b, s, h, :] = softmax(q[b,s,h,:] . K[b, 0:pos+s+1, h/(H/Hkv), :] / sqrt(dh)) V
 * (llama.py:100-135; GQA by head indexing instead of repeat_interleave :101-103).
 * seq_len = 1 is the decode case.  The context is split into `n_split` chunks;
 * partial (max, sum, acc) triples go to `workspace` and the last chunk to finish
 * merges them in chunk order.  workspace bytes = ohara_attn_workspace_bytes(
 * batch*seq_len, h, h_kv, dh, n_split); zero-fill it once before first use (the
 * kernels leave its counters at zero).  n_split = 1 needs no workspace (NULL ok);
 * n_split > 1 needs (h / h_kv) * n_split <= 2048.
 * q / out: (batch*seq_len, h*dh). */
int64_t ohara_attn_workspace_bytes(int batch, int h, int h_kv, int dh, int n_split);
int ohara_attn_cached_bf16(const uint16_t* q, const uint16_t* kcache, const uint16_t* vcache, int batch,
                           int seq_len, int h, int h_kv, int dh, int t_max, int pos, const int32_t* pos_dev,
                           int n_split, void* workspace, uint16_t* out, void* stream);
/* The same with one position per sequence: query s of sequence b sits at seq_pos[b] + s and sees
 * [0, seq_pos[b] + s].  No counterpart in the reference (one scalar position, llama.py:287-299). */
int ohara_attn_cached_ragged_bf16(const uint16_t* q, const uint16_t* kcache, const uint16_t* vcache, int batch,
                                  int seq_len, int h, int h_kv, int dh, int t_max, const int32_t* seq_pos, int n_split,
                                  void* workspace, uint16_t* out, void* stream);
/* seq_pos[b] += by for every b with active[b] != 0 (active NULL: all): advances a ragged batch by one
 * decode step without host involvement (graph replay). */
int ohara_advance_positions(int32_t* seq_pos, const uint8_t* active, int batch, int by, void* stream);
/* The same in one launch with the next step's inputs: next_ids[b] = new_ids[b] for an active sequence, 0 for
 * an idle slot (it rides along at position 0).  No counterpart in the reference (one position for the batch). */
int ohara_advance_ragged(int32_t* seq_pos, const uint8_t* active, const int64_t* new_ids, int64_t* next_ids, int batch,
                         int by, void* stream);

/* ohara_attn_cached_bf16 for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the
 * reference.  Same arguments minus the workspace: the chunk partials and counters live in a
 * device array inside the library (8 MiB + 64 KiB, held by every GPU the library runs on until
 * the process ends), so nothing is allocated or freed, by this library or through any other.
 * Limits: batch*seq_len*h_kv <= 16384 and
 *   align256(batch*seq_len*h*n_split*8) + align256(batch*seq_len*h*n_split*dh*4) <= 8 MiB;
 * anything larger returns OHARA_ESIZE and launches nothing.  The first call on a device looks up
 * the array's address (make it outside graph capture).  All calls on one GPU share the array:
 * calls that overlap in time on one GPU (different streams) race; calls on one stream do not. */
int ohara_attn_cached_bf16_noalloc(const uint16_t* q, const uint16_t* kcache, const uint16_t* vcache, int batch,
                                   int seq_len, int h, int h_kv, int dh, int t_max, int pos, const int32_t* pos_dev,
                                   int n_split, uint16_t* out, void* stream);

/* Same contract for many query positions per sequence (prefill), as a causal flash-style kernel
 * on MFMA: 128 queries per workgroup, keys/values walked in 64-position tiles through LDS,
 * online softmax in fp32, probabilities rounded to bf16 for the second product.  dh 64 or 128.
 * Needs no workspace.  (llama.py:100-135 with S > 1.) */
int ohara_attn_prefill_bf16(const uint16_t* q, const uint16_t* kcache, const uint16_t* vcache, int batch,
                            int seq_len, int h, int h_kv, int dh, int t_max, int pos, uint16_t* out, void* stream);

/* ---- int8 KV cache (ohara/modules/kv_cache.py:15-32, 67-73, 94-102, 116-118) ------------------
 * Every (sequence, position, head) row of dh values is stored as int8 with an fp32 scale and
 * minimum: scale = max((max - min) / 255, 1e-8), q = clamp(round((x - min) / scale - 128), -128,
 * 127), read back as bf16((q + 128) * scale + min).  The quantisation arithmetic is rounded to
 * bf16 after every operation, as the reference's tensor ops on a bf16 cache are, so codes, scales
 * and minima are bit-identical to it.  Caches: (batch_cap, t_max, h_kv, dh) int8.  Statistics:
 * `stats`, (batch_cap, h_kv, t_max, 4) fp32 = one 16-byte record (key scale, key minimum, value
 * scale, value minimum) per row, consecutive positions of a head contiguous (the order decode
 * attention reads them in; the reference's four (B, T, H_kv, 1) tensors, kv_cache.py:67-73, are
 * strided views of it).
 *   ohara_kv_quant_append_int8  quantises k / v rows (batch*seq_len, h_kv*dh) into positions
 *                               pos + s (pos_dev as elsewhere);
 *   ohara_kv_dequant_int8       the first `len` positions of the key (which = 0) or value (which = 1)
 *                               cache tensor as bf16 (batch, len, h_kv, dh) - what KVCache._read returns;
 *   ohara_attn_cached_int8      ohara_attn_cached_bf16 over the quantised cache, dequantising in
 *                               registers.  Scales must be bf16-representable, as the quantiser
 *                               writes them: (q + 128) * scale is then exact in fp32 and the
 *                               kernel's fused multiply-add equals the reference's two roundings. */
int ohara_kv_quant_append_int8(const uint16_t* k, const uint16_t* v, int batch, int seq_len, int h_kv, int dh, int pos,
                               const int32_t* pos_dev, int8_t* kq, int8_t* vq, float* stats, int t_max, void* stream);
int ohara_kv_dequant_int8(const int8_t* q, const float* stats, int which, int batch, int len, int h_kv, int dh,
                          int t_max, uint16_t* out, void* stream);
int ohara_attn_cached_int8(const uint16_t* q, const int8_t* kcache, const int8_t* vcache, const float* stats, int batch,
                           int seq_len, int h, int h_kv, int dh, int t_max, int pos, const int32_t* pos_dev, int n_split,
                           void* workspace, uint16_t* out, void* stream);

/* The append and the attention with one cache position per sequence (seq_pos: device array, `batch`
 * entries; token s of sequence b goes to / sits at seq_pos[b] + s).  No counterpart in the reference,
 * whose forward takes one scalar position for the whole batch (llama.py:287-299); the cache itself
 * (kv_cache.py:94-118) is indifferent to where each sequence stands. */
int ohara_kv_quant_append_ragged_int8(const uint16_t* k, const uint16_t* v, int batch, int seq_len, int h_kv, int dh,
                                      const int32_t* seq_pos, int8_t* kq, int8_t* vq, float* stats, int t_max,
                                      void* stream);
int ohara_attn_cached_ragged_int8(const uint16_t* q, const int8_t* kcache, const int8_t* vcache, const float* stats,
                                  int batch, int seq_len, int h, int h_kv, int dh, int t_max, const int32_t* seq_pos,
                                  int n_split, void* workspace, uint16_t* out, void* stream);

/* ---- greedy selection ---------------------------------------------------------
 * next_ids[b] = first index of max(logits[b, 0:valid_vocab])  (argmax of the last
 * position, ohara/chat_engine.py:61-63, ohara/inference.py:40-45; ids >= valid_vocab
 * are the padded vocabulary masked at chat_engine.py:398-399).  When `step_state`
 * (device, 4 x int32: pos, step, done, pad) is given, the token is also written to
 * history[step * batch + b] (if step < hist_cap) and the last workgroup to finish
 * advances pos and step by one - the device-side loop bookkeeping. */
int ohara_argmax_bf16(const uint16_t* logits, int ldl, int batch, int vocab, int valid_vocab, int64_t* next_ids,
                      int64_t* history, int hist_cap, int32_t* step_state, void* stream);

/* ---- temperature / top-k / top-p sampling ------------------------------------------
 * sample_next_token (ohara/chat_engine.py:51-82) and the nucleus branch of
 * Inference.sampler (ohara/inference.py:46-64) for temperature > 0, fused into one
 * launch, one workgroup per row:
 *   x = logits / temperature, ids >= valid_vocab masked (:398-399); top_k > 0 keeps
 *   x >= the k-th largest (ties survive, :66-69); p = softmax(x); 0 < top_p < 1 keeps the
 *   smallest descending-sorted prefix whose preceding mass does not exceed top_p
 *   (:72-81), renormalised; otherwise all of p in vocabulary order (:82).
 * torch.multinomial is replaced by inverse-CDF sampling with the caller's uniform draw
 * u[b] in [0,1); equal probabilities are ordered lowest id first.  Deterministic.
 * logits: (batch, vocab) bf16 (logits_are_fp32 = 0) or fp32.  vocab <= 131072.
 * history / step_state as in ohara_argmax_bf16.  With step_state and u_step_stride > 0 the draw of
 * row b is u[step * u_step_stride + b] (step = index of the token being produced, read on the
 * device), so a captured decode loop walks a pre-drawn (steps, batch) tensor by itself;
 * otherwise u[b].  temperature == 0 is ohara_argmax_bf16. */
int ohara_sample_topk_topp(const void* logits, int logits_are_fp32, int ldl, int batch, int vocab,
                           int valid_vocab, float temperature, int top_k, float top_p, const float* u,
                           int u_step_stride, int64_t* out_ids, int64_t* history, int hist_cap,
                           int32_t* step_state, void* stream);
/* The same selection, same results, for a caller whose sampler calls on one GPU do not overlap in time
 * (one decode stream, as in ohara/chat_engine.py's generate loop): a small top-k (<= 64) on a long bf16
 * row (8192 < vocab <= 65536, batch <= 64) is spread over one workgroup per 8192 ids, whose candidates
 * meet in a 330 KB scratch array inside the library (nothing is allocated); every other shape runs
 * ohara_sample_topk_topp's kernels.  Overlapping calls of this entry point on one GPU would share
 * that array. */
int ohara_sample_topk_topp_exclusive(const void* logits, int logits_are_fp32, int ldl, int batch, int vocab,
                           int valid_vocab, float temperature, int top_k, float top_p, const float* u,
                           int u_step_stride, int64_t* out_ids, int64_t* history, int hist_cap,
                           int32_t* step_state, void* stream);
/* The same spread selection with the candidates meeting in the CALLER's workspace instead of the library's
 * array: calls with different workspaces may overlap in time (one workspace per decode session / stream).
 * workspace: ohara_sample_workspace_bytes() bytes of device memory, 256-byte aligned, zeroed once before its
 * first use (the kernels leave its counters at zero); calls sharing one workspace must not overlap. */
int64_t ohara_sample_workspace_bytes(void);
int ohara_sample_topk_topp_ws(const void* logits, int logits_are_fp32, int ldl, int batch, int vocab,
                              int valid_vocab, float temperature, int top_k, float top_p, const float* u,
                              int u_step_stride, int64_t* out_ids, int64_t* history, int hist_cap,
                              int32_t* step_state, void* workspace, int64_t workspace_bytes, void* stream);

/* ---- BitNet-b1.58 BitLinear (ternary weights x int8 activations, int32 accumulate) ------
 * Integer form of BitLinear.forward (experiments/bitnet/bitnet.py:29-59):
 *   x_hat = RMSNorm(x; norm_w, eps) in bf16 (:49,53); s = 127 / max(max|x_hat|, 1e-5) and
 *   q = clamp(rint(x_hat * s), -128, 127) per row (:30-33); acc[n] = sum_k q[k] * T[n,k] in
 *   int32; y = bf16((float(acc) / s) * gamma) [+ resid]  (:58-59, bias dropped).
 * T in {-1,0,1} and gamma = max(mean|W|, 1e-5) come from weight_quant (:37-43), done once at
 * load time.  ohara_bitlinear_pack_ternary turns T (n, k) int8 row-major into the packed
 * 2-bit stream the kernels read (16 weights per dword; size through *bytes when dst is NULL).
 * ohara_act_quant_int8 and ohara_gemv_ternary_i8 are the two halves; ohara_bitlinear_bf16
 * fuses them (k <= 6144).  acc_out, when given, receives the raw int32 accumulators - the
 * quantity that must match a CPU int32 matmul bit for bit.  ldq must be a multiple of 16,
 * k and ldx multiples of 8.  pre_norm_w (may be NULL) is the weight of the block-level RMSNorm
 * that precedes the projection (llama.py:199-200), applied in the same pass: x := bf16(
 * RMSNorm(x; pre_norm_w, eps)) before the BitLinear's own norm. */
int ohara_bitlinear_pack_ternary(const int8_t* t, int n, int k, int ldt, uint32_t* dst, int64_t* bytes, void* stream);
int ohara_act_quant_int8(const uint16_t* x, int ldx, const uint16_t* norm_w, float eps, int rows, int k, int8_t* q,
                         int ldq, float* s, int32_t* sumq, void* stream);
int ohara_gemv_ternary_i8(const int8_t* q, int ldq, const float* s, const int32_t* sumq, const uint32_t* wp, int n,
                          int k, float gamma, int rows, const uint16_t* resid, int ldr, uint16_t* out, int ldo,
                          int32_t* acc_out, int ldacc, void* stream);
int ohara_bitlinear_bf16(const uint16_t* x, int ldx, const uint16_t* pre_norm_w, const uint16_t* norm_w, float eps,
                         const uint32_t* wp, int n, int k, float gamma, int rows, const uint16_t* resid, int ldr,
                         uint16_t* out, int ldo, int32_t* acc_out, int ldacc, void* stream);

/* Groups of BitLinears that read the same rows, for decode (rows <= 64), one launch each:
 *   - attn.query / attn.key / attn.value (each with its own norm weight, packed weights and gamma,
 *     index 0..2 of the three arrays) with rotary + cache append as the epilogue: q_out
 *     (rows, h*dh) rotated, rotated k and v written at cache position pos + s (pos_dev as in
 *     ohara_qkv_rope_append_bf16);
 *   - ff.gate and ff.up with SwiGLU as the epilogue: out[b, f] = bf16(bf16(silu(gate)) * up).
 * Same arithmetic as the separate calls (bitnet.py:29-59, rotary.py:55-93, kv_cache.py:104-105,
 * mlp.py:152). */
int ohara_bitlinear_qkv_rope_append_bf16(const uint16_t* x, int ldx, const uint16_t* pre_norm_w, float eps, int k,
                                         const uint16_t* const* norm_w, const uint32_t* const* wp, const float* gamma,
                                         int batch, int seq_len, int h, int h_kv, int dh, const uint16_t* cos,
                                         const uint16_t* sin, int pos, const int32_t* pos_dev, uint16_t* q_out,
                                         uint16_t* kcache, uint16_t* vcache, int t_max, void* stream);
int ohara_bitlinear_gate_up_bf16(const uint16_t* x, int ldx, const uint16_t* pre_norm_w, float eps, int k, int f,
                                 const uint16_t* gate_norm_w, const uint32_t* gate_wp, float gate_gamma,
                                 const uint16_t* up_norm_w, const uint32_t* up_wp, float up_gamma, int rows,
                                 uint16_t* out, int ldo, void* stream);

/* out = bf16(bf16(silu(gate)) * up), elementwise over n values (ohara/modules/mlp.py:152). */
int ohara_silu_mul_bf16(const uint16_t* gate, const uint16_t* up, uint16_t* out, int64_t n, void* stream);

/* Rotary on q (in place) and on k, and append of the rotated k and of v to the cache, for
 * projections that were computed unfused (ohara/embeddings_pos/rotary.py:55-93,
 * ohara/modules/kv_cache.py:104-105).  q: (batch*seq_len, h*dh), k/v: (batch*seq_len, h_kv*dh).
 * t_max == 0: kcache / vcache are row buffers of k's and v's shape instead of caches - the rotated
 * keys and the values of this call, which an int8 cache's append (ohara_kv_quant_append_int8,
 * kv_cache.py:94-102) takes next; the caller keeps pos + seq_len within the rotary tables. */
int ohara_rope_append_bf16(uint16_t* q, const uint16_t* k, const uint16_t* v, int batch, int seq_len, int h, int h_kv,
                           int dh, const uint16_t* cos, const uint16_t* sin, int pos, const int32_t* pos_dev,
                           uint16_t* kcache, uint16_t* vcache, int t_max, void* stream);

/* ---- grouped mixture-of-experts feed-forward (eval mode) -------------------------------------
 * GroupedMoE.forward (ohara/modules/moe_grouped.py:209-228) in five launches:
 *  ohara_moe_route_topk     _route (:122-147) from the bf16 router logits (n_tokens, n_experts):
 *                           experts = top-k of logits [+ router_bias when biased_topk] with ties
 *                           to the lowest id; weights = softmax (or sigmoid, optionally normalised)
 *                           of the k selected unbiased logits, cast to bf16.  k <= 16, E <= 1024.
 *  ohara_moe_sort_pairs     the stable sort by expert of :161-168: offsets (E+1), pair_of[sorted
 *                           position] = token*k + slot, pos_of = its inverse.  n_pairs <= 65536.
 *  ohara_moe_experts_gate_up  act[sorted position] = bf16(silu(bf16(x W_gate[e]))) * bf16(x W_up[e])
 *  ohara_moe_experts_down     y[sorted position]   = bf16(bf16(act W_down[e]) * weight)   (:175-181)
 *                           expert weights: per expert, rows packed by ohara_pack_rows_bf16
 *                           (gate/up rows interleaved with ohara_swiglu_perm), experts
 *                           expert_stride_bytes apart.
 *  ohara_moe_combine        out[token] = resid + (sum over its experts in ascending expert id,
 *                           each add rounded to bf16 (:184) + shared[token]); shared / resid may
 *                           be NULL. */
int ohara_moe_route_topk(const uint16_t* router_logits, int ldl, const uint16_t* router_bias, int n_tokens, int n_experts,
                         int k, int biased_topk, int gate_sigmoid, int normalize, int32_t* expert_idx,
                         uint16_t* expert_w, void* stream);
int ohara_moe_sort_pairs(const int32_t* expert_idx, int n_pairs, int n_experts, int32_t* offsets, int32_t* pair_of,
                         int32_t* pos_of, void* stream);
int ohara_moe_experts_gate_up(const uint16_t* x, int ldx, const uint16_t* wp_gate_up, int64_t expert_stride_bytes,
                              int n_experts, int hidden, int d, int k, const int32_t* offsets, const int32_t* pair_of,
                              uint16_t* act, int ld_act, void* stream);
int ohara_moe_experts_down(const uint16_t* act, int ld_act, const uint16_t* wp_down, int64_t expert_stride_bytes,
                           int n_experts, int d, int hidden, int k, const int32_t* offsets, const int32_t* pair_of,
                           const uint16_t* expert_w, uint16_t* y, int ldy, void* stream);
int ohara_moe_combine(const uint16_t* y, int ldy, const int32_t* expert_idx, const int32_t* pos_of, int n_tokens, int k,
                      const uint16_t* shared, int ld_shared, const uint16_t* resid, int ldr, uint16_t* out, int ldo, int d,
                      void* stream);
/* The same feed-forward for a decode step in four launches (at most 64 experts, 1024 pairs, d <= 4096):
 *  ohara_moe_route_fused    the block's RMSNorm (ohara/modules/norm.py:16-21; ohara/models/llama.py:200) of the rows
 *                           x, the router Linear on the normalised rows (moe_grouped.py:126), _route (:122-147) and
 *                           the sort of :161-168 in ONE launch: x_norm (n_tokens, d) for the experts, expert_idx /
 *                           expert_w, offsets / pair_of / pos_of as above; router_logits (n_tokens, n_experts) may be
 *                           NULL.  counter: one int32 of device memory that is zero between calls (the workgroup
 *                           that finishes last sorts, and leaves it zero); calls that share it must not overlap.
 *  ohara_moe_experts_gate_up_shared / ohara_moe_experts_down_shared
 *                           the expert launches with the shared expert (_shared, :206-207, 219-220) as more
 *                           rows of their grids (16 tokens a row): wp_shared its packed gate/up (down) rows, shared_hidden its width,
 *                           act_shared (n_tokens, shared_hidden), y_shared (n_tokens, d) = bf16(act_shared W_down),
 *                           not scaled - pass y_shared to ohara_moe_combine as `shared`.  wp_shared NULL: as the
 *                           entry points above. */
int ohara_moe_route_fused(const uint16_t* x, int ldx, const uint16_t* norm_w, float eps, const uint16_t* router_wp,
                          const uint16_t* router_bias, int n_tokens, int d, int n_experts, int k, int biased_topk,
                          int gate_sigmoid, int normalize, uint16_t* x_norm, int ld_x_norm, uint16_t* router_logits, int ldl,
                          int32_t* expert_idx, uint16_t* expert_w, int32_t* offsets, int32_t* pair_of, int32_t* pos_of,
                          int32_t* counter, void* stream);
int ohara_moe_experts_gate_up_shared(const uint16_t* x, int ldx, const uint16_t* wp_gate_up, int64_t expert_stride_bytes,
                                     int n_experts, int hidden, int d, int k, const int32_t* offsets,
                                     const int32_t* pair_of, uint16_t* act, int ld_act, const uint16_t* wp_shared,
                                     int shared_hidden, int n_tokens, uint16_t* act_shared, int ld_act_shared,
                                     void* stream);
int ohara_moe_experts_down_shared(const uint16_t* act, int ld_act, const uint16_t* wp_down, int64_t expert_stride_bytes,
                                  int n_experts, int d, int hidden, int k, const int32_t* offsets, const int32_t* pair_of,
                                  const uint16_t* expert_w, uint16_t* y, int ldy, const uint16_t* wp_shared,
                                  int shared_hidden, int n_tokens, const uint16_t* act_shared, int ld_act_shared,
                                  uint16_t* y_shared, int ldy_shared, void* stream);

/* ---- the whole forward pass through the KV cache ---------------------------------
 * Llama.forward(x, kv_cache, position) (ohara/models/llama.py:279-323; Block.forward
 * :191-201) for seq_len new tokens per sequence, as a fixed sequence of the kernels
 * above enqueued on `stream`; optionally followed by greedy selection that feeds the
 * next call, so a generate loop (ohara/chat_engine.py:395-405,
 * ohara/inference.py:110-121) can run without touching the host.
 * Host structs; every pointer inside is a device pointer owned by the caller. */
typedef struct OharaLayer {
  const uint16_t* wqkv;  /* packed rows [W_q; W_k; W_v], each (heads*dh, d)          */
  const uint16_t* wo;    /* packed attn.proj (d, h*dh)                                */
  const uint16_t* wgu;   /* packed ff.gate / ff.up, rows interleaved (swiglu perm)    */
  const uint16_t* wdown; /* packed ff.down (d, f)                                     */
  const uint16_t* norm1; /* (d) */
  const uint16_t* norm2; /* (d) */
} OharaLayer;

typedef struct OharaModel {
  int32_t n_layers, d_model, n_heads, n_kv_heads, head_dim, d_ff, vocab, t_max;
  float eps;
  int32_t reserved;
  const uint16_t* token_emb;  /* (vocab, d) row-major, unpacked */
  const uint16_t* final_norm; /* (d) */
  const uint16_t* w_vocab;    /* packed vocab_proj (vocab, d) */
  const uint16_t* cos;        /* (2*t_max, dh/2) bf16 */
  const uint16_t* sin;
  const OharaLayer* layers;   /* host array [n_layers] */
} OharaModel;

typedef struct OharaDecodeState {
  int32_t batch;         /* sequences                                                     */
  int32_t rows_cap;      /* rows (batch*seq_len) the activation buffers below can hold    */
  int32_t n_split;       /* context chunks of decode attention (seq_len == 1)             */
  int32_t valid_vocab;   /* ids >= this are never selected; 0 = whole vocabulary          */
  int32_t hist_cap;
  int32_t prof_kernel;   /* -1: off; else index of the launch (0 = embedding, 1 + 5*l + i = i-th
                            kernel of layer l, 1 + 5*n_layers = vocabulary projection, then the
                            selection) to bracket with prof_start / prof_stop                    */
  int64_t* ids;          /* (rows) tokens fed; ids[0:batch] overwritten by greedy select  */
  uint16_t* x;           /* (rows, d) residual stream                                     */
  uint16_t* q;           /* (rows, h*dh)                                                  */
  uint16_t* attn;        /* (rows, h*dh)                                                  */
  uint16_t* act;         /* (rows, f)                                                     */
  uint16_t* xn;          /* (rows, d) normalised rows for calls with > 64 rows; may be NULL when
                            rows_cap <= 64 (NULL with more rows: the skinny kernel runs 64 rows at
                            a time instead of the tiled MFMA kernel)                           */
  uint16_t* logits;      /* (batch, vocab) or (rows, vocab), see logits_mode              */
  void* attn_ws;         /* ohara_attn_workspace_bytes(batch, h, h_kv, dh, n_split)       */
  int32_t* step_state;   /* 4 x int32 {pos, step, done, pad}, may be NULL                 */
  int64_t* history;      /* (hist_cap, batch) generated ids, may be NULL                  */
  uint16_t* const* kcache; /* host array [n_layers] of (batch_cap, t_max, h_kv, dh)       */
  uint16_t* const* vcache;
  /* int8 cache mode (kv_int8 != 0): kcache / vcache point at int8 tensors of the same shape,
     kvstats at the per-layer (batch_cap, h_kv, t_max, 4) fp32 statistics records; kstage / vstage
     (rows, h_kv*dh) receive the bf16 rows before they are quantised; kdeq / vdeq ((batch, t_max,
     h_kv, dh) bf16, may be NULL) hold the dequantised cache for calls with >= 16 positions. */
  int32_t kv_int8;
  float* const* kvstats;
  uint16_t* kstage;
  uint16_t* vstage;
  uint16_t* kdeq;
  uint16_t* vdeq;
  /* ragged batches: when non-NULL, sequence b's first fed token sits at cache position seq_pos[b]
     (device array of `batch` entries) and the pos / use_pos_dev arguments are ignored.  The
     reference has one scalar position for the whole batch (llama.py:287-299); this is what lets
     sequences of different lengths decode in one batch.  bf16 caches only. */
  const int32_t* seq_pos;
  void* prof_start;      /* hipEvent_t recorded on `stream` right before launch prof_kernel */
  void* prof_stop;       /* hipEvent_t recorded right after it                             */
} OharaDecodeState;

#define OHARA_LOGITS_NONE 0
#define OHARA_LOGITS_LAST 1 /* logits (batch, vocab) of each sequence's last position     */
#define OHARA_LOGITS_ALL 2  /* logits (batch*seq_len, vocab), what llama.py:321-322 returns */

/* pos: cache position of the first fed token (ignored when use_pos_dev != 0, then
 * step_state->pos is read on the device; that needs seq_len == 1).
 * select_greedy != 0 (needs logits_mode LAST or seq_len == 1) appends the argmax. */
int ohara_llama_forward(const OharaModel* m, const OharaDecodeState* s, int seq_len, int pos, int use_pos_dev,
                        int logits_mode, int select_greedy, void* stream);

/* ---- one decode step as ONE persistent launch (batch <= 16) ------------------------
 * Same result as ohara_llama_forward(seq_len = 1, use_pos_dev = 1, LOGITS_LAST) but the
 * whole step (all layers, vocabulary projection, greedy selection) runs in a single
 * kernel of `n_workgroups` resident workgroups (use the CU count; more than the device can
 * hold of this kernel at once returns OHARA_ESIZE) whose phases are separated by grid-wide barriers
 * (batch > 8) or hand their rows over through memory that the consumers poll (batch <= 8); it has no counterpart in the reference, whose decode step is
 * ~1000 eager launches (llama.py:279-323).  The cache position and step index are read
 * from / advanced in s->step_state; s->attn and s->attn_ws are not used.
 * `workspace`: ohara_persistent_workspace_bytes(m, batch, s->n_split, n_workgroups) of
 * device memory with any contents (it need not be zeroed: the call with init_workspace = 1 sets
 * what a step relies on, every other slot a step reads was written earlier in the same step, and
 * the merge of the attention chunks never uses a chunk no workgroup wrote).  Call once with
 * init_workspace = 1 (copies the layer table and the cache pointers to the device, zeroes the
 * barrier words, the launch counters and the attention partials behind them and fills the
 * hand-off rows of the polled builds (batch <= 8) with 0xFF, their "not written yet"; synchronises the stream;
 * do it outside graph capture) whenever the model or the caches change, and before the workspace
 * is used for the first time or after its memory has been used for anything else; then each call
 * with init_workspace = 0 enqueues one step.  Steps on one workspace must not overlap (each
 * step counts itself in the workspace).  spin_limit bounds every barrier wait and every poll for
 * a hand-off (0 = default); if a wait expires the kernel still drains and the error word reads
 * non-zero.  s->n_split must be 16.
 * Requires head_dim 64 or 128, n_heads / n_kv_heads in {1, 2, 4}, d_model <= 1024,
 * d_model and d_ff multiples of 8. */
int64_t ohara_persistent_workspace_bytes(const OharaModel* m, int batch, int n_split, int n_workgroups);
int ohara_llama_decode_persistent(const OharaModel* m, const OharaDecodeState* s, void* workspace, int n_workgroups,
                                  int init_workspace, int select_greedy, unsigned int spin_limit, void* stream);
/* Byte offsets inside the workspace: the barrier words; the sticky error word (uint32,
 * non-zero after a barrier wait expired); per workgroup 1024 x uint64 samples of the constant
 * 100 MHz clock taken by its thread 0 at every phase boundary when s->prof_kernel == -2 (workgroup
 * w's samples start 8192 w bytes after the offset; measurement only; the samples
 * are compiled into a separate build of the kernel that exists for head_dim 128 with
 * n_kv_heads == n_heads only, other shapes leave the slots untouched). */
int64_t ohara_persistent_barrier_offset(const OharaModel* m, int batch, int n_split, int n_workgroups);
/* Which build of the kernel a launch with this model, batch and grid runs: 0 the general one (a grid
 * barrier between the phases), 1 and 2 the polled ones (one sequence; two to eight).  The polled builds
 * also serve the int8 cache (s->kv_int8: the attention phase dequantises the tiles it reads and
 * quantises the appended row as ohara_kv_quant_append_int8 does, ohara/modules/kv_cache.py:15-32);
 * ohara_llama_decode_persistent returns OHARA_ESIZE for an int8 cache where this returns 0. */
int ohara_persistent_polled(const OharaModel* m, int batch, int n_workgroups);
int64_t ohara_persistent_error_offset(const OharaModel* m, int batch, int n_split, int n_workgroups);
int64_t ohara_persistent_profile_offset(const OharaModel* m, int batch, int n_split, int n_workgroups);

/* ---- one decode step of the BitNet-b1.58 Llama as ONE persistent launch (batch <= 8) --------
 * Llama.forward(x, kv_cache, position) (ohara/models/llama.py:279-323) for one new token per
 * sequence when the seven projections of every block are BitLinears
 * (experiments/bitnet/bitnet.py:29-95, swapped in by apply_bitlinear :70-95 over the target list of
 * experiments/bitnet/train_bitnet.py:240): per projection the BitLinear's own RMSNorm, the
 * per-token int8 codes, the ternary product on the integer matrix cores and the rescale; block
 * norms, rotary, cache append, attention, SwiGLU, residuals, the final norm, the bf16 vocabulary
 * projection and the greedy selection as in ohara_llama_decode_persistent, whose calling
 * convention (init_workspace, step_state, spin_limit, error word) this entry point shares.  The
 * integer accumulators are those of ohara_bitlinear_* on the same rows; the reference's eager
 * step is ~1700 launches.
 * w[i] / norm_w[i] / gamma[i]: packed ternary weight (ohara_bitlinear_pack_ternary), the
 * BitLinear's norm weight and weight scale of attn.query, attn.key, attn.value, attn.proj,
 * ff.gate, ff.up, ff.down in that order.
 * Requires head_dim 64 or 128, n_heads == n_kv_heads, d_model and n_heads * head_dim <= 2048,
 * d_ff <= 6144, d_model and d_ff multiples of 16, n_workgroups >= 4; s->n_split must be 16; uses s->batch, valid_vocab, hist_cap, ids, logits,
 * step_state, history, kcache, vcache. */
#define OHARA_BIT_QUERY 0
#define OHARA_BIT_KEY 1
#define OHARA_BIT_VALUE 2
#define OHARA_BIT_PROJ 3
#define OHARA_BIT_GATE 4
#define OHARA_BIT_UP 5
#define OHARA_BIT_DOWN 6
typedef struct OharaBitLayer {
  const uint32_t* w[7];
  const uint16_t* norm_w[7];
  float gamma[7];
  float reserved;
  const uint16_t* norm1; /* (d) block norms */
  const uint16_t* norm2;
} OharaBitLayer;

typedef struct OharaBitModel {
  int32_t n_layers, d_model, n_heads, n_kv_heads, head_dim, d_ff, vocab, t_max;
  float eps;
  int32_t reserved;
  const uint16_t* token_emb;  /* (vocab, d) row-major, unpacked */
  const uint16_t* final_norm; /* (d) */
  const uint16_t* w_vocab;    /* packed vocab_proj (vocab, d), bf16 (ohara_pack_rows_bf16) */
  const uint16_t* cos;        /* (2*t_max, dh/2) bf16 */
  const uint16_t* sin;
  const OharaBitLayer* layers; /* host array [n_layers] */
} OharaBitModel;

int64_t ohara_bitnet_persistent_workspace_bytes(const OharaBitModel* m, int batch, int n_workgroups);
int64_t ohara_bitnet_persistent_error_offset(const OharaBitModel* m, int batch, int n_workgroups);
/* 1024 x uint64 shader-clock samples of workgroup 0 (six per grid barrier: phase work issued, own
 * stores complete, workgroup barrier passed, arrival issued, prefetch issued, barrier passed), taken
 * when s->prof_kernel == -2 (measurement only; a separate build of the kernel that exists for
 * head_dim 128 only, other shapes leave the slots untouched). */
int64_t ohara_bitnet_persistent_profile_offset(const OharaBitModel* m, int batch, int n_workgroups);
int ohara_bitnet_decode_persistent(const OharaBitModel* m, const OharaDecodeState* s, void* workspace, int n_workgroups,
                                   int init_workspace, int select_greedy, unsigned int spin_limit, void* stream);

/* ---- Phi (ohara/models/phi.py): the parts of its cached decode path that differ from Llama ----
 * nn.Linear WITH bias on packed weights (phi.py:46-47, :63-66, :161), any number of rows (up to 128:
 * the weight-streaming strip kernel, 64 rows per pass; more: the tiled MFMA kernel of ohara_gemm_bf16,
 * same epilogues and rounding points).  n % 4 == 0, k % 8 == 0.
 *   OHARA_LIN_BIAS       out = bf16(x @ W^T + bias)
 *   OHARA_LIN_BIAS_GELU  out = new_gelu(bf16(x @ W^T + bias)), every op of phi.py:37-40 rounded to
 *                        bf16 as the eager ops round                          (MLP.fc1, phi.py:50-51)
 *   OHARA_LIN_BIAS_ADD2  out = bf16(bf16(add1 + bf16(x @ W^T + bias)) + add2): the parallel block's
 *                        `mixer(x) + mlp(x) + residual` with add1 = mixer output, add2 = block input
 *                                                                              (phi.py:151) */
#define OHARA_LIN_BIAS 0
#define OHARA_LIN_BIAS_GELU 1
#define OHARA_LIN_BIAS_ADD2 2
int ohara_linear_bias_bf16(const uint16_t* x, int ldx, const uint16_t* wp, int n, int k, const uint16_t* bias, int rows,
                           int epilogue, const uint16_t* add1, int ld1, const uint16_t* add2, int ld2, uint16_t* out,
                           int ldo, void* stream);
/* The head of a Phi block in one launch (phi.py:150, :81-87, :95, :50-51): h = LayerNorm(x), then
 * [q; k; v; fc1] = h @ W^T + bias with W the packed vertical concatenation of q_proj, k_proj, v_proj
 * (d rows each) and mlp.fc1 (ff rows): q rows -> q (leading dimension ldq), k / v rows -> the
 * caches at position pos + s as they are (un-rotated), fc1 rows -> new_gelu -> act.  Same rounding
 * points as ohara_layernorm_bf16 + ohara_linear_bias_bf16 + ohara_kv_append_bf16, except that the
 * variance comes from the sums of x and x^2.  ln_w == NULL: x already is the normalised input
 * (measured faster at Phi-2's sizes: a separate LayerNorm launch costs less than re-deriving the
 * statistics in each of the 1120 workgroups before their weight loads start).
 * d % 16 == 0, ff % 4 == 0. */
int ohara_phi_block_in_bf16(const uint16_t* x, int ldx, const uint16_t* ln_w, const uint16_t* ln_b, float eps,
                            const uint16_t* wp, const uint16_t* bias, int d, int ff, int batch, int seq_len, int pos,
                            const int32_t* pos_dev, uint16_t* q, int ldq, uint16_t* kcache, uint16_t* vcache, int t_max,
                            uint16_t* act, int ldact, void* stream);
/* nn.LayerNorm over the last dimension (phi.py:132, :160): fp32 mean and biased variance,
 * out = bf16((x - mean) * rstd * weight + bias).  d % 8 == 0. */
int ohara_layernorm_bf16(const uint16_t* x, int ldx, const uint16_t* weight, const uint16_t* bias, uint16_t* out, int ldo,
                         int rows, int d, float eps, void* stream);
/* KVCache.forward for rows that are stored as they are (phi.py:95, kv_cache.py:104-105): row
 * (b, s) of k / v (leading dimension ld, h*dh wide) -> cache[b, pos + s].  pos_dev (seq_len 1):
 * the position is read on the device. */
int ohara_kv_append_bf16(const uint16_t* k, const uint16_t* v, int ld, int batch, int seq_len, int h, int dh, int pos,
                         const int32_t* pos_dev, uint16_t* kcache, uint16_t* vcache, int t_max, void* stream);
/* PhiMHA's attention core (phi.py:98-117): fp32 throughout; the first `rot` features of every head
 * rotate in the half-split layout (feature i with i + rot/2; rotary.py:131-164), queries from
 * position pos (+ s), the cached UN-rotated keys from 0; key t is visible to query s when
 * t <= pos + s; softmax(q k^T / sqrt(dh)) v rounded once to bf16.  cos / sin: (t_max, rot/2) fp32
 * tables of rotary.py:166-184.  q: rows (b, s) with leading dimension ldq; out (batch*seq_len, h*dh).
 * dh % 8 == 0, dh <= 128.  n_split > 1 (seq_len 1 only, at most 64) spreads the context of every
 * (sequence, head) over that many workgroups whose partial results meet in `workspace`
 * (ohara_phi_attn_workspace_bytes, zero-filled once before the first use; calls sharing it must not
 * overlap) and are merged in chunk order by the workgroup that finishes last.  Calls with 16 or more
 * new tokens per sequence (prefill; head widths 16, 32, 64, 80, 128) run queries in tiles of 64
 * against key / value tiles in LDS with fp32 matrix products; other shapes one query per workgroup. */
int64_t ohara_phi_attn_workspace_bytes(int batch, int h, int dh, int n_split);
int ohara_phi_attn_bf16(const uint16_t* q, int ldq, const uint16_t* kcache, const uint16_t* vcache, const float* cos,
                        const float* sin, int rot, int batch, int seq_len, int h, int dh, int t_max, int pos,
                        const int32_t* pos_dev, int n_split, void* workspace, uint16_t* out, void* stream);

/* ---- timing helpers (measurement only; no counterpart in the reference) -----------
 * Thin wrappers over hipEventCreate / hipEventDestroy / hipEventElapsedTime so that a
 * benchmark can time single launches on the stream they run on without another HIP
 * binding.  elapsed needs both events completed (synchronise the stream first). */
int ohara_event_create(void** event);
int ohara_event_destroy(void* event);
int ohara_event_record(void* event, void* stream);
int ohara_event_elapsed_ms(void* start, void* stop, float* ms);

#ifdef __cplusplus
}
#endif
#endif /* OHARA_DECODE_H */
