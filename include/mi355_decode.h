/*
 * mi355_decode.h -- C ABI of libmi355_decode.so
 *
 * MI355X (gfx950) kernels for the decode-step hot path of Megatron-Core's dynamic
 * inference engine: KV-append into the chunked ("paged") KV cache, paged GQA
 * decode / chunked-prefill attention, and the fused q/k norm + rotary embedding.
 *
 * Conventions (all entry points)
 *  - Every pointer except `stream`, names and returned strings is a DEVICE pointer
 *    owned by the caller; the library allocates nothing and keeps no pointer.
 *  - `stream` is a hipStream_t (null = the default stream).  Calls only enqueue
 *    work: they never synchronise and never read device memory on the host, so they
 *    can be recorded into a HIP graph.
 *  - Strides are in ELEMENTS of the tensor they describe unless the name says bytes.
 *  - Return value: 0 = enqueued; negative = rejected, nothing was launched
 *    (MI_ERR_*); mi_last_error() gives the message of the calling thread's last
 *    rejection.
 *  - The library keeps no state between calls: what a call does depends on its
 *    arguments only (kernel timing, mi_profile_enable, is the one exception and is a
 *    measurement aid).  Experiment knobs travel with the call (MiTuning).
 *  - `dtype` is the 16-bit element type of q / k / v / out, of a cache that is not
 *    fp8 and of norm weights: MI_DTYPE_BF16 or MI_DTYPE_FP16 (the reference's
 *    params_dtype, dynamic_context.py:195,287-308).
 *  - KV cache layout is the reference's: key cache = memory_buffer[0, layer],
 *    value cache = memory_buffer[1, layer], each `[n_chunks, chunk_tokens, Hkv, d]`
 *    (megatron/core/inference/contexts/dynamic_context.py:296-308,547-564).
 */
#ifndef MI355_DECODE_H
#define MI355_DECODE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
  MI_OK = 0,
  MI_ERR_NULL = -1,
  MI_ERR_SHAPE = -2,
  MI_ERR_ALIGN = -3,
  MI_ERR_UNSUPPORTED = -4,
  MI_ERR_WORKSPACE = -5,
  MI_ERR_LAUNCH = -6
};

enum { MI_DTYPE_BF16 = 0, MI_DTYPE_FP16 = 1 };
/* KV storage: the 16-bit type given by `dtype`, or fp8-e4m3 bytes with scales (q / out in either 16-bit type). */
enum { MI_KV_16BIT = 0, MI_KV_BF16 = 0, MI_KV_FP8_E4M3 = 1 };
enum { MI_NORM_NONE = 0, MI_NORM_RMS = 1, MI_NORM_L2 = 2 };

/* ABI revision of the loaded library. */
int mi_version(void);

/* Message of the calling thread's most recent rejected call ("" if none). */
const char* mi_last_error(void);

/*
 * Experiment knobs, passed per call.  NULL, or a field left 0, selects the default (the measured best
 * on MI355X); they exist for sweeps and tests.  Out-of-range values are rejected (MI_ERR_UNSUPPORTED).
 * Pass the same knobs to a *_workspace_bytes function and to the attention call it sizes.
 */
typedef struct MiTuning {
  int32_t decode_tile_subtiles;   /* decode kernel, 16-token sub-tiles per loop iteration: 0 = automatic, 1, 2, 4 */
  int32_t decode_min_waves;       /* decode kernel, wavefronts per SIMD to compile for: 0 = default (3), 2..4 */
  int32_t decode_wgs_per_cu;      /* decode kernel, workgroups of 8 wavefronts per CU: 0 = default (1), 1..8 */
  int32_t decode_grid;            /* decode kernels, spans the tile sequence is cut into: 0 = automatic, 1..65535 */
  int32_t decode_waves_per_block; /* decode kernel, KV heads per workgroup: 0 = default (8), 1..8 */
  int32_t prefill_two_phase;      /* prefill tile kernel: 0 = default (3), 1 = two-phase kernel, 2 = the same with its
                                     wave groups in lock-step, 3 = one-stream kernel where it applies (head_dim 128 over a
                                     16-bit cache; the two-phase kernel elsewhere), -1 = register-only kernel */
  int32_t prefill_tile_subtiles;  /* register-only prefill kernel, 16-key sub-tiles per iteration: 0 = default (2), 1, 2 */
  int32_t prefill_row_tiles;      /* register-only prefill kernel, 16-row tiles per wavefront: 0 = default (2), 2, 4 */
  int32_t prefill_kv_split;       /* two-phase kernel, key ranges per request: 0 = from T and max_kv_len, -1 = never,
                                     2..64 = forced where the workspace allows it */
  int32_t norm_rope_vectorised;   /* 16-byte-per-lane norm / rotary kernel: 0 = default (from 256 tokens up, where
                                     alignment and rotary width allow), 1 = wherever they allow, -1 = never */
  int32_t mla_decode_lds;         /* multi-latent decode: 0 = default (latent tiles shared through LDS when the chunk
                                     size is a multiple of 64 and the call has at most 768 requests; with a multiple
                                     of 128 query heads and a chunk size that is a multiple of 32, by the kernel of
                                     four wavefronts with 32 heads each), 2 = the eight-wavefront LDS kernel at
                                     every head count, -1 = one streaming wavefront per 16-head group always */
  int32_t reserved[5];            /* must be 0 */
} MiTuning;

/*
 * Kernel timing.  mi_profile_enable(1) makes the attention entry points bracket their main
 * kernel (decode: the KV-streaming kernel; prefill: the tile kernel, followed by a second pair
 * for the decode kernel of a mixed batch when a workspace is passed) with HIP events on the caller's
 * stream; mi_profile_collect waits for
 * the recorded pairs, writes their durations (milliseconds, HOST pointer) and returns how
 * many there were.  Keep it off while capturing a graph.
 */
int mi_profile_enable(int32_t on);
int32_t mi_profile_collect(float* out_ms_host, int32_t capacity);

/*
 * KV-append with explicit per-token slots.
 * Replaces DynamicInferenceContext.append_key_value_cache
 * (megatron/core/inference/contexts/dynamic_context.py:511-545):
 *   k_cache[token_to_chunk_idx[t], token_to_local_pos[t]] = key[t]   (same for value)
 * key/value: `[T, Hkv*d]` rows of `row_elems` contiguous elements, `src_stride_tok`
 * apart.  Pure copy: the cache receives the source bits.  Tokens that share a slot
 * (batch padding routed to the dummy chunk) race; any one of them wins.
 * value == NULL and v_cache == NULL: only the key rows are written -- the latent cache of
 * multi-latent attention, memory_buffer[layer, chunk_idx, local] = kv_concat
 * (dynamic_context.py:533-538), `row_elems` = kv_lora_rank + qk_pos_emb_head_dim.
 */
int mi_kv_append(const void* key, const void* value, int64_t src_stride_tok, void* k_cache,
                 void* v_cache, int64_t kv_stride_chunk, int64_t kv_stride_tok,
                 const int64_t* token_to_chunk_idx, const int64_t* token_to_local_pos, int32_t T,
                 int32_t row_elems, int32_t elem_bytes, void* stream);

/*
 * KV-append for a decode step with the slot computed on the GPU: request r's new
 * token goes to position kv_lens[r]-1 (kv_lens already counts it), i.e. chunk
 * block_table[r][(kv_lens[r]-1) / chunk_tokens], local (kv_lens[r]-1) % chunk_tokens.
 * Same result as mi_kv_append fed with the rows that
 * DynamicInferenceContext.update_requests writes (dynamic_context.py:1283-1296),
 * without materialising them.  Rows with kv_lens[r] <= 0 write nothing.
 */
int mi_kv_append_decode(const void* key, const void* value, int64_t src_stride_tok, void* k_cache,
                        void* v_cache, int64_t kv_stride_chunk, int64_t kv_stride_tok,
                        const int32_t* block_table, int64_t bt_stride, const int32_t* kv_lens,
                        int32_t R, int32_t chunk_tokens, int32_t row_elems, int32_t elem_bytes,
                        void* stream);

/*
 * fp8 KV storage (no counterpart in the reference, whose cache dtype is always
 * params_dtype, dynamic_context.py:195,287-308).  OCP e4m3fn bytes, one fp32 scale
 * per (chunk, KV head), value = byte * scale.
 * mi_kv_quantize_chunks_fp8: whole chunks, scale = amax(chunk-head tile) / 448.
 * mi_kv_append_decode_fp8  : one new token per request; a token that opens a chunk
 *   sets scale = headroom * amax(token) / 448, later tokens reuse it (saturating).
 * `dtype` (MI_DTYPE_BF16 / MI_DTYPE_FP16) is the type of the source rows.
 */
int mi_kv_quantize_chunks_fp8(const void* src, int64_t src_stride_chunk,
                              int64_t src_stride_tok, void* dst_fp8, int64_t dst_stride_chunk,
                              int64_t dst_stride_tok, float* scales, int32_t n_chunks,
                              int32_t chunk_tokens, int32_t Hkv, int32_t head_dim, int32_t dtype,
                              void* stream);

int mi_kv_append_decode_fp8(const void* key, const void* value, int64_t src_stride_tok,
                            void* k_cache_fp8, void* v_cache_fp8, int64_t kv_stride_chunk,
                            int64_t kv_stride_tok, float* k_scales, float* v_scales,
                            const int32_t* block_table, int64_t bt_stride, const int32_t* kv_lens,
                            int32_t R, int32_t chunk_tokens, int32_t Hkv, int32_t head_dim,
                            float headroom, int32_t dtype, void* stream);

/*
 * fp8 append with explicit per-token slots (prefill / mixed steps; no counterpart in the reference).
 * The tokens a call writes into one chunk must be neighbours in the token dimension with rising
 * local positions, as DynamicInferenceContext lays them out (dynamic_context.py:982-1005,1283-1296).
 * A run that starts at local position 0 opens its chunk: scale = amax(run) / 448, times `headroom`
 * unless the run fills the chunk; any other run reuses the stored scale (saturating).
 */
int mi_kv_append_fp8(const void* key, const void* value, int64_t src_stride_tok,
                     void* k_cache_fp8, void* v_cache_fp8, int64_t kv_stride_chunk,
                     int64_t kv_stride_tok, float* k_scales, float* v_scales,
                     const int64_t* token_to_chunk_idx, const int64_t* token_to_local_pos, int32_t T,
                     int32_t chunk_tokens, int32_t Hkv, int32_t head_dim, float headroom, int32_t dtype,
                     void* stream);

/*
 * Bytes of workspace mi_paged_decode_attention needs for these sizes on the current
 * device (partials of the workgroups that share a request + per-request bookkeeping).  The size
 * depends on R, the head counts, head_dim, the device's CU count and the grid knobs of `tuning`;
 * chunk_tokens, max_kv_len and split_tokens are accepted for symmetry with the attention call and
 * do not change it.  -1 = a knob out of range.
 */
int64_t mi_decode_workspace_bytes(int32_t R, int32_t Hq, int32_t Hkv, int32_t head_dim,
                                  int32_t chunk_tokens, int32_t max_kv_len, int32_t split_tokens,
                                  const MiTuning* tuning);

/*
 * Paged GQA decode attention (one query token per request).
 * Replaces flash_attn_with_kvcache(q, k_cache, v_cache, cache_seqlens=kv_lens,
 * causal=True, block_table=...) as called from Attention.flash_decode_and_prefill
 * (megatron/core/transformer/attention.py:589-600):
 *   out[r,h] = softmax(q[r,h] . K_r[:len_r, h/G]^T * softmax_scale) . V_r[:len_r, h/G]
 *   K_r[j] = k_cache[block_table[r, j / chunk_tokens], j % chunk_tokens], G = Hq/Hkv.
 * q/out: bf16 or fp16 `[R, Hq, d]` with the given token / head strides; d 64, 96, 128, 192 or 256 (an fp8 cache:
 * 64 or 128); G any value up to 64 (not only powers of two; every 16 query heads of a KV head take a wavefront).  kv_lens int32 [R] (0 => that row's output is zeros).  `max_kv_len` bounds every kv_lens[r] (the reference
 * passes max_sequence_length here, dynamic_context.py:791); the grid does not depend on
 * it.  `split_tokens` = minimum tokens one workgroup streams (0 = default 64).
 * kv_dtype MI_KV_FP8_E4M3 reads byte caches with k_scales/v_scales `[n_chunks, Hkv]`.
 */
int mi_paged_decode_attention(const void* q, int64_t q_stride_tok, int64_t q_stride_head,
                              const void* k_cache, const void* v_cache, int64_t kv_stride_chunk,
                              int64_t kv_stride_tok, int64_t kv_stride_head,
                              const int32_t* block_table, int64_t bt_stride, const int32_t* kv_lens,
                              void* out, int64_t o_stride_tok, int64_t o_stride_head,
                              void* workspace, int64_t workspace_bytes, int32_t R, int32_t Hq,
                              int32_t Hkv, int32_t head_dim, int32_t chunk_tokens,
                              int32_t max_kv_len, int32_t split_tokens, float softmax_scale,
                              int32_t kv_dtype, const float* k_scales, const float* v_scales,
                              int32_t dtype, const MiTuning* tuning, void* stream);

/*
 * One decode step of a layer in two launches instead of three: what mi_norm_rope_append (or
 * mi_qkv_norm_rope_append) followed by mi_paged_decode_attention computes for R one-token requests, i.e.
 * the sequence q_layernorm / k_layernorm (attention.py:1026-1030), apply_rotary_emb_query / _key
 * (dynamic_context.py:566-631), append_key_value_cache (dynamic_context.py:511-545) and
 * flash_attn_with_kvcache (attention.py:589-600).  The head norm, the rotary embedding and the append of the
 * step's token ride in the streaming kernel: every span of keys prepares its query rows in registers, and the
 * span that ends a request writes the request's new key and value rows into their cache slot
 * (block_table[r, (kv_lens[r] - 1) / chunk_tokens], position (kv_lens[r] - 1) % chunk_tokens) before it reads
 * them.  q holds the RAW queries: head h * G + u of request r at r * q_stride_tok + h * q_stride_group + u * d
 * (a `[R, Hq, d]` tensor: q_stride_group = G * d; the QKV projection's output `[R, Hkv, (G + 2) * d]`:
 * q_stride_group = (G + 2) * d, k_new = q + G * d, v_new = q + (G + 1) * d, both with head stride
 * (G + 2) * d).  positions int64 [R] index rotary_angles; NULL = kv_lens[r] - 1, the position of the step's token
 * in its request (what token_to_pos_ids holds on a decode step, and one load fewer on the way to the first
 * product).  Same arithmetic and rounding points as
 * mi_norm_rope_append (faithful_rounding as there); the normed queries are not written anywhere.
 * Limits: 16-bit caches, head_dim 64, 96, 128, 192 or 256, half-split rotary pairs with rot_dim / 2 a multiple of
 * 32 (or interleaved pairs, or no rotary embedding); anything else is MI_ERR_UNSUPPORTED and takes the separate calls.
 * Workspace as for mi_paged_decode_attention.  Rows with kv_lens[r] == 0 append nothing and produce zeros.
 */
int mi_decode_step_attention(const void* q, int64_t q_stride_tok, int64_t q_stride_group, const void* k_new,
                             int64_t k_stride_tok, int64_t k_stride_head, const void* v_new,
                             int64_t v_stride_tok, int64_t v_stride_head, const void* q_weight,
                             const void* k_weight, float eps, int32_t norm_kind, const float* rotary_angles,
                             int64_t angles_stride, int32_t rot_dim, int32_t rotary_interleaved, float mscale,
                             const int64_t* positions, void* k_cache, void* v_cache, int64_t kv_stride_chunk,
                             int64_t kv_stride_tok, int64_t kv_stride_head, const int32_t* block_table,
                             int64_t bt_stride, const int32_t* kv_lens, void* out, int64_t o_stride_tok,
                             int64_t o_stride_head, void* workspace, int64_t workspace_bytes, int32_t R,
                             int32_t Hq, int32_t Hkv, int32_t head_dim, int32_t chunk_tokens,
                             int32_t split_tokens, float softmax_scale, int32_t faithful_rounding,
                             int32_t dtype, const MiTuning* tuning, void* stream);

/*
 * The same step over an fp8-e4m3 cache (no counterpart in the reference, like the other fp8 entry points): the
 * span that ends a request quantises the step's key row (after head norm and rotary embedding, rounded to bf16
 * first) and value row into their slot with the policy of mi_kv_append_decode_fp8 -- a token that opens a chunk
 * sets that chunk-head's scale to headroom * amax(token) / 448 (1 for an all-zero row) and stores it, later tokens
 * reuse the stored scale and saturate -- and then streams the cache as mi_paged_decode_attention does with
 * kv_dtype MI_KV_FP8_E4M3.  Bytes and scales are those of mi_norm_rope_append (key_out) followed by
 * mi_kv_append_decode_fp8.  Tensors of the 16-bit type `dtype`, head_dim 128; half-split rotary pairs need rot_dim 128
 * (interleaved pairs: any even width).
 */
int mi_decode_step_attention_fp8(const void* q, int64_t q_stride_tok, int64_t q_stride_group, const void* k_new,
                                 int64_t k_stride_tok, int64_t k_stride_head, const void* v_new,
                                 int64_t v_stride_tok, int64_t v_stride_head, const void* q_weight,
                                 const void* k_weight, float eps, int32_t norm_kind, const float* rotary_angles,
                                 int64_t angles_stride, int32_t rot_dim, int32_t rotary_interleaved, float mscale,
                                 const int64_t* positions, void* k_cache_fp8, void* v_cache_fp8,
                                 int64_t kv_stride_chunk, int64_t kv_stride_tok, int64_t kv_stride_head,
                                 float* k_scales, float* v_scales, float headroom, const int32_t* block_table,
                                 int64_t bt_stride, const int32_t* kv_lens, void* out, int64_t o_stride_tok,
                                 int64_t o_stride_head, void* workspace, int64_t workspace_bytes, int32_t R,
                                 int32_t Hq, int32_t Hkv, int32_t head_dim, int32_t chunk_tokens,
                                 int32_t split_tokens, float softmax_scale, int32_t faithful_rounding,
                                 int32_t dtype, const MiTuning* tuning, void* stream);

/*
 * mi_paged_decode_attention for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference.  Same arguments and results as mi_paged_decode_attention, minus the workspace: the
 * partials live in a device array of MI_NOALLOC_SCRATCH_BYTES that is part of the library image
 * (one copy per GPU the library runs on, held until the process ends).  Sizes for which
 * mi_decode_workspace_bytes() exceeds that are rejected with MI_ERR_WORKSPACE.  The call allocates
 * and frees nothing (keep mi_profile_enable off: it creates events).  All calls on one GPU share the
 * array: calls that overlap on one GPU (two streams, two host threads) race; calls on one stream
 * are ordered and need no clearing in between.  The first call on a device looks the array's
 * address up (hipGetSymbolAddress), so make it before a stream capture starts.
 */
#define MI_NOALLOC_SCRATCH_BYTES (16 * 1024 * 1024)
int mi_paged_decode_attention_noalloc(const void* q, int64_t q_stride_tok, int64_t q_stride_head,
                                      const void* k_cache, const void* v_cache, int64_t kv_stride_chunk,
                                      int64_t kv_stride_tok, int64_t kv_stride_head,
                                      const int32_t* block_table, int64_t bt_stride,
                                      const int32_t* kv_lens, void* out, int64_t o_stride_tok,
                                      int64_t o_stride_head, int32_t R, int32_t Hq, int32_t Hkv,
                                      int32_t head_dim, int32_t chunk_tokens, int32_t max_kv_len,
                                      int32_t split_tokens, float softmax_scale, int32_t kv_dtype,
                                      const float* k_scales, const float* v_scales, int32_t dtype, const MiTuning* tuning, void* stream);

/*
 * Decode attention over the latent cache of multi-latent attention (absorbed form).
 * Replaces flash_mla_with_kvcache(q, kv_cache.unsqueeze(-2), block_table, cache_seqlens, head_dim_v,
 * tile_scheduler_metadata, num_splits, softmax_scale=, causal=True) together with get_mla_metadata
 * as called from Attention.flash_decode_and_prefill
 * (megatron/core/transformer/attention.py:561-587): the cache holds one row of head_dim_k = 576
 * values per token (kv_lora_rank 512 + rotary 64; dynamic_context.py:288-294,533-538), shared by
 * all query heads:
 *   out[r,h] = softmax(q[r,h] . KV_r[:len_r, :576]^T * softmax_scale) . KV_r[:len_r, :512]
 * q bf16 `[R, Hq, 576]`, out bf16 `[R, Hq, 512]`, kv_cache bf16 `[n_chunks, chunk_tokens, 576]` with
 * the given chunk / token strides (elements).  Hq: 1, 2, 4, 8 or a multiple of 16.
 */
int64_t mi_mla_decode_workspace_bytes(int32_t R, int32_t Hq, int32_t head_dim_v, const MiTuning* tuning);

int mi_paged_mla_decode_attention(const void* q, int64_t q_stride_tok, int64_t q_stride_head,
                                  const void* kv_cache, int64_t kv_stride_chunk, int64_t kv_stride_tok,
                                  const int32_t* block_table, int64_t bt_stride, const int32_t* kv_lens,
                                  void* out, int64_t o_stride_tok, int64_t o_stride_head, void* workspace,
                                  int64_t workspace_bytes, int32_t R, int32_t Hq, int32_t head_dim_k,
                                  int32_t head_dim_v, int32_t chunk_tokens, int32_t max_kv_len,
                                  float softmax_scale, int32_t dtype, const MiTuning* tuning, void* stream);

/*
 * Paged varlen causal attention for prefill / mixed prefill+decode batches.
 * Replaces flash_attn_varlen_func(q, k_cache, v_cache, cu_seqlens_q, cu_seqlens_k,
 * max_seqlen_q, max_seqlen_k, softmax_scale, causal=True, block_table=...)
 * (megatron/core/transformer/attention.py:546-557): request r owns query rows
 * cu_seqlens_q[r]..cu_seqlens_q[r+1]-1 and kv_lens[r] keys; query i of Lq sees keys
 * j <= i + (Lk - Lq) (bottom-right aligned causal mask).  Rows past cu_seqlens_q[R] (token
 * padding) are zeroed.  head_dim 64, 96, 128, 192 or 256; Hq / Hkv any value up to 64 (3, 5, 7 ... included; every
 * 16 query heads of a KV head take workgroups of their own).
 * With a workspace of mi_prefill_workspace_bytes() bytes, requests that
 * have exactly one query row (the decode requests of a mixed batch) are streamed by the
 * decode kernels at full bandwidth; with workspace == NULL one kernel handles every request.
 * The same workspace lets the two-phase tile kernel (chunk size a multiple of 64; other
 * chunk sizes run a register-only kernel) cut the keys of every request into ranges when
 * the batch has few query rows over long contexts (a chunk of a prompt, a short turn after a long
 * history: without it a handful of workgroups would walk thousands of keys each): the ranges are
 * computed by separate workgroups and merged by log-sum-exp, as in the decode path.  `max_kv_len` (an
 * upper bound of kv_lens; 0 = unknown, no splitting) and T decide the number of ranges, so pass the same
 * values to mi_prefill_workspace_bytes and to the attention call.
 */
int64_t mi_prefill_workspace_bytes(int32_t T, int32_t R, int32_t Hq, int32_t Hkv, int32_t head_dim,
                                   int32_t max_kv_len, int32_t split_tokens, const MiTuning* tuning);

int mi_paged_prefill_attention(const void* q, int64_t q_stride_tok, int64_t q_stride_head,
                               const void* k_cache, const void* v_cache, int64_t kv_stride_chunk,
                               int64_t kv_stride_tok, int64_t kv_stride_head,
                               const int32_t* block_table, int64_t bt_stride,
                               const int32_t* cu_seqlens_q, const int32_t* kv_lens, void* out,
                               int64_t o_stride_tok, int64_t o_stride_head, void* workspace,
                               int64_t workspace_bytes, int32_t T, int32_t R, int32_t Hq,
                               int32_t Hkv, int32_t head_dim, int32_t chunk_tokens,
                               int32_t max_kv_len, int32_t split_tokens, float softmax_scale,
                               int32_t dtype, const MiTuning* tuning, void* stream);

/*
 * The same call over an fp8-e4m3 cache (byte caches `[n_chunks, chunk_tokens, Hkv, d]`, strides in
 * elements = bytes, fp32 scales `[n_chunks, Hkv]`; no counterpart in the reference).  Tiles are
 * multiplied by their chunk's scale and rounded to bf16 on their way into LDS.  Needs head_dim 64
 * or 128 and a chunk size that is a multiple of 64; `dtype` is the type of q / out (and of the staged tiles).
 */
int mi_paged_prefill_attention_fp8(const void* q, int64_t q_stride_tok, int64_t q_stride_head,
                                   const void* k_cache_fp8, const void* v_cache_fp8,
                                   int64_t kv_stride_chunk, int64_t kv_stride_tok,
                                   int64_t kv_stride_head, const float* k_scales,
                                   const float* v_scales, const int32_t* block_table,
                                   int64_t bt_stride, const int32_t* cu_seqlens_q,
                                   const int32_t* kv_lens, void* out, int64_t o_stride_tok,
                                   int64_t o_stride_head, void* workspace, int64_t workspace_bytes,
                                   int32_t T, int32_t R, int32_t Hq, int32_t Hkv, int32_t head_dim,
                                   int32_t chunk_tokens, int32_t max_kv_len, int32_t split_tokens,
                                   float softmax_scale, int32_t dtype, const MiTuning* tuning,
                                   void* stream);

/*
 * Paged varlen causal attention with keys wider than values: the prefill / mixed step of
 * multi-latent attention, where the reference decompresses the latent cache into a key cache
 * `[n_chunks, chunk_tokens, H, 192]` (128 + the 64 shared rotary values) and a value cache
 * `[.., H, 128]` (MLASelfAttention.uncompress_kv_from_cache,
 * megatron/core/transformer/multi_latent_attention.py:801-825, called from
 * attention.py:406-411) and hands them to flash_attn_varlen_func (attention.py:546-557).
 * Same mask and padding rules as mi_paged_prefill_attention; each cache has its own strides
 * (elements); q `[T, Hq, 192]`, out `[T, Hq, 128]`.  One kernel serves every request: the
 * two-phase LDS-tiled kernel when chunk_tokens is a multiple of 64 (and the knob prefill_pingpong
 * is not 0), a register-only kernel otherwise.  `workspace` may be NULL; one of
 * mi_prefill_workspace_bytes(T, R, Hq, Hkv, head_dim_v, max_kv_len, 0) bytes (256-byte aligned) lets
 * the two-phase kernel cut the keys of every request into ranges when few query rows meet long
 * contexts, as in mi_paged_prefill_attention (`max_kv_len` bounds every kv_lens[r]; it only sizes
 * that split).
 */
int mi_paged_prefill_attention_mla(const void* q, int64_t q_stride_tok, int64_t q_stride_head,
                                   const void* k_cache, int64_t k_stride_chunk, int64_t k_stride_tok,
                                   int64_t k_stride_head, const void* v_cache, int64_t v_stride_chunk,
                                   int64_t v_stride_tok, int64_t v_stride_head,
                                   const int32_t* block_table, int64_t bt_stride,
                                   const int32_t* cu_seqlens_q, const int32_t* kv_lens, void* out,
                                   int64_t o_stride_tok, int64_t o_stride_head, void* workspace,
                                   int64_t workspace_bytes, int32_t T, int32_t R, int32_t Hq, int32_t Hkv,
                                   int32_t head_dim_k, int32_t head_dim_v, int32_t chunk_tokens,
                                   int32_t max_kv_len, float softmax_scale, int32_t dtype, const MiTuning* tuning, void* stream);

/*
 * Fused q/k head norm + rotary embedding (+ KV-append when k_cache is given).
 * Replaces, per layer, q_layernorm/k_layernorm
 * (megatron/core/transformer/attention.py:1026-1030), apply_rotary_emb_key /
 * apply_rotary_emb_query (dynamic_context.py:566-631 ->
 * megatron/core/models/common/embeddings/rope_utils.py:92-126) and, optionally,
 * append_key_value_cache (dynamic_context.py:511-545).
 *  q `[T,Hq,d]` bf16 is read and the result written to q_out (which may be q itself);
 *  k `[T,Hkv,d]` is read, the result goes to k_out (if non-null) and to the cache slot
 *  (if k_cache non-null, together with v).
 *  norm_kind: MI_NORM_NONE | MI_NORM_RMS (weights bf16 [d], may be null) | MI_NORM_L2.
 *  rotary_angles: fp32 `[max_pos, rot_dim]` table of angles as built by
 *  RotaryEmbedding.forward (rotary_pos_embedding.py:151-181), null = no rotary;
 *  q_positions / k_positions int64 [T] index it.  rot_dim < head_dim leaves the tail
 *  unrotated.  Cache slots: token_to_chunk_idx/token_to_local_pos (int64 [T]) if
 *  given, else block_table + kv_lens as in mi_kv_append_decode (then T == R).
 *  faithful_rounding != 0 rounds to bf16 wherever the unfused bf16 op chain does.
 */
int mi_norm_rope_append(const void* q, int64_t q_stride_tok, void* q_out, int64_t q_out_stride_tok,
                        const void* k, int64_t k_stride_tok, void* k_out, int64_t k_out_stride_tok, const void* v, int64_t v_stride_tok,
                        const void* q_weight, const void* k_weight, float eps, int32_t norm_kind,
                        const float* rotary_angles, int64_t angles_stride, int32_t rot_dim,
                        int32_t rotary_interleaved, float mscale, const int64_t* q_positions,
                        const int64_t* k_positions, void* k_cache, void* v_cache,
                        int64_t kv_stride_chunk, int64_t kv_stride_tok,
                        const int64_t* token_to_chunk_idx, const int64_t* token_to_local_pos,
                        const int32_t* block_table, int64_t bt_stride, const int32_t* kv_lens,
                        int32_t chunk_tokens, int32_t T, int32_t Hq, int32_t Hkv, int32_t head_dim,
                        int32_t faithful_rounding, int32_t dtype, const MiTuning* tuning, void* stream);

/*
 * The same launch reading the QKV projection's output directly: replaces the split of
 * SelfAttention.get_query_key_value_tensors (megatron/core/transformer/attention.py:985-1030:
 * view `[T, Hkv, (Hq/Hkv + 2) * d]`, split into G = Hq/Hkv query heads, one key head and one
 * value head per query group, reshape of the query to `[T, Hq, d]`) together with everything
 * mi_norm_rope_append replaces.  mixed_qkv is bf16 `[T][Hkv][(G + 2) * d]` with token stride
 * qkv_stride_tok (elements); the normed / rotated query goes to q_out `[T, Hq, d]`, the key to
 * k_out (if non-null) and to the cache slot (if k_cache non-null, together with the value
 * heads); at least one key destination is required.  Remaining arguments as above.
 */
int mi_qkv_norm_rope_append(const void* mixed_qkv, int64_t qkv_stride_tok, void* q_out,
                            int64_t q_out_stride_tok, void* k_out, int64_t k_out_stride_tok,
                            const void* q_weight, const void* k_weight, float eps, int32_t norm_kind,
                            const float* rotary_angles, int64_t angles_stride, int32_t rot_dim,
                            int32_t rotary_interleaved, float mscale, const int64_t* q_positions,
                            const int64_t* k_positions, void* k_cache, void* v_cache,
                            int64_t kv_stride_chunk, int64_t kv_stride_tok,
                            const int64_t* token_to_chunk_idx, const int64_t* token_to_local_pos,
                            const int32_t* block_table, int64_t bt_stride, const int32_t* kv_lens,
                            int32_t chunk_tokens, int32_t T, int32_t Hq, int32_t Hkv, int32_t head_dim,
                            int32_t faithful_rounding, int32_t dtype, const MiTuning* tuning, void* stream);

/*
 * DynamicInferenceContext.update_requests as one kernel
 * (megatron/core/inference/contexts/dynamic_context.py:1033-1298, allocator
 * dynamic_chunk_allocator.py:56-86): same order of chunk releases, row moves, pauses, LIFO
 * resumes and per-token row rewrites, so every state tensor ends up as the reference leaves
 * it.  All state pointers are the context's own tensors (int32 request rows, int64 token rows,
 * int32 chunk table with `table_stride` elements per row, int32 chunk stack).
 * `active_requests_mask` int32 [total - paused], `new_tokens` int64 [total - paused];
 * `paused_tokens` int64 [max_requests] holds the tokens of the paused rows on entry and on exit;
 * `next_tokens_scratch` int64 [max_requests], `scratch` int32 [4 * max_requests].
 * Results: `newly_paused_request_ids` int32 [max_requests], `finished_request_ids` int32
 * [max_requests] (the ids of the requests whose mask entry is 0, in row order -- what
 * TextGenerationController.async_generate_output_tokens_dynamic_batch reads with nonzero + index at
 * text_generation_controller.py:527-530) and `counters` int32 [8] =
 * {total_request_count, paused_request_count, active_token_count, chunk_count_avail,
 *  number of newly paused ids (-1 = none), status (0 ok, 1 mask/count mismatch - nothing was
 *  changed, 2 no active request left, 3 resumed request not at a chunk start), 1 if the context
 *  was emptied, number of finished ids}; the caller copies `counters` to the host after the call.
 */
int mi_update_requests(int32_t* request_ids, int32_t* request_query_lengths,
                       int32_t* request_output_lengths, int32_t* request_kv_length_offsets,
                       int32_t* request_kv_chunk_counts, int32_t* request_last_kv_chunk_id,
                       int32_t* request_last_kv_chunk_offset, int32_t* request_to_kv_chunk_ids,
                       int64_t table_stride, int32_t max_kv_chunk_count, int64_t* token_to_input_ids,
                       int64_t* token_to_pos_ids, int64_t* token_to_request_idx,
                       int64_t* token_to_position_in_request, int64_t* token_to_chunk_idx,
                       int64_t* token_to_local_position_within_kv_chunk, int32_t* chunk_bag,
                       const int32_t* active_requests_mask, const int64_t* new_tokens,
                       int64_t* paused_tokens, int64_t* next_tokens_scratch, int32_t* scratch,
                       int32_t* newly_paused_request_ids, int32_t* finished_request_ids,
                       int32_t* counters, int32_t total_request_count, int32_t paused_request_count,
                       int32_t chunk_count_avail, int32_t gtd_chunk_count, int32_t gtd_request_count,
                       int32_t chunk_size_tokens, int32_t max_requests, void* stream);

/*
 * The tensor writes of DynamicInferenceContext.add_request (dynamic_context.py:976-1015) as one kernel, after
 * the caller has made the reference's host-side checks (token / request / chunk / sequence-length overflow,
 * dynamic_context.py:945-974) and lowered the allocator's count by `chunk_count`: the request's row of every
 * per-request tensor, the first `chunk_count` entries of its chunk-table row = chunk_bag[stack_first ..
 * stack_first + chunk_count - 1] (the ids the allocator hands out, in stack order; stack_first = the
 * allocator's count after the pop), and the rows token_begin .. token_begin + prompt_length - 1 of the per-token
 * tensors (input id, position, request row, position in request, chunk, position in chunk).  prompt_tokens int64
 * [prompt_length] on the device.
 */
int mi_add_request(int32_t* request_ids, int32_t* request_query_lengths, int32_t* request_output_lengths,
                   int32_t* request_kv_length_offsets, int32_t* request_kv_chunk_counts,
                   int32_t* request_last_kv_chunk_id, int32_t* request_last_kv_chunk_offset,
                   int32_t* request_to_kv_chunk_ids, int64_t table_stride, int64_t* token_to_input_ids,
                   int64_t* token_to_pos_ids, int64_t* token_to_request_idx,
                   int64_t* token_to_position_in_request, int64_t* token_to_chunk_idx,
                   int64_t* token_to_local_position_within_kv_chunk, const int32_t* chunk_bag,
                   const int64_t* prompt_tokens, int32_t request_row, int32_t token_begin,
                   int32_t prompt_length, int32_t chunk_count, int32_t stack_first, int32_t chunk_size_tokens,
                   int32_t request_id, int32_t output_length, void* stream);

/*
 * The decode-only part of DynamicInferenceContext.initialize_attention_state
 * (dynamic_context.py:733-741, 747-750, 785-787, 816-818) as one kernel: copies query lengths,
 * kv lengths (offset + query length) and block-table rows of the active requests into the
 * fixed-address mirrors, and points the padded token rows at the dummy chunk.  The mirrors'
 * padded rows must already be zero (reset_attention_state does that).
 */
int mi_decode_attention_state(const int32_t* request_kv_length_offsets,
                              const int32_t* request_query_lengths,
                              const int32_t* request_to_kv_chunk_ids, int64_t table_stride,
                              int32_t max_kv_chunk_count, int32_t* query_seq_lengths_out,
                              int32_t* kv_seq_lengths_out, int32_t* block_table_out,
                              int64_t block_table_out_stride, int64_t* token_to_chunk_idx,
                              int64_t* token_to_local_position_within_kv_chunk,
                              int64_t* token_to_position_in_request, int32_t paused_request_count,
                              int32_t active_request_count, int32_t active_token_count,
                              int32_t padded_active_token_count, int32_t dummy_chunk_idx,
                              void* stream);

/*
 * The prefill / mixed-step part of DynamicInferenceContext.initialize_attention_state
 * (dynamic_context.py:733-741, 752-775, 794-821) as one kernel: everything mi_decode_attention_state
 * writes, plus cu_query_seq_lengths_out / cu_kv_seq_lengths_out int32 [padded_request_count + 1] (running
 * sums of the query and kv lengths; padded requests add nothing) and max_lengths_out int32 [2] = {largest
 * query length, largest kv length} -- the two values the reference fetches with `.max().item()`
 * (:772, :808).  The mirrors' padded rows must already be zero.
 */
int mi_step_attention_state(const int32_t* request_kv_length_offsets,
                            const int32_t* request_query_lengths,
                            const int32_t* request_to_kv_chunk_ids, int64_t table_stride,
                            int32_t max_kv_chunk_count, int32_t* query_seq_lengths_out,
                            int32_t* kv_seq_lengths_out, int32_t* cu_query_seq_lengths_out,
                            int32_t* cu_kv_seq_lengths_out, int32_t* block_table_out,
                            int64_t block_table_out_stride, int64_t* token_to_chunk_idx,
                            int64_t* token_to_local_position_within_kv_chunk,
                            int64_t* token_to_position_in_request, int32_t* max_lengths_out,
                            int32_t paused_request_count, int32_t active_request_count,
                            int32_t padded_request_count, int32_t active_token_count,
                            int32_t padded_active_token_count, int32_t dummy_chunk_idx, void* stream);

/*
 * DynamicInferenceContext.last_token_logits (dynamic_context.py:890-918) as one launch:
 *   dst[r] = src[cumsum(request_query_lengths)[r] - 1],  r < R
 * with the running sum taken on the GPU.  src `[T, row_elems]`, dst `[R, row_elems]`, row strides
 * in elements, 2- or 4-byte elements (logits or hidden states); request_query_lengths points at
 * the first ACTIVE request's entry.  A bit-exact row copy.
 */
int mi_last_token_gather(const void* src, int64_t src_stride_row, void* dst, int64_t dst_stride_row,
                         const int32_t* request_query_lengths, int32_t R, int32_t row_elems,
                         int32_t elem_bytes, void* stream);

/*
 * The arithmetic of DynamicInferenceContext.calculate_log_probs (dynamic_context.py:1300-1365):
 *   log_probs[t] = log_softmax(float(logits[t, :]))[token_ids[t]],  t < T
 * without materialising the `[T, vocab]` fp32 log-softmax matrix: one read of each row.  logits
 * `[T, vocab]` fp32 (0), bf16 (1) or fp16 (2), row stride in elements; token_ids int64 `[T]` (the caller builds
 * them as the reference does: the prompt token that follows each position, the newly sampled token at
 * the last position of each request); an id outside [0, vocab) yields NaN.  fp32 results.
 */
int mi_selected_log_probs(const void* logits, int64_t stride_row, int32_t logits_dtype, int32_t T,
                          int32_t vocab, const int64_t* token_ids, float* log_probs, void* stream);

/*
 * TextGenerationController.sample_from_logits and the finished-request test that follows it
 * (megatron/core/inference/text_generation_controllers/text_generation_controller.py:172-315,
 * 519-530) as one launch, one workgroup per row of `logits` `[R, vocab]` (logits_dtype 0 = fp32,
 * 1 = bf16, 2 = fp16; row stride in elements):
 *   top_k == 1             : samples[r] = argmax (lowest index among equal maxima);
 *   otherwise              : x = logits * (1 / temperature) (rounded to the logits' type for 16-bit logits, as the
 *                            reference's in-place division rounds), then
 *     top_k > 1            : keep x >= the top_k-th largest value (ties kept, as `logits < kth`),
 *     top_p > 0 (top_k 0)  : order by value, keep the shortest prefix whose softmax mass exceeds
 *                            top_p (the reference's shifted `cumsum > top_p` rule); values equal to
 *                            the last kept one are all kept (the reference keeps an unspecified
 *                            subset of them, torch.sort being unstable),
 *     softmax over the kept values and ONE draw by inverse CDF in vocabulary order:
 *     samples[r] = min{ j : sum_{i<=j} p_i > uniform[r] * sum_i p_i },  uniform[r] in [0, 1)
 *     (the reference draws with torch.multinomial from its own generator: same distribution,
 *     different stream of random numbers), clamped to [0, vocab_clamp-1] when vocab_clamp > 0.
 *   Probability mass is summed as fixed point (each term rounded to 2^-32), so a call is reproducible bit for bit.
 *   cut_values (optional, fp32 [R]) receives the smallest kept value (-inf: nothing filtered).
 *   active_request_mask (optional, uint8 [R]) = (samples[r] != termination_id) &&
 *     (request_kv_length_offsets[r] + request_query_lengths[r] + 1 < request_output_lengths[r]);
 *     the three length rows (optional, all or none) point at the first ACTIVE request's entries.
 *   A row whose maximum is not finite yields its argmax.
 */
int mi_sample_from_logits(const void* logits, int64_t stride_row, int32_t logits_dtype, int32_t R,
                          int32_t vocab, int32_t top_k, float top_p, float temperature,
                          const float* uniform, int32_t vocab_clamp, int64_t* samples,
                          float* cut_values, const int32_t* request_kv_length_offsets,
                          const int32_t* request_query_lengths,
                          const int32_t* request_output_lengths, int64_t termination_id,
                          uint8_t* active_request_mask, void* stream);

/*
 * The projections either side of the attention path at decode size (at most 256 tokens a call):
 *   y[T, N] = x[T, K] . W[N, K]^T (+ bias[N]),   16-bit x / W / bias / y, fp32 accumulation.
 * The weight matrix is streamed from HBM once (it is the traffic: 50 MB for 4096 -> 6144), its rows riding
 * through the matrix cores; K is cut into slices of at most 512 columns whose fp32 partial sums [slice][T][N]
 * live in the caller's workspace and are added in a fixed order by a second small launch (results do not depend
 * on timing).  N a multiple of 16, K a multiple of 32; x, W and y rows 16-byte aligned (y: 8-byte).
 *
 * mi_linear_qkv_decode_step replaces `mixed_qkv, _ = self.linear_qkv(hidden_states)` of
 * Attention.get_query_key_value_tensors (megatron/core/transformer/attention.py:985-992; ColumnParallelLinear at
 * tensor-parallel size 1, megatron/core/tensor_parallel/layers.py:946-1010): qkv_weight is
 * `[(Hq + 2 Hkv) d, hidden]` with the rows of KV group h laid out as [G query heads | key | value], so mixed_qkv
 * is the `[T, Hkv, (G + 2) d]` tensor that mi_decode_step_attention and mi_qkv_norm_rope_append read as it is:
 * the split, q / k head norm, rotary embedding and cache append of attention.py:994-1030 and :394-414 then run in
 * THEIR prologue, and no per-head q / k / v tensor is ever written.
 *
 * mi_attention_out_linear_proj replaces `output, bias = self.linear_proj(core_attn_out)` (attention.py:829-845;
 * RowParallelLinear with skip_bias_add, layers.py:1225-1290: the bias is handed back to the caller, not added):
 * core_attn_out is the `[T, Hq d]` output of the attention call, proj_weight `[hidden, Hq d]`.
 *
 * mi_linear_decode is the product itself, for any (N, K) within the limits above.
 */
int64_t mi_linear_decode_workspace_bytes(int32_t T, int32_t N, int32_t K);

int mi_linear_decode(const void* x, int64_t x_stride_tok, const void* weight, int64_t w_stride_row,
                     const void* bias, void* out, int64_t out_stride_tok, void* workspace,
                     int64_t workspace_bytes, int32_t T, int32_t N, int32_t K, int32_t dtype, void* stream);

int mi_linear_qkv_decode_step(const void* hidden_states, int64_t x_stride_tok, const void* qkv_weight,
                              int64_t w_stride_row, const void* qkv_bias, void* mixed_qkv,
                              int64_t out_stride_tok, void* workspace, int64_t workspace_bytes, int32_t T,
                              int32_t hidden_size, int32_t Hq, int32_t Hkv, int32_t head_dim, int32_t dtype,
                              void* stream);

int mi_attention_out_linear_proj(const void* core_attn_out, int64_t x_stride_tok, const void* proj_weight,
                                 int64_t w_stride_row, void* output, int64_t out_stride_tok, void* workspace,
                                 int64_t workspace_bytes, int32_t T, int32_t hidden_size, int32_t Hq,
                                 int32_t head_dim, int32_t dtype, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* MI355_DECODE_H */
