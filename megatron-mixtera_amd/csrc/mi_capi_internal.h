// Host-side plumbing shared by the C-ABI entry points: error codes, the
// per-thread error message, launch checking and the tuning knobs.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

// Return codes (MI_OK, MI_ERR_*), KV storage formats (MI_KV_*), norm kinds (MI_NORM_*) and the prototype
// of every entry point come from the public header, so a definition that drifts from its declaration
// does not compile.
#include "mi355_decode.h"

// The caller's knobs with every default filled in (a null pointer = all defaults): after this call no field
// is 0 unless 0 is a value of its own (decode_tile_subtiles, decode_grid: 0 = automatic).  "Off" settings
// arrive as -1 and stay -1.  Returns MI_OK, or MI_ERR_UNSUPPORTED with a message for an out-of-range value.
int mi_resolve_tuning(const MiTuning* given, MiTuning* out, const char* who);

int mi_fail(int code, const char* msg);
int mi_check_launch(const char* where);
// Next start/stop event pair when kernel timing is enabled (see mi_profile_enable).
bool mi_profile_next(hipEvent_t* start, hipEvent_t* stop);
// Whether kernel timing is switched on (timed launches may create events, which allocates).
bool mi_profile_is_on();

namespace mi {
int decode_grid_size(int Hq, int Hkv, const MiTuning& tune);
// What a fused decode step hands the streaming kernel beside the attention arguments (see mi_decode_step_attention).
struct FusedStepArgs {
  int64_t q_stride_group;  // elements between the query-head groups of two KV heads (heads of a group are contiguous)
  const void* k_new;
  int64_t k_stride_tok, k_stride_head;
  const void* v_new;
  int64_t v_stride_tok, v_stride_head;
  const void* q_weight;
  const void* k_weight;
  float eps;
  int32_t norm_kind;
  const float* rotary_angles;
  int64_t angles_stride;
  int32_t rot_dim, rotary_interleaved;
  float mscale;
  const int64_t* positions;
  int32_t faithful_rounding;
  float fp8_headroom;  // fp8 cache: scale of a chunk the step's token opens = headroom * amax(token) / 448
};
// Shared by the decode entry point and by the mixed-batch path of the prefill entry point
// (cu_seqlens_q non-null: only requests with one query row take part, at row cu_seqlens_q[r]).
// The workspace checks of launch_paged_decode alone (size for R requests, alignment), for callers that must know
// the decode launches can go ahead before they enqueue anything else.  MI_OK or a negative code with a message.
int check_decode_workspace(const void* workspace, int64_t workspace_bytes, int32_t R, int32_t Hq, int32_t Hkv,
                           int32_t head_dim, int32_t split_tokens, const MiTuning& tune, const char* who);
int launch_paged_decode(const void* q, int64_t q_stride_tok, int64_t q_stride_head, const void* k_cache,
                        const void* v_cache, int64_t kv_stride_chunk, int64_t kv_stride_tok,
                        int64_t kv_stride_head, const int32_t* block_table, int64_t bt_stride,
                        const int32_t* kv_lens, const int32_t* cu_seqlens_q, void* out, int64_t o_stride_tok,
                        int64_t o_stride_head, void* workspace, int64_t workspace_bytes, int32_t R, int32_t Hq,
                        int32_t Hkv, int32_t head_dim, int32_t chunk_tokens, int32_t split_tokens,
                        float softmax_scale, int32_t kv_dtype, const float* k_scales, const float* v_scales,
                        int32_t dtype, const MiTuning& tune, void* stream, const FusedStepArgs* fused = nullptr);
}
