// Host-side plumbing shared by the C-ABI entry points: error codes, the
// per-thread error message, launch checking and the tuning knobs.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

// Return codes (MI_OK, MI_ERR_*), KV storage formats (MI_KV_*), norm kinds (MI_NORM_*) and the prototype
// of every entry point come from the public header, so a definition that drifts from its declaration
// does not compile.
#include "mi355_decode.h"

struct MiTuning {
  int decode_tile_subtiles;  // 16-token sub-tiles per loop iteration of the decode kernel: 0 = automatic, 1, 2, 4 (fp8)
  int prefill_tile_subtiles;
  int prefill_lds_row_tiles;   // LDS-shared prefill kernel (head_dim 128): 16-row tiles per wave, 2 or 3; 0 = off
  int prefill_row_tiles;       // 16-row tiles per wave in the prefill kernel: 2 (8 waves) or 4 (4 waves)
  int decode_min_waves;        // occupancy target of the decode kernel, waves per SIMD: 2, 3 or 4
  int decode_wgs_per_cu;       // decode workgroups (of 8 waves) per CU in the streaming grid
  int decode_grid;             // >0 forces the streaming grid size (tests)
  int decode_waves_per_block;  // cap on wavefronts (= KV heads) per decode workgroup, 1..8
  int norm_rope_vectorised;    // 16-byte-per-lane norm/RoPE kernel: 1 = whenever shapes allow, 2 = and T >= 256 (default), 0 = never
  int mla_decode_lds;          // MLA decode: 1 = latent tile shared through LDS when the chunk size allows, 0 = per-wavefront streaming
  int prefill_kv_split;        // two-phase prefill kernel: key ranges per request, 1 = automatic (default), 0 = never, n > 1 = forced
  int prefill_pingpong;        // head_dim-128 prefill: 1 = two wave groups one phase apart, 2 = same kernel in lock-step, 0 = off
};

MiTuning& mi_tuning();
int mi_fail(int code, const char* msg);
int mi_check_launch(const char* where);
// Next start/stop event pair when kernel timing is enabled (see mi_profile_enable).
bool mi_profile_next(hipEvent_t* start, hipEvent_t* stop);

namespace mi {
int decode_grid_size(int Hkv);
// Shared by the decode entry point and by the mixed-batch path of the prefill entry point
// (cu_seqlens_q non-null: only requests with one query row take part, at row cu_seqlens_q[r]).
int launch_paged_decode(const void* q, int64_t q_stride_tok, int64_t q_stride_head, const void* k_cache,
                        const void* v_cache, int64_t kv_stride_chunk, int64_t kv_stride_tok,
                        int64_t kv_stride_head, const int32_t* block_table, int64_t bt_stride,
                        const int32_t* kv_lens, const int32_t* cu_seqlens_q, void* out, int64_t o_stride_tok,
                        int64_t o_stride_head, void* workspace, int64_t workspace_bytes, int32_t R, int32_t Hq,
                        int32_t Hkv, int32_t head_dim, int32_t chunk_tokens, int32_t split_tokens,
                        float softmax_scale, int32_t kv_dtype, const float* k_scales, const float* v_scales,
                        void* stream);
}
