// Arguments and head mapping shared by the paged varlen prefill kernels (paged_prefill.hip,
// paged_prefill_woven.hip).
#pragma once

#include "mi_common.h"

namespace mi {

struct PrefillParams {
  const uint16_t* q;
  int64_t q_st, q_sh;
  const uint8_t* kc;
  const uint8_t* vc;
  int64_t kv_sc;
  int32_t kv_st, kv_sh;
  int64_t v_sc;          // value cache strides (register-only kernel; equal to the key cache's otherwise)
  int32_t v_st, v_sh;
  const int32_t* bt;
  int64_t bt_stride;
  const int32_t* cu_q;
  const int32_t* lens;
  uint16_t* out;
  int64_t o_st, o_sh;
  uint64_t chunk_magic;  // ceil(2^40 / chunk)
  int32_t T, R, Hq, Hkv, G, g_magic, chunk;  // g_magic = 65536 / G + 1: (n * g_magic) >> 16 == n / G for n <= 64, G <= 16
  int32_t parts;         // workgroups per KV head along the query heads: each takes up to 16 of the G that share it
  int32_t skip_single;  // requests with exactly one query row are handled by the decode kernels
  float scale_log2;
  const float* k_scale;  // fp8 KV only: [n_chunks][Hkv]
  const float* v_scale;
  // Two-phase tile kernel only: the keys of a request cut into gridDim.y ranges, one workgroup each;
  // with more than one range the workgroups write fp32 partials [range][T][Hq][128] and their
  // log-sum-exps [range][T][Hq] (log2 domain) and a merge kernel finishes the rows.
  float* split_o;
  float* split_lse;
};

// The query heads one workgroup serves: with at most 16 query heads per KV head, all G of KV head `hv`; with more,
// `parts` workgroups share a KV head and take 16 query heads each (the last one the rest).
struct HeadSlice {
  int h;        // KV head
  int hq0;      // first query head
  int G;        // query heads (1..16)
  int g_magic;  // 65536 / G + 1
};
static __device__ __forceinline__ HeadSlice head_slice(const PrefillParams& p, int hv) {
  HeadSlice s;
  if (p.parts <= 1) {
    s.h = hv; s.hq0 = hv * p.G; s.G = p.G; s.g_magic = p.g_magic;
  } else {
    s.h = hv / p.parts;
    const int part = hv - s.h * p.parts;
    s.hq0 = s.h * p.G + 16 * part;
    s.G = min(16, p.G - 16 * part);
    s.g_magic = 65536 / s.G + 1;
  }
  return s;
}

// The one-stream ("woven") tile kernel for head_dim 128 over 16-bit caches (paged_prefill_woven.hip).  Same grid
// and request -> workgroup map as the two-phase tile kernel: `grid.x` workgroups of 512 threads, `grid.y` key
// ranges (with more than one, `p.split_o` / `p.split_lse` receive the partials).
void launch_prefill_woven(const PrefillParams& p, dim3 grid, bool f16, hipStream_t stream);

}  // namespace mi
