/*
 * C99 consumer of include/mi355_decode.h: compiled with -std=c99 -pedantic -Wall -Wextra -Werror and
 * linked against libmi355_decode.so by tests/test_capi_library.py.  It takes the address of every entry
 * point through a pointer of the declared type (so the header must parse as C and every symbol must
 * exist in the library) and makes the calls that need no GPU.
 */
#include <stdio.h>
#include <string.h>

#include "mi355_decode.h"

int main(void) {
  /* every declared entry point, taken through a function pointer of its declared type */
  int (*p_version)(void) = mi_version;
  const char* (*p_error)(void) = mi_last_error;
  const void* table[] = {
      (const void*)(size_t)mi_profile_enable,
      (const void*)(size_t)mi_profile_collect, (const void*)(size_t)mi_kv_append,
      (const void*)(size_t)mi_kv_append_decode, (const void*)(size_t)mi_kv_quantize_chunks_fp8,
      (const void*)(size_t)mi_kv_append_decode_fp8, (const void*)(size_t)mi_kv_append_fp8,
      (const void*)(size_t)mi_decode_workspace_bytes, (const void*)(size_t)mi_paged_decode_attention,
      (const void*)(size_t)mi_paged_decode_attention_noalloc,
      (const void*)(size_t)mi_mla_decode_workspace_bytes, (const void*)(size_t)mi_paged_mla_decode_attention,
      (const void*)(size_t)mi_prefill_workspace_bytes, (const void*)(size_t)mi_paged_prefill_attention,
      (const void*)(size_t)mi_paged_prefill_attention_fp8, (const void*)(size_t)mi_paged_prefill_attention_mla,
      (const void*)(size_t)mi_norm_rope_append, (const void*)(size_t)mi_qkv_norm_rope_append,
      (const void*)(size_t)mi_update_requests, (const void*)(size_t)mi_decode_attention_state,
      (const void*)(size_t)mi_step_attention_state,
      (const void*)(size_t)mi_last_token_gather, (const void*)(size_t)mi_selected_log_probs,
      (const void*)(size_t)mi_sample_from_logits};
  size_t i;
  int rc;
  for (i = 0; i < sizeof(table) / sizeof(table[0]); ++i)
    if (!table[i]) return 10;
  if (p_version() < 1) return 1;
  /* T == 0: nothing to do, accepted without looking at the pointers */
  rc = mi_kv_append(NULL, NULL, 8, NULL, NULL, 8, 8, NULL, NULL, 0, 8, 2, NULL);
  if (rc != MI_OK) return 2;
  /* null pointers with T > 0: rejected on the host, with a message */
  rc = mi_kv_append(NULL, NULL, 8, NULL, NULL, 8, 8, NULL, NULL, 4, 8, 2, NULL);
  if (rc != MI_ERR_NULL || !strstr(p_error(), "null")) return 3;
  {
    MiTuning knobs = {0};
    knobs.decode_grid = 7;
    if (mi_decode_workspace_bytes(4, 8, 2, 128, 16, 16, 0, &knobs) != (7 + 4) * 8 * 129 * 4 + 4 * 8) return 4;
    knobs.decode_min_waves = 9;  /* out of range */
    if (mi_decode_workspace_bytes(4, 8, 2, 128, 16, 16, 0, &knobs) != -1) return 4;
  }
  if (mi_decode_workspace_bytes(0, 8, 2, 128, 16, 16, 0, NULL) != 0) return 5;
  if (sizeof(MiTuning) != 64) return 7;
  if (MI_NOALLOC_SCRATCH_BYTES != 16 * 1024 * 1024) return 6;
  printf("capi_consumer ok (ABI revision %d)\n", p_version());
  return 0;
}
