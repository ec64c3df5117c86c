// Error reporting, version and tuning entry points of the C-ABI library.
#include "mi_capi_internal.h"

#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static thread_local char g_err[256] = "";

int mi_fail(int code, const char* msg) {
  snprintf(g_err, sizeof(g_err), "%s", msg);
  return code;
}

int mi_check_launch(const char* where) {
  hipError_t e = hipGetLastError();
  if (e == hipSuccess) return MI_OK;
  snprintf(g_err, sizeof(g_err), "%s: %s", where, hipGetErrorString(e));
  return MI_ERR_LAUNCH;
}

extern "C" int mi_version(void) { return 2; }

extern "C" const char* mi_last_error(void) { return g_err; }

int mi_resolve_tuning(const MiTuning* given, MiTuning* out, const char* who) {
  MiTuning t = {};
  if (given) t = *given;
  char msg[200];
  auto bad = [&](const char* what) {
    snprintf(msg, sizeof msg, "%s: tuning: %s", who, what);
    return mi_fail(MI_ERR_UNSUPPORTED, msg);
  };
  for (int r : t.reserved)
    if (r != 0) return bad("reserved fields must be 0");
  if (t.decode_tile_subtiles != 0 && t.decode_tile_subtiles != 1 && t.decode_tile_subtiles != 2 && t.decode_tile_subtiles != 4)
    return bad("decode_tile_subtiles must be 0 (automatic), 1, 2 or 4");
  if (t.decode_min_waves == 0) t.decode_min_waves = 3;
  if (t.decode_min_waves < 2 || t.decode_min_waves > 4) return bad("decode_min_waves must be 0 (default), 2, 3 or 4");
  if (t.decode_wgs_per_cu == 0) t.decode_wgs_per_cu = 1;
  if (t.decode_wgs_per_cu < 1 || t.decode_wgs_per_cu > 8) return bad("decode_wgs_per_cu must be 0 (default) or 1..8");
  if (t.decode_grid < 0 || t.decode_grid > 65535) return bad("decode_grid must be 0 (automatic) or 1..65535");
  if (t.decode_waves_per_block == 0) t.decode_waves_per_block = 8;
  if (t.decode_waves_per_block < 1 || t.decode_waves_per_block > 8) return bad("decode_waves_per_block must be 0 (default) or 1..8");
  if (t.prefill_two_phase == 0) t.prefill_two_phase = 3;
  if (t.prefill_two_phase != 1 && t.prefill_two_phase != 2 && t.prefill_two_phase != 3 && t.prefill_two_phase != -1)
    return bad("prefill_two_phase must be 0 (default), 1, 2, 3 (one-stream tile kernel) or -1 (register-only kernel)");
  if (t.prefill_tile_subtiles == 0) t.prefill_tile_subtiles = 2;
  if (t.prefill_tile_subtiles != 1 && t.prefill_tile_subtiles != 2) return bad("prefill_tile_subtiles must be 0 (default), 1 or 2");
  if (t.prefill_row_tiles == 0) t.prefill_row_tiles = 2;
  if (t.prefill_row_tiles != 2 && t.prefill_row_tiles != 4) return bad("prefill_row_tiles must be 0 (default), 2 or 4");
  if (t.prefill_kv_split == 0) t.prefill_kv_split = 1;  // 1 = automatic from here on
  if (t.prefill_kv_split != -1 && (t.prefill_kv_split < 1 || t.prefill_kv_split > 64))
    return bad("prefill_kv_split must be 0 (automatic), -1 (never) or 2..64");
  if (t.norm_rope_vectorised == 0) t.norm_rope_vectorised = 2;  // 2 = from 256 tokens up
  if (t.norm_rope_vectorised != 1 && t.norm_rope_vectorised != 2 && t.norm_rope_vectorised != -1)
    return bad("norm_rope_vectorised must be 0 (default), 1 or -1 (never)");
  if (t.mla_decode_lds == 0) t.mla_decode_lds = 1;
  if (t.mla_decode_lds != 1 && t.mla_decode_lds != -1 && t.mla_decode_lds != 2)
    return bad("mla_decode_lds must be 0 (default), -1 (streaming kernel) or 2 (eight-wavefront LDS kernel at every head count)");
  *out = t;
  return MI_OK;
}

// ---- kernel timing with HIP events --------------------------------------------------
// When enabled, the attention entry points bracket their main kernel (decode: the kernel that
// streams the KV cache; prefill: the tile kernel, and after it the streaming kernel of the one-row
// requests) with a start/stop event pair on the caller's stream; the pairs are read back, in
// launch order, with mi_profile_collect.  Host objects only: nothing is allocated on the
// device, and profiling must stay off while a stream is being captured into a graph.
#include <mutex>
#include <vector>

namespace {
struct EventPair { hipEvent_t a, b; };
std::vector<EventPair> g_pool;     // created once, reused
size_t g_used = 0;
bool g_profile = false;
std::mutex g_profile_mutex;        // entry points may be called from several host threads
}  // namespace

bool mi_profile_next(hipEvent_t* a, hipEvent_t* b) {
  std::lock_guard<std::mutex> lock(g_profile_mutex);
  if (!g_profile) return false;
  if (g_used == g_pool.size()) {
    if (g_pool.size() >= 65536) return false;
    EventPair p;
    // no system-scope fence: the events only time device work on one stream
    if (hipEventCreateWithFlags(&p.a, hipEventDisableSystemFence) != hipSuccess ||
        hipEventCreateWithFlags(&p.b, hipEventDisableSystemFence) != hipSuccess)
      return false;
    g_pool.push_back(p);
  }
  *a = g_pool[g_used].a;
  *b = g_pool[g_used].b;
  ++g_used;
  return true;
}

bool mi_profile_is_on() {
  std::lock_guard<std::mutex> lock(g_profile_mutex);
  return g_profile;
}

extern "C" int mi_profile_enable(int32_t on) {
  std::lock_guard<std::mutex> lock(g_profile_mutex);
  g_profile = on != 0;
  g_used = 0;
  return MI_OK;
}

extern "C" int32_t mi_profile_collect(float* out_ms, int32_t capacity) {
  std::lock_guard<std::mutex> lock(g_profile_mutex);
  int32_t n = 0;
  for (size_t i = 0; i < g_used; ++i) {
    if (hipEventSynchronize(g_pool[i].b) != hipSuccess) break;
    float ms = 0.f;
    if (hipEventElapsedTime(&ms, g_pool[i].a, g_pool[i].b) != hipSuccess) break;
    if (out_ms && n < capacity) out_ms[n] = ms;
    ++n;
  }
  g_used = 0;
  return n;
}
