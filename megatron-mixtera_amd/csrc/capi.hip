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

static int env_int(const char* name, int dflt) {
  const char* v = getenv(name);
  return (v && *v) ? atoi(v) : dflt;
}

MiTuning& mi_tuning() {
  static MiTuning t = {env_int("MI355_DECODE_SUBTILES", 0), env_int("MI355_PREFILL_SUBTILES", 4),
                      env_int("MI355_PREFILL_LDS_ROW_TILES", 2), env_int("MI355_PREFILL_ROW_TILES", 2),
                      env_int("MI355_DECODE_MIN_WAVES", 3),
                      env_int("MI355_DECODE_WGS_PER_CU", 1), env_int("MI355_DECODE_GRID", 0),
                      env_int("MI355_DECODE_WAVES_PER_BLOCK", 8), env_int("MI355_NORM_ROPE_VECTORISED", 2),
                      env_int("MI355_MLA_DECODE_LDS", 1), env_int("MI355_PREFILL_KV_SPLIT", 1),
                      env_int("MI355_PREFILL_PINGPONG", 1)};
  return t;
}

extern "C" int mi_version(void) { return 1; }

extern "C" const char* mi_last_error(void) { return g_err; }

extern "C" int mi_set_tuning(const char* name, int32_t value) {
  if (!name) return mi_fail(MI_ERR_NULL, "mi_set_tuning: null name");
  if (!strcmp(name, "decode_tile_subtiles")) {
    if (value != 0 && value != 1 && value != 2 && value != 4)
      return mi_fail(MI_ERR_UNSUPPORTED, "decode_tile_subtiles must be 0 (automatic), 1, 2 or 4");
    mi_tuning().decode_tile_subtiles = value;
    return MI_OK;
  }
  if (!strcmp(name, "prefill_lds_row_tiles")) {
    if (value != 0 && value != 2 && value != 3) return mi_fail(MI_ERR_UNSUPPORTED, "prefill_lds_row_tiles must be 0, 2 or 3");
    mi_tuning().prefill_lds_row_tiles = value;
    return MI_OK;
  }
  if (!strcmp(name, "prefill_row_tiles")) {
    if (value != 2 && value != 4) return mi_fail(MI_ERR_UNSUPPORTED, "prefill_row_tiles must be 2 or 4");
    mi_tuning().prefill_row_tiles = value;
    return MI_OK;
  }
  if (!strcmp(name, "prefill_tile_subtiles")) {
    if (value != 1 && value != 2 && value != 4) return mi_fail(MI_ERR_UNSUPPORTED, "prefill_tile_subtiles must be 1, 2 or 4");
    mi_tuning().prefill_tile_subtiles = value;
    return MI_OK;
  }
  if (!strcmp(name, "decode_min_waves")) {
    if (value < 2 || value > 4) return mi_fail(MI_ERR_UNSUPPORTED, "decode_min_waves must be 2, 3 or 4");
    mi_tuning().decode_min_waves = value;
    return MI_OK;
  }
  if (!strcmp(name, "decode_wgs_per_cu")) {
    if (value < 1 || value > 8) return mi_fail(MI_ERR_UNSUPPORTED, "decode_wgs_per_cu must be 1..8");
    mi_tuning().decode_wgs_per_cu = value;
    return MI_OK;
  }
  if (!strcmp(name, "decode_grid")) {
    if (value < 0 || value > 65535) return mi_fail(MI_ERR_UNSUPPORTED, "decode_grid must be 0..65535");
    mi_tuning().decode_grid = value;
    return MI_OK;
  }
  if (!strcmp(name, "norm_rope_vectorised")) {
    if (value < 0 || value > 2) return mi_fail(MI_ERR_UNSUPPORTED, "norm_rope_vectorised must be 0, 1 or 2");
    mi_tuning().norm_rope_vectorised = value;
    return MI_OK;
  }
  if (!strcmp(name, "prefill_pingpong")) {
    if (value < 0 || value > 2) return mi_fail(MI_ERR_UNSUPPORTED, "prefill_pingpong must be 0, 1 or 2");
    mi_tuning().prefill_pingpong = value;
    return MI_OK;
  }
  if (!strcmp(name, "prefill_kv_split")) {
    if (value < 0 || value > 64) return mi_fail(MI_ERR_UNSUPPORTED, "prefill_kv_split must be 0 (never), 1 (automatic) or 2..64");
    mi_tuning().prefill_kv_split = value;
    return MI_OK;
  }
  if (!strcmp(name, "mla_decode_lds")) {
    if (value != 0 && value != 1) return mi_fail(MI_ERR_UNSUPPORTED, "mla_decode_lds must be 0 or 1");
    mi_tuning().mla_decode_lds = value;
    return MI_OK;
  }
  if (!strcmp(name, "decode_waves_per_block")) {
    if (value < 1 || value > 8) return mi_fail(MI_ERR_UNSUPPORTED, "decode_waves_per_block must be 1..8");
    mi_tuning().decode_waves_per_block = value;
    return MI_OK;
  }
  return mi_fail(MI_ERR_UNSUPPORTED, "mi_set_tuning: unknown knob");
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
