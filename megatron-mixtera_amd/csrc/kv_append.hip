// KV-append into the chunked ("paged") KV cache.
//
// Two addressing modes:
//  * mi_kv_append: the slot of every token is given by the reference's per-token
//    rows `token_to_chunk_idx` / `token_to_local_position_within_kv_chunk`
//    (int64), i.e. memory_buffer[0|1, layer, chunk_idx, local] = key|value
//    (megatron/core/inference/contexts/dynamic_context.py:511-545).
//  * mi_kv_append_decode: one new token per request; the slot is derived on the
//    GPU from the block table and the kv length that already counts the new
//    token: pos = len-1, chunk = block_table[r][pos / C], local = pos % C.
//    Rows with len <= 0 (batch padding) write nothing.
// Both are pure copies: the cache holds the source bits unchanged.
//
// fp8 variants quantise on the way in (OCP e4m3fn, round to nearest even,
// saturating at +-448) with one fp32 scale per (chunk, KV head).
#include "mi_common.h"
#include "mi_capi_internal.h"

namespace mi {

struct AppendParams {
  const uint8_t* key;
  const uint8_t* value;
  int64_t src_stride;  // bytes between tokens in key / value
  uint8_t* kc;
  uint8_t* vc;
  int64_t chunk_bytes;  // bytes between chunks
  int64_t tok_bytes;    // bytes between tokens inside a chunk
  const int64_t* tok_chunk;
  const int64_t* tok_local;
  const int32_t* bt;
  int64_t bt_stride;
  const int32_t* lens;
  int32_t chunk, row_bytes, T;
};

// grid = (T, 2): blockIdx.y selects key / value.  VEC = bytes moved per thread step.
template <int VEC, bool DECODE>
__global__ __launch_bounds__(256) void kv_append_kernel(AppendParams p) {
  const int t = blockIdx.x;
  int64_t c, l;
  if (DECODE) {
    const int len = p.lens[t];
    if (len <= 0) return;
    const int pos = len - 1;
    const int ci = pos / p.chunk;
    c = p.bt[(int64_t)t * p.bt_stride + ci];
    l = pos - ci * p.chunk;
  } else {
    c = p.tok_chunk[t];
    l = p.tok_local[t];
  }
  const uint8_t* src = (blockIdx.y ? p.value : p.key) + (int64_t)t * p.src_stride;
  uint8_t* dst = (blockIdx.y ? p.vc : p.kc) + c * p.chunk_bytes + l * p.tok_bytes;
  for (int i = threadIdx.x * VEC; i < p.row_bytes; i += 256 * VEC) {
    if (VEC == 16) st16(dst + i, ld16(src + i));
    else if (VEC == 4) *reinterpret_cast<uint32_t*>(dst + i) = *reinterpret_cast<const uint32_t*>(src + i);
    else if (VEC == 2) *reinterpret_cast<uint16_t*>(dst + i) = *reinterpret_cast<const uint16_t*>(src + i);
    else dst[i] = src[i];
  }
}

struct QuantParams {
  const uint16_t* src;   // rows in the 16-bit type the kernel is instantiated for
  int64_t src_stride;    // elements between tokens (bulk: between chunk tokens)
  int64_t src_chunk;     // bulk: elements between chunks
  uint8_t* dst;          // fp8 cache
  int64_t chunk_bytes, tok_bytes;
  float* scale;          // [n_chunks][Hkv]
  const int32_t* bt;
  int64_t bt_stride;
  const int32_t* lens;
  int32_t chunk, Hkv, d;
  float headroom;
};

// One workgroup (256 threads) per (chunk, KV head): amax over the whole
// chunk-head tile, scale = amax / 448, then quantise.  Used to fill an fp8 cache
// from bf16 chunks (prefill-style writes and benchmark set-up).
template <bool F16>
__global__ __launch_bounds__(256) void quantize_chunks_fp8_kernel(QuantParams p) {
  const int c = blockIdx.x, h = blockIdx.y;
  const uint16_t* src = p.src + (int64_t)c * p.src_chunk + (int64_t)h * p.d;
  const int n = p.chunk * p.d;
  float amax = 0.f;
  for (int i = threadIdx.x; i < n; i += 256) {
    const int tok = i / p.d, e = i - tok * p.d;
    amax = fmaxf(amax, fabsf(to_f32<F16>(src[(int64_t)tok * p.src_stride + e])));
  }
  __shared__ float red[256];
  red[threadIdx.x] = amax;
  __syncthreads();
  for (int s = 128; s > 0; s >>= 1) {
    if ((int)threadIdx.x < s) red[threadIdx.x] = fmaxf(red[threadIdx.x], red[threadIdx.x + s]);
    __syncthreads();
  }
  amax = red[0];
  const float scale = amax > 0.f ? amax / 448.f : 1.f;
  if (threadIdx.x == 0) p.scale[(int64_t)c * p.Hkv + h] = scale;
  uint8_t* dst = p.dst + (int64_t)c * p.chunk_bytes + (int64_t)h * p.d;
  for (int i = threadIdx.x; i < n; i += 256) {
    const int tok = i / p.d, e = i - tok * p.d;
    const float v = to_f32<F16>(src[(int64_t)tok * p.src_stride + e]) / scale;
    dst[(int64_t)tok * p.tok_bytes + e] = (uint8_t)f32_to_e4m3_sat(v);
  }
}

// One workgroup per (request, KV head): quantise the newly generated token.
// A token that opens a chunk (local position 0) fixes that chunk-head's scale to
// headroom * amax(token) / 448; later tokens reuse the stored scale and saturate.
template <bool F16>
__global__ __launch_bounds__(64) void kv_append_decode_fp8_kernel(QuantParams p) {
  const int r = blockIdx.x, h = blockIdx.y;
  const int len = p.lens[r];
  if (len <= 0) return;
  const int pos = len - 1;
  const int ci = pos / p.chunk;
  const int64_t c = p.bt[(int64_t)r * p.bt_stride + ci];
  const int l = pos - ci * p.chunk;
  const uint16_t* src = p.src + (int64_t)r * p.src_stride + (int64_t)h * p.d;
  float scale;
  if (l == 0) {
    float amax = 0.f;
    for (int e = threadIdx.x; e < p.d; e += 64) amax = fmaxf(amax, fabsf(to_f32<F16>(src[e])));
    for (int o = 32; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));
    scale = amax > 0.f ? p.headroom * amax / 448.f : 1.f;
    if (threadIdx.x == 0) p.scale[c * p.Hkv + h] = scale;
  } else {
    scale = p.scale[c * p.Hkv + h];
  }
  uint8_t* dst = p.dst + c * p.chunk_bytes + (int64_t)l * p.tok_bytes + (int64_t)h * p.d;
  for (int e = threadIdx.x; e < p.d; e += 64) dst[e] = (uint8_t)f32_to_e4m3_sat(to_f32<F16>(src[e]) / scale);
}

// ---- fp8 append of many tokens per request (prefill / mixed steps) ----------------------------
// Slots come from the per-token rows.  Tokens of one chunk are neighbours in the token dimension
// with rising local positions (that is how the context lays requests out), so the tokens a call
// writes into a chunk form one run.  A run that starts at local position 0 opens the chunk and fixes
// the scale of each of its heads: amax over the whole run / 448, times `headroom` unless the run
// fills the chunk (later tokens of a partly filled chunk reuse the scale and saturate).  A run that
// starts further in reuses the stored scale.
struct AppendFp8Params {
  const uint16_t* src[2];   // key, value rows (16-bit)
  int64_t src_stride;       // elements between tokens
  uint8_t* dst[2];          // fp8 caches
  int64_t chunk_bytes, tok_bytes;
  float* scale[2];          // [n_chunks][Hkv] each
  const int64_t* tok_chunk;
  const int64_t* tok_local;
  int32_t T, chunk, Hkv, d;
  float headroom;
};

// grid = (ceil(T / 64), Hkv, 2): a workgroup looks at 64 tokens and, for each of them that opens a
// chunk (local position 0), computes the scale of (chunk, head) of the key (z = 0) or value (z = 1)
// cache from the whole run that starts there.
template <bool F16>
__global__ __launch_bounds__(256) void kv_append_fp8_scales_kernel(AppendFp8Params p) {
  const int t0 = blockIdx.x * 64, h = blockIdx.y, kv = blockIdx.z;
  __shared__ int open_s[64];
  __shared__ int n_open_s;
  __shared__ int run_s[256];
  __shared__ float red[256];
  if (threadIdx.x < 64) {
    const int t = t0 + threadIdx.x;
    const bool opens = t < p.T && p.tok_local[t] == 0;
    const uint64_t m = __builtin_amdgcn_ballot_w64(opens);
    if (opens) open_s[__builtin_popcountll(m & (((uint64_t)1 << threadIdx.x) - 1))] = t;
    if (threadIdx.x == 0) n_open_s = __builtin_popcountll(m);
  }
  __syncthreads();
  const int n_open = n_open_s;
  // 8 elements (16 bytes) per thread step when the rows allow it
  const bool wide = !((p.d | p.src_stride) & 7) && !((uintptr_t)p.src[kv] & 15);
  for (int k = 0; k < n_open; ++k) {
    const int t = open_s[k];
    const int64_t c = p.tok_chunk[t];
    // run length: first i >= 1 where token t+i is not (chunk c, local i)
    int first_bad = p.chunk;
    for (int i = 1 + threadIdx.x; i < p.chunk; i += 256) {
      const bool ok = t + i < p.T && p.tok_chunk[t + i] == c && p.tok_local[t + i] == i;
      if (!ok) { first_bad = i; break; }
    }
    __syncthreads();
    run_s[threadIdx.x] = first_bad;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
      if ((int)threadIdx.x < s) run_s[threadIdx.x] = min(run_s[threadIdx.x], run_s[threadIdx.x + s]);
      __syncthreads();
    }
    const int n = run_s[0];
    const uint16_t* src = p.src[kv] + (int64_t)t * p.src_stride + (int64_t)h * p.d;
    float amax = 0.f;
    if (wide) {
      const int per_row = p.d >> 3;
      for (int i = threadIdx.x; i < n * per_row; i += 256) {
        const int tok = i / per_row, e = (i - tok * per_row) << 3;
        const uint4 w = ld16(src + (int64_t)tok * p.src_stride + e);
        const uint32_t u[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int j = 0; j < 4; ++j)
          amax = fmaxf(amax, fmaxf(fabsf(lo_to_f32<F16>(u[j])), fabsf(hi_to_f32<F16>(u[j]))));
      }
    } else {
      for (int i = threadIdx.x; i < n * p.d; i += 256) {
        const int tok = i / p.d, e = i - tok * p.d;
        amax = fmaxf(amax, fabsf(to_f32<F16>(src[(int64_t)tok * p.src_stride + e])));
      }
    }
    red[threadIdx.x] = amax;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
      if ((int)threadIdx.x < s) red[threadIdx.x] = fmaxf(red[threadIdx.x], red[threadIdx.x + s]);
      __syncthreads();
    }
    if (threadIdx.x == 0) {
      const float hr = n == p.chunk ? 1.f : p.headroom;
      p.scale[kv][c * p.Hkv + h] = red[0] > 0.f ? hr * red[0] / 448.f : 1.f;
    }
  }
}

// grid = (T, 2): quantise the key (y = 0) or value (y = 1) row of one token with its chunk's scales.
template <bool F16>
__global__ __launch_bounds__(256) void kv_append_fp8_rows_kernel(AppendFp8Params p) {
  const int t = blockIdx.x, kv = blockIdx.y;
  const int64_t c = p.tok_chunk[t], l = p.tok_local[t];
  const uint16_t* src = p.src[kv] + (int64_t)t * p.src_stride;
  uint8_t* dst = p.dst[kv] + c * p.chunk_bytes + l * p.tok_bytes;
  const float* scales = p.scale[kv] + c * p.Hkv;
  const int row = p.Hkv * p.d;
  const bool wide = !((p.d | p.src_stride) & 7) && !((uintptr_t)p.src[kv] & 15) &&
                    !(((uintptr_t)p.dst[kv] | (uintptr_t)p.chunk_bytes | (uintptr_t)p.tok_bytes) & 7);
  if (wide) {
    for (int e = threadIdx.x * 8; e < row; e += 256 * 8) {
      const float scale = scales[e / p.d];
      const uint4 w = ld16(src + e);
      const uint32_t u[4] = {w.x, w.y, w.z, w.w};
      uint32_t out[2] = {0u, 0u};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t lo = f32_to_e4m3_sat(lo_to_f32<F16>(u[j]) / scale), hi = f32_to_e4m3_sat(hi_to_f32<F16>(u[j]) / scale);
        out[j >> 1] |= (lo | (hi << 8)) << (16 * (j & 1));
      }
      st8(dst + e, make_uint2(out[0], out[1]));
    }
  } else {
    for (int e = threadIdx.x; e < row; e += 256)
      dst[e] = (uint8_t)f32_to_e4m3_sat(to_f32<F16>(src[e]) / scales[e / p.d]);
  }
}

// n_tensors = 2: key and value; 1: the key alone (a cache with one row per token, e.g. MLA latents)
template <bool DECODE>
static int launch_append(AppendParams& p, hipStream_t st, int n_tensors = 2) {
  const uintptr_t bits = (uintptr_t)p.key | (uintptr_t)p.value | (uintptr_t)p.kc | (uintptr_t)p.vc |
                         (uintptr_t)p.src_stride | (uintptr_t)p.chunk_bytes | (uintptr_t)p.tok_bytes |
                         (uintptr_t)p.row_bytes;
  dim3 grid(p.T, n_tensors), block(256);
  if (!(bits & 15)) hipLaunchKernelGGL((kv_append_kernel<16, DECODE>), grid, block, 0, st, p);
  else if (!(bits & 3)) hipLaunchKernelGGL((kv_append_kernel<4, DECODE>), grid, block, 0, st, p);
  else if (!(bits & 1)) hipLaunchKernelGGL((kv_append_kernel<2, DECODE>), grid, block, 0, st, p);
  else hipLaunchKernelGGL((kv_append_kernel<1, DECODE>), grid, block, 0, st, p);
  return MI_OK;
}

}  // namespace mi

using namespace mi;

extern "C" int mi_kv_append(const void* key, const void* value, int64_t src_stride_tok,
                            void* k_cache, void* v_cache, int64_t kv_stride_chunk,
                            int64_t kv_stride_tok, const int64_t* token_to_chunk_idx,
                            const int64_t* token_to_local_pos, int32_t T, int32_t row_elems,
                            int32_t elem_bytes, void* stream) {
  if (T == 0) return MI_OK;
  if (!key || !k_cache || !token_to_chunk_idx || !token_to_local_pos || (value == nullptr) != (v_cache == nullptr))
    return mi_fail(MI_ERR_NULL, "mi_kv_append: null pointer argument (value and v_cache go together)");
  if (T < 0 || row_elems <= 0 || elem_bytes <= 0 || src_stride_tok < row_elems || kv_stride_tok < row_elems)
    return mi_fail(MI_ERR_SHAPE, "mi_kv_append: bad sizes or strides");
  AppendParams p = {};
  p.key = (const uint8_t*)key; p.value = (const uint8_t*)value;
  p.src_stride = src_stride_tok * elem_bytes;
  p.kc = (uint8_t*)k_cache; p.vc = (uint8_t*)v_cache;
  p.chunk_bytes = kv_stride_chunk * elem_bytes; p.tok_bytes = kv_stride_tok * elem_bytes;
  p.tok_chunk = token_to_chunk_idx; p.tok_local = token_to_local_pos;
  p.row_bytes = row_elems * elem_bytes; p.T = T; p.chunk = 1;
  launch_append<false>(p, (hipStream_t)stream, value ? 2 : 1);
  return mi_check_launch("mi_kv_append");
}

extern "C" int mi_kv_append_decode(const void* key, const void* value, int64_t src_stride_tok,
                                   void* k_cache, void* v_cache, int64_t kv_stride_chunk,
                                   int64_t kv_stride_tok, const int32_t* block_table,
                                   int64_t bt_stride, const int32_t* kv_lens, int32_t R,
                                   int32_t chunk_tokens, int32_t row_elems, int32_t elem_bytes,
                                   void* stream) {
  if (R == 0) return MI_OK;
  if (!key || !value || !k_cache || !v_cache || !block_table || !kv_lens)
    return mi_fail(MI_ERR_NULL, "mi_kv_append_decode: null pointer argument");
  if (R < 0 || row_elems <= 0 || elem_bytes <= 0 || chunk_tokens <= 0 || src_stride_tok < row_elems ||
      kv_stride_tok < row_elems)
    return mi_fail(MI_ERR_SHAPE, "mi_kv_append_decode: bad sizes or strides");
  AppendParams p = {};
  p.key = (const uint8_t*)key; p.value = (const uint8_t*)value;
  p.src_stride = src_stride_tok * elem_bytes;
  p.kc = (uint8_t*)k_cache; p.vc = (uint8_t*)v_cache;
  p.chunk_bytes = kv_stride_chunk * elem_bytes; p.tok_bytes = kv_stride_tok * elem_bytes;
  p.bt = block_table; p.bt_stride = bt_stride; p.lens = kv_lens;
  p.row_bytes = row_elems * elem_bytes; p.T = R; p.chunk = chunk_tokens;
  launch_append<true>(p, (hipStream_t)stream);
  return mi_check_launch("mi_kv_append_decode");
}

extern "C" int mi_kv_quantize_chunks_fp8(const void* src, int64_t src_stride_chunk,
                                         int64_t src_stride_tok, void* dst_fp8,
                                         int64_t dst_stride_chunk, int64_t dst_stride_tok,
                                         float* scales, int32_t n_chunks, int32_t chunk_tokens,
                                         int32_t Hkv, int32_t head_dim, int32_t dtype, void* stream) {
  if (n_chunks == 0) return MI_OK;
  if (dtype != MI_DTYPE_BF16 && dtype != MI_DTYPE_FP16)
    return mi_fail(MI_ERR_UNSUPPORTED, "mi_kv_quantize_chunks_fp8: dtype must be MI_DTYPE_BF16 or MI_DTYPE_FP16");
  if (!src || !dst_fp8 || !scales) return mi_fail(MI_ERR_NULL, "mi_kv_quantize_chunks_fp8: null pointer argument");
  if (n_chunks < 0 || chunk_tokens <= 0 || Hkv <= 0 || head_dim <= 0 || Hkv > 65535)
    return mi_fail(MI_ERR_SHAPE, "mi_kv_quantize_chunks_fp8: bad sizes");
  QuantParams p = {};
  p.src = (const uint16_t*)src; p.src_chunk = src_stride_chunk; p.src_stride = src_stride_tok;
  p.dst = (uint8_t*)dst_fp8; p.chunk_bytes = dst_stride_chunk; p.tok_bytes = dst_stride_tok;
  p.scale = scales; p.chunk = chunk_tokens; p.Hkv = Hkv; p.d = head_dim; p.headroom = 1.f;
  if (dtype == MI_DTYPE_FP16) hipLaunchKernelGGL(quantize_chunks_fp8_kernel<true>, dim3(n_chunks, Hkv), dim3(256), 0, (hipStream_t)stream, p);
  else hipLaunchKernelGGL(quantize_chunks_fp8_kernel<false>, dim3(n_chunks, Hkv), dim3(256), 0, (hipStream_t)stream, p);
  return mi_check_launch("mi_kv_quantize_chunks_fp8");
}

extern "C" int mi_kv_append_decode_fp8(const void* key, const void* value,
                                       int64_t src_stride_tok, void* k_cache_fp8, void* v_cache_fp8,
                                       int64_t kv_stride_chunk, int64_t kv_stride_tok,
                                       float* k_scales, float* v_scales, const int32_t* block_table,
                                       int64_t bt_stride, const int32_t* kv_lens, int32_t R,
                                       int32_t chunk_tokens, int32_t Hkv, int32_t head_dim,
                                       float headroom, int32_t dtype, void* stream) {
  if (R == 0) return MI_OK;
  if (dtype != MI_DTYPE_BF16 && dtype != MI_DTYPE_FP16)
    return mi_fail(MI_ERR_UNSUPPORTED, "mi_kv_append_decode_fp8: dtype must be MI_DTYPE_BF16 or MI_DTYPE_FP16");
  if (!key || !value || !k_cache_fp8 || !v_cache_fp8 || !k_scales || !v_scales || !block_table || !kv_lens)
    return mi_fail(MI_ERR_NULL, "mi_kv_append_decode_fp8: null pointer argument");
  if (R < 0 || chunk_tokens <= 0 || Hkv <= 0 || head_dim <= 0 || Hkv > 65535 || !(headroom > 0.f))
    return mi_fail(MI_ERR_SHAPE, "mi_kv_append_decode_fp8: bad sizes");
  QuantParams p = {};
  p.src_stride = src_stride_tok; p.chunk_bytes = kv_stride_chunk; p.tok_bytes = kv_stride_tok;
  p.bt = block_table; p.bt_stride = bt_stride; p.lens = kv_lens;
  p.chunk = chunk_tokens; p.Hkv = Hkv; p.d = head_dim; p.headroom = headroom;
  const auto kernel = dtype == MI_DTYPE_FP16 ? kv_append_decode_fp8_kernel<true> : kv_append_decode_fp8_kernel<false>;
  p.src = (const uint16_t*)key; p.dst = (uint8_t*)k_cache_fp8; p.scale = k_scales;
  hipLaunchKernelGGL(kernel, dim3(R, Hkv), dim3(64), 0, (hipStream_t)stream, p);
  p.src = (const uint16_t*)value; p.dst = (uint8_t*)v_cache_fp8; p.scale = v_scales;
  hipLaunchKernelGGL(kernel, dim3(R, Hkv), dim3(64), 0, (hipStream_t)stream, p);
  return mi_check_launch("mi_kv_append_decode_fp8");
}

extern "C" int mi_kv_append_fp8(const void* key, const void* value, int64_t src_stride_tok,
                                void* k_cache_fp8, void* v_cache_fp8, int64_t kv_stride_chunk,
                                int64_t kv_stride_tok, float* k_scales, float* v_scales,
                                const int64_t* token_to_chunk_idx, const int64_t* token_to_local_pos,
                                int32_t T, int32_t chunk_tokens, int32_t Hkv, int32_t head_dim,
                                float headroom, int32_t dtype, void* stream) {
  if (T == 0) return MI_OK;
  if (dtype != MI_DTYPE_BF16 && dtype != MI_DTYPE_FP16)
    return mi_fail(MI_ERR_UNSUPPORTED, "mi_kv_append_fp8: dtype must be MI_DTYPE_BF16 or MI_DTYPE_FP16");
  if (!key || !value || !k_cache_fp8 || !v_cache_fp8 || !k_scales || !v_scales || !token_to_chunk_idx ||
      !token_to_local_pos)
    return mi_fail(MI_ERR_NULL, "mi_kv_append_fp8: null pointer argument");
  if (T < 0 || chunk_tokens <= 0 || Hkv <= 0 || head_dim <= 0 || Hkv > 65535 || !(headroom > 0.f) ||
      src_stride_tok < (int64_t)Hkv * head_dim || kv_stride_tok < (int64_t)Hkv * head_dim)
    return mi_fail(MI_ERR_SHAPE, "mi_kv_append_fp8: bad sizes or strides");
  AppendFp8Params p = {};
  p.src[0] = (const uint16_t*)key; p.src[1] = (const uint16_t*)value; p.src_stride = src_stride_tok;
  p.dst[0] = (uint8_t*)k_cache_fp8; p.dst[1] = (uint8_t*)v_cache_fp8;
  p.chunk_bytes = kv_stride_chunk; p.tok_bytes = kv_stride_tok;
  p.scale[0] = k_scales; p.scale[1] = v_scales;
  p.tok_chunk = token_to_chunk_idx; p.tok_local = token_to_local_pos;
  p.T = T; p.chunk = chunk_tokens; p.Hkv = Hkv; p.d = head_dim; p.headroom = headroom;
  hipStream_t st = (hipStream_t)stream;
  if (dtype == MI_DTYPE_FP16) {
    hipLaunchKernelGGL(kv_append_fp8_scales_kernel<true>, dim3((T + 63) / 64, Hkv, 2), dim3(256), 0, st, p);
    hipLaunchKernelGGL(kv_append_fp8_rows_kernel<true>, dim3(T, 2), dim3(256), 0, st, p);
  } else {
    hipLaunchKernelGGL(kv_append_fp8_scales_kernel<false>, dim3((T + 63) / 64, Hkv, 2), dim3(256), 0, st, p);
    hipLaunchKernelGGL(kv_append_fp8_rows_kernel<false>, dim3(T, 2), dim3(256), 0, st, p);
  }
  return mi_check_launch("mi_kv_append_fp8");
}
