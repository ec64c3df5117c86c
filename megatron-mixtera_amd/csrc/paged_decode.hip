// Paged GQA decode attention for gfx950: split-K flash-decode + log-sum-exp merge.
//
// Replaces the `flash_attn_with_kvcache(q, k_cache, v_cache, cache_seqlens,
// causal=True, block_table)` call of the reference
// (megatron/core/transformer/attention.py:589-600): one query token per request
// attends to the request's tokens scattered over fixed-size chunks of a
// `[n_chunks, chunk, Hkv, d]` cache, addressed through a `[R, M]` block table.
//
// Work decomposition
//   grid = (splits, R, Hkv / waves_per_block); one wavefront owns one
//   (request, KV head, split) item and streams `split` tokens of K and V once.
//   The waves of a workgroup take neighbouring KV heads of the SAME tokens, so a
//   workgroup as a whole reads each token's `Hkv*d` row contiguously.
//
// Per 16-token tile (all on the matrix cores, nothing staged in LDS)
//   S^T[token][qrow] = K[token][:] . Q[qrow][:]      4x  mfma 16x16x32 (d = 128)
//     - A operand: lane (m16, g) loads 16 B of token m16's K row;
//     - B operand: the G query heads sharing this KV head, zero padded to 16 rows.
//   The result lands as lane (qrow = m16, g) slot i = token 4g+i, which is
//   exactly the B-operand layout of the next product, so P never moves:
//   O^T[d][qrow] += V^T[d][token] . P^T[token][qrow]  d/16 x mfma 16x16x16
//     - lane (x = m16, g) loads d/16 contiguous values of tokens 4g..4g+3 (four
//       fully coalesced row loads) and transposes the 4 x (d/16) block in
//       registers with byte permutes to build the A operand.
//   Softmax statistics are per query row = per m16, so only the running max
//   needs a cross-lane step (two exchanges across g).
//
// A split that is the only one of its request writes bf16 output directly; else
// it writes a normalised fp32 partial and a base-2 LSE, merged by a second
// kernel: o = sum_s 2^(lse_s - max) o_s / sum_s 2^(lse_s - max).
#include "mi_common.h"
#include "mi_capi_internal.h"

namespace mi {

struct DecodeParams {
  const uint16_t* q;
  int64_t q_st, q_sh;  // element strides: token, head
  const uint8_t* kc;
  const uint8_t* vc;
  int64_t kv_sc;            // elements between chunks
  int32_t kv_st, kv_sh;     // elements between tokens / heads inside a chunk
  const int32_t* bt;
  int64_t bt_stride;
  const int32_t* lens;
  uint16_t* out;
  int64_t o_st, o_sh;
  float* part_o;    // [R][Hq][max_splits][HD]
  float* part_lse;  // [R][Hq][max_splits]
  const float* k_scale;  // fp8 only: [n_chunks][Hkv]
  const float* v_scale;
  int32_t R, Hq, Hkv, G, chunk, chunk_shift, split, max_splits;
  float scale_log2;
};

static __device__ __forceinline__ int chunk_of(int tok, int chunk, int shift) {
  return shift >= 0 ? (tok >> shift) : (tok / chunk);
}

template <int HD, int NT, bool FP8>
__global__ __launch_bounds__(512) void paged_decode_split_kernel(DecodeParams p) {
  constexpr int KS = HD / 32;
  constexpr int DV = HD / 16;
  static_assert(HD == 64 || HD == 128, "head_dim 64 or 128");
  constexpr int ESZ = FP8 ? 1 : 2;

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int m16 = lane & 15, g = lane >> 4;
  const int s = blockIdx.x;
  const int r = blockIdx.y;
  const int h = __builtin_amdgcn_readfirstlane(blockIdx.z * (blockDim.x >> 6) + wave);
  const int G = p.G;
  const int hq = h * G + m16;  // query head of this lane's row (valid when m16 < G)

  const int len = p.lens[r];
  const int start = s * p.split;
  if (len <= 0) {
    // Padded batch rows carry kv-len 0: their output is defined as zeros.
    if (s == 0 && m16 < G) {
      uint16_t* o = p.out + (int64_t)r * p.o_st + (int64_t)hq * p.o_sh + (HD / 4) * g;
      for (int i = 0; i < HD / 4; i += 8) st16(o + i, make_uint4(0, 0, 0, 0));
    }
    return;
  }
  if (start >= len) return;
  const int end = min(start + p.split, len);
  const int nsplit = (len + p.split - 1) / p.split;
  const int last = len - 1;

  // Query fragments: B operand rows are the G heads of this KV head.
  uint4 qf[KS];
  {
    const uint16_t* qrow = p.q + (int64_t)r * p.q_st + (int64_t)hq * p.q_sh;
#pragma unroll
    for (int kk = 0; kk < KS; ++kk) {
      // bf16 cache: lane g owns d = 32kk + 8g .. +7.
      // fp8 cache : K bytes are loaded 16 per lane, d = 64u + 16g + 8half .. +7
      //             for mfma step kk = 2u + half.
      const int d0 = FP8 ? (64 * (kk >> 1) + 16 * g + 8 * (kk & 1)) : (32 * kk + 8 * g);
      qf[kk] = (m16 < G) ? ld16(qrow + d0) : make_uint4(0, 0, 0, 0);
    }
  }

  const uint8_t* kbase = p.kc + (int64_t)h * p.kv_sh * ESZ;
  const uint8_t* vbase = p.vc + (int64_t)h * p.kv_sh * ESZ;
  const int64_t chunk_bytes = p.kv_sc * ESZ;
  const int tok_bytes = p.kv_st * ESZ;

  float m_run = -INFINITY, l_run = 0.f;
  f32x4_t acc[DV];
#pragma unroll
  for (int e = 0; e < DV; ++e) acc[e] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  for (int T = start; T < end; T += 16 * NT) {
    // ---- issue every load of this tile first -------------------------------
    uint4 kf[NT][FP8 ? KS / 2 : KS];
    uint4 vf16[NT][4];  // bf16, HD=128 : 16 B per token
    uint2 vf8[NT][4];   // bf16 HD=64 or fp8 HD=128 : 8 B per token
    float ksc[NT], vsc[NT];
#pragma unroll
    for (int u = 0; u < NT; ++u) {
      const int T0 = T + 16 * u;
      const int tu = min(T0, last);  // wave-uniform
      const int ci = chunk_of(tu, p.chunk, p.chunk_shift);
      const int pc = p.bt[(int64_t)r * p.bt_stride + ci];
      const int cbase = ci * p.chunk;
      const uint8_t* kc = kbase + (int64_t)pc * chunk_bytes;
      const uint8_t* vc = vbase + (int64_t)pc * chunk_bytes;
      if (FP8) {
        ksc[u] = p.k_scale[(int64_t)pc * p.Hkv + h];
        vsc[u] = p.v_scale[(int64_t)pc * p.Hkv + h];
      }
      // Tokens past the end are clamped to the last valid one: the data stays
      // finite and their probabilities are forced to zero below.
      const int tk = min(T0 + m16, last) - cbase;
      const uint8_t* krow = kc + tk * tok_bytes;
      if (FP8) {
#pragma unroll
        for (int kk = 0; kk < KS / 2; ++kk) kf[u][kk] = ld16(krow + 64 * kk + 16 * g);
      } else {
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) kf[u][kk] = ld16(krow + (32 * kk + 8 * g) * 2);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int tv = min(T0 + 4 * g + j, last) - cbase;
        const uint8_t* vrow = vc + tv * tok_bytes + DV * m16 * ESZ;
        if (!FP8 && HD == 128) vf16[u][j] = ld16(vrow);
        else vf8[u][j] = ld8(vrow);
      }
    }

    // ---- S^T = K Q^T ---------------------------------------------------------
    float sc[NT][4];
    float tmax = -INFINITY;
#pragma unroll
    for (int u = 0; u < NT; ++u) {
      f32x4_t sacc = {0.f, 0.f, 0.f, 0.f};
      if (FP8) {
#pragma unroll
        for (int kk = 0; kk < KS / 2; ++kk) {
          const uint2 a0 = fp8x4_to_bf16x4(kf[u][kk].x), a1 = fp8x4_to_bf16x4(kf[u][kk].y);
          const uint2 b0 = fp8x4_to_bf16x4(kf[u][kk].z), b1 = fp8x4_to_bf16x4(kf[u][kk].w);
          sacc = mfma_16x16x32(make_uint4(a0.x, a0.y, a1.x, a1.y), qf[2 * kk], sacc);
          sacc = mfma_16x16x32(make_uint4(b0.x, b0.y, b1.x, b1.y), qf[2 * kk + 1], sacc);
        }
      } else {
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) sacc = mfma_16x16x32(kf[u][kk], qf[kk], sacc);
      }
      const float mul = FP8 ? p.scale_log2 * ksc[u] : p.scale_log2;
      const int tok0 = T + 16 * u + 4 * g;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float v = (tok0 + i < end) ? sacc[i] * mul : -INFINITY;
        sc[u][i] = v;
        tmax = fmaxf(tmax, v);
      }
    }
    tmax = fmaxf(tmax, xor16(tmax));
    tmax = fmaxf(tmax, xor32(tmax));

    // ---- online softmax (row = m16, all lane-local after the max) -----------
    const float m_new = fmaxf(m_run, tmax);
    const float alpha = fast_exp2(m_run - m_new);
    m_run = m_new;
    float psum = 0.f;
    uint2 pf[NT];
#pragma unroll
    for (int u = 0; u < NT; ++u) {
      float pv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        pv[i] = fast_exp2(sc[u][i] - m_new);
        psum += pv[i];
      }
      if (FP8) {
#pragma unroll
        for (int i = 0; i < 4; ++i) pv[i] *= vsc[u];
      }
      pf[u] = make_uint2(pack_bf16x2(pv[0], pv[1]), pack_bf16x2(pv[2], pv[3]));
    }
    l_run = l_run * alpha + psum;
#pragma unroll
    for (int e = 0; e < DV; ++e) {
      acc[e][0] *= alpha; acc[e][1] *= alpha; acc[e][2] *= alpha; acc[e][3] *= alpha;
    }

    // ---- O^T += V^T P^T --------------------------------------------------------
#pragma unroll
    for (int u = 0; u < NT; ++u) {
      if (!FP8 && HD == 128) {
        const uint32_t* r0 = reinterpret_cast<const uint32_t*>(&vf16[u][0]);
        const uint32_t* r1 = reinterpret_cast<const uint32_t*>(&vf16[u][1]);
        const uint32_t* r2 = reinterpret_cast<const uint32_t*>(&vf16[u][2]);
        const uint32_t* r3 = reinterpret_cast<const uint32_t*>(&vf16[u][3]);
#pragma unroll
        for (int pr = 0; pr < 4; ++pr) {
          acc[2 * pr] = mfma_16x16x16(
              make_uint2(low_halves(r1[pr], r0[pr]), low_halves(r3[pr], r2[pr])), pf[u], acc[2 * pr]);
          acc[2 * pr + 1] = mfma_16x16x16(
              make_uint2(high_halves(r1[pr], r0[pr]), high_halves(r3[pr], r2[pr])), pf[u], acc[2 * pr + 1]);
        }
      } else if (!FP8) {  // bf16, HD == 64: four values per token per lane
        const uint2 a = vf8[u][0], b = vf8[u][1], c = vf8[u][2], d = vf8[u][3];
        acc[0] = mfma_16x16x16(make_uint2(low_halves(b.x, a.x), low_halves(d.x, c.x)), pf[u], acc[0]);
        acc[1] = mfma_16x16x16(make_uint2(high_halves(b.x, a.x), high_halves(d.x, c.x)), pf[u], acc[1]);
        acc[2] = mfma_16x16x16(make_uint2(low_halves(b.y, a.y), low_halves(d.y, c.y)), pf[u], acc[2]);
        acc[3] = mfma_16x16x16(make_uint2(high_halves(b.y, a.y), high_halves(d.y, c.y)), pf[u], acc[3]);
      } else {  // fp8, HD == 128: eight bytes per token per lane
        uint2 w[4][2];  // [token j][half] -> two packed bf16 pairs (4 d values)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          w[j][0] = fp8x4_to_bf16x4(vf8[u][j].x);
          w[j][1] = fp8x4_to_bf16x4(vf8[u][j].y);
        }
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
          acc[4 * hf + 0] = mfma_16x16x16(
              make_uint2(low_halves(w[1][hf].x, w[0][hf].x), low_halves(w[3][hf].x, w[2][hf].x)), pf[u], acc[4 * hf + 0]);
          acc[4 * hf + 1] = mfma_16x16x16(
              make_uint2(high_halves(w[1][hf].x, w[0][hf].x), high_halves(w[3][hf].x, w[2][hf].x)), pf[u], acc[4 * hf + 1]);
          acc[4 * hf + 2] = mfma_16x16x16(
              make_uint2(low_halves(w[1][hf].y, w[0][hf].y), low_halves(w[3][hf].y, w[2][hf].y)), pf[u], acc[4 * hf + 2]);
          acc[4 * hf + 3] = mfma_16x16x16(
              make_uint2(high_halves(w[1][hf].y, w[0][hf].y), high_halves(w[3][hf].y, w[2][hf].y)), pf[u], acc[4 * hf + 3]);
        }
      }
    }
  }

  // ---- epilogue ---------------------------------------------------------------
  float l_tot = l_run + xor16(l_run);
  l_tot += xor32(l_tot);
  const float inv = 1.f / l_tot;
  if (m16 >= G) return;
  // acc[e][i] holds d = DV*(4g+i) + e: DV*4 contiguous values per lane.
  if (nsplit == 1) {
    uint16_t* o = p.out + (int64_t)r * p.o_st + (int64_t)hq * p.o_sh + 4 * DV * g;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if constexpr (DV == 8) {
        st16(o + 8 * i, make_uint4(pack_bf16x2(acc[0][i] * inv, acc[1][i] * inv),
                                   pack_bf16x2(acc[2][i] * inv, acc[3][i] * inv),
                                   pack_bf16x2(acc[4][i] * inv, acc[5][i] * inv),
                                   pack_bf16x2(acc[6][i] * inv, acc[7][i] * inv)));
      } else {
        st8(o + 4 * i, make_uint2(pack_bf16x2(acc[0][i] * inv, acc[1][i] * inv),
                                  pack_bf16x2(acc[2][i] * inv, acc[3][i] * inv)));
      }
    }
  } else {
    const int64_t row = ((int64_t)r * p.Hq + hq) * p.max_splits + s;
    float* o = p.part_o + row * HD + 4 * DV * g;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int e = 0; e < DV; e += 4) {
        float4 v = make_float4(acc[e][i] * inv, acc[e + 1][i] * inv, acc[e + 2][i] * inv, acc[e + 3][i] * inv);
        *reinterpret_cast<float4*>(o + DV * i + e) = v;
      }
    }
    if (g == 0) p.part_lse[row] = m_run + fast_log2(l_tot);
  }
}

// One workgroup per (request, query head): merge the split partials.
template <int HD>
__global__ __launch_bounds__(HD) void paged_decode_merge_kernel(DecodeParams p) {
  const int r = blockIdx.y, hq = blockIdx.x, d = threadIdx.x;
  const int len = p.lens[r];
  if (len <= 0) return;
  const int nsplit = (len + p.split - 1) / p.split;
  if (nsplit <= 1) return;
  const int64_t row0 = ((int64_t)r * p.Hq + hq) * p.max_splits;
  const float* lse = p.part_lse + row0;
  const float* po = p.part_o + row0 * HD + d;
  float mx = -INFINITY;
  for (int s = 0; s < nsplit; ++s) mx = fmaxf(mx, lse[s]);
  float num = 0.f, den = 0.f;
#pragma unroll 4
  for (int s = 0; s < nsplit; ++s) {
    const float w = fast_exp2(lse[s] - mx);
    num += w * po[(int64_t)s * HD];
    den += w;
  }
  p.out[(int64_t)r * p.o_st + (int64_t)hq * p.o_sh + d] = f32_to_bf16(num / den);
}

static int pick_waves_per_block(int Hkv) {
  for (int w = 8; w >= 1; --w)
    if (Hkv % w == 0) return w;
  return 1;
}

static int log2_exact(int x) {
  if (x <= 0 || (x & (x - 1))) return -1;
  int s = 0;
  while ((1 << s) < x) ++s;
  return s;
}

int resolve_split_tokens(int R, int Hkv, int chunk, int max_kv_len, int split_tokens) {
  if (split_tokens > 0) return split_tokens;
  int wpb = pick_waves_per_block(Hkv);
  int split = chunk >= 256 ? 256 : chunk;
  if (chunk > 256 && chunk % 256) split = chunk;
  // Keep the grid (mostly early-exit workgroups when lengths are ragged) bounded.
  while ((int64_t)R * (Hkv / wpb) * ((max_kv_len + split - 1) / split) > 16384 && split < 8192) split *= 2;
  return split;
}

}  // namespace mi

using namespace mi;

extern "C" int64_t mi_decode_workspace_bytes(int32_t R, int32_t Hq, int32_t Hkv, int32_t head_dim,
                                             int32_t chunk_tokens, int32_t max_kv_len,
                                             int32_t split_tokens) {
  if (R <= 0 || Hq <= 0 || Hkv <= 0 || head_dim <= 0 || chunk_tokens <= 0 || max_kv_len <= 0) return 0;
  const int split = resolve_split_tokens(R, Hkv, chunk_tokens, max_kv_len, split_tokens);
  const int64_t ms = (max_kv_len + split - 1) / split;
  return (int64_t)R * Hq * ms * (head_dim + 1) * (int64_t)sizeof(float);
}

extern "C" int mi_paged_decode_attention(
    const void* q, int64_t q_stride_tok, int64_t q_stride_head, const void* k_cache,
    const void* v_cache, int64_t kv_stride_chunk, int64_t kv_stride_tok, int64_t kv_stride_head,
    const int32_t* block_table, int64_t bt_stride, const int32_t* kv_lens, void* out,
    int64_t o_stride_tok, int64_t o_stride_head, void* workspace, int64_t workspace_bytes,
    int32_t R, int32_t Hq, int32_t Hkv, int32_t head_dim, int32_t chunk_tokens, int32_t max_kv_len,
    int32_t split_tokens, float softmax_scale, int32_t kv_dtype, const float* k_scales,
    const float* v_scales, void* stream) {
  if (R == 0) return MI_OK;
  if (!q || !k_cache || !v_cache || !block_table || !kv_lens || !out)
    return mi_fail(MI_ERR_NULL, "mi_paged_decode_attention: null pointer argument");
  if (R < 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv)
    return mi_fail(MI_ERR_SHAPE, "mi_paged_decode_attention: need R >= 0 and Hq a multiple of Hkv");
  const int G = Hq / Hkv;
  if (G > 16) return mi_fail(MI_ERR_UNSUPPORTED, "mi_paged_decode_attention: more than 16 query heads per KV head");
  if (head_dim != 64 && head_dim != 128)
    return mi_fail(MI_ERR_UNSUPPORTED, "mi_paged_decode_attention: head_dim must be 64 or 128");
  if (chunk_tokens <= 0 || chunk_tokens % 16)
    return mi_fail(MI_ERR_SHAPE, "mi_paged_decode_attention: chunk size must be a positive multiple of 16");
  if (kv_dtype != MI_KV_BF16 && kv_dtype != MI_KV_FP8_E4M3)
    return mi_fail(MI_ERR_UNSUPPORTED, "mi_paged_decode_attention: unknown kv_dtype");
  if (kv_dtype == MI_KV_FP8_E4M3 && (head_dim != 128 || !k_scales || !v_scales))
    return mi_fail(MI_ERR_UNSUPPORTED, "mi_paged_decode_attention: fp8 KV needs head_dim 128 and both scale arrays");
  const int esz = kv_dtype == MI_KV_FP8_E4M3 ? 1 : 2;
  if (((uintptr_t)q | (uintptr_t)k_cache | (uintptr_t)v_cache | (uintptr_t)out) & 15)
    return mi_fail(MI_ERR_ALIGN, "mi_paged_decode_attention: q/k/v/out must be 16-byte aligned");
  if ((q_stride_tok | q_stride_head | o_stride_tok | o_stride_head) % 8 ||
      ((kv_stride_chunk | kv_stride_tok | kv_stride_head) * esz) % 16)
    return mi_fail(MI_ERR_ALIGN, "mi_paged_decode_attention: strides must keep rows 16-byte aligned");
  if (kv_stride_tok * (int64_t)chunk_tokens * esz >= (int64_t)1 << 31)
    return mi_fail(MI_ERR_SHAPE, "mi_paged_decode_attention: one chunk must span less than 2 GiB");
  if (max_kv_len <= 0) return mi_fail(MI_ERR_SHAPE, "mi_paged_decode_attention: max_kv_len must be positive");

  const int split = resolve_split_tokens(R, Hkv, chunk_tokens, max_kv_len, split_tokens);
  if (split % 16) return mi_fail(MI_ERR_SHAPE, "mi_paged_decode_attention: split_tokens must be a multiple of 16");
  const int max_splits = (max_kv_len + split - 1) / split;
  const int64_t need = (int64_t)R * Hq * max_splits * (head_dim + 1) * (int64_t)sizeof(float);
  if (max_splits > 1 && (!workspace || workspace_bytes < need))
    return mi_fail(MI_ERR_WORKSPACE, "mi_paged_decode_attention: workspace too small (see mi_decode_workspace_bytes)");
  if (max_splits > 1 && ((uintptr_t)workspace & 15))
    return mi_fail(MI_ERR_ALIGN, "mi_paged_decode_attention: workspace must be 16-byte aligned");

  DecodeParams p;
  p.q = (const uint16_t*)q; p.q_st = q_stride_tok; p.q_sh = q_stride_head;
  p.kc = (const uint8_t*)k_cache; p.vc = (const uint8_t*)v_cache;
  p.kv_sc = kv_stride_chunk; p.kv_st = (int32_t)kv_stride_tok; p.kv_sh = (int32_t)kv_stride_head;
  p.bt = block_table; p.bt_stride = bt_stride; p.lens = kv_lens;
  p.out = (uint16_t*)out; p.o_st = o_stride_tok; p.o_sh = o_stride_head;
  p.part_o = (float*)workspace;
  p.part_lse = p.part_o ? p.part_o + (int64_t)R * Hq * max_splits * head_dim : nullptr;
  p.k_scale = k_scales; p.v_scale = v_scales;
  p.R = R; p.Hq = Hq; p.Hkv = Hkv; p.G = G; p.chunk = chunk_tokens;
  p.chunk_shift = log2_exact(chunk_tokens); p.split = split; p.max_splits = max_splits;
  p.scale_log2 = softmax_scale * 1.4426950408889634f;

  const int wpb = pick_waves_per_block(Hkv);
  dim3 grid(max_splits, R, Hkv / wpb), block(64 * wpb);
  hipStream_t st = (hipStream_t)stream;
  const int nt = mi_tuning().decode_tile_subtiles;
  hipEvent_t ev_a, ev_b;
  const bool timed = mi_profile_next(&ev_a, &ev_b);
  if (timed) hipEventRecord(ev_a, st);
  if (kv_dtype == MI_KV_FP8_E4M3) {
    if (nt == 1) hipLaunchKernelGGL((paged_decode_split_kernel<128, 1, true>), grid, block, 0, st, p);
    else if (nt == 4) hipLaunchKernelGGL((paged_decode_split_kernel<128, 4, true>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((paged_decode_split_kernel<128, 2, true>), grid, block, 0, st, p);
  } else if (head_dim == 128) {
    if (nt == 1) hipLaunchKernelGGL((paged_decode_split_kernel<128, 1, false>), grid, block, 0, st, p);
    else if (nt == 4) hipLaunchKernelGGL((paged_decode_split_kernel<128, 4, false>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((paged_decode_split_kernel<128, 2, false>), grid, block, 0, st, p);
  } else {
    if (nt == 1) hipLaunchKernelGGL((paged_decode_split_kernel<64, 1, false>), grid, block, 0, st, p);
    else if (nt == 4) hipLaunchKernelGGL((paged_decode_split_kernel<64, 4, false>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((paged_decode_split_kernel<64, 2, false>), grid, block, 0, st, p);
  }
  if (timed) hipEventRecord(ev_b, st);
  if (max_splits > 1) {
    dim3 mgrid(Hq, R);
    if (head_dim == 128) hipLaunchKernelGGL((paged_decode_merge_kernel<128>), mgrid, dim3(128), 0, st, p);
    else hipLaunchKernelGGL((paged_decode_merge_kernel<64>), mgrid, dim3(64), 0, st, p);
  }
  return mi_check_launch("mi_paged_decode_attention");
}
