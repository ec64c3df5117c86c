// Fused q/k head norm + rotary embedding (+ optional KV-append) for the decode
// and prefill Q/K of one layer.
//
// Replaces, in one launch, what the reference runs as ~20 small kernels per
// layer:
//   q_layernorm / k_layernorm over the head dim
//       (megatron/core/transformer/attention.py:1026-1030; RMSNorm or L2Norm,
//        megatron/core/transformer/torch_norm.py:15-96),
//   apply_rotary_emb_key / apply_rotary_emb_query: gather emb[pos] and
//       t*cos + rotate_half(t)*sin
//       (megatron/core/inference/contexts/dynamic_context.py:566-631,
//        megatron/core/models/common/embeddings/rope_utils.py:73-126),
//   append_key_value_cache (dynamic_context.py:511-545) when a cache is given.
//
// Rounding: with `faithful != 0` every point where the unfused 16-bit (bf16 or fp16) chain rounds
// is rounded here too -- norm output, cos and sin, both products and their sum --
// so the result equals the op-by-op evaluation in that type; with `faithful == 0` the
// whole expression is evaluated in fp32 and rounded once.
//
// grid = (tokens, groups of head vectors); a workgroup of 4 waves handles 4 (d = 128, 192, 256) or 8
// (d = 64, 96) head vectors of one token per pass, each by 64 or 32 lanes, lane i owning elements i,
// i + lanes, ... (two, three or four of them).  The normalised vector goes through a few hundred bytes of
// LDS so that any rotary pairing (half-split, interleaved, partial rotary width) reads its partner from there.
#include <stdio.h>

#include "mi_common.h"
#include "mi_capi_internal.h"

namespace mi {

struct NormRopeParams {
  const uint16_t* q;  // [T][Hq][d]; head h at (h / q_group) * q_gst + (h % q_group) * d of its token
  int64_t q_st, q_gst;
  uint16_t* q_out;  // [T][Hq][d]; may alias q
  int64_t qo_st;
  const uint16_t* k;  // [T][Hkv][d]; head h at h * k_hst of its token
  int64_t k_st, k_hst;
  uint16_t* k_out;  // [T][Hkv][d] or null
  int64_t ko_st;
  const uint16_t* v;  // [T][Hkv][d] or null (append only); head h at h * v_hst of its token
  int64_t v_st, v_hst;
  const uint16_t* q_w;  // [d] bf16 or null
  const uint16_t* k_w;
  const float* emb;  // [max_pos][rot] angles, or null for no rotary
  int64_t emb_stride;
  const int64_t* q_pos;  // [T]
  const int64_t* k_pos;  // [T]
  uint16_t* kc;  // cache or null
  uint16_t* vc;
  int64_t chunk_elems, tok_elems;
  const int64_t* tok_chunk;  // slot mode A
  const int64_t* tok_local;
  const int32_t* bt;  // slot mode B (decode)
  int64_t bt_stride;
  const int32_t* lens;
  int32_t T, Hq, Hkv, d, rot, chunk, norm, interleaved, faithful, q_group;
  uint32_t q_group_magic;  // ceil(2^32 / q_group): h / q_group = umulhi(h, magic) for q_group > 1 (h * q_group < 2^32)
  float eps, mscale;
};

// one rounding to the tensors' 16-bit type and back
template <bool F16>
static __device__ __forceinline__ float round16(float x) { return to_f32<F16>(f32_to_16<F16>(x)); }
// the same for two values: one packed conversion and two unpacks
template <bool F16>
static __device__ __forceinline__ void round16_pair(float& a, float& b) {
  const uint32_t packed = pack2<F16>(a, b);
  a = lo_to_f32<F16>(packed);
  b = hi_to_f32<F16>(packed);
}

// First element of head vector `vec` (query heads first, then key heads) of token t.
static __device__ __forceinline__ const uint16_t* head_vector(const NormRopeParams& p, int t, int vec) {
  if (vec < p.Hq) {
    if (p.q_gst == 0) return p.q + (int64_t)t * p.q_st + (int64_t)vec * p.d;  // one group: contiguous heads
    const int g = p.q_group == 1 ? vec : (int)__umulhi((uint32_t)vec, p.q_group_magic);
    return p.q + (int64_t)t * p.q_st + (int64_t)g * p.q_gst + (int64_t)(vec - g * p.q_group) * p.d;
  }
  return p.k + (int64_t)t * p.k_st + (int64_t)(vec - p.Hq) * p.k_hst;
}

template <int D, bool F16>
__global__ __launch_bounds__(256) void norm_rope_append_kernel(NormRopeParams p) {
  constexpr int LPV = D >= 128 ? 64 : 32;  // lanes per head vector
  constexpr int EPL = D / LPV;             // elements per lane: i, i + LPV, ...
  constexpr int VPW = 64 / LPV;     // head vectors per wave
  constexpr int VPB = 4 * VPW;      // head vectors per workgroup pass
  static_assert(EPL * LPV == D && EPL >= 2 && EPL <= 4, "head widths 64, 96, 128, 192, 256");
  __shared__ float lds[VPB][D];

  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int i = lane % LPV;
  const int slot = wave * VPW + lane / LPV;
  const int nvec = p.Hq + p.Hkv;
  const bool faithful = p.faithful != 0;

  // Destination slot of this token in the cache (wave-uniform).
  int64_t cache_off = -1;
  if (p.kc) {
    if (p.tok_chunk) {
      cache_off = p.tok_chunk[t] * p.chunk_elems + p.tok_local[t] * p.tok_elems;
    } else {
      const int len = p.lens[t];
      if (len > 0) {
        const int pos = len - 1, ci = pos / p.chunk;
        cache_off = (int64_t)p.bt[(int64_t)t * p.bt_stride + ci] * p.chunk_elems +
                    (int64_t)(pos - ci * p.chunk) * p.tok_elems;
      }
    }
  }

  // cos / sin of this lane's elements depend only on the token position, not on the head:
  // evaluate them once (twice if query and key positions differ) and reuse them for every head.
  float cs[2][EPL][2] = {};  // [q|k][element][cos|sin]
  int partner[EPL] = {};
  float sign[EPL] = {};
  bool rotate[EPL] = {};
  if (p.emb) {
    const int64_t qp = p.q_pos ? p.q_pos[t] : 0;
    const int64_t kp = p.k_pos ? p.k_pos[t] : qp;
#pragma unroll
    for (int w = 0; w < EPL; ++w) {
      const int e = i + w * LPV;
      rotate[w] = e < p.rot;
      if (p.interleaved) {
        partner[w] = e ^ 1;
        sign[w] = (e & 1) ? 1.f : -1.f;
      } else {
        const int half = p.rot >> 1;
        partner[w] = e < half ? e + half : e - half;
        sign[w] = e < half ? -1.f : 1.f;
      }
      if (rotate[w]) {
#pragma unroll
        for (int which = 0; which < 2; ++which) {
          if (which == 1 && kp == qp && p.Hq > 0) {
            cs[1][w][0] = cs[0][w][0];
            cs[1][w][1] = cs[0][w][1];
            continue;
          }
          if ((which == 0 && p.Hq == 0) || (which == 1 && p.Hkv == 0)) continue;
          const float a = p.emb[(which ? kp : qp) * p.emb_stride + e];
          float c, sn;
          rotary_sincos(a, &sn, &c);
          c *= p.mscale;
          sn *= p.mscale;
          if (faithful) {
            c = round16<F16>(c);
            sn = round16<F16>(sn);
          }
          cs[which][w][0] = c;
          cs[which][w][1] = sn;
        }
      }
    }
  }

  for (int vec0 = blockIdx.y * VPB; vec0 < nvec; vec0 += gridDim.y * VPB) {
    const int vec = vec0 + slot;
    const bool active = vec < nvec;
    const bool is_q = vec < p.Hq;
    const int head = is_q ? vec : vec - p.Hq;
    float y[EPL] = {};
    if (active) {
      const uint16_t* src = head_vector(p, t, vec);
#pragma unroll
      for (int w = 0; w < EPL; ++w) y[w] = to_f32<F16>(src[i + w * LPV]);
    }
    if (p.norm != MI_NORM_NONE) {
      float ss = y[0] * y[0] + y[1] * y[1];
#pragma unroll
      for (int w = 2; w < EPL; ++w) ss += y[w] * y[w];
#pragma unroll
      for (int o = LPV / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
      const float rstd = rsqrtf(ss * (1.f / D) + p.eps);
      const uint16_t* wt = is_q ? p.q_w : p.k_w;
#pragma unroll
      for (int w = 0; w < EPL; ++w) {
        y[w] *= rstd;
        if (p.norm == MI_NORM_RMS && wt) y[w] *= to_f32<F16>(wt[i + w * LPV]);
        if (faithful) y[w] = round16<F16>(y[w]);
      }
    }
    float o[EPL];
#pragma unroll
    for (int w = 0; w < EPL; ++w) o[w] = y[w];
    if (p.emb) {
#pragma unroll
      for (int w = 0; w < EPL; ++w) lds[slot][i + w * LPV] = y[w];
      __syncthreads();
#pragma unroll
      for (int w = 0; w < EPL; ++w) {
        if (active && rotate[w]) {
          const float c = cs[is_q ? 0 : 1][w][0], sn = cs[is_q ? 0 : 1][w][1];
          const float yp = lds[slot][partner[w]] * sign[w];
          o[w] = faithful ? round16<F16>(y[w] * c) + round16<F16>(yp * sn) : y[w] * c + yp * sn;
        }
      }
      __syncthreads();
    }
    if (active) {
      uint16_t* dst_q = is_q ? p.q_out + (int64_t)t * p.qo_st + (int64_t)head * D : nullptr;
      uint16_t* dst_k = (!is_q && p.k_out) ? p.k_out + (int64_t)t * p.ko_st + (int64_t)head * D : nullptr;
      uint16_t* dst_c = (!is_q && cache_off >= 0) ? p.kc + cache_off + (int64_t)head * D : nullptr;
#pragma unroll
      for (int w = 0; w < EPL; ++w) {
        const uint16_t b = f32_to_16<F16>(o[w]);
        if (dst_q) dst_q[i + w * LPV] = b;
        if (dst_k) dst_k[i + w * LPV] = b;
        if (dst_c) dst_c[i + w * LPV] = b;
      }
    }
  }
  // Value rows are copied unchanged (by the first workgroup of the token).
  if (blockIdx.y == 0 && cache_off >= 0 && p.v) {
    uint32_t* dst = reinterpret_cast<uint32_t*>(p.vc + cache_off);
    for (int e = threadIdx.x; e < p.Hkv * D / 2; e += 256) {
      const int h = e / (D / 2);
      dst[e] = *reinterpret_cast<const uint32_t*>(p.v + (int64_t)t * p.v_st + (int64_t)h * p.v_hst + 2 * (e - h * (D / 2)));
    }
  }
}


// Vectorised variant: a head vector is handled by d/8 lanes with 8 contiguous elements (one 16-byte
// load / store) each.  The rotary partner of an element is in the same lane (interleaved pairs) or
// one lane shuffle away (half-split pairs, when rot/2 is a multiple of 8).  Same rounding points as
// norm_rope_append_kernel; only the order of the sum of squares differs.  grid = (tokens, groups of
// head vectors) as above, 16 (d = 128, 96), 32 (d = 64) or 8 (d = 192, 256) head vectors per workgroup pass;
// at d = 96 and 192 a vector's 12 / 24 lanes sit in a group of 16 / 32 whose other lanes idle.
//
// A token's work starts with a chain of dependent loads (position -> angle row -> cos / sin), so
// the kernel is latency-bound unless enough workgroups are resident and independent loads are in
// flight meanwhile: the first pass's head vector and the value row are requested before the chain,
// and cos / sin / norm weights live in LDS or packed registers to stay within 64 VGPRs (8 waves per
// SIMD).  Each angle's cos and sin are evaluated by exactly one thread of the workgroup.
template <int D, bool F16>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(6, 8))) void norm_rope_append_vec_kernel(NormRopeParams p) {
  constexpr int LPV = D / 8;        // lanes that hold a head vector
  constexpr int LPG = LPV <= 8 ? 8 : LPV <= 16 ? 16 : 32;  // lane group of a head vector (a power of two)
  constexpr int VPW = 64 / LPG;     // head vectors per wave
  constexpr int VPB = 4 * VPW;      // head vectors per workgroup pass
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int li = lane % LPG;
  const bool lane_on = LPG == LPV || li < LPV;
  const int slot = wave * VPW + lane / LPG;
  const int nvec = p.Hq + p.Hkv;
  const bool faithful = p.faithful != 0;
  const int e0 = lane_on ? 8 * li : 0;  // first element of this lane (idle lanes read what lane 0 reads)

  auto load_vec = [&](int vec) -> uint4 {
    if (vec >= nvec || !lane_on) return make_uint4(0, 0, 0, 0);
    return ld16(head_vector(p, t, vec) + e0);
  };
  // Independent of the position chain: first head vector, value row (first workgroup of the token).
  uint4 raw = load_vec(blockIdx.y * VPB + slot);
  const bool copy_v = blockIdx.y == 0 && p.kc && p.v;
  const int v_vecs = p.Hkv * D / 8;  // 16-byte pieces of a value row
  uint4 vraw[2] = {make_uint4(0, 0, 0, 0), make_uint4(0, 0, 0, 0)};
  auto load_v = [&](int piece) -> uint4 {  // piece = 16 bytes of the token's value row
    const int h = piece / LPV;
    return ld16(p.v + (int64_t)t * p.v_st + (int64_t)h * p.v_hst + 8 * (piece - h * LPV));
  };
  if (copy_v) {
#pragma unroll
    for (int r = 0; r < 2; ++r)
      if ((int)threadIdx.x + 256 * r < v_vecs) vraw[r] = load_v(threadIdx.x + 256 * r);
  }

  int64_t cache_off = -1;
  if (p.kc) {
    if (p.tok_chunk) {
      cache_off = p.tok_chunk[t] * p.chunk_elems + p.tok_local[t] * p.tok_elems;
    } else {
      const int len = p.lens[t];
      if (len > 0) {
        const int pos = len - 1, ci = pos / p.chunk;
        cache_off = (int64_t)p.bt[(int64_t)t * p.bt_stride + ci] * p.chunk_elems +
                    (int64_t)(pos - ci * p.chunk) * p.tok_elems;
      }
    }
  }

  __shared__ __align__(16) float cs_lds[2][2][D];  // [query | key position][cos | sin][element]
  const int half = p.rot >> 1;
  int src_lane = lane;   // lane holding the half-split partner elements (same j)
  bool same = true;      // query and key positions agree (uniform over the workgroup)
  if (p.emb) {
    const int64_t qp = p.q_pos ? p.q_pos[t] : 0;
    const int64_t kp = p.k_pos ? p.k_pos[t] : qp;
    same = kp == qp && p.Hq > 0;
    // one thread per (position, element): cos and sin together; the sine carries the sign of the partner term
    // (half-split pairs: minus in the first half; interleaved pairs: minus at even elements)
    for (int job = threadIdx.x; job < 2 * D; job += 256) {
      const int which = job / D, e = job % D;
      if (which == 1 && same) break;
      if ((which == 0 && p.Hq == 0) || (which == 1 && p.Hkv == 0)) continue;
      float c = 1.f, sn = 0.f;
      if (e < p.rot) {
        rotary_sincos(p.emb[(which ? kp : qp) * p.emb_stride + e], &sn, &c);
        c *= p.mscale;
        sn *= p.mscale;
        if (faithful) {
          c = round16<F16>(c);
          sn = round16<F16>(sn);
        }
        if (p.interleaved ? (e & 1) == 0 : e < half) sn = -sn;
      }
      cs_lds[which][0][e] = c;
      cs_lds[which][1][e] = sn;
    }
    if (!p.interleaved) {
      const int pe = e0 < half ? e0 + half : e0 - half;  // partner of this lane's first element
      src_lane = lane - li + pe / 8;
    }
  }
  // norm weights of this lane's elements, kept packed
  uint4 wq_raw = make_uint4(ones2<F16>(), ones2<F16>(), ones2<F16>(), ones2<F16>()), wk_raw = wq_raw;
  if (p.norm == MI_NORM_RMS) {
    if (p.q_w) wq_raw = ld16(p.q_w + e0);
    if (p.k_w) wk_raw = ld16(p.k_w + e0);
  }
  if (copy_v && cache_off >= 0) {
    uint16_t* dst = p.vc + cache_off;
#pragma unroll
    for (int r = 0; r < 2; ++r)
      if ((int)threadIdx.x + 256 * r < v_vecs) st16(dst + 8 * (threadIdx.x + 256 * r), vraw[r]);
    for (int e = threadIdx.x + 512; e < v_vecs; e += 256)  // more than 32 KV heads of 128
      st16(dst + 8 * e, load_v(e));
  }
  if (p.emb) __syncthreads();

  // The loop below is bound by vector-instruction issue (about as many instructions as a copy of the same bytes
  // leaves time for), so everything uniform is decided by scalar branches around whole element loops, lane
  // exchanges are single data-parallel moves where the distance allows, and cos = 1 / sin = 0 past the rotary
  // width make the rotation a pass-through there without a per-element test (non-finite inputs excepted: then the
  // select below keeps the reference's behaviour).
  const bool any_norm = p.norm != MI_NORM_NONE, rms = p.norm == MI_NORM_RMS;
  const int plane = half >> 3;                         // lanes between the partners of a half-split pair
  const bool pow2 = (half & 7) == 0 && plane > 0 && (plane & (plane - 1)) == 0 && 2 * plane <= LPG;
  const bool full_rot = p.rot == D;
  for (int vec0 = blockIdx.y * VPB; vec0 < nvec; vec0 += gridDim.y * VPB) {
    const int vec = vec0 + slot;
    const bool active = vec < nvec;  // uniform over the LPV lanes of a vector
    const bool is_q = vec < p.Hq;
    const int head = is_q ? vec : vec - p.Hq;
    float y[8];
    {
      const uint32_t w4[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) { y[2 * j] = lo_to_f32<F16>(w4[j]); y[2 * j + 1] = hi_to_f32<F16>(w4[j]); }
    }
    raw = load_vec(vec + gridDim.y * VPB);  // next pass, in flight during this one
    if (any_norm) {
      float ss = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) ss += y[j] * y[j];
      ss = lane_group_sum<LPG>(ss);
      const float rstd = rsqrtf(ss * (1.f / D) + p.eps);
#pragma unroll
      for (int j = 0; j < 8; ++j) y[j] *= rstd;
      if (rms) {
        const uint4 wr = is_q ? wq_raw : wk_raw;
        const uint32_t w4[4] = {wr.x, wr.y, wr.z, wr.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) { y[2 * j] *= lo_to_f32<F16>(w4[j]); y[2 * j + 1] *= hi_to_f32<F16>(w4[j]); }
      }
      if (faithful) {
#pragma unroll
        for (int j = 0; j < 8; j += 2) round16_pair<F16>(y[j], y[j + 1]);
      }
    }
    float o[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = y[j];
    if (p.emb) {
      const int which = (is_q || same) ? 0 : 1;
      float c[8], sn[8], yp[8];
#pragma unroll
      for (int j = 0; j < 8; j += 4) {
        const float4 c4 = *reinterpret_cast<const float4*>(&cs_lds[which][0][e0 + j]);
        const float4 s4 = *reinterpret_cast<const float4*>(&cs_lds[which][1][e0 + j]);
        c[j] = c4.x; c[j + 1] = c4.y; c[j + 2] = c4.z; c[j + 3] = c4.w;
        sn[j] = s4.x; sn[j + 1] = s4.y; sn[j + 2] = s4.z; sn[j + 3] = s4.w;
      }
      if (p.interleaved) {
#pragma unroll
        for (int j = 0; j < 8; ++j) yp[j] = y[j ^ 1];
      } else if (pow2) {  // the partner lane is lane ^ plane
#define MI_PARTNERS(P_)                                  \
  _Pragma("unroll") for (int j = 0; j < 8; ++j) yp[j] = lane_xor<P_>(y[j])
        if (plane == 8) { MI_PARTNERS(8); }
        else if (plane == 4) { MI_PARTNERS(4); }
        else if (plane == 16) { MI_PARTNERS(16); }
        else if (plane == 2) { MI_PARTNERS(2); }
        else { MI_PARTNERS(1); }
#undef MI_PARTNERS
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) yp[j] = __shfl(y[j], src_lane, 64);
      }
      if (faithful) {
#pragma unroll
        for (int j = 0; j < 8; j += 2) {
          float a0 = y[j] * c[j], a1 = y[j + 1] * c[j + 1], b0 = yp[j] * sn[j], b1 = yp[j + 1] * sn[j + 1];
          round16_pair<F16>(a0, a1);
          round16_pair<F16>(b0, b1);
          o[j] = a0 + b0;
          o[j + 1] = a1 + b1;
        }
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j] = y[j] * c[j] + yp[j] * sn[j];
      }
      if (!full_rot) {
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j] = e0 + j < p.rot ? o[j] : y[j];
      }
    }
    if (active && lane_on) {
      const uint4 packed = make_uint4(pack2<F16>(o[0], o[1]), pack2<F16>(o[2], o[3]),
                                      pack2<F16>(o[4], o[5]), pack2<F16>(o[6], o[7]));
      if (is_q) {
        st16(p.q_out + (int64_t)t * p.qo_st + (int64_t)head * D + e0, packed);
      } else {
        if (p.k_out) st16(p.k_out + (int64_t)t * p.ko_st + (int64_t)head * D + e0, packed);
        if (cache_off >= 0) st16(p.kc + cache_off + (int64_t)head * D + e0, packed);
      }
    }
  }
}

}  // namespace mi

using namespace mi;

namespace {

// Argument checks shared by both entry points, kernel choice and launch.  `p` carries every pointer,
// stride and size; `name` prefixes error messages.
int norm_rope_launch(NormRopeParams& p, int32_t dtype, const MiTuning* tuning, hipStream_t st, const char* name) {
  char msg[160];
  auto fail = [&](int code, const char* what) {
    snprintf(msg, sizeof msg, "%s: %s", name, what);
    return mi_fail(code, msg);
  };
  if (p.T == 0) return MI_OK;
  p.q_group_magic = p.q_group > 1 ? (uint32_t)((((uint64_t)1 << 32) + p.q_group - 1) / p.q_group) : 0u;
  MiTuning tune;
  const int rc_t = mi_resolve_tuning(tuning, &tune, name);
  if (rc_t != MI_OK) return rc_t;
  if (dtype != MI_DTYPE_BF16 && dtype != MI_DTYPE_FP16) return fail(MI_ERR_UNSUPPORTED, "dtype must be MI_DTYPE_BF16 or MI_DTYPE_FP16");
  const bool f16 = dtype == MI_DTYPE_FP16;
  if (p.T < 0 || p.Hq < 0 || p.Hkv < 0 || p.Hq + p.Hkv == 0) return fail(MI_ERR_SHAPE, "bad sizes");
  if ((p.Hq > 0 && (!p.q || !p.q_out)) || (p.Hkv > 0 && !p.k)) return fail(MI_ERR_NULL, "q / q_out / k missing");
  if (p.d != 64 && p.d != 96 && p.d != 128 && p.d != 192 && p.d != 256)
    return fail(MI_ERR_UNSUPPORTED, "head_dim must be 64, 96, 128, 192 or 256");
  if (p.norm != MI_NORM_NONE && p.norm != MI_NORM_RMS && p.norm != MI_NORM_L2)
    return fail(MI_ERR_UNSUPPORTED, "unknown norm kind");
  if (p.emb) {
    if (p.rot <= 0 || p.rot > p.d || (p.rot & 1) || p.emb_stride < p.rot)
      return fail(MI_ERR_SHAPE, "rot_dim must be even and within head_dim");
    if ((p.Hq > 0 && !p.q_pos) || (p.Hkv > 0 && !p.k_pos)) return fail(MI_ERR_NULL, "rotary positions missing");
  }
  const bool to_cache = p.kc != nullptr;
  if (to_cache) {
    if (!p.vc || !p.v) return fail(MI_ERR_NULL, "append needs v and v_cache");
    const bool mode_a = p.tok_chunk && p.tok_local;
    const bool mode_b = p.bt && p.lens && p.chunk > 0;
    if (!mode_a && !mode_b) return fail(MI_ERR_NULL, "append needs per-token slots or block table + lengths");
    if ((((uintptr_t)p.v | (uintptr_t)p.vc) & 3) || ((p.v_st | p.v_hst | p.chunk_elems | p.tok_elems) & 1))
      return fail(MI_ERR_ALIGN, "value rows must be 4-byte aligned");
  }
  if (!(p.tok_chunk && p.tok_local)) p.tok_chunk = nullptr;
  // Few tokens (decode): spread the heads of a token over several workgroups for latency.
  // Many tokens (prefill): one workgroup per token loops over the heads and reuses cos / sin.
  // The vectorised kernel needs 16-byte rows and every rotary partner in the same lane or a whole
  // number of lanes away; anything else takes the element-wise kernel.
  const bool rot_ok = !p.emb || p.interleaved || (p.rot % 16 == 0);
  const uintptr_t ptrs = (uintptr_t)p.q | (uintptr_t)p.q_out | (uintptr_t)p.k | (uintptr_t)p.k_out | (uintptr_t)p.kc |
                         (uintptr_t)p.q_w | (uintptr_t)p.k_w | (to_cache ? ((uintptr_t)p.v | (uintptr_t)p.vc) : 0);
  const int64_t strides = p.q_st | p.q_gst | p.qo_st | p.k_st | p.k_hst | p.ko_st |
                          (to_cache ? (p.chunk_elems | p.tok_elems | p.v_st | p.v_hst) : 0);
  // The 16-byte-per-lane kernel wins on many tokens; on a decode batch (a few hundred rows at most) the
  // element-wise kernel's shorter dependent chain does (4.8 against 5.7 us at 64 tokens).
  const int mode = tune.norm_rope_vectorised;  // -1 never, 1 whenever the shapes allow, 2 automatic
  const bool vec = rot_ok && (ptrs & 15) == 0 && (strides & 7) == 0 && (mode == 1 || (mode == 2 && p.T >= 256));
  // head vectors per workgroup pass (see the kernels)
  const int vpb = vec ? (p.d == 64 ? 32 : p.d <= 128 ? 16 : 8) : (p.d >= 128 ? 4 : 8);
  const int passes = (p.Hq + p.Hkv + vpb - 1) / vpb;
  int gy = (2048 + p.T - 1) / p.T;
  gy = gy < 1 ? 1 : (gy > passes ? passes : gy);
  dim3 grid(p.T, gy);
#define MI_NR_LAUNCH(KERNEL_)                                                                   \
  do {                                                                                          \
    if (p.d == 128 && f16) hipLaunchKernelGGL((KERNEL_<128, true>), grid, dim3(256), 0, st, p);   \
    else if (p.d == 128) hipLaunchKernelGGL((KERNEL_<128, false>), grid, dim3(256), 0, st, p);    \
    else if (p.d == 64 && f16) hipLaunchKernelGGL((KERNEL_<64, true>), grid, dim3(256), 0, st, p);  \
    else if (p.d == 64) hipLaunchKernelGGL((KERNEL_<64, false>), grid, dim3(256), 0, st, p);      \
    else if (p.d == 96 && f16) hipLaunchKernelGGL((KERNEL_<96, true>), grid, dim3(256), 0, st, p);  \
    else if (p.d == 96) hipLaunchKernelGGL((KERNEL_<96, false>), grid, dim3(256), 0, st, p);      \
    else if (p.d == 192 && f16) hipLaunchKernelGGL((KERNEL_<192, true>), grid, dim3(256), 0, st, p); \
    else if (p.d == 192) hipLaunchKernelGGL((KERNEL_<192, false>), grid, dim3(256), 0, st, p);    \
    else if (f16) hipLaunchKernelGGL((KERNEL_<256, true>), grid, dim3(256), 0, st, p);            \
    else hipLaunchKernelGGL((KERNEL_<256, false>), grid, dim3(256), 0, st, p);                    \
  } while (0)
  if (vec) MI_NR_LAUNCH(norm_rope_append_vec_kernel);
  else MI_NR_LAUNCH(norm_rope_append_kernel);
#undef MI_NR_LAUNCH
  return mi_check_launch(name);
}

}  // namespace

extern "C" int mi_norm_rope_append(
    const void* q, int64_t q_stride_tok, void* q_out, int64_t q_out_stride_tok, const void* k,
    int64_t k_stride_tok, void* k_out,
    int64_t k_out_stride_tok, const void* v, int64_t v_stride_tok, const void* q_weight,
    const void* k_weight, float eps, int32_t norm_kind, const float* rotary_angles,
    int64_t angles_stride, int32_t rot_dim, int32_t rotary_interleaved, float mscale,
    const int64_t* q_positions, const int64_t* k_positions, void* k_cache, void* v_cache,
    int64_t kv_stride_chunk, int64_t kv_stride_tok, const int64_t* token_to_chunk_idx,
    const int64_t* token_to_local_pos, const int32_t* block_table, int64_t bt_stride,
    const int32_t* kv_lens, int32_t chunk_tokens, int32_t T, int32_t Hq, int32_t Hkv,
    int32_t head_dim, int32_t faithful_rounding, int32_t dtype, const MiTuning* tuning, void* stream) {
  NormRopeParams p = {};
  p.q = (const uint16_t*)q; p.q_st = q_stride_tok; p.q_gst = 0; p.q_group = Hq > 0 ? Hq : 1;
  p.q_out = (uint16_t*)q_out; p.qo_st = q_out_stride_tok;
  p.k = (const uint16_t*)k; p.k_st = k_stride_tok; p.k_hst = head_dim;
  p.k_out = (uint16_t*)k_out; p.ko_st = k_out_stride_tok;
  p.v = (const uint16_t*)v; p.v_st = v_stride_tok; p.v_hst = head_dim;
  p.q_w = (const uint16_t*)q_weight; p.k_w = (const uint16_t*)k_weight;
  p.emb = rotary_angles; p.emb_stride = angles_stride;
  p.q_pos = q_positions; p.k_pos = k_positions;
  p.kc = (uint16_t*)k_cache; p.vc = (uint16_t*)v_cache;
  p.chunk_elems = kv_stride_chunk; p.tok_elems = kv_stride_tok;
  p.tok_chunk = token_to_chunk_idx; p.tok_local = token_to_local_pos;
  p.bt = block_table; p.bt_stride = bt_stride; p.lens = kv_lens;
  p.T = T; p.Hq = Hq; p.Hkv = Hkv; p.d = head_dim; p.rot = rot_dim; p.chunk = chunk_tokens;
  p.norm = norm_kind; p.interleaved = rotary_interleaved; p.faithful = faithful_rounding;
  p.eps = eps; p.mscale = mscale;
  return norm_rope_launch(p, dtype, tuning, (hipStream_t)stream, "mi_norm_rope_append");
}

extern "C" int mi_qkv_norm_rope_append(
    const void* mixed_qkv, int64_t qkv_stride_tok, void* q_out, int64_t q_out_stride_tok, void* k_out,
    int64_t k_out_stride_tok, const void* q_weight, const void* k_weight, float eps, int32_t norm_kind,
    const float* rotary_angles, int64_t angles_stride, int32_t rot_dim, int32_t rotary_interleaved,
    float mscale, const int64_t* q_positions, const int64_t* k_positions, void* k_cache, void* v_cache,
    int64_t kv_stride_chunk, int64_t kv_stride_tok, const int64_t* token_to_chunk_idx,
    const int64_t* token_to_local_pos, const int32_t* block_table, int64_t bt_stride,
    const int32_t* kv_lens, int32_t chunk_tokens, int32_t T, int32_t Hq, int32_t Hkv,
    int32_t head_dim, int32_t faithful_rounding, int32_t dtype, const MiTuning* tuning, void* stream) {
  if (T == 0) return MI_OK;
  if (!mixed_qkv) return mi_fail(MI_ERR_NULL, "mi_qkv_norm_rope_append: mixed_qkv missing");
  if (Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0)
    return mi_fail(MI_ERR_SHAPE, "mi_qkv_norm_rope_append: query heads must be a positive multiple of KV heads");
  if (!k_cache && !k_out)
    return mi_fail(MI_ERR_NULL, "mi_qkv_norm_rope_append: the key needs a destination (k_out and/or the cache)");
  const int G = Hq / Hkv;
  const int64_t group = (int64_t)(G + 2) * head_dim;  // elements of one query group: G q heads, k, v
  if (qkv_stride_tok < group * Hkv)
    return mi_fail(MI_ERR_SHAPE, "mi_qkv_norm_rope_append: token stride smaller than (Hq + 2 Hkv) * head_dim");
  const uint16_t* base = (const uint16_t*)mixed_qkv;
  NormRopeParams p = {};
  p.q = base; p.q_st = qkv_stride_tok; p.q_gst = group; p.q_group = G;
  p.q_out = (uint16_t*)q_out; p.qo_st = q_out_stride_tok;
  p.k = base + (int64_t)G * head_dim; p.k_st = qkv_stride_tok; p.k_hst = group;
  p.k_out = (uint16_t*)k_out; p.ko_st = k_out_stride_tok;
  p.v = k_cache ? base + (int64_t)(G + 1) * head_dim : nullptr; p.v_st = qkv_stride_tok; p.v_hst = group;
  p.q_w = (const uint16_t*)q_weight; p.k_w = (const uint16_t*)k_weight;
  p.emb = rotary_angles; p.emb_stride = angles_stride;
  p.q_pos = q_positions; p.k_pos = k_positions;
  p.kc = (uint16_t*)k_cache; p.vc = (uint16_t*)v_cache;
  p.chunk_elems = kv_stride_chunk; p.tok_elems = kv_stride_tok;
  p.tok_chunk = token_to_chunk_idx; p.tok_local = token_to_local_pos;
  p.bt = block_table; p.bt_stride = bt_stride; p.lens = kv_lens;
  p.T = T; p.Hq = Hq; p.Hkv = Hkv; p.d = head_dim; p.rot = rot_dim; p.chunk = chunk_tokens;
  p.norm = norm_kind; p.interleaved = rotary_interleaved; p.faithful = faithful_rounding;
  p.eps = eps; p.mscale = mscale;
  return norm_rope_launch(p, dtype, tuning, (hipStream_t)stream, "mi_qkv_norm_rope_append");
}
