// Paged GQA decode attention for gfx950: split-K flash-decode + log-sum-exp merge.
//
// Replaces the `flash_attn_with_kvcache(q, k_cache, v_cache, cache_seqlens,
// causal=True, block_table)` call of the reference
// (megatron/core/transformer/attention.py:589-600): one query token per request
// attends to the request's tokens scattered over fixed-size chunks of a
// `[n_chunks, chunk, Hkv, d]` cache, addressed through a `[R, M]` block table.
//
// Work decomposition ("flattened stream")
//   Every request is cut into tiles of 16*NT tokens and the tiles of all requests are
//   laid end to end.  A fixed grid of workgroups (a small multiple of the CU count)
//   divides that sequence into equal contiguous spans, so every workgroup streams the
//   same number of bytes whatever the mix of context lengths, and pays its start-up cost
//   once.  A span that crosses a request boundary yields one segment per request; a
//   segment that is a whole request writes bf16 output directly, any other segment
//   writes a normalised fp32 partial + base-2 LSE into slot (workgroup index + request
//   index), which is unique because both indices only grow along the sequence.
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
//   needs a cross-lane step (two exchanges across g); the row sums are one more
//   16x16x16 product with an all-ones A operand.
//
// A second kernel merges the partials of each request,
//   o = sum_s 2^(lse_s - max) o_s / sum_s 2^(lse_s - max),
// and writes zeros for zero-length (padded) rows.
#include <stdio.h>

#include "mi_common.h"

#include <atomic>
#include <type_traits>
#include "mi_capi_internal.h"

namespace mi {

constexpr int MI_FUSED_FP8_NT = 2;  // 16-token sub-tiles per iteration of the one-kernel decode step over an fp8 cache

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
  const int32_t* cu_q;  // null: row r of q/out belongs to request r.  Else (mixed batches): only
                        // requests with exactly one query row take part, at row cu_q[r].
  uint16_t* out;
  int64_t o_st, o_sh;
  float* part_o;     // [slots][Hq][HD], slots = grid + R
  float* part_lse;   // [slots][Hq]
  int32_t* seg_info;  // [R][2]: first and last workgroup that touched request r
  const float* k_scale;  // fp8 only: [n_chunks][Hkv] (written by the fused step when a token opens a chunk)
  const float* v_scale;
  float headroom;        // fp8 fused step: scale of a chunk a token opens = headroom * amax(token) / 448
  uint64_t chunk_magic;  // ceil(2^40 / chunk)
  int32_t R, Hq, Hkv, G, chunk, min_span_tiles, grid;
  int32_t parts;  // wavefronts per KV head: each takes up to 16 of the G query heads that share it
  // Fused decode step only (FUSED kernels): `q` holds the raw queries of the step, head h * G + u of a row at
  // h * q_gst + u * d; the step's new key / value rows, norm weights, rotary table and positions.
  int64_t q_gst;
  const uint16_t* nk;  // [R][Hkv][d]: head h of row r at r * nk_st + h * nk_hst
  int64_t nk_st, nk_hst;
  const uint16_t* nv;
  int64_t nv_st, nv_hst;
  const uint16_t* q_w;  // [d] or null
  const uint16_t* k_w;
  const float* emb;  // [max_pos][rot] angles or null
  int64_t emb_stride;
  const int64_t* pos;  // [R] rotary position of the step's token
  int32_t rot, norm, interleaved, faithful;
  float eps, mscale;
  float scale_log2;
};

// tok / chunk for 0 <= tok < 2^31 via a 40-bit reciprocal (exact while tok * chunk < 2^40).
static __device__ __forceinline__ int chunk_of(int tok, uint64_t magic) {
  return (int)(((uint64_t)(uint32_t)tok * magic) >> 40);
}

// One segment: tokens [start, end) of request r for KV head h (one wavefront) and the `gq` <= 16 query heads
// hq0 .. hq0 + gq - 1 that share it.  `whole` = the segment is the entire request (write the 16-bit output, no
// partial).
// HDK = width of the keys (and queries), HDV = width of the values (and of the output).  They differ
// only for the latent cache of multi-latent attention (576 / 512: the value is the first 512 of the
// shared 576-wide row, the caller points both cache arguments at the same buffer).
//
// FUSED: the segment starts from the RAW queries of the step and does what the separate norm / rotary / append
// launch does (same arithmetic and rounding points as norm_rope_append_kernel): every segment normalises and
// rotates its query rows in registers; the segment that ends the request (`final_seg`: the only one that reads
// the step's new token) first normalises and rotates the new key row of its KV head, writes it and the value
// row into their cache slot, and orders that write before its own reads.  `q_lds` is then this wavefront's
// piece of LDS for cos / sin of the request's position [2][HDK] and the key row [HDK] (fp32).
template <int HDK, int HDV, int NT, bool FP8, bool F16, bool FUSED = false>
static __device__ __forceinline__ void decode_segment(const DecodeParams& p, int r, int row, int h, int hq0, int gq,
                                                      int len, int start, int end, bool whole, bool final_seg,
                                                      int slot, int lane, uint8_t* q_lds) {
  constexpr int KS = HDK / 32;
  // Wide keys (the 576-wide latent rows): the query fragments would take 72 registers per lane next
  // to 128 accumulator registers, so they live in this wavefront's piece of LDS instead (16 rows with
  // a pitch that spreads the 16 rows of a fragment read over all banks).
  constexpr bool Q_IN_LDS = HDK > 256;
  // The latent rows are read twice (as keys, then their first part as values) and by every query
  // group: those loads stay cacheable; an ordinary KV cache is read exactly once and streams past.
  constexpr bool SHARED_KV = HDK != HDV;
  constexpr int kQPitch = HDK * 2 + 16;
  constexpr int DV = HDV / 16;
  constexpr int VD = FP8 ? DV / 4 : DV / 2;  // dwords per token and lane of the value operand
  static_assert(HDK % 32 == 0 && HDV % 32 == 0 && HDK >= 64 && HDV >= 64, "head widths: multiples of 32");
  static_assert(!FP8 || (HDK == HDV && (HDK == 64 || HDK == 128)), "fp8 KV: head_dim 64 or 128");
  static_assert(!FUSED || (HDK == HDV && HDK <= 256), "fused step: an ordinary per-head cache");
  constexpr int ESZ = FP8 ? 1 : 2;
  // Everything that describes the segment is wave-uniform; as scalars, the chunk lookup and the
  // tile base addresses below run on the scalar unit instead of costing vector instructions.
  r = __builtin_amdgcn_readfirstlane(r);
  row = __builtin_amdgcn_readfirstlane(row);
  len = __builtin_amdgcn_readfirstlane(len);
  start = __builtin_amdgcn_readfirstlane(start);
  end = __builtin_amdgcn_readfirstlane(end);
  slot = __builtin_amdgcn_readfirstlane(slot);
  const int m16 = lane & 15, g = lane >> 4;
  const int G = gq;
  const int hq = hq0 + m16;  // query head of this lane's row (valid when m16 < G)
  // Loads are clamped to the last token of this segment (not of the request): the software
  // pipeline requests one tile past the end, and that tile belongs to another workgroup's span --
  // clamped, the request degenerates to re-reading one row instead of streaming 2 tiles from HBM.
  const int last = min(end, len) - 1;

  // Query fragments: B operand rows are the G heads of this KV head.
  uint4 qf[Q_IN_LDS ? 1 : KS];
  const uint8_t* q_frag = q_lds + m16 * kQPitch + 16 * g;  // this lane's fragment of step kk: + 64 kk
  {
    const uint16_t* qrow = FUSED ? p.q + (int64_t)row * p.q_st + (int64_t)h * p.q_gst + (int64_t)(hq - h * p.G) * HDK
                                 : p.q + (int64_t)row * p.q_st + (int64_t)hq * p.q_sh;
    if (Q_IN_LDS) {
#pragma unroll
      for (int kk = 0; kk < KS; ++kk)
        *reinterpret_cast<uint4*>(q_lds + m16 * kQPitch + 16 * g + 64 * kk) =
            (m16 < G) ? ld16(qrow + 32 * kk + 8 * g) : make_uint4(0, 0, 0, 0);
      // (every lane reads back exactly what it wrote, so no cross-lane ordering is needed)
    } else {
#pragma unroll
      for (int kk = 0; kk < KS; ++kk) {
        // bf16 cache: lane g owns d = 32kk + 8g .. +7.
        // fp8 cache : K bytes are loaded 16 per lane, d = 64u + 16g + 8half .. +7
        //             for mfma step kk = 2u + half.
        const int d0 = FP8 ? (64 * (kk >> 1) + 16 * g + 8 * (kk & 1)) : (32 * kk + 8 * g);
        qf[kk] = (m16 < G) ? ld16(qrow + d0) : make_uint4(0, 0, 0, 0);
      }
    }
  }

  const uint8_t* kbase = p.kc + (int64_t)h * p.kv_sh * ESZ;
  const uint8_t* vbase = p.vc + (int64_t)h * p.kv_sh * ESZ;
  const int64_t chunk_bytes = p.kv_sc * ESZ;
  const uint32_t tok_bytes = (uint32_t)(p.kv_st * ESZ);

  // first element of this lane's 8 of fragment kk (see the query loads above)
  auto frag_d0 = [&](int kk) { return FP8 ? 64 * (kk >> 1) + 16 * g + 8 * (kk & 1) : 32 * kk + 8 * g; };
  float* const cs = reinterpret_cast<float*>(q_lds);  // fused: [2][HDK]: cos | sin at the request's position
  float* const kx = cs + 2 * HDK;                     // fused: [HDK]: the normalised key row (rotary partners)
  const bool faithful = FUSED && p.faithful != 0;
  // LDS traffic between the lanes of one wavefront: order it for the compiler, the hardware runs it in order
  auto wave_sync = [] {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };
  // Requested here, ahead of the block-table round trip below, so that the two overlap: the rotary angles of
  // elements lane, lane + 64 at the request's position and the norm weights of this lane's query elements.
  constexpr int NA = (HDK + 63) / 64;
  float ang[NA];
  uint4 qwr[KS];
  if constexpr (FUSED) {
    if (p.emb) {
      // (no position array: the step's token sits at the request's last position, which is already at hand)
      const int64_t pos = p.pos ? p.pos[row] : (int64_t)(len - 1);
#pragma unroll
      for (int i = 0; i < NA; ++i) ang[i] = lane + 64 * i < p.rot ? p.emb[pos * p.emb_stride + lane + 64 * i] : 0.f;
    }
#pragma unroll
    for (int kk = 0; kk < KS; ++kk)
      qwr[kk] = (p.norm == MI_NORM_RMS && p.q_w) ? ld16(p.q_w + frag_d0(kk))
                                                 : make_uint4(ones2<F16>(), ones2<F16>(), ones2<F16>(), ones2<F16>());
  }
  // fp8 fused step: the scales of the chunk that takes the step's token, as this wavefront knows them after its
  // append (it reads them from these registers, never back from memory: the loads of the cursor below may have
  // been issued before the store of a scale this very step set)
  bool own_scale = false;   // the token opened its chunk: own_ksc / own_vsc are that chunk's scales
  float own_ksc = 1.f, own_vsc = 1.f;
  auto fused_cos_sin = [&] {
    if (p.emb) {
#pragma unroll
      for (int i = 0; i < NA; ++i) {
        const int e = lane + 64 * i;
        if (e >= HDK) break;
        float c = 1.f, sn = 0.f;  // elements past the rotary width pass through
        if (e < p.rot) {
          const float a = ang[i];
          rotary_sincos(a, &sn, &c);
          c *= p.mscale;
          sn *= p.mscale;
          if (faithful) {
            c = to_f32<F16>(f32_to_16<F16>(c));
            sn = to_f32<F16>(f32_to_16<F16>(sn));
          }
        }
        cs[e] = c;
        cs[HDK + e] = sn;
      }
      wave_sync();
    }
  };
  // ---- the step's new key / value rows of this KV head -> their cache slot (the request's last position) ----
  // (With more than 16 query heads per KV head every wavefront of the head writes the same bytes: each one orders
  // its own write before its own reads, and none has to wait for another.)
  auto fused_append = [&] {
    {
      constexpr int LPV = HDK >= 128 ? 64 : 32, EPL = HDK / LPV;  // lane i owns elements i, i + LPV, ...
      const bool on = lane < LPV;
      const int i = on ? lane : 0;
      const uint16_t* src = p.nk + (int64_t)row * p.nk_st + (int64_t)h * p.nk_hst;
      float y[EPL];
#pragma unroll
      for (int w = 0; w < EPL; ++w) y[w] = on ? to_f32<F16>(src[i + w * LPV]) : 0.f;
      if (p.norm != MI_NORM_NONE) {
        float ss = y[0] * y[0] + y[1] * y[1];
#pragma unroll
        for (int w = 2; w < EPL; ++w) ss += y[w] * y[w];
#pragma unroll
        for (int o = LPV / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
        const float rstd = rsqrtf(ss * (1.f / HDK) + p.eps);
#pragma unroll
        for (int w = 0; w < EPL; ++w) {
          y[w] *= rstd;
          if (p.norm == MI_NORM_RMS && p.k_w) y[w] *= to_f32<F16>(p.k_w[i + w * LPV]);
          if (faithful) y[w] = to_f32<F16>(f32_to_16<F16>(y[w]));
        }
      }
      float o[EPL];
#pragma unroll
      for (int w = 0; w < EPL; ++w) o[w] = y[w];
      if (p.emb) {
        if (on) {
#pragma unroll
          for (int w = 0; w < EPL; ++w) kx[i + w * LPV] = y[w];
        }
        wave_sync();
        const int half = p.rot >> 1;
#pragma unroll
        for (int w = 0; w < EPL; ++w) {
          const int e = i + w * LPV;
          if (on && e < p.rot) {
            const int partner = p.interleaved ? (e ^ 1) : (e < half ? e + half : e - half);
            const float sign = p.interleaved ? ((e & 1) ? 1.f : -1.f) : (e < half ? -1.f : 1.f);
            const float yp = kx[partner] * sign;
            const float c = cs[e], sn = cs[HDK + e];
            o[w] = faithful ? to_f32<F16>(f32_to_16<F16>(y[w] * c)) + to_f32<F16>(f32_to_16<F16>(yp * sn))
                            : y[w] * c + yp * sn;
          }
        }
      }
      const int cpos = len - 1, ci = chunk_of(cpos, p.chunk_magic);
      const int pc_new = p.bt[(int64_t)r * p.bt_stride + ci];
      const int64_t slot_bytes = (int64_t)pc_new * chunk_bytes + (int64_t)(cpos - ci * p.chunk) * tok_bytes;
      if constexpr (FP8) {
        // Quantising append, the policy of the separate launch (kv_append_decode_fp8_kernel): a token that opens a
        // chunk fixes the chunk-head's scale to headroom * amax(token) / 448, later tokens reuse the stored scale
        // and saturate; the key row is rounded to bf16 first, as the separate norm / rotary launch hands it over.
        const bool opens = cpos == ci * p.chunk;  // wave-uniform
        float* const ksc_p = const_cast<float*>(p.k_scale) + (int64_t)pc_new * p.Hkv + h;
        float* const vsc_p = const_cast<float*>(p.v_scale) + (int64_t)pc_new * p.Hkv + h;
        const uint16_t* vsrc = p.nv + (int64_t)row * p.nv_st + (int64_t)h * p.nv_hst;
        float kq[EPL], vq[EPL];
#pragma unroll
        for (int w = 0; w < EPL; ++w) {
          kq[w] = on ? to_f32<F16>(f32_to_16<F16>(o[w])) : 0.f;
          vq[w] = on ? to_f32<F16>(vsrc[i + w * LPV]) : 0.f;
        }
        float ksc, vsc;
        if (opens) {
          float ka = 0.f, va = 0.f;
#pragma unroll
          for (int w = 0; w < EPL; ++w) {
            ka = fmaxf(ka, fabsf(kq[w]));
            va = fmaxf(va, fabsf(vq[w]));
          }
#pragma unroll
          for (int off = 32; off > 0; off >>= 1) {
            ka = fmaxf(ka, __shfl_xor(ka, off, 64));
            va = fmaxf(va, __shfl_xor(va, off, 64));
          }
          ksc = ka > 0.f ? p.headroom * ka / 448.f : 1.f;
          vsc = va > 0.f ? p.headroom * va / 448.f : 1.f;
          if (lane == 0) {
            *ksc_p = ksc;
            *vsc_p = vsc;
          }
          own_scale = true;
        } else {
          ksc = *ksc_p;
          vsc = *vsc_p;
        }
        own_ksc = ksc;
        own_vsc = vsc;
        uint8_t* kdst8 = const_cast<uint8_t*>(kbase) + slot_bytes;
        uint8_t* vdst8 = const_cast<uint8_t*>(vbase) + slot_bytes;
        if (on) {
#pragma unroll
          for (int w = 0; w < EPL; ++w) {
            kdst8[i + w * LPV] = (uint8_t)f32_to_e4m3_sat(kq[w] / ksc);
            vdst8[i + w * LPV] = (uint8_t)f32_to_e4m3_sat(vq[w] / vsc);
          }
        }
      } else {
      uint16_t* kdst = reinterpret_cast<uint16_t*>(const_cast<uint8_t*>(kbase) + slot_bytes);
      if (on) {
#pragma unroll
        for (int w = 0; w < EPL; ++w) kdst[i + w * LPV] = f32_to_16<F16>(o[w]);
      }
      const uint32_t* vsrc = reinterpret_cast<const uint32_t*>(p.nv + (int64_t)row * p.nv_st + (int64_t)h * p.nv_hst);
      uint32_t* vdst = reinterpret_cast<uint32_t*>(const_cast<uint8_t*>(vbase) + slot_bytes);
      for (int e = lane; e < HDV / 2; e += 64) vdst[e] = vsrc[e];
      }
      // The rows just written are read back below by other lanes of this same wavefront and by nobody else in
      // this launch (it owns the request's last tiles): wait until the stores have reached the L2 (their
      // acknowledgement), then keep the compiler from moving the loads up.  No cache has to be written back or
      // invalidated for that -- the lines cannot sit in this CU's L1 (nothing read them before), and a wider
      // scope would flush the L2 of the whole XCD under the other wavefronts' streams.
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    }
  };
  // ---- this wavefront's query rows: lane (m16, g) holds elements 32 kk + 8 g .. + 7 of head m16 ----
  auto fused_queries = [&] {
    float x[KS][8];
#pragma unroll
    for (int kk = 0; kk < KS; ++kk) {
      const uint32_t w4[4] = {qf[kk].x, qf[kk].y, qf[kk].z, qf[kk].w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        x[kk][2 * j] = lo_to_f32<F16>(w4[j]);
        x[kk][2 * j + 1] = hi_to_f32<F16>(w4[j]);
      }
    }
    if (p.norm != MI_NORM_NONE) {
      float ss = 0.f;
#pragma unroll
      for (int kk = 0; kk < KS; ++kk)
#pragma unroll
        for (int j = 0; j < 8; ++j) ss += x[kk][j] * x[kk][j];
      ss += xor16(ss);
      ss += xor32(ss);
      const float rstd = rsqrtf(ss * (1.f / HDK) + p.eps);
#pragma unroll
      for (int kk = 0; kk < KS; ++kk) {
        const uint32_t w4[4] = {qwr[kk].x, qwr[kk].y, qwr[kk].z, qwr[kk].w};
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          float v = x[kk][j] * rstd;
          if (p.norm == MI_NORM_RMS && p.q_w) v *= (j & 1) ? hi_to_f32<F16>(w4[j >> 1]) : lo_to_f32<F16>(w4[j >> 1]);
          x[kk][j] = faithful ? to_f32<F16>(f32_to_16<F16>(v)) : v;
        }
      }
    }
    if (p.emb) {
      // one rotated element: y cos + (partner, signed) sin, with the op chain's roundings when asked for
      auto rotated = [&](float y, float yp, float c, float sn) {
        return faithful ? to_f32<F16>(f32_to_16<F16>(y * c)) + to_f32<F16>(f32_to_16<F16>(yp * sn)) : y * c + yp * sn;
      };
      // cos | sin of this lane's elements j .. j + 3 of fragment kk (j = 0 or 4)
      auto cos_sin = [&](int kk, int j, float (&c)[4], float (&sn)[4]) {
        const float4 c4 = *reinterpret_cast<const float4*>(&cs[frag_d0(kk) + j]);
        const float4 s4 = *reinterpret_cast<const float4*>(&cs[HDK + frag_d0(kk) + j]);
        c[0] = c4.x; c[1] = c4.y; c[2] = c4.z; c[3] = c4.w;
        sn[0] = s4.x; sn[1] = s4.y; sn[2] = s4.z; sn[3] = s4.w;
      };
      // fragments ka < kb whose elements are each other's partners (half-split pairs), rotated in place
      auto rotate_pair = [&](int ka, int kb) {
#pragma unroll
        for (int j0 = 0; j0 < 8; j0 += 4) {
          float ca[4], sa[4], cb[4], sb[4];
          cos_sin(ka, j0, ca, sa);
          cos_sin(kb, j0, cb, sb);
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float ya = x[ka][j0 + j], yb = x[kb][j0 + j];
            x[ka][j0 + j] = rotated(ya, -yb, ca[j], sa[j]);
            x[kb][j0 + j] = rotated(yb, ya, cb[j], sb[j]);
          }
        }
      };
      if (p.interleaved) {
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) {
#pragma unroll
          for (int j0 = 0; j0 < 8; j0 += 4) {
            float c[4], sn[4];
            cos_sin(kk, j0, c, sn);
#pragma unroll
            for (int j = 0; j < 4; j += 2) {
              if (frag_d0(kk) + j0 + j < p.rot) {  // (rot_dim is even: a pair lies within it or beyond)
                const float ya = x[kk][j0 + j], yb = x[kk][j0 + j + 1];
                x[kk][j0 + j] = rotated(ya, -yb, c[j], sn[j]);
                x[kk][j0 + j + 1] = rotated(yb, ya, c[j + 1], sn[j + 1]);
              }
            }
          }
        }
      } else {
        // half-split pairs: partners are rot_dim / 2 elements = nf fragments apart (the entry point admits only
        // whole numbers of fragments); fragments beyond the rotary width pass through
        const int nf = p.rot >> 6;
        if (nf == 1) {
          rotate_pair(0, 1);
        } else if (nf == 2) {
          if constexpr (KS >= 4) { rotate_pair(0, 2); rotate_pair(1, 3); }
        } else if (nf == 3) {
          if constexpr (KS >= 6) { rotate_pair(0, 3); rotate_pair(1, 4); rotate_pair(2, 5); }
        } else {
          if constexpr (KS >= 8) { rotate_pair(0, 4); rotate_pair(1, 5); rotate_pair(2, 6); rotate_pair(3, 7); }
        }
      }
    }
#pragma unroll
    for (int kk = 0; kk < KS; ++kk)
      qf[kk] = make_uint4(pack2<F16>(x[kk][0], x[kk][1]), pack2<F16>(x[kk][2], x[kk][3]),
                          pack2<F16>(x[kk][4], x[kk][5]), pack2<F16>(x[kk][6], x[kk][7]));
  };

  float m_run = -INFINITY, l_run = 0.f;
  f32x4_t acc[DV];
#pragma unroll
  for (int e = 0; e < DV; ++e) acc[e] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  // Register staging of one tile (NT sub-tiles of 16 tokens).  The loop below is software
  // pipelined with these registers alone: K of the next tile is requested as soon as the
  // scores of the current one exist, V of the next tile as soon as the current P.V is done,
  // so every wave keeps loads in flight while it computes.
  uint4 kf[NT][FP8 ? KS / 2 : KS];
  uint32_t vf[NT][4][VD];  // 16-bit cache: HDV / 8 bytes per token and lane; fp8: HDV / 16 bytes
  float ksc_tile = 1.f, vsc_tile = 1.f;  // fp8: scales of the chunk the staged K / V tile lies in

  // Addressing.  A tile of 16*NT tokens never straddles a chunk (the launcher picks NT so that the
  // tile size divides the chunk size), so its address is
  //   cache + table entry * chunk_bytes + (token inside the chunk) * tok_bytes        -- all scalar --
  // plus a per-lane byte offset that is fixed for the whole kernel:
  //   K: lane (m16, g) reads 16 B at column 16g (+64 per step) of row m16 of a sub-tile;
  //   V: lane (m16, g) reads its DV values of rows 4g .. 4g+3.
  // Tokens past the end are clamped to the last valid one (row offset min(row, rows left)): the
  // data stays finite and their probabilities are forced to zero below.  That also makes a request
  // for a tile beyond `end` harmless (it re-reads the last token's rows).
  const uint32_t k_col = 16u * (uint32_t)g, v_col = (uint32_t)(DV * m16 * ESZ);
  const uint32_t k_lane = (uint32_t)m16 * tok_bytes + k_col;
  uint32_t v_lane[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) v_lane[j] = (uint32_t)(4 * g + j) * tok_bytes + v_col;

  // Block-table cursor: the entries of the current chunk and of the next one as scalars, the one
  // after that still in flight; with fp8 the scale of the next chunk is in flight too.  An entry is
  // requested two chunks (its scale one chunk) before its first use, so after the start of a
  // segment the stream never waits for the table.  One cursor each for K and V (V runs half an
  // iteration behind K).
  const int32_t* bt_row = p.bt + (int64_t)r * p.bt_stride;
  const int ci_last = chunk_of(last, p.chunk_magic);
  struct Cursor {
    int ci;            // chunk the scalars describe
    int pc, pc_next;   // its table entry and the next chunk's
    int pc_after;      // per-lane copy of the entry two chunks ahead (load may be in flight)
    float sc;          // fp8: scale of (pc, h)
    float sc_next;     // per-lane copy of the next chunk's scale (load may be in flight)
  };
  auto entry_load = [&](int ci) { return bt_row[min(ci, ci_last)]; };
  auto scale_load = [&](const float* scales, int pc) { return scales[(int64_t)pc * p.Hkv + h]; };
  auto uniform_f = [](float x) { return __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(x))); };
  // the clamped tile start only ever moves forward, by at most one chunk per tile
  auto cursor_follow = [&](Cursor& c, const float* scales, int ci) {
    if (ci != c.ci) {
      c.ci = ci;
      c.pc = c.pc_next;
      c.pc_next = __builtin_amdgcn_readfirstlane(c.pc_after);
      c.pc_after = entry_load(ci + 2);
      if (FP8) {
        c.sc = uniform_f(c.sc_next);
        c.sc_next = scale_load(scales, c.pc_next);
      }
    }
  };
  // Opening: one round trip for the three table entries, shared by both cursors; the scales are
  // requested next and only waited for after the first tiles' loads have been issued.
  Cursor kcur, vcur;
  float ksc_first = 1.f, vsc_first = 1.f;  // per-lane copies, loads in flight
  {
    const int ci0 = chunk_of(min(start, last), p.chunk_magic);
    const int e0 = entry_load(ci0), e1 = entry_load(ci0 + 1), e2 = entry_load(ci0 + 2);
    kcur.ci = ci0;
    kcur.pc = __builtin_amdgcn_readfirstlane(e0);
    kcur.pc_next = __builtin_amdgcn_readfirstlane(e1);
    kcur.pc_after = e2;
    kcur.sc = kcur.sc_next = 1.f;
    vcur = kcur;
    if (FP8) {
      ksc_first = scale_load(p.k_scale, kcur.pc);
      vsc_first = scale_load(p.v_scale, kcur.pc);
      kcur.sc_next = scale_load(p.k_scale, kcur.pc_next);
      vcur.sc_next = scale_load(p.v_scale, kcur.pc_next);
    }
  }

  // chunk base (scalar) of the tile that starts at T; `row0` = chunk-relative row of token 0 of the chunk
  auto tile_chunk = [&](Cursor& c, const float* scales, const uint8_t* base, int T, int& tok0) {
    const int ci = chunk_of(min(T, last), p.chunk_magic);
    cursor_follow(c, scales, ci);
    tok0 = ci * p.chunk;
    return base + (int64_t)c.pc * chunk_bytes;
  };
  auto load_k = [&](int T) {
    int tok0;
    const uint8_t* chunk = tile_chunk(kcur, p.k_scale, kbase, T, tok0);
    if (FP8) ksc_tile = (FUSED && own_scale && kcur.ci == ci_last) ? own_ksc : kcur.sc;
#pragma unroll
    for (int u = 0; u < NT; ++u) {
      const int t0 = min(T + 16 * u, last);
      const uint32_t lim = (uint32_t)min(last - t0, 15) * tok_bytes;
      const uint8_t* krow = chunk + (uint32_t)(t0 - tok0) * tok_bytes + min(k_lane, lim + k_col);
#pragma unroll
      for (int kk = 0; kk < (FP8 ? KS / 2 : KS); ++kk)
        kf[u][kk] = SHARED_KV ? ld16(krow + 64 * kk) : ld16_stream(krow + 64 * kk);
    }
  };
  auto load_v = [&](int T) {
    int tok0;
    const uint8_t* chunk = tile_chunk(vcur, p.v_scale, vbase, T, tok0);
    if (FP8) vsc_tile = (FUSED && own_scale && vcur.ci == ci_last) ? own_vsc : vcur.sc;
#pragma unroll
    for (int u = 0; u < NT; ++u) {
      const int t0 = min(T + 16 * u, last);
      const uint32_t cap = (uint32_t)min(last - t0, 15) * tok_bytes + v_col;
      const uint8_t* tile = chunk + (uint32_t)(t0 - tok0) * tok_bytes;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint8_t* vrow = tile + min(v_lane[j], cap);
        if constexpr (SHARED_KV) ld_dwords(vrow, vf[u][j]);
        else ld_dwords_stream(vrow, vf[u][j]);
      }
    }
  };

  if constexpr (FUSED) {
    // The segment that ends the request appends before it loads (its tiles hold the new token); every other
    // segment gets its first loads under way and prepares its queries while they are in flight.
    // (The value loads wait until the queries are done: with both tiles in flight the prologue would not fit the
    // registers of three wavefronts per SIMD.)
    if (final_seg) {
      fused_cos_sin();
      fused_append();
      load_k(start);
    } else {
      load_k(start);
      fused_cos_sin();
    }
    fused_queries();
    __builtin_amdgcn_sched_barrier(0);
    load_v(start);
  } else {
    load_k(start);
    load_v(start);
  }
  __builtin_amdgcn_sched_barrier(0);
  if (FP8) {  // the first tile lies in the opening chunk
    kcur.sc = ksc_tile = uniform_f(ksc_first);
    vcur.sc = vsc_tile = uniform_f(vsc_first);
    if (FUSED && own_scale && kcur.ci == ci_last) {  // ... which the step's token has just opened
      ksc_tile = own_ksc;
      vsc_tile = own_vsc;
    }
  }
  const uint2 ones = make_uint2(ones2<F16>(), ones2<F16>());  // four times 1.0
  for (int T = start; T < end; T += 16 * NT) {
    // ---- S^T = K Q^T ---------------------------------------------------------
    // The tile lies in one chunk, so one K scale and one V scale hold for all of it; the score
    // multiplier is positive and wave-uniform, so the maximum is taken over the raw products.
    const float mul = FP8 ? p.scale_log2 * ksc_tile : p.scale_log2;
    const bool ragged = T + 16 * NT > end;  // only the last tile of a segment has masked tokens
    float sc[NT][4];
    float tmax = -INFINITY;
#pragma unroll
    for (int u = 0; u < NT; ++u) {
      f32x4_t sacc = {0.f, 0.f, 0.f, 0.f};
      if (FP8) {
#pragma unroll
        for (int kk = 0; kk < KS / 2; ++kk) {
          const uint2 a0 = fp8x4_to_16x4<F16>(kf[u][kk].x), a1 = fp8x4_to_16x4<F16>(kf[u][kk].y);
          const uint2 b0 = fp8x4_to_16x4<F16>(kf[u][kk].z), b1 = fp8x4_to_16x4<F16>(kf[u][kk].w);
          sacc = mfma_16x16x32<F16>(make_uint4(a0.x, a0.y, a1.x, a1.y), qf[2 * kk], sacc);
          sacc = mfma_16x16x32<F16>(make_uint4(b0.x, b0.y, b1.x, b1.y), qf[2 * kk + 1], sacc);
        }
      } else {
#pragma unroll
        for (int kk = 0; kk < KS; ++kk)
          sacc = mfma_16x16x32<F16>(kf[u][kk], Q_IN_LDS ? lds_ld16(q_frag + 64 * kk) : qf[Q_IN_LDS ? 0 : kk], sacc);
      }
      if (ragged) {
        const int tok0 = T + 16 * u + 4 * g;
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (tok0 + i >= end) sacc[i] = -INFINITY;
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) sc[u][i] = sacc[i];
      tmax = fmaxf(fmaxf(tmax, sacc[0]), fmaxf(sacc[1], fmaxf(sacc[2], sacc[3])));
    }
    const float vscale = FP8 ? vsc_tile : 1.f;
    // The scheduling fences keep each batch of prefetch loads together at this point of the
    // loop instead of letting the compiler sink them next to their uses one by one.
    __builtin_amdgcn_sched_barrier(0);
    load_k(T + 16 * NT);  // prefetch: the K registers are free again
    __builtin_amdgcn_sched_barrier(0);
    tmax = fmaxf(tmax, xor16(tmax));
    tmax = fmaxf(tmax, xor32(tmax));

    // ---- online softmax (row = m16, all lane-local after the max) -----------
    // p = 2^(s * mul - m) [* V scale, folded into the exponent]; the row sums come from the
    // matrix cores (an all-ones A operand), complete over the 16 tokens of a sub-tile.
    const float m_new = fmaxf(m_run, tmax * mul);
    const float alpha = fast_exp2(m_run - m_new);
    m_run = m_new;
    const float neg = FP8 ? fast_log2(vscale) - m_new : -m_new;
    uint2 pf[NT];
    f32x4_t psum4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int u = 0; u < NT; ++u) {
      const float p0 = fast_exp2(__builtin_fmaf(sc[u][0], mul, neg));
      const float p1 = fast_exp2(__builtin_fmaf(sc[u][1], mul, neg));
      const float p2 = fast_exp2(__builtin_fmaf(sc[u][2], mul, neg));
      const float p3 = fast_exp2(__builtin_fmaf(sc[u][3], mul, neg));
      pf[u] = make_uint2(pack2<F16>(p0, p1), pack2<F16>(p2, p3));
      psum4 = mfma_16x16x16<F16>(ones, pf[u], psum4);
    }
    // (every slot of psum4 holds the row sum of this lane's query row)
    l_run = l_run * alpha + (FP8 ? psum4[0] * __builtin_amdgcn_rcpf(vscale) : psum4[0]);
    if (__builtin_amdgcn_ballot_w64(alpha != 1.f)) {  // the running maximum rarely moves after the first tiles
#pragma unroll
      for (int e = 0; e < DV; ++e) {
        acc[e][0] *= alpha; acc[e][1] *= alpha; acc[e][2] *= alpha; acc[e][3] *= alpha;
      }
    }

    // ---- O^T += V^T P^T --------------------------------------------------------
#pragma unroll
    for (int u = 0; u < NT; ++u) {
      if constexpr (!FP8) {  // 16-bit cache: dword dw of a token holds this lane's values 2 dw, 2 dw + 1
#pragma unroll
        for (int dw = 0; dw < VD; ++dw) {
          const uint32_t r0 = vf[u][0][dw], r1 = vf[u][1][dw], r2 = vf[u][2][dw], r3 = vf[u][3][dw];
          acc[2 * dw] = mfma_16x16x16<F16>(make_uint2(low_halves(r1, r0), low_halves(r3, r2)), pf[u], acc[2 * dw]);
          acc[2 * dw + 1] =
              mfma_16x16x16<F16>(make_uint2(high_halves(r1, r0), high_halves(r3, r2)), pf[u], acc[2 * dw + 1]);
        }
      } else {  // fp8: four bytes (width 64) or eight (width 128) per token and lane
        uint2 w[4][VD];  // [token j][dword] -> two packed bf16 pairs (4 d values)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int hf = 0; hf < VD; ++hf) w[j][hf] = fp8x4_to_16x4<F16>(vf[u][j][hf]);
#pragma unroll
        for (int hf = 0; hf < VD; ++hf) {
          acc[4 * hf + 0] = mfma_16x16x16<F16>(
              make_uint2(low_halves(w[1][hf].x, w[0][hf].x), low_halves(w[3][hf].x, w[2][hf].x)), pf[u], acc[4 * hf + 0]);
          acc[4 * hf + 1] = mfma_16x16x16<F16>(
              make_uint2(high_halves(w[1][hf].x, w[0][hf].x), high_halves(w[3][hf].x, w[2][hf].x)), pf[u], acc[4 * hf + 1]);
          acc[4 * hf + 2] = mfma_16x16x16<F16>(
              make_uint2(low_halves(w[1][hf].y, w[0][hf].y), low_halves(w[3][hf].y, w[2][hf].y)), pf[u], acc[4 * hf + 2]);
          acc[4 * hf + 3] = mfma_16x16x16<F16>(
              make_uint2(high_halves(w[1][hf].y, w[0][hf].y), high_halves(w[3][hf].y, w[2][hf].y)), pf[u], acc[4 * hf + 3]);
        }
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    load_v(T + 16 * NT);  // prefetch: the V registers are free again
    __builtin_amdgcn_sched_barrier(0);
  }

  // ---- epilogue ---------------------------------------------------------------
  const float l_tot = l_run;  // already summed over the lanes of a row (matrix-core row sums)
  const float inv = 1.f / l_tot;
  if (m16 >= G) return;  // (no barrier follows inside a segment)
  // acc[e][i] holds d = DV*(4g+i) + e: DV*4 contiguous values per lane.
  if (whole) {
    uint16_t* o = p.out + (int64_t)row * p.o_st + (int64_t)hq * p.o_sh + 4 * DV * g;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      uint32_t ow[DV / 2];
#pragma unroll
      for (int dw = 0; dw < DV / 2; ++dw) ow[dw] = pack2<F16>(acc[2 * dw][i] * inv, acc[2 * dw + 1][i] * inv);
      st_dwords(o + DV * i, ow);
    }
  } else {
    const int64_t row = (int64_t)slot * p.Hq + hq;
    float* o = p.part_o + row * HDV + 4 * DV * g;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if constexpr (DV % 4 == 0) {
#pragma unroll
        for (int e = 0; e < DV; e += 4) {
          float4 v = make_float4(acc[e][i] * inv, acc[e + 1][i] * inv, acc[e + 2][i] * inv, acc[e + 3][i] * inv);
          *reinterpret_cast<float4*>(o + DV * i + e) = v;
        }
      } else {
#pragma unroll
        for (int e = 0; e < DV; e += 2)
          *reinterpret_cast<float2*>(o + DV * i + e) = make_float2(acc[e][i] * inv, acc[e + 1][i] * inv);
      }
    }
    if (g == 0) p.part_lse[row] = m_run + fast_log2(l_tot);
  }
}

// Tiles (of TK tokens) of one request.
static __device__ __forceinline__ int tiles_of(int len, int tk) { return len > 0 ? (len + tk - 1) / tk : 0; }

// Does request r take part in this launch, and which q/out row is its?
static __device__ __forceinline__ bool decode_row(const DecodeParams& p, int r, int& row) {
  if (!p.cu_q) {
    row = r;
    return true;
  }
  row = p.cu_q[r];
  return p.cu_q[r + 1] - row == 1;
}

// Span of this workgroup along the flattened sequence of TK-token tiles, then its segments one after
// the other: seg(r, row, len, first token, one past the last token, whole request?, ends the request?, partial slot).
// Every wavefront of the workgroup walks the same segments.  Dynamic LDS starts with the inclusive
// prefix sums of tiles per request [R] and the request lengths [R].
template <int TK, typename Seg>
static __device__ __forceinline__ void walk_segments(const DecodeParams& p, Seg seg) {
  extern __shared__ int cum[];
  int* const len_s = cum + p.R;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;

  // ---- prefix sum of tiles over the batch (wave 0), shared through LDS -------------
  if (wave == 0) {
    int carry = 0;
    for (int base = 0; base < p.R; base += 64) {
      const int i = base + lane;
      int row_unused;
      const int len_i = i < p.R ? p.lens[i] : 0;
      int v = (i < p.R && decode_row(p, i, row_unused)) ? tiles_of(len_i, TK) : 0;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const int up = __shfl_up(v, o, 64);
        if (lane >= o) v += up;
      }
      if (i < p.R) {
        cum[i] = carry + v;
        len_s[i] = len_i;  // a segment start then costs no trip to memory for the length
      }
      carry += __shfl(v, 63, 64);
    }
  }
  __syncthreads();
  const int total = cum[p.R - 1];
  // equal spans; the remainder goes one tile each to the first workgroups (rounding the span
  // up instead would leave the last workgroups without work)
  int t0, t1;
  if (total >= p.grid * p.min_span_tiles) {
    const int per = total / p.grid, rem = total - per * p.grid;
    t0 = (int)blockIdx.x * per + min((int)blockIdx.x, rem);
    t1 = t0 + per + ((int)blockIdx.x < rem ? 1 : 0);
  } else {
    t0 = blockIdx.x * p.min_span_tiles;
    t1 = min(t0 + p.min_span_tiles, total);
  }
  if (t0 >= t1) return;

  // first request whose tiles extend beyond t0
  int lo = 0, hi = p.R - 1;
  while (lo < hi) {
    const int mid = (lo + hi) >> 1;
    if (cum[mid] > t0) hi = mid; else lo = mid + 1;
  }
  int r = lo;
  while (t0 < t1) {
    const int rb = r ? cum[r - 1] : 0;
    const int re = cum[r];
    if (re > t0) {  // requests without tiles (length 0) are skipped
      const int len = len_s[r];
      const int tb = t0 - rb;             // first tile of the segment, within the request
      const int te = min(t1, re) - rb;    // one past its last tile
      const bool first = tb == 0, final = te == re - rb;
      if (wave == 0 && lane == 0) {
        if (first) p.seg_info[2 * r] = blockIdx.x;
        if (final) p.seg_info[2 * r + 1] = blockIdx.x;
      }
      int row;
      decode_row(p, r, row);
      seg(r, row, len, tb * TK, min(te * TK, len), first && final, final, (int)blockIdx.x + r);
      t0 = rb + te;
    }
    ++r;
  }
}

// The body of the register-streaming kernels: one wavefront per (virtual) KV head.
template <int HDK, int HDV, int NT, bool FP8, bool F16, bool FUSED = false>
static __device__ __forceinline__ void decode_stream_body(const DecodeParams& p) {
  extern __shared__ int cum[];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  // wavefront index along the heads: `parts` consecutive ones share a KV head and split its query heads by 16
  const int hv = __builtin_amdgcn_readfirstlane(blockIdx.y * (blockDim.x >> 6) + wave);
  const int h = p.parts > 1 ? hv / p.parts : hv;
  const int part = hv - h * p.parts;
  const int hq0 = h * p.G + 16 * part;
  const int gq = min(16, p.G - 16 * part);
  // behind the two integer arrays, per wavefront: 16 query rows (wide keys) or the fused step's cos / sin / key
  // row (see decode_segment)
  uint8_t* const q_lds = reinterpret_cast<uint8_t*>(cum) + (((size_t)p.R * 8 + 15) & ~(size_t)15) +
                         (size_t)wave * (FUSED ? 3 * HDK * sizeof(float) : 16 * (HDK * 2 + 16));
  walk_segments<16 * NT>(p, [&](int r, int row, int len, int start, int end, bool whole, bool final_seg, int slot) {
    decode_segment<HDK, HDV, NT, FP8, F16, FUSED>(p, r, row, h, hq0, gq, len, start, end, whole, final_seg, slot, lane,
                                                  q_lds);
  });
}

template <int HD, int NT, bool FP8, int MINW, bool F16>
__global__ __launch_bounds__(512, MINW) void paged_decode_stream_kernel(DecodeParams p) {
  decode_stream_body<HD, HD, NT, FP8, F16>(p);
}

// The same stream over the raw queries, keys and values of a decode step: head norm, rotary embedding and the
// append of the new token ride in the segment prologues (see decode_segment).
template <int HD, int NT, bool F16, int MINW = 3, bool FP8 = false>
__global__ __launch_bounds__(512, MINW) void decode_step_stream_kernel(DecodeParams p) {
  decode_stream_body<HD, HD, NT, FP8, F16, true>(p);
}

// Multi-latent attention, absorbed form: every query head attends to the same 576-wide latent rows
// (scores over all 576 values, output = weighted sum of the first 512).  A wavefront takes 16 query
// heads; with 128 accumulator registers per lane a SIMD holds one wavefront, hence at most four per
// workgroup.
template <bool F16>
__global__ __launch_bounds__(256, 1) void paged_mla_decode_stream_kernel(DecodeParams p) {
  decode_stream_body<576, 512, 1, false, F16>(p);
}

// ---------------------------------------------------------------------------------------------
// Multi-latent attention decode with the latent tile shared through LDS.
//
// A workgroup of 8 wavefronts streams 64-token tiles of the latent rows (64 x 576 bf16 = 72 KB) into
// LDS, double buffered, each row fetched from memory once per workgroup.  Wavefront w works for
// query-head group w / PARTS (16 heads).  Scores: the PARTS wavefronts of a group share the work --
// each takes one of the four 16-token sub-tiles (and, with PARTS = 8, one half of the 576 key
// values), writes its raw partial scores to LDS, and after a barrier every wavefront reads the whole
// 16 x 64 score tile back and runs the (cheap) softmax for itself.  Values: wavefront w owns output
// columns part w % PARTS of the 512 and reads their fragments with transposing LDS reads.
// PARTS = 8 serves one head group per workgroup (up to 16 heads per rank), PARTS = 4 two groups.
// Two barriers per tile; the global loads of tile t+1 are in flight in registers while tile t computes.
// ---------------------------------------------------------------------------------------------
constexpr int kMlaTile = 64;                 // tokens per staged tile
// LDS bytes per staged row.  (By counter a 16-byte fragment read takes 4 conflict cycles on top of its 4 and a
// transposing 8-byte read 2 on top of its 2 at this pitch -- 292 dwords = 36 mod 64; 1 184 bytes, as in the kernel
// for 128 heads below, has none, but two 64-token buffers of it leave room for 512 requests' prefix sums instead
// of 768, and this kernel is no faster for it.)
constexpr int kMlaPitch = 576 * 2 + 16;

template <int PARTS, bool F16>
__global__ __launch_bounds__(512, 2) void paged_mla_decode_lds_kernel(DecodeParams p) {
  constexpr int HDK = 576, HDV = 512, KS = HDK / 32;
  constexpr int NG = 8 / PARTS;               // head groups per workgroup
  constexpr int DVW = HDV / PARTS / 16;       // 16-column output blocks per wavefront
  constexpr int KH = PARTS / 4;               // wavefronts that share the key values of one sub-tile
  constexpr int KSW = KS / KH;                // 32-value steps of the score product per wavefront
  extern __shared__ int cum[];
  uint8_t* const tiles = reinterpret_cast<uint8_t*>(cum) + (((size_t)p.R * 8 + 15) & ~(size_t)15);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int m16 = lane & 15, g = lane >> 4;
  const int group = blockIdx.y * NG + wave / PARTS;   // 16-head query group of this wavefront
  const int c0 = (wave % PARTS) * (HDV / PARTS);      // its first output column
  const int su = wave & 3;                            // sub-tile whose scores it computes
  const int k0 = ((wave % PARTS) >> 2) * KSW;         // first 32-value step of its share of the keys
  // partial scores of this wavefront's group: [key part][sub-tile][lane] float4, behind the two tile buffers
  float4* const sbuf = reinterpret_cast<float4*>(tiles + 2 * kMlaTile * kMlaPitch) + (wave / PARTS) * (KH * 4 * 64);
  const int G = p.G;
  const int hq = group * G + m16;                     // query head of this lane's row (valid when m16 < G)
  const int64_t chunk_bytes = p.kv_sc * 2;
  const uint32_t tok_bytes = (uint32_t)(p.kv_st * 2);
  // loader role: row tid / 8 of a tile, 16-byte pieces (tid % 8) + 8 i, i < 9, of that row
  const int lrow = tid >> 3, lpiece = tid & 7;
  const uint32_t l_src = (uint32_t)lrow * tok_bytes + 16u * lpiece;
  uint8_t* const l_dst = tiles + lrow * kMlaPitch + 16 * lpiece;
  // fragment reads: keys as the A operand of the scores, values transposed as the A operand of P.V
  const int kfrag_off = m16 * kMlaPitch + 16 * g;
  const int vfrag_off = (4 * g + (m16 >> 2)) * kMlaPitch + 2 * c0 + 8 * (m16 & 3);
  const uint4 ones = make_uint4(ones2<F16>(), ones2<F16>(), ones2<F16>(), ones2<F16>());

  walk_segments<kMlaTile>(p, [&](int r, int row, int len, int start, int end, bool whole, bool /*final_seg*/, int slot) {
    r = __builtin_amdgcn_readfirstlane(r);
    row = __builtin_amdgcn_readfirstlane(row);
    len = __builtin_amdgcn_readfirstlane(len);
    start = __builtin_amdgcn_readfirstlane(start);
    end = __builtin_amdgcn_readfirstlane(end);
    slot = __builtin_amdgcn_readfirstlane(slot);
    const int last = min(end, len) - 1;
    const int ntile = (end - start + kMlaTile - 1) / kMlaTile;
    const int32_t* bt_row = p.bt + (int64_t)r * p.bt_stride;

    uint4 qf[KSW];
    {
      const uint16_t* qrow = p.q + (int64_t)row * p.q_st + (int64_t)hq * p.q_sh + 32 * k0;
#pragma unroll
      for (int kk = 0; kk < KSW; ++kk) qf[kk] = (m16 < G) ? ld16(qrow + 32 * kk + 8 * g) : make_uint4(0, 0, 0, 0);
    }
    float m_run = -INFINITY, l_run = 0.f;
    f32x4_t acc[DVW];
#pragma unroll
    for (int e = 0; e < DVW; ++e) acc[e] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    // A tile lies in one chunk (the launcher requires a chunk size that is a multiple of 64); rows past
    // the segment's last token re-read that token's row (their probabilities are forced to zero).
    uint4 stage[9];
    auto fetch = [&](int t) {
      const int T = start + t * kMlaTile;
      const int ci = chunk_of(T, p.chunk_magic);
      const int pc = __builtin_amdgcn_readfirstlane(bt_row[ci]);
      const uint8_t* src = p.kc + (int64_t)pc * chunk_bytes + (int64_t)(uint32_t)(T - ci * p.chunk) * tok_bytes;
      const uint32_t lim = (uint32_t)min(last - T, kMlaTile - 1) * tok_bytes + 16u * lpiece;
      const uint8_t* rowp = src + min(l_src, lim);
#pragma unroll
      for (int i = 0; i < 9; ++i) stage[i] = ld16(rowp + 128 * i);
    };
    auto store = [&](int t) {
      uint8_t* dst = l_dst + (t & 1) * (kMlaTile * kMlaPitch);
#pragma unroll
      for (int i = 0; i < 9; ++i) *reinterpret_cast<uint4*>(dst + 128 * i) = stage[i];
    };

    fetch(0);
    store(0);
    __syncthreads();
    for (int t = 0; t < ntile; ++t) {
      if (t + 1 < ntile) fetch(t + 1);  // workgroup-uniform
      const uint8_t* buf = tiles + (t & 1) * (kMlaTile * kMlaPitch);
      const int T = start + t * kMlaTile;
      // ---- S^T = K Q^T: this wavefront's share, then the whole tile through LDS -----------
      {
        // Key fragments in batches of KB, the reads of batch b+1 issued before the products of batch b (scheduling
        // barriers keep that order): read-wait-multiply one fragment at a time pays the LDS latency KSW times.
        constexpr int KB = KSW % 6 == 0 ? 6 : 3, NB = KSW / KB;
        static_assert(KSW % KB == 0, "18 or 9 fragments");
        const uint8_t* ks = buf + kfrag_off + 16 * su * kMlaPitch + 64 * k0;
        f32x4_t sacc = {0.f, 0.f, 0.f, 0.f};
        uint4 kf[2][KB];
#pragma unroll
        for (int j = 0; j < KB; ++j) kf[0][j] = *reinterpret_cast<const uint4*>(ks + 64 * j);
#pragma unroll
        for (int b = 0; b < NB; ++b) {
          if (b + 1 < NB) {
#pragma unroll
            for (int j = 0; j < KB; ++j) kf[(b + 1) & 1][j] = *reinterpret_cast<const uint4*>(ks + 64 * (KB * (b + 1) + j));
          }
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int j = 0; j < KB; ++j) sacc = mfma_16x16x32<F16>(kf[b & 1][j], qf[KB * b + j], sacc);
          __builtin_amdgcn_sched_barrier(0);
        }
        sbuf[((k0 ? 1 : 0) * 4 + su) * 64 + lane] = make_float4(sacc[0], sacc[1], sacc[2], sacc[3]);
      }
      __syncthreads();
      f32x4_t sc[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        float4 a = sbuf[u * 64 + lane];
        if (KH == 2) {
          const float4 b = sbuf[(4 + u) * 64 + lane];
          a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
        }
        sc[u] = f32x4_t{a.x, a.y, a.z, a.w};
      }
      if (T + kMlaTile > end) {  // only the last tile of a segment has masked tokens
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int tok0 = T + 16 * u + 4 * g;
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (tok0 + i >= end) sc[u][i] = -INFINITY;
        }
      }
      float tmax = -INFINITY;
#pragma unroll
      for (int u = 0; u < 4; ++u) tmax = fmaxf(fmaxf(tmax, sc[u][0]), fmaxf(sc[u][1], fmaxf(sc[u][2], sc[u][3])));
      tmax = rowgroup_max(tmax);
      // ---- online softmax (row = m16) ----------------------------------------------------
      const float mul = p.scale_log2;
      const float m_new = fmaxf(m_run, tmax * mul);
      const float alpha = fast_exp2(m_run - m_new);
      m_run = m_new;
      uint2 pf[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const float p0 = fast_exp2(__builtin_fmaf(sc[u][0], mul, -m_new));
        const float p1 = fast_exp2(__builtin_fmaf(sc[u][1], mul, -m_new));
        const float p2 = fast_exp2(__builtin_fmaf(sc[u][2], mul, -m_new));
        const float p3 = fast_exp2(__builtin_fmaf(sc[u][3], mul, -m_new));
        pf[u] = make_uint2(pack2<F16>(p0, p1), pack2<F16>(p2, p3));
      }
      if (__builtin_amdgcn_ballot_w64(alpha != 1.f)) {
#pragma unroll
        for (int e = 0; e < DVW; ++e) {
          acc[e][0] *= alpha; acc[e][1] *= alpha; acc[e][2] *= alpha; acc[e][3] *= alpha;
        }
      }
      // ---- O^T += V^T P^T, 32 tokens per product; row sums from an all-ones A operand -----
      f32x4_t psum4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        const uint4 pp = make_uint4(pf[2 * s2].x, pf[2 * s2].y, pf[2 * s2 + 1].x, pf[2 * s2 + 1].y);
        const uint8_t* vs = buf + vfrag_off + 32 * s2 * kMlaPitch;
#pragma unroll
        for (int e = 0; e < DVW; ++e) {
          const uint2 a0 = lds_ld8_tr(vs + 32 * e), a1 = lds_ld8_tr(vs + 16 * kMlaPitch + 32 * e);
          acc[e] = mfma_16x16x32<F16>(make_uint4(a0.x, a0.y, a1.x, a1.y), pp, acc[e]);
        }
        psum4 = mfma_16x16x32<F16>(ones, pp, psum4);
      }
      l_run = l_run * alpha + psum4[0];
      if (t + 1 < ntile) store(t + 1);
      __syncthreads();
    }

    // ---- epilogue: acc[e][i] is output column c0 + 16 e + 4 g + i of row m16 ------------------
    const float inv = 1.f / l_run;
    if (m16 < G) {
      if (whole) {
        uint16_t* o = p.out + (int64_t)row * p.o_st + (int64_t)hq * p.o_sh + c0 + 4 * g;
#pragma unroll
        for (int e = 0; e < DVW; ++e)
          st8(o + 16 * e, make_uint2(pack2<F16>(acc[e][0] * inv, acc[e][1] * inv),
                                     pack2<F16>(acc[e][2] * inv, acc[e][3] * inv)));
      } else {
        const int64_t prow = (int64_t)slot * p.Hq + hq;
        float* o = p.part_o + prow * HDV + c0 + 4 * g;
#pragma unroll
        for (int e = 0; e < DVW; ++e)
          *reinterpret_cast<float4*>(o + 16 * e) =
              make_float4(acc[e][0] * inv, acc[e][1] * inv, acc[e][2] * inv, acc[e][3] * inv);
        if (g == 0 && c0 == 0) p.part_lse[prow] = m_run + fast_log2(l_run);
      }
    }
  });
}

// ---------------------------------------------------------------------------------------------
// Multi-latent attention decode, 128 query heads per workgroup.
//
// With 128 heads the latent rows carry 242 flop per byte: the matrix cores, not memory, are the bound,
// and what feeds them is LDS.  A wavefront takes in no more than ~18 B/clk of fragments whatever runs
// beside it, so what counts is how many products each fragment read serves.  Here a workgroup is four
// wavefronts, one per SIMD with the SIMD's whole register file (512 registers per lane); wavefront w
// owns query heads 32 w .. 32 w + 31 (two 16-row tiles: every key fragment and every transposed value
// fragment feeds two products) and all 512 output columns (256 accumulator registers), and shares
// nothing with the others but the staged rows: no score exchange, one barrier per tile.
// 32-token tiles (37 KB) in four LDS buffers, filled by direct loads from memory (no staging registers, no LDS
// stores): iteration t multiplies the scores of tile t, waits until its own loads of tile t+1 have landed, passes
// the barrier, then softmax and the value product of tile t -- under whose products it issues, one by one, the
// loads of tile t+3, and at whose end it requests the first key fragments of tile t+1.  (Four buffers: tile t+3
// replaces tile t-1, which every wavefront left before the barrier of iteration t; tiles t+1 and t+2 are in LDS
// or on their way.)  The accumulators are never rescaled in that loop (see there).
// ---------------------------------------------------------------------------------------------
constexpr int kMlaHeadsTile = 32;  // tokens per staged tile of the 128-head kernel
// LDS bytes per staged row: 296 dwords = 40 mod 64, an odd multiple of 8 banks.  A 16-byte fragment read is served in
// passes of {rows 0-7 at piece g, rows 8-15 at piece g + 1} and a transposing 8-byte read in passes of eight rows: both
// then cover the 64 banks exactly once (no conflict cycle by counter; at 1 168 bytes: 4 and 2 per read).
constexpr int kMlaHeadsPitch = 576 * 2 + 32;
// A tile arrives in LDS by direct loads: each instruction puts its 64 lanes' 16-byte pieces side by side (1 KB), so a
// tile is 37 instructions over a line of 32 x 74 pieces (72 of a row + the 32 bytes of row padding, which receive
// copies of the row's last piece), and a buffer is 37 KB -- exactly.
constexpr int kMlaHeadsLoads = (kMlaHeadsTile * (kMlaHeadsPitch / 16) + 63) / 64;
constexpr int kMlaHeadsBuf = kMlaHeadsLoads * 1024;
constexpr bool mla_piece_division_ok() {
  for (unsigned u = 0; u < 64u * kMlaHeadsLoads; ++u)
    if (((u * 14170u) >> 20) != u / 74u) return false;
  return true;
}
static_assert(kMlaHeadsPitch == 74 * 16 && mla_piece_division_ok(), "piece -> (row, column) by multiplication");

template <bool F16>
__global__ __launch_bounds__(256, 1) void paged_mla_decode_heads_kernel(DecodeParams p) {
  constexpr int HDV = 512, KS = 576 / 32, NE = HDV / 16, TK = kMlaHeadsTile;
  constexpr int KB = 3, NKG = 2 * KS / KB;   // key fragments per group; groups per tile (two 16-token sub-tiles)
  constexpr int VB = 2, NVG = NE / VB;       // 16-column output blocks per group; groups per tile
  // log2 of the factor a row's maximum may grow before the reference of its exponentials follows: probabilities
  // up to that factor must fit the 16-bit type (fp16: 65 504)
  constexpr float kLazy = F16 ? 8.f : 30.f;
  extern __shared__ int cum[];
  uint8_t* const tiles = reinterpret_cast<uint8_t*>(cum) + (((size_t)p.R * 8 + 15) & ~(size_t)15);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int m16 = lane & 15, g = lane >> 4;
  const int hq0 = (blockIdx.y * 4 + wave) * 32 + m16;  // this lane's query head in the first row tile (+16: second)
  const int64_t chunk_bytes = p.kv_sc * 2;
  const uint32_t tok_bytes = (uint32_t)(p.kv_st * 2);
  // the LDS byte address of the tile buffers, for the direct loads
  const uint32_t tiles_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)tiles;
  // The lane number, computed where it is asked for (volatile: neither hoisted nor shared between its uses).
  auto lane_now = []() {
    uint32_t ln;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=&v"(ln));
    return ln;
  };
  // Where a lane's key fragments (the A operand of the scores) and transposed value fragments start within a tile.
  // Worked out afresh for every tile from an opaque copy of the lane number: kept in a register across the kernel,
  // such a value ends up in scratch memory, and its reload in the tile loop waits on the vector-memory counter --
  // for every direct load in flight.
  auto frag_offsets = [&](int& kfrag_off, int& vfrag_off) {
    const uint32_t ln = lane_now();
    const int m = ln & 15, gq = ln >> 4;
    kfrag_off = m * kMlaHeadsPitch + 16 * gq;
    vfrag_off = (4 * gq + (m >> 2)) * kMlaHeadsPitch + 8 * (m & 3);
  };
  const uint4 ones = make_uint4(ones2<F16>(), ones2<F16>(), ones2<F16>(), ones2<F16>());
#define MI_SB() __builtin_amdgcn_sched_barrier(0)

  walk_segments<TK>(p, [&](int r, int row, int len, int start, int end, bool whole, bool /*final_seg*/, int slot) {
    r = __builtin_amdgcn_readfirstlane(r);
    row = __builtin_amdgcn_readfirstlane(row);
    len = __builtin_amdgcn_readfirstlane(len);
    start = __builtin_amdgcn_readfirstlane(start);
    end = __builtin_amdgcn_readfirstlane(end);
    slot = __builtin_amdgcn_readfirstlane(slot);
    const int last = min(end, len) - 1;
    const int ntile = (end - start + TK - 1) / TK;
    const int32_t* bt_row = p.bt + (int64_t)r * p.bt_stride;

    auto load_q = [&](uint4 (&qf)[2][KS]) {
#pragma unroll
      for (int h2 = 0; h2 < 2; ++h2) {
        const uint16_t* qrow = p.q + (int64_t)row * p.q_st + (int64_t)(hq0 + 16 * h2) * p.q_sh + 8 * g;
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) qf[h2][kk] = ld16(qrow + 32 * kk);
      }
    };
    uint4 qf[2][KS];
    load_q(qf);
    // A tile lies in one chunk (the launcher requires a chunk size that is a multiple of 32); rows past
    // the segment's last token re-read that token's row (their probabilities are forced to zero).
    // Tile t goes straight from memory into buffer t % 4: wavefront w issues loads w, w + 4, ... of the tile's 37;
    // lane l of load k fills piece 64 k + l of the buffer's line.  The loads count on the vector-memory counter.
    auto tile_buf = [&](int t) { return ((unsigned)t & 3u) * (unsigned)kMlaHeadsBuf; };
    // The block-table entry of tile t's chunk, by a scalar load the compiler does not see: a vector load in the tile
    // loop would make it wait on the vector-memory counter, i.e. for every direct load in flight.  request / arrived
    // are the two halves (the value may only be used after `arrived`); tiles past the segment ask for its last chunk.
    const int ci_last = chunk_of(last, p.chunk_magic);
    auto bt_request = [&](int t) {
      const int byte_off = 4 * min(chunk_of(start + t * TK, p.chunk_magic), ci_last);
      int pc;
      asm volatile("s_load_dword %0, %1, %2" : "=s"(pc) : "s"(bt_row), "s"(byte_off) : "memory");
      return pc;
    };
    auto bt_arrived = [&](int& pc) { asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(pc)::"memory"); };
    auto tile_src = [&](int t, int pc) {
      const int T = start + t * TK;
      const int ci = chunk_of(T, p.chunk_magic);
      return p.kc + (int64_t)pc * chunk_bytes + (int64_t)(uint32_t)(T - ci * p.chunk) * tok_bytes;
    };
    auto whole_tile = [&](int t) { return last - (start + t * TK) >= TK - 1; };
    // direct load i (of this wavefront's nine or ten) of a whole tile: scalar base + the lane's fixed offset
    auto fetch_piece = [&](int t, const uint8_t* src, int i, uint32_t piece_off_i) {
      const int k = wave + 4 * i;
      if (k < kMlaHeadsLoads) {  // wave-uniform
        const uint32_t m0 = __builtin_amdgcn_readfirstlane(tiles_lds + tile_buf(t) + 1024u * (uint32_t)k);
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(m0), "v"(piece_off_i), "s"(src) : "memory", "m0");
      }
    };
    // any tile, all of this wavefront's loads at once: rows past the segment's last token re-read that token's row
    auto fetch = [&](int t, int pc) {
      const uint8_t* src = tile_src(t, pc);
      const uint32_t row_lim = (uint32_t)min(last - (start + t * TK), TK - 1);
      const uint32_t dst = tiles_lds + tile_buf(t);
      const uint32_t ln = lane_now();
#pragma unroll
      for (int i = 0; i < (kMlaHeadsLoads + 3) / 4; ++i) {
        const int k = wave + 4 * i;
        if (k < kMlaHeadsLoads) {  // wave-uniform
          const uint32_t u = 64u * (uint32_t)k + ln;
          const uint32_t prow = (u * 14170u) >> 20, pcol = u - 74u * prow;
          const uint8_t* g_src = src + min(prow, row_lim) * tok_bytes + 16u * min(pcol, 71u);
          const uint32_t m0 = __builtin_amdgcn_readfirstlane(dst + 1024u * (uint32_t)k);
          asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(m0), "v"(g_src) : "memory", "m0");
          MI_SB();  // one address at a time: the registers are needed elsewhere
        }
      }
    };
    // tile t+1 has landed for this wavefront: nothing in flight but its loads of tile t+2 (ten for wavefront 0, nine
    // for the others), which were issued after those of tile t+1 and complete after them (those of tile t+3 are
    // issued after this wait)
    auto fetch_wait = [&](int t) {
      if (t + 2 >= ntile) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      else if (wave == 0) asm volatile("s_waitcnt vmcnt(10)" ::: "memory");
      else asm volatile("s_waitcnt vmcnt(9)" ::: "memory");
    };
    static_assert(kMlaHeadsLoads == 37, "wavefront 0 issues ten loads per tile, the others nine");
    // key group i of a tile: fragments KB (i % (KS / KB)) .. + KB - 1 of 16-token sub-tile i / (KS / KB)
    auto load_k = [&](const uint8_t* buf, int kfrag_off, int i, uint4 (&kf)[KB]) {
      const uint8_t* ks = buf + kfrag_off + 16 * (i / (KS / KB)) * kMlaHeadsPitch + 64 * KB * (i % (KS / KB));
#pragma unroll
      for (int j = 0; j < KB; ++j) kf[j] = *reinterpret_cast<const uint4*>(ks + 64 * j);
    };
    // value group j: output columns 16 VB j .. + 16 VB - 1, all 32 tokens, transposed
    auto load_v = [&](const uint8_t* buf, int vfrag_off, int j, uint2 (&vf)[VB][2]) {
      const uint8_t* vs = buf + vfrag_off + 32 * VB * j;
#pragma unroll
      for (int e = 0; e < VB; ++e) {
        vf[e][0] = lds_ld8_tr(vs + 32 * e);
        vf[e][1] = lds_ld8_tr(vs + 16 * kMlaHeadsPitch + 32 * e);
      }
    };

    // where this lane's piece of direct load k = wave + 4 i of a whole tile comes from, relative to the tile's first
    // row: piece 64 k + lane of the line = (row, 16-byte column) = divmod by 74, the padding columns doubling the last
    // one.  (Worked out per segment, from a lane number of its own so that it stays so: alive across the whole kernel
    // they would live in scratch memory.)
    uint32_t piece_off[(kMlaHeadsLoads + 3) / 4];
    {
      const uint32_t ln = lane_now();
#pragma unroll
      for (int i = 0; i < (kMlaHeadsLoads + 3) / 4; ++i) {
        const uint32_t u = 64u * (uint32_t)(wave + 4 * i) + ln;
        const uint32_t prow = (u * 14170u) >> 20, pcol = u - 74u * prow;
        piece_off[i] = min(prow, (uint32_t)TK - 1) * tok_bytes + 16u * min(pcol, 71u);
      }
    }
    // a tile of the prologue: whole ones by the fixed offsets, the segment's last one the general way
    auto fetch_first = [&](int t, int pc) {
      if (!whole_tile(t)) return fetch(t, pc);
      const uint8_t* src = tile_src(t, pc);
#pragma unroll
      for (int i = 0; i < (kMlaHeadsLoads + 3) / 4; ++i) fetch_piece(t, src, i, piece_off[i]);
    };

    __syncthreads();  // every wavefront is done with the previous segment's buffers
    int pc0 = bt_request(0), pc1 = bt_request(1), pc2 = bt_request(2);
    bt_arrived(pc2);
    bt_arrived(pc1);
    bt_arrived(pc0);
    fetch_first(0, pc0);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0), in the compiler's sight
    // (the query fragments count as used here: the compiler then waits for their loads now and not in the tile loop,
    // where a wait on the vector-memory counter waits for the direct loads in flight as well)
#pragma unroll
    for (int h2 = 0; h2 < 2; ++h2)
#pragma unroll
      for (int kk = 0; kk < KS; ++kk)
        asm volatile("" ::"v"(qf[h2][kk].x), "v"(qf[h2][kk].y), "v"(qf[h2][kk].z), "v"(qf[h2][kk].w));
    if (ntile > 1) fetch_first(1, pc1);
    if (ntile > 2) fetch_first(2, pc2);
    int pc_ahead = bt_request(3);  // of the tile the loops fetch next; each iteration asks for the one after
    __syncthreads();

    // The accumulators live in accumulation registers, out of the vector ALU's reach, and any other definition of
    // theirs than a matrix product or a zero makes the compiler keep all 256 in vector registers (and the query
    // fragments in scratch memory).  So the tile loop never rescales them: exponentials are taken against the row
    // maxima of the first tile, and when a later maximum leaves the window above those (kLazy: hardly ever) the
    // wavefront moves its sums into this segment's rows of the partial-output buffer -- no other workgroup touches
    // those -- and finishes the segment in a second, slow loop that follows every maximum and keeps them there.
    float m_run[2] = {-INFINITY, -INFINITY}, l_run[2] = {0.f, 0.f};
    const float mul = p.scale_log2;
    // scores of tile t (key fragments of its first group already requested into kf[0]); requests the first value
    // fragments; masks the tokens past the segment's end; row maxima in the exponent's unit
    auto scores = [&](int t, const uint8_t* buf, int kfrag_off, int vfrag_off, const uint4 (&qf)[2][KS], uint4 (&kf)[2][KB],
                      uint2 (&vf0)[VB][2], f32x4_t (&sc)[2][2], float (&tmax)[2]) {
#pragma unroll
      for (int i = 0; i < NKG; ++i) {
        if (i + 1 < NKG) load_k(buf, kfrag_off, i + 1, kf[(i + 1) & 1]);
        else load_v(buf, vfrag_off, 0, vf0);
        MI_SB();
        const int u = i / (KS / KB), k0 = KB * (i % (KS / KB));
#pragma unroll
        for (int j = 0; j < KB; ++j) {
#pragma unroll
          for (int h2 = 0; h2 < 2; ++h2)
            sc[h2][u] = mfma_16x16x32<F16>(kf[i & 1][j], qf[h2][k0 + j], (k0 + j) ? sc[h2][u] : f32x4_t{0.f, 0.f, 0.f, 0.f});
        }
        MI_SB();
      }
      const int T = start + t * TK;
#pragma unroll
      for (int h2 = 0; h2 < 2; ++h2) {
        if (T + TK > end) {  // only the last tile of a segment has masked tokens
          const uint32_t ln = lane_now();
#pragma unroll
          for (int u = 0; u < 2; ++u) {
            const int tok0 = T + 16 * u + 4 * (int)(ln >> 4);
#pragma unroll
            for (int i = 0; i < 4; ++i)
              if (tok0 + i >= end) sc[h2][u][i] = -INFINITY;
          }
        }
        const float mx = fmaxf(fmaxf(fmaxf(sc[h2][0][0], sc[h2][0][1]), fmaxf(sc[h2][0][2], sc[h2][0][3])),
                               fmaxf(fmaxf(sc[h2][1][0], sc[h2][1][1]), fmaxf(sc[h2][1][2], sc[h2][1][3])));
        tmax[h2] = rowgroup_max(mx) * mul;
      }
    };
    // probabilities of a tile against m_run, as the B operand of the value product
    auto probabilities = [&](const f32x4_t (&sc)[2][2], uint4 (&pp)[2]) {
#pragma unroll
      for (int h2 = 0; h2 < 2; ++h2) {
        const float neg = -m_run[h2];
        uint32_t w[4];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          const float p0 = fast_exp2(__builtin_fmaf(sc[h2][u][0], mul, neg));
          const float p1 = fast_exp2(__builtin_fmaf(sc[h2][u][1], mul, neg));
          const float p2 = fast_exp2(__builtin_fmaf(sc[h2][u][2], mul, neg));
          const float p3 = fast_exp2(__builtin_fmaf(sc[h2][u][3], mul, neg));
          w[2 * u] = pack2<F16>(p0, p1);
          w[2 * u + 1] = pack2<F16>(p2, p3);
        }
        pp[h2] = make_uint4(w[0], w[1], w[2], w[3]);
        MI_SB();
      }
    };

    int t = 0;
    {
      f32x4_t acc[2][NE];
#pragma unroll
      for (int h2 = 0; h2 < 2; ++h2)
#pragma unroll
        for (int e = 0; e < NE; ++e) acc[h2][e] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      uint4 kf[2][KB];
      uint2 vf[2][VB][2];
      {
        int kfo, vfo;
        frag_offsets(kfo, vfo);
        load_k(tiles + tile_buf(0), kfo, 0, kf[0]);
      }
      for (; t < ntile; ++t) {
        const uint8_t* buf = tiles + tile_buf(t);
        f32x4_t sc[2][2];
        float tmax[2];
        int kfrag_off, vfrag_off;
        frag_offsets(kfrag_off, vfrag_off);
        scores(t, buf, kfrag_off, vfrag_off, qf, kf, vf[0], sc, tmax);
        if (t == 0) {
          m_run[0] = tmax[0];
          m_run[1] = tmax[1];
        }
        if (__builtin_amdgcn_ballot_w64(tmax[0] > m_run[0] + kLazy || tmax[1] > m_run[1] + kLazy)) break;
        // ---- tile t+1 has landed: every wavefront waits for its own loads, then the barrier ------------
        fetch_wait(t);
        __syncthreads();
        // ---- tile t+3 sets out into the buffer of tile t-1, which every wavefront has left: its loads are issued
        // one by one under the products below (all at once here when it is the segment's last, partial tile) ----
        bt_arrived(pc_ahead);
        const bool more = t + 3 < ntile, piecewise = more && whole_tile(t + 3);
        const uint8_t* const src_ahead = tile_src(t + 3, pc_ahead);
        if (more && !piecewise) fetch(t + 3, pc_ahead);
        pc_ahead = bt_request(t + 4);
        uint4 pp[2];
        probabilities(sc, pp);
        // ---- O^T += V^T P^T: one 32-token product per 16 columns and row tile; row sums from ones ----
        const uint8_t* nbuf = tiles + tile_buf(t + 1);
        static_assert(NVG >= (kMlaHeadsLoads + 3) / 4, "one direct load per group of products");
#pragma unroll
        for (int j = 0; j < NVG; ++j) {
          if (j + 1 < NVG) load_v(buf, vfrag_off, j + 1, vf[(j + 1) & 1]);
          else if (t + 1 < ntile) load_k(nbuf, kfrag_off, 0, kf[0]);
          MI_SB();
#pragma unroll
          for (int e = 0; e < VB; ++e) {
            const uint4 a = make_uint4(vf[j & 1][e][0].x, vf[j & 1][e][0].y, vf[j & 1][e][1].x, vf[j & 1][e][1].y);
#pragma unroll
            for (int h2 = 0; h2 < 2; ++h2) {
              if (VB * j + e >= NE - 3) {
                // The compiler gives every matrix product of the kernel its result in accumulation registers; 256 sums
                // + 16 scores + 8 row sums are 280 of the 256 there are, so it keeps 24 sums in vector registers and
                // moves them in and out around their products (108 moves per tile).  These six tiles are therefore
                // multiplied in the vector-register form, by hand: their registers are touched by nothing else in the
                // loop (next by the same product one tile later, then by the epilogue), the fragment operands come
                // from LDS reads the compiler waits for, and the probabilities were written many instructions ago
                // (the s_nop covers the two wait states a vector write needs before a product reads it).
                typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
                const u32x4_t av = {a.x, a.y, a.z, a.w}, bv = {pp[h2].x, pp[h2].y, pp[h2].z, pp[h2].w};
                if constexpr (F16)
                  asm volatile("s_nop 1\n\tv_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(acc[h2][VB * j + e]) : "v"(av), "v"(bv));
                else
                  asm volatile("s_nop 1\n\tv_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(acc[h2][VB * j + e]) : "v"(av), "v"(bv));
              } else {
                acc[h2][VB * j + e] = mfma_16x16x32<F16>(a, pp[h2], acc[h2][VB * j + e]);
              }
            }
          }
          if (j < (kMlaHeadsLoads + 3) / 4 && piecewise) fetch_piece(t + 3, src_ahead, j, piece_off[j]);
          if (j == 0) {
#pragma unroll
            for (int h2 = 0; h2 < 2; ++h2)
              l_run[h2] += mfma_16x16x32<F16>(ones, pp[h2], f32x4_t{0.f, 0.f, 0.f, 0.f})[0];
          }
          MI_SB();
        }
      }
      // (the hand-written products above are not known to the compiler as such: the wait states a vector instruction
      // needs before it reads a matrix result, spelled out)
      asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");
      // ---- the sums leave the registers: acc[h2][e][i] is output column 16 e + 4 g + i of head hq0 + 16 h2.
      // The segment's result when every tile is done; otherwise as they are, for the loop below ---------
      const bool done = t >= ntile;
#pragma unroll
      for (int h2 = 0; h2 < 2; ++h2) {
        const float inv = done ? 1.f / l_run[h2] : 1.f;
        const int hq = hq0 + 16 * h2;
        const int64_t prow = (int64_t)slot * p.Hq + hq;
        if (done && whole) {
          uint16_t* o = p.out + (int64_t)row * p.o_st + (int64_t)hq * p.o_sh + 4 * g;
#pragma unroll
          for (int e = 0; e < NE; ++e)
            st8(o + 16 * e, make_uint2(pack2<F16>(acc[h2][e][0] * inv, acc[h2][e][1] * inv),
                                       pack2<F16>(acc[h2][e][2] * inv, acc[h2][e][3] * inv)));
        } else {
          float* o = p.part_o + prow * HDV + 4 * g;
#pragma unroll
          for (int e = 0; e < NE; ++e)
            *reinterpret_cast<float4*>(o + 16 * e) =
                make_float4(acc[h2][e][0] * inv, acc[h2][e][1] * inv, acc[h2][e][2] * inv, acc[h2][e][3] * inv);
          if (done && g == 0) p.part_lse[prow] = m_run[h2] + fast_log2(l_run[h2]);
        }
      }
    }
    if (t < ntile) {
      // ---- the slow loop: sums in memory, every lane reading back only what it wrote itself (the fences make
      // its own earlier stores what its loads see) ---------------------------------------------------------
      float* const po0 = p.part_o + ((int64_t)slot * p.Hq + hq0) * HDV + 4 * g;
      float* const po1 = po0 + (int64_t)16 * HDV;
      // (the query fragments are fetched again: kept alive across the stores above, some of them would live in
      // scratch memory -- in the fast loop as well)
      uint4 qs[2][KS];
      load_q(qs);
      for (; t < ntile; ++t) {
        const uint8_t* buf = tiles + tile_buf(t);
        uint4 kf[2][KB];
        uint2 vf[2][VB][2];
        f32x4_t sc[2][2];
        float tmax[2], alpha[2];

        int kfrag_off, vfrag_off;
        frag_offsets(kfrag_off, vfrag_off);
        load_k(buf, kfrag_off, 0, kf[0]);
        scores(t, buf, kfrag_off, vfrag_off, qs, kf, vf[0], sc, tmax);
#pragma unroll
        for (int h2 = 0; h2 < 2; ++h2) {
          const float m_new = fmaxf(m_run[h2], tmax[h2]);
          alpha[h2] = fast_exp2(m_run[h2] - m_new);
          m_run[h2] = m_new;
        }
        fetch_wait(t);
        __syncthreads();
        bt_arrived(pc_ahead);
        if (t + 3 < ntile) fetch(t + 3, pc_ahead);
        pc_ahead = bt_request(t + 4);
        uint4 pp[2];
        probabilities(sc, pp);
        __threadfence();
#pragma unroll
        for (int j = 0; j < NVG; ++j) {
          if (j + 1 < NVG) load_v(buf, vfrag_off, j + 1, vf[(j + 1) & 1]);
          MI_SB();
#pragma unroll
          for (int e = 0; e < VB; ++e) {
            const uint4 a = make_uint4(vf[j & 1][e][0].x, vf[j & 1][e][0].y, vf[j & 1][e][1].x, vf[j & 1][e][1].y);
#pragma unroll
            for (int h2 = 0; h2 < 2; ++h2) {
              const f32x4_t add = mfma_16x16x32<F16>(a, pp[h2], f32x4_t{0.f, 0.f, 0.f, 0.f});
              float4* o = reinterpret_cast<float4*>((h2 ? po1 : po0) + 16 * (VB * j + e));
              float4 v = *o;
              v.x = __builtin_fmaf(v.x, alpha[h2], add[0]); v.y = __builtin_fmaf(v.y, alpha[h2], add[1]);
              v.z = __builtin_fmaf(v.z, alpha[h2], add[2]); v.w = __builtin_fmaf(v.w, alpha[h2], add[3]);
              *o = v;
            }
          }
          MI_SB();
        }
#pragma unroll
        for (int h2 = 0; h2 < 2; ++h2)
          l_run[h2] = l_run[h2] * alpha[h2] + mfma_16x16x32<F16>(ones, pp[h2], f32x4_t{0.f, 0.f, 0.f, 0.f})[0];
      }
      __threadfence();
#pragma unroll
      for (int h2 = 0; h2 < 2; ++h2) {
        const float inv = 1.f / l_run[h2];
        const int hq = hq0 + 16 * h2;
        float* po = h2 ? po1 : po0;
        uint16_t* o = p.out + (int64_t)row * p.o_st + (int64_t)hq * p.o_sh + 4 * g;
#pragma unroll 4
        for (int e = 0; e < NE; ++e) {
          float4 v = *reinterpret_cast<const float4*>(po + 16 * e);
          v.x *= inv; v.y *= inv; v.z *= inv; v.w *= inv;
          if (whole) st8(o + 16 * e, make_uint2(pack2<F16>(v.x, v.y), pack2<F16>(v.z, v.w)));
          else *reinterpret_cast<float4*>(po + 16 * e) = v;
        }
        if (!whole && g == 0) p.part_lse[(int64_t)slot * p.Hq + hq] = m_run[h2] + fast_log2(l_run[h2]);
      }
    }
  });
#undef MI_SB
}

// One workgroup per (request, query head): merge the partials of the workgroups that
// shared the request; zero-length rows get zeros.  blockDim.x = HD * S: S groups of HD threads take the
// segments round-robin in batches of 8 (a request cut over hundreds of workgroups is a chain of dependent
// memory round trips otherwise) and group 0 folds the S running (maximum, numerator, denominator) triples.
// One workgroup per (request, block of heads): a thread owns four neighbouring output values of one head (16-byte
// loads of the fp32 partials, one 8-byte store), `cols` = heads-per-workgroup x head_dim / 4 threads cover the block
// and `groups` such thread groups take the request's segments round-robin in batches of 8 loads; group 0 folds their
// (maximum, numerators, denominator) through LDS.
struct MergeShape {
  int hd;        // width of the output rows (values per head)
  int hpw;       // heads per workgroup
  int cols;      // threads per group = hpw * hd / 4
  int groups;    // thread groups (blockDim.x = cols * groups)
};
template <bool F16>
__global__ __launch_bounds__(1024) void paged_decode_merge_kernel(DecodeParams p, MergeShape ms) {
  __shared__ float red[6][1024];
  const int r = blockIdx.y;
  const int col = threadIdx.x % ms.cols, grp = threadIdx.x / ms.cols;
  const int q4 = ms.hd >> 2;
  const int hq = blockIdx.x * ms.hpw + col / q4, d = 4 * (col % q4);
  int row;
  if (!decode_row(p, r, row)) return;
  // The kernel is a chain of dependent memory round trips, so everything that does not depend
  // on a loaded value is requested at once: length and segment range here, then LSE and partial
  // of every segment together (the running-maximum form below needs no first pass over the LSEs).
  const int len = p.lens[r];
  const int first = p.seg_info[2 * r], last = p.seg_info[2 * r + 1];  // stale for len <= 0: not used then
  const bool live = hq < p.Hq;                                        // (the last block of heads may be partial)
  uint16_t* o = p.out + (int64_t)row * p.o_st + (int64_t)(live ? hq : 0) * p.o_sh + d;
  if (len <= 0) {  // (uniform over the workgroup, like the two returns around it)
    if (grp == 0 && live) st8(o, make_uint2(0u, 0u));
    return;
  }
  if (first == last) return;  // written directly by the streaming kernel
  float mx = -INFINITY, den = 0.f;
  float4 num = make_float4(0.f, 0.f, 0.f, 0.f);
  const int hq_c = live ? hq : p.Hq - 1;
  for (int w0 = first + 8 * grp; w0 <= last; w0 += 8 * ms.groups) {
    float lse[8];
    float4 po[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int64_t slot = (int64_t)(min(w0 + j, last) + r) * p.Hq + hq_c;
      lse[j] = p.part_lse[slot];
      po[j] = *reinterpret_cast<const float4*>(p.part_o + slot * ms.hd + d);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (w0 + j <= last) {
        const float m_new = fmaxf(mx, lse[j]);
        const float a = fast_exp2(mx - m_new), wt = fast_exp2(lse[j] - m_new);
        num.x = num.x * a + wt * po[j].x; num.y = num.y * a + wt * po[j].y;
        num.z = num.z * a + wt * po[j].z; num.w = num.w * a + wt * po[j].w;
        den = den * a + wt;
        mx = m_new;
      }
    }
  }
  if (ms.groups > 1) {
    red[0][threadIdx.x] = mx; red[1][threadIdx.x] = den;
    red[2][threadIdx.x] = num.x; red[3][threadIdx.x] = num.y; red[4][threadIdx.x] = num.z; red[5][threadIdx.x] = num.w;
    __syncthreads();
    if (grp != 0) return;
    for (int g2 = 1; g2 < ms.groups; ++g2) {
      const int t = g2 * ms.cols + col;
      const float m2 = red[0][t];
      if (m2 == -INFINITY) continue;  // that group had no segment
      const float m_new = fmaxf(mx, m2);
      const float a = fast_exp2(mx - m_new), wt = fast_exp2(m2 - m_new);
      num.x = num.x * a + wt * red[2][t]; num.y = num.y * a + wt * red[3][t];
      num.z = num.z * a + wt * red[4][t]; num.w = num.w * a + wt * red[5][t];
      den = den * a + wt * red[1][t];
      mx = m_new;
    }
  }
  if (!live) return;
  const float inv = 1.f / den;
  st8(o, make_uint2(pack2<F16>(num.x * inv, num.y * inv), pack2<F16>(num.z * inv, num.w * inv)));
}

// Shape of the merge launch: about 256 threads per thread group (whole heads), one group per 8 segments a request
// is expected to be cut into, as far as 1024 threads go.
static MergeShape merge_shape(int grid_x, int R, int Hq, int head_dim) {
  MergeShape ms;
  ms.hd = head_dim;
  const int q4 = head_dim / 4;
  ms.hpw = 256 / q4 > 0 ? 256 / q4 : 1;
  if (ms.hpw > Hq) ms.hpw = Hq;
  ms.cols = ms.hpw * q4;
  const int per_request = grid_x / (R > 0 ? R : 1) + 2;
  int g = (per_request + 7) / 8;
  if (g > 1024 / ms.cols) g = 1024 / ms.cols;
  if (g > 8) g = 8;
  ms.groups = g < 1 ? 1 : g;
  return ms;
}
static void launch_merge(const DecodeParams& p, int grid_x, int R, int Hq, int head_dim, bool f16, hipStream_t st) {
  const MergeShape ms = merge_shape(grid_x, R, Hq, head_dim);
  const dim3 mgrid((Hq + ms.hpw - 1) / ms.hpw, R), mblock(ms.cols * ms.groups);
  if (f16) hipLaunchKernelGGL((paged_decode_merge_kernel<true>), mgrid, mblock, 0, st, p, ms);
  else hipLaunchKernelGGL((paged_decode_merge_kernel<false>), mgrid, mblock, 0, st, p, ms);
}

// Requests one launch of the streaming kernels takes: their tile prefix sums and lengths sit in LDS.
constexpr int kMaxRequestsPerLaunch = 7680;

// Wavefronts along the heads: one per KV head and 16 query heads that share it.
static int head_waves(int Hq, int Hkv) { return Hkv * ((Hq / Hkv + 15) / 16); }

static int pick_waves_per_block(int waves, const MiTuning& tune) {
  int cap = tune.decode_waves_per_block;
  if (cap < 1 || cap > 8) cap = 8;
  for (int w = cap; w >= 1; --w)
    if (waves % w == 0) return w;
  return 1;
}

static int device_cu_count() {
  static std::atomic<int> cus[64];  // zero-initialised; callers on several host threads may race to fill a slot
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  int n = cus[dev].load(std::memory_order_relaxed);
  if (!n) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cus[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

// Workgroups along the flattened tile sequence: enough to put `decode_wgs_per_cu`
// workgroups of 8 waves (or the equivalent in smaller workgroups) on every CU.
int decode_grid_size(int Hq, int Hkv, const MiTuning& tune) {
  const int forced = tune.decode_grid;
  if (forced > 0) return forced;
  const int waves = head_waves(Hq, Hkv);
  const int wpb = pick_waves_per_block(waves, tune);
  const int head_groups = waves / wpb;
  int per_cu = tune.decode_wgs_per_cu * (8 / wpb);
  int grid = device_cu_count() * per_cu / head_groups;
  return grid < 1 ? 1 : grid;
}

}  // namespace mi

using namespace mi;

extern "C" int64_t mi_decode_workspace_bytes(int32_t R, int32_t Hq, int32_t Hkv, int32_t head_dim,
                                             int32_t chunk_tokens, int32_t max_kv_len,
                                             int32_t split_tokens, const MiTuning* tuning) {
  (void)chunk_tokens; (void)max_kv_len; (void)split_tokens;  // (the size depends on R, the head counts and the grid only)
  if (R <= 0 || Hq <= 0 || Hkv <= 0 || head_dim <= 0 || Hq % Hkv) return 0;
  MiTuning tune;
  if (mi_resolve_tuning(tuning, &tune, "mi_decode_workspace_bytes") != MI_OK) return -1;
  const int64_t slots = (int64_t)decode_grid_size(Hq, Hkv, tune) + R;
  return slots * Hq * (head_dim + 1) * (int64_t)sizeof(float) + (int64_t)R * 2 * sizeof(int32_t);
}

int mi::check_decode_workspace(const void* workspace, int64_t workspace_bytes, int32_t R, int32_t Hq, int32_t Hkv,
                               int32_t head_dim, int32_t split_tokens, const MiTuning& tune, const char* who) {
  static thread_local char msg[192];
  if (split_tokens < 0 || split_tokens % 16) {
    snprintf(msg, sizeof msg, "%s: split_tokens must be a non-negative multiple of 16", who);
    return mi_fail(MI_ERR_SHAPE, msg);
  }
  // a batch above kMaxRequestsPerLaunch runs in slices of that many requests over the same workspace
  const int64_t n = R < kMaxRequestsPerLaunch ? R : kMaxRequestsPerLaunch;
  const int64_t slots = (int64_t)decode_grid_size(Hq, Hkv, tune) + n;
  const int64_t need = slots * Hq * (head_dim + 1) * (int64_t)sizeof(float) + n * 2 * (int64_t)sizeof(int32_t);
  if (!workspace || workspace_bytes < need) {
    snprintf(msg, sizeof msg, "%s: workspace too small (see mi_decode_workspace_bytes)", who);
    return mi_fail(MI_ERR_WORKSPACE, msg);
  }
  if ((uintptr_t)workspace & 15) {
    snprintf(msg, sizeof msg, "%s: workspace must be 16-byte aligned", who);
    return mi_fail(MI_ERR_ALIGN, msg);
  }
  return MI_OK;
}

int mi::launch_paged_decode(
    const void* q, int64_t q_stride_tok, int64_t q_stride_head, const void* k_cache,
    const void* v_cache, int64_t kv_stride_chunk, int64_t kv_stride_tok, int64_t kv_stride_head,
    const int32_t* block_table, int64_t bt_stride, const int32_t* kv_lens, const int32_t* cu_seqlens_q,
    void* out, int64_t o_stride_tok, int64_t o_stride_head, void* workspace, int64_t workspace_bytes,
    int32_t R, int32_t Hq, int32_t Hkv, int32_t head_dim, int32_t chunk_tokens,
    int32_t split_tokens, float softmax_scale, int32_t kv_dtype, const float* k_scales,
    const float* v_scales, int32_t dtype, const MiTuning& tune, void* stream, const FusedStepArgs* fused) {
  if (R == 0) return MI_OK;
  if (dtype != MI_DTYPE_BF16 && dtype != MI_DTYPE_FP16)
    return mi_fail(MI_ERR_UNSUPPORTED, "mi_paged_decode_attention: dtype must be MI_DTYPE_BF16 or MI_DTYPE_FP16");
  const bool f16 = dtype == MI_DTYPE_FP16;
  if (!q || !k_cache || !v_cache || !block_table || !kv_lens || !out)
    return mi_fail(MI_ERR_NULL, "mi_paged_decode_attention: null pointer argument");
  if (R < 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv)
    return mi_fail(MI_ERR_SHAPE, "mi_paged_decode_attention: need R >= 0 and Hq a multiple of Hkv");
  const int G = Hq / Hkv;
  if (G > 64) return mi_fail(MI_ERR_UNSUPPORTED, "mi_paged_decode_attention: more than 64 query heads per KV head");
  if (head_dim != 64 && head_dim != 96 && head_dim != 128 && head_dim != 192 && head_dim != 256)
    return mi_fail(MI_ERR_UNSUPPORTED, "mi_paged_decode_attention: head_dim must be 64, 96, 128, 192 or 256");
  if (chunk_tokens <= 0 || chunk_tokens % 16)
    return mi_fail(MI_ERR_SHAPE, "mi_paged_decode_attention: chunk size must be a positive multiple of 16");
  if (kv_dtype != MI_KV_BF16 && kv_dtype != MI_KV_FP8_E4M3)
    return mi_fail(MI_ERR_UNSUPPORTED, "mi_paged_decode_attention: unknown kv_dtype");
  if (kv_dtype == MI_KV_FP8_E4M3 && ((head_dim != 64 && head_dim != 128) || !k_scales || !v_scales))
    return mi_fail(MI_ERR_UNSUPPORTED, "mi_paged_decode_attention: fp8 KV needs head_dim 64 or 128 and both scale arrays");
  const int esz = kv_dtype == MI_KV_FP8_E4M3 ? 1 : 2;
  if (((uintptr_t)q | (uintptr_t)k_cache | (uintptr_t)v_cache | (uintptr_t)out) & 15)
    return mi_fail(MI_ERR_ALIGN, "mi_paged_decode_attention: q/k/v/out must be 16-byte aligned");
  if ((q_stride_tok | q_stride_head | o_stride_tok | o_stride_head) % 8 ||
      ((kv_stride_chunk | kv_stride_tok | kv_stride_head) * esz) % 16)
    return mi_fail(MI_ERR_ALIGN, "mi_paged_decode_attention: strides must keep rows 16-byte aligned");
  if (kv_stride_tok * (int64_t)chunk_tokens * esz >= (int64_t)1 << 31)
    return mi_fail(MI_ERR_SHAPE, "mi_paged_decode_attention: one chunk must span less than 2 GiB");
  // The per-request prefix sums and lengths live in LDS (8 bytes per request): a larger batch is streamed in
  // slices of kMaxRequestsPerLaunch requests, one after the other on the same stream and workspace.  Every
  // argument check above is independent of the slice, so either all slices run or none does.
  {
    const int rc_w = check_decode_workspace(workspace, workspace_bytes, R, Hq, Hkv, head_dim, split_tokens, tune,
                                            "mi_paged_decode_attention");
    if (rc_w != MI_OK) return rc_w;
  }
  if (R > kMaxRequestsPerLaunch) {
    for (int r0 = 0; r0 < R; r0 += kMaxRequestsPerLaunch) {
      const int n = R - r0 < kMaxRequestsPerLaunch ? R - r0 : kMaxRequestsPerLaunch;
      // with cu_seqlens_q the rows of q / out are addressed through it, else request r owns row r
      const int64_t row0 = cu_seqlens_q ? 0 : r0;
      FusedStepArgs fs;
      if (fused) {
        fs = *fused;
        fs.k_new = (const uint16_t*)fs.k_new + r0 * fs.k_stride_tok;
        fs.v_new = (const uint16_t*)fs.v_new + r0 * fs.v_stride_tok;
        if (fs.positions) fs.positions += r0;
      }
      const int rc = launch_paged_decode(
          (const uint16_t*)q + row0 * q_stride_tok, q_stride_tok, q_stride_head, k_cache, v_cache, kv_stride_chunk,
          kv_stride_tok, kv_stride_head, block_table + (int64_t)r0 * bt_stride, bt_stride, kv_lens + r0,
          cu_seqlens_q ? cu_seqlens_q + r0 : nullptr, (uint16_t*)out + row0 * o_stride_tok, o_stride_tok, o_stride_head,
          workspace, workspace_bytes, n, Hq, Hkv, head_dim, chunk_tokens, split_tokens, softmax_scale, kv_dtype, k_scales,
          v_scales, dtype, tune, stream, fused ? &fs : nullptr);
      if (rc != MI_OK) return rc;
    }
    return MI_OK;
  }

  const int grid_x = decode_grid_size(Hq, Hkv, tune);
  const int64_t slots = (int64_t)grid_x + R;

  // 16-token sub-tiles per loop iteration (0 = automatic).
  int nt = tune.decode_tile_subtiles;
  if (nt != 1 && nt != 2 && nt != 4) nt = kv_dtype == MI_KV_FP8_E4M3 ? 4 : 2;
  if (head_dim == 256) nt = 1;                 // (registers: 64 accumulators + 32 each for queries, keys, values)
  else if (head_dim == 192 && nt > 2) nt = 2;
  if (fused) nt = kv_dtype == MI_KV_FP8_E4M3 ? MI_FUSED_FP8_NT : 1;  // (the prologue's registers on top of two 16-bit sub-tiles in flight would spill)
  while (chunk_tokens % (16 * nt)) nt >>= 1;  // a tile must not straddle two chunks
  const int minw = head_dim > 128 ? 2 : tune.decode_min_waves;
  const int tk = 16 * nt;
  // a small batch is cut finer than a large one needs: 64 tokens per workgroup put a single 8 192-token
  // request on 128 CUs (17.8 us against 33 us with 256-token spans); large batches get equal spans anyway
  const int min_span_tokens = split_tokens > 0 ? split_tokens : 64;

  DecodeParams p;
  p.q = (const uint16_t*)q; p.q_st = q_stride_tok; p.q_sh = q_stride_head;
  p.kc = (const uint8_t*)k_cache; p.vc = (const uint8_t*)v_cache;
  p.kv_sc = kv_stride_chunk; p.kv_st = (int32_t)kv_stride_tok; p.kv_sh = (int32_t)kv_stride_head;
  p.bt = block_table; p.bt_stride = bt_stride; p.lens = kv_lens; p.cu_q = cu_seqlens_q;
  p.out = (uint16_t*)out; p.o_st = o_stride_tok; p.o_sh = o_stride_head;
  p.part_o = (float*)workspace;
  p.part_lse = p.part_o + slots * Hq * head_dim;
  p.seg_info = (int32_t*)(p.part_lse + slots * Hq);
  p.k_scale = k_scales; p.v_scale = v_scales;
  p.R = R; p.Hq = Hq; p.Hkv = Hkv; p.G = G; p.chunk = chunk_tokens;
  p.parts = (G + 15) / 16;
  p.chunk_magic = (((uint64_t)1 << 40) + chunk_tokens - 1) / chunk_tokens;
  p.min_span_tiles = (min_span_tokens + tk - 1) / tk;
  p.grid = grid_x;
  p.scale_log2 = softmax_scale * 1.4426950408889634f;
  if (fused) {
    p.q_gst = fused->q_stride_group;
    p.nk = (const uint16_t*)fused->k_new; p.nk_st = fused->k_stride_tok; p.nk_hst = fused->k_stride_head;
    p.nv = (const uint16_t*)fused->v_new; p.nv_st = fused->v_stride_tok; p.nv_hst = fused->v_stride_head;
    p.q_w = (const uint16_t*)fused->q_weight; p.k_w = (const uint16_t*)fused->k_weight;
    p.emb = fused->rotary_angles; p.emb_stride = fused->angles_stride; p.pos = fused->positions;
    p.rot = fused->rot_dim; p.norm = fused->norm_kind; p.interleaved = fused->rotary_interleaved;
    p.faithful = fused->faithful_rounding; p.eps = fused->eps; p.mscale = fused->mscale;
    p.headroom = fused->fp8_headroom;
  }

  const int waves = head_waves(Hq, Hkv);
  const int wpb = pick_waves_per_block(waves, tune);
  dim3 grid(grid_x, waves / wpb), block(64 * wpb);
  // (fused step: per wavefront cos | sin | key row in fp32 behind the per-request arrays)
  const size_t lds = fused ? (((size_t)R * 2 * sizeof(int32_t) + 15) & ~(size_t)15) + (size_t)wpb * 3 * head_dim * sizeof(float)
                           : (size_t)R * 2 * sizeof(int32_t);
  hipStream_t st = (hipStream_t)stream;
  hipEvent_t ev_a, ev_b;
  const bool timed = mi_profile_next(&ev_a, &ev_b);
  if (timed) (void)hipEventRecord(ev_a, st);
#define MI_LAUNCH_DECODE(HD_, FP8_, F16_)                                                                              \
  do {                                                                                                                 \
    if (nt == 4) hipLaunchKernelGGL((paged_decode_stream_kernel<HD_, 4, FP8_, 2, F16_>), grid, block, lds, st, p);          \
    else if (nt == 1 && minw >= 4) hipLaunchKernelGGL((paged_decode_stream_kernel<HD_, 1, FP8_, 4, F16_>), grid, block, lds, st, p); \
    else if (nt == 1) hipLaunchKernelGGL((paged_decode_stream_kernel<HD_, 1, FP8_, 3, F16_>), grid, block, lds, st, p);     \
    else if (minw >= 4) hipLaunchKernelGGL((paged_decode_stream_kernel<HD_, 2, FP8_, 4, F16_>), grid, block, lds, st, p);   \
    else if (minw == 3) hipLaunchKernelGGL((paged_decode_stream_kernel<HD_, 2, FP8_, 3, F16_>), grid, block, lds, st, p);   \
    else hipLaunchKernelGGL((paged_decode_stream_kernel<HD_, 2, FP8_, 2, F16_>), grid, block, lds, st, p);                  \
  } while (0)
  // wide heads: two wavefronts per SIMD (256 registers each), tiles of 16 or 32 tokens
#define MI_LAUNCH_DECODE_WIDE(HD_, F16_)                                                                               \
  do {                                                                                                                 \
    if (nt == 2 && HD_ < 256) hipLaunchKernelGGL((paged_decode_stream_kernel<HD_, (HD_ < 256 ? 2 : 1), false, 2, F16_>), grid, block, lds, st, p); \
    else hipLaunchKernelGGL((paged_decode_stream_kernel<HD_, 1, false, 2, F16_>), grid, block, lds, st, p);               \
  } while (0)
#define MI_LAUNCH_STEP(HD_, F16_) hipLaunchKernelGGL((decode_step_stream_kernel<HD_, 1, F16_>), grid, block, lds, st, p)
#define MI_LAUNCH_STEP_WIDE(HD_, F16_) hipLaunchKernelGGL((decode_step_stream_kernel<HD_, 1, F16_, 2>), grid, block, lds, st, p)
  if (fused && kv_dtype == MI_KV_FP8_E4M3 && f16)
    hipLaunchKernelGGL((decode_step_stream_kernel<128, MI_FUSED_FP8_NT, true, 3, true>), grid, block, lds, st, p);
  else if (fused && kv_dtype == MI_KV_FP8_E4M3)
    hipLaunchKernelGGL((decode_step_stream_kernel<128, MI_FUSED_FP8_NT, false, 3, true>), grid, block, lds, st, p);
  else if (fused && head_dim == 128 && f16) MI_LAUNCH_STEP(128, true);
  else if (fused && head_dim == 128) MI_LAUNCH_STEP(128, false);
  else if (fused && head_dim == 64 && f16) MI_LAUNCH_STEP(64, true);
  else if (fused && head_dim == 64) MI_LAUNCH_STEP(64, false);
  else if (fused && head_dim == 96 && f16) MI_LAUNCH_STEP(96, true);
  else if (fused && head_dim == 96) MI_LAUNCH_STEP(96, false);
  else if (fused && head_dim == 192 && f16) MI_LAUNCH_STEP_WIDE(192, true);
  else if (fused && head_dim == 192) MI_LAUNCH_STEP_WIDE(192, false);
  else if (fused && f16) MI_LAUNCH_STEP_WIDE(256, true);
  else if (fused) MI_LAUNCH_STEP_WIDE(256, false);
  else if (kv_dtype == MI_KV_FP8_E4M3 && head_dim == 64 && f16) MI_LAUNCH_DECODE(64, true, true);
  else if (kv_dtype == MI_KV_FP8_E4M3 && head_dim == 64) MI_LAUNCH_DECODE(64, true, false);
  else if (kv_dtype == MI_KV_FP8_E4M3 && f16) MI_LAUNCH_DECODE(128, true, true);
  else if (kv_dtype == MI_KV_FP8_E4M3) MI_LAUNCH_DECODE(128, true, false);
  else if (head_dim == 128 && f16) MI_LAUNCH_DECODE(128, false, true);
  else if (head_dim == 128) MI_LAUNCH_DECODE(128, false, false);
  else if (head_dim == 64 && f16) MI_LAUNCH_DECODE(64, false, true);
  else if (head_dim == 64) MI_LAUNCH_DECODE(64, false, false);
  else if (head_dim == 96 && f16) MI_LAUNCH_DECODE(96, false, true);
  else if (head_dim == 96) MI_LAUNCH_DECODE(96, false, false);
  else if (head_dim == 192 && f16) MI_LAUNCH_DECODE_WIDE(192, true);
  else if (head_dim == 192) MI_LAUNCH_DECODE_WIDE(192, false);
  else if (f16) MI_LAUNCH_DECODE_WIDE(256, true);
  else MI_LAUNCH_DECODE_WIDE(256, false);
#undef MI_LAUNCH_DECODE
#undef MI_LAUNCH_DECODE_WIDE
#undef MI_LAUNCH_STEP
#undef MI_LAUNCH_STEP_WIDE
  if (timed) (void)hipEventRecord(ev_b, st);
  launch_merge(p, p.grid, R, Hq, head_dim, f16, st);
  return mi_check_launch("mi_paged_decode_attention");
}

extern "C" int mi_paged_decode_attention(
    const void* q, int64_t q_stride_tok, int64_t q_stride_head, const void* k_cache,
    const void* v_cache, int64_t kv_stride_chunk, int64_t kv_stride_tok, int64_t kv_stride_head,
    const int32_t* block_table, int64_t bt_stride, const int32_t* kv_lens, void* out,
    int64_t o_stride_tok, int64_t o_stride_head, void* workspace, int64_t workspace_bytes,
    int32_t R, int32_t Hq, int32_t Hkv, int32_t head_dim, int32_t chunk_tokens, int32_t max_kv_len,
    int32_t split_tokens, float softmax_scale, int32_t kv_dtype, const float* k_scales,
    const float* v_scales, int32_t dtype, const MiTuning* tuning, void* stream) {
  (void)max_kv_len;
  MiTuning tune;
  const int rc = mi_resolve_tuning(tuning, &tune, "mi_paged_decode_attention");
  if (rc != MI_OK) return rc;
  return launch_paged_decode(q, q_stride_tok, q_stride_head, k_cache, v_cache, kv_stride_chunk, kv_stride_tok,
                             kv_stride_head, block_table, bt_stride, kv_lens, nullptr, out, o_stride_tok,
                             o_stride_head, workspace, workspace_bytes, R, Hq, Hkv, head_dim, chunk_tokens,
                             split_tokens, softmax_scale, kv_dtype, k_scales, v_scales, dtype, tune, stream);
}

static int decode_step_entry(
    const char* who, const void* q, int64_t q_stride_tok, int64_t q_stride_group, const void* k_new, int64_t k_stride_tok,
    int64_t k_stride_head, const void* v_new, int64_t v_stride_tok, int64_t v_stride_head, const void* q_weight,
    const void* k_weight, float eps, int32_t norm_kind, const float* rotary_angles, int64_t angles_stride,
    int32_t rot_dim, int32_t rotary_interleaved, float mscale, const int64_t* positions, void* k_cache, void* v_cache,
    int64_t kv_stride_chunk, int64_t kv_stride_tok, int64_t kv_stride_head, const int32_t* block_table,
    int64_t bt_stride, const int32_t* kv_lens, void* out, int64_t o_stride_tok, int64_t o_stride_head, void* workspace,
    int64_t workspace_bytes, int32_t R, int32_t Hq, int32_t Hkv, int32_t head_dim, int32_t chunk_tokens,
    int32_t split_tokens, float softmax_scale, int32_t faithful_rounding, int32_t dtype, const MiTuning* tuning,
    void* stream, int32_t kv_dtype, float* k_scales, float* v_scales, float headroom) {
  const bool fp8 = kv_dtype == MI_KV_FP8_E4M3;
  char msg[160];
  auto fail = [&](int code, const char* what) {
    snprintf(msg, sizeof msg, "%s: %s", who, what);
    return mi_fail(code, msg);
  };
  if (R == 0) return MI_OK;
  MiTuning tune;
  const int rc = mi_resolve_tuning(tuning, &tune, who);
  if (rc != MI_OK) return rc;
  if (!q || !k_new || !v_new || !k_cache || !v_cache) return fail(MI_ERR_NULL, "null pointer argument");
  if (R < 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv) return fail(MI_ERR_SHAPE, "need R >= 0 and Hq a multiple of Hkv");
  if (head_dim != 64 && head_dim != 96 && head_dim != 128 && head_dim != 192 && head_dim != 256)
    return fail(MI_ERR_UNSUPPORTED, "head_dim must be 64, 96, 128, 192 or 256");
  if (norm_kind != MI_NORM_NONE && norm_kind != MI_NORM_RMS && norm_kind != MI_NORM_L2)
    return fail(MI_ERR_UNSUPPORTED, "unknown norm kind");
  if (rotary_angles) {
    if (rot_dim <= 0 || rot_dim > head_dim || (rot_dim & 1) || angles_stride < rot_dim)
      return fail(MI_ERR_SHAPE, "rot_dim must be even and within head_dim");
    // a lane holds 8 consecutive elements of every 32: half-split partners must sit a whole number of 32s away
    if (!rotary_interleaved && (rot_dim / 2) % 32)
      return fail(MI_ERR_UNSUPPORTED, "half-split rotary pairs need rot_dim / 2 to be a multiple of 32 (else: the separate calls)");
    // (an fp8 cache's key bytes put a lane's 16 consecutive elements of every 64 into two fragments)
    if (fp8 && !rotary_interleaved && (rot_dim / 2) % 64)
      return fail(MI_ERR_UNSUPPORTED, "over an fp8 cache half-split rotary pairs need rot_dim / 2 to be a multiple of 64 (else: the separate calls)");
  }
  if (fp8 && (head_dim != 128 || !k_scales || !v_scales || !(headroom > 0.f)))
    return fail(MI_ERR_UNSUPPORTED, "an fp8 cache needs head_dim 128, both scale arrays and a positive headroom");
  const int G = Hq / Hkv;
  if (q_stride_group < (int64_t)G * head_dim) return fail(MI_ERR_SHAPE, "query group stride smaller than (Hq / Hkv) * head_dim");
  if ((((uintptr_t)q | (uintptr_t)q_weight) & 15) || (q_stride_tok | q_stride_group) % 8)
    return fail(MI_ERR_ALIGN, "q, the query norm weight and the q strides must keep rows 16-byte aligned");
  if ((((uintptr_t)v_new | (uintptr_t)k_new) & 3) || ((v_stride_tok | v_stride_head) & 1))
    return fail(MI_ERR_ALIGN, "new key / value rows must be 4-byte aligned");
  FusedStepArgs fs;
  fs.q_stride_group = q_stride_group;
  fs.k_new = k_new; fs.k_stride_tok = k_stride_tok; fs.k_stride_head = k_stride_head;
  fs.v_new = v_new; fs.v_stride_tok = v_stride_tok; fs.v_stride_head = v_stride_head;
  fs.q_weight = q_weight; fs.k_weight = k_weight; fs.eps = eps; fs.norm_kind = norm_kind;
  fs.rotary_angles = rotary_angles; fs.angles_stride = angles_stride; fs.rot_dim = rot_dim;
  fs.rotary_interleaved = rotary_interleaved; fs.mscale = mscale; fs.positions = positions;
  fs.faithful_rounding = faithful_rounding;
  fs.fp8_headroom = headroom;
  // (the remaining checks -- cache strides, chunk size, workspace -- are those of the attention entry point; the
  // head stride of q is not used by the fused kernels)
  return launch_paged_decode(q, q_stride_tok, head_dim, k_cache, v_cache, kv_stride_chunk, kv_stride_tok, kv_stride_head,
                             block_table, bt_stride, kv_lens, nullptr, out, o_stride_tok, o_stride_head, workspace,
                             workspace_bytes, R, Hq, Hkv, head_dim, chunk_tokens, split_tokens, softmax_scale,
                             kv_dtype, k_scales, v_scales, dtype, tune, stream, &fs);
}

extern "C" int mi_decode_step_attention(
    const void* q, int64_t q_stride_tok, int64_t q_stride_group, const void* k_new, int64_t k_stride_tok,
    int64_t k_stride_head, const void* v_new, int64_t v_stride_tok, int64_t v_stride_head, const void* q_weight,
    const void* k_weight, float eps, int32_t norm_kind, const float* rotary_angles, int64_t angles_stride,
    int32_t rot_dim, int32_t rotary_interleaved, float mscale, const int64_t* positions, void* k_cache, void* v_cache,
    int64_t kv_stride_chunk, int64_t kv_stride_tok, int64_t kv_stride_head, const int32_t* block_table,
    int64_t bt_stride, const int32_t* kv_lens, void* out, int64_t o_stride_tok, int64_t o_stride_head, void* workspace,
    int64_t workspace_bytes, int32_t R, int32_t Hq, int32_t Hkv, int32_t head_dim, int32_t chunk_tokens,
    int32_t split_tokens, float softmax_scale, int32_t faithful_rounding, int32_t dtype, const MiTuning* tuning,
    void* stream) {
  return decode_step_entry("mi_decode_step_attention", q, q_stride_tok, q_stride_group, k_new, k_stride_tok, k_stride_head,
                           v_new, v_stride_tok, v_stride_head, q_weight, k_weight, eps, norm_kind, rotary_angles,
                           angles_stride, rot_dim, rotary_interleaved, mscale, positions, k_cache, v_cache, kv_stride_chunk,
                           kv_stride_tok, kv_stride_head, block_table, bt_stride, kv_lens, out, o_stride_tok, o_stride_head,
                           workspace, workspace_bytes, R, Hq, Hkv, head_dim, chunk_tokens, split_tokens, softmax_scale,
                           faithful_rounding, dtype, tuning, stream, MI_KV_16BIT, nullptr, nullptr, 1.f);
}

extern "C" int mi_decode_step_attention_fp8(
    const void* q, int64_t q_stride_tok, int64_t q_stride_group, const void* k_new, int64_t k_stride_tok,
    int64_t k_stride_head, const void* v_new, int64_t v_stride_tok, int64_t v_stride_head, const void* q_weight,
    const void* k_weight, float eps, int32_t norm_kind, const float* rotary_angles, int64_t angles_stride,
    int32_t rot_dim, int32_t rotary_interleaved, float mscale, const int64_t* positions, void* k_cache_fp8,
    void* v_cache_fp8, int64_t kv_stride_chunk, int64_t kv_stride_tok, int64_t kv_stride_head, float* k_scales,
    float* v_scales, float headroom, const int32_t* block_table, int64_t bt_stride, const int32_t* kv_lens, void* out,
    int64_t o_stride_tok, int64_t o_stride_head, void* workspace, int64_t workspace_bytes, int32_t R, int32_t Hq,
    int32_t Hkv, int32_t head_dim, int32_t chunk_tokens, int32_t split_tokens, float softmax_scale,
    int32_t faithful_rounding, int32_t dtype, const MiTuning* tuning, void* stream) {
  return decode_step_entry("mi_decode_step_attention_fp8", q, q_stride_tok, q_stride_group, k_new, k_stride_tok,
                           k_stride_head, v_new, v_stride_tok, v_stride_head, q_weight, k_weight, eps, norm_kind,
                           rotary_angles, angles_stride, rot_dim, rotary_interleaved, mscale, positions, k_cache_fp8,
                           v_cache_fp8, kv_stride_chunk, kv_stride_tok, kv_stride_head, block_table, bt_stride, kv_lens, out,
                           o_stride_tok, o_stride_head, workspace, workspace_bytes, R, Hq, Hkv, head_dim, chunk_tokens,
                           split_tokens, softmax_scale, faithful_rounding, dtype, tuning, stream, MI_KV_FP8_E4M3,
                           k_scales, v_scales, headroom);
}

// ---------------------------------------------------------------------------------------------
// Decode attention for callers that cannot allocate (code under HIP graph capture, serving loops and
// harnesses that forbid hipMalloc): the partials and the per-request segment records live in a
// file-scope device array instead of a caller workspace.  Every GPU the library runs on holds its own
// copy of the array until the process ends; `scratch` below is only the host-side stand-in of the
// symbol, so its device address is looked up once per device and only that address is ever handed to
// a kernel.
// ---------------------------------------------------------------------------------------------
namespace {
constexpr int64_t kNoAllocScratchBytes = (int64_t)MI_NOALLOC_SCRATCH_BYTES;
}
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];
static std::atomic<void*> g_scratch_ptr[64];  // per device: address of that device's copy of `scratch`

static int noalloc_scratch(void** out) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64)
    return mi_fail(MI_ERR_LAUNCH, "mi_paged_decode_attention_noalloc: cannot identify the current device");
  void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!ptr) {  // first call on this device (several host threads may race here: they all get the same address)
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      (void)hipGetLastError();
      return mi_fail(MI_ERR_LAUNCH, "mi_paged_decode_attention_noalloc: hipGetSymbolAddress(scratch) failed");
    }
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);
  }
  *out = ptr;
  return MI_OK;
}

extern "C" int mi_paged_decode_attention_noalloc(
    const void* q, int64_t q_stride_tok, int64_t q_stride_head, const void* k_cache,
    const void* v_cache, int64_t kv_stride_chunk, int64_t kv_stride_tok, int64_t kv_stride_head,
    const int32_t* block_table, int64_t bt_stride, const int32_t* kv_lens, void* out,
    int64_t o_stride_tok, int64_t o_stride_head, int32_t R, int32_t Hq, int32_t Hkv, int32_t head_dim,
    int32_t chunk_tokens, int32_t max_kv_len, int32_t split_tokens, float softmax_scale, int32_t kv_dtype,
    const float* k_scales, const float* v_scales, int32_t dtype, const MiTuning* tuning, void* stream) {
  (void)max_kv_len;
  MiTuning tune;
  const int rc_t = mi_resolve_tuning(tuning, &tune, "mi_paged_decode_attention_noalloc");
  if (rc_t != MI_OK) return rc_t;
  if (R > 0 && Hq > 0 && Hkv > 0 && head_dim > 0 &&
      mi_decode_workspace_bytes(R, Hq, Hkv, head_dim, chunk_tokens, max_kv_len, split_tokens, tuning) > kNoAllocScratchBytes)
    return mi_fail(MI_ERR_WORKSPACE,
                   "mi_paged_decode_attention_noalloc: these sizes need more than the 16 MiB of built-in scratch "
                   "(see mi_decode_workspace_bytes); use mi_paged_decode_attention with a workspace");
  // a timed launch takes an event pair from a pool that grows by creating events: not for this entry point
  if (mi_profile_is_on())
    return mi_fail(MI_ERR_UNSUPPORTED,
                   "mi_paged_decode_attention_noalloc: kernel timing is on (mi_profile_enable), and timed launches "
                   "may create events; switch it off for callers that must not allocate");
  void* ptr = nullptr;
  const int rc = noalloc_scratch(&ptr);
  if (rc != MI_OK) return rc;
  // Nothing in the scratch has to start at zero: every partial, log-sum-exp and segment record the merge
  // kernel reads was written by the streaming kernel of the same call, so the previous call's contents
  // (a larger batch's, say) are never looked at.
  return launch_paged_decode(q, q_stride_tok, q_stride_head, k_cache, v_cache, kv_stride_chunk, kv_stride_tok,
                             kv_stride_head, block_table, bt_stride, kv_lens, nullptr, out, o_stride_tok,
                             o_stride_head, ptr, kNoAllocScratchBytes, R, Hq, Hkv, head_dim, chunk_tokens,
                             split_tokens, softmax_scale, kv_dtype, k_scales, v_scales, dtype, tune, stream);
}

// ---------------------------------------------------------------------------------------------
// Multi-latent attention (absorbed decode): one shared latent row per token, every query head
// attends to it.  The streaming kernel sees the 16-head query groups as "KV heads" whose cache
// head stride is zero, and is handed the same buffer as key and value cache.
// ---------------------------------------------------------------------------------------------
namespace mi {
// query groups (wavefronts) per workgroup: at most four, one per SIMD
static int mla_waves_per_block(int groups) {
  for (int w = 4; w >= 1; --w)
    if (groups % w == 0) return w;
  return 1;
}
// spans along the flattened tile sequence: four wavefronts on every CU in total
static int mla_grid_size(int groups, const MiTuning& tune) {
  const int forced = tune.decode_grid;
  if (forced > 0) return forced;
  const int grid = device_cu_count() * 4 / groups;
  return grid < 1 ? 1 : grid;
}
static int mla_groups(int Hq) { return Hq <= 16 ? 1 : Hq / 16; }
// the 128-heads-per-workgroup kernel: one workgroup per CU, Hq / 128 of them per span
static bool mla_heads_kernel_shape(int Hq, int chunk_tokens) { return Hq % 128 == 0 && chunk_tokens % kMlaHeadsTile == 0; }
static int mla_heads_grid_size(int Hq, const MiTuning& tune) {
  if (tune.decode_grid > 0) return tune.decode_grid;
  const int grid = device_cu_count() / (Hq / 128);
  return grid < 1 ? 1 : grid;
}
}  // namespace mi

extern "C" int64_t mi_mla_decode_workspace_bytes(int32_t R, int32_t Hq, int32_t head_dim_v, const MiTuning* tuning) {
  if (R <= 0 || Hq <= 0 || head_dim_v <= 0) return 0;
  MiTuning tune;
  if (mi_resolve_tuning(tuning, &tune, "mi_mla_decode_workspace_bytes") != MI_OK) return -1;
  // (the largest grid any of the kernels may take for this head count: enough for each of them)
  int grid = mla_grid_size(mla_groups(Hq), tune);
  if (Hq % 128 == 0 && mla_heads_grid_size(Hq, tune) > grid) grid = mla_heads_grid_size(Hq, tune);
  const int64_t slots = (int64_t)grid + R;
  return slots * Hq * (head_dim_v + 1) * (int64_t)sizeof(float) + (int64_t)R * 2 * sizeof(int32_t);
}

extern "C" int mi_paged_mla_decode_attention(
    const void* q, int64_t q_stride_tok, int64_t q_stride_head, const void* kv_cache, int64_t kv_stride_chunk,
    int64_t kv_stride_tok, const int32_t* block_table, int64_t bt_stride, const int32_t* kv_lens, void* out,
    int64_t o_stride_tok, int64_t o_stride_head, void* workspace, int64_t workspace_bytes, int32_t R, int32_t Hq,
    int32_t head_dim_k, int32_t head_dim_v, int32_t chunk_tokens, int32_t max_kv_len, float softmax_scale,
    int32_t dtype, const MiTuning* tuning, void* stream) {
  (void)max_kv_len;
  if (R == 0) return MI_OK;
  if (dtype != MI_DTYPE_BF16 && dtype != MI_DTYPE_FP16)
    return mi_fail(MI_ERR_UNSUPPORTED, "mi_paged_mla_decode_attention: dtype must be MI_DTYPE_BF16 or MI_DTYPE_FP16");
  const bool f16 = dtype == MI_DTYPE_FP16;
  MiTuning tune;
  const int rc_t = mi_resolve_tuning(tuning, &tune, "mi_paged_mla_decode_attention");
  if (rc_t != MI_OK) return rc_t;
  if (!q || !kv_cache || !block_table || !kv_lens || !out)
    return mi_fail(MI_ERR_NULL, "mi_paged_mla_decode_attention: null pointer argument");
  if (R < 0 || Hq <= 0) return mi_fail(MI_ERR_SHAPE, "mi_paged_mla_decode_attention: need R >= 0 and Hq > 0");
  if (head_dim_k != 576 || head_dim_v != 512)
    return mi_fail(MI_ERR_UNSUPPORTED, "mi_paged_mla_decode_attention: latent rows of 576 values (512 + 64) only");
  if ((Hq > 16 && Hq % 16) || (Hq < 16 && (Hq & (Hq - 1))))
    return mi_fail(MI_ERR_UNSUPPORTED, "mi_paged_mla_decode_attention: Hq must be 1, 2, 4, 8 or a multiple of 16");
  if (chunk_tokens <= 0 || chunk_tokens % 16)
    return mi_fail(MI_ERR_SHAPE, "mi_paged_mla_decode_attention: chunk size must be a positive multiple of 16");
  if (((uintptr_t)q | (uintptr_t)kv_cache | (uintptr_t)out) & 15)
    return mi_fail(MI_ERR_ALIGN, "mi_paged_mla_decode_attention: q / cache / out must be 16-byte aligned");
  if ((q_stride_tok | q_stride_head | o_stride_tok | o_stride_head | kv_stride_chunk | kv_stride_tok) % 8)
    return mi_fail(MI_ERR_ALIGN, "mi_paged_mla_decode_attention: strides must keep rows 16-byte aligned");
  if (kv_stride_tok < head_dim_k || kv_stride_tok * (int64_t)chunk_tokens * 2 >= (int64_t)1 << 31)
    return mi_fail(MI_ERR_SHAPE, "mi_paged_mla_decode_attention: bad token stride, or a chunk of 2 GiB or more");
  if (!(softmax_scale > 0.f)) return mi_fail(MI_ERR_SHAPE, "mi_paged_mla_decode_attention: softmax_scale must be positive");
  if (R > kMaxRequestsPerLaunch) {  // slices, as in launch_paged_decode
    if (!workspace || workspace_bytes < mi_mla_decode_workspace_bytes(kMaxRequestsPerLaunch, Hq, head_dim_v, tuning))
      return mi_fail(MI_ERR_WORKSPACE, "mi_paged_mla_decode_attention: workspace too small (see mi_mla_decode_workspace_bytes)");
    for (int r0 = 0; r0 < R; r0 += kMaxRequestsPerLaunch) {
      const int n = R - r0 < kMaxRequestsPerLaunch ? R - r0 : kMaxRequestsPerLaunch;
      const int rc = mi_paged_mla_decode_attention(
          (const uint16_t*)q + (int64_t)r0 * q_stride_tok, q_stride_tok, q_stride_head, kv_cache, kv_stride_chunk,
          kv_stride_tok, block_table + (int64_t)r0 * bt_stride, bt_stride, kv_lens + r0,
          (uint16_t*)out + (int64_t)r0 * o_stride_tok, o_stride_tok, o_stride_head, workspace, workspace_bytes, n, Hq,
          head_dim_k, head_dim_v, chunk_tokens, max_kv_len, softmax_scale, dtype, tuning, stream);
      if (rc != MI_OK) return rc;
    }
    return MI_OK;
  }

  const int groups = mla_groups(Hq);
  // Two kernels: the latent tile shared through LDS by the eight wavefronts of a workgroup (needs tiles
  // of 64 tokens that do not straddle chunks), or one wavefront per head group streaming on its own.
  const size_t lds_head = ((size_t)R * 2 * sizeof(int32_t) + 15) & ~(size_t)15;
  const size_t lds_shared = lds_head + (size_t)2 * kMlaTile * kMlaPitch + 8 * 1024;  // tiles + partial scores
  const bool shared_tile = chunk_tokens % kMlaTile == 0 && tune.mla_decode_lds > 0 && lds_shared <= 160 * 1024;
  const int parts = (groups % 2 == 0) ? 4 : 8;            // output-column parts per head group
  const int wg_y = shared_tile ? groups / (8 / parts) : 0;  // workgroups per span (shared-tile kernel)
  // Multiples of 128 heads: four wavefronts with 32 heads each (mla_decode_lds = 2 keeps the kernel above)
  const size_t lds_heads = lds_head + (size_t)4 * kMlaHeadsBuf;
  const bool heads_tile = mla_heads_kernel_shape(Hq, chunk_tokens) && tune.mla_decode_lds == 1 && lds_heads <= 160 * 1024;
  int grid_x = mla_grid_size(groups, tune);
  if (heads_tile) {
    grid_x = mla_heads_grid_size(Hq, tune);
  } else if (shared_tile && tune.decode_grid <= 0) {
    grid_x = device_cu_count() / wg_y;
    if (grid_x < 1) grid_x = 1;
  }
  const int64_t slots = (int64_t)grid_x + R;
  const int64_t need = slots * Hq * (head_dim_v + 1) * (int64_t)sizeof(float) + (int64_t)R * 2 * sizeof(int32_t);
  if (!workspace || workspace_bytes < need)
    return mi_fail(MI_ERR_WORKSPACE, "mi_paged_mla_decode_attention: workspace too small (see mi_mla_decode_workspace_bytes)");
  if ((uintptr_t)workspace & 15)
    return mi_fail(MI_ERR_ALIGN, "mi_paged_mla_decode_attention: workspace must be 16-byte aligned");

  DecodeParams p;
  p.q = (const uint16_t*)q; p.q_st = q_stride_tok; p.q_sh = q_stride_head;
  p.kc = (const uint8_t*)kv_cache; p.vc = (const uint8_t*)kv_cache;  // value = first head_dim_v values of the row
  p.kv_sc = kv_stride_chunk; p.kv_st = (int32_t)kv_stride_tok; p.kv_sh = 0;
  p.bt = block_table; p.bt_stride = bt_stride; p.lens = kv_lens; p.cu_q = nullptr;
  p.out = (uint16_t*)out; p.o_st = o_stride_tok; p.o_sh = o_stride_head;
  p.part_o = (float*)workspace;
  p.part_lse = p.part_o + slots * Hq * head_dim_v;
  p.seg_info = (int32_t*)(p.part_lse + slots * Hq);
  p.k_scale = nullptr; p.v_scale = nullptr;
  p.R = R; p.Hq = Hq; p.Hkv = groups; p.G = Hq < 16 ? Hq : 16; p.parts = 1; p.chunk = chunk_tokens;
  p.chunk_magic = (((uint64_t)1 << 40) + chunk_tokens - 1) / chunk_tokens;
  p.min_span_tiles = heads_tile ? 64 / kMlaHeadsTile : shared_tile ? 64 / kMlaTile : 64 / 16;
  p.grid = grid_x;
  p.scale_log2 = softmax_scale * 1.4426950408889634f;

  hipStream_t st = (hipStream_t)stream;
  const int wpb = mla_waves_per_block(groups);
  const size_t lds = heads_tile ? lds_heads : shared_tile ? lds_shared : lds_head + (size_t)wpb * 16 * (576 * 2 + 16);
  if (lds > 160 * 1024)
    return mi_fail(MI_ERR_UNSUPPORTED, "mi_paged_mla_decode_attention: batch too large for the LDS of one workgroup");
  static std::atomic<bool> lds_limit_raised[64];  // per device: more than the default 64 KB of dynamic LDS
  int dev_id = 0;
  if (hipGetDevice(&dev_id) != hipSuccess || dev_id < 0 || dev_id >= 64) dev_id = 0;
  if (!lds_limit_raised[dev_id].load(std::memory_order_acquire)) {
    const hipFuncAttribute attr = hipFuncAttributeMaxDynamicSharedMemorySize;
    if (hipFuncSetAttribute((const void*)paged_mla_decode_stream_kernel<false>, attr, 160 * 1024) != hipSuccess ||
        hipFuncSetAttribute((const void*)paged_mla_decode_stream_kernel<true>, attr, 160 * 1024) != hipSuccess ||
        hipFuncSetAttribute((const void*)paged_mla_decode_lds_kernel<4, false>, attr, 160 * 1024) != hipSuccess ||
        hipFuncSetAttribute((const void*)paged_mla_decode_lds_kernel<4, true>, attr, 160 * 1024) != hipSuccess ||
        hipFuncSetAttribute((const void*)paged_mla_decode_lds_kernel<8, false>, attr, 160 * 1024) != hipSuccess ||
        hipFuncSetAttribute((const void*)paged_mla_decode_lds_kernel<8, true>, attr, 160 * 1024) != hipSuccess ||
        hipFuncSetAttribute((const void*)paged_mla_decode_heads_kernel<false>, attr, 160 * 1024) != hipSuccess ||
        hipFuncSetAttribute((const void*)paged_mla_decode_heads_kernel<true>, attr, 160 * 1024) != hipSuccess)
      return mi_fail(MI_ERR_LAUNCH, "mi_paged_mla_decode_attention: cannot raise the dynamic LDS limit");
    lds_limit_raised[dev_id].store(true, std::memory_order_release);
  }
  hipEvent_t ev_a, ev_b;
  const bool timed = mi_profile_next(&ev_a, &ev_b);
  if (timed) (void)hipEventRecord(ev_a, st);
#define MI_LAUNCH_MLA(F16_)                                                                                       \
  do {                                                                                                            \
    if (heads_tile)                                                                                               \
      hipLaunchKernelGGL((paged_mla_decode_heads_kernel<F16_>), dim3(grid_x, Hq / 128), dim3(256), lds, st, p);    \
    else if (shared_tile && parts == 4)                                                                           \
      hipLaunchKernelGGL((paged_mla_decode_lds_kernel<4, F16_>), dim3(grid_x, wg_y), dim3(512), lds, st, p);       \
    else if (shared_tile)                                                                                         \
      hipLaunchKernelGGL((paged_mla_decode_lds_kernel<8, F16_>), dim3(grid_x, wg_y), dim3(512), lds, st, p);       \
    else                                                                                                          \
      hipLaunchKernelGGL((paged_mla_decode_stream_kernel<F16_>), dim3(grid_x, groups / wpb), dim3(64 * wpb), lds, st, p); \
  } while (0)
  if (f16) MI_LAUNCH_MLA(true); else MI_LAUNCH_MLA(false);
#undef MI_LAUNCH_MLA
  if (timed) (void)hipEventRecord(ev_b, st);
  launch_merge(p, grid_x, R, Hq, 512, f16, st);
  return mi_check_launch("mi_paged_mla_decode_attention");
}
