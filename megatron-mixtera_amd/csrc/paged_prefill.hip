// Paged varlen causal attention for chunked prefill and mixed prefill+decode
// batches on gfx950.
//
// Replaces flash_attn_varlen_func(q, k_cache, v_cache, cu_seqlens_q, cu_seqlens_k,
// max_seqlen_q, max_seqlen_k, softmax_scale, causal=True, block_table=...)
// as called from Attention.flash_decode_and_prefill
// (megatron/core/transformer/attention.py:546-557).  The new tokens' K/V are
// already in the paged cache (append runs first), so keys are only ever read
// through the block table.  Mask: query i (0-based among the request's Lq new
// tokens) sees keys j <= i + (Lk - Lq).
//
// A wavefront owns 64 "rows" = (64/G query tokens) x (G query heads of one KV
// head) and walks the keys 16 at a time with the same matrix-core scheme as the
// decode kernel, reusing every K / V fragment for four 16-row tiles:
//   S^T[tok][row] = K . Q^T   (mfma 16x16x32),   O^T[d][row] += V^T . P^T (16x16x16).
// The four waves of a workgroup take four consecutive query blocks of the same
// (request, KV head), so they pull identical K/V lines at about the same time.
#include "mi_common.h"
#include "mi_capi_internal.h"
#include "paged_prefill_params.h"

namespace mi {

// NQ = 16-row tiles per wave, WAVES wavefronts per workgroup (256 rows for the narrow heads, 128 at width 256).
// HDK = width of queries and keys, HDV = width of values and of the output (they differ for the
// decompressed caches of multi-latent attention: 192 / 128); the value cache has its own strides.
template <int HDK, int HDV, int NT, int NQ, bool F16, int WAVES = 16 / NQ>
__global__ __launch_bounds__(64 * WAVES) void paged_prefill_kernel(PrefillParams p) {
  constexpr int KS = HDK / 32;
  constexpr int DV = HDV / 16;
  constexpr int VD = DV / 2;  // dwords per token and lane of the value operand

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int m16 = lane & 15, g = lane >> 4;
  const HeadSlice hs = head_slice(p, blockIdx.y);
  const int h = hs.h, G = hs.G, g_magic = hs.g_magic, hq0 = hs.hq0;
  // (the same for every head slice of a launch: the request -> workgroup map depends on it)
  const int BQ = ((16 * NQ) * p.g_magic) >> 16;  // query tokens per wave
  const int SBQ = WAVES * BQ;             // query tokens per workgroup

  // Rows beyond the last request (token padding of the batch) are defined as zeros; the first
  // workgroup of every KV head clears its heads of those rows.
  if (blockIdx.x == 0) {
    const int tq = p.cu_q[p.R];
    const int per_row = G * HDV;  // contiguous elements of this head group in one row
    for (int64_t i = (int64_t)threadIdx.x * 8; i < (int64_t)(p.T - tq) * per_row; i += 64 * WAVES * 8) {
      const int row = (int)(i / per_row), e = (int)(i - (int64_t)row * per_row);
      st16(p.out + (int64_t)(tq + row) * p.o_st + (int64_t)(hq0 + e / HDV) * p.o_sh + (e % HDV), make_uint4(0, 0, 0, 0));
    }
  }

  // ---- which request does this workgroup belong to? ----------------------------
  // Request r's workgroups start at pbs(r) = cu_q[r] / SBQ + r, a strictly
  // increasing sequence that leaves at least ceil(Lq_r / SBQ) indices to r.
  const int sb = blockIdx.x;
  int lo = 0, hi = p.R - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (p.cu_q[mid] / SBQ + mid <= sb) lo = mid; else hi = mid - 1;
  }
  const int r = lo;
  const int q_begin = p.cu_q[r];
  const int Lq = p.cu_q[r + 1] - q_begin;
  const int q0 = (sb - (q_begin / SBQ + r)) * SBQ + wave * BQ;  // first query of this wave
  if (q0 >= Lq) return;
  if (p.skip_single && Lq == 1) return;
  const int Lk = p.lens[r];
  const int shift = Lk - Lq;  // key position of query 0
  const int nq = min(BQ, Lq - q0);
  const int kend = min(Lk, shift + q0 + nq);  // keys [0, kend) are visible to some row
  const int last = Lk - 1;

  // ---- query fragments and per-row causal limits ---------------------------------
  uint4 qf[NQ][KS];
  int qpos[NQ];
#pragma unroll
  for (int nt = 0; nt < NQ; ++nt) {
    const int n = 16 * nt + m16;
    const int qi = (n * g_magic) >> 16, u = n - qi * G;  // n / G, n % G
    const bool valid = qi < nq;
    qpos[nt] = valid ? shift + q0 + qi : last;
    const uint16_t* qrow = p.q + (int64_t)(q_begin + q0 + qi) * p.q_st + (int64_t)(hq0 + u) * p.q_sh;
#pragma unroll
    for (int kk = 0; kk < KS; ++kk)
      qf[nt][kk] = valid ? ld16(qrow + 32 * kk + 8 * g) : make_uint4(0, 0, 0, 0);
  }
  const int ntiles = (nq * G + 15) >> 4;  // 16-row tiles that hold a valid row

  const uint8_t* kbase = p.kc + (int64_t)h * p.kv_sh * 2;
  const uint8_t* vbase = p.vc + (int64_t)h * p.v_sh * 2;
  const int64_t chunk_bytes = p.kv_sc * 2;
  const int tok_bytes = p.kv_st * 2;
  const int64_t v_chunk_bytes = p.v_sc * 2;
  const int v_tok_bytes = p.v_st * 2;

  float m_run[NQ], l_run[NQ];
  f32x4_t acc[NQ][DV];
#pragma unroll
  for (int nt = 0; nt < NQ; ++nt) {
    m_run[nt] = -INFINITY;
    l_run[nt] = 0.f;
#pragma unroll
    for (int e = 0; e < DV; ++e) acc[nt][e] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }

  if (kend <= 0) {
    // No visible key (Lk == 0): rows are defined as zeros.
#pragma unroll
    for (int nt = 0; nt < NQ; ++nt) {
      const int n = 16 * nt + m16;
      const int qi = (n * g_magic) >> 16, u = n - qi * G;  // n / G, n % G
      if (qi < nq) {
        uint16_t* o = p.out + (int64_t)(q_begin + q0 + qi) * p.o_st + (int64_t)(hq0 + u) * p.o_sh + 4 * DV * g;
        for (int i = 0; i < 4 * DV; i += 2) *reinterpret_cast<uint32_t*>(o + i) = 0u;
      }
    }
    return;
  }

  // K / V staging registers of one tile of 16*NT keys; the loop is software pipelined on them
  // (K of the next tile is requested once all scores of this one exist, V once P.V is done).
  uint4 kf[NT][KS];
  uint32_t vf[NT][4][VD];
  auto load_k = [&](int T) {
#pragma unroll
    for (int u = 0; u < NT; ++u) {
      const int T0 = T + 16 * u;
      const int tu = min(T0, last);
      const int ci = (int)(((uint64_t)(uint32_t)tu * p.chunk_magic) >> 40);
      const int pc = p.bt[(int64_t)r * p.bt_stride + ci];
      const uint8_t* krow = kbase + (int64_t)pc * chunk_bytes + (min(T0 + m16, last) - ci * p.chunk) * tok_bytes;
#pragma unroll
      for (int kk = 0; kk < KS; ++kk) kf[u][kk] = ld16(krow + (32 * kk + 8 * g) * 2);
    }
  };
  auto load_v = [&](int T) {
#pragma unroll
    for (int u = 0; u < NT; ++u) {
      const int T0 = T + 16 * u;
      const int tu = min(T0, last);
      const int ci = (int)(((uint64_t)(uint32_t)tu * p.chunk_magic) >> 40);
      const int pc = p.bt[(int64_t)r * p.bt_stride + ci];
      const uint8_t* vc = vbase + (int64_t)pc * v_chunk_bytes;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint8_t* vrow = vc + (min(T0 + 4 * g + j, last) - ci * p.chunk) * v_tok_bytes + DV * m16 * 2;
        ld_dwords(vrow, vf[u][j]);
      }
    }
  };

  // Keys up to and including `full_until` are visible to every valid row of this wave, so a
  // tile that ends there needs no masking.
  const int full_until = shift + q0;
  const float scale = p.scale_log2;

  load_k(0);
  load_v(0);
  __builtin_amdgcn_sched_barrier(0);
  for (int T = 0; T < kend; T += 16 * NT) {
    // ---- S^T = K Q^T for every 16-row tile of the wave (raw, unscaled) ----------------
    f32x4_t s[NQ][NT];
#pragma unroll
    for (int nt = 0; nt < NQ; ++nt) {
      if (nt >= ntiles) break;  // wave-uniform
#pragma unroll
      for (int u = 0; u < NT; ++u) {
        f32x4_t sacc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) sacc = mfma_16x16x32<F16>(kf[u][kk], qf[nt][kk], sacc);
        s[nt][u] = sacc;
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    load_k(T + 16 * NT);
    __builtin_amdgcn_sched_barrier(0);

    // ---- online softmax per 16-row tile ----------------------------------------------
    const bool need_mask = T + 16 * NT - 1 > full_until;  // wave-uniform
    uint2 pf[NQ][NT];
#pragma unroll
    for (int nt = 0; nt < NQ; ++nt) {
      if (nt >= ntiles) break;
      float tmax = -INFINITY;
#pragma unroll
      for (int u = 0; u < NT; ++u) {
        if (need_mask) {
          const int tok0 = T + 16 * u + 4 * g;
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (tok0 + i > qpos[nt]) s[nt][u][i] = -INFINITY;
        }
        tmax = fmaxf(fmaxf(fmaxf(s[nt][u][0], s[nt][u][1]), fmaxf(s[nt][u][2], s[nt][u][3])), tmax);
      }
      tmax = fmaxf(tmax, xor16(tmax));
      tmax = fmaxf(tmax, xor32(tmax));
      // Key 0 is visible to every row of a well-formed request (Lk >= Lq), so m_run is finite
      // after the first tile; a row with no visible key so far keeps m_run = -inf and p = 0.
      const float m_raw = fmaxf(m_run[nt], tmax);
      const float m_use = m_raw == -INFINITY ? 0.f : m_raw;
      const float alpha = fast_exp2((m_run[nt] - m_use) * scale);
      const float neg = -m_use * scale;
      m_run[nt] = m_raw;
      float psum = 0.f;
#pragma unroll
      for (int u = 0; u < NT; ++u) {
        float pv[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          pv[i] = fast_exp2(__builtin_fmaf(s[nt][u][i], scale, neg));
          psum += pv[i];
        }
        pf[nt][u] = make_uint2(pack2<F16>(pv[0], pv[1]), pack2<F16>(pv[2], pv[3]));
      }
      l_run[nt] = l_run[nt] * alpha + psum;
      // The running max rarely moves once a few tiles have been seen: skip the rescale of the
      // accumulators when no lane of the wave needs it.
      if (__builtin_amdgcn_ballot_w64(alpha != 1.f)) {
#pragma unroll
        for (int e = 0; e < DV; ++e) {
          acc[nt][e][0] *= alpha; acc[nt][e][1] *= alpha; acc[nt][e][2] *= alpha; acc[nt][e][3] *= alpha;
        }
      }
    }

    // ---- O^T += V^T P^T: each transposed V fragment serves all row tiles ---------------
    // Two 16-key sub-tiles are contracted by one mfma 16x16x32 (slots 0-3 = tokens 4g..4g+3 of
    // the first sub-tile, slots 4-7 = the same of the second; P is packed the same way).
    auto transpose_v = [&](int u, uint2 (&vt)[DV]) {
#pragma unroll
      for (int dw = 0; dw < VD; ++dw) {
        const uint32_t r0 = vf[u][0][dw], r1 = vf[u][1][dw], r2 = vf[u][2][dw], r3 = vf[u][3][dw];
        vt[2 * dw] = make_uint2(low_halves(r1, r0), low_halves(r3, r2));
        vt[2 * dw + 1] = make_uint2(high_halves(r1, r0), high_halves(r3, r2));
      }
    };
    if constexpr (NT % 2 == 0) {
#pragma unroll
      for (int u = 0; u < NT; u += 2) {
        uint2 va[DV], vb[DV];
        transpose_v(u, va);
        transpose_v(u + 1, vb);
#pragma unroll
        for (int nt = 0; nt < NQ; ++nt) {
          if (nt >= ntiles) break;
          const uint4 pp = make_uint4(pf[nt][u].x, pf[nt][u].y, pf[nt][u + 1].x, pf[nt][u + 1].y);
#pragma unroll
          for (int e = 0; e < DV; ++e)
            acc[nt][e] = mfma_16x16x32<F16>(make_uint4(va[e].x, va[e].y, vb[e].x, vb[e].y), pp, acc[nt][e]);
        }
      }
    } else {
#pragma unroll
      for (int u = 0; u < NT; ++u) {
        uint2 vt[DV];
        transpose_v(u, vt);
#pragma unroll
        for (int nt = 0; nt < NQ; ++nt) {
          if (nt >= ntiles) break;
#pragma unroll
          for (int e = 0; e < DV; ++e) acc[nt][e] = mfma_16x16x16<F16>(vt[e], pf[nt][u], acc[nt][e]);
        }
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    load_v(T + 16 * NT);
    __builtin_amdgcn_sched_barrier(0);
  }

#pragma unroll
  for (int nt = 0; nt < NQ; ++nt) {
    float l_tot = l_run[nt] + xor16(l_run[nt]);
    l_tot += xor32(l_tot);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    const int n = 16 * nt + m16;
    const int qi = (n * g_magic) >> 16, u = n - qi * G;  // n / G, n % G
    if (qi < nq) {
      uint16_t* o = p.out + (int64_t)(q_begin + q0 + qi) * p.o_st + (int64_t)(hq0 + u) * p.o_sh + 4 * DV * g;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        uint32_t ow[VD];
#pragma unroll
        for (int dw = 0; dw < VD; ++dw) ow[dw] = pack2<F16>(acc[nt][2 * dw][i] * inv, acc[nt][2 * dw + 1][i] * inv);
        st_dwords(o + DV * i, ow);
      }
    }
  }
}


// ---------------------------------------------------------------------------------------------
// Two-phase ("ping-pong") LDS-tiled kernel.
//
// A workgroup of 8 wavefronts takes 256 consecutive (query token, head-in-group) rows of one (request, KV head),
// 32 rows per wavefront; each 64-key K tile and V tile is fetched from memory once per workgroup (16 bytes per
// loader thread), staged row-major in LDS, and the wavefronts read their matrix operands from there.
// The per-tile work of a wave is split into a matrix phase  { O^T += V^T P^T of the previous tile,
// S^T = K Q^T of this tile }  and a vector phase  { online softmax of this tile, staging of the
// next tiles into LDS }.  The 8 waves form two groups of four (waves w and w+4 share a SIMD);
// every phase ends in a workgroup barrier and the second group runs one phase behind the first,
// so on every SIMD one wave is feeding the matrix cores while the other one runs the exp / max /
// convert chain.  Because the groups read a staged tile one phase apart, the first group stages
// one tile ahead of its own use and the second group two (see the table in the loop).
//
// V fragments come out of LDS already transposed (ds_read_b64_tr_b16, 288-byte V pitch), so there is no
// permute work; the softmax denominator is accumulated by the matrix cores (an all-ones A fragment), and
// the cross-lane maximum uses the lane-swap instructions instead of LDS permutes -- and is taken only when
// some score of a tile exceeds the reference of its row by a window (2^30 as the largest probability with bf16
// operands, 2^8 with fp16 ones): the exponentials are taken against a reference that rarely moves.
// ---------------------------------------------------------------------------------------------
// bytes per staged K / V row: the row width plus padding that makes the pitch an odd multiple of 8 banks (32 bytes).
// A 16-byte fragment read is served in passes of {rows 0-7 at piece g, rows 8-15 at piece g + 1}, a transposing
// 8-byte read in passes of eight rows; both cover the 64 banks exactly once at such a pitch (288 = 8 x 9 dwords
// reads 0 conflict cycles by counter; 4 x odd dwords -- 144 or 208, as head_dim 64 and 96 once had -- costs a
// fragment read 4 cycles on top of its 4 and a transposing read 2 on top of its 2).
// head_dim 64: 160 (8 x 5 dwords), 96: 224 (8 x 7), 128: 288, 192-wide keys: 416 (8 x 13), 256: 544 (8 x 17).
template <int HD> constexpr int pp_pitch() { return HD == 256 ? 544 : HD == 192 ? 416 : HD == 128 ? 288 : HD == 96 ? 224 : 160; }
// keys per staged tile: 64; 32 at head_dim 256, where five 64-key buffers would not fit the 160 KB of LDS
template <int HD> constexpr int pp_tile() { return HD == 256 ? 32 : 64; }

// FP8: the cache holds e4m3 bytes with one fp32 scale per (chunk, KV head); a piece is multiplied by
// its chunk's scale and rounded to bf16 on its way into LDS, so both matrix phases are the bf16 ones.
// SPLIT: the keys of a request are cut into gridDim.y ranges (a separate instantiation, so that the
// ordinary kernel carries no tile offsets).
// HD = width of values and output, HDK = width of queries and keys: equal, or 192 / 128 for the decompressed
// caches of multi-latent attention, whose value cache has its own strides.
template <bool STAGGER, bool FP8, bool SPLIT, int HD, int HDK, bool F16>
__global__ __launch_bounds__(512, 2) void paged_prefill_pp_kernel(PrefillParams p) {
  static_assert((HD == 128 && HDK == 128) || (HD == 64 && HDK == 64) ||
                    ((HD == 96 || HD == 192 || HD == 256) && HDK == HD && !FP8) || (HD == 128 && HDK == 192 && !FP8),
                "head_dim 64 or 128, or 96 / 192 / 256 with a 16-bit cache, or 192 / 128 with 16-bit caches");
  constexpr bool MLA = HDK != HD;
  // Wide heads (192, 256): 16 rows per wavefront instead of 32 -- the accumulators of 32 rows (96 / 128 registers)
  // plus query fragments (48 / 64) leave no room for the operand fragments in a wavefront's 256 registers.
  constexpr bool WIDE = HD >= 192;
  constexpr int kPPTile = pp_tile<HD>();
  constexpr int KS = HDK / 32, DV = HD / 16, NQ = WIDE ? 1 : 2, NT = kPPTile / 16, WAVES = 8;
  constexpr int kKPitch = pp_pitch<HDK>(), kVPitch = pp_pitch<HD>();
  constexpr int PPRK = HDK * 2 / 16;                 // 16-byte pieces per key row: 24 | 16 | 12 | 8
  constexpr int PPR = HD * 2 / 16;                   // 16-byte pieces (8 elements) per value row: 16 | 12 | 8
  // Rows of 16 or 8 pieces divide the 512 loader threads into whole rows (a thread keeps its piece index and
  // takes rows lkey, lkey + RPP); rows of 24 or 12 pieces do not: a thread then takes pieces tid, tid + 512, ...
  // of the tile's 64 * pieces-per-row, as far as they exist ("flat").
  constexpr bool FLAT_K = 512 % PPRK != 0, FLAT_V = 512 % PPR != 0;
  constexpr int NPK = (kPPTile * PPRK + 511) / 512;  // key pieces per loader thread and tile: 3 | 2 | 2 | 1
  constexpr int RPP = 512 / PPR;         // value rows the 512 loader threads cover in one pass: 32 | - | 64
  constexpr int NPASS = (kPPTile * PPR + 511) / 512;  // value pieces per loader thread and tile: 2 | 2 | 1
  constexpr int NH = HD == 64 ? 1 : WIDE ? HD / 64 : 2;   // column groups of the output: 64 + 64, 48 + 48, 64, or 3 / 4 x 64
  constexpr int EPG = HD / 16 / NH;      // 16-column blocks per group: 4 | 3 | 4
  constexpr int ESZ = FP8 ? 1 : 2;       // bytes per cache element
  constexpr int PIECE = FP8 ? 8 : 16;    // bytes one loader thread fetches of a row (8 elements)
  __shared__ __attribute__((aligned(16))) uint8_t Ks[2][kPPTile * kKPitch];
  __shared__ __attribute__((aligned(16))) uint8_t Vs[3][kPPTile * kVPitch];  // three: see the loop

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform values stay in SGPRs
  const int m16 = lane & 15, g = lane >> 4;
  const int lead = STAGGER ? (wave >> 2) : 0;  // 0: first group, 1: second group (one phase behind)
  const int HV = p.Hkv * p.parts;  // workgroups along the heads
  const HeadSlice hs = head_slice(p, blockIdx.x % HV);
  const int h = hs.h, G = hs.G, g_magic = hs.g_magic, hq0 = hs.hq0;
  const int rank = blockIdx.x / HV;
  // query tokens per workgroup: the same for every head slice of a launch (the request -> workgroup map
  // depends on it), i.e. the count of the widest slice; a narrower last slice leaves rows unused
  const int BQ = ((16 * NQ) * p.g_magic) >> 16;
  const int SBQ = WAVES * BQ;

  if (rank == 0 && (!SPLIT || blockIdx.y == 0)) {
    const int tq = p.cu_q[p.R];
    const int per_row = G * HD;
    for (int64_t i = (int64_t)tid * 8; i < (int64_t)(p.T - tq) * per_row; i += 512 * 8) {
      const int row = (int)(i / per_row), e = (int)(i - (int64_t)row * per_row);
      st16(p.out + (int64_t)(tq + row) * p.o_st + (int64_t)(hq0 + e / HD) * p.o_sh + (e % HD), make_uint4(0, 0, 0, 0));
    }
  }

  const int sb = (int)(gridDim.x / HV) - 1 - rank;
  int lo = 0, hi = p.R - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (p.cu_q[mid] / SBQ + mid <= sb) lo = mid; else hi = mid - 1;
  }
  const int r = lo;
  const int q_begin = p.cu_q[r];
  const int Lq = p.cu_q[r + 1] - q_begin;
  const int q0_wg = (sb - (q_begin / SBQ + r)) * SBQ;
  if (q0_wg >= Lq) return;  // workgroup-uniform
  if (p.skip_single && Lq == 1) return;
  const int Lk = p.lens[r];
  const int shift = Lk - Lq;
  const int last = Lk - 1;
  const int kend_wg = min(Lk, shift + min(q0_wg + SBQ, Lq));
  const int ntl_all = (kend_wg + kPPTile - 1) / kPPTile;  // staged tiles the rows of this workgroup can see
  // this workgroup's share of them: tiles [tb, tb + ntl)
  const int n_split = SPLIT ? (int)gridDim.y : 1, split = SPLIT ? (int)blockIdx.y : 0;
  const int tb = SPLIT ? (int)((int64_t)ntl_all * split / n_split) : 0;
  const int te = SPLIT ? (int)((int64_t)ntl_all * (split + 1) / n_split) : ntl_all;
  const int ntl = te - tb;

  const int q0 = q0_wg + wave * BQ;
  const int nq = max(0, min(BQ, Lq - q0));
  const int full_until = shift + q0;

  uint4 qf[NQ][KS];
  int qpos[NQ];
#pragma unroll
  for (int nt = 0; nt < NQ; ++nt) {
    const int n = 16 * nt + m16;
    const int qi = (n * g_magic) >> 16, u = n - qi * G;  // n / G, n % G
    const bool valid = qi < nq;
    qpos[nt] = valid ? shift + q0 + qi : last;
    const uint16_t* qrow = p.q + (int64_t)(q_begin + q0 + qi) * p.q_st + (int64_t)(hq0 + u) * p.q_sh;
#pragma unroll
    for (int kk = 0; kk < KS; ++kk)
      qf[nt][kk] = valid ? ld16(qrow + 32 * kk + 8 * g) : make_uint4(0, 0, 0, 0);
  }

  float m_run[NQ], neg_run[NQ];
  f32x4_t acc[NQ][DV], accl[NQ];
#pragma unroll
  for (int nt = 0; nt < NQ; ++nt) {
    m_run[nt] = -INFINITY;
    neg_run[nt] = 0.f;
    accl[nt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int e = 0; e < DV; ++e) acc[nt][e] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }

  if (ntl > 0) {
    const uint8_t* kbase = p.kc + (int64_t)h * p.kv_sh * ESZ;
    const uint8_t* vbase = p.vc + (int64_t)h * (MLA ? p.v_sh : p.kv_sh) * ESZ;
    const int64_t chunk_bytes = p.kv_sc * ESZ;
    const int tok_bytes = p.kv_st * ESZ;
    const int64_t v_chunk_bytes = MLA ? p.v_sc * ESZ : chunk_bytes;  // (value cache of its own: multi-latent only)
    const int v_tok_bytes = MLA ? p.v_st * ESZ : tok_bytes;
    // loader role: piece `lpiece` (8 elements) of key rows `lkey` and `lkey + 32` of a tile
    const int lkey = tid / PPR, lpiece = tid % PPR;
    const int k_off = lkey * kKPitch + lpiece * 16;
    const int v_off = lkey * kVPitch + lpiece * 16;
    uint4 kreg[NPK], vreg[NPASS];
    // Staged tiles never straddle a chunk (the launcher only picks this kernel when the chunk size
    // is a multiple of 64), so a tile is addressed by scalars only -- physical chunk, tile index
    // inside the chunk -- plus a per-lane row offset that is fixed for the whole kernel.  The
    // fetch cursor below walks the tiles with adds and compares instead of divisions; it stops
    // on the last tile, so the extra fetches and LDS stores at the end of the loop repeat that
    // tile into a buffer nobody reads any more, which keeps the loop free of branches.
    const int tiles_per_chunk = p.chunk / kPPTile;
    const int tile_bytes = kPPTile * tok_bytes;
    const int v_tile_bytes = kPPTile * v_tok_bytes;
    const uint32_t row_off0 = (uint32_t)(lkey * v_tok_bytes + lpiece * PIECE);
    const uint32_t row_off1 = row_off0 + (uint32_t)(RPP * v_tok_bytes);  // (second pass, head_dim 128 only)
    const uint32_t piece_off = (uint32_t)(lpiece * PIECE);
    // flat loader roles (a piece index past the tile's last repeats piece 0 and is not stored)
    uint32_t mk_row_off[NPK], mk_piece_off[NPK], mv_row_off[NPASS], mv_piece_off[NPASS];
    int mk_lds[NPK], mv_lds[NPASS];
    if constexpr (FLAT_K) {
#pragma unroll
      for (int i = 0; i < NPK; ++i) {
        const int idx = tid + 512 * i < kPPTile * PPRK ? tid + 512 * i : 0, row = idx / PPRK, piece = idx - row * PPRK;
        mk_row_off[i] = (uint32_t)(row * tok_bytes + piece * 16);
        mk_piece_off[i] = (uint32_t)(piece * 16);
        mk_lds[i] = row * kKPitch + piece * 16;
      }
    }
    if constexpr (FLAT_V) {
#pragma unroll
      for (int i = 0; i < NPASS; ++i) {
        const int idx = tid + 512 * i < kPPTile * PPR ? tid + 512 * i : 0, row = idx / PPR, piece = idx - row * PPR;
        mv_row_off[i] = (uint32_t)(row * v_tok_bytes + piece * 16);
        mv_piece_off[i] = (uint32_t)(piece * 16);
        mv_lds[i] = row * kVPitch + piece * 16;
      }
    }
    float ksc_staged = 1.f, vsc_staged = 1.f;  // fp8: scales of the tile held in kreg / vreg (per-lane copies)
    const int32_t* bt_row = p.bt + (int64_t)r * p.bt_stride;
    struct Cursor {   // all members are wave-uniform
      int tile;       // tile index
      int ci, tin;    // logical chunk of the tile and tile index inside the chunk
      int room;       // bytes from the tile's first row to the request's last row (>= 0)
      int room_v;     // the same in the value cache (multi-latent only)
    };
    auto cursor_at = [&](int t) {
      Cursor c;
      c.tile = min(t, te - 1);
      c.ci = c.tile / tiles_per_chunk;
      c.tin = c.tile - c.ci * tiles_per_chunk;
      c.room = (last - c.tile * kPPTile) * tok_bytes;
      c.room_v = MLA ? (last - c.tile * kPPTile) * v_tok_bytes : 0;
      return c;
    };
    auto cursor_next = [&](Cursor& c) {  // one tile forward, sticking to the last tile
      const bool adv = c.tile + 1 < te;
      const bool wrap = adv && (c.tin + 1 == tiles_per_chunk);
      c.tile += adv ? 1 : 0;
      c.room -= adv ? tile_bytes : 0;
      if constexpr (MLA) c.room_v -= adv ? v_tile_bytes : 0;
      c.tin = wrap ? 0 : c.tin + (adv ? 1 : 0);
      c.ci += wrap ? 1 : 0;
    };
    // fp8: the scales of a tile's chunk, requested when the tile's loads are issued
    auto tile_scales = [&](int pc) {
      if (FP8) {
        ksc_staged = p.k_scale[(int64_t)pc * p.Hkv + h];
        vsc_staged = p.v_scale[(int64_t)pc * p.Hkv + h];
      }
    };
    // byte offset of the cursor's tile inside a cache, given its physical chunk
    auto tile_offset = [&](const Cursor& c, int pc_lane) -> int64_t {
      const int pc = __builtin_amdgcn_readfirstlane(pc_lane);
      tile_scales(pc);
      return (int64_t)pc * chunk_bytes + (int64_t)c.tin * tile_bytes;
    };
    auto tile_offset_v = [&](const Cursor& c, int pc_lane) -> int64_t {
      const int pc = __builtin_amdgcn_readfirstlane(pc_lane);
      return (int64_t)pc * v_chunk_bytes + (int64_t)c.tin * v_tile_bytes;
    };
    // this thread's two pieces of a tile (rows past the request's last key re-read the last row,
    // which every query row masks)
    auto tile_loads = [&](const uint8_t* base, int64_t off, int room, uint4 (&reg)[NPASS]) {
      const uint8_t* tb = base + off;
      const uint32_t lim = (uint32_t)room + piece_off;
      if constexpr (FP8) {
        const uint2 a = ld8(tb + min(row_off0, lim));
        reg[0] = make_uint4(a.x, a.y, 0u, 0u);
        if constexpr (NPASS == 2) {
          const uint2 b = ld8(tb + min(row_off1, lim));
          reg[1] = make_uint4(b.x, b.y, 0u, 0u);
        }
      } else {
        reg[0] = ld16(tb + min(row_off0, lim));
        if constexpr (NPASS == 2) reg[1] = ld16(tb + min(row_off1, lim));
      }
    };
    auto tile_loads_k = [&](int64_t off, int room) {
      if constexpr (FLAT_K) {
        const uint8_t* tb = kbase + off;
#pragma unroll
        for (int i = 0; i < NPK; ++i) kreg[i] = ld16(tb + min(mk_row_off[i], (uint32_t)room + mk_piece_off[i]));
      } else {
        tile_loads(kbase, off, room, kreg);
      }
    };
    auto tile_loads_v = [&](int64_t off, int room) {
      if constexpr (FLAT_V) {
        const uint8_t* tb = vbase + off;
#pragma unroll
        for (int i = 0; i < NPASS; ++i) vreg[i] = ld16(tb + min(mv_row_off[i], (uint32_t)room + mv_piece_off[i]));
      } else {
        tile_loads(vbase, off, room, vreg);
      }
    };
    // what goes into LDS for one staged piece: the bf16 bits, or (fp8) 8 bytes -> 8 bf16 of byte * scale
    auto lds_piece = [&](uint4 raw, float scale) {
      if (!FP8) return raw;
      const f32x2_t a = fp8x2_lo_to_f32(raw.x), b = fp8x2_hi_to_f32(raw.x);
      const f32x2_t c = fp8x2_lo_to_f32(raw.y), d = fp8x2_hi_to_f32(raw.y);
      return make_uint4(pack2<F16>(a.x * scale, a.y * scale), pack2<F16>(b.x * scale, b.y * scale),
                        pack2<F16>(c.x * scale, c.y * scale), pack2<F16>(d.x * scale, d.y * scale));
    };
    auto store_k = [&](int t) {
      if constexpr (FLAT_K) {
#pragma unroll
        for (int i = 0; i < NPK; ++i)
          if (tid + 512 * i < kPPTile * PPRK) *reinterpret_cast<uint4*>(&Ks[t & 1][mk_lds[i]]) = kreg[i];
        return;
      }
      uint8_t* dst = &Ks[t & 1][k_off];
      *reinterpret_cast<uint4*>(dst) = lds_piece(kreg[0], ksc_staged);
      if constexpr (NPASS == 2) *reinterpret_cast<uint4*>(dst + RPP * kKPitch) = lds_piece(kreg[1], ksc_staged);
    };
    auto vbuf = [](int t) { return (unsigned)(t + 3) % 3u; };  // tile -1 lives in buffer 2
    auto store_v = [&](int t) {
      if constexpr (FLAT_V) {
#pragma unroll
        for (int i = 0; i < NPASS; ++i)
          if (tid + 512 * i < kPPTile * PPR) *reinterpret_cast<uint4*>(&Vs[vbuf(t)][mv_lds[i]]) = vreg[i];
        return;
      }
      uint8_t* dst = &Vs[vbuf(t)][v_off];
      *reinterpret_cast<uint4*>(dst) = lds_piece(vreg[0], vsc_staged);
      if constexpr (NPASS == 2) *reinterpret_cast<uint4*>(dst + RPP * kVPitch) = lds_piece(vreg[1], vsc_staged);
    };

    const float scale = p.scale_log2;
    const float win = (F16 ? 8.f : 30.f) / scale;  // probabilities stay below 2^8 (fp16 operands) or 2^30
    const uint4 ones = make_uint4(ones2<F16>(), ones2<F16>(), ones2<F16>(), ones2<F16>());
    f32x4_t s[NQ][NT];
    uint2 pf[NQ][NT];
    // fixed per-lane offsets of the fragment reads
    const int kfrag_off = m16 * kKPitch + 16 * g;
    const int vfrag_off = (4 * g + (m16 >> 2)) * kVPitch + 8 * (m16 & 3);

    // ---- matrix phase pieces.  The work is cut into groups of 8-10 MFMAs; the LDS reads of a
    // group are issued before the MFMAs of the previous group (scheduling barriers keep that
    // order), so a read has ~130 cycles of matrix work to hide behind and only two groups of
    // fragments are live at a time.
    // S^T = K Q^T: group u = 16-key sub-tile u (KS K fragments, 2 KS MFMAs)
    auto sc_load = [&](int t, int u, uint4 (&kf)[KS]) {
      const uint8_t* ks = Ks[t & 1] + kfrag_off + 16 * u * kKPitch;
#pragma unroll
      for (int kk = 0; kk < KS; ++kk) kf[kk] = *reinterpret_cast<const uint4*>(ks + 64 * kk);
    };
    auto sc_mma = [&](int u, const uint4 (&kf)[KS]) {
#pragma unroll
      for (int nt = 0; nt < NQ; ++nt) s[nt][u] = mfma_16x16x32<F16>(kf[0], qf[nt][0], f32x4_t{0.f, 0.f, 0.f, 0.f});
#pragma unroll
      for (int kk = 1; kk < KS; ++kk) {
#pragma unroll
        for (int nt = 0; nt < NQ; ++nt) s[nt][u] = mfma_16x16x32<F16>(kf[kk], qf[nt][kk], s[nt][u]);
      }
    };
    // 192-wide keys: a sub-tile's product in two halves of three fragments (half the fragment registers)
    auto sc_load_half = [&](int t, int u, int half, uint4 (&kf)[3]) {
      const uint8_t* ks = Ks[t & 1] + kfrag_off + 16 * u * kKPitch + 192 * half;
#pragma unroll
      for (int j = 0; j < 3; ++j) kf[j] = *reinterpret_cast<const uint4*>(ks + 64 * j);
    };
    auto sc_mma_half = [&](int u, int half, const uint4 (&kf)[3]) {
#pragma unroll
      for (int j = 0; j < 3; ++j) {
        const int kk = 3 * half + j;
#pragma unroll
        for (int nt = 0; nt < NQ; ++nt)
          s[nt][u] = mfma_16x16x32<F16>(kf[j], qf[nt][kk % KS], kk == 0 ? f32x4_t{0.f, 0.f, 0.f, 0.f} : s[nt][u]);
      }
    };
    // O^T += V^T P^T: group grp = (32-key step grp / NH, output column group grp % NH of 64 or 48 columns):
    // 8 (6) transposed reads, 8 (6) MFMAs (+2 for the denominators in the last group of a step)
    auto pv_load = [&](int t, int grp, uint2 (&af)[4][2]) {
      const uint8_t* vs = Vs[vbuf(t)] + vfrag_off + 32 * (grp / NH) * kVPitch + 32 * EPG * (grp % NH);
#pragma unroll
      for (int e = 0; e < EPG; ++e) {
        af[e][0] = lds_ld8_tr(vs + 32 * e);
        af[e][1] = lds_ld8_tr(vs + 16 * kVPitch + 32 * e);
      }
    };
    auto pv_mma = [&](int grp, const uint2 (&af)[4][2]) {
      const int up = 2 * (grp / NH), e0 = EPG * (grp % NH);
      uint4 pp[NQ];
#pragma unroll
      for (int nt = 0; nt < NQ; ++nt) pp[nt] = make_uint4(pf[nt][up].x, pf[nt][up].y, pf[nt][up + 1].x, pf[nt][up + 1].y);
#pragma unroll
      for (int e = 0; e < EPG; ++e) {
        const uint4 a = make_uint4(af[e][0].x, af[e][0].y, af[e][1].x, af[e][1].y);
#pragma unroll
        for (int nt = 0; nt < NQ; ++nt) acc[nt][e0 + e] = mfma_16x16x32<F16>(a, pp[nt], acc[nt][e0 + e]);
      }
      if (grp % NH == NH - 1) {  // once per 32-key step
#pragma unroll
        for (int nt = 0; nt < NQ; ++nt) accl[nt] = mfma_16x16x32<F16>(ones, pp[nt], accl[nt]);
      }
    };
#define MI_SB() __builtin_amdgcn_sched_barrier(0)
    // The whole matrix phase of iteration it: O^T += V^T P^T of tile it-1, S^T = K Q^T of tile it,
    // and -- spread over the first MFMA groups, whose shadow hides the address arithmetic --
    // the staging: store K(it+1) and V(it+1) (fetched during the previous matrix phase) into
    // LDS, then fetch K(it+2) and V(it+2).  (Moving score groups to the vector phase was measured
    // slower; so was reading more than one group of fragments ahead there: the registers run out.)
    Cursor cur = cursor_at(tb + 2);  // the tile fetched during iteration 0
    int pc_cur = 0;             // its block-table entry (a per-lane copy, made scalar at its use)
    // Head width 128, whose matrix phase is the longer one: the fragments of its first value group are requested at
    // the end of the vector phase before it (their tile was staged two phases earlier) and waited for at that
    // phase's barrier, so the matrix phase starts on loaded registers instead of on an LDS round trip.
    constexpr bool kAhead = !WIDE && !MLA && HD == 128;
    uint2 a_first[4][2];
    auto matrix_phase = [&](int it) {
      uint2 a0[4][2], a1[4][2];
      uint4 k0[KS], k1[KS];
      const int ta = it - 1, ts = it;
      if constexpr (WIDE) {
        // One list of operand groups -- the value groups of tile it-1 (a 32-key step x 64 output columns each), then
        // the 16-key score groups of tile it; the fragments of group i+1 are requested before the MFMAs of group i,
        // in alternating registers.  Staging rides behind the first three groups.
        constexpr int NPV = (kPPTile / 32) * NH, NG = NPV + NT;
        static_assert(NG >= 3, "the staging hooks sit behind groups 0, 1 and 2");
        uint2 ab[2][4][2];
        uint4 kb[2][KS];
        auto load = [&](int i) {
          if (i < NPV) pv_load(ta, i, ab[i & 1]);
          else sc_load(ts, i - NPV, kb[(i - NPV) & 1]);
        };
        auto mma = [&](int i) {
          if (i < NPV) pv_mma(i, ab[i & 1]);
          else sc_mma(i - NPV, kb[(i - NPV) & 1]);
        };
        int64_t off = 0;
        int room = 0;
        load(0);
#pragma unroll
        for (int i = 0; i < NG; ++i) {
          if (i + 1 < NG) load(i + 1);
          MI_SB();
          mma(i);
          if (i == 0) {
            store_k(it + 1);
            store_v(it + 1);
          } else if (i == 1) {
            off = tile_offset(cur, pc_cur);
            room = cur.room;
            tile_loads_k(off, room);
            cursor_next(cur);
            pc_cur = bt_row[cur.ci];  // block-table entry of tile it+3, consumed one iteration from now
          } else if (i == 2) {
            tile_loads_v(off, room);
          }
          MI_SB();
        }
        return;
      }
      if constexpr (HD == 64) {  // half the matrix work per tile: two value groups, four 4-MFMA score groups
        pv_load(ta, 0, a0);
        pv_load(ta, 1, a1); MI_SB();
        pv_mma(0, a0);
        store_k(it + 1);
        store_v(it + 1); MI_SB();
        const int64_t off = tile_offset(cur, pc_cur);
        const int room = cur.room;
        tile_loads(kbase, off, room, kreg);
        cursor_next(cur);
        pc_cur = bt_row[cur.ci];  // block-table entry of tile it+3, consumed one iteration from now
#pragma unroll
        for (int i = 0; i < 10; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
          __builtin_amdgcn_sched_group_barrier(0x006, 3, 0);  // up to three scalar / vector ALU instructions
        }
        MI_SB();
        sc_load(ts, 0, k0); MI_SB();
        pv_mma(1, a1);
        tile_loads_v(off, room); MI_SB();
        sc_load(ts, 1, k1); MI_SB(); sc_mma(0, k0); MI_SB();
        sc_load(ts, 2, k0); MI_SB(); sc_mma(1, k1); MI_SB();
        sc_load(ts, 3, k1); MI_SB(); sc_mma(2, k0); MI_SB();
        sc_mma(3, k1);
        return;
      }
      if constexpr (!kAhead) pv_load(ta, 0, a_first);
      pv_load(ta, 1, a1); MI_SB();
      pv_mma(0, a_first);
      store_k(it + 1);
      store_v(it + 1); MI_SB();
      pv_load(ta, 2, a0); MI_SB();
      pv_mma(1, a1);
      const int64_t off = tile_offset(cur, pc_cur);
      const int room = cur.room;
      const int64_t off_v = MLA ? tile_offset_v(cur, pc_cur) : off;
      const int room_v = MLA ? cur.room_v : room;
      tile_loads_k(off, room);
      cursor_next(cur);
      pc_cur = bt_row[cur.ci];  // block-table entry of tile it+3, consumed one iteration from now
      // spread the address arithmetic through the shadow of this group's MFMAs
#pragma unroll
      for (int i = 0; i < 10; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
        __builtin_amdgcn_sched_group_barrier(0x006, 3, 0);  // up to three scalar / vector ALU instructions
      }
      MI_SB();
      pv_load(ta, 3, a1); MI_SB();
      pv_mma(2, a0);
      tile_loads_v(off_v, room_v); MI_SB();
      if constexpr (MLA) {
        uint4 h0[3], h1[3];
        sc_load_half(ts, 0, 0, h0); MI_SB();
        pv_mma(3, a1); MI_SB();
        sc_load_half(ts, 0, 1, h1); MI_SB(); sc_mma_half(0, 0, h0); MI_SB();
        sc_load_half(ts, 1, 0, h0); MI_SB(); sc_mma_half(0, 1, h1); MI_SB();
        sc_load_half(ts, 1, 1, h1); MI_SB(); sc_mma_half(1, 0, h0); MI_SB();
        sc_load_half(ts, 2, 0, h0); MI_SB(); sc_mma_half(1, 1, h1); MI_SB();
        sc_load_half(ts, 2, 1, h1); MI_SB(); sc_mma_half(2, 0, h0); MI_SB();
        sc_load_half(ts, 3, 0, h0); MI_SB(); sc_mma_half(2, 1, h1); MI_SB();
        sc_load_half(ts, 3, 1, h1); MI_SB(); sc_mma_half(3, 0, h0); MI_SB();
        sc_mma_half(3, 1, h1);
        return;
      }
      if constexpr (kAhead) {
        // the next group's four key fragments requested one by one between this group's products, not in a burst:
        // the four wavefronts in this phase run in step and would otherwise queue at the LDS together
        auto weave = [&]() {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);  // two MFMAs
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // one LDS read
          }
        };
        sc_load(ts, 0, k0); pv_mma(3, a1); weave(); MI_SB();
        sc_load(ts, 1, k1); sc_mma(0, k0); weave(); MI_SB();
        sc_load(ts, 2, k0); sc_mma(1, k1); weave(); MI_SB();
        sc_load(ts, 3, k1); sc_mma(2, k0); weave(); MI_SB();
        sc_mma(3, k1);
        return;
      }
      sc_load(ts, 0, k0); MI_SB();
      pv_mma(3, a1); MI_SB();
      sc_load(ts, 1, k1); MI_SB(); sc_mma(0, k0); MI_SB();
      sc_load(ts, 2, k0); MI_SB(); sc_mma(1, k1); MI_SB();
      sc_load(ts, 3, k1); MI_SB(); sc_mma(2, k0); MI_SB();
      sc_mma(3, k1);
    };
    // ---- online softmax of tile t: s -> pf, rescale of the accumulators when the reference moved ----
    auto softmax = [&](int t) {  // t counts from this workgroup's first tile
      const int T = (tb + t) * kPPTile;
      const bool need_mask = T + kPPTile - 1 > full_until;
#pragma unroll
      for (int nt = 0; nt < NQ; ++nt) {
        if (need_mask) {
          int Tm = T;
          // keeps the token positions below out of the tiles that need no mask (the 192-wide keys of the
          // multi-latent form have no register to spare for it)
          if constexpr (!MLA) asm volatile("" : "+s"(Tm));
#pragma unroll
          for (int u = 0; u < NT; ++u) {
            const int tok0 = Tm + 16 * u + 4 * g;
#pragma unroll
            for (int i = 0; i < 4; ++i)
              if (tok0 + i > qpos[nt]) s[nt][u][i] = -INFINITY;
          }
        }
        float tmax = fmaxf(fmaxf(s[nt][0][0], s[nt][0][1]), s[nt][0][2]);
        tmax = fmaxf(fmaxf(tmax, s[nt][0][3]), s[nt][1][0]);
        tmax = fmaxf(fmaxf(tmax, s[nt][1][1]), s[nt][1][2]);
        if constexpr (NT == 4) {
          tmax = fmaxf(fmaxf(tmax, s[nt][1][3]), s[nt][2][0]);
          tmax = fmaxf(fmaxf(tmax, s[nt][2][1]), s[nt][2][2]);
          tmax = fmaxf(fmaxf(tmax, s[nt][2][3]), s[nt][3][0]);
          tmax = fmaxf(fmaxf(tmax, s[nt][3][1]), s[nt][3][2]);
          tmax = fmaxf(tmax, s[nt][3][3]);
        } else {
          tmax = fmaxf(tmax, s[nt][1][3]);
        }
        // The reference the exponentials are taken against moves only when a score of this lane exceeds it by a
        // window (2^kWin as the largest probability): the exchange within the row group, the rescale factor and
        // the rescale are then rare instead of once per tile.
        if (__builtin_amdgcn_ballot_w64(tmax > m_run[nt] + win)) {
          tmax = rowgroup_max(tmax);
          const float m_raw = fmaxf(m_run[nt], tmax);
          const float m_use = m_raw == -INFINITY ? 0.f : m_raw;
          const float alpha = fast_exp2((m_run[nt] - m_use) * scale);
          neg_run[nt] = -m_use * scale;
          m_run[nt] = m_raw;
          if (__builtin_amdgcn_ballot_w64(alpha != 1.f)) {
#pragma unroll
            for (int e = 0; e < DV; ++e) {
              acc[nt][e][0] *= alpha; acc[nt][e][1] *= alpha; acc[nt][e][2] *= alpha; acc[nt][e][3] *= alpha;
            }
            accl[nt][0] *= alpha; accl[nt][1] *= alpha; accl[nt][2] *= alpha; accl[nt][3] *= alpha;
          }
        }
        const float neg = neg_run[nt];
#pragma unroll
        for (int u = 0; u < NT; ++u) {
          const float p0 = fast_exp2(__builtin_fmaf(s[nt][u][0], scale, neg));
          const float p1 = fast_exp2(__builtin_fmaf(s[nt][u][1], scale, neg));
          const float p2 = fast_exp2(__builtin_fmaf(s[nt][u][2], scale, neg));
          const float p3 = fast_exp2(__builtin_fmaf(s[nt][u][3], scale, neg));
          pf[nt][u] = make_uint2(pack2<F16>(p0, p1), pack2<F16>(p2, p3));
        }
      }
      if constexpr (kAhead) pv_load(t, 0, a_first);  // for the matrix phase of iteration t + 1
    };
    // Staging rides in the matrix phase (LDS-write and memory ports are idle there).  Phase
    // numbers: group 0 runs matrix(it) in phase 2it and vector(it) in 2it+1, group 1 one phase
    // later.  matrix(it) reads K(it) and V(it-1), the vector phase reads no LDS; both groups store
    // K(it+1) and V(it+1) during matrix(it), i.e. in phases 2it and 2it+1.
    //   K(t): stored in phases 2t-2, 2t-1; read in 2t, 2t+1           -> two buffers
    //   V(t): stored in phases 2t-2, 2t-1; read in 2t+2, 2t+3         -> three buffers
    // (the tile that shares a buffer is stored from phase 2t+2 resp. 2t+4 on).
#pragma unroll
    for (int nt = 0; nt < NQ; ++nt)
#pragma unroll
      for (int u = 0; u < NT; ++u) pf[nt][u] = make_uint2(0u, 0u);
    for (int i = tid * 16; i < kPPTile * kVPitch; i += 512 * 16)
      *reinterpret_cast<uint4*>(&Vs[2][i]) = make_uint4(0u, 0u, 0u, 0u);  // "tile -1"
    {
      const Cursor c0 = cursor_at(tb), c1 = cursor_at(tb + 1);
      const int pc0 = bt_row[c0.ci], pc1 = bt_row[c1.ci];
      const int64_t off0 = tile_offset(c0, pc0);
      tile_loads_k(off0, c0.room);
      tile_loads_v(MLA ? tile_offset_v(c0, pc0) : off0, MLA ? c0.room_v : c0.room);
      store_k(0);
      store_v(0);
      __syncthreads();  // K(0), V(0) and the zero-filled buffer are visible; the staging registers are free
      const int64_t off1 = tile_offset(c1, pc1);
      tile_loads_k(off1, c1.room);  // K(1), V(1): stored by matrix(0)
      tile_loads_v(MLA ? tile_offset_v(c1, pc1) : off1, MLA ? c1.room_v : c1.room);
      pc_cur = bt_row[cur.ci];
    }
    if (lead) __syncthreads();  // second group idles through phase 0

    // One code path for every iteration.  Every wave runs every staged tile of the workgroup (a
    // wave whose rows cannot see a tile would only wait at the barriers instead; its scores there
    // are all masked, p = 0).  Iteration 0 "accumulates" tile -1: zero probabilities times a
    // zero-filled V buffer; iteration ntl computes scores of a stale K buffer that nobody uses.
    if constexpr (kAhead) pv_load(-1, 0, a_first);
    for (int it = 0; it <= ntl; ++it) {
      // (scheduling barriers: MFMAs touch no memory, so nothing else stops the compiler from
      // sinking them past the workgroup barrier into the other phase)
      __builtin_amdgcn_s_setprio(2);  // the matrix-phase wave issues first: its MFMAs are sparse
      matrix_phase(it);               // and must never wait behind the other wave's ALU stream
      __builtin_amdgcn_s_setprio(0);
      MI_SB();
      __syncthreads();
      MI_SB();
      if (it < ntl) softmax(it);
      MI_SB();
      __syncthreads();
      MI_SB();
    }
    if (!lead && STAGGER) __syncthreads();
#undef MI_SB
  }

  // ---- epilogue: acc[nt][e][i] is output element d = 16e + 4g + i of row (nt, m16) --------------
#pragma unroll
  for (int nt = 0; nt < NQ; ++nt) {
    const float l_tot = accl[nt][0];
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    const int n = 16 * nt + m16;
    const int qi = (n * g_magic) >> 16, u = n - qi * G;  // n / G, n % G
    if (qi < nq) {
      if (!SPLIT) {
        uint16_t* o = p.out + (int64_t)(q_begin + q0 + qi) * p.o_st + (int64_t)(hq0 + u) * p.o_sh + 4 * g;
#pragma unroll
        for (int e = 0; e < DV; ++e)
          st8(o + 16 * e, make_uint2(pack2<F16>(acc[nt][e][0] * inv, acc[nt][e][1] * inv),
                                     pack2<F16>(acc[nt][e][2] * inv, acc[nt][e][3] * inv)));
      } else {  // a range without visible keys (none for short requests) leaves zeros and -inf
        const int64_t prow = ((int64_t)split * p.T + (q_begin + q0 + qi)) * p.Hq + (hq0 + u);
        float* o = p.split_o + prow * HD + 4 * g;
#pragma unroll
        for (int e = 0; e < DV; ++e)
          *reinterpret_cast<float4*>(o + 16 * e) =
              make_float4(acc[nt][e][0] * inv, acc[nt][e][1] * inv, acc[nt][e][2] * inv, acc[nt][e][3] * inv);
        if (g == 0) p.split_lse[prow] = l_tot > 0.f ? m_run[nt] * p.scale_log2 + fast_log2(l_tot) : -INFINITY;
      }
    }
  }
}

// Rows whose keys were split over several workgroups: o = sum_s 2^(lse_s - max) o_s / sum_s 2^(lse_s - max).
// Grid (T, Hq), head_dim threads = the output values of one (row, head).
template <bool F16>
__global__ __launch_bounds__(256) void prefill_split_merge_kernel(PrefillParams p, int n_split, int head_dim) {
  const int row = blockIdx.x, head = blockIdx.y, d = threadIdx.x;
  if (row >= p.cu_q[p.R]) return;  // padding rows: zeroed by the tile kernel
  if (p.skip_single) {             // one-row requests were left to the decode kernels
    int lo = 0, hi = p.R - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (p.cu_q[mid] <= row) lo = mid; else hi = mid - 1;
    }
    if (p.cu_q[lo + 1] - p.cu_q[lo] == 1) return;
  }
  float mx = -INFINITY, num = 0.f, den = 0.f;
  for (int s0 = 0; s0 < n_split; s0 += 8) {
    float lse[8], po[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int64_t prow = ((int64_t)min(s0 + j, n_split - 1) * p.T + row) * p.Hq + head;
      lse[j] = p.split_lse[prow];
      po[j] = p.split_o[prow * head_dim + d];
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (s0 + j < n_split && lse[j] != -INFINITY) {
        const float m_new = fmaxf(mx, lse[j]);
        const float a = fast_exp2(mx - m_new), wt = fast_exp2(lse[j] - m_new);
        num = num * a + wt * po[j];
        den = den * a + wt;
        mx = m_new;
      }
    }
  }
  p.out[(int64_t)row * p.o_st + (int64_t)head * p.o_sh + d] = f32_to_16<F16>(den > 0.f ? num / den : 0.f);
}

}  // namespace mi

using namespace mi;

// Ranges the keys of every request are cut into by the two-phase tile kernel.  Few query rows over a
// long context (a chunk of a prompt, a short turn after a long history) give few workgroups, each
// with thousands of keys to walk: then the keys are split so that about one workgroup per CU exists,
// every one keeping at least sixteen 64-key tiles (a 512-token prompt is not worth the merge).  Host-side quantities only (the lengths live on the GPU).
static int prefill_kv_splits(int T, int Hq, int Hkv, int head_dim, int max_kv_len) {
  if (max_kv_len <= 0) return 1;
  const int G = Hq / Hkv, Gw = G < 16 ? G : 16, parts = (G + 15) / 16;
  const int sbq = 8 * ((head_dim >= 192 ? 16 : 32) / Gw);  // query tokens per workgroup (8 wavefronts x 32 or 16 rows)
  const int64_t useful = (int64_t)Hkv * parts * ((T + sbq - 1) / sbq);
  const int cus = 256;
  if (useful >= cus) return 1;
  int64_t s = (cus + useful - 1) / useful;
  const int64_t by_tiles = ((int64_t)max_kv_len + 63) / 64 / 16;
  if (s > by_tiles) s = by_tiles;
  if (s > 32) s = 32;  // (more ranges cost more in partials than they win: 64 rows over 131 072 keys, 16-32 is best)
  return s < 2 ? 1 : (int)s;
}

// key ranges for these sizes under the caller's knob (1 = automatic, -1 = never, n > 1 = forced)
static int kv_split_count(const MiTuning& tune, int T, int Hq, int Hkv, int head_dim, int max_kv_len) {
  if (tune.prefill_kv_split < 0) return 1;
  return tune.prefill_kv_split > 1 ? tune.prefill_kv_split : prefill_kv_splits(T, Hq, Hkv, head_dim, max_kv_len);
}

extern "C" int64_t mi_prefill_workspace_bytes(int32_t T, int32_t R, int32_t Hq, int32_t Hkv,
                                              int32_t head_dim, int32_t max_kv_len,
                                              int32_t split_tokens, const MiTuning* tuning) {
  MiTuning tune;
  if (mi_resolve_tuning(tuning, &tune, "mi_prefill_workspace_bytes") != MI_OK) return -1;
  // The one-row (decode) requests of a mixed batch are streamed by the decode kernels, whose partials
  // live here; behind them the partials of the tile kernel when it splits the keys.
  int64_t bytes = mi_decode_workspace_bytes(R, Hq, Hkv, head_dim, 16, max_kv_len, split_tokens, tuning);
  bytes = (bytes + 255) & ~(int64_t)255;
  if (T > 0 && Hq > 0 && Hkv > 0 && Hq % Hkv == 0) {
    const int s = kv_split_count(tune, T, Hq, Hkv, head_dim, max_kv_len);  // (a forced count is honoured here too)
    if (s > 1) bytes += (int64_t)s * T * Hq * (head_dim + 1) * (int64_t)sizeof(float);
  }
  return bytes;
}

// The two-phase tile kernel for one combination of (wave groups staggered?, fp8 cache?, keys split?, widths, type).
#define MI_PP_LAUNCH(FP8_, HD_, HDK_, F16_)                                                                         \
  do {                                                                                                              \
    if (n_split > 1 && stagger) hipLaunchKernelGGL((paged_prefill_pp_kernel<true, FP8_, true, HD_, HDK_, F16_>), lgrid, dim3(512), 0, st, p);   \
    else if (n_split > 1) hipLaunchKernelGGL((paged_prefill_pp_kernel<false, FP8_, true, HD_, HDK_, F16_>), lgrid, dim3(512), 0, st, p);      \
    else if (stagger) hipLaunchKernelGGL((paged_prefill_pp_kernel<true, FP8_, false, HD_, HDK_, F16_>), lgrid, dim3(512), 0, st, p);          \
    else hipLaunchKernelGGL((paged_prefill_pp_kernel<false, FP8_, false, HD_, HDK_, F16_>), lgrid, dim3(512), 0, st, p);                      \
  } while (0)

static int launch_paged_prefill(
    const void* q, int64_t q_stride_tok, int64_t q_stride_head, const void* k_cache,
    const void* v_cache, int64_t kv_stride_chunk, int64_t kv_stride_tok, int64_t kv_stride_head,
    const int32_t* block_table, int64_t bt_stride, const int32_t* cu_seqlens_q,
    const int32_t* kv_lens, void* out, int64_t o_stride_tok, int64_t o_stride_head,
    void* workspace, int64_t workspace_bytes, int32_t T, int32_t R, int32_t Hq, int32_t Hkv,
    int32_t head_dim, int32_t chunk_tokens, int32_t max_kv_len, int32_t split_tokens, float softmax_scale,
    int32_t kv_dtype, const float* k_scales, const float* v_scales, int32_t dtype, const MiTuning* tuning,
    void* stream) {
  const bool fp8 = kv_dtype == MI_KV_FP8_E4M3;
  if (T == 0 || R == 0) return MI_OK;
  MiTuning tune;
  const int rc_t = mi_resolve_tuning(tuning, &tune, "mi_paged_prefill_attention");
  if (rc_t != MI_OK) return rc_t;
  if (dtype != MI_DTYPE_BF16 && dtype != MI_DTYPE_FP16)
    return mi_fail(MI_ERR_UNSUPPORTED, "mi_paged_prefill_attention: dtype must be MI_DTYPE_BF16 or MI_DTYPE_FP16");
  const bool f16 = dtype == MI_DTYPE_FP16;
  if (!q || !k_cache || !v_cache || !block_table || !cu_seqlens_q || !kv_lens || !out)
    return mi_fail(MI_ERR_NULL, "mi_paged_prefill_attention: null pointer argument");
  if (T < 0 || R < 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv || Hkv > 65535)
    return mi_fail(MI_ERR_SHAPE, "mi_paged_prefill_attention: need T, R >= 0 and Hq a multiple of Hkv");
  const int G = Hq / Hkv;
  if (G > 64)
    return mi_fail(MI_ERR_UNSUPPORTED, "mi_paged_prefill_attention: at most 64 query heads per KV head");
  if (head_dim != 64 && head_dim != 96 && head_dim != 128 && head_dim != 192 && head_dim != 256)
    return mi_fail(MI_ERR_UNSUPPORTED, "mi_paged_prefill_attention: head_dim must be 64, 96, 128, 192 or 256");
  const int Gw = G < 16 ? G : 16, parts = (G + 15) / 16;  // query heads per workgroup, workgroups per KV head
  if (chunk_tokens <= 0 || chunk_tokens % 16)
    return mi_fail(MI_ERR_SHAPE, "mi_paged_prefill_attention: chunk size must be a positive multiple of 16");
  if (((uintptr_t)q | (uintptr_t)k_cache | (uintptr_t)v_cache | (uintptr_t)out) & 15)
    return mi_fail(MI_ERR_ALIGN, "mi_paged_prefill_attention: q/k/v/out must be 16-byte aligned");
  if ((q_stride_tok | q_stride_head | o_stride_tok | o_stride_head | kv_stride_chunk | kv_stride_tok | kv_stride_head) % 8)
    return mi_fail(MI_ERR_ALIGN, "mi_paged_prefill_attention: strides must keep rows 16-byte aligned");
  if (kv_stride_tok * (int64_t)chunk_tokens * 2 >= (int64_t)1 << 31)
    return mi_fail(MI_ERR_SHAPE, "mi_paged_prefill_attention: one chunk must span less than 2 GiB");
  if (fp8 && (kv_stride_chunk | kv_stride_tok | kv_stride_head) % 16)
    return mi_fail(MI_ERR_ALIGN, "mi_paged_prefill_attention_fp8: cache strides must keep rows 16-byte aligned");
  if (kv_dtype != MI_KV_16BIT && !fp8)
    return mi_fail(MI_ERR_UNSUPPORTED, "mi_paged_prefill_attention: unknown kv_dtype");
  if (fp8 && (!k_scales || !v_scales))
    return mi_fail(MI_ERR_NULL, "mi_paged_prefill_attention_fp8: both scale arrays are required");
  // the two-phase tile kernel stages 64-key tiles that must not straddle chunks; other chunk sizes (and the knob)
  // select the register-only kernel
  const bool two_phase = tune.prefill_two_phase > 0 && chunk_tokens % 64 == 0;
  if (fp8 && ((head_dim != 64 && head_dim != 128) || !two_phase))
    return mi_fail(MI_ERR_UNSUPPORTED,
                   "mi_paged_prefill_attention_fp8: fp8 KV needs head_dim 64 or 128, a chunk size that is a "
                   "multiple of 64 and the two-phase tile kernel");
  if (!(softmax_scale > 0.f)) return mi_fail(MI_ERR_SHAPE, "mi_paged_prefill_attention: softmax_scale must be positive");
  // (no limit on the number of requests: the decode part of a mixed batch runs in slices when it has to)

  PrefillParams p;
  p.q = (const uint16_t*)q; p.q_st = q_stride_tok; p.q_sh = q_stride_head;
  p.kc = (const uint8_t*)k_cache; p.vc = (const uint8_t*)v_cache;
  p.kv_sc = kv_stride_chunk; p.kv_st = (int32_t)kv_stride_tok; p.kv_sh = (int32_t)kv_stride_head;
  p.v_sc = p.kv_sc; p.v_st = p.kv_st; p.v_sh = p.kv_sh;
  p.bt = block_table; p.bt_stride = bt_stride; p.cu_q = cu_seqlens_q; p.lens = kv_lens;
  p.out = (uint16_t*)out; p.o_st = o_stride_tok; p.o_sh = o_stride_head;
  p.T = T; p.R = R; p.Hq = Hq; p.Hkv = Hkv; p.G = G; p.parts = parts;
  p.g_magic = 65536 / Gw + 1;
  p.chunk = chunk_tokens;
  p.chunk_magic = (((uint64_t)1 << 40) + chunk_tokens - 1) / chunk_tokens;
  p.scale_log2 = softmax_scale * 1.4426950408889634f;
  // With a workspace, one-row requests go through the bandwidth-optimised decode kernels.
  p.skip_single = workspace != nullptr;
  p.k_scale = k_scales; p.v_scale = v_scales;
  p.split_o = nullptr; p.split_lse = nullptr;

  // The decode part's own argument checks come before the first launch, so that a negative return still means
  // nothing was enqueued (its remaining checks repeat ones made above).
  if (p.skip_single) {
    const int rc_w = check_decode_workspace(workspace, workspace_bytes, R, Hq, Hkv, head_dim, split_tokens, tune,
                                            "mi_paged_prefill_attention");
    if (rc_w != MI_OK) return rc_w;
  }

  hipStream_t st = (hipStream_t)stream;
  if (two_phase) {
    const int sbq_lds = 8 * ((head_dim >= 192 ? 16 : 32) / Gw);  // 8 wavefronts x whole tokens in a wavefront's 32 (wide heads: 16) rows
    dim3 lgrid(((T + sbq_lds - 1) / sbq_lds + R) * Hkv * parts);
    hipEvent_t ev_a, ev_b;
    const bool timed = mi_profile_next(&ev_a, &ev_b);
    if (timed) (void)hipEventRecord(ev_a, st);
    const bool stagger = tune.prefill_two_phase != 2;
    // key ranges per request (with a workspace only): partials behind the decode part's scratch
    int n_split = 1;
    if (workspace) {
      n_split = kv_split_count(tune, T, Hq, Hkv, head_dim, max_kv_len);
      const int64_t dec_bytes = (mi_decode_workspace_bytes(R, Hq, Hkv, head_dim, 16, max_kv_len, split_tokens, tuning) + 255) &
                                ~(int64_t)255;
      const int64_t sp_bytes = (int64_t)n_split * T * Hq * (head_dim + 1) * (int64_t)sizeof(float);
      if (n_split > 1 && workspace_bytes < dec_bytes + sp_bytes) n_split = 1;  // (a caller-sized workspace without room for them)
      if (n_split > 1) {
        p.split_o = reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(workspace) + dec_bytes);
        p.split_lse = p.split_o + (int64_t)n_split * T * Hq * head_dim;
        lgrid.y = n_split;
        workspace_bytes = dec_bytes;
      }
    }
    // head_dim 128 over a 16-bit cache: the one-stream tile kernel when asked for
    if (!fp8 && head_dim == 128 && tune.prefill_two_phase == 3) launch_prefill_woven(p, lgrid, f16, st);
    else if (fp8 && head_dim == 64 && f16) MI_PP_LAUNCH(true, 64, 64, true);
    else if (fp8 && head_dim == 64) MI_PP_LAUNCH(true, 64, 64, false);
    else if (fp8 && f16) MI_PP_LAUNCH(true, 128, 128, true);
    else if (fp8) MI_PP_LAUNCH(true, 128, 128, false);
    else if (head_dim == 128 && f16) MI_PP_LAUNCH(false, 128, 128, true);
    else if (head_dim == 128) MI_PP_LAUNCH(false, 128, 128, false);
    else if (head_dim == 64 && f16) MI_PP_LAUNCH(false, 64, 64, true);
    else if (head_dim == 64) MI_PP_LAUNCH(false, 64, 64, false);
    else if (head_dim == 96 && f16) MI_PP_LAUNCH(false, 96, 96, true);
    else if (head_dim == 96) MI_PP_LAUNCH(false, 96, 96, false);
    else if (head_dim == 192 && f16) MI_PP_LAUNCH(false, 192, 192, true);
    else if (head_dim == 192) MI_PP_LAUNCH(false, 192, 192, false);
    else if (f16) MI_PP_LAUNCH(false, 256, 256, true);
    else MI_PP_LAUNCH(false, 256, 256, false);
    if (timed) (void)hipEventRecord(ev_b, st);
    if (n_split > 1) {
      if (f16) hipLaunchKernelGGL(prefill_split_merge_kernel<true>, dim3(T, Hq), dim3(head_dim), 0, st, p, n_split, head_dim);
      else hipLaunchKernelGGL(prefill_split_merge_kernel<false>, dim3(T, Hq), dim3(head_dim), 0, st, p, n_split, head_dim);
    }
  } else {
    // register-only kernel: any chunk size that is a multiple of 16; 16 or 32 keys per iteration
    // (wide heads: fewer rows per wavefront and keys per iteration, so that accumulators and fragments fit)
    const int nq = head_dim == 256 ? 1 : head_dim == 192 ? 2 : tune.prefill_row_tiles == 4 ? 4 : 2;
    const int waves = head_dim == 256 ? 8 : 16 / nq;
    const int sbq = waves * ((16 * nq) / Gw);  // query tokens per workgroup: whole tokens in each wavefront's rows
    dim3 grid((T + sbq - 1) / sbq + R, Hkv * parts), block(64 * waves);
    const int nt = (tune.prefill_tile_subtiles == 1 || head_dim >= 192) ? 1 : 2;
    hipEvent_t ev_a, ev_b;
    const bool timed = mi_profile_next(&ev_a, &ev_b);
    if (timed) (void)hipEventRecord(ev_a, st);
#define MI_LAUNCH_PREFILL(HD_, F16_)                                                                           \
  do {                                                                                                         \
    if (nq == 4 && nt == 1) hipLaunchKernelGGL((paged_prefill_kernel<HD_, HD_, 1, 4, F16_>), grid, block, 0, st, p);  \
    else if (nq == 4) hipLaunchKernelGGL((paged_prefill_kernel<HD_, HD_, 2, 4, F16_>), grid, block, 0, st, p);        \
    else if (nt == 1) hipLaunchKernelGGL((paged_prefill_kernel<HD_, HD_, 1, 2, F16_>), grid, block, 0, st, p);        \
    else hipLaunchKernelGGL((paged_prefill_kernel<HD_, HD_, 2, 2, F16_>), grid, block, 0, st, p);                     \
  } while (0)
    if (head_dim == 128 && f16) MI_LAUNCH_PREFILL(128, true);
    else if (head_dim == 128) MI_LAUNCH_PREFILL(128, false);
    else if (head_dim == 64 && f16) MI_LAUNCH_PREFILL(64, true);
    else if (head_dim == 64) MI_LAUNCH_PREFILL(64, false);
    else if (head_dim == 96 && f16) MI_LAUNCH_PREFILL(96, true);
    else if (head_dim == 96) MI_LAUNCH_PREFILL(96, false);
    else if (head_dim == 192 && f16) hipLaunchKernelGGL((paged_prefill_kernel<192, 192, 1, 2, true>), grid, block, 0, st, p);
    else if (head_dim == 192) hipLaunchKernelGGL((paged_prefill_kernel<192, 192, 1, 2, false>), grid, block, 0, st, p);
    else if (f16) hipLaunchKernelGGL((paged_prefill_kernel<256, 256, 1, 1, true, 8>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((paged_prefill_kernel<256, 256, 1, 1, false, 8>), grid, block, 0, st, p);
#undef MI_LAUNCH_PREFILL
    if (timed) (void)hipEventRecord(ev_b, st);
  }
  const int rc = mi_check_launch("mi_paged_prefill_attention");
  if (rc != MI_OK || !p.skip_single) return rc;
  return launch_paged_decode(q, q_stride_tok, q_stride_head, k_cache, v_cache, kv_stride_chunk, kv_stride_tok,
                             kv_stride_head, block_table, bt_stride, kv_lens, cu_seqlens_q, out, o_stride_tok,
                             o_stride_head, workspace, workspace_bytes, R, Hq, Hkv, head_dim, chunk_tokens,
                             split_tokens, softmax_scale, kv_dtype, k_scales, v_scales, dtype, tune, stream);
}

extern "C" int mi_paged_prefill_attention(
    const void* q, int64_t q_stride_tok, int64_t q_stride_head, const void* k_cache,
    const void* v_cache, int64_t kv_stride_chunk, int64_t kv_stride_tok, int64_t kv_stride_head,
    const int32_t* block_table, int64_t bt_stride, const int32_t* cu_seqlens_q,
    const int32_t* kv_lens, void* out, int64_t o_stride_tok, int64_t o_stride_head,
    void* workspace, int64_t workspace_bytes, int32_t T, int32_t R, int32_t Hq, int32_t Hkv,
    int32_t head_dim, int32_t chunk_tokens, int32_t max_kv_len, int32_t split_tokens,
    float softmax_scale, int32_t dtype, const MiTuning* tuning, void* stream) {
  return launch_paged_prefill(q, q_stride_tok, q_stride_head, k_cache, v_cache, kv_stride_chunk, kv_stride_tok,
                              kv_stride_head, block_table, bt_stride, cu_seqlens_q, kv_lens, out, o_stride_tok,
                              o_stride_head, workspace, workspace_bytes, T, R, Hq, Hkv, head_dim, chunk_tokens,
                              max_kv_len, split_tokens, softmax_scale, MI_KV_16BIT, nullptr, nullptr, dtype, tuning,
                              stream);
}

extern "C" int mi_paged_prefill_attention_fp8(
    const void* q, int64_t q_stride_tok, int64_t q_stride_head, const void* k_cache_fp8,
    const void* v_cache_fp8, int64_t kv_stride_chunk, int64_t kv_stride_tok, int64_t kv_stride_head,
    const float* k_scales, const float* v_scales, const int32_t* block_table, int64_t bt_stride,
    const int32_t* cu_seqlens_q, const int32_t* kv_lens, void* out, int64_t o_stride_tok,
    int64_t o_stride_head, void* workspace, int64_t workspace_bytes, int32_t T, int32_t R, int32_t Hq,
    int32_t Hkv, int32_t head_dim, int32_t chunk_tokens, int32_t max_kv_len, int32_t split_tokens,
    float softmax_scale, int32_t dtype, const MiTuning* tuning, void* stream) {
  return launch_paged_prefill(q, q_stride_tok, q_stride_head, k_cache_fp8, v_cache_fp8, kv_stride_chunk,
                              kv_stride_tok, kv_stride_head, block_table, bt_stride, cu_seqlens_q, kv_lens, out,
                              o_stride_tok, o_stride_head, workspace, workspace_bytes, T, R, Hq, Hkv, head_dim,
                              chunk_tokens, max_kv_len, split_tokens, softmax_scale, MI_KV_FP8_E4M3, k_scales, v_scales,
                              dtype, tuning, stream);
}

extern "C" int mi_paged_prefill_attention_mla(
    const void* q, int64_t q_stride_tok, int64_t q_stride_head, const void* k_cache, int64_t k_stride_chunk,
    int64_t k_stride_tok, int64_t k_stride_head, const void* v_cache, int64_t v_stride_chunk, int64_t v_stride_tok,
    int64_t v_stride_head, const int32_t* block_table, int64_t bt_stride, const int32_t* cu_seqlens_q,
    const int32_t* kv_lens, void* out, int64_t o_stride_tok, int64_t o_stride_head, void* workspace,
    int64_t workspace_bytes, int32_t T, int32_t R, int32_t Hq, int32_t Hkv, int32_t head_dim_k, int32_t head_dim_v,
    int32_t chunk_tokens, int32_t max_kv_len, float softmax_scale, int32_t dtype, const MiTuning* tuning,
    void* stream) {
  if (T == 0 || R == 0) return MI_OK;
  MiTuning tune;
  const int rc_t = mi_resolve_tuning(tuning, &tune, "mi_paged_prefill_attention_mla");
  if (rc_t != MI_OK) return rc_t;
  if (dtype != MI_DTYPE_BF16 && dtype != MI_DTYPE_FP16)
    return mi_fail(MI_ERR_UNSUPPORTED, "mi_paged_prefill_attention_mla: dtype must be MI_DTYPE_BF16 or MI_DTYPE_FP16");
  const bool f16 = dtype == MI_DTYPE_FP16;
  if (!q || !k_cache || !v_cache || !block_table || !cu_seqlens_q || !kv_lens || !out)
    return mi_fail(MI_ERR_NULL, "mi_paged_prefill_attention_mla: null pointer argument");
  if (workspace && ((uintptr_t)workspace & 255))
    return mi_fail(MI_ERR_ALIGN, "mi_paged_prefill_attention_mla: the workspace must be 256-byte aligned");
  if (T < 0 || R < 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv || Hkv > 65535)
    return mi_fail(MI_ERR_SHAPE, "mi_paged_prefill_attention_mla: need T, R >= 0 and Hq a multiple of Hkv");
  const int G = Hq / Hkv;
  if (G > 64)
    return mi_fail(MI_ERR_UNSUPPORTED, "mi_paged_prefill_attention_mla: at most 64 query heads per KV head");
  const int Gw = G < 16 ? G : 16, parts = (G + 15) / 16;  // query heads per workgroup, workgroups per KV head
  if (head_dim_k != 192 || head_dim_v != 128)
    return mi_fail(MI_ERR_UNSUPPORTED, "mi_paged_prefill_attention_mla: key width 192 (128 + 64) and value width 128 only");
  if (chunk_tokens <= 0 || chunk_tokens % 16)
    return mi_fail(MI_ERR_SHAPE, "mi_paged_prefill_attention_mla: chunk size must be a positive multiple of 16");
  if (((uintptr_t)q | (uintptr_t)k_cache | (uintptr_t)v_cache | (uintptr_t)out) & 15)
    return mi_fail(MI_ERR_ALIGN, "mi_paged_prefill_attention_mla: q/k/v/out must be 16-byte aligned");
  if ((q_stride_tok | q_stride_head | o_stride_tok | o_stride_head | k_stride_chunk | k_stride_tok | k_stride_head |
       v_stride_chunk | v_stride_tok | v_stride_head) % 8)
    return mi_fail(MI_ERR_ALIGN, "mi_paged_prefill_attention_mla: strides must keep rows 16-byte aligned");
  if (k_stride_tok * (int64_t)chunk_tokens * 2 >= (int64_t)1 << 31 || v_stride_tok * (int64_t)chunk_tokens * 2 >= (int64_t)1 << 31)
    return mi_fail(MI_ERR_SHAPE, "mi_paged_prefill_attention_mla: one chunk must span less than 2 GiB");
  if (!(softmax_scale > 0.f)) return mi_fail(MI_ERR_SHAPE, "mi_paged_prefill_attention_mla: softmax_scale must be positive");

  PrefillParams p;
  p.q = (const uint16_t*)q; p.q_st = q_stride_tok; p.q_sh = q_stride_head;
  p.kc = (const uint8_t*)k_cache; p.vc = (const uint8_t*)v_cache;
  p.kv_sc = k_stride_chunk; p.kv_st = (int32_t)k_stride_tok; p.kv_sh = (int32_t)k_stride_head;
  p.v_sc = v_stride_chunk; p.v_st = (int32_t)v_stride_tok; p.v_sh = (int32_t)v_stride_head;
  p.bt = block_table; p.bt_stride = bt_stride; p.cu_q = cu_seqlens_q; p.lens = kv_lens;
  p.out = (uint16_t*)out; p.o_st = o_stride_tok; p.o_sh = o_stride_head;
  p.T = T; p.R = R; p.Hq = Hq; p.Hkv = Hkv; p.G = G; p.parts = parts;
  p.g_magic = 65536 / Gw + 1;
  p.chunk = chunk_tokens;
  p.chunk_magic = (((uint64_t)1 << 40) + chunk_tokens - 1) / chunk_tokens;
  p.scale_log2 = softmax_scale * 1.4426950408889634f;
  p.skip_single = 0;  // one kernel serves every request, one-row requests included
  p.k_scale = nullptr; p.v_scale = nullptr;
  p.split_o = nullptr; p.split_lse = nullptr;
  const int sbq = 8 * (32 / Gw);  // query tokens per workgroup (8 wavefronts x 32 rows)
  const bool two_phase = tune.prefill_two_phase > 0 && chunk_tokens % 64 == 0;  // staged tiles must not straddle chunks
  hipStream_t st = (hipStream_t)stream;
  hipEvent_t ev_a, ev_b;
  const bool timed = mi_profile_next(&ev_a, &ev_b);
  if (timed) (void)hipEventRecord(ev_a, st);
  int n_split = 1;
  if (two_phase) {
    dim3 lgrid(((T + sbq - 1) / sbq + R) * Hkv * parts);
    const bool stagger = tune.prefill_two_phase != 2;
    // few query rows over long contexts: key ranges per request, partials in the workspace (which holds
    // nothing else here: one-row requests stay in the tile kernel)
    if (workspace) {
      n_split = kv_split_count(tune, T, Hq, Hkv, head_dim_v, max_kv_len);
      const int64_t sp_bytes = (int64_t)n_split * T * Hq * (head_dim_v + 1) * (int64_t)sizeof(float);
      if (n_split > 1 && workspace_bytes < sp_bytes) n_split = 1;
      if (n_split > 1) {
        p.split_o = reinterpret_cast<float*>(workspace);
        p.split_lse = p.split_o + (int64_t)n_split * T * Hq * head_dim_v;
        lgrid.y = n_split;
      }
    }
    if (f16) MI_PP_LAUNCH(false, 128, 192, true);
    else MI_PP_LAUNCH(false, 128, 192, false);
  } else {
    dim3 grid((T + sbq - 1) / sbq + R, Hkv * parts), block(64 * 8);
    if (f16) hipLaunchKernelGGL((paged_prefill_kernel<192, 128, 1, 2, true>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((paged_prefill_kernel<192, 128, 1, 2, false>), grid, block, 0, st, p);
  }
  if (timed) (void)hipEventRecord(ev_b, st);
  if (n_split > 1) {
    if (f16) hipLaunchKernelGGL(prefill_split_merge_kernel<true>, dim3(T, Hq), dim3(head_dim_v), 0, st, p, n_split, head_dim_v);
    else hipLaunchKernelGGL(prefill_split_merge_kernel<false>, dim3(T, Hq), dim3(head_dim_v), 0, st, p, n_split, head_dim_v);
  }
  return mi_check_launch("mi_paged_prefill_attention_mla");
}
#undef MI_PP_LAUNCH
