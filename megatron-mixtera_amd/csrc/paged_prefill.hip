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

extern "C" int64_t mi_decode_workspace_bytes(int32_t, int32_t, int32_t, int32_t, int32_t, int32_t, int32_t);

namespace mi {

struct PrefillParams {
  const uint16_t* q;
  int64_t q_st, q_sh;
  const uint8_t* kc;
  const uint8_t* vc;
  int64_t kv_sc;
  int32_t kv_st, kv_sh;
  const int32_t* bt;
  int64_t bt_stride;
  const int32_t* cu_q;
  const int32_t* lens;
  uint16_t* out;
  int64_t o_st, o_sh;
  uint64_t chunk_magic;  // ceil(2^40 / chunk)
  int32_t T, R, Hq, Hkv, G, g_shift, chunk;
  int32_t skip_single;  // requests with exactly one query row are handled by the decode kernels
  float scale_log2;
};

// NQ = 16-row tiles per wave; a workgroup always covers 256 rows (16 / NQ waves).
template <int HD, int NT, int NQ>
__global__ __launch_bounds__(64 * (16 / NQ)) void paged_prefill_kernel(PrefillParams p) {
  constexpr int KS = HD / 32;
  constexpr int DV = HD / 16;
  constexpr int WAVES = 16 / NQ;

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int m16 = lane & 15, g = lane >> 4;
  const int h = blockIdx.y;
  const int G = p.G;
  const int BQ = (16 * NQ) >> p.g_shift;  // query tokens per wave
  const int SBQ = WAVES * BQ;             // query tokens per workgroup

  // Rows beyond the last request (token padding of the batch) are defined as zeros; the first
  // workgroup of every KV head clears its heads of those rows.
  if (blockIdx.x == 0) {
    const int tq = p.cu_q[p.R];
    const int per_row = G * HD;  // contiguous elements of this head group in one row
    for (int64_t i = (int64_t)threadIdx.x * 8; i < (int64_t)(p.T - tq) * per_row; i += 64 * WAVES * 8) {
      const int row = (int)(i / per_row), e = (int)(i - (int64_t)row * per_row);
      st16(p.out + (int64_t)(tq + row) * p.o_st + (int64_t)(h * G + e / HD) * p.o_sh + (e % HD), make_uint4(0, 0, 0, 0));
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
    const int qi = n >> p.g_shift, u = n & (G - 1);
    const bool valid = qi < nq;
    qpos[nt] = valid ? shift + q0 + qi : last;
    const uint16_t* qrow = p.q + (int64_t)(q_begin + q0 + qi) * p.q_st + (int64_t)(h * G + u) * p.q_sh;
#pragma unroll
    for (int kk = 0; kk < KS; ++kk)
      qf[nt][kk] = valid ? ld16(qrow + 32 * kk + 8 * g) : make_uint4(0, 0, 0, 0);
  }
  const int ntiles = (nq * G + 15) >> 4;  // 16-row tiles that hold a valid row

  const uint8_t* kbase = p.kc + (int64_t)h * p.kv_sh * 2;
  const uint8_t* vbase = p.vc + (int64_t)h * p.kv_sh * 2;
  const int64_t chunk_bytes = p.kv_sc * 2;
  const int tok_bytes = p.kv_st * 2;

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
      const int qi = n >> p.g_shift, u = n & (G - 1);
      if (qi < nq) {
        uint16_t* o = p.out + (int64_t)(q_begin + q0 + qi) * p.o_st + (int64_t)(h * G + u) * p.o_sh + 4 * DV * g;
        for (int i = 0; i < 4 * DV; i += 4) st8(o + i, make_uint2(0, 0));
      }
    }
    return;
  }

  // K / V staging registers of one tile of 16*NT keys; the loop is software pipelined on them
  // (K of the next tile is requested once all scores of this one exist, V once P.V is done).
  uint4 kf[NT][KS];
  uint4 vf16[NT][4];
  uint2 vf8[NT][4];
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
      const uint8_t* vc = vbase + (int64_t)pc * chunk_bytes;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint8_t* vrow = vc + (min(T0 + 4 * g + j, last) - ci * p.chunk) * tok_bytes + DV * m16 * 2;
        if (HD == 128) vf16[u][j] = ld16(vrow);
        else vf8[u][j] = ld8(vrow);
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
        for (int kk = 0; kk < KS; ++kk) sacc = mfma_16x16x32(kf[u][kk], qf[nt][kk], sacc);
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
        pf[nt][u] = make_uint2(pack_bf16x2(pv[0], pv[1]), pack_bf16x2(pv[2], pv[3]));
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
      if constexpr (HD == 128) {
        const uint32_t* r0 = reinterpret_cast<const uint32_t*>(&vf16[u][0]);
        const uint32_t* r1 = reinterpret_cast<const uint32_t*>(&vf16[u][1]);
        const uint32_t* r2 = reinterpret_cast<const uint32_t*>(&vf16[u][2]);
        const uint32_t* r3 = reinterpret_cast<const uint32_t*>(&vf16[u][3]);
#pragma unroll
        for (int pr = 0; pr < 4; ++pr) {
          vt[2 * pr] = make_uint2(low_halves(r1[pr], r0[pr]), low_halves(r3[pr], r2[pr]));
          vt[2 * pr + 1] = make_uint2(high_halves(r1[pr], r0[pr]), high_halves(r3[pr], r2[pr]));
        }
      } else {
        const uint2 a = vf8[u][0], b = vf8[u][1], c = vf8[u][2], d = vf8[u][3];
        vt[0] = make_uint2(low_halves(b.x, a.x), low_halves(d.x, c.x));
        vt[1] = make_uint2(high_halves(b.x, a.x), high_halves(d.x, c.x));
        vt[2] = make_uint2(low_halves(b.y, a.y), low_halves(d.y, c.y));
        vt[3] = make_uint2(high_halves(b.y, a.y), high_halves(d.y, c.y));
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
            acc[nt][e] = mfma_16x16x32(make_uint4(va[e].x, va[e].y, vb[e].x, vb[e].y), pp, acc[nt][e]);
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
          for (int e = 0; e < DV; ++e) acc[nt][e] = mfma_16x16x16(vt[e], pf[nt][u], acc[nt][e]);
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
    const int qi = n >> p.g_shift, u = n & (G - 1);
    if (qi < nq) {
      uint16_t* o = p.out + (int64_t)(q_begin + q0 + qi) * p.o_st + (int64_t)(h * G + u) * p.o_sh + 4 * DV * g;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if constexpr (DV == 8) {
          st16(o + 8 * i, make_uint4(pack_bf16x2(acc[nt][0][i] * inv, acc[nt][1][i] * inv),
                                     pack_bf16x2(acc[nt][2][i] * inv, acc[nt][3][i] * inv),
                                     pack_bf16x2(acc[nt][4][i] * inv, acc[nt][5][i] * inv),
                                     pack_bf16x2(acc[nt][6][i] * inv, acc[nt][7][i] * inv)));
        } else {
          st8(o + 4 * i, make_uint2(pack_bf16x2(acc[nt][0][i] * inv, acc[nt][1][i] * inv),
                                    pack_bf16x2(acc[nt][2][i] * inv, acc[nt][3][i] * inv)));
        }
      }
    }
  }
}


// ---------------------------------------------------------------------------------------------
// LDS-shared variant (head_dim 128): 8 waves x 48 rows = 384 rows per workgroup.  Each 32-key
// K tile and V tile is fetched from HBM/L2 once per workgroup (one 16-byte piece per thread),
// staged row-major in LDS with a 272-byte pitch (conflict-free for both read patterns), double
// buffered with one barrier per tile; the waves read their MFMA operands from LDS.  The tile for
// step t+1 is in flight in registers while step t computes.
// ---------------------------------------------------------------------------------------------
constexpr int kLdsPitch = 272;   // bytes per staged row (256 + 16 padding)

// NQ = 16-row tiles per wave, NT = 16-key sub-tiles per staged tile (2 or 4).
template <int NQ, int NT>
__global__ __launch_bounds__(512, 2) void paged_prefill_lds_kernel(PrefillParams p) {
  constexpr int HD = 128, KS = 4, DV = 8, WAVES = 8;
  constexpr int kLdsTile = 16 * NT;  // keys per staged tile
  constexpr int LP = NT / 2;         // loader passes (512 threads fetch 32 rows per pass)
  static_assert(NT == 2 || NT == 4, "staged tile of 32 or 64 keys");
  __shared__ __attribute__((aligned(16))) uint8_t Ks[2][kLdsTile * kLdsPitch];
  __shared__ __attribute__((aligned(16))) uint8_t Vs[2][kLdsTile * kLdsPitch];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int m16 = lane & 15, g = lane >> 4;
  const int h = blockIdx.y;
  const int G = p.G;
  const int BQ = (16 * NQ) >> p.g_shift;  // query tokens per wave
  const int SBQ = WAVES * BQ;             // query tokens per workgroup

  if (blockIdx.x == 0) {
    const int tq = p.cu_q[p.R];
    const int per_row = G * HD;
    for (int64_t i = (int64_t)tid * 8; i < (int64_t)(p.T - tq) * per_row; i += 512 * 8) {
      const int row = (int)(i / per_row), e = (int)(i - (int64_t)row * per_row);
      st16(p.out + (int64_t)(tq + row) * p.o_st + (int64_t)(h * G + e / HD) * p.o_sh + (e % HD), make_uint4(0, 0, 0, 0));
    }
  }

  const int sb = blockIdx.x;
  int lo = 0, hi = p.R - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (p.cu_q[mid] / SBQ + mid <= sb) lo = mid; else hi = mid - 1;
  }
  const int r = lo;
  const int q_begin = p.cu_q[r];
  const int Lq = p.cu_q[r + 1] - q_begin;
  const int q0_wg = (sb - (q_begin / SBQ + r)) * SBQ;
  // Everything up to here is uniform over the workgroup: nobody is left behind at a barrier.
  if (q0_wg >= Lq) return;
  if (p.skip_single && Lq == 1) return;
  const int Lk = p.lens[r];
  const int shift = Lk - Lq;
  const int last = Lk - 1;
  const int kend_wg = min(Lk, shift + min(q0_wg + SBQ, Lq));  // keys some row of the workgroup sees

  const int q0 = q0_wg + wave * BQ;
  const int nq = max(0, min(BQ, Lq - q0));      // valid query tokens of this wave (may be 0)
  const int kend = nq > 0 ? min(Lk, shift + q0 + nq) : 0;
  const int ntiles = (nq * G + 15) >> 4;

  uint4 qf[NQ][KS];
  int qpos[NQ];
#pragma unroll
  for (int nt = 0; nt < NQ; ++nt) {
    const int n = 16 * nt + m16;
    const int qi = n >> p.g_shift, u = n & (G - 1);
    const bool valid = qi < nq;
    qpos[nt] = valid ? shift + q0 + qi : last;
    const uint16_t* qrow = p.q + (int64_t)(q_begin + q0 + qi) * p.q_st + (int64_t)(h * G + u) * p.q_sh;
#pragma unroll
    for (int kk = 0; kk < KS; ++kk)
      qf[nt][kk] = valid ? ld16(qrow + 32 * kk + 8 * g) : make_uint4(0, 0, 0, 0);
  }

  float m_run[NQ], l_run[NQ];
  f32x4_t acc[NQ][DV];
#pragma unroll
  for (int nt = 0; nt < NQ; ++nt) {
    m_run[nt] = -INFINITY;
    l_run[nt] = 0.f;
#pragma unroll
    for (int e = 0; e < DV; ++e) acc[nt][e] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }

  if (kend_wg > 0) {
    const uint8_t* kbase = p.kc + (int64_t)h * p.kv_sh * 2;
    const uint8_t* vbase = p.vc + (int64_t)h * p.kv_sh * 2;
    const int64_t chunk_bytes = p.kv_sc * 2;
    const int tok_bytes = p.kv_st * 2;
    // loader role of this thread: one 16-byte piece of one key row, for K and for V
    const int lkey = tid >> 4, lpiece = tid & 15;
    const int lds_off = lkey * kLdsPitch + lpiece * 16;
    uint4 kreg[LP], vreg[LP];
    auto gload = [&](int T) {
#pragma unroll
      for (int lp = 0; lp < LP; ++lp) {
        const int tok = min(T + 32 * lp + lkey, last);
        const int ci = (int)(((uint64_t)(uint32_t)tok * p.chunk_magic) >> 40);
        const int pc = p.bt[(int64_t)r * p.bt_stride + ci];
        const int64_t off = (int64_t)pc * chunk_bytes + (int64_t)(tok - ci * p.chunk) * tok_bytes + lpiece * 16;
        kreg[lp] = ld16(kbase + off);
        vreg[lp] = ld16(vbase + off);
      }
    };
    auto lstore = [&](int buf) {
#pragma unroll
      for (int lp = 0; lp < LP; ++lp) {
        *reinterpret_cast<uint4*>(&Ks[buf][lds_off + 32 * lp * kLdsPitch]) = kreg[lp];
        *reinterpret_cast<uint4*>(&Vs[buf][lds_off + 32 * lp * kLdsPitch]) = vreg[lp];
      }
    };
    const int full_until = shift + q0;
    const float scale = p.scale_log2;

    gload(0);
    lstore(0);
    __syncthreads();
    int buf = 0;
    for (int T = 0; T < kend_wg; T += kLdsTile, buf ^= 1) {
      const bool more = T + kLdsTile < kend_wg;  // workgroup-uniform
      if (more) gload(T + kLdsTile);
      if (T < kend) {  // wave-uniform: this wave still has visible keys in the tile
        const uint8_t* ks = Ks[buf];
        const uint8_t* vs = Vs[buf];
        // ---- S^T = K Q^T ---------------------------------------------------------------
        f32x4_t s[NQ][NT];
#pragma unroll
        for (int u = 0; u < NT; ++u) {
          uint4 kf[KS];
#pragma unroll
          for (int kk = 0; kk < KS; ++kk)
            kf[kk] = lds_ld16(ks + (16 * u + m16) * kLdsPitch + (32 * kk + 8 * g) * 2);
#pragma unroll
          for (int nt = 0; nt < NQ; ++nt) {
            if (nt >= ntiles) break;
            f32x4_t sacc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kk = 0; kk < KS; ++kk) sacc = mfma_16x16x32(kf[kk], qf[nt][kk], sacc);
            s[nt][u] = sacc;
          }
        }
        // ---- online softmax ---------------------------------------------------------------
        const bool need_mask = T + kLdsTile - 1 > full_until;
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
            pf[nt][u] = make_uint2(pack_bf16x2(pv[0], pv[1]), pack_bf16x2(pv[2], pv[3]));
          }
          l_run[nt] = l_run[nt] * alpha + psum;
          if (__builtin_amdgcn_ballot_w64(alpha != 1.f)) {
#pragma unroll
            for (int e = 0; e < DV; ++e) {
              acc[nt][e][0] *= alpha; acc[nt][e][1] *= alpha; acc[nt][e][2] *= alpha; acc[nt][e][3] *= alpha;
            }
          }
        }
        // ---- O^T += V^T P^T (k = 32: two 16-key sub-tiles per mfma) ------------------------
#pragma unroll
        for (int up = 0; up < NT; up += 2) {
          uint4 va[4], vb[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            va[j] = lds_ld16(vs + (16 * up + 4 * g + j) * kLdsPitch + 16 * m16);
            vb[j] = lds_ld16(vs + (16 * up + 16 + 4 * g + j) * kLdsPitch + 16 * m16);
          }
          const uint32_t* a0 = reinterpret_cast<const uint32_t*>(&va[0]);
          const uint32_t* a1 = reinterpret_cast<const uint32_t*>(&va[1]);
          const uint32_t* a2 = reinterpret_cast<const uint32_t*>(&va[2]);
          const uint32_t* a3 = reinterpret_cast<const uint32_t*>(&va[3]);
          const uint32_t* b0 = reinterpret_cast<const uint32_t*>(&vb[0]);
          const uint32_t* b1 = reinterpret_cast<const uint32_t*>(&vb[1]);
          const uint32_t* b2 = reinterpret_cast<const uint32_t*>(&vb[2]);
          const uint32_t* b3 = reinterpret_cast<const uint32_t*>(&vb[3]);
#pragma unroll
          for (int pr = 0; pr < 4; ++pr) {
            const uint4 lo4 = make_uint4(low_halves(a1[pr], a0[pr]), low_halves(a3[pr], a2[pr]),
                                         low_halves(b1[pr], b0[pr]), low_halves(b3[pr], b2[pr]));
            const uint4 hi4 = make_uint4(high_halves(a1[pr], a0[pr]), high_halves(a3[pr], a2[pr]),
                                         high_halves(b1[pr], b0[pr]), high_halves(b3[pr], b2[pr]));
#pragma unroll
            for (int nt = 0; nt < NQ; ++nt) {
              if (nt >= ntiles) break;
              const uint4 pp = make_uint4(pf[nt][up].x, pf[nt][up].y, pf[nt][up + 1].x, pf[nt][up + 1].y);
              acc[nt][2 * pr] = mfma_16x16x32(lo4, pp, acc[nt][2 * pr]);
              acc[nt][2 * pr + 1] = mfma_16x16x32(hi4, pp, acc[nt][2 * pr + 1]);
            }
          }
        }
      }
      if (more) lstore(buf ^ 1);
      __syncthreads();
    }
  }

  // ---- epilogue (rows of a request without keys get zeros: l_tot == 0) -------------------
#pragma unroll
  for (int nt = 0; nt < NQ; ++nt) {
    float l_tot = l_run[nt] + xor16(l_run[nt]);
    l_tot += xor32(l_tot);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    const int n = 16 * nt + m16;
    const int qi = n >> p.g_shift, u = n & (G - 1);
    if (qi < nq) {
      uint16_t* o = p.out + (int64_t)(q_begin + q0 + qi) * p.o_st + (int64_t)(h * G + u) * p.o_sh + 4 * DV * g;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        st16(o + 8 * i, make_uint4(pack_bf16x2(acc[nt][0][i] * inv, acc[nt][1][i] * inv),
                                   pack_bf16x2(acc[nt][2][i] * inv, acc[nt][3][i] * inv),
                                   pack_bf16x2(acc[nt][4][i] * inv, acc[nt][5][i] * inv),
                                   pack_bf16x2(acc[nt][6][i] * inv, acc[nt][7][i] * inv)));
    }
  }
}

}  // namespace mi

using namespace mi;

extern "C" int64_t mi_prefill_workspace_bytes(int32_t T, int32_t R, int32_t Hq, int32_t Hkv,
                                              int32_t head_dim, int32_t max_kv_len,
                                              int32_t split_tokens) {
  (void)T;
  // Only the one-row (decode) requests of a mixed batch need scratch: they are streamed by the
  // decode kernels, whose partials live here.
  return mi_decode_workspace_bytes(R, Hq, Hkv, head_dim, 16, max_kv_len, split_tokens);
}

extern "C" int mi_paged_prefill_attention(
    const void* q, int64_t q_stride_tok, int64_t q_stride_head, const void* k_cache,
    const void* v_cache, int64_t kv_stride_chunk, int64_t kv_stride_tok, int64_t kv_stride_head,
    const int32_t* block_table, int64_t bt_stride, const int32_t* cu_seqlens_q,
    const int32_t* kv_lens, void* out, int64_t o_stride_tok, int64_t o_stride_head,
    void* workspace, int64_t workspace_bytes, int32_t T, int32_t R, int32_t Hq, int32_t Hkv,
    int32_t head_dim, int32_t chunk_tokens, int32_t max_kv_len, int32_t split_tokens,
    float softmax_scale, void* stream) {
  (void)max_kv_len;
  if (T == 0 || R == 0) return MI_OK;
  if (!q || !k_cache || !v_cache || !block_table || !cu_seqlens_q || !kv_lens || !out)
    return mi_fail(MI_ERR_NULL, "mi_paged_prefill_attention: null pointer argument");
  if (T < 0 || R < 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv || Hkv > 65535)
    return mi_fail(MI_ERR_SHAPE, "mi_paged_prefill_attention: need T, R >= 0 and Hq a multiple of Hkv");
  const int G = Hq / Hkv;
  if (G > 16 || (G & (G - 1)))
    return mi_fail(MI_ERR_UNSUPPORTED, "mi_paged_prefill_attention: query heads per KV head must be 1, 2, 4, 8 or 16");
  if (head_dim != 64 && head_dim != 128)
    return mi_fail(MI_ERR_UNSUPPORTED, "mi_paged_prefill_attention: head_dim must be 64 or 128");
  if (chunk_tokens <= 0 || chunk_tokens % 16)
    return mi_fail(MI_ERR_SHAPE, "mi_paged_prefill_attention: chunk size must be a positive multiple of 16");
  if (((uintptr_t)q | (uintptr_t)k_cache | (uintptr_t)v_cache | (uintptr_t)out) & 15)
    return mi_fail(MI_ERR_ALIGN, "mi_paged_prefill_attention: q/k/v/out must be 16-byte aligned");
  if ((q_stride_tok | q_stride_head | o_stride_tok | o_stride_head | kv_stride_chunk | kv_stride_tok | kv_stride_head) % 8)
    return mi_fail(MI_ERR_ALIGN, "mi_paged_prefill_attention: strides must keep rows 16-byte aligned");
  if (kv_stride_tok * (int64_t)chunk_tokens * 2 >= (int64_t)1 << 31)
    return mi_fail(MI_ERR_SHAPE, "mi_paged_prefill_attention: one chunk must span less than 2 GiB");

  PrefillParams p;
  p.q = (const uint16_t*)q; p.q_st = q_stride_tok; p.q_sh = q_stride_head;
  p.kc = (const uint8_t*)k_cache; p.vc = (const uint8_t*)v_cache;
  p.kv_sc = kv_stride_chunk; p.kv_st = (int32_t)kv_stride_tok; p.kv_sh = (int32_t)kv_stride_head;
  p.bt = block_table; p.bt_stride = bt_stride; p.cu_q = cu_seqlens_q; p.lens = kv_lens;
  p.out = (uint16_t*)out; p.o_st = o_stride_tok; p.o_sh = o_stride_head;
  p.T = T; p.R = R; p.Hq = Hq; p.Hkv = Hkv; p.G = G;
  p.g_shift = 0;
  while ((1 << p.g_shift) < G) ++p.g_shift;
  p.chunk = chunk_tokens;
  p.chunk_magic = (((uint64_t)1 << 40) + chunk_tokens - 1) / chunk_tokens;
  p.scale_log2 = softmax_scale * 1.4426950408889634f;
  // With a workspace, one-row requests go through the bandwidth-optimised decode kernels.
  p.skip_single = workspace != nullptr;

  hipStream_t st = (hipStream_t)stream;
  if (!(softmax_scale > 0.f)) return mi_fail(MI_ERR_SHAPE, "mi_paged_prefill_attention: softmax_scale must be positive");
  const int lds_tiles = mi_tuning().prefill_lds_row_tiles;  // 0 = register-only kernel
  if (head_dim == 128 && lds_tiles > 0) {
    const int rows = 8 * 16 * (lds_tiles == 2 ? 2 : 3);
    const int sbq_lds = rows / G;
    dim3 lgrid((T + sbq_lds - 1) / sbq_lds + R, Hkv);
    const bool wide = mi_tuning().prefill_tile_subtiles == 4;  // 64-key staged tiles
    hipEvent_t ev_a, ev_b;
    const bool timed = mi_profile_next(&ev_a, &ev_b);
    if (timed) hipEventRecord(ev_a, st);
    if (lds_tiles == 2 && wide) hipLaunchKernelGGL((paged_prefill_lds_kernel<2, 4>), lgrid, dim3(512), 0, st, p);
    else if (lds_tiles == 2) hipLaunchKernelGGL((paged_prefill_lds_kernel<2, 2>), lgrid, dim3(512), 0, st, p);
    else hipLaunchKernelGGL((paged_prefill_lds_kernel<3, 2>), lgrid, dim3(512), 0, st, p);  // (48 rows: 32-key tiles only)
    if (timed) hipEventRecord(ev_b, st);
    int rc0 = mi_check_launch("mi_paged_prefill_attention");
    if (rc0 != MI_OK || !p.skip_single) return rc0;
    return launch_paged_decode(q, q_stride_tok, q_stride_head, k_cache, v_cache, kv_stride_chunk, kv_stride_tok,
                               kv_stride_head, block_table, bt_stride, kv_lens, cu_seqlens_q, out, o_stride_tok,
                               o_stride_head, workspace, workspace_bytes, R, Hq, Hkv, head_dim, chunk_tokens,
                               split_tokens, softmax_scale, MI_KV_BF16, nullptr, nullptr, stream);
  }
  const int nq = mi_tuning().prefill_row_tiles == 4 ? 4 : 2;
  const int sbq = 256 / G;  // query tokens per workgroup (256 rows)
  dim3 grid((T + sbq - 1) / sbq + R, Hkv), block(64 * (16 / nq));
  // register-only kernel (head_dim 64, or LDS variant switched off): 16 or 32 keys per iteration
  const int nt = mi_tuning().prefill_tile_subtiles == 1 ? 1 : 2;
#define MI_LAUNCH_PREFILL(HD_, NT_)                                                                        \
  do {                                                                                                     \
    if (nq == 4) hipLaunchKernelGGL((paged_prefill_kernel<HD_, NT_, 4>), grid, block, 0, st, p);           \
    else hipLaunchKernelGGL((paged_prefill_kernel<HD_, NT_, 2>), grid, block, 0, st, p);                   \
  } while (0)
  if (head_dim == 128) {
    if (nt == 1) MI_LAUNCH_PREFILL(128, 1);
    else MI_LAUNCH_PREFILL(128, 2);
  } else {
    if (nt == 1) MI_LAUNCH_PREFILL(64, 1);
    else MI_LAUNCH_PREFILL(64, 2);
  }
#undef MI_LAUNCH_PREFILL
  int rc = mi_check_launch("mi_paged_prefill_attention");
  if (rc != MI_OK || !p.skip_single) return rc;
  return launch_paged_decode(q, q_stride_tok, q_stride_head, k_cache, v_cache, kv_stride_chunk, kv_stride_tok,
                             kv_stride_head, block_table, bt_stride, kv_lens, cu_seqlens_q, out, o_stride_tok,
                             o_stride_head, workspace, workspace_bytes, R, Hq, Hkv, head_dim, chunk_tokens,
                             split_tokens, softmax_scale, MI_KV_BF16, nullptr, nullptr, stream);
}
