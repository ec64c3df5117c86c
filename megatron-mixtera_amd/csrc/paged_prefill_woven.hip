// Paged varlen causal attention tiles for chunked prefill on gfx950: one instruction stream per wavefront.
//
// Serves the same call as the two-phase tile kernel of paged_prefill.hip -- flash_attn_varlen_func(..., causal=True,
// block_table=...) from Attention.flash_decode_and_prefill (megatron/core/transformer/attention.py:546-557) -- for
// head_dim 128 over a 16-bit cache whose chunk size is a multiple of 64.
//
// A workgroup of 8 wavefronts (two per SIMD, 256 registers each) takes 256 consecutive (query token, head-in-group)
// rows of one (request, KV head), 32 rows per wavefront, and walks the keys in staged tiles of 64.  There are no
// matrix / vector phases and no per-phase barriers: every wavefront runs the whole tile pipeline in ONE stream, cut
// into 32-key steps and software-pipelined so that three independent chains are always open --
//     products    S^T(step s+1) = K Q^T          and  O^T += V^T P^T(step s-1)     (matrix cores)
//     vector ALU  P(step s) = exp2(S(step s) * scale - reference)  and the running maximum of S(step s+1)
//     LDS         the fragments of the products three fragments ahead
// -- and the source orders them product pair / fragment read / a few vector instructions, pinned by scheduling
// barriers.  Whatever one wavefront of a SIMD cannot issue (a product waiting for the matrix core, a wait for LDS),
// the SIMD's other wavefront fills with its own stream; nothing but the one barrier per tile keeps them in step.
//
// Staging: a 64-key tile goes straight from memory into LDS (buffer loads with the LDS destination: no staging
// registers, no LDS stores), as 18 instructions of 64 lanes x 16 bytes over a line of 64 rows x 18 pieces (288-byte
// row pitch, the last two pieces of a row are padding).  The loads go through a buffer descriptor that covers the
// tile's rows up to the request's last key: rows beyond it arrive as zeros (their probabilities are masked to zero,
// and zero times a stale value must not be NaN).  Key tiles are double-buffered and value tiles triple-buffered
// (values are multiplied one tile after their keys); the loads of the next pair are issued right after the tile's
// barrier and are waited for at the next one.
//
// Softmax: exponentials are taken against a per-row reference that moves only when a score exceeds it by a window
// (2^30 as the largest probability with bf16 operands, 2^8 with fp16); the row sums come out of the matrix cores
// (an all-ones A fragment).  A move of the reference rescales the accumulators, the sums and the one step of
// probabilities that is still waiting for its product.
#include <type_traits>

#include "mi_common.h"
#include "mi_capi_internal.h"
#include "paged_prefill_params.h"

namespace mi {

constexpr int kWvTile = 64;                      // keys per staged tile
constexpr int kWvPitch = 288;                    // LDS bytes per staged row (256 + 32: conflict-free fragment reads)
constexpr int kWvPieces = kWvPitch / 16;         // 16-byte pieces per staged row
constexpr int kWvLoads = kWvTile * kWvPieces / 64;  // direct loads (64 lanes x 16 bytes) per tile: 18
constexpr int kWvBuf = kWvLoads * 1024;          // bytes per tile buffer
constexpr int kWvDepth = 1;                      // tiles between the issue of a tile's loads and the barrier that needs them
constexpr int kWvAhead = 3;                      // fragments requested ahead of their products (the stream: 16 per 32-key slot)
constexpr int kWvRing = 4;                       // fragment registers: fragment n lives in slot n % kWvRing
static_assert(kWvAhead < kWvRing && kWvAhead <= 8 && 16 % kWvRing == 0, "next slot's key fragments are requested after the tile's barrier");
constexpr bool wv_piece_division_ok() {
  for (unsigned u = 0; u < 64u * kWvLoads; ++u)
    if (((u * 3641u) >> 16) != u / 18u) return false;
  return true;
}
static_assert((kWvDepth == 1 || kWvDepth == 2) && kWvPieces == 18 && kWvBuf == kWvTile * kWvPitch && wv_piece_division_ok(), "piece -> (row, column) by multiplication");

template <bool SPLIT, bool F16>
__global__ __launch_bounds__(512, 2) void paged_prefill_woven_kernel(PrefillParams p) {
  constexpr int HD = 128, KS = HD / 32, DV = HD / 16, NQ = 2, WAVES = 8;
  constexpr int PITCH = kWvPitch, BUF = kWvBuf;
  // DEPTH: how many tiles ahead of their barrier the loads of a tile pair are issued.  Key tile t lives in
  // Ks[t % KBUFS], value tile t in Vs[(t + 1) % VBUFS] (values are multiplied one tile after their keys).
  constexpr int DEPTH = kWvDepth, KBUFS = DEPTH + 1, VBUFS = DEPTH + 2;
  __shared__ __attribute__((aligned(16))) uint8_t Ks[KBUFS][BUF];
  __shared__ __attribute__((aligned(16))) uint8_t Vs[VBUFS][BUF];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int m16 = lane & 15, g = lane >> 4;
  const int HV = p.Hkv * p.parts;  // workgroups along the heads
  const HeadSlice hs = head_slice(p, blockIdx.x % HV);
  const int h = hs.h, G = hs.G, g_magic = hs.g_magic, hq0 = hs.hq0;
  const int rank = blockIdx.x / HV;
  const int BQ = ((16 * NQ) * p.g_magic) >> 16;  // query tokens per wavefront (the widest head slice's count)
  const int SBQ = WAVES * BQ;

  // rows beyond the last request (token padding of the batch) are defined as zeros
  if (rank == 0 && (!SPLIT || blockIdx.y == 0)) {
    const int tq = p.cu_q[p.R];
    const int per_row = G * HD;
    for (int64_t i = (int64_t)tid * 8; i < (int64_t)(p.T - tq) * per_row; i += 512 * 8) {
      const int row = (int)(i / per_row), e = (int)(i - (int64_t)row * per_row);
      st16(p.out + (int64_t)(tq + row) * p.o_st + (int64_t)(hq0 + e / HD) * p.o_sh + (e % HD), make_uint4(0, 0, 0, 0));
    }
  }

  // Query block sb of the batch: request r's blocks are cu_q[r] / SBQ + r onward; last block (most keys) first.
  // The search takes 64 candidates per pass, one per lane (a pass is one trip to memory, and nothing of the
  // workgroup's work can start before its request is known): the last request whose first block is not past this
  // one.  The same pass fetches what is needed of that request.
  const int sb = (int)(gridDim.x / HV) - 1 - rank;
  int r = 0, q_begin = 0, q_end = 0, Lk = 0;
  for (int n = p.R;;) {  // the answer lies in [r, r + n)
    const int stride = (n + 63) >> 6;
    const int idx = r + lane * stride;
    const bool in = lane * stride < n;
    const int cq = in ? p.cu_q[idx] : 0, cq1 = in ? p.cu_q[idx + 1] : 0, len = in ? p.lens[idx] : 0;
    const int c = __builtin_popcountll(__builtin_amdgcn_ballot_w64(in && cq / SBQ + idx <= sb)) - 1;  // >= 0: the first candidate always qualifies
    r += c * stride;
    n = min(stride, n - c * stride);
    if (stride == 1) {
      q_begin = __builtin_amdgcn_readlane(cq, c);
      q_end = __builtin_amdgcn_readlane(cq1, c);
      Lk = __builtin_amdgcn_readlane(len, c);
      break;
    }
  }
  const int Lq = q_end - q_begin;
  const int q0_wg = (sb - (q_begin / SBQ + r)) * SBQ;
  if (q0_wg >= Lq) return;  // workgroup-uniform
  if (p.skip_single && Lq == 1) return;
  const int shift = Lk - Lq;
  const int last = Lk - 1;
  const int kend_wg = min(Lk, shift + min(q0_wg + SBQ, Lq));
  const int ntl_all = (kend_wg + kWvTile - 1) / kWvTile;  // staged tiles the rows of this workgroup can see
  const int n_split = SPLIT ? (int)gridDim.y : 1, split = SPLIT ? (int)blockIdx.y : 0;
  // (workgroup-uniform values the tile loop's bookkeeping is built from: held in scalar registers)
  const int tb = __builtin_amdgcn_readfirstlane(SPLIT ? (int)((int64_t)ntl_all * split / n_split) : 0);
  const int te = __builtin_amdgcn_readfirstlane(SPLIT ? (int)((int64_t)ntl_all * (split + 1) / n_split) : ntl_all);
  const int ntl = te - tb;  // this workgroup walks tiles [tb, te)

  const int q0 = q0_wg + wave * BQ;
  const int nq = max(0, min(BQ, Lq - q0));
  const int full_until = shift + q0;  // keys up to here are visible to every valid row of the wavefront

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

  float m_run[NQ], neg_run[NQ], mwin[NQ];
  f32x4_t acc[NQ][DV], accl[NQ];
#pragma unroll
  for (int nt = 0; nt < NQ; ++nt) {
    m_run[nt] = -INFINITY;
    mwin[nt] = -INFINITY;
    neg_run[nt] = 0.f;
    accl[nt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int e = 0; e < DV; ++e) acc[nt][e] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }

  if (ntl > 0) {
#define MI_SB() __builtin_amdgcn_sched_barrier(0)
    auto uniform64 = [](uint64_t x) {
      return ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(x >> 32)) << 32) | (uint32_t)__builtin_amdgcn_readfirstlane((int)x);
    };
    // (48-bit addresses: what a descriptor's second word holds above them are its stride and swizzle fields)
    const uint64_t kbase = uniform64((uint64_t)(uintptr_t)(p.kc + (int64_t)h * p.kv_sh * 2)) & 0xffffffffffffull;
    const uint64_t vbase = uniform64((uint64_t)(uintptr_t)(p.vc + (int64_t)h * p.kv_sh * 2)) & 0xffffffffffffull;
    const int last_key = __builtin_amdgcn_readfirstlane(last);
    const int64_t chunk_bytes = p.kv_sc * 2;
    const int tok_bytes = p.kv_st * 2;
    const int tiles_per_chunk = p.chunk / kWvTile;
    const int tile_bytes = kWvTile * tok_bytes;
    const int32_t* bt_row = p.bt + (int64_t)r * p.bt_stride;
    const uint32_t ks_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)&Ks[0][0];
    const uint32_t vs_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)&Vs[0][0];

    // ---- this wavefront's five direct loads of a tile pair {key tile, value tile} -------------------------------
    // Load k of the pair's 36 (0-17: the key tile's line, 18-35: the value tile's) belongs to wavefront k % 8; the
    // fifth load of wavefronts 4-7 repeats their fourth, so that every wavefront issues five per tile.
    // Loads 0 and 1 are key loads and loads 3 and 4 value loads for every wavefront; load 2 is a key load for
    // wavefronts 0 and 1 only.
    static_assert(kWvLoads == 18, "which of a wavefront's five loads belong to the key tile");
    uint32_t ld_off[5];   // per lane: where its piece of the load comes from, relative to the tile's first row
    uint32_t ld_dst[5];   // scalar: LDS offset of the load's 1 KiB inside its tile buffer
    const bool third_is_key = wave < 2;
#pragma unroll
    for (int i = 0; i < 5; ++i) {
      const int k = wave + 8 * i < 2 * kWvLoads ? wave + 8 * i : wave + 8 * i - 8;
      const bool is_key = k < kWvLoads;
      const int kp = is_key ? k : k - kWvLoads;
      ld_dst[i] = (uint32_t)__builtin_amdgcn_readfirstlane(1024 * kp);
      const uint32_t u = 64u * (uint32_t)kp + (uint32_t)lane;
      const uint32_t prow = (u * 3641u) >> 16, pcol = u - 18u * prow;
      ld_off[i] = prow * (uint32_t)tok_bytes + 16u * min(pcol, 15u);
    }
    // descriptor of a tile: its rows up to the request's last key (reads beyond return zeros)
    auto tile_rsrc = [&](uint64_t base, int64_t off, uint32_t nrec) {
      const uint64_t a = base + (uint64_t)off;
      u32x4_t rs;
      rs.x = (uint32_t)a;
      rs.y = (uint32_t)(a >> 32);
      rs.z = nrec;
      rs.w = 0x00020000u;
      return rs;
    };
    auto issue_load = [&](int i, const u32x4_t& rs_k, const u32x4_t& rs_v, uint32_t kdst, uint32_t vdst) {
      const bool is_key = i < 2 || (i == 2 && third_is_key);
      const u32x4_t rs = is_key ? rs_k : rs_v;
      const uint32_t m0 = (is_key ? kdst : vdst) + ld_dst[i];
      asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds" ::"s"(m0), "v"(ld_off[i]), "s"(rs)
                   : "memory", "m0");
    };
    // the tile cursor: all members wave-uniform; it sticks to the workgroup's last tile
    struct Cursor { int tile, ci, tin; };
    auto cursor_at = [&](int t) {
      Cursor c;
      c.tile = __builtin_amdgcn_readfirstlane(min(t, te - 1));
      c.ci = __builtin_amdgcn_readfirstlane(c.tile / tiles_per_chunk);
      c.tin = c.tile - c.ci * tiles_per_chunk;
      return c;
    };
    auto cursor_next = [&](Cursor& c) {
      const bool adv = c.tile + 1 < te;
      const bool wrap = adv && (c.tin + 1 == tiles_per_chunk);
      c.tile += adv ? 1 : 0;
      c.tin = wrap ? 0 : c.tin + (adv ? 1 : 0);
      c.ci += wrap ? 1 : 0;
    };
    auto tile_off = [&](const Cursor& c, int pc) { return (int64_t)pc * chunk_bytes + (int64_t)c.tin * tile_bytes; };
    auto tile_nrec = [&](const Cursor& c) { return (uint32_t)(min(last_key - c.tile * kWvTile, kWvTile - 1) + 1) * (uint32_t)tok_bytes; };
    // block-table entries by scalar loads the compiler does not see (a vector load in the tile loop would make it
    // wait on the vector-memory counter, i.e. for the direct loads in flight)
    auto bt_request = [&](int ci) {
      const int byte_off = 4 * ci;
      int pc;
      asm volatile("s_load_dword %0, %1, %2" : "=s"(pc) : "s"(bt_row), "s"(byte_off) : "memory");
      return pc;
    };
    auto bt_arrived = [&](int& pc) { asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(pc)::"memory"); };

    const float scale = p.scale_log2;
    const float win = (F16 ? 8.f : 30.f) / scale;
    const uint4 ones = make_uint4(ones2<F16>(), ones2<F16>(), ones2<F16>(), ones2<F16>());
    const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
    // per-lane starts of the fragment reads inside a tile buffer
    const uint8_t* const k_lane = &Ks[0][0] + m16 * PITCH + 16 * g;
    const uint8_t* const v_lane = &Vs[0][0] + (4 * g + (m16 >> 2)) * PITCH + 8 * (m16 & 3);

    // S[x]: scores of the even (x = 0) / odd (x = 1) 32-key steps, P[x]: their probabilities as the B operand
    f32x4_t S[2][NQ][2];
    uint4 P[2][NQ];
    constexpr int AHEAD = kWvAhead, RING = kWvRing;
    uint4 fr[RING];  // fragments in flight: fragment n of the stream lives in fr[n % RING]
#pragma unroll
    for (int nt = 0; nt < NQ; ++nt) {
      P[0][nt] = P[1][nt] = make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
      for (int u = 0; u < 2; ++u) S[0][nt][u] = S[1][nt][u] = f32x4_t{-INFINITY, -INFINITY, -INFINITY, -INFINITY};
    }

    auto read_k = [&](const uint8_t* ka, int half, int f) {  // key fragment f of a half tile: sub-tile f & 1, columns 32 (f >> 1)
      return *reinterpret_cast<const uint4*>(ka + (32 * half + 16 * (f & 1)) * PITCH + 64 * (f >> 1));
    };
    auto read_v = [&](const uint8_t* va, int half, int e) {  // transposed value fragment: 32 keys x output columns 16 e
      const uint2 a = lds_ld8_tr(va + 32 * half * PITCH + 32 * e), b = lds_ld8_tr(va + (32 * half + 16) * PITCH + 32 * e);
      return make_uint4(a.x, a.y, b.x, b.y);
    };
    // probabilities of two scores (chunk c of a step's 8 per lane): rows nt = c >> 2, sub-tile (c >> 1) & 1, pair c & 1
    auto exp_chunk = [&](const f32x4_t (&Sx)[NQ][2], uint4 (&Px)[NQ], int c) {
      const int nt = c >> 2, u = (c >> 1) & 1, q2 = 2 * (c & 1);
      const float p0 = fast_exp2(__builtin_fmaf(Sx[nt][u][q2], scale, neg_run[nt]));
      const float p1 = fast_exp2(__builtin_fmaf(Sx[nt][u][q2 + 1], scale, neg_run[nt]));
      const uint32_t w = pack2<F16>(p0, p1);
      const int d = 2 * u + (c & 1);
      if (d == 0) Px[nt].x = w; else if (d == 1) Px[nt].y = w; else if (d == 2) Px[nt].z = w; else Px[nt].w = w;
    };
    // the reference of some row has to move (rare): new reference, rescale of everything taken against the old one
    auto move_reference = [&](float (&tmax)[NQ], uint4 (&Ppend)[NQ]) {
#pragma unroll
      for (int nt = 0; nt < NQ; ++nt) {
        const float tm = rowgroup_max(tmax[nt]);
        const float m_raw = fmaxf(m_run[nt], tm);
        const float m_use = m_raw == -INFINITY ? 0.f : m_raw;
        const float alpha = fast_exp2((m_run[nt] - m_use) * scale);
        neg_run[nt] = -m_use * scale;
        m_run[nt] = m_raw;
        mwin[nt] = m_raw + win;
        if (__builtin_amdgcn_ballot_w64(alpha != 1.f)) {
#pragma unroll
          for (int e = 0; e < DV; ++e) {
            acc[nt][e][0] *= alpha; acc[nt][e][1] *= alpha; acc[nt][e][2] *= alpha; acc[nt][e][3] *= alpha;
          }
          accl[nt][0] *= alpha; accl[nt][1] *= alpha; accl[nt][2] *= alpha; accl[nt][3] *= alpha;
          auto rs = [&](uint32_t w) { return pack2<F16>(lo_to_f32<F16>(w) * alpha, hi_to_f32<F16>(w) * alpha); };
          Ppend[nt] = make_uint4(rs(Ppend[nt].x), rs(Ppend[nt].y), rs(Ppend[nt].z), rs(Ppend[nt].w));
        }
      }
    };

    // ---- one 32-key slot.  H: the half of the key tile whose scores are multiplied (into S[H]); the vector ALU turns
    // S[1-H] into P[1-H]; the value product takes P[H] and half H of the value tile before.  ka / va: this lane's
    // fragment starts in the key tile's and the value tile's buffers, ka_next in the next key tile's.  key0: position
    // of the first key of S[H] (MASK only).  at_barrier (H == 1): runs between the two groups of products.
    auto slot = [&](auto Hc, auto Mc, const uint8_t* ka, const uint8_t* ka_next, const uint8_t* va, int key0,
                    auto&& at_barrier, auto&& under_products) {
      constexpr int H = decltype(Hc)::value;
      constexpr bool MASK = decltype(Mc)::value;
      f32x4_t (&Sn)[NQ][2] = S[H];
      const f32x4_t (&Sx)[NQ][2] = S[1 - H];
      uint4 (&Px)[NQ] = P[1 - H];
      const uint4 (&Pv)[NQ] = P[H];
      // fragment n of the slot's stream: 0-7 key fragments, 8-15 value fragments, from 16 the next slot's first keys
      auto request = [&](int n) {
        if (n < 8) fr[n % RING] = read_k(ka, H, n);
        else if (n < 16) fr[n % RING] = read_v(va, H, n - 8);
        else fr[n % RING] = H == 0 ? read_k(ka, 1, n - 16) : read_k(ka_next, 0, n - 16);
      };
      // The probabilities of S[1-H], two scores ("chunk") at a time in three stages -- scale and subtract, exponential,
      // pack -- one stage of three different chunks per position, so that no instruction waits for the one before it:
      // position n holds stage one of chunk n, stage two of chunk n - 1, stage three of chunk n - 2.
      float xs[8][2], ps[8][2];
      auto exp_stages = [&](int n) {
        if (n >= 2 && n < 10) {
          const int c = n - 2, nt = c >> 2, d = 2 * ((c >> 1) & 1) + (c & 1);
          const uint32_t w = pack2<F16>(ps[c][0], ps[c][1]);
          if (d == 0) Px[nt].x = w; else if (d == 1) Px[nt].y = w; else if (d == 2) Px[nt].z = w; else Px[nt].w = w;
        }
        if (n >= 1 && n < 9) {
          ps[n - 1][0] = fast_exp2(xs[n - 1][0]);
          ps[n - 1][1] = fast_exp2(xs[n - 1][1]);
        }
        if (n < 8) {
          const int nt = n >> 2, u = (n >> 1) & 1, q2 = 2 * (n & 1);
          xs[n][0] = __builtin_fmaf(Sx[nt][u][q2], scale, neg_run[nt]);
          xs[n][1] = __builtin_fmaf(Sx[nt][u][q2 + 1], scale, neg_run[nt]);
        }
      };
      // scores: sub-tiles alternate, so a product meets its accumulator again four products later
#pragma unroll
      for (int n = 0; n < 8; ++n) {
        request(n + AHEAD);
        MI_SB();
        const int u = n & 1, kk = n >> 1;
        Sn[0][u] = mfma_16x16x32<F16>(fr[n % RING], qf[0][kk], kk ? Sn[0][u] : zero4);
        Sn[1][u] = mfma_16x16x32<F16>(fr[n % RING], qf[1][kk], kk ? Sn[1][u] : zero4);
        MI_SB();
        exp_stages(n);
        MI_SB();
      }
      if constexpr (H == 1) at_barrier();
      float tmax[NQ];
      int dpos[NQ];
      // values; beside them the last probabilities, then mask and maximum of the scores just multiplied
#pragma unroll
      for (int n = 8; n < 16; ++n) {
        request(n + AHEAD);
        MI_SB();
        const int e = n - 8;
        acc[0][e] = mfma_16x16x32<F16>(fr[n % RING], Pv[0], acc[0][e]);
        acc[1][e] = mfma_16x16x32<F16>(fr[n % RING], Pv[1], acc[1][e]);
        MI_SB();
        if (n < 10) exp_stages(n);
        if constexpr (H == 1) under_products(n - 8);
        if (n == 11 && MASK) {
          const int tok0 = key0 + 4 * g;
          dpos[0] = qpos[0] - tok0;
          dpos[1] = qpos[1] - tok0;
        }
        if (n >= 11 && n < 15) {  // rows (n - 11) >> 1 of the scores just multiplied, in two parts
          const int nt = (n - 11) >> 1, part = (n - 11) & 1;
          if (MASK && part == 0) {
            // (every masked score is out of the way before the first maximum is taken: a masked key's score in the
            // reference would cost fp16 probabilities their precision)
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
              for (int i = 0; i < 4; ++i)
                if (16 * u + i > dpos[nt]) Sn[nt][u][i] = -INFINITY;
          }
          // a chain of three-operand maxima
          if (MASK ? part == 1 : part == 0) {
            tmax[nt] = fmaxf(fmaxf(Sn[nt][0][0], Sn[nt][0][1]), Sn[nt][0][2]);
            tmax[nt] = fmaxf(fmaxf(tmax[nt], Sn[nt][0][3]), Sn[nt][1][0]);
          }
          if (part == 1) {
            tmax[nt] = fmaxf(fmaxf(tmax[nt], Sn[nt][1][1]), Sn[nt][1][2]);
            tmax[nt] = fmaxf(tmax[nt], Sn[nt][1][3]);
          }
        }
        MI_SB();
      }
      accl[0] = mfma_16x16x32<F16>(ones, Pv[0], accl[0]);
      accl[1] = mfma_16x16x32<F16>(ones, Pv[1], accl[1]);
      MI_SB();
      if (__builtin_amdgcn_ballot_w64(tmax[0] > mwin[0] || tmax[1] > mwin[1])) move_reference(tmax, Px);
      MI_SB();
    };

    // ---- prologue: clear the buffers (the value tile "before the first" must hold zeros), start the first tiles ----
    for (int i = tid * 16; i < KBUFS * BUF; i += 512 * 16) *reinterpret_cast<uint4*>(&Ks[0][0] + i) = make_uint4(0u, 0u, 0u, 0u);
    for (int i = tid * 16; i < VBUFS * BUF; i += 512 * 16) *reinterpret_cast<uint4*>(&Vs[0][0] + i) = make_uint4(0u, 0u, 0u, 0u);
    Cursor cur = cursor_at(tb + DEPTH + 1);
    int64_t off_first[DEPTH + 1];   // tiles tb .. tb + DEPTH, started here
    uint32_t nrec_first[DEPTH + 1];
#pragma unroll
    for (int i = 0; i <= DEPTH; ++i) {
      const Cursor c = cursor_at(tb + i);
      off_first[i] = tile_off(c, __builtin_amdgcn_readfirstlane(bt_row[c.ci]));
      nrec_first[i] = tile_nrec(c);
    }
    int pc_next = __builtin_amdgcn_readfirstlane(bt_row[cur.ci]);
    // (the query fragments count as used here: the compiler then waits for their loads now and not in the tile
    // loop, where a wait on the vector-memory counter would wait for the direct loads in flight as well)
#pragma unroll
    for (int nt = 0; nt < NQ; ++nt)
#pragma unroll
      for (int kk = 0; kk < KS; ++kk)
        asm volatile("" ::"v"(qf[nt][kk].x), "v"(qf[nt][kk].y), "v"(qf[nt][kk].z), "v"(qf[nt][kk].w));
    __syncthreads();  // the cleared buffers are in place before the first direct load can land
    int64_t off_prev;
    uint32_t nrec_prev;
    {
      const u32x4_t rk0 = tile_rsrc(kbase, off_first[0], nrec_first[0]);
#pragma unroll
      for (int i = 0; i < 5; ++i)
        if (i < 2 || (i == 2 && third_is_key)) issue_load(i, rk0, rk0, ks_lds, ks_lds);  // key tile 0 -> Ks[0]
#pragma unroll
      for (int t = 1; t <= DEPTH; ++t) {  // the pairs {key tile t -> Ks[t], value tile t - 1 -> Vs[t]}
        const u32x4_t rk = tile_rsrc(kbase, off_first[t], nrec_first[t]);
        const u32x4_t rv = tile_rsrc(vbase, off_first[t - 1], nrec_first[t - 1]);
#pragma unroll
        for (int i = 0; i < 5; ++i) issue_load(i, rk, rv, ks_lds + t * BUF, vs_lds + t * BUF);
      }
      off_prev = off_first[DEPTH];
      nrec_prev = nrec_first[DEPTH];
    }
    // key tile 0 has landed (this wavefront's share): only the DEPTH pairs issued after it may still be on their way
    if constexpr (DEPTH == 1) asm volatile("s_waitcnt vmcnt(5)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(10)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    MI_SB();

    const int t_mask = max(0, (full_until + 1) >> 6);              // first tile with a masked score for this wavefront
    const int jm = min(max(t_mask - tb, 0), ntl);                  // iterations [0, jm) need no mask
    int j = 0;
    int kbi = 0, vbi = 0;  // j % KBUFS, j % VBUFS
#pragma unroll
    for (int n = 0; n < AHEAD; ++n) fr[n] = read_k(k_lane, 0, n);

    // iteration j: scores of key tile j (Ks[j % KBUFS]), values of tile j-1 (Vs[j % VBUFS]); after its barrier key tile
    // j+1 and value tile j are in LDS, and the loads of key tile j+DEPTH+1 (into the buffer of key tile j, which every
    // wavefront has left) and value tile j+DEPTH (into the buffer of value tile j-2) set out under the products that follow.
    auto iteration = [&](auto Mc) {
      const int kb = kbi * BUF;
      const uint8_t* ka = k_lane + kb;
      const uint8_t* ka_next = k_lane + (kbi == KBUFS - 1 ? 0 : kbi + 1) * BUF;
      const uint8_t* va = v_lane + vbi * BUF;
      const int key0 = (tb + j) * kWvTile;
      u32x4_t rs_k, rs_v;
      const uint32_t kdst = ks_lds + (uint32_t)kb;
      const uint32_t vdst = vs_lds + (uint32_t)((vbi == 0 ? VBUFS - 1 : vbi - 1) * BUF);  // (j - 1) % VBUFS
      slot(std::integral_constant<int, 0>{}, Mc, ka, ka_next, va, key0, [] {}, [](int) {});
      slot(std::integral_constant<int, 1>{}, Mc, ka, ka_next, va, key0 + 32,
           [&] {
             // this wavefront's share of key tile j+1 and value tile j has landed: only younger pairs are on their way
             if constexpr (DEPTH == 1) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
             else asm volatile("s_waitcnt vmcnt(5)" ::: "memory");
             __builtin_amdgcn_s_barrier();
             bt_arrived(pc_next);
             const int64_t off = tile_off(cur, pc_next);
             const uint32_t nrec = tile_nrec(cur);
             rs_k = tile_rsrc(kbase, off, nrec);
             rs_v = tile_rsrc(vbase, off_prev, nrec_prev);
             off_prev = off;
             nrec_prev = nrec;
             cursor_next(cur);
             pc_next = bt_request(cur.ci);
           },
           [&](int i) {
             if (i < 5) issue_load(i, rs_k, rs_v, kdst, vdst);
           });
      ++j;
      kbi = kbi == KBUFS - 1 ? 0 : kbi + 1;
      vbi = vbi == VBUFS - 1 ? 0 : vbi + 1;
    };
    for (; j < jm;) iteration(std::false_type{});
    for (; j < ntl;) iteration(std::true_type{});

    // ---- drain: the last two steps' values (tile ntl - 1 in Vs[ntl % VBUFS]); S[1] is masked and checked already ----
    {
      const uint8_t* va = v_lane + vbi * BUF;
      auto values = [&](int half, const uint4 (&Pv)[NQ]) {
#pragma unroll
        for (int e = 0; e < DV; ++e) {
          const uint4 a = read_v(va, half, e);
          acc[0][e] = mfma_16x16x32<F16>(a, Pv[0], acc[0][e]);
          acc[1][e] = mfma_16x16x32<F16>(a, Pv[1], acc[1][e]);
        }
        accl[0] = mfma_16x16x32<F16>(ones, Pv[0], accl[0]);
        accl[1] = mfma_16x16x32<F16>(ones, Pv[1], accl[1]);
      };
      values(0, P[0]);
#pragma unroll
      for (int c = 0; c < 8; ++c) exp_chunk(S[1], P[1], c);
      values(1, P[1]);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no direct load may still be on its way into this workgroup's LDS
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
      } else {  // a range without visible keys leaves zeros and -inf
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

void launch_prefill_woven(const PrefillParams& p, dim3 grid, bool f16, hipStream_t st) {
  const bool split = grid.y > 1;
  if (split && f16) hipLaunchKernelGGL((paged_prefill_woven_kernel<true, true>), grid, dim3(512), 0, st, p);
  else if (split) hipLaunchKernelGGL((paged_prefill_woven_kernel<true, false>), grid, dim3(512), 0, st, p);
  else if (f16) hipLaunchKernelGGL((paged_prefill_woven_kernel<false, true>), grid, dim3(512), 0, st, p);
  else hipLaunchKernelGGL((paged_prefill_woven_kernel<false, false>), grid, dim3(512), 0, st, p);
}

}  // namespace mi
