// Tail of a decode step: last-token gather, token sampling and the finished-request mask.
//
// What the reference does with torch ops after the forward pass
// (megatron/core/inference/text_generation_controllers/text_generation_controller.py:172-315,
// 519-530 and megatron/core/inference/contexts/dynamic_context.py:890-918):
//   * last_token_logits: rows  cumsum(request_query_lengths) - 1  of the `[T, V]` logits;
//   * sample_from_logits: argmax (top_k == 1), or  logits / temperature -> top-k filter (keep
//     values >= the k-th largest) or top-p filter (sort descending, keep the shortest prefix
//     whose softmax mass exceeds top_p) -> softmax -> one multinomial draw per row;
//   * active_request_mask = (sample != termination_id) & (sequence length + 1 < maximum length).
//
// Here a row is never sorted.  One workgroup of 16 wavefronts owns a row and finds the cut
// value of the filter by selection: a 256-bin histogram over the value range, then four 8-bit
// digit passes over the order-preserving integer image of the floats in the chosen bin (its
// members are listed in LDS; the row is re-read instead when they do not fit).  Probability mass is carried as 64-bit fixed point
// (exp(x - max) rounded to 2^-32), so every sum is an integer sum: the result does not depend on the
// order of the atomic additions and a replay of the same call gives the same token.  The draw
// itself is an inverse-CDF lookup in vocabulary order driven by one caller-supplied uniform
// number per row (three levels: 16 ranges -> 16 sub-ranges -> elements).
#include "mi_common.h"
#include "mi_capi_internal.h"

namespace mi {

struct SampleParams {
  const void* logits; int64_t stride;  // row stride in elements
  int32_t R, V;
  int32_t top_k; float top_p; float inv_temperature;
  const float* uniform;      // [R], unused for top_k == 1
  int32_t vocab_clamp;       // > 0: samples are clamped to [0, vocab_clamp - 1]
  int64_t* samples;          // [R]
  float* cut_out;            // optional [R]: smallest kept (scaled) logit value, -inf = nothing filtered
  const int32_t* kv_off; const int32_t* q_len; const int32_t* out_len;  // optional, [R] each
  int64_t termination_id;
  uint8_t* active_mask;      // optional [R]
};

constexpr int kSampleThreads = 1024;
constexpr int kSampleWaves = kSampleThreads / 64;

// float -> uint32 with the same ordering (and back)
static __device__ __forceinline__ uint32_t order_key(float x) {
  const uint32_t u = __float_as_uint(x);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
static __device__ __forceinline__ float order_key_value(uint32_t k) {
  return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

// Inclusive prefix sum over the 64 lanes with data-parallel-primitive moves (shifts by 1, 2, 4, 8 inside a row of 16
// lanes, then the last lane of row 0 / 2 broadcast into row 1 / 3 and lane 31 into the upper half): six steps of two
// moves and one 64-bit add, where the shuffle form costs twelve dependent trips through the LDS crossbar.  Lanes
// without a source receive zero.
template <int CTRL, int ROW_MASK>
static __device__ __forceinline__ uint64_t dpp_u64(uint64_t v) {
  const uint32_t lo = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(uint32_t)v, CTRL, ROW_MASK, 0xF, false);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(uint32_t)(v >> 32), CTRL, ROW_MASK, 0xF, false);
  return ((uint64_t)hi << 32) | lo;
}
static __device__ __forceinline__ uint64_t wave_scan_incl_u64(uint64_t v, int /*lane*/) {
  v += dpp_u64<0x111, 0xF>(v);  // row_shr:1
  v += dpp_u64<0x112, 0xF>(v);  // row_shr:2
  v += dpp_u64<0x114, 0xF>(v);  // row_shr:4
  v += dpp_u64<0x118, 0xF>(v);  // row_shr:8
  v += dpp_u64<0x142, 0xA>(v);  // row_bcast:15 into rows 1 and 3
  v += dpp_u64<0x143, 0xC>(v);  // row_bcast:31 into rows 2 and 3
  return v;
}
// Sum over the 64 lanes, in every lane: the scan above, then its last lane's value.
static __device__ __forceinline__ uint64_t wave_sum_u64(uint64_t v) {
  v = wave_scan_incl_u64(v, 0);
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v, 63);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(v >> 32), 63);
  return ((uint64_t)hi << 32) | lo;
}

// One row of logits.  DT = element type (0 fp32, 1 bf16, 2 fp16); VEC = elements per 16-byte load (4 fp32,
// 8 of a 16-bit type) when the row is 16-byte aligned, 1 otherwise.
template <int DT, int VEC>
struct RowReader {
  const uint8_t* row; int V; float inv_t; bool scale;
  // the value the filters see: logit * (1 / temperature), rounded to the logits' dtype as the
  // in-place division of the reference rounds it; -0 becomes +0 so that equal values share a key
  __device__ __forceinline__ float finish(float x) const {
    if (scale) {
      x *= inv_t;
      if (DT != 0) x = to_f32<DT == 2>(f32_to_16<DT == 2>(x));
    }
    return x + 0.0f;
  }
  __device__ __forceinline__ float at(int i) const {
    return finish(DT != 0 ? to_f32<DT == 2>(reinterpret_cast<const uint16_t*>(row)[i]) : reinterpret_cast<const float*>(row)[i]);
  }
  // elements i0 .. i0+VEC-1 (i0 a multiple of VEC), all inside the row
  __device__ __forceinline__ void load_full(int i0, float (&x)[VEC]) const {
    if (VEC > 1) {
      const uint4 w = ld16(row + (int64_t)i0 * (DT != 0 ? 2 : 4));
      const uint32_t u[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        float v;
        if (DT != 0) v = (j & 1) ? hi_to_f32<DT == 2>(u[(j >> 1) & 3]) : lo_to_f32<DT == 2>(u[(j >> 1) & 3]);
        else v = __uint_as_float(u[j & 3]);
        x[j] = finish(v);
      }
    } else {
      x[0] = at(i0);
    }
  }
  // the same with slots at or past V set to 0
  __device__ __forceinline__ void load(int i0, float (&x)[VEC]) const {
    if (VEC > 1 && i0 + VEC <= V) {
      const uint4 w = ld16(row + (int64_t)i0 * (DT != 0 ? 2 : 4));
      const uint32_t u[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        float v;
        if (DT != 0) v = (j & 1) ? hi_to_f32<DT == 2>(u[(j >> 1) & 3]) : lo_to_f32<DT == 2>(u[(j >> 1) & 3]);
        else v = __uint_as_float(u[j & 3]);
        x[j] = finish(v);
      }
    } else {
#pragma unroll
      for (int j = 0; j < VEC; ++j) x[j] = i0 + j < V ? at(i0 + j) : 0.f;
    }
  }
};

// Calls f(i, x, i < end) for every slot of [begin, end) rounded up to whole strides: `nthreads`
// threads (this one is `t`) take VEC consecutive elements each, U loads in flight.  Every thread
// makes the same number of calls, so f may use wavefront-wide operations.  begin % VEC == 0.
// Whole blocks of U strides run without any bounds test (the flag is the constant true there);
// only the rest of the range pays for guards.
template <int U, int DT, int VEC, typename F>
static __device__ __forceinline__ void sweep(const RowReader<DT, VEC>& rd, int begin, int end, int t, int nthreads, F f) {
  const int stride = nthreads * VEC;
  const int row_end = rd.V - (rd.V % VEC);  // whole 16-byte groups of the row end here
  int base = begin;
  for (; base + U * stride <= min(end, row_end); base += U * stride) {
    float x[U][VEC];
#pragma unroll
    for (int u = 0; u < U; ++u) rd.load_full(base + u * stride + t * VEC, x[u]);
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) f(base + u * stride + t * VEC + j, x[u][j], true);
    }
  }
  if (base < end) {  // the rest: fewer than U strides, guarded, loads still issued together
    float x[U][VEC];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i0 = base + u * stride + t * VEC;
      if (i0 < end) {
        rd.load(i0, x[u]);
      } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) x[u][j] = 0.f;
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i0 = base + u * stride + t * VEC;
      if (base + u * stride < end) {  // uniform over the participating threads
#pragma unroll
        for (int j = 0; j < VEC; ++j) f(i0 + j, x[u][j], i0 + j < end);
      }
    }
  }
}

// exp(x - mx) as fixed point, rounded to the nearest 2^-32: one 32-bit conversion per element
// (sums are carried in 64 bits).  0 for anything that is not a number at or below the maximum.
constexpr float kMassOne = 4294967040.0f;  // largest fp32 below 2^32
static __device__ __forceinline__ uint64_t mass_of(float x, float neg_mx_log2e) {
  const float e = fmaxf(fast_exp2(__builtin_fmaf(x, 1.4426950408889634f, neg_mx_log2e)), 0.f);  // NaN -> 0
  return (uint64_t)(uint32_t)__builtin_fmaf(e, kMassOne, 0.5f);  // the conversion saturates
}

// Adds weight() to hist[bin] for the active lanes (weight is only evaluated when some lane of the
// wavefront is active).  When every active lane hits the same bin -- values clustered in one bin
// would otherwise serialise 64 atomics on one address -- the wavefront adds its sum once.
template <typename W>
static __device__ __forceinline__ void hist_add(uint64_t* hist, int bin, bool active, int lane, W weight) {
  const uint64_t m = __builtin_amdgcn_ballot_w64(active);
  if (m == 0) return;
  const uint64_t w = active ? weight() : 0;
  const int first = __builtin_ctzll(m);
  const int b0 = __builtin_amdgcn_readlane(bin, first);
  const uint64_t same = __builtin_amdgcn_ballot_w64(active && bin == b0);
  if (same == m) {
    const uint64_t s = wave_sum_u64(w);
    if (lane == first && s) atomicAdd(reinterpret_cast<unsigned long long*>(&hist[b0]), (unsigned long long)s);
  } else if (active && w) {
    atomicAdd(reinterpret_cast<unsigned long long*>(&hist[bin]), (unsigned long long)w);
  }
}

// Wave 0: first bin b (ascending) whose inclusive running sum, started at `above`, exceeds
// `target`.  Writes {bin or -1, running sum before that bin} to res[0..1].
static __device__ void find_crossing(const uint64_t* hist, uint64_t above, uint64_t target, uint64_t* res, int lane) {
  uint64_t h[4], loc = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j) { h[j] = hist[4 * lane + j]; loc += h[j]; }
  const uint64_t incl = wave_scan_incl_u64(loc, lane) + above;
  const bool cross = incl > target;
  const uint64_t m = __builtin_amdgcn_ballot_w64(cross);
  if (m == 0) {
    if (lane == 63) { res[0] = (uint64_t)-1; res[1] = incl; }
    return;
  }
  if (lane == __builtin_ctzll(m)) {
    uint64_t run = incl - loc;
    int b = 4 * lane;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (run + h[j] > target) break;
      run += h[j];
      ++b;
    }
    res[0] = (uint64_t)b;
    res[1] = run;
  }
}

constexpr int kMemberCap = 4096;  // members of the chosen value bin that fit the LDS list
// Top-k with a small k (the usual 20-100) needs none of the row-wide histogram passes: a threshold is estimated
// from kMemberCap values spread over the row so that a thousand or a few thousand elements lie at or above it, ONE pass
// finds the maximum and lists those candidates, and the exact k-th largest value and the draw are then worked out
// on the list.  Top-p does the same with one more pass for the row's total mass; its cut lies inside the list
// whenever the candidates alone hold more than top_p of that mass (peaked rows: the usual case).  When the estimate
// misses (fewer than k candidates, more than the list holds -- flat rows --, too little mass), the general path
// below runs instead; the result is the same either way.
constexpr int kFastTopK = 768;          // largest k the one-pass form is tried for
constexpr int kFastMinVocab = 16384;    // smallest row it is tried for
// expected candidates: 1 024, or 4 k up to 3 072 (standard deviation ~ target / sqrt(sample rank), i.e. ~10-18 %)
static __device__ __forceinline__ int candidate_target(int top_k) { return max(1024, min(4 * top_k, 3072)); }

template <int DT, int VEC>
__global__ __launch_bounds__(kSampleThreads) void sample_kernel(SampleParams p) {
  __shared__ uint64_t hist[256];
  __shared__ uint64_t res[2];
  __shared__ uint64_t wsum[kSampleWaves];
  __shared__ uint32_t red_key[kSampleWaves];
  __shared__ int32_t red_idx[kSampleWaves];
  __shared__ float red_min[kSampleWaves];
  __shared__ int32_t pick[2];
  __shared__ uint32_t member_count;
  __shared__ uint32_t member_key[kMemberCap];
  __shared__ int32_t member_idx[kMemberCap];    // one-pass top-k only: vocabulary index of a candidate
  __shared__ uint64_t member_mass[kMemberCap];

  const int r = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int V = p.V;
  const bool greedy = p.top_k == 1;
  const RowReader<DT, VEC> rd{reinterpret_cast<const uint8_t*>(p.logits) + (int64_t)r * p.stride * (DT != 0 ? 2 : 4), V,
                                p.inv_temperature, !greedy && p.inv_temperature != 1.0f};
  constexpr int U = VEC == 8 ? 4 : 8;  // 16-byte loads in flight per thread (32 values either way)

  // ---- pass A: maximum (lowest index among equals, NaN counts as largest) and finite minimum ----
  // (a thread meets its elements in rising index order, so "strictly greater" keeps the first)
  uint32_t bk = 0; int bi = 0x7fffffff; float mn = INFINITY;
  const bool filtering = !greedy && (p.top_k > 1 || p.top_p > 0.f);
  // `digit_select`: the key with exactly `target` list members (weights: 1, or the members' masses) above it, by four
  // 8-bit digit passes over member_key[0..n) starting from `above` (the weight already counted above the list).
  // With last_digit > 0 the low digits stay zero: a key at or below the exact one (a threshold that errs on the
  // side of more members).
  auto digit_select = [&](int n, uint64_t target, uint64_t above, bool by_mass, int last_digit) -> uint32_t {
    uint32_t pmask = 0, pval = 0;
    __syncthreads();
    if (tid < 256) hist[tid] = 0;
    __syncthreads();
    for (int d = 3; d >= last_digit; --d) {
      for (int j0 = 0; j0 < n; j0 += kSampleThreads) {
        const int j = j0 + tid;
        const bool in = j < n;
        const uint32_t k = in ? member_key[j] : 0;
        hist_add(hist, 255 - (int)((k >> (8 * d)) & 255u), in && (k & pmask) == pval, lane,
                 [&] { return by_mass ? member_mass[j] : (uint64_t)1; });
      }
      __syncthreads();
      if (wave == 0) {  // the wavefront that reads the bins also clears them for the next digit: two barriers a pass
        find_crossing(hist, above, target, res, lane);
#pragma unroll
        for (int j = 0; j < 4; ++j) hist[4 * lane + j] = 0;
      }
      __syncthreads();
      const uint32_t digit = 255u - (uint32_t)res[0];  // the crossing lies inside the list, so a digit is always found
      above = res[1];
      pmask |= 0xffu << (8 * d);
      pval |= digit << (8 * d);
    }
    return pval;
  };
  const bool one_pass = !greedy && V >= kFastMinVocab &&
                        (p.top_k > 1 ? p.top_k <= kFastTopK : p.top_p > 0.f);  // (top-p: one more pass for the total mass)
  constexpr int kSamplesPerThread = kMemberCap / kSampleThreads;
  uint32_t tau = 0;
  if (one_pass) {
    // threshold: the rank-th largest of kMemberCap sampled values, rank chosen for ~candidate_target(k) candidates
    const int blk = V / kSampleThreads;  // >= 16: thread t samples elements t * blk .. + 3
#pragma unroll
    for (int j = 0; j < kSamplesPerThread; ++j)
      member_key[tid * kSamplesPerThread + j] = order_key(rd.at(tid * blk + j));
    const int rank = min(kMemberCap / 2, (int)(((int64_t)candidate_target(p.top_k) * kMemberCap + V - 1) / V));
    // (the upper 16 bits of the key are enough: sign, exponent and 7 bits of the fraction)
    tau = digit_select(kMemberCap, (uint64_t)(rank - 1), 0, false, 2);
    if (tid == 0) member_count = 0;
    __syncthreads();  // the sample has been read by everyone; the list is reused for the candidates
    // one pass: the maximum (and, for top-p, which falls back to the general path often enough, the finite
    // minimum) and the list of candidates
    auto list_candidate = [&](uint32_t k, int i, bool cand) {
      const uint64_t m = __builtin_amdgcn_ballot_w64(cand);
      if (m == 0) return;
      uint32_t base = 0;
      const int first = __builtin_ctzll(m);
      if (lane == first) base = atomicAdd(&member_count, (uint32_t)__builtin_popcountll(m));
      base = __builtin_amdgcn_readlane(base, first);
      const uint32_t at = base + (uint32_t)__builtin_popcountll(m & (((uint64_t)1 << lane) - 1));
      if (cand && at < (uint32_t)kMemberCap) {
        member_key[at] = k;
        member_idx[at] = i;
      }
    };
    if (p.top_k > 1) {
      sweep<U>(rd, 0, V, tid, kSampleThreads, [&](int i, float x, bool in) {
        const uint32_t k = order_key(x);
        const bool up = in && k > bk;
        bk = up ? k : bk; bi = up ? i : bi;
        list_candidate(k, i, in && k >= tau);
      });
    } else {  // (half the loads in flight: with the minimum the full count no longer fits the registers)
      sweep<U / 2>(rd, 0, V, tid, kSampleThreads, [&](int i, float x, bool in) {
        const uint32_t k = order_key(x);
        const bool up = in && k > bk;
        bk = up ? k : bk; bi = up ? i : bi;
        mn = (in && x > -INFINITY) ? fminf(mn, x) : mn;
        list_candidate(k, i, in && k >= tau);
      });
    }
  } else if (filtering) {
    sweep<U>(rd, 0, V, tid, kSampleThreads, [&](int i, float x, bool in) {
      const uint32_t k = order_key(x);
      const bool up = in && k > bk;
      bk = up ? k : bk; bi = up ? i : bi;
      mn = (in && x > -INFINITY) ? fminf(mn, x) : mn;
    });
  } else {
    sweep<U>(rd, 0, V, tid, kSampleThreads, [&](int i, float x, bool in) {
      const uint32_t k = order_key(x);
      const bool up = in && k > bk;
      bk = up ? k : bk; bi = up ? i : bi;
    });
  }
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) {
    const uint32_t ok = __shfl_xor(bk, m, 64); const int oi = __shfl_xor(bi, m, 64);
    if (ok > bk || (ok == bk && oi < bi)) { bk = ok; bi = oi; }
    mn = fminf(mn, __shfl_xor(mn, m, 64));
  }
  if (lane == 0) { red_key[wave] = bk; red_idx[wave] = bi; red_min[wave] = mn; }
  __syncthreads();
  bk = red_key[0]; bi = red_idx[0]; mn = red_min[0];
#pragma unroll
  for (int w = 1; w < kSampleWaves; ++w) {
    const uint32_t ok = red_key[w]; const int oi = red_idx[w];
    if (ok > bk || (ok == bk && oi < bi)) { bk = ok; bi = oi; }
    mn = fminf(mn, red_min[w]);
  }
  if (bi >= V) bi = 0;  // only when no element compared greater than the start value
  const float mx = order_key_value(bk);
  int sample = bi;
  uint32_t cut_key = 0;  // keep everything

  // A maximum that is not a finite number leaves no distribution to draw from: take the argmax.
  const bool drawable = !greedy && fabsf(mx) < INFINITY;
  const float neg_mx = -mx * 1.4426950408889634f;
  if (drawable) {
    const bool by_count = p.top_k > 1;
    const bool filtered = by_count || p.top_p > 0.f;
    bool cut_from_list = false;
    int n_candidates = 0;
    if (one_pass) {
      n_candidates = (int)member_count;  // (published by the barrier of the maximum's reduction)
      bool usable = n_candidates <= kMemberCap && (by_count ? n_candidates >= p.top_k : n_candidates > 0);
      uint64_t target = by_count ? (uint64_t)(p.top_k - 1) : 0;
      if (usable && !by_count) {
        // top-p: the row's total mass (one more pass), then the candidates' masses; the cut lies inside the list
        // when those alone exceed top_p of the total
        auto workgroup_sum = [&](uint64_t v) -> uint64_t {
          v = wave_sum_u64(v);
          __syncthreads();
          if (lane == 0) wsum[wave] = v;
          __syncthreads();
          uint64_t t = 0;
#pragma unroll
          for (int w = 0; w < kSampleWaves; ++w) t += wsum[w];
          return t;
        };
        uint64_t c = 0;
        for (int j = tid; j < n_candidates; j += kSampleThreads) {
          const uint64_t m = mass_of(order_key_value(member_key[j]), neg_mx);
          member_mass[j] = m;
          c += m;
        }
        c = workgroup_sum(c);
        // Worth the pass?  The mass below the threshold is many small terms, so the sample estimates it well
        // (unlike the mass above it, which a few elements can hold); a quarter on top of the estimate as margin, so
        // that rows on the edge do not pay for the total-mass pass and then fail.
        // (the sampled values are read again rather than kept in registers through the passes above)
        uint64_t below = 0;
#pragma unroll
        for (int j = 0; j < kSamplesPerThread; ++j) {
          const float x = rd.at(tid * (V / kSampleThreads) + j);
          below += order_key(x) < tau ? mass_of(x, neg_mx) : 0;
        }
        const double rest = (double)workgroup_sum(below) * ((double)V / kMemberCap) * 1.25;
        usable = (double)c > (double)p.top_p * ((double)c + rest);
        if (usable) {
          uint64_t z = 0;
          sweep<U>(rd, 0, V, tid, kSampleThreads, [&](int, float x, bool in) { z += in ? mass_of(x, neg_mx) : 0; });
          z = workgroup_sum(z);
          target = (uint64_t)((double)p.top_p * (double)z);
          usable = c > target;
        }
      }
      if (usable) {
        cut_key = digit_select(n_candidates, target, 0, !by_count, 0);
        cut_from_list = true;
      } else if (by_count) {
        // the general path needs the finite minimum, which the one-pass sweep did not track for top-k
        sweep<U>(rd, 0, V, tid, kSampleThreads, [&](int, float x, bool in) {
          mn = (in && x > -INFINITY) ? fminf(mn, x) : mn;
        });
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) mn = fminf(mn, __shfl_xor(mn, m, 64));
        __syncthreads();
        if (lane == 0) red_min[wave] = mn;
        __syncthreads();
        mn = red_min[0];
#pragma unroll
        for (int w = 1; w < kSampleWaves; ++w) mn = fminf(mn, red_min[w]);
      }
    }
    if (filtered && !cut_from_list) {
      // ---- pass B: 256 linear bins over [mx - range, mx], bin 0 = largest values ----
      float range = mx - mn;
      if (!by_count) range = fminf(range, 32.f);  // mass below exp(-32) cannot move a top-p cut
      const float inv_w = range > 0.f ? 256.f / range : 0.f;
      auto lin_bin = [&](float x) {
        const float f = (mx - x) * inv_w;
        int b = f >= 255.f ? 255 : (int)f;  // NaN (inf * 0) compares false and converts to 0
        return b < 0 ? 0 : b;
      };
      auto weight_of = [&](float x) -> uint64_t { return by_count ? (uint64_t)1 : mass_of(x, neg_mx); };
      if (tid < 256) hist[tid] = 0;
      if (tid == 0) member_count = 0;
      __syncthreads();
      sweep<U>(rd, 0, V, tid, kSampleThreads, [&](int, float x, bool in) {
        hist_add(hist, lin_bin(x), in, lane, [&] { return weight_of(x); });
      });
      __syncthreads();
      uint64_t target;
      if (by_count) {
        target = (uint64_t)(p.top_k - 1);
      } else {
        uint64_t z = 0;
        for (int j = 0; j < 256; ++j) z += hist[j];  // same LDS words for every lane: broadcast reads
        target = (uint64_t)((double)p.top_p * (double)z);
      }
      if (wave == 0) find_crossing(hist, 0, target, res, lane);
      __syncthreads();
      const int lbin = (int)(int64_t)res[0];
      uint64_t above = res[1];
      if (lbin >= 0) {
        // ---- pass C: list the members of the chosen bin in LDS (wavefront-aggregated append) ----
        sweep<U>(rd, 0, V, tid, kSampleThreads, [&](int, float x, bool in) {
          const bool member = in && lin_bin(x) == lbin;
          const uint64_t m = __builtin_amdgcn_ballot_w64(member);
          if (m == 0) return;
          uint32_t base = 0;
          const int first = __builtin_ctzll(m);
          if (lane == first) base = atomicAdd(&member_count, (uint32_t)__builtin_popcountll(m));
          base = __builtin_amdgcn_readlane(base, first);
          const uint32_t at = base + (uint32_t)__builtin_popcountll(m & (((uint64_t)1 << lane) - 1));
          if (member && at < (uint32_t)kMemberCap) {
            member_key[at] = order_key(x);
            member_mass[at] = weight_of(x);
          }
        });
        __syncthreads();
        const int n_members = (int)member_count;
        const bool listed = n_members <= kMemberCap;
        // ---- four 8-bit digit passes over the members (the LDS list, or the row when it overflowed) ----
        uint32_t pmask = 0, pval = 0;
        for (int d = 3; d >= 0; --d) {
          __syncthreads();
          if (tid < 256) hist[tid] = 0;
          __syncthreads();
          if (listed) {
            for (int j0 = 0; j0 < n_members; j0 += kSampleThreads) {
              const int j = j0 + tid;
              const bool in = j < n_members;
              const uint32_t k = in ? member_key[j] : 0;
              hist_add(hist, 255 - (int)((k >> (8 * d)) & 255u), in && (k & pmask) == pval, lane,
                       [&] { return member_mass[j]; });
            }
          } else {
            sweep<U>(rd, 0, V, tid, kSampleThreads, [&](int, float x, bool in) {
              const uint32_t k = order_key(x);
              hist_add(hist, 255 - (int)((k >> (8 * d)) & 255u), in && lin_bin(x) == lbin && (k & pmask) == pval, lane,
                       [&] { return weight_of(x); });
            });
          }
          __syncthreads();
          if (wave == 0) find_crossing(hist, above, target, res, lane);
          __syncthreads();
          // the crossing lies inside the chosen bin, so a digit is always found
          const uint32_t digit = 255u - (uint32_t)res[0];
          above = res[1];
          pmask |= 0xffu << (8 * d);
          pval |= digit << (8 * d);
        }
        cut_key = pval;
      }
    }

    // ---- draw on the candidate list: the kept elements are among the candidates, so when they are few the
    // inverse CDF in vocabulary order is a direct count over the list (each thread owns one kept element and sums
    // the masses of those at or before it) ----
    bool drawn = false;
    if (cut_from_list) {
      __syncthreads();
      if (tid == 0) member_count = 0;
      __syncthreads();
      for (int j0 = 0; j0 < n_candidates; j0 += kSampleThreads) {
        const int j = j0 + tid;
        const bool kept = j < n_candidates && member_key[j] >= cut_key;
        const uint64_t m = __builtin_amdgcn_ballot_w64(kept);
        if (m == 0) continue;
        uint32_t base = 0;
        const int first = __builtin_ctzll(m);
        if (lane == first) base = atomicAdd(&member_count, (uint32_t)__builtin_popcountll(m));
        base = __builtin_amdgcn_readlane(base, first);
        const uint32_t at = base + (uint32_t)__builtin_popcountll(m & (((uint64_t)1 << lane) - 1));
        // (vocabulary index and mass of a kept element in one word: a mass fits 32 bits)
        if (kept) member_mass[at] = ((uint64_t)(uint32_t)member_idx[j] << 32) | mass_of(order_key_value(member_key[j]), neg_mx);
      }
      __syncthreads();
      const int n_kept = (int)member_count;
      if (n_kept <= kSampleThreads) {
        if (wave * 64 < n_kept) {  // only the wavefronts that own a kept element walk the list
          const uint64_t mine = tid < n_kept ? member_mass[tid] : 0;
          const uint32_t my_idx = (uint32_t)(mine >> 32);
          uint64_t total = 0, upto = 0;  // all kept mass; kept mass at vocabulary indices <= mine
          for (int m = 0; m < n_kept; ++m) {
            const uint64_t e = member_mass[m];  // the same word for every lane: a broadcast read
            const uint64_t w = e & 0xffffffffu;
            total += w;
            upto += (uint32_t)(e >> 32) <= my_idx ? w : 0;
          }
          uint64_t want = (uint64_t)((double)p.uniform[r] * (double)total);
          want = want < total ? want : total - 1;
          const uint64_t w_mine = mine & 0xffffffffu;
          if (tid < n_kept && upto > want && upto - w_mine <= want) pick[0] = (int)my_idx;
        }
        drawn = true;
      }
    }
    auto kept_mass = [&](float x) -> uint64_t { return order_key(x) >= cut_key ? mass_of(x, neg_mx) : 0; };
    if (!drawn) {
      const int L1 = ((V + kSampleWaves - 1) / kSampleWaves + 63) & ~63;  // elements per first-level range
      {
        const int a = min(wave * L1, V), b = min(a + L1, V);
        uint64_t s = 0;
        sweep<U>(rd, a, b, lane, 64, [&](int, float x, bool in) { s += in ? kept_mass(x) : 0; });
        s = wave_sum_u64(s);
        if (lane == 0) wsum[wave] = s;
      }
      __syncthreads();
      uint64_t total = 0;
#pragma unroll
      for (int w = 0; w < kSampleWaves; ++w) total += wsum[w];
      // total > 0: the maximum itself is always kept and has the largest mass
      uint64_t want = (uint64_t)((double)p.uniform[r] * (double)total);
      want = want < total ? want : total - 1;
      int w1 = 0;
#pragma unroll
      for (int w = 0; w < kSampleWaves - 1; ++w) {
        const bool pass = w == w1 && want >= wsum[w];
        want -= pass ? wsum[w] : 0;
        w1 += pass ? 1 : 0;
      }
      // (ranges after the last non-empty one hold no mass, so w1 stops inside the vocabulary)
      const int a1 = min(w1 * L1, V), b1 = min(a1 + L1, V);
      const int L2 = (L1 / kSampleWaves + 63) & ~63;  // elements per second-level range
      __syncthreads();
      {
        const int a = min(a1 + wave * L2, b1), b = min(a + L2, b1);
        uint64_t s = 0;
        sweep<1>(rd, a, b, lane, 64, [&](int, float x, bool in) { s += in ? kept_mass(x) : 0; });
        s = wave_sum_u64(s);
        if (lane == 0) wsum[wave] = s;
      }
      __syncthreads();
      int w2 = 0;
#pragma unroll
      for (int w = 0; w < kSampleWaves - 1; ++w) {
        const bool pass = w == w2 && want >= wsum[w];
        want -= pass ? wsum[w] : 0;
        w2 += pass ? 1 : 0;
      }
      const int a2 = min(a1 + w2 * L2, b1), b2 = min(a2 + L2, b1);
      if (wave == 0) {
        // third level: each lane owns a contiguous run of the sub-range
        const int per = L2 / 64;
        const int a = min(a2 + lane * per, b2), b = min(a + per, b2);
        uint64_t s = 0;
        for (int i = a; i < b; ++i) s += kept_mass(rd.at(i));
        const uint64_t incl = wave_scan_incl_u64(s, lane);
        const uint64_t m = __builtin_amdgcn_ballot_w64(incl > want);
        const int owner = m ? __builtin_ctzll(m) : 63;
        if (lane == owner) {
          uint64_t run = incl - s;
          int found = b > a ? b - 1 : bi;
          for (int i = a; i < b; ++i) {
            run += kept_mass(rd.at(i));
            if (run > want) { found = i; break; }
          }
          pick[0] = found;
        }
      }
    }
    __syncthreads();
    sample = pick[0];
    if (p.vocab_clamp > 0) sample = min(max(sample, 0), p.vocab_clamp - 1);
  }

  if (tid == 0) {
    p.samples[r] = sample;
    if (p.cut_out) p.cut_out[r] = cut_key ? order_key_value(cut_key) : -INFINITY;
    if (p.active_mask) {
      bool active = (int64_t)sample != p.termination_id;
      if (p.kv_off) active = active && (p.kv_off[r] + p.q_len[r] + 1 < p.out_len[r]);
      p.active_mask[r] = active ? 1 : 0;
    }
  }
}

struct GatherParams {
  const uint8_t* src; int64_t src_stride_bytes;
  uint8_t* dst; int64_t dst_stride_bytes;
  const int32_t* q_len; int32_t R; int64_t row_bytes; int32_t vec;
};

// dst[r] = src[sum(q_len[0..r]) - 1]; grid = (R, column blocks)
__global__ __launch_bounds__(256) void last_token_gather_kernel(GatherParams p) {
  __shared__ int32_t part[4];
  const int r = blockIdx.x, tid = threadIdx.x;
  int s = 0;
  for (int i = tid; i <= r; i += 256) s += p.q_len[i];
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) s += __shfl_xor(s, m, 64);
  if ((tid & 63) == 0) part[tid >> 6] = s;
  __syncthreads();
  const int64_t row = (int64_t)part[0] + part[1] + part[2] + part[3] - 1;
  if (row < 0) return;
  const uint8_t* src = p.src + row * p.src_stride_bytes;
  uint8_t* dst = p.dst + (int64_t)r * p.dst_stride_bytes;
  const int64_t step = (int64_t)gridDim.y * 256 * p.vec;
  for (int64_t o = ((int64_t)blockIdx.y * 256 + tid) * p.vec; o < p.row_bytes; o += step) {
    if (p.vec == 16) st16(dst + o, ld16(src + o));
    else if (p.vec == 4) *reinterpret_cast<uint32_t*>(dst + o) = *reinterpret_cast<const uint32_t*>(src + o);
    else *reinterpret_cast<uint16_t*>(dst + o) = *reinterpret_cast<const uint16_t*>(src + o);
  }
}

struct LogProbParams {
  const void* logits; int64_t stride; int32_t T, V;
  const int64_t* token_ids; float* out;
};

constexpr int kLogProbThreads = 512;

// out[t] = log_softmax(logits[t])[token_ids[t]] in fp32: one pass over the row with a running
// (maximum, sum of exp(x - maximum)) pair per thread, merged over the workgroup.  One workgroup per row.
template <int DT, int VEC>
__global__ __launch_bounds__(kLogProbThreads) void selected_log_probs_kernel(LogProbParams p) {
  __shared__ float red_m[kLogProbThreads / 64], red_s[kLogProbThreads / 64];
  const int t = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  RowReader<DT, VEC> rd;
  rd.row = reinterpret_cast<const uint8_t*>(p.logits) + (int64_t)t * p.stride * (DT != 0 ? 2 : 4);
  rd.V = p.V; rd.inv_t = 1.f; rd.scale = false;
  constexpr float kLog2e = 1.4426950408889634f;
  // a finite start keeps exp(-inf - m) = 0 for masked (-inf) logits
  float m = -3.0e38f, sum = 0.f;
  // Whole batches of U 16-byte groups per thread: the batch maximum first (one three-way maximum per
  // two elements), a rescale only when it raises the running maximum (rare after a thread's first
  // batches), then one fused multiply-add, one exp2 and one add per element.
  constexpr int U = 4;
  const int stride = kLogProbThreads * VEC;
  const int row_end = p.V - (p.V % VEC);
  int base = 0;
  if (VEC > 1) {
    for (; base + U * stride <= row_end; base += U * stride) {
      float x[U * VEC];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint4 w = ld16(rd.row + (int64_t)(base + u * stride + tid * VEC) * (DT != 0 ? 2 : 4));
        const uint32_t q[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int j = 0; j < VEC; ++j)
          x[u * VEC + j] = DT != 0 ? ((j & 1) ? hi_to_f32<DT == 2>(q[(j >> 1) & 3]) : lo_to_f32<DT == 2>(q[(j >> 1) & 3]))
                                : __uint_as_float(q[j & 3]);
      }
      float bm = x[0];
#pragma unroll
      for (int j = 1; j + 1 < U * VEC; j += 2) bm = fmaxf(fmaxf(bm, x[j]), x[j + 1]);
      bm = fmaxf(bm, x[U * VEC - 1]);
      if (bm > m) {
        sum *= fast_exp2((m - bm) * kLog2e);
        m = bm;
      }
      const float nm = -m * kLog2e;
      float part = 0.f;
#pragma unroll
      for (int j = 0; j < U * VEC; ++j) part += fast_exp2(__builtin_fmaf(x[j], kLog2e, nm));
      sum += part;
    }
  }
  sweep<U>(rd, base, p.V, tid, kLogProbThreads, [&](int, float x, bool valid) {
    if (valid) {
      if (x > m) {
        sum *= fast_exp2((m - x) * kLog2e);
        m = x;
      }
      sum += fast_exp2((x - m) * kLog2e);
    }
  });
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) {
    const float m2 = __shfl_xor(m, d, 64), s2 = __shfl_xor(sum, d, 64);
    const float mm = fmaxf(m, m2);
    sum = sum * fast_exp2((m - mm) * kLog2e) + s2 * fast_exp2((m2 - mm) * kLog2e);
    m = mm;
  }
  if (lane == 0) { red_m[wave] = m; red_s[wave] = sum; }
  __syncthreads();
  if (tid == 0) {
    float mm = red_m[0];
#pragma unroll
    for (int w = 1; w < kLogProbThreads / 64; ++w) mm = fmaxf(mm, red_m[w]);
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < kLogProbThreads / 64; ++w) total += red_s[w] * fast_exp2((red_m[w] - mm) * kLog2e);
    const int64_t id = p.token_ids[t];
    float r = __builtin_nanf("");
    if (id >= 0 && id < p.V) r = (rd.at((int)id) - mm) - __logf(total);
    p.out[t] = r;
  }
}

}  // namespace mi

using namespace mi;

extern "C" int mi_last_token_gather(const void* src, int64_t src_stride_row, void* dst, int64_t dst_stride_row,
                                    const int32_t* request_query_lengths, int32_t R, int32_t row_elems,
                                    int32_t elem_bytes, void* stream) {
  if (R == 0 || row_elems == 0) return MI_OK;
  if (!src || !dst || !request_query_lengths) return mi_fail(MI_ERR_NULL, "mi_last_token_gather: null pointer argument");
  if (R < 0 || row_elems < 0 || (elem_bytes != 2 && elem_bytes != 4))
    return mi_fail(MI_ERR_SHAPE, "mi_last_token_gather: need R, row_elems >= 0 and 2- or 4-byte elements");
  if (src_stride_row < row_elems || dst_stride_row < row_elems)
    return mi_fail(MI_ERR_SHAPE, "mi_last_token_gather: row strides are shorter than a row");
  GatherParams p;
  p.src = (const uint8_t*)src; p.src_stride_bytes = src_stride_row * elem_bytes;
  p.dst = (uint8_t*)dst; p.dst_stride_bytes = dst_stride_row * elem_bytes;
  p.q_len = request_query_lengths; p.R = R; p.row_bytes = (int64_t)row_elems * elem_bytes;
  const bool wide = !(((uintptr_t)src | (uintptr_t)dst | (uintptr_t)p.src_stride_bytes | (uintptr_t)p.dst_stride_bytes |
                       (uintptr_t)p.row_bytes) & 15);
  p.vec = wide ? 16 : elem_bytes;
  const int64_t per_block = 256 * (int64_t)p.vec;
  int ny = (int)((p.row_bytes + per_block - 1) / per_block);
  ny = ny < 1 ? 1 : (ny > 64 ? 64 : ny);
  hipLaunchKernelGGL(last_token_gather_kernel, dim3(R, ny), dim3(256), 0, (hipStream_t)stream, p);
  return mi_check_launch("mi_last_token_gather");
}

extern "C" int mi_sample_from_logits(const void* logits, int64_t stride_row, int32_t logits_dtype, int32_t R,
                                     int32_t vocab, int32_t top_k, float top_p, float temperature,
                                     const float* uniform, int32_t vocab_clamp, int64_t* samples,
                                     float* cut_values, const int32_t* request_kv_length_offsets,
                                     const int32_t* request_query_lengths, const int32_t* request_output_lengths,
                                     int64_t termination_id, uint8_t* active_request_mask, void* stream) {
  if (R == 0) return MI_OK;
  if (!logits || !samples) return mi_fail(MI_ERR_NULL, "mi_sample_from_logits: null pointer argument");
  if (R < 0 || vocab <= 0 || stride_row < vocab)
    return mi_fail(MI_ERR_SHAPE, "mi_sample_from_logits: need R >= 0, vocab > 0 and a row stride of at least vocab");
  if (logits_dtype < 0 || logits_dtype > 2)
    return mi_fail(MI_ERR_UNSUPPORTED, "mi_sample_from_logits: logits must be fp32 (0), bf16 (1) or fp16 (2)");
  if (top_k < 0 || !(top_p >= 0.f && top_p <= 1.f))
    return mi_fail(MI_ERR_SHAPE, "mi_sample_from_logits: need top_k >= 0 and top_p in [0, 1]");
  if (top_k > 0 && top_p > 0.f)
    return mi_fail(MI_ERR_SHAPE, "mi_sample_from_logits: cannot have top-p and top-k both greater than zero");
  if (top_k > vocab) return mi_fail(MI_ERR_SHAPE, "mi_sample_from_logits: top-k is larger than logit size");
  if (top_k != 1 && !(temperature > 0.f))
    return mi_fail(MI_ERR_SHAPE, "mi_sample_from_logits: temperature must be positive");
  if (top_k != 1 && !uniform)
    return mi_fail(MI_ERR_NULL, "mi_sample_from_logits: sampling needs one uniform number per row");
  const bool any_len = request_kv_length_offsets || request_query_lengths || request_output_lengths;
  if (any_len && !(request_kv_length_offsets && request_query_lengths && request_output_lengths))
    return mi_fail(MI_ERR_NULL, "mi_sample_from_logits: the three request length rows go together");
  if (any_len && !active_request_mask)
    return mi_fail(MI_ERR_NULL, "mi_sample_from_logits: request lengths were given without a mask to write");
  SampleParams p;
  p.logits = logits; p.stride = stride_row; p.R = R; p.V = vocab;
  p.top_k = top_k; p.top_p = top_p; p.inv_temperature = top_k == 1 ? 1.0f : 1.0f / temperature;
  p.uniform = uniform; p.vocab_clamp = vocab_clamp; p.samples = samples; p.cut_out = cut_values;
  p.kv_off = request_kv_length_offsets; p.q_len = request_query_lengths; p.out_len = request_output_lengths;
  p.termination_id = termination_id; p.active_mask = active_request_mask;
  const int esize = logits_dtype != 0 ? 2 : 4;
  const bool wide = !(((uintptr_t)logits | (uintptr_t)(stride_row * esize)) & 15);  // 16-byte loads
  const dim3 grid(R), block(kSampleThreads);
  hipStream_t st = (hipStream_t)stream;
  if (logits_dtype == 2) {
    if (wide) hipLaunchKernelGGL((sample_kernel<2, 8>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((sample_kernel<2, 1>), grid, block, 0, st, p);
  } else if (logits_dtype == 1) {
    if (wide) hipLaunchKernelGGL((sample_kernel<1, 8>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((sample_kernel<1, 1>), grid, block, 0, st, p);
  } else {
    if (wide) hipLaunchKernelGGL((sample_kernel<0, 4>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((sample_kernel<0, 1>), grid, block, 0, st, p);
  }
  return mi_check_launch("mi_sample_from_logits");
}

extern "C" int mi_selected_log_probs(const void* logits, int64_t stride_row, int32_t logits_dtype, int32_t T,
                                     int32_t vocab, const int64_t* token_ids, float* log_probs, void* stream) {
  if (T == 0) return MI_OK;
  if (!logits || !token_ids || !log_probs) return mi_fail(MI_ERR_NULL, "mi_selected_log_probs: null pointer argument");
  if (T < 0 || vocab <= 0 || stride_row < vocab)
    return mi_fail(MI_ERR_SHAPE, "mi_selected_log_probs: need T >= 0, vocab > 0 and a row stride of at least vocab");
  if (logits_dtype < 0 || logits_dtype > 2)
    return mi_fail(MI_ERR_UNSUPPORTED, "mi_selected_log_probs: logits must be fp32 (0), bf16 (1) or fp16 (2)");
  LogProbParams p;
  p.logits = logits; p.stride = stride_row; p.T = T; p.V = vocab; p.token_ids = token_ids; p.out = log_probs;
  const int esize = logits_dtype != 0 ? 2 : 4;
  const bool wide = !(((uintptr_t)logits | (uintptr_t)(stride_row * esize)) & 15);  // 16-byte loads
  const dim3 grid(T), block(kLogProbThreads);
  hipStream_t st = (hipStream_t)stream;
  if (logits_dtype == 2) {
    if (wide) hipLaunchKernelGGL((selected_log_probs_kernel<2, 8>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((selected_log_probs_kernel<2, 1>), grid, block, 0, st, p);
  } else if (logits_dtype == 1) {
    if (wide) hipLaunchKernelGGL((selected_log_probs_kernel<1, 8>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((selected_log_probs_kernel<1, 1>), grid, block, 0, st, p);
  } else {
    if (wide) hipLaunchKernelGGL((selected_log_probs_kernel<0, 4>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((selected_log_probs_kernel<0, 1>), grid, block, 0, st, p);
  }
  return mi_check_launch("mi_selected_log_probs");
}
