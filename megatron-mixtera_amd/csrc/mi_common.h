// Shared device helpers for the gfx950 (MI355X) paged-KV kernels.
//
// Conventions used by every kernel in this directory:
//  * a wavefront is 64 lanes; `m16 = lane & 15` and `g = lane >> 4` are the two
//    coordinates every MFMA operand layout is expressed in;
//  * bf16 / fp16 values travel as raw uint16_t / packed uint32_t pairs and are only
//    reinterpreted by the helpers below (template parameter F16);
//  * all kernels are enqueue-only: no host synchronisation, no device-side
//    allocation, every buffer is owned by the caller.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mi {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short s16x4_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;
typedef __attribute__((ext_vector_type(2))) float f32x2_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;

constexpr int kWave = 64;

// 16-bit element types.  Every kernel that touches q / k / v / out elements is compiled twice, for bf16
// (F16 = false) and for IEEE fp16 (F16 = true); values travel as raw uint16_t / packed uint32_t pairs and the
// helpers below are the only places that know which of the two they are.
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4_t __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));

// D(16x16) += A(16x32) * B(32x16), 16-bit inputs, fp32 accumulate.
// Lane (m16, g) supplies A[m16][8g..8g+7] and B[8g..8g+7][m16]; it receives
// D[4g+i][m16] in slot i.  Only the pairing "A slot j of group g meets B slot j
// of group g" is relied upon, so any consistent assignment of contraction
// indices to (g, j) gives the same dot products.
template <bool F16 = false>
static __device__ __forceinline__ f32x4_t mfma_16x16x32(uint4 a, uint4 b, f32x4_t c) {
  if constexpr (F16)
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

// D(16x16) += A(16x16) * B(16x16), 16-bit inputs, fp32 accumulate.
// Lane (m16, g) supplies A[m16][4g..4g+3] and B[4g..4g+3][m16]; D as above.
template <bool F16 = false>
static __device__ __forceinline__ f32x4_t mfma_16x16x16(uint2 a, uint2 b, f32x4_t c) {
  if constexpr (F16)
    return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4_t, a), __builtin_bit_cast(f16x4_t, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4_t, a), __builtin_bit_cast(s16x4_t, b), c, 0, 0, 0);
}

// Two fp32 -> packed bf16 pair (round to nearest even), `lo` in bits 0..15.
static __device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  f32x2_t v = {lo, hi};
  bf16x2_t r = __builtin_convertvector(v, bf16x2_t);
  return __builtin_bit_cast(uint32_t, r);
}
// Two fp32 -> packed pair of the kernel's 16-bit type (round to nearest even), `lo` in bits 0..15.
template <bool F16>
static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  if constexpr (F16) {
    f32x2_t v = {lo, hi};
    f16x2_t r = __builtin_convertvector(v, f16x2_t);
    return __builtin_bit_cast(uint32_t, r);
  } else {
    return pack_bf16x2(lo, hi);
  }
}

static __device__ __forceinline__ uint16_t f32_to_bf16(float x) {
  return (uint16_t)(pack_bf16x2(x, 0.f) & 0xffffu);
}
template <bool F16>
static __device__ __forceinline__ uint16_t f32_to_16(float x) {
  if constexpr (F16) return __builtin_bit_cast(uint16_t, (_Float16)x);
  else return f32_to_bf16(x);
}

static __device__ __forceinline__ float bf16_to_f32(uint16_t x) {
  return __builtin_bit_cast(float, (uint32_t)x << 16);
}
static __device__ __forceinline__ float bf16lo_to_f32(uint32_t pair) {
  return __builtin_bit_cast(float, pair << 16);
}
static __device__ __forceinline__ float bf16hi_to_f32(uint32_t pair) {
  return __builtin_bit_cast(float, pair & 0xffff0000u);
}
template <bool F16>
static __device__ __forceinline__ float to_f32(uint16_t x) {
  if constexpr (F16) return (float)__builtin_bit_cast(_Float16, x);
  else return bf16_to_f32(x);
}
template <bool F16>
static __device__ __forceinline__ float lo_to_f32(uint32_t pair) {
  if constexpr (F16) return (float)__builtin_bit_cast(_Float16, (uint16_t)(pair & 0xffffu));
  else return bf16lo_to_f32(pair);
}
template <bool F16>
static __device__ __forceinline__ float hi_to_f32(uint32_t pair) {
  if constexpr (F16) return (float)__builtin_bit_cast(_Float16, (uint16_t)(pair >> 16));
  else return bf16hi_to_f32(pair);
}
// 1.0 twice, as a packed pair of the kernel's 16-bit type
template <bool F16>
static __device__ __forceinline__ constexpr uint32_t ones2() { return F16 ? 0x3c003c00u : 0x3f803f80u; }

// (hi16 of a | lo16 ... ) helpers for the in-register 4x4 bf16 transposes.
// low_halves(a, b)  = (a.lo16 << 16) | b.lo16
// high_halves(a, b) = (a.hi16 << 16) | b.hi16
static __device__ __forceinline__ uint32_t low_halves(uint32_t a, uint32_t b) {
  return __builtin_amdgcn_perm(a, b, 0x05040100u);
}
static __device__ __forceinline__ uint32_t high_halves(uint32_t a, uint32_t b) {
  return __builtin_amdgcn_perm(a, b, 0x07060302u);
}

static __device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
static __device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// sin and cos of a rotary angle (position x inverse frequency: non-negative, up to ~1e6 rad for a million positions)
// in ~30 vector instructions for the pair: three-term Cody-Waite reduction by pi/2 with fused multiply-adds, then the
// single-precision minimax polynomials on [-pi/4, pi/4].  Absolute error <= 1.2e-7 for |x| <= 1e6 (160 M random
// arguments against double precision), i.e. within one unit in the last place of the library's sinf / cosf where it
// matters: after rounding to bf16 the two differ on 4 values in a million.  Larger arguments take the library
// functions (their reduction handles any magnitude).
static __device__ __forceinline__ void rotary_sincos(float x, float* sn, float* cs) {
  if (!(fabsf(x) <= 1.0e6f)) {
    *sn = sinf(x);
    *cs = cosf(x);
    return;
  }
  const float k = rintf(x * 0.63661977236758134f);
  float r = __builtin_fmaf(-k, 1.57079637050628662109375f, x);  // pi/2 = hi + mid + lo
  r = __builtin_fmaf(-k, -4.37113900018624283e-8f, r);
  r = __builtin_fmaf(-k, -1.71512567349610e-15f, r);
  const int q = (int)k;
  const float r2 = r * r;
  const float ps = __builtin_fmaf(__builtin_fmaf(-1.9515295891e-4f, r2, 8.3321608736e-3f), r2, -1.6666654611e-1f);
  const float sr = __builtin_fmaf(r * r2, ps, r);
  const float pc = __builtin_fmaf(__builtin_fmaf(2.443315711809948e-5f, r2, -1.388731625493765e-3f), r2, 4.166664568298827e-2f);
  const float cr = __builtin_fmaf(r2 * r2, pc, __builtin_fmaf(-0.5f, r2, 1.0f));
  const float s0 = (q & 1) ? cr : sr, c0 = (q & 1) ? sr : cr;
  *sn = (q & 2) ? -s0 : s0;
  *cs = ((q + 1) & 2) ? -c0 : c0;
}

// Exchange with the lane 16 / 32 positions away (the two "g" bits).
static __device__ __forceinline__ float xor16(float x) { return __shfl_xor(x, 16, 64); }
static __device__ __forceinline__ float xor32(float x) { return __shfl_xor(x, 32, 64); }

// 16-byte global loads / stores through plain pointers.
static __device__ __forceinline__ uint4 ld16(const void* p) { return *reinterpret_cast<const uint4*>(p); }
static __device__ __forceinline__ uint2 ld8(const void* p) { return *reinterpret_cast<const uint2*>(p); }
// Streaming variants: the data is read exactly once, so it is marked non-temporal.
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2_t;
static __device__ __forceinline__ uint4 ld16_stream(const void* p) {
  const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}
static __device__ __forceinline__ uint2 ld8_stream(const void* p) {
  const u32x2_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x2_t*>(p));
  return make_uint2(v.x, v.y);
}
// N consecutive dwords read once from global memory into registers.  The address is aligned to the largest
// power of two that divides 4 N (at most 16): 12 bytes (N = 3) sit at any multiple of 4, so that load is declared
// with 4-byte alignment and the compiler picks an encoding the alignment allows.
typedef uint32_t u32x3a4_t __attribute__((ext_vector_type(3), aligned(4)));
template <int N>
static __device__ __forceinline__ void ld_dwords_stream(const void* p, uint32_t (&dst)[N]) {
  static_assert(N == 1 || N == 3 || N % 2 == 0, "dword counts of the value fragments");
  if constexpr (N == 1) {
    dst[0] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(p));
  } else if constexpr (N % 4 == 0) {
#pragma unroll
    for (int w = 0; w < N / 4; ++w) {
      const uint4 v = ld16_stream(reinterpret_cast<const uint8_t*>(p) + 16 * w);
      dst[4 * w] = v.x; dst[4 * w + 1] = v.y; dst[4 * w + 2] = v.z; dst[4 * w + 3] = v.w;
    }
  } else if constexpr (N % 2 == 0) {
#pragma unroll
    for (int w = 0; w < N / 2; ++w) {
      const uint2 v = ld8_stream(reinterpret_cast<const uint8_t*>(p) + 8 * w);
      dst[2 * w] = v.x; dst[2 * w + 1] = v.y;
    }
  } else {
    const u32x3a4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x3a4_t*>(p));
    dst[0] = v.x; dst[1] = v.y; dst[2] = v.z;
  }
}
template <int N>
static __device__ __forceinline__ void ld_dwords(const void* p, uint32_t (&dst)[N]) {  // the cacheable form
  static_assert(N == 1 || N == 3 || N % 2 == 0, "dword counts of the value fragments");
  if constexpr (N == 1) {
    dst[0] = *reinterpret_cast<const uint32_t*>(p);
  } else if constexpr (N % 4 == 0) {
#pragma unroll
    for (int w = 0; w < N / 4; ++w) {
      const uint4 v = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint8_t*>(p) + 16 * w);
      dst[4 * w] = v.x; dst[4 * w + 1] = v.y; dst[4 * w + 2] = v.z; dst[4 * w + 3] = v.w;
    }
  } else if constexpr (N % 2 == 0) {
#pragma unroll
    for (int w = 0; w < N / 2; ++w) {
      const uint2 v = *reinterpret_cast<const uint2*>(reinterpret_cast<const uint8_t*>(p) + 8 * w);
      dst[2 * w] = v.x; dst[2 * w + 1] = v.y;
    }
  } else {
    const u32x3a4_t v = *reinterpret_cast<const u32x3a4_t*>(p);
    dst[0] = v.x; dst[1] = v.y; dst[2] = v.z;
  }
}
// N consecutive dwords written from registers, same alignment rule.
template <int N>
static __device__ __forceinline__ void st_dwords(void* p, const uint32_t (&src)[N]) {
  static_assert(N == 3 || N % 2 == 0, "dword counts of the output fragments");
  if constexpr (N % 4 == 0) {
#pragma unroll
    for (int w = 0; w < N / 4; ++w)
      *reinterpret_cast<uint4*>(reinterpret_cast<uint8_t*>(p) + 16 * w) =
          make_uint4(src[4 * w], src[4 * w + 1], src[4 * w + 2], src[4 * w + 3]);
  } else if constexpr (N % 2 == 0) {
#pragma unroll
    for (int w = 0; w < N / 2; ++w)
      *reinterpret_cast<uint2*>(reinterpret_cast<uint8_t*>(p) + 8 * w) = make_uint2(src[2 * w], src[2 * w + 1]);
  } else {
    u32x3a4_t v = {src[0], src[1], src[2]};
    *reinterpret_cast<u32x3a4_t*>(p) = v;
  }
}
static __device__ __forceinline__ void st16(void* p, uint4 v) { *reinterpret_cast<uint4*>(p) = v; }
static __device__ __forceinline__ void st8(void* p, uint2 v) { *reinterpret_cast<uint2*>(p) = v; }

// 16-byte LDS read that stays one ds_read_b128: the empty asm uses the whole vector, which keeps
// the compiler from narrowing the load into strided dword reads (those conflict on the banks).
static __device__ __forceinline__ uint4 lds_ld16(const void* p) {
  u32x4_t v = *reinterpret_cast<const u32x4_t*>(p);
  asm volatile("" : "+v"(v));
  return make_uint4(v.x, v.y, v.z, v.w);
}

typedef short s16x4v __attribute__((ext_vector_type(4)));

// Transposing LDS read: within each block of 16 lanes, lane i supplies the address of 4 bf16
// (row i/4, columns 4*(i%4)..+3 of a 4 x 16 matrix) and lane L receives column L of that matrix.
static __device__ __forceinline__ uint2 lds_ld8_tr(const uint8_t* ptr) {
  const s16x4v v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (__attribute__((address_space(3))) s16x4v*)(uintptr_t)(uint32_t)(uintptr_t)ptr);
  return __builtin_bit_cast(uint2, v);
}

// Value of lane (l ^ P), P a power of two: data-parallel-primitive moves inside a row of 16 lanes (quad permutes, the
// rotate by 8), the LDS crossbar's bit-mask swizzle for 4 and 16 (no address register, no bounds arithmetic), the
// generic shuffle for 32.
template <int P>
static __device__ __forceinline__ float lane_xor(float x) {
  const int v = __float_as_int(x);
  if constexpr (P == 1) return __int_as_float(__builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true));        // quad_perm [1,0,3,2]
  else if constexpr (P == 2) return __int_as_float(__builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
  else if constexpr (P == 4) return __int_as_float(__builtin_amdgcn_ds_swizzle(v, 0x101F));                    // lane ^ 4
  else if constexpr (P == 8) return __int_as_float(__builtin_amdgcn_update_dpp(0, v, 0x128, 0xF, 0xF, true));  // row_ror:8
  else if constexpr (P == 16) return __int_as_float(__builtin_amdgcn_ds_swizzle(v, 0x401F));                   // lane ^ 16
  else return __shfl_xor(x, 32, 64);
}
// Sum over the aligned group of N lanes (N = 8, 16, 32) a lane belongs to; every lane ends with the total.
template <int N>
static __device__ __forceinline__ float lane_group_sum(float x) {
  x += lane_xor<1>(x);
  x += lane_xor<2>(x);
  x += lane_xor<4>(x);
  if constexpr (N >= 16) x += lane_xor<8>(x);
  if constexpr (N >= 32) x += lane_xor<16>(x);
  return x;
}

// max over the four lanes {l, l^16, l^32, l^48} with two lane-swap instructions
static __device__ __forceinline__ float rowgroup_max(float x) {
  const uint32_t u = __float_as_uint(x);
  const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  const float y = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  const uint32_t w = __float_as_uint(y);
  const auto b = __builtin_amdgcn_permlane32_swap(w, w, false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}

// OCP e4m3fn byte pairs -> fp32 (gfx950 converts OCP formats natively).
static __device__ __forceinline__ f32x2_t fp8x2_lo_to_f32(uint32_t w) {
  return __builtin_amdgcn_cvt_pk_f32_fp8((int)w, false);
}
static __device__ __forceinline__ f32x2_t fp8x2_hi_to_f32(uint32_t w) {
  return __builtin_amdgcn_cvt_pk_f32_fp8((int)w, true);
}
// Four e4m3fn bytes -> two packed bf16 pairs.  gfx950 converts a pair of OCP fp8 values to
// a packed bf16 pair in one instruction (with a multiplier, 1.0 here); the conversion is
// exact because every e4m3 value is representable in bf16.
static __device__ __forceinline__ uint2 fp8x4_to_bf16x4(uint32_t w) {
  const bf16x2_t lo = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, false);
  const bf16x2_t hi = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, true);
  return make_uint2(__builtin_bit_cast(uint32_t, lo), __builtin_bit_cast(uint32_t, hi));
}

// The same into the operand type of the kernel: bf16 pairs, or fp16 pairs (exact as well: e4m3 has 3 mantissa bits
// and its exponents lie inside fp16's).
template <bool F16>
static __device__ __forceinline__ uint2 fp8x4_to_16x4(uint32_t w) {
  if constexpr (F16) {
    typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
    const f16x2_t lo = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, false);
    const f16x2_t hi = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, true);
    return make_uint2(__builtin_bit_cast(uint32_t, lo), __builtin_bit_cast(uint32_t, hi));
  } else {
    return fp8x4_to_bf16x4(w);
  }
}

// fp32 -> e4m3fn byte, round to nearest even, saturating (no NaN / inf produced).
static __device__ __forceinline__ uint32_t f32_to_e4m3_sat(float x) {
  x = fminf(fmaxf(x, -448.f), 448.f);
  // v_cvt_pk_fp8_f32 packs two conversions into the low 16 bits.
  const int r = __builtin_amdgcn_cvt_pk_fp8_f32(x, 0.f, 0, false);
  return (uint32_t)r & 0xffu;
}

}  // namespace mi
