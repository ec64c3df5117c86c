// Measurement aids for bench.py (not part of the C ABI of the product library): three probes of one compute
// unit that explain what bounds the prefill tile kernel.
//   1. LDS read rate: 1, 4, 8 or 16 wavefronts of a workgroup read fragments the way the tile kernel does
//      (16-byte reads of 16 rows with a 288-byte pitch, or the transposing 8-byte reads); bytes per core clock
//      per wavefront and per CU.
//   2. The same 16-byte fragment pattern straight from global memory (a 128 KiB region per workgroup, resident
//      in the vector L1 after the first pass): what the path through the texture unit delivers per CU.
//   3. Matrix / vector co-execution: wavefronts w and w+4 of a 512-thread workgroup share a SIMD; one streams
//      matrix instructions (16x16x32 or 32x32x16 bf16), the other ordinary fp32 fma or exp2 instructions; core
//      clocks per instruction for each, alone and side by side.
//   4. One or two wavefronts per SIMD running the whole instruction mix of a 64-key attention tile (matrix
//      instructions 16x16x32, key and transposing value fragment reads, the softmax's vector arithmetic) woven into
//      one stream each: clocks per tile, i.e. what the matrix cores can be kept busy at without separate phases.
// Every probe reports core clocks (clock64) and, for the clock itself, the ratio to the 100 MHz wall clock.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
typedef short s16x4v __attribute__((ext_vector_type(4)));
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;

constexpr int kPitch = 288;  // bytes per staged 128-value row, as in the tile kernel

// MODE 0: ds_read_b128 fragments, 1: ds_read_b64_tr_b16 fragments, 2: 16-byte fragments from global memory.
// DEPTH: fragments (16 bytes a lane each) requested before the first of them is waited for.
template <int MODE, int DEPTH>
__global__ __launch_bounds__(1024) void read_probe(uint32_t* sink, long long* cycles, int iters, const uint8_t* gsrc) {
  __shared__ __attribute__((aligned(16))) uint8_t lds[64 * kPitch];
  const int tid = threadIdx.x, lane = tid & 63;
  for (int i = tid * 16; i < 64 * kPitch; i += blockDim.x * 16)
    *reinterpret_cast<u32x4_t*>(lds + i) = u32x4_t{(uint32_t)i, 1u, 2u, 3u};
  __syncthreads();
  const int m16 = lane & 15, g = lane >> 4;
  const uint8_t* kp = lds + m16 * kPitch + 16 * g;
  const uint8_t* vp = lds + (4 * g + (m16 >> 2)) * kPitch + 8 * (m16 & 3);
  const uint8_t* gp = gsrc + (size_t)blockIdx.x * 64 * 2048 + m16 * 2048 + 16 * g;  // rows 2 KiB apart: 8 KV heads
  u32x4_t acc = {0, 0, 0, 0};
  const long long t0 = clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int f0 = 0; f0 < 16; f0 += DEPTH) {
      u32x4_t v[DEPTH];
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        const int f = f0 + d;
        if (MODE == 1) {
          const int s2 = f >> 3, e = f & 7;
          const s16x4v a = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (__attribute__((address_space(3))) s16x4v*)(uintptr_t)(uint32_t)(uintptr_t)(vp + 32 * s2 * kPitch + 32 * e));
          const s16x4v b = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (__attribute__((address_space(3))) s16x4v*)(uintptr_t)(uint32_t)(uintptr_t)(vp + (32 * s2 + 16) * kPitch + 32 * e));
          const uint2 a2 = __builtin_bit_cast(uint2, a), b2 = __builtin_bit_cast(uint2, b);
          v[d] = u32x4_t{a2.x, a2.y, b2.x, b2.y};
        } else {
          const int u = f >> 2, kk = f & 3;
          v[d] = MODE == 0 ? *reinterpret_cast<const u32x4_t*>(kp + 16 * u * kPitch + 64 * kk)
                           : *reinterpret_cast<const u32x4_t*>(gp + 16 * u * 2048 + 64 * kk);
        }
      }
      __builtin_amdgcn_sched_barrier(0);  // all DEPTH requests before the first use
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        asm volatile("" : "+v"(v[d]));
        acc ^= v[d];
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  const long long t1 = clock64();
  sink[blockIdx.x * blockDim.x + tid] = acc.x ^ acc.y ^ acc.z ^ acc.w;
  if (lane == 0 && blockIdx.x == 0) cycles[tid >> 6] = t1 - t0;
}

template <int MODE>
int run_read(int depth, int workgroups, int waves, hipStream_t st, uint32_t* sink, long long* cycles, int iters, const uint8_t* gsrc) {
  if (depth == 1) hipLaunchKernelGGL((read_probe<MODE, 1>), dim3(workgroups), dim3(64 * waves), 0, st, sink, cycles, iters, gsrc);
  else if (depth == 4) hipLaunchKernelGGL((read_probe<MODE, 4>), dim3(workgroups), dim3(64 * waves), 0, st, sink, cycles, iters, gsrc);
  else hipLaunchKernelGGL((read_probe<MODE, 16>), dim3(workgroups), dim3(64 * waves), 0, st, sink, cycles, iters, gsrc);
  return hipGetLastError() == hipSuccess ? 0 : -2;
}

// W: 0 idle, 1 mfma 16x16x32, 2 mfma 32x32x16, 3 fp32 fma, 4 exp2.  32 (W 1, 3, 4) or 16 (W 2) instructions per iteration.
template <int W>
static __device__ __forceinline__ float work(int lane, int iters) {
  if (W == 1 || W == 2) {
    bf16x8_t a, b;
    for (int i = 0; i < 8; ++i) { a[i] = (__bf16)(float)(lane + i); b[i] = (__bf16)(float)(lane - i); }
    if (W == 1) {
      f32x4_t c0 = {}, c1 = {}, c2 = {}, c3 = {};
      for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          c0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c0, 0, 0, 0);
          c1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c1, 0, 0, 0);
          c2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c2, 0, 0, 0);
          c3 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c3, 0, 0, 0);
        }
      }
      return c0[0] + c1[1] + c2[2] + c3[3];
    }
    f32x16_t c0 = {}, c1 = {};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c0, 0, 0, 0);
        c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c1, 0, 0, 0);
      }
    }
    return c0[0] + c1[3];
  }
  if (W == 3 || W == 4) {
    float x[8];
    for (int i = 0; i < 8; ++i) x[i] = lane * 0.001f + i;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] = W == 3 ? __builtin_fmaf(x[i], 0.999f, 0.5f) : __builtin_amdgcn_exp2f(x[i]);
    }
    return x[0] + x[1] + x[2] + x[3] + x[4] + x[5] + x[6] + x[7];
  }
  return 0.f;
}

template <int A, int B>
__global__ __launch_bounds__(512) void coexec_probe(long long* cycles, float* sink, int iters) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  __syncthreads();
  const long long t0 = clock64(), w0 = wall_clock64();
  const float r = wave < 4 ? work<A>(lane, iters) : work<B>(lane, iters);
  const long long t1 = clock64(), w1 = wall_clock64();
  sink[blockIdx.x * 512 + threadIdx.x] = r;
  if (lane == 0 && blockIdx.x == 0) {
    cycles[wave] = t1 - t0;
    cycles[8 + wave] = w1 - w0;
  }
}

template <int A, int B>
int run_coexec(long long* cycles, float* sink, int iters, int workgroups, hipStream_t st) {
  hipLaunchKernelGGL((coexec_probe<A, B>), dim3(workgroups), dim3(512), 0, st, cycles, sink, iters);
  return hipGetLastError() == hipSuccess ? 0 : -2;
}

static __device__ __forceinline__ uint2 lds_tr(const uint8_t* p) {
  const s16x4v v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4v*)(uintptr_t)(uint32_t)(uintptr_t)p);
  return __builtin_bit_cast(uint2, v);
}

// The instruction mix of a 64-key attention tile for ROWS query rows per wavefront at 128 values per head, per tile:
// 16 key fragments (ds_read_b128) and 16 value fragments (two ds_read_b64_tr_b16 each), every fragment feeding ROWS/16
// products 16x16x32; ROWS exponentials per lane with their max / fma / sum; scores out of, probabilities into, the
// product operands.  ROWS 64: four wavefronts a workgroup, the SIMD's whole register file each; ROWS 32: eight.
// WEAVE: vector work between the matrix instructions (true) or all of it after them (false).
// LEAN: per score only fma + exponential (+ pack): no running maximum, no sum (a kernel that takes its exponentials
// against a fixed reference and lets the matrix cores add the denominators).
template <int ROWS, bool WEAVE, bool LEAN>
__global__ __launch_bounds__(ROWS == 64 ? 256 : 512, 1) void woven_probe(long long* cycles, float* sink, int iters) {
  constexpr int R16 = ROWS / 16, kGroups = 16 * R16;
  __shared__ __attribute__((aligned(16))) uint8_t lds[2][64 * kPitch];  // a key and a value tile (contents do not matter)
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int i = tid * 16; i < 2 * 64 * kPitch; i += blockDim.x * 16)
    *reinterpret_cast<u32x4_t*>(&lds[0][0] + i) = u32x4_t{0x3c003c00u, 0x3c003c00u, 0x3c003c00u, 0x3c003c00u};
  __syncthreads();
  const int m16 = lane & 15, g = lane >> 4;
  const uint8_t* kbase = &lds[0][0] + m16 * kPitch + 16 * g;
  const uint8_t* vbase = &lds[1][0] + (4 * g + (m16 >> 2)) * kPitch + 8 * (m16 & 3);
  f32x4_t acc_o[8 * R16], acc_s[4 * R16];
#pragma unroll
  for (int i = 0; i < 8 * R16; ++i) acc_o[i] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int i = 0; i < 4 * R16; ++i) acc_s[i] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  u32x4_t q[4 * R16], pr[2 * R16];
#pragma unroll
  for (int i = 0; i < 4 * R16; ++i) q[i] = u32x4_t{0x3c003c00u + lane, 0x3c003c00u, 0x3c003c00u + i, 0x3c003c00u};
#pragma unroll
  for (int i = 0; i < 2 * R16; ++i) pr[i] = u32x4_t{0x3c003c00u, 0x3c003c00u + lane, 0x3c003c00u, 0x3c003c00u + i};
  float sprev[ROWS];
#pragma unroll
  for (int i = 0; i < ROWS; ++i) sprev[i] = lane * 0.001f + i * 0.01f;
  float mx = -1e30f, sum = 0.f;
  const float scale = 0.125f;
  auto read_k = [&](int f) { return *reinterpret_cast<const u32x4_t*>(kbase + 16 * ((f / 4) % 4) * kPitch + 64 * (f % 4)); };
  auto read_v = [&](int f) {
    const int e = f % 8, ks = (f / 8) % 2;
    const uint2 a = lds_tr(vbase + 32 * ks * kPitch + 32 * e), b = lds_tr(vbase + (32 * ks + 16) * kPitch + 32 * e);
    return u32x4_t{a.x, a.y, b.x, b.y};
  };
  u32x4_t kf[4], vf[4];  // fragment f lives in slot f & 3 and is requested two fragments ahead of its first product
  kf[0] = read_k(0);
  vf[0] = read_v(0);
  kf[1] = read_k(1);
  vf[1] = read_v(1);
#define SB() __builtin_amdgcn_sched_barrier(0)
  __syncthreads();
  const long long t0 = clock64(), w0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
    float e_keep[ROWS];
#pragma unroll
    for (int grp = 0; grp < kGroups; ++grp) {
      const int f = grp / R16;
      if (grp % R16 == 0) {
        kf[(f + 2) & 3] = read_k((f + 2) % 16);
        vf[(f + 2) & 3] = read_v((f + 2) % 16);
      }
      SB();
      acc_s[grp % (4 * R16)] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
          __builtin_bit_cast(bf16x8_t, kf[f & 3]), __builtin_bit_cast(bf16x8_t, q[grp % (4 * R16)]), acc_s[grp % (4 * R16)], 0, 0, 0);
      acc_o[grp % (8 * R16)] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
          __builtin_bit_cast(bf16x8_t, vf[f & 3]), __builtin_bit_cast(bf16x8_t, pr[grp % (2 * R16)]), acc_o[grp % (8 * R16)], 0, 0, 0);
      if (WEAVE) {  // the softmax arithmetic of one score of the previous tile
        if (!LEAN) mx = fmaxf(mx, sprev[grp]);
        const float e = __builtin_amdgcn_exp2f(__builtin_fmaf(sprev[grp], scale, -mx));
        if (!LEAN) sum += e;
        e_keep[grp] = e;
      }
      SB();
    }
    if (!WEAVE) {
#pragma unroll
      for (int grp = 0; grp < kGroups; ++grp) {
        mx = fmaxf(mx, sprev[grp]);
        const float e = __builtin_amdgcn_exp2f(__builtin_fmaf(sprev[grp], scale, -mx));
        sum += e;
        e_keep[grp] = e;
      }
    }
    // the tile's scores become the next tile's softmax input; its probabilities the next value operands
#pragma unroll
    for (int i = 0; i < 4 * R16; ++i) {
#pragma unroll
      for (int j = 0; j < 4; ++j) sprev[4 * i + j] = acc_s[i][j];
      acc_s[i] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int i = 0; i < 2 * R16; ++i) {
      uint32_t w[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float a = e_keep[8 * i + 2 * j], b = e_keep[8 * i + 2 * j + 1];
        w[j] = (__builtin_bit_cast(uint32_t, a) >> 16) | (__builtin_bit_cast(uint32_t, b) & 0xffff0000u);
      }
      pr[i] = u32x4_t{w[0], w[1], w[2], w[3]};
    }
  }
  const long long t1 = clock64(), w1 = wall_clock64();
#undef SB
  float r = mx + sum;
#pragma unroll
  for (int i = 0; i < 8 * R16; ++i) r += acc_o[i][0] + acc_o[i][3];
  sink[blockIdx.x * blockDim.x + tid] = r;
  if (lane == 0 && blockIdx.x == 0) {
    cycles[wave] = t1 - t0;
    cycles[8 + wave] = w1 - w0;
  }
}

}  // namespace

// rows 64: four wavefronts a workgroup, 128 matrix instructions per wavefront and tile; rows 32: eight wavefronts, 64 each.
// `weave` 1: vector work between the matrix instructions, 0: after them, 2: between them and only fma + exponential per score.  cycles_out (device, int64 [16]): [w] core
// clocks of wavefront w (< 8) of workgroup 0, [8 + w] its wall-clock ticks.  sink: device, workgroups * 512 floats.
extern "C" int mi_bench_woven_probe(int32_t rows, int32_t weave, int32_t workgroups, int32_t iters, long long* cycles_out,
                                    float* sink, void* stream) {
  if (!cycles_out || !sink || workgroups < 1 || iters < 1 || (rows != 32 && rows != 64)) return -1;
  hipStream_t st = (hipStream_t)stream;
  if (rows == 64 && weave == 2) hipLaunchKernelGGL((woven_probe<64, true, true>), dim3(workgroups), dim3(256), 0, st, cycles_out, sink, iters);
  else if (rows == 64 && weave) hipLaunchKernelGGL((woven_probe<64, true, false>), dim3(workgroups), dim3(256), 0, st, cycles_out, sink, iters);
  else if (rows == 64) hipLaunchKernelGGL((woven_probe<64, false, false>), dim3(workgroups), dim3(256), 0, st, cycles_out, sink, iters);
  else if (weave == 2) hipLaunchKernelGGL((woven_probe<32, true, true>), dim3(workgroups), dim3(512), 0, st, cycles_out, sink, iters);
  else if (weave) hipLaunchKernelGGL((woven_probe<32, true, false>), dim3(workgroups), dim3(512), 0, st, cycles_out, sink, iters);
  else hipLaunchKernelGGL((woven_probe<32, false, false>), dim3(workgroups), dim3(512), 0, st, cycles_out, sink, iters);
  return hipGetLastError() == hipSuccess ? 0 : -2;
}

// mode 0 / 1 / 2 as read_probe; `depth` fragments in flight per wavefront (1, 4 or 16); `waves` wavefronts per workgroup
// (1..16), one workgroup per CU (`workgroups` of them).
// cycles_out (device, int64 [16]): core clocks each wavefront of workgroup 0 took for `iters` x 16 KiB.
// sink: device, workgroups * 1024 words; gsrc: device, workgroups * 128 KiB (mode 2 only).
extern "C" int mi_bench_read_probe(int32_t mode, int32_t depth, int32_t waves, int32_t workgroups, int32_t iters,
                                   long long* cycles_out, uint32_t* sink, const void* gsrc, void* stream) {
  if (mode < 0 || mode > 2 || (depth != 1 && depth != 4 && depth != 16) || waves < 1 || waves > 16 || workgroups < 1 ||
      iters < 1 || !cycles_out || !sink || (mode == 2 && !gsrc))
    return -1;
  hipStream_t st = (hipStream_t)stream;
  const uint8_t* g = (const uint8_t*)gsrc;
  if (mode == 0) return run_read<0>(depth, workgroups, waves, st, sink, cycles_out, iters, g);
  if (mode == 1) return run_read<1>(depth, workgroups, waves, st, sink, cycles_out, iters, g);
  return run_read<2>(depth, workgroups, waves, st, sink, cycles_out, iters, g);
}

// Work of wavefronts 0-3 (a) and 4-7 (b) of every workgroup: 0 idle, 1 mfma 16x16x32, 2 mfma 32x32x16, 3 fma, 4 exp2.
// cycles_out (device, int64 [16]): [w] core clocks of wavefront w of workgroup 0, [8 + w] its 100 MHz wall-clock ticks.
// sink: device, workgroups * 512 floats.
extern "C" int mi_bench_coexec_probe(int32_t a, int32_t b, int32_t workgroups, int32_t iters, long long* cycles_out,
                                     float* sink, void* stream) {
  if (!cycles_out || !sink || workgroups < 1 || iters < 1) return -1;
  hipStream_t st = (hipStream_t)stream;
  switch (a * 8 + b) {
    case 1 * 8 + 0: return run_coexec<1, 0>(cycles_out, sink, iters, workgroups, st);
    case 2 * 8 + 0: return run_coexec<2, 0>(cycles_out, sink, iters, workgroups, st);
    case 3 * 8 + 0: return run_coexec<3, 0>(cycles_out, sink, iters, workgroups, st);
    case 4 * 8 + 0: return run_coexec<4, 0>(cycles_out, sink, iters, workgroups, st);
    case 3 * 8 + 3: return run_coexec<3, 3>(cycles_out, sink, iters, workgroups, st);
    case 1 * 8 + 3: return run_coexec<1, 3>(cycles_out, sink, iters, workgroups, st);
    case 1 * 8 + 4: return run_coexec<1, 4>(cycles_out, sink, iters, workgroups, st);
    case 2 * 8 + 3: return run_coexec<2, 3>(cycles_out, sink, iters, workgroups, st);
    case 2 * 8 + 4: return run_coexec<2, 4>(cycles_out, sink, iters, workgroups, st);
    case 1 * 8 + 1: return run_coexec<1, 1>(cycles_out, sink, iters, workgroups, st);
    default: return -1;
  }
}
