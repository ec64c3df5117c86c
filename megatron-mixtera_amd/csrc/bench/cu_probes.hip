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

// MODE 0: ds_read_b128 fragments, 1: ds_read_b64_tr_b16 fragments, 2: 16-byte fragments from global memory
template <int MODE>
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
    if (MODE == 1) {
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          s16x4v a = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (__attribute__((address_space(3))) s16x4v*)(uintptr_t)(uint32_t)(uintptr_t)(vp + 32 * s2 * kPitch + 32 * e));
          s16x4v b = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (__attribute__((address_space(3))) s16x4v*)(uintptr_t)(uint32_t)(uintptr_t)(vp + (32 * s2 + 16) * kPitch + 32 * e));
          asm volatile("" : "+v"(a), "+v"(b));
          acc.x ^= (uint32_t)a.x ^ (uint32_t)b.y;
        }
    } else {
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
          u32x4_t v = MODE == 0 ? *reinterpret_cast<const u32x4_t*>(kp + 16 * u * kPitch + 64 * kk)
                                : *reinterpret_cast<const u32x4_t*>(gp + 16 * u * 2048 + 64 * kk);
          asm volatile("" : "+v"(v));
          acc ^= v;
        }
    }
  }
  const long long t1 = clock64();
  sink[blockIdx.x * blockDim.x + tid] = acc.x ^ acc.y ^ acc.z ^ acc.w;
  if (lane == 0 && blockIdx.x == 0) cycles[tid >> 6] = t1 - t0;
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

}  // namespace

// mode 0 / 1 / 2 as read_probe; `waves` wavefronts per workgroup (1..16), one workgroup per CU (`workgroups` of them).
// cycles_out (device, int64 [16]): core clocks each wavefront of workgroup 0 took for `iters` x 16 KiB.
// sink: device, workgroups * 1024 words; gsrc: device, workgroups * 128 KiB (mode 2 only).
extern "C" int mi_bench_read_probe(int32_t mode, int32_t waves, int32_t workgroups, int32_t iters, long long* cycles_out,
                                   uint32_t* sink, const void* gsrc, void* stream) {
  if (mode < 0 || mode > 2 || waves < 1 || waves > 16 || workgroups < 1 || iters < 1 || !cycles_out || !sink ||
      (mode == 2 && !gsrc))
    return -1;
  hipStream_t st = (hipStream_t)stream;
  if (mode == 0) hipLaunchKernelGGL(read_probe<0>, dim3(workgroups), dim3(64 * waves), 0, st, sink, cycles_out, iters, (const uint8_t*)gsrc);
  else if (mode == 1) hipLaunchKernelGGL(read_probe<1>, dim3(workgroups), dim3(64 * waves), 0, st, sink, cycles_out, iters, (const uint8_t*)gsrc);
  else hipLaunchKernelGGL(read_probe<2>, dim3(workgroups), dim3(64 * waves), 0, st, sink, cycles_out, iters, (const uint8_t*)gsrc);
  return hipGetLastError() == hipSuccess ? 0 : -2;
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
