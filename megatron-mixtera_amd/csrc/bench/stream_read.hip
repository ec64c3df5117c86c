// Measurement aid for bench.py, not part of the C ABI of the product library: a plain streaming read of
// a device buffer, used to record what fraction of the published HBM peak a read-only kernel reaches on
// the box the benchmark runs on (the ceiling the KV-streaming decode kernel is compared with).
//
// 512-thread workgroups; every thread issues four independent 16-byte loads per iteration (the same
// bytes in flight per wavefront as the decode kernel's 32-token tile), XOR-reduces what it read and
// writes one word per workgroup, so nothing is optimised away and the write traffic is negligible.
// Built into libmi355_bench.so next to the product library.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;

template <bool NT>
__global__ __launch_bounds__(512) void stream_read_kernel(const u32x4_t* __restrict__ src, int64_t n_vec,
                                                          uint32_t* __restrict__ sink) {
  // contiguous span per workgroup, as the decode kernel cuts its tile sequence
  const int64_t per = (n_vec + gridDim.x - 1) / gridDim.x;
  const int64_t begin = (int64_t)blockIdx.x * per;
  const int64_t end = begin + per < n_vec ? begin + per : n_vec;
  u32x4_t acc = {0u, 0u, 0u, 0u};
  int64_t i = begin + threadIdx.x;
  for (; i + 3 * 512 < end; i += 4 * 512) {
    u32x4_t a, b, c, d;
    if (NT) {
      a = __builtin_nontemporal_load(src + i);
      b = __builtin_nontemporal_load(src + i + 512);
      c = __builtin_nontemporal_load(src + i + 1024);
      d = __builtin_nontemporal_load(src + i + 1536);
    } else {
      a = src[i]; b = src[i + 512]; c = src[i + 1024]; d = src[i + 1536];
    }
    acc ^= a ^ b ^ c ^ d;
  }
  for (; i < end; i += 512) acc ^= NT ? __builtin_nontemporal_load(src + i) : src[i];
  uint32_t x = acc.x ^ acc.y ^ acc.z ^ acc.w;
  for (int o = 32; o > 0; o >>= 1) x ^= __shfl_xor(x, o, 64);
  __shared__ uint32_t part[8];
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = x;
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t y = 0;
    for (int w = 0; w < 8; ++w) y ^= part[w];
    sink[blockIdx.x] = y;
  }
}

}  // namespace

// Enqueue one streaming read of `bytes` bytes (a multiple of 16) at `src` on `stream`.
// `sink` receives one 32-bit word per workgroup (`workgroups` of them).  Returns 0, or -1 for bad arguments.
extern "C" int mi_bench_stream_read(const void* src, int64_t bytes, uint32_t* sink, int32_t workgroups,
                                    int32_t nontemporal, void* stream) {
  if (!src || !sink || bytes <= 0 || bytes % 16 || workgroups <= 0 || ((uintptr_t)src & 15)) return -1;
  const int64_t n_vec = bytes / 16;
  if (nontemporal)
    hipLaunchKernelGGL(stream_read_kernel<true>, dim3(workgroups), dim3(512), 0, (hipStream_t)stream,
                       (const u32x4_t*)src, n_vec, sink);
  else
    hipLaunchKernelGGL(stream_read_kernel<false>, dim3(workgroups), dim3(512), 0, (hipStream_t)stream,
                       (const u32x4_t*)src, n_vec, sink);
  return hipGetLastError() == hipSuccess ? 0 : -2;
}
