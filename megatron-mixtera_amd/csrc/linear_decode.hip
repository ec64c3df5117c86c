// The two projections either side of the attention path, at decode size:  y[T, N] = x[T, K] . W[N, K]^T (+ bias).
//
// Replaces, for steps of at most 256 tokens,
//   mixed_qkv, _ = self.linear_qkv(hidden_states)        (megatron/core/transformer/attention.py:985-992; N = (Hq + 2 Hkv) d)
//   output, bias = self.linear_proj(core_attn_out)       (attention.py:829-845; skip_bias_add: the bias is returned, not added)
// as ColumnParallelLinear / RowParallelLinear compute them at tensor-parallel size 1
// (megatron/core/tensor_parallel/layers.py:946-1010,1225-1290): 16-bit inputs, fp32 accumulation, 16-bit result.
// With a few dozen rows of x the weight matrix is the traffic -- 50 MB for 4096 -> 6144 -- and each of its bytes is
// used once: the kernel is a stream of W from HBM with the products riding along.
//
// Work split: a workgroup of 8 wavefronts takes 128 rows of W (16 per wavefront, the A operand of mfma 16x16x32)
// times one slice of at most 512 columns of K, for a block of at most 64 tokens.  Every wavefront asks for its whole
// share of W at once -- sixteen 16-byte loads per lane, 16 KB per wavefront, non-temporal, whole cache lines per
// instruction -- so the launch has the entire matrix in flight from its second microsecond, and multiplies each
// piece as it arrives; before that the workgroup stages its slice of x in LDS (64 tokens x 512 values, read by all 8
// wavefronts as the B operand).  Slices of K end in fp32 partial sums
// (one contiguous tile of T x 16 per slice and wavefront) that a second, small kernel adds up in a fixed order (so results do not depend on timing), adds the
// bias to and rounds; a call whose K fits one slice writes its 16-bit result directly.
#include "mi_common.h"
#include "mi_capi_internal.h"

namespace mi {

constexpr int kLinRows = 128;    // rows of W per workgroup (8 wavefronts x 16)
constexpr int kLinSlice = 512;   // columns of K per workgroup, at most
constexpr int kLinTok = 64;      // tokens per workgroup, at most
constexpr int kLinPitch = kLinSlice * 2 + 32;  // LDS bytes per staged row of x: an odd multiple of 32 (conflict-free fragments)

struct LinearParams {
  const uint16_t* x; int64_t x_st;
  const uint16_t* w; int64_t w_st;
  const uint16_t* bias;
  uint16_t* out; int64_t o_st;
  float* part;   // S > 1: [S][N / 16][T][16] -- a wavefront's 16 rows of W for every token, contiguous
  int32_t T, N, K, kslice, S;
};

template <bool F16>
__global__ __launch_bounds__(512, 4) void linear_decode_kernel(LinearParams p) {
  __shared__ __attribute__((aligned(16))) uint8_t xs[kLinTok * kLinPitch];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int m16 = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * kLinRows + 16 * wave;     // this wavefront's 16 rows of W
  const int k0 = blockIdx.y * p.kslice;                 // this workgroup's slice of K
  const int klen = min(p.kslice, p.K - k0);             // (a multiple of 32)
  const int t0 = blockIdx.z * kLinTok;
  const int nt = min(kLinTok, p.T - t0);                // tokens of this block
  const int nkk = klen >> 5;                            // 32-column steps of the products (<= 16)
  const bool rows_live = n0 < p.N;                      // (wave-uniform; N is a multiple of 16)

  // ---- x[t0 .. t0 + nt)[k0 .. k0 + klen) -> LDS (rows and columns beyond stay zero).  Before anything of W is asked
  // for: loads are served in the order a CU issued them, and behind sixteen loads of W per lane these few cache
  // hits would wait for microseconds ----
  {
    constexpr int PPR = kLinSlice / 8;  // 16-byte pieces per staged row
#pragma unroll
    for (int i = 0; i < kLinTok * PPR / 512; ++i) {
      const int piece = tid + 512 * i, row = piece / PPR, col = piece - row * PPR;
      uint4 v = make_uint4(0u, 0u, 0u, 0u);
      if (row < nt && 8 * col < klen) v = ld16(p.x + (int64_t)(t0 + row) * p.x_st + k0 + 8 * col);
      *reinterpret_cast<uint4*>(xs + row * kLinPitch + 16 * col) = v;
    }
  }
  __syncthreads();
  // ---- this wavefront's share of W.  The products want lane (m16, g) to hold columns 32 kk + 8 g .. + 7 of row
  // n0 + m16; loaded that way an instruction touches 64 bytes of each of 16 rows, half a cache line each.  So a pair
  // of loads covers whole lines instead -- load 2 j: rows n0 .. + 7, load 2 j + 1: rows n0 + 8 .. + 15, each lane
  // (m16, g) the 16 bytes at column 64 j + 8 (g + 4 (m16 >> 3)) of row (m16 & 7) -- and two moves per register within
  // the 16-lane rows put the halves where the products expect them. ----
  uint4 wf[kLinSlice / 32];
  {
    const int lo = m16 & 7, hi = m16 >> 3;
    const int col = 8 * (g + 4 * hi);   // within a 64-column pair of steps
    const uint16_t* wrow = p.w + (int64_t)min(n0 + lo, p.N - 1) * p.w_st + k0 + col;
    const int64_t half = 8 * p.w_st;    // (N is a multiple of 16: rows n0 + 8 .. exist whenever rows_live)
#pragma unroll
    for (int j = 0; j < kLinSlice / 64; ++j) {
      const bool live = rows_live && 64 * j + col < klen;
      wf[2 * j] = live ? ld16_stream(wrow + 64 * j) : make_uint4(0u, 0u, 0u, 0u);
      wf[2 * j + 1] = live ? ld16_stream(wrow + half + 64 * j) : make_uint4(0u, 0u, 0u, 0u);
    }
  }
  if (!rows_live) return;

  const int ntile = (nt + 15) >> 4;  // 16-token tiles with a live token
  f32x4_t acc[kLinTok / 16];
#pragma unroll
  for (int i = 0; i < kLinTok / 16; ++i) acc[i] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const uint8_t* xfrag = xs + m16 * kLinPitch + 16 * g;  // B operand: lane (token m16, g) supplies x[token][32 kk + 8 g ..]
  // (fully unrolled with wave-uniform guards: the fragments must stay in registers, and a loop that is left early
  // would index them at run time)
#pragma unroll
  for (int kk = 0; kk < kLinSlice / 32; ++kk) {
    if ((kk & 1) == 0 && kk < nkk) {
      // lanes 8-15 of every 16 take the rows-8-15 load's lanes 0-7 (columns 8 g ..), lanes 0-7 the rows-0-7 load's
      // lanes 8-15 (columns 32 + 8 g ..): row_ror:8 with a bank mask writes just those lanes
      const uint4 a = wf[kk], b = wf[kk + 1];
      auto upper = [](uint32_t keep, uint32_t from) { return (uint32_t)__builtin_amdgcn_update_dpp((int)keep, (int)from, 0x128, 0xf, 0xc, false); };
      auto lower = [](uint32_t keep, uint32_t from) { return (uint32_t)__builtin_amdgcn_update_dpp((int)keep, (int)from, 0x128, 0xf, 0x3, false); };
      wf[kk] = make_uint4(upper(a.x, b.x), upper(a.y, b.y), upper(a.z, b.z), upper(a.w, b.w));
      wf[kk + 1] = make_uint4(lower(b.x, a.x), lower(b.y, a.y), lower(b.z, a.z), lower(b.w, a.w));
    }
    if (kk < nkk) {
#pragma unroll
      for (int i = 0; i < kLinTok / 16; ++i) {
        if (i < ntile) {
          const uint4 xf = *reinterpret_cast<const uint4*>(xfrag + 16 * i * kLinPitch + 64 * kk);
          acc[i] = mfma_16x16x32<F16>(wf[kk], xf, acc[i]);
        }
      }
    }
  }
  // ---- acc[i][j] = y[token 16 i + m16][row n0 + 4 g + j] ----
#pragma unroll
  for (int i = 0; i < kLinTok / 16; ++i) {
    const int t = 16 * i + m16;
    if (i >= ntile || t >= nt) continue;
    const int n = n0 + 4 * g;
    if (p.S == 1) {
      float b[4] = {0.f, 0.f, 0.f, 0.f};
      if (p.bias) {
        const uint2 bw = ld8(p.bias + n);
        b[0] = lo_to_f32<F16>(bw.x); b[1] = hi_to_f32<F16>(bw.x); b[2] = lo_to_f32<F16>(bw.y); b[3] = hi_to_f32<F16>(bw.y);
      }
      st8(p.out + (int64_t)(t0 + t) * p.o_st + n,
          make_uint2(pack2<F16>(acc[i][0] + b[0], acc[i][1] + b[1]), pack2<F16>(acc[i][2] + b[2], acc[i][3] + b[3])));
    } else {
      // (lane (token, g) writes 16 bytes at token * 64 + 16 g of its wavefront's tile: whole lines, no gaps)
      float* dst = p.part + (((int64_t)blockIdx.y * (p.N >> 4) + (n0 >> 4)) * p.T + (t0 + t)) * 16 + 4 * g;
      *reinterpret_cast<float4*>(dst) = make_float4(acc[i][0], acc[i][1], acc[i][2], acc[i][3]);
    }
  }
}

// out[t][n .. n + 3] = round(sum over the slices, in their order, of the partial sums + bias[n ..]).  Threads walk the
// partial tiles in their memory order (tile, token, quarter of the 16 rows): neighbouring threads read neighbouring
// 16 bytes.
template <bool F16>
__global__ __launch_bounds__(256) void linear_decode_reduce_kernel(LinearParams p) {
  const int64_t q4 = (int64_t)blockIdx.x * 256 + threadIdx.x;   // group of four neighbouring outputs
  const int64_t per_slice = (int64_t)p.T * p.N;                 // floats per slice
  if (q4 * 4 >= per_slice) return;
  const int tile = (int)(q4 / (4 * p.T)), rest = (int)(q4 - (int64_t)tile * 4 * p.T);
  const int t = rest >> 2, n = 16 * tile + 4 * (rest & 3);
  float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
  const float* src = p.part + q4 * 4;
#pragma unroll 4
  for (int s = 0; s < p.S; ++s) {
    const float4 v = *reinterpret_cast<const float4*>(src + (int64_t)s * per_slice);
    sum.x += v.x; sum.y += v.y; sum.z += v.z; sum.w += v.w;
  }
  if (p.bias) {
    const uint2 bw = ld8(p.bias + n);
    sum.x += lo_to_f32<F16>(bw.x); sum.y += hi_to_f32<F16>(bw.x); sum.z += lo_to_f32<F16>(bw.y); sum.w += hi_to_f32<F16>(bw.y);
  }
  st8(p.out + (int64_t)t * p.o_st + n, make_uint2(pack2<F16>(sum.x, sum.y), pack2<F16>(sum.z, sum.w)));
}

}  // namespace mi

using namespace mi;

// Slices the K columns are cut into: enough workgroups to keep every CU streaming (about one and a half per CU),
// never more than 512 columns a slice (the staged x rows), slices a multiple of 32 columns.
static void linear_split(int T, int N, int K, int* n_slices, int* kslice) {
  const int row_blocks = (N + kLinRows - 1) / kLinRows, tok_blocks = (T + kLinTok - 1) / kLinTok;
  int s = (K + kLinSlice - 1) / kLinSlice;
  const int want = (384 + row_blocks * tok_blocks - 1) / (row_blocks * tok_blocks);
  if (want > s) s = want;
  if (s > K / 128) s = K / 128 > 0 ? K / 128 : 1;  // (a slice keeps at least 128 columns)
  int len = ((K + s - 1) / s + 31) & ~31;
  if (len > kLinSlice) len = kLinSlice;
  *kslice = len;
  *n_slices = (K + len - 1) / len;
}

extern "C" int64_t mi_linear_decode_workspace_bytes(int32_t T, int32_t N, int32_t K) {
  if (T <= 0 || N <= 0 || K <= 0) return 0;
  int s, len;
  linear_split(T, N, K, &s, &len);
  return s > 1 ? (int64_t)s * T * N * (int64_t)sizeof(float) : 0;
}

extern "C" int mi_linear_decode(const void* x, int64_t x_stride_tok, const void* weight, int64_t w_stride_row,
                                const void* bias, void* out, int64_t out_stride_tok, void* workspace,
                                int64_t workspace_bytes, int32_t T, int32_t N, int32_t K, int32_t dtype, void* stream) {
  if (T == 0) return MI_OK;
  if (dtype != MI_DTYPE_BF16 && dtype != MI_DTYPE_FP16)
    return mi_fail(MI_ERR_UNSUPPORTED, "mi_linear_decode: dtype must be MI_DTYPE_BF16 or MI_DTYPE_FP16");
  if (!x || !weight || !out) return mi_fail(MI_ERR_NULL, "mi_linear_decode: null pointer argument");
  if (T < 0 || T > 256) return mi_fail(MI_ERR_SHAPE, "mi_linear_decode: 1..256 tokens per call (decode-sized steps)");
  if (N <= 0 || K <= 0 || N % 16 || K % 32)
    return mi_fail(MI_ERR_SHAPE, "mi_linear_decode: N must be a multiple of 16 and K a multiple of 32");
  if (((uintptr_t)x | (uintptr_t)weight | (uintptr_t)out) & 15 || ((uintptr_t)bias & 7))
    return mi_fail(MI_ERR_ALIGN, "mi_linear_decode: x / weight / out must be 16-byte aligned, bias 8-byte aligned");
  if ((x_stride_tok | w_stride_row) % 8 || out_stride_tok % 4 || x_stride_tok < K || w_stride_row < K || out_stride_tok < N)
    return mi_fail(MI_ERR_ALIGN, "mi_linear_decode: strides must cover a row and keep rows 16-byte (out: 8-byte) aligned");
  LinearParams p;
  p.x = (const uint16_t*)x; p.x_st = x_stride_tok; p.w = (const uint16_t*)weight; p.w_st = w_stride_row;
  p.bias = (const uint16_t*)bias; p.out = (uint16_t*)out; p.o_st = out_stride_tok;
  p.T = T; p.N = N; p.K = K;
  p.part = nullptr;
  hipStream_t st = (hipStream_t)stream;
  linear_split(T, N, K, &p.S, &p.kslice);
  if (p.S > 1) {
    const int64_t need = (int64_t)p.S * T * N * (int64_t)sizeof(float);
    if (!workspace || workspace_bytes < need)
      return mi_fail(MI_ERR_WORKSPACE, "mi_linear_decode: workspace smaller than mi_linear_decode_workspace_bytes()");
    if ((uintptr_t)workspace & 15) return mi_fail(MI_ERR_ALIGN, "mi_linear_decode: the workspace must be 16-byte aligned");
    p.part = (float*)workspace;
  }
  const dim3 grid((N + kLinRows - 1) / kLinRows, p.S, (T + kLinTok - 1) / kLinTok);
  hipEvent_t ev_a, ev_b;
  const bool timed = mi_profile_next(&ev_a, &ev_b);
  if (timed) (void)hipEventRecord(ev_a, st);
  if (dtype == MI_DTYPE_FP16) hipLaunchKernelGGL(linear_decode_kernel<true>, grid, dim3(512), 0, st, p);
  else hipLaunchKernelGGL(linear_decode_kernel<false>, grid, dim3(512), 0, st, p);
  if (timed) (void)hipEventRecord(ev_b, st);
  if (p.S > 1) {
    const int64_t quads = (int64_t)T * (N / 4);
    const dim3 rgrid((unsigned)((quads + 255) / 256));
    if (dtype == MI_DTYPE_FP16) hipLaunchKernelGGL(linear_decode_reduce_kernel<true>, rgrid, dim3(256), 0, st, p);
    else hipLaunchKernelGGL(linear_decode_reduce_kernel<false>, rgrid, dim3(256), 0, st, p);
  }
  return mi_check_launch("mi_linear_decode");
}

extern "C" int mi_linear_qkv_decode_step(const void* hidden_states, int64_t x_stride_tok, const void* qkv_weight,
                                         int64_t w_stride_row, const void* qkv_bias, void* mixed_qkv,
                                         int64_t out_stride_tok, void* workspace, int64_t workspace_bytes, int32_t T,
                                         int32_t hidden_size, int32_t Hq, int32_t Hkv, int32_t head_dim, int32_t dtype,
                                         void* stream) {
  if (Hq <= 0 || Hkv <= 0 || head_dim <= 0 || Hq % Hkv)
    return mi_fail(MI_ERR_SHAPE, "mi_linear_qkv_decode_step: need Hq a positive multiple of Hkv");
  return mi_linear_decode(hidden_states, x_stride_tok, qkv_weight, w_stride_row, qkv_bias, mixed_qkv, out_stride_tok,
                          workspace, workspace_bytes, T, (Hq + 2 * Hkv) * head_dim, hidden_size, dtype, stream);
}

extern "C" int mi_attention_out_linear_proj(const void* core_attn_out, int64_t x_stride_tok, const void* proj_weight,
                                            int64_t w_stride_row, void* output, int64_t out_stride_tok, void* workspace,
                                            int64_t workspace_bytes, int32_t T, int32_t hidden_size, int32_t Hq,
                                            int32_t head_dim, int32_t dtype, void* stream) {
  if (Hq <= 0 || head_dim <= 0) return mi_fail(MI_ERR_SHAPE, "mi_attention_out_linear_proj: need Hq, head_dim > 0");
  return mi_linear_decode(core_attn_out, x_stride_tok, proj_weight, w_stride_row, nullptr, output, out_stride_tok,
                          workspace, workspace_bytes, T, hidden_size, Hq * head_dim, dtype, stream);
}
