// update_requests of the dynamic inference context as ONE kernel.
//
// The reference advances its bookkeeping after every sampled token with ~40 small torch
// kernels and 4-5 device-to-host synchronisations
// (megatron/core/inference/contexts/dynamic_context.py:1033-1298, helper :1017-1030,
// allocator megatron/core/inference/contexts/dynamic_chunk_allocator.py:56-86).  This kernel
// performs the same sequence -- count, release the chunks of finished requests, compact the
// rows into [paused | active | finished], pause requests whose last chunk is full, resume as
// many paused requests as free chunks allow (LIFO), advance lengths / offsets and rewrite the
// per-token rows of the next decode step -- on the device, in the same order, so that every
// tensor the reference exposes ends up with the same contents.  The host reads back one small
// array of counters (a single synchronisation) to refresh its Python integers.
//
// One workgroup of 1024 threads; rows are distributed over the threads and ordered lists
// (holes, movers, ...) are built with a block-wide prefix sum, so the order of every move and
// of every chunk id pushed to / popped from the free stack is the reference's.
#include "mi_common.h"
#include "mi_capi_internal.h"

namespace mi {

struct UpdateParams {
  int32_t* ids; int32_t* q_len; int32_t* out_len; int32_t* kv_off; int32_t* n_chunks;
  int32_t* last_chunk; int32_t* last_off;
  int32_t* table; int64_t table_stride; int32_t M;
  int64_t* tok_input; int64_t* tok_pos; int64_t* tok_req; int64_t* tok_in_req; int64_t* tok_chunk; int64_t* tok_local;
  int32_t* bag;
  const int32_t* mask; const int64_t* new_tokens;
  int64_t* paused_tokens;    // in: tokens of the paused rows; out: tokens of the rows paused afterwards
  int64_t* next_tokens;      // scratch [max_requests]
  int32_t* scratch;          // scratch [4 * max_requests]
  int32_t* newly_paused;     // out [max_requests]
  int32_t* finished;         // out [max_requests]: ids of the requests that finished, in row order
  int32_t* counters;         // out [8]
  int32_t total, paused, avail, gtd_chunks, gtd_requests, chunk, max_requests;
};

constexpr int kThreads = 1024;
constexpr int kWaves = kThreads / 64;

// Inclusive block-wide prefix sum of one value per thread (thread order); *total receives the sum over the block.
// Within a wavefront by lane shuffles, across wavefronts through `sh` (at least kWaves ints).  All threads call.
static __device__ int block_scan(int v, int* sh, int* total) {
  const int t = threadIdx.x, lane = t & 63, w = t >> 6;
  int x = v;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int y = __shfl_up(x, o, 64);
    if (lane >= o) x += y;
  }
  __syncthreads();  // (an earlier call's readers are done with sh)
  if (lane == 63) sh[w] = x;
  __syncthreads();
  int before = 0, all = 0;
#pragma unroll
  for (int i = 0; i < kWaves; ++i) {
    const int s = sh[i];
    before += i < w ? s : 0;
    all += s;
  }
  *total = all;
  return x + before;
}

// Ordered compaction: out[k] = base + i for the k-th i in [0, n) with pred(i); returns the count.
// Must be called by all threads of the block.
template <typename Pred>
static __device__ int compact(int n, int base, int32_t* out, Pred pred, int* sh) {
  const int t = threadIdx.x;
  const int seg = (n + kThreads - 1) / kThreads;
  const int a = min(t * seg, n), b = min(a + seg, n);
  int cnt = 0;
  for (int i = a; i < b; ++i) cnt += pred(i) ? 1 : 0;
  int total;
  int at = block_scan(cnt, sh, &total) - cnt;
  for (int i = a; i < b; ++i)
    if (pred(i)) out[at++] = base + i;
  __syncthreads();
  return total;
}

struct Row { int32_t kv_off, q_len, out_len, id, n_chunks, last_chunk, last_off; int64_t tok; };

static __device__ __forceinline__ Row load_row(const UpdateParams& p, int i) {
  return Row{p.kv_off[i], p.q_len[i], p.out_len[i], p.ids[i], p.n_chunks[i], p.last_chunk[i], p.last_off[i],
             p.next_tokens[i]};
}
static __device__ __forceinline__ void store_row(const UpdateParams& p, int i, const Row& r) {
  p.kv_off[i] = r.kv_off; p.q_len[i] = r.q_len; p.out_len[i] = r.out_len; p.ids[i] = r.id;
  p.n_chunks[i] = r.n_chunks; p.last_chunk[i] = r.last_chunk; p.last_off[i] = r.last_off;
  p.next_tokens[i] = r.tok;
}

// Push the chunk ids owned by the listed rows (ascending list order, ascending column) onto the stack.
// One wavefront per row at a time, its lanes over the columns: the row's ids keep their column order through a
// ballot and a count of the lower lanes.
static __device__ int release_rows(const UpdateParams& p, const int32_t* rows, int n_rows, int avail,
                                   int32_t* counts, int* sh) {
  const int t = threadIdx.x, lane = t & 63, w = t >> 6;
  for (int k = w; k < n_rows; k += kWaves) {
    const int32_t* row = p.table + (int64_t)rows[k] * p.table_stride;
    int c = 0;
    for (int j0 = 0; j0 < p.M; j0 += 64) {
      const int j = j0 + lane;
      c += __popcll(__ballot(j < p.M && row[j] != -1));
    }
    if (lane == 0) counts[k] = c;
  }
  __syncthreads();
  // counts -> where each row's ids start (exclusive prefix sum, in place)
  const int seg = (n_rows + kThreads - 1) / kThreads;
  const int a = min(t * seg, n_rows), b = min(a + seg, n_rows);
  int cnt = 0;
  for (int k = a; k < b; ++k) cnt += counts[k];
  int total;
  int at = block_scan(cnt, sh, &total) - cnt;
  for (int k = a; k < b; ++k) {
    const int c = counts[k];
    counts[k] = at;
    at += c;
  }
  __syncthreads();
  for (int k = w; k < n_rows; k += kWaves) {
    const int32_t* row = p.table + (int64_t)rows[k] * p.table_stride;
    int start = avail + counts[k];
    for (int j0 = 0; j0 < p.M; j0 += 64) {
      const int j = j0 + lane;
      const int32_t v = j < p.M ? row[j] : -1;
      const unsigned long long keep = __ballot(v != -1);
      if (v != -1) p.bag[start + __popcll(keep & ((1ull << lane) - 1))] = v;
      start += __popcll(keep);
    }
  }
  __syncthreads();
  return avail + total;
}

__global__ __launch_bounds__(kThreads) void update_requests_kernel(UpdateParams p) {
  __shared__ int sh[kWaves];
  __shared__ int red[2];
  const int t = threadIdx.x;
  const int P0 = p.paused;
  const int n = p.total - P0;  // rows covered by the mask
  int32_t* list_a = p.scratch;                       // [max_requests]
  int32_t* list_b = p.scratch + p.max_requests;      // [max_requests]
  int32_t* counts = p.scratch + 2 * p.max_requests;  // [max_requests]

  // ---- 1. how many requests continue / finished ---------------------------------------
  if (t < 2) red[t] = 0;
  __syncthreads();
  int c1 = 0, c0 = 0;
  for (int i = t; i < n; i += kThreads) {
    c1 += p.mask[i] == 1;
    c0 += p.mask[i] == 0;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    c1 += __shfl_xor(c1, o, 64);
    c0 += __shfl_xor(c0, o, 64);
  }
  if ((t & 63) == 0) {
    atomicAdd(&red[0], c1);
    atomicAdd(&red[1], c0);
  }
  __syncthreads();
  int n_cont = red[0];
  const int n_fin = red[1];
  int avail = p.avail;
  int paused = P0;
  if (n_cont + n_fin + P0 != p.total || n < 0) {
    if (t == 0) { p.counters[5] = 1; }
    return;
  }

  // ---- 2. nothing left: give everything back --------------------------------------------
  if (n_cont + P0 == 0) {
    if (n_fin > 0) {
      const int nf = compact(n, P0, list_a, [&](int i) { return p.mask[i] == 0; }, sh);
      for (int k = t; k < nf; k += kThreads) p.finished[k] = p.ids[list_a[k]];
      avail = release_rows(p, list_a, nf, avail, counts, sh);
    }
    for (int64_t i = t; i < (int64_t)p.max_requests * p.M; i += kThreads)
      p.table[(i / p.M) * p.table_stride + (i % p.M)] = -1;
    if (t == 0) {
      p.counters[0] = 0; p.counters[1] = P0; p.counters[2] = 0; p.counters[3] = avail;
      p.counters[4] = -1; p.counters[5] = 0; p.counters[6] = 1; p.counters[7] = n_fin;
    }
    return;
  }

  // ---- 3. tokens of paused + active rows, in row order -----------------------------------
  for (int i = t; i < p.total; i += kThreads)
    p.next_tokens[i] = i < P0 ? p.paused_tokens[i] : p.new_tokens[i - P0];
  __syncthreads();

  // ---- 4. finished requests: release chunks, fill their holes from the right ---------------
  if (n_fin > 0) {
    const int nf = compact(n, P0, list_a, [&](int i) { return p.mask[i] == 0; }, sh);
    // their ids, in row order (what the caller of the step reports as finished), before any row moves
    for (int k = t; k < nf; k += kThreads) p.finished[k] = p.ids[list_a[k]];
    avail = release_rows(p, list_a, nf, avail, counts, sh);
    for (int64_t i = t; i < (int64_t)nf * p.M; i += kThreads)
      p.table[(int64_t)list_a[i / p.M] * p.table_stride + (i % p.M)] = -1;
    __syncthreads();
    if (n_cont > 0) {
      const int nh = compact(n_cont, P0, list_a, [&](int i) { return p.mask[i] == 0; }, sh);
      compact(n - n_cont, P0 + n_cont, list_b, [&](int i) { return p.mask[n_cont + i] != 0; }, sh);
      for (int k = t; k < nh; k += kThreads) store_row(p, list_a[k], load_row(p, list_b[k]));
      for (int64_t i = t; i < (int64_t)nh * p.M; i += kThreads) {
        const int k = (int)(i / p.M), j = (int)(i % p.M);
        int32_t* src = p.table + (int64_t)list_b[k] * p.table_stride + j;
        p.table[(int64_t)list_a[k] * p.table_stride + j] = *src;
        *src = -1;
      }
      __syncthreads();
    }
  }

  // ---- 5. requests whose last chunk is full pause: swap them to the left -------------------
  int n_newly = -1;
  if (n_cont > 0) {
    const int C1 = p.chunk - 1;
    const int n_need = compact(n_cont, P0, list_a, [&](int i) { return p.last_off[P0 + i] == C1; }, sh);
    if (n_need > 0 && n_need != n_cont) {
      const int nl = compact(n_need, P0, list_a, [&](int i) { return p.last_off[P0 + i] != C1; }, sh);
      compact(n_cont - n_need, P0 + n_need, list_b, [&](int i) { return p.last_off[P0 + n_need + i] == C1; }, sh);
      for (int k = t; k < nl; k += kThreads) {
        const Row l = load_row(p, list_a[k]), r = load_row(p, list_b[k]);
        store_row(p, list_a[k], r);
        store_row(p, list_b[k], l);
      }
      for (int64_t i = t; i < (int64_t)nl * p.M; i += kThreads) {
        const int k = (int)(i / p.M), j = (int)(i % p.M);
        int32_t* a = p.table + (int64_t)list_a[k] * p.table_stride + j;
        int32_t* b = p.table + (int64_t)list_b[k] * p.table_stride + j;
        const int32_t va = *a, vb = *b;
        *a = vb;
        *b = va;
      }
      __syncthreads();
      // ids at [left positions..., right positions...] after the swap
      for (int k = t; k < nl; k += kThreads) {
        p.newly_paused[k] = p.ids[list_a[k]];
        p.newly_paused[nl + k] = p.ids[list_b[k]];
      }
      n_newly = 2 * nl;
      __syncthreads();
    }
    paused += n_need;
    n_cont -= n_need;
  }

  // ---- 6. how many paused requests get a chunk now ------------------------------------------
  const int spare = max(0, avail - p.gtd_chunks);
  const int n_resume = spare ? min(spare, paused) : min(max(p.gtd_requests - n_cont, 0), paused);
  paused -= n_resume;
  n_cont += n_resume;
  if (n_cont <= 0) {
    if (t == 0) { p.counters[5] = 2; p.counters[7] = n_fin; }
    return;
  }
  if (n_newly >= 0 && n_resume > 0) n_newly = max(0, n_newly - n_resume);

  // ---- 7. next step: one token per active request ---------------------------------------------
  const int total = n_cont + paused;
  for (int i = t; i < paused; i += kThreads) p.paused_tokens[i] = p.next_tokens[i];
  int bad = 0;
  for (int i = t; i < n_cont; i += kThreads) {
    const int r = paused + i;
    p.tok_input[i] = p.next_tokens[r];
    const int off = p.kv_off[r] + p.q_len[r];
    p.kv_off[r] = off;
    p.q_len[r] = 1;
    p.tok_pos[i] = off;
    int lo = (p.last_off[r] + 1) % p.chunk;
    p.last_off[r] = lo;
    // ---- 8. resumed rows take a fresh chunk from the top of the stack --------------------------
    if (i < n_resume) {
      bad |= lo != 0;
      const int32_t c = p.bag[avail - n_resume + i];
      if (p.n_chunks[r] < p.M) p.table[(int64_t)r * p.table_stride + p.n_chunks[r]] = c;
      p.n_chunks[r] += 1;
      p.last_chunk[r] = c;
    }
    // ---- 9. per-token rows ------------------------------------------------------------------------
    p.tok_req[i] = r;
    p.tok_in_req[i] = off;
    p.tok_chunk[i] = p.last_chunk[r];
    p.tok_local[i] = lo;
  }
  if (bad) atomicOr(&red[0], 1 << 30);
  __syncthreads();
  avail -= n_resume;
  if (t == 0) {
    p.counters[0] = total; p.counters[1] = paused; p.counters[2] = n_cont; p.counters[3] = avail;
    p.counters[4] = n_newly; p.counters[5] = (red[0] >> 30) ? 3 : 0; p.counters[6] = 0; p.counters[7] = n_fin;
  }
}

struct DecodeStateParams {
  const int32_t* kv_off; const int32_t* q_len; const int32_t* table; int64_t table_stride; int32_t M;
  int32_t* q_lens_out; int32_t* kv_lens_out; int32_t* table_out; int64_t table_out_stride;
  int64_t* tok_chunk; int64_t* tok_local; int64_t* tok_in_req;
  int32_t paused, n_active, padded, active_tokens, dummy_chunk;
};

// Decode-only initialize_attention_state: fixed-address mirrors of query / kv lengths and of the
// block table for the active rows, plus the padded token rows (dummy chunk, position 0).
__global__ __launch_bounds__(256) void decode_attention_state_kernel(DecodeStateParams p) {
  const int i = blockIdx.x;  // active row
  if (i < p.n_active) {
    const int r = p.paused + i;
    if (threadIdx.x == 0) {
      p.q_lens_out[i] = p.q_len[r];
      p.kv_lens_out[i] = p.kv_off[r] + p.q_len[r];
    }
    for (int j = threadIdx.x; j < p.M; j += 256)
      p.table_out[(int64_t)i * p.table_out_stride + j] = p.table[(int64_t)r * p.table_stride + j];
  }
  if (blockIdx.x == 0) {
    for (int tk = p.active_tokens + threadIdx.x; tk < p.padded; tk += 256) {
      p.tok_chunk[tk] = p.dummy_chunk;
      p.tok_local[tk] = 0;
      p.tok_in_req[tk] = 0;
    }
  }
}


struct StepStateParams {
  const int32_t* kv_off; const int32_t* q_len; const int32_t* table; int64_t table_stride; int32_t M;
  int32_t* q_lens_out; int32_t* kv_lens_out; int32_t* cu_q_out; int32_t* cu_kv_out;
  int32_t* table_out; int64_t table_out_stride;
  int64_t* tok_chunk; int64_t* tok_local; int64_t* tok_in_req;
  int32_t* maxes;  // out [2]: largest query length, largest kv length
  int32_t paused, n_active, R, padded, active_tokens, dummy_chunk;
};

// initialize_attention_state of a prefill / mixed step: what decode_attention_state_kernel does, plus the
// running sums of query and kv lengths over the R (padded) requests and the two maxima.
// Workgroup 0 (1024 threads) owns the length rows: a block-wide scan over R entries; the other
// workgroups copy the block-table rows of the active requests.
__global__ __launch_bounds__(1024) void step_attention_state_kernel(StepStateParams p) {
  const int t = threadIdx.x;
  if (blockIdx.x > 0) {
    const int64_t n = (int64_t)p.n_active * p.M, step = (int64_t)(gridDim.x - 1) * 1024;
    for (int64_t e = (int64_t)(blockIdx.x - 1) * 1024 + t; e < n; e += step) {
      const int i = (int)(e / p.M), j = (int)(e - (int64_t)i * p.M);
      p.table_out[(int64_t)i * p.table_out_stride + j] = p.table[(int64_t)(p.paused + i) * p.table_stride + j];
    }
    return;
  }
  static_assert(kThreads == 1024, "block_scan covers the workgroup of this kernel");
  __shared__ int sh_q[kWaves], sh_k[kWaves];
  __shared__ int red[2];
  if (t < 2) red[t] = 0;
  const int seg = (p.R + 1023) / 1024;
  const int a = min(t * seg, p.R), b = min(a + seg, p.R);
  int sq = 0, sk = 0, mq = 0, mk = 0;
  for (int i = a; i < b; ++i) {
    const int q = i < p.n_active ? p.q_len[p.paused + i] : 0;
    const int k = i < p.n_active ? p.kv_off[p.paused + i] + q : 0;
    if (i < p.n_active) {
      p.q_lens_out[i] = q;
      p.kv_lens_out[i] = k;
    }
    sq += q; sk += k;
    mq = max(mq, q); mk = max(mk, k);
  }
  int all_q, all_k;
  int cq = block_scan(sq, sh_q, &all_q) - sq, ck = block_scan(sk, sh_k, &all_k) - sk;  // sums before this thread's rows
  if (t == 0) { p.cu_q_out[0] = 0; p.cu_kv_out[0] = 0; }
  if (seg == 1) {  // (one row per thread: its lengths are still in sq / sk)
    if (a < b) {
      p.cu_q_out[a + 1] = cq + sq;
      p.cu_kv_out[a + 1] = ck + sk;
    }
  } else {
    for (int i = a; i < b; ++i) {
      const int q = i < p.n_active ? p.q_len[p.paused + i] : 0;
      const int k = i < p.n_active ? p.kv_off[p.paused + i] + q : 0;
      cq += q; ck += k;
      p.cu_q_out[i + 1] = cq;
      p.cu_kv_out[i + 1] = ck;
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {  // one LDS atomic per wavefront instead of one per thread
    mq = max(mq, __shfl_xor(mq, o, 64));
    mk = max(mk, __shfl_xor(mk, o, 64));
  }
  if ((t & 63) == 0) {
    atomicMax(&red[0], mq);
    atomicMax(&red[1], mk);
  }
  for (int tk = p.active_tokens + t; tk < p.padded; tk += 1024) {
    p.tok_chunk[tk] = p.dummy_chunk;
    p.tok_local[tk] = 0;
    p.tok_in_req[tk] = 0;
  }
  __syncthreads();
  if (t < 2) p.maxes[t] = red[t];
}

}  // namespace mi

using namespace mi;

extern "C" int mi_update_requests(
    int32_t* request_ids, int32_t* request_query_lengths, int32_t* request_output_lengths,
    int32_t* request_kv_length_offsets, int32_t* request_kv_chunk_counts, int32_t* request_last_kv_chunk_id,
    int32_t* request_last_kv_chunk_offset, int32_t* request_to_kv_chunk_ids, int64_t table_stride,
    int32_t max_kv_chunk_count, int64_t* token_to_input_ids, int64_t* token_to_pos_ids,
    int64_t* token_to_request_idx, int64_t* token_to_position_in_request, int64_t* token_to_chunk_idx,
    int64_t* token_to_local_position_within_kv_chunk, int32_t* chunk_bag, const int32_t* active_requests_mask,
    const int64_t* new_tokens, int64_t* paused_tokens, int64_t* next_tokens_scratch, int32_t* scratch,
    int32_t* newly_paused_request_ids, int32_t* finished_request_ids, int32_t* counters, int32_t total_request_count,
    int32_t paused_request_count, int32_t chunk_count_avail, int32_t gtd_chunk_count,
    int32_t gtd_request_count, int32_t chunk_size_tokens, int32_t max_requests, void* stream) {
  if (!request_ids || !request_query_lengths || !request_output_lengths || !request_kv_length_offsets ||
      !request_kv_chunk_counts || !request_last_kv_chunk_id || !request_last_kv_chunk_offset ||
      !request_to_kv_chunk_ids || !token_to_input_ids || !token_to_pos_ids || !token_to_request_idx ||
      !token_to_position_in_request || !token_to_chunk_idx || !token_to_local_position_within_kv_chunk ||
      !chunk_bag || !active_requests_mask || !new_tokens || !paused_tokens || !next_tokens_scratch || !scratch ||
      !newly_paused_request_ids || !finished_request_ids || !counters)
    return mi_fail(MI_ERR_NULL, "mi_update_requests: null pointer argument");
  if (total_request_count < 0 || paused_request_count < 0 || paused_request_count > total_request_count ||
      total_request_count > max_requests || max_kv_chunk_count <= 0 || chunk_size_tokens <= 0)
    return mi_fail(MI_ERR_SHAPE, "mi_update_requests: inconsistent counts");
  UpdateParams p;
  p.ids = request_ids; p.q_len = request_query_lengths; p.out_len = request_output_lengths;
  p.kv_off = request_kv_length_offsets; p.n_chunks = request_kv_chunk_counts;
  p.last_chunk = request_last_kv_chunk_id; p.last_off = request_last_kv_chunk_offset;
  p.table = request_to_kv_chunk_ids; p.table_stride = table_stride; p.M = max_kv_chunk_count;
  p.tok_input = token_to_input_ids; p.tok_pos = token_to_pos_ids; p.tok_req = token_to_request_idx;
  p.tok_in_req = token_to_position_in_request; p.tok_chunk = token_to_chunk_idx;
  p.tok_local = token_to_local_position_within_kv_chunk;
  p.bag = chunk_bag; p.mask = active_requests_mask; p.new_tokens = new_tokens;
  p.paused_tokens = paused_tokens; p.next_tokens = next_tokens_scratch; p.scratch = scratch;
  p.newly_paused = newly_paused_request_ids; p.finished = finished_request_ids; p.counters = counters;
  p.total = total_request_count; p.paused = paused_request_count; p.avail = chunk_count_avail;
  p.gtd_chunks = gtd_chunk_count; p.gtd_requests = gtd_request_count; p.chunk = chunk_size_tokens;
  p.max_requests = max_requests;
  hipLaunchKernelGGL(update_requests_kernel, dim3(1), dim3(kThreads), 0, (hipStream_t)stream, p);
  return mi_check_launch("mi_update_requests");
}

extern "C" int mi_decode_attention_state(
    const int32_t* request_kv_length_offsets, const int32_t* request_query_lengths,
    const int32_t* request_to_kv_chunk_ids, int64_t table_stride, int32_t max_kv_chunk_count,
    int32_t* query_seq_lengths_out, int32_t* kv_seq_lengths_out, int32_t* block_table_out,
    int64_t block_table_out_stride, int64_t* token_to_chunk_idx,
    int64_t* token_to_local_position_within_kv_chunk, int64_t* token_to_position_in_request,
    int32_t paused_request_count, int32_t active_request_count, int32_t active_token_count,
    int32_t padded_active_token_count, int32_t dummy_chunk_idx, void* stream) {
  if (!request_kv_length_offsets || !request_query_lengths || !request_to_kv_chunk_ids || !query_seq_lengths_out ||
      !kv_seq_lengths_out || !block_table_out || !token_to_chunk_idx || !token_to_local_position_within_kv_chunk ||
      !token_to_position_in_request)
    return mi_fail(MI_ERR_NULL, "mi_decode_attention_state: null pointer argument");
  if (paused_request_count < 0 || active_request_count < 0 || active_token_count < 0 ||
      padded_active_token_count < active_token_count || max_kv_chunk_count <= 0)
    return mi_fail(MI_ERR_SHAPE, "mi_decode_attention_state: inconsistent counts");
  DecodeStateParams p;
  p.kv_off = request_kv_length_offsets; p.q_len = request_query_lengths; p.table = request_to_kv_chunk_ids;
  p.table_stride = table_stride; p.M = max_kv_chunk_count;
  p.q_lens_out = query_seq_lengths_out; p.kv_lens_out = kv_seq_lengths_out; p.table_out = block_table_out;
  p.table_out_stride = block_table_out_stride;
  p.tok_chunk = token_to_chunk_idx; p.tok_local = token_to_local_position_within_kv_chunk;
  p.tok_in_req = token_to_position_in_request;
  p.paused = paused_request_count; p.n_active = active_request_count; p.padded = padded_active_token_count;
  p.active_tokens = active_token_count; p.dummy_chunk = dummy_chunk_idx;
  const int blocks = active_request_count > 0 ? active_request_count : 1;
  hipLaunchKernelGGL(decode_attention_state_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, p);
  return mi_check_launch("mi_decode_attention_state");
}

extern "C" int mi_step_attention_state(
    const int32_t* request_kv_length_offsets, const int32_t* request_query_lengths,
    const int32_t* request_to_kv_chunk_ids, int64_t table_stride, int32_t max_kv_chunk_count,
    int32_t* query_seq_lengths_out, int32_t* kv_seq_lengths_out, int32_t* cu_query_seq_lengths_out,
    int32_t* cu_kv_seq_lengths_out, int32_t* block_table_out, int64_t block_table_out_stride,
    int64_t* token_to_chunk_idx, int64_t* token_to_local_position_within_kv_chunk,
    int64_t* token_to_position_in_request, int32_t* max_lengths_out, int32_t paused_request_count,
    int32_t active_request_count, int32_t padded_request_count, int32_t active_token_count,
    int32_t padded_active_token_count, int32_t dummy_chunk_idx, void* stream) {
  if (!request_kv_length_offsets || !request_query_lengths || !request_to_kv_chunk_ids || !query_seq_lengths_out ||
      !kv_seq_lengths_out || !cu_query_seq_lengths_out || !cu_kv_seq_lengths_out || !block_table_out ||
      !token_to_chunk_idx || !token_to_local_position_within_kv_chunk || !token_to_position_in_request ||
      !max_lengths_out)
    return mi_fail(MI_ERR_NULL, "mi_step_attention_state: null pointer argument");
  if (paused_request_count < 0 || active_request_count < 0 || padded_request_count < active_request_count ||
      active_token_count < 0 || padded_active_token_count < active_token_count || max_kv_chunk_count <= 0)
    return mi_fail(MI_ERR_SHAPE, "mi_step_attention_state: inconsistent counts");
  StepStateParams p;
  p.kv_off = request_kv_length_offsets; p.q_len = request_query_lengths; p.table = request_to_kv_chunk_ids;
  p.table_stride = table_stride; p.M = max_kv_chunk_count;
  p.q_lens_out = query_seq_lengths_out; p.kv_lens_out = kv_seq_lengths_out;
  p.cu_q_out = cu_query_seq_lengths_out; p.cu_kv_out = cu_kv_seq_lengths_out;
  p.table_out = block_table_out; p.table_out_stride = block_table_out_stride;
  p.tok_chunk = token_to_chunk_idx; p.tok_local = token_to_local_position_within_kv_chunk;
  p.tok_in_req = token_to_position_in_request; p.maxes = max_lengths_out;
  p.paused = paused_request_count; p.n_active = active_request_count; p.R = padded_request_count;
  p.padded = padded_active_token_count; p.active_tokens = active_token_count; p.dummy_chunk = dummy_chunk_idx;
  // enough copy workgroups that a thread moves one or two table entries (every load in flight at once)
  int64_t copy_blocks = ((int64_t)active_request_count * max_kv_chunk_count + 1023) / 1024;
  if (copy_blocks > 512) copy_blocks = 512;
  hipLaunchKernelGGL(step_attention_state_kernel, dim3(1 + (int)copy_blocks), dim3(1024), 0, (hipStream_t)stream, p);
  return mi_check_launch("mi_step_attention_state");
}


// ---------------------------------------------------------------------------------------------
// DynamicInferenceContext.add_request (dynamic_context.py:920-1015) after its host-side checks: the
// request row, its chunk-table row (the ids popped from the top of the chunk stack, in stack order) and the
// per-token rows of the prompt, in one launch instead of about fourteen indexed writes.
// ---------------------------------------------------------------------------------------------
namespace mi {
struct AddRequestParams {
  int32_t* request_ids; int32_t* q_len; int32_t* out_len; int32_t* kv_off; int32_t* chunk_counts;
  int32_t* last_chunk_id; int32_t* last_chunk_off; int32_t* table; int64_t table_stride;
  int64_t* tok_input; int64_t* tok_pos; int64_t* tok_req; int64_t* tok_in_req; int64_t* tok_chunk; int64_t* tok_local;
  const int32_t* chunk_bag;
  const int64_t* tokens;
  int32_t row, token_begin, length, n_chunks, stack_first, chunk, request_id, output_length;
};

__global__ __launch_bounds__(256) void add_request_kernel(AddRequestParams p) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i == 0) {
    p.request_ids[p.row] = p.request_id;
    p.q_len[p.row] = p.length;
    p.out_len[p.row] = p.output_length;
    p.kv_off[p.row] = 0;
    p.chunk_counts[p.row] = p.n_chunks;
    p.last_chunk_id[p.row] = p.chunk_bag[p.stack_first + p.n_chunks - 1];
    p.last_chunk_off[p.row] = (p.length - 1) % p.chunk;
  }
  if (i < p.n_chunks) p.table[(int64_t)p.row * p.table_stride + i] = p.chunk_bag[p.stack_first + i];
  if (i < p.length) {
    const int64_t t = (int64_t)p.token_begin + i;
    const int ci = i / p.chunk;
    p.tok_input[t] = p.tokens[i];
    p.tok_pos[t] = i;
    p.tok_req[t] = p.row;
    p.tok_in_req[t] = i;
    p.tok_chunk[t] = p.chunk_bag[p.stack_first + ci];
    p.tok_local[t] = i - ci * p.chunk;
  }
}
}  // namespace mi

extern "C" int mi_add_request(
    int32_t* request_ids, int32_t* request_query_lengths, int32_t* request_output_lengths,
    int32_t* request_kv_length_offsets, int32_t* request_kv_chunk_counts, int32_t* request_last_kv_chunk_id,
    int32_t* request_last_kv_chunk_offset, int32_t* request_to_kv_chunk_ids, int64_t table_stride,
    int64_t* token_to_input_ids, int64_t* token_to_pos_ids, int64_t* token_to_request_idx,
    int64_t* token_to_position_in_request, int64_t* token_to_chunk_idx,
    int64_t* token_to_local_position_within_kv_chunk, const int32_t* chunk_bag, const int64_t* prompt_tokens,
    int32_t request_row, int32_t token_begin, int32_t prompt_length, int32_t chunk_count, int32_t stack_first,
    int32_t chunk_size_tokens, int32_t request_id, int32_t output_length, void* stream) {
  if (!request_ids || !request_query_lengths || !request_output_lengths || !request_kv_length_offsets ||
      !request_kv_chunk_counts || !request_last_kv_chunk_id || !request_last_kv_chunk_offset ||
      !request_to_kv_chunk_ids || !token_to_input_ids || !token_to_pos_ids || !token_to_request_idx ||
      !token_to_position_in_request || !token_to_chunk_idx || !token_to_local_position_within_kv_chunk || !chunk_bag ||
      !prompt_tokens)
    return mi_fail(MI_ERR_NULL, "mi_add_request: null pointer argument");
  if (request_row < 0 || token_begin < 0 || prompt_length <= 0 || chunk_size_tokens <= 0 || stack_first < 0 ||
      chunk_count != (prompt_length + chunk_size_tokens - 1) / chunk_size_tokens || chunk_count > table_stride)
    return mi_fail(MI_ERR_SHAPE, "mi_add_request: inconsistent counts (chunk_count must be ceil(prompt_length / chunk_size_tokens))");
  mi::AddRequestParams p;
  p.request_ids = request_ids; p.q_len = request_query_lengths; p.out_len = request_output_lengths;
  p.kv_off = request_kv_length_offsets; p.chunk_counts = request_kv_chunk_counts;
  p.last_chunk_id = request_last_kv_chunk_id; p.last_chunk_off = request_last_kv_chunk_offset;
  p.table = request_to_kv_chunk_ids; p.table_stride = table_stride;
  p.tok_input = token_to_input_ids; p.tok_pos = token_to_pos_ids; p.tok_req = token_to_request_idx;
  p.tok_in_req = token_to_position_in_request; p.tok_chunk = token_to_chunk_idx;
  p.tok_local = token_to_local_position_within_kv_chunk;
  p.chunk_bag = chunk_bag; p.tokens = prompt_tokens;
  p.row = request_row; p.token_begin = token_begin; p.length = prompt_length; p.n_chunks = chunk_count;
  p.stack_first = stack_first; p.chunk = chunk_size_tokens; p.request_id = request_id; p.output_length = output_length;
  hipLaunchKernelGGL(mi::add_request_kernel, dim3((prompt_length + 255) / 256), dim3(256), 0, (hipStream_t)stream, p);
  return mi_check_launch("mi_add_request");
}
