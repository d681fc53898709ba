// Token choice from float32 logits: argmax for greedy rows; temperature, top-k, top-p and one
// categorical draw for the others. One workgroup per row, so a row's result depends on nothing but
// its own logits, parameters, seed and draw counter.
//
// The pipeline is the reference's (src/dli/sampling.py:83-117) without the sort:
//   x = logits / temperature
//   top-k: keep x >= (k-th largest value)            [tokens tied with the k-th are all kept]
//   p = softmax over the kept
//   top-p: drop a token iff the mass of strictly more likely tokens reaches top_p
//   draw one token from the renormalised rest with u = Philox4x32-10(seed, counter) in [0, 1),
//   by inverse CDF in vocabulary order.
// Thresholds are found by bitwise search over an order-preserving 32-bit key of the value, each
// probe one reduction over the row; every reduction adds in a fixed order, so the same inputs
// always give the same token.
#include "common.h"

#define SAMPLE_THREADS 1024

__device__ __forceinline__ uint32_t order_key(float x) {  // larger float <=> larger key
  const uint32_t u = __float_as_uint(x);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ uint32_t mulhi32(uint32_t a, uint32_t b) { return __umulhi(a, b); }

// Philox4x32 with 10 rounds; returns the first output word.
__device__ uint32_t philox_first_word(uint64_t seed, uint64_t counter) {
  uint32_t c0 = (uint32_t)counter, c1 = (uint32_t)(counter >> 32), c2 = 0u, c3 = 0u;
  uint32_t k0 = (uint32_t)seed, k1 = (uint32_t)(seed >> 32);
  for (int r = 0; r < 10; ++r) {
    const uint32_t hi0 = mulhi32(0xD2511F53u, c0), lo0 = 0xD2511F53u * c0;
    const uint32_t hi1 = mulhi32(0xCD9E8D57u, c2), lo1 = 0xCD9E8D57u * c2;
    const uint32_t n0 = hi1 ^ c1 ^ k0, n1 = lo1, n2 = hi0 ^ c3 ^ k1, n3 = lo0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  return c0;
}

struct ArgBest {
  float v;
  int i;
};

__device__ __forceinline__ ArgBest better(ArgBest a, ArgBest b) {
  if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
  return a;
}

__device__ float block_sum_f(float v, float* scratch) { return block_sum(v, scratch); }

__device__ int block_sum_i(int v, int* scratch) {
  const int lane = threadIdx.x % DLI_WAVE, wave = threadIdx.x / DLI_WAVE;
  const int nwaves = (blockDim.x + DLI_WAVE - 1) / DLI_WAVE;
#pragma unroll
  for (int m = DLI_WAVE / 2; m > 0; m >>= 1) v += __shfl_xor(v, m, DLI_WAVE);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  int total = 0;
  for (int i = 0; i < nwaves; ++i) total += scratch[i];
  return total;
}

// Stage one of the argmax: each workgroup scans one chunk of one row and leaves its best
// (value, lowest index). grid (chunks, rows).
#define ARGMAX_CHUNKS 64
__global__ __launch_bounds__(256) void argmax_partial_kernel(const float* __restrict__ logits,
                                                             int64_t row_stride, int vocab,
                                                             float* __restrict__ part_val,
                                                             int* __restrict__ part_idx) {
  __shared__ ArgBest best[4];
  const int row = blockIdx.y, chunk = blockIdx.x;
  const int per = (vocab + ARGMAX_CHUNKS - 1) / ARGMAX_CHUNKS;
  const int lo = chunk * per, hi = min(vocab, lo + per);
  const float* x = logits + (int64_t)row * row_stride;
  ArgBest mine = {-INFINITY, 0x7fffffff};
  for (int i = lo + threadIdx.x; i < hi; i += blockDim.x) mine = better(mine, ArgBest{x[i], i});
#pragma unroll
  for (int m = DLI_WAVE / 2; m > 0; m >>= 1) {
    ArgBest o;
    o.v = __shfl_xor(mine.v, m, DLI_WAVE);
    o.i = __shfl_xor(mine.i, m, DLI_WAVE);
    mine = better(mine, o);
  }
  if (threadIdx.x % DLI_WAVE == 0) best[threadIdx.x / DLI_WAVE] = mine;
  __syncthreads();
  if (threadIdx.x == 0) {
    ArgBest top = best[0];
    for (int w = 1; w < (int)(blockDim.x / DLI_WAVE); ++w) top = better(top, best[w]);
    part_val[row * ARGMAX_CHUNKS + chunk] = top.v;
    part_idx[row * ARGMAX_CHUNKS + chunk] = top.i;
  }
}

// Between two decode steps that run back to back on the device: row i's sampled token becomes
// its next input, its position and key count grow by one, its draw counter moves on, and its
// cache slot in each group of layers is looked up in its block table. Rows without keys
// (padding) are left alone. `tokens_out` receives the sampled tokens of the step that has just
// run; with advance == 0 nothing else is done (the last step of a run).
#define ADVANCE_MAX_GROUPS 4
struct AdvanceGroups {
  int* slots[ADVANCE_MAX_GROUPS];
  const int* tables[ADVANCE_MAX_GROUPS];
};
struct AdvanceArgs {
  int* tokens_out;  // null: the sampling kernel does none of this
  int* token_ids;
  int* positions;
  int* kv_len;
  uint64_t* counters;
  AdvanceGroups groups;
  int n_groups, table_stride, page_size, advance;
};

__device__ __forceinline__ void advance_row(const AdvanceArgs& a, int i, int tok) {
  a.tokens_out[i] = tok;
  if (!a.advance || a.kv_len[i] <= 0) return;
  const int pos = a.positions[i] + 1;
  a.token_ids[i] = tok;
  a.positions[i] = pos;
  a.kv_len[i] += 1;
  a.counters[i] += 1;
  for (int g = 0; g < a.n_groups; ++g) {
    const int page = a.groups.tables[g][(int64_t)i * a.table_stride + pos / a.page_size];
    a.groups.slots[g][i] = page * a.page_size + pos % a.page_size;
  }
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(
    const float* __restrict__ logits, int64_t row_stride, int vocab,
    const float* __restrict__ temperature, const int* __restrict__ top_k,
    const float* __restrict__ top_p, const uint64_t* __restrict__ seeds,
    const uint64_t* __restrict__ counters, const float* __restrict__ part_val,
    const int* __restrict__ part_idx, int parts, int* __restrict__ out, AdvanceArgs next) {
  __shared__ float fscratch[16];
  __shared__ int iscratch[16];
  __shared__ ArgBest best[16];
  __shared__ float chunk_sums[SAMPLE_THREADS];
  __shared__ int chosen;

  const int row = blockIdx.x, tid = threadIdx.x;
  const float* x = logits + (int64_t)row * row_stride;
  const float temp = temperature[row];
  const int k = top_k[row];
  const bool greedy = temp == 0.f || k == 1;

  // maximum (and its lowest index), from the `parts` results of stage one
  ArgBest mine = {-INFINITY, 0x7fffffff};
  if (tid < parts) mine = ArgBest{part_val[(int64_t)row * parts + tid], part_idx[(int64_t)row * parts + tid]};
#pragma unroll
  for (int m = DLI_WAVE / 2; m > 0; m >>= 1) {
    ArgBest o;
    o.v = __shfl_xor(mine.v, m, DLI_WAVE);
    o.i = __shfl_xor(mine.i, m, DLI_WAVE);
    mine = better(mine, o);
  }
  if (tid % DLI_WAVE == 0) best[tid / DLI_WAVE] = mine;
  __syncthreads();
  ArgBest top = best[0];
  for (int w = 1; w < (int)(blockDim.x / DLI_WAVE); ++w) top = better(top, best[w]);
  if (greedy) {
    if (tid == 0) {
      out[row] = top.i;
      if (next.tokens_out != nullptr) advance_row(next, row, top.i);
    }
    return;
  }
  // the draw's counter, before this row moves on to its next draw
  const uint64_t draw = counters[row];

  const float inv_t = 1.f / temp;
  const float xmax = top.v * inv_t;

  // top-k threshold: the largest key t with count(key >= t) >= k
  uint32_t keep_key = 0u;  // keep everything
  if (k > 0 && k < vocab) {
    uint32_t t = 0u;
    for (int bit = 31; bit >= 0; --bit) {
      const uint32_t probe = t | (1u << bit);
      int cnt = 0;
      for (int i = tid; i < vocab; i += blockDim.x) cnt += order_key(x[i] * inv_t) >= probe;
      if (block_sum_i(cnt, iscratch) >= k) t = probe;
    }
    keep_key = t;
  }

  // top-p threshold: the smallest key t with mass(key > t) < top_p * mass(kept)
  const float p = top_p[row];
  if (p < 1.f) {
    float z = 0.f;
    for (int i = tid; i < vocab; i += blockDim.x) {
      const float v = x[i] * inv_t;
      if (order_key(v) >= keep_key) z += expf(v - xmax);
    }
    const float limit = p * block_sum_f(z, fscratch);
    // bitwise search for the smallest t where the predicate holds; the predicate is monotone in t
    uint32_t t = 0u;
    for (int bit = 31; bit >= 0; --bit) {
      const uint32_t probe = t | (1u << bit);  // test the predicate at probe - 1
      const uint32_t at = probe - 1u;
      float above = 0.f;
      for (int i = tid; i < vocab; i += blockDim.x) {
        const float v = x[i] * inv_t;
        const uint32_t key = order_key(v);
        if (key >= keep_key && key > at) above += expf(v - xmax);
      }
      if (!(block_sum_f(above, fscratch) < limit)) t = probe;  // predicate false at probe-1: answer >= probe
    }
    if (t > keep_key) keep_key = t;
  }

  // inverse CDF over the kept tokens in vocabulary order; each thread owns a contiguous chunk
  const int chunk = (vocab + blockDim.x - 1) / blockDim.x;
  const int lo = min(vocab, tid * chunk), hi = min(vocab, lo + chunk);
  float s = 0.f;
  for (int i = lo; i < hi; ++i) {
    const float v = x[i] * inv_t;
    if (order_key(v) >= keep_key) s += expf(v - xmax);
  }
  chunk_sums[tid] = s;
  if (tid == 0) chosen = -1;
  __syncthreads();
  if (tid == 0) {
    float total = 0.f;
    for (int i = 0; i < (int)blockDim.x; ++i) total += chunk_sums[i];
    const float u = (float)(philox_first_word(seeds[row], draw) >> 8) * (1.0f / 16777216.0f);
    const float target = u * total;
    float run = 0.f;
    int owner = -1;
    for (int i = 0; i < (int)blockDim.x; ++i) {
      if (chunk_sums[i] > 0.f) {
        owner = i;  // the last chunk with mass takes a target that rounding pushed to the end
        if (run + chunk_sums[i] > target) break;
        run += chunk_sums[i];
      }
    }
    chosen = owner;
    fscratch[0] = target - run;  // what is left to cover inside the owner's chunk
  }
  __syncthreads();
  if (tid == chosen) {
    const float rest = fscratch[0];
    float run = 0.f;
    int pick = -1;
    for (int i = lo; i < hi; ++i) {
      const float v = x[i] * inv_t;
      if (order_key(v) >= keep_key) {
        pick = i;
        run += expf(v - xmax);
        if (run > rest) break;
      }
    }
    out[row] = pick;
    if (next.tokens_out != nullptr) advance_row(next, row, pick);
  }
  if (chosen < 0 && tid == 0) {  // no mass at all (cannot happen: the maximum is kept)
    out[row] = top.i;
    if (next.tokens_out != nullptr) advance_row(next, row, top.i);
  }
}

// Floats and ints of scratch that dli_sample needs per row.
extern "C" int dli_sample_scratch_per_row() { return ARGMAX_CHUNKS; }

extern "C" int dli_sample(const float* logits, int64_t row_stride, int rows, int vocab,
                          const float* temperature, const int* top_k, const float* top_p,
                          const uint64_t* seeds, const uint64_t* counters, float* part_val,
                          int* part_idx, int* out, hipStream_t stream) {
  if (rows <= 0) return DLI_OK;
  if (vocab <= 0 || row_stride < vocab || rows > 65535 || part_val == nullptr || part_idx == nullptr)
    return DLI_ERR_ARGUMENT;
  argmax_partial_kernel<<<dim3(ARGMAX_CHUNKS, rows), 256, 0, stream>>>(logits, row_stride, vocab,
                                                                       part_val, part_idx);
  if (dli_launch_status() != DLI_OK) return DLI_ERR_LAUNCH;
  AdvanceArgs none = {};
  sample_kernel<<<rows, SAMPLE_THREADS, 0, stream>>>(logits, row_stride, vocab, temperature, top_k, top_p, seeds,
                                                     counters, part_val, part_idx, ARGMAX_CHUNKS, out, none);
  return dli_launch_status();
}

static bool fill_groups(AdvanceGroups& groups, int* const* slots, const int* const* tables, int n_groups) {
  if (n_groups < 0 || n_groups > ADVANCE_MAX_GROUPS) return false;
  for (int g = 0; g < ADVANCE_MAX_GROUPS; ++g) {
    groups.slots[g] = g < n_groups ? slots[g] : nullptr;
    groups.tables[g] = g < n_groups ? tables[g] : nullptr;
    if (g < n_groups && (groups.slots[g] == nullptr || groups.tables[g] == nullptr)) return false;
  }
  return true;
}

// dli_sample and dli_decode_advance in one: the thread that chooses a row's token also hands it to
// the row's next step, so a decode step inside a graph ends with one kernel less. `parts` > 0:
// stage one of the argmax has been done by whoever made the logits (dli_head_gemm), part_val and
// part_idx hold [rows][parts]; 0: it runs here (they then need dli_sample_scratch_per_row() per row).
extern "C" int dli_sample_and_advance(const float* logits, int64_t row_stride, int rows, int vocab,
                                      const float* temperature, const int* top_k, const float* top_p,
                                      const uint64_t* seeds, uint64_t* counters, float* part_val, int* part_idx,
                                      int parts, int* out, int* tokens_out, int* token_ids, int* positions,
                                      int* kv_len, int* const* slots, const int* const* tables, int n_groups,
                                      int table_stride, int page_size, int advance, hipStream_t stream) {
  if (rows <= 0) return DLI_OK;
  if (vocab <= 0 || row_stride < vocab || rows > 65535 || part_val == nullptr || part_idx == nullptr ||
      parts < 0 || parts > SAMPLE_THREADS || out == nullptr || tokens_out == nullptr || token_ids == nullptr ||
      positions == nullptr || kv_len == nullptr || counters == nullptr || page_size <= 0 || table_stride <= 0)
    return DLI_ERR_ARGUMENT;
  AdvanceArgs next = {tokens_out, token_ids, positions, kv_len, counters, {}, n_groups, table_stride, page_size,
                      advance};
  if (!fill_groups(next.groups, slots, tables, n_groups)) return DLI_ERR_ARGUMENT;
  if (parts == 0) {
    argmax_partial_kernel<<<dim3(ARGMAX_CHUNKS, rows), 256, 0, stream>>>(logits, row_stride, vocab, part_val,
                                                                         part_idx);
    if (dli_launch_status() != DLI_OK) return DLI_ERR_LAUNCH;
    parts = ARGMAX_CHUNKS;
  }
  sample_kernel<<<rows, SAMPLE_THREADS, 0, stream>>>(logits, row_stride, vocab, temperature, top_k, top_p, seeds,
                                                     counters, part_val, part_idx, parts, out, next);
  return dli_launch_status();
}

// The same hand-over as a kernel of its own (for steps whose tokens were chosen elsewhere).
__global__ void decode_advance_kernel(const int* __restrict__ sampled, AdvanceArgs next, int rows) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < rows) advance_row(next, i, sampled[i]);
}

extern "C" int dli_decode_advance(const int* sampled, int* tokens_out, int* token_ids, int* positions,
                                  int* kv_len, uint64_t* counters, int* const* slots,
                                  const int* const* tables, int n_groups, int table_stride,
                                  int page_size, int rows, int advance, hipStream_t stream) {
  if (rows <= 0) return DLI_OK;
  if (page_size <= 0 || table_stride <= 0 || tokens_out == nullptr) return DLI_ERR_ARGUMENT;
  AdvanceArgs next = {tokens_out, token_ids, positions, kv_len, counters, {}, n_groups, table_stride, page_size,
                      advance};
  if (!fill_groups(next.groups, slots, tables, n_groups)) return DLI_ERR_ARGUMENT;
  decode_advance_kernel<<<(rows + 255) / 256, 256, 0, stream>>>(sampled, next, rows);
  return dli_launch_status();
}
