// Paged attention on the vector units, for every size: any page size, head_dim in steps of 16 up
// to 256, any number of heads and groups, portions of prompts beside single decoded tokens.
// All arithmetic is 32-bit whatever the storage type, so this is the attention of the true 32-bit
// path and the fallback of the bf16 path for shapes that the matrix-core kernels refuse.
//
// One workgroup takes BM consecutive queries of one request (one "tile") and one query head, and
// walks that request's keys in tiles of BN through its block table with an online softmax
// (running maximum m, running sum l, accumulator rescaled by exp(m_old - m_new)).
//
// A query at absolute position p sees key j iff j <= p and (window <= 0 or j > p - window).
// Scores are scaled by `scale` (1/sqrt(head_dim) in the reference: src/dli/model/llama.py:165-177,
// src/dli/model/paged_attention.py:150,274).
//
// Page layout: K [pages][kv_heads][page_size][head_dim], V [pages][kv_heads][head_dim][page_size].
#include "common.h"

template <typename T, int RM, int RN, int DC>
__global__ __launch_bounds__(256) void attention_generic_kernel(
    const T* __restrict__ q, int64_t q_stride, const T* __restrict__ k_pages,
    const T* __restrict__ v_pages, T* __restrict__ out, int64_t out_stride,
    const int* __restrict__ q_start, const int* __restrict__ kv_len,
    const int* __restrict__ block_tables, int table_stride, const int* __restrict__ tile_entry,
    const int* __restrict__ tile_q0, int q_heads, int kv_heads, int head_dim, int page_size,
    float scale, int window) {
  constexpr int BM = 16 * RM, BN = 16 * RN, DMAX = 16 * DC;
  __shared__ float qs[BM][DMAX + 1];
  __shared__ float ks[BN][DMAX + 1];
  __shared__ float vs[BN][DMAX + 1];
  __shared__ float ps[BM][BN + 1];

  const int tid = threadIdx.x, tx = tid % 16, ty = tid / 16;
  const int entry = tile_entry[blockIdx.x];
  const int q0 = tile_q0[blockIdx.x];
  const int head = blockIdx.y;
  const int kvh = head / (q_heads / kv_heads);
  const int tok0 = q_start[entry];
  const int q_len = q_start[entry + 1] - tok0;
  const int n_keys = kv_len[entry];
  const int first_pos = n_keys - q_len;  // absolute position of this request's first query here
  const int rows = min(BM, q_len - q0);
  const int* table = block_tables + (int64_t)entry * table_stride;

  for (int idx = tid; idx < BM * head_dim; idx += 256) {
    const int r = idx / head_dim, c = idx - r * head_dim;
    qs[r][c] = r < rows ? to_f32(q[(int64_t)(tok0 + q0 + r) * q_stride + (int64_t)head * head_dim + c]) * scale : 0.f;
  }

  float m_run[RM], l_run[RM], acc[RM][DC];
#pragma unroll
  for (int i = 0; i < RM; ++i) {
    m_run[i] = -INFINITY;
    l_run[i] = 0.f;
#pragma unroll
    for (int c = 0; c < DC; ++c) acc[i][c] = 0.f;
  }

  const int pos_lo = first_pos + q0, pos_hi = first_pos + q0 + rows - 1;
  int j_begin = 0;
  if (window > 0) j_begin = max(0, pos_lo - window + 1) / BN * BN;
  const int j_end = pos_hi + 1;

  for (int j0 = j_begin; j0 < j_end; j0 += BN) {
    __syncthreads();  // previous tile's reads of ks/vs/ps are done (and qs is written)
    for (int idx = tid; idx < BN * head_dim; idx += 256) {
      const int r = idx / head_dim, c = idx - r * head_dim;
      const int j = j0 + r;
      float kv = 0.f;
      if (j < j_end) {
        const int64_t page = table[j / page_size];
        kv = to_f32(k_pages[((page * kv_heads + kvh) * page_size + j % page_size) * head_dim + c]);
      }
      ks[r][c] = kv;
    }
    for (int idx = tid; idx < BN * head_dim; idx += 256) {
      const int c = idx / BN, r = idx - c * BN;  // key index fastest: contiguous in a V page
      const int j = j0 + r;
      float vv = 0.f;
      if (j < j_end) {
        const int64_t page = table[j / page_size];
        vv = to_f32(v_pages[((page * kv_heads + kvh) * head_dim + c) * page_size + j % page_size]);
      }
      vs[r][c] = vv;
    }
    __syncthreads();

    float s[RM][RN];
#pragma unroll
    for (int i = 0; i < RM; ++i)
#pragma unroll
      for (int jj = 0; jj < RN; ++jj) s[i][jj] = 0.f;
    for (int c = 0; c < head_dim; ++c) {
      float qa[RM], kb[RN];
#pragma unroll
      for (int i = 0; i < RM; ++i) qa[i] = qs[ty * RM + i][c];
#pragma unroll
      for (int jj = 0; jj < RN; ++jj) kb[jj] = ks[tx + 16 * jj][c];
#pragma unroll
      for (int i = 0; i < RM; ++i)
#pragma unroll
        for (int jj = 0; jj < RN; ++jj) s[i][jj] = fmaf(qa[i], kb[jj], s[i][jj]);
    }

#pragma unroll
    for (int i = 0; i < RM; ++i) {
      const int r = ty * RM + i;
      const int pos = first_pos + q0 + r;
      float tile_max = -INFINITY;
#pragma unroll
      for (int jj = 0; jj < RN; ++jj) {
        const int j = j0 + tx + 16 * jj;
        const bool visible = r < rows && j <= pos && (window <= 0 || j > pos - window);
        s[i][jj] = visible ? s[i][jj] : -INFINITY;
        tile_max = fmaxf(tile_max, s[i][jj]);
      }
#pragma unroll
      for (int msk = 8; msk > 0; msk >>= 1) tile_max = fmaxf(tile_max, __shfl_xor(tile_max, msk, DLI_WAVE));
      const float m_new = fmaxf(m_run[i], tile_max);
      float alpha = 1.f, tile_sum = 0.f;
      if (m_new > -INFINITY) {
        alpha = expf(m_run[i] - m_new);  // exp(-inf) = 0 on the first visible tile
#pragma unroll
        for (int jj = 0; jj < RN; ++jj) {
          const float p = expf(s[i][jj] - m_new);
          ps[r][tx + 16 * jj] = p;
          tile_sum += p;
        }
      } else {
#pragma unroll
        for (int jj = 0; jj < RN; ++jj) ps[r][tx + 16 * jj] = 0.f;
      }
#pragma unroll
      for (int msk = 8; msk > 0; msk >>= 1) tile_sum += __shfl_xor(tile_sum, msk, DLI_WAVE);
      l_run[i] = l_run[i] * alpha + tile_sum;
      m_run[i] = m_new;
#pragma unroll
      for (int c = 0; c < DC; ++c) acc[i][c] *= alpha;
    }
    __syncthreads();

    for (int jj = 0; jj < BN; ++jj) {
      float pv[RM];
#pragma unroll
      for (int i = 0; i < RM; ++i) pv[i] = ps[ty * RM + i][jj];
#pragma unroll
      for (int c = 0; c < DC; ++c) {
        if (c * 16 < head_dim) {
          const float vv = vs[jj][tx + 16 * c];
#pragma unroll
          for (int i = 0; i < RM; ++i) acc[i][c] = fmaf(pv[i], vv, acc[i][c]);
        }
      }
    }
  }

#pragma unroll
  for (int i = 0; i < RM; ++i) {
    const int r = ty * RM + i;
    if (r >= rows) continue;
    const float inv = l_run[i] > 0.f ? 1.f / l_run[i] : 0.f;
    T* o = out + (int64_t)(tok0 + q0 + r) * out_stride + (int64_t)head * head_dim;
#pragma unroll
    for (int c = 0; c < DC; ++c)
      if (c * 16 < head_dim) o[tx + 16 * c] = from_f32<T>(acc[i][c] * inv);
  }
}

template <typename T, int RM, int RN, int DC>
static int launch_generic(const void* q, int64_t q_stride, const void* k_pages, const void* v_pages,
                          void* out, int64_t out_stride, const int* q_start, const int* kv_len,
                          const int* block_tables, int table_stride, const int* tile_entry,
                          const int* tile_q0, int tiles, int q_heads, int kv_heads, int head_dim,
                          int page_size, float scale, int window, hipStream_t stream) {
  attention_generic_kernel<T, RM, RN, DC><<<dim3(tiles, q_heads), 256, 0, stream>>>(
      (const T*)q, q_stride, (const T*)k_pages, (const T*)v_pages, (T*)out, out_stride, q_start,
      kv_len, block_tables, table_stride, tile_entry, tile_q0, q_heads, kv_heads, head_dim,
      page_size, scale, window);
  return dli_launch_status();
}

// Queries per tile for a head_dim: the host builds its tile list with this.
extern "C" int dli_attention_generic_tile_rows(int head_dim) {
  if (head_dim <= 0 || head_dim % 16 != 0 || head_dim > 256) return DLI_ERR_ARGUMENT;
  return head_dim <= 128 ? 32 : 16;
}

extern "C" int dli_attention_generic(const void* q, int64_t q_stride, const void* k_pages,
                                     const void* v_pages, void* out, int64_t out_stride,
                                     const int* q_start, const int* kv_len, const int* block_tables,
                                     int table_stride, const int* tile_entry, const int* tile_q0,
                                     int tiles, int q_heads, int kv_heads, int head_dim, int page_size,
                                     float scale, int window, int is_bf16, hipStream_t stream) {
  if (tiles <= 0) return DLI_OK;
  if (head_dim <= 0 || head_dim % 16 != 0 || head_dim > 256 || q_heads <= 0 || kv_heads <= 0 ||
      q_heads % kv_heads != 0 || q_heads > 65535 || page_size <= 0 || table_stride <= 0)
    return DLI_ERR_ARGUMENT;
#define GENERIC_ARGS                                                                              \
  q, q_stride, k_pages, v_pages, out, out_stride, q_start, kv_len, block_tables, table_stride,   \
      tile_entry, tile_q0, tiles, q_heads, kv_heads, head_dim, page_size, scale, window, stream
  if (is_bf16) {
    if (head_dim <= 64) return launch_generic<bf16_t, 2, 2, 4>(GENERIC_ARGS);
    if (head_dim <= 128) return launch_generic<bf16_t, 2, 2, 8>(GENERIC_ARGS);
    return launch_generic<bf16_t, 1, 1, 16>(GENERIC_ARGS);
  }
  if (head_dim <= 64) return launch_generic<float, 2, 2, 4>(GENERIC_ARGS);
  if (head_dim <= 128) return launch_generic<float, 2, 2, 8>(GENERIC_ARGS);
  return launch_generic<float, 1, 1, 16>(GENERIC_ARGS);
#undef GENERIC_ARGS
}
