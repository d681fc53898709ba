// Paged attention on the matrix cores (bfloat16 operands, 32-bit accumulation), for decode
// (one query per request, keys split over workgroups, partial results merged) and for portions of
// prompts (tiles of queries, causal by absolute position).
//
// Both kernels compute the transposed products, so that every per-query statistic of the online
// softmax lives in the lane that owns the query's column and no operand is ever transposed:
//
//   S^T [16 keys x 16 columns]   = K [16 keys x d]   * Q^T [d x 16 columns]
//   O^T [16 dims x 16 columns]  += V^T [16 dims x 16 keys] * P^T [16 keys x 16 columns]
//
// with v_mfma_f32_16x16x16_bf16: operand A gives lane l row l%16 and the four k-indices
// 4*(l/16)..+3; operand B gives lane l column l%16 and the same k-indices; the result gives lane l
// column l%16 and rows 4*(l/16)..+3. So S^T comes out exactly in the layout that P^T needs as
// operand B of the second product. A "column" is a query head of the group in the decode kernel
// and a query position in the prefill kernel.
//
// K pages are [kv_heads][page_size][head_dim] and V pages [kv_heads][head_dim][page_size]: operand
// A of the first product reads head_dim-contiguous keys, operand A of the second reads
// key-contiguous dims. The d index of the first product is permuted (lane group g takes the
// contiguous range [g*d/4, (g+1)*d/4)), identically for K and Q, which leaves the dot product
// unchanged and makes each lane's K load one contiguous run.
//
// Needs page_size % 16 == 0 and head_dim = 16*DCH with DCH <= 8; other shapes take the generic
// kernel. Scores are scaled by `scale`; exp is taken as exp2 with log2(e) folded into the scale.
// P is rounded to bfloat16 for the second product while the running sum keeps the unrounded
// values (as the reference's kernel does: src/dli/model/paged_attention.py:128-168).
#include "common.h"
#include "merge_splits.h"
#include "no_alloc.h"

typedef short short4v __attribute__((ext_vector_type(4)));
typedef float float4v __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float4v mfma16(short4v a, short4v b, float4v c) {
  return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ short bf16_bits(float x) {
  bf16_t b = (bf16_t)x;
  return *reinterpret_cast<short*>(&b);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Maximum as one instruction. fmaxf() asks for a quieted NaN, which costs a second instruction per
// operand that the compiler cannot prove canonical (every matrix-core result); scores are never
// NaN here (masked ones are -inf), and the instruction itself orders -inf and finite values as
// fmaxf does. The prefill kernel is bound by the vector unit's instruction count: 65 -> 59 us a
// layer at 2,048 tokens of the 1B sizes.
__device__ __forceinline__ float max2(float a, float b) {
  float r;
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
__device__ __forceinline__ float max3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}

// Reductions over the four lanes l, l^16, l^32, l^48 (the lane groups that share a column) with
// the gfx950 lane-swap instructions: after v_permlane32_swap of two copies of v, one copy holds
// the lower half's values in both halves and the other the upper half's; v_permlane16_swap does
// the same for neighbouring rows of 16 lanes.
__device__ __forceinline__ float column_max(float v) {
  const unsigned u = __float_as_uint(v);
  const auto a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  const float m = max2(__uint_as_float(a[0]), __uint_as_float(a[1]));
  const unsigned um = __float_as_uint(m);
  const auto b = __builtin_amdgcn_permlane16_swap(um, um, false, false);
  return max2(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float column_sum(float v) {
  const unsigned u = __float_as_uint(v);
  const auto a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  const float m = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  const unsigned um = __float_as_uint(m);
  const auto b = __builtin_amdgcn_permlane16_swap(um, um, false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// Online-softmax state of one column tile (16 columns; this lane owns column lane%16).
template <int DCH>
struct ColumnTile {
  float m, l;
  float4v o[DCH];
  __device__ __forceinline__ void init() {
    m = -INFINITY;
    l = 0.f;
#pragma unroll
    for (int c = 0; c < DCH; ++c) o[c] = float4v{0.f, 0.f, 0.f, 0.f};
  }
};

// One tile of 16 keys starting at logical key `t` (page-aligned by 16) against one column tile.
// `limit[i]` for i in 0..3: the largest visible key for this lane's column (causal / request end),
// `lowest`: the smallest visible key (window); keys outside become -inf.
template <int DCH>
__device__ __forceinline__ void attend_tile(ColumnTile<DCH>& st, const short4v (&kreg)[DCH],
                                            const short4v (&qreg)[DCH], const short4v (&vreg)[DCH],
                                            int t, int grp, int last_visible, int first_visible,
                                            float scale_log2e, bool need_mask) {
  float4v s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int c = 0; c < DCH; ++c) s = mfma16(kreg[c], qreg[c], s);
  float sv[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) sv[i] = s[i] * scale_log2e;
  if (need_mask) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int key = t + 4 * grp + i;
      if (key > last_visible || key < first_visible) sv[i] = -INFINITY;
    }
  }
  const float tile_max = column_max(max2(max3(sv[0], sv[1], sv[2]), sv[3]));
  const float m_new = max2(st.m, tile_max);
  const float m_safe = m_new == -INFINITY ? 0.f : m_new;
  const float alpha = fast_exp2(st.m - m_safe);
  float p[4];
  float tile_sum = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    p[i] = fast_exp2(sv[i] - m_safe);
    tile_sum += p[i];
  }
  tile_sum = column_sum(tile_sum);
  st.l = st.l * alpha + tile_sum;
  st.m = m_new;
  const short4v pb = {bf16_bits(p[0]), bf16_bits(p[1]), bf16_bits(p[2]), bf16_bits(p[3])};
  if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {  // the running maximum rose somewhere
#pragma unroll
    for (int c = 0; c < DCH; ++c) st.o[c] *= alpha;
  }
#pragma unroll
  for (int c = 0; c < DCH; ++c) st.o[c] = mfma16(vreg[c], pb, st.o[c]);
}

template <int DCH>
__device__ __forceinline__ void load_k(short4v (&kreg)[DCH], const bf16_t* __restrict__ k_pages,
                                       int64_t page, int kv_heads, int kvh, int page_size, int off,
                                       int col, int grp) {
  constexpr int D = DCH * 16;
  const bf16_t* p = k_pages + ((page * kv_heads + kvh) * page_size + off + col) * D + grp * (D / 4);
#pragma unroll
  for (int c = 0; c < DCH; ++c) kreg[c] = *reinterpret_cast<const short4v*>(p + c * 4);
}

template <int DCH>
__device__ __forceinline__ void load_v(short4v (&vreg)[DCH], const bf16_t* __restrict__ v_pages,
                                       int64_t page, int kv_heads, int kvh, int page_size, int off,
                                       int col, int grp) {
  constexpr int D = DCH * 16;
  const bf16_t* p = v_pages + ((page * kv_heads + kvh) * D + col) * page_size + off + 4 * grp;
#pragma unroll
  for (int c = 0; c < DCH; ++c) vreg[c] = *reinterpret_cast<const short4v*>(p + (int64_t)c * 16 * page_size);
}

// Values of keys at or beyond `end_key` are replaced by zero so that a zero probability never
// multiplies whatever a not yet written slot holds. Apart from the loads: what looks at loaded
// values waits for them.
template <int DCH>
__device__ __forceinline__ void blank_v(short4v (&vreg)[DCH], int grp, int t, int end_key) {
  if (t + 16 > end_key) {
#pragma unroll
    for (int c = 0; c < DCH; ++c)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (t + 4 * grp + i >= end_key) vreg[c][i] = 0;
  }
}

// ------------------------------------------------------------------------------------ decode
// grid (splits, kv_heads * head_tiles, requests); 256 threads. Request e's single query is row e.
// part_o, part_ml and arrivals without __restrict__: the workgroup that merges reads what other
// workgroups of the launch stored.
template <int DCH>
__global__ __launch_bounds__(256) void attention_decode_kernel(
    const bf16_t* __restrict__ q, int64_t q_stride, const bf16_t* __restrict__ k_pages,
    const bf16_t* __restrict__ v_pages, bf16_t* __restrict__ out, int64_t out_stride,
    float* part_o, float* part_ml, const int* __restrict__ kv_len,
    const int* __restrict__ block_tables, int table_stride, int q_heads, int kv_heads, int page_size,
    float scale_log2e, int window, int splits, unsigned* arrivals) {
  constexpr int D = DCH * 16;
  __shared__ float sm_o[3][D][16];
  __shared__ float sm_m[3][16], sm_l[3][16];

  const int split = blockIdx.x, e = blockIdx.z;
  const int group = q_heads / kv_heads;
  const int head_tiles = (group + 15) / 16;
  const int kvh = blockIdx.y / head_tiles, ht = blockIdx.y % head_tiles;
  const int lane = threadIdx.x % DLI_WAVE;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / DLI_WAVE);  // known to be the same in all lanes
  const int col = lane % 16, grp = lane / 16;
  const int head_in_group = ht * 16 + col;
  const bool valid = head_in_group < group;
  const int head = kvh * group + head_in_group;

  const int n_keys = kv_len[e];
  const int first_visible = window > 0 ? max(0, n_keys - window) : 0;
  const int begin = first_visible / 16 * 16;
  const int chunk = (((n_keys - begin + splits - 1) / splits) + 15) / 16 * 16;
  const int k0 = begin + split * chunk;
  const int k1 = min(n_keys, k0 + chunk);
  const int* table = block_tables + (int64_t)e * table_stride;

  short4v qreg[DCH];
#pragma unroll
  for (int c = 0; c < DCH; ++c) qreg[c] = short4v{0, 0, 0, 0};
  if (valid) {
    const bf16_t* qp = q + (int64_t)e * q_stride + (int64_t)head * D + grp * (D / 4);
#pragma unroll
    for (int c = 0; c < DCH; ++c) qreg[c] = *reinterpret_cast<const short4v*>(qp + c * 4);
  }

  ColumnTile<DCH> st;
  st.init();
  // A wave takes every fourth tile of 16 keys, UN tiles (a group) at a time. A group costs a chain
  // of two trips to memory (its block-table entries, then its keys and values), so the chain is
  // taken apart: while group g is multiplied, the keys and values of group g+1 are on their way
  // (two sets of registers take turns) and the table entries of group g+2 have been asked for.
  // No load hangs on a condition (a tile past the run's end reads the run's last tile again and
  // is skipped by the arithmetic; values of keys past the end are blanked when they are used),
  // so at every wait the number of younger loads is known and only the group's own are waited for.
  constexpr int UN = 1, NG = 4;  // tiles of a group, groups on their way
  constexpr int STEP = 64 * UN;  // keys between a wave's groups
  struct Group {
    short4v k[UN][DCH], v[UN][DCH];
  };
  struct Where {
    int64_t page[UN];
    int off[UN];
  };
  const int t_first = k0 + wave * 16;
  if (t_first < k1) {
    const int t_last = (k1 - 1) / 16 * 16;  // the run's last tile
    auto look_up = [&](Where& w, int tg) __attribute__((always_inline)) {
#pragma unroll
      for (int u = 0; u < UN; ++u) {
        const int t = min(tg + 64 * u, t_last);
        w.page[u] = table[t / page_size];
        w.off[u] = t % page_size;
      }
    };
    auto fetch = [&](Group& g, const Where& w) __attribute__((always_inline)) {
#pragma unroll
      for (int u = 0; u < UN; ++u) {
        load_k<DCH>(g.k[u], k_pages, w.page[u], kv_heads, kvh, page_size, w.off[u], col, grp);
        load_v<DCH>(g.v[u], v_pages, w.page[u], kv_heads, kvh, page_size, w.off[u], col, grp);
      }
    };
    auto attend = [&](const Group& g, int tg) __attribute__((always_inline)) {
#pragma unroll
      for (int u = 0; u < UN; ++u) {
        const int t = tg + 64 * u;
        if (t < k1) {
          const bool need_mask = t + 16 > k1 || t < first_visible;
          short4v v[DCH];  // a copy: the group's registers are written by loads only
#pragma unroll
          for (int c = 0; c < DCH; ++c) v[c] = g.v[u][c];
          blank_v<DCH>(v, grp, t, k1);
          attend_tile<DCH>(st, g.k[u], qreg, v, t, grp, k1 - 1, first_visible, scale_log2e, need_mask);
        }
      }
    };
    // NG sets of registers take turns; set d holds group g = d (mod NG), and where[d] the place of
    // the group that it loads next
    Group sets[NG];
    Where where[NG];
#pragma unroll
    for (int d = 0; d < NG; ++d) look_up(where[d], t_first + d * STEP);
#pragma unroll
    for (int d = 0; d < NG; ++d) {
      fetch(sets[d], where[d]);
      look_up(where[d], t_first + (d + NG) * STEP);
    }
    int tg = t_first;
    for (; tg + NG * STEP < k1; tg += NG * STEP) {  // rounds that have a group behind them
#pragma unroll
      for (int d = 0; d < NG; ++d) {
        attend(sets[d], tg + d * STEP);
        fetch(sets[d], where[d]);
        look_up(where[d], tg + (d + 2 * NG) * STEP);
        __builtin_amdgcn_sched_barrier(0);  // the loads leave before the next group's arithmetic
      }
    }
#pragma unroll
    for (int d = 0; d < NG; ++d) attend(sets[d], tg + d * STEP);  // the last round
  }

  // merge the four waves' states in wave 0
  if (wave > 0) {
    if (grp == 0) {
      sm_m[wave - 1][col] = st.m;
      sm_l[wave - 1][col] = st.l;
    }
#pragma unroll
    for (int c = 0; c < DCH; ++c)
#pragma unroll
      for (int i = 0; i < 4; ++i) sm_o[wave - 1][c * 16 + 4 * grp + i][col] = st.o[c][i];
  }
  __syncthreads();
  if (wave != 0) return;
  float m_all = st.m;
#pragma unroll
  for (int w = 0; w < 3; ++w) m_all = fmaxf(m_all, sm_m[w][col]);
  const float m_safe = m_all == -INFINITY ? 0.f : m_all;
  float scale_own = fast_exp2(st.m - m_safe);
  float l_all = st.l * scale_own;
#pragma unroll
  for (int c = 0; c < DCH; ++c) st.o[c] *= scale_own;
#pragma unroll
  for (int w = 0; w < 3; ++w) {
    const float sw = fast_exp2(sm_m[w][col] - m_safe);
    l_all += sm_l[w][col] * sw;
#pragma unroll
    for (int c = 0; c < DCH; ++c)
#pragma unroll
      for (int i = 0; i < 4; ++i) st.o[c][i] += sm_o[w][c * 16 + 4 * grp + i][col] * sw;
  }
  if (splits == 1) {
    if (!valid) return;
    const float inv = l_all > 0.f ? 1.f / l_all : 0.f;
    bf16_t* op = out + (int64_t)e * out_stride + (int64_t)head * D + 4 * grp;
#pragma unroll
    for (int c = 0; c < DCH; ++c) {
      const short4v packed = {bf16_bits(st.o[c][0] * inv), bf16_bits(st.o[c][1] * inv),
                              bf16_bits(st.o[c][2] * inv), bf16_bits(st.o[c][3] * inv)};
      *reinterpret_cast<short4v*>(op + c * 16) = packed;
    }
    return;
  }
  if (arrivals == nullptr) {  // attention_merge_kernel follows
    if (!valid) return;
    const int64_t slot = ((int64_t)e * q_heads + head) * splits + split;
    float* po = part_o + slot * D + 4 * grp;
#pragma unroll
    for (int c = 0; c < DCH; ++c) *reinterpret_cast<float4v*>(po + c * 16) = st.o[c];
    if (grp == 0) {
      part_ml[slot * 2] = m_all;
      part_ml[slot * 2 + 1] = l_all;
    }
    return;
  }
  // The workgroup that finishes last of those that share (request, kv head, head tile) merges their
  // results, which saves the launch of a kernel that is one trip to memory long. Each workgroup
  // stores its partial results at the device's scope (through the caches that only a part of the
  // chip shares), waits until they have arrived, then counts itself in; who counts last reads
  // everybody's, at the device's scope again, and puts the counter back to zero for the next
  // launch. (Ordinary stores and loads with a release and an acquire fence of the device's scope
  // on the way give the same result, but those fences write back and empty the whole level-2
  // cache under the workgroups that still stream keys: 40 us instead of 16 for the launch.)
  if (valid) {
    const int64_t slot = ((int64_t)e * q_heads + head) * splits + split;
    const __amdgpu_buffer_rsrc_t po = device_scope_buffer(part_o);
#pragma unroll
    for (int c = 0; c < DCH; ++c) device_store4(po, (unsigned)((slot * D + 4 * grp + c * 16) * 4), st.o[c]);
    if (grp == 0) device_store2(device_scope_buffer(part_ml), (unsigned)(slot * 2 * 4), merge_float2{m_all, l_all});
  }
  // every store of this wave has been acknowledged before the count goes up ...
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __builtin_amdgcn_s_waitcnt(0);
  unsigned* counter = arrivals + (int64_t)e * gridDim.y + blockIdx.y;
  unsigned before = 0;
  if (lane == 0) before = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  before = __builtin_amdgcn_readfirstlane(before);
  if (before != (unsigned)splits - 1) return;
  // ... and the loads below are not asked for before the count has come back
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  if (lane == 0) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const int heads_here = min(16, group - ht * 16);
  constexpr int QUADS = D / 4;
  for (int item = lane; item < heads_here * QUADS; item += DLI_WAVE) {
    const int h = item / QUADS, d = (item - h * QUADS) * 4;
    const int merged_head = kvh * group + ht * 16 + h;
    const int64_t base = ((int64_t)e * q_heads + merged_head) * splits;
    const float4v y = merged_quad<true>(part_o, part_ml, base, splits, D, d);
    const short4v packed = {bf16_bits(y[0]), bf16_bits(y[1]), bf16_bits(y[2]), bf16_bits(y[3])};
    *reinterpret_cast<short4v*>(out + (int64_t)e * out_stride + (int64_t)merged_head * D + d) = packed;
  }
}

// One wave per (request, head), four to a workgroup: out = sum_s o_s 2^(m_s - M) / sum_s l_s 2^(m_s - M).
// Lane s reads the statistics of split s and every lane the partial outputs of up to SMAX splits
// for its dims, all before anything is used: the kernel is one round trip to memory long. The
// weights 2^(m_s - M) then go from lane to lane and the splits are added in their order.
// head_dim <= 64 * DV; more than SMAX splits are taken SMAX at a time.
template <int SMAX, int DV>
__global__ __launch_bounds__(256) void attention_merge_kernel(const float* __restrict__ part_o,
                                                              const float* __restrict__ part_ml,
                                                              bf16_t* __restrict__ out,
                                                              int64_t out_stride, int q_heads,
                                                              int head_dim, int splits, int pairs) {
  const int lane = threadIdx.x % DLI_WAVE;
  const int pair = blockIdx.x * 4 + threadIdx.x / DLI_WAVE;  // request * q_heads + head
  if (pair >= pairs) return;
  const int e = pair / q_heads, head = pair % q_heads;
  const int64_t base = (int64_t)pair * splits;
  float m_run = -INFINITY, l_run = 0.f;
  float acc[DV];
#pragma unroll
  for (int v = 0; v < DV; ++v) acc[v] = 0.f;
  for (int s0 = 0; s0 < splits; s0 += SMAX) {
    const int n = min(SMAX, splits - s0);
    float m_s = -INFINITY, l_s = 0.f;
    if (lane < n) {
      m_s = part_ml[(base + s0 + lane) * 2];
      l_s = part_ml[(base + s0 + lane) * 2 + 1];
    }
    float po[SMAX][DV];
#pragma unroll
    for (int j = 0; j < SMAX; ++j)
#pragma unroll
      for (int v = 0; v < DV; ++v) {
        const bool live = j < n && v * DLI_WAVE + lane < head_dim;
        po[j][v] = live ? part_o[(base + s0 + j) * head_dim + v * DLI_WAVE + lane] : 0.f;
      }
    const float m_new = fmaxf(m_run, wave_max(m_s));
    const float m_safe = m_new == -INFINITY ? 0.f : m_new;
    const float keep = fast_exp2(m_run - m_safe);  // rescales what earlier rounds left
    const float weight = lane < n ? fast_exp2(m_s - m_safe) : 0.f;
    l_run = __fmaf_rn(l_run, keep, wave_sum(__fmul_rn(l_s, weight)));
#pragma unroll
    for (int v = 0; v < DV; ++v) acc[v] *= keep;
#pragma unroll
    for (int j = 0; j < SMAX; ++j) {
      const float wj = __shfl(weight, j, DLI_WAVE);
#pragma unroll
      for (int v = 0; v < DV; ++v) acc[v] = __fmaf_rn(po[j][v], wj, acc[v]);
    }
    m_run = m_new;
  }
  const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
#pragma unroll
  for (int v = 0; v < DV; ++v)
    if (v * DLI_WAVE + lane < head_dim)
      out[(int64_t)e * out_stride + (int64_t)head * head_dim + v * DLI_WAVE + lane] = (bf16_t)(acc[v] * inv);
}

// ------------------------------------------------------------------------------------ prefill
// grid (query tiles of 128, q_heads); 256 threads; each wave owns 32 consecutive queries
// (two column tiles) of one request and walks that request's keys up to its last query.
#define PF_TILE_ROWS 128
template <int DCH>
__global__ __launch_bounds__(256) void attention_prefill_kernel(
    const bf16_t* __restrict__ q, int64_t q_stride, const bf16_t* __restrict__ k_pages,
    const bf16_t* __restrict__ v_pages, bf16_t* __restrict__ out, int64_t out_stride,
    const int* __restrict__ q_start, const int* __restrict__ kv_len,
    const int* __restrict__ block_tables, int table_stride, const int* __restrict__ tile_entry,
    const int* __restrict__ tile_q0, int q_heads, int kv_heads, int page_size, float scale_log2e,
    int window) {
  constexpr int D = DCH * 16;
  const int e = tile_entry[blockIdx.x];
  const int head = blockIdx.y;
  const int kvh = head / (q_heads / kv_heads);
  const int lane = threadIdx.x % DLI_WAVE, wave = threadIdx.x / DLI_WAVE;
  const int col = lane % 16, grp = lane / 16;
  const int tok0 = q_start[e];
  const int q_len = q_start[e + 1] - tok0;
  const int n_keys = kv_len[e];
  const int first_pos = n_keys - q_len;
  const int q0 = tile_q0[blockIdx.x] + wave * 32;  // this wave's first query
  if (q0 >= q_len) return;
  const int* table = block_tables + (int64_t)e * table_stride;

  short4v qreg[2][DCH];
  ColumnTile<DCH> st[2];
  int pos[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    st[j].init();
    const int qi = q0 + j * 16 + col;
    pos[j] = qi < q_len ? first_pos + qi : -1;  // -1: no query in this column, nothing is visible
#pragma unroll
    for (int c = 0; c < DCH; ++c) qreg[j][c] = short4v{0, 0, 0, 0};
    if (qi < q_len) {
      const bf16_t* qp = q + (int64_t)(tok0 + qi) * q_stride + (int64_t)head * D + grp * (D / 4);
#pragma unroll
      for (int c = 0; c < DCH; ++c) qreg[j][c] = *reinterpret_cast<const short4v*>(qp + c * 4);
    }
  }
  const int wave_rows = min(32, q_len - q0);
  const int pos_lo = first_pos + q0, pos_hi = first_pos + q0 + wave_rows - 1;
  const int begin = window > 0 ? max(0, pos_lo - window + 1) / 16 * 16 : 0;
  const int end = pos_hi + 1;  // keys [begin, end) may be visible to some query of this wave
  const bool second = wave_rows > 16;

  for (int t = begin; t < end; t += 16) {
    const int64_t page = table[t / page_size];
    const int off = t % page_size;
    short4v kreg[DCH], vreg[DCH];
    load_k<DCH>(kreg, k_pages, page, kv_heads, kvh, page_size, off, col, grp);
    load_v<DCH>(vreg, v_pages, page, kv_heads, kvh, page_size, off, col, grp);
    blank_v<DCH>(vreg, grp, t, end);
    // a tile needs masking if it reaches beyond the first query's position or before the window
    const bool need_mask = t + 15 > pos_lo || (window > 0 && t < pos_hi - window + 1) || wave_rows < 32;
    const int low0 = window > 0 ? pos[0] - window + 1 : 0;
    attend_tile<DCH>(st[0], kreg, qreg[0], vreg, t, grp, pos[0], low0, scale_log2e, need_mask);
    if (second) {
      const int low1 = window > 0 ? pos[1] - window + 1 : 0;
      attend_tile<DCH>(st[1], kreg, qreg[1], vreg, t, grp, pos[1], low1, scale_log2e, need_mask);
    }
  }

#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int qi = q0 + j * 16 + col;
    if (qi >= q_len) continue;
    const float inv = st[j].l > 0.f ? 1.f / st[j].l : 0.f;
    bf16_t* op = out + (int64_t)(tok0 + qi) * out_stride + (int64_t)head * D + 4 * grp;
#pragma unroll
    for (int c = 0; c < DCH; ++c) {
      const short4v packed = {bf16_bits(st[j].o[c][0] * inv), bf16_bits(st[j].o[c][1] * inv),
                              bf16_bits(st[j].o[c][2] * inv), bf16_bits(st[j].o[c][3] * inv)};
      *reinterpret_cast<short4v*>(op + c * 16) = packed;
    }
  }
}

// ------------------------------------------------------------------------------------ prefill, shared tiles
// The waves of a workgroup share every key tile through LDS. Four waves take HW query heads of
// one kv head (HW = 4, 2 or 1, whatever divides the group) times 4/HW blocks of 32 queries, so
// each K/V tile is fetched from memory once for 128 query rows. Every tile of the list has a
// workgroup of its own: listed longest first, the tiles even the causal triangle out through the
// queue of workgroups, and no wave waits for a wave of another tile. Tiles of 32 keys are
// pipelined through a ring of NB buffers in LDS:
// while tile i is consumed, tile i+1 already lies there and tiles i+2..i+NB-1 are on their way
// from memory, written into LDS by the loads themselves (no registers, no second instruction; moving
// a tile through registers took a third of the kernel's time at 8,192 tokens).
// Products use v_mfma_f32_16x16x32_bf16 (lane l: row/column l%16, k-indices 8*(l/16)..+7). For
// P*V the eight k-indices of lane group g stand for the keys 8g..8g+7 of the tile.
// Head sizes of 32 to 128 in steps of 16. Where the size is no multiple of 32 (48, 80, 112) the
// first product's last sixteen dims take one v_mfma_f32_16x16x16_bf16, and K lies in LDS part by
// part (chunk `part` of the tile's 32 keys side by side, the sixteen keys of a product next to
// each other: sixteen lanes then read 256 consecutive bytes whatever the row length), which the
// loads arrange by the address each lane reads from; a block of 64 chunks then holds keys of
// both halves of the tile, so the half's page is chosen lane by lane.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

__device__ __forceinline__ float4v mfma32(bf16x8 a, bf16x8 b, float4v c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

// Which chunk of its row (R chunks of 16 bytes) a K chunk changes places with in LDS. A product
// reads chunk c of the sixteen key rows 8a + 4b + r (a, r = 0..3; b says which of the tile's two
// products), one row a lane: with this the sixteen lanes read sixteen different 16-byte columns
// of the 256 bytes that LDS serves at a time. Rows of 4 or 12 chunks: the four rows of one r share
// a column; of 8: the two of one r / 2; of 16: all.
template <int R>
__device__ __forceinline__ int k_swizzle(int key) {  // key: 0..31 within the tile
  static_assert(R == 4 || R == 8 || R == 12 || R == 16, "rows of 32, 64, 96 or 128 dims");
  const int a = key >> 3;
  return R == 8 ? (a << 1) | ((key >> 1) & 1) : (R == 16 ? (a << 2) | (key & 3) : a);
}

// waits until at most `n` of the wave's vector memory loads are outstanding (nothing else awaited)
template <int N>
__device__ __forceinline__ void wait_loads() {
  static_assert(N >= 0 && N < 64, "6 bits");
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// The barrier between two tiles, without the fence of __syncthreads(): that fence would wait for
// every load that is still writing LDS, the later tiles' too. What the barrier orders is stated by
// hand instead: wait_loads() before it for the tile that is read next; a buffer is written again
// only after the barrier that follows its last read, whose values the wave has used by then.
__device__ __forceinline__ void tile_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// (Held to the registers that let three waves share a SIMD for heads of up to 64 and two for
// larger ones: 126 instead of 176 and 196 instead of 276, nothing spilled, no copies between
// the two register files.)
#define PREFILL_MAX_CUTS 8  // the most runs that a tile's keys are cut into

template <int DCH>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(DCH <= 4 ? 3 : 2)))
void attention_prefill_shared_kernel(
    const bf16_t* __restrict__ q, int64_t q_stride, const bf16_t* __restrict__ k_pages,
    const bf16_t* __restrict__ v_pages, bf16_t* __restrict__ out, int64_t out_stride,
    const int* __restrict__ q_start, const int* __restrict__ kv_len,
    const int* __restrict__ block_tables, int table_stride, const int* __restrict__ tile_entry,
    const int* __restrict__ tile_q0, int q_heads, int kv_heads, int page_size, float scale_log2e,
    int window, int heads_per_wg, const int* __restrict__ tile_cut, int cut_room, float* cut_buf,
    unsigned* cut_count) {
  constexpr int D = DCH * 16, DK = D / 32;      // DK: k-steps of 32 dims of the first product
  constexpr bool ODD = DCH % 2 != 0;            // sixteen dims more, and K part by part in LDS
  static_assert(DCH >= 2 && DCH <= 8, "heads of 32 to 128");
  constexpr int R = D / 8;                      // 16-byte chunks in a key's row of K
  constexpr int NT = 256;                       // threads
  constexpr int NW = NT / DLI_WAVE;             // waves
  constexpr int BLOCKS = 2 * DCH;               // 1 KB blocks of a tile (64 chunks of 16 bytes): DCH of K, DCH of V^T
  constexpr int UCH = (BLOCKS + NW - 1) / NW;   // blocks per wave and tile
  constexpr int NB = DCH <= 4 ? 6 : (DCH <= 6 ? 5 : 4);  // tiles in LDS: one in use, the others on their way
  constexpr int K_ELEMS = 32 * D, VH_ELEMS = 16 * D, TILE_ELEMS = 64 * D;
  // a tile: K rows of 32 keys; V^T rows (one a dim) of the first 16 keys; V^T rows of the other 16
  __shared__ __attribute__((aligned(1024))) bf16_t lds[NB][TILE_ELEMS];

  // Workgroups are dealt to the eight XCDs in turn by their linear index, and each XCD has an L2
  // of its own: the tiles of one kv head are therefore given to one XCD (when the heads divide
  // evenly), so that a head's keys and values are fetched into one L2 instead of all eight.
  // Eight workgroups in a row (one an XCD) take the same tile for eight heads; the next eight the
  // same tile for the next eight heads, and only then the list's next tile: workgroups start in
  // the order of the tile list whatever the number of heads.
  int bx = blockIdx.x, by = blockIdx.y;
  const int linear = blockIdx.x + gridDim.x * blockIdx.y;
  if (gridDim.y % 8 == 0) {
    const int slot = linear / 8, head_blocks = gridDim.y / 8;
    by = linear % 8 + 8 * (slot % head_blocks);
    bx = slot / head_blocks;
  } else {  // the list's order at least: a tile for all heads, then the next tile
    by = linear % (int)gridDim.y;
    bx = linear / (int)gridDim.y;
  }
  const int e = tile_entry[bx];
  const int tok0 = q_start[e];
  const int q_len = q_start[e + 1] - tok0;
  const int tile_rows = (4 / heads_per_wg) * 32;
  const int q0_first = tile_q0[bx];
  // A tile whose keys are cut into runs (short launches: the longest workgroups are then a
  // fraction as long): this workgroup takes run `cut` of `cuts`, and the workgroup that finishes
  // last of a tile's runs adds them up. code: cut | cuts << 4 | place of the tile among the cut
  // ones << 8; cuts is at most PREFILL_MAX_CUTS, and the buffer has room for cut_room runs a tile.
  const int cut_code = tile_cut != nullptr ? tile_cut[bx] : -1;
  const int cut = cut_code >= 0 ? cut_code & 15 : 0, cuts = cut_code >= 0 ? (cut_code >> 4) & 15 : 1;
  const int cut_place = cut_code >= 0 ? cut_code >> 8 : 0;
  const int group = q_heads / kv_heads;
  const int wg_per_kv = group / heads_per_wg;
  const int kvh = by / wg_per_kv;
  const int lane = threadIdx.x % DLI_WAVE, wave = threadIdx.x / DLI_WAVE;
  const int col = lane % 16, grp = lane / 16;
  const int head = kvh * group + (by % wg_per_kv) * heads_per_wg + wave % heads_per_wg;
  const int n_keys = kv_len[e];
  const int first_pos = n_keys - q_len;
  const int q0 = q0_first + (wave / heads_per_wg) * 32;  // this wave's first query
  const int wave_rows = max(0, min(32, q_len - q0));
  const int* table = block_tables + (int64_t)e * table_stride;

  bf16x8 qreg[2][DK];
  short4v qtail[2];   // dims 32 DK + 4 grp .. + 3 (ODD)
  ColumnTile<DCH> st[2];
  // beside st[j].m: the value subtracted in the exponent (m, or 0 while m is -inf), and the raw
  // score above which m has to rise
  float m_ref[2], raise_at[2];
  constexpr float LAZY_LOG2 = 8.f;
  const float inv_scale_log2e = 1.f / scale_log2e;
  int pos[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    st[j].init();
    m_ref[j] = 0.f;
    raise_at[j] = -INFINITY;
    const int qi = q0 + j * 16 + col;
    pos[j] = qi < q_len ? first_pos + qi : -1;
#pragma unroll
    for (int c = 0; c < DK; ++c) qreg[j][c] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
    qtail[j] = short4v{0, 0, 0, 0};
    if (qi < q_len) {
      const bf16_t* qp = q + (int64_t)(tok0 + qi) * q_stride + (int64_t)head * D + grp * 8;
#pragma unroll
      for (int c = 0; c < DK; ++c) qreg[j][c] = *reinterpret_cast<const bf16x8*>(qp + c * 32);
      if constexpr (ODD) qtail[j] = *reinterpret_cast<const short4v*>(qp - grp * 8 + 32 * DK + grp * 4);
    }
  }
  // this wave's span, the same in all its lanes and said so: what is decided from it per tile
  // (whether the wave sees the tile, whether it needs the mask) is then scalar work
  const int pos_lo = __builtin_amdgcn_readfirstlane(first_pos + q0);
  const int pos_hi = __builtin_amdgcn_readfirstlane(first_pos + q0 + wave_rows - 1);
  // the workgroup walks the keys that any of its queries sees
  const int wg_q_lo = q0_first;
  const int wg_q_hi = min(q_len, q0_first + tile_rows) - 1;
  const int first_key = window > 0 ? max(0, first_pos + wg_q_lo - window + 1) / 32 * 32 : 0;
  const int end = first_pos + wg_q_hi + 1;
  const int all_tiles = (end - first_key + 31) / 32;
  const int begin = first_key + all_tiles * cut / cuts * 32;   // this run's tiles
  const int n_tiles = all_tiles * (cut + 1) / cuts - all_tiles * cut / cuts;

  // Staging: a wave moves a block of 64 chunks with one load that writes LDS directly (lane i's 16
  // bytes land at the block's address + 16 i). Blocks 0..DCH-1 are the K rows in order (16-byte
  // chunk p of the region is part p % R of key p / R), blocks DCH.. the two V^T halves (chunk p of
  // a half is 8 keys of dim p / 2). DCH is even, so whether a block is of K or of V, and which half
  // of the tile's keys it holds, is the same for all lanes of a wave: the page's address is made on
  // the scalar unit and each lane adds a constant of its own. Rows are not padded. Instead the
  // chunks of a row change places (an XOR of the chunk's number with bits of the row's number,
  // applied here to the address a lane reads from and below to the address a fragment is read
  // at) so that the 16 lanes that read one column of chunks hit 16 different bank groups.
  const int wave_id = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / DLI_WAVE));
  unsigned lane_off[UCH];   // elements from the half's first key in its page
  int block_at[UCH];        // the block's first element in a tile
  bool second_half[UCH], is_v[UCH];  // the same in all lanes
  bool lane_second[UCH];    // ODD: the half of the tile that this lane's chunk belongs to
#pragma unroll
  for (int r = 0; r < UCH; ++r) {
    // with more waves than blocks, the others load a block a second time (same bytes, same place):
    // every wave then has the same number of loads in flight
    const int blk = (wave_id + r * NW) % BLOCKS;
    is_v[r] = blk >= DCH;
    block_at[r] = blk * 512;
    if constexpr (!ODD) {
      second_half[r] = blk % DCH >= DCH / 2;
      lane_second[r] = second_half[r];
      const int p = (blk % (DCH / 2)) * 64 + lane;  // the lane's chunk within the half's region
      if (!is_v[r]) {
        const int kk = p / R, part = (p % R) ^ k_swizzle<R>(kk + (second_half[r] ? 16 : 0));
        lane_off[r] = kk * D + part * 8;
      } else {
        const int d = p / 2, sub = (p % 2) ^ ((d >> 3) & 1);
        lane_off[r] = d * page_size + sub * 8;
      }
    } else {
      second_half[r] = false;
      const int pg = (blk % DCH) * 64 + lane;       // the lane's chunk within the region of K or of V^T
      if (!is_v[r]) {
        // chunk pg of K's region: part pg / 32 of the key that row pg % 16 of product pg % 32 / 16 takes
        const int part = pg / 32, kp = pg % 32, cl = kp % 16;
        const int key = 8 * (cl / 4) + 4 * (kp / 16) + cl % 4;
        lane_second[r] = key >= 16;
        lane_off[r] = (key % 16) * D + part * 8;
      } else {
        const int p = pg % (32 * DCH);                // the chunk within its half's region
        const int d = p / 2, sub = (p % 2) ^ ((d >> 3) & 1);
        lane_second[r] = pg >= 32 * DCH;
        lane_off[r] = d * page_size + sub * 8;
      }
    }
  }
  // Tiles are fetched in order, so the page of the tile's first key is tracked by addition
  // instead of division: `tile_page` indexes the block table, `tile_off` is the key's offset in it.
  // Tiles start at multiples of 32 and pages hold a multiple of 16 keys, so each half of a tile
  // lies in one page: the two page numbers are the same for every lane and are read through the
  // scalar unit one tile ahead (`page_a`, `page_b`), which keeps the table lookup out of the
  // vector memory queue where it would wait behind the tiles in flight.
  int tile_page = begin / page_size, tile_off = begin % page_size;
  int page_a = 0, page_b = 0, off_a = 0, off_b = 0;
  // Table entries exist only for pages that hold keys: a tile past them reads the last one's.
  // No branch goes around the loads: a condition that outlives its block becomes a lane mask, and
  // what is computed from it (the second entry's index) went through the vector unit and back,
  // which cost 7% of the kernel's time at 8,192 tokens.
  const int last_page = max(n_keys - 1, 0) / page_size;
  auto lookup = [&]() {
    off_a = tile_off;
    const int second = tile_off + 16 >= page_size ? 1 : 0;
    off_b = tile_off + 16 - second * page_size;
    page_a = table[min(tile_page, last_page)];
    page_b = table[min(tile_page + second, last_page)];
    tile_off += 32;
    while (tile_off >= page_size) { tile_off -= page_size; ++tile_page; }
  };
  lookup();
  // Every fetch issues the same loads whatever the tile, also for tiles past the last one (their
  // halves read page 0 and are never used): the count of loads in flight is then known at compile
  // time and a tile is awaited without draining the younger ones behind it. Keys past the last one
  // of a half-filled page may hold anything: K rows there are masked as later than every query, V
  // columns are cleared in the fragments that a wave has read from LDS.
  // (Looking a tile's pages up earlier in the iteration, behind the first product, so that the
  // scalar load's answer arrives during the softmax, needs the lookup inside the branch that a wave
  // takes when it sees the tile: the compiler then keeps the pages in vector registers or, told
  // that the branch is uniform, copies the accumulators at its end: 393 -> 529 us at 8,192 tokens.)
  // Scalar arithmetic counts here: a wave issues it in turn with its vector instructions, and
  // all waves of a compute unit share one scalar unit. So a page's offset is one 32 x 32-bit
  // product onto the kv head's own base (the host checks that a page's elements fit 32 bits).
  const unsigned page_stride = (unsigned)kv_heads * (unsigned)page_size * (unsigned)D;
  const bf16_t* k_head = k_pages + (int64_t)kvh * page_size * D;
  const bf16_t* v_head = v_pages + (int64_t)kvh * page_size * D;
  auto fetch = [&](int buf) __attribute__((always_inline)) {  // the next tile in order
    const uint64_t at_a = (uint64_t)(unsigned)page_a * page_stride, at_b = (uint64_t)(unsigned)page_b * page_stride;
    const unsigned oa = off_a, ob = off_b;
    lookup();
#pragma unroll
    for (int r = 0; r < UCH; ++r) {
      // the same for every lane of the wave: a key's row of K is D long, a key's column of V^T one element
      const bf16_t* base;
      if constexpr (!ODD) {
        const unsigned off = second_half[r] ? ob : oa;
        base = (is_v[r] ? v_head : k_head) + (second_half[r] ? at_b : at_a) + (is_v[r] ? off : off * D);
      } else {  // both halves' places on the scalar unit, the lane takes its own
        const bf16_t* head_base = is_v[r] ? v_head : k_head;
        const bf16_t* base_a = head_base + at_a + (is_v[r] ? oa : oa * D);
        const bf16_t* base_b = head_base + at_b + (is_v[r] ? ob : ob * D);
        base = lane_second[r] ? base_b : base_a;
      }
      __builtin_amdgcn_global_load_lds(
          (const __attribute__((address_space(1))) void*)(base + lane_off[r]),
          (__attribute__((address_space(3))) void*)&lds[buf][block_at[r]], 16, 0, 0);
    }
  };

  // tiles 0..NB-2 set out for LDS; the loop needs the first of them there
#pragma unroll
  for (int T = 0; T < NB - 1; ++T) fetch(T);
  wait_loads<(NB - 2) * UCH>();
  tile_barrier();
  // A tile's work in two parts: `scores` reads the tile's fragments from LDS, makes S^T and the
  // softmax (vector unit, mostly); `values` makes P*V (matrix cores).
  // Where this lane's fragments lie in a tile. Which sixteen keys a product of S^T takes is free,
  // since every lane reads its own key's row: rows 4g..4g+3 of the first product are the keys
  // 8g..8g+3 and those of the second the keys 8g+4..8g+7, so that lane group g ends up with the
  // probabilities of the eight consecutive keys 8g..8g+7, whose values (dim row 16c+col) lie in
  // LDS as one chunk of 16 bytes.
  int k_at[2][DK];
  int k_tail_at[2];   // ODD: the lane's four dims of the last sixteen
  const int key_row = 8 * (col / 4) + col % 4;  // of the first product; the second's: four rows on
#pragma unroll
  for (int b = 0; b < 2; ++b) {
#pragma unroll
    for (int c = 0; c < DK; ++c) {
      if constexpr (!ODD)
        k_at[b][c] = (key_row + 4 * b) * D + ((c * 4 + grp) ^ k_swizzle<R>(key_row + 4 * b)) * 8;
      else
        k_at[b][c] = ((c * 4 + grp) * 32 + b * 16 + col) * 8;
    }
    k_tail_at[b] = ((4 * DK + (grp >> 1)) * 32 + b * 16 + col) * 8 + (grp & 1) * 4;
  }
  const int v_at = (grp >> 1) * VH_ELEMS + col * 16 + ((grp & 1) ^ (col >> 3)) * 8;
  // the tiles that the wave sees, [see_from, see_until], and among them those that need no mask,
  // [plain_until, plain_from] (tile starts; an empty range where there is no such tile)
  const bool has_rows = pos_hi >= pos_lo;
  const int see_until = has_rows ? pos_hi : -1;
  const int see_from = window > 0 ? pos_lo - window + 1 - 31 : 0;
  const int plain_from = pos_hi - pos_lo == 31 ? pos_lo - 31 : -1;
  const int plain_until = window > 0 ? pos_hi - window + 1 : 0;
  auto sees = [&](int it) __attribute__((always_inline)) {  // whether any of the wave's queries sees a key of the tile
    const int t = begin + it * 32;
    return t <= see_until && t >= see_from;
  };
  auto scores = [&](int it, bf16x8 (&vf)[DCH], bf16x8 (&pb)[2]) __attribute__((always_inline)) {
    const int t = begin + it * 32, buf = it % NB;
    {
      const bool need_mask = t > plain_from || t < plain_until;
      const bf16_t* ks = &lds[buf][0];
      const bf16_t* vs = &lds[buf][K_ELEMS];
      // all operand fragments of the tile are requested from LDS first, so that the reads of V
      // overlap the first product and the softmax
      bf16x8 kf0[DK], kf1[DK];
#pragma unroll
      for (int c = 0; c < DK; ++c) {
        kf0[c] = *reinterpret_cast<const bf16x8*>(ks + k_at[0][c]);
        kf1[c] = *reinterpret_cast<const bf16x8*>(ks + k_at[1][c]);
      }
      short4v kt0 = short4v{0, 0, 0, 0}, kt1 = short4v{0, 0, 0, 0};
      if constexpr (ODD) {
        kt0 = *reinterpret_cast<const short4v*>(ks + k_tail_at[0]);
        kt1 = *reinterpret_cast<const short4v*>(ks + k_tail_at[1]);
      }
#pragma unroll
      for (int c = 0; c < DCH; ++c) {
        vf[c] = *reinterpret_cast<const bf16x8*>(vs + c * 256 + v_at);
      }
      // S^T of both column tiles, for the two halves of the tile: keys t+4g+i and t+16+4g+i
      float4v sa[2], sb[2];
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        sa[j] = float4v{0.f, 0.f, 0.f, 0.f};
        sb[j] = float4v{0.f, 0.f, 0.f, 0.f};
      }
#pragma unroll
      for (int c = 0; c < DK; ++c)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          sa[j] = mfma32(kf0[c], qreg[j][c], sa[j]);
          sb[j] = mfma32(kf1[c], qreg[j][c], sb[j]);
        }
      if constexpr (ODD) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          sa[j] = mfma16(kt0, qtail[j], sa[j]);
          sb[j] = mfma16(kt1, qtail[j], sb[j]);
        }
      }
      float sv[2][8];
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          sv[j][i] = sa[j][i];
          sv[j][4 + i] = sb[j][i];
        }
      if (need_mask) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int low = window > 0 ? pos[j] - window + 1 : 0;
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            const int key = t + 8 * grp + i;
            if (key > pos[j] || key < low) sv[j][i] = -INFINITY;
          }
        }
      }
      // The reference point of the exponentials moves lazily: st[j].m is raised (and what has been
      // accumulated rescaled) only when a score of the tile exceeds it by more than 2^LAZY_LOG2,
      // which each lane can tell from its own eight scores. Most tiles then need neither the
      // maximum over the four lanes of a column nor the factor exp2(m_old - m_new); probabilities
      // lie below 2^LAZY_LOG2 instead of below one, which changes nothing in the quotient O / l
      // (32-bit sums, and bfloat16 keeps its eight bits at any magnitude).
      float lane_max[2];
      bool rise = false;
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        lane_max[j] = max3(max3(sv[j][0], sv[j][1], sv[j][2]), max3(sv[j][3], sv[j][4], sv[j][5]),
                           max2(sv[j][6], sv[j][7]));
        rise |= lane_max[j] > raise_at[j];
      }
      if (__builtin_amdgcn_ballot_w64(rise) != 0) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const float tile_max = column_max(lane_max[j]) * scale_log2e;  // the scale is positive
          const float m_new = max2(st[j].m, tile_max);
          const float m_safe = m_new == -INFINITY ? 0.f : m_new;
          const float alpha = fast_exp2(st[j].m - m_safe);  // 0 while nothing was seen, else at most 1
          st[j].l *= alpha;
#pragma unroll
          for (int c = 0; c < DCH; ++c) st[j].o[c] *= alpha;
          st[j].m = m_new;
          m_ref[j] = m_safe;
          raise_at[j] = m_new == -INFINITY ? -INFINITY : (m_new + LAZY_LOG2) * inv_scale_log2e;
        }
      }
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        // l stays a per-lane partial sum (the lanes of a column share m): the four partial sums of
        // a column are added once, after the last tile. (Taking the sum from the matrix cores
        // instead, as the product of P^T with a row of ones, saves sixteen additions a lane and
        // tile and was slower, 62 against 59 us; so was computing S^T of the next tile before the
        // softmax of this one inside a wave, 68 us.)
        float tile_sum = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float p = fast_exp2(fmaf(sv[j][i], scale_log2e, -m_ref[j]));
          tile_sum += p;
          pb[j][i] = (bf16_t)p;
        }
        st[j].l += tile_sum;
      }
      // keys past the request's last one (the rest of a half-filled page) may hold anything, also
      // what no product with zero clears
      if (t + 32 > n_keys) {
#pragma unroll
        for (int c = 0; c < DCH; ++c)
#pragma unroll
          for (int i = 0; i < 8; ++i)
            if (t + 8 * grp + i >= n_keys) vf[c][i] = (__bf16)0.f;
      }
    }
  };
  auto values = [&](bf16x8 (&vf)[DCH], bf16x8 (&pb)[2]) __attribute__((always_inline)) {
#pragma unroll
    for (int c = 0; c < DCH; ++c)
#pragma unroll
      for (int j = 0; j < 2; ++j) st[j].o[c] = mfma32(vf[c], pb[j], st[j].o[c]);
  };
  auto move_on = [&](int it) __attribute__((always_inline)) {
    // tile it+NB-1 sets out for the buffer that tile it-1 left at the last barrier; tile it+1 has
    // to be there before the next one
    fetch((it + NB - 1) % NB);
    wait_loads<(NB - 2) * UCH>();
  };
  // (Tried and 45% slower: S^T of tile it+1 sent to the matrix cores before the softmax of tile it.)
  for (int it0 = 0; it0 < n_tiles; it0 += NB) {
#pragma unroll
    for (int r = 0; r < NB; ++r) {
      const int it = it0 + r;
      if (it >= n_tiles) break;
      if (sees(it)) {
        bf16x8 vf[DCH];
        bf16x8 pb[2];
        scores(it, vf, pb);
        values(vf, pb);
      }
      move_on(it);
      tile_barrier();
    }
  }

  float l_sum[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) l_sum[j] = column_sum(st[j].l);  // every lane takes part
  if (cuts > 1) {
    // This run's state goes to memory at the device's scope: per wave and column tile DCH + 1
    // quads a lane (the output's, then the sum and the exponent's reference point). Then the
    // workgroup counts itself in; the one that counts last reads the other runs' states, adds all
    // of them up in the order of the runs (its own from its registers: the same values), and
    // leaves the counter zero for the next launch.
    constexpr int QUADS = DCH + 1;
    __shared__ unsigned arrived_before;
    const __amdgpu_buffer_rsrc_t cb = device_scope_buffer(cut_buf);
    const unsigned wg_quads = 8u * QUADS * 64u;   // 4 waves x 2 column tiles
    const unsigned tile_at = ((unsigned)cut_place * gridDim.y + (unsigned)by) * (unsigned)cut_room;
    auto at = [&](int run, int j, int quad) {
      return ((tile_at + (unsigned)run) * wg_quads + ((unsigned)(wave * 2 + j) * QUADS + (unsigned)quad) * 64u + (unsigned)lane) * 16u;
    };
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
      for (int c = 0; c < DCH; ++c) device_store4(cb, at(cut, j, c), st[j].o[c]);
      device_store4(cb, at(cut, j, DCH), float4v{l_sum[j], m_ref[j], 0.f, 0.f});
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);   // every store of this wave has been acknowledged
    __syncthreads();
    unsigned* counter = cut_count + (size_t)cut_place * gridDim.y + by;
    if (threadIdx.x == 0) arrived_before = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (arrived_before != (unsigned)cuts - 1) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    if (threadIdx.x == 0) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // the runs' sums and reference points first (all loads leave before the first is used) ...
    merge_float2 stat[2][PREFILL_MAX_CUTS];
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int run = 0; run < PREFILL_MAX_CUTS; ++run)
        stat[j][run] = run < cuts ? device_load2(cb, at(run, j, DCH)) : merge_float2{0.f, 0.f};
    float wgt[2][PREFILL_MAX_CUTS];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      // a run that saw no key of a query (sum 0) has no say in the reference point
      float m_all = -INFINITY;
#pragma unroll
      for (int run = 0; run < PREFILL_MAX_CUTS; ++run) m_all = max2(m_all, stat[j][run][0] > 0.f ? stat[j][run][1] : -INFINITY);
      const float m_safe = m_all == -INFINITY ? 0.f : m_all;
      float l_all = 0.f;
#pragma unroll
      for (int run = 0; run < PREFILL_MAX_CUTS; ++run) {
        wgt[j][run] = stat[j][run][0] > 0.f ? fast_exp2(stat[j][run][1] - m_safe) : 0.f;
        l_all = __fadd_rn(l_all, __fmul_rn(stat[j][run][0], wgt[j][run]));
      }
      l_sum[j] = l_all;
    }
    // ... then their outputs, run by run. Products and sums in the order of the runs and each
    // rounded by itself, so that the result does not depend on which of the workgroups does the
    // adding (left to itself the compiler fuses a product into the sum, and which one depends on
    // whose values sit in registers).
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      float4v acc[DCH];
#pragma unroll
      for (int c = 0; c < DCH; ++c) acc[c] = float4v{0.f, 0.f, 0.f, 0.f};
      for (int run = 0; run < cuts; ++run) {
        float4v o_run[DCH];
#pragma unroll
        for (int c = 0; c < DCH; ++c) o_run[c] = device_load4(cb, at(run, j, c));
        float w = 0.f;
#pragma unroll
        for (int u = 0; u < PREFILL_MAX_CUTS; ++u) w = u == run ? wgt[j][u] : w;
#pragma unroll
        for (int c = 0; c < DCH; ++c)
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[c][i] = __fadd_rn(acc[c][i], __fmul_rn(o_run[c][i], w));
      }
#pragma unroll
      for (int c = 0; c < DCH; ++c) st[j].o[c] = acc[c];
    }
  }
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int qi = q0 + j * 16 + col;
    if (qi >= q_len) continue;
    const float inv = l_sum[j] > 0.f ? 1.f / l_sum[j] : 0.f;
    bf16_t* op = out + (int64_t)(tok0 + qi) * out_stride + (int64_t)head * D + 4 * grp;
#pragma unroll
    for (int c = 0; c < DCH; ++c) {
      const short4v packed = {bf16_bits(st[j].o[c][0] * inv), bf16_bits(st[j].o[c][1] * inv),
                              bf16_bits(st[j].o[c][2] * inv), bf16_bits(st[j].o[c][3] * inv)};
      *reinterpret_cast<short4v*>(op + c * 16) = packed;
    }
  }
}

// ------------------------------------------------------------------------------------ host side
#define LOG2E 1.4426950408889634f

extern "C" int dli_attention_mfma_supports(int head_dim, int page_size) {
  return head_dim > 0 && head_dim % 16 == 0 && head_dim <= 128 && page_size > 0 && page_size % 16 == 0;
}

// Query heads that one workgroup of the shared-tile kernel takes (4, 2 or 1), or 0 if the shape
// has to take the plain kernel (heads of 16).
static int shared_heads_per_wg(int head_dim, int group) {
  if (head_dim % 16 != 0 || head_dim < 32) return 0;
  return group % 4 == 0 ? 4 : (group % 2 == 0 ? 2 : 1);
}

// Queries per tile of the tile list that dli_attention_prefill_bf16 expects for this shape.
extern "C" int dli_attention_prefill_tile_rows(int head_dim, int q_heads, int kv_heads) {
  if (kv_heads <= 0 || q_heads % kv_heads != 0) return DLI_ERR_ARGUMENT;
  const int hw = shared_heads_per_wg(head_dim, q_heads / kv_heads);
  return hw == 0 ? PF_TILE_ROWS : (4 / hw) * 32;
}

// merge: whether the partial results of more than one run of keys are merged into `out` here, or
// left in part_o / part_ml for the kernel that reads them next.
static int attention_decode(const void* q, int64_t q_stride, const void* k_pages, const void* v_pages,
                            void* out, int64_t out_stride, float* part_o, float* part_ml,
                            const int* kv_len, const int* block_tables, int table_stride, int requests,
                            int q_heads, int kv_heads, int head_dim, int page_size, float scale,
                            int window, int splits, bool merge, unsigned* arrivals, hipStream_t stream) {
  if (requests <= 0) return DLI_OK;
  if (!dli_attention_mfma_supports(head_dim, page_size) || q_heads <= 0 || kv_heads <= 0 ||
      q_heads % kv_heads != 0 || splits < 1 || splits > 65535 || requests > 65535 ||
      (splits > 1 && (part_o == nullptr || part_ml == nullptr)) || q_stride % 4 != 0 ||
      out_stride % 4 != 0)
    return DLI_ERR_ARGUMENT;
  const int head_tiles = (q_heads / kv_heads + 15) / 16;
  const dim3 grid(splits, kv_heads * head_tiles, requests);
  // with counters the last workgroup of each (request, kv head, head tile) merges
  const bool self_merging = merge && arrivals != nullptr && splits >= 2 && splits <= MERGE_SPLITS;
  unsigned* counters = self_merging ? arrivals : nullptr;
#define DECODE_CASE(N)                                                                            \
  case N:                                                                                         \
    attention_decode_kernel<N><<<grid, 256, 0, stream>>>(                                         \
        (const bf16_t*)q, q_stride, (const bf16_t*)k_pages, (const bf16_t*)v_pages, (bf16_t*)out, \
        out_stride, part_o, part_ml, kv_len, block_tables, table_stride, q_heads, kv_heads,       \
        page_size, scale * LOG2E, window, splits, counters);                                      \
    break;
  switch (head_dim / 16) {
    DECODE_CASE(1) DECODE_CASE(2) DECODE_CASE(3) DECODE_CASE(4)
    DECODE_CASE(5) DECODE_CASE(6) DECODE_CASE(7) DECODE_CASE(8)
    default: return DLI_ERR_ARGUMENT;
  }
#undef DECODE_CASE
  if (dli_launch_status() != DLI_OK) return DLI_ERR_LAUNCH;
  if (splits > 1 && merge && !self_merging) {
    const int pairs = requests * q_heads;
#define MERGE(S, V)                                                             \
  attention_merge_kernel<S, V><<<(pairs + 3) / 4, 256, 0, stream>>>(part_o, part_ml, (bf16_t*)out, \
                                                                    out_stride, q_heads, head_dim, splits, pairs)
    if (head_dim <= 64) {
      if (splits <= 8) MERGE(8, 1);
      else if (splits <= 16) MERGE(16, 1);
      else MERGE(32, 1);
    } else {
      if (splits <= 8) MERGE(8, 2);
      else MERGE(16, 2);
    }
#undef MERGE
  }
  return dli_launch_status();
}

extern "C" int dli_attention_decode_bf16(const void* q, int64_t q_stride, const void* k_pages,
                                         const void* v_pages, void* out, int64_t out_stride,
                                         float* part_o, float* part_ml, const int* kv_len,
                                         const int* block_tables, int table_stride, int requests,
                                         int q_heads, int kv_heads, int head_dim, int page_size,
                                         float scale, int window, int splits, hipStream_t stream) {
  return attention_decode(q, q_stride, k_pages, v_pages, out, out_stride, part_o, part_ml, kv_len, block_tables,
                          table_stride, requests, q_heads, kv_heads, head_dim, page_size, scale, window, splits,
                          true, nullptr, stream);
}

// The same, and the launch merges by itself where it can (2 to 16 runs of keys): the workgroup
// that finishes last of those that share a request and kv head does what the merge kernel would,
// to the bit. arrivals: requests * kv_heads * ceil(group / 16) counters that are zero before the
// first call and that every call leaves zero; launches that share them must not overlap.
extern "C" int dli_attention_decode_self_merging_bf16(const void* q, int64_t q_stride, const void* k_pages,
                                                      const void* v_pages, void* out, int64_t out_stride,
                                                      float* part_o, float* part_ml, unsigned* arrivals,
                                                      const int* kv_len, const int* block_tables,
                                                      int table_stride, int requests, int q_heads,
                                                      int kv_heads, int head_dim, int page_size, float scale,
                                                      int window, int splits, hipStream_t stream) {
  if (arrivals == nullptr) return DLI_ERR_ARGUMENT;
  return attention_decode(q, q_stride, k_pages, v_pages, out, out_stride, part_o, part_ml, kv_len, block_tables,
                          table_stride, requests, q_heads, kv_heads, head_dim, page_size, scale, window, splits,
                          true, arrivals, stream);
}

// The same without the merge: with two or more runs of keys the partial results stay in part_o
// [requests][q_heads][splits][head_dim] and part_ml [requests][q_heads][splits][2] and `out` is not
// written (dli_skinny_gemm_merged reads them).
extern "C" int dli_attention_decode_partial_bf16(const void* q, int64_t q_stride, const void* k_pages,
                                                 const void* v_pages, float* part_o, float* part_ml,
                                                 const int* kv_len, const int* block_tables,
                                                 int table_stride, int requests, int q_heads, int kv_heads,
                                                 int head_dim, int page_size, float scale, int window,
                                                 int splits, hipStream_t stream) {
  if (splits < 2) return DLI_ERR_ARGUMENT;
  return attention_decode(q, q_stride, k_pages, v_pages, nullptr, 0, part_o, part_ml, kv_len, block_tables,
                          table_stride, requests, q_heads, kv_heads, head_dim, page_size, scale, window, splits,
                          false, nullptr, stream);
}

// ---------------------------------------------------------------- decode without an allocation
// The split-key partial results of dli_attention_decode_bf16_static live in this array instead
// of a buffer that the caller brings. Each GPU holds its own copy at its own address; host code
// never uses the array's name as an address, only what hipGetSymbolAddress returned for the
// current device.
static __device__ __align__(256) float scratch[DLI_STATIC_SCRATCH_FLOATS];

// The array's address on the current device (asked once per device), or nullptr.
static float* static_scratch() {
  static float* of_device[64] = {nullptr};
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
  if (of_device[dev] == nullptr) {
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || ptr == nullptr) return nullptr;
    of_device[dev] = static_cast<float*>(ptr);
  }
  return of_device[dev];
}

extern "C" int64_t dli_attention_decode_static_floats(int requests, int q_heads, int head_dim, int splits) {
  if (requests <= 0 || q_heads <= 0 || head_dim <= 0 || splits <= 1) return 0;
  const int64_t slots = (int64_t)requests * q_heads * splits;
  return (slots * head_dim + 63) / 64 * 64 + slots * 2;
}

extern "C" int dli_attention_decode_bf16_static(const void* q, int64_t q_stride, const void* k_pages,
                                                const void* v_pages, void* out, int64_t out_stride,
                                                const int* kv_len, const int* block_tables,
                                                int table_stride, int requests, int q_heads,
                                                int kv_heads, int head_dim, int page_size, float scale,
                                                int window, int splits, hipStream_t stream) {
  if (requests <= 0) return DLI_OK;
  if (q_heads <= 0 || head_dim <= 0 || splits < 1) return DLI_ERR_ARGUMENT;
  float* part_o = nullptr;
  float* part_ml = nullptr;
  if (splits > 1) {
    if (dli_attention_decode_static_floats(requests, q_heads, head_dim, splits) > DLI_STATIC_SCRATCH_FLOATS)
      return DLI_ERR_SCRATCH;
    float* base = static_scratch();
    if (base == nullptr) return DLI_ERR_LAUNCH;
    const int64_t slots = (int64_t)requests * q_heads * splits;
    part_o = base;
    part_ml = base + (slots * head_dim + 63) / 64 * 64;
  }
  // Nothing has to start at zero: every (request, head, split) writes its partial result and its
  // statistics before the merge reads them.
  return dli_attention_decode_bf16(q, q_stride, k_pages, v_pages, out, out_stride, part_o, part_ml, kv_len,
                                   block_tables, table_stride, requests, q_heads, kv_heads, head_dim, page_size,
                                   scale, window, splits, stream);
}

// 32-bit values that the kernel wants per run of a tile whose keys are cut into runs (the state
// of every workgroup of the tile), or 0 where this shape's kernel cuts no tiles.
extern "C" int dli_attention_prefill_cut_floats(int head_dim, int q_heads, int kv_heads) {
  if (kv_heads <= 0 || q_heads % kv_heads != 0 || q_heads > 65535 || head_dim > 128) return DLI_ERR_ARGUMENT;
  const int hw = shared_heads_per_wg(head_dim, q_heads / kv_heads);
  if (hw == 0) return 0;
  return (q_heads / hw) * 8 * (head_dim / 16 + 1) * 64 * 4;
}

// The most runs that a tile's keys can be cut into.
extern "C" int dli_attention_prefill_max_cuts() { return PREFILL_MAX_CUTS; }

// tile_cut (or null: every tile whole): per entry of the tile list -1, or run | runs << 4 |
// place << 8 for one of the 2 to dli_attention_prefill_max_cuts() runs of a tile whose keys that
// many workgroups share, `place` numbering the cut tiles from 0 to cut_tiles - 1; all runs of a
// tile must be listed. Only without a window and for heads of 32 and more.
// cut_room: the most runs of any tile; cut_buf: cut_tiles * cut_room *
// dli_attention_prefill_cut_floats() values; cut_count: one counter per cut tile and workgroup of
// a tile (cut_tiles * q_heads is enough), zero before the first launch; every launch leaves them
// zero, and launches that share them or cut_buf must not overlap.
extern "C" int dli_attention_prefill_bf16(const void* q, int64_t q_stride, const void* k_pages,
                                          const void* v_pages, void* out, int64_t out_stride,
                                          const int* q_start, const int* kv_len,
                                          const int* block_tables, int table_stride,
                                          const int* tile_entry, const int* tile_q0, int tiles,
                                          int q_heads, int kv_heads, int head_dim, int page_size,
                                          float scale, int window, const int* tile_cut, int cut_tiles,
                                          int cut_room, float* cut_buf, unsigned* cut_count, hipStream_t stream) {
  if (tiles <= 0) return DLI_OK;
  if (!dli_attention_mfma_supports(head_dim, page_size) || q_heads <= 0 || kv_heads <= 0 ||
      q_heads % kv_heads != 0 || q_heads > 65535 || q_stride % 4 != 0 || out_stride % 4 != 0)
    return DLI_ERR_ARGUMENT;
  const int hw = shared_heads_per_wg(head_dim, q_heads / kv_heads);
  if (tile_cut != nullptr &&
      (hw == 0 || window > 0 || cut_tiles <= 0 || cut_tiles >= (1 << 23) || cut_room < 2 || cut_room > PREFILL_MAX_CUTS ||
       cut_buf == nullptr || cut_count == nullptr ||
       (int64_t)cut_tiles * cut_room * dli_attention_prefill_cut_floats(head_dim, q_heads, kv_heads) * 4 >= ((int64_t)1 << 32)))
    return DLI_ERR_ARGUMENT;
  if (hw > 0) {
    if ((int64_t)kv_heads * page_size * head_dim >= ((int64_t)1 << 31)) return DLI_ERR_ARGUMENT;  // the kernel's 32 bits
    const dim3 sgrid(tiles, q_heads / hw);
#define SHARED_CASE(N)                                                                            \
  case N:                                                                                         \
    attention_prefill_shared_kernel<N><<<sgrid, 256, 0, stream>>>(                                \
        (const bf16_t*)q, q_stride, (const bf16_t*)k_pages, (const bf16_t*)v_pages, (bf16_t*)out, \
        out_stride, q_start, kv_len, block_tables, table_stride, tile_entry, tile_q0, q_heads,    \
        kv_heads, page_size, scale * LOG2E, window, hw, tile_cut, cut_room, cut_buf, cut_count);  \
    break;
    switch (head_dim / 16) {
      SHARED_CASE(2) SHARED_CASE(3) SHARED_CASE(4) SHARED_CASE(5) SHARED_CASE(6) SHARED_CASE(7) SHARED_CASE(8)
      default: return DLI_ERR_ARGUMENT;
    }
#undef SHARED_CASE
    return dli_launch_status();
  }
  const dim3 grid(tiles, q_heads);
#define PREFILL_CASE(N)                                                                           \
  case N:                                                                                         \
    attention_prefill_kernel<N><<<grid, 256, 0, stream>>>(                                        \
        (const bf16_t*)q, q_stride, (const bf16_t*)k_pages, (const bf16_t*)v_pages, (bf16_t*)out, \
        out_stride, q_start, kv_len, block_tables, table_stride, tile_entry, tile_q0, q_heads,    \
        kv_heads, page_size, scale * LOG2E, window);                                              \
    break;
  switch (head_dim / 16) {
    PREFILL_CASE(1) PREFILL_CASE(2) PREFILL_CASE(3) PREFILL_CASE(4)
    PREFILL_CASE(5) PREFILL_CASE(6) PREFILL_CASE(7) PREFILL_CASE(8)
    default: return DLI_ERR_ARGUMENT;
  }
#undef PREFILL_CASE
  return dli_launch_status();
}
