// The merge of the partial results that decode attention leaves when a request's keys are cut into
// runs: out = sum_s o_s 2^(m_s - M) / sum_s l_s 2^(m_s - M) with M = max_s m_s, for four
// consecutive dims of one (request, head). Used by the kernels that merge on their own way (the
// o projection of very few rows, the last workgroup of a decode attention launch); sums in the
// order of attention_merge_kernel, so that all three give the same bits: the denominators pairwise
// as its butterfly adds them (lanes 8 apart, then 4, 2, 1), the outputs run by run.
#pragma once
#include "common.h"

#define MERGE_SPLITS 16  // the most runs of keys that merged_quad takes

typedef float merge_float2 __attribute__((ext_vector_type(2)));
typedef float merge_float4 __attribute__((ext_vector_type(4)));

// What one workgroup of a launch hands to another goes through memory at the device's scope, past
// the caches that are private to a part of the chip: buffer loads and stores with the sc1 bit
// (bit 4 of the builtins' cache policy on gfx940 and later), 8 or 16 bytes a lane. The resource
// spans the whole address range behind the pointer (offsets are 32-bit byte offsets).
typedef unsigned merge_u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned merge_u32x2 __attribute__((ext_vector_type(2)));
constexpr int DEVICE_SCOPE = 1 << 4;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t device_scope_buffer(const void* p) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, 0xffffffffu, 0x00020000);
}
__device__ __forceinline__ merge_float4 device_load4(__amdgpu_buffer_rsrc_t r, unsigned byte_offset) {
  union {
    merge_u32x4 raw;
    merge_float4 f;
  } u;
  u.raw = __builtin_amdgcn_raw_buffer_load_b128(r, (int)byte_offset, 0, DEVICE_SCOPE);
  return u.f;
}
__device__ __forceinline__ merge_float2 device_load2(__amdgpu_buffer_rsrc_t r, unsigned byte_offset) {
  union {
    merge_u32x2 raw;
    merge_float2 f;
  } u;
  u.raw = __builtin_amdgcn_raw_buffer_load_b64(r, (int)byte_offset, 0, DEVICE_SCOPE);
  return u.f;
}
__device__ __forceinline__ void device_store4(__amdgpu_buffer_rsrc_t r, unsigned byte_offset, merge_float4 v) {
  union {
    merge_u32x4 raw;
    merge_float4 f;
  } u;
  u.f = v;
  __builtin_amdgcn_raw_buffer_store_b128(u.raw, r, (int)byte_offset, 0, DEVICE_SCOPE);
}
__device__ __forceinline__ void device_store2(__amdgpu_buffer_rsrc_t r, unsigned byte_offset, merge_float2 v) {
  union {
    merge_u32x2 raw;
    merge_float2 f;
  } u;
  u.f = v;
  __builtin_amdgcn_raw_buffer_store_b64(u.raw, r, (int)byte_offset, 0, DEVICE_SCOPE);
}

// part_o [.. slots][head_dim], part_ml [.. slots][2]; `base`: the first of the S slots of this
// (request, head); d: the first of the four dims. All loads are asked for before the first is used.
// SAME_LAUNCH: the partial results were stored by other workgroups of this launch (each array
// under 4 GB).
template <bool SAME_LAUNCH = false>
__device__ __forceinline__ merge_float4 merged_quad(const float* part_o, const float* part_ml, int64_t base, int S,
                                                    int head_dim, int d) {
  merge_float2 ml[MERGE_SPLITS];
  merge_float4 po[MERGE_SPLITS];
#pragma unroll
  for (int j = 0; j < MERGE_SPLITS; ++j) {
    ml[j] = merge_float2{-INFINITY, 0.f};
    po[j] = merge_float4{0.f, 0.f, 0.f, 0.f};
    if (j < S) {
      const float* ml_at = part_ml + (base + j) * 2;
      const float* po_at = part_o + (base + j) * head_dim + d;
      if constexpr (SAME_LAUNCH) {
        ml[j] = device_load2(device_scope_buffer(part_ml), (unsigned)((base + j) * 2 * 4));
        po[j] = device_load4(device_scope_buffer(part_o), (unsigned)(((base + j) * head_dim + d) * 4));
      } else {
        ml[j] = *reinterpret_cast<const merge_float2*>(ml_at);
        po[j] = *reinterpret_cast<const merge_float4*>(po_at);
      }
    }
  }
  float m_all = -INFINITY;
#pragma unroll
  for (int j = 0; j < MERGE_SPLITS; ++j) m_all = fmaxf(m_all, ml[j][0]);
  const float m_safe = m_all == -INFINITY ? 0.f : m_all;
  float wgt[MERGE_SPLITS], t[MERGE_SPLITS];
#pragma unroll
  for (int j = 0; j < MERGE_SPLITS; ++j) {
    wgt[j] = j < S ? __builtin_amdgcn_exp2f(ml[j][0] - m_safe) : 0.f;
    t[j] = __fmul_rn(ml[j][1], wgt[j]);
  }
#pragma unroll
  for (int h = MERGE_SPLITS / 2; h > 0; h >>= 1)
#pragma unroll
    for (int j = 0; j < h; ++j) t[j] = __fadd_rn(t[j], t[j + h]);
  const float inv = t[0] > 0.f ? 1.f / t[0] : 0.f;
  merge_float4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < MERGE_SPLITS; ++j)
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = __fmaf_rn(po[j][i], wgt[j], acc[i]);
#pragma unroll
  for (int i = 0; i < 4; ++i) acc[i] = __fmul_rn(acc[i], inv);
  return acc;
}
