// Rotary position encoding of q and k, fused with the write of k and v into cache pages.
//
// Input rows are the fused projection [tokens, (q_heads + 2*kv_heads) * head_dim]: q heads, then
// k heads, then v heads. q is rotated in place; rotated k and raw v go to the pages:
//   K page: [kv_heads][page_size][head_dim]   (a key's head_dim values are contiguous)
//   V page: [kv_heads][head_dim][page_size]   (one dimension of page_size keys is contiguous,
//                                               which is the operand order of the P*V product)
// Rotation (reference: src/dli/model/rope.py:50-70): angle = float(pos) * inv_freq[i] in 32-bit,
// cos/sin rounded to the activation type, dimension i pairs with i + rotary_dim/2:
//   y[i] = x[i]*cos - x[i+h]*sin ;  y[i+h] = x[i+h]*cos + x[i]*sin.
// Dimensions at and beyond rotary_dim pass through. inv_freq == nullptr means no rotation.
#include "common.h"

// One workgroup per token: cos/sin of the token's angles are computed once into LDS, then the
// threads walk the token's q heads (rotated in place), k heads (rotated into the page) and v heads
// (copied into the transposed page).
#define ROPE_MAX_HALF 128
template <typename T>
__global__ __launch_bounds__(256) void rope_kv_write_kernel(
    T* __restrict__ qkv, int64_t row_stride, const int* __restrict__ positions,
    const float* __restrict__ inv_freq, int rotary_dim, const int* __restrict__ slots,
    T* __restrict__ k_pages, T* __restrict__ v_pages, int q_heads, int kv_heads, int head_dim,
    int page_size) {
  __shared__ float cs[ROPE_MAX_HALF], sn[ROPE_MAX_HALF];
  const int64_t token = blockIdx.x;
  T* row = qkv + token * row_stride;
  const int slot = slots != nullptr ? slots[token] : -1;
  const int64_t page = slot >= 0 ? slot / page_size : 0;
  const int off = slot >= 0 ? slot % page_size : 0;
  const int half = rotary_dim / 2;
  const float pos = (float)positions[token];
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    float c = 1.f, s = 0.f;
    if (inv_freq != nullptr) {
      sincosf(pos * inv_freq[i], &s, &c);
      c = round_to<T>(c);
      s = round_to<T>(s);
    }
    cs[i] = c;
    sn[i] = s;
  }
  __syncthreads();
  const bool cache = slot >= 0 && k_pages != nullptr && v_pages != nullptr;

  // q and k heads: pairs (i, i + half) of the rotary part
  const int rot_heads = q_heads + kv_heads;
  if (half > 0) {
    for (int idx = threadIdx.x; idx < rot_heads * half; idx += blockDim.x) {
      const int head = idx / half, i = idx - head * half;
      T* h = row + (int64_t)head * head_dim;
      const float x1 = to_f32(h[i]), x2 = to_f32(h[i + half]);
      const T y1 = from_f32<T>(x1 * cs[i] - x2 * sn[i]);
      const T y2 = from_f32<T>(x2 * cs[i] + x1 * sn[i]);
      if (head < q_heads) {
        h[i] = y1;
        h[i + half] = y2;
      } else if (cache) {
        T* kd = k_pages + ((page * kv_heads + (head - q_heads)) * page_size + off) * head_dim;
        kd[i] = y1;
        kd[i + half] = y2;
      }
    }
  }
  if (!cache) return;
  // the part of k beyond the rotary dimensions passes through
  const int rest = head_dim - rotary_dim;
  for (int idx = threadIdx.x; idx < kv_heads * rest; idx += blockDim.x) {
    const int h = idx / rest, i = rotary_dim + idx - h * rest;
    k_pages[((page * kv_heads + h) * page_size + off) * head_dim + i] = row[(int64_t)(q_heads + h) * head_dim + i];
  }
  // v heads into the transposed page
  const T* v = row + (int64_t)(q_heads + kv_heads) * head_dim;
  for (int idx = threadIdx.x; idx < kv_heads * head_dim; idx += blockDim.x) {
    const int h = idx / head_dim, i = idx - h * head_dim;
    v_pages[((page * kv_heads + h) * head_dim + i) * page_size + off] = v[idx];
  }
}

extern "C" int dli_rope_kv_write(void* qkv, int64_t row_stride, const int* positions,
                                 const float* inv_freq, int rotary_dim, const int* slots,
                                 void* k_pages, void* v_pages, int tokens, int q_heads, int kv_heads,
                                 int head_dim, int page_size, int is_bf16, hipStream_t stream) {
  if (tokens <= 0) return DLI_OK;
  if (head_dim <= 0 || rotary_dim < 0 || rotary_dim > head_dim || rotary_dim % 2 != 0 ||
      rotary_dim / 2 > ROPE_MAX_HALF || q_heads < 0 || kv_heads < 0 || page_size <= 0 ||
      q_heads + 2 * kv_heads <= 0)
    return DLI_ERR_ARGUMENT;
  if (is_bf16)
    rope_kv_write_kernel<bf16_t><<<tokens, 256, 0, stream>>>(
        (bf16_t*)qkv, row_stride, positions, inv_freq, rotary_dim, slots, (bf16_t*)k_pages,
        (bf16_t*)v_pages, q_heads, kv_heads, head_dim, page_size);
  else
    rope_kv_write_kernel<float><<<tokens, 256, 0, stream>>>(
        (float*)qkv, row_stride, positions, inv_freq, rotary_dim, slots, (float*)k_pages,
        (float*)v_pages, q_heads, kv_heads, head_dim, page_size);
  return dli_launch_status();
}
