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

template <typename T>
__global__ void rope_kv_write_kernel(T* __restrict__ qkv, int64_t row_stride,
                                     const int* __restrict__ positions,
                                     const float* __restrict__ inv_freq, int rotary_dim,
                                     const int* __restrict__ slots, T* __restrict__ k_pages,
                                     T* __restrict__ v_pages, int q_heads, int kv_heads, int head_dim,
                                     int page_size) {
  const int64_t token = blockIdx.x;
  const int head = blockIdx.y;  // [0,q_heads): q; then k heads; then v heads
  T* row = qkv + token * row_stride + (int64_t)head * head_dim;
  const int slot = slots != nullptr ? slots[token] : -1;
  const int64_t page = slot >= 0 ? slot / page_size : 0;
  const int off = slot >= 0 ? slot % page_size : 0;

  if (head >= q_heads + kv_heads) {  // v head: copy to its transposed page
    if (slot < 0 || v_pages == nullptr) return;
    const int h = head - q_heads - kv_heads;
    T* dst = v_pages + ((page * kv_heads + h) * head_dim) * page_size + off;
    for (int i = threadIdx.x; i < head_dim; i += blockDim.x) dst[(int64_t)i * page_size] = row[i];
    return;
  }

  const bool is_k = head >= q_heads;
  T* kdst = nullptr;
  if (is_k) {
    if (slot >= 0 && k_pages != nullptr)
      kdst = k_pages + ((page * kv_heads + (head - q_heads)) * page_size + off) * head_dim;
  }
  const int half = rotary_dim / 2;
  const float pos = (float)positions[token];
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    float c = 1.f, s = 0.f;
    if (inv_freq != nullptr) {
      const float angle = pos * inv_freq[i];
      sincosf(angle, &s, &c);
      c = round_to<T>(c);
      s = round_to<T>(s);
    }
    const float x1 = to_f32(row[i]), x2 = to_f32(row[i + half]);
    const T y1 = from_f32<T>(x1 * c - x2 * s);
    const T y2 = from_f32<T>(x2 * c + x1 * s);
    if (is_k) {
      if (kdst != nullptr) { kdst[i] = y1; kdst[i + half] = y2; }
    } else {
      row[i] = y1;
      row[i + half] = y2;
    }
  }
  if (is_k && kdst != nullptr)
    for (int i = rotary_dim + threadIdx.x; i < head_dim; i += blockDim.x) kdst[i] = row[i];
}

extern "C" int dli_rope_kv_write(void* qkv, int64_t row_stride, const int* positions,
                                 const float* inv_freq, int rotary_dim, const int* slots,
                                 void* k_pages, void* v_pages, int tokens, int q_heads, int kv_heads,
                                 int head_dim, int page_size, int is_bf16, hipStream_t stream) {
  if (tokens <= 0) return DLI_OK;
  if (head_dim <= 0 || rotary_dim < 0 || rotary_dim > head_dim || rotary_dim % 2 != 0 || q_heads < 0 ||
      kv_heads < 0 || page_size <= 0 || q_heads + 2 * kv_heads <= 0)
    return DLI_ERR_ARGUMENT;
  const dim3 grid(tokens, q_heads + 2 * kv_heads);
  const int threads = head_dim / 2 > 64 ? 128 : 64;
  if (is_bf16)
    rope_kv_write_kernel<bf16_t><<<grid, threads, 0, stream>>>(
        (bf16_t*)qkv, row_stride, positions, inv_freq, rotary_dim, slots, (bf16_t*)k_pages,
        (bf16_t*)v_pages, q_heads, kv_heads, head_dim, page_size);
  else
    rope_kv_write_kernel<float><<<grid, threads, 0, stream>>>(
        (float*)qkv, row_stride, positions, inv_freq, rotary_dim, slots, (float*)k_pages,
        (float*)v_pages, q_heads, kv_heads, head_dim, page_size);
  return dli_launch_status();
}
