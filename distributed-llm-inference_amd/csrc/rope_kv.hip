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

// Few tokens (decode): a token's work is a list of items, the rotary pairs of its q and k heads,
// the dimensions of k beyond the rotary part, and the values of v. Workgroup y of a token takes
// the items y*256 + t, (y + gridDim.y)*256 + t, ...; there are as many workgroups per token as it
// takes to give each thread one item. A thread asks for the operands of its first item before the
// angles are computed (every workgroup its own copy in LDS): what it reads does not wait for
// them, and the kernel is one trip to memory long.
#define ROPE_MAX_HALF 128
template <typename T>
struct RopeItem {
  int kind, head, i;  // kind: 0 pair, 1 rest of k, 2 v, 3 nothing
  float x1, x2;
};

template <typename T>
__device__ __forceinline__ RopeItem<T> rope_fetch(const T* __restrict__ row, int item, int half,
                                                  int rest, int rotary_dim, int q_heads, int kv_heads,
                                                  int head_dim) {
  const int n_pairs = (q_heads + kv_heads) * half, n_rest = kv_heads * rest, n_v = kv_heads * head_dim;
  RopeItem<T> it{3, 0, 0, 0.f, 0.f};
  if (item < n_pairs) {
    it.kind = 0;
    it.head = item / half;
    it.i = item - it.head * half;
    const T* h = row + (int64_t)it.head * head_dim;
    it.x1 = to_f32(h[it.i]);
    it.x2 = to_f32(h[it.i + half]);
  } else if (item < n_pairs + n_rest) {
    it.kind = 1;
    it.head = (item - n_pairs) / rest;
    it.i = rotary_dim + (item - n_pairs) - it.head * rest;
    it.x1 = to_f32(row[(int64_t)(q_heads + it.head) * head_dim + it.i]);
  } else if (item < n_pairs + n_rest + n_v) {
    it.kind = 2;
    it.head = (item - n_pairs - n_rest) / head_dim;
    it.i = (item - n_pairs - n_rest) - it.head * head_dim;
    it.x1 = to_f32(row[(int64_t)(q_heads + kv_heads + it.head) * head_dim + it.i]);
  }
  return it;
}

template <typename T>
__global__ __launch_bounds__(256) void rope_kv_write_kernel(
    T* __restrict__ qkv, int64_t row_stride, const int* __restrict__ positions,
    const float* __restrict__ inv_freq, int rotary_dim, const int* __restrict__ slots,
    T* __restrict__ k_pages, T* __restrict__ v_pages, int q_heads, int kv_heads, int head_dim,
    int page_size, int items) {
  __shared__ float cs[ROPE_MAX_HALF], sn[ROPE_MAX_HALF];
  const int64_t token = blockIdx.x;
  T* row = qkv + token * row_stride;
  const int half = rotary_dim / 2, rest = head_dim - rotary_dim;
  int item = blockIdx.y * 256 + threadIdx.x;
  RopeItem<T> it = rope_fetch<T>(row, item, half, rest, rotary_dim, q_heads, kv_heads, head_dim);
  const int slot = slots != nullptr ? slots[token] : -1;
  const float pos = (float)positions[token];
  if (threadIdx.x < half) {
    float c = 1.f, sv = 0.f;
    if (inv_freq != nullptr) {
      sincosf(pos * inv_freq[threadIdx.x], &sv, &c);
      c = round_to<T>(c);
      sv = round_to<T>(sv);
    }
    cs[threadIdx.x] = c;
    sn[threadIdx.x] = sv;
  }
  __syncthreads();
  const bool cache = slot >= 0 && k_pages != nullptr && v_pages != nullptr;
  const int64_t page = slot >= 0 ? slot / page_size : 0;
  const int off = slot >= 0 ? slot % page_size : 0;
  while (true) {
    if (it.kind == 0) {
      const T y1 = from_f32<T>(it.x1 * cs[it.i] - it.x2 * sn[it.i]);
      const T y2 = from_f32<T>(it.x2 * cs[it.i] + it.x1 * sn[it.i]);
      if (it.head < q_heads) {
        T* h = row + (int64_t)it.head * head_dim;
        h[it.i] = y1;
        h[it.i + half] = y2;
      } else if (cache) {
        T* kd = k_pages + ((page * kv_heads + (it.head - q_heads)) * page_size + off) * head_dim;
        kd[it.i] = y1;
        kd[it.i + half] = y2;
      }
    } else if (it.kind == 1) {
      if (cache) k_pages[((page * kv_heads + it.head) * page_size + off) * head_dim + it.i] = from_f32<T>(it.x1);
    } else if (it.kind == 2) {
      if (cache) v_pages[((page * kv_heads + it.head) * head_dim + it.i) * page_size + off] = from_f32<T>(it.x1);
    }
    item += gridDim.y * 256;
    if (item >= items) break;
    it = rope_fetch<T>(row, item, half, rest, rotary_dim, q_heads, kv_heads, head_dim);
  }
}

// Many tokens (prompts): one workgroup per token. cos/sin of the token's angles are computed once
// into LDS, then the threads walk the token's q heads (rotated in place), k heads (rotated into
// the page) and v heads (copied into the transposed page).
template <typename T>
__global__ __launch_bounds__(256) void rope_kv_write_token_kernel(
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

// cos and sin of every token's angles, rounded to the activation type as the rotation uses them:
// table[t][0][i] = cos(pos[t] * inv_freq[i]), table[t][1][i] = sin(...), float32. Computed once a
// step for kernels that rotate on the fly in every layer.
template <typename T>
__global__ void rope_angles_kernel(const int* __restrict__ positions, const float* __restrict__ inv_freq,
                                   float* __restrict__ table, int half) {
  const int64_t token = blockIdx.x;
  const float pos = (float)positions[token];
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    float sv, cv;
    sincosf(pos * inv_freq[i], &sv, &cv);
    table[(token * 2 + 0) * half + i] = round_to<T>(cv);
    table[(token * 2 + 1) * half + i] = round_to<T>(sv);
  }
}

extern "C" int dli_rope_angles(const int* positions, const float* inv_freq, float* table, int tokens,
                               int half, int is_bf16, hipStream_t stream) {
  if (tokens <= 0 || half <= 0) return DLI_OK;
  if (is_bf16) rope_angles_kernel<bf16_t><<<tokens, 64, 0, stream>>>(positions, inv_freq, table, half);
  else rope_angles_kernel<float><<<tokens, 64, 0, stream>>>(positions, inv_freq, table, half);
  return dli_launch_status();
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
  const int half = rotary_dim / 2;
  const int items = (q_heads + kv_heads) * half + kv_heads * (head_dim - rotary_dim) + kv_heads * head_dim;
  if (items <= 0) return DLI_OK;
  if (tokens > 64) {
    if (is_bf16)
      rope_kv_write_token_kernel<bf16_t><<<tokens, 256, 0, stream>>>(
          (bf16_t*)qkv, row_stride, positions, inv_freq, rotary_dim, slots, (bf16_t*)k_pages,
          (bf16_t*)v_pages, q_heads, kv_heads, head_dim, page_size);
    else
      rope_kv_write_token_kernel<float><<<tokens, 256, 0, stream>>>(
          (float*)qkv, row_stride, positions, inv_freq, rotary_dim, slots, (float*)k_pages,
          (float*)v_pages, q_heads, kv_heads, head_dim, page_size);
    return dli_launch_status();
  }
  const dim3 grid(tokens, min((items + 255) / 256, 64));
  if (is_bf16)
    rope_kv_write_kernel<bf16_t><<<grid, 256, 0, stream>>>(
        (bf16_t*)qkv, row_stride, positions, inv_freq, rotary_dim, slots, (bf16_t*)k_pages,
        (bf16_t*)v_pages, q_heads, kv_heads, head_dim, page_size, items);
  else
    rope_kv_write_kernel<float><<<grid, 256, 0, stream>>>(
        (float*)qkv, row_stride, positions, inv_freq, rotary_dim, slots, (float*)k_pages,
        (float*)v_pages, q_heads, kv_heads, head_dim, page_size, items);
  return dli_launch_status();
}
