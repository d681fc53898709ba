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

// Few tokens (decode steps, short portions of prompts): a token's work is a list of items, the rotary pairs of its q and k heads,
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

// Many tokens, vector form: a workgroup takes ROWS consecutive tokens and moves 16 bytes per
// access. v goes through LDS so that one thread writes a dimension's ROWS keys as one contiguous
// run of the transposed page when the tokens' slots are consecutive in one page (a prompt's
// portion, mostly); otherwise element by element. Workgroups that share a page's runs are placed
// on the same XCD (workgroup b runs on XCD b % 8), so that a page's cache lines are completed in
// one L2 instead of being written back in pieces from several.
// Needs rotary_dim/2, head_dim and row_stride to be multiples of the 16-byte vector.
template <typename T, int ROWS>
__global__ __launch_bounds__(256) void rope_kv_write_rows_kernel(
    T* __restrict__ qkv, int64_t row_stride, const int* __restrict__ positions,
    const float* __restrict__ inv_freq, int rotary_dim, const int* __restrict__ slots,
    T* __restrict__ k_pages, T* __restrict__ v_pages, int tokens, int q_heads, int kv_heads,
    int head_dim, int page_size) {
  constexpr int VEC = 16 / sizeof(T);
  typedef T vec_t __attribute__((ext_vector_type(VEC)));
  extern __shared__ __align__(16) unsigned char rope_lds[];
  __shared__ int slot_s[ROWS];
  const int half = rotary_dim / 2, rest = head_dim - rotary_dim, v_width = kv_heads * head_dim;
  float* cs = reinterpret_cast<float*>(rope_lds);
  float* sn = cs + ROWS * half;
  T* vs = reinterpret_cast<T*>(sn + ROWS * half);

  const int xcd = blockIdx.x % 8, local = blockIdx.x / 8;
  const int group = ((local / 2) * 8 + xcd) * 2 + local % 2;
  const int t0 = group * ROWS;
  if (t0 >= tokens) return;
  const int rows = min(ROWS, tokens - t0);
  T* base = qkv + (int64_t)t0 * row_stride;

  // The rotary pairs of the q and k heads: chunk j of a head pairs dimensions [j*VEC, j*VEC+VEC)
  // with the same run + half. A thread asks for U chunk pairs at once, the first U before the
  // angles are computed, so that the workgroup is few trips to memory long.
  constexpr int U = 5;
  const int chunks = half / VEC, rot_heads = q_heads + kv_heads;
  const int total = rows * rot_heads * chunks;
  vec_t lo[U], hi[U];
  int idx0 = threadIdx.x;
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int idx = min(idx0 + u * (int)blockDim.x, total - 1);
    const int r = idx / (rot_heads * chunks), rem = idx - r * rot_heads * chunks;
    const T* h = base + r * row_stride + (int64_t)(rem / chunks) * head_dim + (rem % chunks) * VEC;
    lo[u] = *reinterpret_cast<const vec_t*>(h);
    hi[u] = *reinterpret_cast<const vec_t*>(h + half);
  }

  for (int idx = threadIdx.x; idx < rows * half; idx += blockDim.x) {
    const int r = idx / half, i = idx - r * half;
    float c = 1.f, sv = 0.f;
    if (inv_freq != nullptr) {
      sincosf((float)positions[t0 + r] * inv_freq[i], &sv, &c);
      c = round_to<T>(c);
      sv = round_to<T>(sv);
    }
    cs[idx] = c;
    sn[idx] = sv;
  }
  const bool pages = slots != nullptr && k_pages != nullptr && v_pages != nullptr;
  if (threadIdx.x < ROWS) slot_s[threadIdx.x] = pages && threadIdx.x < rows ? slots[t0 + threadIdx.x] : -1;
  // v rows into LDS
  const int v_chunks = v_width / VEC;
  if (pages) {
    for (int idx = threadIdx.x; idx < rows * v_chunks; idx += blockDim.x) {
      const int r = idx / v_chunks, c = idx - r * v_chunks;
      *reinterpret_cast<vec_t*>(vs + r * v_width + c * VEC) = *reinterpret_cast<const vec_t*>(
          base + r * row_stride + (int64_t)(q_heads + kv_heads) * head_dim + c * VEC);
    }
  }
  __syncthreads();

  while (true) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int idx = idx0 + u * (int)blockDim.x;
      if (idx >= total) break;
      const int r = idx / (rot_heads * chunks), rem = idx - r * rot_heads * chunks;
      const int head = rem / chunks, j = rem - head * chunks;
      const int slot = slot_s[r];
      if (head >= q_heads && slot < 0) continue;
      vec_t ylo, yhi;
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        const float c = cs[r * half + j * VEC + e], sv = sn[r * half + j * VEC + e];
        const float x1 = to_f32(lo[u][e]), x2 = to_f32(hi[u][e]);
        ylo[e] = from_f32<T>(x1 * c - x2 * sv);
        yhi[e] = from_f32<T>(x2 * c + x1 * sv);
      }
      T* dst = base + r * row_stride + (int64_t)head * head_dim + j * VEC;
      if (head >= q_heads)
        dst = k_pages + (((int64_t)(slot / page_size) * kv_heads + (head - q_heads)) * page_size + slot % page_size) * head_dim + j * VEC;
      *reinterpret_cast<vec_t*>(dst) = ylo;
      *reinterpret_cast<vec_t*>(dst + half) = yhi;
    }
    idx0 += U * blockDim.x;
    if (idx0 >= total) break;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int idx = min(idx0 + u * (int)blockDim.x, total - 1);
      const int r = idx / (rot_heads * chunks), rem = idx - r * rot_heads * chunks;
      const T* h = base + r * row_stride + (int64_t)(rem / chunks) * head_dim + (rem % chunks) * VEC;
      lo[u] = *reinterpret_cast<const vec_t*>(h);
      hi[u] = *reinterpret_cast<const vec_t*>(h + half);
    }
  }
  if (!pages) return;
  // the part of k beyond the rotary dimensions passes through
  for (int idx = threadIdx.x; idx < rows * kv_heads * rest; idx += blockDim.x) {
    const int r = idx / (kv_heads * rest), rem = idx - r * kv_heads * rest;
    const int hk = rem / rest, i = rotary_dim + rem - hk * rest;
    const int slot = slot_s[r];
    if (slot < 0) continue;
    k_pages[(((int64_t)(slot / page_size) * kv_heads + hk) * page_size + slot % page_size) * head_dim + i] =
        base[r * row_stride + (int64_t)(q_heads + hk) * head_dim + i];
  }
  // v: a dimension's keys are contiguous in the page
  const int slot0 = slot_s[0];
  bool run = rows == ROWS && slot0 >= 0 && page_size % VEC == 0 && (slot0 % page_size) % VEC == 0 &&
             slot0 % page_size + ROWS <= page_size;
#pragma unroll
  for (int r = 1; r < ROWS; ++r) run = run && slot_s[r] == slot0 + r;
  if (run) {
    const int64_t page = slot0 / page_size;
    const int off = slot0 % page_size;
    for (int c = threadIdx.x; c < v_width; c += blockDim.x) {
      const int hk = c / head_dim, i = c - hk * head_dim;
      T* dst = v_pages + ((page * kv_heads + hk) * head_dim + i) * page_size + off;
#pragma unroll
      for (int r0 = 0; r0 < ROWS; r0 += VEC) {
        vec_t keys;
#pragma unroll
        for (int e = 0; e < VEC; ++e) keys[e] = vs[(r0 + e) * v_width + c];
        *reinterpret_cast<vec_t*>(dst + r0) = keys;
      }
    }
  } else {
    for (int idx = threadIdx.x; idx < rows * v_width; idx += blockDim.x) {
      const int r = idx / v_width, c = idx - r * v_width;
      const int slot = slot_s[r];
      if (slot < 0) continue;
      const int hk = c / head_dim, i = c - hk * head_dim;
      v_pages[(((int64_t)(slot / page_size) * kv_heads + hk) * head_dim + i) * page_size + slot % page_size] = vs[idx];
    }
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
  // Up to 512 tokens one item per thread is ahead (256 tokens at the 1B sizes: 4.6 us for a prompt's
  // rows and 4.9 for rows of 256 requests, against 6.4 and 10.6 in the vector form, which launches
  // a workgroup for eight rows and gains from rows that lie side by side in a page; 1,024 rows of
  // a prompt: 11.7 against 7.1)
  if (tokens > 512) {
    // the vector form where the sizes are multiples of its 16 bytes and a workgroup's v rows fit LDS
    constexpr int ROWS = 8;
    const int vec = is_bf16 ? 8 : 4, elem = is_bf16 ? 2 : 4;
    const size_t lds = (size_t)2 * ROWS * half * sizeof(float) + (size_t)ROWS * kv_heads * head_dim * elem;
    if (half > 0 && half % vec == 0 && head_dim % vec == 0 && row_stride % vec == 0 &&
        (uintptr_t)qkv % 16 == 0 && (uintptr_t)k_pages % 16 == 0 && (uintptr_t)v_pages % 16 == 0 &&
        lds <= 48 * 1024) {
      const int groups = (tokens + ROWS - 1) / ROWS;
      const int grid = (groups + 15) / 16 * 16;  // the XCD-aware order permutes blocks of 16
      if (is_bf16)
        rope_kv_write_rows_kernel<bf16_t, ROWS><<<grid, 256, lds, stream>>>(
            (bf16_t*)qkv, row_stride, positions, inv_freq, rotary_dim, slots, (bf16_t*)k_pages,
            (bf16_t*)v_pages, tokens, q_heads, kv_heads, head_dim, page_size);
      else
        rope_kv_write_rows_kernel<float, ROWS><<<grid, 256, lds, stream>>>(
            (float*)qkv, row_stride, positions, inv_freq, rotary_dim, slots, (float*)k_pages,
            (float*)v_pages, tokens, q_heads, kv_heads, head_dim, page_size);
      return dli_launch_status();
    }
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
