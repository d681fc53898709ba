// Row-wise and element-wise kernels: embedding gather, RMSNorm, SwiGLU gate, residual add,
// row gather, casts and page copies. Each is a template over the activation type
// (float for the 32-bit path, bf16 for serving); all statistics are computed in 32-bit.
#include "common.h"

// ---------------------------------------------------------------- embedding: out[t] = table[id[t]]
template <typename T>
__global__ void embedding_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                                 T* __restrict__ out, int width) {
  const int64_t row = blockIdx.x;
  const T* src = table + (int64_t)ids[row] * width;
  T* dst = out + row * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = src[i];
}

// ---------------------------------------------------------------- RMSNorm
// y = w * cast(x * rsqrt(mean(x^2) + eps)); the normalised value is rounded to the activation
// type before the weight multiplies it (reference: src/dli/model/llama.py:40-44).
// With `delta`, the row is first replaced by x + delta (sum in 32-bit) and written to `sum_out`.
template <typename T>
__global__ void rms_norm_kernel(const T* x, const T* __restrict__ delta,
                                const float* __restrict__ weight, T* sum_out,
                                T* __restrict__ out, int width, float eps) {
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  const T* xr = x + row * width;
  float ss = 0.f;
  if (delta != nullptr) {
    const T* dr = delta + row * width;
    T* sr = sum_out + row * width;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
      const T s = from_f32<T>(to_f32(xr[i]) + to_f32(dr[i]));
      sr[i] = s;
      const float f = to_f32(s);
      ss += f * f;
    }
    xr = sr;
    __syncthreads();  // this block's own writes to sr are read back below
  } else {
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
      const float f = to_f32(xr[i]);
      ss += f * f;
    }
  }
  const float total = block_sum(ss, scratch);
  const float r = rsqrtf(total / (float)width + eps);
  T* yr = out + row * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float normed = round_to<T>(to_f32(xr[i]) * r);
    yr[i] = from_f32<T>(weight[i] * normed);
  }
}

// Eight elements at a time (rows of a multiple of eight elements, 16-byte aligned).
template <typename T> struct Vec8;
template <> struct Vec8<bf16_t> { typedef __bf16 type __attribute__((ext_vector_type(8))); };
template <> struct Vec8<float> { typedef float type __attribute__((ext_vector_type(8))); };

template <typename T>
__global__ void rms_norm_vec_kernel(const T* x, const T* __restrict__ delta,
                                    const float* __restrict__ weight, T* sum_out,
                                    T* __restrict__ out, int width, float eps) {
  typedef typename Vec8<T>::type V;
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  const V* xr = reinterpret_cast<const V*>(x + row * width);
  const V* dr = delta != nullptr ? reinterpret_cast<const V*>(delta + row * width) : nullptr;
  V* sr = delta != nullptr ? reinterpret_cast<V*>(sum_out + row * width) : nullptr;
  const int chunks = width / 8;
  float ss = 0.f;
  if (chunks <= (int)blockDim.x) {
    // one chunk a thread: it stays in registers across the reduction, and the weights are asked
    // for together with it, so the row is one trip to memory long
    const int c = threadIdx.x;
    const bool mine = c < chunks;
    V v;
    float4 w0 = make_float4(0.f, 0.f, 0.f, 0.f), w1 = w0;
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = from_f32<T>(0.f);
    if (mine) {
      v = xr[c];
      w0 = *reinterpret_cast<const float4*>(weight + c * 8);
      w1 = *reinterpret_cast<const float4*>(weight + c * 8 + 4);
      if (dr != nullptr) {
        const V d = dr[c];
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = from_f32<T>(to_f32((T)v[i]) + to_f32((T)d[i]));
        sr[c] = v;
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float f = to_f32((T)v[i]);
        ss += f * f;
      }
    }
    const float r = rsqrtf(block_sum(ss, scratch) / (float)width + eps);
    if (mine) {
      const float wv[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
      V y;
#pragma unroll
      for (int i = 0; i < 8; ++i) y[i] = from_f32<T>(wv[i] * round_to<T>(to_f32((T)v[i]) * r));
      reinterpret_cast<V*>(out + row * width)[c] = y;
    }
    return;
  }
  for (int c = threadIdx.x; c < chunks; c += blockDim.x) {
    V v = xr[c];
    if (dr != nullptr) {
      const V d = dr[c];
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = from_f32<T>(to_f32((T)v[i]) + to_f32((T)d[i]));
      sr[c] = v;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float f = to_f32((T)v[i]);
      ss += f * f;
    }
  }
  const float r = rsqrtf(block_sum(ss, scratch) / (float)width + eps);
  const V* src = dr != nullptr ? reinterpret_cast<const V*>(sum_out + row * width) : xr;
  V* yr = reinterpret_cast<V*>(out + row * width);
  for (int c = threadIdx.x; c < chunks; c += blockDim.x) {
    const V v = src[c];  // re-read of this thread's own chunk
    const float4 w0 = *reinterpret_cast<const float4*>(weight + c * 8);
    const float4 w1 = *reinterpret_cast<const float4*>(weight + c * 8 + 4);
    const float wv[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
    V y;
#pragma unroll
    for (int i = 0; i < 8; ++i) y[i] = from_f32<T>(wv[i] * round_to<T>(to_f32((T)v[i]) * r));
    yr[c] = y;
  }
}

template <typename T>
__global__ void silu_mul_vec_kernel(const T* __restrict__ gu, T* __restrict__ out, int64_t rows, int inter) {
  typedef typename Vec8<T>::type V;
  const int chunks = inter / 8;
  const int64_t total = rows * chunks;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = idx / chunks;
    const int c = (int)(idx - r * chunks);
    const V g = *reinterpret_cast<const V*>(gu + r * 2 * inter + c * 8);
    const V u = *reinterpret_cast<const V*>(gu + r * 2 * inter + inter + c * 8);
    V o;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float gf = to_f32((T)g[i]);
      const float sg = silu<T>(gf);
      o[i] = from_f32<T>(round_to<T>(sg) * to_f32((T)u[i]));
    }
    *reinterpret_cast<V*>(out + r * inter + c * 8) = o;
  }
}

// ---------------------------------------------------------------- SwiGLU gate: out = silu(g) * u
// `gu` holds [rows, 2*inter]: gate columns first, then up columns.
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int64_t rows, int inter) {
  const int64_t total = rows * inter;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = idx / inter;
    const int c = (int)(idx - r * inter);
    const float g = to_f32(gu[r * 2 * inter + c]);
    const float u = to_f32(gu[r * 2 * inter + inter + c]);
    const float s = silu<T>(g);
    out[idx] = from_f32<T>(round_to<T>(s) * u);
  }
}

// ---------------------------------------------------------------- out = a + b (+ bias per column)
template <typename T>
__global__ void add_kernel(const T* __restrict__ a, const T* __restrict__ b, const T* __restrict__ bias,
                           T* __restrict__ out, int64_t rows, int width) {
  const int64_t total = rows * width;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    float v = to_f32(a[idx]);
    if (bias != nullptr) v = round_to<T>(v + to_f32(bias[idx % width]));
    if (b != nullptr) v += to_f32(b[idx]);
    out[idx] = from_f32<T>(v);
  }
}

// ---------------------------------------------------------------- out[i] = x[rows[i]]
template <typename T>
__global__ void gather_rows_kernel(const T* __restrict__ x, const int* __restrict__ rows,
                                   T* __restrict__ out, int width) {
  const int64_t i = blockIdx.x;
  const T* src = x + (int64_t)rows[i] * width;
  T* dst = out + i * width;
  for (int c = threadIdx.x; c < width; c += blockDim.x) dst[c] = src[c];
}

template <typename T>
__global__ void to_float_kernel(const T* __restrict__ x, float* __restrict__ out, int64_t total) {
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x)
    out[idx] = to_f32(x[idx]);
}

// ---------------------------------------------------------------- page copies (copy-on-write)
// pool is [layers][2][pages][page_elems]; copies page src[i] to dst[i] in every layer, K and V.
template <typename T>
__global__ void copy_pages_kernel(T* __restrict__ pool, const int* __restrict__ src,
                                  const int* __restrict__ dst, int64_t pages, int64_t page_elems) {
  const int op = blockIdx.x;
  const int64_t plane = blockIdx.y;  // layer * 2 + (0 for K, 1 for V)
  const T* s = pool + (plane * pages + src[op]) * page_elems;
  T* d = pool + (plane * pages + dst[op]) * page_elems;
  for (int64_t i = threadIdx.x; i < page_elems; i += blockDim.x) d[i] = s[i];
}

template <typename T>
__global__ void fill_kernel(T* __restrict__ x, float value, int64_t total) {
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x)
    x[idx] = from_f32<T>(value);
}

static inline int grid_for(int64_t total, int threads) {
  int64_t g = (total + threads - 1) / threads;
  if (g > 65535 * 4) g = 65535 * 4;
  if (g < 1) g = 1;
  return (int)g;
}

#define DISPATCH_DTYPE(is_bf16, CALL) \
  do {                                \
    if (is_bf16) {                    \
      typedef bf16_t T;               \
      CALL;                           \
    } else {                          \
      typedef float T;                \
      CALL;                           \
    }                                 \
  } while (0)

extern "C" {

int dli_embedding(const void* table, const int* ids, void* out, int rows, int width, int is_bf16,
                  hipStream_t stream) {
  if (rows <= 0) return DLI_OK;
  if (width <= 0) return DLI_ERR_ARGUMENT;
  DISPATCH_DTYPE(is_bf16, (embedding_kernel<T><<<rows, 256, 0, stream>>>((const T*)table, ids, (T*)out, width)));
  return dli_launch_status();
}

int dli_rms_norm(const void* x, const void* delta, const float* weight, void* sum_out, void* out,
                 int rows, int width, float eps, int is_bf16, hipStream_t stream) {
  if (rows <= 0) return DLI_OK;
  if (width <= 0 || (delta != nullptr && sum_out == nullptr)) return DLI_ERR_ARGUMENT;
  const int threads = width >= 2048 ? 512 : 256;
  const bool aligned = (((uintptr_t)x | (uintptr_t)delta | (uintptr_t)sum_out | (uintptr_t)out | (uintptr_t)weight) % 32) == 0;
  if (width % 8 == 0 && aligned) {
    const int vthreads = width / 8 >= 256 ? 256 : (width / 8 >= 128 ? 128 : 64);
    DISPATCH_DTYPE(is_bf16, (rms_norm_vec_kernel<T><<<rows, vthreads, 0, stream>>>(
                                (const T*)x, (const T*)delta, weight, (T*)sum_out, (T*)out, width, eps)));
    return dli_launch_status();
  }
  DISPATCH_DTYPE(is_bf16, (rms_norm_kernel<T><<<rows, threads, 0, stream>>>(
                              (const T*)x, (const T*)delta, weight, (T*)sum_out, (T*)out, width, eps)));
  return dli_launch_status();
}

int dli_silu_mul(const void* gu, void* out, int rows, int inter, int is_bf16, hipStream_t stream) {
  if (rows <= 0) return DLI_OK;
  if (inter <= 0) return DLI_ERR_ARGUMENT;
  const int64_t total = (int64_t)rows * inter;
  if (inter % 8 == 0 && (((uintptr_t)gu | (uintptr_t)out) % 32) == 0) {
    DISPATCH_DTYPE(is_bf16, (silu_mul_vec_kernel<T><<<grid_for(total / 8, 256), 256, 0, stream>>>((const T*)gu, (T*)out, rows, inter)));
    return dli_launch_status();
  }
  DISPATCH_DTYPE(is_bf16, (silu_mul_kernel<T><<<grid_for(total, 256), 256, 0, stream>>>((const T*)gu, (T*)out, rows, inter)));
  return dli_launch_status();
}

int dli_add(const void* a, const void* b, const void* bias, void* out, int rows, int width, int is_bf16,
            hipStream_t stream) {
  if (rows <= 0) return DLI_OK;
  if (width <= 0) return DLI_ERR_ARGUMENT;
  const int64_t total = (int64_t)rows * width;
  DISPATCH_DTYPE(is_bf16, (add_kernel<T><<<grid_for(total, 256), 256, 0, stream>>>(
                              (const T*)a, (const T*)b, (const T*)bias, (T*)out, rows, width)));
  return dli_launch_status();
}

int dli_gather_rows(const void* x, const int* rows, void* out, int count, int width, int is_bf16,
                    hipStream_t stream) {
  if (count <= 0) return DLI_OK;
  if (width <= 0) return DLI_ERR_ARGUMENT;
  DISPATCH_DTYPE(is_bf16, (gather_rows_kernel<T><<<count, 256, 0, stream>>>((const T*)x, rows, (T*)out, width)));
  return dli_launch_status();
}

int dli_to_float(const void* x, float* out, int64_t total, int is_bf16, hipStream_t stream) {
  if (total <= 0) return DLI_OK;
  DISPATCH_DTYPE(is_bf16, (to_float_kernel<T><<<grid_for(total, 256), 256, 0, stream>>>((const T*)x, out, total)));
  return dli_launch_status();
}

int dli_copy_pages(void* pool, const int* src, const int* dst, int ops, int planes, int64_t pages,
                   int64_t page_elems, int is_bf16, hipStream_t stream) {
  if (ops <= 0) return DLI_OK;
  if (planes <= 0 || pages <= 0 || page_elems <= 0) return DLI_ERR_ARGUMENT;
  DISPATCH_DTYPE(is_bf16, (copy_pages_kernel<T><<<dim3(ops, planes), 256, 0, stream>>>((T*)pool, src, dst, pages, page_elems)));
  return dli_launch_status();
}

int dli_fill(void* x, float value, int64_t total, int is_bf16, hipStream_t stream) {
  if (total <= 0) return DLI_OK;
  DISPATCH_DTYPE(is_bf16, (fill_kernel<T><<<grid_for(total, 256), 256, 0, stream>>>((T*)x, value, total)));
  return dli_launch_status();
}

}  // extern "C"
