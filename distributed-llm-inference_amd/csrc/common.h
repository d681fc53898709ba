// Shared device helpers for the gfx950 kernels: element types, conversions and reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16_t;

#define DLI_WAVE 64

// Status codes returned by every extern "C" entry point.
#define DLI_OK 0
#define DLI_ERR_ARGUMENT -1   // sizes that the kernel does not take
#define DLI_ERR_LAUNCH -2     // the runtime refused the launch

__device__ __forceinline__ float to_f32(float x) { return x; }
__device__ __forceinline__ float to_f32(bf16_t x) { return (float)x; }

template <typename T> __device__ __forceinline__ T from_f32(float x);
template <> __device__ __forceinline__ float from_f32<float>(float x) { return x; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float x) { return (bf16_t)x; }

// Round through the storage type: what a value becomes when it is written as T and read back.
template <typename T> __device__ __forceinline__ float round_to(float x) { return to_f32(from_f32<T>(x)); }

// silu(g) = g * sigmoid(g) in 32-bit (reference: src/dli/model/llama.py:190). Faster forms of the
// exponential and the division were tried for bfloat16 and changed no timing: the kernels that
// use it wait for memory.
template <typename T> __device__ __forceinline__ float silu(float g) { return g / (1.f + expf(-g)); }


__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int m = DLI_WAVE / 2; m > 0; m >>= 1) v += __shfl_xor(v, m, DLI_WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int m = DLI_WAVE / 2; m > 0; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, DLI_WAVE));
  return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result. `scratch` holds 16 floats.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x % DLI_WAVE, wave = threadIdx.x / DLI_WAVE;
  const int nwaves = (blockDim.x + DLI_WAVE - 1) / DLI_WAVE;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int i = 0; i < nwaves; ++i) total += scratch[i];  // same order in every thread
  return total;
}

static inline int dli_launch_status() {
  return hipGetLastError() == hipSuccess ? DLI_OK : DLI_ERR_LAUNCH;
}

// Compute units of the current device (256 if the runtime does not say), asked once per device.
static inline int dli_compute_units() {
  static int cached[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev] = n;
  }
  return cached[dev];
}
