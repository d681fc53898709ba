// 32-bit matrix product for the true 32-bit path: out[m][n] = sum_k a[m][k] * w[n][k]
// (+ bias[n]) (+ residual[m][n]). Plain FMA on the vector units, no matrix-core mode, so every
// product and sum is IEEE single precision. Every output element sums its k in the same fixed
// order whatever the tile it falls in, so a row's result does not depend on how many other rows
// are in the batch: runs of GF_RUN consecutive k are summed in ascending order, and the runs'
// sums are added in ascending order (the rounding error of a long sum then grows with the
// length of a run plus the number of runs, not with k).
#include "common.h"

#define GF_BM 64
#define GF_BN 64
#define GF_BK 16
#define GF_RUN 256  // a multiple of GF_BK

__global__ __launch_bounds__(256) void gemm_f32_nt_kernel(
    const float* __restrict__ a, int64_t lda, const float* __restrict__ w, int64_t ldw,
    const float* __restrict__ bias, const float* __restrict__ residual, int64_t ldr,
    float* __restrict__ out, int64_t ldo, int m, int n, int k) {
  __shared__ float as[GF_BK][GF_BM + 4];
  __shared__ float ws[GF_BK][GF_BN + 4];
  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;
  const int m0 = blockIdx.y * GF_BM, n0 = blockIdx.x * GF_BN;
  float acc[4][4] = {};    // the run of k in progress
  float total[4][4] = {};  // the finished runs
  const int lrow = tid / 4;          // 0..63: tile row loaded by this thread
  const int lk = (tid % 4) * 4;      // 0,4,8,12: first of its four k values
  const bool vec = (k % 4 == 0) && (lda % 4 == 0) && (ldw % 4 == 0) &&
                   (((uintptr_t)a | (uintptr_t)w) % 16 == 0);
  for (int k0 = 0; k0 < k; k0 += GF_BK) {
    float av[4] = {0.f, 0.f, 0.f, 0.f}, wv[4] = {0.f, 0.f, 0.f, 0.f};
    const int gm = m0 + lrow, gn = n0 + lrow, gk = k0 + lk;
    if (vec) {
      if (gm < m && gk < k) *(float4*)av = *(const float4*)(a + (int64_t)gm * lda + gk);
      if (gn < n && gk < k) *(float4*)wv = *(const float4*)(w + (int64_t)gn * ldw + gk);
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (gm < m && gk + i < k) av[i] = a[(int64_t)gm * lda + gk + i];
        if (gn < n && gk + i < k) wv[i] = w[(int64_t)gn * ldw + gk + i];
      }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      as[lk + i][lrow] = av[i];
      ws[lk + i][lrow] = wv[i];
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GF_BK; ++kk) {
      const float4 af = *(const float4*)&as[kk][ty * 4];
      const float4 wf = *(const float4*)&ws[kk][tx * 4];
      const float ar[4] = {af.x, af.y, af.z, af.w};
      const float wr[4] = {wf.x, wf.y, wf.z, wf.w};
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(ar[i], wr[j], acc[i][j]);
    }
    if ((k0 + GF_BK) % GF_RUN == 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          total[i][j] += acc[i][j];
          acc[i][j] = 0.f;
        }
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int gm = m0 + ty * 4 + i;
    if (gm >= m) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int gn = n0 + tx * 4 + j;
      if (gn >= n) continue;
      float v = total[i][j] + acc[i][j];
      if (bias != nullptr) v += bias[gn];
      if (residual != nullptr) v += residual[(int64_t)gm * ldr + gn];
      out[(int64_t)gm * ldo + gn] = v;
    }
  }
}

extern "C" int dli_gemm_f32_nt(const float* a, int64_t lda, const float* w, int64_t ldw,
                               const float* bias, const float* residual, int64_t ldr, float* out,
                               int64_t ldo, int m, int n, int k, hipStream_t stream) {
  if (m <= 0 || n <= 0) return DLI_OK;
  if (k <= 0 || lda < k || ldw < k || ldo < n || (residual != nullptr && ldr < n)) return DLI_ERR_ARGUMENT;
  const dim3 grid((n + GF_BN - 1) / GF_BN, (m + GF_BM - 1) / GF_BM);
  if (grid.y > 65535) return DLI_ERR_ARGUMENT;
  gemm_f32_nt_kernel<<<grid, 256, 0, stream>>>(a, lda, w, ldw, bias, residual, ldr, out, ldo, m, n, k);
  return dli_launch_status();
}
