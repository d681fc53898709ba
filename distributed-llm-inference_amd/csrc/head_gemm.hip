// The logits of a decode step of few rows: out[m][n] = sum_k xhat[m][k] * w[n][k] for a
// vocabulary of rows n (src/dli/model/llama.py:305), float32, with the final RMSNorm of x inside
// (src/dli/model/llama.py:40-44). The table is the largest matrix a step reads (half a gigabyte at
// the 1B sizes), so this kernel is a long stream rather than a short one, and it is built for
// that: one workgroup per compute unit stays for the whole launch and walks the table's tiles in
// turn, instead of one short-lived workgroup per pair of tiles.
//   - The activations do not change from tile to tile: each wave normalises the run of k that it
//     multiplies once, keeps it in registers, and from then on reads weights only (a workgroup of
//     the tile-by-tile kernel re-reads all rows and the norm's weights for every pair of tiles,
//     a third as many bytes again as the weights themselves at 8 rows).
//   - The weights of the next block of 128 k are asked for before the products of the current
//     one, also across the end of a pair of tiles, so the stream never drains.
// Weights in tile order (16 features x 128 k contiguous, see skinny_gemm.hip); 4 waves split k and
// add up through LDS in wave order: the same sums in the same order as the tile-by-tile kernel's
// shape of 4 k-waves x 2 tiles, to the bit. Rows: at most 16. K = 512 * KB.
// The wave that stores the logits has every one of them in a register once: asked to, it keeps
// each row's best (value, lowest index) among the logits of its workgroup and leaves it as one
// part of the row's argmax, so that the sampler's first stage (a kernel that reads all logits
// again) need not run.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));

namespace {

constexpr int HEAD_KS = 4;  // waves of a workgroup; they split k

__device__ __forceinline__ float4v mfma32(bf16x8 a, bf16x8 b, float4v c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

template <int KB, bool NORM>
__global__ __launch_bounds__(HEAD_KS * 64) void head_gemm_kernel(
    const bf16_t* __restrict__ x, int64_t ldx, const float* __restrict__ ssq_in, int ssq_parts,
    const float* __restrict__ norm_w, float eps, const bf16_t* __restrict__ w, float* __restrict__ out,
    int64_t ldo, int M, int N, int K, float* __restrict__ best_val, int* __restrict__ best_idx) {
  constexpr int KS = HEAD_KS;
  __shared__ float red[2][KS - 1][2][4][64];  // two pairs of tiles in turn

  const int lane = threadIdx.x % 64, ks = threadIdx.x / 64;
  const int col = lane % 16, grp = lane / 16;
  const int tiles = N / 16, pairs = (tiles + 1) / 2;
  const int kb0 = ks * KB;  // this wave's first block of 128 k

  float rs = 1.f;
  if constexpr (NORM) {
    // rs[m] from the parts of sum x^2 that the producer of x left: dealt out to the lane groups
    // of all waves, added per wave, then in wave order through LDS
    __shared__ float rsum[KS][16];
    const int m = min(col, M - 1);
    float sum = 0.f;
    for (int p0 = ks * 4 + grp; p0 < ssq_parts; p0 += 32 * KS) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int p = p0 + u * 4 * KS;
        const float part = ssq_in[(int64_t)min(p, ssq_parts - 1) * M + m];
        v[u] = p < ssq_parts ? part : 0.f;
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) sum += v[u];
    }
    sum += __shfl_xor(sum, 16, 64);
    sum += __shfl_xor(sum, 32, 64);
    if (grp == 0) rsum[ks][col] = sum;
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int wv = 0; wv < KS; ++wv) total += rsum[wv][col];
    rs = rsqrtf(total / (float)K + eps);
  }

  // the wave's activations, normalised once: lane (col, grp) holds row col, k = 128*(kb0 + b) +
  // 32*grp + 8*q + (0..7) for block b and product q
  bf16x8 xn[KB][4];
  {
    const bf16_t* xrow = x + (int64_t)min(col, M - 1) * ldx;
#pragma unroll
    for (int b = 0; b < KB; ++b)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int k = (kb0 + b) * 128 + grp * 32 + q * 8;
        bf16x8 v = *reinterpret_cast<const bf16x8*>(xrow + k);  // rows past the last: the last again, not stored
        if constexpr (NORM) {
          const float4v w0 = *reinterpret_cast<const float4v*>(norm_w + k);
          const float4v w1 = *reinterpret_cast<const float4v*>(norm_w + k + 4);
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            const float normed = (float)(bf16_t)((float)v[i] * rs);
            v[i] = (bf16_t)((i < 4 ? w0[i] : w1[i - 4]) * normed);
          }
        }
        xn[b][q] = v;
      }
  }

  // tile `tile`, block b of this wave, product q: 1 KB of consecutive memory for the wave
  auto w_at = [&](int tile, int b, int q) __attribute__((always_inline)) {
    return reinterpret_cast<const bf16x8*>(w + (int64_t)tile * 16 * K + (int64_t)(kb0 + b) * 2048 + q * 512 + lane * 8);
  };
  // A pair's second tile may lie past the table's end (an odd number of tiles): it reads the
  // last tile again and is not stored.
  auto load_block = [&](bf16x8 (&dst)[2][4], int pair, int b) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int tile = min(2 * pair + j, tiles - 1);
#pragma unroll
      for (int q = 0; q < 4; ++q) dst[j][q] = *w_at(tile, b, q);
    }
  };

  static_assert(KB % 2 == 0, "the two weight buffers take turns in a fixed order");
  bf16x8 wf[2][2][4];
  float top_v = -INFINITY;  // wave 0: the best logit of row col among those this lane stored, and its index
  int top_i = 0x7fffffff;
  int pair = blockIdx.x;
  if (pair < pairs) load_block(wf[0], pair, 0);
  for (int turn = 0; pair < pairs; pair += gridDim.x, ++turn) {
    float4v acc[2] = {float4v{0.f, 0.f, 0.f, 0.f}, float4v{0.f, 0.f, 0.f, 0.f}};
    const int next_pair = pair + gridDim.x;
#pragma unroll
    for (int b = 0; b < KB; ++b) {
      // the block after this one: of this pair, or the first of the workgroup's next pair
      // (past the last pair the last one's first block again: a load under a condition would leave
      // the number of loads on their way unknown, and every block would be waited for at once)
      if (b + 1 < KB) load_block(wf[(b + 1) % 2], pair, b + 1);
      else load_block(wf[0], min(next_pair, pairs - 1), 0);
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[j] = mfma32(wf[b % 2][j][q], xn[b][q], acc[j]);
    }
    // wave 0 adds the other waves' tiles to its own, in wave order, and stores the logits; the
    // others go on with the next pair meanwhile (the exchange buffers take turns: a wave writes
    // buffer t % 2 again only after the barrier of turn t + 1, which wave 0 reaches after it has
    // read that buffer)
    const int buf = turn % 2;
    if (ks != 0) {
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) red[buf][ks - 1][j][i][lane] = acc[j][i];
    }
    __syncthreads();
    if (ks == 0) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int tile = 2 * pair + j;
        if (tile >= tiles) continue;
        float4v y;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float v = acc[j][i];
          for (int wv = 0; wv < KS - 1; ++wv) v += red[buf][wv][j][i][lane];
          y[i] = v;
          const int n = tile * 16 + 4 * grp + i;
          if (v > top_v || (v == top_v && n < top_i)) {
            top_v = v;
            top_i = n;
          }
        }
        // lane holds y[m = col][n = 16*tile + 4*grp + i] (storing whole lines of a row instead,
        // turned through LDS, changed nothing: the kernel's time is the table's)
        if (col < M) *reinterpret_cast<float4v*>(out + (int64_t)col * ldo + tile * 16 + 4 * grp) = y;
      }
    }
  }
  if (best_val != nullptr && ks == 0) {
    // part blockIdx.x of row col: the best of the four lanes that hold the row's logits
#pragma unroll
    for (int m = 16; m < 64; m <<= 1) {
      const float ov = __shfl_xor(top_v, m, 64);
      const int oi = __shfl_xor(top_i, m, 64);
      if (ov > top_v || (ov == top_v && oi < top_i)) {
        top_v = ov;
        top_i = oi;
      }
    }
    if (grp == 0 && col < M) {
      best_val[(int64_t)col * gridDim.x + blockIdx.x] = top_v;
      best_idx[(int64_t)col * gridDim.x + blockIdx.x] = top_i;
    }
  }
}

}  // namespace

// Whether dli_head_gemm takes this product: at most 16 rows, whole tiles, K = 512 * (2, 4, 6 or 8).
extern "C" int dli_head_gemm_supports(int M, int N, int K) {
  return M > 0 && M <= 16 && N > 0 && N % 16 == 0 && K > 0 && K % 1024 == 0 && K <= 4096;
}

// x bfloat16 [M][K] (row stride ldx, a multiple of 8), w_tiled bfloat16 [N][K] in tile order,
// out float32 [M][N] (row stride ldo, a multiple of 4). norm_w float32 [K] or null (then xhat = x);
// ssq_in float32 [ssq_parts][M]. workgroups: how many stay for the launch (0: one per compute unit,
// which is ahead of two and more at every row count: 93 against 96 us at 8 rows, 97 against 100 at 16).
// best_val / best_idx (both or neither): [M][dli_head_gemm_workgroups(N, workgroups)], each row's best
// logit and its lowest index among the logits of each workgroup (the first stage of an argmax).
extern "C" int dli_head_gemm_workgroups(int N, int workgroups) {
  const int pairs = (N / 16 + 1) / 2;
  const int grid = workgroups > 0 ? workgroups : dli_compute_units();
  return grid > pairs ? pairs : grid;
}

extern "C" int dli_head_gemm(const void* x, int64_t ldx, const float* ssq_in, int ssq_parts, const float* norm_w,
                             float eps, const void* w_tiled, float* out, int64_t ldo, int M, int N, int K,
                             int workgroups, float* best_val, int* best_idx, hipStream_t stream) {
  if (M <= 0 || N <= 0) return DLI_OK;
  if ((best_val == nullptr) != (best_idx == nullptr)) return DLI_ERR_ARGUMENT;
  if (!dli_head_gemm_supports(M, N, K) || x == nullptr || w_tiled == nullptr || out == nullptr || ldx % 8 != 0 ||
      ldx < K || ldo % 4 != 0 || ldo < N || workgroups < 0 ||
      (norm_w != nullptr && (ssq_in == nullptr || ssq_parts <= 0)))
    return DLI_ERR_ARGUMENT;
  const int grid = dli_head_gemm_workgroups(N, workgroups);
#define HEAD_CASE(KB)                                                                                          \
  case KB:                                                                                                     \
    if (norm_w != nullptr)                                                                                     \
      head_gemm_kernel<KB, true><<<grid, HEAD_KS * 64, 0, stream>>>((const bf16_t*)x, ldx, ssq_in, ssq_parts,   \
                                                                   norm_w, eps, (const bf16_t*)w_tiled, out,   \
                                                                   ldo, M, N, K, best_val, best_idx);          \
    else                                                                                                       \
      head_gemm_kernel<KB, false><<<grid, HEAD_KS * 64, 0, stream>>>((const bf16_t*)x, ldx, ssq_in, ssq_parts,  \
                                                                    norm_w, eps, (const bf16_t*)w_tiled, out,  \
                                                                    ldo, M, N, K, best_val, best_idx);         \
    break;
  switch (K / (128 * HEAD_KS)) {
    HEAD_CASE(2) HEAD_CASE(4) HEAD_CASE(6) HEAD_CASE(8)
    default: return DLI_ERR_ARGUMENT;
  }
#undef HEAD_CASE
  return dli_launch_status();
}
