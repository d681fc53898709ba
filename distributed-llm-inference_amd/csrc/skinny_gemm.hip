// Matrix product for a few rows of activations (decode): y[m][n] = sum_k xhat[m][k] * w[n][k],
// m < 64, with the work that surrounds it in a decoder layer fused in, so that a layer needs few
// launches and the weights stream from HBM exactly once.
//
// One workgroup owns 16 output features (rows n of w) for all activation rows; its waves split k
// among themselves and add up through LDS in a fixed order. Products run on the matrix cores as
//   acc[16 n x 16 m] += W[16 n x 32 k] * xhat^T[32 k x 16 m]      (v_mfma_f32_16x16x32_bf16)
// where lane l supplies row/column l%16 and eight k values. Inside a block of 128 k the lane
// group g = l/16 takes the contiguous run [32g, 32g+32) and the four products of the block use its
// four runs of eight: the same permutation of k for both operands, so the sum is unchanged and a
// lane reads 64 contiguous bytes of its weight row.
//
// TILED: the weights are stored tile by tile instead of row by row, as
//   t[tile][block][q][g][c][8] = w[16*tile + c][128*block + 32*g + 8*q + (0..7)],
// so that the 16 features x 128 k of one tile and block are 4 KB of consecutive memory in the
// order in which the lanes take them (lane = 16*g + c) and every load of a wave is 1 KB of
// consecutive bytes. Needs K % 128 == 0 and whole tiles (N % 16 == 0, gate and up parts included).
//
// Fused in (template switches):
//   NORM     xhat = cast(norm_w[k] * cast(x[m][k] * rs[m])), rs[m] = rsqrt(sum_k x^2 / K + eps),
//            the row sums of squares being handed over in parts by the kernel that wrote x
//            (RMSNorm: src/dli/model/llama.py:40-44); otherwise xhat = x.
//   EPI_STORE     y (+ bias) stored as bf16
//   EPI_SWIGLU    two products per workgroup, rows n (gate) and n + up_offset (up) of w:
//                 stores cast(silu(gate)) * up (src/dli/model/llama.py:190)
//   EPI_RESIDUAL  stream[m][n] = cast(stream[m][n] + cast(y + bias)) in place (the residual sum, in
//                 32-bit), and this tile's part of sum_n stream[m][n]^2 for the norm that follows
//   EPI_F32       y stored as float32 (logits)
//   EPI_QKV       the fused q/k/v projection of a decode step with what follows it: rotary
//                 rotation of the q and k heads (src/dli/model/rope.py:50-70) and the write of the
//                 rotated keys and the values into the cache pages, so that no rotation kernel
//                 runs. TILED only, and the tile order of the q and k heads is a special one: tile
//                 t of a head holds its dimensions 8t..8t+7 and half+8t..half+8t+7, i.e. eight
//                 rotary pairs, whose partners sit 32 lanes apart in the product's result. q is
//                 stored to out in the usual order; k and v go to the pages only.
//   MERGED   the activations are not read from x but made in the kernel from the split-key partial
//            results of the decode attention (o_s, m_s, l_s per request, head and run of keys):
//            x[m][head*D + d] = cast(sum_s o_s[d] 2^(m_s - M) / sum_s l_s 2^(m_s - M)), the same
//            arithmetic in the same order as attention_merge_kernel, so that the o projection of a
//            step of one to four rows needs no merge kernel before it. Each wave merges the run of
//            k that it multiplies (all loads of a lane in flight at once) and hands it to its
//            lanes through LDS. TILED, EPI_RESIDUAL, at most 16 runs.
#include "common.h"
#include "merge_splits.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef float float2v __attribute__((ext_vector_type(2)));

enum { EPI_STORE = 0, EPI_SWIGLU = 1, EPI_RESIDUAL = 2, EPI_F32 = 3, EPI_QKV = 4 };

// What EPI_QKV needs beside the product: cos/sin of the rows' positions ([rows][2][head_dim/2]
// float32, rounded to bfloat16 values), the rows' cache slots (negative: not cached), the pages
// (K page [kv_heads][page_size][head_dim], V page [kv_heads][head_dim][page_size]) and the heads.
struct QkvRope {
  const float* angles;
  const int* slots;
  bf16_t* k_pages;
  bf16_t* v_pages;
  int q_heads, kv_heads, head_dim, page_size;
};

// What MERGED reads instead of x: part_o [rows][heads][splits][head_dim] and part_ml
// [rows][heads][splits][2] (running maximum in units of log2, sum) float32.
struct MergedIn {
  const float* part_o;
  const float* part_ml;
  int splits, heads, head_dim;
};
#define MERGE_ROWS 4     // rows of a step whose o projection merges by itself
#define MERGE_RANGE 512  // the longest run of k of one wave

__device__ __forceinline__ float4v mfma32(bf16x8 a, bf16x8 b, float4v c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

// Activation fragment of eight k values: the raw loads, and the norm applied afterwards (so the
// loads can be issued a block ahead of their use).
template <bool NORM>
struct XFrag {
  bf16x8 v;
  float4v w0, w1;
};
template <>
struct XFrag<false> {
  bf16x8 v;
};

template <bool NORM>
__device__ __forceinline__ XFrag<NORM> fetch_x(const bf16_t* __restrict__ xrow,
                                               const float* __restrict__ norm_w, int k) {
  XFrag<NORM> f;
  f.v = *reinterpret_cast<const bf16x8*>(xrow + k);
  if constexpr (NORM) {
    f.w0 = *reinterpret_cast<const float4v*>(norm_w + k);
    f.w1 = *reinterpret_cast<const float4v*>(norm_w + k + 4);
  }
  return f;
}

template <bool NORM>
__device__ __forceinline__ bf16x8 finish_x(const XFrag<NORM>& f, float rs) {
  if constexpr (!NORM) {
    return f.v;
  } else {
    bf16x8 v;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float normed = (float)(bf16_t)((float)f.v[i] * rs);
      v[i] = (bf16_t)((i < 4 ? f.w0[i] : f.w1[i - 4]) * normed);
    }
    return v;
  }
}

// KS waves split k, NS groups of waves split the workgroup's tiles, each wave owns NT tiles:
// a workgroup computes NS*NT tiles of 16 features with KS*NS waves. The activation fragments are
// loaded once per block of k and reused for the wave's NT tiles.
template <int KS, int NS, int NT, int MT, int EPI, bool NORM, bool TILED, bool MERGED = false>
__global__ __launch_bounds__(KS * NS * 64) void skinny_gemm_kernel(
    const bf16_t* __restrict__ x, int64_t ldx, const float* __restrict__ ssq_in, int ssq_parts,
    const float* __restrict__ norm_w, float eps, const bf16_t* __restrict__ w,
    const bf16_t* __restrict__ bias, void* __restrict__ out, int64_t ldo,
    bf16_t* __restrict__ stream, int64_t lds_, float* __restrict__ ssq_out, int M, int N, int K,
    int up_offset, QkvRope qr, MergedIn mi) {
  static_assert(EPI != EPI_QKV || (TILED && MT == 1), "the q/k/v epilogue reads tiled weights, at most 16 rows");
  static_assert(!MERGED || (TILED && MT == 1 && NS == 1 && !NORM), "merged activations: tiled weights, one row tile");
  // MERGED: each wave's run of k for up to MERGE_ROWS rows
  __shared__ __align__(16) bf16_t xs[MERGED ? KS : 1][MERGED ? MERGE_ROWS : 1][MERGED ? MERGE_RANGE : 8];
  constexpr int NA = EPI == EPI_SWIGLU ? 2 : 1;  // weight row sets per tile (gate and up)
  constexpr int KR = KS > 1 ? KS - 1 : 1;
  __shared__ float red[KR][NS][NT][NA][MT][4][64];  // k-split waves 1.. hand their tiles to wave 0

  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  const int ks = wave % KS, ns = wave / KS;
  const int col = lane % 16, grp = lane / 16;
  const int tile0 = (blockIdx.x * NS + ns) * NT;  // first of this wave's tiles

  // weight rows of this lane (clamped at the matrix's end: such rows are computed and dropped)
  const bf16_t* wrow[NT][NA];
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int a = 0; a < NA; ++a) {
      if constexpr (TILED) {
        // the tile's first block, at this lane's 16 bytes of a 1 KB load
        const int tile = min(tile0 + j, (N - 1) / 16) + a * (up_offset / 16);
        wrow[j][a] = w + (int64_t)tile * 16 * K + lane * 8;
      } else {
        const int n = min((tile0 + j) * 16 + col, N - 1) + a * up_offset;
        wrow[j][a] = w + (int64_t)n * K + grp * 32;
      }
    }
  // where a lane finds its eight k values of product q in the block that starts at step s
  auto w_at = [&](const bf16_t* base, int s, int q) __attribute__((always_inline)) {
    return reinterpret_cast<const bf16x8*>(TILED ? base + (s / 4) * 2048 + q * 512 : base + s * 32 + q * 8);
  };

  // EPI_RESIDUAL: the stream values that this lane will add to at the end (lane holds
  // y[m = 16t + col][n = 16*tile + 4*grp + i]) are asked for now, so that the epilogue does not
  // wait for a trip to memory of its own
  bf16_t old_s[EPI == EPI_RESIDUAL ? NT : 1][EPI == EPI_RESIDUAL ? MT : 1][4];
  if constexpr (EPI == EPI_RESIDUAL) {
    // In every wave and for every element (only the first k-split wave uses them; an element past
    // the edge reads the edge's and is not stored): a load under a condition is waited for on
    // the spot, one trip to memory after the other, and leaves the count of loads on their way
    // unknown to everything behind it.
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int n = (tile0 + j) * 16 + 4 * grp + i, m = t * 16 + col;
          old_s[j][t][i] = stream[(int64_t)min(m, M - 1) * lds_ + min(n, N - 1)];
        }
  }

  const bf16_t* xrow[MT];
  float rs[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = t * 16 + col;
    xrow[t] = x + (int64_t)min(m, M - 1) * ldx;
    rs[t] = 1.f;
  }
  float4v acc[NT][NA][MT];
#pragma unroll
  for (int j = 0; j < NT; ++j)
#pragma unroll
    for (int a = 0; a < NA; ++a)
#pragma unroll
      for (int t = 0; t < MT; ++t) acc[j][a][t] = float4v{0.f, 0.f, 0.f, 0.f};

  // this wave's share of the k steps of 32
  const int steps = K / 32;
  const int s_begin = TILED ? 4 * (int)((int64_t)(steps / 4) * ks / KS) : (int)((int64_t)steps * ks / KS);
  const int s_end = TILED ? 4 * (int)((int64_t)(steps / 4) * (ks + 1) / KS) : (int)((int64_t)steps * (ks + 1) / KS);
  int s = s_begin;
  // Blocks of 128: lane group g reads k in [32g, 32g + 32). The weights and activations of the
  // next block are asked for before the products of the current one. The two sets of registers
  // take turns in a loop that is written out for both, with the last block's products apart, so
  // that at every product the number of younger loads is known and the wait is for the block's
  // own loads alone (with one body for every turn, the turn without younger loads decides the
  // wait of all: each block was then waited for right after it had been asked for). Rows past
  // the last read the last row again (their results are dropped), so no load is conditional.
  struct Block {
    bf16x8 a[NT][NA][4];
    XFrag<NORM> x[MT][4];
  };
  auto fetch_weights = [&](Block& b, int at) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int a = 0; a < NA; ++a)
#pragma unroll
        for (int q = 0; q < 4; ++q) b.a[j][a][q] = *w_at(wrow[j][a], at, q);
  };
  auto fetch_rows = [&](Block& b, int at) __attribute__((always_inline)) {
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int q = 0; q < 4; ++q) b.x[t][q] = fetch_x<NORM>(xrow[t], norm_w, at * 32 + grp * 32 + q * 8);
  };
  auto multiply = [&](const Block& b) __attribute__((always_inline)) {
#pragma unroll
    for (int t = 0; t < MT; ++t) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const bf16x8 bf = finish_x<NORM>(b.x[t][q], rs[t]);
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
          for (int a = 0; a < NA; ++a) acc[j][a][t] = mfma32(b.a[j][a][q], bf, acc[j][a][t]);
      }
    }
  };
  int blocks = (s_end - s) / 4;
  Block b0, b1;
  if constexpr (NORM) {
    // rs[m] from the parts of sum x^2 that the producer of x left. The parts are dealt out to
    // all lane groups of all waves (group q of W*4 takes the parts q, q + 4W, ...), eight loads
    // at a time so that they share one trip to memory; a wave adds its four groups, the waves'
    // sums meet in LDS and are added in wave order. The first block of weights and rows is asked
    // for right behind the first eight parts and before anything waits for them, so that it is
    // on its way while the sums are made.
    constexpr int W = KS * NS;
    __shared__ float rsum[W][MT][16];
    float first[MT][8];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const int m = min(t * 16 + col, M - 1);
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        // no load is conditional (a part past the last reads the last and counts as zero), so
        // that the number of loads on their way is known where the first is waited for
        const int p = wave * 4 + grp + u * 4 * W;
        const float part = ssq_in[(int64_t)min(p, ssq_parts - 1) * M + m];
        first[t][u] = p < ssq_parts ? part : 0.f;
      }
    }
    // (a wave without a block of its own, k being short, reads the matrix's first block)
    if (TILED || blocks > 0) {
      fetch_rows(b0, blocks > 0 ? s : 0);
      fetch_weights(b0, blocks > 0 ? s : 0);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const int m = min(t * 16 + col, M - 1);
      float sum = 0.f;
#pragma unroll
      for (int u = 0; u < 8; ++u) sum += first[t][u];
      for (int p0 = wave * 4 + grp + 32 * W; p0 < ssq_parts; p0 += 32 * W) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int p = p0 + u * 4 * W;
          v[u] = p < ssq_parts ? ssq_in[(int64_t)p * M + m] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) sum += v[u];
      }
      sum += __shfl_xor(sum, 16, 64);
      sum += __shfl_xor(sum, 32, 64);
      if (grp == 0) rsum[wave][t][col] = sum;
    }
    __syncthreads();
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      float sum = 0.f;
#pragma unroll
      for (int wv = 0; wv < W; ++wv) sum += rsum[wv][t][col];
      rs[t] = rsqrtf(sum / (float)K + eps);
    }
  } else {
    if (blocks > 0) fetch_weights(b0, s);
  }
  if constexpr (MERGED) {
    // The wave's run of k, four values a lane and turn, merged as attention_merge_kernel does.
    const int kb0 = s_begin * 32, quads = (s_end - s_begin) * 8;
    const int D = mi.head_dim, S = mi.splits;
    for (int item = lane; item < M * quads; item += 64) {
      const int row = item / quads, idx = (item - row * quads) * 4;
      const int k = kb0 + idx, head = k / D, d = k - head * D;
      const int64_t base = ((int64_t)row * mi.heads + head) * S;
      const float4v merged = merged_quad(mi.part_o, mi.part_ml, base, S, D, d);
      bf16_t* dst = &xs[ks][row][idx];
#pragma unroll
      for (int i = 0; i < 4; ++i) dst[i] = (bf16_t)merged[i];
    }
    __syncthreads();
#pragma unroll
    for (int t = 0; t < MT; ++t) xrow[t] = &xs[ks][min(t * 16 + col, M - 1)][0] - kb0;
  }
  if constexpr (!NORM) {
    if (blocks > 0) fetch_rows(b0, s);
  }
  if constexpr (MT > 1) {
    // several row tiles: one body for every turn (the registers do not hold two whole blocks)
    for (; s + 4 <= s_end; s += 4) {
      const bool more = s + 8 <= s_end;
      if (more) {
        fetch_weights(b1, s + 4);
        fetch_rows(b1, s + 4);
      }
      multiply(b0);
      if (more) b0 = b1;
    }
  } else if (blocks > 0) {
    while (blocks >= 3) {
      fetch_rows(b1, s + 4);
      fetch_weights(b1, s + 4);
      __builtin_amdgcn_sched_barrier(0);  // all of the next block's loads leave before the products
      multiply(b0);
      fetch_rows(b0, s + 8);
      fetch_weights(b0, s + 8);
      __builtin_amdgcn_sched_barrier(0);
      multiply(b1);
      s += 8;
      blocks -= 2;
    }
    if (blocks == 2) {
      fetch_rows(b1, s + 4);
      fetch_weights(b1, s + 4);
      __builtin_amdgcn_sched_barrier(0);
      multiply(b0);
      multiply(b1);
    } else {
      multiply(b0);
    }
    s = s_begin + (s_end - s_begin) / 4 * 4;
  }
  for (; !TILED && s < s_end; ++s) {  // single steps: lane group g reads k in [8g, 8g + 8)
    const int kb = s * 32 + grp * 8;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const bf16x8 bf = finish_x<NORM>(fetch_x<NORM>(xrow[t], norm_w, kb), rs[t]);
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int a = 0; a < NA; ++a)
          acc[j][a][t] = mfma32(*reinterpret_cast<const bf16x8*>(wrow[j][a] - grp * 32 + kb), bf, acc[j][a][t]);
    }
  }

  // k-split wave 0 of each group adds the other waves' partial tiles to its own, in wave order
  if (KS > 1) {
    if (ks != 0) {
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int a = 0; a < NA; ++a)
#pragma unroll
          for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) red[ks - 1][ns][j][a][t][i][lane] = acc[j][a][t][i];
    }
    __syncthreads();
    if (ks == 0) {
#pragma unroll
      for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int a = 0; a < NA; ++a)
#pragma unroll
          for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              float v = acc[j][a][t][i];
              for (int wv = 0; wv < KS - 1; ++wv) v += red[wv][ns][j][a][t][i][lane];
              acc[j][a][t][i] = v;
            }
    }
  }

  // lane holds y[m = 16t + col][n = 16*tile + 4*grp + i]
  if (ks == 0) {
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    const int tile = tile0 + j;
    const int nb = tile * 16 + 4 * grp;
    if (tile * 16 >= N) continue;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const int m = t * 16 + col;
      float y[NA][4];
#pragma unroll
      for (int a = 0; a < NA; ++a)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          y[a][i] = acc[j][a][t][i];
          if (bias != nullptr && nb + i < N) y[a][i] += (float)bias[nb + i + a * up_offset];
        }
      if constexpr (EPI == EPI_QKV) {
        // all lanes take part in the exchange of partners; rows beyond M hold zeros
        const int d = qr.head_dim, half = d / 2;
        const int head = tile * 16 / d, t_in = (tile * 16 - head * d) / 16;
        const bool rotary = head < qr.q_heads + qr.kv_heads;
        const int mm = min(m, M - 1);
        const int slot = qr.slots[mm];
        float v[4], partner[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          v[i] = (float)(bf16_t)y[0][i];
          partner[i] = __shfl_xor(v[i], 32, 64);
        }
        if (rotary) {
          const int j = 8 * t_in + 4 * (grp & 1);  // first of this lane's four rotary pairs
          const float4v cs = *reinterpret_cast<const float4v*>(qr.angles + ((int64_t)mm * 2 + 0) * half + j);
          const float4v sn = *reinterpret_cast<const float4v*>(qr.angles + ((int64_t)mm * 2 + 1) * half + j);
          bf16_t r[4];
#pragma unroll
          for (int i = 0; i < 4; ++i)
            r[i] = grp < 2 ? (bf16_t)(v[i] * cs[i] - partner[i] * sn[i]) : (bf16_t)(v[i] * cs[i] + partner[i] * sn[i]);
          const int dim = (grp < 2 ? 0 : half) + j;
          bf16_t* dst = nullptr;
          if (head < qr.q_heads) {
            dst = reinterpret_cast<bf16_t*>(out) + (int64_t)m * ldo + head * d + dim;
          } else if (slot >= 0) {
            const int64_t page = slot / qr.page_size;
            const int off = slot - (int)page * qr.page_size;
            dst = qr.k_pages + ((page * qr.kv_heads + (head - qr.q_heads)) * qr.page_size + off) * d + dim;
          }
          if (m < M && dst != nullptr) {
            typedef bf16_t bf16x4 __attribute__((ext_vector_type(4)));
            *reinterpret_cast<bf16x4*>(dst) = bf16x4{r[0], r[1], r[2], r[3]};
          }
        } else if (m < M && slot >= 0) {
          const int64_t page = slot / qr.page_size;
          const int off = slot - (int)page * qr.page_size;
          const int hv = head - qr.q_heads - qr.kv_heads;
#pragma unroll
          for (int i = 0; i < 4; ++i)
            qr.v_pages[((page * qr.kv_heads + hv) * d + 16 * t_in + 4 * grp + i) * qr.page_size + off] = (bf16_t)v[i];
        }
        continue;
      }
      float sq = 0.f;
      if (m < M) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int n = nb + i;
          if (n >= N) continue;
          if (EPI == EPI_STORE) {
            reinterpret_cast<bf16_t*>(out)[(int64_t)m * ldo + n] = (bf16_t)y[0][i];
          } else if (EPI == EPI_F32) {
            reinterpret_cast<float*>(out)[(int64_t)m * ldo + n] = y[0][i];
          } else if (EPI == EPI_SWIGLU) {
            const float g = (float)(bf16_t)y[0][i], u = (float)(bf16_t)y[NA - 1][i];
            const float sg = (float)(bf16_t)silu<bf16_t>(g);
            reinterpret_cast<bf16_t*>(out)[(int64_t)m * ldo + n] = (bf16_t)(sg * u);
          } else {  // EPI_RESIDUAL
            bf16_t* sp = stream + (int64_t)m * lds_ + n;
            const bf16_t summed = (bf16_t)((float)old_s[EPI == EPI_RESIDUAL ? j : 0][EPI == EPI_RESIDUAL ? t : 0][i] + (float)(bf16_t)y[0][i]);
            *sp = summed;
            sq += (float)summed * (float)summed;
          }
        }
      }
      if (EPI == EPI_RESIDUAL) {
        sq += __shfl_xor(sq, 16, 64);
        sq += __shfl_xor(sq, 32, 64);
        if (grp == 0 && m < M) ssq_out[(int64_t)tile * M + m] = sq;
      }
    }
  }
  }
}

// Embedding rows with the sum of squares of each (one part), for the first layer's norm.
__global__ void embedding_ssq_kernel(const bf16_t* __restrict__ table, const int* __restrict__ ids,
                                     bf16_t* __restrict__ out, float* __restrict__ ssq, int width) {
  __shared__ float scratch[16];
  const int64_t row = blockIdx.x;
  const bf16_t* src = table + (int64_t)ids[row] * width;
  float s = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const bf16_t v = src[i];
    out[row * width + i] = v;
    s += (float)v * (float)v;
  }
  const float total = block_sum(s, scratch);
  if (threadIdx.x == 0) ssq[row] = total;
}

#define SK_PARAMS                                                                                 \
  const void *x, int64_t ldx, const float *ssq_in, int ssq_parts, const float *norm_w, float eps,   \
      const void *w, const void *bias, void *out, int64_t ldo, void *stream_buf, int64_t lds_,      \
      float *ssq_out, int M, int N, int K, int up_offset, QkvRope qr, hipStream_t stream
#define SK_ARGS \
  x, ldx, ssq_in, ssq_parts, norm_w, eps, w, bias, out, ldo, stream_buf, lds_, ssq_out, M, N, K, up_offset, qr, stream

template <int KS, int NS, int NT, int MT, int EPI, bool NORM, bool TILED>
static void launch_skinny(SK_PARAMS) {
  const int tiles = (N + 15) / 16;
  const int groups = (tiles + NS * NT - 1) / (NS * NT);
  skinny_gemm_kernel<KS, NS, NT, MT, EPI, NORM, TILED><<<groups, KS * NS * 64, 0, stream>>>(
      (const bf16_t*)x, ldx, ssq_in, ssq_parts, norm_w, eps, (const bf16_t*)w, (const bf16_t*)bias,
      out, ldo, (bf16_t*)stream_buf, lds_, ssq_out, M, N, K, up_offset, qr, MergedIn{});
}

// shapes of the workgroup: 0: 4 k-waves x 1 tile (few tiles, short k); 1: 8 k-waves x 1 tile (few
// tiles, long k); 2: 4 n-waves x 2 tiles, no k split (many tiles: the activations are read once
// per 8 tiles); 3: 2 k-waves x 2 n-waves x 2 tiles; 4: 4 k-waves x 2 tiles (many tiles in tile order)
template <int MT, int EPI, bool NORM, bool TILED>
static void dispatch_shape(int shape, SK_PARAMS) {
  switch (shape) {
    case 0: launch_skinny<4, 1, 1, MT, EPI, NORM, TILED>(SK_ARGS); break;
    case 1: launch_skinny<8, 1, 1, MT, EPI, NORM, TILED>(SK_ARGS); break;
    case 2: launch_skinny<1, 4, 2, MT, EPI, NORM, TILED>(SK_ARGS); break;
    case 4: launch_skinny<4, 1, 2, MT, EPI, NORM, TILED>(SK_ARGS); break;
    default: launch_skinny<2, 2, 2, MT, EPI, NORM, TILED>(SK_ARGS); break;
  }
}

// tiled weights serve the decode steps of few rows: one row tile only
template <int EPI, bool NORM>
static int dispatch_skinny(int shape, int mt, bool tiled, SK_PARAMS) {
  if (tiled) dispatch_shape<1, EPI, NORM, true>(shape, SK_ARGS);
  else if (mt == 1) dispatch_shape<1, EPI, NORM, false>(shape, SK_ARGS);
  else if (mt == 2) dispatch_shape<2, EPI, NORM, false>(shape, SK_ARGS);
  else dispatch_shape<4, EPI, NORM, false>(shape, SK_ARGS);
  return dli_launch_status();
}

extern "C" int dli_skinny_gemm_max_rows() { return 64; }

// epilogue: 0 store bf16, 1 swiglu (N = features of one half, up rows at +up_offset), 2 residual,
// 3 store float32. norm_w == nullptr: no norm. shape: the workgroup shape, see dispatch_shape.
// tiled: w is in the tile order described at the top (at most 16 rows, K % 128 == 0, whole tiles).
extern "C" int dli_skinny_gemm(const void* x, int64_t ldx, const float* ssq_in, int ssq_parts,
                               const float* norm_w, float eps, const void* w, const void* bias,
                               void* out, int64_t ldo, void* stream_buf, int64_t lds_,
                               float* ssq_out, int M, int N, int K, int up_offset, int epilogue,
                               int shape, int tiled, hipStream_t stream) {
  const QkvRope qr{};
  if (M <= 0 || N <= 0) return DLI_OK;
  if (tiled && (M > 16 || K % 128 != 0 || N % 16 != 0 || up_offset % 16 != 0)) return DLI_ERR_ARGUMENT;
  if (M > 64 || K <= 0 || K % 32 != 0 || ldx % 8 != 0 || shape < 0 || shape > 4 || epilogue < 0 ||
      epilogue > 3 || (norm_w != nullptr && (ssq_in == nullptr || ssq_parts <= 0)) ||
      (epilogue == EPI_RESIDUAL && (stream_buf == nullptr || ssq_out == nullptr || norm_w != nullptr)) ||
      (epilogue != EPI_RESIDUAL && out == nullptr))
    return DLI_ERR_ARGUMENT;
  const int mt = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
  const bool norm = norm_w != nullptr;
  switch (epilogue) {
    case EPI_STORE:
      return norm ? dispatch_skinny<EPI_STORE, true>(shape, mt, tiled != 0, SK_ARGS) : dispatch_skinny<EPI_STORE, false>(shape, mt, tiled != 0, SK_ARGS);
    case EPI_SWIGLU:
      return norm ? dispatch_skinny<EPI_SWIGLU, true>(shape, mt, tiled != 0, SK_ARGS) : dispatch_skinny<EPI_SWIGLU, false>(shape, mt, tiled != 0, SK_ARGS);
    case EPI_RESIDUAL:
      return dispatch_skinny<EPI_RESIDUAL, false>(shape, mt, tiled != 0, SK_ARGS);
    default:
      return norm ? dispatch_skinny<EPI_F32, true>(shape, mt, tiled != 0, SK_ARGS) : dispatch_skinny<EPI_F32, false>(shape, mt, tiled != 0, SK_ARGS);
  }
}

// The fused q/k/v projection of a decode step with rotation and cache write inside (EPI_QKV):
// w_tiled is the [(q_heads + 2*kv_heads) * head_dim, K] matrix in tile order with the q and k
// heads' tiles made of rotary pairs (see the top), bias (optional) in the same feature order.
// q goes to out[row][head*head_dim + dim] (row stride ldo), rotated; rotated k and v go to the
// pages at slots[row]. angles: [M][2][head_dim/2] float32 cos/sin of the rows' positions.
extern "C" int dli_skinny_gemm_qkv_rope(const void* x, int64_t ldx, const float* ssq_in, int ssq_parts,
                                        const float* norm_w, float eps, const void* w_tiled,
                                        const void* bias, void* out, int64_t ldo, const float* angles,
                                        const int* slots, void* k_pages, void* v_pages, int M, int K,
                                        int q_heads, int kv_heads, int head_dim, int page_size,
                                        int shape, hipStream_t stream) {
  if (M <= 0) return DLI_OK;
  if (M > 16 || K <= 0 || K % 128 != 0 || ldx % 8 != 0 || ldo % 8 != 0 || shape < 0 || shape > 4 ||
      q_heads <= 0 || kv_heads <= 0 || head_dim <= 0 || head_dim % 16 != 0 || page_size <= 0 ||
      out == nullptr || angles == nullptr || slots == nullptr || k_pages == nullptr ||
      v_pages == nullptr || (norm_w != nullptr && (ssq_in == nullptr || ssq_parts <= 0)))
    return DLI_ERR_ARGUMENT;
  const QkvRope qr{angles, slots, (bf16_t*)k_pages, (bf16_t*)v_pages, q_heads, kv_heads, head_dim, page_size};
  const int N = (q_heads + 2 * kv_heads) * head_dim, up_offset = 0;
  void* stream_buf = nullptr;
  float* ssq_out = nullptr;
  const int64_t lds_ = 0;
  const void* w = w_tiled;
  if (norm_w != nullptr) dispatch_shape<1, EPI_QKV, true, true>(shape, SK_ARGS);
  else dispatch_shape<1, EPI_QKV, false, true>(shape, SK_ARGS);
  return dli_launch_status();
}

// The o projection of a decode step of at most MERGE_ROWS rows, fed with the split-key partial
// results of the attention instead of its merged output (MERGED above): stream += merge(...) @ w^T
// (+ bias), and the parts of the rows' sums of squares. w_tiled [N, K] in tile order with
// K = heads * head_dim; splits 2..MERGE_SPLITS; shape 0 or 1 (4 or 8 waves split k).
extern "C" int dli_skinny_gemm_merged(const float* part_o, const float* part_ml, int splits, int heads,
                                      int head_dim, const void* w_tiled, const void* bias, void* stream_buf,
                                      int64_t lds_, float* ssq_out, int M, int N, int shape, hipStream_t stream) {
  if (M <= 0 || N <= 0) return DLI_OK;
  const int64_t K64 = (int64_t)heads * head_dim;
  if (M > MERGE_ROWS || splits < 2 || splits > MERGE_SPLITS || heads <= 0 || head_dim <= 0 || head_dim % 4 != 0 ||
      K64 % 128 != 0 || K64 > (1 << 20) || N % 16 != 0 || (shape != 0 && shape != 1) || part_o == nullptr ||
      part_ml == nullptr || w_tiled == nullptr || stream_buf == nullptr || ssq_out == nullptr)
    return DLI_ERR_ARGUMENT;
  const int K = (int)K64, ks = shape == 0 ? 4 : 8;
  if (((K / 128 + ks - 1) / ks) * 128 > MERGE_RANGE) return DLI_ERR_ARGUMENT;
  const MergedIn mi{part_o, part_ml, splits, heads, head_dim};
  const int groups = N / 16;
#define MERGED_LAUNCH(KS)                                                                          \
  skinny_gemm_kernel<KS, 1, 1, 1, EPI_RESIDUAL, false, true, true><<<groups, KS * 64, 0, stream>>>( \
      nullptr, 0, nullptr, 0, nullptr, 0.f, (const bf16_t*)w_tiled, (const bf16_t*)bias, nullptr, 0, \
      (bf16_t*)stream_buf, lds_, ssq_out, M, N, K, 0, QkvRope{}, mi)
  if (shape == 0) MERGED_LAUNCH(4);
  else MERGED_LAUNCH(8);
#undef MERGED_LAUNCH
  return dli_launch_status();
}

extern "C" int dli_skinny_gemm_merged_limits(int* rows, int* splits) {
  *rows = MERGE_ROWS;
  *splits = MERGE_SPLITS;
  return DLI_OK;
}

extern "C" int dli_embedding_ssq(const void* table, const int* ids, void* out, float* ssq, int rows,
                                 int width, hipStream_t stream) {
  if (rows <= 0) return DLI_OK;
  if (width <= 0) return DLI_ERR_ARGUMENT;
  embedding_ssq_kernel<<<rows, 256, 0, stream>>>((const bf16_t*)table, ids, (bf16_t*)out, ssq, width);
  return dli_launch_status();
}
