// Matrix product for a decode step of 17 to 64 rows (it takes 1 to 64):
//   y[m][n] = sum_k xhat[m][k] * w[n][k]
// k is walked in blocks of 128; where k is no multiple of 128 the last block is part empty: the
// activations past k count as zeros (so what the weights hold there does not matter, as long as
// it is finite: row by row it is the next row's start, in tile order the copy's zero filling).
// With this many rows the activations are no longer small beside the weights: a workgroup that
// owns few features and reads every row for them moves more activation bytes than weight bytes.
// So the activations of a block of 128 k are brought into LDS once per workgroup (normalised on
// the way, if a norm is asked for) and shared by its waves, each of which owns 16 features (two
// sets of 16 for the gated product), and k is split over workgroups (grid.y) until the launch
// fills the chip. A split launch leaves its 32-bit partial products in [split][m][n]; the
// elementwise kernel that has to run after the product anyway (residual sum, or rotation and
// cache write) adds them up in the order of the splits, so the result does not depend on timing.
//
// Products run on the matrix cores as in the kernel for few rows:
//   acc[16 n x 16 m] += W[16 n x 32 k] * xhat^T[32 k x 16 m]      (v_mfma_f32_16x16x32_bf16)
// lane l supplies feature/row l%16 and eight k values; inside a block of 128 k lane group g = l/16
// takes the run [32g, 32g+32) and product q of the block its q-th run of eight (the same
// permutation for both operands). Weights come either row by row or in the tile order
//   t[tile][block][q][g][c][8] = w[16*tile + c][128*block + 32*g + 8*q + (0..7)]
// (every load of a wave is then 1 KB of consecutive memory); both are a base and two strides here.
// Weight loads go straight to registers, two blocks ahead of their use.
//
//   norm        xhat = cast(norm_w[k] * cast(x[m][k] * rs[m])), rs[m] = rsqrt(sum_k x^2 / K + eps)
//               from the parts of the row's sum of squares that the producer of x left
//               (RMSNorm: src/dli/model/llama.py:40-44); otherwise xhat = x
//   MID_PARTIAL float32 [split][m][n], no bias
//   MID_STORE   cast(y + bias)                                  (one split only)
//   MID_SWIGLU  cast(silu(cast(gate))) * cast(up), rows n and n + up_offset of w
//               (src/dli/model/llama.py:190)                    (one split only)
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float float4v __attribute__((ext_vector_type(4)));

enum { MID_PARTIAL = 0, MID_SWIGLU = 1, MID_STORE = 2 };

namespace {

__device__ __forceinline__ float4v mfma32(bf16x8 a, bf16x8 b, float4v c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ bf16x8 as_bf16x8(u32x4 raw) {
  union {
    u32x4 r;
    bf16x8 v;
  } u;
  u.r = raw;
  return u.v;
}

constexpr int XPAD = 8;                // elements: rows of the staged block start 16 bytes apart in the banks
constexpr int XROW = 128 + XPAD;

struct MidArgs {
  const bf16_t* x; int64_t ldx;
  const float* ssq_in; int ssq_parts; const float* norm_w; float eps;
  const bf16_t* w; int tiled; int w_rows;
  const bf16_t* bias; void* out; int64_t ldo;
  int M, N, K, up_offset, splits;
};

// MT row tiles of 16; NW x KW waves: wave (nw, kw) owns 16 features (NW tiles a workgroup) and
// every KW-th block of the workgroup's range of k, so that a compute unit has many waves, each
// with its next blocks of weights in flight, from the first cycle on: these launches last only a
// few trips to memory, and what bounds them is how many bytes are under way. The NW waves of one
// kw share that block's activations through LDS; the KW partial tiles of a feature tile meet in
// LDS at the end and are added in the order of kw. grid (ceil(tiles / NW), splits).
template <int MT, int NW, int KW, int EPI>
__global__ __launch_bounds__(NW * KW * 64) void mid_gemm_kernel(MidArgs p) {
  constexpr int NA = EPI == MID_SWIGLU ? 2 : 1;
  constexpr int NG = NW * 64;          // threads that stage one kw's blocks
  constexpr int ROWS = 16 * MT;
  constexpr int PP = ROWS * 16 / NG;   // 16-byte pieces of a block that one thread stages
  static_assert(ROWS * 16 % NG == 0, "the block's pieces divide among the threads");
  constexpr int XS_BYTES = 2 * KW * ROWS * XROW * 2;
  constexpr int RED_BYTES = (KW - 1) * NW * NA * MT * 4 * 64 * 4;
  __shared__ __attribute__((aligned(16))) char smem[XS_BYTES > RED_BYTES ? XS_BYTES : RED_BYTES];
  __shared__ float rs_s[ROWS];
  typedef bf16_t XBuf[KW][ROWS][XROW];
  XBuf* xs = reinterpret_cast<XBuf*>(smem);                     // xs[buffer][kw][row][k]

  const int lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  const int nw = wave % NW, kw = wave / NW;
  const int gtid = threadIdx.x % NG;   // thread within the kw group (its waves are consecutive)
  const int col = lane % 16, grp = lane / 16;
  const int M = p.M, N = p.N, K = p.K;
  const int tiles = (N + 15) / 16;
  const int tile = blockIdx.x * NW + nw;
  const bool owns = tile < tiles;
  const int split = blockIdx.y;
  const int nblk = (K + 127) / 128;
  const int b0 = (int)((int64_t)nblk * split / p.splits), b1 = (int)((int64_t)nblk * (split + 1) / p.splits);
  const int cnt = b1 - b0;
  const int steps = (cnt + KW - 1) / KW;       // the same for every wave: all keep the barriers
  // Workgroups start at different blocks of their range and wrap around: launched together and
  // running in step, they would otherwise all ask for the same offsets inside their weights'
  // 64 KB regions (and for the same activations) at the same time, which lands on few memory
  // channels. The order of a feature's sum thus depends on its tile, never on the rows.
  const int rot = (int)((blockIdx.x * 5u + blockIdx.y * 3u) % (unsigned)cnt);
  // whether this wave has a block in this step (the last step of an uneven split may have none)
  auto live = [&](int step) { return step * KW + kw < cnt; };
  auto block_of = [&](int step) {  // always a block of the range: where there is none, the last
    const int r = min(step * KW + kw, cnt - 1) + rot;
    return b0 + (r >= cnt ? r - cnt : r);
  };

  // Weights and activations are read through buffer resources that end with the matrix and with
  // the last row: a load that is not wanted (a step without a block, a row that does not exist)
  // is sent past the end, where it returns zeros and costs no memory traffic. So every step
  // issues the same loads, the number of loads on their way is known at every wait, and a step
  // waits for its own block only.
  const int KP = nblk * 128;           // a row of the tile-ordered copy: whole blocks
  const unsigned w_bytes = (unsigned)((int64_t)p.w_rows * (p.tiled ? KP : K) * 2);
  const __amdgpu_buffer_rsrc_t wres = __builtin_amdgcn_make_buffer_rsrc((void*)p.w, 0, w_bytes, 0x00020000);
  const unsigned x_bytes = (unsigned)(((int64_t)(M - 1) * p.ldx + K) * 2);
  const __amdgpu_buffer_rsrc_t xres = __builtin_amdgcn_make_buffer_rsrc((void*)p.x, 0, x_bytes, 0x00020000);
  // this lane's first weight fragment (byte offset) and the steps to the next block and product
  unsigned wbase[NA];
  const int blk_stride = p.tiled ? 4096 : 256, q_stride = p.tiled ? 1024 : 16;
#pragma unroll
  for (int a = 0; a < NA; ++a) {
    const int tl = min(tile, tiles - 1);
    if (p.tiled) {
      wbase[a] = (unsigned)(((int64_t)(tl + a * (p.up_offset / 16)) * 16 * KP + lane * 8) * 2);
    } else {
      const int n = min(tl * 16 + col, N - 1) + a * p.up_offset;
      wbase[a] = (unsigned)(((int64_t)n * K + grp * 32) * 2);
    }
  }
  bf16x8 wf[3][NA][4];
  auto load_w = [&](bf16x8 (&dst)[NA][4], int b, bool wanted) __attribute__((always_inline)) {
#pragma unroll
    for (int a = 0; a < NA; ++a)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const unsigned at = wanted ? wbase[a] + (unsigned)(b * blk_stride + q * q_stride) : w_bytes;
        dst[a][q] = as_bf16x8(__builtin_amdgcn_raw_buffer_load_b128(wres, (int)at, 0, 0));
      }
  };
  const bool norm = p.norm_w != nullptr;

  // staging: piece i of this thread is eight k of one row of its kw's block
  int prow[PP], pk[PP];
#pragma unroll
  for (int i = 0; i < PP; ++i) {
    const int piece = gtid + i * NG;
    prow[i] = piece / 16;
    pk[i] = (piece % 16) * 8;
  }
  // every piece of a thread covers the same eight columns of the block (the group's thread
  // count is a multiple of 16), so one pair of norm-weight vectors serves them all
  struct Staged {
    bf16x8 v[PP];
    float4v nw0, nw1;
  };
  const float* nw_at = norm ? p.norm_w : reinterpret_cast<const float*>(p.w);  // always readable
  auto fetch_x = [&](Staged& st, int b, bool wanted) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < PP; ++i) {
      const unsigned at = wanted && prow[i] < M && b * 128 + pk[i] < K
                              ? (unsigned)(((int64_t)prow[i] * p.ldx + b * 128 + pk[i]) * 2) : x_bytes;
      st.v[i] = as_bf16x8(__builtin_amdgcn_raw_buffer_load_b128(xres, (int)at, 0, 0));
    }
    // (without a norm the same two loads, of anything: no load hangs on a condition; past k the
    // last eight weights, for activations that are zero)
    const int nk = min(b * 128 + pk[0], K - 8);
    st.nw0 = *reinterpret_cast<const float4v*>(nw_at + nk);
    st.nw1 = *reinterpret_cast<const float4v*>(nw_at + nk + 4);
  };
  auto stash_x = [&](const Staged& st, int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < PP; ++i) {
      bf16x8 v = st.v[i];
      if (norm) {
        const float r = rs_s[prow[i]];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float normed = (float)(bf16_t)((float)st.v[i][e] * r);
          v[e] = (bf16_t)((e < 4 ? st.nw0[e] : st.nw1[e - 4]) * normed);
        }
      }
      *reinterpret_cast<bf16x8*>(&xs[buf][kw][prow[i]][pk[i]]) = v;
    }
  };

  float4v acc[NA][MT];
#pragma unroll
  for (int a = 0; a < NA; ++a)
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[a][t] = float4v{0.f, 0.f, 0.f, 0.f};

  // Memory answers in the order of the requests, so a wait for one load is a wait for all older
  // ones: the activations of a block are therefore requested before the weights of the same
  // step, two steps ahead like them, and what a step waits for is always the oldest request.
  // A wave whose block lies beyond the range (the last step of an uneven split) stages and
  // multiplies nothing but keeps every barrier.
  Staged sx[2];
  fetch_x(sx[0], block_of(0), live(0));
  load_w(wf[0], block_of(0), live(0));
  fetch_x(sx[1], block_of(1), live(1));
  load_w(wf[1], block_of(1), live(1));
  // rs[m] from the parts of sum x^2, added in the order of the parts
  if (norm) {
    for (int m = threadIdx.x; m < ROWS; m += NW * KW * 64) {
      float sum = 0.f;
      if (m < M)
        for (int part = 0; part < p.ssq_parts; ++part) sum += p.ssq_in[(int64_t)part * M + m];
      rs_s[m] = rsqrtf(sum / (float)K + p.eps);
    }
    __syncthreads();
  }
  if (live(0)) stash_x(sx[0], 0);
  __syncthreads();
  for (int s0 = 0; s0 < steps; s0 += 6) {
#pragma unroll
    for (int r = 0; r < 6; ++r) {
      const int step = s0 + r;
      if (step >= steps) break;
      const int buf = r & 1;
      fetch_x(sx[r & 1], block_of(step + 2), live(step + 2));   // the slot of this step's block, which lies in LDS by now
      load_w(wf[(r + 2) % 3], block_of(step + 2), live(step + 2));
      if (live(step)) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int t = 0; t < MT; ++t) {
            const bf16x8 xf = *reinterpret_cast<const bf16x8*>(&xs[buf][kw][16 * t + col][32 * grp + 8 * q]);
#pragma unroll
            for (int a = 0; a < NA; ++a) acc[a][t] = mfma32(wf[r % 3][a][q], xf, acc[a][t]);
          }
      }
      if (live(step + 1)) stash_x(sx[(r + 1) & 1], buf ^ 1);
      __syncthreads();
    }
  }

  // the kw waves of a feature tile hand their partial tiles to wave kw == 0, which adds them in
  // the order of kw (the staged activations are done with: their memory is reused)
  if constexpr (KW > 1) {
    typedef float Red[NW][NA][MT][4][64];
    Red* red = reinterpret_cast<Red*>(smem);
    if (kw != 0) {
#pragma unroll
      for (int a = 0; a < NA; ++a)
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
          for (int i = 0; i < 4; ++i) red[kw - 1][nw][a][t][i][lane] = acc[a][t][i];
    }
    __syncthreads();
    if (kw != 0) return;
#pragma unroll
    for (int a = 0; a < NA; ++a)
#pragma unroll
      for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          for (int k2 = 0; k2 < KW - 1; ++k2) acc[a][t][i] += red[k2][nw][a][t][i][lane];
  }

  // lane holds y[m = 16t + col][n = 16*tile + 4*grp + i]
  if (!owns) return;
  const int nb = tile * 16 + 4 * grp;
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = 16 * t + col;
    if (m >= M || nb >= N) continue;
    if constexpr (EPI == MID_PARTIAL) {
      float* dst = reinterpret_cast<float*>(p.out) + ((int64_t)split * M + m) * p.ldo + nb;
      if (nb + 3 < N) {
        *reinterpret_cast<float4v*>(dst) = acc[0][t];
      } else {
        for (int i = 0; i < 4 && nb + i < N; ++i) dst[i] = acc[0][t][i];
      }
    } else {
      bf16_t* dst = reinterpret_cast<bf16_t*>(p.out) + (int64_t)m * p.ldo + nb;
      bf16_t r[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = min(nb + i, N - 1);
        float y0 = acc[0][t][i];
        if (p.bias != nullptr) y0 += (float)p.bias[n];
        if constexpr (EPI == MID_SWIGLU) {
          float y1 = acc[NA - 1][t][i];
          if (p.bias != nullptr) y1 += (float)p.bias[n + p.up_offset];
          const float g = (float)(bf16_t)y0, u = (float)(bf16_t)y1;
          r[i] = (bf16_t)((float)(bf16_t)silu<bf16_t>(g) * u);
        } else {
          r[i] = (bf16_t)y0;
        }
      }
      if (nb + 3 < N) {
        *reinterpret_cast<bf16x4*>(dst) = bf16x4{r[0], r[1], r[2], r[3]};
      } else {
        for (int i = 0; i < 4 && nb + i < N; ++i) dst[i] = r[i];
      }
    }
  }
}

// The splits' values of four neighbouring features, added in the order of the splits. The first
// eight are asked for together and without conditions (a split past the last reads the last and
// is not added), apart from their sum, so that a kernel can ask for everything it needs before it
// waits for anything; further splits follow eight at a time.
struct Splits8 {
  float4v v[8];
};
__device__ __forceinline__ Splits8 load_splits(const float* __restrict__ src, int splits, int64_t split_stride) {
  Splits8 s;
#pragma unroll
  for (int u = 0; u < 8; ++u) s.v[u] = *reinterpret_cast<const float4v*>(src + min(u, splits - 1) * split_stride);
  return s;
}
__device__ __forceinline__ float4v sum_splits(const Splits8& first, const float* __restrict__ src, int splits,
                                              int64_t split_stride) {
  float4v y = first.v[0];
#pragma unroll
  for (int u = 1; u < 8; ++u)
    if (u < splits) {
#pragma unroll
      for (int i = 0; i < 4; ++i) y[i] = y[i] + first.v[u][i];
    }
  for (int s0 = 8; s0 < splits; s0 += 8) {
    float4v v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = *reinterpret_cast<const float4v*>(src + min(s0 + u, splits - 1) * split_stride);
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (s0 + u < splits) {
#pragma unroll
        for (int i = 0; i < 4; ++i) y[i] = y[i] + v[u][i];
      }
  }
  return y;
}

// stream[m][n] = cast(stream[m][n] + cast(sum_s partial[s][m][n] + bias[n])), the splits added in
// their order, and ssq_out[part][m] = the sum of stream[m][n]^2 over the part's 1024 features, for
// the norm that follows. One workgroup per row and part.
__global__ __launch_bounds__(256) void mid_finish_residual_kernel(
    const float* __restrict__ partial, int splits, const bf16_t* __restrict__ bias,
    bf16_t* __restrict__ stream, int64_t lds_, float* __restrict__ ssq_out, int M, int N) {
  __shared__ float scratch[16];
  const int m = blockIdx.x, part = blockIdx.y;   // a part of a row: 1024 features
  const int64_t split_stride = (int64_t)M * N;
  const int n = part * 1024 + threadIdx.x * 4;
  float sq = 0.f;
  // (a thread past the row's end reads the row's last four features, for nothing)
  const int nc = min(n, N - 4);
  const bf16x4 old = *reinterpret_cast<const bf16x4*>(stream + (int64_t)m * lds_ + nc);
  const Splits8 first = load_splits(partial + (int64_t)m * N + nc, splits, split_stride);
  if (n < N) {
    bf16_t* sp = stream + (int64_t)m * lds_ + n;
    const float4v y = sum_splits(first, partial + (int64_t)m * N + n, splits, split_stride);
    bf16x4 res;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float b = bias != nullptr ? (float)bias[n + i] : 0.f;
      res[i] = (bf16_t)((float)old[i] + (float)(bf16_t)(y[i] + b));
      sq += (float)res[i] * (float)res[i];
    }
    *reinterpret_cast<bf16x4*>(sp) = res;
  }
  const float total = block_sum(sq, scratch);
  if (threadIdx.x == 0) ssq_out[(int64_t)part * M + m] = total;
}

// The same, and the row normalised for the product that reads it next, so that none of that
// product's 256 workgroups has to normalise all rows again: one workgroup per row holds the row's
// new values in registers (PER x 1024 features at most), adds up its squares and writes
// normed[m][n] = cast(norm_w[n] * cast(stream[m][n] * rs)), rs = rsqrt(sum / N + eps)
// (src/dli/model/llama.py:40-44). ssq_out[m] gets the row's whole sum.
template <int PER>
__global__ __launch_bounds__(256) void mid_finish_residual_normed_kernel(
    const float* __restrict__ partial, int splits, const bf16_t* __restrict__ bias,
    bf16_t* __restrict__ stream, int64_t lds_, float* __restrict__ ssq_out,
    const float* __restrict__ norm_w, float eps, bf16_t* __restrict__ normed, int64_t ldn, int M, int N) {
  __shared__ float scratch[16];
  const int m = blockIdx.x;
  const int64_t split_stride = (int64_t)M * N;
  bf16x4 res[PER], old[PER];
  float4v nw[PER], y[PER];
  // every load of the row is asked for before the first is used: the stream's old values, the
  // norm's weights, and the splits CH at a time for all of the thread's features
  constexpr int CH = PER <= 2 ? 8 : (PER <= 4 ? 4 : 2);
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int n = (j * 256 + threadIdx.x) * 4;
    const int nc = min(n, N - 4);  // past the row's end: its last four features, for nothing
    y[j] = float4v{0.f, 0.f, 0.f, 0.f};
    old[j] = *reinterpret_cast<const bf16x4*>(stream + (int64_t)m * lds_ + nc);
    nw[j] = *reinterpret_cast<const float4v*>(norm_w + nc);
  }
  for (int s0 = 0; s0 < splits; s0 += CH) {
    float4v v[PER][CH];
#pragma unroll
    for (int j = 0; j < PER; ++j) {
      const int n = (j * 256 + threadIdx.x) * 4;
#pragma unroll
      for (int u = 0; u < CH; ++u)  // no load under a condition: a split past the last reads the last
        v[j][u] = *reinterpret_cast<const float4v*>(partial + min(s0 + u, splits - 1) * split_stride +
                                                    (int64_t)m * N + min(n, N - 4));
    }
#pragma unroll
    for (int j = 0; j < PER; ++j)
#pragma unroll
      for (int u = 0; u < CH; ++u)
        if (s0 + u < splits) {
#pragma unroll
          for (int i = 0; i < 4; ++i) y[j][i] = s0 + u == 0 ? v[j][u][i] : y[j][i] + v[j][u][i];
        }
  }
  float sq = 0.f;
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int n = (j * 256 + threadIdx.x) * 4;
    if (n < N) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float b = bias != nullptr ? (float)bias[n + i] : 0.f;
        res[j][i] = (bf16_t)((float)old[j][i] + (float)(bf16_t)(y[j][i] + b));
        sq += (float)res[j][i] * (float)res[j][i];
      }
      *reinterpret_cast<bf16x4*>(stream + (int64_t)m * lds_ + n) = res[j];
    }
  }
  const float total = block_sum(sq, scratch);
  if (threadIdx.x == 0) ssq_out[m] = total;
  const float rs = rsqrtf(total / (float)N + eps);
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int n = (j * 256 + threadIdx.x) * 4;
    if (n < N) {
      bf16x4 out;
#pragma unroll
      for (int i = 0; i < 4; ++i) out[i] = (bf16_t)(nw[j][i] * (float)(bf16_t)((float)res[j][i] * rs));
      *reinterpret_cast<bf16x4*>(normed + (int64_t)m * ldn + n) = out;
    }
  }
}

// The fused q/k/v projection's partial products [split][m][n], n in the feature order of the
// product that rotates (tile t of a q or k head holds the head's dimensions 8t..8t+7 and
// half+8t..half+8t+7; v heads in their own order): the splits are added in their order, the bias
// (same order) joins, q and k are rotated (src/dli/model/rope.py:50-70: pairs (i, i + half), cos
// and sin of the row's position from `angles` [M][2][half]), q goes to out[m][head*d + dim] and
// rotated k and v to the cache pages at slots[m] (negative: not cached). grid (rows, workgroups
// that share a row's items); an item is four rotary pairs of a head, or four dimensions of a v head.
__global__ __launch_bounds__(256) void mid_finish_qkv_kernel(
    const float* __restrict__ partial, int splits, const bf16_t* __restrict__ bias,
    const float* __restrict__ angles, const int* __restrict__ slots, bf16_t* __restrict__ out,
    int64_t ldo, bf16_t* __restrict__ k_pages, bf16_t* __restrict__ v_pages, int M, int q_heads,
    int kv_heads, int d, int page_size) {
  const int m = blockIdx.x;
  const int half = d / 2, N = (q_heads + 2 * kv_heads) * d;
  const int64_t split_stride = (int64_t)M * N;
  const int rot_items = (q_heads + kv_heads) * (half / 4), v_items = kv_heads * (d / 4);
  const int slot = slots[m];
  const int64_t page = slot >= 0 ? slot / page_size : 0;
  const int off = slot >= 0 ? slot - (int)page * page_size : 0;
  auto summed = [&](const Splits8& first, int n) __attribute__((always_inline)) {
    float4v y = sum_splits(first, partial + (int64_t)m * N + n, splits, split_stride);
#pragma unroll
    for (int i = 0; i < 4; ++i) y[i] = (float)(bf16_t)(y[i] + (bias != nullptr ? (float)bias[n + i] : 0.f));
    return y;
  };
  for (int item = blockIdx.y * 256 + threadIdx.x; item < rot_items + v_items; item += 256 * gridDim.y) {
    if (item < rot_items) {
      const int head = item / (half / 4), j = (item % (half / 4)) * 4;   // pairs j..j+3 of the head
      const int pos = head * d + 16 * (j / 8) + j % 8;                   // where pair j's first member lies
      // both members' splits and the angles are asked for before any of them is used
      const Splits8 fa = load_splits(partial + (int64_t)m * N + pos, splits, split_stride);
      const Splits8 fb = load_splits(partial + (int64_t)m * N + pos + 8, splits, split_stride);
      const float4v cs = *reinterpret_cast<const float4v*>(angles + ((int64_t)m * 2 + 0) * half + j);
      const float4v sn = *reinterpret_cast<const float4v*>(angles + ((int64_t)m * 2 + 1) * half + j);
      __builtin_amdgcn_sched_barrier(0);
      const float4v a = summed(fa, pos), b = summed(fb, pos + 8);
      bf16x4 lo, hi;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        lo[i] = (bf16_t)(a[i] * cs[i] - b[i] * sn[i]);
        hi[i] = (bf16_t)(b[i] * cs[i] + a[i] * sn[i]);
      }
      bf16_t* dst = nullptr;
      if (head < q_heads) dst = out + (int64_t)m * ldo + head * d + j;
      else if (slot >= 0) dst = k_pages + ((page * kv_heads + (head - q_heads)) * page_size + off) * d + j;
      if (dst != nullptr) {
        *reinterpret_cast<bf16x4*>(dst) = lo;
        *reinterpret_cast<bf16x4*>(dst + half) = hi;
      }
    } else if (slot >= 0) {
      const int vi = item - rot_items, hv = vi / (d / 4), dim = (vi % (d / 4)) * 4;
      const int pos = (q_heads + kv_heads + hv) * d + dim;
      const float4v v = summed(load_splits(partial + (int64_t)m * N + pos, splits, split_stride), pos);
#pragma unroll
      for (int i = 0; i < 4; ++i)
        v_pages[((page * kv_heads + hv) * d + dim + i) * page_size + off] = (bf16_t)v[i];
    }
  }
}

// The workgroup shapes that are built: four feature tiles a workgroup with one or two waves on
// each for the plain products, two tiles with one, two or four waves on each for the gated one
// (whose waves hold two sets of weights). Others are refused.
template <int MT, int EPI>
int launch_mid(int nw, int kw, const MidArgs& a, hipStream_t stream) {
  const int tiles = (a.N + 15) / 16;
  const dim3 grid((tiles + nw - 1) / nw, a.splits);
#define MID_CASE(NW_, KW_)                                                              \
  if (nw == NW_ && kw == KW_) {                                                         \
    mid_gemm_kernel<MT, NW_, KW_, EPI><<<grid, NW_ * KW_ * 64, 0, stream>>>(a);         \
    return dli_launch_status();                                                         \
  }
  if constexpr (EPI == MID_SWIGLU) {
    MID_CASE(2, 1) MID_CASE(2, 2) MID_CASE(2, 4)
  } else {
    MID_CASE(4, 1) MID_CASE(4, 2)
  }
#undef MID_CASE
  return DLI_ERR_ARGUMENT;
}

template <int EPI>
int launch_mid_rows(int nw, int kw, const MidArgs& a, hipStream_t stream) {
  if (a.M <= 16) return launch_mid<1, EPI>(nw, kw, a, stream);
  if (a.M <= 32) return launch_mid<2, EPI>(nw, kw, a, stream);
  if (a.M <= 48) return launch_mid<3, EPI>(nw, kw, a, stream);
  return launch_mid<4, EPI>(nw, kw, a, stream);
}

}  // namespace

// x [M, K] bfloat16 (row stride ldx), M <= 64, K % 8 == 0. w: [N (+ up part), K] row by row, or
// in tile order if `tiled` (then N % 16 == 0 and up_offset % 16 == 0, and a row of the copy is K
// rounded up to whole blocks of 128, zeros past K). norm_w == nullptr: no norm.
// epilogue 0: out is float32 [splits][M][N] (ldo == N); 1 (gated) and 2 (store): out is bfloat16
// [M][N] with row stride ldo, one split. waves: feature tiles per workgroup; kwaves: waves that
// share a feature tile and split the workgroup's k (the built pairs are listed in launch_mid).
extern "C" int dli_mid_gemm(const void* x, int64_t ldx, const float* ssq_in, int ssq_parts,
                            const float* norm_w, float eps, const void* w, int tiled, const void* bias,
                            void* out, int64_t ldo, int M, int N, int K, int up_offset, int epilogue,
                            int splits, int waves, int kwaves, hipStream_t stream) {
  if (M <= 0 || N <= 0) return DLI_OK;
  if (M > 64 || K <= 0 || K % 8 != 0 || ldx % 8 != 0 || ldx < K || out == nullptr || epilogue < 0 ||
      epilogue > 2 || splits < 1 || splits > (K + 127) / 128 || waves < 1 || kwaves < 1 ||
      (epilogue != MID_PARTIAL && splits != 1) || (epilogue == MID_PARTIAL && (ldo != N || bias != nullptr)) ||
      (epilogue != MID_PARTIAL && (ldo < N || ldo % 4 != 0)) ||
      (norm_w != nullptr && (ssq_in == nullptr || ssq_parts <= 0)) ||
      (tiled && (N % 16 != 0 || up_offset % 16 != 0)) || (epilogue == MID_SWIGLU && up_offset <= 0) ||
      (epilogue == MID_PARTIAL && N % 4 != 0))
    return DLI_ERR_ARGUMENT;
  // the kernel addresses the matrix and the rows with 32-bit byte offsets
  const int64_t w_rows = epilogue == MID_SWIGLU ? (int64_t)up_offset + N : N;
  if (w_rows * ((K + 127) / 128 * 128) * 2 >= ((int64_t)1 << 32) - 4096 || ((int64_t)(M - 1) * ldx + K) * 2 >= ((int64_t)1 << 31))
    return DLI_ERR_ARGUMENT;
  const MidArgs a{(const bf16_t*)x, ldx, ssq_in, ssq_parts, norm_w, eps, (const bf16_t*)w, tiled, (int)w_rows,
                  (const bf16_t*)bias, out, ldo, M, N, K, up_offset, splits};
  if (epilogue == MID_PARTIAL) return launch_mid_rows<MID_PARTIAL>(waves, kwaves, a, stream);
  if (epilogue == MID_SWIGLU) return launch_mid_rows<MID_SWIGLU>(waves, kwaves, a, stream);
  return launch_mid_rows<MID_STORE>(waves, kwaves, a, stream);
}

// partial: float32 [splits][M][N]; stream: bfloat16 [M][N] (row stride lds, a multiple of 4),
// updated in place; ssq_out: float32 [ceil(N / 1024)][M]. N % 4 == 0.
extern "C" int dli_mid_finish_residual(const float* partial, int splits, const void* bias, void* stream_buf,
                                       int64_t lds_, float* ssq_out, int M, int N, hipStream_t stream) {
  if (M <= 0 || N <= 0) return DLI_OK;
  if (partial == nullptr || stream_buf == nullptr || ssq_out == nullptr || splits < 1 || N % 4 != 0 ||
      lds_ < N || lds_ % 4 != 0)
    return DLI_ERR_ARGUMENT;
  mid_finish_residual_kernel<<<dim3(M, (N + 1023) / 1024), 256, 0, stream>>>(
      partial, splits, (const bf16_t*)bias, (bf16_t*)stream_buf, lds_, ssq_out, M, N);
  return dli_launch_status();
}

// The same with the normalised rows beside the stream: normed bfloat16 [M][N] (row stride ldn, a
// multiple of 4), norm_w float32 [N]; ssq_out float32 [1][M]. N at most 8192.
extern "C" int dli_mid_finish_residual_normed(const float* partial, int splits, const void* bias,
                                              void* stream_buf, int64_t lds_, float* ssq_out,
                                              const float* norm_w, float eps, void* normed, int64_t ldn,
                                              int M, int N, hipStream_t stream) {
  if (M <= 0 || N <= 0) return DLI_OK;
  if (partial == nullptr || stream_buf == nullptr || ssq_out == nullptr || norm_w == nullptr || normed == nullptr ||
      splits < 1 || N % 4 != 0 || N > 8192 || lds_ < N || lds_ % 4 != 0 || ldn < N || ldn % 4 != 0)
    return DLI_ERR_ARGUMENT;
#define FINISH_NORMED(PER)                                                                              \
  mid_finish_residual_normed_kernel<PER><<<M, 256, 0, stream>>>(partial, splits, (const bf16_t*)bias,   \
                                                                (bf16_t*)stream_buf, lds_, ssq_out, norm_w, \
                                                                eps, (bf16_t*)normed, ldn, M, N)
  const int per = (N + 1023) / 1024;
  if (per <= 1) FINISH_NORMED(1);
  else if (per <= 2) FINISH_NORMED(2);
  else if (per <= 4) FINISH_NORMED(4);
  else FINISH_NORMED(8);
#undef FINISH_NORMED
  return dli_launch_status();
}

// partial: float32 [splits][M][(q_heads + 2*kv_heads) * head_dim] in the feature order of the
// product that rotates; bias (optional) in the same order; angles float32 [M][2][head_dim/2];
// slots int32 [M]; out bfloat16 [M][>= q_heads*head_dim] (row stride ldo); pages as the attention
// kernels read them. head_dim % 16 == 0.
extern "C" int dli_mid_finish_qkv(const float* partial, int splits, const void* bias, const float* angles,
                                  const int* slots, void* out, int64_t ldo, void* k_pages, void* v_pages,
                                  int M, int q_heads, int kv_heads, int head_dim, int page_size,
                                  hipStream_t stream) {
  if (M <= 0) return DLI_OK;
  if (partial == nullptr || angles == nullptr || slots == nullptr || out == nullptr || k_pages == nullptr ||
      v_pages == nullptr || splits < 1 || q_heads <= 0 || kv_heads <= 0 || head_dim <= 0 ||
      head_dim % 16 != 0 || page_size <= 0 || ldo < (int64_t)q_heads * head_dim || ldo % 4 != 0)
    return DLI_ERR_ARGUMENT;
  const int items = (q_heads + kv_heads) * (head_dim / 8) + kv_heads * (head_dim / 4);
  mid_finish_qkv_kernel<<<dim3(M, (items + 255) / 256), 256, 0, stream>>>(partial, splits, (const bf16_t*)bias, angles, slots, (bf16_t*)out,
                                               ldo, (bf16_t*)k_pages, (bf16_t*)v_pages, M, q_heads, kv_heads,
                                               head_dim, page_size);
  return dli_launch_status();
}
