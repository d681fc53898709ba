// Matrix product for at most 16 rows of activations (decode): y[m][n] = sum_k xhat[m][k] * w[n][k],
// built around the memory system rather than the matrix cores: a decode product streams each
// weight once and is bound by how many bytes a compute unit's vector cache can accept per tag
// lookup, so every load here covers whole 64-byte runs.
//
// Products use v_mfma_f32_4x4x4_16B_bf16: sixteen independent 4x4x4 blocks per instruction. Lane
// l belongs to block l/4; as operand A it supplies row l%4 and four k values, as operand B column
// l%4 and four k values; the result gives it column l%4 and the four rows. Here the sixteen blocks
// are sixteen consecutive runs of eight k (a "chunk" of 128 k), rows are four neighbouring
// features (a "quad") and columns four activation rows: lane l loads the 16 bytes at k = chunk*128
// + 8*(l/4) of its feature's weight row, so that sixteen neighbouring lanes read four rows times 64
// contiguous bytes, and does two products (k halves) per quad and group of four activation rows.
// The blocks' partial sums are added at the end: lanes l, l^16, l^32, l^48 by lane swaps, the rest
// and the waves' shares of k through LDS, always in the same order.
//
// A workgroup has KS waves that split k among themselves and owns FQ quads of features. Few
// quads and many waves suit products with few features (every compute unit still gets a
// workgroup, and many loads are in flight on each); more quads read the activations less often.
//
// With XL the activations go through LDS: all threads of the workgroup read x once (whole lines),
// apply the norm there and then, and leave xhat in LDS, from where the waves take their fragments.
// The loop then holds no loads but the weights' and no arithmetic but the products. Used when
// rows * k fits (64 KB) and the product has many tiles (see launch4).
//
// Fused in (template switches), as in the product for more rows:
//   NORM          xhat = cast(norm_w[k] * cast(x[m][k] * rs[m])), rs[m] = rsqrt(sum_k x^2 / K + eps)
//                 from the parts of the row sums of squares that the producer of x left
//                 (RMSNorm: src/dli/model/llama.py:40-44)
//   EPI_STORE     y (+ bias) stored as bf16
//   EPI_SWIGLU    half of the quads are gate rows n, half up rows n + up_offset:
//                 stores cast(silu(gate)) * up (src/dli/model/llama.py:190)
//   EPI_RESIDUAL  stream[m][n] = cast(stream[m][n] + cast(y + bias)) in place, and this tile's part
//                 of sum_n stream[m][n]^2 for the norm that follows
//   EPI_F32       y stored as float32 (logits)
#include "common.h"

typedef short short4v __attribute__((ext_vector_type(4)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

enum { EPI_STORE = 0, EPI_SWIGLU = 1, EPI_RESIDUAL = 2, EPI_F32 = 3 };

union Frag16 {
  u32x4 raw;
  short4v h[2];
  bf16_t e[8];
};

__device__ __forceinline__ float4v mfma4(short4v a, short4v b, float4v c) {
  return __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(a, b, c, 0, 0, 0);
}

template <int KS, int FQ, int MG, int EPI, bool NORM, bool XL, int DEPTH>
__global__ __launch_bounds__(KS * 64) void skinny4_kernel(
    const bf16_t* __restrict__ x, int64_t ldx, const float* __restrict__ ssq_in, int ssq_parts,
    const float* __restrict__ norm_w, float eps, const bf16_t* __restrict__ w,
    const bf16_t* __restrict__ bias, void* __restrict__ out, int64_t ldo,
    bf16_t* __restrict__ stream, int64_t lds_, float* __restrict__ ssq_out, int M, int N, int K,
    int up_offset) {
  constexpr int PAIRS = FQ * MG;                        // (quad, row group) accumulators per lane
  constexpr int OQ = EPI == EPI_SWIGLU ? FQ / 2 : FQ;   // quads of output features per tile
  __shared__ float4v red[KS][PAIRS][16];
  __shared__ float4v fin[PAIRS][4];
  __shared__ float sqs[OQ][MG][4];
  extern __shared__ __attribute__((aligned(16))) bf16_t xs[];  // XL: xhat, rows of XPAD(K) values

  const int lane = threadIdx.x % 64, ks = threadIdx.x / 64;
  const int r = lane % 4, blk = lane / 4;
  const int tile = blockIdx.x;
  const int n_tile = tile * 4 * OQ;  // first output feature of the tile

  // EPI_RESIDUAL: the stream values that this thread will add to at the end are asked for now, so
  // that the epilogue does not wait for a trip to memory of its own (same thread, same places)
  union Pack4 {
    short4v v;
    bf16_t e[4];
  } old;
  old.v = short4v{0, 0, 0, 0};
  if (EPI == EPI_RESIDUAL) {
    const int t0 = threadIdx.x, p0 = t0 / 4, f0 = p0 / MG;
    const int m0 = 4 * (p0 % MG) + t0 % 4, nb0 = n_tile + 4 * f0;
    if (t0 < 4 * PAIRS && f0 < OQ && m0 < M && nb0 < N) {
      const bf16_t* sp = stream + (int64_t)m0 * lds_ + nb0;
      if (nb0 + 3 < N && lds_ % 4 == 0) {
        old.v = *reinterpret_cast<const short4v*>(sp);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) old.e[i] = nb0 + i < N ? sp[i] : (bf16_t)0.f;
      }
    }
  }

  // weight rows of this lane, one per quad (clamped at the matrix's end: computed and dropped)
  const bf16_t* wrow[FQ];
#pragma unroll
  for (int f = 0; f < FQ; ++f) {
    const int oq = f % OQ;
    const int n = min(n_tile + 4 * oq + r, N - 1) + (f / OQ) * up_offset;
    wrow[f] = w + (int64_t)n * K;
  }
  // activations through a buffer resource that ends after the last row: rows that do not exist
  // and k past the end read zeros and cause no memory traffic
  const unsigned x_bytes = (unsigned)(((int64_t)(M - 1) * ldx + K) * 2);
  const __amdgpu_buffer_rsrc_t xres = __builtin_amdgcn_make_buffer_rsrc((void*)x, 0, x_bytes, 0x00020000);
  int xrow[MG];
  float rs[MG];
#pragma unroll
  for (int g = 0; g < MG; ++g) {
    const int m = 4 * g + r;
    xrow[g] = m < M ? (int)(m * ldx * 2) : (int)x_bytes;  // past the end: what is added stays there
    rs[g] = 1.f;
  }
  float4v acc[FQ][MG];
#pragma unroll
  for (int f = 0; f < FQ; ++f)
#pragma unroll
    for (int g = 0; g < MG; ++g) acc[f][g] = float4v{0.f, 0.f, 0.f, 0.f};

  // chunks of 128 k: this wave's share
  const int chunks = (K + 127) / 128;
  const int c0 = chunks * ks / KS, c1 = chunks * (ks + 1) / KS;

  struct Stage {
    Frag16 wf[FQ], xf[MG];
    float4v g0, g1;
  };
  const int xpad = chunks * 128 + 32;  // XL: values per row of xs; rows 64 bytes apart in the banks
  // Every turn of the loop issues the same loads (a turn past the wave's last chunk reads the
  // last chunk's weights again and zeros for x), so the number of loads in flight is known at
  // compile time and only the current chunk is waited for.
  auto fetch = [&](int c, Stage& st) __attribute__((always_inline)) {
    const int k = max(min(c, c1 - 1), 0) * 128 + blk * 8;  // (a wave without chunks reads the first one, for nothing)
    const bool inside = k < K && c < c1;  // the last chunk may reach past k; K % 8 == 0
    const int kc = k < K ? k : 0;
#pragma unroll
    for (int f = 0; f < FQ; ++f) st.wf[f].raw = *reinterpret_cast<const u32x4*>(wrow[f] + kc);
    if constexpr (!XL) {
      const int k_at = inside ? k * 2 : (int)x_bytes;  // one offset for every case, no branch
#pragma unroll
      for (int g = 0; g < MG; ++g) st.xf[g].raw = __builtin_amdgcn_raw_buffer_load_b128(xres, xrow[g] + k_at, 0, 0);
      if constexpr (NORM) {
        st.g0 = *reinterpret_cast<const float4v*>(norm_w + kc);
        st.g1 = *reinterpret_cast<const float4v*>(norm_w + kc + 4);
      }
    }
  };
  // DEPTH chunks are on their way at a time, each in registers of its own: the loop is written
  // out for all of them, so that no chunk is copied (a copy waits for its loads) and each is
  // waited for only when its turn has come.
  // (4 or 2, as fast as each other where a wave's chunks are a multiple of four: the launch takes 2
  // where they are not, since a wave's turns are a multiple of DEPTH; 3 and 8 are slower: 11.1,
  // 11.8 and 12.7 us for down at the 1B sizes, 8 rows)
  static_assert(DEPTH == 2 || DEPTH == 4, "chunks on their way at a time");
  Stage st[DEPTH];
  auto fetch_first = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) fetch(c0 + d, st[d]);
  };
  // What the prologue needs is asked for before anything is waited for, in the order of its use:
  // the first parts of the rows' sums of squares, the first pieces of x that a thread stages (XL),
  // the first chunks of weights. No load hangs on a condition (a part past the last reads the
  // last and counts as zero, a piece past the end its row's first), so that the sums wait for the
  // parts alone and the staging for the pieces alone, the weights on their way meanwhile.
  constexpr int WG = KS * 64;
  const int per_row = chunks * 16;          // XL: 16-byte pieces of a staged row
  const int pieces = XL ? M * per_row : 0;  // thread t stages pieces t, t + WG, ...
  float first[NORM ? MG : 1][8];
  if constexpr (NORM) {
#pragma unroll
    for (int g = 0; g < MG; ++g) {
      const int m = min(4 * g + r, M - 1);
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int p = ks * 16 + blk + u * 16 * KS;
        const float part = ssq_in[(int64_t)min(p, ssq_parts - 1) * M + m];
        first[g][u] = p < ssq_parts ? part : 0.f;
      }
    }
  }
  Frag16 piece;
  float4v piece_g0, piece_g1;
  if constexpr (XL) {
    const int idx = min((int)threadIdx.x, pieces - 1);
    const int m = idx / per_row, k = (idx - m * per_row) * 8, kc = k < K ? k : 0;
    piece.raw = *reinterpret_cast<const u32x4*>(x + (int64_t)m * ldx + kc);
    if constexpr (NORM) {
      piece_g0 = *reinterpret_cast<const float4v*>(norm_w + kc);
      piece_g1 = *reinterpret_cast<const float4v*>(norm_w + kc + 4);
    }
  }
  fetch_first();
  __builtin_amdgcn_sched_barrier(0);
  if constexpr (NORM) {
    // rs[m] from the parts of sum x^2. The parts are dealt out to all blocks of all waves (block
    // q of 16*KS takes the parts q, q + 16*KS, ...), eight loads at a time so that they share one
    // trip to memory; a wave adds its blocks, the waves' sums meet in LDS and are added in wave
    // order.
    __shared__ float rsum[KS][MG][4];
#pragma unroll
    for (int g = 0; g < MG; ++g) {
      const int m = min(4 * g + r, M - 1);
      float sum = 0.f;
#pragma unroll
      for (int u = 0; u < 8; ++u) sum += first[g][u];
      for (int p0 = ks * 16 + blk + 128 * KS; p0 < ssq_parts; p0 += 128 * KS) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int p = p0 + u * 16 * KS;
          v[u] = p < ssq_parts ? ssq_in[(int64_t)p * M + m] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) sum += v[u];
      }
      sum += __shfl_xor(sum, 4, 64);
      sum += __shfl_xor(sum, 8, 64);
      sum += __shfl_xor(sum, 16, 64);
      sum += __shfl_xor(sum, 32, 64);
      if (blk == 0) rsum[ks][g][r] = sum;
    }
    __syncthreads();
#pragma unroll
    for (int g = 0; g < MG; ++g) {
      float sum = 0.f;
#pragma unroll
      for (int wv = 0; wv < KS; ++wv) sum += rsum[wv][g][r];
      rs[g] = rsqrtf(sum / (float)K + eps);
    }
  }

  if constexpr (XL) {
    // thread t stages the 8 values at k = 8*(t % (chunks*16)) of row t / (chunks*16), and so on
    __shared__ float rs_row[4 * MG];
    if constexpr (NORM) {
      if (ks == 0 && blk == 0) {
#pragma unroll
        for (int g = 0; g < MG; ++g) rs_row[4 * g + r] = rs[g];
      }
      __syncthreads();
    }
    auto stage = [&](int idx, Frag16 v, float4v g0, float4v g1) __attribute__((always_inline)) {
      const int m = idx / per_row, k = (idx - m * per_row) * 8;
      if (k < K) {
        if constexpr (NORM) {
          const float rsm = rs_row[m];
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            const float normed = (float)(bf16_t)((float)v.e[i] * rsm);
            v.e[i] = (bf16_t)((i < 4 ? g0[i] : g1[i - 4]) * normed);
          }
        }
      } else {
        v.raw = u32x4{0, 0, 0, 0};
      }
      *reinterpret_cast<u32x4*>(xs + (int64_t)m * xpad + k) = v.raw;
    };
    if ((int)threadIdx.x < pieces) stage(threadIdx.x, piece, piece_g0, piece_g1);
    for (int idx = threadIdx.x + WG; idx < pieces; idx += WG) {
      const int m = idx / per_row, k = (idx - m * per_row) * 8, kc = k < K ? k : 0;
      Frag16 v;
      float4v g0 = {0.f, 0.f, 0.f, 0.f}, g1 = g0;
      v.raw = *reinterpret_cast<const u32x4*>(x + (int64_t)m * ldx + kc);
      if constexpr (NORM) {
        g0 = *reinterpret_cast<const float4v*>(norm_w + kc);
        g1 = *reinterpret_cast<const float4v*>(norm_w + kc + 4);
      }
      stage(idx, v, g0, g1);
    }
    __syncthreads();
  }
  auto multiply = [&](Stage& cur, int c) __attribute__((always_inline)) {
    if constexpr (XL) {
#pragma unroll
      for (int g = 0; g < MG; ++g) {
        const int m = 4 * g + r;
        cur.xf[g].raw = u32x4{0, 0, 0, 0};
        if (m < M && c < c1)
          cur.xf[g].raw = *reinterpret_cast<const u32x4*>(xs + (int64_t)m * xpad + c * 128 + blk * 8);
      }
    } else if constexpr (NORM) {
#pragma unroll
      for (int g = 0; g < MG; ++g)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float normed = (float)(bf16_t)((float)cur.xf[g].e[i] * rs[g]);
          cur.xf[g].e[i] = (bf16_t)((i < 4 ? cur.g0[i] : cur.g1[i - 4]) * normed);
        }
    }
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int f = 0; f < FQ; ++f)
#pragma unroll
        for (int g = 0; g < MG; ++g) acc[f][g] = mfma4(cur.wf[f].h[h], cur.xf[g].h[h], acc[f][g]);
  };
  if (c0 < c1) {
    int c = c0;
    for (; c + DEPTH < c1; c += DEPTH) {  // groups that have a chunk behind them
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        multiply(st[d], c + d);
        fetch(c + d + DEPTH, st[d]);
      }
    }
#pragma unroll
    for (int d = 0; d < DEPTH; ++d)
      if (c + d < c1) multiply(st[d], c + d);  // the last group (what was loaded past the end is not waited for)
  }

  // blocks l/4 that differ in their upper two bits are added by lane swaps, the remaining four
  // blocks and the waves through LDS
#pragma unroll
  for (int f = 0; f < FQ; ++f)
#pragma unroll
    for (int g = 0; g < MG; ++g)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float v = acc[f][g][i];
        v += __shfl_xor(v, 32, 64);
        v += __shfl_xor(v, 16, 64);
        acc[f][g][i] = v;
      }
  if (lane < 16) {
#pragma unroll
    for (int f = 0; f < FQ; ++f)
#pragma unroll
      for (int g = 0; g < MG; ++g) red[ks][f * MG + g][lane] = acc[f][g];
  }
  __syncthreads();
  // thread t < 4*PAIRS owns the four features of quad f = p / MG for activation row m = 4g + rr
  const int t = threadIdx.x;
  const bool owner = t < 4 * PAIRS;
  const int p = t / 4, rr = t % 4;
  float4v total = {0.f, 0.f, 0.f, 0.f};
  if (owner) {
#pragma unroll
    for (int k = 0; k < KS; ++k)
#pragma unroll
      for (int b = 0; b < 4; ++b) total += red[k][p][4 * b + rr];
  }
  if (EPI == EPI_SWIGLU) {
    if (owner) fin[p][rr] = total;
    __syncthreads();
  }
  const int f = p / MG, g = p % MG;
  const int m = 4 * g + rr;
  const int nb = n_tile + 4 * f;
  float sq = 0.f;
  if (owner && f < OQ && m < M && nb < N) {
    const bool whole = nb + 3 < N;
    float y[2][4];
#pragma unroll
    for (int a = 0; a < (EPI == EPI_SWIGLU ? 2 : 1); ++a) {
      const float4v src = EPI == EPI_SWIGLU ? fin[(f + a * OQ) * MG + g][rr] : total;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        y[a][i] = src[i] + (bias != nullptr && nb + i < N ? (float)bias[nb + i + a * up_offset] : 0.f);
    }
    if (EPI == EPI_F32) {
      float* op = reinterpret_cast<float*>(out) + (int64_t)m * ldo + nb;
      if (whole && ldo % 4 == 0) {
        *reinterpret_cast<float4v*>(op) = float4v{y[0][0], y[0][1], y[0][2], y[0][3]};
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (nb + i < N) op[i] = y[0][i];
      }
    } else {
      bf16_t* op = EPI == EPI_RESIDUAL ? stream + (int64_t)m * lds_ + nb
                                       : reinterpret_cast<bf16_t*>(out) + (int64_t)m * ldo + nb;
      const bool vec = whole && (EPI == EPI_RESIDUAL ? lds_ : ldo) % 4 == 0;
      Pack4 res;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (EPI == EPI_STORE) {
          res.e[i] = (bf16_t)y[0][i];
        } else if (EPI == EPI_SWIGLU) {
          const float gt = (float)(bf16_t)y[0][i], up = (float)(bf16_t)y[1][i];
          const float sg = (float)(bf16_t)silu<bf16_t>(gt);
          res.e[i] = (bf16_t)(sg * up);
        } else {  // EPI_RESIDUAL: the sum in 32-bit, rounded to the stream's type
          res.e[i] = (bf16_t)((float)old.e[i] + (float)(bf16_t)y[0][i]);
          if (nb + i < N) sq += (float)res.e[i] * (float)res.e[i];
        }
      }
      if (vec) {
        *reinterpret_cast<short4v*>(op) = res.v;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (nb + i < N) op[i] = res.e[i];
      }
    }
  }
  if (EPI == EPI_RESIDUAL) {
    // the tile's part of the row's sum of squares: the quads' shares, added in quad order
    if (owner) sqs[f][g][rr] = sq;
    __syncthreads();
    if (owner && f == 0 && m < M) {
      float s = 0.f;
#pragma unroll
      for (int q = 0; q < OQ; ++q) s += sqs[q][g][rr];
      ssq_out[(int64_t)tile * M + m] = s;
    }
  }
}

#define S4_PARAMS                                                                                 \
  const void *x, int64_t ldx, const float *ssq_in, int ssq_parts, const float *norm_w, float eps,   \
      const void *w, const void *bias, void *out, int64_t ldo, void *stream_buf, int64_t lds_,      \
      float *ssq_out, int M, int N, int K, int up_offset, hipStream_t stream
#define S4_ARGS \
  x, ldx, ssq_in, ssq_parts, norm_w, eps, w, bias, out, ldo, stream_buf, lds_, ssq_out, M, N, K, up_offset, stream

template <int KS, int FQ, int MG, int EPI, bool NORM>
static void launch4(S4_PARAMS) {
  constexpr int OQ = EPI == EPI_SWIGLU ? FQ / 2 : FQ;
  const int tiles = (N + 4 * OQ - 1) / (4 * OQ);
  // The activations are staged through LDS when they fit 64 KB there and the product has many
  // tiles: staging costs a workgroup a barrier and a trip to memory before its first product, which
  // pays when each compute unit works through several workgroups, and does not for a short kernel.
  const int64_t x_lds = (int64_t)M * ((K + 127) / 128 * 128 + 32) * 2;
  const bool staged = x_lds <= 64 * 1024 && tiles >= 4 * dli_compute_units();
  // A wave walks its chunks of 128 k in groups of DEPTH turns: four at a time where every wave's
  // share is a multiple of four, else two (rows of 2,560 or 3,072 k on four waves are five or six
  // chunks a wave: eight turns in groups of four, six in groups of two; the sums are the same
  // whichever way, each wave adds its chunks in their order).
  const int chunks = (K + 127) / 128;
  const bool by_four = chunks % (4 * KS) == 0;
#define S4_LAUNCH(XL_, DEPTH_)                                                                              \
  skinny4_kernel<KS, FQ, MG, EPI, NORM, XL_, DEPTH_><<<tiles, KS * 64, XL_ ? (size_t)x_lds : 0, stream>>>( \
      (const bf16_t*)x, ldx, ssq_in, ssq_parts, norm_w, eps, (const bf16_t*)w, (const bf16_t*)bias, out,    \
      ldo, (bf16_t*)stream_buf, lds_, ssq_out, M, N, K, up_offset)
  if (staged && by_four) S4_LAUNCH(true, 4);
  else if (staged) S4_LAUNCH(true, 2);
  else if (by_four) S4_LAUNCH(false, 4);
  else S4_LAUNCH(false, 2);
#undef S4_LAUNCH
}

template <int KS, int FQ, int EPI, bool NORM>
static void dispatch_rows(int mg, S4_PARAMS) {
  if (mg == 1) launch4<KS, FQ, 1, EPI, NORM>(S4_ARGS);
  else if (mg == 2) launch4<KS, FQ, 2, EPI, NORM>(S4_ARGS);
  else launch4<KS, FQ, 4, EPI, NORM>(S4_ARGS);
}

// shapes of the workgroup: 0: 4 waves x 4 quads, 1: 8 waves x 2 quads, 2: 16 waves x 2 quads
template <int EPI, bool NORM>
static int dispatch4(int shape, int mg, S4_PARAMS) {
  switch (shape) {
    case 0: dispatch_rows<4, 4, EPI, NORM>(mg, S4_ARGS); break;
    case 1: dispatch_rows<8, 2, EPI, NORM>(mg, S4_ARGS); break;
    default: dispatch_rows<16, 2, EPI, NORM>(mg, S4_ARGS); break;
  }
  return dli_launch_status();
}

extern "C" int dli_skinny4_max_rows() { return 16; }

// Output features per tile of workgroup shape `shape`: the residual epilogue leaves one part of
// each row's sum of squares per tile.
extern "C" int dli_skinny4_tile_features(int shape, int epilogue) {
  const int fq = shape == 0 ? 4 : 2;
  return epilogue == EPI_SWIGLU ? 2 * fq : 4 * fq;
}

// epilogue: 0 store bf16, 1 swiglu (N = features of one half, up rows at +up_offset), 2 residual,
// 3 store float32. norm_w == nullptr: no norm. shape: see dispatch4.
extern "C" int dli_skinny4_gemm(const void* x, int64_t ldx, const float* ssq_in, int ssq_parts,
                                const float* norm_w, float eps, const void* w, const void* bias,
                                void* out, int64_t ldo, void* stream_buf, int64_t lds_,
                                float* ssq_out, int M, int N, int K, int up_offset, int epilogue,
                                int shape, hipStream_t stream) {
  if (M <= 0 || N <= 0) return DLI_OK;
  if (M > 16 || K <= 0 || K % 8 != 0 || ldx % 8 != 0 || ldx < K || (int64_t)M * ldx * 2 >= (int64_t)1 << 31 ||
      shape < 0 || shape > 2 || epilogue < 0 || epilogue > 3 ||
      (norm_w != nullptr && (ssq_in == nullptr || ssq_parts <= 0)) ||
      (epilogue == EPI_RESIDUAL && (stream_buf == nullptr || ssq_out == nullptr || norm_w != nullptr)) ||
      (epilogue != EPI_RESIDUAL && out == nullptr))
    return DLI_ERR_ARGUMENT;
  const int mg = M <= 4 ? 1 : (M <= 8 ? 2 : 4);
  const bool norm = norm_w != nullptr;
  switch (epilogue) {
    case EPI_STORE:
      return norm ? dispatch4<EPI_STORE, true>(shape, mg, S4_ARGS) : dispatch4<EPI_STORE, false>(shape, mg, S4_ARGS);
    case EPI_SWIGLU:
      return norm ? dispatch4<EPI_SWIGLU, true>(shape, mg, S4_ARGS) : dispatch4<EPI_SWIGLU, false>(shape, mg, S4_ARGS);
    case EPI_RESIDUAL:
      return dispatch4<EPI_RESIDUAL, false>(shape, mg, S4_ARGS);
    default:
      return norm ? dispatch4<EPI_F32, true>(shape, mg, S4_ARGS) : dispatch4<EPI_F32, false>(shape, mg, S4_ARGS);
  }
}
