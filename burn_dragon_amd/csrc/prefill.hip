// Chunked (all tokens at once) form of the recurrent path on the bf16 matrix cores of gfx950.
//
// The sequential definition (src/model/bdh.rs:288-302, no ALiBi) for T tokens starting from a
// state rho0 is, per (b,h) slice with Q = rope(x) [T,N] and V [T,d]:
//     out  = tril(-1)(Q Q^T) V + Q rho0          (readout before update => strictly causal)
//     rho  = rho0 + Q^T V
// Stages (all stream-ordered on the context's stream):
//   1. k_rope_bf16      Q = bf16(rope_f32(x)); the sin/cos of a (t, pair) is computed once and
//                       reused for every (b,h) slice.
//   2. k_gemm<SCORES>   S = tril(-1)(Q Q^T) as bf16, lower-triangular 256x256 tiles only, K = N.
//   3. k_gemm<ACC>      out = S V  (K limited to the causal extent of each row tile)
//                       (+ Q rho0 first when the state is not known to be zero)
//   4. k_gemm<ACC>      rho += Q^T V
// One GEMM kernel serves all products: C[m,n] = sum_k A[m,k] B[n,k] with 256x256x64 workgroup
// tiles, 8 wavefronts (2x4) of 128x64 each, v_mfma_f32_32x32x16_bf16, f32 accumulators.  B is
// always k-contiguous in memory (V and rho0 are transposed once by a small kernel).  A is either
// k-contiguous (copied to LDS as is, fragments read with one 16-byte LDS load) or, for Q^T V,
// k-major (Q [T,N] with the reduction over T): that tile is also copied as is, [k][m], and the
// fragments are read with the transposing LDS load of gfx950 (ds_read_b64_tr_b16); a 64-byte
// column swizzle on every other group of eight k rows keeps the two half-waves on different banks.
#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstring>
#include <type_traits>

#include "bdh_internal.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

constexpr float kTwoPi = 6.28318530717958647692f;
constexpr int BM = 256, BN = 256, BK = 64;
constexpr int LDS_STRIDE = BK + 8;  // bf16 elements per LDS row: 144 bytes, conflict-free b128 reads

__device__ __forceinline__ unsigned short f32_to_bf16_bits(float f) {
  unsigned int u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (unsigned short)((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (unsigned short)(u >> 16);
}
__device__ __forceinline__ float bf16_bits_to_f32(unsigned short v) { return __uint_as_float((unsigned int)v << 16); }

// ------------------------------------------------------------------------------------
// 1. rotation: x bf16 [S, T, N] -> q bf16 [S, T, N]   (S = B*h slices)
// thread = (t, group of 4 pairs); loops over the slices
// ------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_rope_bf16(const uint4 *__restrict__ x, uint4 *__restrict__ q,
                                                   const float *__restrict__ freqs, int S, int T, int N,
                                                   long x_slice_groups, long pos0) {
  const int groups = N >> 3;  // 8 elements (4 pairs) per thread
  const long gid = (long)blockIdx.x * 256 + threadIdx.x;
  if (gid >= (long)T * groups) return;
  const int t = (int)(gid / groups), g = (int)(gid - (long)t * groups);
  const float pos = (float)(pos0 + t);
  float cs[8], sn[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float f = freqs[g * 8 + e];
    const float raw = pos * f;
    const float ph = (raw - floorf(raw)) * kTwoPi;
    sincosf(ph, &sn[e], &cs[e]);
  }
  auto rotate = [&](const uint4 in) -> uint4 {
    if (!(in.x | in.y | in.z | in.w)) return make_uint4(0u, 0u, 0u, 0u);
    const unsigned int w[4] = {in.x, in.y, in.z, in.w};
    unsigned int o[4];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const float xe = bf16_bits_to_f32((unsigned short)(w[p] & 0xffffu));
      const float xo = bf16_bits_to_f32((unsigned short)(w[p] >> 16));
      // q[2j] = x[2j] cos + (-x[2j+1]) sin ; q[2j+1] = x[2j+1] cos + x[2j] sin  (attention.rs:305-321)
      const float a0 = xe * cs[2 * p], r0 = (-xo) * sn[2 * p];
      const float a1 = xo * cs[2 * p + 1], r1 = xe * sn[2 * p + 1];
      o[p] = (unsigned int)f32_to_bf16_bits(a0 + r0) | ((unsigned int)f32_to_bf16_bits(a1 + r1) << 16);
    }
    return make_uint4(o[0], o[1], o[2], o[3]);
  };
  // eight slices at a time: the loads are issued together, so eight requests per thread are in flight
  int s = 0;
  for (; s + 8 <= S; s += 8) {
    uint4 in[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) in[u] = x[(long)(s + u) * x_slice_groups + (long)t * groups + g];
#pragma unroll
    for (int u = 0; u < 8; ++u) q[((long)(s + u) * T + t) * groups + g] = rotate(in[u]);
  }
  for (; s < S; ++s) {
    q[((long)s * T + t) * groups + g] = rotate(x[(long)s * x_slice_groups + (long)t * groups + g]);
  }
}

// ------------------------------------------------------------------------------------
// batched transpose to bf16: in [batch][R][C] (f32 or bf16) -> out [batch][C][ldo], ldo >= R,
// columns R..ldo-1 of the output are zero-filled.  64x64 tiles through LDS.
// ------------------------------------------------------------------------------------
template <typename TIn>
__global__ __launch_bounds__(256) void k_transpose_to_bf16(const TIn *__restrict__ in, unsigned short *__restrict__ out,
                                                          int R, int C, int ldo, long in_batch) {
  __shared__ unsigned short tile[64][66];
  const long batch = blockIdx.z;
  const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  const TIn *src = in + batch * in_batch;
  unsigned short *dst = out + batch * (long)C * ldo;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int rr = ty; rr < 64; rr += 4) {
    const int r = r0 + rr, c = c0 + tx;
    unsigned short v = 0;
    if (r < R && c < C) {
      if constexpr (sizeof(TIn) == 4) v = f32_to_bf16_bits((float)src[(long)r * C + c]);
      else v = (unsigned short)src[(long)r * C + c];
    }
    tile[rr][tx] = v;
  }
  __syncthreads();
  for (int cc = ty; cc < 64; cc += 4) {
    const int c = c0 + cc, r = r0 + tx;
    if (c < C && r < ldo) dst[(long)c * ldo + r] = tile[tx][cc];  // rows >= R were staged as zero
  }
}

struct HeadPar {
  float v[64];
};

// V^T per (b,h) slice for a decaying state (src/model/bdh.rs:299-301): in bf16 [B][R][C] -> out bf16
// [B*h][C][ldo] with row r (token r of R) scaled by exp((R - r) * log_decay[head]) -- the decay a token's update
// has seen by the end of the pass.  Columns R..ldo-1 of the output are zero-filled.
__global__ __launch_bounds__(256) void k_transpose_decay_bf16(const unsigned short *__restrict__ in,
                                                              unsigned short *__restrict__ out, int R, int C, int ldo,
                                                              long in_batch, int h, HeadPar log_decay) {
  __shared__ unsigned short tile[64][66];
  const long slice = blockIdx.z;
  const float ld = log_decay.v[slice % h];
  const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  const unsigned short *src = in + (slice / h) * in_batch;
  unsigned short *dst = out + slice * (long)C * ldo;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int rr = ty; rr < 64; rr += 4) {
    const int r = r0 + rr, c = c0 + tx;
    unsigned short v = 0;
    if (r < R && c < C) v = f32_to_bf16_bits(bf16_bits_to_f32(src[(long)r * C + c]) * expf((float)(R - r) * ld));
    tile[rr][tx] = v;
  }
  __syncthreads();
  for (int cc = ty; cc < 64; cc += 4) {
    const int c = c0 + cc, r = r0 + tx;
    if (c < C && r < ldo) dst[(long)c * ldo + r] = tile[tx][cc];
  }
}

// PoPE (src/model/attention.rs:323-330): x bf16 [S, T, N] -> q bf16 [S, T, 2N] = cat(softplus(x) cos, softplus(x) sin).
// thread = (t, group of 8 neurons); loops over the slices
__global__ __launch_bounds__(256) void k_pope_bf16(const uint4 *__restrict__ x, uint4 *__restrict__ q,
                                                   const float *__restrict__ freqs, int S, int T, int N,
                                                   long x_slice_groups, long pos0) {
  const int groups = N >> 3;
  const long gid = (long)blockIdx.x * 256 + threadIdx.x;
  if (gid >= (long)T * groups) return;
  const int t = (int)(gid / groups), g = (int)(gid - (long)t * groups);
  const float pos = (float)(pos0 + t);
  float cs[8], sn[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float raw = pos * freqs[g * 8 + e];
    sincosf((raw - floorf(raw)) * kTwoPi, &sn[e], &cs[e]);
  }
  for (int s = 0; s < S; ++s) {
    const uint4 in = x[(long)s * x_slice_groups + (long)t * groups + g];
    const unsigned int w[4] = {in.x, in.y, in.z, in.w};
    unsigned int re[4], im[4];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const float m0 = logf(expf(bf16_bits_to_f32((unsigned short)(w[p] & 0xffffu))) + 1.0f);
      const float m1 = logf(expf(bf16_bits_to_f32((unsigned short)(w[p] >> 16))) + 1.0f);
      re[p] = (unsigned int)f32_to_bf16_bits(m0 * cs[2 * p]) | ((unsigned int)f32_to_bf16_bits(m1 * cs[2 * p + 1]) << 16);
      im[p] = (unsigned int)f32_to_bf16_bits(m0 * sn[2 * p]) | ((unsigned int)f32_to_bf16_bits(m1 * sn[2 * p + 1]) << 16);
    }
    uint4 *row = q + ((long)s * T + t) * (2 * groups);
    row[g] = make_uint4(re[0], re[1], re[2], re[3]);
    row[groups + g] = make_uint4(im[0], im[1], im[2], im[3]);
  }
}

// denom[slice][row] = sum over the column tiles of norm_part + eps (src/kernel/linear_attention.rs:8,108), in tile
// order; tri: only the tiles up to the row's own exist
__global__ __launch_bounds__(256) void k_norm_reduce(const float *__restrict__ norm_part, float *__restrict__ denom,
                                                     int M, int nt, int tri, float eps) {
  const int row = blockIdx.x * 256 + threadIdx.x;
  const long slice = blockIdx.y;
  if (row >= M) return;
  const int last = tri ? row / BM : nt - 1;
  float sum = 0.0f;
  for (int tj = 0; tj <= last; ++tj) sum += norm_part[(slice * nt + tj) * M + row];
  denom[slice * M + row] = sum + eps;
}

// ------------------------------------------------------------------------------------
// batched GEMM  C[m,n] (+)= sum_k A[m,k] B[n,k]
// ------------------------------------------------------------------------------------
// EPI_SCORES / EPI_ACC: the two epilogues of the RoPE path.  The _X variants add what ALiBi, the row
// normalisation of kernel::linear_attention::fused_state_aligned and a decaying state need (GemmArgs::mode).
enum { EPI_SCORES = 0, EPI_ACC = 1, EPI_SCORES_X = 2, EPI_ACC_X = 3 };
enum {
  GM_DECAY_SCORES = 1,  // scores:  S[t,s] *= exp((t - s) * par)            (src/model/bdh.rs:299-301 unrolled)
  GM_ADD_ALIBI = 2,     // scores:  S[t,s] += par * (s - t) on every element of the causal time blocks
                        //          (src/kernel/linear_attention.rs:97-100: whole blocks, the diagonal one included)
  GM_ROWNORM = 4,       // scores:  also write sum_s |S[t,s]| of this tile's columns to norm_part
  GM_DECAY_ROWS = 8,    // acc:     row t *= exp(t * par)                   (the Q rho0 term of a decaying state)
  GM_DECAY_STATE = 16,  // acc:     C = exp(K * par) * C + acc              (the state after K decaying tokens)
  GM_DIVNORM = 32       // acc:     C = acc / denom[row]                    (src/kernel/linear_attention.rs:108-109)
};

struct GemmArgs {
  const void *A;  // bf16
  const void *B;  // bf16 or f32
  void *C;        // bf16 (scores) or f32
  long a_batch, b_batch, c_batch;  // element strides between slices (B may be shared by heads: see b_div)
  int lda, ldb, ldc;
  int M, N, K;
  int b_div;           // B slice index = slice / b_div (V is shared by the h heads of a batch entry)
  int beta;            // EPI_ACC: add to the existing C
  int causal_k;        // limit K of row tile i to min(K, (i+1)*BM)   (S V product)
  int tri;             // 1: tiles enumerate the lower triangle (row tile >= col tile) of an mt x mt grid
  int mt, nt;          // tile grid (rows, cols); rows are visited from the last (largest causal K) down
  int n_tiles, n_slices;
  // _X epilogues only
  int mode;            // GM_* bits
  int h;               // heads: slice % h selects head_par
  int block_size;      // GM_ADD_ALIBI: tokens per time block of the causal layout
  float *norm_part;    // GM_ROWNORM: [slice][nt][M] sums of |S| per column tile
  const float *denom;  // GM_DIVNORM: [slice][M]
  float head_par[64];  // per head: log of the per-token decay factor, or the additive slope
};

// Epilogues of the _X variants.  Accumulator element e of lane l in a 32x32 tile: row = (e/4)*8 + (l/32)*4 +
// (e%4), col = l%32.  s_red: 1024 floats of LDS that no wave reads any more (GM_ROWNORM only).
template <int EPI>
__device__ __forceinline__ void gemm_epilogue_x(const GemmArgs &g, f32x16 (&acc)[4][2], int slice, int m0, int n0,
                                                int tj, int wm, int wn, int lane, int tid, float *s_red) {
  const float par = g.head_par[slice % g.h];
  if constexpr (EPI == EPI_SCORES_X) {
    unsigned short *C = static_cast<unsigned short *>(g.C) + (long)slice * g.c_batch;
    const int bs = g.block_size > 0 ? g.block_size : 1;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int row = m0 + wm * 128 + i * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
        const int rblk = (g.mode & GM_ADD_ALIBI) ? row / bs : 0;
        float rsum = 0.0f;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int col = n0 + wn * 64 + j * 32 + (lane & 31);
          float v = col < row ? acc[i][j][e] : 0.0f;  // tril(-1)
          if ((g.mode & GM_DECAY_SCORES) && col < row) v *= expf((float)(row - col) * par);
          if ((g.mode & GM_ADD_ALIBI) && col / bs <= rblk) v += par * (float)(col - row);
          if (col >= g.N) v = 0.0f;  // padding columns of the score matrix
          const unsigned short bits = f32_to_bf16_bits(v);
          if (row < g.M && col < g.ldc) C[(long)row * g.ldc + col] = bits;
          rsum += fabsf(bf16_bits_to_f32(bits));  // what the next product multiplies with
        }
        if (g.mode & GM_ROWNORM) {
#pragma unroll
          for (int off = 16; off >= 1; off >>= 1) rsum += __shfl_xor(rsum, off);  // the 32 columns of a half-wave
          if ((lane & 31) == 0) s_red[wn * 256 + wm * 128 + i * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3)] = rsum;
        }
      }
    if (g.mode & GM_ROWNORM) {
      __syncthreads();
      if (tid < 256 && m0 + tid < g.M) {
        const float sum = ((s_red[tid] + s_red[256 + tid]) + s_red[512 + tid]) + s_red[768 + tid];
        g.norm_part[((long)slice * g.nt + tj) * g.M + m0 + tid] = sum;
      }
    }
  } else {
    float *C = static_cast<float *>(g.C) + (long)slice * g.c_batch;
    const float sdecay = (g.mode & GM_DECAY_STATE) ? expf((float)g.K * par) : 1.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int row = m0 + wm * 128 + i * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
        if (row >= g.M) continue;
        const float rscale = (g.mode & GM_DECAY_ROWS) ? expf((float)row * par) : 1.0f;
        const float dn = (g.mode & GM_DIVNORM) ? g.denom[(long)slice * g.M + row] : 1.0f;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int col = n0 + wn * 64 + j * 32 + (lane & 31);
          if (col >= g.N) continue;
          float v = acc[i][j][e];
          if (g.mode & GM_DECAY_ROWS) v *= rscale;
          if (g.mode & GM_DIVNORM) v = v / dn;
          float *p = C + (long)row * g.ldc + col;
          if (g.beta) v = ((g.mode & GM_DECAY_STATE) ? *p * sdecay : *p) + v;
          *p = v;
        }
      }
  }
}

// bf16 elements per k row of a k-major tile in LDS: 576 bytes = 64 mod 256, so the four k rows of 64 bytes
// that 32 lanes of a transposing read touch fall on disjoint quarters of the 64 banks
constexpr int KM_STRIDE = BM + 32;

template <bool A_KMAJOR, int EPI>
__global__ __launch_bounds__(512) void k_gemm(GemmArgs g) {
  __shared__ __attribute__((aligned(16))) unsigned short s_a[BM * LDS_STRIDE];
  __shared__ __attribute__((aligned(16))) unsigned short s_b[BN * LDS_STRIDE];
  static_assert(BK * KM_STRIDE <= BM * LDS_STRIDE, "k-major tile must fit");

  // XCD-aware mapping: workgroup ids are dealt round-robin to the 8 XCDs, so workgroups with the
  // same (id % 8) share an L2; all tiles of one slice go to one XCD.
  const int xcd = blockIdx.x & 7;
  const int r = blockIdx.x >> 3;
  const int slice = xcd + 8 * (r / g.n_tiles);
  if (slice >= g.n_slices) return;
  int ti, tj;
  {
    const int t = r % g.n_tiles;
    if (g.tri) {  // t = i(i+1)/2 + j, 0 <= j <= i
      int i = (int)((sqrtf(8.0f * (float)t + 1.0f) - 1.0f) * 0.5f);
      while (i * (i + 1) / 2 > t) --i;
      while ((i + 1) * (i + 2) / 2 <= t) ++i;
      tj = t - i * (i + 1) / 2;
      ti = i;
    } else {  // row tiles from the last (largest causal K) down
      ti = g.mt - 1 - t / g.nt;
      tj = t % g.nt;
    }
  }
  const int m0 = ti * BM, n0 = tj * BN;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 2, wn = wave & 3;  // 2 x 4 waves, 128 x 64 each

  const unsigned short *A = static_cast<const unsigned short *>(g.A) + (long)slice * g.a_batch;
  const unsigned short *Bh = static_cast<const unsigned short *>(g.B) + (long)(slice / g.b_div) * g.b_batch;

  int K = g.K;
  if (g.causal_k) K = min(K, m0 + BM);

  f32x16 acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  // staging registers: 4 chunks of 8 elements per operand per thread
  uint4 ra[4], rb[4];

  auto load_a = [&](int k0) {
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int chunk = c * 512 + tid;  // 2048 chunks of 8 elements
      uint4 v = make_uint4(0u, 0u, 0u, 0u);
      if (!A_KMAJOR) {
        const int row = chunk >> 3, kc = (chunk & 7) * 8;  // 8 chunks per row of 64 k
        if (m0 + row < g.M && k0 + kc < K) v = *reinterpret_cast<const uint4 *>(A + (long)(m0 + row) * g.lda + k0 + kc);
      } else {
        const int kr = chunk >> 5, mc = (chunk & 31) * 8;  // 32 chunks per k row of 256 m
        if (k0 + kr < K && m0 + mc < g.M) v = *reinterpret_cast<const uint4 *>(A + (long)(k0 + kr) * g.lda + m0 + mc);
      }
      ra[c] = v;
    }
  };
  auto load_b = [&](int k0) {
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int chunk = c * 512 + tid;
      const int row = chunk >> 3, kc = (chunk & 7) * 8;
      uint4 v = make_uint4(0u, 0u, 0u, 0u);
      if (n0 + row < g.N && k0 + kc < K) v = *reinterpret_cast<const uint4 *>(Bh + (long)(n0 + row) * g.ldb + k0 + kc);
      rb[c] = v;
    }
  };
  auto store_tiles = [&]() {
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int chunk = c * 512 + tid;
      const int row = chunk >> 3, kc = (chunk & 7) * 8;
      *reinterpret_cast<uint4 *>(s_b + row * LDS_STRIDE + kc) = rb[c];
      if (!A_KMAJOR) {
        *reinterpret_cast<uint4 *>(s_a + row * LDS_STRIDE + kc) = ra[c];
      } else {
        const int kr = chunk >> 5, mc = (chunk & 31) * 8;
        *reinterpret_cast<uint4 *>(s_a + kr * KM_STRIDE + (mc ^ (((kr >> 3) & 1) << 5))) = ra[c];
      }
    }
  };

  load_a(0);
  load_b(0);
  for (int k0 = 0; k0 < K; k0 += BK) {
    __syncthreads();  // the previous step's fragment reads are done
    store_tiles();
    __syncthreads();
    if (k0 + BK < K) {  // prefetch the next k tile while the matrix cores work on this one
      load_a(k0 + BK);
      load_b(k0 + BK);
    }
#pragma unroll
    for (int kk = 0; kk < BK; kk += 16) {
      bf16x8 fa[4], fb[2];
      const int kof = kk + (lane >> 5) * 8;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int mrow = wm * 128 + i * 32 + (lane & 31);
        if (!A_KMAJOR) {
          fa[i] = *reinterpret_cast<const bf16x8 *>(s_a + mrow * LDS_STRIDE + kof);
        } else {
          // transposing LDS read (ds_read_b64_tr_b16): a group of 16 lanes reads a 4(k) x 16(m)
          // block, lane j of the group supplying the address of row j/4, columns (j%4)*4..+3, and
          // receives column j for the four k rows.  Two reads give the 8 consecutive k of lane
          // (m = lane%32, k-group = lane/32).  Rows kof..kof+7 share bit 3 = lane>>5: one swizzle.
          const int j16 = lane & 15;
          const int mcol = (wm * 128 + i * 32 + ((lane >> 4) & 1) * 16) ^ ((lane >> 5) << 5);
          const unsigned short *src = s_a + (kof + (j16 >> 2)) * KM_STRIDE + mcol + (j16 & 3) * 4;
          typedef short s16x4 __attribute__((ext_vector_type(4)));
          typedef short s16x8 __attribute__((ext_vector_type(8)));
          typedef __attribute__((address_space(3))) s16x4 *lds_s16x4_t;
          const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_t)(src));
          const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_t)(src + 4 * KM_STRIDE));
          const s16x8 pk = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
          fa[i] = __builtin_bit_cast(bf16x8, pk);
        }
      }
#pragma unroll
      for (int j = 0; j < 2; ++j)
        fb[j] = *reinterpret_cast<const bf16x8 *>(s_b + (wn * 64 + j * 32 + (lane & 31)) * LDS_STRIDE + kof);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
  }

  if constexpr (EPI == EPI_SCORES_X || EPI == EPI_ACC_X) {
    __syncthreads();  // every wave is past its fragment reads: s_a can hold the row sums
    gemm_epilogue_x<EPI>(g, acc, slice, m0, n0, tj, wm, wn, lane, tid, reinterpret_cast<float *>(s_a));
    return;
  }
  // epilogue.  Accumulator element e of lane l in a 32x32 tile:
  //   row = (e/4)*8 + (l/32)*4 + (e%4), col = l%32
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int col = n0 + wn * 64 + j * 32 + (lane & 31);
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int row = m0 + wm * 128 + i * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
        if (row < g.M && col < (EPI == EPI_SCORES ? g.ldc : g.N)) {
          float v = acc[i][j][e];
          if (EPI == EPI_SCORES) {
            unsigned short *C = static_cast<unsigned short *>(g.C) + (long)slice * g.c_batch;
            C[(long)row * g.ldc + col] = col < row ? f32_to_bf16_bits(v) : (unsigned short)0;  // tril(-1)
          } else {
            float *C = static_cast<float *>(g.C) + (long)slice * g.c_batch;
            float *p = C + (long)row * g.ldc + col;
            *p = g.beta ? *p + v : v;
          }
        }
      }
    }
}

// ------------------------------------------------------------------------------------
// Fast variant for full tiles (M, N multiples of 256, K a multiple of 64, both operands
// k-contiguous): the tiles go from global memory straight into LDS (global_load_lds_dwordx4, no
// VGPR staging, no ds_write), double buffered.  LDS tile layout: blocks of 8 rows x 128 bytes
// (1 KiB, one wave-wide load each); inside a block the 16-byte slot of (row R, k-chunk c) is
// (R%8)*8 + (c ^ ((R/2)%8)): the LDS has 64 banks and serves a 16-byte read 16 lanes at a time, and
// 16 consecutive rows at one k-chunk then cover all 64 banks once (no conflicts, no padding).
// Same accumulation order as k_gemm, so both give identical results.
// ------------------------------------------------------------------------------------
typedef __attribute__((address_space(1))) const void *gptr_t;
typedef __attribute__((address_space(3))) void *lptr_t;

template <int EPI>
__global__ __launch_bounds__(512) void k_gemm_direct(GemmArgs g) {
  extern __shared__ __attribute__((aligned(1024))) unsigned short s_dyn[];
  constexpr int TILE = 256 * 64;  // elements per operand tile (32 KiB)
  constexpr int BUF = 2 * TILE;
  const int xcd = blockIdx.x & 7;
  const int r = blockIdx.x >> 3;
  const int slice = xcd + 8 * (r / g.n_tiles);
  if (slice >= g.n_slices) return;
  int ti, tj;
  {
    const int t = r % g.n_tiles;
    if (g.tri) {
      int i = (int)((sqrtf(8.0f * (float)t + 1.0f) - 1.0f) * 0.5f);
      while (i * (i + 1) / 2 > t) --i;
      while ((i + 1) * (i + 2) / 2 <= t) ++i;
      tj = t - i * (i + 1) / 2;
      ti = i;
    } else {
      ti = g.mt - 1 - t / g.nt;
      tj = t % g.nt;
    }
  }
  const int m0 = ti * BM, n0 = tj * BN;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 2, wn = wave & 3;
  const unsigned short *A = static_cast<const unsigned short *>(g.A) + (long)slice * g.a_batch;
  const unsigned short *Bh = static_cast<const unsigned short *>(g.B) + (long)(slice / g.b_div) * g.b_batch;
  int K = g.K;
  if (g.causal_k) K = min(K, m0 + BM);

  f32x16 acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  // source chunk of this lane inside an 8-row block: row lr, k-chunk lc (the XOR swizzle)
  const int lr = lane >> 3, lc = (lane & 7) ^ ((lr >> 1) | ((wave & 1) << 2));
  const unsigned short *pa[4], *pb[4];
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int bi = c * 8 + wave;  // 32 blocks of 8 rows per operand, 4 per wave
    pa[c] = A + (long)(m0 + bi * 8 + lr) * g.lda + lc * 8;
    pb[c] = Bh + (long)(n0 + bi * 8 + lr) * g.ldb + lc * 8;
  }
  // scores: A and B are the same matrix, so a tile on the diagonal needs its rows only once
  const bool same_ab = (EPI == EPI_SCORES || EPI == EPI_SCORES_X) && ti == tj && g.A == g.B && g.b_div == 1 &&
                       g.a_batch == g.b_batch;
#define BDH_ISSUE_TILE(buf, k0)                                                                              \
  _Pragma("unroll") for (int c = 0; c < 4; ++c) {                                                            \
    const int bi = c * 8 + wave;                                                                             \
    __builtin_amdgcn_global_load_lds((gptr_t)(pa[c] + (k0)), (lptr_t)(s_dyn + (buf)*BUF + bi * 512), 16, 0, 0);        \
    if (!same_ab)                                                                                            \
      __builtin_amdgcn_global_load_lds((gptr_t)(pb[c] + (k0)), (lptr_t)(s_dyn + (buf)*BUF + TILE + bi * 512), 16, 0, 0); \
  }
  BDH_ISSUE_TILE(0, 0)
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  int cur = 0;
  for (int k0 = 0; k0 < K; k0 += BK) {
    if (k0 + BK < K) { BDH_ISSUE_TILE(cur ^ 1, k0 + BK) }  // lands while the matrix cores work on this tile
    const unsigned short *sa = s_dyn + cur * BUF, *sb = same_ab ? sa : sa + TILE;
#pragma unroll
    for (int kk = 0; kk < BK; kk += 16) {
      bf16x8 fa[4], fb[2];
      const int C = (kk >> 3) + (lane >> 5);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int R = wm * 128 + i * 32 + (lane & 31);
        fa[i] = *reinterpret_cast<const bf16x8 *>(sa + (R >> 3) * 512 + (((R & 7) << 3) + (C ^ ((R >> 1) & 7))) * 8);
      }
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int R = wn * 64 + j * 32 + (lane & 31);
        fb[j] = *reinterpret_cast<const bf16x8 *>(sb + (R >> 3) * 512 + (((R & 7) << 3) + (C ^ ((R >> 1) & 7))) * 8);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    cur ^= 1;
  }
#undef BDH_ISSUE_TILE
  if constexpr (EPI == EPI_SCORES_X || EPI == EPI_ACC_X) {  // the loop ended with a barrier: s_dyn is free
    gemm_epilogue_x<EPI>(g, acc, slice, m0, n0, tj, wm, wn, lane, tid, reinterpret_cast<float *>(s_dyn));
    return;
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int col = n0 + wn * 64 + j * 32 + (lane & 31);
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int row = m0 + wm * 128 + i * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
        const float v = acc[i][j][e];
        if (EPI == EPI_SCORES) {
          unsigned short *C = static_cast<unsigned short *>(g.C) + (long)slice * g.c_batch;
          C[(long)row * g.ldc + col] = col < row ? f32_to_bf16_bits(v) : (unsigned short)0;  // tril(-1)
        } else {
          float *C = static_cast<float *>(g.C) + (long)slice * g.c_batch;
          float *p = C + (long)row * g.ldc + col;
          *p = g.beta ? *p + v : v;
        }
      }
    }
}

// ====================================================================================
// Chunk-recurrent form for aligned shapes (T a multiple of 256, N a multiple of 256, d = 256):
//   per 256-token chunk c of a (b,h) slice, with rho_c the state before the chunk,
//     out_c = tril(-1)(Q_c Q_c^T) V_c + Q_c rho_c        rho_{c+1} = rho_c + Q_c^T V_c
// It executes 45 % of the matrix work of the all-scores form at T = 2048 (one 256x256 score tile and
// one 256x256 state product per chunk instead of (T/256+1)/2 score tiles), and its workspace is linear
// in T.  Two kernels:
//   k_state_stream  one workgroup per (slice, 64 neurons): walks all tokens, keeps its 64x256 tile of
//                   rho in the accumulators (f32, started from the caller's state), rotates x on the way
//                   in (RoPE; Q = bf16(rope(x)) is also written out for the second kernel) and, at every
//                   chunk boundary, writes bf16(rho_c) transposed (value-major, the k-contiguous B operand
//                   of Q_c rho_c).  Q and the state copies are stored k-tile by k-tile, [N/64][rows][64].
//   k_chunk_out     one workgroup per (slice, chunk): S = Q_c Q_c^T on the matrix cores (operands straight
//                   from global memory into LDS), mask + round to bf16 into LDS, out = S V_c, then
//                   out += Q_c bf16(rho_c) with the same accumulators, written once.
// ====================================================================================

// The k loop of k_gemm_direct as a function: acc += A[0..255, k] * B[0..255, k] over K (a multiple of 64);
// A_rows / B_rows point at the first row of the 256-row operand panels, whose 64 columns of k-tile t start
// t * a_kstride (b_kstride) elements further on (64 for a plain row-major operand; a panel stored tile by tile,
// [k / 64][row][64], has row stride 64 and the tile size as the k-tile stride).  Ends with every wave past its
// last LDS read.  SAME: B is A (a diagonal score tile), loaded once.
// cache policy of the operand copies of direct_mainloop: streaming (in the chunk-recurrent form every tile is used
// once: k_chunk_out 560 -> 545 us)
constexpr int BDH_K2_LOAD_AUX = 2;
template <bool SAME>
__device__ __forceinline__ void direct_mainloop(f32x16 (&acc)[4][2], const unsigned short *A_rows, long lda,
                                                long a_kstride, const unsigned short *B_rows, long ldb,
                                                long b_kstride, int K, unsigned short *s_dyn, int wave, int lane) {
  constexpr int TILE = 256 * 64;
  constexpr int BUF = 2 * TILE;
  const int wm = wave >> 2, wn = wave & 3;
  const int lr = lane >> 3, lc = (lane & 7) ^ ((lr >> 1) | ((wave & 1) << 2));
  const unsigned short *pa[4], *pb[4];
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int bi = c * 8 + wave;
    pa[c] = A_rows + (long)(bi * 8 + lr) * lda + lc * 8;
    pb[c] = B_rows + (long)(bi * 8 + lr) * ldb + lc * 8;
  }
#define BDH_ISSUE(buf, k0)                                                                                          \
  _Pragma("unroll") for (int c = 0; c < 4; ++c) {                                                                   \
    const int bi = c * 8 + wave;                                                                                    \
    __builtin_amdgcn_global_load_lds((gptr_t)(pa[c] + ((k0) >> 6) * a_kstride),                                      \
                                     (lptr_t)(s_dyn + (buf)*BUF + bi * 512), 16, 0, BDH_K2_LOAD_AUX);                             \
    if (!SAME)                                                                                                      \
      __builtin_amdgcn_global_load_lds((gptr_t)(pb[c] + ((k0) >> 6) * b_kstride),                                    \
                                       (lptr_t)(s_dyn + (buf)*BUF + TILE + bi * 512), 16, 0, BDH_K2_LOAD_AUX);                    \
  }
  BDH_ISSUE(0, 0)
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  int cur = 0;
  for (int k0 = 0; k0 < K; k0 += BK) {
    if (k0 + BK < K) { BDH_ISSUE(cur ^ 1, k0 + BK) }
    const unsigned short *sa = s_dyn + cur * BUF, *sb = SAME ? sa : sa + TILE;
#pragma unroll
    for (int kk = 0; kk < BK; kk += 16) {
      bf16x8 fa[4], fb[2];
      const int C = (kk >> 3) + (lane >> 5);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int R = wm * 128 + i * 32 + (lane & 31);
        fa[i] = *reinterpret_cast<const bf16x8 *>(sa + (R >> 3) * 512 + (((R & 7) << 3) + (C ^ ((R >> 1) & 7))) * 8);
      }
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int R = wn * 64 + j * 32 + (lane & 31);
        fb[j] = *reinterpret_cast<const bf16x8 *>(sb + (R >> 3) * 512 + (((R & 7) << 3) + (C ^ ((R >> 1) & 7))) * 8);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    cur ^= 1;
  }
#undef BDH_ISSUE
}

// Workgroup barrier that orders LDS accesses only: global loads and stores issued before it stay in flight
// (__syncthreads also waits for every outstanding global access).
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

struct ChunkOutArgs {
  const unsigned short *Q;   // [S][N/64][Tc][64] rotated activations of this pass, Tc = 256 nc
  long q_slice;
  const unsigned short *P;   // [slot][S][N/64][256][64]: bf16(rho_c)^T, slot c = the state before chunk c
  long p_slot, p_slice;
  const unsigned short *Vt;  // [B][256][ldv]: V^T of this pass
  long vt_batch;
  float *out;                // row 0 of this pass in out [S][T][256]
  long out_slice;
  int N, ldv, nc, n_slices, h;
  int has_state;             // chunk 0 has a state term as well
  int lo_slot;               // >= 0: chunk 0 also adds Q_0 * P[lo_slot] (the rounding remainder of the carried state)
};

constexpr int S_ROW = 256 + 8;  // bf16 elements per row of the score tile in LDS (528 bytes: 16-byte reads of 16
                                // consecutive rows cover the 64 banks once)
constexpr int CHUNK_OUT_LDS = 256 * S_ROW * 2;  // 135168 bytes >= the 128 KiB of the operand buffers

__global__ __launch_bounds__(512) void k_chunk_out(ChunkOutArgs g) {
  extern __shared__ __attribute__((aligned(1024))) unsigned short s_dyn[];
  const int xcd = blockIdx.x & 7;
  const int r = blockIdx.x >> 3;
  const int slice = xcd + 8 * (r / g.nc);
  if (slice >= g.n_slices) return;
  const int c = g.nc - 1 - r % g.nc;  // later chunks first: they all have a state term
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 2, wn = wave & 3;
  // Q [slice][N/64][Tc][64] and P [slot][slice][N/64][256][64]: operand panels stored k-tile by k-tile, so that a
  // k-step of a panel is 32 KiB of consecutive bytes (and so that the state update writes whole strips)
  const unsigned short *Qc = g.Q + (long)slice * g.q_slice + (long)c * 256 * 64;
  const long q_kstride = (long)g.nc * 256 * 64, p_kstride = 256 * 64;

  f32x16 acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  // 1. S = Q_c Q_c^T
  direct_mainloop<true>(acc, Qc, 64, q_kstride, Qc, 64, q_kstride, g.N, s_dyn, wave, lane);

  // 2. tril(-1), rounded to bf16, into LDS as the A operand of S V (the operand buffers are free now)
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int col = wn * 64 + j * 32 + (lane & 31);
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int row = wm * 128 + i * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
        s_dyn[row * S_ROW + col] = col < row ? f32_to_bf16_bits(acc[i][j][e]) : (unsigned short)0;
        acc[i][j][e] = 0.0f;
      }
    }
  __syncthreads();

  // 3. out = S V_c: A fragments from LDS, B fragments (V^T rows = value columns, k = token) straight from
  //    global memory (128 KiB per workgroup, shared by the heads of a sequence).  Rows 0..127 (wm = 0) see
  //    only the first 128 tokens of the chunk.
  {
    const unsigned short *vt = g.Vt + (long)(slice / g.h) * g.vt_batch + (long)c * 256 + (lane >> 5) * 8;
    const unsigned short *vrow[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) vrow[j] = vt + (long)(wn * 64 + j * 32 + (lane & 31)) * g.ldv;
    const int kend = wm == 0 ? 128 : 256;
    for (int k0 = 0; k0 < kend; k0 += 64) {
      bf16x8 fb[4][2];
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int j = 0; j < 2; ++j) fb[q][j] = *reinterpret_cast<const bf16x8 *>(vrow[j] + k0 + q * 16);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        bf16x8 fa[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int R = wm * 128 + i * 32 + (lane & 31);
          fa[i] = *reinterpret_cast<const bf16x8 *>(s_dyn + R * S_ROW + k0 + q * 16 + (lane >> 5) * 8);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[q][j], acc[i][j], 0, 0, 0);
      }
    }
  }
  __syncthreads();  // the score tile is overwritten by the operand buffers of the next product

  // 4. out += Q_c bf16(rho_c)   (+ Q_0 times the rounding remainder of a carried state)
  if (c > 0 || g.has_state) {
    const unsigned short *Pc = g.P + (long)c * g.p_slot + (long)slice * g.p_slice;
    direct_mainloop<false>(acc, Qc, 64, q_kstride, Pc, 64, p_kstride, g.N, s_dyn, wave, lane);
    if (c == 0 && g.lo_slot >= 0) {
      const unsigned short *Pl = g.P + (long)g.lo_slot * g.p_slot + (long)slice * g.p_slice;
      direct_mainloop<false>(acc, Qc, 64, q_kstride, Pl, 64, p_kstride, g.N, s_dyn, wave, lane);
    }
  }

  float *o = g.out + (long)slice * g.out_slice + (long)c * 256 * 256;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int col = wn * 64 + j * 32 + (lane & 31);
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int row = wm * 128 + i * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
        __builtin_nontemporal_store(acc[i][j][e], o + (long)row * 256 + col);  // streaming: 542 -> 528 us for the kernel
      }
    }
}

struct StateUpdArgs {
  const unsigned short *X;   // x bf16, token 0 of this pass; rows of N
  long x_slice;
  unsigned short *Q;         // [S][N/64][Tc][64] out: bf16(rope(x))
  long q_slice;
  const unsigned short *Vf;  // [B][Tc/64][8][4][64][8]: V in B-fragment order (k_v_layouts), batch stride vt_batch
  long vt_batch;
  const float *freqs;        // [N]
  float *rho;                // [S][N][256] in/out
  unsigned short *P;         // [slot][S][N/64][256][64]
  long p_slot, p_slice;
  long pos0;                 // position of token 0 of this pass
  int N, Tc, h, n_slices;
  int has_state;             // the accumulators start from rho, and slot 0 is written
  int lo_slot;               // >= 0: bf16(rho_0 - float(bf16(rho_0))) goes to that slot
  const int *pairs_equal;    // device flag written by k_v_layouts
};

// The layouts of V that a pass consumes, and the frequency table's flag, in one launch.
// Vf[b][step][dt][kk][lane][8] holds V[b][token 64 step + 16 kk + 8 (lane >> 5) + e][value 32 dt + (lane & 31)]: the
// order the state update's B operand is consumed in, one fragment load of a wavefront = 1 KiB of consecutive bytes.
// Vt[b][value][token] is V^T, the B operand of the score-times-value product.  in: [B][Tc][256] bf16 (batch stride
// in_batch), Tc a multiple of 64.  Workgroup (0, 0) also writes flag[0] = 1 when the two elements of every lane pair
// share a frequency (what build_freqs makes), else 0.
__global__ __launch_bounds__(256) void k_v_layouts(const unsigned short *__restrict__ in, long in_batch,
                                                   unsigned short *__restrict__ vf, unsigned short *__restrict__ vt, int Tc,
                                                   const float *__restrict__ freqs, int N, int *__restrict__ flag) {
  // a workgroup takes 64 tokens x 64 value columns (quarter q of the 256)
  __shared__ unsigned short s_v[64][64 + 2];
  const int step = blockIdx.x, b = blockIdx.y, q = blockIdx.z, tid = threadIdx.x;
  const unsigned short *src = in + (long)b * in_batch + (long)step * 64 * 256 + q * 64;
  for (int i = tid; i < 64 * 32; i += 256) {  // two bf16 per access
    const int t = i >> 5, c2 = (i & 31) * 2;
    const unsigned int v = *reinterpret_cast<const unsigned int *>(src + t * 256 + c2);
    s_v[t][c2] = (unsigned short)(v & 0xffffu);
    s_v[t][c2 + 1] = (unsigned short)(v >> 16);
  }
  __syncthreads();
  unsigned short *dst = vf + ((long)b * (Tc / 64) + step) * (64 * 256) + (long)q * (2 * 4 * 64 * 8);
  for (int piece = tid; piece < 2 * 4 * 64; piece += 256) {
    const int lane = piece & 63, kk = (piece >> 6) & 3, dt = piece >> 8;
    const int t0 = kk * 16 + (lane >> 5) * 8, c = dt * 32 + (lane & 31);
    unsigned int w[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) w[e] = (unsigned int)s_v[t0 + 2 * e][c] | ((unsigned int)s_v[t0 + 2 * e + 1][c] << 16);
    *reinterpret_cast<uint4 *>(dst + (long)piece * 8) = make_uint4(w[0], w[1], w[2], w[3]);
  }
  // V^T: value row c, tokens 64 step + 8 t8 .. + 8 (16 bytes); eight consecutive threads write one 128-byte row piece
  unsigned short *dt_ = vt + ((long)b * 256 + q * 64) * Tc + step * 64;
  for (int piece = tid; piece < 64 * 8; piece += 256) {
    const int c = piece >> 3, t8 = (piece & 7) * 8;
    unsigned int w[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) w[e] = (unsigned int)s_v[t8 + 2 * e][c] | ((unsigned int)s_v[t8 + 2 * e + 1][c] << 16);
    *reinterpret_cast<uint4 *>(dt_ + (long)c * Tc + t8) = make_uint4(w[0], w[1], w[2], w[3]);
  }
  if (blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0) {
    int ok = 1;
    for (int p = tid; p < N / 2; p += 256) {
      const float2 f = reinterpret_cast<const float2 *>(freqs)[p];
      ok &= f.x == f.y;
    }
    ok = __syncthreads_and(ok);
    if (tid == 0) flag[0] = ok;
  }
}

// ---- the state update as a streaming kernel ---------------------------------------------------------------------
// Workgroups of four wavefronts own 64 neurons x 256 value columns of a slice's state (wavefront w: value columns
// 64w..64w+63, accumulators in 64 registers), two workgroups per CU.  The update moves ~3.5 GiB through HBM at the
// headline shape and needs ~0.11 ms of matrix-core time: it is a memory stream, laid out for many independent
// workgroups whose loads, stores, rotations and matrix products overlap each other, not for operand reuse.  Per
// 64-token step a workgroup reads a [64 tokens x 64 neurons] tile of x (128-byte row pieces), rotates it in
// registers, stores Q, keeps the tile in LDS for the transposing reads of the A operand; the B operand (V in
// fragment order, L2-resident) goes straight from global memory into the registers the matrix instructions just
// consumed, a whole step ahead.
// sine and cosine of a fraction of a turn in [0, 1): the hardware instructions take their argument in turns
// (absolute error below 2e-6 on that interval), no range reduction and no branches
__device__ __forceinline__ void turn_sincos(float turns, float &sn, float &cs) {
  sn = __builtin_amdgcn_sinf(turns);
  cs = __builtin_amdgcn_cosf(turns);
}

constexpr int ST_LOOK = 4;  // k-steps of B fragments in flight (1, 2 or 4): a whole step
constexpr int ST_TN = 64;
constexpr int ST_ASTRIDE = ST_TN + 32;           // bf16 per token row of the LDS tile: 48 dwords, the four rows a
                                                 // transposing read touches cover the 64 banks once
constexpr int ST_A_TILE = 64 * ST_ASTRIDE;       // elements per stage
constexpr int ST_DUMP_ROW = ST_TN + 8;           // bf16 per staged value row of a state copy (144 bytes)
constexpr int ST_DUMP_WAVE = 32 * ST_DUMP_ROW;   // a wavefront stages 32 value rows at a time
constexpr int ST_LDS = (2 * ST_A_TILE + 4 * ST_DUMP_WAVE) * 2 + 64 * 4;  // + the tile's frequencies

// Buffer addressing: a wavefront-uniform descriptor and byte offset in scalar registers plus one constant 32-bit
// offset per lane, so the token loop keeps no per-lane 64-bit addresses alive and spends no vector arithmetic on
// them.  Offsets stay below 2 GiB (checked by the host).
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ __amdgpu_buffer_rsrc_t buffer_of(const void *base) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, 0x7fffffff, 0x00020000);
}
template <int AUX = 0>
__device__ __forceinline__ uint4 buffer_load16(__amdgpu_buffer_rsrc_t r, unsigned int lane_bytes, int uniform_bytes) {
  const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(r, (int)lane_bytes, uniform_bytes, AUX);
  return make_uint4(v[0], v[1], v[2], v[3]);
}
// Stores carry the whole offset in the lane's register.  With the uniform part in a scalar offset operand the
// compiler assumes that a 16-byte store needs no idle cycles before the next write of its data registers; on this
// chip it does (seen as corrupted state copies when a vector instruction followed the store directly), and with a
// zero scalar offset the compiler inserts them.
__device__ __forceinline__ void buffer_store16(uint4 q, __amdgpu_buffer_rsrc_t r, unsigned int lane_bytes, int uniform_bytes) {
  const u32x4 v = {q.x, q.y, q.z, q.w};
  // streaming ("slc") stores: Q and the state copies are read once, by the next kernel, long after they have left
  // the caches; marked so, that kernel starts with cleaner caches (k_chunk_out 586 -> 562 us at config 3)
  __builtin_amdgcn_raw_buffer_store_b128(v, r, (int)(lane_bytes + (unsigned int)uniform_bytes), 0, 2);
}

template <bool EQ>
__device__ __forceinline__ void state_stream_body(const StateUpdArgs &g, unsigned short *s_dyn) {
  const int nt = g.N / ST_TN;
  const int xcd = blockIdx.x & 7;
  const int r = blockIdx.x >> 3;
  const int slice = xcd + 8 * (r / nt);
  if (slice >= g.n_slices) return;
  const int n0 = (r % nt) * ST_TN;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  const unsigned short *X = g.X + (long)slice * g.x_slice + n0;
  unsigned short *Qo = g.Q + (long)slice * g.q_slice + (long)(r % nt) * g.Tc * 64;  // this tile's [Tc][64] strip
  const unsigned short *Vf = g.Vf + (long)(slice / g.h) * g.vt_batch;  // fragment order, as many elements as V^T
  float *rho = g.rho + ((long)slice * g.N + n0) * 256;
  unsigned short *s_stage = s_dyn + 2 * ST_A_TILE + wave * ST_DUMP_WAVE;  // this wavefront's own staging rows

  // this thread rotates neurons mc..mc+7 of the tile at tokens tk + 32 j
  const int mc = (tid & 7) * 8, tk = tid >> 3;
  constexpr bool eq = EQ;
  float cse[4], sne[4], cso[EQ ? 1 : 4], sno[EQ ? 1 : 4];
  float c32e[4], s32e[4], c32o[EQ ? 1 : 4], s32o[EQ ? 1 : 4];  // the phase advance of 32 tokens
  {
    const float4 f0 = *reinterpret_cast<const float4 *>(g.freqs + n0 + mc);
    const float4 f1 = *reinterpret_cast<const float4 *>(g.freqs + n0 + mc + 4);
    const float fre[4] = {f0.x, f0.z, f1.x, f1.z}, fro[4] = {f0.y, f0.w, f1.y, f1.w};
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const float raw = 32.0f * fre[p];  // exact in binary32; the fraction is taken as the reference takes it
      turn_sincos(raw - floorf(raw), s32e[p], c32e[p]);
      if constexpr (!eq) {
        const float rawo = 32.0f * fro[p];
        turn_sincos(rawo - floorf(rawo), s32o[p], c32o[p]);
      }
    }
  }
  // exact phases (src/model/attention.rs:338-343) at the first tokens of a chunk; 32-token steps inside it
  // (the tile's frequencies sit in LDS after the prologue: a global load here would make the token loop wait for
  // every activation and value load in flight)
  float *s_freq = reinterpret_cast<float *>(s_dyn + 2 * ST_A_TILE + 4 * ST_DUMP_WAVE);
  auto seed = [&](int token, auto from_lds_t) {
    const float pos = (float)(g.pos0 + token);
    const float *fsrc = decltype(from_lds_t)::value ? s_freq + mc : g.freqs + n0 + mc;
    const float4 f0 = *reinterpret_cast<const float4 *>(fsrc);
    const float4 f1 = *reinterpret_cast<const float4 *>(fsrc + 4);
    const float fre[4] = {f0.x, f0.z, f1.x, f1.z}, fro[4] = {f0.y, f0.w, f1.y, f1.w};
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const float raw = pos * fre[p];
      turn_sincos(raw - floorf(raw), sne[p], cse[p]);
      if constexpr (!eq) {
        const float rawo = pos * fro[p];
        turn_sincos(rawo - floorf(rawo), sno[p], cso[p]);
      }
    }
  };
  auto advance = [&]() {
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const float c0 = cse[p] * c32e[p] - sne[p] * s32e[p], s0 = sne[p] * c32e[p] + cse[p] * s32e[p];
      cse[p] = c0; sne[p] = s0;
      if constexpr (!eq) {
        const float c1 = cso[p] * c32o[p] - sno[p] * s32o[p], s1 = sno[p] * c32o[p] + cso[p] * s32o[p];
        cso[p] = c1; sno[p] = s1;
      }
    }
  };
  // q[2j] = x[2j] cos + (-x[2j+1]) sin ; q[2j+1] = x[2j+1] cos + x[2j] sin  (src/model/attention.rs:305-321),
  // rounded to bf16 (nearest even) by the conversion instruction
  auto rotate = [&](const uint4 in) -> uint4 {
    const unsigned int w[4] = {in.x, in.y, in.z, in.w};
    unsigned int o[4];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      const float xe = __uint_as_float(w[p] << 16), xo = __uint_as_float(w[p] & 0xffff0000u);
      const float co = eq ? cse[p] : cso[eq ? 0 : p], so = eq ? sne[p] : sno[eq ? 0 : p];
      const float a0 = xe * cse[p], r0 = (-xo) * sne[p];
      const float a1 = xo * co, r1 = xe * so;
      const f32x2 qv = {a0 + r0, a1 + r1};
      o[p] = __builtin_bit_cast(unsigned int, __builtin_convertvector(qv, bf16x2));
    }
    return make_uint4(o[0], o[1], o[2], o[3]);
  };

  // the state's loads and stores (outside the token loop) are a wavefront-uniform base plus this lane's unsigned
  // 32-bit byte offset; the accesses of the token loop go through buffer descriptors (buffer_of)
  auto at = [](const void *base, unsigned int byte_off) { return static_cast<const char *>(base) + byte_off; };
  auto at_w = [](void *base, unsigned int byte_off) { return static_cast<char *>(base) + byte_off; };
  // accumulators: rows = neurons 32 i + 8 (e >> 2) + 4 (lane >> 5) + (e & 3), column = value 64 wave + 32 j + (lane & 31)
  f32x16 acc[2][2];
  if (g.has_state) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int col = wave * 64 + j * 32 + (lane & 31);
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int row = i * 32 + (e >> 2) * 8 + (e & 3);  // + 4 (lane >> 5), in the lane's offset
          acc[i][j][e] = *reinterpret_cast<const float *>(at(rho + row * 256, (unsigned int)((lane >> 5) * 1024 + col) * 4u));
        }
      }
  } else {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;
  }

  // activations: requested in the middle of step kt for the staging at the start of step kt + 2, in two register
  // slots that alternate by step parity (under load a read from HBM takes longer than the matrix products of a step)
  uint4 ra[2][2];
  const unsigned int lane_off = (unsigned int)(tk * g.N + mc) * 2u, q_off = (unsigned int)(tk * 64 + mc) * 2u;
  const __amdgpu_buffer_rsrc_t r_x = buffer_of(X), r_v = buffer_of(Vf), r_q = buffer_of(Qo);
  const int row_bytes = g.N * 2;
  auto load_piece = [&](int step, auto slot_t, int c) {  // activations of 32 tokens of a step
    constexpr int SLOT = decltype(slot_t)::value;
    // streaming load: x is read once (k_state_stream 802 -> 784 us)
    ra[SLOT][c] = buffer_load16<2>(r_x, lane_off, (step * 64 + c * 32) * row_bytes);
  };
  // B fragments of a step: fb[kk][j] = V[tokens 16 kk + 8 (lane >> 5) .. + 8)[value 64 wave + 32 j + (lane & 31)],
  // 1 KiB of consecutive bytes per wavefront and fragment in the fragment-order copy of V
  // a ring of ST_LOOK k-steps: fragment kk + ST_LOOK is fetched into the slot the products of kk just read
  bf16x8 fb[ST_LOOK][2];
  const unsigned int vb_off = (unsigned int)(wave * 2 * 4 * 64 + lane) * 16u;
  auto load_b = [&](int step, int kk) {
    const int so = (step * (64 * 256) + kk * (64 * 8)) * 2;
#pragma unroll
    for (int j = 0; j < 2; ++j)
      fb[kk % ST_LOOK][j] = __builtin_bit_cast(bf16x8, buffer_load16(r_v, vb_off, so + j * (4 * 64 * 8 * 2)));
  };
  auto stage_piece = [&](int step, auto slot_t, int c) {  // rotate, write Q, put the A operand into the stage's LDS tile
    constexpr int SLOT = decltype(slot_t)::value;
    unsigned short *sa = s_dyn + SLOT * ST_A_TILE;
    const uint4 q = rotate(ra[SLOT][c]);
    advance();
    const int kr = c * 32 + tk;
    buffer_store16(q, r_q, q_off, (step * 64 + c * 32) * 64 * 2);
    *reinterpret_cast<uint4 *>(sa + kr * ST_ASTRIDE + (mc ^ (((kr >> 3) & 1) << 5))) = q;
  };
  // bf16 of the accumulators, transposed to [value column][neuron]: each wavefront stages its own 64 value rows,
  // 32 at a time, in LDS rows of its own (LDS operations of one wavefront execute in order: no barrier), and
  // writes them as whole 128-byte row pieces
  auto dump = [&](int slot, bool remainder) {
    const __amdgpu_buffer_rsrc_t r_p = buffer_of(g.P + (long)slot * g.p_slot + (long)slice * g.p_slice + (long)(r % nt) * (256 * 64));
    const unsigned int dst_off = (unsigned int)((wave * 64 + (lane >> 3)) * 64 + (lane & 7) * 8) * 2u;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int e4 = 0; e4 < 4; ++e4) {
          unsigned int b[2];
#pragma unroll
          for (int e2 = 0; e2 < 2; ++e2) {  // round to nearest even by the conversion instruction, no branches
            const f32x2 v = {acc[i][j][e4 * 4 + 2 * e2], acc[i][j][e4 * 4 + 2 * e2 + 1]};
            unsigned int hi = __builtin_bit_cast(unsigned int, __builtin_convertvector(v, bf16x2));
            if (remainder) {
              const f32x2 rest = {v[0] - __uint_as_float(hi << 16), v[1] - __uint_as_float(hi & 0xffff0000u)};
              hi = __builtin_bit_cast(unsigned int, __builtin_convertvector(rest, bf16x2));
            }
            b[e2] = hi;
          }
          *reinterpret_cast<uint2 *>(s_stage + (lane & 31) * ST_DUMP_ROW + i * 32 + e4 * 8 + (lane >> 5) * 4) =
              make_uint2(b[0], b[1]);
        }
#pragma unroll
      for (int pass = 0; pass < 4; ++pass)
        buffer_store16(*reinterpret_cast<const uint4 *>(s_stage + (pass * 8 + (lane >> 3)) * ST_DUMP_ROW + (lane & 7) * 8),
                       r_p, dst_off, (j * 32 + pass * 8) * 64 * 2);
    }
  };

  // The token loop is laid out as straight-line code per 256-token chunk (four steps, no run-time branches
  // inside): the compiler counts outstanding memory operations statically, and only in a branch-free body does
  // it let the loads of the next step, the Q stores and the state copies stay in flight across the matrix
  // products instead of draining them at every join.  Tc is a multiple of 256 here.
  const int nc = g.Tc / 256;
  // step kt = 4 c + S_: staging of step kt + 1 (MORE), then the matrix products of step kt from LDS tile S_ & 1.
  // Memory operations of a wavefront complete in issue order, so a wait for a value fragment is also a wait for
  // every load and store issued before it.  Hence the order below: value fragments a whole step ahead (ST_LOOK = 4),
  // and the activations of step kt + 3 (MORE3; from HBM, the slowest) requested only after the third k-step's
  // fragment loads, into the registers the staging freed: the first wait that covers them is then a full step
  // away.  (Requested at the start of the step they stalled the second half of the same step's products;
  // fragments two k-steps ahead left every k-step waiting on the L2 latency.  Placing the rotation inside the
  // product regions or reading the A fragments one k-step ahead gained nothing.)
  auto step = [&](int kt, auto s_t, auto more_t, auto more3_t) {
    constexpr int S_ = decltype(s_t)::value;
    constexpr bool MORE = decltype(more_t)::value, MORE3 = decltype(more3_t)::value;
    using Next = std::integral_constant<int, (S_ + 1) & 1>;
    const unsigned short *s_a = s_dyn + (S_ & 1) * ST_A_TILE;
    if constexpr (MORE) {
#pragma unroll
      for (int c = 0; c < 2; ++c) stage_piece(kt + 1, Next{}, c);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      bf16x8 fa[2];
      const int kof = kk * 16 + (lane >> 5) * 8;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        // transposing LDS read: see k_gemm
        const int j16 = lane & 15;
        const int mcol = (i * 32 + ((lane >> 4) & 1) * 16) ^ ((lane >> 5) << 5);
        const unsigned short *src = s_a + (kof + (j16 >> 2)) * ST_ASTRIDE + mcol + (j16 & 3) * 4;
        typedef short s16x4 __attribute__((ext_vector_type(4)));
        typedef short s16x8 __attribute__((ext_vector_type(8)));
        typedef __attribute__((address_space(3))) s16x4 *lds_s16x4_t;
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_t)(src));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_t)(src + 4 * ST_ASTRIDE));
        const s16x8 pk = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        fa[i] = __builtin_bit_cast(bf16x8, pk);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[kk % ST_LOOK][j], acc[i][j], 0, 0, 0);
      // into the registers the products above just read: nothing may be scheduled across, or the compiler
      // hoists these loads over the products and keeps more sets of fragments alive
      __builtin_amdgcn_sched_barrier(0);
      if (kk + ST_LOOK < 4) load_b(kt, kk + ST_LOOK);
      else if constexpr (MORE) load_b(kt + 1, kk + ST_LOOK - 4);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (MORE3) {
        if (kk == 2) {
#pragma unroll
          for (int c = 0; c < 2; ++c) load_piece(kt + 3, Next{}, c);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
    lds_barrier();
  };
  auto chunk = [&](int c, auto last_t) {
    constexpr bool LAST = decltype(last_t)::value;
    using T = std::true_type;
    using NotLast = std::integral_constant<bool, !LAST>;
    const int kt = 4 * c;
    if (c != 0) dump(c, false);  // (slot 0 is the carried-in state, written in the prologue)
    step(kt, std::integral_constant<int, 0>{}, T{}, T{});
    step(kt + 1, std::integral_constant<int, 1>{}, T{}, NotLast{});
    step(kt + 2, std::integral_constant<int, 2>{}, T{}, NotLast{});
    if constexpr (!LAST) seed((kt + 4) * 64 + tk, std::true_type{});  // the next step opens a chunk: exact phases
    step(kt + 3, std::integral_constant<int, 3>{}, NotLast{}, NotLast{});
  };

  if (g.has_state) {
    dump(0, false);
    if (g.lo_slot >= 0) dump(g.lo_slot, true);
  }
  using Slot0 = std::integral_constant<int, 0>;
  using Slot1 = std::integral_constant<int, 1>;
  // every load the first step needs goes out before anything waits: the activations of steps 0 and 1, the value
  // fragments of step 0 (the first wait, for the activations of step 0, leaves the others in flight)
#pragma unroll
  for (int c = 0; c < 2; ++c) load_piece(0, Slot0{}, c);
#pragma unroll
  for (int c = 0; c < 2; ++c) load_piece(1, Slot1{}, c);
#pragma unroll
  for (int kk = 0; kk < ST_LOOK; ++kk) load_b(0, kk);
  __builtin_amdgcn_sched_barrier(0);
  if (tid < 64) s_freq[tid] = g.freqs[n0 + tid];
  seed(tk, std::false_type{});
#pragma unroll
  for (int c = 0; c < 2; ++c) stage_piece(0, Slot0{}, c);
#pragma unroll
  for (int c = 0; c < 2; ++c) load_piece(2, Slot0{}, c);
  lds_barrier();
#pragma unroll 1
  for (int c = 0; c + 1 < nc; ++c) chunk(c, std::false_type{});
  chunk(nc - 1, std::true_type{});
  // the addresses of the final stores equal those of the initial loads: hidden from the compiler here, or it
  // keeps all of them in registers across the token loop
  asm volatile("" : "+s"(rho));
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int col = wave * 64 + j * 32 + (lane & 31);
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int row = i * 32 + (e >> 2) * 8 + (e & 3);  // + 4 (lane >> 5), in the lane's offset
        *reinterpret_cast<float *>(at_w(rho + row * 256, (unsigned int)((lane >> 5) * 1024 + col) * 4u)) = acc[i][j][e];
      }
    }
}

#ifndef BDH_ST_WAVES
#define BDH_ST_WAVES 2
#endif
// one launch for both kinds of frequency table: the flag k_v_layouts wrote picks the body (uniform over the grid)
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(BDH_ST_WAVES, BDH_ST_WAVES))) void k_state_stream(StateUpdArgs g) {
  extern __shared__ __attribute__((aligned(1024))) unsigned short s_dyn[];
  if (g.pairs_equal[0] != 0) state_stream_body<true>(g, s_dyn);
  else state_stream_body<false>(g, s_dyn);
}

template <bool AK, int EPI>
hipError_t launch_gemm(hipStream_t st, const GemmArgs &g) {
  const int groups = (g.n_slices + 7) / 8;
  const bool full = !AK && g.M % BM == 0 && g.N % BN == 0 && g.K % BK == 0 && g.lda % 8 == 0 && g.ldb % 8 == 0 &&
                    ((EPI != EPI_SCORES && EPI != EPI_SCORES_X) || g.ldc == g.N);
  if constexpr (!AK) {
    if (full) {
      constexpr int lds = 4 * 256 * 64 * 2;  // two buffers of two 32 KiB tiles
      // the attribute belongs to the (kernel, device) pair: remember the devices already configured
      static std::atomic<uint64_t> configured{0};
      int dev = 0;
      hipError_t e = hipGetDevice(&dev);
      if (e != hipSuccess) return e;
      const uint64_t bit = 1ull << (dev & 63);
      if (!(configured.load(std::memory_order_acquire) & bit)) {
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(k_gemm_direct<EPI>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (e != hipSuccess) return e;
        configured.fetch_or(bit, std::memory_order_release);
      }
      hipLaunchKernelGGL((k_gemm_direct<EPI>), dim3(8 * groups * g.n_tiles), dim3(512), lds, st, g);
      return hipSuccess;
    }
  }
  hipLaunchKernelGGL((k_gemm<AK, EPI>), dim3(8 * groups * g.n_tiles), dim3(512), 0, st, g);
  return hipSuccess;
}

// What a pass of the all-scores form does beyond the RoPE recurrence.
struct PassMode {
  int rotary = BDH_ROPE;
  bool decay = false;       // ALiBi, recurrent semantics: rho <- (rho + q (x) v) * exp(-slope) per token
  bool row_norm = false;    // the stateless, row-normalised form of kernel::linear_attention::fused_state_aligned
  bool add_alibi = false;   // row_norm only: + slope * (s - t) on the causal time blocks
  int block_size = 1;       // row_norm + add_alibi: tokens per time block
  float head_par[64] = {};  // per head: log of the decay factor (decay) or the slope (add_alibi)
  bool extended() const { return rotary != BDH_ROPE || decay || row_norm; }
};

// One pass of the all-scores form (any T; N and d multiples of 8): tokens [0, T) of the pointers given,
// x / out slices x_slice / out_slice elements apart.  rho [S, Nq, d], Nq = 2N for PoPE.
static int prefill_pass_scores(bdh_ctx *ctx, int B, int h, int T, int N, int d, const uint16_t *x_bf16, long x_slice,
                               const uint16_t *v_bf16, long v_batch, const float *freqs, int64_t position,
                               int state_is_zero, float *rho, float *out, long out_slice,
                               const PassMode &pm = PassMode()) {
  const int S = B * h;
  const int Nq = pm.rotary == BDH_POPE ? 2 * N : N;
  const bool ext = pm.extended();
  const bool stateless = pm.row_norm;
  const int Tp = (T + 7) / 8 * 8;  // leading dimension of the score matrix
  const int mt = (T + BM - 1) / BM;  // row/col tiles of the score matrix
  const int nt_rho = (Nq + BM - 1) / BM, nt_d = (d + BN - 1) / BN;
  // a time block that straddles two score tiles has additive terms above the tile diagonal: all tiles then
  const bool full_grid = pm.row_norm && pm.add_alibi && (BM % pm.block_size) != 0;
  const int n_score_tiles = full_grid ? mt * mt : mt * (mt + 1) / 2;
  const int n_out_tiles = mt * nt_d, n_rho_tiles = nt_rho * nt_d;
  const bool own_q = pm.rotary != BDH_ALIBI;  // ALiBi does not rotate: the products read x itself

  // workspace: Q bf16 [S,T,Nq] | scores bf16 [S,T,Tp] | V^T bf16 [B or S,d,Tp] | rho0^T bf16 [S,d,Nq] |
  //            norm partials f32 [S,mt,T] | denominators f32 [S,T]
  const size_t q_bytes = own_q ? bdh_align_up((size_t)S * T * Nq * 2, 256) : 0;
  const size_t s_bytes = bdh_align_up((size_t)S * T * Tp * 2, 256);
  const size_t vt_bytes = bdh_align_up((size_t)(pm.decay ? S : B) * d * Tp * 2, 256);
  const size_t vs_bytes = pm.decay ? bdh_align_up((size_t)B * d * Tp * 2, 256) : 0;  // undecayed V^T for S V
  const size_t rt_bytes = (state_is_zero || stateless) ? 0 : bdh_align_up((size_t)S * d * Nq * 2, 256);
  const size_t np_bytes = pm.row_norm ? bdh_align_up((size_t)S * mt * T * 4, 256) : 0;
  const size_t dn_bytes = pm.row_norm ? bdh_align_up((size_t)S * T * 4, 256) : 0;
  int rc = bdh_ws_reserve(ctx, q_bytes + s_bytes + vt_bytes + vs_bytes + rt_bytes + np_bytes + dn_bytes);
  if (rc != BDH_OK) return rc;
  char *ws = static_cast<char *>(ctx->ws);
  size_t off = 0;
  auto take = [&](size_t bytes) { char *p = ws + off; off += bytes; return p; };
  unsigned short *Qw = reinterpret_cast<unsigned short *>(take(q_bytes));
  unsigned short *Sc = reinterpret_cast<unsigned short *>(take(s_bytes));
  unsigned short *Vt = reinterpret_cast<unsigned short *>(take(vt_bytes));   // decayed per slice when pm.decay
  unsigned short *Vs = pm.decay ? reinterpret_cast<unsigned short *>(take(vs_bytes)) : Vt;  // plain, per batch entry
  unsigned short *Rt = reinterpret_cast<unsigned short *>(take(rt_bytes));
  float *norm_part = reinterpret_cast<float *>(take(np_bytes));
  float *denom = reinterpret_cast<float *>(take(dn_bytes));
  const unsigned short *Q = own_q ? Qw : reinterpret_cast<const unsigned short *>(x_bf16);
  const long q_slice = own_q ? (long)T * Nq : x_slice;
  if ((long)S * n_score_tiles > 0x7fffffffL / 16 || (long)S * n_rho_tiles > 0x7fffffffL / 16)
    return bdh_fail(ctx, BDH_E_SHAPE, "too many tiles (T=%d N=%d)", T, N);
  auto with_mode = [&](GemmArgs &g, int mode) {
    g.mode = mode; g.h = h; g.block_size = pm.block_size; g.norm_part = norm_part; g.denom = denom;
    memcpy(g.head_par, pm.head_par, sizeof(g.head_par));
  };

  // 0. V^T (and rho0^T): make every B operand k-contiguous
  hipLaunchKernelGGL(k_transpose_to_bf16<unsigned short>, dim3((d + 63) / 64, (Tp + 63) / 64, B), dim3(256), 0,
                     ctx->stream, v_bf16, Vs, T, d, Tp, v_batch);
  BDH_LAUNCH_CHECK(ctx, "k_transpose_to_bf16<V>");
  if (pm.decay) {
    HeadPar hp;
    memcpy(hp.v, pm.head_par, sizeof(hp.v));
    hipLaunchKernelGGL(k_transpose_decay_bf16, dim3((d + 63) / 64, (Tp + 63) / 64, S), dim3(256), 0, ctx->stream,
                       v_bf16, Vt, T, d, Tp, v_batch, h, hp);
    BDH_LAUNCH_CHECK(ctx, "k_transpose_decay_bf16");
  }
  if (!state_is_zero && !stateless) {
    hipLaunchKernelGGL(k_transpose_to_bf16<float>, dim3((d + 63) / 64, (Nq + 63) / 64, S), dim3(256), 0, ctx->stream,
                       rho, Rt, Nq, d, Nq, (long)Nq * d);
    BDH_LAUNCH_CHECK(ctx, "k_transpose_to_bf16<rho0>");
  }
  // 1. rotation
  if (own_q) {
    const long work = (long)T * (N / 8);
    if (pm.rotary == BDH_POPE)
      hipLaunchKernelGGL(k_pope_bf16, dim3((unsigned)((work + 255) / 256)), dim3(256), 0, ctx->stream,
                         reinterpret_cast<const uint4 *>(x_bf16), reinterpret_cast<uint4 *>(Qw), freqs, S, T, N,
                         x_slice / 8, (long)position);
    else
      hipLaunchKernelGGL(k_rope_bf16, dim3((unsigned)((work + 255) / 256)), dim3(256), 0, ctx->stream,
                         reinterpret_cast<const uint4 *>(x_bf16), reinterpret_cast<uint4 *>(Qw), freqs, S, T, N,
                         x_slice / 8, (long)position);
    BDH_LAUNCH_CHECK(ctx, "k_rope_bf16 / k_pope_bf16");
  }
  // 2. scores = tril(-1)(Q Q^T), lower tiles only
  {
    GemmArgs g{};
    g.A = Q; g.B = Q; g.C = Sc;
    g.a_batch = q_slice; g.b_batch = q_slice; g.c_batch = (long)T * Tp;
    g.lda = Nq; g.ldb = Nq; g.ldc = Tp;
    g.M = T; g.N = T; g.K = Nq; g.b_div = 1; g.beta = 0; g.causal_k = 0;
    g.tri = full_grid ? 0 : 1; g.mt = mt; g.nt = mt; g.n_tiles = n_score_tiles; g.n_slices = S;
    if (ext) {
      with_mode(g, (pm.decay ? GM_DECAY_SCORES : 0) | (pm.add_alibi ? GM_ADD_ALIBI : 0) | (pm.row_norm ? GM_ROWNORM : 0));
      BDH_HIP_CHECK(ctx, (launch_gemm<false, EPI_SCORES_X>(ctx->stream, g)));
    } else {
      BDH_HIP_CHECK(ctx, (launch_gemm<false, EPI_SCORES>(ctx->stream, g)));
    }
    BDH_LAUNCH_CHECK(ctx, "k_gemm<scores>");
  }
  if (pm.row_norm) {
    hipLaunchKernelGGL(k_norm_reduce, dim3((T + 255) / 256, S), dim3(256), 0, ctx->stream, norm_part, denom, T, mt,
                       full_grid ? 0 : 1, 1e-6f);
    BDH_LAUNCH_CHECK(ctx, "k_norm_reduce");
  }
  // 3a. out = Q rho0 (skipped for a fresh state; a decaying state has lost exp(-slope)^t by row t)
  if (!state_is_zero && !stateless) {
    GemmArgs g{};
    g.A = Q; g.B = Rt; g.C = out;
    g.a_batch = q_slice; g.b_batch = (long)d * Nq; g.c_batch = out_slice;
    g.lda = Nq; g.ldb = Nq; g.ldc = d;
    g.M = T; g.N = d; g.K = Nq; g.b_div = 1; g.beta = 0; g.causal_k = 0;
    g.tri = 0; g.mt = mt; g.nt = nt_d; g.n_tiles = n_out_tiles; g.n_slices = S;
    if (pm.decay) {
      with_mode(g, GM_DECAY_ROWS);
      BDH_HIP_CHECK(ctx, (launch_gemm<false, EPI_ACC_X>(ctx->stream, g)));
    } else {
      BDH_HIP_CHECK(ctx, (launch_gemm<false, EPI_ACC>(ctx->stream, g)));
    }
    BDH_LAUNCH_CHECK(ctx, "k_gemm<Q rho0>");
  }
  // 3b. out (+)= scores V   (row-normalised form: divided by the row's sum of |scores| + eps)
  {
    GemmArgs g{};
    g.A = Sc; g.B = Vs; g.C = out;
    g.a_batch = (long)T * Tp; g.b_batch = (long)d * Tp; g.c_batch = out_slice;
    g.lda = Tp; g.ldb = Tp; g.ldc = d;
    g.M = T; g.N = d; g.K = T; g.b_div = h; g.beta = (state_is_zero || stateless) ? 0 : 1;
    g.causal_k = full_grid ? 0 : 1;
    g.tri = 0; g.mt = mt; g.nt = nt_d; g.n_tiles = n_out_tiles; g.n_slices = S;
    if (pm.row_norm) {
      with_mode(g, GM_DIVNORM);
      BDH_HIP_CHECK(ctx, (launch_gemm<false, EPI_ACC_X>(ctx->stream, g)));
    } else {
      BDH_HIP_CHECK(ctx, (launch_gemm<false, EPI_ACC>(ctx->stream, g)));
    }
    BDH_LAUNCH_CHECK(ctx, "k_gemm<S V>");
  }
  // 4. rho (+)= Q^T V   (A = Q read k-major; a decaying state: rho = g^T rho + sum_s g^(T-s) q_s (x) v_s)
  if (!stateless) {
    GemmArgs g{};
    g.A = Q; g.B = Vt; g.C = rho;
    g.a_batch = q_slice; g.b_batch = (long)d * Tp; g.c_batch = (long)Nq * d;
    g.lda = Nq; g.ldb = Tp; g.ldc = d;
    g.M = Nq; g.N = d; g.K = T; g.b_div = pm.decay ? 1 : h; g.beta = state_is_zero ? 0 : 1; g.causal_k = 0;
    g.tri = 0; g.mt = nt_rho; g.nt = nt_d; g.n_tiles = n_rho_tiles; g.n_slices = S;
    if (pm.decay) {
      with_mode(g, GM_DECAY_STATE);
      BDH_HIP_CHECK(ctx, (launch_gemm<true, EPI_ACC_X>(ctx->stream, g)));
    } else {
      BDH_HIP_CHECK(ctx, (launch_gemm<true, EPI_ACC>(ctx->stream, g)));
    }
    BDH_LAUNCH_CHECK(ctx, "k_gemm<Q^T V>");
  }
  return BDH_OK;
}

// dynamic LDS beyond 64 KiB must be allowed per (kernel, device)
template <typename K>
static hipError_t allow_lds(K kernel, int bytes, std::atomic<uint64_t> &configured) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  const uint64_t bit = 1ull << (dev & 63);
  if (configured.load(std::memory_order_acquire) & bit) return hipSuccess;
  e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e == hipSuccess) configured.fetch_or(bit, std::memory_order_release);
  return e;
}

// One pass of the chunk-recurrent form: Tc tokens (a multiple of 256), N a multiple of 256, d = 256.
static int prefill_pass_chunks(bdh_ctx *ctx, int B, int h, int Tc, int N, const uint16_t *x_bf16, long x_slice,
                               const uint16_t *v_bf16, long v_batch, const float *freqs, int64_t position,
                               int state_is_zero, int hilo, float *rho, float *out, long out_slice) {
  constexpr int d = 256;
  const int S = B * h, nc = Tc / 256;
  const int lo_slot = (!state_is_zero && hilo) ? nc : -1;
  const int slots = nc + (lo_slot >= 0 ? 1 : 0);
  // workspace: Q bf16 [S,N/64,Tc,64] | P bf16 [slots,S,N/64,d,64] | V^T bf16 [B,d,Tc] | V in fragment order (same size)
  const size_t q_bytes = bdh_align_up((size_t)S * Tc * N * 2, 256);
  const size_t p_bytes = bdh_align_up((size_t)slots * S * d * N * 2, 256);
  const size_t vt_bytes = bdh_align_up((size_t)B * d * Tc * 2, 256);
  int rc = bdh_ws_reserve(ctx, q_bytes + p_bytes + 2 * vt_bytes + 256);
  if (rc != BDH_OK) return rc;
  char *ws = static_cast<char *>(ctx->ws);
  unsigned short *Q = reinterpret_cast<unsigned short *>(ws);
  unsigned short *P = reinterpret_cast<unsigned short *>(ws + q_bytes);
  unsigned short *Vt = reinterpret_cast<unsigned short *>(ws + q_bytes + p_bytes);
  unsigned short *Vf = reinterpret_cast<unsigned short *>(ws + q_bytes + p_bytes + vt_bytes);
  int *flag = reinterpret_cast<int *>(ws + q_bytes + p_bytes + 2 * vt_bytes);
  const int groups = (S + 7) / 8;
  if ((long)groups * 8 * std::max(N / ST_TN, nc) > 0x7fffffffL) return bdh_fail(ctx, BDH_E_SHAPE, "too many tiles");
  // k_state_stream addresses a slice's activations by 32-bit byte offsets
  if ((long)Tc * N * 2 > 0x7fffffffL) return bdh_fail(ctx, BDH_E_SHAPE, "pass too long for 32-bit offsets (Tc=%d N=%d)", Tc, N);

  hipLaunchKernelGGL(k_v_layouts, dim3(Tc / 64, B, 4), dim3(256), 0, ctx->stream, v_bf16, v_batch, Vf, Vt, Tc, freqs, N, flag);
  BDH_LAUNCH_CHECK(ctx, "k_v_layouts");
  {
    static std::atomic<uint64_t> configured_st{0};
    BDH_HIP_CHECK(ctx, allow_lds(k_state_stream, ST_LDS, configured_st));
    StateUpdArgs g{};
    g.X = x_bf16; g.x_slice = x_slice;
    g.Q = Q; g.q_slice = (long)Tc * N;
    g.Vf = Vf; g.vt_batch = (long)d * Tc;
    g.freqs = freqs; g.rho = rho;
    g.P = P; g.p_slot = (long)S * d * N; g.p_slice = (long)d * N;
    g.pos0 = (long)position;
    g.N = N; g.Tc = Tc; g.h = h; g.n_slices = S;
    g.has_state = state_is_zero ? 0 : 1; g.lo_slot = lo_slot;
    g.pairs_equal = flag;
    const int nts = N / ST_TN;
    hipLaunchKernelGGL(k_state_stream, dim3(8 * groups * nts), dim3(256), ST_LDS, ctx->stream, g);
    BDH_LAUNCH_CHECK(ctx, "k_state_stream");
  }
  {
    static std::atomic<uint64_t> configured{0};
    BDH_HIP_CHECK(ctx, allow_lds(k_chunk_out, CHUNK_OUT_LDS, configured));
    ChunkOutArgs g{};
    g.Q = Q; g.q_slice = (long)Tc * N;
    g.P = P; g.p_slot = (long)S * d * N; g.p_slice = (long)d * N;
    g.Vt = Vt; g.vt_batch = (long)d * Tc; g.ldv = Tc;
    g.out = out; g.out_slice = out_slice;
    g.N = N; g.nc = nc; g.n_slices = S; g.h = h;
    g.has_state = state_is_zero ? 0 : 1; g.lo_slot = lo_slot;
    hipLaunchKernelGGL(k_chunk_out, dim3(8 * groups * nc), dim3(512), CHUNK_OUT_LDS, ctx->stream, g);
    BDH_LAUNCH_CHECK(ctx, "k_chunk_out");
  }
  return BDH_OK;
}

}  // namespace

// Shared body of the two entry points.  pm: what goes beyond the RoPE recurrence (all-scores form only).
static int prefill_chunked_impl(bdh_ctx *ctx, int B, int h, int T, int N, int d, const uint16_t *x_bf16,
                                const uint16_t *v_bf16, const float *freqs, int64_t position, int chunk, int flags,
                                float *rho, float *out, const PassMode &pm) {
  if (B < 0 || h < 0 || T < 0 || N < 0 || d < 0) return bdh_fail(ctx, BDH_E_INVAL, "negative dimension");
  if (position < 0) return bdh_fail(ctx, BDH_E_INVAL, "negative position");
  if (chunk < 0) return bdh_fail(ctx, BDH_E_INVAL, "negative chunk length");
  if (B == 0 || h == 0 || T == 0) return BDH_OK;
  // RoPE keeps the contract of bdh_prefill_chunked (N and d multiples of 8); the other forms only read x in
  // 16-byte pieces
  if ((N & 7) || N == 0 || d == 0 || (!pm.extended() && (d & 7)))
    return bdh_fail(ctx, BDH_E_SHAPE, "chunked prefill needs N%s to be positive multiples of 8 (N=%d d=%d)",
                    pm.extended() ? "" : " and d", N, d);
  const bool stateless = pm.row_norm;
  if (!x_bf16 || !v_bf16 || !out || (!stateless && !rho) || (pm.rotary != BDH_ALIBI && !freqs))
    return bdh_fail(ctx, BDH_E_INVAL, "null data pointer");
  if (!bdh_aligned(x_bf16, 16) || !bdh_aligned(v_bf16, 16) || (rho && !bdh_aligned(rho, 16)) || !bdh_aligned(out, 16))
    return bdh_fail(ctx, BDH_E_ALIGN, "x, v, rho and out need 16-byte alignment");
  if (B > 65535 || B * h > 65535) return bdh_fail(ctx, BDH_E_SHAPE, "batch too large for the transpose grid");
  // tokens per pass: the workspace holds the rotated activations (and, in the all-scores form, the score
  // matrix) of one pass only; the state is carried from pass to pass in the caller's f32 rho
  const int pass_default = 2048;
  int pass = chunk > 0 ? chunk : pass_default;
  if (stateless) {  // the normaliser needs whole score rows: one pass
    if ((double)B * h * T * T * 2.0 > 64.0 * 1024 * 1024 * 1024)
      return bdh_fail(ctx, BDH_E_SHAPE, "row-normalised form: the score matrix of B*h=%d, T=%d exceeds 64 GiB", B * h, T);
    pass = T;
  }
  const bool aligned = !pm.extended() && !(flags & BDH_PREFILL_ALL_SCORES) && d == 256 && N % 256 == 0;
  int zero = ((flags & BDH_PREFILL_STATE_IS_ZERO) || stateless) ? 1 : 0;
  const int hilo = (flags & BDH_PREFILL_STATE_HILO) ? 1 : 0;
  for (int t0 = 0; t0 < T;) {
    int Tc = std::min(pass, T - t0);
    const uint16_t *xp = x_bf16 + (long)t0 * N;
    const uint16_t *vp = v_bf16 + (long)t0 * d;
    float *op = out + (long)t0 * d;
    int rc;
    if (aligned && Tc >= 256) {
      Tc -= Tc % 256;  // a ragged tail goes to the all-scores form below
      rc = prefill_pass_chunks(ctx, B, h, Tc, N, xp, (long)T * N, vp, (long)T * d, freqs, position + t0, zero, hilo, rho,
                               op, (long)T * d);
    } else {
      rc = prefill_pass_scores(ctx, B, h, Tc, N, d, xp, (long)T * N, vp, (long)T * d, freqs, position + t0, zero, rho,
                               op, (long)T * d, pm);
    }
    if (rc != BDH_OK) return rc;
    zero = 0;
    t0 += Tc;
  }
  return BDH_OK;
}

namespace {

// in f32 [n] -> out bf16 [n], rounded to nearest even
__global__ __launch_bounds__(256) void k_f32_to_bf16(const float *__restrict__ in, unsigned short *__restrict__ out, size_t n) {
  const size_t n4 = n / 4;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n4; i += (size_t)gridDim.x * 256) {
    const float4 v = reinterpret_cast<const float4 *>(in)[i];
    uint2 o;
    o.x = (unsigned int)f32_to_bf16_bits(v.x) | ((unsigned int)f32_to_bf16_bits(v.y) << 16);
    o.y = (unsigned int)f32_to_bf16_bits(v.z) | ((unsigned int)f32_to_bf16_bits(v.w) << 16);
    reinterpret_cast<uint2 *>(out)[i] = o;
  }
  if (blockIdx.x == 0 && threadIdx.x < n - n4 * 4) out[n4 * 4 + threadIdx.x] = f32_to_bf16_bits(in[n4 * 4 + threadIdx.x]);
}

__global__ __launch_bounds__(256) void k_fill_i32(int32_t *__restrict__ p, long n, int32_t v) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = v;
}

}  // namespace

int bdh_launch_state_prefill_bf16(bdh_ctx *ctx, const StateStepParams &p, float *out_ln) {
  const int B = p.B, h = p.h, T = p.T, N = p.N, d = p.d;
  if (p.rho_dtype != BDH_F32 || p.positions_dev || p.bitmask || p.rows_touched)
    return bdh_fail(ctx, BDH_E_UNSUPPORTED, "the bf16 prompt form takes an f32 state, a host position and no by-products");
  if (p.stamps && p.rotary != BDH_ALIBI) return bdh_fail(ctx, BDH_E_INVAL, "decay stamps only apply to ALiBi");
  if (p.stamps && p.position + T > 0x7fffffffLL) return bdh_fail(ctx, BDH_E_INVAL, "position beyond the stamp range");
  PassMode pm;
  pm.rotary = p.rotary;
  if (p.rotary == BDH_ALIBI) {
    if (h > 64) return bdh_fail(ctx, BDH_E_SHAPE, "at most 64 heads with ALiBi slopes (h=%d)", h);
    pm.decay = true;
    for (int i = 0; i < h; ++i) pm.head_par[i] = (float)log((double)expf(-p.slopes_host[i]));
  }
  if (p.stamps) {  // a lazily decayed state: apply what is pending, the products decay every row themselves
    const int rc0 = bdh_launch_alibi_materialize(ctx, B, h, N, d, p.slopes_host, p.position, nullptr, p.rho, p.rho_dtype,
                                                 p.stamps);
    if (rc0 != BDH_OK) return rc0;
  }
  const size_t nx = (size_t)B * h * T * N, nv = (size_t)B * T * d;
  const size_t x_bytes = bdh_align_up(nx * 2, 256);
  int rc = bdh_stage_reserve(ctx, x_bytes + bdh_align_up(nv * 2, 256));
  if (rc != BDH_OK) return rc;
  unsigned short *xb = static_cast<unsigned short *>(ctx->stage);
  unsigned short *vb = reinterpret_cast<unsigned short *>(static_cast<char *>(ctx->stage) + x_bytes);
  hipLaunchKernelGGL(k_f32_to_bf16, dim3((unsigned)std::min<size_t>((nx / 4 + 255) / 256 + 1, 1u << 16)), dim3(256), 0,
                     ctx->stream, p.x, xb, nx);
  BDH_LAUNCH_CHECK(ctx, "k_f32_to_bf16<x>");
  hipLaunchKernelGGL(k_f32_to_bf16, dim3((unsigned)std::min<size_t>((nv / 4 + 255) / 256 + 1, 1u << 16)), dim3(256), 0,
                     ctx->stream, p.v, vb, nv);
  BDH_LAUNCH_CHECK(ctx, "k_f32_to_bf16<v>");
  rc = prefill_chunked_impl(ctx, B, h, T, N, d, xb, vb, p.freqs, p.position, 0, 0, static_cast<float *>(p.rho), p.out, pm);
  if (rc != BDH_OK) return rc;
  if (p.stamps) {  // every row is now up to date as of the end of the call
    const long rows = (long)B * h * N;
    hipLaunchKernelGGL(k_fill_i32, dim3((unsigned)((rows + 255) / 256)), dim3(256), 0, ctx->stream, p.stamps, rows,
                       (int32_t)(p.position + T));
    BDH_LAUNCH_CHECK(ctx, "k_fill_i32");
  }
  if (out_ln) return bdh_launch_layer_norm_rows(ctx, (int64_t)B * h * T, d, p.out, out_ln);
  return BDH_OK;
}

// kernel::linear_attention::fused_state_aligned with the dense causal layout on the bf16 matrix cores: f32 inputs
// rounded to bf16 in the context's staging buffer, then the row-normalised form of bdh_prefill_chunked_ex.
int bdh_launch_fsa_bf16(bdh_ctx *ctx, int B, int h, int T, int N, int dv, const float *query, const float *value,
                        const float *freqs, const float *alibi_slopes_host, int block_size, int rotary, float *out) {
  PassMode pm;
  pm.rotary = rotary;
  pm.row_norm = true;
  pm.block_size = block_size > 0 ? block_size : 1;
  pm.add_alibi = alibi_slopes_host != nullptr;
  if (pm.add_alibi) {
    if (h > 64) return bdh_fail(ctx, BDH_E_SHAPE, "at most 64 heads with ALiBi slopes (h=%d)", h);
    memcpy(pm.head_par, alibi_slopes_host, sizeof(float) * h);
  }
  const size_t nx = (size_t)B * h * T * N, nv = (size_t)B * T * dv;
  const size_t x_bytes = bdh_align_up(nx * 2, 256);
  int rc = bdh_stage_reserve(ctx, x_bytes + bdh_align_up(nv * 2, 256));
  if (rc != BDH_OK) return rc;
  unsigned short *xb = static_cast<unsigned short *>(ctx->stage);
  unsigned short *vb = reinterpret_cast<unsigned short *>(static_cast<char *>(ctx->stage) + x_bytes);
  hipLaunchKernelGGL(k_f32_to_bf16, dim3((unsigned)std::min<size_t>((nx / 4 + 255) / 256 + 1, 1u << 16)), dim3(256), 0,
                     ctx->stream, query, xb, nx);
  BDH_LAUNCH_CHECK(ctx, "k_f32_to_bf16<query>");
  hipLaunchKernelGGL(k_f32_to_bf16, dim3((unsigned)std::min<size_t>((nv / 4 + 255) / 256 + 1, 1u << 16)), dim3(256), 0,
                     ctx->stream, value, vb, nv);
  BDH_LAUNCH_CHECK(ctx, "k_f32_to_bf16<value>");
  return prefill_chunked_impl(ctx, B, h, T, N, dv, xb, vb, freqs, 0, 0, 0, nullptr, out, pm);
}

extern "C" int bdh_prefill_chunked(bdh_ctx *ctx, int B, int h, int T, int N, int d, const uint16_t *x_bf16,
                                   const uint16_t *v_bf16, const float *freqs, int64_t position, int chunk,
                                   int flags, float *rho, float *out) {
  if (!ctx) return BDH_E_INVAL;
  if (flags & ~(BDH_PREFILL_STATE_IS_ZERO | BDH_PREFILL_STATE_HILO | BDH_PREFILL_ALL_SCORES))
    return bdh_fail(ctx, BDH_E_INVAL, "unknown flag bits 0x%x", flags);
  return prefill_chunked_impl(ctx, B, h, T, N, d, x_bf16, v_bf16, freqs, position, chunk, flags, rho, out, PassMode());
}

extern "C" int bdh_prefill_chunked_ex(bdh_ctx *ctx, int B, int h, int T, int N, int d, int rotary,
                                      const uint16_t *x_bf16, const uint16_t *v_bf16, const float *freqs,
                                      const float *alibi_slopes_host, int64_t position, int chunk, int flags,
                                      int block_size, float *rho, float *out) {
  if (!ctx) return BDH_E_INVAL;
  if (flags & ~(BDH_PREFILL_STATE_IS_ZERO | BDH_PREFILL_STATE_HILO | BDH_PREFILL_ALL_SCORES | BDH_PREFILL_ROW_NORMALIZE))
    return bdh_fail(ctx, BDH_E_INVAL, "unknown flag bits 0x%x", flags);
  if (rotary != BDH_ROPE && rotary != BDH_ALIBI && rotary != BDH_POPE)
    return bdh_fail(ctx, BDH_E_INVAL, "unknown rotary mode %d", rotary);
  PassMode pm;
  pm.rotary = rotary;
  pm.row_norm = (flags & BDH_PREFILL_ROW_NORMALIZE) != 0;
  pm.block_size = block_size > 0 ? block_size : 1;
  float slopes[64];
  if (pm.row_norm) {
    // kernel::linear_attention::fused_state_aligned: the additive term exists when slopes are given (:44-51)
    pm.add_alibi = alibi_slopes_host != nullptr;
    if (pm.add_alibi) {
      if (h > 64) return bdh_fail(ctx, BDH_E_SHAPE, "at most 64 heads with ALiBi slopes (h=%d)", h);
      memcpy(pm.head_par, alibi_slopes_host, sizeof(float) * h);
    }
  } else if (rotary == BDH_ALIBI) {
    // BDH::recurrent_attention: the state decays by exp(-slope) after every token (src/model/bdh.rs:299-301)
    if (h > 64) return bdh_fail(ctx, BDH_E_SHAPE, "at most 64 heads with ALiBi slopes (h=%d)", h);
    if (alibi_slopes_host) memcpy(slopes, alibi_slopes_host, sizeof(float) * h);
    else bdh_default_alibi_slopes(h, slopes);
    pm.decay = true;
    // log of the ROUNDED per-token factor (src/model/attention.rs:181-186), as the lazily decayed step uses it
    for (int i = 0; i < h; ++i) pm.head_par[i] = (float)log((double)expf(-slopes[i]));
  }
  return prefill_chunked_impl(ctx, B, h, T, N, d, x_bf16, v_bf16, freqs, position, chunk, flags, rho, out, pm);
}
