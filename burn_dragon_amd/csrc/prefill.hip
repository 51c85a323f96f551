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
#include <atomic>

#include "bdh_internal.h"

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

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
                                                   float pos0_f, long pos0) {
  const int groups = N >> 3;  // 8 elements (4 pairs) per thread
  const long gid = (long)blockIdx.x * 256 + threadIdx.x;
  if (gid >= (long)T * groups) return;
  const int t = (int)(gid / groups), g = (int)(gid - (long)t * groups);
  const float pos = (float)(pos0 + t);
  (void)pos0_f;
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
    for (int u = 0; u < 8; ++u) in[u] = x[((long)(s + u) * T + t) * groups + g];
#pragma unroll
    for (int u = 0; u < 8; ++u) q[((long)(s + u) * T + t) * groups + g] = rotate(in[u]);
  }
  for (; s < S; ++s) {
    const long off = ((long)s * T + t) * groups + g;
    q[off] = rotate(x[off]);
  }
}

// ------------------------------------------------------------------------------------
// batched transpose to bf16: in [batch][R][C] (f32 or bf16) -> out [batch][C][ldo], ldo >= R,
// columns R..ldo-1 of the output are zero-filled.  64x64 tiles through LDS.
// ------------------------------------------------------------------------------------
template <typename TIn>
__global__ __launch_bounds__(256) void k_transpose_to_bf16(const TIn *__restrict__ in, unsigned short *__restrict__ out,
                                                          int R, int C, int ldo) {
  __shared__ unsigned short tile[64][66];
  const long batch = blockIdx.z;
  const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  const TIn *src = in + batch * (long)R * C;
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

// ------------------------------------------------------------------------------------
// batched GEMM  C[m,n] (+)= sum_k A[m,k] B[n,k]
// ------------------------------------------------------------------------------------
enum { EPI_SCORES = 0, EPI_ACC = 1 };

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
};

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
  const bool same_ab = EPI == EPI_SCORES && g.tri && ti == tj && g.A == g.B && g.b_div == 1;
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

template <bool AK, int EPI>
hipError_t launch_gemm(hipStream_t st, const GemmArgs &g) {
  const int groups = (g.n_slices + 7) / 8;
  const bool full = !AK && g.M % BM == 0 && g.N % BN == 0 && g.K % BK == 0 && g.lda % 8 == 0 && g.ldb % 8 == 0 &&
                    (EPI != EPI_SCORES || g.ldc == g.N);
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

}  // namespace

extern "C" int bdh_prefill_chunked(bdh_ctx *ctx, int B, int h, int T, int N, int d, const uint16_t *x_bf16,
                                   const uint16_t *v_bf16, const float *freqs, int64_t position,
                                   int state_is_zero, float *rho, float *out) {
  if (!ctx) return BDH_E_INVAL;
  if (B < 0 || h < 0 || T < 0 || N < 0 || d < 0) return bdh_fail(ctx, BDH_E_INVAL, "negative dimension");
  if (position < 0) return bdh_fail(ctx, BDH_E_INVAL, "negative position");
  if (B == 0 || h == 0 || T == 0) return BDH_OK;
  if ((N & 7) || (d & 7) || N == 0 || d == 0)
    return bdh_fail(ctx, BDH_E_SHAPE, "chunked prefill needs N and d to be positive multiples of 8 (N=%d d=%d)", N, d);
  if (!x_bf16 || !v_bf16 || !freqs || !rho || !out) return bdh_fail(ctx, BDH_E_INVAL, "null data pointer");
  if (!bdh_aligned(x_bf16, 16) || !bdh_aligned(v_bf16, 16) || !bdh_aligned(rho, 16) || !bdh_aligned(out, 16))
    return bdh_fail(ctx, BDH_E_ALIGN, "x, v, rho and out need 16-byte alignment");
  const int S = B * h;
  const int Tp = (T + 7) / 8 * 8;  // leading dimension of the score matrix
  const int mt = (T + BM - 1) / BM;  // row/col tiles of the score matrix
  const int nt_rho = (N + BM - 1) / BM, nt_d = (d + BN - 1) / BN;
  const int n_score_tiles = mt * (mt + 1) / 2;
  const int n_out_tiles = mt * nt_d, n_rho_tiles = nt_rho * nt_d;

  // workspace: Q bf16 [S,T,N] | scores bf16 [S,T,Tp] | V^T bf16 [B,d,Tp] | rho0^T bf16 [S,d,N]
  const size_t q_bytes = bdh_align_up((size_t)S * T * N * 2, 256);
  const size_t s_bytes = bdh_align_up((size_t)S * T * Tp * 2, 256);
  const size_t vt_bytes = bdh_align_up((size_t)B * d * Tp * 2, 256);
  const size_t rt_bytes = state_is_zero ? 0 : bdh_align_up((size_t)S * d * N * 2, 256);
  int rc = bdh_ws_reserve(ctx, q_bytes + s_bytes + vt_bytes + rt_bytes);
  if (rc != BDH_OK) return rc;
  char *ws = static_cast<char *>(ctx->ws);
  unsigned short *Q = reinterpret_cast<unsigned short *>(ws);
  unsigned short *Sc = reinterpret_cast<unsigned short *>(ws + q_bytes);
  unsigned short *Vt = reinterpret_cast<unsigned short *>(ws + q_bytes + s_bytes);
  unsigned short *Rt = reinterpret_cast<unsigned short *>(ws + q_bytes + s_bytes + vt_bytes);
  if ((long)S * n_score_tiles > 0x7fffffffL / 16 || (long)S * n_rho_tiles > 0x7fffffffL / 16)
    return bdh_fail(ctx, BDH_E_SHAPE, "too many tiles (T=%d N=%d)", T, N);
  if (B > 65535 || S > 65535) return bdh_fail(ctx, BDH_E_SHAPE, "batch too large for the transpose grid");

  // 0. V^T (and rho0^T): make every B operand k-contiguous
  hipLaunchKernelGGL(k_transpose_to_bf16<unsigned short>, dim3((d + 63) / 64, (Tp + 63) / 64, B), dim3(256), 0,
                     ctx->stream, v_bf16, Vt, T, d, Tp);
  BDH_LAUNCH_CHECK(ctx, "k_transpose_to_bf16<V>");
  if (!state_is_zero) {
    hipLaunchKernelGGL(k_transpose_to_bf16<float>, dim3((d + 63) / 64, (N + 63) / 64, S), dim3(256), 0, ctx->stream,
                       rho, Rt, N, d, N);
    BDH_LAUNCH_CHECK(ctx, "k_transpose_to_bf16<rho0>");
  }
  // 1. rotation
  {
    const long work = (long)T * (N / 8);
    hipLaunchKernelGGL(k_rope_bf16, dim3((unsigned)((work + 255) / 256)), dim3(256), 0, ctx->stream,
                       reinterpret_cast<const uint4 *>(x_bf16), reinterpret_cast<uint4 *>(Q), freqs, S, T, N,
                       (float)position, (long)position);
    BDH_LAUNCH_CHECK(ctx, "k_rope_bf16");
  }
  // 2. scores = tril(-1)(Q Q^T), lower tiles only
  {
    GemmArgs g{};
    g.A = Q; g.B = Q; g.C = Sc;
    g.a_batch = (long)T * N; g.b_batch = (long)T * N; g.c_batch = (long)T * Tp;
    g.lda = N; g.ldb = N; g.ldc = Tp;
    g.M = T; g.N = T; g.K = N; g.b_div = 1; g.beta = 0; g.causal_k = 0;
    g.tri = 1; g.mt = mt; g.nt = mt; g.n_tiles = n_score_tiles; g.n_slices = S;
    BDH_HIP_CHECK(ctx, (launch_gemm<false, EPI_SCORES>(ctx->stream, g)));
    BDH_LAUNCH_CHECK(ctx, "k_gemm<scores>");
  }
  // 3a. out = Q rho0 (skipped for a fresh state)
  if (!state_is_zero) {
    GemmArgs g{};
    g.A = Q; g.B = Rt; g.C = out;
    g.a_batch = (long)T * N; g.b_batch = (long)d * N; g.c_batch = (long)T * d;
    g.lda = N; g.ldb = N; g.ldc = d;
    g.M = T; g.N = d; g.K = N; g.b_div = 1; g.beta = 0; g.causal_k = 0;
    g.tri = 0; g.mt = mt; g.nt = nt_d; g.n_tiles = n_out_tiles; g.n_slices = S;
    BDH_HIP_CHECK(ctx, (launch_gemm<false, EPI_ACC>(ctx->stream, g)));
    BDH_LAUNCH_CHECK(ctx, "k_gemm<Q rho0>");
  }
  // 3b. out (+)= scores V
  {
    GemmArgs g{};
    g.A = Sc; g.B = Vt; g.C = out;
    g.a_batch = (long)T * Tp; g.b_batch = (long)d * Tp; g.c_batch = (long)T * d;
    g.lda = Tp; g.ldb = Tp; g.ldc = d;
    g.M = T; g.N = d; g.K = T; g.b_div = h; g.beta = state_is_zero ? 0 : 1; g.causal_k = 1;
    g.tri = 0; g.mt = mt; g.nt = nt_d; g.n_tiles = n_out_tiles; g.n_slices = S;
    BDH_HIP_CHECK(ctx, (launch_gemm<false, EPI_ACC>(ctx->stream, g)));
    BDH_LAUNCH_CHECK(ctx, "k_gemm<S V>");
  }
  // 4. rho (+)= Q^T V   (A = Q read k-major)
  {
    GemmArgs g{};
    g.A = Q; g.B = Vt; g.C = rho;
    g.a_batch = (long)T * N; g.b_batch = (long)d * Tp; g.c_batch = (long)N * d;
    g.lda = N; g.ldb = Tp; g.ldc = d;
    g.M = N; g.N = d; g.K = T; g.b_div = h; g.beta = state_is_zero ? 0 : 1; g.causal_k = 0;
    g.tri = 0; g.mt = nt_rho; g.nt = nt_d; g.n_tiles = n_rho_tiles; g.n_slices = S;
    BDH_HIP_CHECK(ctx, (launch_gemm<true, EPI_ACC>(ctx->stream, g)));
    BDH_LAUNCH_CHECK(ctx, "k_gemm<Q^T V>");
  }
  return BDH_OK;
}
