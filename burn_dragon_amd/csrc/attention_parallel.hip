// Parallel (all tokens at once) normalised causal linear attention in f32:
// kernel::linear_attention::fused_state_aligned (src/kernel/linear_attention.rs:11-115) and, with
// the dense block pattern, Attention::forward (src/model/attention.rs:142-175).
//
// This is the reference's training-path form; it is kept in f32 and follows the reference's
// block semantics exactly (including the ALiBi term being added to every entry of an active
// block).  Small problems take a row-per-workgroup kernel; from T = 128 on the two products run
// on the f32 matrix cores (v_mfma_f32_32x32x2_f32): S = mask(Q Q^T) + bias is materialised per
// slice, a row pass sums |S|, and out = (S V) / (norm + eps).  The bf16 form for inference is in
// prefill.hip.
#include <algorithm>
#include <cstring>
#include <vector>

#include "bdh_internal.h"

namespace {

struct FsaSlopes {
  float v[64];
};


constexpr float kTwoPi = 6.28318530717958647692f;
constexpr float kRowNormEps = 1e-6f;  // src/kernel/linear_attention.rs:9

// q_rot [S,T,Nq] from query [S,T,N], positions 0..T (src/kernel/linear_attention.rs:23-40)
__global__ __launch_bounds__(256) void k_rotate_f32(const float *__restrict__ x, const float *__restrict__ freqs,
                                                    float *__restrict__ q, int T, int N, int rotary) {
  const long row = blockIdx.x;  // slice * T + t
  const int t = (int)(row % T);
  const float pos = (float)t;
  const float *xr = x + row * N;
  const int Nq = rotary == BDH_POPE ? 2 * N : N;
  float *qr = q + row * Nq;
  for (int n = threadIdx.x; n < N; n += 256) {
    if (rotary == BDH_ALIBI) {
      qr[n] = xr[n];
      continue;
    }
    const float raw = pos * freqs[n];
    const float ph = (raw - floorf(raw)) * kTwoPi;
    float s, c;
    sincosf(ph, &s, &c);
    if (rotary == BDH_ROPE) {
      const float rot = (n & 1) ? xr[n - 1] : -xr[n + 1];
      const float a = xr[n] * c, r = rot * s;
      qr[n] = a + r;
    } else {
      const float m = logf(expf(xr[n] * 1.0f) + 1.0f) / 1.0f;  // softplus(x, 1)
      qr[n] = m * c;
      qr[N + n] = m * s;
    }
  }
}

// q [S,Tc,Nq] from rows t0..t0+Tc of x [S][T][N] (x points at row t0 of slice 0), token t of the chunk at
// position pos0 + t, or pos_dev[b] + pos_add + t with per-sequence positions.  The arithmetic is that of
// the decode step kernels (src/model/attention.rs:305-330), so the rotated values are the same bits.
__global__ __launch_bounds__(256) void k_rotate_chunk_f32(const float *__restrict__ x, long x_slice_stride,
                                                          const float *__restrict__ freqs, float *__restrict__ q,
                                                          int Tc, int N, int rotary, long pos0,
                                                          const int32_t *__restrict__ pos_dev, int pos_add, int h) {
  const long row = blockIdx.x;  // slice * Tc + t
  const long slice = row / Tc;
  const int t = (int)(row - slice * Tc);
  const float pos = (float)((pos_dev ? (long)pos_dev[slice / h] + pos_add : pos0) + t);
  const float *xr = x + slice * x_slice_stride + (long)t * N;
  const int Nq = rotary == BDH_POPE ? 2 * N : N;
  float *qr = q + row * Nq;
  if (rotary == BDH_ROPE) {  // N is even: one lane per pair
    for (int pr = threadIdx.x; pr < (N >> 1); pr += 256) {
      const float2 xv = reinterpret_cast<const float2 *>(xr)[pr];
      float2 o = make_float2(0.0f, 0.0f);
      if (xv.x != 0.0f || xv.y != 0.0f) {
        const float2 fv = reinterpret_cast<const float2 *>(freqs)[pr];
        const float raw0 = pos * fv.x, raw1 = pos * fv.y;
        float s0, c0, s1, c1;
        sincosf((raw0 - floorf(raw0)) * kTwoPi, &s0, &c0);
        sincosf((raw1 - floorf(raw1)) * kTwoPi, &s1, &c1);
        const float a0 = xv.x * c0, r0 = (-xv.y) * s0;
        const float a1 = xv.y * c1, r1 = xv.x * s1;
        o.x = a0 + r0;
        o.y = a1 + r1;
      }
      reinterpret_cast<float2 *>(qr)[pr] = o;
    }
    return;
  }
  for (int n = threadIdx.x; n < N; n += 256) {
    const float raw = pos * freqs[n];
    const float ph = (raw - floorf(raw)) * kTwoPi;
    float sn, cs;
    sincosf(ph, &sn, &cs);
    const float m = logf(expf(xr[n] * 1.0f) + 1.0f) / 1.0f;  // softplus(x, 1)
    qr[n] = m * cs;
    qr[N + n] = m * sn;
  }
}

// stamps[b,h,n] = clock (or clocks_dev[b] + add), saturated to the stamp range
__global__ __launch_bounds__(256) void k_set_stamps(int32_t *__restrict__ stamps, long rows, long rows_per_seq,
                                                    long clock, const int32_t *__restrict__ clocks_dev, int add) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= rows) return;
  const long c = clocks_dev ? (long)clocks_dev[i / rows_per_seq] + add : clock;
  stamps[i] = (int32_t)min(c, 0x7fffffffL);
}

// bf16 <-> f32 copies of a whole state (grid-stride); f32 -> bf16 rounds to nearest even
__global__ __launch_bounds__(256) void k_widen_bf16(const unsigned short *__restrict__ in, float *__restrict__ out,
                                                    size_t n) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256)
    out[i] = __uint_as_float(static_cast<unsigned int>(in[i]) << 16);
}
__global__ __launch_bounds__(256) void k_narrow_bf16(const float *__restrict__ in, unsigned short *__restrict__ out,
                                                     size_t n) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
    unsigned int u = __float_as_uint(in[i]);
    if ((u & 0x7fffffffu) > 0x7f800000u) {
      out[i] = static_cast<unsigned short>((u >> 16) | 0x40);
    } else {
      u += 0x7fffu + ((u >> 16) & 1u);
      out[i] = static_cast<unsigned short>(u >> 16);
    }
  }
}

// one workgroup per (slice, query row i)
__global__ __launch_bounds__(256) void k_fsa_row(const float *__restrict__ q, const float *__restrict__ v,
                                                 FsaSlopes slopes_dev, int use_alibi, int h,
                                                 int T, int Nq, int dv, int block_size,
                                                 const unsigned char *__restrict__ active,  // [tb*tb] or null
                                                 int tb, int row_normalize, float *__restrict__ out) {
  extern __shared__ float s_mem[];
  float *s_q = s_mem;          // [Nq]
  float *s_sc = s_mem + Nq;    // [T]
  __shared__ float s_part[4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const long slice = blockIdx.x / T;
  const int i = (int)(blockIdx.x - slice * T);
  const int hh = (int)(slice % h);
  const long b = slice / h;
  const float *Q = q + slice * (long)T * Nq;
  const float *V = v + b * (long)T * dv;
  const int rb = i / block_size;
  const float slope = use_alibi ? slopes_dev.v[hh] : 0.0f;
  for (int n = tid; n < Nq; n += 256) s_q[n] = Q[(long)i * Nq + n];
  __syncthreads();
  bool any = false;
  float nsum = 0.0f;
  for (int j = wave; j < T; j += 4) {
    const int cb = j / block_size;
    const bool act = active ? (active[(long)rb * tb + cb] != 0) : (cb <= rb);
    float s = 0.0f;
    if (act) {
      any = true;
      if (!(rb == cb && j >= i)) {  // tril(-1) on diagonal blocks
        const float *qj = Q + (long)j * Nq;
        float part = 0.0f;
        for (int n = lane; n < Nq; n += 64) part = __builtin_fmaf(s_q[n], qj[n], part);
        for (int o = 32; o > 0; o >>= 1) part += __shfl_xor(part, o);
        s = part;
      }
      if (use_alibi) {
        const float al = slope * ((float)j - (float)i);
        s = s + al;
      }
      nsum += fabsf(s);
    }
    if (lane == 0) s_sc[j] = s;
  }
  // any / norm across waves (each wave saw a different subset of j; lanes of a wave agree)
  if (lane == 0) s_part[wave] = nsum;
  const int any_all = __syncthreads_or(any ? 1 : 0);
  const float norm = s_part[0] + s_part[1] + s_part[2] + s_part[3];
  const float den = norm + kRowNormEps;
  float *o = out + (slice * (long)T + i) * dv;
  for (int c = tid; c < dv; c += 256) {
    float acc = 0.0f;
    for (int j = 0; j < T; ++j) {
      const float s = s_sc[j];
      if (s != 0.0f) acc = __builtin_fmaf(s, V[(long)j * dv + c], acc);
    }
    o[c] = (any_all && row_normalize) ? acc / den : acc;
  }
}

// ------------------------------------------------------------------------------------
// f32 matrix-core path
// ------------------------------------------------------------------------------------
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// Eight floats as three bf16x8 operands h + m + l that add up to the floats exactly: each term is the remainder so far
// rounded to bf16 (v_cvt_pk_bf16_f32, round to nearest even); a remainder is a difference of neighbours and therefore
// exact, and the third one has at most eight significant bits.  A product of two such sums is taken as the six matrix
// instructions l h, h l, m m, m h, h m, h h (smallest terms first); what is left out (m l, l m, l l) is below 2^-23 of
// |a b|, the size of one f32 rounding.  An infinite input, or a finite one that rounds to an infinite bf16 (above
// 3.389e38), gives NaN (inf - inf in the remainder).
__device__ __forceinline__ void fsa_split3(const float (&a)[8], bf16x8 &h, bf16x8 &m, bf16x8 &l) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  u32x4 ph, pm, pl;
#pragma unroll
  for (int q = 0; q < 4; ++q) {  // element 2q in the low half of a dword, 2q + 1 in the high half
    const f32x2 a2 = {a[2 * q], a[2 * q + 1]};
    ph[q] = __builtin_bit_cast(unsigned int, __builtin_convertvector(a2, bf16x2));
    const f32x2 r1 = {a2[0] - __uint_as_float(ph[q] << 16), a2[1] - __uint_as_float(ph[q] & 0xffff0000u)};
    pm[q] = __builtin_bit_cast(unsigned int, __builtin_convertvector(r1, bf16x2));
    const f32x2 r2 = {r1[0] - __uint_as_float(pm[q] << 16), r1[1] - __uint_as_float(pm[q] & 0xffff0000u)};
    pl[q] = __builtin_bit_cast(unsigned int, __builtin_convertvector(r2, bf16x2));
  }
  h = __builtin_bit_cast(bf16x8, ph);
  m = __builtin_bit_cast(bf16x8, pm);
  l = __builtin_bit_cast(bf16x8, pl);
}
constexpr int FK = 16;    // k per LDS stage
constexpr int FLD = 20;   // LDS row stride in floats (80 bytes: 16-byte aligned, spreads the banks)

struct FsaArgs {
  const float *A;   // A_KMAJOR ? [slices][K][lda] (m contiguous) : [slices][M][lda] (k contiguous)
  const float *Bm;  // B_KMAJOR ? [b][K][ldb] (n contiguous) : [slices][N][ldb] (k contiguous)
  float *C;         // [slices][M][ldc]
  long a_batch, b_batch, c_batch;
  int lda, ldb, ldc, M, N, K;
  int b_div;        // B slice = slice / b_div
  int n_slices;
  int mt, nt;       // tile grid (rows, columns) of one slice
  // scores epilogue
  int block_size, tb, h, use_alibi, dense;
  const unsigned char *active;  // [tb*tb] when !dense
  float slopes[64];             // per head, by value (no device copy, no host synchronisation)
  // output epilogue
  const float *norm;            // [slices][M] or null
  int beta;                     // EPI 2: C += acc instead of C = acc
  // mod > 0: slice = s1 * mod + s2 and operand X starts at s1 * x_batch + s2 * x_mod_stride
  int mod;
  long a_mod_stride, b_mod_stride, c_mod_stride;
  // ALiBi state decay (src/model/bdh.rs:299-301) in the many-token form, g = exp(log_decay[slice % h]):
  //   FSA_DECAY_SCORES  EPI 0: S[t,s] *= g^(t-s)
  //   FSA_DECAY_ROWS    EPI 2: acc[t,:] *= g^t
  //   FSA_DECAY_STATE   EPI 2, A k-major: A[k,:] *= g^(K-k) on load and C = g^K * C + acc
  int decay_mode;
  float log_decay[64];
  // EPI 3, relu_lowrank (src/kernel/relu_lowrank.rs:7-37): C = gate * mask * relu(acc + bias - thr), head = slice % mod
  const float *rl_bias;            // [h][N] or null
  float rl_thr;
  const unsigned char *rl_mask;    // one byte per latent block (device) or null
  int rl_block, rl_nblocks;
  const float *rl_gate;            // laid out like C, or null
};
constexpr int FSA_DECAY_SCORES = 1, FSA_DECAY_ROWS = 2, FSA_DECAY_STATE = 4;

__device__ __forceinline__ float4 fsa_ld4(const float *p, int n_valid, bool vec_ok) {
  if (n_valid >= 4 && vec_ok) return *reinterpret_cast<const float4 *>(p);
  float4 r = make_float4(0.f, 0.f, 0.f, 0.f);
  if (n_valid > 0) r.x = p[0];
  if (n_valid > 1) r.y = p[1];
  if (n_valid > 2) r.z = p[2];
  if (n_valid > 3) r.w = p[3];
  return r;
}

// EPI 0: scores (mask, ALiBi term, zero outside the pattern); EPI 1: out = acc / (norm + eps);
// EPI 2: C = acc or C += acc; EPI 3: the relu_lowrank epilogue.
// SEQK: the eight matrix instructions of a 16-wide k stage take k = 0,1 | 2,3 | ... instead of 0,8 | 1,9 | ...; an
// instruction adds its two k-steps one after the other as fused multiply-adds, so every output is then ONE
// k-sequential fmaf chain -- the same bits as a scalar loop over k (A rows k-contiguous, B k-major only).
// A k-major operand (its reduction index is the slow one in memory) is staged as it lies, [k][m] with a
// row stride of tile + 4 floats: float4 stores, and fragment reads of one float per lane in which the
// 32 lanes of a half-wave take consecutive addresses and the two halves (k and k + 8) fall on the two
// halves of the 64 banks.
// SPLIT3: the products run on the bf16 matrix instructions (16 times the f32 rate) with every f32 operand split into
// three bf16 terms in registers, six instructions per f32 one: f32-level accuracy (the result differs from the f32
// instruction's by about one rounding of a product), not the bits of any particular summation order.  The fragment a
// lane holds for eight f32 steps (k = half*8 .. +7 of its row) is the fragment of one 32 x 32 x 16 instruction.
// Tile BM x BN, NWM x NWN waves, each wave (BM/NWM) x (BN/NWN).  The 128 x 128 tile needs 8 bytes per
// clock and workgroup from the L2, which three resident workgroups per CU do not get; the
// 256 x 256 tile halves that per FLOP and is the one that keeps the matrix cores busy.
template <int EPI, bool A_KMAJOR, bool B_KMAJOR, int BM, int BN, int NWM, int NWN, bool SEQK = false, bool SPLIT3 = false>
__global__ __launch_bounds__(NWM * NWN * 64) void k_fsa_gemm_f32(FsaArgs g) {
  static_assert(!(SEQK && SPLIT3), "the split product does not keep the bits of a scalar loop");
  static_assert(!SEQK || (!A_KMAJOR && B_KMAJOR), "sequential k order is built for row-major A and k-major B");
  constexpr int NT = NWM * NWN * 64;
  constexpr int KLA = BM + 4, KLB = BN + 4;  // row strides of the k-major LDS layouts
  static_assert(FK * KLA <= BM * FLD && FK * KLB <= BN * FLD, "k-major tile must fit");
  constexpr int MI = BM / NWM / 32, NJ = BN / NWN / 32;
  constexpr int CA = BM * 4 / NT, CB = BN * 4 / NT;  // float4 chunks per thread and stage
  static_assert(CA >= 1 && CB >= 1 && CA * NT == BM * 4 && CB * NT == BN * 4, "tile does not divide over the threads");
  __shared__ __attribute__((aligned(16))) float s_a[BM * FLD];
  __shared__ __attribute__((aligned(16))) float s_b[BN * FLD];
  // XCD-aware mapping: workgroup ids are dealt round-robin to the 8 XCDs, so ids with the same
  // (id % 8) share an L2; all tiles of one slice go to one XCD and reuse its operand rows there.
  const int xcd = blockIdx.x & 7;
  const int rr = blockIdx.x >> 3;
  const int tiles = g.mt * g.nt;
  const int slice = xcd + 8 * (rr / tiles);
  if (slice >= g.n_slices) return;
  const int tile = rr % tiles;
  const int m0 = (tile / g.nt) * BM, n0 = (tile % g.nt) * BN;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / NWN, wn = wave % NWN;
  const float *A = g.A + (long)slice * g.a_batch;
  const float *Bm = g.Bm + (long)(slice / g.b_div) * g.b_batch;
  float *C = g.C + (long)slice * g.c_batch;
  if (g.mod > 0) {
    const long s1 = slice / g.mod, s2 = slice % g.mod;
    A = g.A + s1 * g.a_batch + s2 * g.a_mod_stride;
    Bm = g.Bm + s1 * g.b_batch + s2 * g.b_mod_stride;
    C = g.C + s1 * g.c_batch + s2 * g.c_mod_stride;
  }
  const int bs = g.block_size;

  int K = g.K;
  bool tile_active = true;
  if (EPI == 0) {
    // dense pattern: block (rb, cb) is active iff cb <= rb; a tile all of whose blocks lie above
    // the diagonal only writes zeros
    if (g.dense && n0 / bs > (min(m0 + BM, g.M) - 1) / bs) tile_active = false;
  } else if (g.dense) {
    K = min(K, ((min(m0 + BM, g.M) - 1) / bs + 1) * bs);  // S is zero beyond the row tile's last block
  }
  if (K <= 0) tile_active = false;
  const float ld = g.decay_mode ? g.log_decay[slice % g.h] : 0.0f;

  f32x16 acc[MI][NJ];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  if (tile_active) {
    const bool a_vec = (g.lda % 4 == 0) && (reinterpret_cast<uintptr_t>(A) % 16 == 0);
    const bool b_vec = (g.ldb % 4 == 0) && (reinterpret_cast<uintptr_t>(Bm) % 16 == 0);
    float4 ra[1][CA], rb[1][CB];
    // a tile that lies inside both operands, 16-byte aligned: its loads need no checks, and loads that sit
    // under no branch are issued back to back
    const bool tile_full = a_vec && b_vec && m0 + BM <= g.M && n0 + BN <= g.N;
    auto load = [&](float4 *pa, float4 *pb, int k0) {
      if (tile_full && k0 + FK <= K) {
#pragma unroll
        for (int c = 0; c < CA; ++c) {
          const int chunk = c * NT + tid;
          if (!A_KMAJOR) {
            const int row = chunk >> 2, kc = (chunk & 3) * 4;
            pa[c] = *reinterpret_cast<const float4 *>(A + (long)(m0 + row) * g.lda + k0 + kc);
          } else {
            const int kr = chunk / (BM / 4), mc = (chunk % (BM / 4)) * 4;
            pa[c] = *reinterpret_cast<const float4 *>(A + (long)(k0 + kr) * g.lda + m0 + mc);
          }
        }
#pragma unroll
        for (int c = 0; c < CB; ++c) {
          const int chunk = c * NT + tid;
          if (!B_KMAJOR) {
            const int row = chunk >> 2, kc = (chunk & 3) * 4;
            pb[c] = *reinterpret_cast<const float4 *>(Bm + (long)(n0 + row) * g.ldb + k0 + kc);
          } else {
            const int kr = chunk / (BN / 4), nc = (chunk % (BN / 4)) * 4;
            pb[c] = *reinterpret_cast<const float4 *>(Bm + (long)(k0 + kr) * g.ldb + n0 + nc);
          }
        }
        if (A_KMAJOR && EPI == 2 && (g.decay_mode & FSA_DECAY_STATE)) {
#pragma unroll
          for (int c = 0; c < CA; ++c) {
            const int kr = (c * NT + tid) / (BM / 4);
            const float f = expf((float)(K - (k0 + kr)) * ld);
            pa[c].x *= f; pa[c].y *= f; pa[c].z *= f; pa[c].w *= f;
          }
        }
        return;
      }
#pragma unroll
      for (int c = 0; c < CA; ++c) {
        const int chunk = c * NT + tid;
        if (!A_KMAJOR) {
          const int row = chunk >> 2, kc = (chunk & 3) * 4;
          pa[c] = (m0 + row < g.M && k0 < K) ? fsa_ld4(A + (long)(m0 + row) * g.lda + k0 + kc, K - (k0 + kc), a_vec)
                                             : make_float4(0.f, 0.f, 0.f, 0.f);
        } else {
          const int kr = chunk / (BM / 4), mc = (chunk % (BM / 4)) * 4;  // BM/4 chunks of 4 rows per k row
          pa[c] = (k0 + kr < K) ? fsa_ld4(A + (long)(k0 + kr) * g.lda + m0 + mc, g.M - (m0 + mc), a_vec)
                                : make_float4(0.f, 0.f, 0.f, 0.f);
          if (EPI == 2 && (g.decay_mode & FSA_DECAY_STATE)) {  // token k of K is decayed K - k times by the end
            const float f = expf((float)(K - (k0 + kr)) * ld);
            pa[c].x *= f; pa[c].y *= f; pa[c].z *= f; pa[c].w *= f;
          }
        }
      }
#pragma unroll
      for (int c = 0; c < CB; ++c) {
        const int chunk = c * NT + tid;
        if (!B_KMAJOR) {
          const int row = chunk >> 2, kc = (chunk & 3) * 4;
          pb[c] = (n0 + row < g.N && k0 < K) ? fsa_ld4(Bm + (long)(n0 + row) * g.ldb + k0 + kc, K - (k0 + kc), b_vec)
                                             : make_float4(0.f, 0.f, 0.f, 0.f);
        } else {
          const int kr = chunk / (BN / 4), nc = (chunk % (BN / 4)) * 4;  // BN/4 chunks of 4 columns per k row
          pb[c] = (k0 + kr < K) ? fsa_ld4(Bm + (long)(k0 + kr) * g.ldb + n0 + nc, g.N - (n0 + nc), b_vec)
                                : make_float4(0.f, 0.f, 0.f, 0.f);
        }
      }
    };
    auto store = [&](const float4 *pa, const float4 *pb) {
#pragma unroll
      for (int c = 0; c < CA; ++c) {
        const int chunk = c * NT + tid;
        if (!A_KMAJOR) {
          const int row = chunk >> 2, kc = (chunk & 3) * 4;
          if (SEQK) {  // k = kc, kc + 2 to places kc / 2, kc / 2 + 1; k = kc + 1, kc + 3 to places 8 + kc / 2, ...
            *reinterpret_cast<float2 *>(s_a + row * FLD + (kc >> 1)) = make_float2(pa[c].x, pa[c].z);
            *reinterpret_cast<float2 *>(s_a + row * FLD + 8 + (kc >> 1)) = make_float2(pa[c].y, pa[c].w);
          } else {
            *reinterpret_cast<float4 *>(s_a + row * FLD + kc) = pa[c];
          }
        } else {
          const int kr = chunk / (BM / 4), mc = (chunk % (BM / 4)) * 4;
          *reinterpret_cast<float4 *>(s_a + kr * KLA + mc) = pa[c];
        }
      }
#pragma unroll
      for (int c = 0; c < CB; ++c) {
        const int chunk = c * NT + tid;
        if (!B_KMAJOR) {
          const int row = chunk >> 2, kc = (chunk & 3) * 4;
          *reinterpret_cast<float4 *>(s_b + row * FLD + kc) = pb[c];
        } else {
          const int kr = chunk / (BN / 4), nc = (chunk % (BN / 4)) * 4;
          *reinterpret_cast<float4 *>(s_b + kr * KLB + nc) = pb[c];
        }
      }
    };
    auto multiply = [&]() {
      // lane (r = lane % 32, half = lane / 32) feeds k = half*8 + q to the q-th of eight 32x32x2 steps
      const int r = lane & 31, kb = (lane >> 5) * 8;
      float fa[MI][8], fb[NJ][8];
#pragma unroll
      for (int i = 0; i < MI; ++i) {
        if (A_KMAJOR) {
          const float *p = s_a + kb * KLA + wm * (BM / NWM) + i * 32 + r;
#pragma unroll
          for (int q = 0; q < 8; ++q) fa[i][q] = p[q * KLA];
          continue;
        }
        // (SEQK: the stage was stored with its even k in the first eight places of a row and its odd k in the
        // last eight, so the same two reads give this half-wave k = 2 q + half)
        const float *p = s_a + (wm * (BM / NWM) + i * 32 + r) * FLD + kb;
        const float4 lo = *reinterpret_cast<const float4 *>(p), hi = *reinterpret_cast<const float4 *>(p + 4);
        fa[i][0] = lo.x; fa[i][1] = lo.y; fa[i][2] = lo.z; fa[i][3] = lo.w;
        fa[i][4] = hi.x; fa[i][5] = hi.y; fa[i][6] = hi.z; fa[i][7] = hi.w;
      }
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        if (B_KMAJOR) {
          const float *p = s_b + (SEQK ? (lane >> 5) : kb) * KLB + wn * (BN / NWN) + j * 32 + r;
#pragma unroll
          for (int q = 0; q < 8; ++q) fb[j][q] = p[(SEQK ? 2 * q : q) * KLB];
          continue;
        }
        const float *p = s_b + (wn * (BN / NWN) + j * 32 + r) * FLD + kb;
        const float4 lo = *reinterpret_cast<const float4 *>(p), hi = *reinterpret_cast<const float4 *>(p + 4);
        fb[j][0] = lo.x; fb[j][1] = lo.y; fb[j][2] = lo.z; fb[j][3] = lo.w;
        fb[j][4] = hi.x; fb[j][5] = hi.y; fb[j][6] = hi.z; fb[j][7] = hi.w;
      }
      if (SPLIT3) {
        bf16x8 ah[MI], am[MI], al[MI], bh[NJ], bm[NJ], bl[NJ];
#pragma unroll
        for (int i = 0; i < MI; ++i) fsa_split3(fa[i], ah[i], am[i], al[i]);
#pragma unroll
        for (int j = 0; j < NJ; ++j) fsa_split3(fb[j], bh[j], bm[j], bl[j]);
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
          for (int j = 0; j < NJ; ++j) {
            f32x16 c = acc[i][j];
            c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(al[i], bh[j], c, 0, 0, 0);
            c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah[i], bl[j], c, 0, 0, 0);
            c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(am[i], bm[j], c, 0, 0, 0);
            c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(am[i], bh[j], c, 0, 0, 0);
            c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah[i], bm[j], c, 0, 0, 0);
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ah[i], bh[j], c, 0, 0, 0);
          }
        return;
      }
#pragma unroll
      for (int q = 0; q < 8; ++q)
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
          for (int j = 0; j < NJ; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i][q], fb[j][q], acc[i][j], 0, 0, 0);
    };
    // one register stage: a second one (loads two k-steps ahead) measured no faster
    load(ra[0], rb[0], 0);
    for (int k0 = 0; k0 < K; k0 += FK) {
      __syncthreads();  // the previous step's fragment reads are done
      store(ra[0], rb[0]);
      __syncthreads();
      load(ra[0], rb[0], k0 + FK);  // an out-of-range stage loads nothing
      multiply();
    }
  }

  // accumulator element e of lane l in a 32x32 tile: row = (e/4)*8 + (l/32)*4 + (e%4), col = l%32
  const float slope = (EPI == 0 && g.use_alibi) ? g.slopes[slice % g.h] : 0.0f;
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int col = n0 + wn * (BN / NWN) + j * 32 + (lane & 31);
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int row = m0 + wm * (BM / NWM) + i * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
        if (row >= g.M) continue;
        if (EPI == 0) {
          if (col >= g.ldc) continue;
          float v = 0.0f;
          if (col < g.N) {
            const int rbk = row / bs, cbk = col / bs;
            const bool act = g.dense ? (cbk <= rbk) : (g.active[(long)rbk * g.tb + cbk] != 0);
            if (act) {
              v = (rbk == cbk && col >= row) ? 0.0f : acc[i][j][e];  // tril(-1) on diagonal blocks (:88-90)
              if ((g.decay_mode & FSA_DECAY_SCORES) && col < row) v = v * expf((float)(row - col) * ld);
              if (g.use_alibi) {  // added to every entry of an active block (:97-100)
                const float al = slope * ((float)col - (float)row);
                v = v + al;
              }
            }
          }
          C[(long)row * g.ldc + col] = v;
        } else if (EPI == 1) {
          if (col >= g.N) continue;
          float v = acc[i][j][e];
          if (g.norm) v = v / (g.norm[(long)slice * g.M + row] + kRowNormEps);
          C[(long)row * g.ldc + col] = v;
        } else if (EPI == 3) {
          if (col >= g.N) continue;
          const int hh = g.mod > 0 ? slice % g.mod : 0;
          float pv = acc[i][j][e];
          if (g.rl_bias) pv = pv + g.rl_bias[(long)hh * g.N + col];
          if (g.rl_thr != 0.0f) pv = pv - g.rl_thr;
          float y = pv > 0.0f ? pv : 0.0f;
          if (g.rl_mask) {
            const int blk = col / g.rl_block;
            y = y * ((blk < g.rl_nblocks && g.rl_mask[blk]) ? 1.0f : 0.0f);
          }
          const long o = (long)row * g.ldc + col;
          // the gate and the output are touched once per call: streaming accesses leave the L2 to the operand tiles
          // ([8192 x 512] x [512 x 131072]: 9.98 -> 9.69 ms)
          if (g.rl_gate) y = __builtin_nontemporal_load(g.rl_gate + (C - g.C) + o) * y;
          __builtin_nontemporal_store(y, C + o);
        } else {
          if (col >= g.N) continue;
          float *p = C + (long)row * g.ldc + col;
          float v = acc[i][j][e];
          if (g.decay_mode & FSA_DECAY_ROWS) v = v * expf((float)row * ld);
          if (g.decay_mode & FSA_DECAY_STATE)
            *p = *p * expf((float)g.K * ld) + v;
          else if (g.beta)
            // C += acc as one no-return add per element, done by the L2: the wavefront does not wait for C to arrive,
            // so a short-K tile's epilogue overlaps the next workgroup's products (rho += Q^T V at B=32, h=8,
            // N=16384, d=512, K=256: 12.1 -> 10.1 ms).  One add per element and call: the same rounding as
            // *p + v and no race; the L2's adder flushes results below the smallest normal float to zero.
            unsafeAtomicAdd(p, v);
          else
            *p = v;
        }
      }
    }
}

// norm[row] = sum_s |S[row, s]|: one wave per row
__global__ __launch_bounds__(256) void k_fsa_row_abs_sum(const float *__restrict__ S, long rows, int T, int ld,
                                                         float *__restrict__ norm) {
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int lane = threadIdx.x & 63;
  const float *p = S + row * ld;
  float a = 0.0f;
  for (int c = lane; c < T; c += 64) a += fabsf(p[c]);
  for (int o = 32; o > 0; o >>= 1) a += __shfl_xor(a, o);
  if (lane == 0) norm[row] = a;
}

}  // namespace

extern "C" int bdh_fused_state_aligned(bdh_ctx *ctx, int B, int h, int T, int N, int dv, const float *query,
                                       const float *value, const float *freqs, const float *alibi_slopes_host,
                                       int block_size, const int32_t *block_pairs_host, int n_pairs, int rotary,
                                       int row_normalize, float *out) {
  if (!ctx) return BDH_E_INVAL;
  if (B < 0 || h < 0 || T < 0 || N < 0 || dv < 0) return bdh_fail(ctx, BDH_E_INVAL, "negative dimension");
  if (rotary != BDH_ROPE && rotary != BDH_ALIBI && rotary != BDH_POPE)
    return bdh_fail(ctx, BDH_E_INVAL, "rotary %d is not a bdh_rotary value", rotary);
  if (rotary == BDH_ROPE && (N & 1)) return bdh_fail(ctx, BDH_E_SHAPE, "RoPE needs an even latent size, got N=%d", N);
  if (h > 64) return bdh_fail(ctx, BDH_E_SHAPE, "n_head %d > 64", h);
  if (n_pairs < 0 || (n_pairs > 0 && !block_pairs_host)) return bdh_fail(ctx, BDH_E_INVAL, "bad block pair list");
  if (B == 0 || h == 0 || T == 0 || dv == 0) return BDH_OK;
  if (!query || !value || !out || (rotary != BDH_ALIBI && !freqs)) return bdh_fail(ctx, BDH_E_INVAL, "null data pointer");
  if (block_size < 1) block_size = 1;  // usize::max(layout.block_size(), 1), linear_attention.rs:46
  const int Nq = rotary == BDH_POPE ? 2 * N : N;
  const long S = (long)B * h;
  const int tb = (T + block_size - 1) / block_size;
  const bool sparse = block_pairs_host != nullptr;
  if (sparse && tb > 4096) return bdh_fail(ctx, BDH_E_SHAPE, "sparse time pattern with %d blocks", tb);
  // opt-in: the dense layout, row-normalised, on the bf16 matrix cores (inputs and scores rounded to bf16: 2e-2)
  if (ctx->opt_fsa_path == 2 && !sparse && row_normalize && (N & 7) == 0 && bdh_aligned(query, 16) && bdh_aligned(out, 16))
    return bdh_launch_fsa_bf16(ctx, B, h, T, N, dv, query, value, freqs, alibi_slopes_host, block_size, rotary, out);
  const size_t lds = sizeof(float) * ((size_t)Nq + T);
  int path = ctx->opt_fsa_path == 2 ? -1 : ctx->opt_fsa_path;  // -1 choose, 0 row kernel, 1 matrix cores
  if (path < 0) path = T >= 128 ? 1 : 0;
  if (path == 0 && lds > 150 * 1024) path = 1;
  if (S * T > 0x7fffffffL || (S + 7) / 8 * 8 * (long)(((T + 127) / 128) * ((T + 127) / 128)) > 0x7fffffffL) return bdh_fail(ctx, BDH_E_SHAPE, "B*h*T too large");

  const int Tp = (T + 3) & ~3;  // row stride of the score matrix
  const size_t q_bytes = bdh_align_up(sizeof(float) * (size_t)S * T * Nq, 256);
  const size_t act_bytes = sparse ? bdh_align_up((size_t)tb * tb, 256) : 0;
  const size_t sc_bytes = path == 1 ? bdh_align_up(sizeof(float) * (size_t)S * T * Tp, 256) : 0;
  const size_t nm_bytes = path == 1 ? bdh_align_up(sizeof(float) * (size_t)S * T, 256) : 0;
  int rc = bdh_ws_reserve(ctx, q_bytes + sc_bytes + nm_bytes);
  if (rc != BDH_OK) return rc;
  char *ws = static_cast<char *>(ctx->ws);
  float *q = reinterpret_cast<float *>(ws);
  float *scores = reinterpret_cast<float *>(ws + q_bytes);
  float *norm = reinterpret_cast<float *>(ws + q_bytes + sc_bytes);
  // The time-block mask of a sparse pattern lives in memory the context owns and is uploaded only when the
  // pattern differs from the one already there (a model calls with the same pattern every time): no copy and
  // no host synchronisation on the usual call.  The ALiBi slopes travel as a kernel argument.
  unsigned char *active = nullptr;
  if (sparse) {
    std::vector<int> key;
    key.reserve(2 * (size_t)n_pairs + 1);
    key.push_back(tb);
    key.insert(key.end(), block_pairs_host, block_pairs_host + 2 * (size_t)n_pairs);
    if (!ctx->fsa_mask || ctx->fsa_mask_key != key) {
      std::vector<unsigned char> m((size_t)tb * tb, 0);
      for (int p = 0; p < n_pairs; ++p) {
        const int r = block_pairs_host[2 * p], c = block_pairs_host[2 * p + 1];
        if (r >= 0 && r < tb && c >= 0 && c < tb) m[(size_t)r * tb + c] = 1;  // iter_cols drops c >= total_blocks
      }
      BDH_HIP_CHECK(ctx, hipStreamSynchronize(ctx->stream));  // earlier calls may still read the old mask
      if (ctx->fsa_mask_bytes < m.size()) {
        if (ctx->fsa_mask) BDH_HIP_CHECK(ctx, hipFree(ctx->fsa_mask));
        ctx->fsa_mask = nullptr;
        ctx->fsa_mask_bytes = 0;
        ctx->fsa_mask_key.clear();
        if (hipMalloc(&ctx->fsa_mask, m.size()) != hipSuccess) {
          (void)hipGetLastError();
          return bdh_fail(ctx, BDH_E_NOMEM, "time-block mask of %zu bytes", m.size());
        }
        ctx->fsa_mask_bytes = m.size();
      }
      BDH_HIP_CHECK(ctx, hipMemcpy(ctx->fsa_mask, m.data(), m.size(), hipMemcpyHostToDevice));
      ctx->fsa_mask_key = std::move(key);
    }
    active = static_cast<unsigned char *>(ctx->fsa_mask);
  }
  FsaSlopes slopes_dev{};
  if (alibi_slopes_host) memcpy(slopes_dev.v, alibi_slopes_host, sizeof(float) * h);
  hipLaunchKernelGGL(k_rotate_f32, dim3((unsigned)(S * T)), dim3(256), 0, ctx->stream, query, freqs, q, T, N, rotary);
  BDH_LAUNCH_CHECK(ctx, "k_rotate_f32");
  if (path == 1) {
    FsaArgs g{};
    g.A = q; g.Bm = q; g.C = scores;
    g.a_batch = g.b_batch = (long)T * Nq; g.c_batch = (long)T * Tp;
    g.lda = g.ldb = Nq; g.ldc = Tp; g.M = g.N = T; g.K = Nq; g.b_div = 1; g.n_slices = (int)S;
    g.block_size = block_size; g.tb = tb; g.h = h; g.use_alibi = alibi_slopes_host ? 1 : 0; g.dense = sparse ? 0 : 1;
    g.active = active; g.norm = nullptr;
    memcpy(g.slopes, slopes_dev.v, sizeof(g.slopes));
    // big tiles once there are enough of them to cover the chip; small ones for short sequences
    const bool big = (long)S * ((T + 255) / 256) * ((T + 255) / 256) >= 256;
    const unsigned groups = (unsigned)((S + 7) / 8);
    if (big) {
      g.mt = g.nt = (T + 255) / 256;
      hipLaunchKernelGGL((k_fsa_gemm_f32<0, false, false, 256, 256, 2, 4, false, true>), dim3(8 * groups * g.mt * g.nt), dim3(512), 0,
                         ctx->stream, g);
    } else {
      g.mt = g.nt = (T + 127) / 128;
      hipLaunchKernelGGL((k_fsa_gemm_f32<0, false, false, 128, 128, 2, 2, false, true>), dim3(8 * groups * g.mt * g.nt), dim3(256), 0,
                         ctx->stream, g);
    }
    BDH_LAUNCH_CHECK(ctx, "k_fsa_gemm_f32<scores>");
    if (row_normalize) {
      hipLaunchKernelGGL(k_fsa_row_abs_sum, dim3((unsigned)((S * T + 3) / 4)), dim3(256), 0, ctx->stream, scores,
                         S * T, T, Tp, norm);
      BDH_LAUNCH_CHECK(ctx, "k_fsa_row_abs_sum");
    }
    FsaArgs o{};
    o.A = scores; o.Bm = value; o.C = out;
    o.a_batch = (long)T * Tp; o.b_batch = (long)T * dv; o.c_batch = (long)T * dv;
    o.lda = Tp; o.ldb = dv; o.ldc = dv; o.M = T; o.N = dv; o.K = T; o.b_div = h; o.n_slices = (int)S;
    o.block_size = block_size; o.tb = tb; o.h = h; o.dense = sparse ? 0 : 1;
    o.norm = row_normalize ? norm : nullptr;
    o.mt = (T + 127) / 128;
    o.nt = (dv + 127) / 128;
    hipLaunchKernelGGL((k_fsa_gemm_f32<1, false, true, 128, 128, 2, 2, false, true>), dim3(8 * groups * o.mt * o.nt), dim3(256), 0,
                       ctx->stream, o);
    BDH_LAUNCH_CHECK(ctx, "k_fsa_gemm_f32<out>");
    return BDH_OK;
  }
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(k_fsa_row),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return bdh_fail(ctx, BDH_E_HIP, "dynamic LDS of %zu bytes refused: %s", lds, hipGetErrorString(e));
  }
  hipLaunchKernelGGL(k_fsa_row, dim3((unsigned)(S * T)), dim3(256), lds, ctx->stream, q, value, slopes_dev,
                     alibi_slopes_host ? 1 : 0, h, T, Nq, dv, block_size, active, tb, row_normalize, out);
  BDH_LAUNCH_CHECK(ctx, "k_fsa_row");
  return BDH_OK;
}

// ------------------------------------------------------------------------------------
// BDH::recurrent_attention (src/model/bdh.rs:258-307) over many tokens at once, f32, RoPE or PoPE:
// for a chunk of Tc tokens  out = tril(-1)(Q Q^T) V + Q rho,  rho += Q^T V  — the same sums as the
// token-by-token loop, reassociated, as four products on the f32 matrix cores.  The cost does not
// depend on how many neurons are active, which is what a prompt through a densely firing model needs
// (the sparse step kernels move every touched state row once per token).
// ------------------------------------------------------------------------------------
int bdh_launch_state_chunks_f32(bdh_ctx *ctx, const StateStepParams &p, float *out_ln) {
  const int B = p.B, h = p.h, T = p.T, N = p.N, d = p.d;
  const int Nq = p.rotary == BDH_POPE ? 2 * N : N;
  const long S = (long)B * h;
  const bool bf16_state = p.rho_dtype == BDH_BF16;
  const bool alibi = p.rotary == BDH_ALIBI;
  if (p.stamps && !alibi) return bdh_fail(ctx, BDH_E_INVAL, "decay stamps only apply to ALiBi");
  float log_decay[64] = {0};
  if (alibi)  // log of the ROUNDED per-token factor, as in the lazily decayed step (src/model/attention.rs:181-186)
    for (int i = 0; i < h; ++i) log_decay[i] = (float)log((double)expf(-p.slopes_host[i]));
  if (p.stamps) {  // a lazily decayed state: apply what is pending, the products below decay every row themselves
    int rc0 = bdh_launch_alibi_materialize(ctx, B, h, N, d, p.slopes_host, p.position, p.positions_dev, p.rho,
                                           p.rho_dtype, p.stamps);
    if (rc0 != BDH_OK) return rc0;
  }
  if (S > 0x7fffffffL / 4096) return bdh_fail(ctx, BDH_E_SHAPE, "B*h too large");
  // chunk length: a multiple of 128 between 128 and 512 whose rotated activations stay under 4 GiB
  const size_t per_token = sizeof(float) * (size_t)S * Nq;
  long Tc = (long)((size_t(4) << 30) / per_token) / 128 * 128;
  Tc = std::min<long>(512, std::max<long>(128, Tc));
  Tc = std::min<long>(Tc, T);
  const int Tcp = ((int)Tc + 3) & ~3;
  const size_t q_bytes = alibi ? 0 : bdh_align_up(per_token * (size_t)Tc, 256);  // ALiBi does not rotate: q = x
  const size_t sc_bytes = bdh_align_up(sizeof(float) * (size_t)S * Tc * Tcp, 256);
  // a bf16 state is widened to f32 for the call and rounded back once at its end (the token loop rounds
  // after every token)
  const size_t n_state = (size_t)S * Nq * d;
  const size_t wide_bytes = bf16_state ? bdh_align_up(sizeof(float) * n_state, 256) : 0;
  int rc = bdh_ws_reserve(ctx, q_bytes + sc_bytes + wide_bytes);
  if (rc != BDH_OK) return rc;
  float *q = static_cast<float *>(ctx->ws);
  float *scores = reinterpret_cast<float *>(static_cast<char *>(ctx->ws) + q_bytes);
  float *rho = static_cast<float *>(p.rho);
  if (bf16_state) {
    rho = reinterpret_cast<float *>(static_cast<char *>(ctx->ws) + q_bytes + sc_bytes);
    hipLaunchKernelGGL(k_widen_bf16, dim3((unsigned)std::min<size_t>((n_state + 255) / 256, 1u << 20)), dim3(256), 0,
                       ctx->stream, static_cast<const unsigned short *>(p.rho), rho, n_state);
    BDH_LAUNCH_CHECK(ctx, "k_widen_bf16");
  }
  const unsigned groups = (unsigned)((S + 7) / 8);
  const int nt_d = (d + 127) / 128;
  if ((long)groups * 8 * ((Nq + 127) / 128) * nt_d > 0x7fffffffL) return bdh_fail(ctx, BDH_E_SHAPE, "too many tiles");

  const int n_cu = ctx->n_cu > 0 ? ctx->n_cu : 256;
  for (int t0 = 0; t0 < T; t0 += (int)Tc) {
    const int tc = (int)std::min<long>(Tc, T - t0);
    // a small model or a short call: with 128 x 128 tiles the products would run on a few CUs, each a chain of
    // load latencies; 32 x 64 tiles give sixteen times the workgroups
    const bool small_tiles = (long)8 * groups * ((tc + 127) / 128) * nt_d < n_cu;
    const float *qc = q;           // this chunk's rotated activations [S][tc][Nq]
    long q_batch = (long)tc * Nq;
    if (alibi) {
      qc = p.x + (long)t0 * N;
      q_batch = (long)T * N;
    } else {
      hipLaunchKernelGGL(k_rotate_chunk_f32, dim3((unsigned)(S * tc)), dim3(256), 0, ctx->stream, p.x + (long)t0 * N,
                         (long)T * N, p.freqs, q, tc, N, p.rotary, (long)(p.position + t0), p.positions_dev, t0, h);
      BDH_LAUNCH_CHECK(ctx, "k_rotate_chunk_f32");
    }
    auto with_decay = [&](FsaArgs &g, int mode) {
      if (!alibi) return;
      g.decay_mode = mode;
      memcpy(g.log_decay, log_decay, sizeof(log_decay));
    };
    {  // S = tril(-1)(Q Q^T)   (ALiBi: S[t,s] *= decay^(t-s))
      FsaArgs g{};
      g.A = qc; g.Bm = qc; g.C = scores;
      g.a_batch = g.b_batch = q_batch; g.c_batch = (long)Tc * Tcp;
      g.lda = g.ldb = Nq; g.ldc = Tcp; g.M = g.N = tc; g.K = Nq; g.b_div = 1; g.n_slices = (int)S;
      g.block_size = 1; g.tb = tc; g.h = h; g.use_alibi = 0; g.dense = 1;
      with_decay(g, FSA_DECAY_SCORES);
      const bool big = S * ((tc + 255) / 256) * ((tc + 255) / 256) >= 256;
      if (small_tiles) {
        g.mt = (tc + 31) / 32; g.nt = (tc + 63) / 64;
        hipLaunchKernelGGL((k_fsa_gemm_f32<0, false, false, 32, 64, 1, 2>), dim3(8 * groups * g.mt * g.nt), dim3(128),
                           0, ctx->stream, g);
      } else if (big) {
        g.mt = g.nt = (tc + 255) / 256;
        hipLaunchKernelGGL((k_fsa_gemm_f32<0, false, false, 256, 256, 2, 4, false, true>), dim3(8 * groups * g.mt * g.nt), dim3(512),
                           0, ctx->stream, g);
      } else {
        g.mt = g.nt = (tc + 127) / 128;
        hipLaunchKernelGGL((k_fsa_gemm_f32<0, false, false, 128, 128, 2, 2, false, true>), dim3(8 * groups * g.mt * g.nt), dim3(256),
                           0, ctx->stream, g);
      }
      BDH_LAUNCH_CHECK(ctx, "k_fsa_gemm_f32<chunk scores>");
    }
    {  // out = Q rho   (the state before this chunk; B = rho [Nq,d] is k-major; ALiBi: row t *= decay^t)
      FsaArgs g{};
      g.A = qc; g.Bm = rho; g.C = p.out + (long)t0 * d;
      g.a_batch = q_batch; g.b_batch = (long)Nq * d; g.c_batch = (long)T * d;
      g.lda = Nq; g.ldb = d; g.ldc = d; g.M = tc; g.N = d; g.K = Nq; g.b_div = 1; g.n_slices = (int)S;
      g.block_size = 1; g.h = h; g.dense = 0; g.beta = 0;
      with_decay(g, FSA_DECAY_ROWS);
      if (small_tiles) {
        g.mt = (tc + 31) / 32; g.nt = (d + 63) / 64;
        hipLaunchKernelGGL((k_fsa_gemm_f32<2, false, true, 32, 64, 1, 2>), dim3(8 * groups * g.mt * g.nt), dim3(128), 0,
                           ctx->stream, g);
      } else {
        g.mt = (tc + 127) / 128; g.nt = nt_d;
        hipLaunchKernelGGL((k_fsa_gemm_f32<2, false, true, 128, 128, 2, 2, false, true>), dim3(8 * groups * g.mt * g.nt), dim3(256), 0,
                           ctx->stream, g);
      }
      BDH_LAUNCH_CHECK(ctx, "k_fsa_gemm_f32<Q rho>");
    }
    {  // out += S V   (K limited to the causal prefix of each row tile)
      FsaArgs g{};
      g.A = scores; g.Bm = p.v + (long)t0 * d; g.C = p.out + (long)t0 * d;
      g.a_batch = (long)Tc * Tcp; g.b_batch = (long)T * d; g.c_batch = (long)T * d;
      g.lda = Tcp; g.ldb = d; g.ldc = d; g.M = tc; g.N = d; g.K = tc; g.b_div = h; g.n_slices = (int)S;
      g.block_size = 1; g.h = h; g.dense = 1; g.beta = 1;
      if (small_tiles) {
        g.mt = (tc + 31) / 32; g.nt = (d + 63) / 64;
        hipLaunchKernelGGL((k_fsa_gemm_f32<2, false, true, 32, 64, 1, 2>), dim3(8 * groups * g.mt * g.nt), dim3(128), 0,
                           ctx->stream, g);
      } else {
        g.mt = (tc + 127) / 128; g.nt = nt_d;
        hipLaunchKernelGGL((k_fsa_gemm_f32<2, false, true, 128, 128, 2, 2, false, true>), dim3(8 * groups * g.mt * g.nt), dim3(256), 0,
                           ctx->stream, g);
      }
      BDH_LAUNCH_CHECK(ctx, "k_fsa_gemm_f32<S V>");
    }
    {  // rho += Q^T V   (both operands k-major: the reduction runs over the tokens)
       // ALiBi: rho = decay^tc * rho + sum_s decay^(tc-s) q_s (x) v_s
      FsaArgs g{};
      g.A = qc; g.Bm = p.v + (long)t0 * d; g.C = rho;
      g.a_batch = q_batch; g.b_batch = (long)T * d; g.c_batch = (long)Nq * d;
      g.lda = Nq; g.ldb = d; g.ldc = d; g.M = Nq; g.N = d; g.K = tc; g.b_div = h; g.n_slices = (int)S;
      g.block_size = 1; g.h = h; g.dense = 0; g.beta = 1;
      with_decay(g, FSA_DECAY_STATE);
      if (small_tiles) {
        g.mt = (Nq + 31) / 32; g.nt = (d + 63) / 64;
        hipLaunchKernelGGL((k_fsa_gemm_f32<2, true, true, 32, 64, 1, 2>), dim3(8 * groups * g.mt * g.nt), dim3(128), 0,
                           ctx->stream, g);
      } else {
        g.mt = (Nq + 127) / 128; g.nt = nt_d;
        hipLaunchKernelGGL((k_fsa_gemm_f32<2, true, true, 128, 128, 2, 2, false, true>), dim3(8 * groups * g.mt * g.nt), dim3(256), 0,
                           ctx->stream, g);
      }
      BDH_LAUNCH_CHECK(ctx, "k_fsa_gemm_f32<Q^T V>");
    }
  }
  if (bf16_state) {
    hipLaunchKernelGGL(k_narrow_bf16, dim3((unsigned)std::min<size_t>((n_state + 255) / 256, 1u << 20)), dim3(256), 0,
                       ctx->stream, rho, static_cast<unsigned short *>(p.rho), n_state);
    BDH_LAUNCH_CHECK(ctx, "k_narrow_bf16");
  }
  if (p.stamps) {  // every row is now up to date as of the end of the call
    const long rows = S * N;
    hipLaunchKernelGGL(k_set_stamps, dim3((unsigned)((rows + 255) / 256)), dim3(256), 0, ctx->stream, p.stamps, rows,
                       (long)h * N, (long)(p.position + T), p.positions_dev, T);
    BDH_LAUNCH_CHECK(ctx, "k_set_stamps");
  }
  if (out_ln) return bdh_launch_layer_norm_rows(ctx, (int64_t)S * T, d, p.out, out_ln);
  return BDH_OK;
}

// The encoder E over many rows (src/model/bdh.rs:383,436-438): mixed [B*T, h*N] . decoder [h*N, d], as one
// product per (sequence, head) on the f32 matrix cores.  partial [h][B*T][d] receives the h per-head terms
// of every output row; the caller sums them in head order.
int bdh_launch_decoder_partials_f32(bdh_ctx *ctx, int B, int T, int h, int N, int d, const float *xy,
                                    const float *decoder, float *partial) {
  const long S = (long)B * h;
  const unsigned groups = (unsigned)((S + 7) / 8);
  FsaArgs g{};
  g.A = xy; g.Bm = decoder; g.C = partial;
  g.mod = h;
  g.a_batch = (long)h * T * N; g.a_mod_stride = (long)T * N;  // xy [B,h,T,N]
  g.b_batch = 0; g.b_mod_stride = (long)N * d;                // decoder rows hh*N .. hh*N+N-1
  g.c_batch = (long)T * d; g.c_mod_stride = (long)B * T * d;
  g.lda = N; g.ldb = d; g.ldc = d; g.M = T; g.N = d; g.K = N; g.b_div = 1; g.n_slices = (int)S;
  g.block_size = 1; g.h = h; g.dense = 0; g.beta = 0;
  g.mt = (T + 127) / 128; g.nt = (d + 127) / 128;
  if ((long)groups * 8 * g.mt * g.nt > 0x7fffffffL) return bdh_fail(ctx, BDH_E_SHAPE, "too many tiles");
  hipLaunchKernelGGL((k_fsa_gemm_f32<2, false, true, 128, 128, 2, 2, false, true>), dim3(8 * groups * g.mt * g.nt), dim3(256), 0,
                     ctx->stream, g);
  BDH_LAUNCH_CHECK(ctx, "k_fsa_gemm_f32<decoder>");
  return BDH_OK;
}

extern "C" int bdh_rotate(bdh_ctx *ctx, int B, int h, int T, int N, int rotary, const float *x, const float *freqs,
                          int64_t position, const int32_t *positions_dev, float *q) {
  if (!ctx) return BDH_E_INVAL;
  if (B < 0 || h < 0 || T < 0 || N < 0) return bdh_fail(ctx, BDH_E_INVAL, "negative dimension");
  if (rotary != BDH_ROPE && rotary != BDH_ALIBI && rotary != BDH_POPE)
    return bdh_fail(ctx, BDH_E_INVAL, "rotary %d is not a bdh_rotary value", rotary);
  if (position < 0) return bdh_fail(ctx, BDH_E_INVAL, "negative position");
  if (rotary == BDH_ROPE && (N & 1)) return bdh_fail(ctx, BDH_E_SHAPE, "RoPE needs an even latent size, got N=%d", N);
  const long rows = (long)B * h * T;
  if (rows == 0 || N == 0) return BDH_OK;
  if (!x || !q || (rotary != BDH_ALIBI && !freqs)) return bdh_fail(ctx, BDH_E_INVAL, "null data pointer");
  if (!bdh_aligned(x, 8) || !bdh_aligned(q, 8) || !bdh_aligned(freqs, 8))
    return bdh_fail(ctx, BDH_E_ALIGN, "x, q and freqs need 8-byte alignment");
  if (rows > 0x7fffffffL) return bdh_fail(ctx, BDH_E_SHAPE, "B*h*T too large");
  if (rotary == BDH_ALIBI) {  // Attention::rotate returns its input (src/model/attention.rs:333-335)
    if (q != x)
      BDH_HIP_CHECK(ctx, hipMemcpyAsync(q, x, sizeof(float) * (size_t)rows * N, hipMemcpyDeviceToDevice, ctx->stream));
    return BDH_OK;
  }
  hipLaunchKernelGGL(k_rotate_chunk_f32, dim3((unsigned)rows), dim3(256), 0, ctx->stream, x, (long)T * N, freqs, q, T, N,
                     rotary, (long)position, positions_dev, 0, h);
  BDH_LAUNCH_CHECK(ctx, "k_rotate_chunk_f32");
  return BDH_OK;
}

// The encoder E of a decode step for a batch of sequences (T = 1, src/model/bdh.rs:383,436-438): mixed [B, h*N] is
// contiguous per sequence, so the product is one [B x K] . [K x d] GEMM split over K: slice s takes k in
// [s*KB, (s+1)*KB) and writes partial[s][B][d].  With 8 or more sequences nearly every row of E is needed by some
// sequence, so the weights are streamed once through the matrix cores instead of skipping inactive rows.
int bdh_launch_decoder_splitk_f32(bdh_ctx *ctx, int M, long K, int d, int KB, const float *xy, const float *decoder,
                                  float *partial) {
  const long KBN = (K + KB - 1) / KB;
  const unsigned groups = (unsigned)((KBN + 7) / 8);
  FsaArgs g{};
  g.A = xy; g.Bm = decoder; g.C = partial;
  g.a_batch = KB; g.b_batch = (long)KB * d; g.c_batch = (long)M * d;
  g.lda = (int)K; g.ldb = d; g.ldc = d; g.M = M; g.N = d; g.K = KB; g.b_div = 1; g.n_slices = (int)KBN;
  g.block_size = 1; g.h = 1; g.dense = 0; g.beta = 0;
  g.mt = (M + 31) / 32; g.nt = (d + 63) / 64;
  if (K % KB != 0) return bdh_fail(ctx, BDH_E_SHAPE, "split-K block %d does not divide K=%ld", KB, K);
  if ((long)groups * 8 * g.mt * g.nt > 0x7fffffffL) return bdh_fail(ctx, BDH_E_SHAPE, "too many tiles");
  hipLaunchKernelGGL((k_fsa_gemm_f32<2, false, true, 32, 64, 1, 2>), dim3(8 * groups * g.mt * g.nt), dim3(128), 0,
                     ctx->stream, g);
  BDH_LAUNCH_CHECK(ctx, "k_fsa_gemm_f32<decoder split-K>");
  return BDH_OK;
}

// relu_lowrank for many rows per (sequence, head) on the f32 matrix cores: one product [T, d] x [d, N] per slice with
// the k order of a scalar loop (SEQK), so the outputs are the bits of k_relu_lowrank.  mask_dev: one byte per latent
// block in device memory, or null.
int bdh_launch_relu_lowrank_gemm(bdh_ctx *ctx, const ReluLowrankParams &p, const unsigned char *mask_dev) {
  FsaArgs g{};
  g.A = p.in;
  g.Bm = p.weight;
  g.C = p.out;
  g.mod = p.h;                                   // slice = b * h + head
  g.a_batch = (long)p.h_in * p.T * p.d;
  g.a_mod_stride = p.h_in == 1 ? 0 : (long)p.T * p.d;
  g.b_batch = 0;
  g.b_mod_stride = (long)p.d * p.N;
  g.c_batch = (long)p.h * p.T * p.N;
  g.c_mod_stride = (long)p.T * p.N;
  g.lda = p.d;
  g.ldb = p.N;
  g.ldc = p.N;
  g.M = p.T;
  g.N = p.N;
  g.K = p.d;
  g.b_div = 1;
  g.n_slices = p.B * p.h;
  g.block_size = 1;
  g.h = p.h;
  g.rl_bias = p.bias;
  g.rl_thr = p.threshold;
  g.rl_mask = mask_dev;
  g.rl_block = p.block_size > 0 ? p.block_size : 1;
  g.rl_nblocks = p.n_blocks;
  g.rl_gate = p.gate;
  const int groups = (g.n_slices + 7) / 8;
  // 128 x 128 tiles: K = d is short (a 256 x 256 tile spends as long in its prologue and 256 KiB epilogue as in its
  // 32 k stages: 12.1 against 10.8 ms for [8192 x 512] x [512 x 131072])
  // 128 x 256 tiles for wide matrices: 10.8 -> 10.1 ms for [8192 x 512] x [512 x 131072]
  g.mt = (p.T + 127) / 128;
  const bool wide = p.N % 256 == 0 && (long)p.B * p.h * g.mt * (p.N / 256) >= 2L * (ctx->n_cu > 0 ? ctx->n_cu : 256);
  g.nt = wide ? p.N / 256 : (p.N + 127) / 128;
  if ((long)8 * groups * g.mt * g.nt > 0x7fffffffL) return bdh_fail(ctx, BDH_E_SHAPE, "too many tiles");
  if (wide)
    hipLaunchKernelGGL((k_fsa_gemm_f32<3, false, true, 128, 256, 2, 4, true>), dim3(8 * groups * g.mt * g.nt), dim3(512), 0,
                       ctx->stream, g);
  else
    hipLaunchKernelGGL((k_fsa_gemm_f32<3, false, true, 128, 128, 2, 2, true>), dim3(8 * groups * g.mt * g.nt), dim3(256), 0,
                       ctx->stream, g);
  BDH_LAUNCH_CHECK(ctx, "k_fsa_gemm_f32<relu_lowrank>");
  return BDH_OK;
}
