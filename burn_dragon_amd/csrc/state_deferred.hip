// The decode state step with DEFERRED updates (RoPE, d in {256,512}, f32 or bf16 state) on gfx950.
// Reference semantics: BDH::recurrent_attention at T = 1 (src/model/bdh.rs:258-307, rotation
// src/model/attention.rs:305-349): out_t = sum_n rho_{t-1}[n,:] q_t[n], then rho_t = rho_{t-1} + q_t (x) v_t.
//
// The eager step (state_step.hip) reads every active state row and writes it back.  Here a step only
// READS its active rows and appends its update to a log; the rows are written once per flush:
//
//   out_t   = sum_n rho_base[n,:] q_t[n]  +  sum_{s logged} (q_t . q_s) v_s           (readout)
//   log    <- (which pairs q_t touches, their rotated values, v_t)                      (append)
//   flush:    every state row that some logged step touched takes its updates in step order,
//             row + (q_s[n] * v_s) with the product rounded before the add -- the operations and the
//             order of the eager step, so the flushed state holds the same bits.
//
// Layout of the log (device memory owned by a bdh_state_log): a "unit" is 256 adjacent lane pairs (512
// neurons) of one (b,h) slice, the share of one workgroup.  The log is kept PER PAIR, so that a step finds the
// pending updates of its active pairs, and the flush those of a row, in one contiguous piece:
//   pmask  [unit][256][2]  uint64: bit s % 64 of word s / 64 set iff logged step s touched the pair
//   pvals  [unit][256][K]  float2: the pair's rotated (q_even, q_odd) of those steps, in step order
//   vlog   [K][B][d]       the value rows of the logged steps
//   scores [unit][128]     this step's partial dot products q_t . q_s over the unit's pairs (scratch)
#include <algorithm>
#include <new>
#include <type_traits>

#include "bdh_internal.h"
#include "state_common.h"

struct bdh_state_log {
  int device = 0;
  int B = 0, h = 0, N = 0, d = 0, rho_dtype = BDH_F32, K = 0;
  int S = 0;               // units per (b,h) slice
  int count = 0;           // steps logged and not yet applied
  const void *rho = nullptr;  // the state the logged steps belong to
  void *mem = nullptr;     // one allocation holding the four arrays below
  size_t mem_bytes = 0;
  ulonglong2 *pmask = nullptr;
  float2 *pvals = nullptr;
  float *vlog = nullptr;
  float *scores = nullptr;
};

namespace {

constexpr int kUnitPairs = 256;  // lane pairs per unit = per workgroup of four wavefronts
constexpr int kMaxLog = 128;     // two logged steps per lane of a wavefront
constexpr int kScoreAhead = 6;   // active pairs of a wavefront whose logged values are fetched ahead of the state rows

// The part of a lane pair's two state rows (2*D adjacent elements) that one lane of a wavefront holds:
// NG groups of GW adjacent elements of one row.  f32: a lane owns four columns per 256 of both rows (16-byte
// accesses); bf16: a lane owns 16-byte pieces of the 4*D-byte chunk (eight elements of one row each).
template <typename RhoT, int D>
struct PairFrag {
  static constexpr bool kF32 = sizeof(RhoT) == 4;
  static constexpr int GW = kF32 ? 4 : 8;
  static constexpr int NG = kF32 ? 2 * (D / 256) : D / 256;
  __device__ static __forceinline__ int row(int g, int lane) { return kF32 ? g / (D / 256) : ((g * 64 + lane) * 8) / D; }
  __device__ static __forceinline__ int col(int g, int lane) {
    return kF32 ? ((g % (D / 256)) * 64 + lane) * 4 : ((g * 64 + lane) * 8) % D;
  }
  // Rows are streamed: every access is non-temporal, so that the lines of the log, which are read again on the
  // next step, are the ones the caches keep.  A group travels as one 16-byte register quad (Raw) and is widened to
  // floats where it is used, so that many groups can be in flight per lane.
  typedef float v4f __attribute__((ext_vector_type(4)));
  typedef unsigned int v4u __attribute__((ext_vector_type(4)));
  using Raw = typename std::conditional<kF32, v4f, v4u>::type;
  __device__ static __forceinline__ Raw load_raw(const RhoT *pair, int g, int lane) {
    if constexpr (kF32)
      return __builtin_nontemporal_load(reinterpret_cast<const v4f *>(pair + row(g, lane) * D + col(g, lane)));
    else
      return __builtin_nontemporal_load(reinterpret_cast<const v4u *>(pair + (g * 64 + lane) * 8));
  }
  __device__ static __forceinline__ void expand(const Raw &t, float (&f)[GW]) {
    if constexpr (kF32) {
      f[0] = t.x; f[1] = t.y; f[2] = t.z; f[3] = t.w;
    } else {
      const unsigned int w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        f[2 * k] = __uint_as_float(w[k] << 16);
        f[2 * k + 1] = __uint_as_float(w[k] & 0xffff0000u);
      }
    }
  }
  __device__ static __forceinline__ void load_nt(const RhoT *pair, int g, int lane, float (&f)[GW]) {
    expand(load_raw(pair, g, lane), f);
  }
  // two floats rounded to bf16 (nearest even, the hardware conversion; the bits of f32_to_bf16 for every finite
  // value), packed low | high
  __device__ static __forceinline__ unsigned int pack_bf16(float lo, float hi) {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    const f32x2 a = {lo, hi};
    return __builtin_bit_cast(unsigned int, __builtin_convertvector(a, bf16x2));
  }
  // a bf16 state holds bf16 values after every step: the floats of a group rounded in place
  __device__ static __forceinline__ void round_in_place(float (&f)[GW]) {
    if constexpr (!kF32) {
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const unsigned int pk = pack_bf16(f[2 * k], f[2 * k + 1]);
        f[2 * k] = __uint_as_float(pk << 16);
        f[2 * k + 1] = __uint_as_float(pk & 0xffff0000u);
      }
    }
  }
  __device__ static __forceinline__ void store_nt(RhoT *pair, int g, int lane, const float (&f)[GW]) {
    if constexpr (kF32) {
      v4f t; t.x = f[0]; t.y = f[1]; t.z = f[2]; t.w = f[3];
      __builtin_nontemporal_store(t, reinterpret_cast<v4f *>(pair + row(g, lane) * D + col(g, lane)));
    } else {
      v4u o;
      o.x = pack_bf16(f[0], f[1]);
      o.y = pack_bf16(f[2], f[3]);
      o.z = pack_bf16(f[4], f[5]);
      o.w = pack_bf16(f[6], f[7]);
      __builtin_nontemporal_store(o, reinterpret_cast<v4u *>(pair + (g * 64 + lane) * 8));
    }
  }
};

__device__ __forceinline__ unsigned long long readlane64(unsigned long long v, int lane) {
  const unsigned int lo = __builtin_amdgcn_readlane((int)(unsigned int)v, lane);
  const unsigned int hi = __builtin_amdgcn_readlane((int)(unsigned int)(v >> 32), lane);
  return ((unsigned long long)hi << 32) | lo;
}
__device__ __forceinline__ float readlane_f(float v, int lane) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}

struct DeferArgs {
  const float *x;
  long x_slice_stride;
  const float *v;  // [B][d]
  const float *freqs;
  long pos_int;
  const int32_t *pos_dev;
  float *partial;  // [units][d]
  int *pair_cnt;   // [units]
  unsigned long long *bitmask;
  long bitmask_slice_stride;
  int h, N, S, B;
  ulonglong2 *pmask;
  float2 *pvals;
  float *vlog;
  float *scores;
  int K, count;
};

// ------------------------------------------------------------------------------------
// The step: rotate + compact (as the eager kernel), read the active rows, score the logged steps against
// this one, append to the log.  One workgroup of four wavefronts per unit, U pairs in flight per wave.
// ------------------------------------------------------------------------------------
template <typename RhoT, int D, int U, bool HI>
__global__ __launch_bounds__(256) void k_step_deferred(DeferArgs a, const RhoT *__restrict__ rho) {
  using F = PairFrag<RhoT, D>;
  constexpr int NG = F::NG, GW = F::GW;
  __shared__ int s_cnt[4];
  __shared__ unsigned short s_idx[kUnitPairs];
  __shared__ float2 s_q[kUnitPairs];
  __shared__ float s_red[4][2][D];
  __shared__ float s_score[4][kMaxLog];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int unit = blockIdx.x;
  const int slice = unit / a.S;
  const int seg = unit - slice * a.S;
  const int b = slice / a.h;
  const int NP = a.N >> 1;
  const int p = seg * kUnitPairs + tid;

  float2 xv = make_float2(0.0f, 0.0f), fv = make_float2(0.0f, 0.0f);
  // which logged steps touched this lane's pair (independent of x: in flight together with it)
  ulonglong2 pm = make_ulonglong2(0ull, 0ull);
  if (p < NP) {
    xv = reinterpret_cast<const float2 *>(a.x + (long)slice * a.x_slice_stride)[p];
    fv = reinterpret_cast<const float2 *>(a.freqs)[p];
    pm = a.pmask[(long)unit * kUnitPairs + tid];
  }
  const float pos = (float)(a.pos_dev ? (long)a.pos_dev[b] : a.pos_int);

  const bool ae = xv.x != 0.0f, ao = xv.y != 0.0f;
  const bool act = ae || ao;
  const unsigned long long m_act = __ballot(act);
  if (a.bitmask) {
    const unsigned long long me = __ballot(ae), mo = __ballot(ao);
    if (lane == 0) {
      const int w0 = (seg * kUnitPairs + wave * 64) >> 5;
      const int NW = (a.N + 63) >> 6;
      unsigned long long *bm = a.bitmask + (long)slice * a.bitmask_slice_stride;
      if (w0 < NW) bm[w0] = spread_bits((unsigned int)me) | (spread_bits((unsigned int)mo) << 1);
      if (w0 + 1 < NW)
        bm[w0 + 1] = spread_bits((unsigned int)(me >> 32)) | (spread_bits((unsigned int)(mo >> 32)) << 1);
    }
  }
  // rotation of this lane's pair (src/model/attention.rs:305-321), the arithmetic of the eager kernel
  float2 q = make_float2(0.0f, 0.0f);
  if (act) {
    float s0, c0, s1, c1;
    sincosf(rope_phase(pos, fv.x), &s0, &c0);
    if (fv.y == fv.x) {
      s1 = s0;
      c1 = c0;
    } else {
      sincosf(rope_phase(pos, fv.y), &s1, &c1);
    }
    const float a0 = xv.x * c0, r0 = (-xv.y) * s0;
    const float a1 = xv.y * c1, r1 = xv.x * s1;
    q.x = a0 + r0;
    q.y = a1 + r1;
  }
  if (lane == 0) s_cnt[wave] = __popcll(m_act);
  __syncthreads();
  int offset = 0, total = 0;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const int c = s_cnt[w];
    if (w < wave) offset += c;
    total += c;
  }
  const unsigned long long below = (1ull << lane) - 1ull;
  if (act) {
    const int rank = offset + __popcll(m_act & below);
    s_idx[rank] = (unsigned short)tid;
    s_q[rank] = q;
  }
  __syncthreads();

  // Scores of the logged steps against this one over this wavefront's 64 pairs: lane s collects q_t . q_s for the
  // logged steps s and s + 64.  The wavefront walks its active pairs in pair order; for a pair, the lanes of the
  // steps that touched it fetch that step's values -- adjacent entries of the pair's list, one coalesced access.
  // The accesses of the first kScoreAhead pairs (steps below 64) are issued here, ahead of the state rows (a
  // wavefront's memory operations complete in issue order, so the first wait for rows covers them); their
  // products are added after the row loop, where the remaining pairs and the steps from 64 on follow.
  const float2 *pv = a.pvals + ((long)unit * kUnitPairs + wave * 64) * a.K;
  const unsigned long long m_all = a.count > 0 ? m_act : 0ull;
  unsigned long long m_sc = m_all;
  float2 se[kScoreAhead];
  int sp[kScoreAhead];
  bool sb0[kScoreAhead];
#pragma unroll
  for (int j = 0; j < kScoreAhead; ++j) {
    const bool has = m_sc != 0ull;
    sp[j] = has ? __builtin_ctzll(m_sc) : 0;
    m_sc &= m_sc - 1ull;  // stays zero once it is
    const unsigned long long lo = readlane64(pm.x, sp[j]);
    sb0[j] = has && ((lo >> lane) & 1ull);
    se[j] = make_float2(0.0f, 0.0f);
    if (sb0[j]) se[j] = pv[(long)sp[j] * a.K + __popcll(lo & below)];
  }

  // readout against the stored rows (read only)
  float acc[NG][GW];
#pragma unroll
  for (int g = 0; g < NG; ++g)
#pragma unroll
    for (int e = 0; e < GW; ++e) acc[g][e] = 0.0f;
  const RhoT *base = rho + ((long)slice * a.N + 2L * seg * kUnitPairs) * D;
  for (int i0 = wave; i0 < total; i0 += 4 * U) {
    typename F::Raw r[U][NG];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i = i0 + u * 4;
      if (i < total) {
        const RhoT *pp = base + (long)s_idx[i] * (2 * D);
#pragma unroll
        for (int g = 0; g < NG; ++g) r[u][g] = F::load_raw(pp, g, lane);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i = i0 + u * 4;
      if (i < total) {
        const float2 qq = s_q[i];
#pragma unroll
        for (int g = 0; g < NG; ++g) {
          const float qf = F::row(g, lane) ? qq.y : qq.x;
          float f[GW];
          F::expand(r[u][g], f);
#pragma unroll
          for (int e = 0; e < GW; ++e) acc[g][e] = __builtin_fmaf(f[e], qf, acc[g][e]);
        }
      }
    }
  }

  {
    float sc0 = 0.0f, sc1 = 0.0f;
#pragma unroll
    for (int j = 0; j < kScoreAhead; ++j) {
      const float qx = readlane_f(q.x, sp[j]), qy = readlane_f(q.y, sp[j]);
      if (sb0[j]) sc0 = __builtin_fmaf(qy, se[j].y, __builtin_fmaf(qx, se[j].x, sc0));
    }
    while (m_sc) {  // a wavefront with more active pairs: the rest, four in flight
      float2 e0[4], qt[4];
      bool b0[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const bool has = m_sc != 0ull;
        const int pj = has ? __builtin_ctzll(m_sc) : 0;
        m_sc &= m_sc - 1ull;
        const unsigned long long lo = readlane64(pm.x, pj);
        qt[j] = make_float2(readlane_f(q.x, pj), readlane_f(q.y, pj));
        b0[j] = has && ((lo >> lane) & 1ull);
        if (b0[j]) e0[j] = pv[(long)pj * a.K + __popcll(lo & below)];
      }
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (b0[j]) sc0 = __builtin_fmaf(qt[j].y, e0[j].y, __builtin_fmaf(qt[j].x, e0[j].x, sc0));
    }
    if (HI && a.count > 64) {  // the steps from 64 on: the entries behind those of the first word in each list
      unsigned long long m_hi = m_all;
      while (m_hi) {
        float2 e1[4], qt[4];
        bool b1[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const bool has = m_hi != 0ull;
          const int pj = has ? __builtin_ctzll(m_hi) : 0;
          m_hi &= m_hi - 1ull;
          const unsigned long long lo = readlane64(pm.x, pj), hi = readlane64(pm.y, pj);
          qt[j] = make_float2(readlane_f(q.x, pj), readlane_f(q.y, pj));
          b1[j] = has && ((hi >> lane) & 1ull);
          if (b1[j]) e1[j] = pv[(long)pj * a.K + __popcll(lo) + __popcll(hi & below)];
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (b1[j]) sc1 = __builtin_fmaf(qt[j].y, e1[j].y, __builtin_fmaf(qt[j].x, e1[j].x, sc1));
      }
    }
    s_score[wave][lane] = sc0;
    s_score[wave][64 + lane] = sc1;
  }
  // log append: the pair's list grows by this step's values, its mask by this step's bit.  Last, so that the
  // list's cache line, which the scores above have just read, is in the L2 when the 8-byte store arrives.
  if (act) {
    a.pvals[((long)unit * kUnitPairs + tid) * a.K + __popcll(pm.x) + __popcll(pm.y)] = q;
    if (a.count < 64) pm.x |= 1ull << a.count; else pm.y |= 1ull << (a.count - 64);
    a.pmask[(long)unit * kUnitPairs + tid] = pm;
  }

  // cross-wave reduction of the readout and of the scores, fixed order
#pragma unroll
  for (int g = 0; g < NG; ++g) {
    float *dst = &s_red[wave][F::row(g, lane)][F::col(g, lane)];
#pragma unroll
    for (int e = 0; e < GW; ++e) dst[e] = acc[g][e];
  }
  __syncthreads();
  float *pout = a.partial + (long)unit * D;
  for (int c = tid; c < D; c += 256) {
    float s = 0.0f;
#pragma unroll
    for (int w = 0; w < 4; ++w) s += s_red[w][0][c] + s_red[w][1][c];
    pout[c] = s;
  }
  if (tid < a.count) a.scores[(long)unit * kMaxLog + tid] = (s_score[0][tid] + s_score[1][tid]) + (s_score[2][tid] + s_score[3][tid]);
  if (tid == 0) a.pair_cnt[unit] = total;
}

// ------------------------------------------------------------------------------------
// Second stage: out[slice,:] = sum of the unit partials (index order) + sum_s (q_t . q_s) v_s over the
// logged steps; optional LayerNorm (src/model/bdh.rs:359); appends v_t to the log.
// One workgroup finishes CW columns of one slice (blockIdx.y = which): thread (g, c4) = (tid / (CW/4), tid % (CW/4))
// takes four columns and, of the units and of the logged steps, every G-th (G = 1024 / CW): all of its loads (score
// partials, readout partials, logged value rows) are issued before the first of them is needed, and the G groups
// are added in group order through LDS.  KMAX = 64 or 128 bounds the logged steps.  LN needs CW = d.
// ------------------------------------------------------------------------------------
template <bool LN, int CW, int KMAX>
__global__ __launch_bounds__(256) void k_deferred_finalize(DeferArgs a, int d, float *__restrict__ out,
                                                           float *__restrict__ out_ln, int *__restrict__ rows) {
  constexpr int NC4 = CW / 4, G = 256 / NC4, NI = KMAX / G, UG = 256 / KMAX;
  static_assert(NI * G == KMAX && NI >= 1, "the step groups must cover the log");
  __shared__ float s_tp[UG][KMAX];
  __shared__ float4 s_acc[G][NC4];
  const int tid = threadIdx.x, g = tid / NC4, c4 = tid - g * NC4;
  const int slice = blockIdx.x;
  const int col0 = blockIdx.y * CW;
  const int b = slice / a.h, hh = slice - b * a.h;
  const int S = a.S, count = a.count;
  const int nc4 = d >> 2;

  {  // score partials: thread (ug, s) adds every UG-th unit's q_t . q_s
    const int ug = tid / KMAX, s = tid - ug * KMAX;
    float tpart = 0.0f;
    if (s < count) {
#pragma unroll 8
      for (int u = ug; u < S; u += UG) tpart += a.scores[((long)slice * S + u) * kMaxLog + s];
    }
    s_tp[ug][s] = tpart;
  }
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f), vl[NI];
  {
    const float4 *p4 = reinterpret_cast<const float4 *>(a.partial + (long)slice * S * d + col0) + c4;
#pragma unroll 4
    for (int u = g; u < S; u += G) {
      const float4 t = p4[(long)u * nc4];
      acc.x += t.x; acc.y += t.y; acc.z += t.z; acc.w += t.w;
    }
    if (count > 0) {
      const float4 *v4 = reinterpret_cast<const float4 *>(a.vlog + (long)b * d + col0) + c4;
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const int st = min(g + G * i, count - 1);  // steps at or beyond count re-read the last row; their score is zero
        vl[i] = v4[(long)st * a.B * nc4];
      }
    }
  }
  __syncthreads();
  if (count > 0) {
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int st = g + G * i;
      float tot = s_tp[0][st];
#pragma unroll
      for (int ug = 1; ug < UG; ++ug) tot += s_tp[ug][st];
      acc.x = __builtin_fmaf(tot, vl[i].x, acc.x);
      acc.y = __builtin_fmaf(tot, vl[i].y, acc.y);
      acc.z = __builtin_fmaf(tot, vl[i].z, acc.z);
      acc.w = __builtin_fmaf(tot, vl[i].w, acc.w);
    }
  }
  s_acc[g][c4] = acc;
  __syncthreads();
  float vals[(CW + 255) / 256];
  float lsum = 0.0f;
#pragma unroll
  for (int j = 0; j < (CW + 255) / 256; ++j) {
    const int c = j * 256 + tid;
    vals[j] = 0.0f;
    if (c < CW) {
      const float *sa = reinterpret_cast<const float *>(&s_acc[0][0]);
      float sv = sa[c];
#pragma unroll
      for (int gg = 1; gg < G; ++gg) sv += sa[gg * CW + c];
      out[(long)slice * d + col0 + c] = sv;
      vals[j] = sv;
      lsum += sv;
      if (hh == 0) a.vlog[((long)count * a.B + b) * d + col0 + c] = a.v[(long)b * d + col0 + c];  // log append: v_t
    }
  }
  if (rows && tid == 0 && blockIdx.y == 0) {
    int np = 0;
    for (int u = 0; u < S; ++u) np += a.pair_cnt[(long)slice * S + u];
    rows[slice] = 2 * np;
  }
  if constexpr (LN) {  // CW == d: this workgroup holds the whole row
    __shared__ float s_part[4];
    __shared__ float s_stat[2];
    const int lane = tid & 63, wave = tid >> 6;
    for (int o = 32; o > 0; o >>= 1) lsum += __shfl_xor(lsum, o);
    if (lane == 0) s_part[wave] = lsum;
    __syncthreads();
    if (tid == 0) s_stat[0] = (s_part[0] + s_part[1] + s_part[2] + s_part[3]) / (float)d;
    __syncthreads();
    const float mean = s_stat[0];
    float lsq = 0.0f;
#pragma unroll
    for (int j = 0; j < (CW + 255) / 256; ++j) {
      const int c = j * 256 + tid;
      if (c < CW) {
        const float t = vals[j] - mean;
        lsq += t * t;
      }
    }
    for (int o = 32; o > 0; o >>= 1) lsq += __shfl_xor(lsq, o);
    __syncthreads();
    if (lane == 0) s_part[wave] = lsq;
    __syncthreads();
    if (tid == 0) s_stat[1] = sqrtf((s_part[0] + s_part[1] + s_part[2] + s_part[3]) / (float)d + 1e-5f);
    __syncthreads();
    const float den = s_stat[1];
#pragma unroll
    for (int j = 0; j < (CW + 255) / 256; ++j) {
      const int c = j * 256 + tid;
      if (c < CW) out_ln[(long)slice * d + c] = (vals[j] - mean) / den;
    }
  }
}

// ------------------------------------------------------------------------------------
// The flush: a workgroup of 16 wavefronts takes four consecutive units of one batch entry (they share the logged
// value rows, staged once in LDS); four wavefronts per unit, each owning 64 of its pairs.  For a pair, the pair's
// mask lists the steps that touched it; lane s of the wavefront fetches the values of steps s and s + 64 from the
// pair's list (coalesced) and the steps are applied in order: row + (q * v_s), product rounded before the add
// (src/model/bdh.rs:298); a bf16 state is rounded after every step, as the eager step stores it.  The pair masks are
// cleared on the way.  PB pairs in flight per wavefront.
// ------------------------------------------------------------------------------------
constexpr int kFlushUnits = 4;  // units per workgroup

template <typename RhoT, int D, int NG_, int GW_>
__device__ __forceinline__ void flush_apply(float (&r)[NG_][GW_], const float *vs, float qe, float qo, int lane) {
  using F = PairFrag<RhoT, D>;
#pragma unroll
  for (int g = 0; g < F::NG; ++g) {
    const float qf = F::row(g, lane) ? qo : qe;
    const float *vg = vs + F::col(g, lane);
#pragma unroll
    for (int e4 = 0; e4 < F::GW; e4 += 4) {
      const float4 v4 = *reinterpret_cast<const float4 *>(vg + e4);
      float t;
      t = qf * v4.x; r[g][e4 + 0] = r[g][e4 + 0] + t;
      t = qf * v4.y; r[g][e4 + 1] = r[g][e4 + 1] + t;
      t = qf * v4.z; r[g][e4 + 2] = r[g][e4 + 2] + t;
      t = qf * v4.w; r[g][e4 + 3] = r[g][e4 + 3] + t;
    }
    F::round_in_place(r[g]);  // the eager step stores bf16 after every token
  }
}

template <typename RhoT, int D, int PB>
__global__ __launch_bounds__(256 * kFlushUnits) void k_state_flush(DeferArgs a, RhoT *__restrict__ rho) {
  using F = PairFrag<RhoT, D>;
  constexpr int NG = F::NG, GW = F::GW;
  extern __shared__ float s_v[];  // [count][D]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = (tid >> 6) & 3;  // the quarter of the unit this wavefront owns
  const int b = blockIdx.y;
  const int ub = blockIdx.x * kFlushUnits + (tid >> 8);  // unit within the batch entry
  const int hS = a.h * a.S;
  for (int i = tid; i < a.count * (D / 4); i += 256 * kFlushUnits) {
    const int st = i / (D / 4), c4 = i - st * (D / 4);
    reinterpret_cast<float4 *>(s_v)[i] = reinterpret_cast<const float4 *>(a.vlog + ((long)st * a.B + b) * D)[c4];
  }
  const bool valid = ub < hS;
  const int unit = b * hS + (valid ? ub : 0);
  const int slice = unit / a.S;
  const int seg = unit - slice * a.S;
  // lane p: which logged steps touched pair p of this wavefront's 64
  ulonglong2 pm = make_ulonglong2(0ull, 0ull);
  ulonglong2 *pmp = a.pmask + (long)unit * kUnitPairs + wave * 64 + lane;
  if (valid) pm = *pmp;
  __syncthreads();
  if (pm.x | pm.y) *pmp = make_ulonglong2(0ull, 0ull);  // the log is empty after this launch
  const unsigned long long below = (1ull << lane) - 1ull;
  const float2 *pv = a.pvals + ((long)unit * kUnitPairs + wave * 64) * a.K;
  RhoT *base = rho + ((long)slice * a.N + 2L * (seg * kUnitPairs + wave * 64)) * D;

  for (int p0 = 0; p0 < 64; p0 += PB) {
    unsigned long long lo[PB], hi[PB];
    float2 q0[PB], q1[PB];
    float r[PB][NG][GW];
#pragma unroll
    for (int j = 0; j < PB; ++j) {
      lo[j] = readlane64(pm.x, p0 + j);
      hi[j] = readlane64(pm.y, p0 + j);
      q0[j] = q1[j] = make_float2(0.0f, 0.0f);
      // lane s: the values of steps s and s + 64 of the pair, entry (number of earlier steps in its list)
      const float2 *pl = pv + (long)(p0 + j) * a.K;
      if ((lo[j] >> lane) & 1ull) q0[j] = pl[__popcll(lo[j] & below)];
      if ((hi[j] >> lane) & 1ull) q1[j] = pl[__popcll(lo[j]) + __popcll(hi[j] & below)];
      if (lo[j] | hi[j]) {
        const RhoT *pp = base + (long)(p0 + j) * (2 * D);
#pragma unroll
        for (int g = 0; g < NG; ++g) {
          F::load_nt(pp, g, lane, r[j][g]);
        }
      }
    }
#pragma unroll
    for (int j = 0; j < PB; ++j) {
      if (!(lo[j] | hi[j])) continue;
      unsigned long long m = lo[j];
      while (m) {
        const int s = __builtin_ctzll(m);
        m &= m - 1ull;
        flush_apply<RhoT, D>(r[j], s_v + s * D, readlane_f(q0[j].x, s), readlane_f(q0[j].y, s), lane);
      }
      m = hi[j];
      while (m) {
        const int s = __builtin_ctzll(m);
        m &= m - 1ull;
        flush_apply<RhoT, D>(r[j], s_v + (64 + s) * D, readlane_f(q1[j].x, s), readlane_f(q1[j].y, s), lane);
      }
      RhoT *pp = base + (long)(p0 + j) * (2 * D);
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        F::store_nt(pp, g, lane, r[j][g]);
      }
    }
  }
}

__global__ __launch_bounds__(256) void k_fill_zero_u64(unsigned long long *__restrict__ p, size_t n) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = 0ull;
}

size_t log_layout(int B, int h, int N, int d, int K, size_t *o_masks, size_t *o_values, size_t *o_vlog, size_t *o_scores) {
  const size_t S = ((size_t)(N / 2) + kUnitPairs - 1) / kUnitPairs;
  const size_t units = (size_t)B * h * S;
  size_t off = 0;
  *o_masks = off;
  off += bdh_align_up(units * kUnitPairs * sizeof(ulonglong2), 256);
  *o_values = off;
  off += bdh_align_up(units * kUnitPairs * K * sizeof(float2), 256);
  *o_vlog = off;
  off += bdh_align_up((size_t)K * B * d * sizeof(float), 256);
  *o_scores = off;
  off += bdh_align_up(units * kMaxLog * sizeof(float), 256);
  return off;
}

DeferArgs make_args(const bdh_state_log *log) {
  DeferArgs a{};
  a.h = log->h;
  a.N = log->N;
  a.S = log->S;
  a.B = log->B;
  a.pmask = log->pmask;
  a.pvals = log->pvals;
  a.vlog = log->vlog;
  a.scores = log->scores;
  a.K = log->K;
  a.count = log->count;
  return a;
}

template <typename RhoT, int D>
int launch_flush(bdh_ctx *ctx, const DeferArgs &a, dim3 grid, size_t lds, void *rho) {
  auto kernel = k_state_flush<RhoT, D, 4>;
  if (lds > (size_t(64) << 10))
    BDH_HIP_CHECK(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  hipLaunchKernelGGL(kernel, grid, dim3(256 * kFlushUnits), lds, ctx->stream, a, static_cast<RhoT *>(rho));
  BDH_LAUNCH_CHECK(ctx, "k_state_flush");
  return BDH_OK;
}

template <bool LN, int CW>
void launch_finalize(bdh_ctx *ctx, const DeferArgs &a, int slices, int d, float *out, float *out_ln, int32_t *rows) {
  const dim3 grid(slices, d / CW), block(256);
  if (a.K > 64)
    hipLaunchKernelGGL((k_deferred_finalize<LN, CW, 128>), grid, block, 0, ctx->stream, a, d, out, out_ln, rows);
  else
    hipLaunchKernelGGL((k_deferred_finalize<LN, CW, 64>), grid, block, 0, ctx->stream, a, d, out, out_ln, rows);
}

}  // namespace

int bdh_launch_state_flush(bdh_ctx *ctx, bdh_state_log *log, void *rho) {
  if (log->count == 0) return BDH_OK;
  if (rho != log->rho)
    return bdh_fail(ctx, BDH_E_INVAL, "the %d logged steps belong to another state tensor", log->count);
  DeferArgs a = make_args(log);
  const int hS = log->h * log->S;
  const size_t lds = (size_t)log->count * log->d * sizeof(float);
  const dim3 grid((hS + kFlushUnits - 1) / kFlushUnits, log->B);
  int rc;
  if (log->rho_dtype == BDH_F32)
    rc = log->d == 256 ? launch_flush<float, 256>(ctx, a, grid, lds, rho) : launch_flush<float, 512>(ctx, a, grid, lds, rho);
  else
    rc = log->d == 256 ? launch_flush<unsigned short, 256>(ctx, a, grid, lds, rho)
                       : launch_flush<unsigned short, 512>(ctx, a, grid, lds, rho);
  if (rc != BDH_OK) return rc;
  log->count = 0;
  return BDH_OK;
}

int bdh_launch_state_step_deferred(bdh_ctx *ctx, bdh_state_log *log, const float *x, const float *v, const float *freqs,
                                   int64_t position, const int32_t *positions_dev, void *rho, float *out, float *out_ln,
                                   uint64_t *bitmask, int32_t *rows_touched) {
  if (log->count > 0 && rho != log->rho)
    return bdh_fail(ctx, BDH_E_INVAL, "the %d logged steps belong to another state tensor: flush it first", log->count);
  if (log->count == log->K) {
    int rc = bdh_launch_state_flush(ctx, log, rho);
    if (rc != BDH_OK) return rc;
  }
  const int B = log->B, h = log->h, N = log->N, d = log->d;
  const int slices = B * h, units = slices * log->S;
  const size_t partial_bytes = bdh_align_up(sizeof(float) * (size_t)units * d, 256);
  const size_t cnt_bytes = bdh_align_up(sizeof(int) * (size_t)units, 256);
  int rc = bdh_ws_reserve(ctx, partial_bytes + cnt_bytes);
  if (rc != BDH_OK) return rc;
  DeferArgs a = make_args(log);
  a.x = x;
  a.x_slice_stride = N;
  a.v = v;
  a.freqs = freqs;
  a.pos_int = (long)position;
  a.pos_dev = positions_dev;
  a.partial = reinterpret_cast<float *>(ctx->ws);
  a.pair_cnt = reinterpret_cast<int *>(static_cast<char *>(ctx->ws) + partial_bytes);
  a.bitmask = reinterpret_cast<unsigned long long *>(bitmask);
  a.bitmask_slice_stride = (N + 63) / 64;
  const dim3 grid(units), block(256);
#define BDH_STEP(T_, D_, U_)                                                                                        \
  do {                                                                                                              \
    if (a.K > 64)                                                                                                   \
      hipLaunchKernelGGL((k_step_deferred<T_, D_, U_, true>), grid, block, 0, ctx->stream, a, static_cast<const T_ *>(rho)); \
    else                                                                                                            \
      hipLaunchKernelGGL((k_step_deferred<T_, D_, U_, false>), grid, block, 0, ctx->stream, a, static_cast<const T_ *>(rho)); \
  } while (0)
  if (log->rho_dtype == BDH_F32) {
    if (d == 256) BDH_STEP(float, 256, 2); else BDH_STEP(float, 512, 2);
  } else {
    if (d == 256) BDH_STEP(unsigned short, 256, 8); else BDH_STEP(unsigned short, 512, 4);
  }
#undef BDH_STEP
  BDH_LAUNCH_CHECK(ctx, "k_step_deferred");
  if (out_ln) {
    if (d == 256) launch_finalize<true, 256>(ctx, a, slices, d, out, out_ln, rows_touched);
    else launch_finalize<true, 512>(ctx, a, slices, d, out, out_ln, rows_touched);
  } else {
    launch_finalize<false, 64>(ctx, a, slices, d, out, out_ln, rows_touched);
  }
  BDH_LAUNCH_CHECK(ctx, "k_deferred_finalize");
  log->rho = rho;
  log->count += 1;
  return BDH_OK;
}

extern "C" {

int bdh_state_log_create(bdh_ctx *ctx, int B, int h, int N, int d, int rho_dtype, int capacity, bdh_state_log **out) {
  if (!ctx || !out) return BDH_E_INVAL;
  *out = nullptr;
  if (B <= 0 || h <= 0 || N <= 0) return bdh_fail(ctx, BDH_E_INVAL, "B=%d h=%d N=%d must be positive", B, h, N);
  if (rho_dtype != BDH_F32 && rho_dtype != BDH_BF16) return bdh_fail(ctx, BDH_E_INVAL, "rho_dtype %d is not a bdh_dtype value", rho_dtype);
  if (h > 64) return bdh_fail(ctx, BDH_E_SHAPE, "n_head %d > 64", h);
  if (N & 1) return bdh_fail(ctx, BDH_E_SHAPE, "RoPE needs an even latent size, got N=%d", N);
  if (d != 256 && d != 512) return bdh_fail(ctx, BDH_E_SHAPE, "the deferred step is built for d in {256, 512}, got %d", d);
  if (capacity < 1 || capacity > kMaxLog || (long)capacity * d > 32768)
    return bdh_fail(ctx, BDH_E_SHAPE, "log capacity %d outside 1..%d for d=%d (capacity * d <= 32768: the flush keeps the logged value rows in LDS)",
                    capacity, std::min(kMaxLog, 32768 / d), d);
  bdh_state_log *log = new (std::nothrow) bdh_state_log();
  if (!log) return bdh_fail(ctx, BDH_E_NOMEM, "host allocation failed");
  log->device = ctx->device;
  log->B = B; log->h = h; log->N = N; log->d = d; log->rho_dtype = rho_dtype; log->K = capacity;
  log->S = ((N / 2) + kUnitPairs - 1) / kUnitPairs;
  if ((long)B * h * log->S > 0x7fffffffL / 2 || B > 65535) {
    delete log;
    return bdh_fail(ctx, BDH_E_SHAPE, "B*h*N too large");
  }
  size_t om, ov, ol, os;
  log->mem_bytes = log_layout(B, h, N, d, capacity, &om, &ov, &ol, &os);
  hipError_t e = hipMalloc(&log->mem, log->mem_bytes);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    delete log;
    return bdh_fail(ctx, BDH_E_NOMEM, "state log of %zu bytes: %s", log->mem_bytes, hipGetErrorString(e));
  }
  char *m = static_cast<char *>(log->mem);
  log->pmask = reinterpret_cast<ulonglong2 *>(m + om);
  log->pvals = reinterpret_cast<float2 *>(m + ov);
  log->vlog = reinterpret_cast<float *>(m + ol);
  log->scores = reinterpret_cast<float *>(m + os);
  {  // an empty log: no pair has a logged step
    const size_t n = (size_t)B * h * log->S * kUnitPairs * 2;
    hipLaunchKernelGGL(k_fill_zero_u64, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, ctx->stream,
                       reinterpret_cast<unsigned long long *>(log->pmask), n);
    if (hipGetLastError() != hipSuccess) {
      (void)hipFree(log->mem);
      delete log;
      return bdh_fail(ctx, BDH_E_HIP, "launch of k_fill_zero_u64 failed");
    }
  }
  *out = log;
  return BDH_OK;
}

int bdh_state_log_destroy(bdh_ctx *ctx, bdh_state_log *log) {
  if (!log) return BDH_OK;
  if (log->mem) {
    if (ctx) (void)hipStreamSynchronize(ctx->stream);
    (void)hipFree(log->mem);
  }
  delete log;
  return BDH_OK;
}

int bdh_state_log_pending(const bdh_state_log *log) { return log ? log->count : BDH_E_INVAL; }

size_t bdh_state_log_bytes(const bdh_state_log *log) { return log ? log->mem_bytes : 0; }

int bdh_state_step_deferred(bdh_ctx *ctx, bdh_state_log *log, const float *x, const float *v, const float *freqs,
                            int64_t position, const int32_t *positions_dev, void *rho, float *out,
                            uint64_t *active_bitmask, int32_t *rows_touched) {
  if (!ctx) return BDH_E_INVAL;
  if (!log) return bdh_fail(ctx, BDH_E_INVAL, "null state log");
  if (log->device != ctx->device) return bdh_fail(ctx, BDH_E_INVAL, "the state log lives on device %d, the context on %d", log->device, ctx->device);
  if (position < 0) return bdh_fail(ctx, BDH_E_INVAL, "negative position");
  if (!x || !v || !freqs || !rho || !out) return bdh_fail(ctx, BDH_E_INVAL, "null data pointer");
  if (!bdh_aligned(x, 8) || !bdh_aligned(v, 16) || !bdh_aligned(rho, 16) || !bdh_aligned(out, 16) || !bdh_aligned(freqs, 8))
    return bdh_fail(ctx, BDH_E_ALIGN, "x/freqs need 8-byte, v/rho/out 16-byte alignment");
  return bdh_launch_state_step_deferred(ctx, log, x, v, freqs, position, positions_dev, rho, out, nullptr, active_bitmask,
                                        rows_touched);
}

int bdh_state_flush(bdh_ctx *ctx, bdh_state_log *log, void *rho) {
  if (!ctx) return BDH_E_INVAL;
  if (!log) return bdh_fail(ctx, BDH_E_INVAL, "null state log");
  if (log->device != ctx->device) return bdh_fail(ctx, BDH_E_INVAL, "the state log lives on device %d, the context on %d", log->device, ctx->device);
  if (log->count > 0 && (!rho || !bdh_aligned(rho, 16))) return bdh_fail(ctx, BDH_E_INVAL, "rho is null or not 16-byte aligned");
  return bdh_launch_state_flush(ctx, log, rho);
}

}  // extern "C"
