// The recurrent state step of the BDH cached path on gfx950:
//   rotate (RoPE / PoPE / none)  ->  readout with the OLD state  ->  rank-1 update.
// Reference semantics: src/model/bdh.rs:258-307 and src/model/attention.rs:305-349.
//
// Layout in HBM: rho [B,h,Nq,d] row-major; one state row = d contiguous values.  The two
// rows of a RoPE lane pair (2j, 2j+1) are adjacent, so an active pair is one contiguous
// 2*d*sizeof(T) chunk.  A 64-lane wavefront covers one d=256 f32 row with one 16-byte
// load per lane (1 KiB, eight 128-byte segments).
//
// Fast path (RoPE, d in {256,512}): one workgroup owns WAVES*64 lane pairs of one
// (b,h) slice.  Lane l of wave w loads pair w*64+l of x, rotates it, and the wavefront
// ballot gives the 64-bit active-pair mask; popcount prefix sums compact the active pairs
// of the workgroup into an LDS list, which the waves then walk round-robin, U pairs in
// flight per wave.  Every touched byte of rho is read once and written once.  The readout
// is reduced across waves in LDS and written as one partial per workgroup; a second small
// kernel adds the partials in a fixed order (deterministic, no atomics).
#include <hip/hip_bf16.h>

#include <algorithm>
#include <mutex>

#include "bdh_internal.h"
#include "state_common.h"

namespace {

struct HeadScalars {
  float v[64];
};

struct StepPtrs {
  const float *x;        // token t of slice 0
  long x_slice_stride;   // elements between (b,h) slices
  const float *v;        // token t of batch 0
  long v_batch_stride;
  const float *freqs;
  float pos_scalar;             // f32(position + t)
  long pos_int;                 // position + t as an integer (the clock of a lazily decayed state)
  const int32_t *pos_dev;       // optional per-sequence start positions
  int pos_add;                  // t, added to pos_dev[b]
  float *partial;               // [slices, S, d]
  int *pair_cnt;                // [slices, S]
  unsigned long long *bitmask;  // token t of slice 0, or null
  long bitmask_slice_stride;
  int h, N, S;
  // k_step_rope_f32 only: the launch walks nt consecutive tokens (each workgroup owns its state rows, so
  // it can take the tokens one after the other without leaving the kernel); per-token element strides
  int nt = 1;
  long x_t_stride = 0, v_t_stride = 0, partial_t_stride = 0, cnt_t_stride = 0, bm_t_stride = 0;
};

// ------------------------------------------------------------------------------------
// fast path: RoPE, f32 state, D in {256, 512}
// ------------------------------------------------------------------------------------
// SPLIT > 1: the workgroup still has WAVES waves but owns only WAVES*64/SPLIT lane pairs; the
// first WAVES/SPLIT waves compact them and all waves walk the list.  Used when there are few
// (b,h) slices, so that a small batch still spreads over every CU with enough loads in flight.
template <int D, int WAVES, int U, int SPLIT, bool MULTI>
__global__ __launch_bounds__(WAVES * 64) void k_step_rope_f32(StepPtrs a, float *__restrict__ rho) {
  constexpr int VPL = D / 256;             // float4 per lane per row
  constexpr int PPB = WAVES * 64 / SPLIT;  // lane pairs per workgroup
  constexpr int OW = WAVES / SPLIT;        // waves that own pairs
  static_assert(OW >= 1 && OW * SPLIT == WAVES, "SPLIT must divide WAVES");
  __shared__ int s_cnt[OW];
  __shared__ unsigned short s_idx[PPB];
  __shared__ float2 s_q[PPB];
  __shared__ float4 s_red[WAVES][D / 4];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int slice = blockIdx.x / a.S;
  const int seg = blockIdx.x - slice * a.S;
  const int b = slice / a.h;
  const int NP = a.N >> 1;
  const bool owner = wave < OW;
  const int p = seg * PPB + tid;
  float2 fv = make_float2(0.0f, 0.0f);

  // Tokens of this launch, in order.  A workgroup touches only its own state rows and its barriers
  // order the row stores of one token before the row loads of the next.
  const int nt = MULTI ? a.nt : 1;  // the single-token kernel keeps its straight-line code
  for (int t = 0; t < nt; ++t) {
  float2 xv = make_float2(0.0f, 0.0f);
  if (owner && p < NP) {  // one block, so that both loads are in flight together
    xv = reinterpret_cast<const float2 *>(a.x + t * a.x_t_stride + (long)slice * a.x_slice_stride)[p];
    if (t == 0) fv = reinterpret_cast<const float2 *>(a.freqs)[p];
  }
  const float pos = (float)((a.pos_dev ? (long)a.pos_dev[b] + a.pos_add : a.pos_int) + t);

  const bool ae = xv.x != 0.0f, ao = xv.y != 0.0f;
  const bool act = ae || ao;
  const unsigned long long m_act = __ballot(act);

  // element bitmask: two 64-bit words per wave (128 consecutive neurons)
  if (a.bitmask && owner) {
    const unsigned long long me = __ballot(ae), mo = __ballot(ao);
    if (lane == 0) {
      const int w0 = (seg * PPB + wave * 64) >> 5;
      const int NW = (a.N + 63) >> 6;
      unsigned long long *bm = a.bitmask + t * a.bm_t_stride + (long)slice * a.bitmask_slice_stride;
      if (w0 < NW) bm[w0] = spread_bits((unsigned int)me) | (spread_bits((unsigned int)mo) << 1);
      if (w0 + 1 < NW)
        bm[w0 + 1] = spread_bits((unsigned int)(me >> 32)) | (spread_bits((unsigned int)(mo >> 32)) << 1);
    }
  }

  // rotate this lane's pair (src/model/attention.rs:305-321):
  //   q[2j]   = x[2j]  *cos(ph[2j])   + (-x[2j+1])*sin(ph[2j])
  //   q[2j+1] = x[2j+1]*cos(ph[2j+1]) +   x[2j]   *sin(ph[2j+1])
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

  // workgroup-wide compaction of the active pairs
  if (lane == 0 && owner) s_cnt[wave] = __popcll(m_act);
  __syncthreads();
  int offset = 0, total = 0;
#pragma unroll
  for (int w = 0; w < OW; ++w) {
    const int c = s_cnt[w];
    if (w < wave) offset += c;
    total += c;
  }
  if (act) {
    const int rank = offset + __popcll(m_act & ((1ull << lane) - 1ull));
    s_idx[rank] = (unsigned short)tid;
    s_q[rank] = q;
  }
  __syncthreads();

  float4 acc[VPL];
  float4 vv[VPL];
  {
    const float4 *vrow = reinterpret_cast<const float4 *>(a.v + t * a.v_t_stride + (long)b * a.v_batch_stride);
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
      acc[j] = make_float4(0.f, 0.f, 0.f, 0.f);
      vv[j] = vrow[j * 64 + lane];
    }
  }
  float *base = rho + ((long)slice * a.N + 2L * seg * PPB) * D;

  for (int i0 = wave; i0 < total; i0 += WAVES * U) {
    float4 r0[U][VPL], r1[U][VPL];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i = i0 + u * WAVES;
      if (i < total) {
        const float4 *rp = reinterpret_cast<const float4 *>(base + (long)s_idx[i] * (2 * D));
#pragma unroll
        for (int j = 0; j < VPL; ++j) {
          r0[u][j] = rp[j * 64 + lane];
          r1[u][j] = rp[D / 4 + j * 64 + lane];
        }
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i = i0 + u * WAVES;
      if (i < total) {
        const float2 qq = s_q[i];
        float4 *wp = reinterpret_cast<float4 *>(base + (long)s_idx[i] * (2 * D));
#pragma unroll
        for (int j = 0; j < VPL; ++j) {
          float4 e = r0[u][j], o = r1[u][j];
          // readout with the old state (src/model/bdh.rs:293-295)
          acc[j].x = __builtin_fmaf(e.x, qq.x, acc[j].x);
          acc[j].y = __builtin_fmaf(e.y, qq.x, acc[j].y);
          acc[j].z = __builtin_fmaf(e.z, qq.x, acc[j].z);
          acc[j].w = __builtin_fmaf(e.w, qq.x, acc[j].w);
          acc[j].x = __builtin_fmaf(o.x, qq.y, acc[j].x);
          acc[j].y = __builtin_fmaf(o.y, qq.y, acc[j].y);
          acc[j].z = __builtin_fmaf(o.z, qq.y, acc[j].z);
          acc[j].w = __builtin_fmaf(o.w, qq.y, acc[j].w);
          // rank-1 update: rho + (q*v), product rounded before the add (src/model/bdh.rs:298)
          const float4 vj = vv[j];
          float t;
          t = qq.x * vj.x; e.x = e.x + t;
          t = qq.x * vj.y; e.y = e.y + t;
          t = qq.x * vj.z; e.z = e.z + t;
          t = qq.x * vj.w; e.w = e.w + t;
          t = qq.y * vj.x; o.x = o.x + t;
          t = qq.y * vj.y; o.y = o.y + t;
          t = qq.y * vj.z; o.z = o.z + t;
          t = qq.y * vj.w; o.w = o.w + t;
          wp[j * 64 + lane] = e;
          wp[D / 4 + j * 64 + lane] = o;
        }
      }
    }
  }

  // cross-wave reduction of the readout, fixed order
#pragma unroll
  for (int j = 0; j < VPL; ++j) s_red[wave][j * 64 + lane] = acc[j];
  __syncthreads();
  float *pout = a.partial + t * a.partial_t_stride + (long)blockIdx.x * D;
  for (int c4 = tid; c4 < D / 4; c4 += WAVES * 64) {
    float4 s = s_red[0][c4];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) {
      const float4 t = s_red[w][c4];
      s.x += t.x; s.y += t.y; s.z += t.z; s.w += t.w;
    }
    reinterpret_cast<float4 *>(pout)[c4] = s;
  }
  if (tid == 0) a.pair_cnt[t * a.cnt_t_stride + blockIdx.x] = total;
  }  // tokens
}

// ------------------------------------------------------------------------------------
// fast path: ALiBi with a lazily decayed f32 state, D in {256, 512}.  Same shape as the RoPE
// kernel (one workgroup of WAVES waves owns WAVES*128 neurons of one slice, ballot compaction
// into an LDS list, U rows in flight per wave), but the unit is a single state row: ALiBi does
// not rotate, so a neuron's row is touched only when that neuron is active.  The thread that
// owns a neuron also reads its stamp, turns it into the catch-up factor decay^(clock - stamp)
// and writes the new stamp clock + 1.
// ------------------------------------------------------------------------------------
template <int D, int WAVES, int U>
__global__ __launch_bounds__(WAVES * 64) void k_step_alibi_lazy_f32(StepPtrs a, float *__restrict__ rho,
                                                                   int32_t *__restrict__ stamps, HeadScalars decay,
                                                                   HeadScalars log_decay) {
  constexpr int VPL = D / 256;
  constexpr int RPB = WAVES * 128;  // state rows (neurons) per workgroup
  __shared__ int s_cnt[2][WAVES];
  __shared__ unsigned short s_idx[RPB];
  __shared__ float2 s_qs[RPB];  // (activation, catch-up factor)
  __shared__ float4 s_red[WAVES][D / 4];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int slice = blockIdx.x / a.S;
  const int seg = blockIdx.x - slice * a.S;
  const int b = slice / a.h, hh = slice - b * a.h;
  const int p = seg * (RPB / 2) + tid;  // this thread owns neurons 2p and 2p+1
  const long clock = a.pos_dev ? (long)a.pos_dev[b] + a.pos_add : a.pos_int;
  const float dec = decay.v[hh], ld = log_decay.v[hh];

  float2 xv = make_float2(0.0f, 0.0f);
  if (2 * p + 1 < a.N) {
    xv = reinterpret_cast<const float2 *>(a.x + (long)slice * a.x_slice_stride)[p];
  } else if (2 * p < a.N) {
    xv.x = a.x[(long)slice * a.x_slice_stride + 2 * p];
  }
  const bool ae = xv.x != 0.0f, ao = xv.y != 0.0f;
  const unsigned long long me = __ballot(ae), mo = __ballot(ao);
  if (a.bitmask && lane == 0) {
    const int w0 = (seg * RPB + wave * 128) >> 6;
    const int NW = (a.N + 63) >> 6;
    unsigned long long *bm = a.bitmask + (long)slice * a.bitmask_slice_stride;
    if (w0 < NW) bm[w0] = spread_bits((unsigned int)me) | (spread_bits((unsigned int)mo) << 1);
    if (w0 + 1 < NW) bm[w0 + 1] = spread_bits((unsigned int)(me >> 32)) | (spread_bits((unsigned int)(mo >> 32)) << 1);
  }
  float se = 1.0f, so = 1.0f;
  {
    int32_t *st = stamps + (long)slice * a.N;
    const int32_t next = (int32_t)min(clock + 1, 0x7fffffffL);
    if (ae) {
      const long k = clock - (long)st[2 * p];
      if (k > 0) se = expf((float)k * ld);
      st[2 * p] = next;
    }
    if (ao) {
      const long k = clock - (long)st[2 * p + 1];
      if (k > 0) so = expf((float)k * ld);
      st[2 * p + 1] = next;
    }
  }
  if (lane == 0) {
    s_cnt[0][wave] = __popcll(me);
    s_cnt[1][wave] = __popcll(mo);
  }
  __syncthreads();
  int off_e = 0, off_o = 0, total_e = 0, total = 0;
#pragma unroll
  for (int w = 0; w < WAVES; ++w) {
    const int ce = s_cnt[0][w], co = s_cnt[1][w];
    if (w < wave) {
      off_e += ce;
      off_o += co;
    }
    total_e += ce;
    total += ce + co;
  }
  const unsigned long long below = (1ull << lane) - 1ull;
  if (ae) {
    const int rank = off_e + __popcll(me & below);
    s_idx[rank] = (unsigned short)(2 * tid);
    s_qs[rank] = make_float2(xv.x, se);
  }
  if (ao) {
    const int rank = total_e + off_o + __popcll(mo & below);
    s_idx[rank] = (unsigned short)(2 * tid + 1);
    s_qs[rank] = make_float2(xv.y, so);
  }
  __syncthreads();

  float4 acc[VPL], vv[VPL];
  {
    const float4 *vrow = reinterpret_cast<const float4 *>(a.v + (long)b * a.v_batch_stride);
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
      acc[j] = make_float4(0.f, 0.f, 0.f, 0.f);
      vv[j] = vrow[j * 64 + lane];
    }
  }
  float *base = rho + ((long)slice * a.N + (long)seg * RPB) * D;
  for (int i0 = wave; i0 < total; i0 += WAVES * U) {
    float4 r[U][VPL];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i = i0 + u * WAVES;
      if (i < total) {
        const float4 *rp = reinterpret_cast<const float4 *>(base + (long)s_idx[i] * D);
#pragma unroll
        for (int j = 0; j < VPL; ++j) r[u][j] = rp[j * 64 + lane];
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i = i0 + u * WAVES;
      if (i < total) {
        const float2 qs = s_qs[i];
        float4 *wp = reinterpret_cast<float4 *>(base + (long)s_idx[i] * D);
#pragma unroll
        for (int j = 0; j < VPL; ++j) {
          float4 e = r[u][j];
          e.x = e.x * qs.y; e.y = e.y * qs.y; e.z = e.z * qs.y; e.w = e.w * qs.y;  // pending decay
          acc[j].x = __builtin_fmaf(e.x, qs.x, acc[j].x);  // readout with the old row (src/model/bdh.rs:293-295)
          acc[j].y = __builtin_fmaf(e.y, qs.x, acc[j].y);
          acc[j].z = __builtin_fmaf(e.z, qs.x, acc[j].z);
          acc[j].w = __builtin_fmaf(e.w, qs.x, acc[j].w);
          const float4 vj = vv[j];
          float t;
          t = qs.x * vj.x; e.x = (e.x + t) * dec;  // update (:298), then this token's decay (:299-301)
          t = qs.x * vj.y; e.y = (e.y + t) * dec;
          t = qs.x * vj.z; e.z = (e.z + t) * dec;
          t = qs.x * vj.w; e.w = (e.w + t) * dec;
          wp[j * 64 + lane] = e;
        }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < VPL; ++j) s_red[wave][j * 64 + lane] = acc[j];
  __syncthreads();
  float *pout = a.partial + (long)blockIdx.x * D;
  for (int c4 = tid; c4 < D / 4; c4 += WAVES * 64) {
    float4 sum = s_red[0][c4];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) {
      const float4 t = s_red[w][c4];
      sum.x += t.x; sum.y += t.y; sum.z += t.z; sum.w += t.w;
    }
    reinterpret_cast<float4 *>(pout)[c4] = sum;
  }
  if (tid == 0) a.pair_cnt[blockIdx.x] = total;
}

// ------------------------------------------------------------------------------------
// fast path: RoPE, bf16 state (f32 accumulate), D in {256, 512}.  A lane pair's two rows are
// 4*D contiguous bytes; each lane owns D/256 16-byte pieces (8 bf16) of that chunk.
// ------------------------------------------------------------------------------------
template <int D, int WAVES, int U, int SPLIT>
__global__ __launch_bounds__(WAVES * 64) void k_step_rope_bf16(StepPtrs a, unsigned short *__restrict__ rho) {
  constexpr int PL = D / 256;      // 16-byte pieces per lane per pair (D=256: 1, D=512: 2)
  constexpr int PPB = WAVES * 64 / SPLIT;
  constexpr int OW = WAVES / SPLIT;
  static_assert(OW >= 1 && OW * SPLIT == WAVES, "SPLIT must divide WAVES");
  __shared__ int s_cnt[OW];
  __shared__ unsigned short s_idx[PPB];
  __shared__ float2 s_q[PPB];
  __shared__ float s_red[WAVES][2][D];  // per wave, per row of the pair

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int slice = blockIdx.x / a.S;
  const int seg = blockIdx.x - slice * a.S;
  const int b = slice / a.h;
  const int NP = a.N >> 1;
  const bool owner = wave < OW;
  const int p = seg * PPB + tid;

  float2 xv = make_float2(0.0f, 0.0f), fv = make_float2(0.0f, 0.0f);
  if (owner && p < NP) {
    xv = reinterpret_cast<const float2 *>(a.x + (long)slice * a.x_slice_stride)[p];
    fv = reinterpret_cast<const float2 *>(a.freqs)[p];
  }
  const float pos = a.pos_dev ? (float)((long)a.pos_dev[b] + a.pos_add) : a.pos_scalar;
  const bool ae = xv.x != 0.0f, ao = xv.y != 0.0f;
  const bool act = ae || ao;
  const unsigned long long m_act = __ballot(act);
  if (a.bitmask && owner) {
    const unsigned long long me = __ballot(ae), mo = __ballot(ao);
    if (lane == 0) {
      const int w0 = (seg * PPB + wave * 64) >> 5;
      const int NW = (a.N + 63) >> 6;
      unsigned long long *bm = a.bitmask + (long)slice * a.bitmask_slice_stride;
      if (w0 < NW) bm[w0] = spread_bits((unsigned int)me) | (spread_bits((unsigned int)mo) << 1);
      if (w0 + 1 < NW)
        bm[w0 + 1] = spread_bits((unsigned int)(me >> 32)) | (spread_bits((unsigned int)(mo >> 32)) << 1);
    }
  }
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
  if (lane == 0 && owner) s_cnt[wave] = __popcll(m_act);
  __syncthreads();
  int offset = 0, total = 0;
#pragma unroll
  for (int w = 0; w < OW; ++w) {
    const int c = s_cnt[w];
    if (w < wave) offset += c;
    total += c;
  }
  if (act) {
    const int rank = offset + __popcll(m_act & ((1ull << lane) - 1ull));
    s_idx[rank] = (unsigned short)tid;
    s_q[rank] = q;
  }
  __syncthreads();

  // piece j of this lane covers elements e0 = (j*64 + lane)*8 .. +7 of the 2*D-element pair chunk
  int prow[PL], pcol[PL];
  float vv[PL][8], acc[PL][8];
  const float *vrow = a.v + (long)b * a.v_batch_stride;
#pragma unroll
  for (int j = 0; j < PL; ++j) {
    const int e0 = (j * 64 + lane) * 8;
    prow[j] = e0 / D;
    pcol[j] = e0 - prow[j] * D;
    const float4 v0 = *reinterpret_cast<const float4 *>(vrow + pcol[j]);
    const float4 v1 = *reinterpret_cast<const float4 *>(vrow + pcol[j] + 4);
    vv[j][0] = v0.x; vv[j][1] = v0.y; vv[j][2] = v0.z; vv[j][3] = v0.w;
    vv[j][4] = v1.x; vv[j][5] = v1.y; vv[j][6] = v1.z; vv[j][7] = v1.w;
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[j][e] = 0.0f;
  }
  unsigned short *base = rho + ((long)slice * a.N + 2L * seg * PPB) * D;

  for (int i0 = wave; i0 < total; i0 += WAVES * U) {
    uint4 r[U][PL];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i = i0 + u * WAVES;
      if (i < total) {
        const uint4 *rp = reinterpret_cast<const uint4 *>(base + (long)s_idx[i] * (2 * D));
#pragma unroll
        for (int j = 0; j < PL; ++j) r[u][j] = rp[j * 64 + lane];
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i = i0 + u * WAVES;
      if (i < total) {
        const float2 qq = s_q[i];
        uint4 *wp = reinterpret_cast<uint4 *>(base + (long)s_idx[i] * (2 * D));
#pragma unroll
        for (int j = 0; j < PL; ++j) {
          const float qf = prow[j] ? qq.y : qq.x;
          const unsigned int w[4] = {r[u][j].x, r[u][j].y, r[u][j].z, r[u][j].w};
          unsigned int o[4];
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            float lo = __uint_as_float(w[k] << 16), hi = __uint_as_float(w[k] & 0xffff0000u);
            acc[j][2 * k] = __builtin_fmaf(lo, qf, acc[j][2 * k]);
            acc[j][2 * k + 1] = __builtin_fmaf(hi, qf, acc[j][2 * k + 1]);
            const float t0 = qf * vv[j][2 * k], t1 = qf * vv[j][2 * k + 1];
            lo = lo + t0;
            hi = hi + t1;
            o[k] = pack_bf16_rne(lo, hi);
          }
          wp[j * 64 + lane] = make_uint4(o[0], o[1], o[2], o[3]);
        }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < PL; ++j) {
    // D=256: both rows are covered by one piece (lanes 0-31 row 0, 32-63 row 1);
    // D=512: piece 0 is row 0, piece 1 is row 1.
    float *dst = &s_red[wave][prow[j]][pcol[j]];
#pragma unroll
    for (int e = 0; e < 8; ++e) dst[e] = acc[j][e];
  }
  __syncthreads();
  float *pout = a.partial + (long)blockIdx.x * D;
  for (int c = tid; c < D; c += WAVES * 64) {
    float s = 0.0f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) s += s_red[w][0][c] + s_red[w][1][c];
    pout[c] = s;
  }
  if (tid == 0) a.pair_cnt[blockIdx.x] = total;
}

// ------------------------------------------------------------------------------------
// generic path: any d <= 1024, any rotary, f32 or bf16 state.  One workgroup owns ROWS
// state rows of one slice; waves take rows round-robin, lanes stride over columns.
// ------------------------------------------------------------------------------------
constexpr int kGenRows = 64;
constexpr int kGenMaxCols = 16;  // d <= 64 * 16

template <typename RhoT>
__device__ __forceinline__ float rho_load(const RhoT *p);
template <>
__device__ __forceinline__ float rho_load<float>(const float *p) { return *p; }
template <>
__device__ __forceinline__ float rho_load<unsigned short>(const unsigned short *p) { return bf16_to_f32(*p); }
__device__ __forceinline__ void rho_store(float *p, float v) { *p = v; }
__device__ __forceinline__ void rho_store(unsigned short *p, float v) { *p = f32_to_bf16(v); }

// Per state row (all d columns) of the generic path: readout with the old row, rank-1 update, optional
// decay; a lazily decayed row is brought up to date first.
// stamps != nullptr (ALiBi only): the state is kept lazily decayed.  Row n of a slice holds the
// value it had when the sequence had absorbed stamps[n] tokens; its current value is that times
// decay^(clock - stamps[n]).  Only rows with a non-zero activation are read, brought up to date,
// updated, decayed once (src/model/bdh.rs:299-301) and stamped clock+1; all other rows are left
// alone, so the step stays as sparse as the activations.
template <typename RhoT, int MAXC, int FL>  // d <= 64 * MAXC; FL state rows in flight per wave
__global__ __launch_bounds__(256) void k_step_generic(StepPtrs a, RhoT *__restrict__ rho, int d, int Nq,
                                                      int rotary, int has_decay, HeadScalars decay,
                                                      HeadScalars log_decay, int32_t *__restrict__ stamps) {
  __shared__ float s_red[4][64 * MAXC];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int slice = blockIdx.x / a.S;
  const int seg = blockIdx.x - slice * a.S;
  const int b = slice / a.h, hh = slice - b * a.h;
  const float dec = has_decay ? decay.v[hh] : 1.0f;
  const int ncol = (d + 63) >> 6;

  // Lane l < 16 prepares row wave + 4l of this segment: its query value, whether the row is visited and,
  // for a lazily decayed state, the factor that brings it up to date.  The ballot lists the rows to visit;
  // they are then walked in index order, FL rows in flight at a time.
  const bool lazy = rotary == BDH_ALIBI && stamps != nullptr;
  const long clock0 = a.pos_dev ? (long)a.pos_dev[b] + a.pos_add : a.pos_int;
  int32_t *st = lazy ? stamps + (long)slice * Nq : nullptr;
  const int n_l = seg * kGenRows + wave + 4 * lane;
  const bool in_range = lane < kGenRows / 4 && n_l < Nq;
  // the stamp of this lane's row lives in a register over the tokens of the launch
  long stamp_l = (lazy && in_range) ? (long)st[n_l] : 0;
  bool stamp_dirty = false;

  // Tokens of this launch, in order.  A workgroup touches only its own state rows, and the barriers of a
  // token order its row stores before the row loads of the next.
  for (int t = 0; t < a.nt; ++t) {
  const long clock = clock0 + t;
  const float pos = (float)clock;
  const float *xs = a.x + (long)t * a.x_t_stride + (long)slice * a.x_slice_stride;
  const float *vrow = a.v + (long)t * a.v_t_stride + (long)b * a.v_batch_stride;
  float acc[MAXC];
#pragma unroll
  for (int j = 0; j < MAXC; ++j) acc[j] = 0.0f;
  float q_l = 0.0f, scale_l = 1.0f;
  bool touch_l = false;
  if (in_range) {
    if (rotary == BDH_ALIBI) {
      // q = x (src/model/attention.rs:332-349: ALiBi does not rotate)
      q_l = xs[n_l];
      touch_l = lazy ? (q_l != 0.0f) : true;
      if (lazy && touch_l) {
        const long k = clock - stamp_l;
        if (k > 0) scale_l = expf((float)k * log_decay.v[hh]);
      }
    } else if (rotary == BDH_ROPE) {
      const float xn = xs[n_l], xo = xs[n_l ^ 1];
      touch_l = (xn != 0.0f) || (xo != 0.0f);
      float sn, cs;
      sincosf(rope_phase(pos, a.freqs[n_l]), &sn, &cs);
      const float rot = (n_l & 1) ? xo : -xo;
      const float t0 = xn * cs, t1 = rot * sn;
      q_l = t0 + t1;
    } else {
      const int m = n_l < a.N ? n_l : n_l - a.N;
      const float mag = softplus1(xs[m]);
      const float ph = rope_phase(pos, a.freqs[m]);
      q_l = n_l < a.N ? mag * cosf(ph) : mag * sinf(ph);
      touch_l = true;
    }
  }
  const bool has_dec = rotary == BDH_ALIBI;  // src/model/bdh.rs:299-301
  float vv[MAXC];
#pragma unroll
  for (int j = 0; j < MAXC; ++j) {
    const int c = j * 64 + lane;
    vv[j] = (j < ncol && c < d) ? vrow[c] : 0.0f;
  }
  unsigned long long m = __ballot(touch_l);
  while (m) {
    int ls[FL];
    bool ok[FL];
    float rv[FL][MAXC];
#pragma unroll
    for (int u = 0; u < FL; ++u) {
      ok[u] = m != 0ull;
      ls[u] = ok[u] ? __builtin_ctzll(m) : 0;
      if (ok[u]) m &= m - 1;
    }
#pragma unroll
    for (int u = 0; u < FL; ++u) {
      if (ok[u]) {
        const RhoT *row = rho + ((long)slice * Nq + seg * kGenRows + wave + 4 * ls[u]) * d;
#pragma unroll
        for (int j = 0; j < MAXC; ++j) {
          const int c = j * 64 + lane;
          if (j < ncol && c < d) rv[u][j] = rho_load<RhoT>(row + c);
        }
      }
    }
#pragma unroll
    for (int u = 0; u < FL; ++u) {
      const int lu = __builtin_amdgcn_readfirstlane(ls[u]);  // the row list is the same in every lane
            const float qn = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(q_l), lu));
      const float scale = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(scale_l), lu));
      if (ok[u]) {
        RhoT *row = rho + ((long)slice * Nq + seg * kGenRows + wave + 4 * ls[u]) * d;
#pragma unroll
        for (int j = 0; j < MAXC; ++j) {
          const int c = j * 64 + lane;
          if (j < ncol && c < d) {
            float r = rv[u][j];
            if (lazy) r = r * scale;
            acc[j] = __builtin_fmaf(r, qn, acc[j]);
            const float outer = qn * vv[j];
            r = r + outer;
            if (has_dec) r = r * dec;
            rho_store(row + c, r);
          }
        }
      }
    }
  }
  if (lazy && touch_l) {
    stamp_l = min(clock + 1, 0x7fffffffL);
    stamp_dirty = true;
  }
#pragma unroll
  for (int j = 0; j < MAXC; ++j) s_red[wave][j * 64 + lane] = acc[j];
  __syncthreads();
  float *pout = a.partial + (long)t * a.partial_t_stride + (long)blockIdx.x * d;
  for (int c = tid; c < d; c += 256) {
    float s = s_red[0][c];
    s += s_red[1][c];
    s += s_red[2][c];
    s += s_red[3][c];
    pout[c] = s;
  }
  __syncthreads();  // s_red is written again by the next token
  }
  if (stamp_dirty) st[n_l] = (int32_t)stamp_l;
}

// ------------------------------------------------------------------------------------
// dense path, D in {256, 512}: PoPE (2N rows) and ALiBi with the eager decay touch every state row on
// every token, so the step is a streaming read-modify-write of the whole slice.  Same work split and
// the same order of operations per element as k_step_generic (a workgroup owns 64 rows, wave w takes
// rows w, w+4, ...), but a lane owns four adjacent columns (one 16-byte access per row) and U rows are
// in flight per wave.
// ------------------------------------------------------------------------------------
__device__ __forceinline__ float4 dense_load4(const float *p) { return *reinterpret_cast<const float4 *>(p); }
__device__ __forceinline__ float4 dense_load4(const unsigned short *p) {
  const uint2 v = *reinterpret_cast<const uint2 *>(p);
  return make_float4(__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u), __uint_as_float(v.y << 16),
                     __uint_as_float(v.y & 0xffff0000u));
}
__device__ __forceinline__ void dense_store4(float *p, float4 v) { *reinterpret_cast<float4 *>(p) = v; }
__device__ __forceinline__ void dense_store4(unsigned short *p, float4 v) {
  uint2 o;
  o.x = (unsigned int)f32_to_bf16(v.x) | ((unsigned int)f32_to_bf16(v.y) << 16);
  o.y = (unsigned int)f32_to_bf16(v.z) | ((unsigned int)f32_to_bf16(v.w) << 16);
  *reinterpret_cast<uint2 *>(p) = o;
}

template <typename RhoT, int D, int U>
__global__ __launch_bounds__(256) void k_step_dense(StepPtrs a, RhoT *__restrict__ rho, int Nq, int rotary,
                                                    HeadScalars decay) {
  constexpr int VPL = D / 256;  // groups of four columns per lane
  __shared__ float4 s_red[4][D / 4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int slice = blockIdx.x / a.S;
  const int seg = blockIdx.x - slice * a.S;
  const int b = slice / a.h, hh = slice - b * a.h;
  const long clock0 = a.pos_dev ? (long)a.pos_dev[b] + a.pos_add : a.pos_int;
  const bool has_decay = rotary == BDH_ALIBI;
  const float dec = has_decay ? decay.v[hh] : 1.0f;

  // Tokens of this launch, in order.  A workgroup touches only its own state rows, and the barriers of a
  // token order its row stores before the row loads of the next.
  for (int t = 0; t < a.nt; ++t) {
  const float pos = (float)(clock0 + t);
  const float *xs = a.x + (long)t * a.x_t_stride + (long)slice * a.x_slice_stride;
  float4 acc[VPL], vv[VPL];
  {
    const float4 *vrow = reinterpret_cast<const float4 *>(a.v + (long)t * a.v_t_stride + (long)b * a.v_batch_stride);
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
      acc[j] = make_float4(0.f, 0.f, 0.f, 0.f);
      vv[j] = vrow[j * 64 + lane];
    }
  }
  RhoT *base = rho + ((long)slice * Nq + (long)seg * kGenRows) * D;
  for (int r0 = wave; r0 < kGenRows; r0 += 4 * U) {
    float4 rv[U][VPL];
    float qn[U];
    bool ok[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int r = r0 + 4 * u;
      ok[u] = r < kGenRows && seg * kGenRows + r < Nq;
      if (ok[u]) {
#pragma unroll
        for (int j = 0; j < VPL; ++j) rv[u][j] = dense_load4(base + (long)r * D + (j * 64 + lane) * 4);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      qn[u] = 0.0f;
      if (ok[u]) {
        const int n = seg * kGenRows + r0 + 4 * u;
        if (rotary == BDH_ALIBI) {
          qn[u] = xs[n];  // ALiBi does not rotate (src/model/attention.rs:333-335)
        } else {          // PoPE (src/model/attention.rs:323-330): rows N..2N-1 are the imaginary parts
          const int m = n < a.N ? n : n - a.N;
          const float mag = softplus1(xs[m]);
          const float ph = rope_phase(pos, a.freqs[m]);
          qn[u] = n < a.N ? mag * cosf(ph) : mag * sinf(ph);
        }
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (ok[u]) {
        const float q = qn[u];
        RhoT *row = base + (long)(r0 + 4 * u) * D;
#pragma unroll
        for (int j = 0; j < VPL; ++j) {
          float4 e = rv[u][j];
          // readout with the old state (src/model/bdh.rs:293-295), update with the product rounded
          // before the add (:298), ALiBi decay after the update (:299-301)
          acc[j].x = __builtin_fmaf(e.x, q, acc[j].x);
          acc[j].y = __builtin_fmaf(e.y, q, acc[j].y);
          acc[j].z = __builtin_fmaf(e.z, q, acc[j].z);
          acc[j].w = __builtin_fmaf(e.w, q, acc[j].w);
          float t;
          t = q * vv[j].x; e.x = e.x + t;
          t = q * vv[j].y; e.y = e.y + t;
          t = q * vv[j].z; e.z = e.z + t;
          t = q * vv[j].w; e.w = e.w + t;
          if (has_decay) {
            e.x = e.x * dec; e.y = e.y * dec; e.z = e.z * dec; e.w = e.w * dec;
          }
          dense_store4(row + (j * 64 + lane) * 4, e);
        }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < VPL; ++j) s_red[wave][j * 64 + lane] = acc[j];
  __syncthreads();
  float *pout = a.partial + (long)t * a.partial_t_stride + (long)blockIdx.x * D;
  for (int c4 = tid; c4 < D / 4; c4 += 256) {
    float4 s = s_red[0][c4];
#pragma unroll
    for (int w = 1; w < 4; ++w) {
      const float4 p4 = s_red[w][c4];
      s.x += p4.x; s.y += p4.y; s.z += p4.z; s.w += p4.w;
    }
    reinterpret_cast<float4 *>(pout)[c4] = s;
  }
  __syncthreads();  // s_red is written again by the next token
  }
}

// Brings every row of a lazily decayed ALiBi state up to date: row *= decay^(clock - stamp),
// stamp = clock.  Afterwards rho is the state the reference would hold.
template <typename RhoT>
__global__ __launch_bounds__(256) void k_alibi_materialize(RhoT *__restrict__ rho, int32_t *__restrict__ stamps, int h,
                                                           int N, int d, long total_rows, long clock_scalar,
                                                           const int32_t *__restrict__ clocks_dev,
                                                           HeadScalars log_decay) {
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);  // one wave per state row
  const int lane = threadIdx.x & 63;
  if (row >= total_rows) return;
  const long slice = row / N;
  const int b = (int)(slice / h), hh = (int)(slice - (long)b * h);
  const long clock = clocks_dev ? (long)clocks_dev[b] : clock_scalar;
  const long k = clock - (long)stamps[row];
  if (k > 0) {
    const float scale = expf((float)k * log_decay.v[hh]);
    RhoT *p = rho + row * d;
    if ((d & 3) == 0) {  // rows start on 16-byte (f32) / 8-byte (bf16) boundaries: four elements per access
      for (int c = lane * 4; c < d; c += 256) {
        float4 e = dense_load4(p + c);
        e.x = e.x * scale; e.y = e.y * scale; e.z = e.z * scale; e.w = e.w * scale;
        dense_store4(p + c, e);
      }
    } else {
      for (int c = lane; c < d; c += 64) rho_store(p + c, rho_load<RhoT>(p + c) * scale);
    }
  }
  if (lane == 0) stamps[row] = (int32_t)min(clock, 0x7fffffffL);
}

// bitmask + touched-row count for the generic path: one workgroup per slice
__global__ __launch_bounds__(256) void k_bitmask_rows(StepPtrs a, int rotary, int Nq, int *__restrict__ rows,
                                                      long rows_slice_stride, int lazy) {
  __shared__ int s_pairs[4], s_elems[4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int slice = blockIdx.x;
  const float *xs = a.x + (long)slice * a.x_slice_stride;
  const int NW = (a.N + 63) >> 6;
  int pairs = 0, elems = 0;
  for (int w = wave; w < NW; w += 4) {
    const int n = w * 64 + lane;
    const float xv = n < a.N ? xs[n] : 0.0f;
    const unsigned long long m = __ballot(xv != 0.0f);
    if (a.bitmask && lane == 0) a.bitmask[(long)slice * a.bitmask_slice_stride + w] = m;
    const unsigned long long pm = (m | (m >> 1)) & 0x5555555555555555ull;
    pairs += __popcll(pm);
    elems += __popcll(m);
  }
  if (lane == 0) {
    s_pairs[wave] = pairs;
    s_elems[wave] = elems;
  }
  __syncthreads();
  if (tid == 0 && rows) {
    const int np = s_pairs[0] + s_pairs[1] + s_pairs[2] + s_pairs[3];
    const int ne = s_elems[0] + s_elems[1] + s_elems[2] + s_elems[3];
    rows[(long)slice * rows_slice_stride] = rotary == BDH_ROPE ? 2 * np : (lazy ? ne : Nq);
  }
}

// ------------------------------------------------------------------------------------
// second stage: out[slice,:] = sum over the S partials in index order; optional
// LayerNorm of the result (src/model/bdh.rs:359) and touched-row count.
// ------------------------------------------------------------------------------------
template <bool LN>
__global__ __launch_bounds__(256) void k_step_finalize(const float *__restrict__ partial,
                                                       const int *__restrict__ pair_cnt, int S, int d,
                                                       float *__restrict__ out, long out_slice_stride,
                                                       float *__restrict__ out_ln, int *__restrict__ rows,
                                                       long rows_slice_stride, int rows_per_count,
                                                       long partial_t_stride, long cnt_t_stride) {
  const int tid = threadIdx.x;
  const int slice = blockIdx.x;
  // blockIdx.y = token of a multi-token launch: partials and counts advance by their per-token
  // strides, the outputs by one row of d (tokens are adjacent in out [slices, T, d] and rows [slices, T])
  partial += blockIdx.y * partial_t_stride;
  if (pair_cnt) pair_cnt += blockIdx.y * cnt_t_stride;
  out += (long)blockIdx.y * d;
  if (LN) out_ln += (long)blockIdx.y * d;
  if (rows) rows += blockIdx.y;
  const float *p = partial + (long)slice * S * d;
  float vals[4];  // d <= 1024
  float lsum = 0.0f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int c = j * 256 + tid;
    float s = 0.0f;
    if (c < d) {
#pragma unroll 16
      for (int g = 0; g < S; ++g) s += p[(long)g * d + c];
      out[(long)slice * out_slice_stride + c] = s;
      lsum += s;
    }
    vals[j] = s;
  }
  if (rows && pair_cnt && tid == 0) {
    int np = 0;
#pragma unroll 16
    for (int g = 0; g < S; ++g) np += pair_cnt[(long)slice * S + g];
    rows[(long)slice * rows_slice_stride] = rows_per_count * np;
  }
  if (!LN) return;
  // LayerNorm over d: mean, biased variance, (x-mean)/sqrt(var+eps)
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
  for (int j = 0; j < 4; ++j) {
    const int c = j * 256 + tid;
    if (c < d) {
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
  for (int j = 0; j < 4; ++j) {
    const int c = j * 256 + tid;
    if (c < d) out_ln[(long)slice * out_slice_stride + c] = (vals[j] - mean) / den;
  }
}

void launch_finalize(hipStream_t st, int slices, const float *partial, const int *pair_cnt, int S, int d, float *out,
                     long out_stride, float *out_ln, int *rows, long rows_stride, int rows_per_count = 2, int nt = 1,
                     long partial_t_stride = 0, long cnt_t_stride = 0) {
  if (out_ln)
    hipLaunchKernelGGL(k_step_finalize<true>, dim3(slices, nt), dim3(256), 0, st, partial, pair_cnt, S, d, out,
                       out_stride, out_ln, rows, rows_stride, rows_per_count, partial_t_stride, cnt_t_stride);
  else
    hipLaunchKernelGGL(k_step_finalize<false>, dim3(slices, nt), dim3(256), 0, st, partial, pair_cnt, S, d, out,
                       out_stride, out_ln, rows, rows_stride, rows_per_count, partial_t_stride, cnt_t_stride);
}

__global__ __launch_bounds__(256) void k_fill_zero_u32(uint32_t *__restrict__ p, size_t n) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = 0u;
}

template <int D, int WAVES, int U, int SPLIT>
void launch_fast(hipStream_t st, int blocks, const StepPtrs &a, float *rho) {
  if (a.nt > 1)
    hipLaunchKernelGGL((k_step_rope_f32<D, WAVES, U, SPLIT, true>), dim3(blocks), dim3(WAVES * 64), 0, st, a, rho);
  else
    hipLaunchKernelGGL((k_step_rope_f32<D, WAVES, U, SPLIT, false>), dim3(blocks), dim3(WAVES * 64), 0, st, a, rho);
}

}  // namespace

// ------------------------------------------------------------------------------------
// Scratch of the allocation-free decode step (bdh_state_step_noalloc): the readout partials
// [slices, S, d] and the per-workgroup pair counts live in this array instead of the context's
// growable workspace.  Every device the library runs on holds its own copy at its own address
// until the process ends; the address is resolved once per device, with that device current,
// and only that address (never the array's name) is handed to kernels.
// ------------------------------------------------------------------------------------
constexpr size_t kStepScratchBytes = (size_t(32) << 20) + (size_t(256) << 10);
static __device__ __align__(256) unsigned char scratch[kStepScratchBytes];
constexpr int kStepScratchDevices = 64;
static void *g_step_scratch[kStepScratchDevices];
static std::mutex g_step_scratch_mutex;

size_t bdh_step_scratch_bytes() { return kStepScratchBytes; }

int bdh_step_scratch_resolve(bdh_ctx *ctx) {
  if (ctx->device < 0 || ctx->device >= kStepScratchDevices) return BDH_OK;  // such a device has no allocation-free step
  std::lock_guard<std::mutex> lock(g_step_scratch_mutex);
  if (g_step_scratch[ctx->device]) return BDH_OK;
  void *ptr = nullptr;
  BDH_HIP_CHECK(ctx, hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
  if (!ptr) return bdh_fail(ctx, BDH_E_HIP, "hipGetSymbolAddress gave a null scratch address");
  g_step_scratch[ctx->device] = ptr;
  return BDH_OK;
}

void *bdh_step_scratch_ptr(const bdh_ctx *ctx) {
  if (ctx->device < 0 || ctx->device >= kStepScratchDevices) return nullptr;
  std::lock_guard<std::mutex> lock(g_step_scratch_mutex);
  return g_step_scratch[ctx->device];
}

int bdh_launch_state_steps_ln(bdh_ctx *ctx, const StateStepParams &p, float *out_ln) {
  return bdh_launch_state_steps_in(ctx, p, out_ln, nullptr, 0);
}

// fixed != nullptr: partials and counts go to that buffer of fixed_bytes instead of the context's workspace,
// and nothing is allocated (the call fails when they do not fit)
int bdh_launch_state_steps_in(bdh_ctx *ctx, const StateStepParams &p, float *out_ln, void *fixed, size_t fixed_bytes) {
  const int B = p.B, h = p.h, T = p.T, N = p.N, d = p.d;
  const int Nq = p.rotary == BDH_POPE ? 2 * N : N;
  const int slices = B * h;
  if (d > 64 * kGenMaxCols) return bdh_fail(ctx, BDH_E_SHAPE, "d=%d exceeds the supported maximum %d", d, 64 * kGenMaxCols);
  if (N > 65536 * 2 && p.rotary == BDH_ROPE) { /* pair index within a workgroup is 16 bit: always fits */ }
  if ((long)slices > 0x7fffffffL / 4096) return bdh_fail(ctx, BDH_E_SHAPE, "B*h too large");

  const bool fast = p.rotary == BDH_ROPE && (d == 256 || d == 512) && N >= 2;
  if (p.partials_out && (!fast || T != 1 || fixed || p.bitmask || p.rows_touched))
    return bdh_fail(ctx, BDH_E_UNSUPPORTED, "readout partials are only handed over by a single-token RoPE step at d in {256, 512}");
  // few slices (small batch): 64 pairs per workgroup of 8 waves, so the grid still covers the chip
  const int n_cu = ctx->n_cu > 0 ? ctx->n_cu : 256;
  const bool split = fast && (ctx->opt_step_split >= 0 ? ctx->opt_step_split == 1
                                                       : (long)slices * (((N / 2) + 255) / 256) < 2L * n_cu);
  const int ppb = split ? 64 : 256;
  // lazily decayed ALiBi state, f32, d in {256,512}: row-compaction kernel, 512 neurons per workgroup
  const bool fast_lazy = p.rotary == BDH_ALIBI && p.stamps && p.rho_dtype == BDH_F32 && (d == 256 || d == 512) &&
                         (N % 2 == 0);  // the kernel reads x two neurons at a time
  // PoPE, and ALiBi with the eager decay, at d in {256,512}: the dense streaming kernel (the generic kernel's split)
  const bool fast_dense = !fast && !fast_lazy && (d == 256 || d == 512) && ctx->opt_step_dense_kernel != 0 &&
                          (p.rotary == BDH_POPE || (p.rotary == BDH_ALIBI && !p.stamps));
  const int S = fast ? ((N / 2) + ppb - 1) / ppb : fast_lazy ? (N + 511) / 512 : (Nq + kGenRows - 1) / kGenRows;
  if (N == 0 || d == 0) {
    // nothing to read or update: the readout is an empty sum
    // cleared by a kernel, not a memset node, so that a caller may capture this call in a HIP graph
    if (out_ln && d > 0) return bdh_fail(ctx, BDH_E_SHAPE, "LayerNorm of an empty readout");
    const size_t n_out = (size_t)slices * T * d, n_rows = p.rows_touched ? (size_t)slices * T : 0;
    if (n_out) {
      hipLaunchKernelGGL(k_fill_zero_u32, dim3((unsigned)((n_out + 255) / 256)), dim3(256), 0, ctx->stream,
                         reinterpret_cast<uint32_t *>(p.out), n_out);
      BDH_LAUNCH_CHECK(ctx, "k_fill_zero_u32");
    }
    if (n_rows) {
      hipLaunchKernelGGL(k_fill_zero_u32, dim3((unsigned)((n_rows + 255) / 256)), dim3(256), 0, ctx->stream,
                         reinterpret_cast<uint32_t *>(p.rows_touched), n_rows);
      BDH_LAUNCH_CHECK(ctx, "k_fill_zero_u32");
    }
    return BDH_OK;
  }
  // opt-in ("state_step.prompt_bf16" = T0): calls of T0+ tokens on an f32 state, positions given by the host and no
  // per-token by-products run on the bf16 matrix cores (inputs and scores rounded to bf16: tolerance class 2e-2)
  if (!fixed && !p.bitmask && !p.rows_touched && ctx->opt_step_prompt_bf16 > 0 && T >= ctx->opt_step_prompt_bf16 &&
      p.rho_dtype == BDH_F32 && !p.positions_dev && N % 8 == 0 && (p.rotary != BDH_ROPE || d % 8 == 0) &&
      (p.rotary != BDH_ALIBI || h <= 64))
    return bdh_launch_state_prefill_bf16(ctx, p, out_ln);
  // many tokens, no per-token by-products: the dense form on the f32 matrix cores (a bf16 state is widened for the call)
  // (not when even a 128-token chunk of rotated activations would pass 16 GiB of workspace)
  const bool chunk_fits = sizeof(float) * (size_t)slices * Nq * 128 <= (size_t(16) << 30) &&
                          (p.rho_dtype == BDH_F32 || sizeof(float) * (size_t)slices * Nq * d <= (size_t(64) << 30));
  // By default from 128 tokens on (from 8 for the cases below); where the token loop is cheap (the f32 RoPE kernel walks many tokens per
  // launch) only once the products have enough tiles to cover the chip (measured at N=8192, d=256, T=512:
  // B*h = 4 or 8 slices lose to the loop at 5 % density, 16 slices win at any density).
  const bool loop_is_cheap = fast && p.rho_dtype == BDH_F32;
  const long state_tiles = (long)slices * ((std::min(T, 512) + 127) / 128) * ((d + 127) / 128);
  // From 8 tokens on where the token loop has nothing to gain from sparsity: an f32 state that every token
  // streams in full anyway (PoPE, eager ALiBi), or one so small (up to 64 MiB) that the loop is a chain of launch
  // and barrier latencies (a 64-token prompt of the reference's tiny / base / large sizes: 1.5 / 1.4 / 3.5 ms
  // token by token, 0.27 / 0.34 / 0.95 ms as dense products; at 8 tokens 0.30 / 0.29 / 0.69 against 0.22 / 0.27 /
  // 0.59 ms, at 4 tokens the loop is ahead).
  const bool streamed = p.rho_dtype == BDH_F32 && (p.rotary == BDH_POPE || (p.rotary == BDH_ALIBI && !p.stamps));
  const bool small_state = p.rho_dtype == BDH_F32 && !loop_is_cheap &&
                           sizeof(float) * (size_t)slices * Nq * d <= (size_t(64) << 20);
  const bool dense_auto = (T >= 128 && (!loop_is_cheap || state_tiles >= n_cu / 2)) ||
                          (T >= 8 && (streamed || small_state));
  if (!fixed && !p.bitmask && !p.rows_touched && chunk_fits &&
      (ctx->opt_step_dense >= 0 ? ctx->opt_step_dense == 1 : dense_auto))
    return bdh_launch_state_chunks_f32(ctx, p, out_ln);
  // tokens per launch: the f32 RoPE kernel, the generic and the dense streaming kernel walk several, as many as
  // 64 MiB of partials allow
  const size_t partial_one = bdh_align_up(sizeof(float) * (size_t)slices * S * d, 256);
  const size_t cnt_one = bdh_align_up(sizeof(int) * (size_t)slices * S, 256);
  // (the latter two only when no per-token by-products are asked for)
  const bool generic = !fast && !fast_lazy;  // k_step_generic or k_step_dense
  int group = 1;
  if (T > 1 && ((fast && p.rho_dtype == BDH_F32) || (generic && !p.bitmask && !p.rows_touched)))
    group = (int)std::max<size_t>(1, std::min<size_t>((size_t)T, (size_t(64) << 20) / partial_one));
  if (fixed) group = 1;
  const size_t partial_bytes = partial_one * group;
  const size_t cnt_bytes = cnt_one * group;
  if (fixed) {
    if (partial_bytes + cnt_bytes > fixed_bytes)
      return bdh_fail(ctx, BDH_E_SHAPE,
                      "the allocation-free step needs %zu bytes of scratch for B*h=%d, N=%d, d=%d; the fixed array holds %zu",
                      partial_bytes + cnt_bytes, slices, N, d, fixed_bytes);
  } else {
    int rc = bdh_ws_reserve(ctx, partial_bytes + cnt_bytes);
    if (rc != BDH_OK) return rc;
  }
  char *ws = static_cast<char *>(fixed ? fixed : ctx->ws);
  float *partial = reinterpret_cast<float *>(ws);
  int *pair_cnt = reinterpret_cast<int *>(ws + partial_bytes);

  HeadScalars decay{}, log_decay{};
  const int has_decay = p.rotary == BDH_ALIBI;
  if (has_decay)
    for (int i = 0; i < h; ++i) {
      decay.v[i] = expf(-p.slopes_host[i]);  // src/model/attention.rs:181-186
      // k single-precision multiplications by decay are decay^k = exp(k * log(decay)), with the
      // logarithm of the ROUNDED factor so that the lazy form follows the reference's product
      log_decay.v[i] = (float)log((double)decay.v[i]);
    }
  if (p.stamps && p.rotary != BDH_ALIBI) return bdh_fail(ctx, BDH_E_INVAL, "decay stamps only apply to ALiBi");

  const int NW = (N + 63) / 64;
  for (int t = 0; t < T; t += group) {
    const int nt = std::min(group, T - t);
    StepPtrs a{};
    a.nt = nt;
    a.x_t_stride = N;
    a.v_t_stride = d;
    a.partial_t_stride = (long)(partial_one / sizeof(float));
    a.cnt_t_stride = (long)(cnt_one / sizeof(int));
    a.bm_t_stride = NW;
    a.x = p.x + (long)t * N;
    a.x_slice_stride = (long)T * N;
    a.v = p.v + (long)t * d;
    a.v_batch_stride = (long)T * d;
    a.freqs = p.freqs;
    a.pos_scalar = (float)(p.position + (int64_t)t);
    a.pos_int = (long)(p.position + (int64_t)t);
    a.pos_dev = p.positions_dev;
    a.pos_add = t;
    a.partial = partial;
    a.pair_cnt = pair_cnt;
    a.bitmask = p.bitmask ? reinterpret_cast<unsigned long long *>(p.bitmask) + (long)t * NW : nullptr;
    a.bitmask_slice_stride = (long)T * NW;
    a.h = h;
    a.N = N;
    a.S = S;
    float *out_t = p.out + (long)t * d;
    float *out_ln_t = out_ln ? out_ln + (long)t * d : nullptr;
    int32_t *rows_t = p.rows_touched ? p.rows_touched + t : nullptr;
    if (fast) {
      const int blocks = slices * S;
      if (p.rho_dtype == BDH_F32) {
        float *rho = static_cast<float *>(p.rho);
        if (d == 256 && !split) launch_fast<256, 4, 2, 1>(ctx->stream, blocks, a, rho);
        if (d == 256 && split) launch_fast<256, 8, 8, 8>(ctx->stream, blocks, a, rho);
        if (d == 512 && !split) launch_fast<512, 4, 2, 1>(ctx->stream, blocks, a, rho);
        if (d == 512 && split) launch_fast<512, 8, 2, 8>(ctx->stream, blocks, a, rho);
      } else {
        unsigned short *rho = static_cast<unsigned short *>(p.rho);
        if (d == 256 && !split)
          hipLaunchKernelGGL((k_step_rope_bf16<256, 4, 8, 1>), dim3(blocks), dim3(256), 0, ctx->stream, a, rho);
        if (d == 256 && split)
          hipLaunchKernelGGL((k_step_rope_bf16<256, 8, 4, 8>), dim3(blocks), dim3(512), 0, ctx->stream, a, rho);
        if (d == 512 && !split)
          hipLaunchKernelGGL((k_step_rope_bf16<512, 4, 2, 1>), dim3(blocks), dim3(256), 0, ctx->stream, a, rho);
        if (d == 512 && split)
          hipLaunchKernelGGL((k_step_rope_bf16<512, 8, 2, 8>), dim3(blocks), dim3(512), 0, ctx->stream, a, rho);
      }
      BDH_LAUNCH_CHECK(ctx, "k_step_rope");
      if (p.partials_out) {  // the caller's next kernel adds the partials up
        p.partials_out->partial = partial;
        p.partials_out->S = S;
        return BDH_OK;
      }
      launch_finalize(ctx->stream, slices, partial, pair_cnt, S, d, out_t, (long)T * d, out_ln_t, rows_t, (long)T, 2, nt,
                      a.partial_t_stride, a.cnt_t_stride);
      BDH_LAUNCH_CHECK(ctx, "k_step_finalize");
    } else if (fast_lazy) {
      float *rho = static_cast<float *>(p.rho);
      if (d == 256)
        hipLaunchKernelGGL((k_step_alibi_lazy_f32<256, 4, 4>), dim3(slices * S), dim3(256), 0, ctx->stream, a, rho,
                           p.stamps, decay, log_decay);
      else
        hipLaunchKernelGGL((k_step_alibi_lazy_f32<512, 4, 4>), dim3(slices * S), dim3(256), 0, ctx->stream, a, rho,
                           p.stamps, decay, log_decay);
      BDH_LAUNCH_CHECK(ctx, "k_step_alibi_lazy_f32");
      launch_finalize(ctx->stream, slices, partial, pair_cnt, S, d, out_t, (long)T * d, out_ln_t, rows_t, (long)T, 1);
      BDH_LAUNCH_CHECK(ctx, "k_step_finalize");
    } else if (fast_dense) {
      const dim3 grid(slices * S);
      if (p.rho_dtype == BDH_F32) {
        float *rho = static_cast<float *>(p.rho);
        if (d == 256) hipLaunchKernelGGL((k_step_dense<float, 256, 4>), grid, dim3(256), 0, ctx->stream, a, rho, Nq, p.rotary, decay);
        else hipLaunchKernelGGL((k_step_dense<float, 512, 4>), grid, dim3(256), 0, ctx->stream, a, rho, Nq, p.rotary, decay);
      } else {
        unsigned short *rho = static_cast<unsigned short *>(p.rho);
        if (d == 256) hipLaunchKernelGGL((k_step_dense<unsigned short, 256, 4>), grid, dim3(256), 0, ctx->stream, a, rho, Nq, p.rotary, decay);
        else hipLaunchKernelGGL((k_step_dense<unsigned short, 512, 4>), grid, dim3(256), 0, ctx->stream, a, rho, Nq, p.rotary, decay);
      }
      BDH_LAUNCH_CHECK(ctx, "k_step_dense");
      launch_finalize(ctx->stream, slices, partial, nullptr, S, d, out_t, (long)T * d, out_ln_t, nullptr, (long)T, 2, nt,
                      a.partial_t_stride, a.cnt_t_stride);
      BDH_LAUNCH_CHECK(ctx, "k_step_finalize");
      if (a.bitmask || rows_t) {
        hipLaunchKernelGGL(k_bitmask_rows, dim3(slices), dim3(256), 0, ctx->stream, a, p.rotary, Nq, rows_t,
                           (long)T, 0);
        BDH_LAUNCH_CHECK(ctx, "k_bitmask_rows");
      }
    } else {
      // registers for the columns a row really has: the narrower the rows, the more of them in flight
#define BDH_GEN(T_, MAXC_, FL_)                                                                                   \
  hipLaunchKernelGGL((k_step_generic<T_, MAXC_, FL_>), dim3(slices * S), dim3(256), 0, ctx->stream, a,           \
                     static_cast<T_ *>(p.rho), d, Nq, p.rotary, has_decay, decay, log_decay, p.stamps)
      if (p.rho_dtype == BDH_F32) {
        if (d <= 128) BDH_GEN(float, 2, 16); else if (d <= 256) BDH_GEN(float, 4, 8);
        else if (d <= 512) BDH_GEN(float, 8, 4); else BDH_GEN(float, 16, 4);
      } else {
        if (d <= 128) BDH_GEN(unsigned short, 2, 16); else if (d <= 256) BDH_GEN(unsigned short, 4, 8);
        else if (d <= 512) BDH_GEN(unsigned short, 8, 4); else BDH_GEN(unsigned short, 16, 4);
      }
#undef BDH_GEN
      BDH_LAUNCH_CHECK(ctx, "k_step_generic");
      launch_finalize(ctx->stream, slices, partial, nullptr, S, d, out_t, (long)T * d, out_ln_t, nullptr, (long)T, 2, nt,
                      a.partial_t_stride, a.cnt_t_stride);
      BDH_LAUNCH_CHECK(ctx, "k_step_finalize");
      if (a.bitmask || rows_t) {
        hipLaunchKernelGGL(k_bitmask_rows, dim3(slices), dim3(256), 0, ctx->stream, a, p.rotary, Nq, rows_t,
                           (long)T, p.stamps ? 1 : 0);
        BDH_LAUNCH_CHECK(ctx, "k_bitmask_rows");
      }
    }
  }
  return BDH_OK;
}

int bdh_launch_alibi_materialize(bdh_ctx *ctx, int B, int h, int N, int d, const float *slopes_host, int64_t clock,
                                 const int32_t *clocks_dev, void *rho, int rho_dtype, int32_t *stamps) {
  HeadScalars log_decay{};
  for (int i = 0; i < h; ++i) log_decay.v[i] = (float)log((double)expf(-slopes_host[i]));
  const long rows = (long)B * h * N;
  if (rows == 0 || d == 0) return BDH_OK;
  const long blocks = (rows + 3) / 4;
  if (blocks > 0x7fffffffL) return bdh_fail(ctx, BDH_E_SHAPE, "state has too many rows");
  if (rho_dtype == BDH_F32)
    hipLaunchKernelGGL(k_alibi_materialize<float>, dim3((unsigned)blocks), dim3(256), 0, ctx->stream,
                       static_cast<float *>(rho), stamps, h, N, d, rows, (long)clock, clocks_dev, log_decay);
  else
    hipLaunchKernelGGL(k_alibi_materialize<unsigned short>, dim3((unsigned)blocks), dim3(256), 0, ctx->stream,
                       static_cast<unsigned short *>(rho), stamps, h, N, d, rows, (long)clock, clocks_dev, log_decay);
  BDH_LAUNCH_CHECK(ctx, "k_alibi_materialize");
  return BDH_OK;
}

int bdh_launch_state_steps(bdh_ctx *ctx, const StateStepParams &p) {
  return bdh_launch_state_steps_ln(ctx, p, nullptr);
}
