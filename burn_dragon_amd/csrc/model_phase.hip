// A decode step (one token per sequence) of a mid-size model in TWO launches per layer instead of six.
// Kernel by kernel a layer of BDH::forward_with_state (src/model/bdh.rs:336-441) is D_x, state step, its second
// stage, D_y, encoder partials, encoder second stage; at a few sequences each of those is a launch latency plus a
// trip or two to memory.  The only points where a layer needs data from the whole sequence are the LayerNorm of
// a head's readout and the LayerNorm of the encoder output, so a workgroup that owns 64 neurons of one head of
// one sequence can run everything between them on its own:
//   phase A: [previous layer's cur = LN(cur + LN(sum of encoder partials))]  D_x for its 64 neurons, their state
//            rows (readout, update, decay), the readout partial of the workgroup;
//   phase B: LN(sum of the head's readout partials), D_y and the gate for its 64 neurons, the encoder partial of
//            those 64 rows of E.
// The sums over partials are redone by every workgroup that needs them (a few KiB from the L2).  Projections
// keep the k-sequential fmaf chain of k_relu_lowrank; the other sums are taken in a fixed tree of their own
// (results agree with the kernel-by-kernel step to rounding, not bit for bit).
#include "bdh_internal.h"

namespace {

constexpr float kLnEps = 1e-5f;                    // src/model/bdh.rs:17
constexpr float kTwoPi = 6.28318530717958647692f;  // f32(2*PI), src/model/attention.rs:343

struct PhaseArgs {
  const int64_t *tokens;      // first layer only: [B] tokens, the layer's input is LN(embed[token]) (else null)
  const float *embed;         // [V][d]
  int V;
  const float *cur_in;        // [B][d] the layer's input (before the pending encoder second stage, if any)
  float *cur_out;             // [B][d] written by the first workgroup of a sequence when it computed the input itself
  const float *dec_partial;   // [G][B][d] encoder partials of the previous layer, or null
  float *x;                   // [B][h*N]
  float *attn_partial;        // [B][h][N/64][d]
  float *dec_partial_out;     // [G][B][d], G = h * N / 64
  const float *enc, *enc_v, *dec, *freqs;
  void *rho;                  // this layer's state [B][h][Nq][d], f32 or bf16
  int32_t *stamps;            // this layer's stamps [B][h][N] or null
  const int32_t *pos_dev;
  long pos;
  int B, d, h, N, rotary;
  float thr;
  float decay[64], log_decay[64];
};

__device__ __forceinline__ float wave_sum(float v) {
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}

// LayerNorm statistics of d <= 64 * NW values held one per thread by threads 0..d-1; every thread calls it.
template <int NW>
__device__ __forceinline__ void block_ln_stats(float v, bool has, int d, float *s_st, float &mean, float &den) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  __syncthreads();  // s_st may still be read from an earlier use
  const float s = wave_sum(has ? v : 0.0f);
  if (lane == 0) s_st[wave] = s;
  __syncthreads();
  float t = s_st[0];
#pragma unroll
  for (int w = 1; w < NW; ++w) t += s_st[w];
  mean = t / (float)d;
  const float c = has ? v - mean : 0.0f;
  const float q = wave_sum(c * c);
  if (lane == 0) s_st[NW + wave] = q;
  __syncthreads();
  float u = s_st[NW];
#pragma unroll
  for (int w = 1; w < NW; ++w) u += s_st[NW + w];
  den = sqrtf(u / (float)d + kLnEps);
}

// The 64 weights of this wave's span of k for column n, asked for at once (rows past d are clamped to the last
// one and weighted zero: loads under a branch would not be issued back to back).
__device__ __forceinline__ void load_span(const float *__restrict__ w, int hh, int d, int N, int n, int k_lo, float *wv) {
  const float *wp = w + (long)hh * d * N + n;
#pragma unroll
  for (int u = 0; u < 64; ++u) {
    const float t = wp[(long)min(k_lo + u, d - 1) * N];
    wv[u] = k_lo + u < d ? t : 0.0f;
  }
}

// The column's fmaf chain, extended span by span in k order; the accumulator travels through LDS.  s_in holds
// the input row, zero beyond d.  Returns the full sum in the last wave.
template <int NW>
__device__ __forceinline__ float chain_spans(const float *s_in, const float *wv, float *s_acc) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int k_lo = wave * 64;
  float acc = 0.0f;
#pragma unroll
  for (int stage = 0; stage < NW; ++stage) {
    if (wave == stage) {
      if (stage > 0) acc = s_acc[lane];
#pragma unroll
      for (int u = 0; u < 64; ++u) acc = __builtin_fmaf(s_in[k_lo + u], wv[u], acc);
      if (stage < NW - 1) s_acc[lane] = acc;
    }
    if (stage < NW - 1) __syncthreads();
  }
  return acc;
}

// ---- phase A ---------------------------------------------------------------------------------------------------
template <int NW, typename RhoT>
__global__ __launch_bounds__(NW * 64) void k_layer_phase_a(PhaseArgs a) {
  constexpr int VPL = (NW + 3) / 4;  // float4 per lane per state row: columns (j*64 + lane)*4
  constexpr int kFlight = 64 / NW < 16 ? 64 / NW : 16;  // state rows in flight per wave: all of its share of a dense block
  __shared__ __align__(16) float s_cur[NW * 64];
  __shared__ float s_x[64];
  __shared__ float s_acc[64];
  __shared__ float s_st[2 * NW];
  __shared__ unsigned char s_list[NW][64];
  __shared__ float4 s_red[NW][VPL * 64];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int d = a.d, h = a.h, N = a.N;
  const int nblk_n = N >> 6;
  const int nblk = blockIdx.x % nblk_n;
  const int hh = (blockIdx.x / nblk_n) % h;
  const int b = blockIdx.x / (nblk_n * h);
  const int n = nblk * 64 + lane;  // this lane's neuron of the head
  const long pos = a.pos_dev ? (long)a.pos_dev[b] : a.pos;
  const float posf = (float)pos;

  // weights of D_x first: they do not depend on anything computed here
  float wv[64];
  load_span(a.enc, hh, d, N, n, wave * 64, wv);

  // the layer's input: cur, after the pending second stage of the previous layer's encoder
  // (src/model/bdh.rs:383, 436-441: cur = LN(cur + LN(mixed . decoder)))
  {
    const bool has = tid < d;
    float cur = 0.0f;
    if (a.tokens) {  // embedding row and its LayerNorm (src/model/bdh.rs:319-322); a bad token poisons the row
      const int64_t tok = a.tokens[b];
      const bool bad = tok < 0 || tok >= a.V;
      const float v = has ? (bad ? __int_as_float(0x7fc00000) : a.embed[(long)tok * d + tid]) : 0.0f;
      float mean, den;
      block_ln_stats<NW>(v, has, d, s_st, mean, den);
      cur = has ? (v - mean) / den : 0.0f;
      if (has && hh == 0 && nblk == 0) a.cur_out[(long)b * d + tid] = cur;
    } else if (has) {
      cur = a.cur_in[(long)b * d + tid];
    }
    if (a.dec_partial) {
      const int G = h * nblk_n;
      float mlp = 0.0f;
      if (has) {
        int g = 0;
        for (; g + 8 <= G; g += 8) {
          float t[8];
#pragma unroll
          for (int u = 0; u < 8; ++u) t[u] = a.dec_partial[((long)(g + u) * a.B + b) * d + tid];
#pragma unroll
          for (int u = 0; u < 8; ++u) mlp += t[u];
        }
        for (; g < G; ++g) mlp += a.dec_partial[((long)g * a.B + b) * d + tid];
      }
      float mean, den;
      block_ln_stats<NW>(mlp, has, d, s_st, mean, den);
      const float z = has ? cur + (mlp - mean) / den : 0.0f;
      block_ln_stats<NW>(z, has, d, s_st, mean, den);
      cur = has ? (z - mean) / den : 0.0f;
      if (has && hh == 0 && nblk == 0) a.cur_out[(long)b * d + tid] = cur;
    }
    s_cur[tid] = cur;  // zero beyond d
  }
  __syncthreads();

  // x = relu(cur . encoder - thr) for the 64 neurons (src/model/bdh.rs:337-351)
  {
    const float acc = chain_spans<NW>(s_cur, wv, s_acc);
    if (wave == NW - 1) {
      float p = acc;
      if (a.thr != 0.0f) p = p - a.thr;
      const float xv = p > 0.0f ? p : 0.0f;
      s_x[lane] = xv;
      a.x[((long)b * h + hh) * N + n] = xv;
    }
  }
  __syncthreads();

  // the state rows of these neurons (src/model/bdh.rs:232-306): readout with the old rows, rank-1 update with
  // value = cur, ALiBi decay; only visited rows are touched.  Every wave prepares the same list (lane = neuron)
  // and takes every NW-th entry of it.
  const bool alibi = a.rotary == BDH_ALIBI, pope = a.rotary == BDH_POPE;
  const int Nq = pope ? 2 * N : N;
  RhoT *rho = static_cast<RhoT *>(a.rho) + ((long)b * h + hh) * (long)Nq * d;
  int32_t *st = a.stamps ? a.stamps + ((long)b * h + hh) * N : nullptr;
  const bool lazy = alibi && st != nullptr;
  const float dec = alibi ? a.decay[hh] : 1.0f;
  float4 acc[VPL], vv[VPL];
#pragma unroll
  for (int j = 0; j < VPL; ++j) {
    const int c = (j * 64 + lane) * 4;
    acc[j] = make_float4(0.f, 0.f, 0.f, 0.f);
    vv[j] = c < d ? *reinterpret_cast<const float4 *>(&s_cur[c]) : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  for (int part = 0; part < (pope ? 2 : 1); ++part) {  // PoPE: real rows n, then imaginary rows N + n
    float q_l = 0.0f, scale_l = 1.0f;
    bool touch_l = false;
    const float xn = s_x[lane];
    if (alibi) {  // q = x (src/model/attention.rs:332-349)
      q_l = xn;
      touch_l = lazy ? (q_l != 0.0f) : true;
      if (lazy && touch_l) {
        const long k = pos - (long)st[n];
        if (k > 0) scale_l = expf((float)k * a.log_decay[hh]);
      }
    } else if (pope) {  // src/model/attention.rs:323-330
      const float mag = logf(expf(xn * 1.0f) + 1.0f) / 1.0f;
      const float raw = posf * a.freqs[n];
      const float ph = (raw - floorf(raw)) * kTwoPi;
      q_l = part == 0 ? mag * cosf(ph) : mag * sinf(ph);
      touch_l = true;
    } else {  // RoPE (src/model/attention.rs:305-321)
      const float xo = s_x[lane ^ 1];
      touch_l = (xn != 0.0f) || (xo != 0.0f);
      if (touch_l) {
        const float raw = posf * a.freqs[n];
        const float ph = (raw - floorf(raw)) * kTwoPi;
        float sn, cs;
        sincosf(ph, &sn, &cs);
        const float rot = (n & 1) ? xo : -xo;
        const float t0 = xn * cs, t1 = rot * sn;
        q_l = t0 + t1;
      }
    }
    const unsigned long long m = __ballot(touch_l);
    const int count = __popcll(m);
    if (touch_l) s_list[wave][__popcll(m & ((1ull << lane) - 1ull))] = (unsigned char)lane;
    // (LDS operations of one wave execute in order: the list is read back below without a barrier)
    const long row_base = (long)(part * N + nblk * 64);
    for (int i0 = wave; i0 < count; i0 += NW * kFlight) {
      int src[kFlight];
      bool ok[kFlight];
      float4 rv[kFlight][VPL];
#pragma unroll
      for (int u = 0; u < kFlight; ++u) {
        const int idx = i0 + u * NW;
        const int listed = s_list[wave][idx & 63];  // read whether or not the slot is used: no branch
        ok[u] = idx < count;
        src[u] = ok[u] ? listed : 0;
      }
#pragma unroll
      for (int u = 0; u < kFlight; ++u) {
        const RhoT *row = rho + (row_base + src[u]) * d;
#pragma unroll
        for (int j = 0; j < VPL; ++j) {
          const int c = (j * 64 + lane) * 4;
          rv[u][j] = bdh_rho_load4(row + (c < d ? c : 0));
        }
      }
#pragma unroll
      for (int u = 0; u < kFlight; ++u) {
        const int lu = __builtin_amdgcn_readfirstlane(src[u]);
        const float q_src = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(q_l), lu));
        const float scale = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(scale_l), lu));
        const float qn = ok[u] ? q_src : 0.0f;
        RhoT *row = rho + (row_base + src[u]) * d;
#pragma unroll
        for (int j = 0; j < VPL; ++j) {
          const int c = (j * 64 + lane) * 4;
          float4 e = rv[u][j];
          if (!ok[u]) e = make_float4(0.f, 0.f, 0.f, 0.f);
          if (lazy) {
            e.x *= scale; e.y *= scale; e.z *= scale; e.w *= scale;
          }
          acc[j].x = __builtin_fmaf(e.x, qn, acc[j].x);
          acc[j].y = __builtin_fmaf(e.y, qn, acc[j].y);
          acc[j].z = __builtin_fmaf(e.z, qn, acc[j].z);
          acc[j].w = __builtin_fmaf(e.w, qn, acc[j].w);
          float t;
          t = qn * vv[j].x; e.x = e.x + t;
          t = qn * vv[j].y; e.y = e.y + t;
          t = qn * vv[j].z; e.z = e.z + t;
          t = qn * vv[j].w; e.w = e.w + t;
          if (alibi) {  // src/model/bdh.rs:299-301
            e.x *= dec; e.y *= dec; e.z *= dec; e.w *= dec;
          }
          if (ok[u] && c < d) bdh_rho_store4(row + c, e);
        }
      }
    }
    __syncthreads();  // every wave has read the stamps before the first one replaces them
    if (lazy && touch_l && wave == 0) st[n] = (int32_t)min(pos + 1, 0x7fffffffL);
  }
#pragma unroll
  for (int j = 0; j < VPL; ++j) s_red[wave][j * 64 + lane] = acc[j];
  __syncthreads();
  float *pout = a.attn_partial + (((long)b * h + hh) * nblk_n + nblk) * d;
  for (int c4 = tid; c4 < d / 4; c4 += NW * 64) {
    const int j = c4 >> 6, l = c4 & 63;  // column group c4 lives in lane l, piece j
    float4 s = s_red[0][j * 64 + l];
#pragma unroll
    for (int w = 1; w < NW; ++w) {
      const float4 t = s_red[w][j * 64 + l];
      s.x += t.x; s.y += t.y; s.z += t.z; s.w += t.w;
    }
    reinterpret_cast<float4 *>(pout)[c4] = s;
  }
}

// ---- phase B ---------------------------------------------------------------------------------------------------
template <int NW>
__global__ __launch_bounds__(NW * 64) void k_layer_phase_b(PhaseArgs a) {
  __shared__ float s_in[NW * 64];
  __shared__ float s_xy[64];
  __shared__ float s_acc[64];
  __shared__ float s_st[2 * NW];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int d = a.d, h = a.h, N = a.N;
  const int nblk_n = N >> 6;
  const int nblk = blockIdx.x % nblk_n;
  const int hh = (blockIdx.x / nblk_n) % h;
  const int b = blockIdx.x / (nblk_n * h);
  const int n = nblk * 64 + lane;

  float wv[64];
  load_span(a.enc_v, hh, d, N, n, wave * 64, wv);
  const float xg = wave == NW - 1 ? a.x[((long)b * h + hh) * N + n] : 0.0f;  // the gate, needed last

  // LayerNorm of the head's readout (src/model/bdh.rs:359): the partials of the head's workgroups, in order
  {
    const bool has = tid < d;
    float at = 0.0f;
    if (has) {
      const float *pp = a.attn_partial + ((long)b * h + hh) * nblk_n * d + tid;
      int g = 0;
      for (; g + 8 <= nblk_n; g += 8) {
        float t[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) t[u] = pp[(long)(g + u) * d];
#pragma unroll
        for (int u = 0; u < 8; ++u) at += t[u];
      }
      for (; g < nblk_n; ++g) at += pp[(long)g * d];
    }
    float mean, den;
    block_ln_stats<NW>(at, has, d, s_st, mean, den);
    s_in[tid] = has ? (at - mean) / den : 0.0f;
  }
  __syncthreads();

  // xy = x * relu(LN(attn) . encoder_v - thr) for the 64 neurons (src/model/bdh.rs:361-381)
  {
    const float acc = chain_spans<NW>(s_in, wv, s_acc);
    if (wave == NW - 1) {
      float p = acc;
      if (a.thr != 0.0f) p = p - a.thr;
      const float y = p > 0.0f ? p : 0.0f;
      s_xy[lane] = xg * y;
    }
  }
  __syncthreads();

  // encoder partial of these 64 rows of E (src/model/bdh.rs:383): one column per thread, the 64 rows in flight
  if (tid < d) {
    const float *ep = a.dec + ((long)hh * N + nblk * 64) * d + tid;
    float ev[64];
#pragma unroll
    for (int u = 0; u < 64; ++u) ev[u] = ep[(long)u * d];
    float acc = 0.0f;
#pragma unroll
    for (int u = 0; u < 64; ++u) acc = __builtin_fmaf(s_xy[u], ev[u], acc);
    const int g = hh * nblk_n + nblk;
    a.dec_partial_out[((long)g * a.B + b) * d + tid] = acc;
  }
}

// ---- head -----------------------------------------------------------------------------------------------------
// The last layer's pending second stage, then the logits and the greedy token (src/model/bdh.rs:436-449): one
// workgroup of 16 waves per sequence.  logits[v] = sum_k cur[k] * lm_head[k][v]: 1024 / pad64(V) groups split k,
// each one fmaf chain over its span with 32 rows in flight; the groups are added in order; the lowest index wins ties.
__global__ __launch_bounds__(1024) void k_phase_head(const float *__restrict__ cur_in, const float *__restrict__ dec_partial,
                                                     int G, int B, int d, const float *__restrict__ lm_head, int V,
                                                     float *__restrict__ logits, int64_t *__restrict__ next) {
  __shared__ float s_cur[512];
  __shared__ float s_st[32];
  __shared__ float s_grp[1024];
  __shared__ float s_best[16];
  __shared__ int s_arg[16];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int b = blockIdx.x;
  {
    const bool has = tid < d;
    float mlp = 0.0f;
    if (has) {
      int g = 0;
      for (; g + 8 <= G; g += 8) {
        float t[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) t[u] = dec_partial[((long)(g + u) * B + b) * d + tid];
#pragma unroll
        for (int u = 0; u < 8; ++u) mlp += t[u];
      }
      for (; g < G; ++g) mlp += dec_partial[((long)g * B + b) * d + tid];
    }
    const float base = has ? cur_in[(long)b * d + tid] : 0.0f;
    float mean, den;
    block_ln_stats<16>(mlp, has, d, s_st, mean, den);
    const float z = has ? base + (mlp - mean) / den : 0.0f;
    block_ln_stats<16>(z, has, d, s_st, mean, den);
    if (tid < 512) s_cur[tid] = has ? (z - mean) / den : 0.0f;
  }
  __syncthreads();
  const int Vp = (V + 63) & ~63;
  const int GK = 1024 / Vp;
  const int g = tid / Vp, c = tid - g * Vp;
  const int per = (d + GK - 1) / GK;
  if (g < GK && c < V) {
    const int k0 = min(d, g * per), k1 = min(d, k0 + per);
    float acc = 0.0f;
    int k = k0;
    for (; k + 32 <= k1; k += 32) {
      float wv[32];
#pragma unroll
      for (int u = 0; u < 32; ++u) wv[u] = lm_head[(long)(k + u) * V + c];
#pragma unroll
      for (int u = 0; u < 32; ++u) acc = __builtin_fmaf(s_cur[k + u], wv[u], acc);
    }
    for (; k + 8 <= k1; k += 8) {
      float wv[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) wv[u] = lm_head[(long)(k + u) * V + c];
#pragma unroll
      for (int u = 0; u < 8; ++u) acc = __builtin_fmaf(s_cur[k + u], wv[u], acc);
    }
    for (; k < k1; ++k) acc = __builtin_fmaf(s_cur[k], lm_head[(long)k * V + c], acc);
    s_grp[g * Vp + c] = acc;
  }
  __syncthreads();
  float best = -INFINITY;
  int arg = 0x7fffffff;
  if (tid < V) {
    float v = s_grp[tid];
    for (int gg = 1; gg < GK; ++gg) v += s_grp[gg * Vp + tid];
    logits[(long)b * V + tid] = v;
    if (v > best) {
      best = v;
      arg = tid;
    }
  }
  if (!next) return;  // uniform
  for (int o = 32; o > 0; o >>= 1) {
    const float ob = __shfl_xor(best, o);
    const int oa = __shfl_xor(arg, o);
    if (ob > best || (ob == best && oa < arg)) {
      best = ob;
      arg = oa;
    }
  }
  if (lane == 0) {
    s_best[wave] = best;
    s_arg[wave] = arg;
  }
  __syncthreads();
  if (tid == 0) {
    for (int w = 1; w < 16; ++w)
      if (s_best[w] > best || (s_best[w] == best && s_arg[w] < arg)) {
        best = s_best[w];
        arg = s_arg[w];
      }
    next[b] = arg == 0x7fffffff ? 0 : arg;
  }
}

}  // namespace

bool bdh_model_phase_fits(const bdh_model_config &c) {
  if (c.rotary != BDH_ROPE && c.rotary != BDH_ALIBI && c.rotary != BDH_POPE) return false;
  if (c.n_embd < 128 || c.n_embd > 512 || (c.n_embd & 3) != 0) return false;
  if (c.latent < 64 || (c.latent & 63) != 0) return false;  // whole 64-neuron blocks
  if (c.n_head < 1 || c.n_head > 64 || c.n_layer < 1) return false;
  // every workgroup of a sequence sums the partials of all the others: only while those are few
  if ((long)c.n_head * (c.latent / 64) > 64) return false;
  return true;
}

size_t bdh_model_phase_scratch_floats(const bdh_model_config &c, int B) {
  const size_t d = c.n_embd, cols = (size_t)c.n_head * c.latent, G = cols / 64;
  // cur ping-pong | x | readout partials | encoder partials
  return 2 * bdh_align_up((size_t)B * d, 64) + bdh_align_up((size_t)B * cols, 64) + bdh_align_up((size_t)B * G * d, 64) +
         bdh_align_up(G * (size_t)B * d, 64);
}

// On return cur_final points at the buffer holding the last layer's input and dec_partial at its encoder partials
// [G][B][d]: the caller runs the encoder's second stage and the head.
int bdh_launch_model_phases(bdh_model *m, const int64_t *tokens, int B, float *scratch, void *rho, int rho_dtype,
                            int32_t *stamps, int64_t position,
                            const int32_t *positions_dev, float **cur_final, float **dec_partial, int *G_out) {
  bdh_ctx *ctx = m->ctx;
  const bdh_model_config &c = m->cfg;
  if (!bdh_model_phase_fits(c)) return bdh_fail(ctx, BDH_E_SHAPE, "model does not fit the two-launch layer");
  const int d = c.n_embd, h = c.n_head, N = c.latent, L = c.n_layer;
  const size_t cols = (size_t)h * N, G = cols / 64;
  const long grid = (long)B * h * (N / 64);
  if (grid > 0x7fffffffL) return bdh_fail(ctx, BDH_E_SHAPE, "grid too large");
  float *cur[2] = {scratch, scratch + bdh_align_up((size_t)B * d, 64)};
  float *x = cur[1] + bdh_align_up((size_t)B * d, 64);
  float *attn_partial = x + bdh_align_up((size_t)B * cols, 64);
  float *dpart = attn_partial + bdh_align_up((size_t)B * G * d, 64);
  const size_t Nq = c.rotary == BDH_POPE ? 2 * (size_t)N : (size_t)N;
  PhaseArgs a{};
  a.x = x;
  a.attn_partial = attn_partial;
  a.dec_partial_out = dpart;
  a.enc = m->w.encoder;
  a.enc_v = m->w.encoder_v;
  a.dec = m->w.decoder;
  a.freqs = m->freqs;
  a.pos_dev = positions_dev;
  a.pos = (long)position;
  a.B = B;
  a.d = d;
  a.h = h;
  a.N = N;
  a.rotary = c.rotary;
  a.thr = c.relu_threshold;
  if (c.rotary == BDH_ALIBI)
    for (int i = 0; i < h; ++i) {
      a.decay[i] = expf(-m->slopes[i]);                 // src/model/attention.rs:181-186
      a.log_decay[i] = (float)log((double)a.decay[i]);  // of the rounded factor, as the lazy state step
    }
  const int nw = (d + 63) / 64;
  int in = 0;  // cur[in] is the layer's input; a layer with a pending second stage writes cur[in ^ 1]
  a.embed = m->w.embed;
  a.V = c.vocab;
  for (int l = 0; l < L; ++l) {
    a.tokens = l == 0 ? tokens : nullptr;  // the first layer makes its own input and leaves it in cur[0]
    a.cur_in = cur[in];
    a.cur_out = l == 0 ? cur[0] : cur[in ^ 1];
    a.dec_partial = l > 0 ? dpart : nullptr;
    a.rho = static_cast<char *>(rho) + (size_t)l * B * h * Nq * d * (rho_dtype == BDH_BF16 ? 2 : 4);
    a.stamps = stamps ? stamps + (size_t)l * B * h * N : nullptr;
#define BDH_PHASE(K_, NW_) hipLaunchKernelGGL((K_<NW_>), dim3((unsigned)grid), dim3(NW_ * 64), 0, ctx->stream, a)
#define BDH_PHASE_A(NW_)                                                                                           \
  do {                                                                                                             \
    if (rho_dtype == BDH_BF16)                                                                                     \
      hipLaunchKernelGGL((k_layer_phase_a<NW_, unsigned short>), dim3((unsigned)grid), dim3(NW_ * 64), 0, ctx->stream, a); \
    else                                                                                                           \
      hipLaunchKernelGGL((k_layer_phase_a<NW_, float>), dim3((unsigned)grid), dim3(NW_ * 64), 0, ctx->stream, a);   \
  } while (0)
    if (nw <= 2) BDH_PHASE_A(2); else if (nw <= 4) BDH_PHASE_A(4); else BDH_PHASE_A(8);
    BDH_LAUNCH_CHECK(ctx, "k_layer_phase_a");
    if (l > 0) in ^= 1;  // phase A has applied the pending second stage: the layer's input is now cur[in ^ 1]
    if (nw <= 2) BDH_PHASE(k_layer_phase_b, 2); else if (nw <= 4) BDH_PHASE(k_layer_phase_b, 4); else BDH_PHASE(k_layer_phase_b, 8);
    BDH_LAUNCH_CHECK(ctx, "k_layer_phase_b");
#undef BDH_PHASE
#undef BDH_PHASE_A
  }
  *cur_final = cur[in];
  *dec_partial = dpart;
  *G_out = (int)G;
  return BDH_OK;
}

// The last layer's second stage and the output head in one launch (V <= 1024).
int bdh_launch_phase_head(bdh_model *m, int B, const float *cur, const float *dec_partial, int G, float *logits,
                          int64_t *next_tokens) {
  bdh_ctx *ctx = m->ctx;
  const bdh_model_config &c = m->cfg;
  if (c.vocab > 1024 || c.n_embd > 512) return bdh_fail(ctx, BDH_E_SHAPE, "head kernel needs V <= 1024 and d <= 512");
  hipLaunchKernelGGL(k_phase_head, dim3((unsigned)B), dim3(1024), 0, ctx->stream, cur, dec_partial, G, B, c.n_embd,
                     m->w.lm_head, c.vocab, logits, next_tokens);
  BDH_LAUNCH_CHECK(ctx, "k_phase_head");
  return BDH_OK;
}
