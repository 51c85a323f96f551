// A whole decode step (one token per sequence) of a small model in ONE launch: one workgroup of 16 waves
// carries one sequence through the embedding, every layer and the output head of
// BDH::forward_with_state (src/model/bdh.rs:309-450).  At these sizes (d <= 256, h*N <= 2048: the
// reference's shipped checkpoints) the weights sit in the L2 and a layer is a few hundred KiB of state, so
// the step of the kernel-per-operation path is nothing but launch latencies; here the activations never
// leave LDS and the only global traffic is weights in, state rows in and out, logits out.
//
// Values: the projections keep the k-sequential fmaf chain of k_relu_lowrank; sums over state rows, over
// the decoder's k and the LayerNorm statistics are taken in a fixed tree of their own (results differ
// from the kernel-per-operation path in the last bits, and are the same for every batch size and replay).
#include "bdh_internal.h"

namespace {

constexpr float kLnEps = 1e-5f;  // src/model/bdh.rs:17
constexpr float kTwoPi = 6.28318530717958647692f;  // f32(2*PI), src/model/attention.rs:343
constexpr int kThreads = 1024;
constexpr int kWaves = 16;
constexpr int kMaxD = 256;      // embedding width
constexpr int kMaxCols = 2048;  // h * N

struct SmallArgs {
  const int64_t *tokens;
  const float *embed, *enc, *enc_v, *dec, *lm_head, *freqs;
  void *rho;  // f32 or bf16 elements
  int32_t *stamps;
  const int32_t *pos_dev;
  long pos;
  float *logits;
  int64_t *next;
  int B, d, h, N, V, L, rotary;
  float thr;
  size_t rho_layer_stride;    // elements
  size_t stamps_layer_stride;  // entries
  float decay[16], log_decay[16];
};

__device__ __forceinline__ float wave_sum(float v) {
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}

// LayerNorm statistics of a row of d <= 256 values held one per thread by threads 0..d-1 (`has`): mean,
// then sqrt(biased variance + eps).  Every thread of the workgroup calls it.
__device__ __forceinline__ void block_ln_stats(float v, bool has, int d, float *s_st, float &mean, float &den) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  __syncthreads();  // s_st may still be read from an earlier use
  if (wave < 4) {
    const float s = wave_sum(has ? v : 0.0f);
    if (lane == 0) s_st[wave] = s;
  }
  __syncthreads();
  mean = (((s_st[0] + s_st[1]) + s_st[2]) + s_st[3]) / (float)d;
  if (wave < 4) {
    const float c = has ? v - mean : 0.0f;
    const float q = wave_sum(c * c);
    if (lane == 0) s_st[4 + wave] = q;
  }
  __syncthreads();
  den = sqrtf((((s_st[4] + s_st[5]) + s_st[6]) + s_st[7]) / (float)d + kLnEps);
}

// out[col] = relu(sum_k in[head(col)][k] * w[head][k][n] - thr) (* gate[col]); one thread per latent column,
// k-sequential fmaf chain, 32 weight rows in flight (src/model/bdh.rs:337-351, 361-381)
__device__ __forceinline__ void project(const float *s_in, int in_head_stride, const float *__restrict__ w, int d, int N,
                                        int cols, float thr, const float *s_gate, float *s_out) {
  for (int col = threadIdx.x; col < cols; col += kThreads) {
    const int hh = col / N, n = col - hh * N;
    const float *in = s_in + hh * in_head_stride;
    // uniform row pointer + 32-bit per-thread offset: a load needs no vector address arithmetic
    const unsigned voff = (unsigned)hh * (unsigned)d * (unsigned)N + (unsigned)n;
    float acc = 0.0f;
    int k0 = 0;
    for (; k0 + 32 <= d; k0 += 32) {
      float wv[32];
#pragma unroll
      for (int u = 0; u < 32; ++u) wv[u] = (w + (size_t)(k0 + u) * N)[voff];
#pragma unroll
      for (int u = 0; u < 32; ++u) acc = __builtin_fmaf(in[k0 + u], wv[u], acc);
    }
    for (; k0 < d; ++k0) acc = __builtin_fmaf(in[k0], (w + (size_t)k0 * N)[voff], acc);
    float p = acc;
    if (thr != 0.0f) p = p - thr;
    float y = p > 0.0f ? p : 0.0f;
    if (s_gate) y = s_gate[col] * y;
    s_out[col] = y;
  }
}

// out[c] = sum_k in[k] * w[k][c] for c < C (C <= 1024): 1024 / pad64(C) groups split k, each group one
// fmaf chain over its span with 32 rows in flight; the groups are added in order.
__device__ __forceinline__ float matvec_cols(const float *s_in, int K, const float *__restrict__ w, int C,
                                             float (*s_red)[kMaxD]) {
  const int Cp = (C + 63) & ~63;
  const int G = kThreads / Cp;
  const int g = threadIdx.x / Cp, c = threadIdx.x - g * Cp;
  const int per = (K + G - 1) / G;
  __syncthreads();  // s_red may still be read from an earlier use
  if (g < G && c < C) {
    const int k0 = min(K, g * per), k1 = min(K, k0 + per);
    float acc = 0.0f;
    int k = k0;
    for (; k + 32 <= k1; k += 32) {
      float wv[32];
#pragma unroll
      for (int u = 0; u < 32; ++u) wv[u] = w[(long)(k + u) * C + c];
#pragma unroll
      for (int u = 0; u < 32; ++u) acc = __builtin_fmaf(s_in[k + u], wv[u], acc);
    }
    for (; k + 16 <= k1; k += 16) {
      float wv[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) wv[u] = w[(long)(k + u) * C + c];
#pragma unroll
      for (int u = 0; u < 16; ++u) acc = __builtin_fmaf(s_in[k + u], wv[u], acc);
    }
    for (; k < k1; ++k) acc = __builtin_fmaf(s_in[k], w[(long)k * C + c], acc);
    (&s_red[0][0])[g * Cp + c] = acc;
  }
  __syncthreads();
  float v = 0.0f;
  if ((int)threadIdx.x < C) {
    v = (&s_red[0][0])[threadIdx.x];
    for (int gg = 1; gg < G; ++gg) v += (&s_red[0][0])[gg * Cp + threadIdx.x];
  }
  return v;
}

// LPR: lanes per state row, four adjacent columns each (d <= 4 * LPR); a wave instruction covers 64 / LPR rows and
// 8 such groups of rows are in flight per wave
template <int LPR, typename RhoT>
__global__ __launch_bounds__(kThreads) void k_model_step_small(SmallArgs a) {
  constexpr int RPI = 64 / LPR;  // rows per instruction
  constexpr int kFlight = 8;
  __shared__ float s_cur[kMaxD];
  __shared__ float s_x[kMaxCols];
  __shared__ float s_xy[kMaxCols];
  __shared__ float s_attn[16 * kMaxD];  // [h][d]: readout, then its LayerNorm
  __shared__ float s_red[kWaves][kMaxD];
  __shared__ float s_st[8];
  __shared__ unsigned char s_list[kWaves][64];  // per wave: the lanes whose rows are visited, compacted
  __shared__ float s_best[kWaves];
  __shared__ int s_arg[kWaves];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int b = blockIdx.x;
  const int d = a.d, h = a.h, N = a.N, V = a.V;
  const int cols = h * N;
  const long pos = a.pos_dev ? (long)a.pos_dev[b] : a.pos;
  const float posf = (float)pos;

  // embedding row and its LayerNorm (src/model/bdh.rs:319-322); a token outside the vocabulary poisons the row
  {
    const int64_t tok = a.tokens[b];
    const bool bad = tok < 0 || tok >= V;
    const bool has = tid < d;
    const float v = has ? (bad ? __int_as_float(0x7fc00000) : a.embed[(long)tok * d + tid]) : 0.0f;
    float mean, den;
    block_ln_stats(v, has, d, s_st, mean, den);
    if (has) s_cur[tid] = (v - mean) / den;
  }
  __syncthreads();

  const bool alibi = a.rotary == BDH_ALIBI, pope = a.rotary == BDH_POPE;
  const int Nq = pope ? 2 * N : N;     // PoPE: rows N..2N-1 of a head are the imaginary parts
  const int srows = h * Nq;            // state rows of a sequence
  const int rpw = srows / kWaves;      // state rows per wave, all of one head
  const int row0 = wave * rpw;
  const int hh_w = row0 / Nq;
  const int wph = kWaves / h;          // waves per head

  for (int l = 0; l < a.L; ++l) {  // src/model/bdh.rs:336 -- the same weights in every layer
    // x = relu(cur . encoder - thr)
    project(s_cur, 0, a.enc, d, N, cols, a.thr, nullptr, s_x);
    __syncthreads();

    // recurrent attention with value = cur (src/model/bdh.rs:353-359, 232-306): readout with the old rows,
    // then the rank-1 update (and the ALiBi decay); only visited rows are touched
    {
      RhoT *rho = static_cast<RhoT *>(a.rho) + (size_t)l * a.rho_layer_stride + (size_t)b * srows * d;
      int32_t *st = a.stamps ? a.stamps + (size_t)l * a.stamps_layer_stride + (size_t)b * cols : nullptr;
      const bool lazy = alibi && st != nullptr;
      const float dec = alibi ? a.decay[hh_w] : 1.0f;
      const int sub = lane / LPR, cl = lane - sub * LPR;  // this lane's row within an instruction, its column group
      const bool has_c = cl * 4 < d;                      // d % 4 == 0
      const int coff = has_c ? cl * 4 : 0;
      float acc[4], vv[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        acc[j] = 0.0f;
        vv[j] = has_c ? s_cur[cl * 4 + j] : 0.0f;
      }
      for (int base = 0; base < rpw; base += 64) {
        const int r_l = row0 + base + lane;  // this lane prepares row r_l
        const bool in_range = base + lane < rpw;
        float q_l = 0.0f, scale_l = 1.0f;
        bool touch_l = false;
        if (in_range) {
          if (alibi) {  // q = x (src/model/attention.rs:332-349)
            q_l = s_x[r_l];
            touch_l = lazy ? (q_l != 0.0f) : true;
            if (lazy && touch_l) {
              const long k = pos - (long)st[r_l];
              if (k > 0) scale_l = expf((float)k * a.log_decay[hh_w]);
            }
          } else if (pope) {  // PoPE (src/model/attention.rs:323-330): every row is visited
            const int n = r_l - hh_w * Nq;
            const int m = n < N ? n : n - N;
            const float mag = logf(expf(s_x[hh_w * N + m] * 1.0f) + 1.0f) / 1.0f;  // softplus, beta = 1
            const float raw = posf * a.freqs[m];
            const float ph = (raw - floorf(raw)) * kTwoPi;
            q_l = n < N ? mag * cosf(ph) : mag * sinf(ph);
            touch_l = true;
          } else {  // RoPE (src/model/attention.rs:305-321)
            const int n = r_l - hh_w * N;
            const float xn = s_x[r_l], xo = s_x[r_l ^ 1];
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
        }
        const unsigned long long m = __ballot(touch_l);
        const int count = __popcll(m);
        if (touch_l) s_list[wave][__popcll(m & ((1ull << lane) - 1ull))] = (unsigned char)lane;
        // (LDS operations of one wave execute in order: the list is read back below without a barrier)
        for (int i0 = 0; i0 < count; i0 += kFlight * RPI) {
          int src[kFlight];
          bool ok[kFlight];
          float4 rv[kFlight];
#pragma unroll
          for (int u = 0; u < kFlight; ++u) {
            const int idx = i0 + u * RPI + sub;
            const int listed = s_list[wave][idx & 63];  // read whether or not the slot is used: no branch
            ok[u] = idx < count;
            src[u] = ok[u] ? listed : 0;
          }
          // unconditional loads (an unused slot reads the wave's first row again): loads under a branch are not
          // issued back to back
#pragma unroll
          for (int u = 0; u < kFlight; ++u)
            rv[u] = bdh_rho_load4(rho + (size_t)(row0 + base + src[u]) * d + coff);
#pragma unroll
          for (int u = 0; u < kFlight; ++u) {
            const float q_src = __shfl(q_l, src[u], 64);
            const float scale = __shfl(scale_l, src[u], 64);
            const float qn = ok[u] ? q_src : 0.0f;
            float r[4] = {rv[u].x, rv[u].y, rv[u].z, rv[u].w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              float e = ok[u] ? r[j] : 0.0f;
              if (lazy) e = e * scale;
              acc[j] = __builtin_fmaf(e, qn, acc[j]);
              const float outer = qn * vv[j];
              e = e + outer;
              if (alibi) e = e * dec;  // src/model/bdh.rs:299-301
              r[j] = e;
            }
            if (ok[u] && has_c)
              bdh_rho_store4(rho + (size_t)(row0 + base + src[u]) * d + coff, make_float4(r[0], r[1], r[2], r[3]));
          }
        }
        if (lazy && touch_l) st[r_l] = (int32_t)min(pos + 1, 0x7fffffffL);
      }
      // the rows of one instruction sit side by side in the wave: fold them onto the first LPR lanes
#pragma unroll
      for (int o = LPR; o < 64; o <<= 1)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[j] += __shfl_xor(acc[j], o, 64);
      if (sub == 0 && has_c) {
#pragma unroll
        for (int j = 0; j < 4; ++j) s_red[wave][cl * 4 + j] = acc[j];
      }
    }
    __syncthreads();
    for (int i = tid; i < h * d; i += kThreads) {  // the waves of a head, in order
      const int hh = i / d, c = i - hh * d;
      float s = s_red[hh * wph][c];
      for (int w = 1; w < wph; ++w) s += s_red[hh * wph + w][c];
      s_attn[i] = s;
    }
    __syncthreads();
    // LayerNorm of each head's readout: wave hh takes head hh
    if (wave < h) {
      float v[4], s = 0.0f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v[j] = (lane + 64 * j < d) ? s_attn[wave * d + lane + 64 * j] : 0.0f;
        s += v[j];
      }
      const float mean = wave_sum(s) / (float)d;
      float q = 0.0f;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (lane + 64 * j < d) {
          const float c = v[j] - mean;
          q += c * c;
        }
      const float den = sqrtf(wave_sum(q) / (float)d + kLnEps);
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (lane + 64 * j < d) s_attn[wave * d + lane + 64 * j] = (v[j] - mean) / den;
    }
    __syncthreads();

    // xy = x * relu(LN(attn) . encoder_v - thr)
    project(s_attn, d, a.enc_v, d, N, cols, a.thr, s_x, s_xy);
    __syncthreads();

    // cur = LN(cur + LN(xy . decoder))  (src/model/bdh.rs:383, 436-441)
    {
      const float mlp = matvec_cols(s_xy, cols, a.dec, d, s_red);
      const bool has = tid < d;
      float mean, den;
      block_ln_stats(mlp, has, d, s_st, mean, den);
      const float z = has ? s_cur[tid] + (mlp - mean) / den : 0.0f;
      block_ln_stats(z, has, d, s_st, mean, den);
      if (has) s_cur[tid] = (z - mean) / den;  // only thread tid reads s_cur[tid] above
    }
    __syncthreads();
  }

  // logits and the greedy token (src/model/bdh.rs:446-449); the lowest index wins ties
  const float logit = matvec_cols(s_cur, d, a.lm_head, V, s_red);
  float best = -INFINITY;
  int arg = 0x7fffffff;
  if (tid < V) {
    a.logits[(long)b * V + tid] = logit;
    if (logit > best) {
      best = logit;
      arg = tid;
    }
  }
  if (!a.next) return;  // uniform
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
    for (int w = 1; w < kWaves; ++w)
      if (s_best[w] > best || (s_best[w] == best && s_arg[w] < arg)) {
        best = s_best[w];
        arg = s_arg[w];
      }
    a.next[b] = arg == 0x7fffffff ? 0 : arg;
  }
}

}  // namespace

bool bdh_model_small_fits(const bdh_model_config &c) {
  const long cols = (long)c.n_head * c.latent;
  const int h = c.n_head;
  if (c.rotary != BDH_ROPE && c.rotary != BDH_ALIBI && c.rotary != BDH_POPE) return false;
  if ((c.n_embd & 3) != 0) return false;  // a lane reads up to four adjacent columns of a state row at once
  if (c.n_embd < 1 || c.n_embd > kMaxD || c.vocab < 1 || c.vocab > kThreads || c.n_layer < 1) return false;
  if (h != 1 && h != 2 && h != 4 && h != 8 && h != 16) return false;
  if (cols < 32 || cols > kMaxCols || (cols % (2 * kWaves)) != 0) return false;  // whole RoPE pairs per wave; PoPE doubles the rows, not the columns
  return true;
}

int bdh_launch_model_small(bdh_model *m, const int64_t *tokens, int B, void *rho, int rho_dtype, int32_t *stamps,
                           int64_t position,
                           const int32_t *positions_dev, float *logits, int64_t *next_tokens) {
  bdh_ctx *ctx = m->ctx;
  const bdh_model_config &c = m->cfg;
  if (!bdh_model_small_fits(c)) return bdh_fail(ctx, BDH_E_SHAPE, "model too large for the one-launch decode step");
  SmallArgs a{};
  a.tokens = tokens;
  a.embed = m->w.embed;
  a.enc = m->w.encoder;
  a.enc_v = m->w.encoder_v;
  a.dec = m->w.decoder;
  a.lm_head = m->w.lm_head;
  a.freqs = m->freqs;
  a.rho = rho;
  a.stamps = stamps;
  a.pos_dev = positions_dev;
  a.pos = (long)position;
  a.logits = logits;
  a.next = next_tokens;
  a.B = B;
  a.d = c.n_embd;
  a.h = c.n_head;
  a.N = c.latent;
  a.V = c.vocab;
  a.L = c.n_layer;
  a.rotary = c.rotary;
  a.thr = c.relu_threshold;
  a.rho_layer_stride = (size_t)B * c.n_head * (c.rotary == BDH_POPE ? 2 : 1) * c.latent * c.n_embd;
  a.stamps_layer_stride = (size_t)B * c.n_head * c.latent;
  if (c.rotary == BDH_ALIBI)
    for (int i = 0; i < c.n_head; ++i) {
      a.decay[i] = expf(-m->slopes[i]);                 // src/model/attention.rs:181-186
      a.log_decay[i] = (float)log((double)a.decay[i]);  // of the rounded factor, as the lazy state step
    }
#define BDH_SMALL(LPR)                                                                                              \
  do {                                                                                                               \
    if (rho_dtype == BDH_BF16)                                                                                       \
      hipLaunchKernelGGL((k_model_step_small<LPR, unsigned short>), dim3((unsigned)B), dim3(kThreads), 0, ctx->stream, a); \
    else                                                                                                             \
      hipLaunchKernelGGL((k_model_step_small<LPR, float>), dim3((unsigned)B), dim3(kThreads), 0, ctx->stream, a);     \
  } while (0)
  if (a.d <= 64)
    BDH_SMALL(16);
  else if (a.d <= 128)
    BDH_SMALL(32);
  else
    BDH_SMALL(64);
#undef BDH_SMALL
  BDH_LAUNCH_CHECK(ctx, "k_model_step_small");
  return BDH_OK;
}
