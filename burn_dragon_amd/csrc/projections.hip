// Dense stages around the state step: ReLU low-rank projections (D_x, D_y), LayerNorm,
// embedding gather, the decoder E with the residual LayerNorms, and lm_head.
// Reference semantics: src/kernel/relu_lowrank.rs:7-37, src/model/bdh.rs:86-89, :319-322,
// :346-350, :370-384, :436-449.
#include "bdh_internal.h"

#include <algorithm>
#include <atomic>
#include <type_traits>

namespace {

constexpr float kLnEps = 1e-5f;  // src/model/bdh.rs:17

// Sum of `v` over a 256-thread workgroup; every thread gets the result.
__device__ __forceinline__ float block_sum_256(float v, float *s_part) {
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  __syncthreads();  // protects s_part against the previous use
  if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6] = v;
  __syncthreads();
  return s_part[0] + s_part[1] + s_part[2] + s_part[3];
}

// ------------------------------------------------------------------------------------
// relu_lowrank: out[b,hh,t,n] = relu(sum_k in[b,hh|0,t,k] w[hh,k,n] + bias - thr) * mask
// One thread per latent column n (coalesced weight rows), RT input rows per workgroup
// staged in LDS, one k-sequential fmaf chain per output.
// ------------------------------------------------------------------------------------
template <int RT, int UK, int NTHR>
__global__ __launch_bounds__(NTHR) void k_relu_lowrank(const float *__restrict__ in, int h_in, int T, int d,
                                                      const float *__restrict__ w, int h, int N,
                                                      const float *__restrict__ bias, float thr,
                                                      const unsigned char *__restrict__ block_active,
                                                      int block_size, int n_blocks,
                                                      const float *__restrict__ gate, float *__restrict__ out,
                                                      int M) {
  extern __shared__ float s_in[];  // [RT][d]
  const int tid = threadIdx.x;
  const int hh = blockIdx.y;
  const int n = blockIdx.x * NTHR + tid;
  const int m0 = blockIdx.z * RT;
  for (int i = tid; i < RT * d; i += NTHR) {
    const int r = i / d, k = i - r * d;
    const int m = m0 + r;
    float val = 0.0f;
    if (m < M) {
      const int b = m / T, t = m - b * T;
      val = in[(((long)b * h_in + (h_in == 1 ? 0 : hh)) * T + t) * d + k];
    }
    s_in[i] = val;
  }
  __syncthreads();
  if (n >= N) return;

  float acc[RT];
#pragma unroll
  for (int r = 0; r < RT; ++r) acc[r] = 0.0f;
  const float *wp = w + (long)hh * d * N + n;
  int k0 = 0;
  for (; k0 + UK <= d; k0 += UK) {
    float wv[UK];
#pragma unroll
    for (int u = 0; u < UK; ++u) wv[u] = wp[(long)(k0 + u) * N];
#pragma unroll
    for (int u = 0; u < UK; ++u)
#pragma unroll
      for (int r = 0; r < RT; ++r) acc[r] = __builtin_fmaf(s_in[r * d + k0 + u], wv[u], acc[r]);
  }
  if (UK > 16) {  // what a large batch leaves over, 16 rows at a time
    for (; k0 + 16 <= d; k0 += 16) {
      float wv[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) wv[u] = wp[(long)(k0 + u) * N];
#pragma unroll
      for (int u = 0; u < 16; ++u)
#pragma unroll
        for (int r = 0; r < RT; ++r) acc[r] = __builtin_fmaf(s_in[r * d + k0 + u], wv[u], acc[r]);
    }
  }
  for (; k0 < d; ++k0) {
    const float wv = wp[(long)k0 * N];
#pragma unroll
    for (int r = 0; r < RT; ++r) acc[r] = __builtin_fmaf(s_in[r * d + k0], wv, acc[r]);
  }

  const float bv = bias ? bias[(long)hh * N + n] : 0.0f;
  float maskv = 1.0f;
  if (block_active) {
    const int blk = n / block_size;
    maskv = (blk < n_blocks && block_active[blk]) ? 1.0f : 0.0f;
  }
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    const int m = m0 + r;
    if (m < M) {
      const int b = m / T, t = m - b * T;
      float p = acc[r];
      if (bias) p = p + bv;
      if (thr != 0.0f) p = p - thr;
      float y = p > 0.0f ? p : 0.0f;
      if (block_active) y = y * maskv;
      const long o = (((long)b * h + hh) * T + t) * N + n;
      if (gate) y = gate[o] * y;
      out[o] = y;
    }
  }
}

// One input row per head that the kernel makes itself (a decode step of one sequence).  The reductions of a layer whose
// inputs come from other CUs -- the sum of the state step's readout partials with its LayerNorm (src/model/bdh.rs:359),
// the sum of the encoder's partials with the two LayerNorms and the residual (:436-441) -- run in front of the
// projection that consumes their result, in every workgroup, behind the workgroup's first UK weight loads: as launches
// of their own each is a launch gap plus a chain of dependent trips to memory.
//   MODE 1: row(hh) = LN(sum_g partial[hh][g][:])                      rows = S partial rows per head
//   MODE 2: row     = LN(cur_old + LN(sum_kb partial[kb][:]))          rows = KBN, the same row for every head;
//           workgroup (0, 0) writes it to cur_new (another buffer than cur_old: other workgroups still read that)
//   MODE 3: row     = LN(embed[tokens[0]][:])   (src/model/bdh.rs:319-322; a token outside [0, V) gives a NaN row, as
//           k_embed_ln does)                      partial = the embedding table, rows = V; written to cur_new too
// The NW waves split the partial rows, a lane owns four adjacent columns of up to four column groups (d <= 1024),
// every wave then finishes the row on its own with wave shuffles (the same arithmetic in every wave and workgroup, so
// all of them hold the same bits).  Then k_relu_lowrank's one k-sequential fmaf chain per output.
struct RowArgs {
  const float *partial;
  int rows;
  const float *cur_old;
  float *cur_new;
  const int64_t *tokens;  // MODE 3
};

template <int MODE, int UK, int NTHR>
__global__ __launch_bounds__(NTHR) void k_relu_lowrank_row1(RowArgs a, int d, const float *__restrict__ w, int h, int N,
                                                           float thr, const float *__restrict__ gate,
                                                           float *__restrict__ out) {
  constexpr int NW = NTHR / 64;
  extern __shared__ float s_row[];  // [d] the finished row | [NW][d] the waves' partial sums
  float *s_in = s_row;
  float *s_grp = s_row + d;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int hh = blockIdx.y;
  const int n = blockIdx.x * NTHR + tid;
  const bool col = n < N;
  const float *wp = w + (long)hh * d * N + (col ? n : 0);
  float wv[UK];
  const float *src = a.partial + (MODE == 1 ? (long)hh * a.rows * d : 0);
  int n_rows = a.rows;
  bool bad_token = false;
  if (MODE == 3) {
    const long tok = a.tokens[0];
    bad_token = tok < 0 || tok >= a.rows;
    src = a.partial + (bad_token ? 0 : tok) * d;
    n_rows = 1;
  }
  const int per = (n_rows + NW - 1) / NW;
  const int r0 = min(n_rows, wave * per), r1 = min(n_rows, r0 + per);
  // Order of the requests (a wavefront has at most 63 memory operations outstanding and they complete in issue order):
  // the first 32 partial rows of the lane's first column group, then the first UK weight rows, so that the row is
  // being made while the weights are on their way (d >= UK).
  const bool head32 = r0 + 32 <= r1;  // uniform over the wave
  float4 t0[32];
  if (head32) {
#pragma unroll
    for (int u = 0; u < 32; ++u) t0[u] = *reinterpret_cast<const float4 *>(src + (long)(r0 + u) * d + lane * 4);
  }
#pragma unroll
  for (int u = 0; u < UK; ++u) wv[u] = wp[(long)u * N];
  float4 res[4];
  if (MODE == 2) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = (j * 64 + lane) * 4;
      res[j] = c < d ? *reinterpret_cast<const float4 *>(a.cur_old + c) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int c = (j * 64 + lane) * 4;
    if (c < d) {
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      int r = r0;
      if (j == 0 && head32) {
#pragma unroll
        for (int u = 0; u < 32; ++u) {
          v.x += t0[u].x; v.y += t0[u].y; v.z += t0[u].z; v.w += t0[u].w;
        }
        r += 32;
      }
      for (; r + 32 <= r1; r += 32) {  // 32 rows in flight: the sum is a chain of trips to the L2
        float4 t[32];
#pragma unroll
        for (int u = 0; u < 32; ++u) t[u] = *reinterpret_cast<const float4 *>(src + (long)(r + u) * d + c);
#pragma unroll
        for (int u = 0; u < 32; ++u) {
          v.x += t[u].x; v.y += t[u].y; v.z += t[u].z; v.w += t[u].w;
        }
      }
      if (r < r1) {  // up to 31 rows left: all asked for at once
        float4 t[31];
#pragma unroll
        for (int u = 0; u < 31; ++u)
          t[u] = r + u < r1 ? *reinterpret_cast<const float4 *>(src + (long)(r + u) * d + c) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int u = 0; u < 31; ++u)
          if (r + u < r1) {
            v.x += t[u].x; v.y += t[u].y; v.z += t[u].z; v.w += t[u].w;
          }
      }
      if (MODE == 3 && bad_token) v = make_float4(NAN, NAN, NAN, NAN);
      *reinterpret_cast<float4 *>(s_grp + wave * d + c) = v;
    }
  }
  __syncthreads();
  {
    auto wave_sum = [](float v) {
      for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
      return v;
    };
    float4 vals[4];
    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = (j * 64 + lane) * 4;
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (c < d) {
        v = *reinterpret_cast<const float4 *>(s_grp + c);
#pragma unroll
        for (int g = 1; g < NW; ++g) {
          const float4 t = *reinterpret_cast<const float4 *>(s_grp + g * d + c);
          v.x += t.x; v.y += t.y; v.z += t.z; v.w += t.w;
        }
        s += (v.x + v.y) + (v.z + v.w);
      }
      vals[j] = v;
    }
    auto layer_norm4 = [&](float total) {  // vals <- (vals - mean) / sqrt(var + eps) over the d columns
      const float mean = wave_sum(total) / (float)d;
      float q = 0.0f;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if ((j * 64 + lane) * 4 < d) {
          const float tx = vals[j].x - mean, ty = vals[j].y - mean, tz = vals[j].z - mean, tw = vals[j].w - mean;
          q += (tx * tx + ty * ty) + (tz * tz + tw * tw);
        }
      const float den = sqrtf(wave_sum(q) / (float)d + kLnEps);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        vals[j].x = (vals[j].x - mean) / den; vals[j].y = (vals[j].y - mean) / den;
        vals[j].z = (vals[j].z - mean) / den; vals[j].w = (vals[j].w - mean) / den;
      }
    };
    layer_norm4(s);
    if (MODE == 2) {
      s = 0.0f;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if ((j * 64 + lane) * 4 < d) {
          vals[j].x += res[j].x; vals[j].y += res[j].y; vals[j].z += res[j].z; vals[j].w += res[j].w;
          s += (vals[j].x + vals[j].y) + (vals[j].z + vals[j].w);
        }
      layer_norm4(s);
    }
    if (wave == 0) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int c = (j * 64 + lane) * 4;
        if (c < d) {
          *reinterpret_cast<float4 *>(s_in + c) = vals[j];
          if (MODE != 1 && blockIdx.x == 0 && hh == 0) *reinterpret_cast<float4 *>(a.cur_new + c) = vals[j];
        }
      }
    }
  }
  __syncthreads();

  float acc = 0.0f;
#pragma unroll
  for (int u = 0; u < UK; ++u) acc = __builtin_fmaf(s_in[u], wv[u], acc);
  int k0 = UK;
  for (; k0 + UK <= d; k0 += UK) {
#pragma unroll
    for (int u = 0; u < UK; ++u) wv[u] = wp[(long)(k0 + u) * N];
#pragma unroll
    for (int u = 0; u < UK; ++u) acc = __builtin_fmaf(s_in[k0 + u], wv[u], acc);
  }
  for (; k0 < d; ++k0) acc = __builtin_fmaf(s_in[k0], wp[(long)k0 * N], acc);
  if (!col) return;
  float pv = acc;
  if (thr != 0.0f) pv = pv - thr;
  float y = pv > 0.0f ? pv : 0.0f;
  const long o = (long)hh * N + n;
  if (gate) y = gate[o] * y;
  out[o] = y;
}

// A few input rows against a SMALL weight matrix (a few MiB: it sits in the L2): with one thread per column there
// are only a handful of workgroups and each thread walks k in rounds of loads.  Here NW waves share 64
// columns: each wave asks for its own 64-row span of k at once, so every weight of the matrix is in flight
// together, and the waves then extend the column's fmaf chain one after the other in k order (the accumulator
// is handed on through LDS) -- the same k-sequential chain per output as k_relu_lowrank.  Measured per decode
// step of a whole model: 4 x 1 MiB (d=256) 141 -> 132 us, 8 x 4 MiB (d=512) 389 -> 317 us; 32 MiB a tie; at
// 256 MiB the column-per-thread kernel is 1 % ahead, hence the size limit at the call site.
template <int NW, int RT>
__global__ __launch_bounds__(NW * 64) void k_relu_lowrank_row(const float *__restrict__ in, int h_in, int T, int d,
                                                             const float *__restrict__ w, int h, int N,
                                                             const float *__restrict__ bias, float thr,
                                                             const unsigned char *__restrict__ block_active,
                                                             int block_size, int n_blocks,
                                                             const float *__restrict__ gate, float *__restrict__ out,
                                                             int M) {
  __shared__ float s_in[RT][NW * 64];
  __shared__ float s_acc[RT][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int hh = blockIdx.y;
  const int n = blockIdx.x * 64 + lane;
  const int m0 = blockIdx.z * RT;
  const bool valid = n < N;
  const int k_lo = wave * 64;
  // loads return in issue order: the input rows first, they are needed first
  float xin[RT];
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    const int m = m0 + r;
    xin[r] = 0.0f;
    if ((int)threadIdx.x < d && m < M) {
      const int b = m / T, t = m - b * T;
      xin[r] = in[(((long)b * h_in + (h_in == 1 ? 0 : hh)) * T + t) * d + threadIdx.x];
    }
  }
  // unconditional loads (rows past d are clamped to the last one and not used): a load under a branch would
  // be waited for before the next one is issued
  const float *wp = w + (long)hh * d * N + (valid ? n : 0);
  float wv[64];
#pragma unroll
  for (int u = 0; u < 64; ++u) {
    const float t = wp[(long)min(k_lo + u, d - 1) * N];
    wv[u] = k_lo + u < d ? t : 0.0f;  // a select, not a branch; s_in is zero there too, so the term is +0
  }
  float gv[RT], bv = 0.0f;
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    const int m = m0 + r;
    gv[r] = 1.0f;
    if (wave == NW - 1 && valid && gate && m < M) {
      const int b = m / T, t = m - b * T;
      gv[r] = gate[(((long)b * h + hh) * T + t) * N + n];
    }
  }
  if (wave == NW - 1 && valid && bias) bv = bias[(long)hh * N + n];
#pragma unroll
  for (int r = 0; r < RT; ++r) s_in[r][threadIdx.x] = xin[r];
  __syncthreads();
  float acc[RT];
#pragma unroll
  for (int r = 0; r < RT; ++r) acc[r] = 0.0f;
#pragma unroll
  for (int stage = 0; stage < NW; ++stage) {
    if (wave == stage) {
      if (stage > 0) {
#pragma unroll
        for (int r = 0; r < RT; ++r) acc[r] = s_acc[r][lane];
      }
      // unconditional, so that the LDS reads of the inputs are issued together
#pragma unroll
      for (int u = 0; u < 64; ++u)
#pragma unroll
        for (int r = 0; r < RT; ++r) acc[r] = __builtin_fmaf(s_in[r][k_lo + u], wv[u], acc[r]);
      if (stage < NW - 1) {
#pragma unroll
        for (int r = 0; r < RT; ++r) s_acc[r][lane] = acc[r];
      }
    }
    if (stage < NW - 1) __syncthreads();
  }
  if (wave != NW - 1 || !valid) return;
  float maskv = 1.0f;
  if (block_active) {
    const int blk = n / block_size;
    maskv = (blk < n_blocks && block_active[blk]) ? 1.0f : 0.0f;
  }
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    const int m = m0 + r;
    if (m < M) {
      const int b = m / T, t = m - b * T;
      float p = acc[r];
      if (bias) p = p + bv;
      if (thr != 0.0f) p = p - thr;
      float y = p > 0.0f ? p : 0.0f;
      if (block_active) y = y * maskv;
      if (gate) y = gv[r] * y;
      out[(((long)b * h + hh) * T + t) * N + n] = y;
    }
  }
}

// A few input rows (a batch of 8 to 63 sequences decoding together) without LDS: the inputs of a row tile
// are the same for every lane, so they are read through the scalar cache (wave-uniform addresses, read
// only) and feed the FMAs as scalar operands; the vector memory pipe carries only the weights.  With the
// inputs staged in LDS instead, three quarters of the wave wait cycles were waits for the broadcast reads.
// Same k-sequential fmaf chain per output as k_relu_lowrank.
template <int RT, int UK>
__global__ __launch_bounds__(256) void k_relu_lowrank_sc(const float *__restrict__ in, int h_in, int T, int d,
                                                        const float *__restrict__ w, int h, int N,
                                                        const float *__restrict__ bias, float thr,
                                                        const unsigned char *__restrict__ block_active,
                                                        int block_size, int n_blocks,
                                                        const float *__restrict__ gate, float *__restrict__ out,
                                                        int M) {
  const int hh = blockIdx.y;
  const int n = blockIdx.x * 256 + threadIdx.x;
  const int m0 = blockIdx.z * RT;
  if (n >= N) return;
  const float *rows[RT];  // wave-uniform row pointers (rows past M alias the last valid row; never stored)
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    const int m = min(m0 + r, M - 1);
    const int b = m / T, t = m - b * T;
    rows[r] = in + (((long)b * h_in + (h_in == 1 ? 0 : hh)) * T + t) * d;
  }
  float acc[RT];
#pragma unroll
  for (int r = 0; r < RT; ++r) acc[r] = 0.0f;
  const float *wp = w + (long)hh * d * N + n;
  int k0 = 0;
  for (; k0 + UK <= d; k0 += UK) {
    float wv[UK];
#pragma unroll
    for (int u = 0; u < UK; ++u) wv[u] = wp[(long)(k0 + u) * N];
#pragma unroll
    for (int r = 0; r < RT; ++r) {
#pragma unroll
      for (int u = 0; u < UK; ++u) acc[r] = __builtin_fmaf(rows[r][k0 + u], wv[u], acc[r]);
    }
  }
  for (; k0 < d; ++k0) {
    const float wv = wp[(long)k0 * N];
#pragma unroll
    for (int r = 0; r < RT; ++r) acc[r] = __builtin_fmaf(rows[r][k0], wv, acc[r]);
  }
  const float bv = bias ? bias[(long)hh * N + n] : 0.0f;
  float maskv = 1.0f;
  if (block_active) {
    const int blk = n / block_size;
    maskv = (blk < n_blocks && block_active[blk]) ? 1.0f : 0.0f;
  }
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    const int m = m0 + r;
    if (m < M) {
      const int b = m / T, t = m - b * T;
      float p = acc[r];
      if (bias) p = p + bv;
      if (thr != 0.0f) p = p - thr;
      float y = p > 0.0f ? p : 0.0f;
      if (block_active) y = y * maskv;
      const long o = (((long)b * h + hh) * T + t) * N + n;
      if (gate) y = gate[o] * y;
      out[o] = y;
    }
  }
}

// Many input rows (a prompt, a large batch): a 64-row x 256-column tile per workgroup, 16 rows x 4
// adjacent columns per thread.  Wave w owns rows 16w..16w+15, so an input value is one LDS broadcast
// for the whole wave; a weight row segment is one float4 per lane.  The inputs are staged 64 k at a
// time.  Every output is still one k-sequential fmaf chain, so the values are those of k_relu_lowrank
// bit for bit; the tile only cuts the weight re-reads from one per 8 rows to one per 64.
__global__ __launch_bounds__(256) void k_relu_lowrank_tile(const float *__restrict__ in, int h_in, int T, int d,
                                                          const float *__restrict__ w, int h, int N,
                                                          const float *__restrict__ bias, float thr,
                                                          const unsigned char *__restrict__ block_active,
                                                          int block_size, int n_blocks,
                                                          const float *__restrict__ gate, float *__restrict__ out,
                                                          int M) {
  constexpr int RT = 16, KC = 64;
  __shared__ __attribute__((aligned(16))) float s_x[64 * KC];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int hh = blockIdx.y;
  const int n = (blockIdx.x * 64 + lane) * 4;  // N % 4 == 0: a thread's four columns are all in or all out
  const int m0 = blockIdx.z * 64;
  const bool live = n < N;

  float4 acc[RT];
#pragma unroll
  for (int r = 0; r < RT; ++r) acc[r] = make_float4(0.f, 0.f, 0.f, 0.f);
  const float *wp = w + (long)hh * d * N + (live ? n : 0);
  const float *sx = s_x + wave * RT * KC;
  for (int kc = 0; kc < d; kc += KC) {  // d % 4 == 0
    const int kn = min(KC, d - kc);
    __syncthreads();
    for (int i = tid; i < 64 * KC / 4; i += 256) {
      const int r = i / (KC / 4), k4 = (i - r * (KC / 4)) * 4;
      const int m = m0 + r;
      float4 val = make_float4(0.f, 0.f, 0.f, 0.f);
      if (m < M && k4 < kn) {
        const int b = m / T, t = m - b * T;
        val = *reinterpret_cast<const float4 *>(in + (((long)b * h_in + (h_in == 1 ? 0 : hh)) * T + t) * d + kc + k4);
      }
      *reinterpret_cast<float4 *>(s_x + r * KC + k4) = val;
    }
    __syncthreads();
    if (live) {
      for (int k0 = 0; k0 < kn; k0 += 4) {
        float4 wv[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) wv[u] = *reinterpret_cast<const float4 *>(wp + (long)(kc + k0 + u) * N);
#pragma unroll
        for (int r = 0; r < RT; ++r) {
          const float4 xin = *reinterpret_cast<const float4 *>(sx + r * KC + k0);
          const float xs[4] = {xin.x, xin.y, xin.z, xin.w};
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            acc[r].x = __builtin_fmaf(xs[u], wv[u].x, acc[r].x);
            acc[r].y = __builtin_fmaf(xs[u], wv[u].y, acc[r].y);
            acc[r].z = __builtin_fmaf(xs[u], wv[u].z, acc[r].z);
            acc[r].w = __builtin_fmaf(xs[u], wv[u].w, acc[r].w);
          }
        }
      }
    }
  }
  if (!live) return;
  float4 bv = make_float4(0.f, 0.f, 0.f, 0.f);
  if (bias) bv = *reinterpret_cast<const float4 *>(bias + (long)hh * N + n);
  float mk[4] = {1.f, 1.f, 1.f, 1.f};
  if (block_active)
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int blk = (n + c) / block_size;
      mk[c] = (blk < n_blocks && block_active[blk]) ? 1.0f : 0.0f;
    }
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    const int m = m0 + wave * RT + r;
    if (m < M) {
      const int b = m / T, t = m - b * T;
      const long o = (((long)b * h + hh) * T + t) * N + n;
      float p[4] = {acc[r].x, acc[r].y, acc[r].z, acc[r].w};
      const float bb[4] = {bv.x, bv.y, bv.z, bv.w};
      float4 gv = make_float4(1.f, 1.f, 1.f, 1.f);
      if (gate) gv = *reinterpret_cast<const float4 *>(gate + o);
      const float gg[4] = {gv.x, gv.y, gv.z, gv.w};
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        if (bias) p[c] = p[c] + bb[c];
        if (thr != 0.0f) p[c] = p[c] - thr;
        float y = p[c] > 0.0f ? p[c] : 0.0f;
        if (block_active) y = y * mk[c];
        if (gate) y = gg[c] * y;
        p[c] = y;
      }
      *reinterpret_cast<float4 *>(out + o) = make_float4(p[0], p[1], p[2], p[3]);
    }
  }
}

// ------------------------------------------------------------------------------------
// LayerNorm rows (one workgroup per row); in == out allowed.  The row is staged in LDS and
// every thread walks it in index order, so mean and variance are the same left-to-right f32
// sums a scalar loop produces, independent of the launch shape.
// ------------------------------------------------------------------------------------
// (s_row is 16-byte aligned; four values per LDS read, added one after the other in index order)
__device__ __forceinline__ void ln_stats_in_order(const float *s_row, int d, float &mean, float &den) {
  float sum = 0.0f;
  int i = 0;
#pragma unroll 4
  for (; i + 4 <= d; i += 4) {
    const float4 v = *reinterpret_cast<const float4 *>(s_row + i);
    sum += v.x;
    sum += v.y;
    sum += v.z;
    sum += v.w;
  }
  for (; i < d; ++i) sum += s_row[i];
  mean = sum / (float)d;
  float sq = 0.0f;
  i = 0;
#pragma unroll 4
  for (; i + 4 <= d; i += 4) {
    const float4 v = *reinterpret_cast<const float4 *>(s_row + i);
    float c;
    c = v.x - mean; sq += c * c;
    c = v.y - mean; sq += c * c;
    c = v.z - mean; sq += c * c;
    c = v.w - mean; sq += c * c;
  }
  for (; i < d; ++i) {
    const float c = s_row[i] - mean;
    sq += c * c;
  }
  den = sqrtf(sq / (float)d + kLnEps);
}

__global__ __launch_bounds__(256) void k_layer_norm(const float *__restrict__ in, float *__restrict__ out, int d) {
  extern __shared__ float s_row[];
  const float *x = in + (long)blockIdx.x * d;
  float *y = out + (long)blockIdx.x * d;
  for (int c = threadIdx.x; c < d; c += 256) s_row[c] = x[c];
  __syncthreads();
  float mean, den;
  ln_stats_in_order(s_row, d, mean, den);
  for (int c = threadIdx.x; c < d; c += 256) y[c] = (s_row[c] - mean) / den;
}

// LayerNorm of many rows for internal use (the readout of a many-token state step): one wave per row, the
// statistics by wave reduction instead of the index-order sums above (d <= 1024)
__global__ __launch_bounds__(256) void k_layer_norm_wave(const float *__restrict__ in, float *__restrict__ out, int d,
                                                         long rows) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const long row = (long)blockIdx.x * 4 + wave;
  if (row >= rows) return;
  const float *x = in + row * d;
  float *y = out + row * d;
  float v[16], s = 0.0f;
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    const int c = j * 64 + lane;
    v[j] = c < d ? x[c] : 0.0f;
    s += v[j];
  }
  for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
  const float mean = s / (float)d;
  float q = 0.0f;
#pragma unroll
  for (int j = 0; j < 16; ++j)
    if (j * 64 + lane < d) {
      const float c = v[j] - mean;
      q += c * c;
    }
  for (int o = 32; o > 0; o >>= 1) q += __shfl_xor(q, o);
  const float den = sqrtf(q / (float)d + kLnEps);
#pragma unroll
  for (int j = 0; j < 16; ++j)
    if (j * 64 + lane < d) y[j * 64 + lane] = (v[j] - mean) / den;
}

// embed gather + LayerNorm (src/model/bdh.rs:319-322)
__global__ __launch_bounds__(256) void k_embed_ln(const int64_t *__restrict__ tokens, int d, int V,
                                                  const float *__restrict__ embed, float *__restrict__ out) {
  extern __shared__ float s_row[];
  const int64_t tok = tokens[blockIdx.x];
  float *y = out + (long)blockIdx.x * d;
  if (tok < 0 || tok >= V) {  // the reference's gather would panic; poison the row instead
    for (int c = threadIdx.x; c < d; c += 256) y[c] = __int_as_float(0x7fc00000);
    return;
  }
  const float *x = embed + (long)tok * d;
  for (int c = threadIdx.x; c < d; c += 256) s_row[c] = x[c];
  __syncthreads();
  float mean, den;
  ln_stats_in_order(s_row, d, mean, den);
  for (int c = threadIdx.x; c < d; c += 256) y[c] = (s_row[c] - mean) / den;
}

// ------------------------------------------------------------------------------------
// decoder: partial[kb][m][:] = sum_{k in block kb} mixed[m,k] * E[k,:]
// mixed[m = b*T+t, k = hh*N+n] = xy[b,hh,t,n].  Rows of E whose xy is zero for every row
// of the tile are never loaded.
// ------------------------------------------------------------------------------------
template <int RT, int MAXV, int UF = 4>
__global__ __launch_bounds__(256) void k_decoder_partial(const float *__restrict__ xy,
                                                         const float *__restrict__ E,
                                                         float *__restrict__ partial, int T, int h, int N,
                                                         int d, int KB, int M) {
  extern __shared__ float s_mem[];  // [RT][KB] xy tile, then reused for the wave reduction
  // MAXV float4 column groups per lane: columns c = (j*64+lane)*4, d <= 256*MAXV
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int kb = blockIdx.x;
  const int m0 = blockIdx.y * RT;
  const int K = h * N;
  const int nv = (d + 255) >> 8;  // float4 groups per lane
  float *s_xy = s_mem;
  for (int i = tid; i < RT * KB; i += 256) {
    const int r = i / KB, kk = i - r * KB;
    const int m = m0 + r, k = kb * KB + kk;
    float val = 0.0f;
    if (m < M && k < K) {
      const int b = m / T, t = m - b * T;
      const int hh = k / N, n = k - hh * N;
      val = xy[(((long)b * h + hh) * T + t) * N + n];
    }
    s_xy[i] = val;
  }
  __syncthreads();

  float4 acc[RT][MAXV];
#pragma unroll
  for (int r = 0; r < RT; ++r)
#pragma unroll
    for (int j = 0; j < MAXV; ++j) acc[r][j] = make_float4(0.f, 0.f, 0.f, 0.f);

  // each wave takes k = wave, wave+4, ...; UF of its E rows are in flight at a time
  for (int kk0 = wave; kk0 < KB; kk0 += 4 * UF) {
    float xs[UF][RT];
    bool any[UF];
    float4 e[UF][MAXV];
#pragma unroll
    for (int u = 0; u < UF; ++u) {
      const int kk = kk0 + 4 * u;
      const int k = kb * KB + kk;
      any[u] = false;
      if (kk < KB && k < K) {
#pragma unroll
        for (int r = 0; r < RT; ++r) {
          xs[u][r] = s_xy[r * KB + kk];
          any[u] = any[u] || (xs[u][r] != 0.0f);
        }
      }
      if (any[u]) {
        const float *erow = E + (long)k * d;
#pragma unroll
        for (int j = 0; j < MAXV; ++j) {
          const int c = (j * 64 + lane) * 4;
          if (j < nv && c < d) e[u][j] = *reinterpret_cast<const float4 *>(erow + c);
        }
      }
    }
#pragma unroll
    for (int u = 0; u < UF; ++u) {
      if (any[u]) {
#pragma unroll
        for (int j = 0; j < MAXV; ++j) {
          const int c = (j * 64 + lane) * 4;
          if (j < nv && c < d) {
#pragma unroll
            for (int r = 0; r < RT; ++r) {
              acc[r][j].x = __builtin_fmaf(xs[u][r], e[u][j].x, acc[r][j].x);
              acc[r][j].y = __builtin_fmaf(xs[u][r], e[u][j].y, acc[r][j].y);
              acc[r][j].z = __builtin_fmaf(xs[u][r], e[u][j].z, acc[r][j].z);
              acc[r][j].w = __builtin_fmaf(xs[u][r], e[u][j].w, acc[r][j].w);
            }
          }
        }
      }
    }
  }
  __syncthreads();
  // cross-wave reduction, one row of the tile at a time, through LDS [4][d]
  float *s_red = s_mem;
  for (int r = 0; r < RT; ++r) {
#pragma unroll
    for (int j = 0; j < MAXV; ++j) {
      const int c = (j * 64 + lane) * 4;
      if (j < nv && c < d) *reinterpret_cast<float4 *>(s_red + wave * d + c) = acc[r][j];
    }
    __syncthreads();
    const int m = m0 + r;
    if (m < M)
      for (int c = tid; c < d; c += 256)
        partial[((long)kb * M + m) * d + c] = s_red[c] + s_red[d + c] + s_red[2 * d + c] + s_red[3 * d + c];
    __syncthreads();
  }
}

// The encoder's first stage for ONE row (a decode step of one sequence): partial[kb][:] = sum over the KB rows of
// k-block kb of xy[k] * E[k,:], rows whose xy is zero never loaded.  Grid (k-blocks, column parts): a workgroup of NWV
// waves owns 64 * VW adjacent columns, a lane VW of them; wave w takes k = w, w + NWV, ... with UF rows in flight.
// More column parts mean fewer, larger k-blocks for the same number of waves in flight -- fewer partial rows for the
// consumer to add.
template <int VW, int UF, int NWV>
__global__ __launch_bounds__(NWV * 64) void k_decoder_partial_row(const float *__restrict__ xy,
                                                                  const float *__restrict__ E,
                                                                  float *__restrict__ partial, long K, int d, int KB) {
  extern __shared__ float s_mem[];  // [KB] xy of the block, then [NWV][64 * VW] for the wave reduction
  typedef float vec_t __attribute__((ext_vector_type(VW)));
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int kb = blockIdx.x;
  const int c = (blockIdx.y * 64 + lane) * VW;
  for (int i = tid; i < KB; i += NWV * 64) {
    const long k = (long)kb * KB + i;
    s_mem[i] = k < K ? xy[k] : 0.0f;
  }
  __syncthreads();
  float acc[VW];
#pragma unroll
  for (int e = 0; e < VW; ++e) acc[e] = 0.0f;
  for (int kk0 = wave; kk0 < KB; kk0 += NWV * UF) {
    float xs[UF];
    vec_t ev[UF];
#pragma unroll
    for (int u = 0; u < UF; ++u) {
      const int kk = kk0 + NWV * u;
      xs[u] = kk < KB ? s_mem[kk] : 0.0f;
      if (xs[u] != 0.0f && c < d) ev[u] = *reinterpret_cast<const vec_t *>(E + ((long)kb * KB + kk) * d + c);
    }
#pragma unroll
    for (int u = 0; u < UF; ++u)
      if (xs[u] != 0.0f && c < d) {
#pragma unroll
        for (int e = 0; e < VW; ++e) acc[e] = __builtin_fmaf(xs[u], ev[u][e], acc[e]);
      }
  }
  __syncthreads();
  float *s_red = s_mem;
#pragma unroll
  for (int e = 0; e < VW; ++e) s_red[wave * 64 * VW + lane * VW + e] = acc[e];
  __syncthreads();
  for (int j = tid; j < 64 * VW; j += NWV * 64) {
    const int cc = blockIdx.y * 64 * VW + j;
    if (cc < d) {
      float v = s_red[j];
#pragma unroll
      for (int g = 1; g < NWV; ++g) v += s_red[g * 64 * VW + j];
      partial[(long)kb * d + cc] = v;
    }
  }
}

// logits[m,:] = cur[m,:] . lm_head ; optional argmax of the last token of each sequence.
// 1024 threads: 256 vocabulary columns x 4 groups over k; the four partial dot products of a
// logit are added in group order.  s_cur holds the input row (every thread sees it), s_acc has 1024 floats.
__device__ __forceinline__ void lm_head_row(const float *s_cur, float *s_acc, float *s_best, int *s_arg, int m,
                                            const float *__restrict__ W, int T, int d, int V,
                                            float *__restrict__ logits, int64_t *__restrict__ next_tokens) {
  const int tid = threadIdx.x & 255, grp = threadIdx.x >> 8;
  const int lane = tid & 63, wave = tid >> 6;
  const int per = (d + 3) >> 2;
  const int k0 = grp * per, k1 = min(d, k0 + per);
  float best = -INFINITY;
  int arg = 0x7fffffff;
  for (int c0 = 0; c0 < V; c0 += 256) {
    const int c = c0 + tid;
    float acc = 0.0f;
    if (c < V) {
      int k = k0;
      for (; k + 16 <= k1; k += 16) {  // 16 independent loads in flight, then the chain
        float w[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) w[u] = W[(long)(k + u) * V + c];
#pragma unroll
        for (int u = 0; u < 16; ++u) acc = __builtin_fmaf(s_cur[k + u], w[u], acc);
      }
      for (; k < k1; ++k) acc = __builtin_fmaf(s_cur[k], W[(long)k * V + c], acc);
    }
    s_acc[grp * 256 + tid] = acc;
    __syncthreads();
    if (grp == 0 && c < V) {
      const float v = ((s_acc[tid] + s_acc[256 + tid]) + s_acc[512 + tid]) + s_acc[768 + tid];
      logits[(long)m * V + c] = v;
      if (v > best) {  // increasing c: keeps the lowest index on ties
        best = v;
        arg = c;
      }
    }
    __syncthreads();
  }
  const int b = m / T, t = m - b * T;
  const bool want = next_tokens && t == T - 1;  // uniform over the workgroup
  if (!want) return;
  for (int o = 32; o > 0; o >>= 1) {
    const float ob = __shfl_xor(best, o);
    const int oa = __shfl_xor(arg, o);
    if (ob > best || (ob == best && oa < arg)) {
      best = ob;
      arg = oa;
    }
  }
  if (grp == 0 && lane == 0) {
    s_best[wave] = best;
    s_arg[wave] = arg;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w)
      if (s_best[w] > best || (s_best[w] == best && s_arg[w] < arg)) {
        best = s_best[w];
        arg = s_arg[w];
      }
    next_tokens[b] = arg == 0x7fffffff ? 0 : arg;
  }
}

// cur[m,:] = LN(cur[m,:] + LN(sum_kb partial[kb][m][:]))   (src/model/bdh.rs:438-441)
// 1024 threads = 16 groups of 64 lanes; a lane owns four adjacent columns (one 16-byte load per partial
// row), a group adds a sixteenth of the k-block partials in index order with up to 16 loads in flight,
// the groups are combined in order; after the one barrier the first wavefront applies the two LayerNorms
// with wave shuffles only.
// HEAD: the output head of the same row follows in the same launch (the last layer of a model): the finished row
// goes to LDS as well, and all 1024 threads run lm_head_row on it -- the arithmetic of k_lm_head, one launch less.
template <bool HEAD>
__global__ __launch_bounds__(1024) void k_decoder_finalize(const float *__restrict__ partial, int KBN, int M,
                                                           int d, float *__restrict__ cur, DecoderHead head) {
  __shared__ float s_grp[16][1024];
  __shared__ float s_best[4];
  __shared__ int s_arg[4];
  const int m = blockIdx.x, lane = threadIdx.x & 63, grp = threadIdx.x >> 6;
  const int per = (KBN + 15) >> 4;
  const int kb0 = min(KBN, grp * per), kb1 = min(KBN, kb0 + per);
  // the residual row is fetched while the partials are summed: it was written by another
  // workgroup of an earlier launch, so the load is a trip to memory
  float res[16];
  if (grp == 0) {
#pragma unroll
    for (int j = 0; j < 16; ++j) res[j] = (j * 64 + lane < d) ? cur[(long)m * d + j * 64 + lane] : 0.0f;
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int c = (j * 64 + lane) * 4;  // d % 4 == 0
    if (c < d) {
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      int kb = kb0;
      for (; kb + 16 <= kb1; kb += 16) {
        float4 t[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) t[u] = *reinterpret_cast<const float4 *>(partial + ((long)(kb + u) * M + m) * d + c);
#pragma unroll
        for (int u = 0; u < 16; ++u) {
          v.x += t[u].x; v.y += t[u].y; v.z += t[u].z; v.w += t[u].w;
        }
      }
      for (; kb < kb1; ++kb) {
        const float4 t = *reinterpret_cast<const float4 *>(partial + ((long)kb * M + m) * d + c);
        v.x += t.x; v.y += t.y; v.z += t.z; v.w += t.w;
      }
      *reinterpret_cast<float4 *>(&s_grp[grp][c]) = v;
    }
  }
  __syncthreads();
  if (threadIdx.x >= 64) {  // the first wave finishes the row alone
    if (!HEAD) return;      // (no barrier follows)
  } else {
  float vals[16];  // column c = j*64 + lane, d <= 1024
  float s = 0.0f;
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    const int c = j * 64 + lane;
    float v = 0.0f;
    if (c < d) {
      v = s_grp[0][c];
#pragma unroll
      for (int g = 1; g < 16; ++g) v += s_grp[g][c];
      s += v;
    }
    vals[j] = v;
  }
  auto wave_sum = [](float v) {
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
  };
  float mean = wave_sum(s) / (float)d;
  float q = 0.0f;
#pragma unroll
  for (int j = 0; j < 16; ++j)
    if (j * 64 + lane < d) {
      const float t = vals[j] - mean;
      q += t * t;
    }
  float den = sqrtf(wave_sum(q) / (float)d + kLnEps);
  s = 0.0f;
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    const int c = j * 64 + lane;
    if (c < d) {
      const float mlp = (vals[j] - mean) / den;
      vals[j] = res[j] + mlp;
      s += vals[j];
    }
  }
  mean = wave_sum(s) / (float)d;
  q = 0.0f;
#pragma unroll
  for (int j = 0; j < 16; ++j)
    if (j * 64 + lane < d) {
      const float t = vals[j] - mean;
      q += t * t;
    }
  den = sqrtf(wave_sum(q) / (float)d + kLnEps);
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    const int c = j * 64 + lane;
    if (c < d) {
      const float y = (vals[j] - mean) / den;
      cur[(long)m * d + c] = y;
      if (HEAD) s_grp[2][c] = y;  // only this wave reads s_grp after the barrier above, and it has read all of it
    }
  }
  }
  if (!HEAD) return;
  __syncthreads();  // the row is in s_grp[2]; rows 3.. are free for the partial dot products
  lm_head_row(s_grp[2], s_grp[3], s_best, s_arg, m, head.lm_head, head.T, d, head.V, head.logits, head.next_tokens);
}

__global__ __launch_bounds__(1024) void k_lm_head(const float *__restrict__ cur, const float *__restrict__ W,
                                                  int T, int d, int V, float *__restrict__ logits,
                                                  int64_t *__restrict__ next_tokens) {
  extern __shared__ float s_dyn[];  // [d] input row, then [4][256] partials
  __shared__ float s_best[4];
  __shared__ int s_arg[4];
  const int m = blockIdx.x;
  for (int k = threadIdx.x; k < d; k += 1024) s_dyn[k] = cur[(long)m * d + k];
  __syncthreads();
  lm_head_row(s_dyn, s_dyn + d, s_best, s_arg, m, W, T, d, V, logits, next_tokens);
}

__global__ void k_advance_positions(int32_t *pos, int B, int delta) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b < B) {
    const long v = (long)pos[b] + delta;
    pos[b] = v > 0x7fffffffL ? 0x7fffffff : (int32_t)v;  // saturating, as state.position (src/model/bdh.rs:445)
  }
}

template <int RT>
void launch_relu(hipStream_t st, dim3 grid, size_t lds, const ReluLowrankParams &p, const unsigned char *mask,
                 int M) {
  constexpr int UK = RT == 1 ? 64 : 16;      // weight rows in flight per thread (the counter of outstanding loads ends at 63)
  constexpr int NTHR = RT == 1 ? 128 : 256;  // a single input row: smaller workgroups, one per CU at N*h = 32768
  grid.x = (p.N + NTHR - 1) / NTHR;
  hipLaunchKernelGGL((k_relu_lowrank<RT, UK, NTHR>), grid, dim3(NTHR), lds, st, p.in, p.h_in, p.T, p.d, p.weight,
                     p.h, p.N, p.bias, p.threshold, mask, p.block_size, p.n_blocks, p.gate, p.out, M);
}

// ------------------------------------------------------------------------------------
// relu_lowrank on the f32 matrix cores, for 8 rows and more.  v_mfma_f32_32x32x2_f32 adds its two k-steps one
// after the other, each as one fused multiply-add, so a chain of these instructions over k = 0, 1, 2, ... is the
// same k-sequential fmaf chain per output as k_relu_lowrank computes, bit for bit (checked on the device against
// the scalar chain, including denormal results): the active sets do not change, the weights are streamed once
// for up to 32 * RT rows, and the arithmetic runs at the matrix rate.
//   A operand (32 rows x 2 k): lane l holds in[row l % 32][k0 + l / 32], from an LDS copy of the input rows laid
//   out [k][row]; B operand (2 k x 32 columns): lane l holds w[k0 + l / 32][column].  A lane loads four adjacent
//   columns of a weight row at once (16 bytes, a wavefront reads two 512-byte row pieces per k-pair) and uses
//   them in four matrix instructions: instruction j owns the columns n0 + 4 c + j, c = 0..31, so that the four
//   results a lane holds for a row are again four adjacent columns (16-byte stores).
// One workgroup = NW wavefronts x 128 columns; grid (column blocks, heads, row groups of 32 * RT).  Each wavefront
// asks for its first UK k-pairs of weights before the input rows are staged, so the staging hides behind them.
// ------------------------------------------------------------------------------------
typedef float f32x16_t __attribute__((ext_vector_type(16)));

template <int RT, int UK, int NW>  // RT row tiles of 32 rows per workgroup; UK k-pairs of weights in flight per wavefront
__global__ __launch_bounds__(NW * 64) void k_relu_lowrank_mfma(const float *__restrict__ in, int h_in, int T, int d,
                                                           const float *__restrict__ w, int h, int N,
                                                           const float *__restrict__ bias, float thr,
                                                           const unsigned char *__restrict__ block_active,
                                                           int block_size, int n_blocks,
                                                           const float *__restrict__ gate, float *__restrict__ out,
                                                           int M) {
  extern __shared__ float s_in[];  // [d][32 * RT + 1], zero for rows past M (the odd row stride keeps the
                                   // transposing writes below and the two k-rows of a read off each other's banks)
  constexpr int R = 32 * RT, RS = R + 1;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int hh = blockIdx.y;
  // grid.x = column blocks (rounded up to 8) x row groups: the workgroups that share a block of weight columns
  // follow each other on one XCD (blockIdx.x % 8 picks the XCD), so the block is fetched from memory once
  const int row_groups = (M + R - 1) / R;
  const int xj = blockIdx.x >> 3;
  const int col_block = (xj / row_groups) * 8 + (blockIdx.x & 7);
  const int m0 = (xj % row_groups) * R;
  if (col_block * NW * 128 >= N) return;        // a workgroup of the rounding-up: nothing to do (uniform)
  const int n0 = (col_block * NW + wave) * 128;  // first column of this wavefront
  const bool wave_ok = n0 < N;
  const int ncol = n0 + 4 * (lane & 31);          // this lane's four columns ncol .. ncol + 3 (N % 4 == 0)
  const bool col_ok = ncol < N;
  const float *wp = w + (long)hh * d * N + (long)(lane >> 5) * N + (col_ok ? ncol : (wave_ok ? n0 : 0));
  float4 wv[UK];
#pragma unroll
  for (int u = 0; u < UK; ++u) wv[u] = *reinterpret_cast<const float4 *>(wp + (long)(2 * u) * N);
  // the input rows of this group, transposed on the way in: four adjacent k per access (d % 4 == 0), sixteen
  // accesses of a thread in flight at a time (one at a time, the staging is a chain of trips to the L2)
  {
    const int d4 = d >> 2;
    const int total = R * d4;
    for (int i0 = 0; i0 < total; i0 += NW * 64 * 16) {
      float4 v[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const int i = i0 + u * NW * 64 + tid;
        const int r = i / d4, k4 = i - r * d4;
        const int m = m0 + r;
        v[u] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (i < total && m < M) {
          const int b = m / T, t = m - b * T;
          v[u] = *reinterpret_cast<const float4 *>(in + (((long)b * h_in + (h_in == 1 ? 0 : hh)) * T + t) * d + 4 * k4);
        }
      }
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const int i = i0 + u * NW * 64 + tid;
        const int r = i / d4, k4 = i - r * d4;
        if (i < total) {
          s_in[(4 * k4 + 0) * RS + r] = v[u].x;
          s_in[(4 * k4 + 1) * RS + r] = v[u].y;
          s_in[(4 * k4 + 2) * RS + r] = v[u].z;
          s_in[(4 * k4 + 3) * RS + r] = v[u].w;
        }
      }
    }
  }
  __syncthreads();
  if (!wave_ok) return;
  const float *ap = s_in + (lane >> 5) * RS + (lane & 31);

  f32x16_t acc[RT][4];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[rt][j][e] = 0.0f;

  // k-pairs in groups of UK (d is a multiple of 2 * UK): the loop body has no branches, so the loads of the next
  // group stay in flight across the matrix instructions of this one
  const int groups = d / (2 * UK);
  auto group = [&](int g, auto more_t) {
    constexpr bool MORE = decltype(more_t)::value;
#pragma unroll
    for (int u = 0; u < UK; ++u) {
      const int pr = g * UK + u;
      const float4 b4 = wv[u];
      if constexpr (MORE) wv[u] = *reinterpret_cast<const float4 *>(wp + (long)(2 * (pr + UK)) * N);
      float a[RT];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) a[rt] = ap[(2 * pr) * RS + rt * 32];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        acc[rt][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[rt], b4.x, acc[rt][0], 0, 0, 0);
        acc[rt][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[rt], b4.y, acc[rt][1], 0, 0, 0);
        acc[rt][2] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[rt], b4.z, acc[rt][2], 0, 0, 0);
        acc[rt][3] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[rt], b4.w, acc[rt][3], 0, 0, 0);
      }
      // keeps the load above where it is: left alone, the scheduler sinks all the loads of a group below its
      // matrix instructions, and the next group then starts by waiting for every one of them
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  for (int g = 0; g + 1 < groups; ++g) group(g, std::true_type{});
  group(groups - 1, std::false_type{});
  if (!col_ok) return;

  float4 bv = make_float4(0.f, 0.f, 0.f, 0.f);
  if (bias) bv = *reinterpret_cast<const float4 *>(bias + (long)hh * N + ncol);
  float mk[4] = {1.0f, 1.0f, 1.0f, 1.0f};
  if (block_active) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int blk = (ncol + j) / block_size;
      mk[j] = (blk < n_blocks && block_active[blk]) ? 1.0f : 0.0f;
    }
  }
  const float bvv[4] = {bv.x, bv.y, bv.z, bv.w};
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int m = m0 + rt * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
      if (m < M) {
        const int b = m / T, t = m - b * T;
        const long o = (((long)b * h + hh) * T + t) * N + ncol;
        float y[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          float pv = acc[rt][j][e];
          if (bias) pv = pv + bvv[j];
          if (thr != 0.0f) pv = pv - thr;
          float yy = pv > 0.0f ? pv : 0.0f;
          if (block_active) yy = yy * mk[j];
          y[j] = yy;
        }
        if (gate) {
          const float4 g4 = *reinterpret_cast<const float4 *>(gate + o);
          y[0] = g4.x * y[0]; y[1] = g4.y * y[1]; y[2] = g4.z * y[2]; y[3] = g4.w * y[3];
        }
        *reinterpret_cast<float4 *>(out + o) = make_float4(y[0], y[1], y[2], y[3]);
      }
    }
}

}  // namespace

#ifndef BDH_RL_UK
#define BDH_RL_UK 16
#endif
// lets a kernel take up to 144 KiB of dynamic LDS; once per device
template <typename K>
static hipError_t allow_big_lds(K kernel, std::atomic<uint64_t> &configured) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  const uint64_t bit = 1ull << (dev & 63);
  if (configured.load(std::memory_order_acquire) & bit) return hipSuccess;
  e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 144 * 1024);
  if (e == hipSuccess) configured.fetch_or(bit, std::memory_order_release);
  return e;
}

int bdh_launch_relu_lowrank(bdh_ctx *ctx, const ReluLowrankParams &p) {
  const long M = (long)p.B * p.T;
  if (M > 0x7fffffffL) return bdh_fail(ctx, BDH_E_SHAPE, "B*T too large");
  const unsigned char *mask_dev = nullptr;
  if (p.active_blocks_host) {
    // The device copy of the mask is kept with the bytes it was made from: the two projections of every layer of
    // a call (and the calls after it) pass the same pattern, and only a new pattern costs a copy and a wait (the
    // caller's host buffer may go away on return, and kernels still queued may read the old copy).
    const size_t nb = (size_t)std::max(p.n_blocks, 0);
    const bool same = ctx->lat_mask && ctx->lat_mask_key.size() == nb &&
                      (nb == 0 || memcmp(ctx->lat_mask_key.data(), p.active_blocks_host, nb) == 0);
    if (!same) {
      BDH_HIP_CHECK(ctx, hipStreamSynchronize(ctx->stream));
      if (ctx->lat_mask_bytes < nb + 256) {
        if (ctx->lat_mask) BDH_HIP_CHECK(ctx, hipFree(ctx->lat_mask));
        ctx->lat_mask = nullptr;
        ctx->lat_mask_bytes = 0;
        ctx->lat_mask_key.clear();
        if (hipMalloc(&ctx->lat_mask, nb + 256) != hipSuccess) {
          (void)hipGetLastError();
          return bdh_fail(ctx, BDH_E_NOMEM, "latent block mask of %zu bytes", nb);
        }
        ctx->lat_mask_bytes = nb + 256;
      }
      if (nb > 0) BDH_HIP_CHECK(ctx, hipMemcpy(ctx->lat_mask, p.active_blocks_host, nb, hipMemcpyHostToDevice));
      ctx->lat_mask_key.assign(p.active_blocks_host, p.active_blocks_host + nb);
    }
    mask_dev = static_cast<const unsigned char *>(ctx->lat_mask);
  }
  const bool aligned16 = bdh_aligned(p.in, 16) && bdh_aligned(p.weight, 16) && bdh_aligned(p.out, 16) &&
                         bdh_aligned(p.bias, 16) && bdh_aligned(p.gate, 16);
  // 8 to 64 rows (a batch of sequences decoding together): the f32 matrix cores, same values, the weights streamed
  // once.  (Beyond 64 rows this kernel would stream them once per 64 rows; the 64 x 256 tile kernel below reuses them.)
  // (a negative option value -r takes it from r rows on whatever the width)
  const int mf_rows = ctx->opt_lowrank_mfma_rows < 0 ? -ctx->opt_lowrank_mfma_rows : ctx->opt_lowrank_mfma_rows;
  const bool mf_any_width = ctx->opt_lowrank_mfma_rows < 0;
  if (mf_rows > 0 && M >= mf_rows && M <= 64 && (p.N & 3) == 0 && (p.d % (2 * BDH_RL_UK)) == 0 &&
      p.d >= 2 * BDH_RL_UK && aligned16) {
    // one 32-row tile per workgroup; 33 to 64 rows make two row groups that follow each other on one XCD.  (Two row
    // tiles per workgroup would stream the weights once for 64 rows too, but need 133 KiB of LDS at d = 512, one
    // workgroup per CU: a decode step of the reference's large model at B = 64 took 2.5 ms that way against 1.4.)
    const size_t lds = sizeof(float) * (size_t)p.d * 33;
    // a wavefront owns 128 columns: only for matrices wide enough to give every CU a wavefront or two (a model with
    // 256 neurons per head would run on 16 workgroups; it keeps the kernels below)
    const long row_groups = (M + 31) / 32;
    const int n_cu_mf = ctx->n_cu > 0 ? ctx->n_cu : 256;
    const long waves = (long)((p.N + 127) / 128) * p.h * row_groups;
    if (lds <= 144 * 1024 && (waves >= n_cu_mf || mf_any_width)) {
      constexpr int UK = BDH_RL_UK;
      const int nw = waves >= 4L * n_cu_mf ? 2 : 1;
      const long col_blocks8 = ((p.N + nw * 128 - 1) / (nw * 128) + 7) / 8 * 8;
      if (col_blocks8 * row_groups > 0x7fffffffL || p.h > 65535)
        return bdh_fail(ctx, BDH_E_SHAPE, "grid too large (row groups %ld)", row_groups);
      const dim3 grid((unsigned)(col_blocks8 * row_groups), p.h, 1);
      static std::atomic<uint64_t> cfg1{0}, cfg2{0};
      if (nw == 2) {
        BDH_HIP_CHECK(ctx, allow_big_lds(k_relu_lowrank_mfma<1, UK, 2>, cfg2));
        hipLaunchKernelGGL((k_relu_lowrank_mfma<1, UK, 2>), grid, dim3(128), lds, ctx->stream, p.in, p.h_in, p.T, p.d,
                           p.weight, p.h, p.N, p.bias, p.threshold, mask_dev, p.block_size, p.n_blocks, p.gate, p.out, (int)M);
      } else {
        BDH_HIP_CHECK(ctx, allow_big_lds(k_relu_lowrank_mfma<1, UK, 1>, cfg1));
        hipLaunchKernelGGL((k_relu_lowrank_mfma<1, UK, 1>), grid, dim3(64), lds, ctx->stream, p.in, p.h_in, p.T, p.d,
                           p.weight, p.h, p.N, p.bias, p.threshold, mask_dev, p.block_size, p.n_blocks, p.gate, p.out, (int)M);
      }
      BDH_LAUNCH_CHECK(ctx, "k_relu_lowrank_mfma");
      return BDH_OK;
    }
  }
  // many tokens per sequence: one f32 matrix-core product per (sequence, head), same values
  // (a negative option value -r takes it from r tokens on whatever the grid)
  const int gemm_rows = ctx->opt_lowrank_gemm_rows;
  // (the product kernel deals whole (sequence, head) slices to the 8 XCDs: with fewer than 16 of them half the chip
  // idles -- config 1 at B = 1, four slices, took 24 ms for a 64-token prompt that way against 14)
  const bool gemm_grid = (long)p.B * p.h >= 16 &&
                         (long)p.B * p.h * ((p.T + 127) / 128) * ((p.N + 127) / 128) >= (ctx->n_cu > 0 ? ctx->n_cu : 256);
  if (p.d > 0 && p.N > 0 && (gemm_rows > 0 ? (p.T >= gemm_rows && gemm_grid) : (gemm_rows < 0 && p.T >= -gemm_rows)))
    return bdh_launch_relu_lowrank_gemm(ctx, p, mask_dev);
  // many rows: the 64 x 256 tile (same values, an eighth of the weight traffic)
  const long tile_wgs = (long)((p.N / 4 + 63) / 64) * p.h * ((M + 63) / 64);  // enough of them to cover the chip
  if (M >= 64 && ctx->opt_lowrank_tile != 0 && (p.N & 3) == 0 && (p.d & 3) == 0 && p.d > 0 && aligned16 &&
      (ctx->opt_lowrank_tile == 2 || tile_wgs >= (ctx->n_cu > 0 ? ctx->n_cu : 256))) {
    const long row_tiles = (M + 63) / 64;
    if (row_tiles > 65535 || p.h > 65535) return bdh_fail(ctx, BDH_E_SHAPE, "grid too large (row tiles %ld)", row_tiles);
    hipLaunchKernelGGL(k_relu_lowrank_tile, dim3((p.N / 4 + 63) / 64, p.h, (unsigned)row_tiles), dim3(256), 0, ctx->stream,
                       p.in, p.h_in, p.T, p.d, p.weight, p.h, p.N, p.bias, p.threshold, mask_dev, p.block_size, p.n_blocks,
                       p.gate, p.out, (int)M);
    BDH_LAUNCH_CHECK(ctx, "k_relu_lowrank_tile");
    return BDH_OK;
  }
  // A matrix of up to 16 MiB (it sits in the L2) whose column-per-thread grid would leave most CUs idle, or a single
  // row: 64 columns per workgroup, every weight in flight at once, as many rows per workgroup (1, 2, 4, 8) as still
  // give a workgroup per CU
  const int n_cu_rl = ctx->n_cu > 0 ? ctx->n_cu : 256;
  if (p.d >= 128 && p.d <= 512 && ctx->opt_lowrank_row != 0 &&
      sizeof(float) * (size_t)p.h * p.d * p.N <= (size_t(16) << 20) &&
      (M == 1 || (long)((p.N + 255) / 256) * p.h * ((M + 15) / 16) < n_cu_rl)) {
    const long col_blocks = (p.N + 63) / 64;
    int rt = 1;
    if (M > 1) {
      rt = 8;
      while (rt > 1 && col_blocks * p.h * ((M + rt - 1) / rt) < n_cu_rl) rt >>= 1;
      while (rt > M) rt >>= 1;
    }
    const long row_tiles = (M + rt - 1) / rt;
    if (row_tiles > 65535 || p.h > 65535) return bdh_fail(ctx, BDH_E_SHAPE, "grid too large (row tiles %ld)", row_tiles);
    const dim3 grid((unsigned)col_blocks, p.h, (unsigned)row_tiles);
#define BDH_ROW(NW_, RT_)                                                                                             \
  hipLaunchKernelGGL((k_relu_lowrank_row<NW_, RT_>), grid, dim3(NW_ * 64), 0, ctx->stream, p.in, p.h_in, p.T, p.d,   \
                     p.weight, p.h, p.N, p.bias, p.threshold, mask_dev, p.block_size, p.n_blocks, p.gate, p.out, (int)M)
#define BDH_ROW_RT(NW_)                                                                           \
  do {                                                                                            \
    if (rt == 8) BDH_ROW(NW_, 8); else if (rt == 4) BDH_ROW(NW_, 4); else if (rt == 2) BDH_ROW(NW_, 2); \
    else BDH_ROW(NW_, 1);                                                                         \
  } while (0)
    if (p.d <= 128) BDH_ROW_RT(2); else if (p.d <= 256) BDH_ROW_RT(4); else BDH_ROW_RT(8);
#undef BDH_ROW_RT
#undef BDH_ROW
    BDH_LAUNCH_CHECK(ctx, "k_relu_lowrank_row");
    return BDH_OK;
  }
  if (M >= 8 && ctx->opt_lowrank_scalar != 0) {
    // 8 to 63 rows: inputs through the scalar cache, 16 rows (two SGPR batches of 8 k) or 8 rows per pass
    const int rt = M >= 16 ? 16 : 8;
    const long row_tiles = (M + rt - 1) / rt;
    if (row_tiles > 65535 || p.h > 65535) return bdh_fail(ctx, BDH_E_SHAPE, "grid too large (row tiles %ld)", row_tiles);
    const dim3 grid((p.N + 255) / 256, p.h, (unsigned)row_tiles);
    if (rt == 16)
      hipLaunchKernelGGL((k_relu_lowrank_sc<16, 8>), grid, dim3(256), 0, ctx->stream, p.in, p.h_in, p.T, p.d, p.weight,
                         p.h, p.N, p.bias, p.threshold, mask_dev, p.block_size, p.n_blocks, p.gate, p.out, (int)M);
    else
      hipLaunchKernelGGL((k_relu_lowrank_sc<8, 8>), grid, dim3(256), 0, ctx->stream, p.in, p.h_in, p.T, p.d, p.weight,
                         p.h, p.N, p.bias, p.threshold, mask_dev, p.block_size, p.n_blocks, p.gate, p.out, (int)M);
    BDH_LAUNCH_CHECK(ctx, "k_relu_lowrank_sc");
    return BDH_OK;
  }
  const int RT = M >= 8 ? 8 : (M >= 4 ? 4 : (M >= 2 ? 2 : 1));
  const size_t lds = sizeof(float) * (size_t)RT * (p.d > 0 ? p.d : 1);
  if (lds > 64 * 1024) return bdh_fail(ctx, BDH_E_SHAPE, "d=%d too large for the projection tile", p.d);
  const long row_tiles = (M + RT - 1) / RT;
  if (row_tiles > 65535 || p.h > 65535) return bdh_fail(ctx, BDH_E_SHAPE, "grid too large (row tiles %ld)", row_tiles);
  dim3 grid((p.N + 255) / 256, p.h, (unsigned)row_tiles);
  switch (RT) {
    case 8: launch_relu<8>(ctx->stream, grid, lds, p, mask_dev, (int)M); break;
    case 4: launch_relu<4>(ctx->stream, grid, lds, p, mask_dev, (int)M); break;
    case 2: launch_relu<2>(ctx->stream, grid, lds, p, mask_dev, (int)M); break;
    default: launch_relu<1>(ctx->stream, grid, lds, p, mask_dev, (int)M); break;
  }
  BDH_LAUNCH_CHECK(ctx, "k_relu_lowrank");
  return BDH_OK;
}

int bdh_launch_layer_norm(bdh_ctx *ctx, int64_t rows, int d, const float *in, float *out) {
  if (rows > 0x7fffffffL) return bdh_fail(ctx, BDH_E_SHAPE, "too many rows");
  if (d > 16384) return bdh_fail(ctx, BDH_E_SHAPE, "LayerNorm row of %d floats does not fit in LDS", d);
  hipLaunchKernelGGL(k_layer_norm, dim3((unsigned)rows), dim3(256), sizeof(float) * (size_t)d, ctx->stream, in, out, d);
  BDH_LAUNCH_CHECK(ctx, "k_layer_norm");
  return BDH_OK;
}

int bdh_launch_layer_norm_rows(bdh_ctx *ctx, int64_t rows, int d, const float *in, float *out) {
  if (d > 1024) return bdh_launch_layer_norm(ctx, rows, d, in, out);
  const int64_t blocks = (rows + 3) / 4;
  if (blocks > 0x7fffffffL) return bdh_fail(ctx, BDH_E_SHAPE, "too many rows");
  if (rows == 0) return BDH_OK;
  hipLaunchKernelGGL(k_layer_norm_wave, dim3((unsigned)blocks), dim3(256), 0, ctx->stream, in, out, d, (long)rows);
  BDH_LAUNCH_CHECK(ctx, "k_layer_norm_wave");
  return BDH_OK;
}

int bdh_launch_embed_ln(bdh_ctx *ctx, const int64_t *tokens, int64_t rows, int d, int V, const float *embed,
                        float *out) {
  hipLaunchKernelGGL(k_embed_ln, dim3((unsigned)rows), dim3(256), sizeof(float) * (size_t)d, ctx->stream, tokens, d, V, embed, out);
  BDH_LAUNCH_CHECK(ctx, "k_embed_ln");
  return BDH_OK;
}

static void launch_decoder_finalize(bdh_ctx *ctx, const float *partial, int KBN, int M, int d, float *cur,
                                    const DecoderHead *head) {
  if (head)
    hipLaunchKernelGGL(k_decoder_finalize<true>, dim3(M), dim3(1024), 0, ctx->stream, partial, KBN, M, d, cur, *head);
  else
    hipLaunchKernelGGL(k_decoder_finalize<false>, dim3(M), dim3(1024), 0, ctx->stream, partial, KBN, M, d, cur,
                       DecoderHead{});
}

int bdh_launch_decoder_residual(bdh_ctx *ctx, int B, int T, int h, int N, int d, const float *xy,
                                const float *decoder, float *cur, const DecoderHead *head) {
  const int M = B * T;
  const long K = (long)h * N;
  if (d > 1024 || (d & 3)) return bdh_fail(ctx, BDH_E_SHAPE, "decoder needs d %% 4 == 0 and d <= 1024, got %d", d);
  // (the matrix-core form needs enough (sequence, head, tile) products to cover the chip)
  const long mfma_tiles = (long)B * h * ((T + 127) / 128) * ((d + 127) / 128);
  if (T >= 128 && ctx->opt_decoder_mfma != 0 && mfma_tiles >= (ctx->n_cu > 0 ? ctx->n_cu : 256) / 2) {
    // many tokens per sequence: one product per (sequence, head) on the f32 matrix cores, h partials per row
    int rc = bdh_ws_reserve(ctx, sizeof(float) * (size_t)h * M * d);
    if (rc != BDH_OK) return rc;
    float *partial = static_cast<float *>(ctx->ws);
    rc = bdh_launch_decoder_partials_f32(ctx, B, T, h, N, d, xy, decoder, partial);
    if (rc != BDH_OK) return rc;
    launch_decoder_finalize(ctx, partial, h, M, d, cur, head);
    BDH_LAUNCH_CHECK(ctx, "k_decoder_finalize");
    return BDH_OK;
  }
  // (only when its 32 x 64 tiles over k-blocks of 1024 are enough workgroups for half the chip: not for a small model)
  // (a negative option value -r takes it from r rows on whatever the grid)
  const int sk_rows = ctx->opt_decoder_splitk_rows;
  const bool sk_grid = (K / 1024) * ((d + 63) / 64) * ((M + 31) / 32) >= (ctx->n_cu > 0 ? ctx->n_cu : 256) / 2;
  if (T == 1 && (K % 1024) == 0 && (sk_rows > 0 ? (M >= sk_rows && sk_grid) : M >= -(long)sk_rows)) {
    // a batch of decoding sequences: split-K product on the f32 matrix cores, KB = 1024
    const int KB = 1024;
    const int KBN = (int)(K / KB);
    int rc = bdh_ws_reserve(ctx, sizeof(float) * (size_t)KBN * M * d);
    if (rc != BDH_OK) return rc;
    float *partial = static_cast<float *>(ctx->ws);
    rc = bdh_launch_decoder_splitk_f32(ctx, M, K, d, KB, xy, decoder, partial);
    if (rc != BDH_OK) return rc;
    launch_decoder_finalize(ctx, partial, KBN, M, d, cur, head);
    BDH_LAUNCH_CHECK(ctx, "k_decoder_finalize");
    return BDH_OK;
  }
  const int RT = M >= 8 ? 8 : (M >= 4 ? 4 : (M >= 2 ? 2 : 1));
  const int row_tiles = (M + RT - 1) / RT;
  // k-block size: enough workgroups to fill the chip, few enough partials
  // about two workgroups per CU: more k-blocks only add partials for the second stage to read
  int KB = 1024;
  while (KB > 128 && ((K + KB - 1) / KB) * row_tiles < 2L * (ctx->n_cu > 0 ? ctx->n_cu : 256)) KB >>= 1;
  // a small model: down to 32 rows of E per workgroup, until there is a workgroup per CU
  while (KB > 32 && ((K + KB - 1) / KB) * row_tiles < (ctx->n_cu > 0 ? ctx->n_cu : 256)) KB >>= 1;
  const int KBN = (int)((K + KB - 1) / KB);
  size_t lds = sizeof(float) * (size_t)RT * KB;
  if (lds < sizeof(float) * 4u * d) lds = sizeof(float) * 4u * d;
  const size_t pbytes = sizeof(float) * (size_t)KBN * M * d;
  int rc = bdh_ws_reserve(ctx, pbytes);
  if (rc != BDH_OK) return rc;
  float *partial = static_cast<float *>(ctx->ws);
  dim3 grid(KBN, row_tiles);
#define BDH_DEC(RT_, MV_)                                                                                   \
  hipLaunchKernelGGL((k_decoder_partial<RT_, MV_>), grid, dim3(256), lds, ctx->stream, xy, decoder, partial, T, h, \
                     N, d, KB, M)
  const int mv = d <= 256 ? 1 : (d <= 512 ? 2 : 4);
  if (mv == 1) {
    if (RT == 8) BDH_DEC(8, 1); else if (RT == 4) BDH_DEC(4, 1); else if (RT == 2) BDH_DEC(2, 1);
    else  // one row: the kernel is a chain of round trips, so more E rows per trip
      hipLaunchKernelGGL((k_decoder_partial<1, 1, 16>), grid, dim3(256), lds, ctx->stream, xy, decoder, partial, T, h, N, d,
                         KB, M);
  } else if (mv == 2) {
    if (RT == 8) BDH_DEC(8, 2); else if (RT == 4) BDH_DEC(4, 2); else if (RT == 2) BDH_DEC(2, 2);
    else
      hipLaunchKernelGGL((k_decoder_partial<1, 2, 8>), grid, dim3(256), lds, ctx->stream, xy, decoder, partial, T, h, N, d,
                         KB, M);
  } else {
    if (RT >= 4) BDH_DEC(4, 4); else if (RT == 2) BDH_DEC(2, 4); else BDH_DEC(1, 4);
  }
#undef BDH_DEC
  BDH_LAUNCH_CHECK(ctx, "k_decoder_partial");
  launch_decoder_finalize(ctx, partial, KBN, M, d, cur, head);
  BDH_LAUNCH_CHECK(ctx, "k_decoder_finalize");
  return BDH_OK;
}

bool bdh_relu_lowrank_row_fits(int d, int rows) { return d >= 64 && d <= 1024 && (d & 3) == 0 && rows >= 1; }

int bdh_launch_relu_lowrank_row(bdh_ctx *ctx, const ReluLowrankRowParams &p) {
  if (!bdh_relu_lowrank_row_fits(p.d, p.rows)) return bdh_fail(ctx, BDH_E_SHAPE, "fused row projection: d=%d rows=%d", p.d, p.rows);
  constexpr int NTHR = 128, UK = 64;
  const dim3 grid((p.N + NTHR - 1) / NTHR, p.h);
  const size_t lds = sizeof(float) * (size_t)p.d * (1 + NTHR / 64);
  const RowArgs a{p.partial, p.rows, p.cur_old, p.cur_new, p.tokens};
  if (p.mode == 1)
    hipLaunchKernelGGL((k_relu_lowrank_row1<1, UK, NTHR>), grid, dim3(NTHR), lds, ctx->stream, a, p.d, p.weight, p.h, p.N,
                       p.threshold, p.gate, p.out);
  else if (p.mode == 3)
    hipLaunchKernelGGL((k_relu_lowrank_row1<3, UK, NTHR>), grid, dim3(NTHR), lds, ctx->stream, a, p.d, p.weight, p.h, p.N,
                       p.threshold, p.gate, p.out);
  else
    hipLaunchKernelGGL((k_relu_lowrank_row1<2, UK, NTHR>), grid, dim3(NTHR), lds, ctx->stream, a, p.d, p.weight, p.h, p.N,
                       p.threshold, p.gate, p.out);
  BDH_LAUNCH_CHECK(ctx, "k_relu_lowrank_row1");
  return BDH_OK;
}

int bdh_launch_decoder_partial_row(bdh_ctx *ctx, int h, int N, int d, const float *xy, const float *decoder, int KB,
                                   float *partial, int *KBN_out) {
  const long K = (long)h * N;
  if (d > 1024 || (d & 3)) return bdh_fail(ctx, BDH_E_SHAPE, "decoder needs d %% 4 == 0 and d <= 1024, got %d", d);
  const int KBN = (int)((K + KB - 1) / KB);
  // 16 waves per workgroup; two columns per lane (128-column parts) up to d = 256, four beyond
  constexpr int NWV = 16;
  const int VW = d <= 256 ? 2 : 4;
  const size_t lds = sizeof(float) * std::max<size_t>((size_t)KB, (size_t)NWV * 64 * VW);
  const dim3 grid(KBN, (d + 64 * VW - 1) / (64 * VW));
  if (VW == 2)
    hipLaunchKernelGGL((k_decoder_partial_row<2, 16, NWV>), grid, dim3(NWV * 64), lds, ctx->stream, xy, decoder, partial, K, d, KB);
  else
    hipLaunchKernelGGL((k_decoder_partial_row<4, 16, NWV>), grid, dim3(NWV * 64), lds, ctx->stream, xy, decoder, partial, K, d, KB);
  BDH_LAUNCH_CHECK(ctx, "k_decoder_partial_row");
  *KBN_out = KBN;
  return BDH_OK;
}

int bdh_launch_decoder_finalize_head(bdh_ctx *ctx, const float *partial, int KBN, int M, int d, float *cur,
                                     const DecoderHead *head) {
  if (d > 1024 || (d & 3) != 0) return bdh_fail(ctx, BDH_E_SHAPE, "encoder second stage needs d %% 4 == 0 and d <= 1024");
  launch_decoder_finalize(ctx, partial, KBN, M, d, cur, head);
  BDH_LAUNCH_CHECK(ctx, "k_decoder_finalize");
  return BDH_OK;
}

int bdh_launch_decoder_finalize(bdh_ctx *ctx, const float *partial, int KBN, int M, int d, float *cur) {
  if (d > 1024 || (d & 3) != 0) return bdh_fail(ctx, BDH_E_SHAPE, "encoder second stage needs d %% 4 == 0 and d <= 1024");
  launch_decoder_finalize(ctx, partial, KBN, M, d, cur, nullptr);
  BDH_LAUNCH_CHECK(ctx, "k_decoder_finalize");
  return BDH_OK;
}

int bdh_launch_lm_head(bdh_ctx *ctx, int B, int T, int d, int V, const float *cur, const float *lm_head,
                       float *logits, int64_t *next_tokens) {
  const int M = B * T;
  hipLaunchKernelGGL(k_lm_head, dim3(M), dim3(1024), sizeof(float) * ((size_t)d + 1024), ctx->stream, cur, lm_head,
                     T, d, V, logits, next_tokens);
  BDH_LAUNCH_CHECK(ctx, "k_lm_head");
  return BDH_OK;
}

int bdh_launch_advance_positions(bdh_ctx *ctx, int32_t *positions_dev, int B, int delta) {
  hipLaunchKernelGGL(k_advance_positions, dim3((B + 255) / 256), dim3(256), 0, ctx->stream, positions_dev, B, delta);
  BDH_LAUNCH_CHECK(ctx, "k_advance_positions");
  return BDH_OK;
}
