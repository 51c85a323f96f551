// Parallel (all tokens at once) normalised causal linear attention in f32:
// kernel::linear_attention::fused_state_aligned (src/kernel/linear_attention.rs:11-115) and, with
// the dense block pattern, Attention::forward (src/model/attention.rs:142-175).
//
// This is the reference's training-path form; it is kept in f32 and follows the reference's
// block semantics exactly (including the ALiBi term being added to every entry of an active
// block).  It is a straightforward row-per-workgroup kernel, not tuned: the large-shape
// inference form is the bf16 matrix-core path in prefill.hip.
#include <vector>

#include "bdh_internal.h"

namespace {

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

// one workgroup per (slice, query row i)
__global__ __launch_bounds__(256) void k_fsa_row(const float *__restrict__ q, const float *__restrict__ v,
                                                 const float *__restrict__ slopes_dev, int use_alibi, int h,
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
  const float slope = use_alibi ? slopes_dev[hh] : 0.0f;
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
  const size_t lds = sizeof(float) * ((size_t)Nq + T);
  if (lds > 150 * 1024) return bdh_fail(ctx, BDH_E_SHAPE, "Nq + T = %ld floats exceed the LDS budget", (long)Nq + T);
  if (S * T > 0x7fffffffL) return bdh_fail(ctx, BDH_E_SHAPE, "B*h*T too large");

  const size_t q_bytes = bdh_align_up(sizeof(float) * (size_t)S * T * Nq, 256);
  const size_t act_bytes = sparse ? bdh_align_up((size_t)tb * tb, 256) : 0;
  int rc = bdh_ws_reserve(ctx, q_bytes + act_bytes + 512);
  if (rc != BDH_OK) return rc;
  char *ws = static_cast<char *>(ctx->ws);
  float *q = reinterpret_cast<float *>(ws);
  unsigned char *active = sparse ? reinterpret_cast<unsigned char *>(ws + q_bytes) : nullptr;
  float *slopes_dev = reinterpret_cast<float *>(ws + q_bytes + act_bytes);
  if (sparse) {
    std::vector<unsigned char> m((size_t)tb * tb, 0);
    for (int p = 0; p < n_pairs; ++p) {
      const int r = block_pairs_host[2 * p], c = block_pairs_host[2 * p + 1];
      if (r >= 0 && r < tb && c >= 0 && c < tb) m[(size_t)r * tb + c] = 1;  // iter_cols drops c >= total_blocks
    }
    BDH_HIP_CHECK(ctx, hipMemcpyAsync(active, m.data(), m.size(), hipMemcpyHostToDevice, ctx->stream));
    BDH_HIP_CHECK(ctx, hipStreamSynchronize(ctx->stream));  // m is a local buffer
  }
  if (alibi_slopes_host) {
    BDH_HIP_CHECK(ctx, hipMemcpyAsync(slopes_dev, alibi_slopes_host, sizeof(float) * h, hipMemcpyHostToDevice, ctx->stream));
    BDH_HIP_CHECK(ctx, hipStreamSynchronize(ctx->stream));
  }
  hipLaunchKernelGGL(k_rotate_f32, dim3((unsigned)(S * T)), dim3(256), 0, ctx->stream, query, freqs, q, T, N, rotary);
  BDH_LAUNCH_CHECK(ctx, "k_rotate_f32");
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
