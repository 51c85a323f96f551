// Temperature / top-k sampling of the next token on the device: sample_from_logits_values and the
// temperature division of sample_next_token (src/generation.rs:26-72, :117).  One workgroup per
// sequence; the uniform variate comes from the caller, so the token never visits the host.
#include "bdh_internal.h"

namespace {

constexpr int SAMPLE_THREADS = 256;
constexpr int SAMPLE_MAX_V = 8192;

// Monotone map float -> uint32 (larger float = larger key), so the k-th largest value can be found
// by a bitwise search over keys.
__device__ __forceinline__ uint32_t order_key(float f) {
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ int block_sum_int(int v, int *s_red) {
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  __syncthreads();
  if (lane == 0) s_red[wave] = v;
  __syncthreads();
  int total = 0;
  for (int w = 0; w < SAMPLE_THREADS / 64; ++w) total += s_red[w];
  return total;
}

__global__ __launch_bounds__(SAMPLE_THREADS) void k_sample_top_k(const float *__restrict__ logits, long ld, int V,
                                                                 float temperature, int top_k,
                                                                 const float *__restrict__ uniforms,
                                                                 int64_t *__restrict__ next_tokens) {
  __shared__ float s_val[SAMPLE_MAX_V];
  __shared__ int s_red[SAMPLE_THREADS / 64];
  __shared__ float s_redf[SAMPLE_THREADS / 64];
  const int b = blockIdx.x, tid = threadIdx.x;
  const float *row = logits + (long)b * ld;
  for (int i = tid; i < V; i += SAMPLE_THREADS) s_val[i] = row[i] / temperature;  // :117 div_scalar
  __syncthreads();

  if (top_k > 0 && top_k < V) {  // :35-47 — everything below the k-th largest value becomes -inf
    uint32_t thr = 0;
    for (int bit = 31; bit >= 0; --bit) {
      const uint32_t cand = thr | (1u << bit);
      int c = 0;
      for (int i = tid; i < V; i += SAMPLE_THREADS) c += order_key(s_val[i]) >= cand;
      if (block_sum_int(c, s_red) >= top_k) thr = cand;  // uniform across the workgroup
    }
    for (int i = tid; i < V; i += SAMPLE_THREADS)
      if (order_key(s_val[i]) < thr) s_val[i] = -INFINITY;
    __syncthreads();
  }

  float m = -INFINITY;  // :49-52 (f32::max ignores NaN operands, as fmaxf does)
  for (int i = tid; i < V; i += SAMPLE_THREADS) m = fmaxf(m, s_val[i]);
  for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_down(m, off, 64));
  if ((tid & 63) == 0) s_redf[tid >> 6] = m;
  __syncthreads();
  m = s_redf[0];
  for (int w = 1; w < SAMPLE_THREADS / 64; ++w) m = fmaxf(m, s_redf[w]);
  for (int i = tid; i < V; i += SAMPLE_THREADS) s_val[i] = expf(s_val[i] - m);  // :53-56
  __syncthreads();

  if (tid == 0) {  // the sums of :57-67 and of WeightedIndex run in index order, so one lane does them
    float sum = 0.f;
    for (int i = 0; i < V; ++i) sum += s_val[i];
    const bool flat = (sum == 0.f) || (sum != sum);
    const float uniform = 1.0f / (float)V;
    float total = 0.f;
    for (int i = 0; i < V; ++i) {
      const float p = flat ? uniform : s_val[i] / sum;
      s_val[i] = p;
      total += p;
    }
    // WeightedIndex: cumulative weights of the first V-1 entries; the variate is uniform in
    // [0, total); the index is the number of cumulative weights <= the variate.
    float u = uniforms[b];
    u = fminf(fmaxf(u, 0.f), 0.99999994f);
    const float chosen = u * total;
    float cum = 0.f;
    int idx = 0;
    for (int i = 0; i < V - 1; ++i) {
      cum += s_val[i];
      if (cum <= chosen) idx = i + 1;
      else break;
    }
    next_tokens[b] = idx;
  }
}

}  // namespace

extern "C" int bdh_sample_top_k(bdh_ctx *ctx, int B, int V, const float *logits, int64_t row_stride,
                                float temperature, int top_k, const float *uniforms, int64_t *next_tokens) {
  if (!ctx) return BDH_E_INVAL;
  if (B < 0 || V < 1) return bdh_fail(ctx, BDH_E_INVAL, "bad batch %d or vocabulary %d", B, V);
  if (V > SAMPLE_MAX_V) return bdh_fail(ctx, BDH_E_SHAPE, "vocabulary %d > %d", V, SAMPLE_MAX_V);
  if (row_stride < V) return bdh_fail(ctx, BDH_E_INVAL, "row stride %lld < vocabulary %d", (long long)row_stride, V);
  if (B == 0) return BDH_OK;
  if (!logits || !uniforms || !next_tokens) return bdh_fail(ctx, BDH_E_INVAL, "null data pointer");
  hipLaunchKernelGGL(k_sample_top_k, dim3(B), dim3(SAMPLE_THREADS), 0, ctx->stream, logits, (long)row_stride, V,
                     temperature, top_k, uniforms, next_tokens);
  BDH_LAUNCH_CHECK(ctx, "k_sample_top_k");
  return BDH_OK;
}
