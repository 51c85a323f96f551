// By-products of the cached step that the reference keeps when built with its "viz" feature
// (LayerVizState, src/model/state.rs:17-24; filled at src/model/bdh.rs:386-434): the last token's
// x, y and x*y of the first sequence, and the energy map of the updated state.
#include "bdh_internal.h"

namespace {

struct VizHeadScalars {
  float v[64];
};

__device__ __forceinline__ float viz_load(const float *p) { return *p; }
__device__ __forceinline__ float viz_load(const unsigned short *p) {
  return __uint_as_float(static_cast<unsigned int>(*p) << 16);
}

__device__ __forceinline__ float viz_abs_sum4(const float *p) {
  const float4 v = *reinterpret_cast<const float4 *>(p);
  return (fabsf(v.x) + fabsf(v.y)) + (fabsf(v.z) + fabsf(v.w));
}
__device__ __forceinline__ float viz_abs_sum4(const unsigned short *p) {
  const uint2 v = *reinterpret_cast<const uint2 *>(p);
  const float a = __uint_as_float((v.x << 16) & 0x7fffffffu), b = __uint_as_float(v.x & 0x7fff0000u);
  const float c = __uint_as_float((v.y << 16) & 0x7fffffffu), e = __uint_as_float(v.y & 0x7fff0000u);
  return (a + b) + (c + e);
}

// out[hh,n] = (sum_b (sum_c |rho[b,hh,n,c]|) / d) / B   (src/model/bdh.rs:411-419)
// One wave per (head, neuron): the B rows of d elements are read coalesced, one after the other.
// A lazily decayed ALiBi state (stamps != null) is read as the state it stands for: row (b,hh,n)
// counts with the factor decay_hh^(clock_b - stamp).
template <typename RhoT>
__global__ __launch_bounds__(256) void k_rho_energy(const RhoT *__restrict__ rho, const int32_t *__restrict__ stamps,
                                                    int B, int h, int N, int d, long clock_scalar,
                                                    const int32_t *__restrict__ clocks_dev, int clock_add,
                                                    VizHeadScalars log_decay, float *__restrict__ out) {
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= (long)h * N) return;
  const int hh = (int)(row / N);
  const int n = (int)(row - (long)hh * N);
  float acc = 0.0f;
  const bool vec = (d & 3) == 0;  // rows are 16-byte (f32) / 8-byte (bf16) aligned: four elements per load
  for (int b = 0; b < B; ++b) {
    const long r = ((long)b * h + hh) * N + n;
    const RhoT *p = rho + r * d;
    float s = 0.0f;
    if (vec) {
      for (int c = lane * 4; c < d; c += 256) s += viz_abs_sum4(p + c);
    } else {
      for (int c = lane; c < d; c += 64) s += fabsf(viz_load(p + c));
    }
    for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
    if (stamps) {
      const long clock = clocks_dev ? (long)clocks_dev[b] + clock_add : clock_scalar;
      const long k = clock - (long)stamps[r];
      if (k > 0) s = s * expf((float)k * log_decay.v[hh]);
    }
    acc = acc + s / (float)d;
  }
  if (lane == 0) out[row] = acc / (float)B;
}

// dst[hh, c] = src[hh * head_stride + offset + c]: row `offset / cols` of every head of one sequence
__global__ __launch_bounds__(256) void k_gather_head_rows(const float *__restrict__ src, long head_stride, long offset,
                                                          int cols, float *__restrict__ dst) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c < cols) dst[(long)blockIdx.y * cols + c] = src[(long)blockIdx.y * head_stride + offset + c];
}

__global__ __launch_bounds__(256) void k_fill_zero_f32(float *__restrict__ p, long n) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = 0.0f;
}

}  // namespace

int bdh_launch_rho_energy(bdh_ctx *ctx, int B, int h, int N, int d, const void *rho, int rho_dtype,
                          const int32_t *stamps, const float *slopes_host, int64_t clock, const int32_t *clocks_dev,
                          int clock_add, float *out) {
  const long rows = (long)h * N;
  if (rows == 0) return BDH_OK;
  if (B == 0 || d == 0) {  // an empty mean: the reference would divide by zero; report zeros
    hipLaunchKernelGGL(k_fill_zero_f32, dim3((unsigned)((rows + 255) / 256)), dim3(256), 0, ctx->stream, out, rows);
    BDH_LAUNCH_CHECK(ctx, "k_fill_zero_f32");
    return BDH_OK;
  }
  VizHeadScalars log_decay{};
  if (stamps)
    for (int i = 0; i < h; ++i) log_decay.v[i] = (float)log((double)expf(-slopes_host[i]));
  const dim3 grid((unsigned)((rows + 3) / 4));
  if (rho_dtype == BDH_F32)
    hipLaunchKernelGGL(k_rho_energy<float>, grid, dim3(256), 0, ctx->stream, static_cast<const float *>(rho), stamps, B,
                       h, N, d, (long)clock, clocks_dev, clock_add, log_decay, out);
  else
    hipLaunchKernelGGL(k_rho_energy<unsigned short>, grid, dim3(256), 0, ctx->stream,
                       static_cast<const unsigned short *>(rho), stamps, B, h, N, d, (long)clock, clocks_dev, clock_add,
                       log_decay, out);
  BDH_LAUNCH_CHECK(ctx, "k_rho_energy");
  return BDH_OK;
}

int bdh_launch_gather_head_rows(bdh_ctx *ctx, const float *src, int h, long head_stride, long offset, int cols,
                                float *dst) {
  if (h == 0 || cols == 0) return BDH_OK;
  hipLaunchKernelGGL(k_gather_head_rows, dim3((unsigned)((cols + 255) / 256), (unsigned)h), dim3(256), 0, ctx->stream,
                     src, head_stride, offset, cols, dst);
  BDH_LAUNCH_CHECK(ctx, "k_gather_head_rows");
  return BDH_OK;
}

int bdh_launch_fill_zero_f32(bdh_ctx *ctx, float *p, long n) {
  if (n == 0) return BDH_OK;
  hipLaunchKernelGGL(k_fill_zero_f32, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, ctx->stream, p, n);
  BDH_LAUNCH_CHECK(ctx, "k_fill_zero_f32");
  return BDH_OK;
}
