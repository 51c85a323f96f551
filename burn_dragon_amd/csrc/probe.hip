// Memory-system probes: what the decode state step's access pattern can reach on this GPU with all of
// the step's arithmetic, compaction and reduction taken away.  Measurement aid for bench.py; no part of
// the model path calls these kernels.
#include "bdh_internal.h"

namespace {

// One wave per 1 KiB piece (64 lanes x 16 bytes) of a listed chunk; grid-stride over the pieces.
// MODE 0: read, scale, write back in place; 1: read only; 2: write only.
template <int MODE>
__global__ __launch_bounds__(256) void k_probe_chunks(float4 *__restrict__ region, const int32_t *__restrict__ idx,
                                                      long pieces, int chunk_kib, long region_chunks, float s,
                                                      float *__restrict__ sink) {
  const long nw = ((long)gridDim.x * blockDim.x) >> 6;
  const int lane = threadIdx.x & 63;
  float acc = 0.0f;
  for (long w = ((long)blockIdx.x * blockDim.x + threadIdx.x) >> 6; w < pieces; w += nw) {
    const long c = w / chunk_kib;
    const int sub = (int)(w - c * chunk_kib);
    if ((unsigned long)idx[c] >= (unsigned long)region_chunks) continue;  // an index outside the region is skipped
    float4 *p = region + ((size_t)idx[c] * chunk_kib + sub) * 64 + lane;
    if (MODE == 2) {
      *p = make_float4(s, s, s, s);
    } else {
      float4 v = *p;
      if (MODE == 0) {
        v.x *= s; v.y *= s; v.z *= s; v.w *= s;
        *p = v;
      } else {
        acc += v.x + v.y + v.z + v.w;
      }
    }
  }
  if (MODE == 1 && acc == 1.2345f) sink[0] = acc;  // keeps the loads alive
}

}  // namespace

extern "C" int bdh_probe_chunks(bdh_ctx *ctx, void *region, size_t region_bytes, const int32_t *chunk_index,
                                int n_chunks, int chunk_kib, int mode, int workgroups) {
  if (!ctx) return BDH_E_INVAL;
  if (!region || !chunk_index || n_chunks < 0 || chunk_kib < 1 || mode < 0 || mode > 2 || workgroups < 1)
    return bdh_fail(ctx, BDH_E_INVAL, "bad probe arguments");
  if (!bdh_aligned(region, 16)) return bdh_fail(ctx, BDH_E_ALIGN, "region needs 16-byte alignment");
  if (region_bytes < 64) return bdh_fail(ctx, BDH_E_INVAL, "region too small");
  if (n_chunks == 0) return BDH_OK;
  const long pieces = (long)n_chunks * chunk_kib;
  const long region_chunks = (long)(region_bytes / ((size_t)chunk_kib << 10));
  float *sink = reinterpret_cast<float *>(region);  // never written: the read-only kernel's condition is never true
  const dim3 grid((unsigned)workgroups), block(256);
  if (mode == 0)
    hipLaunchKernelGGL(k_probe_chunks<0>, grid, block, 0, ctx->stream, static_cast<float4 *>(region), chunk_index, pieces,
                       chunk_kib, region_chunks, 1.0f, sink);
  else if (mode == 1)
    hipLaunchKernelGGL(k_probe_chunks<1>, grid, block, 0, ctx->stream, static_cast<float4 *>(region), chunk_index, pieces,
                       chunk_kib, region_chunks, 1.0f, sink);
  else
    hipLaunchKernelGGL(k_probe_chunks<2>, grid, block, 0, ctx->stream, static_cast<float4 *>(region), chunk_index, pieces,
                       chunk_kib, region_chunks, 0.0f, sink);
  BDH_LAUNCH_CHECK(ctx, "k_probe_chunks");
  return BDH_OK;
}
