// Context management, argument validation and the host-side tables of the C ABI.
#include <cmath>
#include <new>

#include "bdh_internal.h"

int bdh_fail(bdh_ctx *ctx, int status, const char *fmt, ...) {
  if (ctx) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(ctx->err, sizeof(ctx->err), fmt, ap);
    va_end(ap);
  }
  return status;
}

int bdh_ws_reserve(bdh_ctx *ctx, size_t bytes) {
  if (bytes <= ctx->ws_bytes) return BDH_OK;
  bytes = bdh_align_up(bytes, size_t(1) << 20);
  if (ctx->ws) {
    BDH_HIP_CHECK(ctx, hipStreamSynchronize(ctx->stream));
    BDH_HIP_CHECK(ctx, hipFree(ctx->ws));
    ctx->ws = nullptr;
    ctx->ws_bytes = 0;
  }
  hipError_t e = hipMalloc(&ctx->ws, bytes);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return bdh_fail(ctx, BDH_E_NOMEM, "workspace of %zu bytes: %s", bytes, hipGetErrorString(e));
  }
  ctx->ws_bytes = bytes;
  return BDH_OK;
}

int bdh_stage_reserve(bdh_ctx *ctx, size_t bytes) {
  if (bytes <= ctx->stage_bytes) return BDH_OK;
  bytes = bdh_align_up(bytes, size_t(1) << 20);
  if (ctx->stage) {
    BDH_HIP_CHECK(ctx, hipStreamSynchronize(ctx->stream));
    BDH_HIP_CHECK(ctx, hipFree(ctx->stage));
    ctx->stage = nullptr;
    ctx->stage_bytes = 0;
  }
  hipError_t e = hipMalloc(&ctx->stage, bytes);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return bdh_fail(ctx, BDH_E_NOMEM, "staging buffer of %zu bytes: %s", bytes, hipGetErrorString(e));
  }
  ctx->stage_bytes = bytes;
  return BDH_OK;
}

extern "C" {

const char *bdh_version(void) { return "bdh_mi355x 0.1.0 (gfx950)"; }

const char *bdh_status_string(int status) {
  switch (status) {
    case BDH_OK: return "ok";
    case BDH_E_INVAL: return "invalid argument";
    case BDH_E_SHAPE: return "unsupported shape";
    case BDH_E_ALIGN: return "misaligned pointer";
    case BDH_E_HIP: return "HIP runtime error";
    case BDH_E_NOMEM: return "out of device memory";
    case BDH_E_UNSUPPORTED: return "unsupported combination";
    default: return "unknown status";
  }
}

int bdh_ctx_create(int device_id, void *hip_stream, bdh_ctx **out) {
  if (!out) return BDH_E_INVAL;
  *out = nullptr;
  int count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) {
    (void)hipGetLastError();
    return BDH_E_HIP;  // no device: there is no CPU path to fall back to
  }
  if (device_id < 0 || device_id >= count) return BDH_E_INVAL;
  bdh_ctx *ctx = new (std::nothrow) bdh_ctx();
  if (!ctx) return BDH_E_NOMEM;
  ctx->device = device_id;
  ctx->stream = static_cast<hipStream_t>(hip_stream);
  if (hipSetDevice(device_id) != hipSuccess) {
    delete ctx;
    return BDH_E_HIP;
  }
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, device_id) != hipSuccess) {
    delete ctx;
    return BDH_E_HIP;
  }
  ctx->n_cu = prop.multiProcessorCount;
  // the device is current: resolve this device's copy of the fixed scratch array of bdh_state_step_noalloc
  if (bdh_step_scratch_resolve(ctx) != BDH_OK) {
    delete ctx;
    return BDH_E_HIP;
  }
  *out = ctx;
  return BDH_OK;
}

int bdh_ctx_destroy(bdh_ctx *ctx) {
  if (!ctx) return BDH_OK;
  if (ctx->ws || ctx->fsa_mask || ctx->lat_mask || ctx->stage) (void)hipStreamSynchronize(ctx->stream);
  if (ctx->stage) (void)hipFree(ctx->stage);
  if (ctx->ws) (void)hipFree(ctx->ws);
  if (ctx->fsa_mask) (void)hipFree(ctx->fsa_mask);
  if (ctx->lat_mask) (void)hipFree(ctx->lat_mask);
  delete ctx;
  return BDH_OK;
}

int bdh_ctx_set_stream(bdh_ctx *ctx, void *hip_stream) {
  if (!ctx) return BDH_E_INVAL;
  ctx->stream = static_cast<hipStream_t>(hip_stream);
  return BDH_OK;
}

int bdh_ctx_synchronize(bdh_ctx *ctx) {
  if (!ctx) return BDH_E_INVAL;
  BDH_HIP_CHECK(ctx, hipStreamSynchronize(ctx->stream));
  return BDH_OK;
}

const char *bdh_last_error(const bdh_ctx *ctx) { return ctx ? ctx->err : "null context"; }

int bdh_ctx_set_option(bdh_ctx *ctx, const char *name, int value) {
  if (!ctx || !name) return BDH_E_INVAL;
  if (strcmp(name, "state_step.split") == 0) {
    if (value < -1 || value > 1) return bdh_fail(ctx, BDH_E_INVAL, "state_step.split takes -1, 0 or 1");
    ctx->opt_step_split = value;
    return BDH_OK;
  }
  if (strcmp(name, "state_step.dense_chunks") == 0) {
    if (value < -1 || value > 1) return bdh_fail(ctx, BDH_E_INVAL, "state_step.dense_chunks takes -1, 0 or 1");
    ctx->opt_step_dense = value;
    return BDH_OK;
  }
  if (strcmp(name, "relu_lowrank.tile") == 0) {
    if (value < 0 || value > 2) return bdh_fail(ctx, BDH_E_INVAL, "relu_lowrank.tile takes 0, 1 or 2");
    ctx->opt_lowrank_tile = value;
    return BDH_OK;
  }
  if (strcmp(name, "decoder.mfma") == 0) {
    if (value < 0 || value > 1) return bdh_fail(ctx, BDH_E_INVAL, "decoder.mfma takes 0 or 1");
    ctx->opt_decoder_mfma = value;
    return BDH_OK;
  }
  if (strcmp(name, "relu_lowrank.scalar") == 0) {
    if (value < 0 || value > 1) return bdh_fail(ctx, BDH_E_INVAL, "relu_lowrank.scalar takes 0 or 1");
    ctx->opt_lowrank_scalar = value;
    return BDH_OK;
  }
  if (strcmp(name, "relu_lowrank.gemm_rows") == 0) {
    ctx->opt_lowrank_gemm_rows = value;
    return BDH_OK;
  }
  if (strcmp(name, "relu_lowrank.mfma_rows") == 0) {
    ctx->opt_lowrank_mfma_rows = value;
    return BDH_OK;
  }
  if (strcmp(name, "model.one_launch") == 0) {
    if (value < 0 || value > 2) return bdh_fail(ctx, BDH_E_INVAL, "model.one_launch takes 0, 1 or 2");
    ctx->opt_model_one_launch = value;
    return BDH_OK;
  }
  if (strcmp(name, "model.phase_batch") == 0) {
    if (value < 0) return bdh_fail(ctx, BDH_E_INVAL, "model.phase_batch takes a batch size >= 0");
    ctx->opt_model_phase_batch = value;
    return BDH_OK;
  }
  if (strcmp(name, "relu_lowrank.row") == 0) {
    if (value < 0 || value > 1) return bdh_fail(ctx, BDH_E_INVAL, "relu_lowrank.row takes 0 or 1");
    ctx->opt_lowrank_row = value;
    return BDH_OK;
  }
  if (strcmp(name, "state_step.dense_kernel") == 0) {
    if (value < 0 || value > 1) return bdh_fail(ctx, BDH_E_INVAL, "state_step.dense_kernel takes 0 or 1");
    ctx->opt_step_dense_kernel = value;
    return BDH_OK;
  }
  if (strcmp(name, "decoder.splitk_rows") == 0) {
    if (value == 0) return bdh_fail(ctx, BDH_E_INVAL, "decoder.splitk_rows takes a non-zero row count");
    ctx->opt_decoder_splitk_rows = value;
    return BDH_OK;
  }
  if (strcmp(name, "fused_state_aligned.path") == 0) {
    if (value < -1 || value > 2) return bdh_fail(ctx, BDH_E_INVAL, "fused_state_aligned.path takes -1, 0, 1 or 2");
    ctx->opt_fsa_path = value;
    return BDH_OK;
  }
  if (strcmp(name, "model.fused_rows") == 0) {
    if (value < 0 || value > 1) return bdh_fail(ctx, BDH_E_INVAL, "model.fused_rows takes 0 or 1");
    ctx->opt_model_fused_rows = value;
    return BDH_OK;
  }
  if (strcmp(name, "model.fused_kb") == 0) {
    if (value != 128 && value != 256 && value != 512 && value != 1024 && value != 2048)
      return bdh_fail(ctx, BDH_E_INVAL, "model.fused_kb takes 128, 256, 512, 1024 or 2048");
    ctx->opt_model_fused_kb = value;
    return BDH_OK;
  }
  if (strcmp(name, "state_step.prompt_bf16") == 0) {
    if (value < 0) return bdh_fail(ctx, BDH_E_INVAL, "state_step.prompt_bf16 takes 0 (never) or a token count");
    ctx->opt_step_prompt_bf16 = value;
    return BDH_OK;
  }
  return bdh_fail(ctx, BDH_E_INVAL, "unknown option '%s'", name);
}

int bdh_build_freqs(int latent, float theta, int rotary, float *freqs_host) {
  if (latent < 0 || !freqs_host) return BDH_E_INVAL;
  if (rotary != BDH_ROPE && rotary != BDH_ALIBI && rotary != BDH_POPE) return BDH_E_INVAL;
  const float two_pi = 2.0f * 3.14159265358979323846f;
  for (int i = 0; i < latent; ++i) {
    float value = 0.0f;
    if (rotary == BDH_ROPE) {
      const float e = (floorf((float)i / 2.0f) * 2.0f) / (float)latent;
      value = 1.0f / powf(theta, e) / two_pi;
    } else if (rotary == BDH_POPE) {
      const float e = (float)i / (float)latent;
      value = 1.0f / powf(theta, e) / two_pi;
    }
    freqs_host[i] = value;
  }
  return BDH_OK;
}

int bdh_default_alibi_slopes(int n_head, float *slopes_host) {
  if (n_head < 0 || (n_head > 0 && !slopes_host)) return BDH_E_INVAL;
  for (int i = 0; i < n_head; ++i) slopes_host[i] = 1.0f / powf(2.0f, (float)i / (float)n_head);
  return BDH_OK;
}

static int validate_state_args(bdh_ctx *ctx, int B, int h, int T, int N, int d, int rotary,
                               const float *x, const float *v, const float *freqs,
                               int64_t position, void *rho, int rho_dtype, float *out) {
  if (!ctx) return BDH_E_INVAL;
  if (B < 0 || h < 0 || T < 0 || N < 0 || d < 0)
    return bdh_fail(ctx, BDH_E_INVAL, "negative dimension B=%d h=%d T=%d N=%d d=%d", B, h, T, N, d);
  if (rotary != BDH_ROPE && rotary != BDH_ALIBI && rotary != BDH_POPE)
    return bdh_fail(ctx, BDH_E_INVAL, "rotary %d is not a bdh_rotary value", rotary);
  if (rho_dtype != BDH_F32 && rho_dtype != BDH_BF16)
    return bdh_fail(ctx, BDH_E_INVAL, "rho_dtype %d is not a bdh_dtype value", rho_dtype);
  if (position < 0) return bdh_fail(ctx, BDH_E_INVAL, "negative position");
  if (h > 64) return bdh_fail(ctx, BDH_E_SHAPE, "n_head %d > 64", h);
  if (rotary == BDH_ROPE && (N & 1))
    return bdh_fail(ctx, BDH_E_SHAPE, "RoPE needs an even latent size, got N=%d", N);
  const bool empty = (B == 0 || h == 0 || T == 0);
  if (!empty) {
    if (!v || !out || (N > 0 && (!x || !rho)) || (rotary != BDH_ALIBI && N > 0 && !freqs))
      return bdh_fail(ctx, BDH_E_INVAL, "null data pointer");
    if (!bdh_aligned(x, 8) || !bdh_aligned(v, 16) || !bdh_aligned(rho, 16) || !bdh_aligned(out, 16) ||
        !bdh_aligned(freqs, 8))
      return bdh_fail(ctx, BDH_E_ALIGN, "x/freqs need 8-byte, v/rho/out 16-byte alignment");
  }
  return BDH_OK;
}

int bdh_recurrent_attention(bdh_ctx *ctx, int B, int h, int T, int N, int d, int rotary,
                            const float *x, const float *v, const float *freqs,
                            int64_t position, const int32_t *positions_dev,
                            const float *alibi_slopes_host, void *rho, int rho_dtype,
                            float *out, uint64_t *active_bitmask, int32_t *rows_touched) {
  int rc = validate_state_args(ctx, B, h, T, N, d, rotary, x, v, freqs, position, rho, rho_dtype, out);
  if (rc != BDH_OK) return rc;
  if (B == 0 || h == 0 || T == 0) return BDH_OK;
  float slopes[64];
  if (rotary == BDH_ALIBI) {
    if (alibi_slopes_host)
      memcpy(slopes, alibi_slopes_host, sizeof(float) * h);
    else
      bdh_default_alibi_slopes(h, slopes);
  }
  StateStepParams p{B, h, T, N, d, rotary, rho_dtype, x, v, freqs, position, positions_dev,
                    rotary == BDH_ALIBI ? slopes : nullptr, rho, out, active_bitmask, rows_touched};
  return bdh_launch_state_steps(ctx, p);
}

int bdh_recurrent_attention_lazy_alibi(bdh_ctx *ctx, int B, int h, int T, int N, int d, const float *x,
                                       const float *v, int64_t clock, const int32_t *clocks_dev,
                                       const float *alibi_slopes_host, void *rho, int rho_dtype,
                                       int32_t *stamps, float *out, uint64_t *active_bitmask,
                                       int32_t *rows_touched) {
  int rc = validate_state_args(ctx, B, h, T, N, d, BDH_ALIBI, x, v, nullptr, clock, rho, rho_dtype, out);
  if (rc != BDH_OK) return rc;
  if (B == 0 || h == 0 || T == 0) return BDH_OK;
  if (N > 0 && !stamps) return bdh_fail(ctx, BDH_E_INVAL, "null stamps");
  if (clock + T > 0x7fffffffLL) return bdh_fail(ctx, BDH_E_INVAL, "clock beyond the 31-bit stamp range");
  float slopes[64];
  if (alibi_slopes_host)
    memcpy(slopes, alibi_slopes_host, sizeof(float) * h);
  else
    bdh_default_alibi_slopes(h, slopes);
  StateStepParams p{B, h, T, N, d, BDH_ALIBI, rho_dtype, x, v, nullptr, clock, clocks_dev, slopes, rho, out,
                    active_bitmask, rows_touched, stamps};
  return bdh_launch_state_steps(ctx, p);
}

int bdh_alibi_materialize(bdh_ctx *ctx, int B, int h, int N, int d, int64_t clock, const int32_t *clocks_dev,
                          const float *alibi_slopes_host, void *rho, int rho_dtype, int32_t *stamps) {
  if (!ctx) return BDH_E_INVAL;
  if (B < 0 || h < 0 || N < 0 || d < 0) return bdh_fail(ctx, BDH_E_INVAL, "negative dimension");
  if (h > 64) return bdh_fail(ctx, BDH_E_SHAPE, "n_head %d > 64", h);
  if (rho_dtype != BDH_F32 && rho_dtype != BDH_BF16) return bdh_fail(ctx, BDH_E_INVAL, "bad rho_dtype");
  if (clock < 0 || clock > 0x7fffffffLL) return bdh_fail(ctx, BDH_E_INVAL, "clock outside the 31-bit stamp range");
  if (B == 0 || h == 0 || N == 0) return BDH_OK;
  if (!rho || !stamps) return bdh_fail(ctx, BDH_E_INVAL, "null data pointer");
  if (!bdh_aligned(rho, 16)) return bdh_fail(ctx, BDH_E_ALIGN, "rho needs 16-byte alignment");
  float slopes[64];
  if (alibi_slopes_host)
    memcpy(slopes, alibi_slopes_host, sizeof(float) * h);
  else
    bdh_default_alibi_slopes(h, slopes);
  return bdh_launch_alibi_materialize(ctx, B, h, N, d, slopes, clock, clocks_dev, rho, rho_dtype, stamps);
}

int bdh_rho_energy(bdh_ctx *ctx, int B, int h, int N, int d, const void *rho, int rho_dtype,
                   const int32_t *stamps, int64_t clock, const int32_t *clocks_dev,
                   const float *alibi_slopes_host, float *out) {
  if (!ctx) return BDH_E_INVAL;
  if (B < 0 || h < 0 || N < 0 || d < 0) return bdh_fail(ctx, BDH_E_INVAL, "negative dimension");
  if (h > 64) return bdh_fail(ctx, BDH_E_SHAPE, "n_head %d > 64", h);
  if (rho_dtype != BDH_F32 && rho_dtype != BDH_BF16) return bdh_fail(ctx, BDH_E_INVAL, "bad rho_dtype");
  if (stamps && (clock < 0 || clock > 0x7fffffffLL))
    return bdh_fail(ctx, BDH_E_INVAL, "clock outside the 31-bit stamp range");
  if (h == 0 || N == 0) return BDH_OK;
  if (!out || (!rho && B > 0 && d > 0)) return bdh_fail(ctx, BDH_E_INVAL, "null data pointer");
  if (!bdh_aligned(rho, 16)) return bdh_fail(ctx, BDH_E_ALIGN, "rho needs 16-byte alignment");
  float slopes[64] = {0};
  if (stamps) {
    if (alibi_slopes_host)
      memcpy(slopes, alibi_slopes_host, sizeof(float) * h);
    else
      bdh_default_alibi_slopes(h, slopes);
  }
  return bdh_launch_rho_energy(ctx, B, h, N, d, rho, rho_dtype, stamps, slopes, clock, clocks_dev, 0, out);
}

int bdh_state_step(bdh_ctx *ctx, int B, int h, int N, int d, int rotary, const float *x,
                   const float *v, const float *freqs, int64_t position,
                   const int32_t *positions_dev, const float *alibi_slopes_host, void *rho,
                   int rho_dtype, float *out, uint64_t *active_bitmask, int32_t *rows_touched) {
  return bdh_recurrent_attention(ctx, B, h, 1, N, d, rotary, x, v, freqs, position, positions_dev,
                                 alibi_slopes_host, rho, rho_dtype, out, active_bitmask,
                                 rows_touched);
}

int bdh_state_step_noalloc(bdh_ctx *ctx, int B, int h, int N, int d, int rotary, const float *x,
                           const float *v, const float *freqs, int64_t position,
                           const int32_t *positions_dev, const float *alibi_slopes_host, void *rho,
                           int rho_dtype, float *out, uint64_t *active_bitmask, int32_t *rows_touched) {
  int rc = validate_state_args(ctx, B, h, 1, N, d, rotary, x, v, freqs, position, rho, rho_dtype, out);
  if (rc != BDH_OK) return rc;
  if (B == 0 || h == 0) return BDH_OK;
  void *fixed = bdh_step_scratch_ptr(ctx);
  if (!fixed) return bdh_fail(ctx, BDH_E_UNSUPPORTED, "no fixed scratch array was resolved for device %d", ctx->device);
  float slopes[64];
  if (rotary == BDH_ALIBI) {
    if (alibi_slopes_host)
      memcpy(slopes, alibi_slopes_host, sizeof(float) * h);
    else
      bdh_default_alibi_slopes(h, slopes);
  }
  StateStepParams p{B, h, 1, N, d, rotary, rho_dtype, x, v, freqs, position, positions_dev,
                    rotary == BDH_ALIBI ? slopes : nullptr, rho, out, active_bitmask, rows_touched};
  return bdh_launch_state_steps_in(ctx, p, nullptr, fixed, bdh_step_scratch_bytes());
}

int bdh_relu_lowrank(bdh_ctx *ctx, int B, int h_in, int T, int d, int h, int N, const float *in,
                     const float *weight, const float *bias, float threshold, int block_size,
                     const uint8_t *active_blocks_host, int n_blocks, const float *gate,
                     float *out) {
  if (!ctx) return BDH_E_INVAL;
  if (B < 0 || T < 0 || d < 0 || h < 0 || N < 0)
    return bdh_fail(ctx, BDH_E_INVAL, "negative dimension");
  if (h_in != 1 && h_in != h)
    return bdh_fail(ctx, BDH_E_SHAPE, "input head dim %d must be 1 or %d", h_in, h);
  if (active_blocks_host && (block_size < 1 || n_blocks < 0))
    return bdh_fail(ctx, BDH_E_INVAL, "bad block pattern");
  if (B == 0 || T == 0 || h == 0 || N == 0) return BDH_OK;
  if (!out || !weight || (d > 0 && !in)) return bdh_fail(ctx, BDH_E_INVAL, "null data pointer");
  ReluLowrankParams p{B, h_in, T, d, h, N, in, weight, bias, threshold, block_size,
                      active_blocks_host, n_blocks, gate, out};
  return bdh_launch_relu_lowrank(ctx, p);
}

int bdh_layer_norm(bdh_ctx *ctx, int64_t rows, int d, const float *in, float *out) {
  if (!ctx) return BDH_E_INVAL;
  if (rows < 0 || d < 0) return bdh_fail(ctx, BDH_E_INVAL, "negative dimension");
  if (rows == 0 || d == 0) return BDH_OK;
  if (!in || !out) return bdh_fail(ctx, BDH_E_INVAL, "null data pointer");
  return bdh_launch_layer_norm(ctx, rows, d, in, out);
}

}  // extern "C"
