/*
 * bdh_oracle.c — CPU restatement of the BDH cached-inference path of
 * mosure/burn_dragon (crate burn_dragon_hatchling 0.3.0).
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker that the HIP kernels are
 * compared against and the "restated reference CPU path" timed by the benchmark.
 * Nothing that ships (the C-ABI library, the host mirror) links, loads or calls it.
 *
 * Every function cites the reference lines it follows.  All arithmetic is IEEE
 * binary32 with the operation order of the reference's tensor-op sequence: where
 * the reference materialises a product tensor and then adds it, the product is
 * rounded before the add (the file is built with -ffp-contract=off, so the only
 * fused multiply-adds are the explicit fmaf() calls of the matmul chains).
 *
 * Matmul order.  The reference's matmuls run inside the third-party crates
 * burn-ndarray 0.19.1 / ndarray 0.16.1 / matrixmultiply 0.3.10, whose sources are
 * not part of the reference tree.  Their published algorithm (a register-tiled
 * GEMM micro-kernel that walks k in order and accumulates a*b into one register
 * per output element, using hardware FMA when the CPU has it) is restated here as
 * one k-sequential fmaf() chain per output element.  The summation order inside
 * those crates cannot be confirmed from this tree: parity of values is therefore
 * tolerance-based, and "bit-exact active sets" means bit-exact against THIS order.
 *
 * Pinning status (what independent check fixes each function) is listed in
 * tests/test_oracle.py and tests/test_record.py; functions with no such check are marked "parity
 * unpinned" below.
 *
 *   orc_build_freqs            pinned: closed form + second statement in
 *                              tests/fused_kernel_tests.rs:172-196
 *   orc_rotate (rope/pope)     pinned: tests/fused_kernel_tests.rs:198-220 formulas,
 *                              pos=0 identity, pair-norm invariance, relative-shift
 *   orc_layer_norm             pinned: library routine (torch layer_norm, CPU)
 *   orc_relu_lowrank           pinned: tests/fused_kernel_tests.rs:35-68 recipe
 *                              against numpy matmul
 *   orc_fused_state_aligned    pinned: tests/fused_kernel_tests.rs:70-170 recipe
 *                              (blocked == dense), both rotaries
 *   orc_attention_forward      pinned: KAT src/model/attention.rs:405-432
 *   orc_alibi_decay            pinned: KAT src/model/attention.rs:384-403
 *   orc_recurrent_attention    reference holds no value test for it ("parity
 *                              unpinned" by the reference); pinned here by brute
 *                              force against tril(-1)(QQ^T)V in float64, chunk
 *                              consistency, first-token and final-rho closed forms
 *   orc_forward_with_state     reference pins shapes/position only
 *                              (tests/model_paths.rs:33-91); values pinned here by the
 *                              trained checkpoint the reference ships
 *                              (www/assets/model/tiny_shakespeare, ALiBi): 1.16 nats
 *                              per character on Shakespeare text against 4.23 for a
 *                              uniform guess, and back to >= 3.5 with the wrong
 *                              positional scheme or swapped encoders
 *                              (tests/test_record.py); also decode-vs-prefill
 *                              consistency and agreement with the independent numpy
 *                              restatement.  The RoPE and PoPE variants share
 *                              everything but orc_rotate (pinned above) with it.
 *   orc_sample_from_logits     pinned: library softmax, float64 inverse CDF, argmax
 *                              for top_k = 1, draw frequencies (tests/test_oracle.py);
 *                              the reference's own draw uses thread_rng and cannot be
 *                              replayed
 *   forward_fast (numpy only,  composition of the pinned relu_lowrank, attention_forward /
 *   oracle/bdh_oracle.py)      fused_state_aligned and layer_norm; the reference checks its shape
 *                              only (tests/model_paths.rs:48,81): "parity unpinned" as a whole
 *   orc_rho_energy,            pinned: numpy float64 mean(|rho|) over d and the batch;
 *   orc_forward_with_state_viz the other three taps are slices of x, y and x*y of the
 *                              pinned forward pass, checked against the numpy
 *                              restatement; PoPE gives a zero energy map (state rows
 *                              2N != N, src/model/bdh.rs:413-424)
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_ROPE 0
#define ORC_ALIBI 1
#define ORC_POPE 2

/* src/model/attention.rs:1  `use std::f32::consts::PI` */
static const float ORC_PI = 3.14159265358979323846f;
/* src/model/bdh.rs:17 */
static const float ORC_LN_EPS = 1e-5f;
/* src/model/attention.rs:11, src/kernel/linear_attention.rs:9 */
static const float ORC_ROW_NORM_EPS = 1e-6f;

/* ------------------------------------------------------------------------- */
/* src/model/attention.rs:351-373  Attention::build_freqs                     */
void orc_build_freqs(int latent, float theta, int rotary, float *out) {
  for (int idx = 0; idx < latent; ++idx) {
    float value;
    if (rotary == ORC_ROPE) {
      float exponent = (floorf((float)idx / 2.0f) * 2.0f) / (float)latent;
      value = 1.0f / powf(theta, exponent) / (2.0f * ORC_PI);
    } else if (rotary == ORC_POPE) {
      float exponent = (float)idx / (float)latent;
      value = 1.0f / powf(theta, exponent) / (2.0f * ORC_PI);
    } else {
      value = 0.0f;
    }
    out[idx] = value;
  }
}

/* src/kernel/linear_attention.rs:152-163  default_alibi_slopes */
void orc_default_alibi_slopes(int n_head, float *out) {
  for (int i = 0; i < n_head; ++i) {
    float ratio = (float)i / (float)n_head;
    out[i] = 1.0f / powf(2.0f, ratio);
  }
}

/* src/model/attention.rs:181-186  alibi_decay = exp(-slope) */
void orc_alibi_decay(int n_head, const float *slopes, float *out) {
  for (int i = 0; i < n_head; ++i) out[i] = expf(-slopes[i]);
}

/* burn activation::softplus(x, beta=1) = log(1 + exp(beta x)) / beta, as called
 * at src/model/attention.rs:324 */
static inline float orc_softplus1(float x) {
  return logf(expf(x * 1.0f) + 1.0f) / 1.0f;
}

/* src/model/attention.rs:332-349 rotate, :305-321 rope, :323-330 pope.
 * x [B,h,T,N] -> q [B,h,T,Nq]; Nq = N (rope, alibi) or 2N (pope).
 * One `start` for the whole batch; position = f32(start + t). */
void orc_rotate(const float *x, int B, int h, int T, int N, const float *freqs,
                int rotary, int64_t start, float *q) {
  const int Nq = rotary == ORC_POPE ? 2 * N : N;
  for (int b = 0; b < B; ++b)
    for (int hh = 0; hh < h; ++hh)
      for (int t = 0; t < T; ++t) {
        const float *xr = x + (((size_t)b * h + hh) * T + t) * N;
        float *qr = q + (((size_t)b * h + hh) * T + t) * Nq;
        if (rotary == ORC_ALIBI) {
          memcpy(qr, xr, sizeof(float) * N);
          continue;
        }
        const float pos = (float)(start + (int64_t)t);
        for (int n = 0; n < N; ++n) {
          float raw = pos * freqs[n];
          float phase = (raw - floorf(raw)) * (2.0f * ORC_PI);
          float c = cosf(phase), s = sinf(phase);
          if (rotary == ORC_ROPE) {
            /* rotated[2j] = -x[2j+1]; rotated[2j+1] = x[2j] */
            float rot = (n & 1) ? xr[n - 1] : -xr[n + 1];
            float a = xr[n] * c;
            float r = rot * s;
            qr[n] = a + r;
          } else {
            float m = orc_softplus1(xr[n]);
            qr[n] = m * c;
            qr[N + n] = m * s;
          }
        }
      }
}

/* src/model/bdh.rs:86-89  layer_norm: (x - mean) / sqrt(var_biased + eps), no affine */
void orc_layer_norm(const float *in, int64_t rows, int d, float *out) {
#pragma omp parallel for if (rows > 64)
  for (int64_t r = 0; r < rows; ++r) {
    const float *x = in + r * d;
    float *y = out + r * d;
    float sum = 0.0f;
    for (int i = 0; i < d; ++i) sum += x[i];
    float mean = sum / (float)d;
    float sq = 0.0f;
    for (int i = 0; i < d; ++i) {
      float c = x[i] - mean;
      sq += c * c;
    }
    float var = sq / (float)d;
    float den = sqrtf(var + ORC_LN_EPS);
    for (int i = 0; i < d; ++i) y[i] = (x[i] - mean) / den;
  }
}

/* src/kernel/block_sparse.rs:48-63  BlockPattern1d::mask (1.0 inside active blocks) */
static inline float orc_block_mask_at(int n, int block_size, const uint8_t *active,
                                      int n_active_entries) {
  if (!active) return 1.0f;
  if (block_size < 1) block_size = 1;
  int blk = n / block_size;
  return (blk < n_active_entries && active[blk]) ? 1.0f : 0.0f;
}

/* src/kernel/relu_lowrank.rs:7-37  fused_forward, which is also the unfused
 * sequence at src/model/bdh.rs:346-350 / :370-374 when bias=NULL and no mask.
 * in [B,hin,T,d] with hin in {1,h} (Burn matmul broadcasts dim 1), w [h,d,N],
 * bias [h,N] or NULL, active_blocks: one byte per latent block or NULL (dense).
 * out [B,h,T,N] = relu(in.w + bias - thr) * mask. */
void orc_relu_lowrank(const float *in, int B, int hin, int T, int d, const float *w,
                      int h, int N, const float *bias, float thr, int block_size,
                      const uint8_t *active_blocks, int n_blocks, float *out) {
#pragma omp parallel for collapse(2)
  for (int b = 0; b < B; ++b)
    for (int hh = 0; hh < h; ++hh) {
      float *acc = (float *)malloc(sizeof(float) * N);
      for (int t = 0; t < T; ++t) {
        const float *xr = in + (((size_t)b * hin + (hin == 1 ? 0 : hh)) * T + t) * d;
        float *yr = out + (((size_t)b * h + hh) * T + t) * N;
        for (int n = 0; n < N; ++n) acc[n] = 0.0f;
        for (int k = 0; k < d; ++k) {
          const float a = xr[k];
          const float *wr = w + ((size_t)hh * d + k) * N;
          for (int n = 0; n < N; ++n) acc[n] = fmaf(a, wr[n], acc[n]);
        }
        for (int n = 0; n < N; ++n) {
          float p = acc[n];
          if (bias) p = p + bias[(size_t)hh * N + n];
          if (thr != 0.0f) p = p - thr;
          float r = p > 0.0f ? p : 0.0f; /* relu */
          if (active_blocks) r = r * orc_block_mask_at(n, block_size, active_blocks, n_blocks);
          yr[n] = r;
        }
      }
      free(acc);
    }
}

/* src/model/bdh.rs:258-307  recurrent_attention AFTER the rotate at :265.
 * q [B,h,T,Nq] (already rotated), v [B,T,d] (shared by all heads, :290),
 * rho [B,h,Nq,d] in/out, decay [h] or NULL (ALiBi only, :299-301),
 * out [B,h,T,d].  Dense and faithful: the readout materialises rho*q and sums over
 * the latent axis in index order with the OLD rho (:293-295); the update
 * materialises q*v and adds it (:298). */
void orc_recurrent_attention(const float *q, const float *v, float *rho, const float *decay,
                             int B, int h, int T, int Nq, int d, float *out) {
#pragma omp parallel for collapse(2)
  for (int b = 0; b < B; ++b)
    for (int hh = 0; hh < h; ++hh) {
      float *R = rho + ((size_t)b * h + hh) * (size_t)Nq * d;
      for (int t = 0; t < T; ++t) {
        const float *qt = q + (((size_t)b * h + hh) * T + t) * Nq;
        const float *vt = v + ((size_t)b * T + t) * d;
        float *o = out + (((size_t)b * h + hh) * T + t) * d;
        for (int c = 0; c < d; ++c) o[c] = 0.0f;
        for (int n = 0; n < Nq; ++n) {
          const float qn = qt[n];
          float *Rn = R + (size_t)n * d;
          for (int c = 0; c < d; ++c) {
            float prod = Rn[c] * qn;
            o[c] = o[c] + prod;
          }
        }
        for (int n = 0; n < Nq; ++n) {
          const float qn = qt[n];
          float *Rn = R + (size_t)n * d;
          for (int c = 0; c < d; ++c) {
            float outer = qn * vt[c];
            float r = Rn[c] + outer;
            if (decay) r = r * decay[hh];
            Rn[c] = r;
          }
        }
      }
    }
}

/* Same function restricted to rows whose q is non-zero.  Skipped rows contribute
 * rho*0 = +-0 to the readout and q*v = +-0 to the update, so every output and
 * every state element compares equal (==) to the dense form; only usable when
 * decay == NULL (a decay touches every row).  Used to make config-sized oracle
 * runs finish in seconds. */
void orc_recurrent_attention_sparse(const float *q, const float *v, float *rho, int B, int h,
                                    int T, int Nq, int d, float *out) {
#pragma omp parallel for collapse(2)
  for (int b = 0; b < B; ++b)
    for (int hh = 0; hh < h; ++hh) {
      float *R = rho + ((size_t)b * h + hh) * (size_t)Nq * d;
      for (int t = 0; t < T; ++t) {
        const float *qt = q + (((size_t)b * h + hh) * T + t) * Nq;
        const float *vt = v + ((size_t)b * T + t) * d;
        float *o = out + (((size_t)b * h + hh) * T + t) * d;
        for (int c = 0; c < d; ++c) o[c] = 0.0f;
        for (int n = 0; n < Nq; ++n) {
          const float qn = qt[n];
          if (qn == 0.0f) continue;
          float *Rn = R + (size_t)n * d;
          for (int c = 0; c < d; ++c) {
            float prod = Rn[c] * qn;
            o[c] = o[c] + prod;
          }
          for (int c = 0; c < d; ++c) {
            float outer = qn * vt[c];
            Rn[c] = Rn[c] + outer;
          }
        }
      }
    }
}

/* k-sequential matmul helper: C[m,n] = sum_k A[m,k] B[k,n]  (fmaf chain) */
static void orc_matmul(const float *A, const float *Bm, int M, int K, int N, float *C) {
  for (int m = 0; m < M; ++m) {
    float *c = C + (size_t)m * N;
    for (int n = 0; n < N; ++n) c[n] = 0.0f;
    for (int k = 0; k < K; ++k) {
      const float a = A[(size_t)m * K + k];
      const float *br = Bm + (size_t)k * N;
      for (int n = 0; n < N; ++n) c[n] = fmaf(a, br[n], c[n]);
    }
  }
}

/* src/kernel/block_sparse.rs:96-117 dense BlockPattern2d: active iff col <= row;
 * a sparse pattern is passed as pairs[] = (row, col) entries. */
static int orc_pair_active(int row, int col, const int32_t *pairs, int n_pairs) {
  if (!pairs) return col <= row;
  for (int i = 0; i < n_pairs; ++i)
    if (pairs[2 * i] == row && pairs[2 * i + 1] == col) return 1;
  return 0;
}

/* src/kernel/linear_attention.rs:11-115  fused_state_aligned.
 * query [B,h,T,N] (un-rotated), value [B,T,dv] (dim-1 of size 1 repeated over
 * heads, :44), freqs [N], slopes [h] or NULL, time-block size, optional sparse
 * (row,col) block pairs.  Positions are 0..T (:23-25).  out [B,h,T,dv].
 * The ALiBi term (:97-100) is added to every entry of an active block, including
 * the entries of a diagonal block that tril(-1) has just zeroed (:88-90); this is
 * what the reference computes and it is restated as is. */
void orc_fused_state_aligned(const float *query, const float *value, const float *freqs,
                             const float *slopes, int B, int h, int T, int N, int dv,
                             int block_size, const int32_t *pairs, int n_pairs, int rotary,
                             float *out) {
  const int Nq = rotary == ORC_POPE ? 2 * N : N;
  float *qrot = (float *)malloc(sizeof(float) * (size_t)B * h * T * Nq);
  orc_rotate(query, B, h, T, N, freqs, rotary, 0, qrot);
  if (block_size < 1) block_size = 1;
  const int total_blocks = (T + block_size - 1) / block_size;
  float *scores = (float *)malloc(sizeof(float) * (size_t)block_size * block_size);
  float *contrib = (float *)malloc(sizeof(float) * (size_t)block_size * dv);
  float *acc = (float *)malloc(sizeof(float) * (size_t)block_size * dv);
  float *norm = (float *)malloc(sizeof(float) * (size_t)block_size);
  for (int b = 0; b < B; ++b)
    for (int hh = 0; hh < h; ++hh) {
      const float *Q = qrot + ((size_t)b * h + hh) * (size_t)T * Nq;
      const float *V = value + (size_t)b * T * dv;
      float *O = out + ((size_t)b * h + hh) * (size_t)T * dv;
      for (int row = 0; row < total_blocks; ++row) {
        const int r0 = row * block_size;
        const int r1 = r0 + block_size < T ? r0 + block_size : T;
        const int rl = r1 - r0;
        for (int i = 0; i < rl * dv; ++i) acc[i] = 0.0f;
        for (int i = 0; i < rl; ++i) norm[i] = 0.0f;
        int any = 0;
        for (int col = 0; col < total_blocks; ++col) {
          /* iter_cols (:103-117) then is_active (:96-101) */
          if (!pairs && col > row) break;
          if (!orc_pair_active(row, col, pairs, n_pairs)) continue;
          any = 1;
          const int c0 = col * block_size;
          const int c1 = c0 + block_size < T ? c0 + block_size : T;
          const int cl = c1 - c0;
          for (int i = 0; i < rl; ++i)
            for (int j = 0; j < cl; ++j) {
              float s = 0.0f;
              for (int k = 0; k < Nq; ++k)
                s = fmaf(Q[(size_t)(r0 + i) * Nq + k], Q[(size_t)(c0 + j) * Nq + k], s);
              if (row == col && j >= i) s = 0.0f; /* tril(-1) */
              if (slopes) {
                float al = slopes[hh] * ((float)(c0 + j) - (float)(r0 + i));
                s = s + al;
              }
              scores[i * cl + j] = s;
            }
          for (int i = 0; i < rl; ++i) {
            float a = 0.0f;
            for (int j = 0; j < cl; ++j) a += fabsf(scores[i * cl + j]);
            norm[i] = norm[i] + a;
          }
          orc_matmul(scores, V + (size_t)c0 * dv, rl, cl, dv, contrib);
          /* orc_matmul reads B rows with stride dv and K = cl */
          for (int i = 0; i < rl * dv; ++i) acc[i] = acc[i] + contrib[i];
        }
        (void)any; /* rows with no active column keep acc = 0 and are pushed as is (:70-73) */
        for (int i = 0; i < rl; ++i) {
          float den = any ? norm[i] + ORC_ROW_NORM_EPS : 1.0f;
          for (int c = 0; c < dv; ++c)
            O[(size_t)(r0 + i) * dv + c] = any ? acc[i * dv + c] / den : acc[i * dv + c];
        }
      }
    }
  free(qrot);
  free(scores);
  free(contrib);
  free(acc);
  free(norm);
}

/* src/model/attention.rs:142-175  Attention::forward, unfused branch (:154-174):
 * rotate at position 0, scores = (q q^T).tril(-1), ALiBi bias
 * slopes*(pos_col-pos_row).tril(-1), row_normalize (:300-303), scores.V.
 * row_normalize = 0 gives the un-normalised causal form that equals the recurrent
 * path of bdh.rs:288-302. */
void orc_attention_forward(const float *query, const float *value, const float *freqs,
                           const float *slopes, int B, int h, int T, int N, int dv, int rotary,
                           int row_normalize, float *out) {
  const int Nq = rotary == ORC_POPE ? 2 * N : N;
  float *qrot = (float *)malloc(sizeof(float) * (size_t)B * h * T * Nq);
  orc_rotate(query, B, h, T, N, freqs, rotary, 0, qrot);
  float *scores = (float *)malloc(sizeof(float) * (size_t)T * T);
  for (int b = 0; b < B; ++b)
    for (int hh = 0; hh < h; ++hh) {
      const float *Q = qrot + ((size_t)b * h + hh) * (size_t)T * Nq;
      const float *V = value + (size_t)b * T * dv;
      float *O = out + ((size_t)b * h + hh) * (size_t)T * dv;
      for (int i = 0; i < T; ++i)
        for (int j = 0; j < T; ++j) {
          float s = 0.0f;
          if (j < i) {
            for (int k = 0; k < Nq; ++k)
              s = fmaf(Q[(size_t)i * Nq + k], Q[(size_t)j * Nq + k], s);
            if (slopes) s = s + slopes[hh] * ((float)j - (float)i);
          }
          scores[(size_t)i * T + j] = s;
        }
      if (row_normalize)
        for (int i = 0; i < T; ++i) {
          float a = 0.0f;
          for (int j = 0; j < T; ++j) a += fabsf(scores[(size_t)i * T + j]);
          float den = a + ORC_ROW_NORM_EPS;
          for (int j = 0; j < T; ++j) scores[(size_t)i * T + j] = scores[(size_t)i * T + j] / den;
        }
      orc_matmul(scores, V, T, T, dv, O);
    }
  free(qrot);
  free(scores);
}

/* ------------------------------------------------------------------------- */
/* src/model/bdh.rs:309-450  BDH::forward_with_state (inference: dropout is the
 * identity, :381).  Parameters in the record order of the reference module
 * (src/model/bdh.rs:27-33): embed [V,d], encoder [h,d,N] (= D_x), encoder_v
 * [h,d,N] (= D_y), decoder [h*N,d] (= E), lm_head [d,V].
 * rho: L buffers [B,h,Nq,d] laid out back to back; *position is read as the start
 * position and advanced by T with saturation (:445).
 * Optional taps (may be NULL): x_tap [L,B,h,T,N] sparse activations per layer,
 * attn_tap [L,B,h,T,d] un-normalised readout per layer.
 * sparse_state != 0 uses orc_recurrent_attention_sparse (identical values, see
 * there); it is ignored for ALiBi.                                              */
typedef struct {
  int n_layer, n_embd, n_head, latent, vocab; /* latent = N per head */
  int rotary;                                 /* ORC_ROPE / ORC_ALIBI / ORC_POPE */
  float rope_theta, relu_threshold;           /* src/model/config.rs:20-31 */
  const float *alibi_slopes;                  /* [h] or NULL -> default slopes */
  const float *embed, *encoder, *encoder_v, *decoder, *lm_head;
} orc_model;

/* src/model/bdh.rs:411-419: rho_energy[h,n] = mean over the batch of (sum_c |rho[b,h,n,c]|) / d.
 * Sums run in index order; the batch mean is sum_dim(0) followed by div_scalar(batch). */
void orc_rho_energy(const float *rho, int B, int h, int N, int d, float *out) {
  for (int hh = 0; hh < h; ++hh)
    for (int n = 0; n < N; ++n) {
      float acc = 0.0f;
      for (int b = 0; b < B; ++b) {
        const float *row = rho + (((size_t)b * h + hh) * N + n) * (size_t)d;
        float s = 0.0f;
        for (int c = 0; c < d; ++c) s = s + fabsf(row[c]);
        acc = acc + s / (float)d;
      }
      out[(size_t)hh * N + n] = acc / (float)B;
    }
}

static int orc_forward_impl(const orc_model *m, const int64_t *tokens, int B, int T, float *rho,
                            int64_t *position, float *logits, float *x_tap, float *attn_tap,
                            int sparse_state, float *viz) {
  const int d = m->n_embd, h = m->n_head, N = m->latent, V = m->vocab, L = m->n_layer;
  const int Nq = m->rotary == ORC_POPE ? 2 * N : N;
  const size_t rows = (size_t)B * T;
  float *freqs = (float *)malloc(sizeof(float) * N);
  orc_build_freqs(N, m->rope_theta, m->rotary, freqs);
  float *slopes = NULL, *decay = NULL;
  if (m->rotary == ORC_ALIBI) {
    slopes = (float *)malloc(sizeof(float) * h);
    decay = (float *)malloc(sizeof(float) * h);
    if (m->alibi_slopes)
      memcpy(slopes, m->alibi_slopes, sizeof(float) * h);
    else
      orc_default_alibi_slopes(h, slopes);
    orc_alibi_decay(h, slopes, decay);
  }
  float *cur = (float *)malloc(sizeof(float) * rows * d);
  float *tmp = (float *)malloc(sizeof(float) * rows * d);
  float *x = (float *)malloc(sizeof(float) * (size_t)B * h * T * N);
  float *y = (float *)malloc(sizeof(float) * (size_t)B * h * T * N);
  float *q = (float *)malloc(sizeof(float) * (size_t)B * h * T * Nq);
  float *attn = (float *)malloc(sizeof(float) * (size_t)B * h * T * d);
  float *attn_ln = (float *)malloc(sizeof(float) * (size_t)B * h * T * d);
  float *mixed = (float *)malloc(sizeof(float) * rows * (size_t)h * N);
  float *mlp = (float *)malloc(sizeof(float) * rows * d);

  /* :319-322 embed, reshape [B,1,T,d], layer_norm */
  for (size_t r = 0; r < rows; ++r) {
    int64_t tok = tokens[r];
    if (tok < 0 || tok >= V) {
      free(freqs); free(slopes); free(decay); free(cur); free(tmp); free(x); free(y); free(q);
      free(attn); free(attn_ln); free(mixed); free(mlp);
      return -1;
    }
    memcpy(tmp + r * d, m->embed + (size_t)tok * d, sizeof(float) * d);
  }
  orc_layer_norm(tmp, (int64_t)rows, d, cur);
  const int64_t start_pos = *position; /* :334 */

  for (int l = 0; l < L; ++l) { /* :336, same weights every layer */
    float *rho_l = rho + (size_t)l * B * h * (size_t)Nq * d;
    /* :337-351 x = relu(cur . encoder - thr) */
    orc_relu_lowrank(cur, B, 1, T, d, m->encoder, h, N, NULL, m->relu_threshold, 1, NULL, 0, x);
    if (x_tap) memcpy(x_tap + (size_t)l * B * h * T * N, x, sizeof(float) * (size_t)B * h * T * N);
    /* :353-358 recurrent attention, value = cur */
    orc_rotate(x, B, h, T, N, freqs, m->rotary, start_pos, q);
    if (sparse_state && !decay)
      orc_recurrent_attention_sparse(q, cur, rho_l, B, h, T, Nq, d, attn);
    else
      orc_recurrent_attention(q, cur, rho_l, decay, B, h, T, Nq, d, attn);
    if (attn_tap)
      memcpy(attn_tap + (size_t)l * B * h * T * d, attn, sizeof(float) * (size_t)B * h * T * d);
    /* :359 */
    orc_layer_norm(attn, (int64_t)B * h * T, d, attn_ln);
    /* :361-375 y = relu(LN(attn) . encoder_v - thr) */
    orc_relu_lowrank(attn_ln, B, h, T, d, m->encoder_v, h, N, NULL, m->relu_threshold, 1, NULL, 0, y);
    /* :380 xy = x*y ; :383 swap_dims(1,2) ; :436 reshape [B*T, h*N] */
    for (int b = 0; b < B; ++b)
      for (int hh = 0; hh < h; ++hh)
        for (int t = 0; t < T; ++t) {
          const float *xr = x + (((size_t)b * h + hh) * T + t) * N;
          const float *yr = y + (((size_t)b * h + hh) * T + t) * N;
          float *mr = mixed + ((size_t)b * T + t) * (size_t)h * N + (size_t)hh * N;
          for (int n = 0; n < N; ++n) mr[n] = xr[n] * yr[n];
        }
    /* :386-434 (feature "viz"): x, y, x*y of the first sequence's last token, and the energy of
     * the updated state (zeros when the state is not [B,h,N,d], i.e. for PoPE's 2N rows) */
    if (viz && T > 0) {
      float *vz = viz + (size_t)l * 4 * h * N;
      for (int hh = 0; hh < h; ++hh) {
        const size_t src = ((size_t)hh * T + (T - 1)) * N; /* b = 0 */
        memcpy(vz + (size_t)hh * N, x + src, sizeof(float) * N);
        memcpy(vz + (size_t)(h + hh) * N, y + src, sizeof(float) * N);
        for (int n = 0; n < N; ++n) vz[(size_t)(2 * h + hh) * N + n] = x[src + n] * y[src + n];
      }
      if (Nq == N)
        orc_rho_energy(rho_l, B, h, N, d, vz + (size_t)3 * h * N);
      else
        memset(vz + (size_t)3 * h * N, 0, sizeof(float) * (size_t)h * N);
    }
    /* :438 mlp = mixed . decoder */
#pragma omp parallel for
    for (int64_t r = 0; r < (int64_t)rows; ++r)
      orc_matmul(mixed + (size_t)r * h * N, m->decoder, 1, h * N, d, mlp + (size_t)r * d);
    /* :440-441 cur = LN(cur + LN(mlp)) */
    orc_layer_norm(mlp, (int64_t)rows, d, tmp);
    for (size_t i = 0; i < rows * d; ++i) tmp[i] = cur[i] + tmp[i];
    orc_layer_norm(tmp, (int64_t)rows, d, cur);
  }
  /* :445 saturating_add */
  if (*position > INT64_MAX - (int64_t)T)
    *position = INT64_MAX;
  else
    *position += T;
  /* :446-449 logits = cur . lm_head */
  orc_matmul(cur, m->lm_head, (int)rows, d, V, logits);

  free(freqs); free(slopes); free(decay); free(cur); free(tmp); free(x); free(y); free(q);
  free(attn); free(attn_ln); free(mixed); free(mlp);
  return 0;
}

int orc_forward_with_state(const orc_model *m, const int64_t *tokens, int B, int T, float *rho,
                           int64_t *position, float *logits, float *x_tap, float *attn_tap,
                           int sparse_state) {
  return orc_forward_impl(m, tokens, B, T, rho, position, logits, x_tap, attn_tap, sparse_state, NULL);
}

/* forward_with_state built with the reference's "viz" feature: viz [L,4,h,N] receives, per layer,
 * x_last, y_last, xy_last and rho_last of LayerVizState (src/model/state.rs:17-24). */
int orc_forward_with_state_viz(const orc_model *m, const int64_t *tokens, int B, int T, float *rho,
                               int64_t *position, float *logits, int sparse_state, float *viz) {
  return orc_forward_impl(m, tokens, B, T, rho, position, logits, NULL, NULL, sparse_state, viz);
}

/* src/generation.rs:26-72 with top_k = Some(1): everything below the maximum is
 * masked to -inf, softmax is one-hot on the maxima and WeightedIndex draws among
 * them; with a unique maximum that is argmax.  Ties resolve to the lowest index
 * here (the reference would draw at random among tied maxima). */
int orc_greedy_token(const float *logits, int V) {
  int best = 0;
  for (int i = 1; i < V; ++i)
    if (logits[i] > logits[best]) best = i;
  return best;
}

/* sample_next_token's temperature division (src/generation.rs:117) followed by
 * sample_from_logits_values (:26-72), with the random draw made explicit: `u` in
 * [0,1) stands for the uniform variate WeightedIndex takes from thread_rng.
 * WeightedIndex (rand 0.8) keeps the running sums of the first V-1 weights, draws
 * `chosen` uniformly in [0, total) and returns the number of running sums that
 * are <= chosen.  All sums run in index order in binary32, as the iterator sums
 * of the reference do.  The k-th largest value is found by a full descending sort
 * like the reference's (:40-41); ties with it survive the mask (:43-45). */
static int orc_cmp_desc(const void *a, const void *b) {
  const float x = *(const float *)a, y = *(const float *)b;
  return (x < y) - (x > y);
}
int orc_sample_from_logits(const float *logits, int V, float temperature, int top_k, float u,
                           float *probs_out) {
  float *v = (float *)malloc(sizeof(float) * (size_t)V * 2);
  float *sorted = v + V;
  for (int i = 0; i < V; ++i) v[i] = logits[i] / temperature;
  if (top_k > 0 && top_k < V) {
    memcpy(sorted, v, sizeof(float) * (size_t)V);
    qsort(sorted, (size_t)V, sizeof(float), orc_cmp_desc);
    const float threshold = sorted[top_k - 1];
    for (int i = 0; i < V; ++i)
      if (v[i] < threshold) v[i] = -INFINITY;
  }
  float m = -INFINITY;
  for (int i = 0; i < V; ++i) m = fmaxf(m, v[i]);
  float sum = 0.f;
  for (int i = 0; i < V; ++i) {
    v[i] = expf(v[i] - m);
    sum += v[i];
  }
  const int flat = (sum == 0.f) || (sum != sum);
  float total = 0.f;
  for (int i = 0; i < V; ++i) {
    v[i] = flat ? 1.0f / (float)V : v[i] / sum;
    total += v[i];
  }
  if (probs_out) memcpy(probs_out, v, sizeof(float) * (size_t)V);
  if (u < 0.f) u = 0.f;
  if (u > 0.99999994f) u = 0.99999994f;
  const float chosen = u * total;
  float cum = 0.f;
  int idx = 0;
  for (int i = 0; i < V - 1; ++i) {
    cum += v[i];
    if (cum <= chosen) idx = i + 1;
    else break;
  }
  free(v);
  return idx;
}

/* One dense decode step of the single-layer microbenchmark shape (rotate +
 * recurrent_attention with T = 1), used as the timed CPU baseline. */
void orc_state_step_dense(const float *x, const float *v, const float *freqs, int64_t position,
                          float *rho, int B, int h, int N, int d, float *q_scratch, float *out) {
  orc_rotate(x, B, h, 1, N, freqs, ORC_ROPE, position, q_scratch);
  orc_recurrent_attention(q_scratch, v, rho, NULL, B, h, 1, N, d, out);
}
