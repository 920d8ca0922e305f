/*
 * CPU restatement (C, fp32 storage, OpenMP) of mograd's backward hot path.
 *
 * TEST INFRASTRUCTURE ONLY: loaded by the tests and by the benchmark's CPU-baseline
 * leg through ctypes.  The shipped library never links or calls it.
 *
 * mograd has no CPU runtime (mograd/runtime/__init__.mojo:58,67-68), so this file
 * follows the pass structure of the reference's GPU kernels, one row per OpenMP
 * iteration, and is what the benchmark times as "the reference's arithmetic on the
 * host cores".  Accumulators are fp32 like the kernels' (`get_accum_type[f32]` is
 * f32), except where noted.  Each function cites the lines it restates.
 *
 * Checked in tests/test_oracle.py against the float64 numpy oracle, which is in
 * turn pinned by the reference's golden vectors.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

int orc_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* ---- LayerNorm forward: mograd/nn/modules/normalization.mojo:17-27 -------- */
void orc_layer_norm_fwd_f32(const float* x, const float* gamma, const float* beta, float* y,
                            int64_t rows, int64_t cols, float eps) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    const float* xr = x + r * cols;
    float sx = 0.f, sx2 = 0.f;
    for (int64_t c = 0; c < cols; ++c) { sx += xr[c]; sx2 += xr[c] * xr[c]; }
    float mu = sx / (float)cols;
    float var = fmaxf(sx2 / (float)cols - mu * mu, 0.f);
    float rstd = 1.0f / sqrtf(var + eps);
    for (int64_t c = 0; c < cols; ++c) y[r * cols + c] = (xr[c] - mu) * rstd * gamma[c] + beta[c];
  }
}

/* ---- LayerNorm backward: kernels/normalization.mojo:85-178 (three passes per row,
 * per-group partial dgamma/dbeta) and :281-303 (group reduction).  `groups` plays the
 * role of num_sm. ------------------------------------------------------------------ */
void orc_layer_norm_bwd_f32(const float* dy, const float* x, const float* gamma, float* dx,
                            float* dgamma, float* dbeta, int64_t rows, int64_t cols, float eps,
                            int64_t groups) {
  if (groups > rows) groups = rows;
  if (groups < 1) groups = 1;
  int64_t group_size = (rows + groups - 1) / groups;
  float* tmp_g = (float*)calloc((size_t)(groups * cols), sizeof(float));
  float* tmp_b = (float*)calloc((size_t)(groups * cols), sizeof(float));
#pragma omp parallel for schedule(static)
  for (int64_t g = 0; g < groups; ++g) {
    int64_t r0 = g * group_size, r1 = r0 + group_size;
    if (r1 > rows) r1 = rows;
    float* pg = tmp_g + g * cols;
    float* pb = tmp_b + g * cols;
    for (int64_t r = r0; r < r1; ++r) {
      const float* xr = x + r * cols;
      const float* dyr = dy + r * cols;
      float sx = 0.f, sx2 = 0.f;
      for (int64_t c = 0; c < cols; ++c) { sx += xr[c]; sx2 += xr[c] * xr[c]; }
      float n = (float)cols;
      float mu = sx / n;
      float rstd = 1.0f / sqrtf(fmaxf(sx2 / n - mu * mu, 0.f) + eps);
      float t1 = 0.f, t2 = 0.f;
      for (int64_t c = 0; c < cols; ++c) {
        float xhat = (xr[c] - mu) * rstd;
        float dyg = dyr[c] * gamma[c];
        t1 += dyg;
        t2 += dyg * xhat;
      }
      float c1 = t1 / n, c2 = t2 / n;
      for (int64_t c = 0; c < cols; ++c) {
        float xhat = (xr[c] - mu) * rstd;
        dx[r * cols + c] = rstd * (dyr[c] * gamma[c] - c1 - xhat * c2);
        pg[c] += dyr[c] * xhat;
        pb[c] += dyr[c];
      }
    }
  }
#pragma omp parallel for schedule(static)
  for (int64_t c = 0; c < cols; ++c) {
    float ag = 0.f, ab = 0.f;
    for (int64_t g = 0; g < groups; ++g) { ag += tmp_g[g * cols + c]; ab += tmp_b[g * cols + c]; }
    dgamma[c] = ag;
    dbeta[c] = ab;
  }
  free(tmp_g);
  free(tmp_b);
}

/* ---- Cross-entropy forward, dense labels: kernels/cross_entropy.mojo:35-77 then
 * sum_rows :155-177. ------------------------------------------------------------- */
float orc_cross_entropy_f32(const float* logits, const float* labels, int64_t N, int64_t C) {
  float* rowloss = (float*)malloc((size_t)N * sizeof(float));
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < N; ++r) {
    const float* xr = logits + r * C;
    const float* yr = labels + r * C;
    float m = -INFINITY;
    for (int64_t c = 0; c < C; ++c) m = xr[c] > m ? xr[c] : m;
    float s = 0.f;
    for (int64_t c = 0; c < C; ++c) s += expf(xr[c] - m);
    float lse = logf(s);
    float acc = 0.f;
    for (int64_t c = 0; c < C; ++c) acc += (xr[c] - m - lse) * yr[c];
    rowloss[r] = -acc / (float)N;
  }
  float total = 0.f;
  for (int64_t r = 0; r < N; ++r) total += rowloss[r];
  free(rowloss);
  return total;
}

/* ---- Cross-entropy gradient, dense labels: kernels/cross_entropy.mojo:207-241. -- */
void orc_cross_entropy_grad_f32(const float* logits, const float* labels, const float* upstream,
                                float* dst, int64_t N, int64_t C) {
  float d_by_n = upstream[0] / (float)N;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < N; ++r) {
    const float* xr = logits + r * C;
    const float* yr = labels + r * C;
    float m = -INFINITY;
    for (int64_t c = 0; c < C; ++c) m = xr[c] > m ? xr[c] : m;
    float s = 0.f;
    for (int64_t c = 0; c < C; ++c) s += expf(xr[c] - m);
    float inv = 1.0f / s;
    for (int64_t c = 0; c < C; ++c) dst[r * C + c] = (expf(xr[c] - m) * inv - yr[c]) * d_by_n;
  }
}

/* ---- Integer-label forms (same arithmetic with label = one_hot(id)). ----------- */
float orc_cross_entropy_ids_f32(const float* logits, const int32_t* ids, int64_t N, int64_t C) {
  float* rowloss = (float*)malloc((size_t)N * sizeof(float));
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < N; ++r) {
    const float* xr = logits + r * C;
    float m = -INFINITY;
    for (int64_t c = 0; c < C; ++c) m = xr[c] > m ? xr[c] : m;
    float s = 0.f;
    for (int64_t c = 0; c < C; ++c) s += expf(xr[c] - m);
    rowloss[r] = -(xr[ids[r]] - m - logf(s)) / (float)N;
  }
  float total = 0.f;
  for (int64_t r = 0; r < N; ++r) total += rowloss[r];
  free(rowloss);
  return total;
}

void orc_cross_entropy_grad_ids_f32(const float* logits, const int32_t* ids, const float* upstream,
                                    float* dst, int64_t N, int64_t C) {
  float d_by_n = upstream[0] / (float)N;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < N; ++r) {
    const float* xr = logits + r * C;
    float m = -INFINITY;
    for (int64_t c = 0; c < C; ++c) m = xr[c] > m ? xr[c] : m;
    float s = 0.f;
    for (int64_t c = 0; c < C; ++c) s += expf(xr[c] - m);
    float inv = 1.0f / s;
    for (int64_t c = 0; c < C; ++c) {
      float y = (c == ids[r]) ? 1.f : 0.f;
      dst[r * C + c] = (expf(xr[c] - m) * inv - y) * d_by_n;
    }
  }
}

/* ---- Linear forward and gradients.  Forward: kernels/__init__.mojo:778-809
 * (X W^T + b[n]).  dX = dY W and dW^T = X^T dY: mograd/grad.mojo:183, run by the
 * strided naive kernel, one fp32 accumulator per output element in k order
 * (kernels/__init__.mojo:663-682,734-753).  db: kernels/reduce.mojo:137-173. ----- */
void orc_matmul_bias_bt_f32(const float* x, const float* w, const float* b, float* y, int64_t M,
                            int64_t N, int64_t K) {
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m)
    for (int64_t n = 0; n < N; ++n) {
      float acc = 0.f;
      for (int64_t k = 0; k < K; ++k) acc += x[m * K + k] * w[n * K + k];
      y[m * N + n] = b ? acc + b[n] : acc;
    }
}

/* dX(M,K) = dY(M,N) W(N,K) */
void orc_linear_grad_x_f32(const float* dy, const float* w, float* dx, int64_t M, int64_t N,
                           int64_t K) {
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    float* out = dx + m * K;
    for (int64_t k = 0; k < K; ++k) out[k] = 0.f;
    for (int64_t n = 0; n < N; ++n) {
      float a = dy[m * N + n];
      const float* wr = w + n * K;
      for (int64_t k = 0; k < K; ++k) out[k] += a * wr[k];
    }
  }
}

/* dW(N,K) = dY(M,N)^T X(M,K) */
void orc_linear_grad_w_f32(const float* dy, const float* x, float* dw, int64_t M, int64_t N,
                           int64_t K) {
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < N; ++n) {
    float* out = dw + n * K;
    for (int64_t k = 0; k < K; ++k) out[k] = 0.f;
    for (int64_t m = 0; m < M; ++m) {
      float a = dy[m * N + n];
      const float* xr = x + m * K;
      for (int64_t k = 0; k < K; ++k) out[k] += a * xr[k];
    }
  }
}

void orc_linear_grad_b_f32(const float* dy, float* db, int64_t M, int64_t N) {
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < N; ++n) {
    float acc = 0.f;
    for (int64_t m = 0; m < M; ++m) acc += dy[m * N + n];
    db[n] = acc;
  }
}

void orc_relu_grad_f32(const float* out, const float* up, float* dst, int64_t n) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) dst[i] = out[i] > 0.f ? up[i] : 0.f;
}

/* ---- Attention, naive O(S^2): tests/kernels/attention/harness.mojo:58-175, with fp32
 * storage and fp32 math (the generic kernels compute in fp32 after load,
 * attention/generic.mojo:287-713).  Q,K,V,dQ,dK,dV BSHD; O,dO BHSD; mask (B,H,S,S);
 * lse natural log.  `bh_limit` bounds the (b,h) pairs processed (for bounded timing
 * samples); pass B*H for everything. -------------------------------------------- */
void orc_sdpa_fwd_f32(const float* q, const float* k, const float* v, const float* mask,
                      int has_mask, int causal, float* out, float* lse, int64_t B, int64_t S,
                      int64_t H, int64_t D, float scale, int64_t bh_limit) {
  int64_t BH = B * H;
  if (bh_limit < BH) BH = bh_limit;
#pragma omp parallel for schedule(dynamic, 8) collapse(2)
  for (int64_t bh = 0; bh < BH; ++bh)
    for (int64_t i = 0; i < S; ++i) {
      int64_t b = bh / H, h = bh % H;
      float* sc = (float*)malloc((size_t)S * sizeof(float));
      int64_t j_end = causal ? i + 1 : S;
      const float* qi = q + ((b * S + i) * H + h) * D;
      float row_max = -INFINITY;
      for (int64_t j = 0; j < j_end; ++j) {
        const float* kj = k + ((b * S + j) * H + h) * D;
        float s = 0.f;
        for (int64_t d = 0; d < D; ++d) s += qi[d] * kj[d];
        s *= scale;
        if (has_mask) s += mask[(bh * S + i) * S + j];
        sc[j] = s;
        if (s > row_max) row_max = s;
      }
      float denom = 0.f;
      for (int64_t j = 0; j < j_end; ++j) { sc[j] = expf(sc[j] - row_max); denom += sc[j]; }
      float* oi = out + (bh * S + i) * D;
      for (int64_t d = 0; d < D; ++d) oi[d] = 0.f;
      for (int64_t j = 0; j < j_end; ++j) {
        const float* vj = v + ((b * S + j) * H + h) * D;
        for (int64_t d = 0; d < D; ++d) oi[d] += sc[j] * vj[d];
      }
      for (int64_t d = 0; d < D; ++d) oi[d] /= denom;
      lse[bh * S + i] = row_max + logf(denom);
      free(sc);
    }
}

void orc_sdpa_bwd_f32(const float* q, const float* k, const float* v, const float* dy,
                      const float* mask, int has_mask, int causal, float* dq, float* dk, float* dv,
                      int64_t B, int64_t S, int64_t H, int64_t D, float scale, int64_t bh_limit) {
  int64_t BH = B * H;
  if (bh_limit < BH) BH = bh_limit;
  /* zero the (b,h) slices that will be written */
  for (int64_t bh = 0; bh < BH; ++bh) {
    int64_t b = bh / H, h = bh % H;
    for (int64_t s = 0; s < S; ++s) {
      int64_t base = ((b * S + s) * H + h) * D;
      memset(dq + base, 0, (size_t)D * sizeof(float));
      memset(dk + base, 0, (size_t)D * sizeof(float));
      memset(dv + base, 0, (size_t)D * sizeof(float));
    }
  }
  /* one (b,h) per iteration: dK/dV rows are shared across query rows */
#pragma omp parallel for schedule(dynamic, 1)
  for (int64_t bh = 0; bh < BH; ++bh) {
    int64_t b = bh / H, h = bh % H;
    float* p = (float*)malloc((size_t)S * sizeof(float));
    for (int64_t i = 0; i < S; ++i) {
      int64_t j_end = causal ? i + 1 : S;
      const float* qi = q + ((b * S + i) * H + h) * D;
      const float* dyi = dy + (bh * S + i) * D;
      float row_max = -INFINITY;
      for (int64_t j = 0; j < j_end; ++j) {
        const float* kj = k + ((b * S + j) * H + h) * D;
        float s = 0.f;
        for (int64_t d = 0; d < D; ++d) s += qi[d] * kj[d];
        s *= scale;
        if (has_mask) s += mask[(bh * S + i) * S + j];
        p[j] = s;
        if (s > row_max) row_max = s;
      }
      float denom = 0.f;
      for (int64_t j = 0; j < j_end; ++j) { p[j] = expf(p[j] - row_max); denom += p[j]; }
      for (int64_t j = 0; j < j_end; ++j) p[j] /= denom;
      float delta = 0.f;
      for (int64_t d = 0; d < D; ++d) {
        float od = 0.f;
        for (int64_t j = 0; j < j_end; ++j) od += p[j] * v[((b * S + j) * H + h) * D + d];
        delta += dyi[d] * od;
      }
      float* dqi = dq + ((b * S + i) * H + h) * D;
      for (int64_t j = 0; j < j_end; ++j) {
        const float* kj = k + ((b * S + j) * H + h) * D;
        const float* vj = v + ((b * S + j) * H + h) * D;
        float dp = 0.f;
        for (int64_t d = 0; d < D; ++d) dp += dyi[d] * vj[d];
        float ds = p[j] * (dp - delta) * scale;
        float* dkj = dk + ((b * S + j) * H + h) * D;
        float* dvj = dv + ((b * S + j) * H + h) * D;
        for (int64_t d = 0; d < D; ++d) {
          dqi[d] += ds * kj[d];
          dkj[d] += ds * qi[d];
          dvj[d] += p[j] * dyi[d];
        }
      }
    }
    free(p);
  }
}

/* ---- Pool size class: mograd/memory.mojo:59-72 -------------------------------- */
int64_t orc_round_class(int64_t nbytes) {
  if (nbytes <= 512) return 512;
  int64_t p = 1;
  while ((p << 1) <= nbytes) p <<= 1;
  if (p == nbytes) return nbytes;
  int64_t step = p / 8;
  return ((nbytes + step - 1) / step) * step;
}
