/*
 * CPU oracle for the rembrandt single-GPU operator hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or calls this file;
 * it exists to check the HIP kernels (tests, the smoke check) and to provide the timed CPU
 * baseline of the benchmark.  It restates, in plain C, what the reference's operators ask of
 * their (un-vendored) cuDNN / cuBLAS / custom-kernel back ends; every function cites the
 * reference call site it follows (paths relative to the reference tree).
 *
 * Two families:
 *   orc_*       "precise": fp32 storage, fp64 accumulation, direct loops.  The parity checker.
 *   orc_fast_*  fp32 im2col + blocked SGEMM with OpenMP.  The timed CPU baseline; itself
 *               checked against the precise family in the CPU test-suite.
 *
 * Parity status: the reference holds no golden vectors, known-answer tests or fixtures for this
 * path (its tests assert nothing) and its arithmetic lives in crates that are not in its tree,
 * so no function here can be pinned against reference outputs.  Each function is pinned
 * instead by the CPU test-suite against independent statements of the same mathematics
 * (torch CPU fp64 library routines, numpy brute force on tiny inputs, adjoint identities,
 * closed forms, finite differences).  Semantic choices the reference leaves to code outside
 * its tree ("parity unpinned" against the reference itself): cross-correlation convolution mode,
 * ReLU sub-gradient 0 at y == 0, first-maximum tie rule for max-pool and arg-max, max-pool
 * padding never wins, average-pool divisor size*size also for clipped ceil-mode windows,
 * max-subtracted softmax, the trailing float of softmax_kl_loss1 taken as an accumulate factor.
 *
 * Layouts: activations NCHW (W fastest), filters [K][C][R][S], affine weights [out][in],
 * affine activations [batch][chan] (src/operator/mod.rs:1471-1474, src/arch_new.rs:141-145).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

typedef struct { int32_t N, C, H, W, K, R, S, stride, pad; } orc_conv_geom;
typedef struct { int32_t N, C, H, W, size, stride, pad, mode, round; } orc_pool_geom;
enum { ORC_POOL_MAX = 0, ORC_POOL_AVG = 1 };
enum { ORC_ROUND_FLOOR = 0, ORC_ROUND_CEIL = 1 };

int orc_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* Output extent of a convolution / operator-style pooling window:
 * max(0, in + 2*pad - size + stride) / stride   (src/operator/mod.rs:1393-1398, 2022-2027). */
int32_t orc_out_dim_floor(int32_t in, int32_t size, int32_t stride, int32_t pad) {
  int32_t t = in + 2 * pad - size + stride;
  if (t < 0) t = 0;
  return t / stride;
}

/* Gen-1 pooling extent (ceil): max(0, in + 2*pad - size + stride - 1)/stride + 1 (src/layer.rs:1741-1747). */
int32_t orc_out_dim_ceil(int32_t in, int32_t size, int32_t stride, int32_t pad) {
  int32_t t = in + 2 * pad - size + stride - 1;
  if (t < 0) t = 0;
  return t / stride + 1;
}

static int32_t pool_out_dim(int32_t in, const orc_pool_geom* g) {
  return g->round == ORC_ROUND_CEIL ? orc_out_dim_ceil(in, g->size, g->stride, g->pad)
                                    : orc_out_dim_floor(in, g->size, g->stride, g->pad);
}

/* ------------------------------------------------------------------------------------------
 * Convolution, precise family.
 * ---------------------------------------------------------------------------------------- */

/* K1: y = alpha * corr(x, w) + beta * y   (CudnnConvFwdOp::forward, src/operator/mod.rs:1684-1696) */
void orc_conv2d_fwd(const orc_conv_geom* g, float alpha, const float* x, const float* w,
                    float beta, float* y) {
  const int N = g->N, C = g->C, H = g->H, W = g->W, K = g->K, R = g->R, S = g->S;
  const int st = g->stride, pad = g->pad;
  const int P = orc_out_dim_floor(H, R, st, pad), Q = orc_out_dim_floor(W, S, st, pad);
  if (P <= 0 || Q <= 0) return;
#pragma omp parallel
  {
    double* acc = (double*)malloc(sizeof(double) * (size_t)Q);
#pragma omp for collapse(2) schedule(static)
    for (int n = 0; n < N; ++n)
      for (int k = 0; k < K; ++k)
        for (int p = 0; p < P; ++p) {
          for (int q = 0; q < Q; ++q) acc[q] = 0.0;
          for (int c = 0; c < C; ++c)
            for (int r = 0; r < R; ++r) {
              const int h = p * st + r - pad;
              if (h < 0 || h >= H) continue;
              const float* xrow = x + (((size_t)n * C + c) * H + h) * W;
              const float* wrow = w + (((size_t)k * C + c) * R + r) * S;
              for (int s = 0; s < S; ++s) {
                const double wv = wrow[s];
                for (int q = 0; q < Q; ++q) {
                  const int ww = q * st + s - pad;
                  if (ww >= 0 && ww < W) acc[q] += wv * (double)xrow[ww];
                }
              }
            }
          float* yrow = y + (((size_t)n * K + k) * P + p) * Q;
          for (int q = 0; q < Q; ++q) {
            double v = (double)alpha * acc[q];
            if (beta != 0.0f) v += (double)beta * (double)yrow[q];
            yrow[q] = (float)v;
          }
        }
    free(acc);
  }
}

/* One output element of K1 (no alpha/beta), for sampled checks at sizes where the full
 * oracle would take minutes. idx is a flat index into y[N][K][P][Q]. */
void orc_conv2d_fwd_at(const orc_conv_geom* g, const float* x, const float* w,
                       const int64_t* idx, int64_t n_idx, float* out) {
  const int C = g->C, H = g->H, W = g->W, K = g->K, R = g->R, S = g->S;
  const int st = g->stride, pad = g->pad;
  const int P = orc_out_dim_floor(H, R, st, pad), Q = orc_out_dim_floor(W, S, st, pad);
#pragma omp parallel for schedule(dynamic, 64)
  for (int64_t i = 0; i < n_idx; ++i) {
    int64_t t = idx[i];
    const int q = (int)(t % Q); t /= Q;
    const int p = (int)(t % P); t /= P;
    const int k = (int)(t % K); t /= K;
    const int n = (int)t;
    double acc = 0.0;
    for (int c = 0; c < C; ++c)
      for (int r = 0; r < R; ++r) {
        const int h = p * st + r - pad;
        if (h < 0 || h >= H) continue;
        for (int s = 0; s < S; ++s) {
          const int ww = q * st + s - pad;
          if (ww < 0 || ww >= W) continue;
          acc += (double)w[(((size_t)k * C + c) * R + r) * S + s] *
                 (double)x[(((size_t)n * C + c) * H + h) * W + ww];
        }
      }
    out[i] = (float)acc;
  }
}

/* K5: dw = beta*dw + alpha * sum_{n,p,q} dy * x   (backward_filter, src/operator/mod.rs:1765-1774) */
void orc_conv2d_bwd_filter(const orc_conv_geom* g, float alpha, const float* x, const float* dy,
                           float beta, float* dw) {
  const int N = g->N, C = g->C, H = g->H, W = g->W, K = g->K, R = g->R, S = g->S;
  const int st = g->stride, pad = g->pad;
  const int P = orc_out_dim_floor(H, R, st, pad), Q = orc_out_dim_floor(W, S, st, pad);
#pragma omp parallel for collapse(2) schedule(static)
  for (int k = 0; k < K; ++k)
    for (int c = 0; c < C; ++c)
      for (int r = 0; r < R; ++r)
        for (int s = 0; s < S; ++s) {
          double acc = 0.0;
          for (int n = 0; n < N; ++n)
            for (int p = 0; p < P; ++p) {
              const int h = p * st + r - pad;
              if (h < 0 || h >= H) continue;
              const float* xrow = x + (((size_t)n * C + c) * H + h) * W;
              const float* dyrow = dy + (((size_t)n * K + k) * P + p) * Q;
              for (int q = 0; q < Q; ++q) {
                const int ww = q * st + s - pad;
                if (ww >= 0 && ww < W) acc += (double)dyrow[q] * (double)xrow[ww];
              }
            }
          float* d = dw + (((size_t)k * C + c) * R + r) * S + s;
          double v = (double)alpha * acc;
          if (beta != 0.0f) v += (double)beta * (double)*d;
          *d = (float)v;
        }
}

/* Sampled K5 (no alpha/beta): idx flat into dw[K][C][R][S]. */
void orc_conv2d_bwd_filter_at(const orc_conv_geom* g, const float* x, const float* dy,
                              const int64_t* idx, int64_t n_idx, float* out) {
  const int N = g->N, C = g->C, H = g->H, W = g->W, K = g->K, R = g->R, S = g->S;
  const int st = g->stride, pad = g->pad;
  const int P = orc_out_dim_floor(H, R, st, pad), Q = orc_out_dim_floor(W, S, st, pad);
#pragma omp parallel for schedule(dynamic, 1)
  for (int64_t i = 0; i < n_idx; ++i) {
    int64_t t = idx[i];
    const int s = (int)(t % S); t /= S;
    const int r = (int)(t % R); t /= R;
    const int c = (int)(t % C); t /= C;
    const int k = (int)t;
    double acc = 0.0;
    for (int n = 0; n < N; ++n)
      for (int p = 0; p < P; ++p) {
        const int h = p * st + r - pad;
        if (h < 0 || h >= H) continue;
        const float* xrow = x + (((size_t)n * C + c) * H + h) * W;
        const float* dyrow = dy + (((size_t)n * K + k) * P + p) * Q;
        for (int q = 0; q < Q; ++q) {
          const int ww = q * st + s - pad;
          if (ww >= 0 && ww < W) acc += (double)dyrow[q] * (double)xrow[ww];
        }
      }
    out[i] = (float)acc;
  }
}

/* K6: db[k] = beta*db + alpha * sum_{n,p,q} dy[n,k,p,q]  (backward_bias, src/operator/mod.rs:1775-1781) */
void orc_conv2d_bwd_bias(int32_t N, int32_t K, int32_t plane, float alpha, const float* dy,
                         float beta, float* db) {
#pragma omp parallel for schedule(static)
  for (int k = 0; k < K; ++k) {
    double acc = 0.0;
    for (int n = 0; n < N; ++n) {
      const float* p = dy + ((size_t)n * K + k) * plane;
      for (int i = 0; i < plane; ++i) acc += (double)p[i];
    }
    double v = (double)alpha * acc;
    if (beta != 0.0f) v += (double)beta * (double)db[k];
    db[k] = (float)v;
  }
}

/* K7: dx = alpha * corr^T(dy, w) + beta*dx   (backward_data, src/operator/mod.rs:1783-1793) */
void orc_conv2d_bwd_data(const orc_conv_geom* g, float alpha, const float* w, const float* dy,
                         float beta, float* dx) {
  const int N = g->N, C = g->C, H = g->H, W = g->W, K = g->K, R = g->R, S = g->S;
  const int st = g->stride, pad = g->pad;
  const int P = orc_out_dim_floor(H, R, st, pad), Q = orc_out_dim_floor(W, S, st, pad);
#pragma omp parallel
  {
    double* acc = (double*)malloc(sizeof(double) * (size_t)H * W);
#pragma omp for collapse(2) schedule(static)
    for (int n = 0; n < N; ++n)
      for (int c = 0; c < C; ++c) {
        for (int i = 0; i < H * W; ++i) acc[i] = 0.0;
        for (int k = 0; k < K; ++k)
          for (int r = 0; r < R; ++r)
            for (int s = 0; s < S; ++s) {
              const double wv = w[(((size_t)k * C + c) * R + r) * S + s];
              for (int p = 0; p < P; ++p) {
                const int h = p * st + r - pad;
                if (h < 0 || h >= H) continue;
                const float* dyrow = dy + (((size_t)n * K + k) * P + p) * Q;
                double* arow = acc + (size_t)h * W;
                for (int q = 0; q < Q; ++q) {
                  const int ww = q * st + s - pad;
                  if (ww >= 0 && ww < W) arow[ww] += wv * (double)dyrow[q];
                }
              }
            }
        float* d = dx + ((size_t)n * C + c) * H * W;
        for (int i = 0; i < H * W; ++i) {
          double v = (double)alpha * acc[i];
          if (beta != 0.0f) v += (double)beta * (double)d[i];
          d[i] = (float)v;
        }
      }
    free(acc);
  }
}

/* Sampled K7 (no alpha/beta): idx flat into dx[N][C][H][W]; gather form. */
void orc_conv2d_bwd_data_at(const orc_conv_geom* g, const float* w, const float* dy,
                            const int64_t* idx, int64_t n_idx, float* out) {
  const int C = g->C, H = g->H, W = g->W, K = g->K, R = g->R, S = g->S;
  const int st = g->stride, pad = g->pad;
  const int P = orc_out_dim_floor(H, R, st, pad), Q = orc_out_dim_floor(W, S, st, pad);
#pragma omp parallel for schedule(dynamic, 64)
  for (int64_t i = 0; i < n_idx; ++i) {
    int64_t t = idx[i];
    const int ww = (int)(t % W); t /= W;
    const int h = (int)(t % H); t /= H;
    const int c = (int)(t % C); t /= C;
    const int n = (int)t;
    double acc = 0.0;
    for (int k = 0; k < K; ++k)
      for (int r = 0; r < R; ++r) {
        const int hp = h + pad - r;
        if (hp < 0 || hp % st) continue;
        const int p = hp / st;
        if (p >= P) continue;
        for (int s = 0; s < S; ++s) {
          const int wq = ww + pad - s;
          if (wq < 0 || wq % st) continue;
          const int q = wq / st;
          if (q >= Q) continue;
          acc += (double)dy[(((size_t)n * K + k) * P + p) * Q + q] *
                 (double)w[(((size_t)k * C + c) * R + r) * S + s];
        }
      }
    out[i] = (float)acc;
  }
}

/* ------------------------------------------------------------------------------------------
 * Bias add, ReLU.
 * ---------------------------------------------------------------------------------------- */

/* K2: y[n,k,:] = alpha*bias[k] + beta*y[n,k,:]  (CudnnAddOp::forward, src/operator/mod.rs:1097-1103, 1697-1704) */
void orc_add_bias_nchw(const float* bias, float* y, int32_t plane, int32_t K, int32_t N,
                       float alpha, float beta) {
#pragma omp parallel for collapse(2) schedule(static)
  for (int n = 0; n < N; ++n)
    for (int k = 0; k < K; ++k) {
      float* p = y + ((size_t)n * K + k) * plane;
      const float b = alpha * bias[k];
      for (int i = 0; i < plane; ++i) p[i] = b + beta * p[i];
    }
}

/* K3: y = max(y, 0) in place (rembrandt_kernel_batch_map_rect_inplace, src/operator/mod.rs:1108-1113) */
void orc_rect_inplace(float* y, int32_t frame_len, int32_t batch) {
  const size_t n = (size_t)frame_len * batch;
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; ++i) y[i] = y[i] > 0.0f ? y[i] : 0.0f;
}

/* K4: dy *= [y > 0] in place (rembrandt_kernel_batch_map_rect_backprop_inplace, src/operator/mod.rs:1154-1160) */
void orc_rect_backprop_inplace(const float* y, int32_t frame_len, int32_t batch, float* dy) {
  const size_t n = (size_t)frame_len * batch;
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; ++i) dy[i] = y[i] > 0.0f ? dy[i] : 0.0f;
}

/* ------------------------------------------------------------------------------------------
 * Column-major SGEMM (K8) and BLAS-1 (K14), precise.
 * C(m,n) = alpha * op(A)(m,k) * op(B)(k,n) + beta * C   (matrix_prod, src/operator/mod.rs:1094,1168-1174)
 * ---------------------------------------------------------------------------------------- */
void orc_sgemm(int transA, int transB, int32_t m, int32_t n, int32_t k, float alpha,
               const float* A, int32_t lda, const float* B, int32_t ldb, float beta, float* C,
               int32_t ldc) {
#pragma omp parallel for collapse(2) schedule(static)
  for (int j = 0; j < n; ++j)
    for (int i = 0; i < m; ++i) {
      double acc = 0.0;
      for (int l = 0; l < k; ++l) {
        const double a = transA ? A[(size_t)i * lda + l] : A[(size_t)l * lda + i];
        const double b = transB ? B[(size_t)l * ldb + j] : B[(size_t)j * ldb + l];
        acc += a * b;
      }
      float* c = C + (size_t)j * ldc + i;
      double v = (double)alpha * acc;
      if (beta != 0.0f) v += (double)beta * (double)*c;
      *c = (float)v;
    }
}

/* y += alpha * x  (matrix_sum / row_vector_sum, src/operator/mod.rs:1186-1189) -- single fma-free fp32 ops */
void orc_saxpy(int64_t n, float alpha, const float* x, float* y) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) y[i] = (float)((double)y[i] + (double)alpha * (double)x[i]);
}

/* x *= alpha (matrix_scale / row_vector_scale, src/operator/mod.rs:1199-1202) */
void orc_sscal(int64_t n, float alpha, float* x) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) x[i] = alpha * x[i];
}

/* ------------------------------------------------------------------------------------------
 * Pooling (K9 operator-style batch pooling, K9' gen-1 with arg-max mask and ceil rounding).
 * src/operator/mod.rs:2044-2123, src/layer.rs:1741-1843
 * argmax (optional, may be NULL) receives, per output, the flat h*W+w index inside the input
 * plane of the selected tap, or -1 if the window holds no in-range tap.
 * ---------------------------------------------------------------------------------------- */
void orc_pool2d_fwd(const orc_pool_geom* g, const float* x, float* y, int32_t* argmax) {
  const int N = g->N, C = g->C, H = g->H, W = g->W, k = g->size, st = g->stride, pad = g->pad;
  const int P = pool_out_dim(H, g), Q = pool_out_dim(W, g);
  const float inv = 1.0f / (float)(k * k);
#pragma omp parallel for schedule(static)
  for (int nc = 0; nc < N * C; ++nc) {
    const float* xp = x + (size_t)nc * H * W;
    float* yp = y + (size_t)nc * P * Q;
    int32_t* ap = argmax ? argmax + (size_t)nc * P * Q : NULL;
    for (int p = 0; p < P; ++p)
      for (int q = 0; q < Q; ++q) {
        if (g->mode == ORC_POOL_MAX) {
          float best = -INFINITY;
          int bi = -1;
          for (int r = 0; r < k; ++r) {
            const int h = p * st + r - pad;
            if (h < 0 || h >= H) continue;
            for (int s = 0; s < k; ++s) {
              const int w = q * st + s - pad;
              if (w < 0 || w >= W) continue;
              const float v = xp[h * W + w];
              if (bi < 0 || v > best) { best = v; bi = h * W + w; }
            }
          }
          yp[p * Q + q] = bi < 0 ? 0.0f : best;
          if (ap) ap[p * Q + q] = bi;
        } else {
          double acc = 0.0;
          for (int r = 0; r < k; ++r) {
            const int h = p * st + r - pad;
            if (h < 0 || h >= H) continue;
            for (int s = 0; s < k; ++s) {
              const int w = q * st + s - pad;
              if (w < 0 || w >= W) continue;
              acc += (double)xp[h * W + w];
            }
          }
          yp[p * Q + q] = (float)(acc * (double)inv);
        }
      }
  }
}

/* dx is overwritten.  Max: dy routed to the first maximum of each window (r outer, s inner),
 * recomputed from x unless argmax is given; contributions of overlapping windows add.
 * Average: every in-range tap receives dy / size^2. */
void orc_pool2d_bwd(const orc_pool_geom* g, const float* x, const float* y, const float* dy,
                    float* dx, const int32_t* argmax) {
  (void)y;
  const int N = g->N, C = g->C, H = g->H, W = g->W, k = g->size, st = g->stride, pad = g->pad;
  const int P = pool_out_dim(H, g), Q = pool_out_dim(W, g);
  const double inv = 1.0 / (double)(k * k);
#pragma omp parallel
  {
    double* acc = (double*)malloc(sizeof(double) * (size_t)H * W);
#pragma omp for schedule(static)
    for (int nc = 0; nc < N * C; ++nc) {
      const float* xp = x + (size_t)nc * H * W;
      const float* dyp = dy + (size_t)nc * P * Q;
      const int32_t* ap = argmax ? argmax + (size_t)nc * P * Q : NULL;
      for (int i = 0; i < H * W; ++i) acc[i] = 0.0;
      for (int p = 0; p < P; ++p)
        for (int q = 0; q < Q; ++q) {
          const double d = dyp[p * Q + q];
          if (g->mode == ORC_POOL_MAX) {
            int bi = -1;
            if (ap) {
              bi = ap[p * Q + q];
            } else {
              float best = -INFINITY;
              for (int r = 0; r < k; ++r) {
                const int h = p * st + r - pad;
                if (h < 0 || h >= H) continue;
                for (int s = 0; s < k; ++s) {
                  const int w = q * st + s - pad;
                  if (w < 0 || w >= W) continue;
                  const float v = xp[h * W + w];
                  if (bi < 0 || v > best) { best = v; bi = h * W + w; }
                }
              }
            }
            if (bi >= 0) acc[bi] += d;
          } else {
            for (int r = 0; r < k; ++r) {
              const int h = p * st + r - pad;
              if (h < 0 || h >= H) continue;
              for (int s = 0; s < k; ++s) {
                const int w = q * st + s - pad;
                if (w < 0 || w >= W) continue;
                acc[h * W + w] += d * inv;
              }
            }
          }
        }
      float* dxp = dx + (size_t)nc * H * W;
      for (int i = 0; i < H * W; ++i) dxp[i] = (float)acc[i];
    }
    free(acc);
  }
}

/* ------------------------------------------------------------------------------------------
 * Softmax / KL loss / reductions (K10-K13), src/operator/loss.rs:118-261
 * ---------------------------------------------------------------------------------------- */

/* K10: p[n,:] = softmax(x[n,:]), max-subtracted (CudnnSoftmaxOp::forward, loss.rs:121-126) */
void orc_softmax_fwd(const float* x, float* p, int32_t C, int32_t N) {
#pragma omp parallel for schedule(static)
  for (int n = 0; n < N; ++n) {
    const float* xr = x + (size_t)n * C;
    float* pr = p + (size_t)n * C;
    float mx = xr[0];
    for (int c = 1; c < C; ++c) mx = xr[c] > mx ? xr[c] : mx;
    double z = 0.0;
    for (int c = 0; c < C; ++c) z += exp((double)xr[c] - (double)mx);
    for (int c = 0; c < C; ++c) pr[c] = (float)(exp((double)xr[c] - (double)mx) / z);
  }
}

/* K11: dx[n,c] = weights[n] * (p[n,c] - [c == labels[n]])  (softmax_kl_backward, loss.rs:132-140) */
void orc_softmax_kl_backward(const float* p, int32_t C, int32_t N, const int32_t* labels,
                             const float* weights, float* dx) {
#pragma omp parallel for schedule(static)
  for (int n = 0; n < N; ++n)
    for (int c = 0; c < C; ++c) {
      const float ind = (c == labels[n]) ? 1.0f : 0.0f;
      dx[(size_t)n * C + c] = weights[n] * (p[(size_t)n * C + c] - ind);
    }
}

/* K12a: loss1[n] = beta*loss1[n] - weights[n]*log p[n,labels[n]]  (softmax_kl_loss1, loss.rs:191-200) */
void orc_softmax_kl_loss1(const float* p, int32_t C, int32_t N, const int32_t* labels,
                          const float* weights, float beta, float* loss1) {
  for (int n = 0; n < N; ++n) {
    const double v = -(double)weights[n] * log((double)p[(size_t)n * C + labels[n]]);
    loss1[n] = (float)(beta != 0.0f ? (double)beta * (double)loss1[n] + v : v);
  }
}

/* K12b: dst[b] = beta*dst[b] + sum_i src[b*len + i]  (batch_blockreduce_sum, loss.rs:203-210) */
void orc_blockreduce_sum(const float* src, int32_t len, int32_t batch, float* dst, float beta) {
  for (int b = 0; b < batch; ++b) {
    double acc = 0.0;
    for (int i = 0; i < len; ++i) acc += (double)src[(size_t)b * len + i];
    dst[b] = (float)(beta != 0.0f ? (double)beta * (double)dst[b] + acc : acc);
  }
}

/* K13: per-row maximum and its first index (batch_blockreduce_argmax, loss.rs:229-239) */
void orc_blockreduce_argmax(const float* src, int32_t len, int32_t batch, float* max_out,
                            int32_t* idx_out) {
  for (int b = 0; b < batch; ++b) {
    const float* r = src + (size_t)b * len;
    int bi = 0;
    float best = r[0];
    for (int i = 1; i < len; ++i)
      if (r[i] > best) { best = r[i]; bi = i; }
    max_out[b] = best;
    idx_out[b] = bi;
  }
}

/* accuracy_count: #{n : labels[n] == cats[n]}  (loss.rs:246-261) */
int32_t orc_accuracy_count(const int32_t* labels, const int32_t* cats, int32_t batch) {
  int32_t c = 0;
  for (int i = 0; i < batch; ++i) c += labels[i] == cats[i];
  return c;
}

/* ------------------------------------------------------------------------------------------
 * SGD on operators, the BLAS-1 sequence of src/operator/mod.rs:1178-1236,1355-1363, each
 * step rounded to fp32 exactly as separate SAXPY / SSCAL calls would.
 * ---------------------------------------------------------------------------------------- */

/* g += l2*W ; v = mu*v ; v += scale*g ; W += apply*v ; optionally g = 0 */
void orc_sgd_momentum_step(int64_t n, float* W, float* g, float* v, float l2, float scale,
                           float mu, float apply, int zero_grad) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    float gi = g[i];
    if (l2 > 0.0f) gi = fmaf(l2, W[i], gi);
    float vi = mu * v[i];
    vi = fmaf(scale, gi, vi);
    W[i] = fmaf(apply, vi, W[i]);
    v[i] = vi;
    g[i] = zero_grad ? 0.0f : gi;
  }
}

/* Gen-1/gen-2 descend: g += l2*W ; W -= s*g   (src/layer_new.rs:596-617, src/layer.rs:1710-1715) */
void orc_descend(int64_t n, float* W, float* g, float s, float l2) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    float gi = g[i];
    if (l2 > 0.0f) gi = fmaf(l2, W[i], gi);
    g[i] = gi;
    W[i] = fmaf(-s, gi, W[i]);
  }
}

/* cast_bytes / cast_bytes_normalized (src/operator/mod.rs:735-737): y = scale * (float)x */
void orc_cast_u8_f32(const uint8_t* x, float* y, int64_t n, float scale) {
  for (int64_t i = 0; i < n; ++i) y[i] = scale * (float)x[i];
}

/* Operand rounding of the bf16 math mode (no counterpart in the reference, which is fp32 only; the mode is
 * this build's RH_MATH_BF16_MFMA_FP32ACC): fp32 -> bf16 round-to-nearest-even -> back to fp32, in place.
 * NaN stays NaN (quieted).  Pinned against torch's float32 -> bfloat16 -> float32 round trip. */
void orc_round_bf16(float* x, int64_t n) {
  for (int64_t i = 0; i < n; ++i) {
    uint32_t u;
    memcpy(&u, &x[i], 4);
    if ((u & 0x7f800000u) == 0x7f800000u && (u & 0x007fffffu)) {
      u = (u | 0x00400000u) & 0xffff0000u;
    } else {
      u += 0x7fffu + ((u >> 16) & 1u);
      u &= 0xffff0000u;
    }
    memcpy(&x[i], &u, 4);
  }
}

/* ------------------------------------------------------------------------------------------
 * Fast family: fp32 im2col + blocked SGEMM with OpenMP.  The timed CPU baseline.
 * Row-major helper:  Cm[M][N] (+)= Am[M][K] * Bm[K][N]
 * ---------------------------------------------------------------------------------------- */
static void sgemm_rm_nn(int M, int N, int K, const float* restrict A, int lda,
                        const float* restrict B, int ldb, float* restrict C, int ldc,
                        int accumulate) {
  enum { MB = 64, KB = 256, NB = 512 };
#pragma omp parallel for collapse(2) schedule(dynamic, 1)
  for (int i0 = 0; i0 < M; i0 += MB)
    for (int j0 = 0; j0 < N; j0 += NB) {
      const int i1 = i0 + MB < M ? i0 + MB : M;
      const int j1 = j0 + NB < N ? j0 + NB : N;
      if (!accumulate)
        for (int i = i0; i < i1; ++i)
          for (int j = j0; j < j1; ++j) C[(size_t)i * ldc + j] = 0.0f;
      for (int k0 = 0; k0 < K; k0 += KB) {
        const int k1 = k0 + KB < K ? k0 + KB : K;
        int i = i0;
        for (; i + 4 <= i1; i += 4) {
          float* restrict c0 = C + (size_t)(i + 0) * ldc;
          float* restrict c1 = C + (size_t)(i + 1) * ldc;
          float* restrict c2 = C + (size_t)(i + 2) * ldc;
          float* restrict c3 = C + (size_t)(i + 3) * ldc;
          for (int k = k0; k < k1; ++k) {
            const float a0 = A[(size_t)(i + 0) * lda + k], a1 = A[(size_t)(i + 1) * lda + k];
            const float a2 = A[(size_t)(i + 2) * lda + k], a3 = A[(size_t)(i + 3) * lda + k];
            const float* restrict b = B + (size_t)k * ldb;
#pragma omp simd
            for (int j = j0; j < j1; ++j) {
              const float bv = b[j];
              c0[j] += a0 * bv; c1[j] += a1 * bv; c2[j] += a2 * bv; c3[j] += a3 * bv;
            }
          }
        }
        for (; i < i1; ++i) {
          float* restrict c0 = C + (size_t)i * ldc;
          for (int k = k0; k < k1; ++k) {
            const float a0 = A[(size_t)i * lda + k];
            const float* restrict b = B + (size_t)k * ldb;
#pragma omp simd
            for (int j = j0; j < j1; ++j) c0[j] += a0 * b[j];
          }
        }
      }
    }
}

/* col[(c,r,s)][(p,q)] for one image */
static void im2col(const orc_conv_geom* g, int P, int Q, const float* x, float* col) {
  const int C = g->C, H = g->H, W = g->W, R = g->R, S = g->S, st = g->stride, pad = g->pad;
  for (int c = 0; c < C; ++c)
    for (int r = 0; r < R; ++r)
      for (int s = 0; s < S; ++s) {
        float* dst = col + (((size_t)c * R + r) * S + s) * P * Q;
        for (int p = 0; p < P; ++p) {
          const int h = p * st + r - pad;
          if (h < 0 || h >= H) { memset(dst + (size_t)p * Q, 0, sizeof(float) * Q); continue; }
          const float* xr = x + ((size_t)c * H + h) * W;
          for (int q = 0; q < Q; ++q) {
            const int w = q * st + s - pad;
            dst[(size_t)p * Q + q] = (w >= 0 && w < W) ? xr[w] : 0.0f;
          }
        }
      }
}

static void col2im_add(const orc_conv_geom* g, int P, int Q, const float* col, float* dx) {
  const int C = g->C, H = g->H, W = g->W, R = g->R, S = g->S, st = g->stride, pad = g->pad;
  for (int c = 0; c < C; ++c)
    for (int r = 0; r < R; ++r)
      for (int s = 0; s < S; ++s) {
        const float* src = col + (((size_t)c * R + r) * S + s) * P * Q;
        for (int p = 0; p < P; ++p) {
          const int h = p * st + r - pad;
          if (h < 0 || h >= H) continue;
          float* xr = dx + ((size_t)c * H + h) * W;
          for (int q = 0; q < Q; ++q) {
            const int w = q * st + s - pad;
            if (w >= 0 && w < W) xr[w] += src[(size_t)p * Q + q];
          }
        }
      }
}

/* y = corr(x, w), overwrite.  Per image: y_n[K][PQ] = w[K][CRS] * col_n[CRS][PQ]. */
void orc_fast_conv2d_fwd(const orc_conv_geom* g, const float* x, const float* w, float* y) {
  const int P = orc_out_dim_floor(g->H, g->R, g->stride, g->pad);
  const int Q = orc_out_dim_floor(g->W, g->S, g->stride, g->pad);
  const int CRS = g->C * g->R * g->S, PQ = P * Q;
  float* col = (float*)malloc(sizeof(float) * (size_t)CRS * PQ);
  for (int n = 0; n < g->N; ++n) {
    im2col(g, P, Q, x + (size_t)n * g->C * g->H * g->W, col);
    sgemm_rm_nn(g->K, PQ, CRS, w, CRS, col, PQ, y + (size_t)n * g->K * PQ, PQ, 0);
  }
  free(col);
}

/* dx = corr^T(dy, w), overwrite.  col_n[CRS][PQ] = w^T[CRS][K] * dy_n[K][PQ]; dx_n = col2im(col_n). */
void orc_fast_conv2d_bwd_data(const orc_conv_geom* g, const float* w, const float* dy, float* dx) {
  const int P = orc_out_dim_floor(g->H, g->R, g->stride, g->pad);
  const int Q = orc_out_dim_floor(g->W, g->S, g->stride, g->pad);
  const int CRS = g->C * g->R * g->S, PQ = P * Q, K = g->K;
  float* col = (float*)malloc(sizeof(float) * (size_t)CRS * PQ);
  float* wt = (float*)malloc(sizeof(float) * (size_t)CRS * K);
  for (int k = 0; k < K; ++k)
    for (int j = 0; j < CRS; ++j) wt[(size_t)j * K + k] = w[(size_t)k * CRS + j];
  for (int n = 0; n < g->N; ++n) {
    sgemm_rm_nn(CRS, PQ, K, wt, K, dy + (size_t)n * K * PQ, PQ, col, PQ, 0);
    float* dxn = dx + (size_t)n * g->C * g->H * g->W;
    memset(dxn, 0, sizeof(float) * (size_t)g->C * g->H * g->W);
    col2im_add(g, P, Q, col, dxn);
  }
  free(col);
  free(wt);
}

/* dw += sum_n dy_n[K][PQ] * col_n^T[PQ][CRS]  (beta = 1 accumulation as in the reference) */
void orc_fast_conv2d_bwd_filter(const orc_conv_geom* g, const float* x, const float* dy, float* dw) {
  const int P = orc_out_dim_floor(g->H, g->R, g->stride, g->pad);
  const int Q = orc_out_dim_floor(g->W, g->S, g->stride, g->pad);
  const int CRS = g->C * g->R * g->S, PQ = P * Q, K = g->K;
  float* col = (float*)malloc(sizeof(float) * (size_t)CRS * PQ);
  float* colt = (float*)malloc(sizeof(float) * (size_t)CRS * PQ);
  for (int n = 0; n < g->N; ++n) {
    im2col(g, P, Q, x + (size_t)n * g->C * g->H * g->W, col);
#pragma omp parallel for schedule(static)
    for (int j = 0; j < CRS; ++j)
      for (int i = 0; i < PQ; ++i) colt[(size_t)i * CRS + j] = col[(size_t)j * PQ + i];
    sgemm_rm_nn(K, CRS, PQ, dy + (size_t)n * K * PQ, PQ, colt, CRS, dw, CRS, 1);
  }
  free(col);
  free(colt);
}

/* Row-major fast GEMM entry for the affine layers of the timed baseline:
 * Cm[M][N] = (accumulate ? Cm : 0) + Am[M][K] * Bm[K][N], with optional transposes done by copy. */
void orc_fast_gemm_rm(int transA, int transB, int M, int N, int K, const float* A, const float* B,
                      float* C, int accumulate) {
  float* At = NULL;
  float* Bt = NULL;
  if (transA) { /* A given as [K][M] */
    At = (float*)malloc(sizeof(float) * (size_t)M * K);
#pragma omp parallel for schedule(static)
    for (int i = 0; i < M; ++i)
      for (int k = 0; k < K; ++k) At[(size_t)i * K + k] = A[(size_t)k * M + i];
    A = At;
  }
  if (transB) { /* B given as [N][K] */
    Bt = (float*)malloc(sizeof(float) * (size_t)N * K);
#pragma omp parallel for schedule(static)
    for (int k = 0; k < K; ++k)
      for (int j = 0; j < N; ++j) Bt[(size_t)k * N + j] = B[(size_t)j * K + k];
    B = Bt;
  }
  sgemm_rm_nn(M, N, K, A, K, B, N, C, N, accumulate);
  free(At);
  free(Bt);
}
