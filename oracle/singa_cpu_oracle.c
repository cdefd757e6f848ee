/*
 * CPU oracle: a plain-C restatement of the algorithms SINGA's CppCPU path uses for the
 * backward pass and the SGD-momentum update.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only the test-suite, the smoke check and
 * the CPU-baseline leg of the benchmark may load it; the shipped library never calls it.
 *
 * Every function cites the reference file:line whose algorithm it restates (paths are
 * relative to the apache/singa tree).  Where the reference delegates to a third-party
 * library that is not vendored in its tree (OpenBLAS sgemm/saxpy, oneDNN, cuDNN) the
 * published definition of that routine is restated; the summation ORDER of those libraries
 * is not reproduced ("parity unpinned" for the bit pattern, covered by the stated float
 * tolerances).  See the header comment of each function for what pins it.
 *
 * Build:  gcc -O3 -mavx2 -mfma -fopenmp -shared -fPIC singa_cpu_oracle.c -o libsinga_cpu_oracle.so -lm
 */
#include <float.h>
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_API __attribute__((visibility("default")))
/* separate multiply and add roundings, like the reference's op-by-op tensor calls */
#define NO_CONTRACT __attribute__((optimize("fp-contract=off")))

/* ---------------------------------------------------------------- threads */

ORACLE_API void oracle_set_threads(int n) {
#ifdef _OPENMP
  if (n > 0) omp_set_num_threads(n);
#else
  (void)n;
#endif
}

ORACLE_API int oracle_get_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* ---------------------------------------------------------------- SGEMM
 * Row-major C = alpha*op(A)*op(B) + beta*C with the argument meaning of cblas_sgemm as it
 * is called from GEMM<float, lang::Cpp> (src/core/tensor/tensor_math_cpp.h:877-899).
 * OpenBLAS itself is not vendored in the reference; this is the textbook definition with
 * fp32 accumulation.  Pinned by tests against float64 NumPy matmul.
 */
static void sgemm_nn(int M, int N, int K, float alpha, const float *A, int lda,
                     const float *B, int ldb, float *C, int ldc) {
#pragma omp parallel for schedule(static) if ((long)M * N * K > 200000)
  for (int i0 = 0; i0 < M; i0 += 4) {
    int im = i0 + 4 <= M ? 4 : M - i0;
    for (int k = 0; k < K; ++k) {
      const float *b = B + (size_t)k * ldb;
      for (int ii = 0; ii < im; ++ii) {
        float a = alpha * A[(size_t)(i0 + ii) * lda + k];
        float *c = C + (size_t)(i0 + ii) * ldc;
        for (int j = 0; j < N; ++j) c[j] += a * b[j];
      }
    }
  }
}

static void sgemm_tn(int M, int N, int K, float alpha, const float *A, int lda,
                     const float *B, int ldb, float *C, int ldc) {
  /* A stored K x M */
#pragma omp parallel for schedule(static) if ((long)M * N * K > 200000)
  for (int i0 = 0; i0 < M; i0 += 4) {
    int im = i0 + 4 <= M ? 4 : M - i0;
    for (int k = 0; k < K; ++k) {
      const float *b = B + (size_t)k * ldb;
      for (int ii = 0; ii < im; ++ii) {
        float a = alpha * A[(size_t)k * lda + i0 + ii];
        float *c = C + (size_t)(i0 + ii) * ldc;
        for (int j = 0; j < N; ++j) c[j] += a * b[j];
      }
    }
  }
}

static void sgemm_nt(int M, int N, int K, float alpha, const float *A, int lda,
                     const float *B, int ldb, float *C, int ldc) {
  /* B stored N x K */
#pragma omp parallel for schedule(static) if ((long)M * N * K > 200000)
  for (int i = 0; i < M; ++i) {
    const float *a = A + (size_t)i * lda;
    for (int j = 0; j < N; ++j) {
      const float *b = B + (size_t)j * ldb;
      float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f, s4 = 0.f, s5 = 0.f, s6 = 0.f, s7 = 0.f;
      int k = 0;
      for (; k + 8 <= K; k += 8) {
        s0 += a[k] * b[k];
        s1 += a[k + 1] * b[k + 1];
        s2 += a[k + 2] * b[k + 2];
        s3 += a[k + 3] * b[k + 3];
        s4 += a[k + 4] * b[k + 4];
        s5 += a[k + 5] * b[k + 5];
        s6 += a[k + 6] * b[k + 6];
        s7 += a[k + 7] * b[k + 7];
      }
      float s = ((s0 + s1) + (s2 + s3)) + ((s4 + s5) + (s6 + s7));
      for (; k < K; ++k) s += a[k] * b[k];
      C[(size_t)i * ldc + j] += alpha * s;
    }
  }
}

static void sgemm_tt(int M, int N, int K, float alpha, const float *A, int lda,
                     const float *B, int ldb, float *C, int ldc) {
  for (int i = 0; i < M; ++i)
    for (int j = 0; j < N; ++j) {
      float s = 0.f;
      for (int k = 0; k < K; ++k) s += A[(size_t)k * lda + i] * B[(size_t)j * ldb + k];
      C[(size_t)i * ldc + j] += alpha * s;
    }
}

ORACLE_API void oracle_sgemm(int transA, int transB, int M, int N, int K, float alpha,
                             const float *A, int lda, const float *B, int ldb, float beta,
                             float *C, int ldc) {
  for (int i = 0; i < M; ++i) {
    float *c = C + (size_t)i * ldc;
    if (beta == 0.f)
      for (int j = 0; j < N; ++j) c[j] = 0.f;
    else if (beta != 1.f)
      for (int j = 0; j < N; ++j) c[j] *= beta;
  }
  if (!transA && !transB) sgemm_nn(M, N, K, alpha, A, lda, B, ldb, C, ldc);
  else if (transA && !transB) sgemm_tn(M, N, K, alpha, A, lda, B, ldb, C, ldc);
  else if (!transA && transB) sgemm_nt(M, N, K, alpha, A, lda, B, ldb, C, ldc);
  else sgemm_tt(M, N, K, alpha, A, lda, B, ldb, C, ldc);
}

/* ---------------------------------------------------------------- elementwise */

/* ReLU forward: ReLU<float, lang::Cpp>, src/core/tensor/tensor_math_cpp.h:585-589
 * (a >= 0 ? a : 0).  Pinned by test/python/test_operation.py:717-741. */
ORACLE_API void oracle_relu_fwd(const float *x, float *y, size_t n) {
#pragma omp parallel for schedule(static) if (n > 100000)
  for (size_t i = 0; i < n; ++i) y[i] = (x[i] >= 0.f) ? x[i] : 0.f;
}

/* ReLUBackward<float, lang::Cpp>, src/core/tensor/tensor_math_cpp.h:446-451:
 * out = (in2 > 0) ? in1 : 0, in1 = dy, in2 = the ReLU INPUT, strict '>'.
 * Pinned by test/python/test_operation.py:717-741 and test/singa/test_activation.cc:84-129. */
ORACLE_API void oracle_relu_bwd(const float *dy, const float *x, float *dx, size_t n) {
#pragma omp parallel for schedule(static) if (n > 100000)
  for (size_t i = 0; i < n; ++i) dx[i] = (x[i] > 0.f) ? dy[i] : 0.f;
}

/* Axpy<float, lang::Cpp>, src/core/tensor/tensor_math_cpp.h:788-823: y += alpha * x
 * (cblas_saxpy; one multiply and one add per element, no fused rounding assumed). */
NO_CONTRACT ORACLE_API void oracle_axpy(float alpha, const float *x, float *y, size_t n) {
#pragma omp parallel for schedule(static) if (n > 100000)
  for (size_t i = 0; i < n; ++i) {
    float t = alpha * x[i];
    y[i] = y[i] + t;
  }
}

/* EltwiseMult<float, lang::Cpp>, src/core/tensor/tensor_math_cpp.h:432-444; the stride-0
 * broadcast of a 1-element right operand (python/singa/opt.py:299-300, "buf *= mom")
 * is the b_is_scalar case. */
ORACLE_API void oracle_eltwise_mult(const float *a, const float *b, int b_is_scalar, float *out,
                                    size_t n) {
#pragma omp parallel for schedule(static) if (n > 100000)
  for (size_t i = 0; i < n; ++i) out[i] = a[i] * (b_is_scalar ? b[0] : b[i]);
}

/* Tensor::operator+= used for gradient fan-in, python/singa/autograd.py:204 ->
 * src/core/tensor/tensor.cc:579-586 (Add). */
ORACLE_API void oracle_add(const float *a, const float *b, float *out, size_t n) {
#pragma omp parallel for schedule(static) if (n > 100000)
  for (size_t i = 0; i < n; ++i) out[i] = a[i] + b[i];
}

/* SGD.apply, python/singa/opt.py:269-310, op by op, each op rounding to fp32 like the
 * separate Axpy / EltwiseMult calls of the reference do:
 *   if wd != 0:        g += wd * p                      (:286-287)
 *   if mu != 0:        v *= mu ; v += (1 - damp) * g    (:298-302)
 *        nesterov:     g += mu * v                      (:304-305)
 *        else:         g := v                           (:306-307)
 *   p += (-lr) * g                                      (:309-310)
 * g is updated in place like the reference ("the values may be updated", :275-276).
 * Pinned by test/python/test_opt.py:97-228 (plain, momentum x2 steps, weight decay,
 * nesterov). */
NO_CONTRACT ORACLE_API void oracle_sgd_momentum(float *p, float *g, float *v, size_t n, float lr, float mu,
                                    float damp, float wd, int nesterov) {
  const float one_minus_damp = 1.0f - damp;
  const float minus_lr = 0.0f - lr;
#pragma omp parallel for schedule(static) if (n > 100000)
  for (size_t i = 0; i < n; ++i) {
    float t;
    float gi = g[i];
    if (wd != 0.f) {
      t = wd * p[i];
      gi = gi + t;
    }
    if (mu != 0.f) {
      float vi = v[i] * mu;
      t = one_minus_damp * gi;
      vi = vi + t;
      v[i] = vi;
      if (nesterov) {
        t = mu * vi;
        gi = gi + t;
      } else {
        gi = vi;
      }
    }
    g[i] = gi;
    t = minus_lr * gi;
    p[i] = p[i] + t;
  }
}

/* ---------------------------------------------------------------- softmax / CE */

/* Native SoftMax<float, lang::Cpp>, src/core/tensor/tensor_math_cpp.h:361-379, including
 * the CPU RowMax quirk (max seeded with 0, :1132).  Forward helper only. */
ORACLE_API void oracle_softmax(const float *x, float *p, size_t batch, size_t dim) {
  for (size_t i = 0; i < batch; ++i) {
    float mx = 0.f;
    for (size_t j = 0; j < dim; ++j) mx = x[i * dim + j] > mx ? x[i * dim + j] : mx;
    float s = 0.f;
    for (size_t j = 0; j < dim; ++j) {
      float e = expf(x[i * dim + j] - mx);
      p[i * dim + j] = e;
      s += e;
    }
    for (size_t j = 0; j < dim; ++j) p[i * dim + j] /= s;
  }
}

/* ComputeCrossEntropy<float, lang::Cpp>, src/core/tensor/tensor_math_cpp.h:1058-1088.
 * Returns -1 if a label is negative (the reference CHECK_GE aborts), -2 if it is >= dim.
 * Pinned by test/singa/test_cross_entropy.cc:43-71. */
ORACLE_API int oracle_cross_entropy_fwd(const float *p, const int *t, int int_target, size_t batch,
                                        size_t dim, float *loss) {
  if (int_target) {
    for (size_t i = 0; i < batch; ++i) {
      int k = t[i];
      if (k < 0) return -1;
      if ((size_t)k >= dim) return -2; /* the reference reads out of bounds here; the oracle refuses */
      float pr = p[i * dim + k];
      loss[i] = -logf(pr > FLT_MIN ? pr : FLT_MIN);
    }
  } else {
    for (size_t i = 0; i < batch; ++i) {
      float sum = 0.f;
      for (size_t j = 0; j < dim; ++j) sum += t[i * dim + j];
      float lv = 0.f;
      for (size_t j = 0; j < dim; ++j) {
        float pr = p[i * dim + j];
        lv -= t[i * dim + j] / sum * logf(pr > FLT_MIN ? pr : FLT_MIN);
      }
      loss[i] = lv;
    }
  }
  return 0;
}

/* SoftmaxCrossEntropyBwd<float, lang::Cpp>, src/core/tensor/tensor_math_cpp.h:1090-1119,
 * in place on grad (which the caller pre-fills with p: src/core/tensor/tensor.cc:1717-1721).
 * The target is read as int32 in both modes.  Returns -1 on a negative label, -2 on one >= dim.
 * All labels are validated before anything is written.
 * Pinned by test/singa/test_cross_entropy.cc:73-111. */
ORACLE_API int oracle_softmax_ce_bwd(float *grad, const int *t, int int_target, size_t batch,
                                     size_t dim) {
  if (int_target) {
    for (size_t i = 0; i < batch; ++i) {
      if (t[i] < 0) return -1;
      if ((size_t)t[i] >= dim) return -2; /* the reference writes out of bounds here; the oracle refuses */
    }
    for (size_t i = 0; i < batch; ++i) grad[i * dim + t[i]] -= 1.0f;
  } else {
    for (size_t i = 0; i < batch; ++i) {
      float sum = 0.f;
      for (size_t j = 0; j < dim; ++j) sum += t[i * dim + j];
      for (size_t j = 0; j < dim; ++j) grad[i * dim + j] -= t[i * dim + j] / sum;
    }
  }
  return 0;
}

/* Div(tensor, scalar) multiplies by the fp32 reciprocal: src/core/tensor/tensor_math.h:149-153;
 * this is the "dx /= N" of python/singa/autograd.py:1321. */
ORACLE_API void oracle_div_scalar(float *x, float d, size_t n) {
  const float r = 1.0f / d;
  for (size_t i = 0; i < n; ++i) x[i] *= r;
}

/* ---------------------------------------------------------------- convolution */

/* Im2col, src/model/layer/convolution.cc:197-222. */
static void im2col(const float *im, int C, int H, int W, int R, int S, int ph, int pw, int sh,
                   int sw, float *col) {
  const int P = (H + 2 * ph - R) / sh + 1;
  const int Q = (W + 2 * pw - S) / sw + 1;
  const int CC = C * R * S;
  for (int c = 0; c < CC; ++c) {
    const int wo = c % S, ho = (c / S) % R, ci = c / R / S;
    for (int h = 0; h < P; ++h)
      for (int w = 0; w < Q; ++w) {
        const int hp = h * sh - ph + ho, wp = w * sw - pw + wo;
        col[((size_t)c * P + h) * Q + w] =
            (hp >= 0 && hp < H && wp >= 0 && wp < W) ? im[((size_t)ci * H + hp) * W + wp] : 0.f;
      }
  }
}

/* Col2im, src/model/layer/convolution.cc:224-248. */
static void col2im(const float *col, int C, int H, int W, int R, int S, int ph, int pw, int sh,
                   int sw, float *im) {
  memset(im, 0, sizeof(float) * (size_t)C * H * W);
  const int P = (H + 2 * ph - R) / sh + 1;
  const int Q = (W + 2 * pw - S) / sw + 1;
  const int CC = C * R * S;
  for (int c = 0; c < CC; ++c) {
    const int wo = c % S, ho = (c / S) % R, ci = c / R / S;
    for (int h = 0; h < P; ++h)
      for (int w = 0; w < Q; ++w) {
        const int hp = h * sh - ph + ho, wp = w * sw - pw + wo;
        if (hp >= 0 && hp < H && wp >= 0 && wp < W)
          im[((size_t)ci * H + hp) * W + wp] += col[((size_t)c * P + h) * Q + w];
      }
  }
}

ORACLE_API void oracle_im2col(const float *im, int C, int H, int W, int R, int S, int ph, int pw,
                              int sh, int sw, float *col) {
  im2col(im, C, H, W, R, S, ph, pw, sh, sw, col);
}

ORACLE_API void oracle_col2im(const float *col, int C, int H, int W, int R, int S, int ph, int pw,
                              int sh, int sw, float *im) {
  col2im(col, C, H, W, R, S, ph, pw, sh, sw, im);
}

/* Convolution::Forward, src/model/layer/convolution.cc:107-136 (= the commented native body
 * of CpuConvForward, src/model/operation/convolution.cc:191-223): per image
 * y_b = W[K, CRS] * im2col(x_b) (+ bias per row).  b may be NULL.
 * Pinned by test/singa/test_convolution.cc:58-106. */
ORACLE_API void oracle_conv_fwd(const float *x, const float *Wt, const float *b, float *y, int N,
                                int C, int H, int W, int K, int R, int S, int sh, int sw, int ph,
                                int pw) {
  const int P = (H + 2 * ph - R) / sh + 1, Q = (W + 2 * pw - S) / sw + 1;
  const int CRS = C * R * S, PQ = P * Q;
  float *col = (float *)malloc(sizeof(float) * (size_t)CRS * PQ);
  for (int n = 0; n < N; ++n) {
    im2col(x + (size_t)n * C * H * W, C, H, W, R, S, ph, pw, sh, sw, col);
    float *yb = y + (size_t)n * K * PQ;
    oracle_sgemm(0, 0, K, PQ, CRS, 1.f, Wt, CRS, col, PQ, 0.f, yb, PQ);
    if (b)
      for (int k = 0; k < K; ++k)
        for (int j = 0; j < PQ; ++j) yb[(size_t)k * PQ + j] += b[k];
  }
  free(col);
}

/* Convolution::Backward, src/model/layer/convolution.cc:139-190 (= the commented native
 * bodies of CpuConvBackwardx / CpuConvBackwardW, src/model/operation/convolution.cc:288-309,
 * :383-407).  Per image b, in order:  dw += dy_b[K,PQ] * col^T  (a GEMM into a temporary,
 * then an elementwise add, :177);  dcol = W^T * dy_b (:178);  dx_b = Col2im(dcol) (:180-182).
 * dx and/or dw may be NULL to skip that output.
 * Pinned by test/singa/test_convolution.cc:108-207 and by brute-force direct convolution. */
ORACLE_API void oracle_conv_bwd(const float *dy, const float *x, const float *Wt, float *dx,
                                float *dw, int N, int C, int H, int W, int K, int R, int S, int sh,
                                int sw, int ph, int pw) {
  const int P = (H + 2 * ph - R) / sh + 1, Q = (W + 2 * pw - S) / sw + 1;
  const int CRS = C * R * S, PQ = P * Q;
  float *col = (float *)malloc(sizeof(float) * (size_t)CRS * PQ);
  float *tmp = dw ? (float *)malloc(sizeof(float) * (size_t)K * CRS) : NULL;
  if (dw) memset(dw, 0, sizeof(float) * (size_t)K * CRS);
  for (int n = 0; n < N; ++n) {
    const float *dyb = dy + (size_t)n * K * PQ;
    if (dw) {
      im2col(x + (size_t)n * C * H * W, C, H, W, R, S, ph, pw, sh, sw, col);
      oracle_sgemm(0, 1, K, CRS, PQ, 1.f, dyb, PQ, col, PQ, 0.f, tmp, CRS);
      for (size_t i = 0; i < (size_t)K * CRS; ++i) dw[i] += tmp[i];
    }
    if (dx) {
      oracle_sgemm(1, 0, CRS, PQ, K, 1.f, Wt, CRS, dyb, PQ, 0.f, col, PQ);
      col2im(col, C, H, W, R, S, ph, pw, sh, sw, dx + (size_t)n * C * H * W);
    }
  }
  free(col);
  free(tmp);
}

/* CpuConvBackwardb native body, src/model/operation/convolution.cc:425-440
 * (= src/model/layer/convolution.cc:154-164): SumColumns over [N*K, PQ] then SumRows over
 * [N, K]; each is a GEMV with a ones vector, i.e. a sequential fp32 sum.
 * Pinned by test/singa/test_convolution.cc:184-186. */
ORACLE_API void oracle_conv_bgrad(const float *dy, float *db, int N, int K, int PQ) {
  float *t = (float *)malloc(sizeof(float) * (size_t)N * K);
  for (int i = 0; i < N * K; ++i) {
    float s = 0.f;
    for (int j = 0; j < PQ; ++j) s += dy[(size_t)i * PQ + j];
    t[i] = s;
  }
  for (int k = 0; k < K; ++k) {
    float s = 0.f;
    for (int n = 0; n < N; ++n) s += t[(size_t)n * K + k];
    db[k] = s;
  }
  free(t);
}

/* ---------------------------------------------------------------- pooling */

/* Pooling::ForwardMaxPooling, src/model/layer/pooling.cc:162-206: row-major scan of the
 * clipped window, strict '>' so the FIRST maximum wins; mask holds the flat h*W+w index
 * inside the (n,c) plane (-1 if the window is empty / all -FLT_MAX).
 * Pinned by test/singa/test_pooling.cc:53-89; ties only by the source rule. */
ORACLE_API void oracle_pool_max_fwd(const float *x, float *y, int *mask, int N, int C, int H, int W,
                                    int kh, int kw, int sh, int sw, int ph, int pw) {
  const int P = (H + 2 * ph - kh) / sh + 1, Q = (W + 2 * pw - kw) / sw + 1;
#pragma omp parallel for schedule(static)
  for (int nc = 0; nc < N * C; ++nc) {
    const float *b = x + (size_t)nc * H * W;
    float *t = y + (size_t)nc * P * Q;
    int *m = mask + (size_t)nc * P * Q;
    for (int p = 0; p < P; ++p)
      for (int q = 0; q < Q; ++q) {
        int hs = p * sh - ph, ws = q * sw - pw;
        int he = hs + kh < H ? hs + kh : H, we = ws + kw < W ? ws + kw : W;
        hs = hs > 0 ? hs : 0;
        ws = ws > 0 ? ws : 0;
        float best = -FLT_MAX;
        int bi = -1;
        for (int h = hs; h < he; ++h)
          for (int w = ws; w < we; ++w)
            if (b[h * W + w] > best) {
              best = b[h * W + w];
              bi = h * W + w;
            }
        t[p * Q + q] = best;
        m[p * Q + q] = bi;
      }
  }
}

/* Pooling::BackwardMaxPooling, src/model/layer/pooling.cc:208-233: zero dx, then for each
 * output position in row-major order dx[mask] += dy (overlapping windows accumulate in that
 * order).  Entries with mask < 0 are skipped (the reference would write out of bounds).
 * Pinned by test/singa/test_pooling.cc:91-140. */
ORACLE_API void oracle_pool_max_bwd(const float *dy, const int *mask, float *dx, int N, int C,
                                    int H, int W, int P, int Q) {
#pragma omp parallel for schedule(static)
  for (int nc = 0; nc < N * C; ++nc) {
    float *b = dx + (size_t)nc * H * W;
    const float *t = dy + (size_t)nc * P * Q;
    const int *m = mask + (size_t)nc * P * Q;
    for (int i = 0; i < H * W; ++i) b[i] = 0.f;
    for (int i = 0; i < P * Q; ++i)
      if (m[i] >= 0) b[m[i]] += t[i];
  }
}

/* Average pooling.  Loop structure of Pooling::ForwardAvgPooling / BackwardAvgPooling,
 * src/model/layer/pooling.cc:235-317, with the divisor switchable:
 *   include_pad = 1: the legacy layer's divisor (window clipped to H+pad, :252-254)
 *   include_pad = 0: count-exclude-padding, the mode the operation API selects for both its
 *                    CPU and GPU paths (src/model/operation/pooling.cc:70-72, :172).
 * Pinned by test/python/test_api.py:605-634 (no-padding case, where both agree). */
ORACLE_API void oracle_pool_avg_fwd(const float *x, float *y, int N, int C, int H, int W, int kh,
                                    int kw, int sh, int sw, int ph, int pw, int include_pad) {
  const int P = (H + 2 * ph - kh) / sh + 1, Q = (W + 2 * pw - kw) / sw + 1;
#pragma omp parallel for schedule(static)
  for (int nc = 0; nc < N * C; ++nc) {
    const float *b = x + (size_t)nc * H * W;
    float *t = y + (size_t)nc * P * Q;
    for (int p = 0; p < P; ++p)
      for (int q = 0; q < Q; ++q) {
        int hs = p * sh - ph, ws = q * sw - pw;
        int he = hs + kh < H + ph ? hs + kh : H + ph, we = ws + kw < W + pw ? ws + kw : W + pw;
        int pool = (he - hs) * (we - ws);
        hs = hs > 0 ? hs : 0;
        ws = ws > 0 ? ws : 0;
        he = he < H ? he : H;
        we = we < W ? we : W;
        if (!include_pad) pool = (he - hs) * (we - ws);
        float s = 0.f;
        for (int h = hs; h < he; ++h)
          for (int w = ws; w < we; ++w) s += b[h * W + w];
        t[p * Q + q] = s / pool;
      }
  }
}

ORACLE_API void oracle_pool_avg_bwd(const float *dy, float *dx, int N, int C, int H, int W, int kh,
                                    int kw, int sh, int sw, int ph, int pw, int include_pad) {
  const int P = (H + 2 * ph - kh) / sh + 1, Q = (W + 2 * pw - kw) / sw + 1;
#pragma omp parallel for schedule(static)
  for (int nc = 0; nc < N * C; ++nc) {
    float *b = dx + (size_t)nc * H * W;
    const float *t = dy + (size_t)nc * P * Q;
    for (int i = 0; i < H * W; ++i) b[i] = 0.f;
    for (int p = 0; p < P; ++p)
      for (int q = 0; q < Q; ++q) {
        int hs = p * sh - ph, ws = q * sw - pw;
        int he = hs + kh < H + ph ? hs + kh : H + ph, we = ws + kw < W + pw ? ws + kw : W + pw;
        int pool = (he - hs) * (we - ws);
        hs = hs > 0 ? hs : 0;
        ws = ws > 0 ? ws : 0;
        he = he < H ? he : H;
        we = we < W ? we : W;
        if (!include_pad) pool = (he - hs) * (we - ws);
        for (int h = hs; h < he; ++h)
          for (int w = ws; w < we; ++w) b[h * W + w] += t[p * Q + q] / pool;
      }
  }
}

/* ---------------------------------------------------------------- batch norm (spatial)
 * CppCPU has no native 4-D training BatchNorm (src/model/layer/batchnorm.cc:98-101,
 * :236-239 LOG(FATAL)); the operation API delegates to oneDNN / cuDNN
 * (src/model/operation/batchnorm.cc:123-258, :287-404).  These functions restate the
 * published definition of those routines as SINGA calls them:
 *   mean_c = E[x], var_c = biased batch variance, invstd = 1/sqrt(var + eps), eps = 1e-5
 *   (batchnorm.cc:46, :313), y = gamma * (x - mean) * invstd + beta,
 *   running = (1 - factor) * running + factor * batch  with the UNBIASED variance
 *   (cuDNN rule; test/python/test_api.py:44-50),
 * the saved statistics are (mean, invstd) as on the cuDNN path (batchnorm.cc:318-321).
 * Sums are accumulated in double.  Pinned by test/singa/test_cudnn_batchnorm.cc:44-231,
 * test/python/test_api.py:488-529 and float64 closed forms. */
ORACLE_API void oracle_bn_fwd_train(const float *x, const float *gamma, const float *beta,
                                    float *running_mean, float *running_var, float factor,
                                    float eps, float *y, float *save_mean, float *save_invstd,
                                    int N, int C, int HW) {
  const double M = (double)N * HW;
#pragma omp parallel for schedule(static)
  for (int c = 0; c < C; ++c) {
    double s = 0, ss = 0;
    for (int n = 0; n < N; ++n) {
      const float *xp = x + ((size_t)n * C + c) * HW;
      for (int i = 0; i < HW; ++i) s += xp[i];
    }
    const double mean = s / M;
    for (int n = 0; n < N; ++n) {
      const float *xp = x + ((size_t)n * C + c) * HW;
      for (int i = 0; i < HW; ++i) {
        double d = xp[i] - mean;
        ss += d * d;
      }
    }
    const double var = ss / M;
    const float invstd = (float)(1.0 / sqrt(var + (double)eps));
    const float fmean = (float)mean;
    save_mean[c] = fmean;
    save_invstd[c] = invstd;
    if (running_mean) running_mean[c] = (1.f - factor) * running_mean[c] + factor * fmean;
    if (running_var) {
      const double unb = M > 1 ? var * M / (M - 1) : var;
      running_var[c] = (1.f - factor) * running_var[c] + factor * (float)unb;
    }
    for (int n = 0; n < N; ++n) {
      const float *xp = x + ((size_t)n * C + c) * HW;
      float *yp = y + ((size_t)n * C + c) * HW;
      for (int i = 0; i < HW; ++i) yp[i] = gamma[c] * ((xp[i] - fmean) * invstd) + beta[c];
    }
  }
}

/* BatchNorm backward as GpuBatchNormBackward's callee defines it
 * (src/model/operation/batchnorm.cc:368-404):  dbeta_c = sum dy, dgamma_c = sum dy * xhat,
 * dx = gamma * invstd / M * (M * dy - dbeta - xhat * dgamma), xhat = (x - mean) * invstd.
 * Pinned by test/singa/test_cudnn_batchnorm.cc:117-231 and test/python/test_api.py:488-529. */
ORACLE_API void oracle_bn_bwd(const float *dy, const float *x, const float *gamma,
                              const float *save_mean, const float *save_invstd, float *dx,
                              float *dgamma, float *dbeta, int N, int C, int HW) {
  const double M = (double)N * HW;
#pragma omp parallel for schedule(static)
  for (int c = 0; c < C; ++c) {
    const float mean = save_mean[c], invstd = save_invstd[c];
    double sdy = 0, sdyx = 0;
    for (int n = 0; n < N; ++n) {
      const float *xp = x + ((size_t)n * C + c) * HW;
      const float *dp = dy + ((size_t)n * C + c) * HW;
      for (int i = 0; i < HW; ++i) {
        sdy += dp[i];
        sdyx += (double)dp[i] * ((xp[i] - mean) * invstd);
      }
    }
    dbeta[c] = (float)sdy;
    dgamma[c] = (float)sdyx;
    const double k = (double)gamma[c] * invstd / M;
    for (int n = 0; n < N; ++n) {
      const float *xp = x + ((size_t)n * C + c) * HW;
      const float *dp = dy + ((size_t)n * C + c) * HW;
      float *op = dx + ((size_t)n * C + c) * HW;
      for (int i = 0; i < HW; ++i) {
        double xh = (double)((xp[i] - mean) * invstd);
        op[i] = (float)(k * (M * dp[i] - sdy - xh * sdyx));
      }
    }
  }
}

/* ---------------------------------------------------------------- reductions */

/* Sum(dy, 0) / SumRows: the bias gradient of AddBias.backward
 * (python/singa/autograd.py:696-709 -> src/core/tensor/tensor.cc:1523-1538, a GEMV with a
 * ones vector): out[j] = sum_i m[i][j], sequential over rows. */
ORACLE_API void oracle_sum_rows(const float *m, float *out, int rows, int cols) {
  for (int j = 0; j < cols; ++j) out[j] = 0.f;
  for (int i = 0; i < rows; ++i)
    for (int j = 0; j < cols; ++j) out[j] += m[(size_t)i * cols + j];
}

/* ------------------------------------------------------------- the remaining tensor functions */

/* Transform<float, lang::Cpp>, src/core/tensor/tensor_math_cpp.h:685-689 = traverse_unary with the
 * identity over a view that is not dense: the offset walk of next_offset, :126-138 (the last
 * dimension moves first; `stride` in elements, 0 for a broadcast dimension).
 * Pinned by: NumPy's as_strided / broadcast_to / transpose on random views. */
ORACLE_API void oracle_transform(const float *in, float *out, int ndim, const size_t *shape,
                                 const long *stride) {
  size_t n = 1;
  for (int d = 0; d < ndim; ++d) n *= shape[d];
  size_t index[16] = {0};
  long offset = 0;
  for (size_t i = 0; i < n; ++i) {
    out[i] = in[offset];
    for (int k = ndim - 1; k >= 0; --k) {
      if (index[k] + 1 < shape[k]) {
        offset += stride[k];
        index[k] += 1;
        break;
      }
      index[k] = 0;
      offset -= stride[k] * (long)(shape[k] - 1);
    }
  }
}

/* RowMax<float, lang::Cpp>, tensor_math_cpp.h:1122-1140: the running maximum starts at 0, not at
 * the row's first element.  Pinned by: numpy.maximum(0, x.max(axis=1)) incl. all-negative rows. */
ORACLE_API void oracle_row_max(const float *in, float *out, size_t nrow, size_t ncol) {
  for (size_t r = 0; r < nrow; ++r) {
    float maxval = 0;
    for (size_t c = 0; c < ncol; ++c) maxval = in[r * ncol + c] > maxval ? in[r * ncol + c] : maxval;
    out[r] = maxval;
  }
}

/* Dot<float, lang::Cpp>, tensor_math_cpp.h:827-849: cblas_sdot (OpenBLAS, not vendored: its
 * summation order is not reproduced; the published definition sum_i x[i] * y[i] is, accumulated
 * in order).  Sum<float, lang::Cpp>, :655-663: a sequential float sum.
 * Pinned by: float64 NumPy within |error| <= 1e-6 * sum |terms|. */
ORACLE_API NO_CONTRACT float oracle_dot(const float *a, const float *b, size_t n) {
  float s = 0.f;
  for (size_t i = 0; i < n; ++i) s += a[i] * b[i];
  return s;
}
ORACLE_API float oracle_sum_all(const float *a, size_t n) {
  float s = 0.f;
  for (size_t i = 0; i < n; ++i) s += a[i];
  return s;
}

/* ------------------------------------------------------------- seeded synthetic inputs
 * A counter-based generator, so that the benchmark's inputs do not depend on any library's random
 * stream: the k-th output of splitmix64 seeded with `seed` is mix(seed + (k + 1) * golden).
 * uniform: (out >> 11) * 2^-53 in [0, 1); normal: Box-Muller in double on outputs 2i and 2i + 1,
 * rounded to float once; integers: out % hi.  The Python twin is singa_amd/rng.py; the test-suite
 * holds the two to each other and to known splitmix64 outputs.  (Not a restatement of the
 * reference: SINGA draws from std::mt19937, tensor_math_cpp.h:712-740, whose streams no reference
 * test depends on.) */
static uint64_t splitmix64_at(uint64_t seed, uint64_t k) {
  uint64_t z = seed + (k + 1u) * 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
ORACLE_API uint64_t oracle_rng_raw(uint64_t seed, uint64_t k) { return splitmix64_at(seed, k); }
ORACLE_API void oracle_rng_uniform(uint64_t seed, uint64_t offset, double low, double high, float *out, size_t n) {
  for (size_t i = 0; i < n; ++i)
    out[i] = (float)(low + (double)(splitmix64_at(seed, offset + i) >> 11) * 0x1.0p-53 * (high - low));
}
ORACLE_API void oracle_rng_normal(uint64_t seed, uint64_t offset, double mean, double std, float *out, size_t n) {
  for (size_t i = 0; i < n; ++i) {
    const double u1 = (double)(splitmix64_at(seed, offset + 2 * i) >> 11) * 0x1.0p-53;
    const double u2 = (double)(splitmix64_at(seed, offset + 2 * i + 1) >> 11) * 0x1.0p-53;
    out[i] = (float)(mean + std * (sqrt(-2.0 * log(1.0 - u1)) * cos(6.283185307179586476925286766559 * u2)));
  }
}
ORACLE_API void oracle_rng_integers(uint64_t seed, uint64_t offset, uint64_t hi, int *out, size_t n) {
  for (size_t i = 0; i < n; ++i) out[i] = (int)(splitmix64_at(seed, offset + i) % hi);
}
