/*
 * TEST INFRASTRUCTURE ONLY - plain C restatement, on the host, of the matrix ops
 * the benchmark times on the GPU.  Only tests/, __graft_entry__.smoke() and
 * bench.py's cpu_baseline leg may load this; the product never links it.
 *
 * It serves two purposes:
 *  1. a third, independent coding of the multiply-with-carry generator
 *     (cudamat/cudamat_kernels.cu:96-167) next to the two in mwc.py;
 *  2. the CPU baseline: column-major fp32 loops shaped like the reference's CPU
 *     backend eigenmat/eigenmat.cc (dot :1059-1086, apply_sigmoid :869-878,
 *     add_col_vec :260-278, add_mult :1109-1122, apply_softmax :808-826,
 *     max_by_axis :617-639, sum_by_axis :747-760).  Eigen is not available, so
 *     the product in `hb_gemm` is a cache-blocked loop nest, not Eigen's kernel;
 *     like the reference build (eigenmat/Makefile has no -fopenmp) it runs on
 *     one thread unless hb_set_threads() asks for more.
 *
 * Pins: mwc_* against mwc.py on seeds 0/1/42 (tests/test_oracle_mwc.py); hb_gemm
 * and the loops against numpy float64 (tests/test_oracle_host.py).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define NUM_RND_STREAMS 12288
#define NUM_RND_BURNIN 100

static int g_threads = 1;

void hb_set_threads(int n) { g_threads = n > 0 ? n : 1; }
int hb_get_threads(void) { return g_threads; }
int hb_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* ------------------------------------------------------------------ MWC */

static inline uint64_t mwc_step(uint64_t w, uint32_t mult) { return (uint64_t)mult * (w & 0xffffffffu) + (w >> 32); }
static inline float mwc_unif(uint64_t w) { return ((float)(uint32_t)(w & 0xffffffffu) + 1.0f) / 4294967296.0f; }

/* cudamat_kernels.cu:96-111 */
void mwc_seed(const uint32_t* mults, uint64_t* words, uint32_t seed) {
  for (int t = 0; t < NUM_RND_STREAMS; ++t) {
    uint64_t w = ((uint64_t)seed << 32) + 1u;
    for (int i = 0; i < NUM_RND_BURNIN; ++i) w = mwc_step(w, mults[t]);
    words[t] = w;
  }
}

/* cudamat_kernels.cu:113-123 */
void mwc_uniform(const uint32_t* mults, uint64_t* words, float* out, size_t n) {
  for (size_t t = 0; t < NUM_RND_STREAMS; ++t) {
    uint64_t w = words[t];
    for (size_t i = t; i < n; i += NUM_RND_STREAMS) {
      w = mwc_step(w, mults[t]);
      out[i] = mwc_unif(w);
    }
    words[t] = w;
  }
}

/* cudamat_kernels.cu:157-167 */
void mwc_bernoulli(const uint32_t* mults, uint64_t* words, const float* p, float* out, size_t n) {
  for (size_t t = 0; t < NUM_RND_STREAMS; ++t) {
    uint64_t w = words[t];
    for (size_t i = t; i < n; i += NUM_RND_STREAMS) {
      w = mwc_step(w, mults[t]);
      out[i] = mwc_unif(w) < p[i] ? 1.f : 0.f;
    }
    words[t] = w;
  }
}

/* cudamat_kernels.cu:145-155 */
void mwc_dropout(const uint32_t* mults, uint64_t* words, float* data, size_t n, float dropprob, float val) {
  for (size_t t = 0; t < NUM_RND_STREAMS; ++t) {
    uint64_t w = words[t];
    for (size_t i = t; i < n; i += NUM_RND_STREAMS) {
      w = mwc_step(w, mults[t]);
      data[i] = mwc_unif(w) > dropprob ? data[i] : val;
    }
    words[t] = w;
  }
}

/* ------------------------------------------------------------------ GEMM */
/* C = beta*C + alpha*op(A)*op(B), column-major.  ta/tb: 0 = as stored, 1 = transposed. */

#define at(P, ld, i, j) (P)[(size_t)(j) * (ld) + (i)]

static void gemm_cols(int ta, int tb, int m, int k, float alpha, const float* A, int lda, const float* B, int ldb,
                      float beta, float* C, int ldc, int j0, int j1) {
  enum { KB = 256 };
  for (int j = j0; j < j1; ++j) {
    float* c = &at(C, ldc, 0, j);
    if (beta == 0.f) memset(c, 0, (size_t)m * sizeof(float));
    else if (beta != 1.f) for (int i = 0; i < m; ++i) c[i] *= beta;
  }
  if (!ta) {
    /* A is m x k with contiguous columns: rank-1 updates of a block of C columns. */
    for (int p0 = 0; p0 < k; p0 += KB) {
      const int p1 = p0 + KB < k ? p0 + KB : k;
      for (int j = j0; j < j1; ++j) {
        float* c = &at(C, ldc, 0, j);
        for (int p = p0; p < p1; ++p) {
          const float b = alpha * (tb ? at(B, ldb, j, p) : at(B, ldb, p, j));
          const float* a = &at(A, lda, 0, p);
          for (int i = 0; i < m; ++i) c[i] += a[i] * b;
        }
      }
    }
  } else {
    /* A stored k x m: each output is a dot product down a contiguous column of A. */
    float* bcol = (float*)malloc((size_t)k * sizeof(float));
    for (int j = j0; j < j1; ++j) {
      const float* b = bcol;
      if (tb) for (int p = 0; p < k; ++p) bcol[p] = at(B, ldb, j, p);
      else b = &at(B, ldb, 0, j);
      float* c = &at(C, ldc, 0, j);
      for (int i = 0; i < m; ++i) {
        const float* a = &at(A, lda, 0, i);
        float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
        int p = 0;
        for (; p + 3 < k; p += 4) {
          s0 += a[p] * b[p]; s1 += a[p + 1] * b[p + 1]; s2 += a[p + 2] * b[p + 2]; s3 += a[p + 3] * b[p + 3];
        }
        for (; p < k; ++p) s0 += a[p] * b[p];
        c[i] += alpha * ((s0 + s1) + (s2 + s3));
      }
    }
    free(bcol);
  }
}

void hb_gemm(int ta, int tb, int m, int n, int k, float alpha, const float* A, int lda, const float* B, int ldb,
             float beta, float* C, int ldc) {
#ifdef _OPENMP
  if (g_threads > 1 && n >= 2 * g_threads) {
#pragma omp parallel num_threads(g_threads)
    {
      const int t = omp_get_thread_num(), T = omp_get_num_threads();
      const int j0 = (int)((long long)n * t / T), j1 = (int)((long long)n * (t + 1) / T);
      gemm_cols(ta, tb, m, k, alpha, A, lda, B, ldb, beta, C, ldc, j0, j1);
    }
    return;
  }
#endif
  gemm_cols(ta, tb, m, k, alpha, A, lda, B, ldb, beta, C, ldc, 0, n);
}

/* ------------------------------------------------------------------ elementwise / reductions */

#ifdef _OPENMP
#define PAR_FOR _Pragma("omp parallel for num_threads(g_threads) if (g_threads > 1)")
#else
#define PAR_FOR
#endif

void hb_add_mult(float* a, const float* b, float alpha, size_t n) {
  PAR_FOR for (size_t i = 0; i < n; ++i) a[i] += alpha * b[i];
}
void hb_mult(const float* a, const float* b, float* t, size_t n) {
  PAR_FOR for (size_t i = 0; i < n; ++i) t[i] = a[i] * b[i];
}
void hb_mult_scalar(const float* a, float s, float* t, size_t n) {
  PAR_FOR for (size_t i = 0; i < n; ++i) t[i] = a[i] * s;
}
void hb_sigmoid(const float* a, float* t, size_t n) {
  PAR_FOR for (size_t i = 0; i < n; ++i) t[i] = 1.f / (1.f + expf(-a[i]));
}
void hb_exp(const float* a, float* t, size_t n) {
  PAR_FOR for (size_t i = 0; i < n; ++i) t[i] = expf(a[i]);
}
void hb_lower_bound_scalar(const float* a, float s, float* t, size_t n) {
  PAR_FOR for (size_t i = 0; i < n; ++i) t[i] = a[i] < s ? s : a[i];
}
void hb_greater_than_scalar(const float* a, float s, float* t, size_t n) {
  PAR_FOR for (size_t i = 0; i < n; ++i) t[i] = a[i] > s ? 1.f : 0.f;
}
void hb_relu_deriv(const float* a, const float* b, float* t, size_t n) {
  PAR_FOR for (size_t i = 0; i < n; ++i) t[i] = a[i] * (b[i] > 0.f ? 1.f : 0.f);
}
void hb_add_col_vec(const float* a, const float* v, float* t, int h, int w) {
  PAR_FOR for (int j = 0; j < w; ++j)
    for (int i = 0; i < h; ++i) t[(size_t)j * h + i] = a[(size_t)j * h + i] + v[i];
}
void hb_mult_by_col(const float* a, const float* v, float* t, int h, int w) {
  PAR_FOR for (int j = 0; j < w; ++j)
    for (int i = 0; i < h; ++i) t[(size_t)j * h + i] = a[(size_t)j * h + i] * v[i];
}
void hb_add_row_vec(const float* a, const float* v, float* t, int h, int w) {
  PAR_FOR for (int j = 0; j < w; ++j)
    for (int i = 0; i < h; ++i) t[(size_t)j * h + i] = a[(size_t)j * h + i] + v[j];
}
/* t = beta*t + mult * sums; axis 0: per column (t has w entries); axis 1: per row (h entries). */
void hb_add_sums(const float* a, float* t, int h, int w, int axis, float beta, float mult) {
  if (axis == 0) {
    PAR_FOR for (int j = 0; j < w; ++j) {
      float s = 0.f;
      for (int i = 0; i < h; ++i) s += a[(size_t)j * h + i];
      t[j] = (beta == 0.f ? 0.f : beta * t[j]) + mult * s;
    }
  } else {
    float* acc = (float*)calloc((size_t)h, sizeof(float));
    for (int j = 0; j < w; ++j)
      for (int i = 0; i < h; ++i) acc[i] += a[(size_t)j * h + i];
    for (int i = 0; i < h; ++i) t[i] = (beta == 0.f ? 0.f : beta * t[i]) + mult * acc[i];
    free(acc);
  }
}
void hb_max(const float* a, float* t, int h, int w, int axis) {
  if (axis == 0) {
    PAR_FOR for (int j = 0; j < w; ++j) {
      float m = a[(size_t)j * h];
      for (int i = 1; i < h; ++i) if (m < a[(size_t)j * h + i]) m = a[(size_t)j * h + i];
      t[j] = m;
    }
  } else {
    for (int i = 0; i < h; ++i) t[i] = a[i];
    for (int j = 1; j < w; ++j)
      for (int i = 0; i < h; ++i) if (t[i] < a[(size_t)j * h + i]) t[i] = a[(size_t)j * h + i];
  }
}
void hb_softmax(const float* a, float* t, int h, int w) {
  PAR_FOR for (int j = 0; j < w; ++j) {
    const float* x = a + (size_t)j * h;
    float* y = t + (size_t)j * h;
    float m = x[0];
    for (int i = 1; i < h; ++i) if (m < x[i]) m = x[i];
    float s = 0.f;
    for (int i = 0; i < h; ++i) { y[i] = expf(x[i] - m); s += y[i]; }
    for (int i = 0; i < h; ++i) y[i] /= s;
  }
}

/* ------------------------------------------------------------------ RBM CD-1 step
 * One contrastive-divergence step written against the ops above, the sequence of
 * cudamat/examples/rbm_cudamat.py:46-89 (momentum 0) with the sufficient
 * statistics applied straight to the parameters:
 *   h  = sigm(W^T v + b_h)
 *   hs = bernoulli(h)
 *   v' = sigm(W hs + b_v);   h' = sigm(W^T v' + b_h)
 *   W  += lr/B * v h^T;  W  -= lr/B * v' h'^T
 *   b_v += lr/B * (sum v - sum v');  b_h += lr/B * (sum h - sum h')
 * W is nv x nh, v is nv x B.  Scratch buffers h, hs, v2, h2 are caller-provided.
 */
void hb_rbm_cd1_step(float* W, float* bv, float* bh, const float* v, int nv, int nh, int B, float lr,
                     const uint32_t* mults, uint64_t* words, float* h, float* hs, float* v2, float* h2) {
  const float eps = lr / (float)B;
  hb_gemm(1, 0, nh, B, nv, 1.f, W, nv, v, nv, 0.f, h, nh);
  hb_add_col_vec(h, bh, h, nh, B);
  hb_sigmoid(h, h, (size_t)nh * B);
  mwc_bernoulli(mults, words, h, hs, (size_t)nh * B);
  hb_gemm(0, 0, nv, B, nh, 1.f, W, nv, hs, nh, 0.f, v2, nv);
  hb_add_col_vec(v2, bv, v2, nv, B);
  hb_sigmoid(v2, v2, (size_t)nv * B);
  hb_gemm(1, 0, nh, B, nv, 1.f, W, nv, v2, nv, 0.f, h2, nh);
  hb_add_col_vec(h2, bh, h2, nh, B);
  hb_sigmoid(h2, h2, (size_t)nh * B);
  hb_gemm(0, 1, nv, nh, B, eps, v, nv, h, nh, 1.f, W, nv);
  hb_gemm(0, 1, nv, nh, B, -eps, v2, nv, h2, nh, 1.f, W, nv);
  hb_add_sums(v, bv, nv, B, 1, 1.f, eps);
  hb_add_sums(v2, bv, nv, B, 1, 1.f, -eps);
  hb_add_sums(h, bh, nh, B, 1, 1.f, eps);
  hb_add_sums(h2, bh, nh, B, 1, 1.f, -eps);
}

/* ------------------------------------------------------------------ MLP step
 * One momentum-SGD step of a ReLU net with dropout 0.5 on the hidden layers and a
 * softmax output, written against the ops above in the order deepnet issues them
 * (forward deepnet/neuralnet.py:138-205, loss and its gradient softmax_layer.py:40-66,
 * backward neuralnet.py:207-291, update parameter.py:80-106 with momentum only):
 *   a[i+1] = W[i]^T a[i] + b[i];  hidden: max(.,0) * (u > 0.5), u from the MWC streams;
 *   top: softmax;  loss[j] = -log(p[label_j, j] + 1e-10);  d[nl-1] = p - onehot(label)
 *   gW[i] = a[i] d[i]^T / B;  gb[i] = rowsum(d[i]) / B;  d[i-1] = (W[i] d[i]) * (a[i] > 0)
 *   dX = mom * dX + gX;  X -= lr * dX      for X in W[i], b[i]
 * nl weight layers, sizes[0..nl]; every array column-major with the unit index fastest.
 * Pinned by tests/test_oracle_host.py against oracle/net_oracle.py fed the masks drawn here.
 */
void hb_mlp_step(int nl, const int* sizes, int B, float lr, float mom, float** W, float** b, float** dW, float** db,
                 float** gW, float** gb, float** act, float** mask, float** delta, const float* labels, float* loss,
                 const uint32_t* mults, uint64_t* words) {
  for (int i = 0; i < nl; ++i) {
    const int in = sizes[i], out = sizes[i + 1];
    const size_t n = (size_t)out * B;
    hb_gemm(1, 0, out, B, in, 1.f, W[i], in, act[i], in, 0.f, act[i + 1], out);
    hb_add_col_vec(act[i + 1], b[i], act[i + 1], out, B);
    if (i < nl - 1) {
      hb_lower_bound_scalar(act[i + 1], 0.f, act[i + 1], n);
      mwc_uniform(mults, words, mask[i], n);
      hb_greater_than_scalar(mask[i], 0.5f, mask[i], n);
      hb_mult(act[i + 1], mask[i], act[i + 1], n);
    } else {
      hb_softmax(act[i + 1], act[i + 1], out, B);
    }
  }
  {
    const int out = sizes[nl];
    const float* p = act[nl];
    float* d = delta[nl - 1];
    for (int j = 0; j < B; ++j) {
      const int label = (int)labels[j];
      loss[j] = -logf(p[(size_t)j * out + label] + 1e-10f);
      for (int i = 0; i < out; ++i) d[(size_t)j * out + i] = p[(size_t)j * out + i] - (i == label ? 1.f : 0.f);
    }
  }
  const float invB = 1.f / (float)B;
  for (int i = nl - 1; i >= 0; --i) {
    const int in = sizes[i], out = sizes[i + 1];
    /* gradients accumulate (neuralnet.py:269, 284); Update() leaves them at zero (parameter.py:105) */
    hb_gemm(0, 1, in, out, B, invB, act[i], in, delta[i], out, 1.f, gW[i], in);
    hb_add_sums(delta[i], gb[i], out, B, 1, 1.f, invB);
    if (i > 0) {
      hb_gemm(0, 0, in, B, out, 1.f, W[i], in, delta[i], out, 0.f, delta[i - 1], in);
      hb_mult(delta[i - 1], mask[i - 1], delta[i - 1], (size_t)in * B);      /* the layer's dropout mask (neuralnet.py:212-213) */
      hb_relu_deriv(delta[i - 1], act[i], delta[i - 1], (size_t)in * B);
    }
  }
  for (int i = 0; i < nl; ++i) {
    const size_t nw = (size_t)sizes[i] * sizes[i + 1], nb = (size_t)sizes[i + 1];
    hb_mult_scalar(dW[i], mom, dW[i], nw); hb_add_mult(dW[i], gW[i], 1.f, nw); hb_add_mult(W[i], dW[i], -lr, nw);
    hb_mult_scalar(db[i], mom, db[i], nb); hb_add_mult(db[i], gb[i], 1.f, nb); hb_add_mult(b[i], db[i], -lr, nb);
    memset(gW[i], 0, sizeof(float) * nw);
    memset(gb[i], 0, sizeof(float) * nb);
  }
}
