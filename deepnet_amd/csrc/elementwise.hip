// Elementwise, scalar, comparison and broadcast ops over column-major fp32.
// Replaces the grid-stride kernels of cudamat/cudamat_kernels.cu:298-716 and
// their wrappers cudamat/cudamat.cu:592-1146, 1318-1669, 1763-2102.
//
// All of these are HBM-bound.  One templated kernel moves one 16-byte vector per
// lane (non-temporal for large operands); operands that are not 16-byte aligned
// (column views) are peeled to alignment when they share the same offset and
// fall back to 4-byte accesses otherwise.
#include "common.h"
#include "rng.h"
#include "wide_math.h"
#include <math.h>

// ------------------------------------------------------------------ functors
// f(a, b): a = first input, b = second input (unused for unary ops).

#define DN_FUNCTOR0(NAME, EXPR)                                           \
  struct NAME {                                                           \
    __device__ __forceinline__ float operator()(float a, float b) const { \
      (void)a; (void)b;                                                   \
      return (EXPR);                                                      \
    }                                                                     \
  };
#define DN_FUNCTOR1(NAME, EXPR)                                           \
  struct NAME {                                                           \
    float s;                                                              \
    __device__ __forceinline__ float operator()(float a, float b) const { \
      (void)a; (void)b;                                                   \
      return (EXPR);                                                      \
    }                                                                     \
  };

// unary (cudamat_kernels.cu:386-506)
DN_FUNCTOR0(FSign, a ? copysignf(1.f, a) : 0.f)
DN_FUNCTOR0(FCos, (float)dn_cos_wide(a))
DN_FUNCTOR0(FSin, (float)dn_sin_wide(a))
DN_FUNCTOR0(FSigmoid, dn_sigmoid(a))
DN_FUNCTOR0(FTanh, dn_tanh(a))
DN_FUNCTOR0(FAbs, a * (float)((a > 0.f) - (a < 0.f)))
DN_FUNCTOR0(FLog1pExp, dn_softplus(a))
DN_FUNCTOR1(FLog, dn_log(a + s))
DN_FUNCTOR0(FExp, dn_exp(a))
DN_FUNCTOR0(FCeil, ceilf(a))
DN_FUNCTOR0(FFloor, floorf(a))
DN_FUNCTOR0(FSqrt, sqrtf(a))
DN_FUNCTOR1(FPow, dn_pow(a, s))
DN_FUNCTOR0(FRecip, (float)(1.0 / (double)a))
// binary (cudamat_kernels.cu:298-364, 476-500, 600-685)
DN_FUNCTOR0(FLt, a < b ? 1.f : 0.f)
DN_FUNCTOR0(FLe, a <= b ? 1.f : 0.f)
DN_FUNCTOR0(FGt, a > b ? 1.f : 0.f)
DN_FUNCTOR0(FGe, a >= b ? 1.f : 0.f)
DN_FUNCTOR0(FUpper, a > b ? b : a)
DN_FUNCTOR0(FLower, a < b ? b : a)
DN_FUNCTOR0(FAdd, a + b)
DN_FUNCTOR0(FSub, a - b)
DN_FUNCTOR0(FDiv, a / b)
DN_FUNCTOR0(FMul, a * b)
DN_FUNCTOR0(FPowMat, dn_pow(a, b))
DN_FUNCTOR0(FCosDeriv, (float)(-(double)a * dn_sin_wide(b)))
DN_FUNCTOR0(FSinDeriv, (float)((double)a * dn_cos_wide(b)))
DN_FUNCTOR0(FLogisticDeriv, (float)((double)(a * b) * (1.0 - (double)b)))
DN_FUNCTOR0(FTanhDeriv, (float)((double)a * (1.0 + (double)b) * (1.0 - (double)b) * 0.5))
DN_FUNCTOR0(FReluDeriv, a * (b > 0.f ? 1.f : 0.f))
DN_FUNCTOR0(FReluSmoothDeriv, (float)((double)a * -dn_expm1_wide(-(double)b)))
DN_FUNCTOR1(FAxpy, a + s * b)
DN_FUNCTOR1(FAddMultSign, a + ((b > 0.f) ? s : ((b < 0.f) ? -s : 0.f)))
DN_FUNCTOR1(FCrossEntropy, (float)(-(double)a * dn_log_wide(b + s)))
DN_FUNCTOR1(FCrossEntropyBernoulli,
            (float)(-(double)a * dn_log_wide(b + s) - (double)(1.f - a) * dn_log_wide(1.f - b + s)))
DN_FUNCTOR1(FCorrectPreds, a * (float)(b >= s) + (1.f - a) * (float)(b < s))
// matrix (op) scalar (cudamat_kernels.cu:310-364, 687-716)
DN_FUNCTOR1(FLtS, a < s ? 1.f : 0.f)
DN_FUNCTOR1(FLeS, a <= s ? 1.f : 0.f)
DN_FUNCTOR1(FGtS, a > s ? 1.f : 0.f)
DN_FUNCTOR1(FGeS, a >= s ? 1.f : 0.f)
DN_FUNCTOR1(FUpperS, a > s ? s : a)
DN_FUNCTOR1(FLowerS, a < s ? s : a)
DN_FUNCTOR1(FMulS, s * a)
DN_FUNCTOR1(FDivS, a / s)
DN_FUNCTOR1(FAddS, a + s)
DN_FUNCTOR1(FAssignS, s)

// ------------------------------------------------------------------ kernels

#define EW_THREADS 256

// NIN inputs (0, 1 or 2) -> one output, one 16-byte vector per lane (the shape
// that measures fastest on this part: every lane issues its loads at once and
// the grid is large enough to cover the latency).  [head, head + 4*n4) is moved
// as vectors; the up-to-3 leading and trailing elements by single lanes.
template <int NIN, bool STREAM, class F>
__global__ void __launch_bounds__(EW_THREADS)
k_ew(const float* a, const float* b, float* t, long long n, int head, long long n4, F f) {
  const long long tid = (long long)blockIdx.x * EW_THREADS + threadIdx.x;
  if (tid < n4) {
    const long long e = head + 4 * tid;
    float4 va = make_float4(0.f, 0.f, 0.f, 0.f), vb = va;
    if (NIN >= 1) va = dn_ld4<STREAM>(a + e);
    if (NIN >= 2) vb = dn_ld4<STREAM>(b + e);
    float4 r;
    r.x = f(va.x, vb.x);
    r.y = f(va.y, vb.y);
    r.z = f(va.z, vb.z);
    r.w = f(va.w, vb.w);
    dn_st4<STREAM>(t + e, r);
  }
  // ragged ends
  const long long tail0 = head + 4 * n4;
  if (tid < head) {
    t[tid] = f(NIN >= 1 ? a[tid] : 0.f, NIN >= 2 ? b[tid] : 0.f);
  } else if (tid - head < n - tail0) {
    const long long j = tail0 + (tid - head);
    t[j] = f(NIN >= 1 ? a[j] : 0.f, NIN >= 2 ? b[j] : 0.f);
  }
}

// Fallback for operands whose 16-byte phases differ: 4-byte accesses.
template <int NIN, class F>
__global__ void __launch_bounds__(EW_THREADS) k_ew_scalar(const float* a, const float* b, float* t, long long n, F f) {
  const long long stride = (long long)gridDim.x * EW_THREADS;
  for (long long i = (long long)blockIdx.x * EW_THREADS + threadIdx.x; i < n; i += stride)
    t[i] = f(NIN >= 1 ? a[i] : 0.f, NIN >= 2 ? b[i] : 0.f);
}

static inline int head_of(const void* p) {  // elements until the next 16-byte boundary
  return (int)(((16u - (reinterpret_cast<uintptr_t>(p) & 15u)) & 15u) >> 2);
}

template <int NIN, class F>
static int launch_ew(const float* a, const float* b, float* t, long long n, F f) {
  if (n <= 0) return 0;
  const int cus = dn_num_cus();
  const int ht = head_of(t);
  const bool same_phase = (NIN < 1 || head_of(a) == ht) && (NIN < 2 || head_of(b) == ht) &&
                          ((reinterpret_cast<uintptr_t>(t) & 3u) == 0);
  if (same_phase) {
    const int head = (int)(ht < n ? ht : n);
    const long long n4 = (n - head) / 4;
    long long blocks = (n4 + EW_THREADS - 1) / EW_THREADS;
    if (blocks < 1) blocks = 1;
    if (blocks > 0x7fffffffll) return ERROR_UNSUPPORTED;
    if (n >= DN_STREAM_MIN_ELEMS)
      hipLaunchKernelGGL((k_ew<NIN, true, F>), dim3((unsigned)blocks), dim3(EW_THREADS), 0, dn_stream(), a, b, t, n, head, n4, f);
    else
      hipLaunchKernelGGL((k_ew<NIN, false, F>), dim3((unsigned)blocks), dim3(EW_THREADS), 0, dn_stream(), a, b, t, n, head, n4, f);
  } else {
    long long blocks = (n + EW_THREADS - 1) / EW_THREADS;
    const long long cap = (long long)cus * 32;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL((k_ew_scalar<NIN, F>), dim3((unsigned)blocks), dim3(EW_THREADS), 0, dn_stream(), a, b, t, n, f);
  }
  return dn_launch_status();
}

// Broadcast of a vector along rows (vec[i % h], a column vector) or along
// columns (vec[i / h], a row vector) into a flat pass over the matrix.  The
// row / column of the first element of each 16-byte group comes from one
// multiply-high; the other three follow by increment-and-wrap.
template <bool COLVEC, bool STREAM, bool VEC4, class F>
__global__ void __launch_bounds__(EW_THREADS)
k_bcast(const float* a, const float* vec, float* t, long long n, int head, long long n4, FastDiv fd, F f) {
  const long long tid = (long long)blockIdx.x * EW_THREADS + threadIdx.x;
  const uint32_t h = fd.d;
  if (tid < n4) {
    const uint32_t e = (uint32_t)(head + 4 * tid);
    const float4 va = dn_ld4<STREAM>(a + e);
    uint32_t q = fd_div(e, fd);
    uint32_t r = e - q * h;
    float v[4];
    const float x[4] = {va.x, va.y, va.z, va.w};
    if constexpr (VEC4) {
      // COLVEC, no head, h a multiple of 4, aligned vector: the four rows are one 16-byte
      // group of the vector and never wrap into the next column
      const float4 vv = *reinterpret_cast<const float4*>(vec + r);
      v[0] = f(x[0], vv.x); v[1] = f(x[1], vv.y); v[2] = f(x[2], vv.z); v[3] = f(x[3], vv.w);
    } else {
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        v[k] = f(x[k], vec[COLVEC ? r : q]);
        if (++r == h) { r = 0; ++q; }
      }
    }
    dn_st4<STREAM>(t + e, make_float4(v[0], v[1], v[2], v[3]));
  }
  const long long tail0 = head + 4 * n4;
  long long j = -1;
  if (tid < head) j = tid;
  else if (tid - head < n - tail0) j = tail0 + (tid - head);
  if (j >= 0) {
    const uint32_t q = fd_div((uint32_t)j, fd);
    const uint32_t r = (uint32_t)j - q * h;
    t[j] = f(a[j], vec[COLVEC ? r : q]);
  }
}

template <bool COLVEC, class F>
__global__ void __launch_bounds__(EW_THREADS)
k_bcast_scalar(const float* a, const float* vec, float* t, long long n, FastDiv fd, F f) {
  const long long stride = (long long)gridDim.x * EW_THREADS;
  for (long long i = (long long)blockIdx.x * EW_THREADS + threadIdx.x; i < n; i += stride) {
    const uint32_t q = fd_div((uint32_t)i, fd);
    const uint32_t r = (uint32_t)i - q * fd.d;
    t[i] = f(a[i], vec[COLVEC ? r : q]);
  }
}

template <bool COLVEC, class F>
static int launch_bcast(const float* a, const float* vec, float* t, int h, int w, F f) {
  const long long n = (long long)h * w;
  if (n <= 0) return 0;
  if (n >= (1ll << 32)) return ERROR_UNSUPPORTED;  // 32-bit element index inside the kernel
  const FastDiv fd = make_fastdiv((uint32_t)h);
  const int cus = dn_num_cus();
  const int ht = head_of(t);
  if (head_of(a) == ht) {
    const int head = (int)(ht < n ? ht : n);
    const long long n4 = (n - head) / 4;
    long long blocks = (n4 + EW_THREADS - 1) / EW_THREADS;
    if (blocks < 1) blocks = 1;
    const bool vec4 = COLVEC && head == 0 && h % 4 == 0 && dn_aligned16(vec);
#define BCAST_LAUNCH(ST, V4)                                                                                  \
  hipLaunchKernelGGL((k_bcast<COLVEC, ST, V4, F>), dim3((unsigned)blocks), dim3(EW_THREADS), 0, dn_stream(), a, vec, t, n, \
                     head, n4, fd, f)
    if (n >= DN_STREAM_MIN_ELEMS) {
      if (vec4) BCAST_LAUNCH(true, COLVEC); else BCAST_LAUNCH(true, false);
    } else {
      if (vec4) BCAST_LAUNCH(false, COLVEC); else BCAST_LAUNCH(false, false);
    }
#undef BCAST_LAUNCH
  } else {
    long long blocks = (n + EW_THREADS - 1) / EW_THREADS;
    const long long cap = (long long)cus * 32;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL((k_bcast_scalar<COLVEC, F>), dim3((unsigned)blocks), dim3(EW_THREADS), 0, dn_stream(), a, vec, t, n, fd,
                       f);
  }
  return dn_launch_status();
}

// Diagonal of a square w x w matrix: element i*(w+1).  vec may be null (scalar form).
template <class F>
__global__ void k_diag(const float* a, const float* vec, float* t, int w, F f) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < w) {
    const size_t p = (size_t)i * w + i;
    t[p] = f(a[p], vec ? vec[i] : 0.f);
  }
}

template <class F>
static int launch_diag(const float* a, const float* vec, float* t, int w, F f) {
  if (w <= 0) return 0;
  hipLaunchKernelGGL((k_diag<F>), dim3((w + 255) / 256), dim3(256), 0, dn_stream(), a, vec, t, w, f);
  return dn_launch_status();
}

// ------------------------------------------------------------------ argument checks
// Each family keeps the order of checks of the wrappers it replaces.

static inline bool same_dims(const cudamat* a, const cudamat* b) {
  return a->size[0] == b->size[0] && a->size[1] == b->size[1];
}

// unary math (cudamat.cu:1339-1546): device, then dims.
static inline int check_unary(const cudamat* mat, const cudamat* target) {
  if (!mat->on_device || !target->on_device) return ERROR_NOT_ON_DEVICE;
  if (!same_dims(mat, target)) return ERROR_INCOMPATIBLE_DIMENSIONS;
  return 0;
}
// sign and matrix-vs-scalar comparisons (cudamat.cu:923-966, 1060-1146, 1318-1338):
// device, transposedness of mat vs target, dims.
static inline int check_unary_trans(const cudamat* mat, const cudamat* target) {
  if (!mat->on_device || !target->on_device) return ERROR_NOT_ON_DEVICE;
  if (mat->is_trans != target->is_trans) return ERROR_TRANSPOSEDNESS;
  if (!same_dims(mat, target)) return ERROR_INCOMPATIBLE_DIMENSIONS;
  return 0;
}
// binary elementwise (cudamat.cu:878-1059, 1803-2030): device, transposedness
// of the two inputs, dims.
static inline int check_binary(const cudamat* m1, const cudamat* m2, const cudamat* target) {
  if (!m1->on_device || !m2->on_device || !target->on_device) return ERROR_NOT_ON_DEVICE;
  if (m1->is_trans != m2->is_trans) return ERROR_TRANSPOSEDNESS;
  if (!same_dims(m1, m2) || !same_dims(m1, target)) return ERROR_INCOMPATIBLE_DIMENSIONS;
  return 0;
}
// pow_matrix / cross-entropy family (cudamat.cu:1566-1650): device of mat and
// target, dims of target, dims of the second input.
static inline int check_binary_notrans(const cudamat* mat, const cudamat* p, const cudamat* target) {
  if (!mat->on_device || !target->on_device || !p->on_device) return ERROR_NOT_ON_DEVICE;
  if (!same_dims(mat, target)) return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (!same_dims(mat, p)) return ERROR_INCOMPATIBLE_DIMENSIONS;
  return 0;
}
// column-vector broadcasts (cudamat.cu:592-639, 783-853): device, mat not
// transposed, vec is h x 1 and target matches.
static inline int check_colvec(const cudamat* mat, const cudamat* vec, const cudamat* target) {
  if (!mat->on_device || !vec->on_device || !target->on_device) return ERROR_NOT_ON_DEVICE;
  if (mat->is_trans) return ERROR_TRANSPOSED;
  if (mat->size[0] != vec->size[0] || vec->size[1] != 1 || !same_dims(mat, target))
    return ERROR_INCOMPATIBLE_DIMENSIONS;
  return 0;
}
// row-vector broadcasts (cudamat.cu:735-781, 807-877): vec is 1 x w.
static inline int check_rowvec(const cudamat* mat, const cudamat* vec, const cudamat* target) {
  if (!mat->on_device || !vec->on_device || !target->on_device) return ERROR_NOT_ON_DEVICE;
  if (mat->is_trans) return ERROR_TRANSPOSED;
  if (mat->size[1] != vec->size[1] || vec->size[0] != 1 || !same_dims(mat, target))
    return ERROR_INCOMPATIBLE_DIMENSIONS;
  return 0;
}

#define DN_UNARY(NAME, CHECK, FUNCTOR)                                                        \
  int NAME(cudamat* mat, cudamat* target) {                                                   \
    if (int e = CHECK(mat, target)) return e;                                                 \
    return launch_ew<1>(mat->data_device, nullptr, target->data_device, dn_len(mat), FUNCTOR); \
  }
#define DN_BINARY(NAME, CHECK, FUNCTOR)                                                                   \
  int NAME(cudamat* mat1, cudamat* mat2, cudamat* target) {                                               \
    if (int e = CHECK(mat1, mat2, target)) return e;                                                      \
    return launch_ew<2>(mat1->data_device, mat2->data_device, target->data_device, dn_len(mat1), FUNCTOR); \
  }
#define DN_SCALAR(NAME, CHECK, FUNCTOR)                                                                 \
  int NAME(cudamat* mat, float val, cudamat* target) {                                                  \
    if (int e = CHECK(mat, target)) return e;                                                           \
    return launch_ew<1>(mat->data_device, nullptr, target->data_device, dn_len(mat), FUNCTOR{val});      \
  }
#define DN_BINARY_PARAM(NAME, FUNCTOR)                                                                          \
  int NAME(cudamat* mat, cudamat* p, cudamat* target, float s) {                                                \
    if (int e = check_binary_notrans(mat, p, target)) return e;                                                 \
    return launch_ew<2>(mat->data_device, p->data_device, target->data_device, dn_len(mat), FUNCTOR{s});         \
  }
#define DN_COLVEC(NAME, FUNCTOR)                                                                   \
  int NAME(cudamat* mat, cudamat* vec, cudamat* target) {                                          \
    if (int e = check_colvec(mat, vec, target)) return e;                                          \
    return launch_bcast<true>(mat->data_device, vec->data_device, target->data_device, mat->size[0], \
                              mat->size[1], FUNCTOR);                                              \
  }
#define DN_ROWVEC(NAME, FUNCTOR)                                                                    \
  int NAME(cudamat* mat, cudamat* vec, cudamat* target) {                                           \
    if (int e = check_rowvec(mat, vec, target)) return e;                                           \
    return launch_bcast<false>(mat->data_device, vec->data_device, target->data_device, mat->size[0], \
                               mat->size[1], FUNCTOR);                                              \
  }

extern "C" {

// ---- unary
DN_UNARY(sign, check_unary_trans, FSign{})
DN_UNARY(apply_cos, check_unary, FCos{})
DN_UNARY(apply_sin, check_unary, FSin{})
DN_UNARY(apply_abs, check_unary, FAbs{})
DN_UNARY(apply_log_1_plus_exp, check_unary, FLog1pExp{})
DN_UNARY(apply_exp, check_unary, FExp{})
DN_UNARY(apply_ceil, check_unary, FCeil{})
DN_UNARY(apply_floor, check_unary, FFloor{})
DN_UNARY(apply_sqrt, check_unary, FSqrt{})
DN_UNARY(reciprocal, check_unary, FRecip{})

int apply_log(cudamat* mat, cudamat* target, float tiny) {
  if (int e = check_unary(mat, target)) return e;
  return launch_ew<1>(mat->data_device, nullptr, target->data_device, dn_len(mat), FLog{tiny});
}

// ---- matrix (op) scalar
DN_SCALAR(apply_pow, check_unary, FPow)
DN_SCALAR(less_than_eq_scalar, check_unary_trans, FLeS)
DN_SCALAR(less_than_scalar, check_unary_trans, FLtS)
DN_SCALAR(greater_than_eq_scalar, check_unary_trans, FGeS)
DN_SCALAR(upper_bound_scalar, check_unary_trans, FUpperS)
DN_SCALAR(divide_by_scalar, check_unary, FDivS)
DN_SCALAR(add_scalar, check_unary, FAddS)

// ---- binary
DN_BINARY(less_than_eq, check_binary, FLe{})
// (defined with the held-back fill_with_rand below: r.fill_with_rand(); r.less_than(h, target = h) is a sample)
int less_than(cudamat* mat1, cudamat* mat2, cudamat* target);
DN_BINARY(greater_than_eq, check_binary, FGe{})
DN_BINARY(greater_than, check_binary, FGt{})
DN_BINARY(upper_bound, check_binary, FUpper{})
DN_BINARY(lower_bound, check_binary, FLower{})
DN_BINARY(add_elementwise, check_binary, FAdd{})
DN_BINARY(subtract_elementwise, check_binary, FSub{})
DN_BINARY(divide_elementwise, check_binary, FDiv{})
DN_BINARY(apply_sin_deriv, check_binary, FSinDeriv{})
DN_BINARY(apply_cos_deriv, check_binary, FCosDeriv{})
DN_BINARY(apply_logistic_deriv, check_binary, FLogisticDeriv{})
DN_BINARY(apply_tanh_deriv, check_binary, FTanhDeriv{})
// (defined with the deferred epilogues below: a held-back product may take it along)
int apply_rectified_linear_deriv(cudamat* mat1, cudamat* mat2, cudamat* target);
DN_BINARY(apply_rectified_linear_smooth_deriv, check_binary, FReluSmoothDeriv{})
DN_BINARY(apply_pow_matrix, check_binary_notrans, FPowMat{})
DN_BINARY_PARAM(compute_cross_entropy, FCrossEntropy)
DN_BINARY_PARAM(compute_cross_entropy_bernoulli, FCrossEntropyBernoulli)
DN_BINARY_PARAM(correct_preds, FCorrectPreds)

// ---- broadcasts
DN_COLVEC(mult_by_col_vec, FMul{})
DN_COLVEC(div_by_col_vec, FDiv{})
DN_ROWVEC(add_row_vec, FAdd{})
DN_ROWVEC(mult_by_row_vec, FMul{})
DN_ROWVEC(div_by_row_vec, FDiv{})

int add_col_mult(cudamat* mat, cudamat* vec, cudamat* target, float mult) {
  if (int e = check_colvec(mat, vec, target)) return e;
  return launch_bcast<true>(mat->data_device, vec->data_device, target->data_device, mat->size[0], mat->size[1],
                            FAxpy{mult});
}

int add_row_mult(cudamat* mat, cudamat* vec, cudamat* target, float mult) {
  if (int e = check_rowvec(mat, vec, target)) return e;
  return launch_bcast<false>(mat->data_device, vec->data_device, target->data_device, mat->size[0], mat->size[1],
                             FAxpy{mult});
}

// ---- diagonal (cudamat.cu:641-733): only the w diagonal entries of target are written.
static inline int check_diag(const cudamat* mat, const cudamat* vec, const cudamat* target) {
  if (!mat->on_device || (vec && !vec->on_device) || !target->on_device) return ERROR_NOT_ON_DEVICE;
  if (mat->is_trans) return ERROR_TRANSPOSED;
  if ((vec && mat->size[0] != vec->size[1] * vec->size[0]) || !same_dims(mat, target))
    return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (mat->size[0] < mat->size[1]) return ERROR_INCOMPATIBLE_DIMENSIONS;  // diagonal index i*w+i must stay inside
  return 0;
}

int mult_diagonal_scalar(cudamat* mat, float val, cudamat* target) {
  if (int e = check_diag(mat, nullptr, target)) return e;
  return launch_diag(mat->data_device, nullptr, target->data_device, mat->size[1], FMulS{val});
}
int add_diagonal_scalar(cudamat* mat, float val, cudamat* target) {
  if (int e = check_diag(mat, nullptr, target)) return e;
  return launch_diag(mat->data_device, nullptr, target->data_device, mat->size[1], FAddS{val});
}
int mult_diagonal(cudamat* mat, cudamat* vec, cudamat* target) {
  if (int e = check_diag(mat, vec, target)) return e;
  return launch_diag(mat->data_device, vec->data_device, target->data_device, mat->size[1], FMul{});
}
int add_diagonal(cudamat* mat, cudamat* vec, cudamat* target) {
  if (int e = check_diag(mat, vec, target)) return e;
  return launch_diag(mat->data_device, vec->data_device, target->data_device, mat->size[1], FAdd{});
}

}  // extern "C"

int dn_gemm_fused(bool a_trans, bool b_trans, int M, int N, int K, const float* A, int lda, const float* B, int ldb,
                  float* C, int ldc, const float* bias, int act, bool* fused, const DnGemmSample* smp, bool* sampled,
                  const float* gate, int drop, float drop_p, const float* mul);

// ------------------------------------------------------------------ deferred epilogues
// Every layer of deepnet computes its state as  dot -> add_col_vec -> apply_sigmoid (or
// lower_bound(0), apply_tanh) [-> sample_bernoulli]  (deepnet/dbm.py:95-105,
// neuralnet.py:138-160, cudamat/examples/rbm_cudamat.py:46-70): three or four launches of 2-5 us
// each, and as many trips through the runtime's launch path, which is what such a step spends its
// time on.  The product kernels can carry the bias, the activation and the sample in their
// epilogue (dot_bias_act), so dot() with alpha = 1, beta = 0 does not launch at once: it is held
// back, and while the calls that follow are exactly the rest of that sequence on the product's
// own target they are folded into it; the launch happens at tanh, at the sample, or at the first
// call of any other kind (everything that queues work, hands out a workspace, moves data or waits
// for the device passes through dn_flush()).  Behind lower_bound(0) the product waits once more: the
// dropout mask of its target (fill_with_rand -> greater_than -> mult, neuralnet.py:194-198) is drawn
// in its epilogue when it follows.  apply_rectified_linear_deriv(target, state) directly behind the
// product (a layer's backward pass, neuralnet.py:203-222) is folded likewise.  The arithmetic is
// that of the separate calls, bit for bit (tests/test_gpu_deferred.py), work reaches the stream
// in call order, and a sequence that does not continue costs one kernel as before.
struct DnPending {
  bool active;
  cudamat a, b, t, bias, gate, mul;
  bool has_bias, has_gate, has_mul;
  int act;            // 0 none yet, 1 sigmoid (waiting for a possible sample), 2 max(x, 0) (waiting for a possible mask)
};
static DnPending g_pend = {};
static bool g_no_defer = false;      // the library is issuing the calls of a sequence itself
static bool g_defer_enabled = true;

static void refresh_pending();      // tells the library whether anything is still held back
static bool held_besides_updates();
static inline bool pend_is(const cudamat* x);
static inline bool pend_open();

static int dot_bias_act_impl(rnd_struct* rnd, cudamat* mat1, cudamat* mat2, cudamat* bias, cudamat* target,
                             cudamat* sample, int act, cudamat* gate = nullptr, bool drop = false, float drop_p = 0.f,
                             cudamat* mul = nullptr);

// Launches the held-back sequence (with the sample, when one is given).
static int run_pending(rnd_struct* rnd, cudamat* sample) {
  DnPending p = g_pend;
  g_pend.active = false;
  refresh_pending();
  const bool saved = g_no_defer;
  g_no_defer = true;
  const int e = dot_bias_act_impl(rnd, &p.a, &p.b, p.has_bias ? &p.bias : nullptr, &p.t, sample, p.act, p.has_gate ? &p.gate : nullptr,
                                  false, 0.f, p.has_mul ? &p.mul : nullptr);
  g_no_defer = saved;
  return e;
}
static int run_queue(bool reset);
static int queued_calls();
static int run_batch();
static int stash_ready(bool reset);
static bool update_ready();
static int batched_updates();

// ---- products that accumulate into their target (add_dot / subtract_dot, beta = 1) and sums along
// the rows added to a vector (add_sums).  A contrastive-divergence step ends with
//   W.add_dot(v, h.T, eps); W.add_dot(v', h'.T, -eps); bv.add_sums(v, 1, eps); bv.add_sums(v', 1, -eps);
//   bh.add_sums(h, 1, eps); bh.add_sums(h', 1, -eps)
// (cudamat/examples/rbm_cudamat.py:73-86): six launches of 2-5 us.  A product with beta = 1 waits for
// a second product of the same shape into the same target, the pair waits for row sums, and up to
// four row sums onto at most two vectors wait for each other: all of it runs as one launch
// (dn_gemm_pair_sums; sums without a pair: dn_row_sum_jobs).  Each result has the bits of the
// separate launches; sums that touch the pair's operands or target, and anything else that
// arrives, launch what is held back first, in call order.
struct PendAcc {
  bool active;
  bool paired;          // the second product has arrived: the pair waits for the sums that may follow
  cudamat a, b, t, a2, b2;
  float alpha, beta, alpha2;
  int m, n, k;
};
static PendAcc g_acc = {};
static DnRowSumJob g_sums[4];
static int g_nsums = 0;

// Launches the held-back product (or pair), together with the queued row sums when both wait.
static int run_stats() {
  const PendAcc p = g_acc;
  DnRowSumJob jobs[4];
  const int n = g_nsums;
  for (int i = 0; i < n; ++i) jobs[i] = g_sums[i];
  g_acc.active = false;
  g_nsums = 0;
  refresh_pending();
  if (!p.active) return n > 0 ? dn_row_sum_jobs(jobs, n) : 0;
  const bool ta = p.a.is_trans != 0, tb = p.b.is_trans != 0;
  if (p.paired)
    return dn_gemm_pair_sums(ta, tb, p.m, p.n, p.k, p.alpha, p.a.data_device, p.a.size[0], p.b.data_device, p.b.size[0], p.beta,
                             p.alpha2, p.a2.data_device, p.a2.size[0], p.b2.data_device, p.b2.size[0], p.t.data_device,
                             p.t.size[0], jobs, n);
  return dn_gemm_sums(ta, tb, p.m, p.n, p.k, p.alpha, p.a.data_device, p.a.size[0], p.b.data_device, p.b.size[0], p.beta,
                      p.t.data_device, p.t.size[0], jobs, n);
}

// ---- the dropout mask: mask.fill_with_rand(); mask.greater_than(p); state.mult(mask)
// (deepnet/neuralnet.py:194-198) as one pass over the generator's streams.
struct PendDrop {
  int stage;            // 0 nothing, 1 fill_with_rand held back, 2 ... and its threshold
  bool with_pend;       // ... behind a held-back product with max(x, 0), whose target the mask may be meant for
  rnd_struct* rnd;
  cudamat mask;
  float p;
};
static PendDrop g_drop = {};

extern "C" int fill_with_rand(rnd_struct* rnd_state, cudamat* mat);

static int run_drop(cudamat* state) {
  const PendDrop d = g_drop;
  g_drop.stage = 0;
  refresh_pending();
  const bool saved = g_no_defer;
  g_no_defer = true;
  int e;
  cudamat mask = d.mask;
  if (d.stage == 1) e = fill_with_rand(d.rnd, &mask);
  else e = dn_rng_dropmask(d.rnd, mask.data_device, state ? state->data_device : nullptr, (size_t)dn_len(&mask), d.p);
  g_no_defer = saved;
  return e;
}

static bool g_flushing = false;
static void flush_pending() {
  // (the launches below come back here through dn_stream(): what is still held back is launched by this
  // call, in order, not by theirs)
  if (g_flushing) return;
  g_flushing = true;
  if (update_ready()) stash_ready(false);          // (a complete update joins the ones that wait)
  if (batched_updates() > 0) run_batch();          // older than anything else that is held back
  if (g_pend.active) run_pending(nullptr, nullptr);
  if (queued_calls() > 0) run_queue(false);
  if (g_acc.active || g_nsums > 0) run_stats();
  if (g_drop.stage) run_drop(nullptr);
  dn_softmax_flush();
  g_flushing = false;
  refresh_pending();
}
static const int g_flush_registered = (dn_set_flush_hook(flush_pending), 0);

static inline bool overlap(const float* p, long long np, const float* q, long long nq) {
  return p < q + nq && q < p + np;
}

bool dn_defer_dot(cudamat* mat1, cudamat* mat2, cudamat* target, float beta, float alpha, int m, int n, int k, int* err) {
  *err = 0;
  if (g_no_defer || !g_defer_enabled) return false;
  if (target->is_trans || m <= 1 || n <= 1 || k <= 0) return false;
  if (beta == 1.f) {
    // the second product of a pair: same target, same shapes and transposes, operands that the first does not write
    if (g_acc.active && target->data_device == g_acc.t.data_device && target->size[0] == g_acc.t.size[0] && m == g_acc.m &&
        n == g_acc.n && k == g_acc.k && (mat1->is_trans != 0) == (g_acc.a.is_trans != 0) &&
        (mat2->is_trans != 0) == (g_acc.b.is_trans != 0) &&
        !overlap(mat1->data_device, dn_len(mat1), target->data_device, dn_len(target)) &&
        !overlap(mat2->data_device, dn_len(mat2), target->data_device, dn_len(target)) && !g_acc.paired && g_nsums == 0) {
      g_acc.paired = true;            // (stays held back: the sums of the same statistics may follow)
      g_acc.a2 = *mat1; g_acc.b2 = *mat2; g_acc.alpha2 = alpha;
      return true;
    }
    dn_flush();
    if (k > 128) return false;        // (pairs run as one launch only for short reductions)
    g_acc.active = true;
    g_acc.paired = false;
    g_acc.a = *mat1; g_acc.b = *mat2; g_acc.t = *target;
    g_acc.alpha = alpha; g_acc.beta = beta;
    g_acc.m = m; g_acc.n = n; g_acc.k = k;
    dn_set_pending(true);
    return true;
  }
  if (alpha != 1.f || beta != 0.f) return false;
  dn_flush();                         // at most one product is held back
  g_pend.active = true;
  g_pend.a = *mat1; g_pend.b = *mat2; g_pend.t = *target;
  g_pend.has_bias = false;
  g_pend.has_gate = false;
  g_pend.has_mul = false;
  g_pend.act = 0;
  dn_set_pending(true);
  return true;
}

bool dn_defer_fill_rand(rnd_struct* rnd, cudamat* mat, int* err) {
  *err = 0;
  if (g_no_defer || !g_defer_enabled || mat->is_trans || dn_len(mat) <= 0) return false;
  // behind a product with max(x, 0) that waits (and nothing else does): a mask of its target's shape, apart from
  // its operands, may turn out to be its dropout mask; both wait then
  bool with = g_pend.active && g_pend.act == 2 && !g_pend.has_gate && !g_pend.has_mul && queued_calls() == 0 && batched_updates() == 0 && !g_acc.active && g_nsums == 0 &&
              g_drop.stage == 0 && !dn_softmax_held() && rnd && rnd->dev_mults && rnd->dev_words &&
              mat->size[0] == g_pend.t.size[0] && mat->size[1] == g_pend.t.size[1];
  if (with) {
    const cudamat* ops[4] = {&g_pend.t, &g_pend.a, &g_pend.b, &g_pend.bias};
    for (int i = 0; i < (g_pend.has_bias ? 4 : 3) && with; ++i)
      with = !overlap(mat->data_device, dn_len(mat), ops[i]->data_device, dn_len(ops[i]));
  }
  if (!with) dn_flush();
  g_drop.stage = 1;
  g_drop.with_pend = with;
  g_drop.rnd = rnd;
  g_drop.mask = *mat;
  g_drop.p = 0.f;
  dn_set_pending(true);
  return true;
}
static inline bool drop_mask_is(const cudamat* x) {
  return x->on_device && !x->is_trans && x->data_device == g_drop.mask.data_device && x->size[0] == g_drop.mask.size[0] &&
         x->size[1] == g_drop.mask.size[1];
}

extern "C" {

int greater_than_scalar(cudamat* mat, float val, cudamat* target) {
  if (g_drop.stage == 1 && !g_no_defer && drop_mask_is(mat) && drop_mask_is(target)) {
    g_drop.stage = 2;
    g_drop.p = val;
    return 0;
  }
  if (int e = check_unary_trans(mat, target)) return e;
  return launch_ew<1>(mat->data_device, nullptr, target->data_device, dn_len(mat), FGtS{val});
}

// r.fill_with_rand(); r.less_than(h, target = h): the hidden sample as cudamat/examples/rbm_cudamat.py:63-65
// spells it, in one pass over the generator's streams (h gets the sample, r the uniforms).
int less_than(cudamat* mat1, cudamat* mat2, cudamat* target) {
  if (g_drop.stage == 1 && !g_no_defer && drop_mask_is(mat1) && mat2->on_device && !mat2->is_trans && target->on_device &&
      !target->is_trans && target->data_device == mat2->data_device && mat2->size[0] == mat1->size[0] &&
      mat2->size[1] == mat1->size[1] && target->size[0] == mat2->size[0] && target->size[1] == mat2->size[1] &&
      !overlap(mat1->data_device, dn_len(mat1), mat2->data_device, dn_len(mat2))) {
    const PendDrop d = g_drop;
    g_drop.stage = 0;
    if (g_pend.active) {              // (a product that waits with the fill comes first, by itself)
      if (int e = run_pending(nullptr, nullptr)) return e;
    }
    refresh_pending();
    return dn_rng_bernoulli_keep(d.rnd, d.mask.data_device, mat2->data_device, (size_t)dn_len(mat2));
  }
  if (int e = check_binary(mat1, mat2, target)) return e;
  return launch_ew<2>(mat1->data_device, mat2->data_device, target->data_device, dn_len(mat1), FLt{});
}

int mult_elementwise(cudamat* mat1, cudamat* mat2, cudamat* target) {
  if (g_drop.stage == 2 && !g_no_defer && drop_mask_is(mat2) && mat1->on_device && !mat1->is_trans && target->on_device &&
      !target->is_trans && target->data_device == mat1->data_device && mat1->size[0] == mat2->size[0] &&
      mat1->size[1] == mat2->size[1] && target->size[0] == mat1->size[0] && target->size[1] == mat1->size[1] &&
      !overlap(mat1->data_device, dn_len(mat1), mat2->data_device, dn_len(mat2))) {
    if (g_drop.with_pend && g_pend.active && g_pend.act == 2 && pend_is(mat1)) {
      // the mask is for the product that waits: product, bias, max(x, 0), mask and masking in one launch
      const PendDrop d = g_drop;
      DnPending p = g_pend;
      g_drop.stage = 0;
      g_pend.active = false;
      refresh_pending();
      const bool saved = g_no_defer;
      g_no_defer = true;
      cudamat mask = d.mask;
      const int e = dot_bias_act_impl(d.rnd, &p.a, &p.b, p.has_bias ? &p.bias : nullptr, &p.t, &mask, p.act, nullptr, true, d.p);
      g_no_defer = saved;
      return e;
    }
    if (g_pend.active) {              // (the product that waits is another matter: it comes first, by itself)
      const PendDrop d = g_drop;
      g_drop.stage = 0;
      const int e = run_pending(nullptr, nullptr);
      g_drop = d;
      refresh_pending();
      if (e) return e;
    }
    return run_drop(mat1);
  }
  // deriv = dot(w, deriv_above); deriv.mult(mask) [; deriv.apply_rectified_linear_deriv(state)]: the backward pass
  // of a layer with dropout (deepnet/neuralnet.py:203-222): the factor rides in the product's epilogue
  if (pend_open() && g_pend.act == 0 && !g_pend.has_bias && !g_pend.has_gate && !g_pend.has_mul && g_drop.stage == 0 &&
      pend_is(mat1) && pend_is(target) && mat2->on_device && !mat2->is_trans && mat2->size[0] == target->size[0] &&
      mat2->size[1] == target->size[1] && !overlap(mat2->data_device, dn_len(mat2), target->data_device, dn_len(target))) {
    g_pend.mul = *mat2;
    g_pend.has_mul = true;            // stays held back: the derivative of the activation may follow
    return 0;
  }
  if (int e = check_binary(mat1, mat2, target)) return e;
  return launch_ew<2>(mat1->data_device, mat2->data_device, target->data_device, dn_len(mat1), FMul{});
}

}  // extern "C"

bool dn_defer_row_sum(const float* M, float* y, int h, int w, float alpha, float beta, int* err) {
  *err = 0;
  const int kind = (g_no_defer || !g_defer_enabled || beta != 1.f) ? 0 : dn_row_sum_job_kind(M, h, w);
  if (kind == 0) return false;
  if (overlap(M, (long long)h * w, y, h)) return false;
  // does the call join what is queued?  At most two vectors with two sums each; no vector may share
  // memory with another one or with a matrix that a queued sum reads (the order of the launches
  // would matter then)
  bool fits = g_nsums > 0;
  const float* ys[2] = {nullptr, nullptr};
  int cnt[2] = {0, 0}, nys = 0, mine = -1;
  for (int i = 0; i < g_nsums && fits; ++i) {
    const DnRowSumJob& q = g_sums[i];
    int t = -1;
    for (int u = 0; u < nys; ++u) if (ys[u] == q.y) t = u;
    if (t < 0) { t = nys; ys[nys++] = q.y; }
    ++cnt[t];
    if (q.y == y && q.h == h) mine = t;
    else if (overlap(q.y, q.h, y, h)) fits = false;
    if (overlap(q.M, (long long)q.h * q.w, y, h) || overlap(M, (long long)h * w, q.y, q.h)) fits = false;
  }
  if (fits && (mine >= 0 ? cnt[mine] >= 2 : nys >= 2)) fits = false;
  // a sum may join the product (or the pair of products) that waits, unless it writes what they read
  // or write, or reads what they write
  if (g_acc.active && (fits || g_nsums == 0)) {
    const cudamat* ops[5] = {&g_acc.t, &g_acc.a, &g_acc.b, &g_acc.a2, &g_acc.b2};
    const int nops = g_acc.paired ? 5 : 3;
    fits = !overlap(M, (long long)h * w, g_acc.t.data_device, dn_len(&g_acc.t));
    for (int i = 0; i < nops && fits; ++i) fits = !overlap(y, h, ops[i]->data_device, dn_len(ops[i]));
  }
  if (!fits) dn_flush();
  g_sums[g_nsums++] = DnRowSumJob{M, y, h, w, alpha, beta, kind == 2 ? 1 : 0};
  dn_set_pending(true);
  if (g_nsums == 4) *err = run_stats();
  return true;
}

// x is the held-back product's target, as it was handed to dot()
static inline bool pend_is(const cudamat* x) {
  return x->on_device && !x->is_trans && x->data_device == g_pend.t.data_device && x->size[0] == g_pend.t.size[0] &&
         x->size[1] == g_pend.t.size[1];
}
static inline bool pend_open() { return g_pend.active && !g_no_defer; }

bool dn_defer_enabled() { return g_defer_enabled && !g_no_defer; }

extern "C" {

// Extension: switches the deferred epilogues on or off (on by default); returns the previous setting.
int set_deferred_epilogues(int on) {
  dn_flush();
  const int before = g_defer_enabled ? 1 : 0;
  g_defer_enabled = on != 0;
  return before;
}

int launch_deferred(void) {
  dn_flush();
  return dn_launch_status();
}

int add_col_vec(cudamat* mat, cudamat* vec, cudamat* target) {
  if (pend_open() && !g_pend.has_bias && !g_pend.has_mul && g_pend.act == 0 && pend_is(mat) && pend_is(target) && vec->on_device &&
      !vec->is_trans && vec->size[0] == mat->size[0] && vec->size[1] == 1 && vec->data_device != mat->data_device) {
    g_pend.bias = *vec;
    g_pend.has_bias = true;
    return 0;
  }
  if (int e = check_colvec(mat, vec, target)) return e;
  return launch_bcast<true>(mat->data_device, vec->data_device, target->data_device, mat->size[0], mat->size[1], FAdd{});
}

int apply_sigmoid(cudamat* mat, cudamat* target) {
  if (pend_open() && g_pend.act == 0 && !g_pend.has_mul && pend_is(mat) && pend_is(target)) {
    g_pend.act = 1;                   // stays held back: a sample of it may follow
    return 0;
  }
  if (int e = check_unary(mat, target)) return e;
  return launch_ew<1>(mat->data_device, nullptr, target->data_device, dn_len(mat), FSigmoid{});
}

int apply_tanh(cudamat* mat, cudamat* target) {
  if (pend_open() && g_pend.act == 0 && !g_pend.has_mul && pend_is(mat) && pend_is(target)) {
    g_pend.act = 3;
    return run_pending(nullptr, nullptr);
  }
  if (int e = check_unary(mat, target)) return e;
  return launch_ew<1>(mat->data_device, nullptr, target->data_device, dn_len(mat), FTanh{});
}

// deriv = dot(w, deriv_above); deriv.apply_rectified_linear_deriv(state): the backward pass of a layer of
// rectified linear units (deepnet/neuralnet.py:203-222, layer.py:168-172) in the product's launch.
int apply_rectified_linear_deriv(cudamat* mat1, cudamat* mat2, cudamat* target) {
  if (pend_open() && g_pend.act == 0 && !g_pend.has_bias && pend_is(mat1) && pend_is(target) && mat2->on_device &&
      !mat2->is_trans && mat2->size[0] == target->size[0] && mat2->size[1] == target->size[1] &&
      !overlap(mat2->data_device, dn_len(mat2), target->data_device, dn_len(target))) {
    g_pend.gate = *mat2;
    g_pend.has_gate = true;
    return run_pending(nullptr, nullptr);
  }
  if (int e = check_binary(mat1, mat2, target)) return e;
  return launch_ew<2>(mat1->data_device, mat2->data_device, target->data_device, dn_len(mat1), FReluDeriv{});
}

int lower_bound_scalar(cudamat* mat, float val, cudamat* target) {
  if (pend_open() && g_pend.act == 0 && !g_pend.has_mul && val == 0.f && !signbit(val) && pend_is(mat) && pend_is(target)) {
    g_pend.act = 2;                   // stays held back: a dropout mask for it may follow
    return 0;
  }
  if (int e = check_unary_trans(mat, target)) return e;
  return launch_ew<1>(mat->data_device, nullptr, target->data_device, dn_len(mat), FLowerS{val});
}

}  // extern "C"


// ---- the parameter update.  deepnet/parameter.py:80-106 spells it
//   w_delta.mult(momentum) [; w_delta.add_mult(w, l2)] [; w_delta.add_mult_sign(w, l1)] ; w_delta.add_mult(gradient)
//   ; w.add_mult(w_delta, -epsilon) [; gradient.assign(0)]
// four to six launches over the same three arrays; k_momentum_update does it in one pass with the same
// roundings.  An in-place mult_by_scalar is held back, the add_mult / add_mult_sign calls into the same
// matrix that follow it are queued, and when the add_mult that reads that matrix arrives and the queue spells
// the update, one launch does it all (an assign_scalar(gradient, 0) that follows directly rides along);
// any other call, or a queue that spells something else, launches the queued calls one by one, in order.
enum { EQ_MULS, EQ_AXPY, EQ_AXPYSIGN };
struct EqOp {
  int kind;
  cudamat dst, src;
  float s;
};
static EqOp g_eq[4];
static int g_eqn = 0;
static bool g_eq_ready = false;       // the queue spells an update; w, -epsilon and the roles are in g_up
static struct {
  cudamat w, g;
  float eps, l2, l1;
  int flags;
} g_up;

static inline bool same_mat(const cudamat* a, const cudamat* b) {
  return a->data_device == b->data_device && a->size[0] == b->size[0] && a->size[1] == b->size[1] &&
         a->is_trans == b->is_trans;
}
static inline bool eq_open() { return g_eqn > 0 && !g_no_defer; }
static int queued_calls() { return g_eqn; }

extern "C" int momentum_update(cudamat* w, cudamat* w_delta, cudamat* gradient, float momentum, float l2_decay,
                               float l1_decay, float epsilon, int flags);

// Updates that are complete wait for each other: deepnet updates all parameters of a net one after the
// other (neuralnet.py:300-312), and up to MOM_MANY of them run as one launch (k_momentum_update_many, the
// arithmetic of the single update).  An update that touches an array of one that waits launches those first.
#define UPD_BATCH 8
struct UpdSpec {
  cudamat w, wd, g;
  float mom, l2, l1, eps;
  int flags;
};
static UpdSpec g_ub[UPD_BATCH];
static int g_ubn = 0;

static bool update_ready() { return g_eqn > 0 && g_eq_ready; }
static int batched_updates() { return g_ubn; }
// anything held back besides complete updates that wait for more of their kind
static bool held_besides_updates() {
  return g_pend.active || g_eqn > 0 || g_acc.active || g_nsums > 0 || g_drop.stage != 0 || dn_softmax_held();
}
static void refresh_pending() { dn_set_pending(held_besides_updates() || g_ubn > 0); }
void dn_refresh_pending() { refresh_pending(); }

extern "C" int momentum_update_many(int count, cudamat** w, cudamat** w_delta, cudamat** gradient, const float* momentum,
                                    const float* l2_decay, const float* l1_decay, const float* epsilon, const int* flags);

static int run_batch() {
  UpdSpec u[UPD_BATCH];
  const int n = g_ubn;
  for (int i = 0; i < n; ++i) u[i] = g_ub[i];
  g_ubn = 0;
  refresh_pending();
  const bool saved = g_no_defer;
  g_no_defer = true;
  int e = 0;
  if (n == 1) {
    e = momentum_update(&u[0].w, &u[0].wd, &u[0].g, u[0].mom, u[0].l2, u[0].l1, u[0].eps, u[0].flags);
  } else if (n > 1) {
    cudamat *w[UPD_BATCH], *wd[UPD_BATCH], *g[UPD_BATCH];
    float mom[UPD_BATCH], l2[UPD_BATCH], l1[UPD_BATCH], eps[UPD_BATCH];
    int flags[UPD_BATCH];
    for (int i = 0; i < n; ++i) {
      w[i] = &u[i].w; wd[i] = &u[i].wd; g[i] = &u[i].g;
      mom[i] = u[i].mom; l2[i] = u[i].l2; l1[i] = u[i].l1; eps[i] = u[i].eps; flags[i] = u[i].flags;
    }
    e = momentum_update_many(n, w, wd, g, mom, l2, l1, eps, flags);
  }
  g_no_defer = saved;
  return e;
}

static inline bool mats_overlap(const cudamat* a, const cudamat* b) {
  return overlap(a->data_device, dn_len(a), b->data_device, dn_len(b));
}

// The queue spells an update and nothing more belongs to it: it joins the updates that wait.
static int stash_ready(bool reset) {
  UpdSpec u;
  u.w = g_up.w; u.wd = g_eq[0].dst; u.g = g_up.g;
  u.mom = g_eq[0].s; u.l2 = g_up.l2; u.l1 = g_up.l1; u.eps = g_up.eps;
  u.flags = g_up.flags | (reset ? 4 : 0);
  g_eqn = 0;
  g_eq_ready = false;
  bool alone = g_ubn == UPD_BATCH;
  for (int i = 0; i < g_ubn && !alone; ++i) {
    const cudamat* mine[3] = {&u.w, &u.wd, &u.g};
    const cudamat* theirs[3] = {&g_ub[i].w, &g_ub[i].wd, &g_ub[i].g};
    for (int a = 0; a < 3; ++a)
      for (int b = 0; b < 3; ++b)
        if (mats_overlap(mine[a], theirs[b])) alone = true;
  }
  int e = 0;
  if (alone) e = run_batch();
  g_ub[g_ubn++] = u;
  dn_set_pending(true);
  return e;
}

// Launches what the queue holds: the one-pass update if it spells one, else its calls one by one.
static int run_queue(bool reset) {
  EqOp q[4];
  const int n = g_eqn;
  for (int i = 0; i < n; ++i) q[i] = g_eq[i];
  const bool ready = g_eq_ready;
  g_eqn = 0;
  g_eq_ready = false;
  refresh_pending();
  const bool saved = g_no_defer;
  g_no_defer = true;
  int e = 0;
  if (ready) {
    e = momentum_update(&g_up.w, &q[0].dst, &g_up.g, q[0].s, g_up.l2, g_up.l1, g_up.eps, g_up.flags | (reset ? 4 : 0));
  } else {
    for (int i = 0; i < n && !e; ++i) {
      if (q[i].kind == EQ_MULS) e = mult_by_scalar(&q[i].dst, q[i].s, &q[i].dst);
      else if (q[i].kind == EQ_AXPY) e = add_mult(&q[i].dst, &q[i].src, q[i].s);
      else e = add_mult_sign(&q[i].dst, &q[i].src, q[i].s);
    }
  }
  g_no_defer = saved;
  return e;
}

// The add_mult that reads the scaled matrix has arrived (w += alpha * w_delta): does the queue spell the update?
static bool queue_spells_update(const cudamat* w, float alpha) {
  const cudamat* wd = &g_eq[0].dst;
  if (same_mat(w, wd) || w->data_device == wd->data_device || !same_dims(w, wd) || w->is_trans != wd->is_trans) return false;
  int i = 1;
  g_up.flags = 0; g_up.l2 = 0.f; g_up.l1 = 0.f;
  if (i < g_eqn - 1 && g_eq[i].kind == EQ_AXPY && same_mat(&g_eq[i].src, w)) { g_up.l2 = g_eq[i].s; g_up.flags |= 1; ++i; }
  if (i < g_eqn - 1 && g_eq[i].kind == EQ_AXPYSIGN && same_mat(&g_eq[i].src, w)) { g_up.l1 = g_eq[i].s; g_up.flags |= 2; ++i; }
  if (i != g_eqn - 1 || g_eq[i].kind != EQ_AXPY || g_eq[i].s != 1.f) return false;
  const cudamat* g = &g_eq[i].src;
  if (g->data_device == w->data_device || g->data_device == wd->data_device) return false;
  g_up.w = *w;
  g_up.g = *g;
  g_up.eps = -alpha;
  return true;
}

extern "C" {

int mult_by_scalar(cudamat* mat, float val, cudamat* target) {
  if (int e = check_unary(mat, target)) return e;
  if (!g_no_defer && g_defer_enabled && mat->data_device == target->data_device && dn_len(mat) > 0) {
    // (a complete update before this one waits on; anything else that is held back is launched now)
    int e = 0;
    if (update_ready()) e = stash_ready(false);
    dn_flush_ext();
    if (held_besides_updates()) dn_flush();
    if (e) return e;
    g_eq[0].kind = EQ_MULS; g_eq[0].dst = *mat; g_eq[0].src = *mat; g_eq[0].s = val;
    g_eqn = 1;
    g_eq_ready = false;
    dn_set_pending(true);
    return 0;
  }
  return launch_ew<1>(mat->data_device, nullptr, target->data_device, dn_len(mat), FMulS{val});
}

int assign_scalar(cudamat* mat, float alpha) {
  if (!mat->on_device) return ERROR_NOT_ON_DEVICE;
  if (eq_open() && g_eq_ready && alpha == 0.f && !signbit(alpha) && same_mat(mat, &g_up.g)) return stash_ready(true);
  return launch_ew<0>(nullptr, nullptr, mat->data_device, dn_len(mat), FAssignS{alpha});
}

// mat1 += alpha * mat2 (cudamat.cu:1763-1781): device, transposedness, dims; no target.
int add_mult(cudamat* mat1, cudamat* mat2, float alpha) {
  if (!mat1->on_device || !mat2->on_device) return ERROR_NOT_ON_DEVICE;
  if (mat1->is_trans != mat2->is_trans) return ERROR_TRANSPOSEDNESS;
  if (!same_dims(mat1, mat2)) return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (eq_open() && !g_eq_ready) {
    if (same_mat(mat1, &g_eq[0].dst) && mat2->data_device != mat1->data_device && g_eqn < 4) {
      g_eq[g_eqn].kind = EQ_AXPY; g_eq[g_eqn].dst = *mat1; g_eq[g_eqn].src = *mat2; g_eq[g_eqn].s = alpha;
      ++g_eqn;
      return 0;
    }
    if (same_mat(mat2, &g_eq[0].dst) && g_eqn >= 2 && queue_spells_update(mat1, alpha)) {
      g_eq_ready = true;          // held back one more call: the gradient's reset may follow
      return 0;
    }
  }
  return launch_ew<2>(mat1->data_device, mat2->data_device, mat1->data_device, dn_len(mat1), FAxpy{alpha});
}

int add_mult_sign(cudamat* mat1, cudamat* mat2, float mult) {
  if (!mat1->on_device || !mat2->on_device) return ERROR_NOT_ON_DEVICE;
  if (mat1->is_trans != mat2->is_trans) return ERROR_TRANSPOSEDNESS;
  if (!same_dims(mat1, mat2)) return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (eq_open() && !g_eq_ready && same_mat(mat1, &g_eq[0].dst) && mat2->data_device != mat1->data_device && g_eqn < 4) {
    g_eq[g_eqn].kind = EQ_AXPYSIGN; g_eq[g_eqn].dst = *mat1; g_eq[g_eqn].src = *mat2; g_eq[g_eqn].s = mult;
    ++g_eqn;
    return 0;
  }
  return launch_ew<2>(mat1->data_device, mat2->data_device, mat1->data_device, dn_len(mat1), FAddMultSign{mult});
}

}  // extern "C"

// sample_bernoulli(rnd, mat, target) right after the held-back product's sigmoid: drawn by the
// product's own launch.  Returns true when it took the call (*err is its result).
bool dn_pending_sample(rnd_struct* rnd, cudamat* mat, cudamat* target, int* err) {
  if (!(pend_open() && g_pend.act == 1 && pend_is(mat))) return false;
  if (!target->on_device || target->is_trans || target->size[0] != mat->size[0] || target->size[1] != mat->size[1] ||
      target->data_device == mat->data_device || !rnd || !rnd->dev_mults || !rnd->dev_words)
    return false;
  *err = run_pending(rnd, target);
  return true;
}


// target = act(op(mat1) * op(mat2) + bias) and, with a generator and a sample matrix,
// sample = (uniform < target), in as few launches as the shapes allow.
// drop: the sample is a dropout mask instead, sample = (uniform > drop_p), and target is multiplied by it.
static int dot_bias_act_impl(rnd_struct* rnd, cudamat* mat1, cudamat* mat2, cudamat* bias, cudamat* target,
                             cudamat* sample, int act, cudamat* gate, bool drop, float drop_p, cudamat* mul) {
  if (!mat1->on_device || !mat2->on_device || !target->on_device || (bias && !bias->on_device)) return ERROR_NOT_ON_DEVICE;
  if (target->is_trans || (bias && bias->is_trans)) return ERROR_TRANSPOSED;
  if (act < 0 || act > 3) return ERROR_UNSUPPORTED;
  if (get_leading_dimension(mat1) != target->size[0] || get_nonleading_dimension(mat2) != target->size[1] ||
      get_nonleading_dimension(mat1) != get_leading_dimension(mat2))
    return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (bias && (bias->size[0] != target->size[0] || bias->size[1] != 1)) return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (sample) {
    if (!rnd || !rnd->dev_mults || !rnd->dev_words) return ERROR_GENERIC;
    if (!sample->on_device) return ERROR_NOT_ON_DEVICE;
    if (sample->is_trans) return ERROR_TRANSPOSED;
    if (sample->size[0] != target->size[0] || sample->size[1] != target->size[1]) return ERROR_INCOMPATIBLE_DIMENSIONS;
    if (sample->data_device == target->data_device) return ERROR_UNSUPPORTED;     // both are written
  }
  const int m = target->size[0], n = target->size[1], k = get_leading_dimension(mat2);
  if (m <= 0 || n <= 0) return 0;
  bool fused = false, sampled = false;
  int err;
  if (n == 1 || k <= 0) {
    err = dot(mat1, mat2, target, 0.f, 1.f);                 // vector-shaped: the streaming kernels
  } else {
    DnGemmSample smp = {nullptr, nullptr, nullptr, nullptr};
    const bool try_sample = sample && rng_pin_if_recording(rnd);
    if (try_sample) smp = DnGemmSample{sample->data_device, rnd->dev_mults, rnd->dev_words, rng_other(rnd->dev_words)};
    err = dn_gemm_fused(mat1->is_trans != 0, mat2->is_trans != 0, m, n, k, mat1->data_device, mat1->size[0],
                        mat2->data_device, mat2->size[0], target->data_device, m, bias ? bias->data_device : nullptr,
                        act, &fused, try_sample ? &smp : nullptr, &sampled, gate ? gate->data_device : nullptr,
                        drop ? 1 : 0, drop_p, mul ? mul->data_device : nullptr);
    if (!err && sampled) rng_publish(rnd);
  }
  if (err) return err;
  if (!fused) {
    if (bias && (err = add_col_vec(target, bias, target))) return err;
    if (act == 1) err = apply_sigmoid(target, target);
    else if (act == 2) err = lower_bound_scalar(target, 0.f, target);
    else if (act == 3) err = apply_tanh(target, target);
    if (err) return err;
    if (mul && (err = mult_elementwise(target, mul, target))) return err;
    if (gate && (err = apply_rectified_linear_deriv(target, gate, target))) return err;
  }
  if (sample && !sampled)
    return drop ? dn_rng_dropmask(rnd, sample->data_device, target->data_device, (size_t)dn_len(target), drop_p)
                : sample_bernoulli(rnd, target, sample);
  return 0;
}

extern "C" {

// Extension (no counterpart in cudamat.cu): target = act(op(mat1) * op(mat2) + bias), the
// sequence dot -> add_col_vec -> apply_sigmoid / lower_bound(0) / apply_tanh that every
// layer of deepnet issues (deepnet/dbm.py:95-105, deepnet/neuralnet.py:138-160), in one
// launch where the product runs as a single kernel, bit-identical to the three calls.
// bias: rows(target) x 1 or null.  act: 0 none, 1 sigmoid, 2 max(x, 0), 3 tanh.
int dot_bias_act(cudamat* mat1, cudamat* mat2, cudamat* bias, cudamat* target, int act) {
  dn_flush();
  const bool saved = g_no_defer;
  g_no_defer = true;
  const int e = dot_bias_act_impl(nullptr, mat1, mat2, bias, target, nullptr, act);
  g_no_defer = saved;
  return e;
}

// Extension: dot_bias_act followed by sample_bernoulli(rnd_state, target, sample), the
// up-pass of an RBM with its hidden sample (deepnet/dbm.py:95-105), bit-identical to the two
// calls (same states, same samples, same generator state afterwards).  One launch where the
// product runs as a single kernel over at most 16 * 12288 outputs; otherwise the separate
// kernels.
int dot_bias_act_sample(rnd_struct* rnd_state, cudamat* mat1, cudamat* mat2, cudamat* bias, cudamat* target,
                        cudamat* sample, int act) {
  if (!sample) return ERROR_GENERIC;
  dn_flush();
  const bool saved = g_no_defer;
  g_no_defer = true;
  const int e = dot_bias_act_impl(rnd_state, mat1, mat2, bias, target, sample, act);
  g_no_defer = saved;
  return e;
}

}  // extern "C"


// ------------------------------------------------------------------ fused parameter update
// The update of deepnet/parameter.py:80-106 in one pass over the parameter:
//   w_delta = momentum*w_delta [+ l2*w] [+ l1*sign(w)] + gradient;  w -= epsilon*w_delta;
//   [gradient = 0]
// Each step rounds as the separate calls do (mult by a scalar: one multiply; add_mult: one
// fused multiply-add; add_mult_sign: one add), so the results are the same bits.
template <bool VEC>
__global__ void __launch_bounds__(EW_THREADS)
k_momentum_update(float* w, float* wd, float* g, long long n, float momentum, float l2, float l1, float eps,
                  int use_l2, int use_l1, int reset) {
  auto one = [&](float wv, float dv, float gv, float& w_out, float& d_out) {
    float d = __fmul_rn(momentum, dv);
    if (use_l2) d = __fmaf_rn(l2, wv, d);
    if (use_l1) d = __fadd_rn(d, (wv > 0.f) ? l1 : ((wv < 0.f) ? -l1 : 0.f));
    d = __fmaf_rn(1.f, gv, d);
    d_out = d;
    w_out = __fmaf_rn(-eps, d, wv);
  };
  const long long tid = (long long)blockIdx.x * EW_THREADS + threadIdx.x;
  if (VEC) {
    if (tid * 4 >= n) return;
    const float4 wv = *reinterpret_cast<const float4*>(w + 4 * tid);
    const float4 dv = *reinterpret_cast<const float4*>(wd + 4 * tid);
    const float4 gv = *reinterpret_cast<const float4*>(g + 4 * tid);
    float4 wo, dox;
    one(wv.x, dv.x, gv.x, wo.x, dox.x);
    one(wv.y, dv.y, gv.y, wo.y, dox.y);
    one(wv.z, dv.z, gv.z, wo.z, dox.z);
    one(wv.w, dv.w, gv.w, wo.w, dox.w);
    *reinterpret_cast<float4*>(wd + 4 * tid) = dox;
    *reinterpret_cast<float4*>(w + 4 * tid) = wo;
    if (reset) *reinterpret_cast<float4*>(g + 4 * tid) = make_float4(0.f, 0.f, 0.f, 0.f);
  } else {
    if (tid >= n) return;
    float wo, dox;
    one(w[tid], wd[tid], g[tid], wo, dox);
    wd[tid] = dox;
    w[tid] = wo;
    if (reset) g[tid] = 0.f;
  }
}

// Extension (no counterpart in cudamat.cu).  Checks as add_mult: device, transposedness, dims.
extern "C" int momentum_update(cudamat* w, cudamat* w_delta, cudamat* gradient, float momentum, float l2_decay,
                               float l1_decay, float epsilon, int flags) {
  if (!w->on_device || !w_delta->on_device || !gradient->on_device) return ERROR_NOT_ON_DEVICE;
  if (w->is_trans != w_delta->is_trans || w->is_trans != gradient->is_trans) return ERROR_TRANSPOSEDNESS;
  if (!same_dims(w, w_delta) || !same_dims(w, gradient)) return ERROR_INCOMPATIBLE_DIMENSIONS;
  const long long n = dn_len(w);
  if (n <= 0) return 0;
  const int use_l2 = flags & 1, use_l1 = (flags >> 1) & 1, reset = (flags >> 2) & 1;
  const bool vec = n % 4 == 0 && dn_aligned16(w->data_device) && dn_aligned16(w_delta->data_device) &&
                   dn_aligned16(gradient->data_device);
  const long long lanes = vec ? n / 4 : n;
  const long long blocks = (lanes + EW_THREADS - 1) / EW_THREADS;
  if (blocks > 0x7fffffffll) return ERROR_UNSUPPORTED;
  if (vec)
    hipLaunchKernelGGL((k_momentum_update<true>), dim3((unsigned)blocks), dim3(EW_THREADS), 0, dn_stream(), w->data_device,
                       w_delta->data_device, gradient->data_device, n, momentum, l2_decay, l1_decay, epsilon, use_l2,
                       use_l1, reset);
  else
    hipLaunchKernelGGL((k_momentum_update<false>), dim3((unsigned)blocks), dim3(EW_THREADS), 0, dn_stream(), w->data_device,
                       w_delta->data_device, gradient->data_device, n, momentum, l2_decay, l1_decay, epsilon, use_l2,
                       use_l1, reset);
  return dn_launch_status();
}

// The same update of up to MOM_MANY parameters in one launch (a net's weights and biases after
// a step): workgroup b works on the parameter whose range of workgroups holds b.  Every
// element goes through the arithmetic of k_momentum_update, so the results are the same bits.
#define MOM_MANY 8
struct MomTable {
  float* w[MOM_MANY];
  float* wd[MOM_MANY];
  float* g[MOM_MANY];
  long long n[MOM_MANY];
  float momentum[MOM_MANY], l2[MOM_MANY], l1[MOM_MANY], eps[MOM_MANY];
  int flags[MOM_MANY];               // bit 0: l2, bit 1: l1, bit 2: reset the gradient, bit 3: 16-byte groups
  unsigned first_block[MOM_MANY + 1];
  int count;
};

__global__ void __launch_bounds__(EW_THREADS) k_momentum_update_many(MomTable t) {
  int k = 0;
  while (k + 1 < t.count && blockIdx.x >= t.first_block[k + 1]) ++k;   // (uniform over the workgroup)
  float* w = t.w[k];
  float* wd = t.wd[k];
  float* g = t.g[k];
  const long long n = t.n[k];
  const float momentum = t.momentum[k], l2 = t.l2[k], l1 = t.l1[k], eps = t.eps[k];
  const int flags = t.flags[k];
  const bool use_l2 = flags & 1, use_l1 = flags & 2, reset = flags & 4;
  auto one = [&](float wv, float dv, float gv, float& w_out, float& d_out) {
    float d = __fmul_rn(momentum, dv);
    if (use_l2) d = __fmaf_rn(l2, wv, d);
    if (use_l1) d = __fadd_rn(d, (wv > 0.f) ? l1 : ((wv < 0.f) ? -l1 : 0.f));
    d = __fmaf_rn(1.f, gv, d);
    d_out = d;
    w_out = __fmaf_rn(-eps, d, wv);
  };
  const long long tid = (long long)(blockIdx.x - t.first_block[k]) * EW_THREADS + threadIdx.x;
  if (flags & 8) {
    if (tid * 4 >= n) return;
    const float4 wv = *reinterpret_cast<const float4*>(w + 4 * tid);
    const float4 dv = *reinterpret_cast<const float4*>(wd + 4 * tid);
    const float4 gv = *reinterpret_cast<const float4*>(g + 4 * tid);
    float4 wo, dox;
    one(wv.x, dv.x, gv.x, wo.x, dox.x);
    one(wv.y, dv.y, gv.y, wo.y, dox.y);
    one(wv.z, dv.z, gv.z, wo.z, dox.z);
    one(wv.w, dv.w, gv.w, wo.w, dox.w);
    *reinterpret_cast<float4*>(wd + 4 * tid) = dox;
    *reinterpret_cast<float4*>(w + 4 * tid) = wo;
    if (reset) *reinterpret_cast<float4*>(g + 4 * tid) = make_float4(0.f, 0.f, 0.f, 0.f);
  } else {
    if (tid >= n) return;
    float wo, dox;
    one(w[tid], wd[tid], g[tid], wo, dox);
    wd[tid] = dox;
    w[tid] = wo;
    if (reset) g[tid] = 0.f;
  }
}

// Extension (no counterpart in cudamat.cu): momentum_update over count parameters, arguments as
// arrays of count entries.  All parameters are checked (as momentum_update checks one) before
// anything is launched; more than MOM_MANY take several launches.
extern "C" int momentum_update_many(int count, cudamat** w, cudamat** w_delta, cudamat** gradient, const float* momentum,
                                    const float* l2_decay, const float* l1_decay, const float* epsilon, const int* flags) {
  if (count < 0) return ERROR_GENERIC;
  for (int i = 0; i < count; ++i) {
    if (!w[i]->on_device || !w_delta[i]->on_device || !gradient[i]->on_device) return ERROR_NOT_ON_DEVICE;
    if (w[i]->is_trans != w_delta[i]->is_trans || w[i]->is_trans != gradient[i]->is_trans) return ERROR_TRANSPOSEDNESS;
    if (!same_dims(w[i], w_delta[i]) || !same_dims(w[i], gradient[i])) return ERROR_INCOMPATIBLE_DIMENSIONS;
    const long long lanes = dn_len(w[i]);
    if ((lanes + EW_THREADS - 1) / EW_THREADS > 0x0fffffffll) return ERROR_UNSUPPORTED;
  }
  for (int i0 = 0; i0 < count; i0 += MOM_MANY) {
    MomTable t;
    t.count = 0;
    unsigned blocks = 0;
    for (int i = i0; i < count && i < i0 + MOM_MANY; ++i) {
      const long long n = dn_len(w[i]);
      if (n <= 0) continue;
      const int k = t.count++;
      const bool vec = n % 4 == 0 && dn_aligned16(w[i]->data_device) && dn_aligned16(w_delta[i]->data_device) &&
                       dn_aligned16(gradient[i]->data_device);
      t.w[k] = w[i]->data_device; t.wd[k] = w_delta[i]->data_device; t.g[k] = gradient[i]->data_device;
      t.n[k] = n;
      t.momentum[k] = momentum[i]; t.l2[k] = l2_decay[i]; t.l1[k] = l1_decay[i]; t.eps[k] = epsilon[i];
      t.flags[k] = (flags[i] & 7) | (vec ? 8 : 0);
      t.first_block[k] = blocks;
      const long long lanes = vec ? n / 4 : n;
      blocks += (unsigned)((lanes + EW_THREADS - 1) / EW_THREADS);
    }
    if (t.count == 0) continue;
    t.first_block[t.count] = blocks;
    hipLaunchKernelGGL(k_momentum_update_many, dim3(blocks), dim3(EW_THREADS), 0, dn_stream(), t);
    if (int e = dn_launch_status()) return e;
  }
  return 0;
}
