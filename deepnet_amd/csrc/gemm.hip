// dot(): target = beta*target + alpha*op(mat1)*op(mat2), fp32, column-major.
// Replaces the cublasSgemm call of cudamat/cudamat.cu:1671-1696.
//
// Matrix-shaped products run on the fp32 matrix cores (v_mfma_f32_32x32x2_f32):
// a 256-lane workgroup owns a (64*WM) x (64*WN) tile of the output, stages
// 16-deep slabs of both operands through LDS (double buffered, next slab
// prefetched into registers while the current one is multiplied) and each of
// its 4 wavefronts accumulates WM x WN blocks of 32 x 32.  Vector-shaped
// products (a single row or column on either side, which is how sum(axis) and
// add_sums arrive) go to the streaming matrix-vector kernels instead.
#include "common.h"

int dn_gemv_cols(const float* M, int ld, int h, int w, const float* x, float* y, float alpha, float beta);
int dn_gemv_rows(const float* M, int ld, int h, int w, const float* x, float* y, float alpha, float beta);

typedef float f32x16 __attribute__((ext_vector_type(16)));

#define GEMM_BK 16
#define GEMM_PAD 4

// Four consecutive floats along the contiguous index c (limit c_lim) at the
// strided index o (limit o_lim); zero outside.  vec_ok: base and ld allow a
// 16-byte load whenever the four are all inside.
__device__ __forceinline__ float4 gemm_load4(const float* base, int c, int c_lim, int o, int o_lim, int ld,
                                             bool vec_ok) {
  float4 r = make_float4(0.f, 0.f, 0.f, 0.f);
  if (o < o_lim) {
    const float* p = base + (size_t)o * ld + c;
    if (vec_ok && c + 3 < c_lim) {
      r = *reinterpret_cast<const float4*>(p);
    } else {
      if (c < c_lim) r.x = p[0];
      if (c + 1 < c_lim) r.y = p[1];
      if (c + 2 < c_lim) r.z = p[2];
      if (c + 3 < c_lim) r.w = p[3];
    }
  }
  return r;
}

// opA(m,k) = A_KC ? A[k + m*lda] : A[m + k*lda];  opB(k,n) = B_KC ? B[k + n*ldb] : B[n + k*ldb].
// gridDim.z > 1 splits K; then each z-slice writes its raw partial tile to
// `partial` (M x N, ld = M, one slab per slice) and a second kernel applies
// alpha/beta.  K slices are multiples of GEMM_BK.
template <int WM, int WN, bool A_KC, bool B_KC>
__global__ void __launch_bounds__(256)
k_gemm(const float* __restrict__ A, int lda, const float* __restrict__ B, int ldb, float* C, int ldc, int M, int N,
       int K, int k_per_split, float alpha, float beta, float* partial, bool a_vec, bool b_vec) {
  constexpr int BM = 64 * WM, BN = 64 * WN;
  constexpr int LA = BM + GEMM_PAD, LB = BN + GEMM_PAD;
  constexpr int A4 = BM * GEMM_BK / 4 / 256, B4 = BN * GEMM_BK / 4 / 256;  // float4 per lane per slab
  __shared__ __attribute__((aligned(16))) float As[2][GEMM_BK][LA];
  __shared__ __attribute__((aligned(16))) float Bs[2][GEMM_BK][LB];

  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int wm = wv & 1, wn = wv >> 1;
  const int m0 = blockIdx.x * BM, n0 = blockIdx.y * BN;
  const int kbeg = blockIdx.z * k_per_split;
  const int kend = (kbeg + k_per_split < K) ? kbeg + k_per_split : K;

  f32x16 acc[WN][WM];
#pragma unroll
  for (int j = 0; j < WN; ++j)
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[j][i][v] = 0.f;

  float4 ra[A4], rb[B4];

  auto fetch = [&](int k0) {
#pragma unroll
    for (int u = 0; u < A4; ++u) {
      const int f = tid + u * 256;
      if (A_KC) {  // k contiguous: 4 lanes cover the 16 k of one m
        const int m = f >> 2, k = (f & 3) << 2;
        ra[u] = gemm_load4(A, k0 + k, kend, m0 + m, M, lda, a_vec);
      } else {     // m contiguous
        const int k = f / (BM / 4), m = (f % (BM / 4)) << 2;
        ra[u] = gemm_load4(A, m0 + m, M, k0 + k, kend, lda, a_vec);
      }
    }
#pragma unroll
    for (int u = 0; u < B4; ++u) {
      const int f = tid + u * 256;
      if (B_KC) {
        const int n = f >> 2, k = (f & 3) << 2;
        rb[u] = gemm_load4(B, k0 + k, kend, n0 + n, N, ldb, b_vec);
      } else {
        const int k = f / (BN / 4), n = (f % (BN / 4)) << 2;
        rb[u] = gemm_load4(B, n0 + n, N, k0 + k, kend, ldb, b_vec);
      }
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int u = 0; u < A4; ++u) {
      const int f = tid + u * 256;
      if (A_KC) {
        const int m = f >> 2, k = (f & 3) << 2;
        As[buf][k][m] = ra[u].x; As[buf][k + 1][m] = ra[u].y;
        As[buf][k + 2][m] = ra[u].z; As[buf][k + 3][m] = ra[u].w;
      } else {
        const int k = f / (BM / 4), m = (f % (BM / 4)) << 2;
        *reinterpret_cast<float4*>(&As[buf][k][m]) = ra[u];
      }
    }
#pragma unroll
    for (int u = 0; u < B4; ++u) {
      const int f = tid + u * 256;
      if (B_KC) {
        const int n = f >> 2, k = (f & 3) << 2;
        Bs[buf][k][n] = rb[u].x; Bs[buf][k + 1][n] = rb[u].y;
        Bs[buf][k + 2][n] = rb[u].z; Bs[buf][k + 3][n] = rb[u].w;
      } else {
        const int k = f / (BN / 4), n = (f % (BN / 4)) << 2;
        *reinterpret_cast<float4*>(&Bs[buf][k][n]) = rb[u];
      }
    }
  };

  const int lk = lane >> 5, li = lane & 31;
  int buf = 0;
  if (kbeg < kend) {
    fetch(kbeg);
    stash(0);
  }
  __syncthreads();
  for (int k0 = kbeg; k0 < kend; k0 += GEMM_BK) {
    const bool more = k0 + GEMM_BK < kend;
    if (more) fetch(k0 + GEMM_BK);
#pragma unroll
    for (int kk = 0; kk < GEMM_BK; kk += 2) {
      float av[WM], bv[WN];
#pragma unroll
      for (int i = 0; i < WM; ++i) av[i] = As[buf][kk + lk][wm * 32 * WM + i * 32 + li];
#pragma unroll
      for (int j = 0; j < WN; ++j) bv[j] = Bs[buf][kk + lk][wn * 32 * WN + j * 32 + li];
#pragma unroll
      for (int j = 0; j < WN; ++j)
#pragma unroll
        for (int i = 0; i < WM; ++i)
          acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x2f32(bv[j], av[i], acc[j][i], 0, 0, 0);
    }
    if (more) stash(buf ^ 1);
    __syncthreads();
    buf ^= 1;
  }

  // acc[j][i][v] holds output (m, n) with m = ... + li and n = ... + 8*(v/4) + 4*lk + v%4.
  const bool split = gridDim.z > 1;
  float* out = split ? partial + (size_t)blockIdx.z * M * N : C;
  const int ldo = split ? M : ldc;
#pragma unroll
  for (int j = 0; j < WN; ++j)
#pragma unroll
    for (int i = 0; i < WM; ++i) {
      const int m = m0 + wm * 32 * WM + i * 32 + li;
      if (m >= M) continue;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int n = n0 + wn * 32 * WN + j * 32 + 8 * (v >> 2) + 4 * lk + (v & 3);
        if (n < N) {
          float* p = out + (size_t)n * ldo + m;
          if (split) *p = acc[j][i][v];
          else *p = (beta == 0.f ? 0.f : beta * *p) + alpha * acc[j][i][v];
        }
      }
    }
}

__global__ void k_gemm_splitk_finish(const float* partial, int splits, float* C, int ldc, int M, int N, float alpha,
                                     float beta) {
  const size_t total = (size_t)M * N;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += stride) {
    float s = 0.f;
    for (int z = 0; z < splits; ++z) s += partial[(size_t)z * total + e];
    const size_t m = e % M, n = e / M;
    float* p = C + n * ldc + m;
    *p = (beta == 0.f ? 0.f : beta * *p) + alpha * s;
  }
}

// C = beta*C where the product is empty (K == 0).
__global__ void k_scale(float* C, int ldc, int M, int N, float beta) {
  const size_t total = (size_t)M * N;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += stride) {
    float* p = C + (e / M) * ldc + (e % M);
    *p = beta == 0.f ? 0.f : beta * *p;
  }
}

template <int WM, int WN>
static void launch_gemm(bool a_kc, bool b_kc, dim3 grid, const float* A, int lda, const float* B, int ldb, float* C,
                        int ldc, int M, int N, int K, int kps, float alpha, float beta, float* partial, bool a_vec,
                        bool b_vec) {
#define GEMM_GO(AK, BK_)                                                                                         \
  hipLaunchKernelGGL((k_gemm<WM, WN, AK, BK_>), grid, dim3(256), 0, 0, A, lda, B, ldb, C, ldc, M, N, K, kps, alpha, \
                     beta, partial, a_vec, b_vec)
  if (a_kc && b_kc) GEMM_GO(true, true);
  else if (a_kc) GEMM_GO(true, false);
  else if (b_kc) GEMM_GO(false, true);
  else GEMM_GO(false, false);
#undef GEMM_GO
}

// Host-side dispatch shared with tests through dot().
static int gemm(bool a_trans, bool b_trans, int M, int N, int K, float alpha, const float* A, int lda, const float* B,
                int ldb, float beta, float* C, int ldc) {
  if (M <= 0 || N <= 0) return 0;
  const int cus = dn_num_cus();
  if (K <= 0) {
    size_t total = (size_t)M * N;
    unsigned blocks = (unsigned)((total + 255) / 256 < (size_t)cus * 8 ? (total + 255) / 256 : (size_t)cus * 8);
    hipLaunchKernelGGL(k_scale, dim3(blocks), dim3(256), 0, 0, C, ldc, M, N, beta);
    return dn_launch_status();
  }
  const bool a_kc = a_trans, b_kc = !b_trans;
  const bool a_vec = dn_aligned16(A) && (lda % 4 == 0);
  const bool b_vec = dn_aligned16(B) && (ldb % 4 == 0);

  // Tile choice: big tiles when they already fill the chip, else 64x64 tiles,
  // and split K when even those leave most CUs idle.
  const long long tiles_big = (long long)((M + 127) / 128) * ((N + 127) / 128);
  const bool big = tiles_big >= cus;
  const int BM = big ? 128 : 64, BN = big ? 128 : 64;
  const int gx = (M + BM - 1) / BM, gy = (N + BN - 1) / BN;
  int splits = 1;
  if (!big) {
    const long long tiles = (long long)gx * gy;
    const int kslabs = (K + GEMM_BK - 1) / GEMM_BK;
    long long want = (2ll * cus + tiles - 1) / tiles;
    if (want > kslabs / 4) want = kslabs / 4;  // at least 4 slabs (64 deep) per slice
    if (want > 32) want = 32;
    if (want > 1) splits = (int)want;
  }
  int kps = ((K + splits - 1) / splits + GEMM_BK - 1) / GEMM_BK * GEMM_BK;
  splits = (K + kps - 1) / kps;
  float* partial = nullptr;
  if (splits > 1) {
    partial = (float*)dn_scratch((size_t)splits * M * N * sizeof(float));
    if (!partial) return CUDA_ERROR;
  }
  dim3 grid(gx, gy, splits);
  if (big) launch_gemm<2, 2>(a_kc, b_kc, grid, A, lda, B, ldb, C, ldc, M, N, K, kps, alpha, beta, partial, a_vec, b_vec);
  else launch_gemm<1, 1>(a_kc, b_kc, grid, A, lda, B, ldb, C, ldc, M, N, K, kps, alpha, beta, partial, a_vec, b_vec);
  if (splits > 1) {
    size_t total = (size_t)M * N;
    unsigned blocks = (unsigned)((total + 255) / 256 < (size_t)cus * 8 ? (total + 255) / 256 : (size_t)cus * 8);
    hipLaunchKernelGGL(k_gemm_splitk_finish, dim3(blocks), dim3(256), 0, 0, partial, splits, C, ldc, M, N, alpha, beta);
  }
  return dn_launch_status();
}

// C = beta*C + alpha*op(A)*op(B) on raw column-major buffers, for the other kernels of the library.
int dn_gemm(bool a_trans, bool b_trans, int M, int N, int K, float alpha, const float* A, int lda, const float* B,
            int ldb, float beta, float* C, int ldc) {
  return gemm(a_trans, b_trans, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc);
}

extern "C" {

int dot(cudamat* mat1, cudamat* mat2, cudamat* target, float beta, float alpha) {
  if (!mat1->on_device || !mat2->on_device || !target->on_device) return ERROR_NOT_ON_DEVICE;
  if (get_leading_dimension(mat1) != get_leading_dimension(target) ||
      get_nonleading_dimension(mat2) != get_nonleading_dimension(target) ||
      get_nonleading_dimension(mat1) != get_leading_dimension(mat2))
    return ERROR_INCOMPATIBLE_DIMENSIONS;
  const int m = get_leading_dimension(mat1), k = get_leading_dimension(mat2), n = get_nonleading_dimension(mat2);
  const float* A = mat1->data_device;
  const float* B = mat2->data_device;
  float* C = target->data_device;
  const int lda = mat1->size[0], ldb = mat2->size[0], ldc = target->size[0];
  const bool ta = mat1->is_trans != 0, tb = mat2->is_trans != 0;
  if (m <= 0 || n <= 0) return 0;
  // The target's own is_trans is ignored and its size[0] is used as the leading
  // dimension; refuse the combinations where that would write past its buffer.
  if ((long long)(n - 1) * ldc + m > dn_len(target)) return ERROR_INCOMPATIBLE_DIMENSIONS;

  // One output column: C(:,0) = op(A) * b with b = op(B)(:,0), k contiguous
  // values of B whichever way it is flagged (a k x 1 or 1 x k array).
  if (n == 1 && k > 0) {
    if (!ta) return dn_gemv_rows(A, lda, m, k, B, C, alpha, beta);  // A is m x k
    return dn_gemv_cols(A, lda, k, m, B, C, alpha, beta);           // A stored k x m
  }
  // One output row with contiguous outputs (ldc == 1): C(0,:) = a^T * op(B),
  // a = the k values of A.
  if (m == 1 && k > 0 && ldc == 1) {
    if (!tb) return dn_gemv_cols(B, ldb, k, n, A, C, alpha, beta);  // B is k x n
    return dn_gemv_rows(B, ldb, n, k, A, C, alpha, beta);           // B stored n x k
  }
  return gemm(ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc);
}

}  // extern "C"
