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
#include "rowsum_jobs.h"
#include "rng.h"
#include "wide_math.h"

int dn_gemv_cols(const float* M, int ld, int h, int w, const float* x, float* y, float alpha, float beta);
int dn_gemv_rows(const float* M, int ld, int h, int w, const float* x, float* y, float alpha, float beta);

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// What dot_bias_act() appends to the product, element by element and in the order of
// the separate calls it replaces (add_col_vec, then the activation), so that the fused
// result is bit-identical to theirs: bias is a column vector over the rows of C or null.
enum { GEMM_ACT_NONE = 0, GEMM_ACT_SIGMOID = 1, GEMM_ACT_RELU = 2, GEMM_ACT_TANH = 3 };
// sample != null (dot_bias_act_sample): the kernels that finish every output in one launch also
// draw sample(i) = uniform_i < C(i) for element i = n * ldc + m of a C without gaps (ldc = M),
// with the uniform that sample_bernoulli would use: draw number i / 12288 of stream i % 12288,
// counted from the words the call starts with.  Those words are only read; the lane that makes
// a stream's last draw writes the stream's new word to `next`, and the host makes `next` the
// generator's current buffer afterwards.
struct GemmEpilogue {
  const float* bias;
  int act;
  float* sample;
  const unsigned int* mults;
  const unsigned long long* words;
  unsigned long long* next;
  unsigned int total;            // M * N
  const float* gate;             // an array laid out as C (or null): outputs are multiplied by (gate > 0 ? 1 : 0)
  int drop;                      // the draws make a dropout mask: sample = (uniform > drop_p), C = C * sample
  float drop_p;
  const float* mul;              // an array laid out as C (or null): outputs are multiplied by it, before the gate
};
#define GEMM_SAMPLE_MAX_DRAWS 16
// (m: the output's row; off: its offset in C)
__device__ __forceinline__ float gemm_finish(float v, int m, size_t off, const GemmEpilogue& e) {
  if (e.bias) v = v + e.bias[m];
  if (e.act == GEMM_ACT_SIGMOID) v = dn_sigmoid(v);
  else if (e.act == GEMM_ACT_RELU) v = v < 0.f ? 0.f : v;
  else if (e.act == GEMM_ACT_TANH) v = dn_tanh(v);
  if (e.mul) v = v * e.mul[off];                            // mult_elementwise's expression
  if (e.gate) v = v * (e.gate[off] > 0.f ? 1.f : 0.f);      // apply_rectified_linear_deriv's expression
  return v;
}
// The generator's word and multiplier for element i, fetched early so that the loads are over
// when the product is.
struct GemmDraw { unsigned long long w; unsigned int mult; };
__device__ __forceinline__ GemmDraw gemm_draw_fetch(unsigned int i, bool ok, const GemmEpilogue& e) {
  GemmDraw d = {0ull, 0u};
  if (e.sample && ok) {
    const unsigned int s = i % NUM_RND_STREAMS;
    d.w = e.words[s];
    d.mult = e.mults[s];
  }
  return d;
}
__device__ __forceinline__ void gemm_draw_store(GemmDraw d, unsigned int i, float p, const GemmEpilogue& e) {
  const unsigned int s = i % NUM_RND_STREAMS, nd = i / NUM_RND_STREAMS;
  unsigned long long w = d.w;
  for (unsigned int k = 0; k <= nd; ++k) w = mwc_step(w, d.mult);
  e.sample[i] = mwc_uniform(w) < p ? 1.f : 0.f;
  if (i + NUM_RND_STREAMS >= e.total) e.next[s] = w;
}
// The same draw as a dropout mask (fill_with_rand -> greater_than(drop_p), deepnet/neuralnet.py:194-198):
// stores and returns (uniform > drop_p ? 1 : 0).
__device__ __forceinline__ float gemm_draw_mask(GemmDraw d, unsigned int i, const GemmEpilogue& e) {
  const unsigned int s = i % NUM_RND_STREAMS, nd = i / NUM_RND_STREAMS;
  unsigned long long w = d.w;
  for (unsigned int k = 0; k <= nd; ++k) w = mwc_step(w, d.mult);
  const float mk = mwc_uniform(w) > e.drop_p ? 1.f : 0.f;
  e.sample[i] = mk;
  if (i + NUM_RND_STREAMS >= e.total) e.next[s] = w;
  return mk;
}
// Streams without a draw (fewer outputs than streams) keep their word: one workgroup copies them.
__device__ __forceinline__ void gemm_draw_idle_streams(int tid, int nthreads, const GemmEpilogue& e) {
  if (e.sample && blockIdx.x == 0 && blockIdx.y == 0)
    for (unsigned int s = e.total + tid; s < NUM_RND_STREAMS; s += nthreads) e.next[s] = e.words[s];
}

struct __attribute__((packed, aligned(4))) gemm_f4u { float x, y, z, w; };   // four floats at any 4-byte boundary

#define GEMM_BK 16
#define GEMM_PAD 4

// Four consecutive floats along the contiguous index c (limit c_lim) at the
// strided index o (limit o_lim); zero outside.  vec_ok: base and ld allow a
// 16-byte load whenever the four are all inside.
__device__ __forceinline__ f32x4 gemm_load4(const float* base, int c, int c_lim, int o, int o_lim, int ld,
                                             bool vec_ok) {
  f32x4 r = {0.f, 0.f, 0.f, 0.f};
  if (o < o_lim) {
    const float* p = base + (size_t)o * ld + c;
    if (vec_ok && c + 3 < c_lim) {
      r = *reinterpret_cast<const f32x4*>(p);
    } else if (c + 3 < c_lim) {
      // a leading dimension or base that is not a multiple of 16 bytes: still one 16-byte
      // request (global memory takes it at 4-byte alignment), not four 4-byte ones
      const gemm_f4u t = *reinterpret_cast<const gemm_f4u*>(p);
      r.x = t.x; r.y = t.y; r.z = t.z; r.w = t.w;
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
// PF (even): the number of register sets that take slabs from global memory in the main loop, where the
// fragments of a slab are read from LDS one iteration ahead of their MFMAs, into a second register set.
template <int WM, int WN, bool A_KC, bool B_KC, int PF = 2>
__global__ void __launch_bounds__(256)
k_gemm(const float* __restrict__ A, int lda, const float* __restrict__ B, int ldb, float* C, int ldc, int M, int N,
       int K, int k_per_split, float alpha, float beta, float* partial, bool a_vec, bool b_vec, GemmEpilogue epi) {
  constexpr int BM = 64 * WM, BN = 64 * WN;
  // Row pitch in LDS: a k-contiguous operand is written transposed, one float per lane
  // (lane = 4 k-quads x rows), which is free of bank conflicts when pitch % 8 == 2; the
  // other kind is written 16 bytes at a time and needs pitch % 4 == 0.
  constexpr int LA = BM + (A_KC ? 2 : GEMM_PAD), LB = BN + (B_KC ? 2 : GEMM_PAD);
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

  f32x4 ra[A4], rb[B4];    // slab on its way from global memory to LDS ...
  f32x4 sa[A4], sb[B4];    // ... and, in the loop for interior tiles, the one after it

  // Tiles that lie wholly inside both operands, on 16-byte aligned data, fetch through
  // per-lane pointers that advance one slab at a time: no index arithmetic and no
  // branch around any load.  Edge tiles and the last partial slab take the checked path.
  // A tile that hangs over the last row or column takes the same path when no 16-byte group
  // straddles the edge (the extent along a contiguous index is a multiple of 4): the rows /
  // columns beyond the edge read a clamped, valid address, and whatever they read only
  // reaches outputs that are never stored.  (One workgroup per CU: the slowest tile is the
  // kernel's time, and the checked path made every 2000 x 2000 x 2000 product wait for its
  // edge tiles, 203 us against 154 us for 2048.)
  // (Global memory takes a 16-byte request at any 4-byte boundary, so operands whose base or leading
  // dimension is not a multiple of 16 bytes run the same loop: 1000 x 1000 x 1001 42 -> 23 us, 3001^3 635 -> 490 us.)
  const bool a_fast = m0 + BM <= M || A_KC || (M % 4 == 0 && M >= 4);
  const bool b_fast = n0 + BN <= N || B_KC || (N % 4 == 0 && N >= 4);
  typedef float f32x4_any __attribute__((ext_vector_type(4), aligned(4)));
  typedef const __attribute__((address_space(1))) f32x4_any* gptr4;   // keeps the loads global_load, never flat
  gptr4 pa[A4];
  gptr4 pb[B4];
#pragma unroll
  for (int u = 0; u < A4; ++u) {
    const int f = tid + u * 256;
    if (A_KC) {
      const int m = m0 + (f >> 2);
      pa[u] = (gptr4)(A + (size_t)(m < M ? m : M - 1) * lda + kbeg + ((f & 3) << 2));
    } else {
      const int m = m0 + ((f % (BM / 4)) << 2);
      pa[u] = (gptr4)(A + (size_t)(kbeg + f / (BM / 4)) * lda + (m + 3 < M ? m : (M >= 4 ? M - 4 : 0)));
    }
  }
#pragma unroll
  for (int u = 0; u < B4; ++u) {
    const int f = tid + u * 256;
    if (B_KC) {
      const int n = n0 + (f >> 2);
      pb[u] = (gptr4)(B + (size_t)(n < N ? n : N - 1) * ldb + kbeg + ((f & 3) << 2));
    } else {
      const int n = n0 + ((f % (BN / 4)) << 2);
      pb[u] = (gptr4)(B + (size_t)(kbeg + f / (BN / 4)) * ldb + (n + 3 < N ? n : (N >= 4 ? N - 4 : 0)));
    }
  }
  // steps in 16-byte units (the fast path has lda, ldb multiples of 4)
  const size_t a_step = A_KC ? GEMM_BK / 4 : (size_t)(GEMM_BK / 4) * lda, b_step = B_KC ? GEMM_BK / 4 : (size_t)(GEMM_BK / 4) * ldb;

  // (macros rather than lambdas taking the register sets by reference: those made the
  // compiler keep the sets in scratch memory)
#define GEMM_FETCH_FAST(XA, XB)                                      \
  do {                                                               \
    _Pragma("unroll") for (int u = 0; u < A4; ++u) {                 \
      XA[u] = *pa[u];                                                \
      pa[u] += a_step;                                               \
    }                                                                \
    _Pragma("unroll") for (int u = 0; u < B4; ++u) {                 \
      XB[u] = *pb[u];                                                \
      pb[u] += b_step;                                               \
    }                                                                \
  } while (0)
  auto fetch_checked = [&](int k0) {
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
#define GEMM_STASH(BUF, XA, XB)                                                     \
  do {                                                                              \
    _Pragma("unroll") for (int u = 0; u < A4; ++u) {                                \
      const int f = tid + u * 256;                                                  \
      if (A_KC) {                                                                   \
        const int m = f >> 2, k = (f & 3) << 2;                                     \
        As[BUF][k][m] = XA[u].x; As[BUF][k + 1][m] = XA[u].y;                       \
        As[BUF][k + 2][m] = XA[u].z; As[BUF][k + 3][m] = XA[u].w;                   \
      } else {                                                                      \
        const int k = f / (BM / 4), m = (f % (BM / 4)) << 2;                        \
        *reinterpret_cast<f32x4*>(&As[BUF][k][m]) = XA[u];                          \
      }                                                                             \
    }                                                                               \
    _Pragma("unroll") for (int u = 0; u < B4; ++u) {                                \
      const int f = tid + u * 256;                                                  \
      if (B_KC) {                                                                   \
        const int n = f >> 2, k = (f & 3) << 2;                                     \
        Bs[BUF][k][n] = XB[u].x; Bs[BUF][k + 1][n] = XB[u].y;                       \
        Bs[BUF][k + 2][n] = XB[u].z; Bs[BUF][k + 3][n] = XB[u].w;                   \
      } else {                                                                      \
        const int k = f / (BN / 4), n = (f % (BN / 4)) << 2;                        \
        *reinterpret_cast<f32x4*>(&Bs[BUF][k][n]) = XB[u];                          \
      }                                                                             \
    }                                                                               \
  } while (0)

  const int lk = lane >> 5, li = lane & 31;
  // One slab: all of its fragments are asked of LDS first (the scheduling fence keeps
  // the compiler from sinking the reads back to their uses), so the MFMAs of one k
  // pair run while the reads of the following pairs are still in flight.
  auto multiply = [&](int buf) {
    float av[GEMM_BK / 2][WM], bv[GEMM_BK / 2][WN];
#pragma unroll
    for (int kk = 0; kk < GEMM_BK / 2; ++kk) {  // rows kk and kk + BK/2: 32 banks apart, no conflict
#pragma unroll
      for (int i = 0; i < WM; ++i) av[kk][i] = As[buf][kk + (GEMM_BK / 2) * lk][wm * 32 * WM + i * 32 + li];
#pragma unroll
      for (int j = 0; j < WN; ++j) bv[kk][j] = Bs[buf][kk + (GEMM_BK / 2) * lk][wn * 32 * WN + j * 32 + li];
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int kk = 0; kk < GEMM_BK / 2; ++kk)
#pragma unroll
      for (int j = 0; j < WN; ++j)
#pragma unroll
        for (int i = 0; i < WM; ++i)
          acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x2f32(bv[kk][j], av[kk][i], acc[j][i], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);  // the wait for the next slab's global loads stays behind the MFMAs
  };

  // Tiles wholly inside both operands run their full slabs through a loop whose loads
  // are unconditional; what is left (edge tiles, the last partial slab) goes through
  // the checked loop.
  const bool fast = a_fast && b_fast;
  int buf = 0, k0 = kbeg;
#define GEMM_FRAGS(BUF, AV, BV)                                                                        \
  do {                                                                                                 \
    _Pragma("unroll") for (int kk = 0; kk < GEMM_BK / 2; ++kk) {                                       \
      _Pragma("unroll") for (int i = 0; i < WM; ++i)                                                   \
        AV[kk][i] = As[BUF][kk + (GEMM_BK / 2) * lk][wm * 32 * WM + i * 32 + li];                      \
      _Pragma("unroll") for (int j = 0; j < WN; ++j)                                                   \
        BV[kk][j] = Bs[BUF][kk + (GEMM_BK / 2) * lk][wn * 32 * WN + j * 32 + li];                      \
    }                                                                                                  \
  } while (0)
#define GEMM_MFMAS(AV, BV)                                                                             \
  do {                                                                                                 \
    _Pragma("unroll") for (int kk = 0; kk < GEMM_BK / 2; ++kk)                                         \
      _Pragma("unroll") for (int j = 0; j < WN; ++j)                                                   \
        _Pragma("unroll") for (int i = 0; i < WM; ++i) {                                               \
          if (TWO_ACC && (kk & 1))                                                                     \
            accb[j][i] = __builtin_amdgcn_mfma_f32_32x32x2f32(BV[kk][j], AV[kk][i], accb[j][i], 0, 0, 0); \
          else                                                                                         \
            acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x2f32(BV[kk][j], AV[kk][i], acc[j][i], 0, 0, 0); \
        }                                                                                              \
  } while (0)
  if (PF && fast && kbeg + (PF + 1) * GEMM_BK <= kend) {
    // fa/fb[c]: fragments of the slab at k0; LDS[buf ^ 1]: the slab after it; ga/gb: the PF - 1 slabs after
    // that, on their way from global memory (a workgroup alone on its CU has nobody to hide that
    // latency behind: the requests run PF + 1 slabs ahead of the MFMAs).  Every fetch asks for a full
    // slab inside [kbeg, kend).
    float fa[2][GEMM_BK / 2][WM], fb[2][GEMM_BK / 2][WN];
    // a wavefront alone on its SIMD issues its MFMAs one after the other: two chains of accumulators, so
    // that an MFMA does not wait for the one before it
    constexpr bool TWO_ACC = WM * WN == 1;
    f32x16 accb[TWO_ACC ? WN : 1][TWO_ACC ? WM : 1];
    if (TWO_ACC) {
#pragma unroll
      for (int v = 0; v < 16; ++v) accb[0][0][v] = 0.f;
    }
    constexpr int NS = PF > 0 ? PF : 1;   // (PF == 0 never runs this branch)
    f32x4 ga[NS][A4], gb[NS][B4];
    // (the first slabs are all asked for before the first wait: one trip to memory in front of the
    // first MFMA instead of three)
    GEMM_FETCH_FAST(ra, rb);
    GEMM_FETCH_FAST(ga[NS - 1], gb[NS - 1]);
#pragma unroll
    for (int q = 0; q < PF - 1; ++q) GEMM_FETCH_FAST(ga[q], gb[q]);
    GEMM_STASH(0, ra, rb);
    __syncthreads();
    GEMM_FRAGS(0, fa[0], fb[0]);
    GEMM_STASH(1, ga[NS - 1], gb[NS - 1]);
    __syncthreads();
    while (k0 + (2 * PF + 1) * GEMM_BK <= kend) {
#pragma unroll
      for (int q = 0; q < PF; ++q) {
        // LDS traffic first, then the MFMAs (the fences keep the compiler from sinking the reads to
        // their uses one phase later, behind a wait): the chain of MFMAs runs while LDS answers
        GEMM_FETCH_FAST(ga[(q + NS - 1) % NS], gb[(q + NS - 1) % NS]);
        GEMM_FRAGS(buf ^ 1, fa[(q + 1) % 2], fb[(q + 1) % 2]);
        GEMM_STASH(buf, ga[q], gb[q]);
        GEMM_MFMAS(fa[q % 2], fb[q % 2]);
        {
          // The order of issue: the global loads, then one LDS read (and, in the second half, one LDS
          // write) in the shadow of every MFMA; left to itself the compiler sinks the reads to their uses
          // one phase later, behind a wait.  (4096 x 4096 x 4096: 1068 -> 933 us, 2048^3: 153 -> 133 us,
          // 1024^3 on one workgroup per CU: 26.6 -> 24 us; four register sets instead of two gain nothing.)
          __builtin_amdgcn_sched_group_barrier(0x020, A4 + B4, 0);
#pragma unroll
          for (int g = 0; g < GEMM_BK / 2 * WM * WN; ++g) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            if (g >= GEMM_BK / 4 * WM * WN) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        buf ^= 1; k0 += GEMM_BK;
      }
    }
#pragma unroll
    for (int q = 0; q < PF - 1; ++q) {
      GEMM_FRAGS(buf ^ 1, fa[(q + 1) % 2], fb[(q + 1) % 2]);
      GEMM_STASH(buf, ga[q], gb[q]);
      __builtin_amdgcn_sched_barrier(0);
      GEMM_MFMAS(fa[q % 2], fb[q % 2]);
      __builtin_amdgcn_sched_barrier(0);
      __syncthreads();
      __builtin_amdgcn_sched_barrier(0);
      buf ^= 1; k0 += GEMM_BK;
    }
    GEMM_MFMAS(fa[(PF - 1) % 2], fb[(PF - 1) % 2]);
    if (TWO_ACC) {
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[0][0][v] += accb[0][0][v];
    }
    buf ^= 1; k0 += GEMM_BK;         // LDS[buf] holds the full slab at k0, nothing is in flight
  } else if (fast && kbeg + 2 * GEMM_BK <= kend) {
    // Global loads run two slabs ahead of the MFMAs: while slab i is multiplied, slab
    // i+1 (asked for one iteration ago) is written to LDS and slab i+2 is requested.
    GEMM_FETCH_FAST(ra, rb);
    GEMM_STASH(0, ra, rb);
    GEMM_FETCH_FAST(ra, rb);
    __syncthreads();
    while (k0 + 4 * GEMM_BK <= kend) {   // two slabs per trip, so the two register sets swap roles statically
      GEMM_FETCH_FAST(sa, sb);
      multiply(buf);
      GEMM_STASH(buf ^ 1, ra, rb);
      __syncthreads();
      buf ^= 1; k0 += GEMM_BK;
      GEMM_FETCH_FAST(ra, rb);
      multiply(buf);
      GEMM_STASH(buf ^ 1, sa, sb);
      __syncthreads();
      buf ^= 1; k0 += GEMM_BK;
    }
    multiply(buf);
    GEMM_STASH(buf ^ 1, ra, rb);
    __syncthreads();
    buf ^= 1; k0 += GEMM_BK;         // LDS now holds the full slab at k0, nothing is in flight
  } else {
    if (kbeg < kend) {
      fetch_checked(kbeg);
      GEMM_STASH(0, ra, rb);
    }
    __syncthreads();
  }
  for (; k0 < kend; k0 += GEMM_BK) {
    const bool more = k0 + GEMM_BK < kend;
    if (more) fetch_checked(k0 + GEMM_BK);
    multiply(buf);
    if (more) GEMM_STASH(buf ^ 1, ra, rb);
    __syncthreads();
    buf ^= 1;
  }

  // acc[j][i][v] holds output (m, n) with m = ... + li and n = ... + 8*(v/4) + 4*lk + v%4.
  const bool split = gridDim.z > 1;
  float* out = split ? partial + (size_t)blockIdx.z * M * N : C;
  const int ldo = split ? M : ldc;
  if (!split && beta != 0.f) {
    // Read-modify-write: the sixteen old values of a block are requested before its first
    // store.  (A load placed after a store to the same array cannot be moved above it, so
    // sixteen load -> store pairs would be sixteen round trips one after the other:
    // 4096 x 4096 x 128 with beta = 1 took 88 us that way, 72 us this way.)
#pragma unroll
    for (int j = 0; j < WN; ++j) {
      const int nb = n0 + wn * 32 * WN + j * 32 + 4 * lk;
      float cold[WM][16];
#pragma unroll
      for (int i = 0; i < WM; ++i) {
        const int m = m0 + wm * 32 * WM + i * 32 + li;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int n = nb + 8 * (v >> 2) + (v & 3);
          cold[i][v] = (m < M && n < N) ? out[(size_t)n * ldo + m] : 0.f;
        }
      }
#pragma unroll
      for (int i = 0; i < WM; ++i) {
        const int m = m0 + wm * 32 * WM + i * 32 + li;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int n = nb + 8 * (v >> 2) + (v & 3);
          if (m < M && n < N) out[(size_t)n * ldo + m] = gemm_finish(beta * cold[i][v] + alpha * acc[j][i][v], m, (size_t)n * ldo + m, epi);
        }
      }
    }
    return;
  }
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
          else *p = gemm_finish(alpha * acc[j][i][v], m, (size_t)n * ldo + m, epi);
        }
      }
    }
}

#undef GEMM_FETCH_FAST
#undef GEMM_STASH
#undef GEMM_FRAGS
#undef GEMM_MFMAS

// Products too small to fill the chip with 64 x 64 tiles (the RBM / MLP layer shapes):
// a workgroup owns one 32 x 32 block of C; its NW wavefronts each take every NW-th
// 32-deep chunk of K, loading their operands straight from global memory in the
// matrix-core operand layout (no LDS staging, nothing to synchronise while
// accumulating, two chunks in flight per wavefront), and add their accumulators up
// through LDS in a fixed order.  One launch, no second kernel.  Within a chunk, lane
// (row i, half h) supplies k0 + 16h + 4u + v to the (4u+v)-th of 16 successive MFMAs:
// any order of the k terms is fine as long as both operands use the same one, and
// this one gives a k-contiguous operand four 16-byte loads per lane that together
// cover whole 128-byte lines.
__device__ __forceinline__ float small_ldg(const float* base, unsigned byte_off) {
  return *reinterpret_cast<const float*>(reinterpret_cast<const char*>(base) + byte_off);
}

// r[q] = op(P)(row, k0 + 16*lk + q) for q < 16, zero where k >= K.  `row` is already
// clamped into the matrix, k0 is wave-uniform, and all offsets fit 32 bits (the
// dispatcher checks), so every load is an SGPR base plus one 32-bit lane offset and
// none of them sits behind a lane-dependent branch.
template <bool KC>
__device__ __forceinline__ void small_load(const float* __restrict__ P, unsigned ld, unsigned row, int k0, int lk, int K,
                                           bool vec, float (&r)[16]) {
  if (k0 >= K) {
#pragma unroll
    for (int q = 0; q < 16; ++q) r[q] = 0.f;
    return;
  }
  const int kl = k0 + 16 * lk;
  if (k0 + 32 <= K) {
    if (KC) {
      const unsigned off = (row * ld + (unsigned)kl) * 4u;
      if (vec) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const float4 t =
              *reinterpret_cast<const float4*>(reinterpret_cast<const char*>(P) + (off + 16u * u));
          r[4 * u] = t.x; r[4 * u + 1] = t.y; r[4 * u + 2] = t.z; r[4 * u + 3] = t.w;
        }
      } else {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const gemm_f4u t = *reinterpret_cast<const gemm_f4u*>(reinterpret_cast<const char*>(P) + (off + 16u * u));
          r[4 * u] = t.x; r[4 * u + 1] = t.y; r[4 * u + 2] = t.z; r[4 * u + 3] = t.w;
        }
      }
    } else {
      const float* pu = P + (size_t)k0 * ld;                 // wave-uniform
      const unsigned off = (16u * lk * ld + row) * 4u;
#pragma unroll
      for (int q = 0; q < 16; ++q) r[q] = small_ldg(pu, off + 4u * q * ld);
    }
  } else {                                                   // the chunk that crosses K
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      const unsigned kk = (unsigned)min(kl + q, K - 1);
      r[q] = small_ldg(P, (KC ? row * ld + kk : kk * ld + row) * 4u);
    }
#pragma unroll
    for (int q = 0; q < 16; ++q) r[q] = kl + q < K ? r[q] : 0.f;
  }
}

// K-contiguous operands, whole chunks, 16-byte aligned: the 32 x 32 chunk is read the
// way it lies in memory (8 lanes per row, 128-byte runs: 8 cache lines per instruction
// instead of 64) and turned into the MFMA layout through a wavefront-private LDS tile.
// r[4u + j] = op(P)(row0 + lane/8 + 8u, k0 + 4*(lane%8) + j); rows past the edge repeat the last one.
// (aligned: rows start on 16-byte boundaries; otherwise the same requests at 4-byte alignment)
__device__ __forceinline__ void small_load_rows(const float* __restrict__ P, unsigned ld, unsigned row0, unsigned last_row,
                                                int k0, int lane, bool aligned, float (&r)[16]) {
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const unsigned row = min(row0 + (unsigned)(lane >> 3) + 8u * u, last_row);
    const unsigned off = (row * ld + (unsigned)k0 + 4u * (lane & 7)) * 4u;
    if (aligned) {
      const float4 t = *reinterpret_cast<const float4*>(reinterpret_cast<const char*>(P) + off);
      r[4 * u] = t.x; r[4 * u + 1] = t.y; r[4 * u + 2] = t.z; r[4 * u + 3] = t.w;
    } else {
      const gemm_f4u t = *reinterpret_cast<const gemm_f4u*>(reinterpret_cast<const char*>(P) + off);
      r[4 * u] = t.x; r[4 * u + 1] = t.y; r[4 * u + 2] = t.z; r[4 * u + 3] = t.w;
    }
  }
}
// In: r as small_load_rows left it.  Out: r[q] = chunk(row lane%32, k = 16*(lane/32) + q).
// The pitch of 33 floats keeps both the writes (4 rows x 8 quads per half wavefront) and
// the reads (32 rows, one column) on 32 different banks.  Only this wavefront touches `tile`.
__device__ __forceinline__ void small_restage(float (*tile)[33], int lane, float (&r)[16]) {
#pragma unroll
  for (int u = 0; u < 4; ++u)
#pragma unroll
    for (int j = 0; j < 4; ++j) tile[(lane >> 3) + 8 * u][4 * (lane & 7) + j] = r[4 * u + j];
  __builtin_amdgcn_wave_barrier();
#pragma unroll
  for (int q = 0; q < 16; ++q) r[q] = tile[lane & 31][16 * (lane >> 5) + q];
  __builtin_amdgcn_wave_barrier();
}

// beta*c + alpha*s as one multiplication and one fused multiply-add, spelled out so that every
// kernel that finishes an output this way rounds alike (beta = 0 ignores c, NaN or not).
__device__ __forceinline__ float small_axpby(float beta, float c, float alpha, float s) {
  return __fmaf_rn(alpha, s, beta == 0.f ? 0.f : __fmul_rn(beta, c));
}

template <bool A_KC, bool B_KC, int NW>
__device__ __forceinline__ void gemm_small_body(const float* __restrict__ A, int lda, const float* __restrict__ B, int ldb, float* C,
                                                int ldc, int M, int N, int K, float alpha, float beta, bool a_vec, bool b_vec,
                                                const GemmEpilogue& epi) {
  constexpr int RED = NW / 2 > 4 ? NW / 2 : 4;
  __shared__ float red[RED][16 * 64];
  constexpr int NSTAGE = (A_KC ? 1 : 0) + (B_KC ? 1 : 0);
  __shared__ float stage[NW][NSTAGE > 0 ? NSTAGE : 1][32][33];  // wavefront-private restaging tiles
  const int tid = threadIdx.x, lane = tid & 63;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);   // tell the compiler it is wave-uniform
  const int li = lane & 31, lk = lane >> 5;
  const int m = blockIdx.x * 32 + li, n = blockIdx.y * 32 + li;
  const bool m_ok = m < M;
  const unsigned mc = min(m, M - 1), nc = min(n, N - 1);    // rows past the edge repeat the last one; never stored

  f32x16 acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.f;
  // beta != 0: the outputs this lane will finish are read now, under the operand loads
  constexpr int EPL = 1024 / (NW * 64);
  float cprev[EPL];
#pragma unroll
  for (int u = 0; u < EPL; ++u) {
    const int v = (tid + u * NW * 64) >> 6;
    const int nn = blockIdx.y * 32 + 8 * (v >> 2) + 4 * lk + (v & 3);
    cprev[u] = (beta != 0.f && m_ok && nn < N) ? C[(size_t)nn * ldc + m] : 0.f;
  }
  // Four chunks per wavefront are requested before the first MFMA (for the RBM / MLP
  // products that is all of a wavefront's share of K, the ragged last chunk included):
  // these kernels live on memory latency, not on throughput.
  constexpr int DEPTH = 4;
  constexpr int STEP = 32 * NW;
  float a[DEPTH][16], b[DEPTH][16];
  int k0 = wv * 32;
  // (a chunk takes the row-wise path when it is K-contiguous and whole)
  auto load_a = [&](int kc, float (&r)[16]) __attribute__((always_inline)) {
    if (A_KC && kc + 32 <= K) small_load_rows(A, lda, blockIdx.x * 32, M - 1, kc, lane, a_vec, r);
    else small_load<A_KC>(A, lda, mc, kc, lk, K, a_vec, r);
  };
  auto load_b = [&](int kc, float (&r)[16]) __attribute__((always_inline)) {
    if (B_KC && kc + 32 <= K) small_load_rows(B, ldb, blockIdx.y * 32, N - 1, kc, lane, b_vec, r);
    else small_load<B_KC>(B, ldb, nc, kc, lk, K, b_vec, r);
  };
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) {
    load_a(k0 + d * STEP, a[d]);
    load_b(k0 + d * STEP, b[d]);
  }
  for (; k0 < K; k0 += DEPTH * STEP) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      if (k0 + d * STEP < K) {                               // wave-uniform
        if (A_KC && k0 + d * STEP + 32 <= K) small_restage(stage[wv][0], lane, a[d]);
        if (B_KC && k0 + d * STEP + 32 <= K) small_restage(stage[wv][NSTAGE - 1], lane, b[d]);
#pragma unroll
        for (int q = 0; q < 16; ++q) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(b[d][q], a[d][q], acc, 0, 0, 0);
        if (k0 + (d + DEPTH) * STEP < K) {                   // refill the set with the chunk DEPTH further on
          load_a(k0 + (d + DEPTH) * STEP, a[d]);
          load_b(k0 + (d + DEPTH) * STEP, b[d]);
        }
      }
    }
  }
  // Halve the number of live accumulators until four are left ...
#pragma unroll
  for (int half = NW / 2; half >= 4; half >>= 1) {
    if (wv >= half && wv < 2 * half) {
#pragma unroll
      for (int v = 0; v < 16; ++v) red[wv - half][v * 64 + lane] = acc[v];
    }
    __syncthreads();
    if (wv < half) {
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[v] += red[wv][v * 64 + lane];
    }
    __syncthreads();
  }
  if (wv < 4) {
#pragma unroll
    for (int v = 0; v < 16; ++v) red[wv][v * 64 + lane] = acc[v];
  }
  __syncthreads();
  // ... and let every lane finish its share of the 1024 outputs: element e = v*64 + lane
  // is C(m, n) with m = tile + lane%32, n = tile + 8*(v/4) + 4*(lane/32) + v%4.
#pragma unroll
  for (int u = 0; u < EPL; ++u) {
    const int e = tid + u * NW * 64;
    const int v = e >> 6;
    const float sum = (red[0][e] + red[1][e]) + (red[2][e] + red[3][e]);
    const int nn = blockIdx.y * 32 + 8 * (v >> 2) + 4 * lk + (v & 3);
    if (m_ok && nn < N) {
      float out = gemm_finish(small_axpby(beta, cprev[u], alpha, sum), m, (size_t)nn * ldc + m, epi);
      const unsigned int i = (unsigned int)nn * ldc + m;
      if (epi.sample && epi.drop) out = out * gemm_draw_mask(gemm_draw_fetch(i, true, epi), i, epi);
      C[(size_t)nn * ldc + m] = out;
      if (epi.sample && !epi.drop) gemm_draw_store(gemm_draw_fetch(i, true, epi), i, out, epi);
    }
  }
  gemm_draw_idle_streams(tid, NW * 64, epi);
}

template <bool A_KC, bool B_KC, int NW>
__global__ void __launch_bounds__(NW * 64)
k_gemm_small(const float* __restrict__ A, int lda, const float* __restrict__ B, int ldb, float* C, int ldc, int M, int N,
             int K, float alpha, float beta, bool a_vec, bool b_vec, GemmEpilogue epi) {
  gemm_small_body<A_KC, B_KC, NW>(A, lda, B, ldb, C, ldc, M, N, K, alpha, beta, a_vec, b_vec, epi);
}

// The four-wavefront form with up to four sums along the rows (rowsum_jobs.h) behind its blocks, as
// k_gemm_tile16_sums below.
template <bool A_KC, bool B_KC>
__global__ void __launch_bounds__(256)
k_gemm_small_sums(const float* __restrict__ A, int lda, const float* __restrict__ B, int ldb, float* C, int ldc, int M, int N,
                  int K, float alpha, float beta, bool a_vec, bool b_vec, GemmEpilogue epi, int gy, RowSumJobs J, int jblocks) {
  if ((int)blockIdx.y < gy) {
    gemm_small_body<A_KC, B_KC, 4>(A, lda, B, ldb, C, ldc, M, N, K, alpha, beta, a_vec, b_vec, epi);
  } else {
    const int b = ((int)blockIdx.y - gy) * (int)gridDim.x + (int)blockIdx.x;
    if (b < jblocks) rows_sum_jobs_body(J, b);
  }
}

// Two products into the same C, one after the other, in one launch:
//   C = beta*C + alpha*op(A)*op(B);  C = C + alpha2*op(A2)*op(B2)
// for reductions of at most 128 terms (one chunk per wavefront and product).  Each product is
// computed, summed over the wavefronts and rounded exactly as k_gemm_small<.., 4> does it alone,
// so the result has the bits of the two launches (the statistics of a contrastive-divergence
// step, W += eps * v h^T; W -= eps * v' h'^T: cudamat/examples/rbm_cudamat.py:73-74, 83-84).
struct GemmPairArgs {
  const float* A; const float* B; const float* A2; const float* B2;
  float* C;
  int lda, ldb, lda2, ldb2, ldc, M, N, K;
  float alpha, beta, alpha2;
  bool a_vec, b_vec, a2_vec, b2_vec;
};

// block (bx, by) of the pair: the 32 x 32 outputs at (32 bx, 32 by)
template <bool A_KC, bool B_KC>
__device__ __forceinline__ void gemm_small_pair_body(const GemmPairArgs& g, int bx, int by) {
  const float* __restrict__ A = g.A; const float* __restrict__ B = g.B;
  const float* __restrict__ A2 = g.A2; const float* __restrict__ B2 = g.B2;
  float* C = g.C;
  const int lda = g.lda, ldb = g.ldb, lda2 = g.lda2, ldb2 = g.ldb2, ldc = g.ldc, M = g.M, N = g.N, K = g.K;
  const float alpha = g.alpha, beta = g.beta, alpha2 = g.alpha2;
  const bool a_vec = g.a_vec, b_vec = g.b_vec, a2_vec = g.a2_vec, b2_vec = g.b2_vec;
  constexpr int NW = 4;
  __shared__ float red[2][NW][16 * 64];
  constexpr int NSTAGE = (A_KC ? 1 : 0) + (B_KC ? 1 : 0);
  __shared__ float stage[NW][NSTAGE > 0 ? NSTAGE : 1][32][33];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int li = lane & 31, lk = lane >> 5;
  const int m = bx * 32 + li, n = by * 32 + li;
  const bool m_ok = m < M;
  const unsigned mc = min(m, M - 1), nc = min(n, N - 1);
  constexpr int EPL = 1024 / (NW * 64);
  float cprev[EPL];
#pragma unroll
  for (int u = 0; u < EPL; ++u) {
    const int v = (tid + u * NW * 64) >> 6;
    const int nn = by * 32 + 8 * (v >> 2) + 4 * lk + (v & 3);
    cprev[u] = (beta != 0.f && m_ok && nn < N) ? C[(size_t)nn * ldc + m] : 0.f;
  }
  const int k0 = wv * 32;
  float a[2][16], b[2][16];
  // (the same requests as k_gemm_small: row-wise for a whole chunk of a K-contiguous operand)
  auto load = [&](const float* __restrict__ Pa, int la, bool va, const float* __restrict__ Pb, int lb, bool vb, float (&ra)[16],
                  float (&rb)[16]) __attribute__((always_inline)) {
    if (A_KC && k0 + 32 <= K) small_load_rows(Pa, la, bx * 32, M - 1, k0, lane, va, ra);
    else small_load<A_KC>(Pa, la, mc, k0, lk, K, va, ra);
    if (B_KC && k0 + 32 <= K) small_load_rows(Pb, lb, by * 32, N - 1, k0, lane, vb, rb);
    else small_load<B_KC>(Pb, lb, nc, k0, lk, K, vb, rb);
  };
  load(A, lda, a_vec, B, ldb, b_vec, a[0], b[0]);
  load(A2, lda2, a2_vec, B2, ldb2, b2_vec, a[1], b[1]);
#pragma unroll
  for (int pr = 0; pr < 2; ++pr) {
    f32x16 acc;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = 0.f;
    if (k0 < K) {                                             // wave-uniform
      if (A_KC && k0 + 32 <= K) small_restage(stage[wv][0], lane, a[pr]);
      if (B_KC && k0 + 32 <= K) small_restage(stage[wv][NSTAGE - 1], lane, b[pr]);
#pragma unroll
      for (int q = 0; q < 16; ++q) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(b[pr][q], a[pr][q], acc, 0, 0, 0);
    }
#pragma unroll
    for (int v = 0; v < 16; ++v) red[pr][wv][v * 64 + lane] = acc[v];
  }
  __syncthreads();
#pragma unroll
  for (int u = 0; u < EPL; ++u) {
    const int e = tid + u * NW * 64;
    const int v = e >> 6;
    const float sum1 = (red[0][0][e] + red[0][1][e]) + (red[0][2][e] + red[0][3][e]);
    const float sum2 = (red[1][0][e] + red[1][1][e]) + (red[1][2][e] + red[1][3][e]);
    const int nn = by * 32 + 8 * (v >> 2) + 4 * lk + (v & 3);
    if (m_ok && nn < N) C[(size_t)nn * ldc + m] = small_axpby(1.f, small_axpby(beta, cprev[u], alpha, sum1), alpha2, sum2);
  }
}

template <bool A_KC, bool B_KC>
__global__ void __launch_bounds__(256) k_gemm_small_pair(GemmPairArgs g) {
  gemm_small_pair_body<A_KC, B_KC>(g, (int)blockIdx.x, (int)blockIdx.y);
}

// The pair and up to four sums along the rows (rowsum_jobs.h) in one launch: the first gx * gy
// workgroups are the blocks of the products, the rest the row blocks of the sums (the statistics of
// a contrastive-divergence step: weights and both biases, cudamat/examples/rbm_cudamat.py:73-86).
// Every workgroup runs the code it would run in the separate kernels.
template <bool A_KC, bool B_KC>
__global__ void __launch_bounds__(256) k_gemm_small_pair_sums(GemmPairArgs g, int gx, int nprod, RowSumJobs J) {
  const int b = (int)blockIdx.x;
  if (b < nprod) gemm_small_pair_body<A_KC, B_KC>(g, b % gx, b / gx);
  else rows_sum_jobs_body(J, b - nprod);
}

// The same single-launch scheme on 16 x 16 output blocks (v_mfma_f32_16x16x4_f32), for products
// whose 32 x 32 blocks would occupy less than two fifths of the CUs (the products of the RBM
// configuration with 500 x 100 and 784 x 100 outputs): four times the workgroups, so
// the matrix-core time of a block (K/32 chunks of 8 instructions) spreads over the whole chip.
// Lane (i, kq) of a wavefront holds, for chunk c, row i of an operand at k = 32c + 8kq + j,
// j < 8: two 16-byte loads when the operand is K-contiguous, 64-byte runs per 16 lanes when
// it is not; step j of a chunk multiplies the four k values {8kq + j}.  The NW wavefronts take
// every NW-th chunk, four in flight each, and add up through LDS in wavefront order.
typedef float f32x4m __attribute__((ext_vector_type(4)));

// One whole chunk, without lane-dependent conditions: the loads of a wavefront's first four chunks
// are all in flight before its first multiplication (16-byte requests are taken at 4-byte alignment).
template <bool KC>
__device__ __forceinline__ void tile16_load(const float* __restrict__ P, unsigned ld, unsigned row, int chunk, int kq,
                                            float (&r)[8]) {
  const unsigned kl = 32u * (unsigned)chunk + 8u * (unsigned)kq;
  if (KC) {
    const char* base = reinterpret_cast<const char*>(P) + ((size_t)row * ld + kl) * 4u;
    const gemm_f4u t0 = *reinterpret_cast<const gemm_f4u*>(base), t1 = *reinterpret_cast<const gemm_f4u*>(base + 16);
    r[0] = t0.x; r[1] = t0.y; r[2] = t0.z; r[3] = t0.w; r[4] = t1.x; r[5] = t1.y; r[6] = t1.z; r[7] = t1.w;
  } else {
    const float* pu = P + (size_t)kl * ld + row;
#pragma unroll
    for (int j = 0; j < 8; ++j) r[j] = pu[(size_t)j * ld];
  }
}
// The chunk that crosses K: element by element, zero beyond K.
template <bool KC>
__device__ __forceinline__ void tile16_load_tail(const float* __restrict__ P, unsigned ld, unsigned row, int chunk, int kq,
                                                 int K, float (&r)[8]) {
  const int kl = 32 * chunk + 8 * kq;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const unsigned kk = (unsigned)min(kl + j, K - 1);
    r[j] = KC ? P[(size_t)row * ld + kk] : P[(size_t)kk * ld + row];
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) r[j] = kl + j < K ? r[j] : 0.f;
}

template <bool A_KC, bool B_KC, int NW>
__device__ __forceinline__ void gemm_tile16_body(const float* __restrict__ A, int lda, const float* __restrict__ B, int ldb, float* C,
                                                 int ldc, int M, int N, int K, float alpha, float beta, const GemmEpilogue& epi) {
  __shared__ float red[NW][4 * 64];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int li = lane & 15, kq = lane >> 4;
  const int m0 = blockIdx.x * 16, n0 = blockIdx.y * 16;
  const unsigned mc = min(m0 + li, M - 1), nc = min(n0 + li, N - 1);   // rows past the edge repeat the last one; never stored
  // the output this lane finishes after the wavefronts have met: element e = tid (NW * 64 >= 256)
  const int ev = tid >> 6;                                   // accumulator register v of element e
  const int em = m0 + li, en = n0 + 4 * kq + ev;
  const bool e_ok = tid < 256 && em < M && en < N;
  const float cprev = (beta != 0.f && e_ok) ? C[(size_t)en * ldc + em] : 0.f;
  const unsigned int ei = (unsigned int)en * ldc + em;
  const GemmDraw draw = gemm_draw_fetch(ei, e_ok, epi);

  constexpr int DEPTH = 4;
  const int nfull = K >> 5;                                  // whole chunks; wavefront wv takes wv, wv + NW, ...
  f32x4m acc = {0.f, 0.f, 0.f, 0.f};
  if (nfull > 0) {
    float a[DEPTH][8], b[DEPTH][8];
    int c = wv;
    // Only chunks that exist are asked for (the conditions are wave-uniform): a set that re-read
    // the last chunk instead made every wavefront of the chip hit the same few lines at once,
    // which cost 1 us of the 4.8 us of a 500 x 100 x 784 product.
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      if (c + d * NW < nfull) {
        tile16_load<A_KC>(A, lda, mc, c + d * NW, kq, a[d]);
        tile16_load<B_KC>(B, ldb, nc, c + d * NW, kq, b[d]);
      }
    }
    for (; c < nfull; c += DEPTH * NW) {
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        if (c + d * NW < nfull) {
#pragma unroll
          for (int j = 0; j < 8; ++j) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(b[d][j], a[d][j], acc, 0, 0, 0);
        }
        if (c + (d + DEPTH) * NW < nfull) {
          tile16_load<A_KC>(A, lda, mc, c + (d + DEPTH) * NW, kq, a[d]);
          tile16_load<B_KC>(B, ldb, nc, c + (d + DEPTH) * NW, kq, b[d]);
        }
      }
    }
  }
  if ((K & 31) && wv == nfull % NW) {                        // the ragged end of K, once
    float ta[8], tb[8];
    tile16_load_tail<A_KC>(A, lda, mc, nfull, kq, K, ta);
    tile16_load_tail<B_KC>(B, ldb, nc, nfull, kq, K, tb);
#pragma unroll
    for (int j = 0; j < 8; ++j) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(tb[j], ta[j], acc, 0, 0, 0);
  }
  // acc[v] of lane (i, kq) is C(m0 + i, n0 + 4*kq + v)
#pragma unroll
  for (int v = 0; v < 4; ++v) red[wv][v * 64 + lane] = acc[v];
  __syncthreads();
  if (e_ok) {
    float sum = red[0][tid];
#pragma unroll
    for (int w = 1; w < NW; ++w) sum += red[w][tid];
    float out = gemm_finish((beta == 0.f ? 0.f : beta * cprev) + alpha * sum, em, (size_t)en * ldc + em, epi);
    if (epi.sample && epi.drop) out = out * gemm_draw_mask(draw, ei, epi);
    C[(size_t)en * ldc + em] = out;
    if (epi.sample && !epi.drop) gemm_draw_store(draw, ei, out, epi);
  }
  gemm_draw_idle_streams(tid, NW * 64, epi);
}

template <bool A_KC, bool B_KC, int NW>
__global__ void __launch_bounds__(NW * 64)
k_gemm_tile16(const float* __restrict__ A, int lda, const float* __restrict__ B, int ldb, float* C, int ldc, int M, int N,
              int K, float alpha, float beta, GemmEpilogue epi) {
  gemm_tile16_body<A_KC, B_KC, NW>(A, lda, B, ldb, C, ldc, M, N, K, alpha, beta, epi);
}

// A product and up to four sums along the rows (rowsum_jobs.h) in one launch: the rows of the grid
// below gy are the blocks of the product, the workgroups behind them the row blocks of the sums
// (a weight gradient and the bias gradient of the same layer: deepnet/edge.py:236-242,
// layer.py:206-211).  Every workgroup runs the code it would run in the separate kernels.
template <bool A_KC, bool B_KC, int NW>
__global__ void __launch_bounds__(NW * 64)
k_gemm_tile16_sums(const float* __restrict__ A, int lda, const float* __restrict__ B, int ldb, float* C, int ldc, int M, int N,
                   int K, float alpha, float beta, GemmEpilogue epi, int gy, RowSumJobs J, int jblocks) {
  if ((int)blockIdx.y < gy) {
    gemm_tile16_body<A_KC, B_KC, NW>(A, lda, B, ldb, C, ldc, M, N, K, alpha, beta, epi);
  } else {
    const int b = ((int)blockIdx.y - gy) * (int)gridDim.x + (int)blockIdx.x;
    if (b < jblocks) rows_sum_jobs_body(J, b);
  }
}

// Short reductions (K <= 128) on 64 x 64 tiles: the whole K extent of a tile's two operands is
// asked for at once (two 16-byte loads per lane and operand), written to LDS once and multiplied
// without another wait.  The slab loop of k_gemm spends such a product waiting for one global
// round trip after the other (its tiles have two slabs in flight; 128 deep is eight slabs).
// Sixteen wavefronts: (2 x 2) blocks of 32 x 32 outputs times four interleaved quarters of K,
// so a tile's matrix-core time is 16 instructions per wavefront; the quarters are added up
// through LDS (in the space of the operands) in a fixed order, every lane finishing four outputs.
// LDS layouts: a K-contiguous operand is kept [row][k] (pitch 132: 16-byte writes and 16-byte
// fragment reads, both free of bank conflicts), the other kind [k][row] (pitch 68).  Step t
// of the multiplication takes k = 8t + 4 (lane / 32) + j, j < 4, from both.
#define BOX_K 128
#define BOX_PITCH_KC 132
#define BOX_PITCH_MC 68
#define BOX_THREADS 1024
#define BOX_KW 4
// One operand's 64 x 128 block into registers; zero where k >= kn.  fast: every 16-byte group
// is either whole or unused (see the host side); otherwise element by element with clamped
// indices.  Rows beyond the matrix repeat valid ones and only reach outputs that are not stored.
template <bool KC>
__device__ __forceinline__ void box_fetch(const float* __restrict__ P, int ld, int row0, int rows, int kn, int tid, bool fast,
                                          gemm_f4u (&r)[2]) {
  if (fast) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int f = tid + u * BOX_THREADS;
      if (KC) {
        const int rr = min(row0 + (f >> 5), rows - 1), kq = (f & 31) << 2;
        r[u] = *reinterpret_cast<const gemm_f4u*>(P + (size_t)rr * ld + (kq < kn ? kq : 0));
        if (kq >= kn) r[u] = gemm_f4u{0.f, 0.f, 0.f, 0.f};
      } else {
        const int k = f >> 4, mq = min(row0 + ((f & 15) << 2), rows - 4);
        r[u] = *reinterpret_cast<const gemm_f4u*>(P + (size_t)(k < kn ? k : 0) * ld + mq);
        if (k >= kn) r[u] = gemm_f4u{0.f, 0.f, 0.f, 0.f};
      }
    }
  } else {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int f = tid + u * BOX_THREADS;
      float v[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        int rr, k;
        if (KC) { rr = row0 + (f >> 5); k = ((f & 31) << 2) + j; }
        else { k = f >> 4; rr = row0 + ((f & 15) << 2) + j; }
        const int rc = min(rr, rows - 1), kc = min(k, kn - 1);
        const float x = KC ? P[(size_t)rc * ld + kc] : P[(size_t)kc * ld + rc];
        v[j] = k < kn ? x : 0.f;
      }
      r[u] = gemm_f4u{v[0], v[1], v[2], v[3]};
    }
  }
}
template <bool KC>
__device__ __forceinline__ void box_stash(float* S, int tid, const gemm_f4u (&r)[2]) {
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int f = tid + u * BOX_THREADS;
    if (KC) *reinterpret_cast<gemm_f4u*>(S + (f >> 5) * BOX_PITCH_KC + ((f & 31) << 2)) = r[u];
    else *reinterpret_cast<gemm_f4u*>(S + (f >> 4) * BOX_PITCH_MC + ((f & 15) << 2)) = r[u];
  }
}
template <bool KC>
__device__ __forceinline__ void box_frag(const float* S, int row, int lk, int t, float (&v)[4]) {
  if (KC) {
    const gemm_f4u x = *reinterpret_cast<const gemm_f4u*>(S + row * BOX_PITCH_KC + 8 * t + 4 * lk);
    v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = S[(8 * t + 4 * lk + j) * BOX_PITCH_MC + row];
  }
}
template <bool A_KC, bool B_KC>
__device__ __forceinline__ void gemm_box_body(const float* __restrict__ A, int lda, const float* __restrict__ B, int ldb, float* C,
                                              int ldc, int M, int N, int K, float alpha, float beta, bool a_fast, bool b_fast,
                                              const GemmEpilogue& epi) {
  constexpr int A_FLOATS = A_KC ? 64 * BOX_PITCH_KC : BOX_K * BOX_PITCH_MC;
  constexpr int B_FLOATS = B_KC ? 64 * BOX_PITCH_KC : BOX_K * BOX_PITCH_MC;
  static_assert(A_FLOATS + B_FLOATS >= BOX_KW * 4096, "the partial tiles reuse the operands' space");
  __shared__ __attribute__((aligned(16))) float lds[A_FLOATS + B_FLOATS];
  float* As = lds;
  float* Bs = lds + A_FLOATS;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wv & 1, wn = (wv >> 1) & 1, wk = wv >> 2, li = lane & 31, lk = lane >> 5;
  const int m0 = blockIdx.x * 64, n0 = blockIdx.y * 64;
  gemm_f4u ra[2], rb[2];
  box_fetch<A_KC>(A, lda, m0, M, K, tid, a_fast, ra);
  box_fetch<B_KC>(B, ldb, n0, N, K, tid, b_fast, rb);
  // the four outputs this lane finishes: e = tid + 1024 u is C(m0 + e % 64, n0 + e / 64)
  const int em = m0 + (tid & 63);
  float cold[4];
  if (beta != 0.f) {    // asked for under the operand loads
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int en = n0 + (tid >> 6) + 16 * u;
      cold[u] = (em < M && en < N) ? C[(size_t)en * ldc + em] : 0.f;
    }
  }
  box_stash<A_KC>(As, tid, ra);
  box_stash<B_KC>(Bs, tid, rb);
  __syncthreads();
  f32x16 acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.f;
  const int steps = (K + 7) >> 3;
  for (int t = wk; t < steps; t += BOX_KW) {
    float a[4], b[4];
    box_frag<A_KC>(As, wm * 32 + li, lk, t, a);
    box_frag<B_KC>(Bs, wn * 32 + li, lk, t, b);
#pragma unroll
    for (int j = 0; j < 4; ++j) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(b[j], a[j], acc, 0, 0, 0);
  }
  __syncthreads();                      // every wavefront is done with the operands
  // acc[v] is the tile's (m, n) = (32 wm + li, 32 wn + 8 (v / 4) + 4 lk + v % 4); partial tiles are [n][m]
  float* part = lds + wk * 4096;
#pragma unroll
  for (int v = 0; v < 16; ++v) part[(wn * 32 + 8 * (v >> 2) + 4 * lk + (v & 3)) * 64 + wm * 32 + li] = acc[v];
  __syncthreads();
  if (em >= M) return;
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int e = tid + BOX_THREADS * u;
    const int en = n0 + (tid >> 6) + 16 * u;
    const float sum = (lds[e] + lds[4096 + e]) + (lds[8192 + e] + lds[12288 + e]);
    if (en < N) C[(size_t)en * ldc + em] = gemm_finish((beta != 0.f ? beta * cold[u] : 0.f) + alpha * sum, em, (size_t)en * ldc + em, epi);
  }
}

template <bool A_KC, bool B_KC>
__global__ void __launch_bounds__(BOX_THREADS)
k_gemm_box(const float* __restrict__ A, int lda, const float* __restrict__ B, int ldb, float* C, int ldc, int M, int N, int K,
           float alpha, float beta, bool a_fast, bool b_fast, GemmEpilogue epi) {
  gemm_box_body<A_KC, B_KC>(A, lda, B, ldb, C, ldc, M, N, K, alpha, beta, a_fast, b_fast, epi);
}

// ... and beside the 1024-lane blocks of this kernel (the sums use the first 256 lanes of theirs)
template <bool A_KC, bool B_KC>
__global__ void __launch_bounds__(BOX_THREADS)
k_gemm_box_sums(const float* __restrict__ A, int lda, const float* __restrict__ B, int ldb, float* C, int ldc, int M, int N, int K,
                float alpha, float beta, bool a_fast, bool b_fast, GemmEpilogue epi, int gy, RowSumJobs J, int jblocks) {
  if ((int)blockIdx.y < gy) {
    gemm_box_body<A_KC, B_KC>(A, lda, B, ldb, C, ldc, M, N, K, alpha, beta, a_fast, b_fast, epi);
  } else {
    const int b = ((int)blockIdx.y - gy) * (int)gridDim.x + (int)blockIdx.x;
    if (b < jblocks) rows_sum_jobs_body(J, b);
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

// The same, four rows at a time (M and ldc multiples of 4, C on a 16-byte boundary): the sums and the
// expression per element are those of the kernel above.
__global__ void __launch_bounds__(256)
k_gemm_splitk_finish4(const float* partial, int splits, float* C, int ldc, int M, int N, float alpha, float beta) {
  const size_t total4 = (size_t)M * N / 4;
  const size_t e4 = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (e4 >= total4) return;
  const f32x4* p4 = reinterpret_cast<const f32x4*>(partial) + e4;
  f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
  for (int z = 0; z < splits; ++z) s += p4[(size_t)z * total4];
  const size_t e = e4 * 4, m = e % M, n = e / M;
  f32x4* c = reinterpret_cast<f32x4*>(C + n * ldc + m);
  f32x4 o;
  if (beta == 0.f) {
#pragma unroll
    for (int v = 0; v < 4; ++v) o[v] = 0.f + alpha * s[v];
  } else {
    const f32x4 old = *c;
#pragma unroll
    for (int v = 0; v < 4; ++v) o[v] = beta * old[v] + alpha * s[v];
  }
  *c = o;
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
                        bool b_vec, GemmEpilogue epi) {
#define GEMM_GO(AK, BK_)                                                                                         \
  hipLaunchKernelGGL((k_gemm<WM, WN, AK, BK_>), grid, dim3(256), 0, dn_stream(), A, lda, B, ldb, C, ldc, M, N, K, kps, alpha, \
                     beta, partial, a_vec, b_vec, epi)
  if (a_kc && b_kc) GEMM_GO(true, true);
  else if (a_kc) GEMM_GO(true, false);
  else if (b_kc) GEMM_GO(false, true);
  else GEMM_GO(false, false);
#undef GEMM_GO
}

// Host-side dispatch shared with tests through dot().
// epi: what to append to each output (bias / activation); *fused tells the caller whether
// the launch could carry it (the split-K and empty-K paths cannot).
// Sums along the rows that the next product may take along in its launch (dn_gemm_sums sets them;
// the launch site that does so clears the count).
static const RowSumJobs* g_side_jobs = nullptr;
static int g_side_blocks = 0;
static inline bool side_jobs_fit(const GemmEpilogue& epi) {
  return g_side_blocks > 0 && g_side_jobs && !epi.bias && epi.act == GEMM_ACT_NONE && !epi.sample && !epi.gate && !epi.mul;
}

static int gemm(bool a_trans, bool b_trans, int M, int N, int K, float alpha, const float* A, int lda, const float* B,
                int ldb, float beta, float* C, int ldc, GemmEpilogue epi = GemmEpilogue{nullptr, GEMM_ACT_NONE, nullptr, nullptr, nullptr, nullptr, 0u, nullptr, 0, 0.f, nullptr},
                bool* fused = nullptr, bool* sampled = nullptr) {
  if (fused) *fused = false;
  if (sampled) *sampled = false;
  if (M <= 0 || N <= 0) return 0;
  const int cus = dn_num_cus();
  if (K <= 0) {
    size_t total = (size_t)M * N;
    unsigned blocks = (unsigned)((total + 255) / 256 < (size_t)cus * 8 ? (total + 255) / 256 : (size_t)cus * 8);
    hipLaunchKernelGGL(k_scale, dim3(blocks), dim3(256), 0, dn_stream(), C, ldc, M, N, beta);
    return dn_launch_status();
  }
  const bool a_kc = a_trans, b_kc = !b_trans;
  const bool a_vec = dn_aligned16(A) && (lda % 4 == 0);
  const bool b_vec = dn_aligned16(B) && (ldb % 4 == 0);

  // Tile choice: big tiles when they already fill the chip, else 64x64 tiles; when
  // even those cannot fill it, the 32x32-per-workgroup kernel that splits K over
  // its own wavefronts.
  const long long tiles64 = (long long)((M + 63) / 64) * ((N + 63) / 64);
  const bool off32 = (size_t)lda * (a_kc ? M : K) < (1u << 30) && (size_t)ldb * (b_kc ? N : K) < (1u << 30);
  // The kernels that split K over the wavefronts of a workgroup read their operands straight from L2
  // and L1, and a CU's time goes with what it pulls through: per 1024 of K about 4 us while the
  // 16 x 16 blocks fit one round of the CUs, 6.2 us up to one 32 x 32 block per CU (or a second round
  // of 16 x 16 blocks), 15.5 us up to two.  LDS tiles with a split K cost about 12 us plus 1.5 us per
  // 1e8 multiply-adds, second kernel included, and take over where that is less (measured, us:
  // 4096 x 128 x 4096 66 -> 53, 1024 x 128 x 8192 45 -> 29, 3000 x 128 x 3000 44 -> 36, 1024 x 128 x 4096
  // 24.1 -> 19.5; they stay behind on 2048 x 128 x 2048, 15.1 against 20.3, and 4096 x 128 x 1024,
  // 17.2 against 19.2).
  const long long tiles32 = (long long)((M + 31) / 32) * ((N + 31) / 32);
  const long long tiles16 = (long long)((M + 15) / 16) * ((N + 15) / 16);
  const double per_1024 = tiles16 <= cus ? 4.0 : tiles32 <= cus ? 6.2 : 15.5;
  const bool heavy = 12.0 + 1.5e-8 * (double)M * (double)N * (double)K < per_1024 * (double)K / 1024.0;
  if (K <= BOX_K && tiles64 >= cus / 2 && tiles64 <= 2 * cus) {
    // short reductions on about one 64 x 64 tile per CU: the whole K extent at once (measured against
    // the kernels below: 784 x 1024 x 128 6.3 us against 8.4, 1024 x 1024 x 128 with beta = 1 6.1
    // against 8.7, 1280 x 1280 x 128 9.4 against 10.8; fewer than half a tile per CU and the
    // kernels that split K over wavefronts win, 640 x 640 x 128 4.6 us against 5.7; from about
    // 2.3 tiles per CU on the slab loop does, 1536 x 1536 x 64 8.4 us against 9.6)
    // 16-byte groups run along K for a K-contiguous operand (whole or unused when K % 4 == 0) and
    // along the rows for the other kind (rows % 4 == 0; the last group of an edge tile then starts
    // at rows - 4 or earlier)
    const bool a_fast = a_kc ? K % 4 == 0 : (M % 4 == 0 && M >= 4);
    const bool b_fast = b_kc ? K % 4 == 0 : (N % 4 == 0 && N >= 4);
    dim3 grid((M + 63) / 64, (N + 63) / 64);
#define GEMM_BOX(AK, BK_)                                                                                        \
  hipLaunchKernelGGL((k_gemm_box<AK, BK_>), grid, dim3(BOX_THREADS), 0, dn_stream(), A, lda, B, ldb, C, ldc, M, N, K, alpha, \
                     beta, a_fast, b_fast, epi)
#define GEMM_BOX_SUMS(AK, BK_)                                                                                    \
  hipLaunchKernelGGL((k_gemm_box_sums<AK, BK_>), sgrid, dim3(BOX_THREADS), 0, dn_stream(), A, lda, B, ldb, C, ldc, M, N, K, \
                     alpha, beta, a_fast, b_fast, epi, (int)grid.y, *g_side_jobs, g_side_blocks)
    if (side_jobs_fit(epi)) {
      const dim3 sgrid(grid.x, grid.y + (g_side_blocks + grid.x - 1) / grid.x);
      if (a_kc && b_kc) GEMM_BOX_SUMS(true, true);
      else if (a_kc) GEMM_BOX_SUMS(true, false);
      else if (b_kc) GEMM_BOX_SUMS(false, true);
      else GEMM_BOX_SUMS(false, false);
      g_side_blocks = 0;                // taken along
    }
    else if (a_kc && b_kc) GEMM_BOX(true, true);
    else if (a_kc) GEMM_BOX(true, false);
    else if (b_kc) GEMM_BOX(false, true);
    else GEMM_BOX(false, false);
#undef GEMM_BOX_SUMS
#undef GEMM_BOX
    if (fused) *fused = true;
    return dn_launch_status();
  }
  // Two K-contiguous operands whose rows lie a multiple of 1 KiB apart: the 16 x 16 block kernel
  // reads 16 such rows per load instruction and they meet in the same memory channels (measured
  // 1024 x 128 x 1024 with both leading dimensions 1024: 9.2 us against 8.5 us on 32 x 32 blocks).
  const bool kc_aliased = a_kc && b_kc && (lda % 256 == 0 || ldb % 256 == 0);
  // With both operands K-contiguous a CU's time goes with the operand bytes it pulls through its L1:
  // more 16 x 16 blocks than CUs then means a second round on some of them, and from K = 1024 on the
  // 32 x 32 blocks below are faster (1536 x 64 x 4096: 30.3 us against 2048 x 64 x 4096 on them in 25.9).
  const bool t16_second_round = a_kc && b_kc && tiles16 > cus && K >= 1024;
  if (tiles64 < cus && off32 && !heavy && !t16_second_round &&
      (tiles32 * 5 <= cus * 2 || (tiles32 * 2 <= cus && !kc_aliased))) {
    // 32 x 32 blocks would leave half or more of the CUs idle: 16 x 16 blocks, K over 4 wavefronts
    // (measured against 32 x 32 blocks: 500 x 100 x 784 4.4 us against 7.7, 1024 x 128 x 784 6.5 against
    // 7.9, 1024 x 128 x 1024 with an M-contiguous first operand 7.2 against 8.8; against 8 wavefronts per
    // block: 500 x 100 x 784 5.4 us against 6.0)
    dim3 grid((M + 15) / 16, (N + 15) / 16);
#define GEMM_T16(AK, BK_)                                                                                  \
  hipLaunchKernelGGL((k_gemm_tile16<AK, BK_, 4>), grid, dim3(256), 0, dn_stream(), A, lda, B, ldb, C, ldc, M, N, K, \
                     alpha, beta, epi)
#define GEMM_T16_SUMS(AK, BK_)                                                                                   \
  hipLaunchKernelGGL((k_gemm_tile16_sums<AK, BK_, 4>), sgrid, dim3(256), 0, dn_stream(), A, lda, B, ldb, C, ldc, M, N, K, \
                     alpha, beta, epi, (int)grid.y, *g_side_jobs, g_side_blocks)
    if (side_jobs_fit(epi)) {
      const dim3 sgrid(grid.x, grid.y + (g_side_blocks + grid.x - 1) / grid.x);
      if (a_kc && b_kc) GEMM_T16_SUMS(true, true);
      else if (a_kc) GEMM_T16_SUMS(true, false);
      else if (b_kc) GEMM_T16_SUMS(false, true);
      else GEMM_T16_SUMS(false, false);
      g_side_blocks = 0;                // taken along
    }
    else if (a_kc && b_kc) GEMM_T16(true, true);
    else if (a_kc) GEMM_T16(true, false);
    else if (b_kc) GEMM_T16(false, true);
    else GEMM_T16(false, false);
#undef GEMM_T16_SUMS
#undef GEMM_T16
    if (fused) *fused = true;
    if (sampled) *sampled = epi.sample != nullptr;
    return dn_launch_status();
  }
  // 32 x 32 blocks, K over 8 wavefronts: a CU takes them two at a time in rounds of about 5 us per 512
  // of K, so up to two rounds they beat one 64 x 64 tile per CU (512 x 1024 x 512: 10.2 us against
  // 15.0, x 1024: 17.2 against 25.4) and from the third round on they do not (784 x 1000 x 200: 14.8 us
  // against 9.0, x 1024: 37.6 against 25.9; 832 x 832 x 2048: 53.3 against 37.2). Two rounds of long
  // reductions over operands that are both contiguous along the rows of the product lose to tiles with
  // a split K (512 x 1024 x 2048: 39.2 us against 27.5).
  const bool mn_both = !a_kc && !b_kc;
  if (tiles32 <= 2ll * cus && !(mn_both && K >= 2048 && tiles32 > cus) && off32 && !heavy) {
    dim3 grid((M + 31) / 32, (N + 31) / 32);
#define GEMM_SMALL(AK, BK_)                                                                                  \
  do {                                                                                                       \
    if (K <= 128)                                                                                            \
      hipLaunchKernelGGL((k_gemm_small<AK, BK_, 4>), grid, dim3(256), 0, dn_stream(), A, lda, B, ldb, C, ldc, M, N, K,  \
                         alpha, beta, a_vec, b_vec, epi);                                                    \
    else                                                                                                     \
      hipLaunchKernelGGL((k_gemm_small<AK, BK_, 8>), grid, dim3(512), 0, dn_stream(), A, lda, B, ldb, C, ldc, M, N, K,  \
                         alpha, beta, a_vec, b_vec, epi);                                                    \
  } while (0)
#define GEMM_SMALL_SUMS(AK, BK_)                                                                              \
  hipLaunchKernelGGL((k_gemm_small_sums<AK, BK_>), sgrid, dim3(256), 0, dn_stream(), A, lda, B, ldb, C, ldc, M, N, K, \
                     alpha, beta, a_vec, b_vec, epi, (int)grid.y, *g_side_jobs, g_side_blocks)
    if (K <= 128 && side_jobs_fit(epi)) {
      const dim3 sgrid(grid.x, grid.y + (g_side_blocks + grid.x - 1) / grid.x);
      if (a_kc && b_kc) GEMM_SMALL_SUMS(true, true);
      else if (a_kc) GEMM_SMALL_SUMS(true, false);
      else if (b_kc) GEMM_SMALL_SUMS(false, true);
      else GEMM_SMALL_SUMS(false, false);
      g_side_blocks = 0;                // taken along
    }
    else if (a_kc && b_kc) GEMM_SMALL(true, true);
    else if (a_kc) GEMM_SMALL(true, false);
    else if (b_kc) GEMM_SMALL(false, true);
    else GEMM_SMALL(false, false);
#undef GEMM_SMALL_SUMS
#undef GEMM_SMALL
    if (fused) *fused = true;
    if (sampled) *sampled = epi.sample != nullptr;
    return dn_launch_status();
  }
  const long long tiles_big = (long long)((M + 127) / 128) * ((N + 127) / 128);
  // 128 x 128 tiles (two workgroups per CU) against 64 x 64 tiles (five), as measured:
  // short reductions are mostly prologue and epilogue, which more resident workgroups hide
  // (4096 x 4096 x 128, beta = 1: 71 us against 60 us; up to K = 512 when C is also read, K = 256 otherwise); and
  // a tile count that leaves the last round of a CU half empty costs more than the smaller
  // tile's lower matrix-core rate of about 0.92 (3072 x 3072 x 2048: 404 us against 336 us).
  // (with the present main loop: 4096 x 4096 x 256 84 us on 64 x 64 tiles against 88 us, x 512 even, x 1024 268 us
  // against 254 us; fewer than two big tiles per CU leave the CU to one or two workgroups, and the small
  // tiles win up to K = 1024: 2048 x 2048 x 256 24.2 us against 30.3 us, x 512 39.6 against 46.7, x 1024 71.4
  // against 75.5)
  const int kmax64 = tiles_big < 2ll * cus ? 1024 : beta != 0.f ? 512 : 256;
  auto fill = [&](long long t) { return (double)t / (double)(((t + cus - 1) / cus) * cus); };
  const bool big = tiles_big >= cus && K > kmax64 && fill(tiles_big) >= 0.92 * fill(tiles64);
  const int BM = big ? 128 : 64, BN = big ? 128 : 64;
  const int gx = (M + BM - 1) / BM, gy = (N + BN - 1) / BN;
  int splits = 1;
  if (!big) {
    const long long tiles = (long long)gx * gy;
    const int kslabs = (K + GEMM_BK - 1) / GEMM_BK;
    long long want = (2ll * cus + tiles - 1) / tiles;
    if (want > kslabs / 4) want = kslabs / 4;  // at least 4 slabs (64 deep) per slice
    if (want > 32) want = 32;
    // The second kernel costs about 5 us and a split slice starts its pipeline anew: measured
    // on 1024 x 1024 outputs a split only pays from K = 2048 on (K = 128: 13 us split, 7.5 us
    // whole), and with 1.5 tiles per CU (1280 x 1280) it never does.
    // With four slices or more (tiles on two thirds of the CUs at most) it pays from K = 1024 on
    // (768 x 768 x 1024: 23.4 us against 25.9, x 1536: 29.9 against 36.3).
    if ((K < 2048 && !(K >= 1024 && (heavy || want >= 4))) || tiles * 4 >= (long long)cus * 5) want = 1;
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
  const GemmEpilogue none = {nullptr, GEMM_ACT_NONE, nullptr, nullptr, nullptr, nullptr, 0u, nullptr, 0, 0.f, nullptr};
  if (big) launch_gemm<2, 2>(a_kc, b_kc, grid, A, lda, B, ldb, C, ldc, M, N, K, kps, alpha, beta, partial, a_vec, b_vec, splits > 1 ? none : epi);
  else launch_gemm<1, 1>(a_kc, b_kc, grid, A, lda, B, ldb, C, ldc, M, N, K, kps, alpha, beta, partial, a_vec, b_vec, splits > 1 ? none : epi);
  if (fused) *fused = splits == 1;
  if (splits > 1) {
    size_t total = (size_t)M * N;
    unsigned blocks = (unsigned)((total + 255) / 256 < (size_t)cus * 8 ? (total + 255) / 256 : (size_t)cus * 8);
    if (M % 4 == 0 && ldc % 4 == 0 && dn_aligned16(C))
      hipLaunchKernelGGL(k_gemm_splitk_finish4, dim3((unsigned)((total / 4 + 255) / 256)), dim3(256), 0, dn_stream(), partial, splits, C, ldc, M, N, alpha, beta);
    else
      hipLaunchKernelGGL(k_gemm_splitk_finish, dim3(blocks), dim3(256), 0, dn_stream(), partial, splits, C, ldc, M, N, alpha, beta);
  }
  return dn_launch_status();
}

// C = beta*C + alpha*op(A)*op(B) and the sums of `jobs`, which touch nothing the product reads or writes:
// one launch where the product's kernel can take the sums along, otherwise the product, then the sums.
int dn_gemm_sums(bool a_trans, bool b_trans, int M, int N, int K, float alpha, const float* A, int lda, const float* B, int ldb,
                 float beta, float* C, int ldc, const DnRowSumJob* jobs, int njobs) {
  RowSumJobs J = {};
  const int jblocks = njobs > 0 ? rows_sum_jobs_table(jobs, njobs, &J) : 0;
  if (jblocks < 0) return ERROR_GENERIC;
  dn_flush();                     // (no other product may be launched from inside this one's launch and take the sums)
  g_side_jobs = &J;
  g_side_blocks = jblocks;
  const int e = gemm(a_trans, b_trans, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc);
  const bool taken = g_side_blocks == 0;
  g_side_jobs = nullptr;
  g_side_blocks = 0;
  if (e) return e;
  return (taken || njobs <= 0) ? 0 : dn_row_sum_jobs(jobs, njobs);
}

// Whether gemm() would hand this product to k_gemm_small<.., 4> (the conditions of its dispatch, in its order).
static bool gemm_goes_small4(bool a_kc, bool b_kc, int M, int N, int K, int lda, int ldb) {
  if (M <= 0 || N <= 0 || K <= 0 || K > 128) return false;
  const int cus = dn_num_cus();
  const long long tiles64 = (long long)((M + 63) / 64) * ((N + 63) / 64);
  const bool off32 = (size_t)lda * (a_kc ? M : K) < (1u << 30) && (size_t)ldb * (b_kc ? N : K) < (1u << 30);
  const long long tiles32 = (long long)((M + 31) / 32) * ((N + 31) / 32);
  const long long tiles16 = (long long)((M + 15) / 16) * ((N + 15) / 16);
  const double per_1024 = tiles16 <= cus ? 4.0 : tiles32 <= cus ? 6.2 : 15.5;
  const bool heavy = 12.0 + 1.5e-8 * (double)M * (double)N * (double)K < per_1024 * (double)K / 1024.0;
  if (K <= BOX_K && tiles64 >= cus / 2 && tiles64 <= 2 * cus) return false;            // k_gemm_box
  const bool kc_aliased = a_kc && b_kc && (lda % 256 == 0 || ldb % 256 == 0);
  const bool t16_second_round = a_kc && b_kc && tiles16 > cus && K >= 1024;
  if (tiles64 < cus && off32 && !heavy && !t16_second_round &&
      (tiles32 * 5 <= cus * 2 || (tiles32 * 2 <= cus && !kc_aliased)))
    return false;                                                                      // k_gemm_tile16
  const bool mn_both = !a_kc && !b_kc;
  return tiles32 <= 2ll * cus && !(mn_both && K >= 2048 && tiles32 > cus) && off32 && !heavy;
}

// C = beta*C + alpha*op(A)*op(B), then C = C + alpha2*op(A2)*op(B2) (the second pair of operands has the
// first pair's shapes and transposes).  One launch with the bits of the two when both products are
// k_gemm_small's with one chunk per wavefront; otherwise the two launches.
int dn_gemm_pair_sums(bool a_trans, bool b_trans, int M, int N, int K, float alpha, const float* A, int lda, const float* B,
                      int ldb, float beta, float alpha2, const float* A2, int lda2, const float* B2, int ldb2, float* C, int ldc,
                      const DnRowSumJob* jobs, int njobs) {
  const bool a_kc = a_trans, b_kc = !b_trans;
  RowSumJobs J = {};
  const int jblocks = njobs > 0 ? rows_sum_jobs_table(jobs, njobs, &J) : 0;
  if (jblocks < 0) return ERROR_GENERIC;
  if (gemm_goes_small4(a_kc, b_kc, M, N, K, lda, ldb) && gemm_goes_small4(a_kc, b_kc, M, N, K, lda2, ldb2)) {
    GemmPairArgs g;
    g.A = A; g.B = B; g.A2 = A2; g.B2 = B2; g.C = C;
    g.lda = lda; g.ldb = ldb; g.lda2 = lda2; g.ldb2 = ldb2; g.ldc = ldc; g.M = M; g.N = N; g.K = K;
    g.alpha = alpha; g.beta = beta; g.alpha2 = alpha2;
    g.a_vec = dn_aligned16(A) && (lda % 4 == 0); g.b_vec = dn_aligned16(B) && (ldb % 4 == 0);
    g.a2_vec = dn_aligned16(A2) && (lda2 % 4 == 0); g.b2_vec = dn_aligned16(B2) && (ldb2 % 4 == 0);
    const int gx = (M + 31) / 32, gy = (N + 31) / 32;
    if (jblocks == 0) {
      dim3 grid(gx, gy);
#define GEMM_PAIR(AK, BK_) hipLaunchKernelGGL((k_gemm_small_pair<AK, BK_>), grid, dim3(256), 0, dn_stream(), g)
      if (a_kc && b_kc) GEMM_PAIR(true, true);
      else if (a_kc) GEMM_PAIR(true, false);
      else if (b_kc) GEMM_PAIR(false, true);
      else GEMM_PAIR(false, false);
#undef GEMM_PAIR
    } else {
      const int nprod = gx * gy;
      dim3 grid(nprod + jblocks);
#define GEMM_PAIR_SUMS(AK, BK_) \
  hipLaunchKernelGGL((k_gemm_small_pair_sums<AK, BK_>), grid, dim3(256), 0, dn_stream(), g, gx, nprod, J)
      if (a_kc && b_kc) GEMM_PAIR_SUMS(true, true);
      else if (a_kc) GEMM_PAIR_SUMS(true, false);
      else if (b_kc) GEMM_PAIR_SUMS(false, true);
      else GEMM_PAIR_SUMS(false, false);
#undef GEMM_PAIR_SUMS
    }
    return dn_launch_status();
  }
  if (int e = gemm(a_trans, b_trans, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc)) return e;
  if (int e = gemm(a_trans, b_trans, M, N, K, alpha2, A2, lda2, B2, ldb2, 1.f, C, ldc)) return e;
  return njobs > 0 ? dn_row_sum_jobs(jobs, njobs) : 0;
}

// C = beta*C + alpha*op(A)*op(B) on raw column-major buffers, for the other kernels of the library.
int dn_gemm(bool a_trans, bool b_trans, int M, int N, int K, float alpha, const float* A, int lda, const float* B,
            int ldb, float beta, float* C, int ldc) {
  return gemm(a_trans, b_trans, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc);
}

// C = act(op(A)*op(B) + bias) [* (gate > 0)] for dot_bias_act(); *fused: whether the launch carried bias, act and gate
// (gate and mul, when given, are laid out as C with leading dimension ldc: C = C * mul * (gate > 0)).  drop: the sample is a dropout mask,
// (uniform > drop_p), and C is multiplied by it.
// smp (may be null): the sample to draw in the same launch; *sampled says whether it was drawn
// (then the generator's next words are in smp->next and the caller publishes them).
int dn_gemm_fused(bool a_trans, bool b_trans, int M, int N, int K, const float* A, int lda, const float* B, int ldb,
                  float* C, int ldc, const float* bias, int act, bool* fused, const DnGemmSample* smp, bool* sampled,
                  const float* gate, int drop, float drop_p, const float* mul) {
  GemmEpilogue epi = {bias, act, nullptr, nullptr, nullptr, nullptr, 0u, gate, drop, drop_p, mul};
  const unsigned long long total = (unsigned long long)M * (unsigned long long)N;
  if (smp && ldc == M && total <= (unsigned long long)GEMM_SAMPLE_MAX_DRAWS * NUM_RND_STREAMS) {
    epi.sample = smp->sample;
    epi.mults = smp->mults;
    epi.words = smp->words;
    epi.next = smp->next;
    epi.total = (unsigned int)total;
  }
  // (only the kernels that finish every output in one launch look at epi.sample)
  return gemm(a_trans, b_trans, M, N, K, 1.f, A, lda, B, ldb, 0.f, C, ldc, epi, fused, sampled);
}

// ------------------------------------------------------------------ contrastive-divergence statistics
// W += eps * (v h^T - v2 h2^T), bv += eps * (rowsums(v) - rowsums(v2)), bh += eps * (rowsums(h) - rowsums(h2))
// as ONE product over the concatenated reduction [v | v2] * [h | -h2]^T (2 * batch terms) with a row
// of ones appended to each operand: output row nv is the hidden bias statistic, output column nh
// the visible one (cudamat/examples/rbm_cudamat.py:57-85 spends two add_dot and four add_sums on it;
// deepnet/edge.py:236-242 and layer.py:206-211 collect the same statistics).
// A workgroup owns a 32 x 32 block of the (nv + 1) x (nh + 1) output; its NW wavefronts take
// every NW-th pair of terms, operands straight from global memory in the MFMA operand layout
// (both are contiguous along the output index: 128-byte runs), and meet in LDS in a fixed order.
// Lanes run along the visible index, which is the contiguous one of W.
template <int NW>
__global__ void __launch_bounds__(64 * NW)
k_cd_update(float* W, float* bv, float* bh, const float* v, const float* h, const float* v2, const float* h2,
            int nv, int nh, int B, float eps) {
  constexpr int EPL = 1024 / (64 * NW);     // outputs a lane finishes
  __shared__ float red[NW][16][64];
  const int tid = threadIdx.x, lane = tid & 63, li = lane & 31, half = lane >> 5;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int vis = blockIdx.x * 32 + li, hid = blockIdx.y * 32 + li;   // this lane's row of either operand
  // rows past the operands read row 0 and are replaced: by the ones of the appended row, or by zero
  const unsigned vis_c = vis < nv ? vis : 0, hid_c = hid < nh ? hid : 0;
  const bool vis_in = vis < nv, hid_in = hid < nh;
  const float vis_else = vis == nv ? 1.f : 0.f, hid_else = hid == nh ? 1.f : 0.f;
  // the old values of this lane's four outputs are requested before the operands, so that the
  // read-modify-write at the end does not wait for memory again
  float old[EPL];
  float* dst[EPL];
#pragma unroll
  for (int rr = 0; rr < EPL; ++rr) {
    const int o = tid + 64 * NW * rr, r = o >> 6, ln = o & 63;
    const int vi = blockIdx.x * 32 + (ln & 31);
    const int hi = blockIdx.y * 32 + 8 * (r >> 2) + 4 * (ln >> 5) + (r & 3);
    dst[rr] = vi < nv && hi < nh ? W + (size_t)hi * nv + vi
              : vi < nv && hi == nh ? (bv ? bv + vi : nullptr)
              : vi == nv && hi < nh ? (bh ? bh + hi : nullptr) : nullptr;
    old[rr] = *(dst[rr] ? dst[rr] : W);
  }
  f32x16 acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.f;
  // The reduction runs over the pairs of columns of (v, h), then over those of (v2, -h2): a pair
  // belongs to one of the two, so which operands it reads is a scalar question.  Wavefront w
  // takes pairs w, w + NW, ...; PF of them at a time (batches up to 128: all), 2 * PF loads in flight.
  const int ppp = (B + 1) >> 1, pairs = 2 * ppp;
  auto fetch = [&](int p, float& a, float& b) __attribute__((always_inline)) {
    const bool second = p >= ppp;                                  // wave-uniform
    const int k = 2 * (second ? p - ppp : p) + half;               // column of this lane
    const bool live = p < pairs && k < B;
    const unsigned col = live ? (unsigned)k : 0u;
    const float* vs = second ? v2 : v;
    const float* hs = second ? h2 : h;
    const float x = hs[col * (unsigned)nh + hid_c], y = vs[col * (unsigned)nv + vis_c];
    const float sign = second ? -1.f : 1.f;
    a = live ? sign * (hid_in ? x : hid_else) : 0.f;               // rows of the result block: hidden
    b = live ? (vis_in ? y : vis_else) : 0.f;                      // columns: visible
  };
  constexpr int PF = 128 / NW;
  for (int p0 = wv; p0 < pairs; p0 += 128) {
    float a[PF], b[PF];
#pragma unroll
    for (int u = 0; u < PF; ++u) fetch(p0 + NW * u, a[u], b[u]);
#pragma unroll
    for (int u = 0; u < PF; ++u) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u], b[u], acc, 0, 0, 0);
  }
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const float val = acc[i];
    red[wv][i][lane] = val;
  }
  __syncthreads();
  // acc[r] of lane (li, half): visible index li, hidden index 8 * (r / 4) + 4 * half + r % 4
#pragma unroll
  for (int rr = 0; rr < EPL; ++rr) {
    const int o = tid + 64 * NW * rr, r = o >> 6, ln = o & 63;
    float s = red[0][r][ln];
#pragma unroll
    for (int w = 1; w < NW; ++w) s += red[w][r][ln];
    if (dst[rr]) *dst[rr] = __fmaf_rn(eps, s, old[rr]);
  }
}

extern "C" {

// Extension (no counterpart in cudamat.cu): the contrastive-divergence update of an RBM in one
// launch.  W is nv x nh, v and v2 are nv x batch, h and h2 are nh x batch, bv is nv x 1 and bh is
// nh x 1 (either may be null); nothing may be transposed.
int cd_update(cudamat* W, cudamat* bv, cudamat* bh, cudamat* v, cudamat* h, cudamat* v2, cudamat* h2, float eps) {
  if (!W->on_device || !v->on_device || !h->on_device || !v2->on_device || !h2->on_device || (bv && !bv->on_device) ||
      (bh && !bh->on_device))
    return ERROR_NOT_ON_DEVICE;
  if (W->is_trans || v->is_trans || h->is_trans || v2->is_trans || h2->is_trans || (bv && bv->is_trans) || (bh && bh->is_trans))
    return ERROR_TRANSPOSED;
  const int nv = W->size[0], nh = W->size[1], B = v->size[1];
  if (v->size[0] != nv || v2->size[0] != nv || v2->size[1] != B || h->size[0] != nh || h->size[1] != B || h2->size[0] != nh ||
      h2->size[1] != B || (bv && (bv->size[0] != nv || bv->size[1] != 1)) || (bh && (bh->size[0] != nh || bh->size[1] != 1)))
    return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (nv <= 0 || nh <= 0 || B <= 0) return 0;
  if ((long long)nv * B >= (1ll << 31) || (long long)nh * B >= (1ll << 31)) return ERROR_UNSUPPORTED;   // (32-bit offsets into the operands)
  // Batches of up to 128: the two products and the four sums of the reference's spelling as they
  // are, in one launch (k_gemm_small_pair_sums: the bits of the six calls, and faster than the
  // augmented product below: 784 x 500, batch 100: 8 us against 11 under the tracer)
  if (gemm_goes_small4(false, false, nv, nh, B, nv, nh) &&
      (!bv || (dn_row_sum_job_ok(v->data_device, nv, B) && dn_row_sum_job_ok(v2->data_device, nv, B))) &&
      (!bh || (dn_row_sum_job_ok(h->data_device, nh, B) && dn_row_sum_job_ok(h2->data_device, nh, B)))) {
    DnRowSumJob jobs[4];
    int nj = 0;
    if (bv) {
      jobs[nj++] = DnRowSumJob{v->data_device, bv->data_device, nv, B, eps, 1.f, 0};
      jobs[nj++] = DnRowSumJob{v2->data_device, bv->data_device, nv, B, -eps, 1.f, 0};
    }
    if (bh) {
      jobs[nj++] = DnRowSumJob{h->data_device, bh->data_device, nh, B, eps, 1.f, 0};
      jobs[nj++] = DnRowSumJob{h2->data_device, bh->data_device, nh, B, -eps, 1.f, 0};
    }
    return dn_gemm_pair_sums(false, true, nv, nh, B, eps, v->data_device, nv, h->data_device, nh, 1.f, -eps, v2->data_device, nv,
                             h2->data_device, nh, W->data_device, nv, jobs, nj);
  }
  const dim3 grid((unsigned)(nv / 32 + 1), (unsigned)(nh / 32 + 1));
  // (8 wavefronts per block measured against 4 and 16 on 784 x 500, batch 100: 7.9 us against 9.9 and 7.7)
  hipLaunchKernelGGL(k_cd_update<8>, grid, dim3(512), 0, dn_stream(), W->data_device, bv ? bv->data_device : nullptr,
                     bh ? bh->data_device : nullptr, (const float*)v->data_device, (const float*)h->data_device,
                     (const float*)v2->data_device, (const float*)h2->data_device, nv, nh, B, eps);
  return dn_launch_status();
}

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
  // (held back when the calls that follow may ride in its epilogue)
  int held = 0;
  if (dn_defer_dot(mat1, mat2, target, beta, alpha, m, n, k, &held)) return held;

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
