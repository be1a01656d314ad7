// Several sums along the rows in one launch: the job table and the body of a workgroup, shared by
// the kernel that runs such jobs alone (reduce.hip) and the one that runs them beside a pair of
// products (gemm.hip).  A job adds alpha * rowsums(M) to a vector y (M is h x w, leading dimension
// h); up to two vectors with up to two jobs each, applied in the order given.  Every sum is taken
// in the order of k_rows_one<ROW_SUM, 4, ., false> with one column slice (lane groups on
// neighbouring columns, four wavefronts, fixed order in LDS; a job marked scalar: in the order of
// k_rows_stage1<false, ROW_SUM, 4, 4, false>) and finished by the same expression,
// so the results have the bits of the separate launches.
#pragma once
#include "common.h"

struct RowSumJob { const float* M; int w; float alpha, beta; int scalar; };
struct RowSumJobs {
  float* y0; float* y1;
  int h0, h1, n0, n1, bx0;
  RowSumJob a0, a1, b0, b1;       // a*: jobs of y0, b*: jobs of y1
};

// beta*y + alpha*s as one multiplication and one fused multiply-add, spelled out so that every
// kernel that finishes a row this way rounds alike
__device__ __forceinline__ float rowsum_finish(float yold, float s, float alpha, float beta) {
  return __fmaf_rn(alpha, s, beta == 0.f ? 0.f : __fmul_rn(beta, yold));
}

// Workgroup `block` of the jobs: 64 rows of one of the vectors, on the first 256 lanes (a larger
// workgroup's other lanes only keep the barriers company).
__device__ __forceinline__ void rows_sum_jobs_body(const RowSumJobs& J, int block) {
  __shared__ float sv[4][64];
  const bool live = threadIdx.x < 256;
  const bool second = block >= J.bx0;                        // block-uniform
  const int bx = block - (second ? J.bx0 : 0);
  const int h = second ? J.h1 : J.h0, nj = second ? J.n1 : J.n0;
  float* y = second ? J.y1 : J.y0;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int r = lane & 15, c = lane >> 4;
  const int row0 = (bx * 16 + r) * 4;
  const int row = bx * 64 + (int)threadIdx.x;
  const bool mine = threadIdx.x < 64 && row < h;
  float yv = mine ? y[row] : 0.f;
  constexpr int NW = 4, U = 8;
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    if (q >= nj) break;
    const RowSumJob job = second ? (q ? J.b1 : J.b0) : (q ? J.a1 : J.a0);
    const int w = job.w;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    if (job.scalar) {
      // matrices whose rows do not come in aligned groups of four: a lane owns one row, in the order of
      // k_rows_stage1<false, ROW_SUM, 4, 4, false> with one column slice (wavefront v the columns v, v + 4, ..,
      // four in flight; a column past the end adds a zero)
      const int srow = bx * 64 + lane;
      float a1 = 0.f;
      if (live && srow < h) {
        for (int j = wv; j < w; j += 16) {
          float v[4];
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const int jj = j + 4 * u;
            v[u] = jj < w ? job.M[(size_t)jj * h + srow] : 0.f;
          }
#pragma unroll
          for (int u = 0; u < 4; ++u) a1 += v[u];
        }
      }
      if (live) sv[wv][lane] = a1;
      __syncthreads();
      if (mine) {
        float s = sv[0][threadIdx.x];
#pragma unroll
        for (int k = 1; k < NW; ++k) s += sv[k][threadIdx.x];
        yv = rowsum_finish(yv, s, job.alpha, job.beta);
      }
      __syncthreads();
      continue;
    }
    if (live && row0 < h) {
      for (int j = wv * 4 + c; j < w; j += NW * 4 * U) {
        float4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int jj = j + NW * 4 * u;
          v[u] = jj < w ? dn_ld4<false>(job.M + (size_t)jj * h + row0) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) { acc[0] += v[u].x; acc[1] += v[u].y; acc[2] += v[u].z; acc[3] += v[u].w; }
      }
    }
#pragma unroll
    for (int o = 16; o < 64; o <<= 1)
#pragma unroll
      for (int k = 0; k < 4; ++k) acc[k] += __shfl_xor(acc[k], o, 64);
    if (live && c == 0) *reinterpret_cast<float4*>(&sv[wv][r * 4]) = make_float4(acc[0], acc[1], acc[2], acc[3]);
    __syncthreads();
    if (mine) {
      float s = sv[0][threadIdx.x];
#pragma unroll
      for (int k = 1; k < NW; ++k) s += sv[k][threadIdx.x];
      yv = rowsum_finish(yv, s, job.alpha, job.beta);
    }
    __syncthreads();
  }
  if (mine) y[row] = yv;
}

// Fills the table from jobs in call order (at most two different y, at most two jobs each);
// returns the number of workgroups, 0 for an empty table, -1 when the jobs do not fit.
static inline int rows_sum_jobs_table(const DnRowSumJob* jobs, int n, RowSumJobs* out) {
  RowSumJobs J = {};
  for (int i = 0; i < n; ++i) {
    const RowSumJob rj = {jobs[i].M, jobs[i].w, jobs[i].alpha, jobs[i].beta, jobs[i].scalar};
    if (J.n0 == 0 || jobs[i].y == J.y0) {
      if (J.n0 >= 2) return -1;
      J.y0 = jobs[i].y; J.h0 = jobs[i].h;
      (J.n0 == 0 ? J.a0 : J.a1) = rj;
      ++J.n0;
    } else {
      if ((J.n1 > 0 && jobs[i].y != J.y1) || J.n1 >= 2) return -1;
      J.y1 = jobs[i].y; J.h1 = jobs[i].h;
      (J.n1 == 0 ? J.b0 : J.b1) = rj;
      ++J.n1;
    }
  }
  *out = J;
  if (J.n0 == 0) return 0;
  J.bx0 = (J.h0 + 63) / 64;
  out->bx0 = J.bx0;
  return J.bx0 + (J.n1 ? (J.h1 + 63) / 64 : 0);
}
