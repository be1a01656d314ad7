// Reductions: per-column / per-row max, argmax, sum of squares, norm clipping,
// column softmax and its loss helpers, weighted sums (matrix-vector products),
// flat dot product and Euclidean norm.
// Replaces cudamat/cudamat.cu:1148-1315, 1733-1761, 2104-2118, 2192-2346 and
// the kernels cudamat_kernels.cu:5-92, 819-1088.
//
// A column is h contiguous floats.  One wavefront (or one 256-lane workgroup
// for tall, few columns) streams a column with 16-byte loads and finishes with
// cross-lane shuffles; rows are reduced by tiles of 64 rows x 4 wavefronts with
// the lanes running down the rows so every load is a 256-byte run.
#include "common.h"
#include "rowsum_jobs.h"
#include <float.h>
#include <math.h>
#include <string.h>


// ------------------------------------------------------------------ column walkers

// Visit every element of one column with TPC cooperating lanes: fn(row, value).
// Four 16-byte loads are issued before any of them is consumed.
template <int TPC, class Fn>
__device__ __forceinline__ void for_each_in_col(const float* c, int h, int lane, Fn fn, bool stream = false) {
  int head = (int)(((16u - (unsigned)(reinterpret_cast<uintptr_t>(c) & 15u)) & 15u) >> 2);
  if (head > h) head = h;
  if (lane < head) fn(lane, c[lane]);
  const float4* c4 = reinterpret_cast<const float4*>(c + head);
  const int n4 = (h - head) >> 2;
  int j = lane;
  for (; j + 3 * TPC < n4; j += 4 * TPC) {
    float4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) v[u] = dn_ld4_rt(reinterpret_cast<const float*>(c4 + j + u * TPC), stream);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int b = head + 4 * (j + u * TPC);
      fn(b, v[u].x); fn(b + 1, v[u].y); fn(b + 2, v[u].z); fn(b + 3, v[u].w);
    }
  }
  for (; j < n4; j += TPC) {
    const float4 v = dn_ld4_rt(reinterpret_cast<const float*>(c4 + j), stream);
    const int b = head + 4 * j;
    fn(b, v.x); fn(b + 1, v.y); fn(b + 2, v.z); fn(b + 3, v.w);
  }
  const int t0 = head + 4 * n4;
  if (lane < h - t0) fn(t0 + lane, c[t0 + lane]);
}

// Combine one float per lane across the TPC lanes that share a column.
// TPC == 64: shuffles only.  TPC == 256: shuffles, then 4 partials through LDS.
template <int TPC, bool IS_MAX>
__device__ __forceinline__ float col_combine(float v, float* lds4) {
  v = IS_MAX ? wave_max(v) : wave_sum(v);
  if (TPC == 64) return v;
  const int wv = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) lds4[wv] = v;
  __syncthreads();
  const float a = lds4[0], b = lds4[1], c = lds4[2], d = lds4[3];
  return IS_MAX ? fmaxf(fmaxf(a, b), fmaxf(c, d)) : ((a + b) + (c + d));
}

// Arg-max candidate.  The reference scans a column with 32 lanes, lane t taking
// rows t, t+32, ..., keeps the first strictly larger value per lane and then
// the first strictly larger lane (cudamat_kernels.cu:1020-1050); among equal
// maxima that selects the smallest (row % 32, row).  key reproduces that order;
// the start value (-FLT_MAX, row 0) wins every tie, as it does there.
struct ArgCand {
  float v;
  long long key;  // -1 for the start value, else ((row % 32) << 32) | row
  int row;
};
__device__ __forceinline__ bool arg_better(float v1, long long k1, float v2, long long k2) {
  return v1 > v2 || (v1 == v2 && k1 < k2);
}
__device__ __forceinline__ void arg_visit(ArgCand& c, int row, float v) {
  const long long k = ((long long)(row & 31) << 32) | (long long)row;
  if (arg_better(v, k, c.v, c.key)) { c.v = v; c.key = k; c.row = row; }
}
template <int TPC>
__device__ __forceinline__ ArgCand arg_combine(ArgCand c, ArgCand* lds4) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float v = __shfl_xor(c.v, o, WAVE);
    const long long k = __shfl_xor(c.key, o, WAVE);
    const int r = __shfl_xor(c.row, o, WAVE);
    if (arg_better(v, k, c.v, c.key)) { c.v = v; c.key = k; c.row = r; }
  }
  if (TPC == 64) return c;
  const int wv = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) lds4[wv] = c;
  __syncthreads();
  ArgCand best = lds4[0];
#pragma unroll
  for (int i = 1; i < 4; ++i)
    if (arg_better(lds4[i].v, lds4[i].key, best.v, best.key)) best = lds4[i];
  return best;
}

#define COL_SETUP(TPC)                                                 \
  const int cols_per_block = 256 / TPC;                                \
  const int col = blockIdx.x * cols_per_block + (int)threadIdx.x / TPC; \
  const int lane = (int)threadIdx.x % TPC;                             \
  const bool active = col < w;

// ------------------------------------------------------------------ column kernels (axis 0)

template <int TPC>
__global__ void __launch_bounds__(256) k_col_max(const float* mat, float* target, int w, int h) {
  __shared__ float lds4[4];
  COL_SETUP(TPC)
  const bool stream = (long long)w * h >= DN_STREAM_MIN_ELEMS;
  float m = -FLT_MAX;
  if (active) for_each_in_col<TPC>(mat + (size_t)col * h, h, lane, [&](int, float v) { if (v > m) m = v; }, stream);
  m = col_combine<TPC, true>(m, lds4);
  if (active && lane == 0) target[col] = m;
}

// mode 0: target[col] = argmax; 1: one-hot column into target; 2: target(argmax, col) += 1;
// 3: target[col] = (argmax == (int)labels[col]).
template <int TPC>
__global__ void __launch_bounds__(256)
k_col_argmax(const float* mat, float* target, const float* labels, int w, int h, int mode) {
  __shared__ ArgCand lds4[4];
  COL_SETUP(TPC)
  ArgCand c;
  c.v = -FLT_MAX; c.key = -1; c.row = 0;
  if (active) for_each_in_col<TPC>(mat + (size_t)col * h, h, lane, [&](int r, float v) { arg_visit(c, r, v); });
  c = arg_combine<TPC>(c, lds4);
  if (!active) return;
  if (mode == 0) {
    if (lane == 0) target[col] = (float)c.row;
  } else if (mode == 1) {
    float* t = target + (size_t)col * h;
    for (int i = lane; i < h; i += TPC) t[i] = (i == c.row) ? 1.f : 0.f;
  } else if (mode == 2) {
    if (lane == 0) target[(size_t)col * h + c.row] += 1.f;
  } else {
    if (lane == 0) target[col] = (c.row == (int)labels[col]) ? 1.f : 0.f;
  }
}

template <int TPC>
__global__ void __launch_bounds__(256) k_col_sqsum(const float* mat, float* target, int w, int h, float mult, float p) {
  __shared__ float lds4[4];
  COL_SETUP(TPC)
  const bool stream = (long long)w * h >= DN_STREAM_MIN_ELEMS;
  float s = 0.f;
  if (active) for_each_in_col<TPC>(mat + (size_t)col * h, h, lane, [&](int, float v) { s += v * v; }, stream);
  s = col_combine<TPC, false>(s, lds4);
  // p == 0 overwrites: the previous contents (possibly uninitialised) are not read.
  if (active && lane == 0) target[col] = (p == 0.f ? 0.f : p * target[col]) + mult * s;
}

template <int TPC>
__global__ void __launch_bounds__(256) k_col_normlimit(const float* mat, float* target, int w, int h, float norm) {
  __shared__ float lds4[4];
  COL_SETUP(TPC)
  float s = 0.f;
  const float* c = mat + (size_t)col * h;
  if (active) for_each_in_col<TPC>(c, h, lane, [&](int, float v) { s += v * v; });
  s = col_combine<TPC, false>(s, lds4);
  if (!active) return;
  float scale = sqrtf(s);
  scale = (scale < norm) ? 1.f : (norm / scale);
  float* t = target + (size_t)col * h;
  for_each_in_col<TPC>(c, h, lane, [&](int r, float v) { t[r] = v * scale; });
}

// The same for aligned columns of at most 64 * 4 * NV floats (h % 4 == 0), one wavefront per column: the
// column stays in registers between the two passes, one read and one write of HBM per element.
template <int NV>
__global__ void __launch_bounds__(256) k_col_normlimit_reg(const float* mat, float* target, int w, int h, float norm) {
  const int col = blockIdx.x * 4 + (int)(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (col >= w) return;
  const float* c4 = mat + (size_t)col * h;
  float* t4 = target + (size_t)col * h;
  const int n4 = h >> 2;
  const bool stream = (long long)w * h >= DN_STREAM_MIN_ELEMS;
  float4 v[NV];
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int j = lane + k * 64;
    v[k] = j < n4 ? dn_ld4_rt(c4 + 4 * j, stream) : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  float s = 0.f;
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    if (lane + k * 64 < n4) { s += v[k].x * v[k].x; s += v[k].y * v[k].y; s += v[k].z * v[k].z; s += v[k].w * v[k].w; }
  }
  s = wave_sum(s);
  float scale = sqrtf(s);
  scale = (scale < norm) ? 1.f : (norm / scale);
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int j = lane + k * 64;
    if (j < n4) dn_st4_rt(t4 + 4 * j, make_float4(v[k].x * scale, v[k].y * scale, v[k].z * scale, v[k].w * scale), stream);
  }
}

// e^t for t <= 0 in softmax: t*log2(e) as a two-term product (the rounding of the first
// term and the tail of the constant go into a correction factor), then the hardware exp2.
// Relative error about 1.5 ulp over the whole range, against the 1e-5 these outputs are
// held to; a result below the normal range may come out as 0.  t = -inf gives 0, NaN stays NaN.
__device__ __forceinline__ float softmax_exp(float t) {
  t = t < -128.f ? -128.f : t;      // (e^-128 is 0 in fp32; keeps -inf out of the correction term)
  const float L2E = 1.44269502162933349609375f, L2E_LO = 1.925963033500011e-08f;
  const float p = t * L2E;
  const float lo = __fmaf_rn(t, L2E_LO, __fmaf_rn(t, L2E, -p));
  const float e = __builtin_amdgcn_exp2f(p);
  return __fmaf_rn(e, lo * 0.693147182464599609375f, e);
}

// Column softmax: max, sum of exp(x - max), divide (cudamat_kernels.cu:868-934).
// The column is re-read from cache for the second and third pass.
// Optional extras of the fused loss step (all three null for plain softmax): with
// labels, loss[col] = -log(p[label] + tiny) and grad = p - onehot(label), each value
// computed from the stored p exactly as get_softmax_cross_entropy / apply_softmax_grad do.
struct SoftmaxExtras {
  const float* labels;
  float* loss;
  float* grad;
  float tiny;
};

template <int TPC>
__global__ void __launch_bounds__(256) k_col_softmax(const float* mat, float* target, int w, int h, SoftmaxExtras x) {
  __shared__ float lds4[4];
  COL_SETUP(TPC)
  const float* c = mat + (size_t)col * h;
  float* t = target + (size_t)col * h;
  float m = -FLT_MAX;
  if (active) for_each_in_col<TPC>(c, h, lane, [&](int, float v) { if (v > m) m = v; });
  m = col_combine<TPC, true>(m, lds4);
  float s = 0.f;
  if (active) for_each_in_col<TPC>(c, h, lane, [&](int, float v) { s += softmax_exp(v - m); });
  s = col_combine<TPC, false>(s, lds4);
  if (!active) return;
  const float inv = 1.f / s;
  if (!x.labels) {
    for_each_in_col<TPC>(c, h, lane, [&](int r, float v) { t[r] = softmax_exp(v - m) * inv; });
  } else {
    const int label = (int)x.labels[col];
    float* gcol = x.grad ? x.grad + (size_t)col * h : nullptr;
    for_each_in_col<TPC>(c, h, lane, [&](int r, float v) {
      const float pr = softmax_exp(v - m) * inv;
      t[r] = pr;
      if (gcol) gcol[r] = pr - ((label == r) ? 1.f : 0.f);
      if (x.loss && r == label) x.loss[col] = -logf(pr + x.tiny);
    });
  }
}

// Columns of at most 64 * 4 * NV floats stay in registers between the passes:
// one read and one write of HBM per element.  Requires h % 4 == 0 and 16-byte
// aligned columns.
template <int NV>
__global__ void __launch_bounds__(256) k_col_softmax_reg(const float* mat, float* target, int w, int h, SoftmaxExtras x) {
  const int col = blockIdx.x * 4 + (int)(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (col >= w) return;
  const float* c4 = mat + (size_t)col * h;
  float* t4 = target + (size_t)col * h;
  const int n4 = h >> 2;
  const bool stream = (long long)w * h >= DN_STREAM_MIN_ELEMS;
  float4 v[NV];
  float m = -FLT_MAX;
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int j = lane + k * 64;
    if (j < n4) {
      v[k] = dn_ld4_rt(c4 + 4 * j, stream);
      m = fmaxf(m, fmaxf(fmaxf(v[k].x, v[k].y), fmaxf(v[k].z, v[k].w)));
    }
  }
  m = wave_max(m);
  float s = 0.f;
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int j = lane + k * 64;
    if (j < n4) {
      v[k].x = softmax_exp(v[k].x - m); v[k].y = softmax_exp(v[k].y - m);
      v[k].z = softmax_exp(v[k].z - m); v[k].w = softmax_exp(v[k].w - m);
      s += (v[k].x + v[k].y) + (v[k].z + v[k].w);
    }
  }
  s = wave_sum(s);
  const float inv = 1.f / s;
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int j = lane + k * 64;
    if (j < n4) {
      const float4 pr = make_float4(v[k].x * inv, v[k].y * inv, v[k].z * inv, v[k].w * inv);
      dn_st4_rt(t4 + 4 * j, pr, stream);
      if (x.labels) {
        const int label = (int)x.labels[col], r0 = 4 * j;
        if (x.grad)
          dn_st4_rt(x.grad + (size_t)col * h + r0,
                    make_float4(pr.x - ((label == r0) ? 1.f : 0.f), pr.y - ((label == r0 + 1) ? 1.f : 0.f),
                                pr.z - ((label == r0 + 2) ? 1.f : 0.f), pr.w - ((label == r0 + 3) ? 1.f : 0.f)),
                    stream);
        if (x.loss && label >= r0 && label < r0 + 4) {
          const float pl = label == r0 ? pr.x : (label == r0 + 1 ? pr.y : (label == r0 + 2 ? pr.z : pr.w));
          x.loss[col] = -logf(pl + x.tiny);
        }
      }
    }
  }
}

// The same for tall columns (1024 < h <= 4096) when there are enough of them: the
// 256 lanes of a workgroup run down CB neighbouring columns at once (NVB 16-byte
// groups per lane and column), so that a load instruction of the workgroup covers
// 4 KiB of one column; maxima and sums meet through LDS.
template <int NVB, int CB, bool STREAM>
__global__ void __launch_bounds__(256) k_col_softmax_blk(const float* mat, float* target, int w, int h, SoftmaxExtras x) {
  __shared__ float red[2][4][CB];
  const int col0 = blockIdx.x * CB;
  const int n4 = h >> 2;
  const int wv = threadIdx.x >> 6;
  float4 v[CB][NVB];
#pragma unroll
  for (int cb = 0; cb < CB; ++cb) {
    const float* c4 = mat + (size_t)(col0 + cb < w ? col0 + cb : w - 1) * h;
#pragma unroll
    for (int k = 0; k < NVB; ++k) {
      const int j = threadIdx.x + k * 256;
      v[cb][k] = j < n4 ? dn_ld4<STREAM>(c4 + 4 * j) : make_float4(-FLT_MAX, -FLT_MAX, -FLT_MAX, -FLT_MAX);
    }
  }
  float m[CB];
#pragma unroll
  for (int cb = 0; cb < CB; ++cb) {
    float t = -FLT_MAX;
#pragma unroll
    for (int k = 0; k < NVB; ++k) t = fmaxf(t, fmaxf(fmaxf(v[cb][k].x, v[cb][k].y), fmaxf(v[cb][k].z, v[cb][k].w)));
    t = wave_max(t);
    if ((threadIdx.x & 63) == 0) red[0][wv][cb] = t;
  }
  __syncthreads();
#pragma unroll
  for (int cb = 0; cb < CB; ++cb) m[cb] = fmaxf(fmaxf(red[0][0][cb], red[0][1][cb]), fmaxf(red[0][2][cb], red[0][3][cb]));
#pragma unroll
  for (int cb = 0; cb < CB; ++cb) {
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < NVB; ++k) {
      const int j = threadIdx.x + k * 256;
      if (j < n4) {
        v[cb][k].x = softmax_exp(v[cb][k].x - m[cb]); v[cb][k].y = softmax_exp(v[cb][k].y - m[cb]);
        v[cb][k].z = softmax_exp(v[cb][k].z - m[cb]); v[cb][k].w = softmax_exp(v[cb][k].w - m[cb]);
        s += (v[cb][k].x + v[cb][k].y) + (v[cb][k].z + v[cb][k].w);
      }
    }
    s = wave_sum(s);
    if ((threadIdx.x & 63) == 0) red[1][wv][cb] = s;
  }
  __syncthreads();
#pragma unroll
  for (int cb = 0; cb < CB; ++cb) {
    const int col = col0 + cb;
    if (col >= w) break;
    const float inv = 1.f / ((red[1][0][cb] + red[1][1][cb]) + (red[1][2][cb] + red[1][3][cb]));
    float* t4 = target + (size_t)col * h;
#pragma unroll
    for (int k = 0; k < NVB; ++k) {
      const int j = threadIdx.x + k * 256;
      if (j < n4) {
        const float4 pr = make_float4(v[cb][k].x * inv, v[cb][k].y * inv, v[cb][k].z * inv, v[cb][k].w * inv);
        dn_st4<STREAM>(t4 + 4 * j, pr);
        if (x.labels) {
          const int label = (int)x.labels[col], r0 = 4 * j;
          if (x.grad)
            dn_st4<STREAM>(x.grad + (size_t)col * h + r0,
                           make_float4(pr.x - ((label == r0) ? 1.f : 0.f), pr.y - ((label == r0 + 1) ? 1.f : 0.f),
                                       pr.z - ((label == r0 + 2) ? 1.f : 0.f), pr.w - ((label == r0 + 3) ? 1.f : 0.f)));
          if (x.loss && label >= r0 && label < r0 + 4) {
            const float pl = label == r0 ? pr.x : (label == r0 + 1 ? pr.y : (label == r0 + 2 ? pr.z : pr.w));
            x.loss[col] = -logf(pl + x.tiny);
          }
        }
      }
    }
  }
}

__global__ void k_softmax_grad(const float* mat, const float* labels, float* target, int w, int h, FastDiv fd) {
  const size_t n = (size_t)w * h;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const uint32_t q = fd_div((uint32_t)i, fd);
    const uint32_t r = (uint32_t)i - q * (uint32_t)h;
    target[i] = mat[i] - (((int)labels[q] == (int)r) ? 1.f : 0.f);
  }
}
// The same with 16-byte groups (h a multiple of 4, aligned operands: a group stays inside its
// column), one group per lane.
template <bool STREAM>
__global__ void __launch_bounds__(256) k_softmax_grad4(const float* mat, const float* labels, float* target, long long n4, int h, FastDiv fd) {
  const long long tid = (long long)blockIdx.x * 256 + threadIdx.x;
  if (tid >= n4) return;
  const uint32_t e = (uint32_t)(4 * tid);
  const uint32_t q = fd_div(e, fd);
  const int r = (int)(e - q * (uint32_t)h), lab = (int)labels[q];
  float4 v = dn_ld4<STREAM>(mat + e);
  v.x -= lab == r ? 1.f : 0.f; v.y -= lab == r + 1 ? 1.f : 0.f; v.z -= lab == r + 2 ? 1.f : 0.f; v.w -= lab == r + 3 ? 1.f : 0.f;
  dn_st4<STREAM>(target + e, v);
}

__global__ void k_softmax_ce(const float* mat, const float* labels, float* target, int w, int h, float tiny) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < w) target[i] = -logf(mat[(size_t)h * i + (int)labels[i]] + tiny);
}

// ------------------------------------------------------------------ row kernels (axis 1)
// 64 rows per workgroup, lanes down the rows, the 4 wavefronts take columns
// j = wave, wave + 4, ... and meet in LDS.  First-occurrence ties and a start
// value taken "before column 0", as in eigenmat/eigenmat.cc:617-731.

// op 0: max, 1: argmax, 2: one-hot row into target, 3: sqsum (target = p*target + mult*sum)
__global__ void __launch_bounds__(256)
k_row_reduce(const float* mat, float* target, int w, int h, int op, float mult, float p) {
  __shared__ float sv[4][64];
  __shared__ int si[4][64];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int row = blockIdx.x * 64 + lane;
  float acc = (op == 3) ? 0.f : -INFINITY;
  int idx = 0;
  if (row < h) {
    for (int j = wv; j < w; j += 4) {
      const float v = mat[(size_t)j * h + row];
      if (op == 3) acc += v * v;
      else if (v > acc) { acc = v; idx = j; }
    }
  }
  sv[wv][lane] = acc;
  si[wv][lane] = idx;
  __syncthreads();
  if (row >= h) return;
  float best = sv[0][lane];
  int bidx = si[0][lane];
  if (op == 3) {
    best = (sv[0][lane] + sv[1][lane]) + (sv[2][lane] + sv[3][lane]);
  } else {
#pragma unroll
    for (int k = 1; k < 4; ++k) {
      const float v = sv[k][lane];
      const int i2 = si[k][lane];
      if (v > best || (v == best && i2 < bidx)) { best = v; bidx = i2; }
    }
  }
  if (op == 0) { if (wv == 0) target[row] = best; }
  else if (op == 1) { if (wv == 0) target[row] = (float)bidx; }
  else if (op == 3) { if (wv == 0) target[row] = (p == 0.f ? 0.f : p * target[row]) + mult * best; }
  else { for (int j = wv; j < w; j += 4) target[(size_t)j * h + row] = (j == bidx) ? 1.f : 0.f; }
}


// ------------------------------------------------------------------ weighted sums (matrix-vector)

// y[j] = beta*y[j] + alpha * sum_i M[i + j*ld] * x[i]   (one output per contiguous column)
template <int TPC>
__global__ void __launch_bounds__(256)
k_gemv_cols(const float* M, int ld, int h, int w, const float* x, float* y, float alpha, float beta) {
  __shared__ float lds4[4];
  COL_SETUP(TPC)
  const bool stream = (long long)w * h >= DN_STREAM_MIN_ELEMS;
  float s = 0.f;
  if (active) for_each_in_col<TPC>(M + (size_t)col * ld, h, lane, [&](int r, float v) { s += x ? v * x[r] : v; }, stream);   // (no weights: a plain sum)
  s = col_combine<TPC, false>(s, lds4);
  if (active && lane == 0) y[col] = (beta == 0.f ? 0.f : beta * y[col]) + alpha * s;
}

// Column reductions of tall matrices with many columns: the 256 lanes of a
// workgroup run down CB neighbouring columns at once, 4 x CB 16-byte loads in
// flight per lane (a 4096-row column is one trip), the weights of the weighted
// sum held in registers across the CB columns.  Requires 16-byte aligned
// columns (M aligned, ld % 4 == 0) and h % 4 == 0.
//   COL_DOT: y[j] = beta*y[j] + alpha * sum_i M(i,j) x[i]    COL_SQSUM: the same over M(i,j)^2
//   COL_MAX: y[j] = max_i M(i,j), starting from -FLT_MAX
//   COL_SUM: COL_DOT with every x[i] = 1, the additions in the same order (so the same bits), no loads of x
enum { COL_DOT = 0, COL_SQSUM = 1, COL_MAX = 2, COL_SUM = 3 };

template <int CB, int OP, bool STREAM>
__global__ void __launch_bounds__(256)
k_colblock(const float* M, int ld, int h, int w, const float* x, float* y, float alpha, float beta) {
  __shared__ float lds[4][CB];
  const int n4 = h >> 2;
  const int col0 = blockIdx.x * CB;
  const float neutral = OP == COL_MAX ? -FLT_MAX : 0.f;
  const float* cp[CB];
#pragma unroll
  for (int cb = 0; cb < CB; ++cb) cp[cb] = M + (size_t)(col0 + cb < w ? col0 + cb : w - 1) * ld;
  float acc[CB];
#pragma unroll
  for (int cb = 0; cb < CB; ++cb) acc[cb] = neutral;
  for (int j0 = threadIdx.x; j0 < n4; j0 += 1024) {
    float4 v[4][CB], xv[4];
    // loads issued column by column, down each column: the workgroup walks its CB
    // neighbouring columns as one sequential range (measured 8% faster than chunk by chunk)
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int j = j0 + 256 * k;
      xv[k] = (OP == COL_DOT && j < n4) ? *reinterpret_cast<const float4*>(x + 4 * j) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int cb = 0; cb < CB; ++cb)
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int j = j0 + 256 * k;
        v[k][cb] = j < n4 ? dn_ld4<STREAM>(cp[cb] + 4 * j) : make_float4(neutral, neutral, neutral, neutral);
      }
#pragma unroll
    for (int k = 0; k < 4; ++k)
#pragma unroll
      for (int cb = 0; cb < CB; ++cb) {
        const float4 t = v[k][cb];
        if (OP == COL_DOT) { acc[cb] += t.x * xv[k].x; acc[cb] += t.y * xv[k].y; acc[cb] += t.z * xv[k].z; acc[cb] += t.w * xv[k].w; }
        else if (OP == COL_SQSUM) { acc[cb] += t.x * t.x; acc[cb] += t.y * t.y; acc[cb] += t.z * t.z; acc[cb] += t.w * t.w; }
        else if (OP == COL_SUM) { acc[cb] += t.x; acc[cb] += t.y; acc[cb] += t.z; acc[cb] += t.w; }
        else acc[cb] = fmaxf(fmaxf(acc[cb], fmaxf(t.x, t.y)), fmaxf(t.z, t.w));
      }
  }
#pragma unroll
  for (int cb = 0; cb < CB; ++cb) {
    const float r = OP == COL_MAX ? wave_max(acc[cb]) : wave_sum(acc[cb]);
    if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6][cb] = r;
  }
  __syncthreads();
  const int cb = threadIdx.x;
  if (cb < CB && col0 + cb < w) {
    const float a = lds[0][cb], b = lds[1][cb], c = lds[2][cb], d = lds[3][cb];
    if (OP == COL_MAX) y[col0 + cb] = fmaxf(fmaxf(a, b), fmaxf(c, d));
    else y[col0 + cb] = (beta == 0.f ? 0.f : beta * y[col0 + cb]) + alpha * ((a + b) + (c + d));
  }
}

// Launches k_colblock when the shape suits it (tall, aligned, enough columns to
// fill the chip with 256-lane workgroups); returns false otherwise.
template <int OP>
static bool colblock_launch(const float* M, int ld, int h, int w, const float* x, float* y, float alpha, float beta) {
  if (h < 1024 || (h & 3) || (ld & 3) || !dn_aligned16(M) || (OP == COL_DOT && !dn_aligned16(x))) return false;
  const int cus = dn_num_cus();
  const bool stream = (long long)w * h >= DN_STREAM_MIN_ELEMS;
  if (w >= 4 * cus && h >= 2048 && stream) {
    // two columns per workgroup: measured against four at 4096 x 4096 (max 12.1 -> 11.1 us, sum of
    // squares 11.9 -> 11.1, sum unchanged at 11.9) and from 3072 x 4096 to 8192 x 8192 (1-4 % faster);
    // columns of 1024 rows keep four (65536 of them: max 40.3 against 45.0 us)
    hipLaunchKernelGGL((k_colblock<2, OP, true>), dim3((w + 1) / 2), dim3(256), 0, dn_stream(), M, ld, h, w, x, y, alpha, beta);
  } else if (w >= 8 * cus) {
    if (stream)
      hipLaunchKernelGGL((k_colblock<4, OP, true>), dim3((w + 3) / 4), dim3(256), 0, dn_stream(), M, ld, h, w, x, y, alpha, beta);
    else
      hipLaunchKernelGGL((k_colblock<4, OP, false>), dim3((w + 3) / 4), dim3(256), 0, dn_stream(), M, ld, h, w, x, y, alpha, beta);
  } else if (w >= 4 * cus) {
    hipLaunchKernelGGL((k_colblock<2, OP, false>), dim3((w + 1) / 2), dim3(256), 0, dn_stream(), M, ld, h, w, x, y, alpha, beta);
  } else {
    return false;
  }
  return true;
}

// Two-stage reduction along rows (over the columns j of M[i + j*ld]), for
//   ROW_DOT:   sum_j M(i,j) * x[j]      ROW_SQSUM: sum_j M(i,j)^2      ROW_MAX: max_j M(i,j)
// Stage 1: workgroup (bx, by) reduces columns [by*cps, (by+1)*cps) for rows
// 256*bx .. 256*bx+255 when VEC (4 rows per lane, one 16-byte load per column)
// or 64*bx .. 64*bx+63 otherwise; its 4 wavefronts take every 4th column, four
// loads in flight each, and meet in LDS.  With one split the result is final.
//   ROW_SUM:   ROW_DOT with every x[j] = 1 (the same additions in the same order)
enum { ROW_DOT = 0, ROW_SQSUM = 1, ROW_MAX = 2, ROW_SUM = 3 };


template <int OP>
__device__ __forceinline__ float row_combine(float a, float b) { return OP == ROW_MAX ? fmaxf(a, b) : a + b; }

// y = finish(y_old, s): DOT: beta*y + alpha*s; SQSUM: beta*y + alpha*s; MAX: s.
template <int OP>
__device__ __forceinline__ float row_finish(float yold, float s, float alpha, float beta) {
  if (OP == ROW_MAX) return s;
  return rowsum_finish(yold, s, alpha, beta);
}

template <bool VEC, int OP, int NW, int U, bool STREAM>
__global__ void __launch_bounds__(NW * 64)
k_rows_stage1(const float* M, int ld, int h, int w, int cps, const float* x, float* y, float* partial, float alpha,
              float beta) {
  constexpr int RPL = VEC ? 4 : 1;
  __shared__ float sv[NW][64 * RPL];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int row0 = (blockIdx.x * 64 + lane) * RPL;
  const int j0 = blockIdx.y * cps;
  const int j1 = (j0 + cps < w) ? j0 + cps : w;
  const float init = OP == ROW_MAX ? -INFINITY : 0.f;
  float acc[RPL];
#pragma unroll
  for (int k = 0; k < RPL; ++k) acc[k] = init;
  auto take = [&](int k, float v, float xj) {
    if (OP == ROW_DOT) acc[k] += v * xj;
    else if (OP == ROW_SQSUM) acc[k] += v * v;
    else if (OP == ROW_SUM) acc[k] += v;
    else acc[k] = fmaxf(acc[k], v);
  };
  if (row0 < h) {
    // U columns of this wavefront in flight per trip; a column past the range is
    // read as the neutral element
    for (int j = j0 + wv; j < j1; j += NW * U) {
      float xs[U];
      if constexpr (VEC) {
        float4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int jj = j + NW * u;
          if (jj < j1) {
            v[u] = dn_ld4<STREAM>(M + (size_t)jj * ld + row0);
            xs[u] = OP == ROW_DOT ? x[jj] : 0.f;
          } else {
            v[u] = make_float4(init, init, init, init);
            xs[u] = 0.f;
          }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) { take(0, v[u].x, xs[u]); take(1, v[u].y, xs[u]); take(2, v[u].z, xs[u]); take(3, v[u].w, xs[u]); }
      } else {
        float v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int jj = j + NW * u;
          if (jj < j1) {
            v[u] = M[(size_t)jj * ld + row0];
            xs[u] = OP == ROW_DOT ? x[jj] : 0.f;
          } else {
            v[u] = init;
            xs[u] = 0.f;
          }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) take(0, v[u], xs[u]);
      }
    }
  }
#pragma unroll
  for (int k = 0; k < RPL; ++k) sv[wv][lane * RPL + k] = acc[k];
  __syncthreads();
  for (int r = threadIdx.x; r < 64 * RPL; r += NW * 64) {
    const int row = blockIdx.x * 64 * RPL + r;
    if (row < h) {
      float s = sv[0][r];
#pragma unroll
      for (int k = 1; k < NW; ++k) s = row_combine<OP>(s, sv[k][r]);
      if (partial) partial[(size_t)blockIdx.y * h + row] = s;
      else y[row] = row_finish<OP>(y[row], s, alpha, beta);
    }
  }
}

// Stage 2: a lane owns RPL neighbouring rows (one 16-byte load per split when
// VEC), the 4 wavefronts of a workgroup take every 4th split, 8 loads in flight,
// and meet in LDS; the order of the additions is fixed.
template <bool VEC, int OP>
__global__ void __launch_bounds__(256)
k_rows_stage2(const float* partial, int splits, int h, float* y, float alpha, float beta) {
  constexpr int RPL = VEC ? 4 : 1;
  __shared__ float sv[4][64 * RPL];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int row0 = (blockIdx.x * 64 + lane) * RPL;
  const float init = OP == ROW_MAX ? -INFINITY : 0.f;
  float acc[RPL];
#pragma unroll
  for (int k = 0; k < RPL; ++k) acc[k] = init;
  if (row0 < h) {
    for (int s = wv; s < splits; s += 32) {
      if constexpr (VEC) {
        float4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int ss = s + 4 * u;
          v[u] = ss < splits ? *reinterpret_cast<const float4*>(partial + (size_t)ss * h + row0)
                             : make_float4(init, init, init, init);
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          acc[0] = row_combine<OP>(acc[0], v[u].x); acc[1] = row_combine<OP>(acc[1], v[u].y);
          acc[2] = row_combine<OP>(acc[2], v[u].z); acc[3] = row_combine<OP>(acc[3], v[u].w);
        }
      } else {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int ss = s + 4 * u;
          v[u] = ss < splits ? partial[(size_t)ss * h + row0] : init;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) acc[0] = row_combine<OP>(acc[0], v[u]);
      }
    }
  }
#pragma unroll
  for (int k = 0; k < RPL; ++k) sv[wv][lane * RPL + k] = acc[k];
  __syncthreads();
  for (int r = threadIdx.x; r < 64 * RPL; r += 256) {
    const int row = blockIdx.x * 64 * RPL + r;
    if (row < h) {
      const float s = row_combine<OP>(row_combine<OP>(sv[0][r], sv[1][r]), row_combine<OP>(sv[2][r], sv[3][r]));
      y[row] = row_finish<OP>(y[row], s, alpha, beta);
    }
  }
}

// One launch for 16-byte aligned operands: a workgroup owns 64 rows (16 lanes x 4 rows,
// the 4 lane groups of a wavefront on 4 neighbouring columns: 256-byte runs) and the
// columns [by*cps, (by+1)*cps); NW wavefronts x U loads in flight.  With more than one
// column slice (at most ROWS_ONE_MAX_SPLITS, chosen so that about one workgroup per CU
// runs) a workgroup publishes its 64 partial results and counts itself in; the one that
// arrives last adds the slices up in slice order, so the result does not depend on the
// order of arrival.  Partials travel as agent-scope atomic stores and loads (they bypass
// the non-coherent cache levels; a release fence per wavefront was measured 5-10x slower
// than the whole kernel), the counter returns to zero for the next launch.
#define ROWS_ONE_MAX_SPLITS 8

template <int OP, int NW, int U, bool STREAM>
__global__ void __launch_bounds__(NW * 64)
k_rows_one(const float* M, int ld, int h, int w, int cps, const float* x, float* y, float* partial,
           unsigned* counters, float alpha, float beta) {
  __shared__ float sv[NW][64];
  __shared__ int s_last;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int r = lane & 15, c = lane >> 4;
  const int row0 = (blockIdx.x * 16 + r) * 4;
  const int j0 = blockIdx.y * cps;
  const int j1 = (j0 + cps < w) ? j0 + cps : w;
  const float init = OP == ROW_MAX ? -INFINITY : 0.f;
  float acc[4] = {init, init, init, init};
  auto take = [&](int k, float v, float xj) {
    if (OP == ROW_DOT) acc[k] += v * xj;
    else if (OP == ROW_SQSUM) acc[k] += v * v;
    else if (OP == ROW_SUM) acc[k] += v;
    else acc[k] = fmaxf(acc[k], v);
  };
  if (row0 < h) {
    for (int j = j0 + wv * 4 + c; j < j1; j += NW * 4 * U) {
      float4 v[U];
      float xs[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int jj = j + NW * 4 * u;
        if (jj < j1) {
          v[u] = dn_ld4<STREAM>(M + (size_t)jj * ld + row0);
          xs[u] = OP == ROW_DOT ? x[jj] : 0.f;
        } else {
          v[u] = make_float4(init, init, init, init);
          xs[u] = 0.f;
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) { take(0, v[u].x, xs[u]); take(1, v[u].y, xs[u]); take(2, v[u].z, xs[u]); take(3, v[u].w, xs[u]); }
    }
  }
#pragma unroll
  for (int o = 16; o < 64; o <<= 1)
#pragma unroll
    for (int k = 0; k < 4; ++k) acc[k] = row_combine<OP>(acc[k], __shfl_xor(acc[k], o, WAVE));
  if (c == 0) *reinterpret_cast<float4*>(&sv[wv][r * 4]) = make_float4(acc[0], acc[1], acc[2], acc[3]);
  __syncthreads();
  const int splits = gridDim.y;
  const int row = blockIdx.x * 64 + (int)threadIdx.x;
  const bool mine = threadIdx.x < 64 && row < h;
  if (mine) {
    float s = sv[0][threadIdx.x];
#pragma unroll
    for (int k = 1; k < NW; ++k) s = row_combine<OP>(s, sv[k][threadIdx.x]);
    if (splits == 1) y[row] = row_finish<OP>(y[row], s, alpha, beta);
    else __hip_atomic_store(partial + (size_t)blockIdx.y * h + row, s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  if (splits == 1) return;
  __builtin_amdgcn_s_waitcnt(0);   // the stores of this wavefront have been acknowledged
  __syncthreads();
  if (threadIdx.x == 0) {
    const unsigned old = __hip_atomic_fetch_add(counters + blockIdx.x, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    s_last = (old == (unsigned)splits - 1u);
    if (s_last) __hip_atomic_store(counters + blockIdx.x, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();
  if (!s_last || !mine) return;
  float pv[ROWS_ONE_MAX_SPLITS];
#pragma unroll
  for (int k = 0; k < ROWS_ONE_MAX_SPLITS; ++k)
    pv[k] = k < splits ? __hip_atomic_load(partial + (size_t)k * h + row, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : init;
  float t = pv[0];
#pragma unroll
  for (int k = 1; k < ROWS_ONE_MAX_SPLITS; ++k)
    if (k < splits) t = row_combine<OP>(t, pv[k]);
  y[row] = row_finish<OP>(y[row], t, alpha, beta);
}

// Workspace of k_rows_one: slice partials and one arrival counter per 64-row block.
struct RowsWorkspace {
  float* partial;      // room for partial_floats floats
  size_t partial_floats;
  unsigned* counters;  // zero between launches
  int num_counters;
};

// Number of column slices for the one-launch kernel: about one workgroup per CU, a slice
// at least 256 columns wide.  0 when that would take more than ROWS_ONE_MAX_SPLITS slices
// (few rows, very many columns): such shapes keep the two-stage kernels.
static int rows_one_splits(int h, int w) {
  const int bx = (h + 63) / 64;
  const int cus = dn_num_cus();
  int splits = (cus + bx / 2) / bx;
  if (splits > w / 256) splits = w / 256;
  if (splits < 1) splits = 1;
  if (splits > ROWS_ONE_MAX_SPLITS) return 0;
  // A few workgroups more than CUs double the time of the busiest CU (65 row blocks x 4 slices on
  // 256 CUs: 22.4 us where 64 x 4 take 13.3): among the slice counts allowed, take the one with
  // the smallest (workgroups on the busiest CU) x (columns per workgroup).
  if (bx * splits > cus) {
    long long best = -1;
    int best_s = splits;
    for (int s = 1; s <= ROWS_ONE_MAX_SPLITS && s <= (w / 256 > 1 ? w / 256 : 1); ++s) {
      const long long cost = (long long)((bx * s + cus - 1) / cus) * ((w + s - 1) / s);
      if (best < 0 || cost < best) { best = cost; best_s = s; }
    }
    splits = best_s;
  }
  return splits;
}

__global__ void k_fill_u32(unsigned* p, int n, unsigned v);

// The arrival counters are zero between launches because every launch returns them to zero.  A
// launch that the runtime reports as failed may not have done so: clear them with a kernel (best
// effort; on a device that has gone away this fails like everything after it).
static void rezero_counters(unsigned* counters, int n) {
  if (!counters || n <= 0 || dn_capturing()) return;
  hipGetLastError();
  hipLaunchKernelGGL(k_fill_u32, dim3((n + 255) / 256), dim3(256), 0, dn_stream(), counters, n, 0u);
  hipGetLastError();
}

template <int OP>
static int rows_reduce_one(const float* M, int ld, int h, int w, const float* x, float* y, float alpha, float beta,
                           const RowsWorkspace& ws) {
  const int bx = (h + 63) / 64;
  int splits = rows_one_splits(h, w);
  if (splits > 1 && (bx > ws.num_counters || (size_t)splits * h > ws.partial_floats)) return ERROR_GENERIC;
  const int cps = (w + splits - 1) / splits;
  splits = (w + cps - 1) / cps;
  dim3 grid(bx, splits);
  const bool stream = (long long)w * h >= DN_STREAM_MIN_ELEMS;
  if (cps <= 64)
    hipLaunchKernelGGL((k_rows_one<OP, 4, 4, false>), grid, dim3(256), 0, dn_stream(), M, ld, h, w, cps, x, y, ws.partial, ws.counters, alpha, beta);
  else if ((long long)w * h <= (1 << 18))   // layer states (a few hundred units x a batch): 256 lanes start sooner than 1024
    hipLaunchKernelGGL((k_rows_one<OP, 4, 8, false>), grid, dim3(256), 0, dn_stream(), M, ld, h, w, cps, x, y, ws.partial, ws.counters, alpha, beta);
  else if (stream)
    hipLaunchKernelGGL((k_rows_one<OP, 16, 8, true>), grid, dim3(1024), 0, dn_stream(), M, ld, h, w, cps, x, y, ws.partial, ws.counters, alpha, beta);
  else
    hipLaunchKernelGGL((k_rows_one<OP, 16, 8, false>), grid, dim3(1024), 0, dn_stream(), M, ld, h, w, cps, x, y, ws.partial, ws.counters, alpha, beta);
  const int status = dn_launch_status();
  if (status && splits > 1) rezero_counters(ws.counters, bx);
  return status;
}

static inline bool rows_one_ok(const float* M, int ld, int h) {
  return dn_aligned16(M) && (ld % 4 == 0) && (h % 4 == 0);
}

// The library's own workspace: arrival counters for 16384 row blocks (matrices with more rows
// than that have no column slices), partials from the grow-only scratch.
static int rows_workspace(int h, int w, RowsWorkspace* ws) {
  const int kCounters = 16384;
  ws->partial = nullptr; ws->partial_floats = 0; ws->counters = nullptr; ws->num_counters = 0;
  const int splits = rows_one_splits(h, w);
  if (splits == 1) return 0;
  unsigned* counters = dn_zero_words(kCounters);
  if (!counters) return CUDA_ERROR;
  ws->partial = (float*)dn_scratch((size_t)splits * h * sizeof(float));
  if (!ws->partial) return CUDA_ERROR;
  ws->partial_floats = (size_t)splits * h;
  ws->counters = counters;
  ws->num_counters = kCounters;
  return 0;
}

template <int OP>
static int rows_reduce(const float* M, int ld, int h, int w, const float* x, float* y, float alpha, float beta) {
  if (h <= 0) return 0;
  if (rows_one_ok(M, ld, h) && rows_one_splits(h, w) > 0) {
    RowsWorkspace ws;
    if (int e = rows_workspace(h, w, &ws)) return e;
    return rows_reduce_one<OP>(M, ld, h, w, x, y, alpha, beta, ws);
  }
  const bool vec = rows_one_ok(M, ld, h) && h >= 1024;
  const int rows_per_block = vec ? 256 : 64;
  const int bx = (h + rows_per_block - 1) / rows_per_block;
  int splits = (8 * dn_num_cus()) / bx;
  if (splits > (w + 63) / 64) splits = (w + 63) / 64;
  if (w <= 128) splits = 1;   // (layer states of up to 128 cases: the rows alone fill the chip, one launch)
  if (splits < 1 || (size_t)h * w <= (1u << 18)) splits = 1;   // small: one launch beats two
  int cps = (w + splits - 1) / splits;
  if (cps < 1) cps = 1;
  splits = w > 0 ? (w + cps - 1) / cps : 1;
  float* partial = nullptr;
  if (splits > 1) {
    partial = (float*)dn_scratch((size_t)splits * h * sizeof(float));
    if (!partial) return CUDA_ERROR;
  }
  dim3 grid(bx, splits);
  if (vec) {
    // 8 wavefronts x 8 columns in flight: a 64-column slice is one trip
    if (cps > 16 && (long long)w * h >= DN_STREAM_MIN_ELEMS)
      hipLaunchKernelGGL((k_rows_stage1<true, OP, 8, 8, true>), grid, dim3(512), 0, dn_stream(), M, ld, h, w, cps, x, y, partial, alpha, beta);
    else if (cps > 16)
      hipLaunchKernelGGL((k_rows_stage1<true, OP, 8, 8, false>), grid, dim3(512), 0, dn_stream(), M, ld, h, w, cps, x, y, partial, alpha, beta);
    else
      hipLaunchKernelGGL((k_rows_stage1<true, OP, 4, 4, false>), grid, dim3(256), 0, dn_stream(), M, ld, h, w, cps, x, y, partial, alpha, beta);
  } else {
    hipLaunchKernelGGL((k_rows_stage1<false, OP, 4, 4, false>), grid, dim3(256), 0, dn_stream(), M, ld, h, w, cps, x, y, partial, alpha, beta);
  }
  if (splits > 1) {
    if (h % 4 == 0)
      hipLaunchKernelGGL((k_rows_stage2<true, OP>), dim3((h + 255) / 256), dim3(256), 0, dn_stream(), (const float*)partial, splits,
                         h, y, alpha, beta);
    else
      hipLaunchKernelGGL((k_rows_stage2<false, OP>), dim3((h + 63) / 64), dim3(256), 0, dn_stream(), (const float*)partial, splits,
                         h, y, alpha, beta);
  }
  return dn_launch_status();
}

// ------------------------------------------------------------------ several row sums in one launch
// y += alpha * rowsums(M) for up to two vectors y with up to two matrices each, applied in the
// order given (the bias statistics of a contrastive-divergence step: bv += eps * sums(v);
// bv -= eps * sums(v'); bh += eps * sums(h); bh -= eps * sums(h'), cudamat/examples/rbm_cudamat.py:
// 75-76, 85-86).  Every sum is taken in the order of k_rows_one<ROW_SUM, 4, ., false> with one
// column slice (lane groups on neighbouring columns, four wavefronts, fixed order in LDS) and
// finished by the same expression, so the results have the bits of the separate launches.
__global__ void __launch_bounds__(256) k_rows_sum_jobs(RowSumJobs J) { rows_sum_jobs_body(J, (int)blockIdx.x); }

// Whether sums along the rows of this h x w matrix run as k_rows_one<ROW_SUM, 4, ., false> with one column slice.
bool dn_row_sum_job_ok(const float* M, int h, int w) {
  if (h <= 0 || w <= 0 || !rows_one_ok(M, h, h) || rows_one_splits(h, w) != 1) return false;
  return w <= 64 || (long long)w * h <= (1 << 18);
}
// 1: as above; 2: rows that do not come in aligned groups of four, small enough for rows_reduce() to take
// k_rows_stage1<false, ROW_SUM, 4, 4, false> with one column slice; 0: neither.
int dn_row_sum_job_kind(const float* M, int h, int w) {
  if (dn_row_sum_job_ok(M, h, w)) return 1;
  if (h <= 0 || w <= 0 || rows_one_ok(M, h, h)) return 0;
  return (long long)w * h <= (1 << 18) ? 2 : 0;
}

// jobs in call order: at most two different y, at most two jobs each (the caller has checked that)
int dn_row_sum_jobs(const DnRowSumJob* jobs, int n) {
  RowSumJobs J;
  const int blocks = rows_sum_jobs_table(jobs, n, &J);
  if (blocks < 0) return ERROR_GENERIC;
  if (blocks == 0) return 0;
  hipLaunchKernelGGL(k_rows_sum_jobs, dim3(blocks), dim3(256), 0, dn_stream(), J);
  return dn_launch_status();
}

// ------------------------------------------------------------------ reductions that allocate nothing
// A fixed workspace for k_rows_one inside the code object, for callers that may not
// allocate (HIP graph capture, serving loops): room for NOALLOC_PARTIAL_FLOATS slice
// partials and NOALLOC_COUNTERS arrival counters.  Every GPU holds its own copy of the
// array at its own address; the address is looked up once per device.
#define NOALLOC_PARTIAL_FLOATS 65536
#define NOALLOC_COUNTERS 1024
#define NOALLOC_MAX_DEVICES 16
static __device__ __align__(256) unsigned char scratch[(NOALLOC_PARTIAL_FLOATS + NOALLOC_COUNTERS) * 4];
static unsigned char* g_noalloc_ptr[NOALLOC_MAX_DEVICES] = {nullptr};

__global__ void k_fill_u32(unsigned* p, int n, unsigned v) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}

// Looks up the current device's copy of the workspace and clears its counters (with a
// kernel, not a memset: a memset node must not end up in a caller's graph).
int dn_noalloc_setup() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return CUDA_ERROR;
  if (dev < 0 || dev >= NOALLOC_MAX_DEVICES) return ERROR_UNSUPPORTED;
  if (g_noalloc_ptr[dev]) return 0;
  unsigned char* ptr = nullptr;
  if (hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return CUDA_ERROR;
  hipLaunchKernelGGL(k_fill_u32, dim3((NOALLOC_COUNTERS + 255) / 256), dim3(256), 0, dn_stream(),
                     reinterpret_cast<unsigned*>(ptr + (size_t)NOALLOC_PARTIAL_FLOATS * 4), NOALLOC_COUNTERS, 0u);
  if (dn_launch_status()) return CUDA_ERROR;
  g_noalloc_ptr[dev] = ptr;
  return 0;
}

// Host entry points used by dot() for vector-shaped products.
int dn_gemv_cols(const float* M, int ld, int h, int w, const float* x, float* y, float alpha, float beta) {
  if (w <= 0) return 0;
  if (x && colblock_launch<COL_DOT>(M, ld, h, w, x, y, alpha, beta)) return dn_launch_status();   // (x NULL: plain sums)
  const int cus = dn_num_cus();
  if (w < cus * 2 && h >= 4096) {
    hipLaunchKernelGGL((k_gemv_cols<256>), dim3(w), dim3(256), 0, dn_stream(), M, ld, h, w, x, y, alpha, beta);
  } else {
    hipLaunchKernelGGL((k_gemv_cols<64>), dim3((w + 3) / 4), dim3(256), 0, dn_stream(), M, ld, h, w, x, y, alpha, beta);
  }
  return dn_launch_status();
}

int dn_gemv_rows(const float* M, int ld, int h, int w, const float* x, float* y, float alpha, float beta) {
  return rows_reduce<ROW_DOT>(M, ld, h, w, x, y, alpha, beta);
}

// ------------------------------------------------------------------ flat dot / norm

// Sum of a[i] * b[i] over everything, returned to the host.  One launch: a workgroup sums
// a grid-stride slice (fp32 per lane over four independent chains, fp64 across lanes and
// workgroups; 16-byte loads when VEC, four of each operand in flight), publishes its partial
// sum and counts itself in; the one that arrives last adds the partials in block order, so
// the result does not depend on the order of arrival, and writes {value, tag} as one 8-byte
// word into pinned host memory.  The counters (one of groups, then one per group of
// workgroups) return to zero for the next launch.
#define DOT_U 4
#define DOT_GROUP 32
#define DOT_COUNTER_PITCH 64   // words between two counters: every counter in a memory line of its own
// MODE 0: two operands; 1: b is a; 2: b is all ones and is not read (the products keep their
// operand's bits, so the sum has the bits of a product with a stored vector of ones).
template <bool VEC, bool STREAM, int MODE>
__global__ void __launch_bounds__(256)
k_dot_one(const float* a, const float* b, long long n, double* partial, unsigned* counter,
          unsigned long long* result, unsigned tag, int take_sqrt) {
  __shared__ double lds[4];
  __shared__ int s_last;
  const long long stride = (long long)gridDim.x * 256;
  float s[DOT_U] = {0.f, 0.f, 0.f, 0.f};
  if (VEC) {
    const long long n4 = n >> 2;
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n4; i += DOT_U * stride) {
      float4 x[DOT_U], y[DOT_U];
#pragma unroll
      for (int u = 0; u < DOT_U; ++u) {
        const long long j = i + u * stride;
        const bool ok = j < n4;
        x[u] = ok ? dn_ld4<STREAM>(a + 4 * j) : make_float4(0.f, 0.f, 0.f, 0.f);
        y[u] = MODE == 1 ? x[u] : MODE == 2 ? make_float4(1.f, 1.f, 1.f, 1.f) : ok ? dn_ld4<STREAM>(b + 4 * j) : make_float4(0.f, 0.f, 0.f, 0.f);
      }
#pragma unroll
      for (int u = 0; u < DOT_U; ++u) s[u] += (x[u].x * y[u].x + x[u].y * y[u].y) + (x[u].z * y[u].z + x[u].w * y[u].w);
    }
    if (blockIdx.x == 0 && (long long)threadIdx.x < n - 4 * n4) s[0] += a[4 * n4 + threadIdx.x] * (MODE == 2 ? 1.f : b[4 * n4 + threadIdx.x]);
  } else {
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += DOT_U * stride) {
      float x[DOT_U], y[DOT_U];
#pragma unroll
      for (int u = 0; u < DOT_U; ++u) {
        const long long j = i + u * stride;
        x[u] = j < n ? a[j] : 0.f;
        y[u] = MODE == 1 ? x[u] : MODE == 2 ? 1.f : j < n ? b[j] : 0.f;
      }
#pragma unroll
      for (int u = 0; u < DOT_U; ++u) s[u] += x[u] * y[u];
    }
  }
  double t = wave_sum_d(((double)s[0] + (double)s[1]) + ((double)s[2] + (double)s[3]));
  if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = t;
  __syncthreads();
  const int nblocks = gridDim.x;
  if (threadIdx.x == 0) {
    t = (lds[0] + lds[1]) + (lds[2] + lds[3]);
    if (nblocks == 1) {
      s_last = 1;
      lds[0] = t;
    } else {
      __hip_atomic_store(partial + blockIdx.x, t, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __builtin_amdgcn_s_waitcnt(0);   // the store has been acknowledged
      // Arrivals at one address are served one after the other (about 15 ns each), so the
      // workgroups count themselves in by groups of DOT_GROUP and only the last of a group
      // goes on to the counter of groups.
      const int g = blockIdx.x / DOT_GROUP;
      const int ng = (nblocks + DOT_GROUP - 1) / DOT_GROUP;
      const int gsize = nblocks - g * DOT_GROUP < DOT_GROUP ? nblocks - g * DOT_GROUP : DOT_GROUP;
      int last = 0;
      if (__hip_atomic_fetch_add(counter + DOT_COUNTER_PITCH * (1 + g), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == (unsigned)gsize - 1u) {
        __hip_atomic_store(counter + DOT_COUNTER_PITCH * (1 + g), 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (__hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == (unsigned)ng - 1u) {
          __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          last = 1;
        }
      }
      s_last = last;
    }
  }
  __syncthreads();
  if (!s_last) return;
  if (nblocks > 1) {
    // (atomic loads would be served one at a time; after the fence plain loads see what the
    // other workgroups' acknowledged stores left at the device's point of coherence)
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    double p = 0.0;
    for (int i = threadIdx.x; i < nblocks; i += 256) p += partial[i];
    p = wave_sum_d(p);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = p;
    __syncthreads();
    if (threadIdx.x == 0) lds[0] = (lds[0] + lds[1]) + (lds[2] + lds[3]);
  }
  if (threadIdx.x == 0) {
    const float v = (float)(take_sqrt ? sqrt(lds[0]) : lds[0]);
    __hip_atomic_store(result, ((unsigned long long)tag << 32) | __float_as_uint(v), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_SYSTEM);
  }
}

// The host's side of the result word: pinned memory that the kernel writes directly, so a
// scalar result costs no copy call.  The host polls the word for this call's tag for a
// while (a result of a short kernel arrives within microseconds) and otherwise waits for
// the stream.
static unsigned long long* g_result_host = nullptr;
static unsigned long long* g_result_dev = nullptr;
static unsigned g_result_tag = 0;

static bool result_word() {
  if (g_result_host) return true;
  void* h = nullptr;
  void* d = nullptr;
  if (hipHostMalloc(&h, 64, hipHostMallocCoherent | hipHostMallocMapped) != hipSuccess) { hipGetLastError(); return false; }
  if (hipHostGetDevicePointer(&d, h, 0) != hipSuccess) { hipGetLastError(); hipHostFree(h); return false; }
  g_result_host = (unsigned long long*)h;
  g_result_dev = (unsigned long long*)d;
  *g_result_host = 0ull;
  return true;
}

#define DOT_POLLS (1 << 16)
static int flat_dot(const float* a, const float* b, long long n, int take_sqrt, float* result) {
  *result = 0.f;
  if (dn_capturing()) return ERROR_UNSUPPORTED;        // the result is read back: nothing to record
  if (n <= 0) return 0;
  const bool vec = dn_aligned16(a) && (!b || dn_aligned16(b)) && n >= 1024;   // b == nullptr: a vector of ones
  long long nb = (n + (vec ? 4095 : 1023)) / (vec ? 4096 : 1024);
  const long long cap = (long long)dn_num_cus() * 2;   // (more workgroups: more arrivals; 4 per CU cost 2 us at 4096 x 4096)
  if (nb > cap) nb = cap;
  double* partial = (double*)dn_scratch((size_t)nb * sizeof(double));
  unsigned* counter = dn_zero_words(DOT_COUNTER_PITCH * (1 + (int)((nb + DOT_GROUP - 1) / DOT_GROUP)));
  if (!partial || !counter || !result_word()) return CUDA_ERROR;
  const unsigned tag = ++g_result_tag ? g_result_tag : ++g_result_tag;   // never 0, the word's first content
  const dim3 grid((unsigned)nb), block(256);
#define DOT_GO(VEC, STREAM, MODE) \
  hipLaunchKernelGGL((k_dot_one<VEC, STREAM, MODE>), grid, block, 0, dn_stream(), a, b, n, partial, counter, g_result_dev, tag, take_sqrt)
#define DOT_SAME(VEC, STREAM) do { if (a == b) DOT_GO(VEC, STREAM, 1); else if (!b) DOT_GO(VEC, STREAM, 2); else DOT_GO(VEC, STREAM, 0); } while (0)
  if (vec && n >= DN_STREAM_MIN_ELEMS) DOT_SAME(true, true);
  else if (vec) DOT_SAME(true, false);
  else DOT_SAME(false, false);
#undef DOT_SAME
#undef DOT_GO
  const int n_counters = DOT_COUNTER_PITCH * (1 + (int)((nb + DOT_GROUP - 1) / DOT_GROUP));
  if (hipGetLastError() != hipSuccess) { rezero_counters(counter, n_counters); return CUDA_ERROR; }
  unsigned long long word = 0;
  for (int i = 0; i < DOT_POLLS; ++i) {
    word = __atomic_load_n(g_result_host, __ATOMIC_ACQUIRE);
    if ((unsigned)(word >> 32) == tag) break;
  }
  if ((unsigned)(word >> 32) != tag) {
    if (hipStreamSynchronize(dn_stream()) != hipSuccess) { rezero_counters(counter, n_counters); return CUDA_ERROR; }
    word = __atomic_load_n(g_result_host, __ATOMIC_ACQUIRE);
    if ((unsigned)(word >> 32) != tag) { rezero_counters(counter, n_counters); return CUDA_ERROR; }
  }
  const unsigned bits = (unsigned)word;
  memcpy(result, &bits, sizeof(float));
  return 0;
}

// ------------------------------------------------------------------ C ABI

template <class K64, class K256, class... Args>
static int launch_cols(K64 k64, K256 k256, int w, int h, Args... args) {
  if (w <= 0) return 0;
  if (w < dn_num_cus() * 2 && h >= 4096)
    hipLaunchKernelGGL(k256, dim3(w), dim3(256), 0, dn_stream(), args...);
  else
    hipLaunchKernelGGL(k64, dim3((w + 3) / 4), dim3(256), 0, dn_stream(), args...);
  return dn_launch_status();
}

static inline int check_axis_common(const cudamat* mat, const cudamat* target) {
  if (!mat->on_device || !target->on_device) return ERROR_NOT_ON_DEVICE;
  if (mat->is_trans) return ERROR_TRANSPOSED;
  return 0;
}

extern "C" {

int max_by_axis(cudamat* mat, cudamat* target, int axis) {
  const int h = mat->size[0], w = mat->size[1];
  if (int e = check_axis_common(mat, target)) return e;
  if (axis == 0) {
    if (target->size[0] != 1 || target->size[1] != w) return ERROR_INCOMPATIBLE_DIMENSIONS;
    if (w > 0 && colblock_launch<COL_MAX>(mat->data_device, h, h, w, nullptr, target->data_device, 1.f, 0.f))
      return dn_launch_status();
    return launch_cols(k_col_max<64>, k_col_max<256>, w, h, (const float*)mat->data_device, target->data_device, w, h);
  } else if (axis == 1) {
    if (target->size[0] != h || target->size[1] != 1) return ERROR_INCOMPATIBLE_DIMENSIONS;
    if (w <= 0) return 0;
    return rows_reduce<ROW_MAX>(mat->data_device, h, h, w, nullptr, target->data_device, 1.f, 0.f);
  }
  return ERROR_UNSUPPORTED;
}

// max_by_axis without any allocation (no counterpart in cudamat.cu; for callers that cannot
// allocate device memory).  Same kernels and the same results as max_by_axis; the slice
// partials and arrival counters of the axis-1 kernel live in this library's fixed workspace
// instead of the grow-only scratch.  Returns ERROR_UNSUPPORTED when a call would need more
// than NOALLOC_PARTIAL_FLOATS partials or NOALLOC_COUNTERS row blocks of 64 rows with
// column slices.  Calls that overlap on one GPU (different streams or threads) race on the
// workspace; its counters are zero between calls.
int max_by_axis_noalloc(cudamat* mat, cudamat* target, int axis) {
  const int h = mat->size[0], w = mat->size[1];
  if (int e = check_axis_common(mat, target)) return e;
  if (axis == 0) {
    if (target->size[0] != 1 || target->size[1] != w) return ERROR_INCOMPATIBLE_DIMENSIONS;
    if (w > 0 && colblock_launch<COL_MAX>(mat->data_device, h, h, w, nullptr, target->data_device, 1.f, 0.f))
      return dn_launch_status();
    return launch_cols(k_col_max<64>, k_col_max<256>, w, h, (const float*)mat->data_device, target->data_device, w, h);
  }
  if (axis != 1) return ERROR_UNSUPPORTED;
  if (target->size[0] != h || target->size[1] != 1) return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (w <= 0 || h <= 0) return 0;
  const float* M = mat->data_device;
  if (!rows_one_ok(M, h, h) || rows_one_splits(h, w) == 0) {
    // unaligned operand, or few rows and very many columns: the 64-row kernel over all columns,
    // one launch and no partials
    hipLaunchKernelGGL((k_rows_stage1<false, ROW_MAX, 4, 4, false>), dim3((h + 63) / 64, 1), dim3(256), 0, dn_stream(), M, h, h, w,
                       w, (const float*)nullptr, target->data_device, (float*)nullptr, 1.f, 0.f);
    return dn_launch_status();
  }
  RowsWorkspace ws = {nullptr, 0, nullptr, 0};
  const int splits = rows_one_splits(h, w);
  if (splits > 1) {
    if ((size_t)splits * h > NOALLOC_PARTIAL_FLOATS || (h + 63) / 64 > NOALLOC_COUNTERS) return ERROR_UNSUPPORTED;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return CUDA_ERROR;
    if (dev < 0 || dev >= NOALLOC_MAX_DEVICES) return ERROR_UNSUPPORTED;
    if (!g_noalloc_ptr[dev])
      if (int e = dn_noalloc_setup()) return e;
    unsigned char* ptr = g_noalloc_ptr[dev];
    ws.partial = reinterpret_cast<float*>(ptr);
    ws.partial_floats = NOALLOC_PARTIAL_FLOATS;
    ws.counters = reinterpret_cast<unsigned*>(ptr + (size_t)NOALLOC_PARTIAL_FLOATS * 4);
    ws.num_counters = NOALLOC_COUNTERS;
  }
  return rows_reduce_one<ROW_MAX>(M, h, h, w, nullptr, target->data_device, 1.f, 0.f, ws);
}

int argmax_by_axis(cudamat* mat, cudamat* target, int axis) {
  const int h = mat->size[0], w = mat->size[1];
  if (int e = check_axis_common(mat, target)) return e;
  if (axis == 0) {
    if (target->size[0] != 1 || target->size[1] != w) return ERROR_INCOMPATIBLE_DIMENSIONS;
    return launch_cols(k_col_argmax<64>, k_col_argmax<256>, w, h, (const float*)mat->data_device,
                       target->data_device, (const float*)nullptr, w, h, 0);
  } else if (axis == 1) {
    if (target->size[0] != h || target->size[1] != 1) return ERROR_INCOMPATIBLE_DIMENSIONS;
    if (h <= 0) return 0;
    hipLaunchKernelGGL(k_row_reduce, dim3((h + 63) / 64), dim3(256), 0, dn_stream(), (const float*)mat->data_device,
                       target->data_device, w, h, 1, 0.f, 0.f);
    return dn_launch_status();
  }
  return ERROR_UNSUPPORTED;
}

// One-hot of the arg-max of every column (axis 0) or row (axis 1).  The reference
// kernel clears rows of column 0 instead of the column it is working on
// (cudamat_kernels.cu:980); every column is cleared here.
int choose_max_by_axis(cudamat* mat, cudamat* target, int axis) {
  const int h = mat->size[0], w = mat->size[1];
  if (int e = check_axis_common(mat, target)) return e;
  if (target->size[0] != h || target->size[1] != w) return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (axis == 0) {
    return launch_cols(k_col_argmax<64>, k_col_argmax<256>, w, h, (const float*)mat->data_device,
                       target->data_device, (const float*)nullptr, w, h, 1);
  } else if (axis == 1) {
    if (h <= 0) return 0;
    hipLaunchKernelGGL(k_row_reduce, dim3((h + 63) / 64), dim3(256), 0, dn_stream(), (const float*)mat->data_device,
                       target->data_device, w, h, 2, 0.f, 0.f);
    return dn_launch_status();
  }
  return ERROR_UNSUPPORTED;
}

int choose_max_and_accumulate(cudamat* mat, cudamat* acc) {
  const int h = mat->size[0], w = mat->size[1];
  if (int e = check_axis_common(mat, acc)) return e;
  if (acc->size[0] != h || acc->size[1] != w) return ERROR_INCOMPATIBLE_DIMENSIONS;
  return launch_cols(k_col_argmax<64>, k_col_argmax<256>, w, h, (const float*)mat->data_device, acc->data_device,
                     (const float*)nullptr, w, h, 2);
}

int sqsum_by_axis(cudamat* mat, cudamat* target, int axis, float mult, float p) {
  const int h = mat->size[0], w = mat->size[1];
  if (int e = check_axis_common(mat, target)) return e;
  if (axis == 0) {
    if (target->size[0] != 1 || target->size[1] != w) return ERROR_INCOMPATIBLE_DIMENSIONS;
    if (w > 0 && colblock_launch<COL_SQSUM>(mat->data_device, h, h, w, nullptr, target->data_device, mult, p))
      return dn_launch_status();
    return launch_cols(k_col_sqsum<64>, k_col_sqsum<256>, w, h, (const float*)mat->data_device, target->data_device,
                       w, h, mult, p);
  } else if (axis == 1) {
    if (target->size[0] != h || target->size[1] != 1) return ERROR_INCOMPATIBLE_DIMENSIONS;
    return rows_reduce<ROW_SQSUM>(mat->data_device, h, h, w, nullptr, target->data_device, mult, p);
  }
  return ERROR_UNSUPPORTED;
}

// target = beta * target + alpha * (sums of mat along axis), the kernels that dot() with a vector
// of ones runs, without the vector: the same additions in the same order, so the same bits.
// A transposed operand is summed along its other stored axis, as dot() would.  The target is
// checked the way dot() checks it (cudamat.cu:1675-1679: leading and non-leading dimension,
// the target's is_trans otherwise ignored), so a vector handed over as the transposed view
// of its other orientation is accepted as it is there; it is the same memory.
static int sums_impl(cudamat* mat, cudamat* target, int axis, float beta, float alpha) {
  if (!mat->on_device || !target->on_device) return ERROR_NOT_ON_DEVICE;
  if (axis != 0 && axis != 1) return ERROR_UNSUPPORTED;
  const int h = mat->size[0], w = mat->size[1];
  const bool along_stored_columns = (axis == 0) != (mat->is_trans != 0);   // one result per stored column
  const int results = along_stored_columns ? w : h;
  const int t_lead = target->is_trans ? target->size[1] : target->size[0];
  const int t_nonlead = target->is_trans ? target->size[0] : target->size[1];
  if (axis == 0 ? (t_lead != 1 || t_nonlead != results) : (t_lead != results || t_nonlead != 1))
    return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (results <= 0) return 0;
  if (along_stored_columns) {
    if (colblock_launch<COL_SUM>(mat->data_device, h, h, w, nullptr, target->data_device, alpha, beta)) return dn_launch_status();
    return dn_gemv_cols(mat->data_device, h, h, w, nullptr, target->data_device, alpha, beta);
  }
  int held = 0;
  if (dn_defer_row_sum(mat->data_device, target->data_device, h, w, alpha, beta, &held)) return held;
  return rows_reduce<ROW_SUM>(mat->data_device, h, h, w, nullptr, target->data_device, alpha, beta);
}

// eigenmat.cc:747-760 (the reference's CPU backend exports these; its cudamat.py spells them as
// dot() with a vector of ones, cudamat.py:1546-1577 and 724-748).
int sum_by_axis(cudamat* mat, cudamat* target, int axis) { return sums_impl(mat, target, axis, 0.f, 1.f); }
int add_sum_by_axis(cudamat* mat, cudamat* target, int axis, float mult) { return sums_impl(mat, target, axis, 1.f, mult); }

}  // extern "C"

// t(i, j) = a(i, j) * (n_i < norm ? 1 : norm / n_i) with n_i = sqrt(sq[i]): the second pass of
// normlimit_by_axis along the rows, given the rows' sums of squares.  Axis 1 is an extension:
// the reference returns ERROR_UNSUPPORTED for it (cudamat.cu:1300-1311); the rule is that of its
// column kernel (kNormLimitColumnwise, cudamat_kernels.cu:1068-1098) applied to rows, and is
// checked against the host restatement only.  A flat pass over the matrix; VEC: 16-byte groups (h a multiple of 4, aligned
// operands), whose four rows are one 16-byte group of sq.
template <bool VEC, bool STREAM>
__global__ void __launch_bounds__(256)
k_scale_rows_to_norm(const float* a, const float* sq, float* t, long long n, FastDiv fd, float norm) {
  auto one = [&](float x, float s) {
    const float nn = sqrtf(s);
    return x * (nn < norm ? 1.f : norm / nn);
  };
  const long long tid = (long long)blockIdx.x * 256 + threadIdx.x;
  if (VEC) {
    const long long e = tid * 4;
    if (e >= n) return;
    const uint32_t r = (uint32_t)e - fd_div((uint32_t)e, fd) * fd.d;
    const float4 x = dn_ld4<STREAM>(a + e);
    const float4 s = *reinterpret_cast<const float4*>(sq + r);
    dn_st4<STREAM>(t + e, make_float4(one(x.x, s.x), one(x.y, s.y), one(x.z, s.z), one(x.w, s.w)));
  } else {
    if (tid >= n) return;
    const uint32_t r = (uint32_t)tid - fd_div((uint32_t)tid, fd) * fd.d;
    t[tid] = one(a[tid], sq[r]);
  }
}

extern "C" {

int normlimit_by_axis(cudamat* mat, cudamat* target, int axis, float norm) {
  const int h = mat->size[0], w = mat->size[1];
  if (int e = check_axis_common(mat, target)) return e;
  if (target->size[0] != h || target->size[1] != w) return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (axis == 0) {
    const float* a = mat->data_device;
    float* t = target->data_device;
    // columns that fit a wavefront's registers are read once (4096 x 4096: 36.7 -> 23 us)
    if (w > 0 && h > 0 && h % 4 == 0 && h <= 64 * 4 * 16 && dn_aligned16(a) && dn_aligned16(t) &&
        !(w < dn_num_cus() * 2 && h >= 4096)) {   // (few tall columns: a workgroup per column below)
      const dim3 grid((w + 3) / 4), block(256);
      const int n4 = h / 4;
      if (n4 <= 64 * 2) hipLaunchKernelGGL(k_col_normlimit_reg<2>, grid, block, 0, dn_stream(), a, t, w, h, norm);
      else if (n4 <= 64 * 4) hipLaunchKernelGGL(k_col_normlimit_reg<4>, grid, block, 0, dn_stream(), a, t, w, h, norm);
      else if (n4 <= 64 * 8) hipLaunchKernelGGL(k_col_normlimit_reg<8>, grid, block, 0, dn_stream(), a, t, w, h, norm);
      else hipLaunchKernelGGL(k_col_normlimit_reg<16>, grid, block, 0, dn_stream(), a, t, w, h, norm);
      return dn_launch_status();
    }
    return launch_cols(k_col_normlimit<64>, k_col_normlimit<256>, w, h, a, t, w, h, norm);
  } else if (axis == 1) {
    if (h <= 0 || w <= 0) return 0;
    // two passes, each at streaming rate: the rows' sums of squares (the axis-1 reduction), then the
    // scaling as a column-vector broadcast (4096 x 4096: 37 us; one workgroup per 64 rows walking
    // all columns twice took 640 us).  The sums live in scratch slot 1, which nothing else of the
    // matrix library uses (slot 0 holds the reduction's own partials).
    float* sq = (float*)dn_scratch((size_t)h * sizeof(float), 1);
    if (!sq) return CUDA_ERROR;
    if (int e = rows_reduce<ROW_SQSUM>(mat->data_device, h, h, w, nullptr, sq, 1.f, 0.f)) return e;
    const long long n = (long long)h * w;
    if (n >= (1ll << 32)) return ERROR_UNSUPPORTED;    // 32-bit element index inside the kernel
    const FastDiv fd = make_fastdiv((uint32_t)h);
    const float* a = mat->data_device;
    float* t = target->data_device;
    if (h % 4 == 0 && dn_aligned16(a) && dn_aligned16(t)) {
      const unsigned blocks = (unsigned)((n / 4 + 255) / 256);
      if (n >= DN_STREAM_MIN_ELEMS) hipLaunchKernelGGL((k_scale_rows_to_norm<true, true>), dim3(blocks), dim3(256), 0, dn_stream(), a, (const float*)sq, t, n, fd, norm);
      else hipLaunchKernelGGL((k_scale_rows_to_norm<true, false>), dim3(blocks), dim3(256), 0, dn_stream(), a, (const float*)sq, t, n, fd, norm);
    } else {
      hipLaunchKernelGGL((k_scale_rows_to_norm<false, false>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, dn_stream(), a, (const float*)sq, t, n, fd, norm);
    }
    return dn_launch_status();
  }
  return ERROR_UNSUPPORTED;
}

static int softmax_impl(const float* in, float* out, int w, int h, SoftmaxExtras x = SoftmaxExtras{nullptr, nullptr, nullptr, 0.f}) {
  if (w <= 0 || h <= 0) return 0;
  const bool reg_ok = (h % 4 == 0) && dn_aligned16(in) && dn_aligned16(out) && h <= 64 * 4 * 16 &&
                      (!x.grad || dn_aligned16(x.grad));
  // (4096 x 4096 measured faster on one wavefront per column, 24.0 against 26.3 us; every
  // other tall shape on the workgroup kernel: 4000 x 4224 29.4 against 34.2 us, 3400 x 5000 27.8
  // against 32.7, 4096 x 8192 46.2 against 49.9)
  const bool one_wave_per_column = h == 4096 && (long long)w * h >= DN_STREAM_MIN_ELEMS && (long long)w * h < (1ll << 25);
  if (reg_ok && h > 1024 && w >= 8 * dn_num_cus() && !one_wave_per_column) {
    const int n4 = h / 4;
    dim3 grid((w + 3) / 4), block(256);
    const bool stream = (long long)w * h >= DN_STREAM_MIN_ELEMS;
    if (n4 <= 512) hipLaunchKernelGGL((k_col_softmax_blk<2, 4, false>), grid, block, 0, dn_stream(), in, out, w, h, x);
    else if (n4 <= 768) hipLaunchKernelGGL((k_col_softmax_blk<3, 4, false>), grid, block, 0, dn_stream(), in, out, w, h, x);
    else hipLaunchKernelGGL((k_col_softmax_blk<4, 4, false>), grid, block, 0, dn_stream(), in, out, w, h, x);
    return dn_launch_status();
  }
  if (reg_ok) {
    const int n4 = h / 4;
    dim3 grid((w + 3) / 4), block(256);
    if (n4 <= 64) hipLaunchKernelGGL((k_col_softmax_reg<1>), grid, block, 0, dn_stream(), in, out, w, h, x);
    else if (n4 <= 128) hipLaunchKernelGGL((k_col_softmax_reg<2>), grid, block, 0, dn_stream(), in, out, w, h, x);
    else if (n4 <= 256) hipLaunchKernelGGL((k_col_softmax_reg<4>), grid, block, 0, dn_stream(), in, out, w, h, x);
    else if (n4 <= 512) hipLaunchKernelGGL((k_col_softmax_reg<8>), grid, block, 0, dn_stream(), in, out, w, h, x);
    else hipLaunchKernelGGL((k_col_softmax_reg<16>), grid, block, 0, dn_stream(), in, out, w, h, x);
    return dn_launch_status();
  }
  // columns of 4097 to 16384 rows still fit the registers of a workgroup (two columns or one at
  // a time): one read and one write instead of the three passes below
  if ((h % 4 == 0) && dn_aligned16(in) && dn_aligned16(out) && (!x.grad || dn_aligned16(x.grad)) && h > 4096 && h <= 16384) {
    if (h <= 8192) hipLaunchKernelGGL((k_col_softmax_blk<8, 2, false>), dim3((w + 1) / 2), dim3(256), 0, dn_stream(), in, out, w, h, x);
    else hipLaunchKernelGGL((k_col_softmax_blk<16, 1, false>), dim3(w), dim3(256), 0, dn_stream(), in, out, w, h, x);
    return dn_launch_status();
  }
  return launch_cols(k_col_softmax<64>, k_col_softmax<256>, w, h, in, out, w, h, x);
}

}  // extern "C"

// ---- softmax held back.  A softmax layer's loss is spelled  state.apply_softmax();
// state.get_softmax_cross_entropy(labels, loss); state.apply_softmax_grad(labels, target=deriv)
// (deepnet/softmax_layer.py:25-28, 40-62): the softmax does not launch at once, the loss and the
// gradient of its result join it while they follow directly, and the three run as softmax_ce_grad's one
// launch (same kernels, same bits).  Any other call launches what is held back first.
struct PendSoftmax {
  int stage;                      // 0 nothing, 1 the softmax waits, 2 ... and its loss
  cudamat in, probs, labels, loss;
  float tiny;
};
static PendSoftmax g_sm = {};

bool dn_softmax_held() { return g_sm.stage != 0; }

void dn_softmax_flush() {
  if (g_sm.stage == 0) return;
  const PendSoftmax p = g_sm;
  g_sm.stage = 0;
  dn_refresh_pending();
  if (p.stage == 1) softmax_impl(p.in.data_device, p.probs.data_device, p.in.size[1], p.in.size[0]);
  else softmax_impl(p.in.data_device, p.probs.data_device, p.in.size[1], p.in.size[0],
                    SoftmaxExtras{p.labels.data_device, p.loss.data_device, nullptr, p.tiny});
}

static inline bool sm_overlap(const cudamat* a, const cudamat* b) {
  const float *p = a->data_device, *q = b->data_device;
  const long long np = dn_len(a), nq = dn_len(b);
  return p < q + nq && q < p + np;
}
static inline bool sm_same(const cudamat* a, const cudamat* b) {
  return a->data_device == b->data_device && a->size[0] == b->size[0] && a->size[1] == b->size[1] && !a->is_trans;
}

// (the arguments have passed the entry point's checks)
static bool softmax_hold(cudamat* mat, cudamat* target) {
  if (!dn_defer_enabled() || mat->size[0] <= 0 || mat->size[1] <= 0 || target->is_trans) return false;
  if (mat->data_device != target->data_device && sm_overlap(mat, target)) return false;
  dn_flush();                     // (what else is held back comes first)
  g_sm.stage = 1;
  g_sm.in = *mat; g_sm.probs = *target;
  dn_set_pending(true);
  return true;
}

// the loss of the held-back softmax: labels and loss are 1 x w vectors apart from everything else
static bool softmax_join_loss(cudamat* mat, cudamat* labels, cudamat* target, float tiny) {
  if (g_sm.stage != 1 || !dn_defer_enabled() || !sm_same(mat, &g_sm.probs)) return false;
  const int w = mat->size[1];
  if (!labels->on_device || !target->on_device || labels->size[0] != 1 || labels->size[1] != w || target->size[0] != 1 ||
      target->size[1] != w)
    return false;
  for (const cudamat* m : {&g_sm.in, &g_sm.probs})
    if (sm_overlap(labels, m) || sm_overlap(target, m)) return false;
  if (sm_overlap(labels, target)) return false;
  g_sm.labels = *labels; g_sm.loss = *target; g_sm.tiny = tiny;
  g_sm.stage = 2;
  return true;
}

// the gradient of the held-back softmax: launches the sequence
static bool softmax_join_grad(cudamat* mat, cudamat* labels, cudamat* target, int* err) {
  if (g_sm.stage == 0 || !dn_defer_enabled() || !sm_same(mat, &g_sm.probs)) return false;
  const int h = mat->size[0], w = mat->size[1];
  if (!labels->on_device || !target->on_device || target->is_trans || labels->size[0] != 1 || labels->size[1] != w ||
      target->size[0] != h || target->size[1] != w || !dn_aligned16(target->data_device))
    return false;
  if (g_sm.stage == 2 && !(labels->data_device == g_sm.labels.data_device)) return false;
  for (const cudamat* m : {&g_sm.in, &g_sm.probs})
    if (sm_overlap(labels, m) || sm_overlap(target, m)) return false;
  if (sm_overlap(labels, target) || (g_sm.stage == 2 && sm_overlap(target, &g_sm.loss))) return false;
  const PendSoftmax p = g_sm;
  g_sm.stage = 0;
  dn_refresh_pending();
  *err = softmax_impl(p.in.data_device, p.probs.data_device, w, h,
                      SoftmaxExtras{labels->data_device, p.stage == 2 ? p.loss.data_device : nullptr, target->data_device,
                                    p.stage == 2 ? p.tiny : 0.f});
  return true;
}

extern "C" {

int softmax(cudamat* mat, cudamat* target) {
  const int h = mat->size[0], w = mat->size[1];
  if (int e = check_axis_common(mat, target)) return e;
  if (target->size[0] != h || target->size[1] != w) return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (softmax_hold(mat, target)) return 0;
  return softmax_impl(mat->data_device, target->data_device, w, h);
}

// Extension (no counterpart in cudamat.cu): softmax -> get_softmax_cross_entropy ->
// apply_softmax_grad in one launch; loss and grad may each be NULL.
int softmax_ce_grad(cudamat* mat, cudamat* labels, cudamat* probs, cudamat* loss, cudamat* grad, float tiny) {
  const int h = mat->size[0], w = mat->size[1];
  if (int e = check_axis_common(mat, probs)) return e;
  if (!labels->on_device || (loss && !loss->on_device) || (grad && !grad->on_device)) return ERROR_NOT_ON_DEVICE;
  if (probs->size[0] != h || probs->size[1] != w) return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (labels->size[0] != 1 || labels->size[1] != w) return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (loss && (loss->size[0] != 1 || loss->size[1] != w)) return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (grad && (grad->size[0] != h || grad->size[1] != w)) return ERROR_INCOMPATIBLE_DIMENSIONS;
  return softmax_impl(mat->data_device, probs->data_device, w, h,
                      SoftmaxExtras{labels->data_device, loss ? loss->data_device : nullptr,
                                    grad ? grad->data_device : nullptr, tiny});
}

int softmax_overwrite(cudamat* mat) {
  if (!mat->on_device) return ERROR_NOT_ON_DEVICE;
  if (mat->is_trans) return ERROR_TRANSPOSED;
  if (softmax_hold(mat, mat)) return 0;
  return softmax_impl(mat->data_device, mat->data_device, mat->size[1], mat->size[0]);
}

int apply_softmax_grad(cudamat* mat, cudamat* labels, cudamat* target) {
  const int h = mat->size[0], w = mat->size[1];
  if (int e = check_axis_common(mat, target)) return e;
  if (target->size[0] != h || target->size[1] != w) return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (labels->size[0] != 1 || labels->size[1] != w) return ERROR_INCOMPATIBLE_DIMENSIONS;
  { int held = 0; if (softmax_join_grad(mat, labels, target, &held)) return held; }
  const long long n = (long long)h * w;
  if (n <= 0) return 0;
  if (n >= (1ll << 32)) return ERROR_UNSUPPORTED;
  const FastDiv fd = make_fastdiv((uint32_t)h);
  if (h % 4 == 0 && dn_aligned16(mat->data_device) && dn_aligned16(target->data_device)) {
    const long long n4 = n / 4;
    const unsigned blocks4 = (unsigned)((n4 + 255) / 256);
    if (n >= DN_STREAM_MIN_ELEMS)
      hipLaunchKernelGGL((k_softmax_grad4<true>), dim3(blocks4), dim3(256), 0, dn_stream(), (const float*)mat->data_device,
                         (const float*)labels->data_device, target->data_device, n4, h, fd);
    else
      hipLaunchKernelGGL((k_softmax_grad4<false>), dim3(blocks4), dim3(256), 0, dn_stream(), (const float*)mat->data_device,
                         (const float*)labels->data_device, target->data_device, n4, h, fd);
    return dn_launch_status();
  }
  long long blocks = (n + 255) / 256;
  if (blocks > dn_num_cus() * 32ll) blocks = dn_num_cus() * 32ll;
  hipLaunchKernelGGL(k_softmax_grad, dim3((unsigned)blocks), dim3(256), 0, dn_stream(), (const float*)mat->data_device,
                     (const float*)labels->data_device, target->data_device, w, h, fd);
  return dn_launch_status();
}

int get_softmax_correct(cudamat* mat, cudamat* labels, cudamat* target) {
  const int h = mat->size[0], w = mat->size[1];
  if (int e = check_axis_common(mat, target)) return e;
  if (target->size[0] != 1 || target->size[1] != w) return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (labels->size[0] != 1 || labels->size[1] != w) return ERROR_INCOMPATIBLE_DIMENSIONS;
  return launch_cols(k_col_argmax<64>, k_col_argmax<256>, w, h, (const float*)mat->data_device, target->data_device,
                     (const float*)labels->data_device, w, h, 3);
}

int get_softmax_cross_entropy(cudamat* mat, cudamat* labels, cudamat* target, float tiny) {
  const int h = mat->size[0], w = mat->size[1];
  if (int e = check_axis_common(mat, target)) return e;
  if (target->size[0] != 1 || target->size[1] != w) return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (labels->size[0] != 1 || labels->size[1] != w) return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (softmax_join_loss(mat, labels, target, tiny)) return 0;
  if (w <= 0) return 0;
  hipLaunchKernelGGL(k_softmax_ce, dim3((w + 255) / 256), dim3(256), 0, dn_stream(), (const float*)mat->data_device,
                     (const float*)labels->data_device, target->data_device, w, h, tiny);
  return dn_launch_status();
}

float vdot(cudamat* mat1, cudamat* mat2, int* err_code) {
  const long long len = dn_len(mat1);
  if (!mat1->on_device || !mat2->on_device) { *err_code = ERROR_NOT_ON_DEVICE; return 0.f; }
  if (mat1->is_trans != mat2->is_trans) { *err_code = ERROR_TRANSPOSEDNESS; return 0.f; }
  if (dn_len(mat2) != len) { *err_code = ERROR_INCOMPATIBLE_DIMENSIONS; return 0.f; }
  float res = 0.f;
  const int e = flat_dot(mat1->data_device, mat2->data_device, len, 0, &res);
  *err_code = e;
  return e ? -1.f : res;
}

float sum_all(cudamat* mat, int* err_code) {
  if (!mat->on_device) { *err_code = ERROR_NOT_ON_DEVICE; return 0.f; }
  float res = 0.f;
  const int e = flat_dot(mat->data_device, nullptr, dn_len(mat), 0, &res);
  *err_code = e;
  return e ? -1.f : res;
}

float euclid_norm(cudamat* mat, int* err_code) {
  if (!mat->on_device) { *err_code = ERROR_NOT_ON_DEVICE; return 0.f; }
  float res = 0.f;
  const int e = flat_dot(mat->data_device, mat->data_device, dn_len(mat), 1, &res);
  *err_code = e;
  return e ? -1.f : res;
}

}  // extern "C"
