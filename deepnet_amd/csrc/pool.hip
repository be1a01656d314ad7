// Local max pooling, its gradient, and within-channel response / contrast
// normalisation with their gradient, in the (channels, rows, cols, batch) layout.
// Replaces cudamat/cudamat_conv.cu:1021-1387, cudamat_conv_kernels.cuh:1238-2023
// and cudamat_conv_kernels.cu:30-441.
//
// These are HBM-bound.  The batch index is the fastest one, so a lane owns VW
// neighbouring images (one 16-byte access when VW == 4) of one (channel, output)
// and walks the window; every lane of a wavefront walks the same window, and the
// overlap between neighbouring windows is served from cache.
#include "common.h"
#include "wide_math.h"
#include "../../include/cudamat_conv_amd.h"
#include <math.h>

// Cache policy of the 16-byte accesses below, one bit per place (1, 4: loads of the un-pooled map in the pooling
// gradients; 2, 8, 16, 32, 64: stores of the pooling gradient, the fused kernels, the LDS normalisation kernels
// and the pooling kernel).  Measured at 64 maps of 32 x 32, batch 128: non-temporal stores gain 0.5-2.3 us per
// kernel (MaxPool + ResponseNorm in one launch 11.5 -> 9.2 us), non-temporal loads cost 1.5-3 us.
#define POOL_NT 122
// 16-byte accesses to data that this kernel touches once (non-temporal: they do not displace what the caches hold)
__device__ __forceinline__ float4 ld4_once(const float* p, bool nt) { return nt ? dn_ld4<true>(p) : dn_ld4<false>(p); }
__device__ __forceinline__ void st4_once(float* p, float4 v, bool nt) { if (nt) dn_st4<true>(p, v); else dn_st4<false>(p, v); }

void conv_set_error(const char* where, const char* what);
void conv_clear_error();

#define POOL_REQUIRE(cond, where)        \
  do {                                   \
    if (!(cond)) {                       \
      conv_set_error(where, #cond);      \
      return;                            \
    }                                    \
  } while (0)

template <int VW> struct Vec;
template <> struct Vec<1> {
  float v[1];
  __device__ __forceinline__ static Vec load(const float* p) { Vec r; r.v[0] = *p; return r; }
  __device__ __forceinline__ void store(float* p) const { *p = v[0]; }
};
template <> struct Vec<4> {
  float v[4];
  __device__ __forceinline__ static Vec load(const float* p) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    Vec r; r.v[0] = t.x; r.v[1] = t.y; r.v[2] = t.z; r.v[3] = t.w; return r;
  }
  __device__ __forceinline__ void store(float* p) const { *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]); }
};

struct PoolGeom {
  int N, NV;        // images, images / VW
  int F, S, O;      // channels, input size, output size (per side)
  int subs, start, stride;
  FastDiv dNV, dO, dS;
};

// e -> (image group, x, y, channel) for a (NV, X, X, F) index space
__device__ __forceinline__ void decode4(uint32_t e, const FastDiv& dNV, const FastDiv& dX, int X, int* nv, int* x, int* y,
                                        int* f) {
  uint32_t q = fd_div(e, dNV);
  *nv = (int)(e - q * dNV.d);
  uint32_t q2 = fd_div(q, dX);
  *x = (int)(q - q2 * (uint32_t)X);
  uint32_t q3 = fd_div(q2, dX);
  *y = (int)(q2 - q3 * (uint32_t)X);
  *f = (int)q3;
}

// mode 0: max over the clipped window (start value -2e38, cudamat_conv_kernels.cuh:31-42).
// mode 1: the reference's "probabilistic max" scan (:44-55, :1550-1623): the candidate
//         replaces the running value unless running*r_running > candidate*r_candidate.
template <int VW, int MODE>
__global__ void __launch_bounds__(256) k_pool(const float* imgs, const float* rnd, float* target, PoolGeom g) {
  const uint32_t total = (uint32_t)g.NV * g.O * g.O * g.F;
  for (uint32_t e = blockIdx.x * 256u + threadIdx.x; e < total; e += gridDim.x * 256u) {
    int nv, ox, oy, f;
    decode4(e, g.dNV, g.dO, g.O, &nv, &ox, &oy, &f);
    const int sx = g.start + ox * g.stride, sy = g.start + oy * g.stride;
    const int x0 = sx > 0 ? sx : 0, y0 = sy > 0 ? sy : 0;
    const int x1 = sx + g.subs < g.S ? sx + g.subs : g.S, y1 = sy + g.subs < g.S ? sy + g.subs : g.S;
    const float* base = imgs + (size_t)g.N * ((size_t)f * g.S * g.S) + nv * VW;
    const float* rbase = MODE == 1 ? rnd + (size_t)g.N * ((size_t)f * g.S * g.S) + nv * VW : nullptr;
    Vec<VW> acc, racc;
#pragma unroll
    for (int i = 0; i < VW; ++i) { acc.v[i] = -2e38f; racc.v[i] = -2e38f; }
    for (int y = y0; y < y1; ++y)
      for (int x = x0; x < x1; ++x) {
        const size_t off = (size_t)g.N * (y * g.S + x);
        const Vec<VW> v = Vec<VW>::load(base + off);
        if (MODE == 0) {
#pragma unroll
          for (int i = 0; i < VW; ++i) acc.v[i] = acc.v[i] > v.v[i] ? acc.v[i] : v.v[i];
        } else {
          const Vec<VW> r = Vec<VW>::load(rbase + off);
#pragma unroll
          for (int i = 0; i < VW; ++i) {
            const bool keep = acc.v[i] * racc.v[i] > v.v[i] * r.v[i];
            acc.v[i] = keep ? acc.v[i] : v.v[i];
            racc.v[i] = keep ? racc.v[i] : r.v[i];
          }
        }
      }
    if (VW == 4 && (POOL_NT & 64)) st4_once(target + (size_t)g.N * ((size_t)(f * g.O + oy) * g.O + ox) + nv * VW, make_float4(acc.v[0], acc.v[1], acc.v[2], acc.v[3]), true);
    else acc.store(target + (size_t)g.N * ((size_t)(f * g.O + oy) * g.O + ox) + nv * VW);
  }
}

// Gradient of max pooling (cudamat_conv_kernels.cuh:1439-1530): each pixel collects
// maxGrad from every output whose window holds it and whose max equals the pixel.
template <int VW>
__global__ void __launch_bounds__(256)
k_pool_undo(const float* imgs, const float* maxGrads, const float* maxActs, float* target, PoolGeom g) {
  const uint32_t total = (uint32_t)g.NV * g.S * g.S * g.F;
  for (uint32_t e = blockIdx.x * 256u + threadIdx.x; e < total; e += gridDim.x * 256u) {
    int nv, px, py, f;
    decode4(e, g.dNV, g.dS, g.S, &nv, &px, &py, &f);
    Vec<VW> acc;
#pragma unroll
    for (int i = 0; i < VW; ++i) acc.v[i] = 0.f;
    const size_t poff = (size_t)g.N * ((size_t)(f * g.S + py) * g.S + px) + nv * VW;
    const int span = g.start + g.stride * (g.O - 1) + g.subs;
    if (px >= g.start && px < span && py >= g.start && py < span) {
      const int oy0 = py - g.start < g.subs ? 0 : 1 + (py - g.start - g.subs) / g.stride;
      const int oy1 = 1 + (py - g.start) / g.stride < g.O ? 1 + (py - g.start) / g.stride : g.O;
      const int ox0 = px - g.start < g.subs ? 0 : 1 + (px - g.start - g.subs) / g.stride;
      const int ox1 = 1 + (px - g.start) / g.stride < g.O ? 1 + (px - g.start) / g.stride : g.O;
      const Vec<VW> img = Vec<VW>::load(imgs + poff);
      for (int oy = oy0; oy < oy1; ++oy)
        for (int ox = ox0; ox < ox1; ++ox) {
          const size_t ooff = (size_t)g.N * ((size_t)(f * g.O + oy) * g.O + ox) + nv * VW;
          const Vec<VW> ma = Vec<VW>::load(maxActs + ooff);
          const Vec<VW> mg = Vec<VW>::load(maxGrads + ooff);
#pragma unroll
          for (int i = 0; i < VW; ++i) acc.v[i] += (img.v[i] == ma.v[i] ? 1.f : 0.f) * mg.v[i];
        }
    }
    acc.store(target + poff);
  }
}

// Gradient of max pooling for the usual shapes (window and stride known at compile time,
// 4 images per lane): a pixel is covered by at most NC x NC windows; every load is
// unconditional, from window coordinates clamped into the map, so that all of a lane's
// loads are in flight together, and what fell outside is dropped by a select.  (The same
// treatment of the forward pass measured slower than its loop and is not used.)
template <int SUBS, int STRIDE>
__global__ void __launch_bounds__(256)
k_pool_undo_fixed(const float* imgs, const float* maxGrads, const float* maxActs, float* target, PoolGeom g) {
  constexpr int NC = (SUBS + STRIDE - 1) / STRIDE;
  const uint32_t total = (uint32_t)g.NV * g.S * g.S * g.F;
  for (uint32_t e = blockIdx.x * 256u + threadIdx.x; e < total; e += gridDim.x * 256u) {
    int nv, px, py, f;
    decode4(e, g.dNV, g.dS, g.S, &nv, &px, &py, &f);
    const size_t poff = (size_t)g.N * ((size_t)(f * g.S + py) * g.S + px) + nv * 4;
    const int ty = py - g.start, tx = px - g.start;
    const int oy_hi = ty >= 0 ? ty / STRIDE : 0, ox_hi = tx >= 0 ? tx / STRIDE : 0;
    const Vec<4> img = Vec<4>::load(imgs + poff);
    Vec<4> ma[NC][NC], mg[NC][NC];
    bool ok[NC][NC];
#pragma unroll
    for (int jy = 0; jy < NC; ++jy) {
      const int oy = oy_hi - (NC - 1 - jy);                  // ascending, as the reference scans
      const bool vy = (ty >= 0) & (oy >= 0) & (oy < g.O) & (ty - oy * STRIDE < SUBS);
      const int oyc = oy < 0 ? 0 : (oy >= g.O ? g.O - 1 : oy);
#pragma unroll
      for (int jx = 0; jx < NC; ++jx) {
        const int ox = ox_hi - (NC - 1 - jx);
        ok[jy][jx] = vy & (tx >= 0) & (ox >= 0) & (ox < g.O) & (tx - ox * STRIDE < SUBS);
        const int oxc = ox < 0 ? 0 : (ox >= g.O ? g.O - 1 : ox);
        const size_t ooff = (size_t)g.N * ((size_t)(f * g.O + oyc) * g.O + oxc) + nv * 4;
        ma[jy][jx] = Vec<4>::load(maxActs + ooff);
        mg[jy][jx] = Vec<4>::load(maxGrads + ooff);
      }
    }
    Vec<4> acc;
#pragma unroll
    for (int i = 0; i < 4; ++i) acc.v[i] = 0.f;
#pragma unroll
    for (int jy = 0; jy < NC; ++jy)
#pragma unroll
      for (int jx = 0; jx < NC; ++jx)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float t = (img.v[i] == ma[jy][jx].v[i] ? 1.f : 0.f) * mg[jy][jx].v[i];
          acc.v[i] += ok[jy][jx] ? t : 0.f;
        }
    acc.store(target + poff);
  }
}

// The same for stride 2 on larger maps, start 0: a lane takes a 2 x 2 block of pixels (rows
// 2i, 2i+1, columns 2j, 2j+1).  The windows that cover any of them are (i-1 | i, j-1 | j), so
// the block's four pixels share four loads of each pooled array where one pixel at a time
// asks for four of its own: a quarter of the requests to the caches, which is what bounds
// the one-pixel kernel (96 maps of 55 x 55 at batch 128: 95 -> 68 us).  Every
// pixel adds its windows in the order of the one-pixel kernel, so the results are the same bits.
template <int SUBS>
__global__ void __launch_bounds__(256)
k_pool_undo_block2(const float* imgs, const float* maxGrads, const float* maxActs, float* target, PoolGeom g, int B, FastDiv dB) {
  const uint32_t total = (uint32_t)g.NV * B * B * g.F;
  for (uint32_t e = blockIdx.x * 256u + threadIdx.x; e < total; e += gridDim.x * 256u) {
    int nv, bx, by, f;
    decode4(e, g.dNV, dB, B, &nv, &bx, &by, &f);
    Vec<4> ma[2][2], mg[2][2];
    bool in[2][2];
#pragma unroll
    for (int jy = 0; jy < 2; ++jy) {
      const int oy = by - 1 + jy;
      const int oyc = oy < 0 ? 0 : (oy >= g.O ? g.O - 1 : oy);
#pragma unroll
      for (int jx = 0; jx < 2; ++jx) {
        const int ox = bx - 1 + jx;
        const int oxc = ox < 0 ? 0 : (ox >= g.O ? g.O - 1 : ox);
        in[jy][jx] = (oy >= 0) & (oy < g.O) & (ox >= 0) & (ox < g.O);
        const size_t ooff = (size_t)g.N * ((size_t)(f * g.O + oyc) * g.O + oxc) + nv * 4;
        ma[jy][jx] = Vec<4>::load(maxActs + ooff);
        mg[jy][jx] = Vec<4>::load(maxGrads + ooff);
      }
    }
    Vec<4> img[2][2];
#pragma unroll
    for (int dy = 0; dy < 2; ++dy)
#pragma unroll
      for (int dx = 0; dx < 2; ++dx) {
        const int py = 2 * by + dy, px = 2 * bx + dx;
        const int pyc = py < g.S ? py : g.S - 1, pxc = px < g.S ? px : g.S - 1;
        { const float4 t4 = ld4_once(imgs + (size_t)g.N * ((size_t)(f * g.S + pyc) * g.S + pxc) + nv * 4, POOL_NT & 1);
          img[dy][dx].v[0] = t4.x; img[dy][dx].v[1] = t4.y; img[dy][dx].v[2] = t4.z; img[dy][dx].v[3] = t4.w; }
      }
#pragma unroll
    for (int dy = 0; dy < 2; ++dy)
#pragma unroll
      for (int dx = 0; dx < 2; ++dx) {
        const int py = 2 * by + dy, px = 2 * bx + dx;
        if (py >= g.S || px >= g.S) continue;
        Vec<4> acc;
#pragma unroll
        for (int i = 0; i < 4; ++i) acc.v[i] = 0.f;
#pragma unroll
        for (int jy = 0; jy < 2; ++jy)
#pragma unroll
          for (int jx = 0; jx < 2; ++jx) {
            // window (by - 1 + jy, bx - 1 + jx) starts at row 2*(by - 1 + jy): the pixel is inside it
            // when its offset from that row, 2 - 2*jy + dy, is below SUBS (likewise along x)
            const bool ok = in[jy][jx] & (2 - 2 * jy + dy < SUBS) & (2 - 2 * jx + dx < SUBS);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const float t = (img[dy][dx].v[i] == ma[jy][jx].v[i] ? 1.f : 0.f) * mg[jy][jx].v[i];
              acc.v[i] += ok ? t : 0.f;
            }
          }
        st4_once(target + (size_t)g.N * ((size_t)(f * g.S + py) * g.S + px) + nv * 4, make_float4(acc.v[0], acc.v[1], acc.v[2], acc.v[3]), POOL_NT & 2);
      }
  }
}

// Loads the 16 bytes at p when ok, else returns `other`: from an address that is valid either way
// (`safe`), so that the compiler emits a global load and a select (a conditional expression over the
// load itself becomes a load through a pointer that may point at a stack copy of `other`).
__device__ __forceinline__ float4 load4_or(const float* p, const float* safe, bool ok, float4 other) {
  const float4 v = *reinterpret_cast<const float4*>(ok ? p : safe);
  return ok ? v : other;
}

// x^y for the normalisation layers through the hardware log2 / exp2 (the reference uses
// __powf there, cudamat_conv_kernels.cu:112-176); relative error below 1e-6 for the
// denominators these layers see (1 <= x < ~1e3).
__device__ __forceinline__ float norm_pow(float x, float y) {
  return __builtin_amdgcn_exp2f(y * __builtin_amdgcn_logf(x));
}

// Sum of v (or v*v) over the part of the size x size window with origin (oy, ox) that
// lies inside the S x S map (any window size; the usual sizes take k_norm_rows below).
template <int VW, bool SQUARE>
__device__ __forceinline__ Vec<VW> window_sum(const float* base, int N, int S, int oy, int ox, int size) {
  Vec<VW> acc;
#pragma unroll
  for (int i = 0; i < VW; ++i) acc.v[i] = 0.f;
  const int y0 = oy > 0 ? oy : 0, x0 = ox > 0 ? ox : 0;
  const int y1 = oy + size < S ? oy + size : S, x1 = ox + size < S ? ox + size : S;
  for (int y = y0; y < y1; ++y)
    for (int x = x0; x < x1; ++x) {
      const Vec<VW> v = Vec<VW>::load(base + (size_t)N * (y * S + x));
#pragma unroll
      for (int i = 0; i < VW; ++i) acc.v[i] += SQUARE ? v.v[i] * v.v[i] : v.v[i];
    }
  return acc;
}

// denoms = 1 + addScale * sum over the clipped sizeX x sizeX window (origin -sizeX/2)
// of meanDiffs^2;  target = imgs * denoms^-powScale   (cudamat_conv_kernels.cu:112-176).
template <int VW>
__global__ void __launch_bounds__(256)
k_cnorm(const float* imgs, const float* meanDiffs, float* denoms, float* target, PoolGeom g, int sizeX, float addScale,
        float powScale) {
  const uint32_t total = (uint32_t)g.NV * g.S * g.S * g.F;
  for (uint32_t e = blockIdx.x * 256u + threadIdx.x; e < total; e += gridDim.x * 256u) {
    int nv, px, py, f;
    decode4(e, g.dNV, g.dS, g.S, &nv, &px, &py, &f);
    const float* base = meanDiffs + (size_t)g.N * ((size_t)f * g.S * g.S) + nv * VW;
    const Vec<VW> acc = window_sum<VW, true>(base, g.N, g.S, py - sizeX / 2, px - sizeX / 2, sizeX);
    const size_t poff = (size_t)g.N * ((size_t)(f * g.S + py) * g.S + px) + nv * VW;
    const Vec<VW> in = Vec<VW>::load(imgs + poff);
    Vec<VW> d, t;
#pragma unroll
    for (int i = 0; i < VW; ++i) {
      d.v[i] = 1.f + addScale * acc.v[i];
      t.v[i] = in.v[i] * norm_pow(d.v[i], -powScale);
    }
    d.store(denoms + poff);
    t.store(target + poff);
  }
}

// The same two layers for the usual window sizes, with a sliding window in registers: a
// lane owns SEG consecutive rows of one column of one map (for VW images), sums each
// window row once (SIZE loads) and adds up the SIZE most recent row sums per output, so
// an output costs (SEG + SIZE - 1) * SIZE / SEG loads instead of SIZE * SIZE.
// UNDO == false: denoms / target of the forward pass (window origin -SIZE/2, squares);
// UNDO == true: the backward pass over the prepared acts (mirrored window, plain sums).
template <int VW, int SIZE, int SEG, bool UNDO>
__global__ void __launch_bounds__(256)
k_norm_rows(const float* a0, const float* a1, const float* a2, const float* win, float* out0, float* out1, PoolGeom g,
            int nseg, FastDiv dseg, float addScale, float powScale) {
  // forward: a0 = imgs, win = meanDiffs, out0 = denoms, out1 = target
  // backward: a0 = outGrads, a1 = denoms, a2 = inputs, win = acts, out1 = target
  constexpr int ORG = UNDO ? SIZE / 2 - SIZE + 1 : -(SIZE / 2);
  const int S = g.S, N = g.N;
  const uint32_t total = (uint32_t)g.NV * S * nseg * g.F;
  for (uint32_t e = blockIdx.x * 256u + threadIdx.x; e < total; e += gridDim.x * 256u) {
    uint32_t q = fd_div(e, g.dNV);
    const int nv = (int)(e - q * g.dNV.d);
    uint32_t q2 = fd_div(q, g.dS);
    const int px = (int)(q - q2 * (uint32_t)S);
    const uint32_t f = fd_div(q2, dseg);
    const int y0 = (int)(q2 - f * (uint32_t)nseg) * SEG;
    const float* base = win + (size_t)N * ((size_t)f * S * S) + nv * VW;
    // clamped column offsets and their validity, shared by all rows
    int xoff[SIZE];
    bool xok[SIZE];
#pragma unroll
    for (int dx = 0; dx < SIZE; ++dx) {
      const int x = px + ORG + dx;
      xok[dx] = (unsigned)x < (unsigned)S;
      xoff[dx] = N * (x < 0 ? 0 : (x >= S ? S - 1 : x));
    }
    Vec<VW> ring[SIZE];
#pragma unroll
    for (int j = 0; j < SEG + SIZE - 1; ++j) {
      const int y = y0 + ORG + j;
      const bool yok = (unsigned)y < (unsigned)S;
      const float* row = base + (size_t)N * S * (y < 0 ? 0 : (y >= S ? S - 1 : y));
      Vec<VW> v[SIZE];
#pragma unroll
      for (int dx = 0; dx < SIZE; ++dx) v[dx] = Vec<VW>::load(row + xoff[dx]);
      Vec<VW> rs;
#pragma unroll
      for (int i = 0; i < VW; ++i) rs.v[i] = 0.f;
#pragma unroll
      for (int dx = 0; dx < SIZE; ++dx) {
        const bool ok = yok & xok[dx];
#pragma unroll
        for (int i = 0; i < VW; ++i) {
          const float t = UNDO ? v[dx].v[i] : v[dx].v[i] * v[dx].v[i];
          rs.v[i] += ok ? t : 0.f;
        }
      }
      ring[j % SIZE] = rs;
      if (j >= SIZE - 1) {
        const int py = y0 + j - (SIZE - 1);
        if (py < S) {
          Vec<VW> acc = ring[0];
#pragma unroll
          for (int r = 1; r < SIZE; ++r)
#pragma unroll
            for (int i = 0; i < VW; ++i) acc.v[i] += ring[r].v[i];
          const size_t poff = (size_t)N * ((size_t)(f * S + py) * S + px) + nv * VW;
          if (!UNDO) {
            const Vec<VW> in = Vec<VW>::load(a0 + poff);
            Vec<VW> d, t;
#pragma unroll
            for (int i = 0; i < VW; ++i) {
              d.v[i] = 1.f + addScale * acc.v[i];
              t.v[i] = in.v[i] * norm_pow(d.v[i], -powScale);
            }
            d.store(out0 + poff);
            t.store(out1 + poff);
          } else {
            const Vec<VW> og = Vec<VW>::load(a0 + poff), den = Vec<VW>::load(a1 + poff), inp = Vec<VW>::load(a2 + poff);
            Vec<VW> t;
#pragma unroll
            for (int i = 0; i < VW; ++i) t.v[i] = inp.v[i] * acc.v[i] + og.v[i] * norm_pow(den.v[i], -powScale);
            t.store(out1 + poff);
          }
        }
      }
    }
  }
}

// acts := scale * outGrads * acts / denoms   (cudamat_conv_kernels.cuh:2010-2023)
template <int VW>
__global__ void __launch_bounds__(256)
k_rnorm_undo_prelim(float* acts, const float* denoms, const float* outGrads, size_t nv, float scale) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < nv; i += stride) {
    const Vec<VW> a = Vec<VW>::load(acts + i * VW), d = Vec<VW>::load(denoms + i * VW), o = Vec<VW>::load(outGrads + i * VW);
    Vec<VW> t;
#pragma unroll
    for (int k = 0; k < VW; ++k) t.v[k] = (scale * o.v[k] * a.v[k]) / d.v[k];
    t.store(acts + i * VW);
  }
}

// target = inputs * (sum of the prepared acts over the mirrored window) + outGrads * denoms^-powScale
// (cudamat_conv_kernels.cuh:1920-2004); the window of pixel p is [p + sizeX/2 - sizeX + 1, p + sizeX/2].
template <int VW>
__global__ void __launch_bounds__(256)
k_rnorm_undo(const float* outGrads, const float* denoms, const float* inputs, const float* acts, float* target,
             PoolGeom g, int sizeX, float powScale) {
  const uint32_t total = (uint32_t)g.NV * g.S * g.S * g.F;
  for (uint32_t e = blockIdx.x * 256u + threadIdx.x; e < total; e += gridDim.x * 256u) {
    int nv, px, py, f;
    decode4(e, g.dNV, g.dS, g.S, &nv, &px, &py, &f);
    const float* base = acts + (size_t)g.N * ((size_t)f * g.S * g.S) + nv * VW;
    const Vec<VW> acc =
        window_sum<VW, false>(base, g.N, g.S, py + sizeX / 2 - sizeX + 1, px + sizeX / 2 - sizeX + 1, sizeX);
    const size_t poff = (size_t)g.N * ((size_t)(f * g.S + py) * g.S + px) + nv * VW;
    const Vec<VW> inp = Vec<VW>::load(inputs + poff), og = Vec<VW>::load(outGrads + poff),
                  den = Vec<VW>::load(denoms + poff);
    Vec<VW> t;
#pragma unroll
    for (int i = 0; i < VW; ++i) t.v[i] = inp.v[i] * acc.v[i] + og.v[i] * norm_pow(den.v[i], -powScale);
    t.store(target + poff);
  }
}

// The normalisation layers on maps that fit in LDS: a workgroup owns one map of IB
// neighbouring images (QB = IB/4 groups of 4 images), reads every element once from global
// memory (a lane of the 1024 holds up to NORM_LDS_SLOTS 16-byte groups of it in registers, all loads in
// flight together), and forms the window sums in two passes through LDS: sums along x of
// the squares (forward) or of the prepared acts (backward) into a second tile, then sums
// along y of those.  Any window size; reads of a workgroup all come before its writes and
// cover only its own tile, so operands may alias.
//   forward:  denoms = 1 + addScale * sum(win^2);  target = imgs * denoms^-powScale
//   backward: acts := scale * outGrads * acts / denoms (stored, as the reference's first
//             kernel does), target = inputs * sum(acts) + outGrads * denoms^-powScale
#define NORM_LDS_SLOTS 2
#define NORM_LDS_THREADS 1024
#define NORM_LDS_MAX_GROUPS (NORM_LDS_SLOTS * NORM_LDS_THREADS)   // 16-byte groups per tile (32 KiB)

// SIZE > 0: window size known at compile time (all LDS reads of a lane independent and in
// flight together); SIZE == 0: any size, a loop.
template <int QB, bool UNDO, bool SAME, int SIZE>
__global__ void __launch_bounds__(NORM_LDS_THREADS)
k_norm_lds(const float* a0, const float* a1, const float* a2, const float* win, float* out0, float* out1, int N, int S,
           FastDiv dS, int nblk, int size_rt, float addScale, float powScale) {
  const int size = SIZE > 0 ? SIZE : size_rt;
  // forward: a0 = imgs, win = meanDiffs (SAME: the same array), out0 = denoms, out1 = target
  // backward: a0 = outGrads, a1 = denoms, a2 = inputs, win = acts (also written), out1 = target
  extern __shared__ float4 lds[];
  const int f = blockIdx.x / nblk, b = blockIdx.x - f * nblk;
  const int n0 = b * (QB * 4);
  const int qn = (N - n0) / 4 < QB ? (N - n0) / 4 : QB;      // image groups of this block that exist
  const int SS = S * S;
  const int groups = SS * QB;
  float4* tileA = lds;
  float4* tileB = lds + groups;
  const size_t map0 = (size_t)N * ((size_t)f * SS) + n0;
  const int org = UNDO ? size / 2 - size + 1 : -(size / 2);
  float4 keep0[NORM_LDS_SLOTS], keep1[NORM_LDS_SLOTS];
  // keep0: forward imgs / backward inputs;  keep1: backward outGrads * denoms^-powScale
  {
    float4 w[NORM_LDS_SLOTS], og[NORM_LDS_SLOTS], den[NORM_LDS_SLOTS];
#pragma unroll
    for (int k = 0; k < NORM_LDS_SLOTS; ++k) {
      const int i = (int)threadIdx.x + NORM_LDS_THREADS * k;
      const int pix = i / QB, q = i - pix * QB;
      const bool ok = i < groups && q < qn;
      const size_t off = map0 + (size_t)N * pix + 4 * q;
      const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
      w[k] = load4_or(win + off, win + map0, ok, z);
      if (UNDO) {
        og[k] = load4_or(a0 + off, a0 + map0, ok, z);
        den[k] = load4_or(a1 + off, a1 + map0, ok, make_float4(1.f, 1.f, 1.f, 1.f));
        keep0[k] = load4_or(a2 + off, a2 + map0, ok, z);
      } else if (!SAME) {
        keep0[k] = load4_or(a0 + off, a0 + map0, ok, z);
      }
    }
#pragma unroll
    for (int k = 0; k < NORM_LDS_SLOTS; ++k) {
      const int i = (int)threadIdx.x + NORM_LDS_THREADS * k;
      if (i >= groups) continue;
      if (UNDO) {
        const float sc = addScale;                 // -2 * addScale * powScale, prepared by the host
        float4 t;
        t.x = (sc * og[k].x * w[k].x) / den[k].x; t.y = (sc * og[k].y * w[k].y) / den[k].y;
        t.z = (sc * og[k].z * w[k].z) / den[k].z; t.w = (sc * og[k].w * w[k].w) / den[k].w;
        tileA[i] = t;
        const int pix = i / QB, q = i - pix * QB;
        if (q < qn) *reinterpret_cast<float4*>(const_cast<float*>(win) + map0 + (size_t)N * pix + 4 * q) = t;
        keep1[k] = make_float4(og[k].x * norm_pow(den[k].x, -powScale), og[k].y * norm_pow(den[k].y, -powScale),
                               og[k].z * norm_pow(den[k].z, -powScale), og[k].w * norm_pow(den[k].w, -powScale));
      } else {
        if (SAME) keep0[k] = w[k];
        tileA[i] = make_float4(w[k].x * w[k].x, w[k].y * w[k].y, w[k].z * w[k].z, w[k].w * w[k].w);
      }
    }
  }
  __syncthreads();
  // sums along x
#pragma unroll
  for (int k = 0; k < NORM_LDS_SLOTS; ++k) {
    const int i = (int)threadIdx.x + NORM_LDS_THREADS * k;
    if (i >= groups) continue;
    const int pix = i / QB;
    const int y = (int)fd_div((uint32_t)pix, dS), x = pix - y * S;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    if (SIZE > 0) {
      float4 t[SIZE > 0 ? SIZE : 1];
#pragma unroll
      for (int d = 0; d < SIZE; ++d) {
        const bool ok = (unsigned)(x + org + d) < (unsigned)S;
        t[d] = tileA[i + (ok ? (org + d) * QB : 0)];
      }
#pragma unroll
      for (int d = 0; d < SIZE; ++d) {
        const bool ok = (unsigned)(x + org + d) < (unsigned)S;
        acc.x += ok ? t[d].x : 0.f; acc.y += ok ? t[d].y : 0.f; acc.z += ok ? t[d].z : 0.f; acc.w += ok ? t[d].w : 0.f;
      }
    } else {
      const int x0 = x + org > 0 ? x + org : 0, x1 = x + org + size < S ? x + org + size : S;
      for (int xx = x0; xx < x1; ++xx) {
        const float4 t = tileA[i + (xx - x) * QB];
        acc.x += t.x; acc.y += t.y; acc.z += t.z; acc.w += t.w;
      }
    }
    tileB[i] = acc;
  }
  __syncthreads();
  // sums along y, then the output
#pragma unroll
  for (int k = 0; k < NORM_LDS_SLOTS; ++k) {
    const int i = (int)threadIdx.x + NORM_LDS_THREADS * k;
    if (i >= groups) continue;
    const int pix = i / QB, q = i - pix * QB;
    if (q >= qn) continue;
    const int y = (int)fd_div((uint32_t)pix, dS);
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    if (SIZE > 0) {
      float4 t[SIZE > 0 ? SIZE : 1];
#pragma unroll
      for (int d = 0; d < SIZE; ++d) {
        const bool ok = (unsigned)(y + org + d) < (unsigned)S;
        t[d] = tileB[i + (ok ? (org + d) * S * QB : 0)];
      }
#pragma unroll
      for (int d = 0; d < SIZE; ++d) {
        const bool ok = (unsigned)(y + org + d) < (unsigned)S;
        acc.x += ok ? t[d].x : 0.f; acc.y += ok ? t[d].y : 0.f; acc.z += ok ? t[d].z : 0.f; acc.w += ok ? t[d].w : 0.f;
      }
    } else {
      const int y0 = y + org > 0 ? y + org : 0, y1 = y + org + size < S ? y + org + size : S;
      for (int yy = y0; yy < y1; ++yy) {
        const float4 t = tileB[i + (yy - y) * S * QB];
        acc.x += t.x; acc.y += t.y; acc.z += t.z; acc.w += t.w;
      }
    }
    const size_t off = map0 + (size_t)N * pix + 4 * q;
    if (!UNDO) {
      const float4 d = make_float4(1.f + addScale * acc.x, 1.f + addScale * acc.y, 1.f + addScale * acc.z, 1.f + addScale * acc.w);
      const float4 in = keep0[k];
      st4_once(out0 + off, d, POOL_NT & 32);
      st4_once(out1 + off, make_float4(in.x * norm_pow(d.x, -powScale), in.y * norm_pow(d.y, -powScale),
                                       in.z * norm_pow(d.z, -powScale), in.w * norm_pow(d.w, -powScale)), POOL_NT & 32);
    } else {
      const float4 in = keep0[k], pw = keep1[k];
      st4_once(out1 + off, make_float4(in.x * acc.x + pw.x, in.y * acc.y + pw.y, in.z * acc.z + pw.z, in.w * acc.w + pw.w),
               POOL_NT & 32);
    }
  }
}

// ------------------------------------------------------------------ pooling and normalisation in one launch
// deepnet runs MaxPool -> ResponseNorm on the way up and ResponseNormUndo -> MaxPoolUndo on the way
// down (deepnet/convolutions.py:58-66, 120-134).  The pooled map of a block of images is small
// (15 x 15 x 32 images = 28.8 KB), so both pairs run as one kernel with it in LDS: the pooled
// values never make the round trip through memory between the two stages, and the four
// launches of a conv stage (each a 7-41 MB kernel whose load, compute and store phases do not
// overlap at one workgroup per CU) become two.  The arithmetic of each stage is that of the
// separate kernels above (same expressions, same order of additions): same bits.
//
// Up: a workgroup owns one map of QB * 4 images; a lane pools its (pooled pixel, 4 images)
// groups straight from the un-pooled map (all window loads in flight), stores them, and the
// workgroup goes on as k_norm_lds does.
template <int QB, int SUBS, int STRIDE, int SIZE>
__global__ void __launch_bounds__(NORM_LDS_THREADS)
k_pool_norm_lds(const float* imgs, float* pooled, float* denoms, float* target, int N, int Sin, int start, int S,
                FastDiv dS, int nblk, float addScale, float powScale) {
  extern __shared__ float4 lds[];
  const int f = blockIdx.x / nblk, b = blockIdx.x - f * nblk;
  const int n0 = b * (QB * 4);
  const int qn = (N - n0) / 4 < QB ? (N - n0) / 4 : QB;      // image groups of this block that exist
  const int SS = S * S;
  const int groups = SS * QB;
  float4* tileA = lds;
  float4* tileB = lds + groups;
  const size_t in0 = (size_t)N * ((size_t)f * Sin * Sin) + n0;
  const size_t map0 = (size_t)N * ((size_t)f * SS) + n0;
  constexpr int org = -(SIZE / 2);
  float4 keep0[NORM_LDS_SLOTS];
#pragma unroll
  for (int k = 0; k < NORM_LDS_SLOTS; ++k) {
    const int i = (int)threadIdx.x + NORM_LDS_THREADS * k;
    const int pix = i / QB, q = i - pix * QB;
    const bool ok = i < groups && q < qn;
    const int oy = (int)fd_div((uint32_t)pix, dS), ox = pix - oy * S;
    const int sy = start + oy * STRIDE, sx = start + ox * STRIDE;
    float4 w[SUBS][SUBS];
    bool in[SUBS][SUBS];
#pragma unroll
    for (int dy = 0; dy < SUBS; ++dy)
#pragma unroll
      for (int dx = 0; dx < SUBS; ++dx) {
        const int y = sy + dy, x = sx + dx;
        in[dy][dx] = ok && (unsigned)y < (unsigned)Sin && (unsigned)x < (unsigned)Sin;
        const int yc = y < 0 ? 0 : (y >= Sin ? Sin - 1 : y), xc = x < 0 ? 0 : (x >= Sin ? Sin - 1 : x);
        w[dy][dx] = load4_or(imgs + in0 + (size_t)N * (yc * Sin + xc) + 4 * q, imgs + in0, ok, make_float4(0.f, 0.f, 0.f, 0.f));
      }
    float4 acc = make_float4(-2e38f, -2e38f, -2e38f, -2e38f);    // the start value of the pooling kernel
#pragma unroll
    for (int dy = 0; dy < SUBS; ++dy)
#pragma unroll
      for (int dx = 0; dx < SUBS; ++dx) {
        const float4 v = w[dy][dx];
        if (in[dy][dx]) {
          acc.x = acc.x > v.x ? acc.x : v.x; acc.y = acc.y > v.y ? acc.y : v.y;
          acc.z = acc.z > v.z ? acc.z : v.z; acc.w = acc.w > v.w ? acc.w : v.w;
        }
      }
    if (!ok) acc = make_float4(0.f, 0.f, 0.f, 0.f);
    keep0[k] = acc;
    if (ok) st4_once(pooled + map0 + (size_t)N * pix + 4 * q, acc, POOL_NT & 16);
    if (i < groups) tileA[i] = make_float4(acc.x * acc.x, acc.y * acc.y, acc.z * acc.z, acc.w * acc.w);
  }
  __syncthreads();
  // sums along x
#pragma unroll
  for (int k = 0; k < NORM_LDS_SLOTS; ++k) {
    const int i = (int)threadIdx.x + NORM_LDS_THREADS * k;
    if (i >= groups) continue;
    const int pix = i / QB;
    const int y = (int)fd_div((uint32_t)pix, dS), x = pix - y * S;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    float4 t[SIZE];
#pragma unroll
    for (int d = 0; d < SIZE; ++d) {
      const bool ok = (unsigned)(x + org + d) < (unsigned)S;
      t[d] = tileA[i + (ok ? (org + d) * QB : 0)];
    }
#pragma unroll
    for (int d = 0; d < SIZE; ++d) {
      const bool ok = (unsigned)(x + org + d) < (unsigned)S;
      acc.x += ok ? t[d].x : 0.f; acc.y += ok ? t[d].y : 0.f; acc.z += ok ? t[d].z : 0.f; acc.w += ok ? t[d].w : 0.f;
    }
    tileB[i] = acc;
  }
  __syncthreads();
  // sums along y, then the output
#pragma unroll
  for (int k = 0; k < NORM_LDS_SLOTS; ++k) {
    const int i = (int)threadIdx.x + NORM_LDS_THREADS * k;
    if (i >= groups) continue;
    const int pix = i / QB, q = i - pix * QB;
    if (q >= qn) continue;
    const int y = (int)fd_div((uint32_t)pix, dS);
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    float4 t[SIZE];
#pragma unroll
    for (int d = 0; d < SIZE; ++d) {
      const bool ok = (unsigned)(y + org + d) < (unsigned)S;
      t[d] = tileB[i + (ok ? (org + d) * S * QB : 0)];
    }
#pragma unroll
    for (int d = 0; d < SIZE; ++d) {
      const bool ok = (unsigned)(y + org + d) < (unsigned)S;
      acc.x += ok ? t[d].x : 0.f; acc.y += ok ? t[d].y : 0.f; acc.z += ok ? t[d].z : 0.f; acc.w += ok ? t[d].w : 0.f;
    }
    const size_t off = map0 + (size_t)N * pix + 4 * q;
    const float4 d = make_float4(1.f + addScale * acc.x, 1.f + addScale * acc.y, 1.f + addScale * acc.z, 1.f + addScale * acc.w);
    const float4 in = keep0[k];
    st4_once(denoms + off, d, POOL_NT & 16);
    st4_once(target + off, make_float4(in.x * norm_pow(d.x, -powScale), in.y * norm_pow(d.y, -powScale),
                                       in.z * norm_pow(d.z, -powScale), in.w * norm_pow(d.w, -powScale)), POOL_NT & 16);
  }
}

// Down: the gradient of the normalisation for the pooled map (the arithmetic of k_norm_lds's
// backward form; `acts` is only read) stays in LDS next to the pooled activations, and every
// pixel of the un-pooled map then collects it from the windows that hold the pixel and whose
// maximum it is, in the order of k_pool_undo_fixed.  target may be imgs (a lane reads its pixel
// before it writes it).
#ifndef UNDO_PRE
#define UNDO_PRE 2
#endif
template <int QB, int SUBS, int STRIDE, int SIZE>
__global__ void __launch_bounds__(NORM_LDS_THREADS)
k_normundo_poolundo_lds(const float* outGrads, const float* denoms, const float* inputs, const float* acts, const float* imgs,
                        float* target, int N, int Sin, FastDiv dSin, int start, int S, FastDiv dS, int nblk, float scale,
                        float powScale) {
  constexpr int NC = (SUBS + STRIDE - 1) / STRIDE;
  extern __shared__ float4 lds[];
  const int f = blockIdx.x / nblk, b = blockIdx.x - f * nblk;
  const int n0 = b * (QB * 4);
  const int qn = (N - n0) / 4 < QB ? (N - n0) / 4 : QB;
  const int SS = S * S;
  const int groups = SS * QB;
  float4* tileA = lds;                 // the prepared acts, later the pooled map's gradient
  float4* tileB = lds + groups;        // sums along x
  float4* tileC = lds + 2 * groups;    // the pooled activations
  const size_t in0 = (size_t)N * ((size_t)f * Sin * Sin) + n0;
  const size_t map0 = (size_t)N * ((size_t)f * SS) + n0;
  constexpr int org = SIZE / 2 - SIZE + 1;
  float4 keep0[NORM_LDS_SLOTS], keep1[NORM_LDS_SLOTS];
#pragma unroll
  for (int k = 0; k < NORM_LDS_SLOTS; ++k) keep1[k] = make_float4(0.f, 0.f, 0.f, 0.f);
  // The un-pooled map does not depend on the normalisation's gradient: the groups of the first
  // UNDO_PRE trips of the last phase are requested here, together with the pooled arrays.
  const int items = Sin * Sin * QB;
  float4 pre[4 * UNDO_PRE];
#pragma unroll
  for (int u = 0; u < 4 * UNDO_PRE; ++u) {
    const int j = (int)threadIdx.x + u * NORM_LDS_THREADS;
    const int pin = j / QB, q = j - pin * QB;
    const bool ok = j < items && q < qn;
    const float4 v4 = ld4_once(ok ? imgs + in0 + (size_t)N * pin + 4 * q : imgs + in0, POOL_NT & 4);
    pre[u] = ok ? v4 : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  {
    float4 w[NORM_LDS_SLOTS], og[NORM_LDS_SLOTS], den[NORM_LDS_SLOTS];
#pragma unroll
    for (int k = 0; k < NORM_LDS_SLOTS; ++k) {
      const int i = (int)threadIdx.x + NORM_LDS_THREADS * k;
      const int pix = i / QB, q = i - pix * QB;
      const bool ok = i < groups && q < qn;
      const size_t off = map0 + (size_t)N * pix + 4 * q;
      const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
      w[k] = load4_or(acts + off, acts + map0, ok, z);
      og[k] = load4_or(outGrads + off, outGrads + map0, ok, z);
      den[k] = load4_or(denoms + off, denoms + map0, ok, make_float4(1.f, 1.f, 1.f, 1.f));
      keep0[k] = load4_or(inputs + off, inputs + map0, ok, z);
    }
#pragma unroll
    for (int k = 0; k < NORM_LDS_SLOTS; ++k) {
      const int i = (int)threadIdx.x + NORM_LDS_THREADS * k;
      if (i >= groups) continue;
      float4 t;
      t.x = (scale * og[k].x * w[k].x) / den[k].x; t.y = (scale * og[k].y * w[k].y) / den[k].y;
      t.z = (scale * og[k].z * w[k].z) / den[k].z; t.w = (scale * og[k].w * w[k].w) / den[k].w;
      tileA[i] = t;
      tileC[i] = w[k];
      keep1[k] = make_float4(og[k].x * norm_pow(den[k].x, -powScale), og[k].y * norm_pow(den[k].y, -powScale),
                             og[k].z * norm_pow(den[k].z, -powScale), og[k].w * norm_pow(den[k].w, -powScale));
    }
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < NORM_LDS_SLOTS; ++k) {
    const int i = (int)threadIdx.x + NORM_LDS_THREADS * k;
    if (i >= groups) continue;
    const int pix = i / QB;
    const int y = (int)fd_div((uint32_t)pix, dS), x = pix - y * S;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    float4 t[SIZE];
#pragma unroll
    for (int d = 0; d < SIZE; ++d) {
      const bool ok = (unsigned)(x + org + d) < (unsigned)S;
      t[d] = tileA[i + (ok ? (org + d) * QB : 0)];
    }
#pragma unroll
    for (int d = 0; d < SIZE; ++d) {
      const bool ok = (unsigned)(x + org + d) < (unsigned)S;
      acc.x += ok ? t[d].x : 0.f; acc.y += ok ? t[d].y : 0.f; acc.z += ok ? t[d].z : 0.f; acc.w += ok ? t[d].w : 0.f;
    }
    tileB[i] = acc;
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < NORM_LDS_SLOTS; ++k) {
    const int i = (int)threadIdx.x + NORM_LDS_THREADS * k;
    if (i >= groups) continue;
    const int pix = i / QB;
    const int y = (int)fd_div((uint32_t)pix, dS);
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    float4 t[SIZE];
#pragma unroll
    for (int d = 0; d < SIZE; ++d) {
      const bool ok = (unsigned)(y + org + d) < (unsigned)S;
      t[d] = tileB[i + (ok ? (org + d) * S * QB : 0)];
    }
#pragma unroll
    for (int d = 0; d < SIZE; ++d) {
      const bool ok = (unsigned)(y + org + d) < (unsigned)S;
      acc.x += ok ? t[d].x : 0.f; acc.y += ok ? t[d].y : 0.f; acc.z += ok ? t[d].z : 0.f; acc.w += ok ? t[d].w : 0.f;
    }
    const float4 in = keep0[k], pw = keep1[k];
    // (tileA was last read before the barrier above)
    tileA[i] = make_float4(in.x * acc.x + pw.x, in.y * acc.y + pw.y, in.z * acc.z + pw.z, in.w * acc.w + pw.w);
  }
  __syncthreads();
  // the un-pooled map: every (pixel, 4 images) group of it, four per trip with their loads in flight together
  auto scatter = [&](int j0, const float4* img) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = j0 + u * NORM_LDS_THREADS;
      const int pin = j / QB, q = j - pin * QB;
      if (j >= items || q >= qn) continue;
      const int py = (int)fd_div((uint32_t)pin, dSin), px = pin - py * Sin;
      const int ty = py - start, tx = px - start;
      const int oy_hi = ty >= 0 ? ty / STRIDE : 0, ox_hi = tx >= 0 ? tx / STRIDE : 0;
      float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int jy = 0; jy < NC; ++jy) {
        const int oy = oy_hi - (NC - 1 - jy);                  // ascending, as the reference scans
        const bool vy = (ty >= 0) & (oy >= 0) & (oy < S) & (ty - oy * STRIDE < SUBS);
        const int oyc = oy < 0 ? 0 : (oy >= S ? S - 1 : oy);
#pragma unroll
        for (int jx = 0; jx < NC; ++jx) {
          const int ox = ox_hi - (NC - 1 - jx);
          const bool ok = vy & (tx >= 0) & (ox >= 0) & (ox < S) & (tx - ox * STRIDE < SUBS);
          const int oxc = ox < 0 ? 0 : (ox >= S ? S - 1 : ox);
          const float4 ma = tileC[(oyc * S + oxc) * QB + q], mg = tileA[(oyc * S + oxc) * QB + q];
          const float tx_ = (img[u].x == ma.x ? 1.f : 0.f) * mg.x, ty_ = (img[u].y == ma.y ? 1.f : 0.f) * mg.y;
          const float tz_ = (img[u].z == ma.z ? 1.f : 0.f) * mg.z, tw_ = (img[u].w == ma.w ? 1.f : 0.f) * mg.w;
          acc.x += ok ? tx_ : 0.f; acc.y += ok ? ty_ : 0.f; acc.z += ok ? tz_ : 0.f; acc.w += ok ? tw_ : 0.f;
        }
      }
      st4_once(target + in0 + (size_t)N * pin + 4 * q, acc, POOL_NT & 8);
    }
  };
#pragma unroll
  for (int t = 0; t < UNDO_PRE; ++t) scatter((int)threadIdx.x + t * 4 * NORM_LDS_THREADS, pre + 4 * t);
  for (int j0 = (int)threadIdx.x + UNDO_PRE * 4 * NORM_LDS_THREADS; j0 < items; j0 += 4 * NORM_LDS_THREADS) {
    float4 img[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int j = j0 + u * NORM_LDS_THREADS;
      const int pin = j / QB, q = j - pin * QB;
      const bool ok = j < items && q < qn;
      { const float4 v4 = ld4_once(ok ? imgs + in0 + (size_t)N * pin + 4 * q : imgs + in0, POOL_NT & 4); img[u] = ok ? v4 : make_float4(0.f, 0.f, 0.f, 0.f); }
    }
    scatter(j0, img);
  }
}

// Largest image block (in groups of 4 images) whose two LDS tiles fit; 0 if none does or it
// would be narrow.
static int norm_lds_qb(int N, int S) {
  const long long ss = (long long)S * S;
  int qb = 8;
  while (qb >= 1 && ss * qb > NORM_LDS_MAX_GROUPS) qb >>= 1;
  while (qb > 1 && (qb / 2) * 4 >= N) qb >>= 1;      // no wider than the batch
  // blocks of fewer than 16 images read runs of 32 bytes or less: the row-window kernels, whose
  // lanes run along all the images, are faster then (96 maps of 27 x 27 at batch 128: ResponseNorm
  // 48.8 -> 30.2 us, its gradient 116.5 -> 54.9 us)
  if (qb < 4 && qb * 4 < N) return 0;
  return qb;
}

template <bool UNDO>
static void norm_lds_launch(int qb, bool same, const float* a0, const float* a1, const float* a2, const float* win,
                            float* out0, float* out1, int N, int S, int F, int size, float addScale, float powScale) {
  const int nblk = (N + qb * 4 - 1) / (qb * 4);
  const dim3 grid((unsigned)(F * nblk)), block(NORM_LDS_THREADS);
  const size_t lds = (size_t)2 * S * S * qb * sizeof(float4);
  const FastDiv dS = make_fastdiv((uint32_t)S);
#define NORM_LDS_GO(QB, SM, SZ) \
  hipLaunchKernelGGL((k_norm_lds<QB, UNDO, SM, SZ>), grid, block, lds, dn_stream(), a0, a1, a2, win, out0, out1, N, S, dS, nblk, size, addScale, powScale)
#define NORM_LDS_SZ(QB, SM) do { if (size == 3) NORM_LDS_GO(QB, SM, 3); else if (size == 5) NORM_LDS_GO(QB, SM, 5); \
                                 else if (size == 7) NORM_LDS_GO(QB, SM, 7); else NORM_LDS_GO(QB, SM, 0); } while (0)
#define NORM_LDS_QB(QB) do { if (same && !UNDO) NORM_LDS_SZ(QB, true); else NORM_LDS_SZ(QB, false); } while (0)
  if (qb == 8) NORM_LDS_QB(8);
  else if (qb == 4) NORM_LDS_QB(4);
  else if (qb == 2) NORM_LDS_QB(2);
  else NORM_LDS_QB(1);
#undef NORM_LDS_QB
#undef NORM_LDS_SZ
#undef NORM_LDS_GO
}

// ------------------------------------------------------------------ host side

#define NORM_SEG 5   // rows per lane in k_norm_rows

static int isqrt_exact_p(int v) {
  if (v < 0) return -1;
  int r = (int)(sqrt((double)v) + 0.5);
  return r * r == v ? r : -1;
}

static bool make_geom(PoolGeom& g, int N, int F, int S, int O, int subs, int start, int stride, int vw) {
  g.N = N; g.NV = N / vw; g.F = F; g.S = S; g.O = O; g.subs = subs; g.start = start; g.stride = stride;
  g.dNV = make_fastdiv((uint32_t)g.NV); g.dO = make_fastdiv((uint32_t)(O > 0 ? O : 1));
  g.dS = make_fastdiv((uint32_t)S);
  return true;
}

static unsigned grid_for(long long total) {
  long long b = (total + 255) / 256;
  const long long cap = (long long)dn_num_cus() * 32;
  if (b > cap) b = cap;
  return (unsigned)(b > 0 ? b : 1);
}

static bool all_aligned16(std::initializer_list<const void*> ps) {
  for (const void* p : ps)
    if (!dn_aligned16(p)) return false;
  return true;
}

static void pool_impl(cudamat* images, cudamat* rnd, cudamat* targets, int numFilters, int subsX, int startX,
                      int strideX, int outputsX, const char* where) {
  conv_clear_error();
  POOL_REQUIRE(images->on_device && targets->on_device && (!rnd || rnd->on_device), where);
  POOL_REQUIRE(numFilters > 0 && subsX > 0 && strideX > 0 && outputsX > 0, where);
  const int N = images->size[0];
  POOL_REQUIRE(N > 0 && images->size[1] % numFilters == 0, where);
  const int S = isqrt_exact_p(images->size[1] / numFilters);
  POOL_REQUIRE(S > 0, where);
  POOL_REQUIRE(targets->size[0] == N && targets->size[1] == numFilters * outputsX * outputsX, where);
  POOL_REQUIRE(!rnd || (rnd->size[0] == N && rnd->size[1] == images->size[1]), where);
  const long long outs = (long long)N * outputsX * outputsX * numFilters;
  POOL_REQUIRE(outs < (1ll << 32) && (long long)N * images->size[1] < (1ll << 32), where);
  const bool v4 = N % 4 == 0 && all_aligned16({images->data_device, targets->data_device, rnd ? rnd->data_device : nullptr});
  PoolGeom g;
  make_geom(g, N, numFilters, S, outputsX, subsX, startX, strideX, v4 ? 4 : 1);
  const unsigned grid = grid_for(outs / (v4 ? 4 : 1));
  const float* r = rnd ? rnd->data_device : nullptr;
  if (!rnd) {
    if (v4) hipLaunchKernelGGL((k_pool<4, 0>), dim3(grid), dim3(256), 0, dn_stream(), images->data_device, r, targets->data_device, g);
    else hipLaunchKernelGGL((k_pool<1, 0>), dim3(grid), dim3(256), 0, dn_stream(), images->data_device, r, targets->data_device, g);
  } else {
    if (v4) hipLaunchKernelGGL((k_pool<4, 1>), dim3(grid), dim3(256), 0, dn_stream(), images->data_device, r, targets->data_device, g);
    else hipLaunchKernelGGL((k_pool<1, 1>), dim3(grid), dim3(256), 0, dn_stream(), images->data_device, r, targets->data_device, g);
  }
  if (dn_launch_status()) conv_set_error(where, hipGetErrorString(hipGetLastError()));
}

// ---- MaxPool held back.  deepnet's conv stage calls MaxPool and then ResponseNorm on the pooled map
// (deepnet/convolutions.py:58-66): where the two can run as one launch (MaxPoolResponseNorm's LDS
// kernel: the same bits in the pooled map, the denominators and the result), MaxPool does not
// launch at once; a ResponseNorm of its target takes it along, and any other call -- of this
// library or of the matrix library -- launches it first (every launch passes through dn_stream()).
struct PendPool {
  bool active;
  cudamat images, targets;
  int numFilters, subsX, startX, strideX, outputsX;
};
static PendPool g_pp = {};
static int norm_lds_qb(int N, int S);

static void pool_flush() {
  if (!g_pp.active) return;
  PendPool q = g_pp;
  g_pp.active = false;
  pool_impl(&q.images, nullptr, &q.targets, q.numFilters, q.subsX, q.startX, q.strideX, q.outputsX, "MaxPool");
}
static const int g_pool_flush_registered = (dn_set_ext_flush_hook(pool_flush), 0);

// Holds the call back when MaxPoolResponseNorm's one-launch kernel could serve it (the conditions of
// that entry point on the pooling side; anything else, errors included, takes the usual path).
static bool pool_hold(cudamat* images, cudamat* targets, int numFilters, int subsX, int startX, int strideX, int outputsX) {
  if (!dn_defer_enabled()) return false;
  if (!images->on_device || !targets->on_device || numFilters <= 0 || outputsX <= 0) return false;
  if (!(strideX == 2 && (subsX == 2 || subsX == 3))) return false;
  const int N = images->size[0];
  if (N <= 0 || N % 4 != 0 || images->size[1] % numFilters != 0 || isqrt_exact_p(images->size[1] / numFilters) <= 0) return false;
  if (targets->size[0] != N || targets->size[1] != numFilters * outputsX * outputsX) return false;
  if (!all_aligned16({images->data_device, targets->data_device}) || images->data_device == targets->data_device) return false;
  if (norm_lds_qb(N, outputsX) <= 0 || (long long)N * images->size[1] >= (1ll << 31)) return false;
  dn_flush();                       // (what either library holds back comes first)
  conv_clear_error();
  g_pp.active = true;
  g_pp.images = *images; g_pp.targets = *targets;
  g_pp.numFilters = numFilters; g_pp.subsX = subsX; g_pp.startX = startX; g_pp.strideX = strideX; g_pp.outputsX = outputsX;
  dn_set_ext_pending(true);
  return true;
}

static void cnorm_impl(cudamat* images, cudamat* meanDiffs, cudamat* denoms, cudamat* targets, int numFilters,
                       int sizeX, float addScale, float powScale, const char* where) {
  conv_clear_error();
  POOL_REQUIRE(images->on_device && meanDiffs->on_device && denoms->on_device && targets->on_device, where);
  POOL_REQUIRE(numFilters > 0 && sizeX > 0, where);
  const int N = images->size[0];
  POOL_REQUIRE(N > 0 && images->size[1] % numFilters == 0, where);
  const int S = isqrt_exact_p(images->size[1] / numFilters);
  POOL_REQUIRE(S > 0, where);
  for (cudamat* m : {meanDiffs, denoms, targets})
    POOL_REQUIRE(m->size[0] == N && m->size[1] == images->size[1], where);
  const long long total = (long long)N * images->size[1];
  POOL_REQUIRE(total < (1ll << 32), where);
  const bool v4 = N % 4 == 0 && all_aligned16({images->data_device, meanDiffs->data_device, denoms->data_device,
                                               targets->data_device});
  PoolGeom g;
  make_geom(g, N, numFilters, S, S, 0, 0, 1, v4 ? 4 : 1);
  const unsigned grid = grid_for(total / (v4 ? 4 : 1));
#define CNORM_GO(VW)                                                                                           \
  hipLaunchKernelGGL((k_cnorm<VW>)    , dim3(grid), dim3(256), 0, dn_stream(), (const float*)images->data_device,         \
                     (const float*)meanDiffs->data_device, denoms->data_device, targets->data_device, g, sizeX, \
                     addScale, powScale)
#define CNORM_ROWS(SZ)                                                                                          \
  hipLaunchKernelGGL((k_norm_rows<4, SZ, NORM_SEG, false>), dim3(grid_for((long long)g.NV * S * nseg * numFilters)), \
                     dim3(256), 0, dn_stream(), (const float*)images->data_device, (const float*)nullptr,                  \
                     (const float*)nullptr, (const float*)meanDiffs->data_device, denoms->data_device,           \
                     targets->data_device, g, nseg, make_fastdiv((uint32_t)nseg), addScale, powScale)
  const int nseg = (S + NORM_SEG - 1) / NORM_SEG;
  const int qb = v4 ? norm_lds_qb(N, S) : 0;
  if (qb > 0 && (long long)numFilters * ((N + qb * 4 - 1) / (qb * 4)) <= 0x7fffffffll) {
    norm_lds_launch<false>(qb, images->data_device == meanDiffs->data_device, images->data_device, nullptr, nullptr,
                           meanDiffs->data_device, denoms->data_device, targets->data_device, N, S, numFilters, sizeX,
                           addScale, powScale);
  } else if (v4) {
    if (sizeX == 3) CNORM_ROWS(3);
    else if (sizeX == 5) CNORM_ROWS(5);
    else if (sizeX == 7) CNORM_ROWS(7);
    else CNORM_GO(4);
  } else {
    CNORM_GO(1);
  }
#undef CNORM_GO
#undef CNORM_ROWS
  if (dn_launch_status()) conv_set_error(where, hipGetErrorString(hipGetLastError()));
}

static void rnorm_undo_impl(cudamat* outGrads, cudamat* denoms, cudamat* inputs, cudamat* acts, cudamat* targets,
                            int numFilters, int sizeX, float addScale, float powScale, const char* where) {
  conv_clear_error();
  POOL_REQUIRE(outGrads->on_device && denoms->on_device && inputs->on_device && acts->on_device && targets->on_device,
               where);
  POOL_REQUIRE(numFilters > 0 && sizeX > 0, where);
  const int N = outGrads->size[0];
  POOL_REQUIRE(N > 0 && outGrads->size[1] % numFilters == 0, where);
  const int S = isqrt_exact_p(outGrads->size[1] / numFilters);
  POOL_REQUIRE(S > 0, where);
  for (cudamat* m : {denoms, inputs, acts, targets})
    POOL_REQUIRE(m->size[0] == N && m->size[1] == outGrads->size[1], where);
  const long long total = (long long)N * outGrads->size[1];
  POOL_REQUIRE(total < (1ll << 32), where);
  {
    const bool v4all = N % 4 == 0 && all_aligned16({outGrads->data_device, denoms->data_device, inputs->data_device,
                                                    acts->data_device, targets->data_device});
    const int qb = v4all ? norm_lds_qb(N, S) : 0;
    if (qb > 0) {
      norm_lds_launch<true>(qb, false, outGrads->data_device, denoms->data_device, inputs->data_device, acts->data_device,
                            nullptr, targets->data_device, N, S, numFilters, sizeX, -2.f * addScale * powScale, powScale);
      if (dn_launch_status()) conv_set_error(where, hipGetErrorString(hipGetLastError()));
      return;
    }
  }
  if (total % 4 == 0 && all_aligned16({acts->data_device, denoms->data_device, outGrads->data_device}))
    hipLaunchKernelGGL((k_rnorm_undo_prelim<4>), dim3(grid_for(total / 4)), dim3(256), 0, dn_stream(), acts->data_device,
                       (const float*)denoms->data_device, (const float*)outGrads->data_device, (size_t)(total / 4),
                       -2.f * addScale * powScale);
  else
    hipLaunchKernelGGL((k_rnorm_undo_prelim<1>), dim3(grid_for(total)), dim3(256), 0, dn_stream(), acts->data_device,
                       (const float*)denoms->data_device, (const float*)outGrads->data_device, (size_t)total,
                       -2.f * addScale * powScale);
  const bool v4 = N % 4 == 0 && all_aligned16({outGrads->data_device, denoms->data_device, inputs->data_device,
                                               acts->data_device, targets->data_device});
  PoolGeom g;
  make_geom(g, N, numFilters, S, S, 0, 0, 1, v4 ? 4 : 1);
  const unsigned grid = grid_for(total / (v4 ? 4 : 1));
#define RUNDO_GO(VW)                                                                                          \
  hipLaunchKernelGGL((k_rnorm_undo<VW>)    , dim3(grid), dim3(256), 0, dn_stream(), (const float*)outGrads->data_device, \
                     (const float*)denoms->data_device, (const float*)inputs->data_device,                     \
                     (const float*)acts->data_device, targets->data_device, g, sizeX, powScale)
#define RUNDO_ROWS(SZ)                                                                                         \
  hipLaunchKernelGGL((k_norm_rows<4, SZ, NORM_SEG, true>), dim3(grid_for((long long)g.NV * S * nseg * numFilters)), \
                     dim3(256), 0, dn_stream(), (const float*)outGrads->data_device, (const float*)denoms->data_device,   \
                     (const float*)inputs->data_device, (const float*)acts->data_device, (float*)nullptr,       \
                     targets->data_device, g, nseg, make_fastdiv((uint32_t)nseg), 0.f, powScale)
  const int nseg = (S + NORM_SEG - 1) / NORM_SEG;
  if (v4) {
    if (sizeX == 3) RUNDO_ROWS(3);
    else if (sizeX == 5) RUNDO_ROWS(5);
    else if (sizeX == 7) RUNDO_ROWS(7);
    else RUNDO_GO(4);
  } else {
    RUNDO_GO(1);
  }
#undef RUNDO_GO
#undef RUNDO_ROWS
  if (dn_launch_status()) conv_set_error(where, hipGetErrorString(hipGetLastError()));
}

extern "C" {

void MaxPool(cudamat* images, cudamat* targets, int numFilters, int subsX, int startX, int strideX, int outputsX) {
  if (pool_hold(images, targets, numFilters, subsX, startX, strideX, outputsX)) return;
  pool_impl(images, nullptr, targets, numFilters, subsX, startX, strideX, outputsX, "MaxPool");
}

void ProbMaxPool(cudamat* images, cudamat* rnd, cudamat* targets, int numFilters, int subsX, int startX, int strideX,
                 int outputsX) {
  conv_clear_error();
  POOL_REQUIRE(rnd != nullptr, "ProbMaxPool");
  pool_impl(images, rnd, targets, numFilters, subsX, startX, strideX, outputsX, "ProbMaxPool");
}

void MaxPoolUndo(cudamat* images, cudamat* maxGrads, cudamat* maxActs, cudamat* targets, int subsX, int startX,
                 int strideX, int outputsX) {
  const char* where = "MaxPoolUndo";
  conv_clear_error();
  POOL_REQUIRE(images->on_device && maxGrads->on_device && maxActs->on_device && targets->on_device, where);
  POOL_REQUIRE(subsX > 0 && strideX > 0 && outputsX > 0, where);
  const int N = images->size[0];
  const int outputs = outputsX * outputsX;
  POOL_REQUIRE(N > 0 && maxGrads->size[1] % outputs == 0, where);
  const int F = maxGrads->size[1] / outputs;
  POOL_REQUIRE(F > 0 && images->size[1] % F == 0, where);
  const int S = isqrt_exact_p(images->size[1] / F);
  POOL_REQUIRE(S > 0, where);
  POOL_REQUIRE(maxGrads->size[0] == N && maxActs->size[0] == N && maxActs->size[1] == maxGrads->size[1], where);
  POOL_REQUIRE(targets->size[0] == N && targets->size[1] == images->size[1], where);
  const long long total = (long long)N * images->size[1];
  POOL_REQUIRE(total < (1ll << 32), where);
  const bool v4 = N % 4 == 0 && all_aligned16({images->data_device, maxGrads->data_device, maxActs->data_device,
                                               targets->data_device});
  PoolGeom g;
  make_geom(g, N, F, S, outputsX, subsX, startX, strideX, v4 ? 4 : 1);
  const unsigned grid = grid_for(total / (v4 ? 4 : 1));
  // (measured against the one-pixel kernel at batch 128: 64 maps of 32 x 32 17.7 -> 16.2 us, of
  // 24 x 24 12.8 -> 9.4 us, 256 of 27 x 27 56.9 -> 42.8 us, 96 of 55 x 55 95 -> 68 us; 64 maps of
  // 32 x 32 at batch 256 30.5 -> 31.9 us)
  if (v4 && g.stride == 2 && g.start == 0 && (g.subs == 2 || g.subs == 3) && g.S >= 4) {
    const int B = (g.S + 1) / 2;
    const FastDiv dB = make_fastdiv((uint32_t)B);
    const unsigned grid2 = grid_for((long long)g.NV * B * B * g.F);
    if (g.subs == 3)
      hipLaunchKernelGGL((k_pool_undo_block2<3>), dim3(grid2), dim3(256), 0, dn_stream(), (const float*)images->data_device,
                         (const float*)maxGrads->data_device, (const float*)maxActs->data_device, targets->data_device, g, B, dB);
    else
      hipLaunchKernelGGL((k_pool_undo_block2<2>), dim3(grid2), dim3(256), 0, dn_stream(), (const float*)images->data_device,
                         (const float*)maxGrads->data_device, (const float*)maxActs->data_device, targets->data_device, g, B, dB);
  } else if (v4 && g.subs == 3 && g.stride == 2)
    hipLaunchKernelGGL((k_pool_undo_fixed<3, 2>), dim3(grid), dim3(256), 0, dn_stream(), (const float*)images->data_device,
                       (const float*)maxGrads->data_device, (const float*)maxActs->data_device, targets->data_device, g);
  else if (v4 && g.subs == 2 && g.stride == 2)
    hipLaunchKernelGGL((k_pool_undo_fixed<2, 2>), dim3(grid), dim3(256), 0, dn_stream(), (const float*)images->data_device,
                       (const float*)maxGrads->data_device, (const float*)maxActs->data_device, targets->data_device, g);
  else if (v4)
    hipLaunchKernelGGL((k_pool_undo<4>), dim3(grid), dim3(256), 0, dn_stream(), (const float*)images->data_device,
                       (const float*)maxGrads->data_device, (const float*)maxActs->data_device, targets->data_device, g);
  else
    hipLaunchKernelGGL((k_pool_undo<1>), dim3(grid), dim3(256), 0, dn_stream(), (const float*)images->data_device,
                       (const float*)maxGrads->data_device, (const float*)maxActs->data_device, targets->data_device, g);
  if (dn_launch_status()) conv_set_error(where, hipGetErrorString(hipGetLastError()));
}

void MaxPoolResponseNorm(cudamat* images, cudamat* pooled, cudamat* denoms, cudamat* targets, int numFilters, int subsX,
                         int startX, int strideX, int outputsX, int sizeX, float addScale, float powScale);

void ResponseNorm(cudamat* images, cudamat* denoms, cudamat* targets, int numFilters, int sizeX, float addScale,
                  float powScale) {
  // (the normalisation of a pooled map whose MaxPool is being held back: both in one launch)
  if (g_pp.active && images->on_device && images->data_device == g_pp.targets.data_device && images->size[0] == g_pp.targets.size[0] &&
      images->size[1] == g_pp.targets.size[1] && numFilters == g_pp.numFilters && sizeX > 0 && denoms->on_device &&
      targets->on_device && denoms->size[0] == images->size[0] && denoms->size[1] == images->size[1] &&
      targets->size[0] == images->size[0] && targets->size[1] == images->size[1]) {
    PendPool q = g_pp;
    g_pp.active = false;
    dn_set_ext_pending(false);
    MaxPoolResponseNorm(&q.images, images, denoms, targets, numFilters, q.subsX, q.startX, q.strideX, q.outputsX, sizeX,
                        addScale, powScale);
    return;
  }
  cnorm_impl(images, images, denoms, targets, numFilters, sizeX, addScale, powScale, "ResponseNorm");
}

void ContrastNorm(cudamat* images, cudamat* meanDiffs, cudamat* denoms, cudamat* targets, int numFilters, int sizeX,
                  float addScale, float powScale) {
  cnorm_impl(images, meanDiffs, denoms, targets, numFilters, sizeX, addScale, powScale, "ContrastNorm");
}

void ResponseNormUndo(cudamat* outGrads, cudamat* denoms, cudamat* inputs, cudamat* acts, cudamat* targets,
                      int numFilters, int sizeX, float addScale, float powScale) {
  rnorm_undo_impl(outGrads, denoms, inputs, acts, targets, numFilters, sizeX, addScale, powScale, "ResponseNormUndo");
}

void ContrastNormUndo(cudamat* outGrads, cudamat* denoms, cudamat* meanDiffs, cudamat* acts, cudamat* targets,
                      int numFilters, int sizeX, float addScale, float powScale) {
  rnorm_undo_impl(outGrads, denoms, meanDiffs, acts, targets, numFilters, sizeX, addScale, powScale,
                  "ContrastNormUndo");
}

// ---- Extensions (no counterpart in cudamat_conv.cu): the two pairs of calls deepnet always makes
// back to back (deepnet/convolutions.py:58-66, 120-134), each in one launch where the pooled map of
// 32 (16, 8, 4) images fits in LDS, the separate kernels otherwise; the same results either way.

// pooled = MaxPool(images); (denoms, targets) = ResponseNorm(pooled)
void MaxPoolResponseNorm(cudamat* images, cudamat* pooled, cudamat* denoms, cudamat* targets, int numFilters, int subsX,
                         int startX, int strideX, int outputsX, int sizeX, float addScale, float powScale) {
  const char* where = "MaxPoolResponseNorm";
  conv_clear_error();
  POOL_REQUIRE(images->on_device && pooled->on_device && denoms->on_device && targets->on_device, where);
  POOL_REQUIRE(numFilters > 0 && subsX > 0 && strideX > 0 && outputsX > 0 && sizeX > 0, where);
  const int N = images->size[0];
  POOL_REQUIRE(N > 0 && images->size[1] % numFilters == 0, where);
  const int Sin = isqrt_exact_p(images->size[1] / numFilters);
  POOL_REQUIRE(Sin > 0, where);
  for (cudamat* m : {pooled, denoms, targets})
    POOL_REQUIRE(m->size[0] == N && m->size[1] == numFilters * outputsX * outputsX, where);
  const bool v4 = N % 4 == 0 && all_aligned16({images->data_device, pooled->data_device, denoms->data_device, targets->data_device});
  const int qb = v4 ? norm_lds_qb(N, outputsX) : 0;
  const bool shapes = (strideX == 2 && (subsX == 2 || subsX == 3)) && (sizeX == 3 || sizeX == 5 || sizeX == 7);
  const bool distinct = pooled->data_device != denoms->data_device && pooled->data_device != targets->data_device &&
                        denoms->data_device != targets->data_device && images->data_device != pooled->data_device &&
                        images->data_device != denoms->data_device && images->data_device != targets->data_device;
  if (qb > 0 && shapes && distinct && (long long)N * images->size[1] < (1ll << 31)) {
    const int nblk = (N + qb * 4 - 1) / (qb * 4);
    const dim3 grid((unsigned)(numFilters * nblk)), block(NORM_LDS_THREADS);
    const size_t lds = (size_t)2 * outputsX * outputsX * qb * sizeof(float4);
    const FastDiv dS = make_fastdiv((uint32_t)outputsX);
#define PN_GO(QB, SU, SZ) \
  hipLaunchKernelGGL((k_pool_norm_lds<QB, SU, 2, SZ>), grid, block, lds, dn_stream(), (const float*)images->data_device, \
                     pooled->data_device, denoms->data_device, targets->data_device, N, Sin, startX, outputsX, dS, nblk, addScale, powScale)
#define PN_SZ(QB, SU) do { if (sizeX == 3) PN_GO(QB, SU, 3); else if (sizeX == 5) PN_GO(QB, SU, 5); else PN_GO(QB, SU, 7); } while (0)
#define PN_SU(QB) do { if (subsX == 3) PN_SZ(QB, 3); else PN_SZ(QB, 2); } while (0)
    if (qb == 8) PN_SU(8); else if (qb == 4) PN_SU(4); else if (qb == 2) PN_SU(2); else PN_SU(1);
#undef PN_SU
#undef PN_SZ
#undef PN_GO
    if (dn_launch_status()) conv_set_error(where, hipGetErrorString(hipGetLastError()));
    return;
  }
  pool_impl(images, nullptr, pooled, numFilters, subsX, startX, strideX, outputsX, where);
  if (conv_last_error()) return;
  cnorm_impl(pooled, pooled, denoms, targets, numFilters, sizeX, addScale, powScale, where);
}

// targets = MaxPoolUndo(images, maxGrads = ResponseNormUndo(outGrads, denoms, inputs, acts), maxActs = acts):
// `acts` are the pooled activations, and unlike ResponseNormUndo this call leaves them as they are.
// targets may be images.
void ResponseNormUndoMaxPoolUndo(cudamat* outGrads, cudamat* denoms, cudamat* inputs, cudamat* acts, cudamat* images,
                                 cudamat* targets, int numFilters, int subsX, int startX, int strideX, int outputsX, int sizeX,
                                 float addScale, float powScale) {
  const char* where = "ResponseNormUndoMaxPoolUndo";
  conv_clear_error();
  POOL_REQUIRE(outGrads->on_device && denoms->on_device && inputs->on_device && acts->on_device && images->on_device &&
               targets->on_device, where);
  POOL_REQUIRE(numFilters > 0 && subsX > 0 && strideX > 0 && outputsX > 0 && sizeX > 0, where);
  const int N = images->size[0];
  POOL_REQUIRE(N > 0 && images->size[1] % numFilters == 0, where);
  const int Sin = isqrt_exact_p(images->size[1] / numFilters);
  POOL_REQUIRE(Sin > 0, where);
  for (cudamat* m : {outGrads, denoms, inputs, acts})
    POOL_REQUIRE(m->size[0] == N && m->size[1] == numFilters * outputsX * outputsX, where);
  POOL_REQUIRE(targets->size[0] == N && targets->size[1] == images->size[1], where);
  const bool v4 = N % 4 == 0 && all_aligned16({outGrads->data_device, denoms->data_device, inputs->data_device, acts->data_device,
                                               images->data_device, targets->data_device});
  const int qb = v4 ? norm_lds_qb(N, outputsX) : 0;
  const bool shapes = (strideX == 2 && (subsX == 2 || subsX == 3)) && (sizeX == 3 || sizeX == 5 || sizeX == 7);
  const size_t lds = (size_t)3 * outputsX * outputsX * (qb > 0 ? qb : 1) * sizeof(float4);
  if (qb > 0 && shapes && lds <= 144 * 1024 && (long long)N * images->size[1] < (1ll << 31)) {
    const int nblk = (N + qb * 4 - 1) / (qb * 4);
    const dim3 grid((unsigned)(numFilters * nblk)), block(NORM_LDS_THREADS);
    const FastDiv dS = make_fastdiv((uint32_t)outputsX), dSin = make_fastdiv((uint32_t)Sin);
    const float scale = -2.f * addScale * powScale;
    bool attr_ok = true;
#define NP_GO(QB, SU, SZ)                                                                                                    \
  do {                                                                                                                       \
    static bool raised = false;   /* more than 64 KiB of dynamic LDS has to be asked for once per kernel */                  \
    if (!raised && lds > 64 * 1024) {                                                                                        \
      attr_ok = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_normundo_poolundo_lds<QB, SU, 2, SZ>),                  \
                                    hipFuncAttributeMaxDynamicSharedMemorySize, 144 * 1024) == hipSuccess;                   \
      raised = attr_ok;                                                                                                      \
    }                                                                                                                        \
    if (attr_ok)                                                                                                             \
      hipLaunchKernelGGL((k_normundo_poolundo_lds<QB, SU, 2, SZ>), grid, block, lds, dn_stream(),                            \
                         (const float*)outGrads->data_device, (const float*)denoms->data_device,                             \
                         (const float*)inputs->data_device, (const float*)acts->data_device, (const float*)images->data_device, \
                         targets->data_device, N, Sin, dSin, startX, outputsX, dS, nblk, scale, powScale);                   \
  } while (0)
#define NP_SZ(QB, SU) do { if (sizeX == 3) NP_GO(QB, SU, 3); else if (sizeX == 5) NP_GO(QB, SU, 5); else NP_GO(QB, SU, 7); } while (0)
#define NP_SU(QB) do { if (subsX == 3) NP_SZ(QB, 3); else NP_SZ(QB, 2); } while (0)
    if (qb == 8) NP_SU(8); else if (qb == 4) NP_SU(4); else if (qb == 2) NP_SU(2); else NP_SU(1);
#undef NP_SU
#undef NP_SZ
#undef NP_GO
    if (attr_ok) {
      if (dn_launch_status()) conv_set_error(where, hipGetErrorString(hipGetLastError()));
      return;
    }
    hipGetLastError();
  }
  // the separate kernels, on a copy of the pooled activations (ResponseNormUndo overwrites its acts) and a
  // temporary for the pooled map's gradient
  const size_t pooled_floats = (size_t)N * acts->size[1];
  float* ws = (float*)dn_scratch(2 * pooled_floats * sizeof(float), 2);
  if (!ws) { conv_set_error(where, "out of device memory for the temporaries"); return; }
  cudamat acts_copy = *acts, grad = *acts;
  acts_copy.data_device = ws; acts_copy.owns_data = 0; acts_copy.is_trans = 0;
  grad.data_device = ws + pooled_floats; grad.owns_data = 0; grad.is_trans = 0;
  if (copy_on_device(acts, &acts_copy)) { conv_set_error(where, "copy of the pooled activations failed"); return; }
  rnorm_undo_impl(outGrads, denoms, inputs, &acts_copy, &grad, numFilters, sizeX, addScale, powScale, where);
  if (conv_last_error()) return;
  MaxPoolUndo(images, &grad, acts, targets, subsX, startX, strideX, outputsX);
}

}  // extern "C"
