// Shared-filter convolution in cuda-convnet's (channels, rows, cols, batch)
// layout: forward (convUp), gradient w.r.t. the images (convDown) and w.r.t. the
// filters (convOutp).  Replaces cudamat/cudamat_conv.cu:15-1015 and the kernel
// templates cudamat_conv_kernels.cuh:82-1235.
//
// All three passes are one implicit GEMM  C(r, c) = sum_kk A(r, kk) * B(kk, c)  on
// the fp32 matrix cores (v_mfma_f32_32x32x2_f32), with 16-deep operand slabs
// gathered straight from the tensors into LDS (double buffered):
//
//   pass   rows r                 cols c            kk                 A                 B
//   Up     (module, image)        filter of group   (colour, ky, kx)   image patch       filters
//   Down   (pixel of phase, img)  colour of group   (tap, filter)      hidden acts       filters
//   Outp   filter of group        (colour, ky, kx)  (module, image)    hidden acts       image patch
//
// The batch index is the fastest-varying one everywhere, so rows of Up/Down and
// the kk of Outp are contiguous runs of images: every gather is a 16-byte load of
// four neighbouring images.  Down with stride s runs as s*s "phases" (pixels with
// equal (y - pad) mod s share their set of filter taps), which turns the strided
// transpose convolution into stride-1 problems without multiplying by zeros.
// Outp reduces over modules x images with few outputs, so K is split across
// workgroups and summed by a second kernel.
//
// The matrix-core path needs numImages % 16 == 0, filters-per-group % 16 == 0 and
// 16-byte aligned buffers; other batches above 16 images and other filter counts (one
// group) are padded into a workspace by the entry points (see padded_batch,
// padded_filters), and anything else takes the one-thread-per-output
// kernels below, which are also the cross-check of the fast path in the tests.
//
// First-layer shapes (few colours, few filters) have their own kernels further down,
// because a 16-deep, 128-column LDS pipeline is mostly prologue and padding for them:
//   k_conv_up_regs     convUp with colours*k*k <= 80: filter bank in registers
//   k_conv_patch_regs  convDown, stride 1, <= 16 colours: P = hid * W in registers,
//                      then k_conv_down_gather(_s1) sums the entries that land on a pixel
//   k_conv_outp_regs   convOutp with <= 64 x 80 outputs: both operands straight from global
//                      memory into 16 x 16 x 4 matrix-core operands, no LDS tiles
//   k_conv_outp_small  convOutp with <= 64 x 96 outputs: [row][image] LDS tiles, every
//                      wavefront holds the whole output block
#include "common.h"
#include <type_traits>

#include "../../include/cudamat_conv_amd.h"
#include <math.h>
#include <stdio.h>

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// CONV_DOWNM: convDown for strided layers with few colours, all stride*stride pixel
// phases merged into the columns of one product (uniform-row kernels only).
enum { CONV_UP = 0, CONV_DOWN = 1, CONV_OUTP = 2, CONV_DOWNM = 3 };

struct ConvArgs {
  const float* img;   // images: input of Up/Outp
  const float* flt;   // filters: input of Up/Down
  const float* hid;   // hidden activations / their gradients: input of Down/Outp
  float* out;         // Up: hidden acts, Down: images, Outp: filter gradients
  float* partial;     // Outp split-K workspace
  int N, C, Cg, H, F, Fg, k, Mx, s, pad0, G;
  int M, HH, kk2;     // Mx*Mx, H*H, k*k
  int m_begin, m_count;  // Outp: module chunk [m_begin, m_begin + m_count)
  int chunks;            // Outp, general kernel: chunks of m_count modules batched along grid z (1: one chunk)
  int splits, slabs_per_split;   // Outp always; Up / Down (stride 1) when the tiles alone cannot fill the chip
  long long split_stride;        // Up / Down with splits > 1: elements between the partial outputs in `partial`
  int local;          // 1: one filter bank per module (locally connected layers); direct and uniform-row kernels
  float scale_t, scale_o;
  unsigned a_bytes, b_bytes;  // sizes of the two gathered arrays (uniform-row kernels: buffer ranges)
  int yq;             // CONV_DOWNM: stride x stride pixel blocks per image side
  FastDiv dN, dMx, dk, dkk2, dS, dSS;
};

// ------------------------------------------------------------------ direct kernels
// One lane per output element; images are the fastest index, so neighbouring
// lanes read neighbouring addresses.

__global__ void k_conv_up_direct(ConvArgs p) {
  const long long total = (long long)p.N * p.M * p.F;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += stride) {
    const int n = (int)(e % p.N);
    const int m = (int)((e / p.N) % p.M);
    const int f = (int)(e / ((long long)p.N * p.M));
    const int g = f / p.Fg;
    const int y0 = (m / p.Mx) * p.s + p.pad0, x0 = (m % p.Mx) * p.s + p.pad0;
    const float* flt = p.flt + (p.local ? (size_t)m * p.Cg * p.kk2 * p.F : 0);
    float acc = 0.f;
    for (int c = 0; c < p.Cg; ++c)
      for (int ky = 0; ky < p.k; ++ky) {
        const int y = y0 + ky;
        if (y < 0 || y >= p.H) continue;
        for (int kx = 0; kx < p.k; ++kx) {
          const int x = x0 + kx;
          if (x < 0 || x >= p.H) continue;
          acc += p.img[(size_t)p.N * ((size_t)(g * p.Cg + c) * p.HH + y * p.H + x) + n] *
                 flt[(size_t)p.F * ((c * p.k + ky) * p.k + kx) + f];
        }
      }
    p.out[e] = (p.scale_t == 0.f ? 0.f : p.scale_t * p.out[e]) + p.scale_o * acc;
  }
}

__global__ void k_conv_down_direct(ConvArgs p) {
  const long long total = (long long)p.N * p.HH * p.C;
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += stride) {
    const int n = (int)(e % p.N);
    const int pix = (int)((e / p.N) % p.HH);
    const int c = (int)(e / ((long long)p.N * p.HH));
    const int g = c / p.Cg, cl = c % p.Cg;
    const int y = pix / p.H - p.pad0, x = pix % p.H - p.pad0;  // coordinates in the padded frame
    float acc = 0.f;
    for (int my = 0; my < p.Mx; ++my) {
      const int ky = y - my * p.s;
      if (ky < 0 || ky >= p.k) continue;
      for (int mx = 0; mx < p.Mx; ++mx) {
        const int kx = x - mx * p.s;
        if (kx < 0 || kx >= p.k) continue;
        const size_t wbase = (size_t)p.F * ((cl * p.k + ky) * p.k + kx) +
                             (p.local ? (size_t)(my * p.Mx + mx) * p.Cg * p.kk2 * p.F : 0);
        for (int fl = 0; fl < p.Fg; ++fl) {
          const int f = g * p.Fg + fl;
          acc += p.hid[(size_t)p.N * ((size_t)f * p.M + my * p.Mx + mx) + n] * p.flt[wbase + f];
        }
      }
    }
    p.out[e] = (p.scale_t == 0.f ? 0.f : p.scale_t * p.out[e]) + p.scale_o * acc;
  }
}

// One workgroup per output (f, c, ky, kx): 256 lanes stride over (module, image)
// of the chunk and meet in LDS.
__global__ void __launch_bounds__(256) k_conv_outp_direct(ConvArgs p) {
  __shared__ float red[4];
  const int q = blockIdx.x % (p.Cg * p.kk2);
  const int f = blockIdx.x / (p.Cg * p.kk2);
  const int g = f / p.Fg;
  const int c = q / p.kk2, ky = (q % p.kk2) / p.k, kx = q % p.k;
  const long long total = (long long)p.m_count * p.N;
  float acc = 0.f;
  for (long long e = threadIdx.x; e < total; e += 256) {
    const int n = (int)(e % p.N);
    const int m = p.m_begin + (int)(e / p.N);
    const int y = (m / p.Mx) * p.s + p.pad0 + ky, x = (m % p.Mx) * p.s + p.pad0 + kx;
    if (y < 0 || y >= p.H || x < 0 || x >= p.H) continue;
    acc += p.img[(size_t)p.N * ((size_t)(g * p.Cg + c) * p.HH + y * p.H + x) + n] *
           p.hid[(size_t)p.N * ((size_t)f * p.M + m) + n];
  }
  acc = wave_sum(acc);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    const float s = (red[0] + red[1]) + (red[2] + red[3]);
    float* t = p.out + (size_t)p.F * q + f;
    *t = (p.scale_t == 0.f ? 0.f : p.scale_t * *t) + p.scale_o * s;
  }
}

// ------------------------------------------------------------------ matrix-core kernel

#define CV_BK 16
#define CV_PAD 4

// Geometry of one Down phase (py, px): the pixels y = y_first + s*i, i < QY, whose
// taps are ky = py + s*t, t < TY, reaching module my = qy_first + i - t.
struct DownPhase {
  int py, px, y_first, x_first, QY, QX, qy_first, qx_first, TY, TX;
};
__device__ __forceinline__ void down_axis(int ph, int s, int pad0, int H, int k, int* first, int* Q, int* qfirst,
                                          int* T) {
  // smallest y >= 0 with (y - pad0) % s == ph   (pad0 <= 0)
  int y = ph + pad0;            // (y - pad0) == ph
  if (y < 0) y += ((-y + s - 1) / s) * s;
  *first = y;
  *Q = y < H ? (H - 1 - y) / s + 1 : 0;
  *qfirst = (y - pad0 - ph) / s;
  *T = ph < k ? (k - ph + s - 1) / s : 0;
}

// UNI (Up / Down, 128-row tiles, batch a multiple of 128): all rows of a tile belong to
// one module (Up) or one pixel (Down), so whether a tap falls into the padding is a
// scalar question.  The gathers then are buffer loads -- lane offset fixed for the whole
// kernel, slab offset in an SGPR, an out-of-range offset for a tap in the padding, which
// the hardware answers with zeros -- and cost no vector instructions, which matters
// because fp32 MFMA and the vector ALU share lanes.  Both operands run two slabs ahead.
// INSIDE (general gathers of the image: convUp rows, convOutp columns): no padding and the
// last module ends inside the image, so no image group is ever masked and its gather is
// an add and a load.  convUp: the rows fill their tiles, and a tap beyond the reduction
// re-reads the last one against a zero filter row.  convOutp: rows and columns beyond
// the output are computed on whatever valid data was read and never stored.
// (the merged-phase convDown kernels are asked to fit four wavefronts per SIMD, 128 registers: the
// 3 colours x 16 phases of config 5a then run 288 us instead of 307; the same request costs every
// other variant time -- config 5b's convOutp 530 -> 675 us with 168 registers and spills)
template <int MODE, int WAVES_M, int WM, int WN, bool UNI = false, int N16 = 0, bool INSIDE = false, bool LOCAL = false>
__global__ void __launch_bounds__(256, (MODE == CONV_DOWNM && WM * WN <= 2 ? 4 : 0)) k_conv_mfma(ConvArgs p) {
  static_assert(!LOCAL || UNI, "one filter bank per module: uniform-row kernels only");
  static_assert(!INSIDE || ((MODE == CONV_UP || MODE == CONV_OUTP) && !UNI), "INSIDE: the general gathers of the image");
  constexpr int WAVES_N = 4 / WAVES_M;
  constexpr int BM = 32 * WM * WAVES_M, BN = 32 * WN * WAVES_N;
  // Row pitch in LDS: operands written transposed one float per lane want pitch % 8 == 2
  // (no bank conflicts), those written 16 bytes at a time need pitch % 4 == 0.
  // (16-wide blocks read k rows 4 apart per lane group: both pitches are then 4 mod 8, rows 16 banks apart)
  constexpr int LA = BM + (MODE == CONV_OUTP ? 2 : CV_PAD), LB = BN + (MODE == CONV_UP || N16 > 0 ? CV_PAD : 2);
  constexpr int TA = BM * CV_BK / 4, TB = BN * CV_BK / 4;  // 16-byte groups per slab
  constexpr int NA = (TA + 255) / 256, NB = (TB + 255) / 256;
  __shared__ __attribute__((aligned(16))) float As[2][CV_BK][LA];
  __shared__ __attribute__((aligned(16))) float Bs[2][CV_BK][LB];

  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int wm = wv % WAVES_M, wn = wv / WAVES_M;
  const int lk = lane >> 5, li = lane & 31;
  const int N = p.N, H = p.H, HH = p.HH, Mx = p.Mx, M = p.M, F = p.F, Fg = p.Fg, Cg = p.Cg, k = p.k, s = p.s;

  // ---- what this workgroup computes
  int g, rows, cols, nslabs, slab_beg, slab_end, zsplit = 0, out_chunk = 0;
  DownPhase ph;
  if (MODE == CONV_UP) {
    g = blockIdx.z / p.splits;
    zsplit = blockIdx.z % p.splits;
    rows = M * N; cols = Fg;
    nslabs = (Cg * p.kk2 + CV_BK - 1) / CV_BK;
    slab_beg = p.splits > 1 ? zsplit * p.slabs_per_split : 0;
    slab_end = p.splits > 1 && slab_beg + p.slabs_per_split < nslabs ? slab_beg + p.slabs_per_split : nslabs;
  } else if (MODE == CONV_DOWNM) {
    // Rows: (Y, X, image) over blocks of s x s pixels in padded coordinates, pixel
    // y = Y*s + py + pad0.  Columns: (colour, py, px).  K: (t, u, filter) with the tap
    // ky = t*s + py of module Y - t (zero weight where ky >= k).
    g = blockIdx.z;
    const int T = (k + s - 1) / s;
    ph.py = ph.px = 0; ph.y_first = ph.x_first = p.pad0;
    ph.QY = ph.QX = p.yq; ph.qy_first = ph.qx_first = 0; ph.TY = ph.TX = T;
    rows = p.yq * p.yq * N; cols = Cg * s * s;
    nslabs = T * T * (Fg / CV_BK);
    slab_beg = 0; slab_end = nslabs;
  } else if (MODE == CONV_DOWN) {
    const int nph = s * s;
    const int zz = blockIdx.z / p.splits;             // (splits > 1 only with stride 1: one phase)
    zsplit = blockIdx.z % p.splits;
    g = zz / nph;
    const int phase = zz % nph;
    ph.py = phase / s; ph.px = phase % s;
    down_axis(ph.py, s, p.pad0, H, k, &ph.y_first, &ph.QY, &ph.qy_first, &ph.TY);
    down_axis(ph.px, s, p.pad0, H, k, &ph.x_first, &ph.QX, &ph.qx_first, &ph.TX);
    rows = ph.QY * ph.QX * N; cols = Cg;
    nslabs = ph.TY * ph.TX * (Fg / CV_BK);
    slab_beg = p.splits > 1 ? zsplit * p.slabs_per_split : 0;
    slab_end = p.splits > 1 && slab_beg + p.slabs_per_split < nslabs ? slab_beg + p.slabs_per_split : nslabs;
  } else {
    const int zz = blockIdx.z / p.splits;               // (chunk, group)
    g = zz % p.G;
    out_chunk = zz / p.G;
    zsplit = blockIdx.z % p.splits;
    rows = Fg; cols = Cg * p.kk2;
    nslabs = p.m_count * (N / CV_BK);
    slab_beg = zsplit * p.slabs_per_split;
    slab_end = slab_beg + p.slabs_per_split < nslabs ? slab_beg + p.slabs_per_split : nslabs;
  }
  const int row0 = blockIdx.x * BM, col0 = blockIdx.y * BN;
  if (row0 >= rows || col0 >= cols) return;  // uniform for the workgroup

  // ---- loop-invariant part of each lane's gathers
  // The gathers that can fall into the padding (images for Up and Outp, hidden
  // activations for Down) are addressed as  base + 32-bit lane offset, where
  //   lane offset = (what depends on the lane, fixed for the whole kernel)
  //               + (what depends on the slab: wave-uniform, computed on the scalar unit).
  // base sits `bias` elements below the array so that no lane offset is negative, and a
  // group outside the image reads the first element of the array (offset = bias) and is
  // zeroed when it is written to LDS.  Per slab and group this costs a handful of
  // vector instructions; the index decomposition runs on the scalar unit.
  const int wvu = __builtin_amdgcn_readfirstlane(wv);
  constexpr int A_ROWLANES = BM / 4;                               // lanes per kk row of the A tile
  constexpr bool DOWNISH = MODE == CONV_DOWN || MODE == CONV_DOWNM;
  constexpr bool A_TWO = MODE != CONV_OUTP && A_ROWLANES == 32;    // a wavefront spans two kk rows
  static_assert(MODE == CONV_OUTP || A_ROWLANES == 32 || A_ROWLANES == 64, "Up/Down tiles are 128 or 256 rows");
  const int padw = p.pad0 < 0 ? -p.pad0 : 0;
  const unsigned img_bias = (unsigned)N * (unsigned)(padw * H + padw);
  unsigned hid_bias = 0;
  if (MODE == CONV_DOWN) hid_bias = (unsigned)N * (unsigned)(ph.TY * Mx + ph.TX);
  const char* a_base = nullptr;
  const char* b_base = nullptr;
  if (MODE == CONV_UP) a_base = reinterpret_cast<const char*>(p.img) - 4ll * img_bias;
  if (MODE == CONV_DOWN) a_base = reinterpret_cast<const char*>(p.hid) - 4ll * hid_bias;
  if (MODE == CONV_OUTP) b_base = reinterpret_cast<const char*>(p.img) - 4ll * img_bias;

  // A groups: Up/Down are row-contiguous (4 rows of one kk); Outp is kk-contiguous (4 kk of one row).
  int a_k[NA], a_r[NA], a_y[NA], a_x[NA], a_ks[NA];
  unsigned a_voff[NA];
  long long a_off[NA];
  bool a_ok[NA];
#pragma unroll
  for (int u = 0; u < NA; ++u) {
    const int f = tid + u * 256;
    a_ok[u] = f < TA;
    a_ks[u] = 0; a_voff[u] = 0; a_off[u] = 0;
    if (MODE == CONV_OUTP) {
      a_r[u] = f >> 2; a_k[u] = (f & 3) << 2;
      const int r = row0 + a_r[u];
      a_ok[u] = a_ok[u] && r < rows;
      a_off[u] = (long long)N * M * (g * Fg + r) + (long long)N * (p.m_begin + out_chunk * p.m_count);
      a_y[u] = a_x[u] = 0;
    } else {
      a_k[u] = f / A_ROWLANES; a_r[u] = (f % A_ROWLANES) << 2;
      a_ks[u] = (wvu * 64 + u * 256) / A_ROWLANES;                 // kk row of lanes 0-31 (scalar)
      const int r = row0 + a_r[u];
      a_ok[u] = a_ok[u] && r < rows;
      const int pos = (int)fd_div((uint32_t)r, p.dN);  // module (Up) or pixel-of-phase (Down)
      const int n = r - pos * N;
      if (MODE == CONV_UP) {
        const int my = (int)fd_div((uint32_t)pos, p.dMx), mx = pos - my * Mx;
        a_y[u] = my * s + p.pad0; a_x[u] = mx * s + p.pad0;
        a_voff[u] = 4u * (unsigned)(n + N * (a_y[u] * H + a_x[u]) + (int)img_bias);
      } else {
        const int qyi = ph.QX > 0 ? pos / ph.QX : 0, qxi = pos - qyi * ph.QX;
        a_y[u] = ph.qy_first + qyi; a_x[u] = ph.qx_first + qxi;  // module coordinate before the tap shift
        a_voff[u] = 4u * (unsigned)(n + N * (a_y[u] * Mx + a_x[u]) + (A_TWO && lk ? N * M : 0));
      }
    }
  }
  // B groups: Up is column-contiguous (4 filters of one kk); Down/Outp are kk-contiguous.
  int b_k[NB], b_c[NB], b_y[NB], b_x[NB];
  unsigned b_voff[NB];
  long long b_off[NB];
  bool b_ok[NB];
#pragma unroll
  for (int u = 0; u < NB; ++u) {
    const int f = tid + u * 256;
    b_ok[u] = f < TB;
    b_voff[u] = 0; b_off[u] = 0;
    if (MODE == CONV_UP) {
      b_k[u] = f / (BN / 4); b_c[u] = (f % (BN / 4)) << 2;
      const int c = col0 + b_c[u];
      b_ok[u] = b_ok[u] && c < cols;
      b_off[u] = (long long)g * Fg + c;
      b_y[u] = b_x[u] = 0;
    } else {
      b_c[u] = f >> 2; b_k[u] = (f & 3) << 2;
      const int c = col0 + b_c[u];
      b_ok[u] = b_ok[u] && c < cols;
      if (MODE == CONV_DOWN) {
        b_off[u] = (long long)g * Fg + (long long)F * c * p.kk2;  // + F*(ky*k + kx) + f per slab
        b_y[u] = b_x[u] = 0;
      } else {
        const int cc = (int)fd_div((uint32_t)c, p.dkk2);
        const int pp = c - cc * p.kk2;
        const int ky = (int)fd_div((uint32_t)pp, p.dk), kx = pp - ky * k;
        b_y[u] = p.pad0 + ky; b_x[u] = p.pad0 + kx;
        b_voff[u] = 4u * (unsigned)(N * ((g * Cg + cc) * HH + b_y[u] * H + b_x[u]) + b_k[u] + (int)img_bias);
        if (INSIDE && !b_ok[u]) b_voff[u] = 4u * (unsigned)b_k[u];   // a column beyond the output: any valid address
      }
    }
  }

  // ---- uniform-row variant: buffer resources, fixed lane offsets, the tile's module / pixel
  __amdgpu_buffer_rsrc_t u_ra = __builtin_amdgcn_make_buffer_rsrc((void*)(MODE == CONV_UP ? p.img : p.hid), 0,
                                                                    (int)p.a_bytes, 0x00020000);
  __amdgpu_buffer_rsrc_t u_rb = __builtin_amdgcn_make_buffer_rsrc((void*)p.flt, 0, (int)p.b_bytes, 0x00020000);
  // The two halves of a wavefront (lanes 0-31, 32-63) gather the tile's 128 rows at two
  // consecutive kk.
  unsigned u_avo[NA], u_bvo[NB];
  int u_bks[NB], m_py[NB], m_px[NB];
  int u_y = 0, u_x = 0;
  unsigned u_n0 = 0;
  // locally connected layers: one filter bank per module, F * Cg * k * k floats apart
  // (filters laid out (module, colour, ky, kx, filter)); convolution: one bank
  const unsigned bank_bytes = LOCAL ? 4u * (unsigned)F * (unsigned)(Cg * p.kk2) : 0u;
  unsigned u_bank = 0;
  if constexpr (UNI) {
    static_assert(MODE != CONV_OUTP && BM == 128, "uniform rows: Up / Down with 128-row tiles");
    const int pos = (int)fd_div((uint32_t)row0, p.dN);       // scalar: module (Up) or pixel of the phase (Down)
    u_n0 = 4u * (unsigned)(row0 - pos * N);
    if (MODE == CONV_UP) {
      const int my = (int)fd_div((uint32_t)pos, p.dMx), mx = pos - my * Mx;
      u_y = my * s + p.pad0; u_x = mx * s + p.pad0;
      u_bank = bank_bytes * (unsigned)pos;                     // this tile's module
    } else {
      const int qyi = ph.QX > 0 ? pos / ph.QX : 0, qxi = pos - qyi * ph.QX;
      u_y = ph.qy_first + qyi; u_x = ph.qx_first + qxi;
    }
#pragma unroll
    for (int u = 0; u < NA; ++u) u_avo[u] = 4u * (unsigned)(a_r[u] + (DOWNISH && lk ? M * N : 0));
#pragma unroll
    for (int u = 0; u < NB; ++u) {
      u_bks[u] = __builtin_amdgcn_readfirstlane(b_k[u]);
      if (MODE == CONV_UP) {
        u_bvo[u] = 4u * (unsigned)(g * Fg + col0 + b_c[u] + F * (b_k[u] - u_bks[u]));
      } else if (MODE == CONV_DOWNM) {
        const int j = col0 + b_c[u];                           // column -> (colour, py, px)
        const int c = (int)fd_div((uint32_t)j, p.dSS), q = j - c * s * s;
        m_py[u] = (int)fd_div((uint32_t)q, p.dS); m_px[u] = q - m_py[u] * s;
        if (j >= cols) m_py[u] = k;                            // never a valid tap
        u_bvo[u] = 4u * (unsigned)(g * Fg + b_k[u] + F * (c * p.kk2 + m_py[u] * k + m_px[u]));
      } else {
        u_bvo[u] = 4u * (unsigned)(g * Fg + b_k[u] + F * (col0 + b_c[u]) * p.kk2);
      }
    }
  }

  // ---- slab state (uniform across the workgroup)
  // Down: slab -> (t, u, f0); Outp: slab -> (my, mx, n0).
  int st_a = 0, st_b = 0, st_c = 0;
  if (DOWNISH) {
    const int per_tap = Fg / CV_BK;
    const int tap = slab_beg / per_tap;
    st_c = (slab_beg - tap * per_tap) * CV_BK;            // f0
    st_a = ph.TX > 0 ? tap / ph.TX : 0; st_b = tap - st_a * ph.TX;  // t, u
  } else if (MODE == CONV_OUTP) {
    const int per_mod = N / CV_BK;
    const int m = p.m_begin + out_chunk * p.m_count + slab_beg / per_mod;
    st_c = (slab_beg % per_mod) * CV_BK;                  // n0
    st_a = m / Mx; st_b = m - st_a * Mx;                  // my, mx
  }

  // Two register sets: the gathers run two slabs ahead of the MFMAs.  SET is a
  // compile-time constant so that every index into them is one too.
  f32x4 ra[2][NA], rb[2][NB];
  bool ra_ok[2][NA], rb_ok[2][NB];
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
  typedef std::integral_constant<int, 0> Set0;
  typedef std::integral_constant<int, 1> Set1;
  const int Kup = Cg * p.kk2;

  // Every gather is an unconditional 16-byte load (see above); no load sits behind a
  // branch, so all of a slab's loads are in flight together.
  auto fetch = [&](auto set_tag, int slab) {
    constexpr int SET = decltype(set_tag)::value;
    const int kk0 = slab * CV_BK;
    if constexpr (UNI) {
#pragma unroll
      for (int u = 0; u < NA; ++u) {
        unsigned voff = u_avo[u], so;
        if (MODE == CONV_UP) {
          // per half (kk row): byte offset of its 128 images, or "in the padding"; all scalar
          // and free of branches (a branch here would split up the slab's loads)
          unsigned off[2];
          bool ok[2];
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const int kk = kk0 + a_ks[u] + h;
            const int c = (int)fd_div((uint32_t)kk, p.dkk2);
            const int pp = kk - c * p.kk2;
            const int ky = (int)fd_div((uint32_t)pp, p.dk), kx = pp - ky * k;
            const int y = u_y + ky, x = u_x + kx;
            ok[h] = (kk < Kup) & ((unsigned)y < (unsigned)H) & ((unsigned)x < (unsigned)H);
            off[h] = 4u * (unsigned)N * (unsigned)((g * Cg + c) * HH + y * H + x) + u_n0;
          }
          const unsigned lo = ok[0] ? off[0] : 0xffffffffu, hi = ok[1] ? off[1] : 0xffffffffu;
          so = lo < hi ? lo : hi;                              // the smaller valid offset ...
          if (!(ok[0] | ok[1])) so = 0u;
          const unsigned dlo = ok[0] ? off[0] - so : p.a_bytes, dhi = ok[1] ? off[1] - so : p.a_bytes;   // ... plus a non-negative rest
          voff += lk ? dhi : dlo;
        } else {
          // both halves read the same module, one filter apart (a constant in the lane offset)
          const int my = u_y - st_a, mx = u_x - st_b;
          const bool ok = ((unsigned)my < (unsigned)Mx) & ((unsigned)mx < (unsigned)Mx);
          so = ok ? 4u * (unsigned)N * (unsigned)((g * Fg + st_c + a_ks[u]) * M + my * Mx + mx) + u_n0 : p.a_bytes;
        }
        ra[SET][u] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(u_ra, (int)voff, (int)so, 0));
      }
#pragma unroll
      for (int u = 0; u < NB; ++u) {
        unsigned so;
        unsigned voff = u_bvo[u];
        if (MODE == CONV_UP) {
          so = 4u * (unsigned)F * (unsigned)(kk0 + u_bks[u]) + u_bank;
        } else {
          so = 4u * (unsigned)(F * ((ph.py + s * st_a) * k + ph.px + s * st_b) + st_c);
          if constexpr (LOCAL) {
            // the bank of the module this slab's tap reaches (a module outside the map has zero
            // activations: any bank will do)
            const int my = u_y - st_a, mx = u_x - st_b;
            const bool in_map = ((unsigned)my < (unsigned)Mx) & ((unsigned)mx < (unsigned)Mx);
            so += in_map ? bank_bytes * (unsigned)(my * Mx + mx) : 0u;
          }
        }
        if (MODE == CONV_DOWNM) {                              // this column's tap of module (Y - t, X - u), if it has one
          const bool ok = (m_py[u] + s * st_a < k) & (m_px[u] + s * st_b < k);
          voff = ok ? voff : p.b_bytes;
        }
        rb[SET][u] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(u_rb, (int)voff, (int)so, 0));
      }
      if (DOWNISH) {
        st_c += CV_BK;
        if (st_c == Fg) { st_c = 0; if (++st_b == ph.TX) { st_b = 0; ++st_a; } }
      }
      return;
    }
#pragma unroll
    for (int u = 0; u < NA; ++u) {
      bool ok = a_ok[u];
      if (MODE == CONV_UP) {
        // scalar: where tap kk of this wavefront's row(s) lies relative to the module origin
        int sy[2], sx[2];
        unsigned so[2];
        bool sv[2];
#pragma unroll
        for (int h = 0; h < (A_TWO ? 2 : 1); ++h) {
          int kk = kk0 + a_ks[u] + h;
          sv[h] = kk < Kup;
          if (INSIDE && !sv[h]) kk = Kup - 1;
          const int c = (int)fd_div((uint32_t)kk, p.dkk2);
          const int pp = kk - c * p.kk2;
          sy[h] = (int)fd_div((uint32_t)pp, p.dk); sx[h] = pp - sy[h] * k;
          so[h] = 4u * (unsigned)N * (unsigned)((g * Cg + c) * HH + sy[h] * H + sx[h]);   // unused when !sv[h]
        }
        const bool hi = A_TWO && lk;
        if constexpr (INSIDE) {
          ra[SET][u] = *reinterpret_cast<const f32x4*>(a_base + (a_voff[u] + (hi ? so[1] : so[0])));
        } else {
          const int y = a_y[u] + (hi ? sy[1] : sy[0]), x = a_x[u] + (hi ? sx[1] : sx[0]);
          ok = ok & (hi ? sv[1] : sv[0]) & ((unsigned)y < (unsigned)H) & ((unsigned)x < (unsigned)H);
          const unsigned voff = ok ? a_voff[u] + (hi ? so[1] : so[0]) : 4u * img_bias;
          ra[SET][u] = *reinterpret_cast<const f32x4*>(a_base + voff);
        }
      } else if (MODE == CONV_DOWN) {
        const int my = a_y[u] - st_a, mx = a_x[u] - st_b;
        ok = ok & ((unsigned)my < (unsigned)Mx) & ((unsigned)mx < (unsigned)Mx);
        const unsigned so = 4u * ((unsigned)N * (unsigned)((g * Fg + st_c + a_ks[u]) * M - st_a * Mx - st_b) + hid_bias);  // scalar
        const unsigned voff = ok ? a_voff[u] + so : 4u * hid_bias;
        ra[SET][u] = *reinterpret_cast<const f32x4*>(a_base + voff);
      } else {
        const float* src = p.hid + a_off[u] + (long long)(slab * CV_BK + a_k[u]);
        if (!ok) src = p.hid;
        ra[SET][u] = *reinterpret_cast<const f32x4*>(src);
      }
      ra_ok[SET][u] = ok;
    }
#pragma unroll
    for (int u = 0; u < NB; ++u) {
      bool ok = b_ok[u];
      if (MODE == CONV_UP) {
        const int kk = kk0 + b_k[u];
        ok = ok && kk < Kup;
        const float* src = p.flt + b_off[u] + (long long)F * kk;
        if (!ok) src = p.flt;
        rb[SET][u] = *reinterpret_cast<const f32x4*>(src);
      } else if (MODE == CONV_DOWN) {
        const int ky = ph.py + s * st_a, kx = ph.px + s * st_b;
        const float* src = p.flt + b_off[u] + (long long)F * (ky * k + kx) + st_c + b_k[u];
        if (!ok) src = p.flt;
        rb[SET][u] = *reinterpret_cast<const f32x4*>(src);
      } else {
        const unsigned so = 4u * ((unsigned)N * (unsigned)(st_a * s * H + st_b * s) + (unsigned)st_c);  // scalar
        if constexpr (INSIDE) {
          rb[SET][u] = *reinterpret_cast<const f32x4*>(b_base + (b_voff[u] + so));
        } else {
          const int y = st_a * s + b_y[u], x = st_b * s + b_x[u];
          ok = ok & ((unsigned)y < (unsigned)H) & ((unsigned)x < (unsigned)H);
          const unsigned voff = ok ? b_voff[u] + so : 4u * img_bias;
          rb[SET][u] = *reinterpret_cast<const f32x4*>(b_base + voff);
        }
      }
      rb_ok[SET][u] = ok;
    }
    // advance the uniform slab state
    if (MODE == CONV_DOWN) {
      st_c += CV_BK;
      if (st_c == Fg) { st_c = 0; if (++st_b == ph.TX) { st_b = 0; ++st_a; } }
    } else if (MODE == CONV_OUTP) {
      st_c += CV_BK;
      if (st_c == N) { st_c = 0; if (++st_b == Mx) { st_b = 0; ++st_a; } }
    }
  };
  auto stash = [&](auto set_tag, int buf) {
    constexpr int SET = decltype(set_tag)::value;
#pragma unroll
    for (int u = 0; u < NA; ++u) {
      if (tid + u * 256 >= TA) continue;
      if (!UNI && !INSIDE && !ra_ok[SET][u]) ra[SET][u] = zero4;
      if (MODE == CONV_OUTP) {
        As[buf][a_k[u]][a_r[u]] = ra[SET][u].x; As[buf][a_k[u] + 1][a_r[u]] = ra[SET][u].y;
        As[buf][a_k[u] + 2][a_r[u]] = ra[SET][u].z; As[buf][a_k[u] + 3][a_r[u]] = ra[SET][u].w;
      } else {
        *reinterpret_cast<f32x4*>(&As[buf][a_k[u]][a_r[u]]) = ra[SET][u];
      }
    }
#pragma unroll
    for (int u = 0; u < NB; ++u) {
      if (tid + u * 256 >= TB) continue;
      if (!UNI && !(INSIDE && MODE == CONV_OUTP) && !rb_ok[SET][u]) rb[SET][u] = zero4;
      if (MODE == CONV_UP) {
        *reinterpret_cast<f32x4*>(&Bs[buf][b_k[u]][b_c[u]]) = rb[SET][u];
      } else {
        Bs[buf][b_k[u]][b_c[u]] = rb[SET][u].x; Bs[buf][b_k[u] + 1][b_c[u]] = rb[SET][u].y;
        Bs[buf][b_k[u] + 2][b_c[u]] = rb[SET][u].z; Bs[buf][b_k[u] + 3][b_c[u]] = rb[SET][u].w;
      }
    }
  };

  f32x16 acc[WN][WM];
#pragma unroll
  for (int j = 0; j < WN; ++j)
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[j][i][v] = 0.f;
  // N16 > 0: the columns are covered by N16 blocks of 16 with v_mfma_f32_16x16x4_f32
  // (48 columns, e.g. colours x stride^2 of a merged-phase convDown or 48 colours per
  // group, cost three blocks of 16 instead of two of 32).  A wavefront's 32 rows are two
  // blocks of 16.
  static_assert(N16 == 0 || (MODE != CONV_OUTP && WM == 1 && WAVES_M == 4 && N16 * 16 <= BN), "16-wide blocks: 128-row Up / Down tiles");
  constexpr int N16A = N16 > 0 ? N16 : 1;
  f32x4 acc16[N16A][2];
#pragma unroll
  for (int j = 0; j < N16A; ++j)
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc16[j][i][v] = 0.f;
  const int l16 = lane & 15, k16 = lane >> 4;

  // One slab: all of its fragments are asked of LDS first (the scheduling fences keep
  // the compiler from sinking the reads back to their uses and from hoisting the wait
  // for the gathers in flight above the MFMAs).
  auto multiply = [&](int buf) {
    if constexpr (N16 > 0) {
      // lane (l16, k16): operand element (row or column l16 of its block, k = step + 4*k16:
      // any assignment of the slab's 16 k to (step, k16) will do as long as both operands
      // use the same one, and rows 4 apart sit 16 banks apart)
      float av[CV_BK / 4][2], bv[CV_BK / 4][N16A];
#pragma unroll
      for (int kk = 0; kk < CV_BK / 4; ++kk) {
#pragma unroll
        for (int i = 0; i < 2; ++i) av[kk][i] = As[buf][kk + 4 * k16][wm * 32 + i * 16 + l16];
#pragma unroll
        for (int j = 0; j < N16A; ++j) bv[kk][j] = Bs[buf][kk + 4 * k16][j * 16 + l16];
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int kk = 0; kk < CV_BK / 4; ++kk)
#pragma unroll
        for (int j = 0; j < N16A; ++j)
#pragma unroll
          for (int i = 0; i < 2; ++i)
            acc16[j][i] = __builtin_amdgcn_mfma_f32_16x16x4f32(bv[kk][j], av[kk][i], acc16[j][i], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      return;
    }
    float av[CV_BK / 2][WM], bv[CV_BK / 2][WN];
#pragma unroll
    for (int kk = 0; kk < CV_BK / 2; ++kk) {
#pragma unroll
      for (int i = 0; i < WM; ++i) av[kk][i] = As[buf][kk + (CV_BK / 2) * lk][(wm * WM + i) * 32 + li];
#pragma unroll
      for (int j = 0; j < WN; ++j) bv[kk][j] = Bs[buf][kk + (CV_BK / 2) * lk][(wn * WN + j) * 32 + li];
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int kk = 0; kk < CV_BK / 2; ++kk)
#pragma unroll
      for (int j = 0; j < WN; ++j)
#pragma unroll
        for (int i = 0; i < WM; ++i)
          acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x2f32(bv[kk][j], av[kk][i], acc[j][i], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
  };

  // While slab i is multiplied, slab i+1 (asked for one iteration ago) is written to
  // LDS and slab i+2 is requested; two slabs per trip so the register sets swap roles
  // statically.  fetch() is always called with consecutive slabs.
  // (Measured: the deeper prefetch pays for Outp, whose K runs over modules and images;
  // for Up and Down its extra registers cost more than it hides.)
  constexpr bool TWO_AHEAD = MODE == CONV_OUTP || UNI;
  int buf = 0, slab = slab_beg;
  if (TWO_AHEAD && slab_end - slab_beg >= 2) {
    fetch(Set0(), slab);
    stash(Set0(), 0);
    fetch(Set0(), slab + 1);
    __syncthreads();
    while (slab + 4 <= slab_end) {
      fetch(Set1(), slab + 2);
      multiply(buf);
      stash(Set0(), buf ^ 1);
      __syncthreads();
      buf ^= 1; ++slab;
      fetch(Set0(), slab + 2);
      multiply(buf);
      stash(Set1(), buf ^ 1);
      __syncthreads();
      buf ^= 1; ++slab;
    }
    multiply(buf);
    stash(Set0(), buf ^ 1);
    __syncthreads();
    buf ^= 1; ++slab;                // LDS holds slab `slab`, nothing is in flight
  } else {
    if (slab_beg < slab_end) {
      fetch(Set0(), slab_beg);
      stash(Set0(), 0);
    }
    __syncthreads();
  }
  for (; slab < slab_end; ++slab) {
    const bool more = slab + 1 < slab_end;
    if (more) fetch(Set0(), slab + 1);
    multiply(buf);
    if (more) stash(Set0(), buf ^ 1);
    __syncthreads();
    buf ^= 1;
  }

  // Up / Down with a split reduction: this workgroup's sums go to its own copy of the output.
  float* const outb = (MODE == CONV_UP || MODE == CONV_DOWN) && p.splits > 1 ? p.partial + zsplit * p.split_stride : p.out;
  if constexpr (N16 > 0) {
    // acc16[j][i][v] is C(row, col) with row = ... + i*16 + l16, col = j*16 + 4*k16 + v
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int r = row0 + wm * 32 + i * 16 + l16;
      if (r >= rows) continue;
      const int pos = (int)fd_div((uint32_t)r, p.dN);
      const int n = r - pos * N;
      if constexpr (MODE == CONV_DOWNM) {
        const int Y = pos / p.yq, X = pos - Y * p.yq;
#pragma unroll
        for (int j = 0; j < N16A; ++j)
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            const int cc = col0 + j * 16 + 4 * k16 + v;
            if (cc >= cols) continue;
            const int c = (int)fd_div((uint32_t)cc, p.dSS), q = cc - c * s * s;
            const int py = (int)fd_div((uint32_t)q, p.dS), px = q - py * s;
            const int y = Y * s + py + p.pad0, x = X * s + px + p.pad0;
            if ((unsigned)y < (unsigned)H && (unsigned)x < (unsigned)H) {
              float* t = p.out + (long long)N * ((long long)(g * Cg + c) * HH + y * H + x) + n;
              *t = (p.scale_t == 0.f ? 0.f : p.scale_t * *t) + p.scale_o * acc16[j][i][v];
            }
          }
      } else {
        long long rbase, cstride;
        if (MODE == CONV_UP) {
          rbase = (long long)g * Fg * M * N + r;
          cstride = (long long)M * N;
        } else {
          const int qyi = pos / ph.QX, qxi = pos - qyi * ph.QX;
          const int y = ph.y_first + s * qyi, x = ph.x_first + s * qxi;
          rbase = (long long)N * ((long long)g * Cg * HH + y * H + x) + n;
          cstride = (long long)N * HH;
        }
#pragma unroll
        for (int j = 0; j < N16A; ++j)
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            const int c = col0 + j * 16 + 4 * k16 + v;
            if (c >= cols) continue;
            float* t = outb + rbase + cstride * c;
            *t = (p.scale_t == 0.f ? 0.f : p.scale_t * *t) + p.scale_o * acc16[j][i][v];
          }
      }
    }
    return;
  }
  // ---- epilogue: acc[j][i][v] is C(row, col) with row = ... + li, col = ... + 8*(v/4) + 4*lk + v%4
#pragma unroll
  for (int i = 0; i < WM; ++i) {
    const int r = row0 + (wm * WM + i) * 32 + li;
    if (r >= rows) continue;
    long long rbase;
    long long cstride;
    if (MODE == CONV_UP) {
      rbase = (long long)g * Fg * M * N + r;            // + c * M*N
      cstride = (long long)M * N;
    } else if (MODE == CONV_DOWNM) {
      const int pos = (int)fd_div((uint32_t)r, p.dN);
      const int n = r - pos * N;
      const int Y = pos / p.yq, X = pos - Y * p.yq;
#pragma unroll
      for (int j = 0; j < WN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int cc = col0 + (wn * WN + j) * 32 + 8 * (v >> 2) + 4 * lk + (v & 3);
          if (cc >= cols) continue;
          const int c = (int)fd_div((uint32_t)cc, p.dSS), q = cc - c * s * s;
          const int py = (int)fd_div((uint32_t)q, p.dS), px = q - py * s;
          const int y = Y * s + py + p.pad0, x = X * s + px + p.pad0;
          if ((unsigned)y < (unsigned)H && (unsigned)x < (unsigned)H) {
            float* t = p.out + (long long)N * ((long long)(g * Cg + c) * HH + y * H + x) + n;
            *t = (p.scale_t == 0.f ? 0.f : p.scale_t * *t) + p.scale_o * acc[j][i][v];
          }
        }
      continue;
    } else if (MODE == CONV_DOWN) {
      const int pos = (int)fd_div((uint32_t)r, p.dN);
      const int n = r - pos * N;
      const int qyi = pos / ph.QX, qxi = pos - qyi * ph.QX;
      const int y = ph.y_first + s * qyi, x = ph.x_first + s * qxi;
      rbase = (long long)N * ((long long)g * Cg * HH + y * H + x) + n;  // + c * N*HH
      cstride = (long long)N * HH;
    } else {
      rbase = ((long long)out_chunk * p.splits + zsplit) * ((long long)p.G * Fg * Cg * p.kk2) + ((long long)g * Cg * p.kk2) * Fg + r;
      cstride = Fg;                                     // partial[zsplit][g][q][f]
    }
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int c = col0 + (wn * WN + j) * 32 + 8 * (v >> 2) + 4 * lk + (v & 3);
        if (c >= cols) continue;
        if (MODE == CONV_OUTP) {
          p.partial[rbase + cstride * c] = acc[j][i][v];
        } else {
          float* t = outb + rbase + cstride * c;
          *t = (p.scale_t == 0.f ? 0.f : p.scale_t * *t) + p.scale_o * acc[j][i][v];
        }
      }
  }
}

// ------------------------------------------------------------------ convOutp, small outputs
// Weight gradients of a layer with at most 32*RT filters per group and at most 32*CT
// patch columns (a first layer over RGB: 64 x 75).  Both operands are contiguous along
// the images, which is the reduction index here, so a chunk of (one module, 64 images)
// is read row by row in whole 256-byte runs and kept in LDS as [row][image] with a pitch
// of 68: the 16-byte groups go to LDS as they came, and a lane's operands of four MFMA
// steps (lane = row, four neighbouring images) are one conflict-free 16-byte LDS read.  The four wavefronts each hold the whole RT x CT block of accumulators and
// split the 32 steps of a chunk between them (no columns are padded to a wavefront
// grid, one barrier per chunk); they are summed through LDS once, at the end, and every
// workgroup writes one partial block for k_conv_outp_finish.
template <int RT, int CT>
__global__ void __launch_bounds__(256, 1) k_conv_outp_small(ConvArgs p) {
  constexpr unsigned FAR = 0x80000000u;  // beyond any buffer here: sizes are below 2^31 bytes
  constexpr int PITCH = 68;              // 64 images + 4: 16-byte groups stay aligned, 8 neighbouring rows on different banks
  constexpr int NAV = RT * 2, NBV = CT * 2;   // 16-byte loads per lane and chunk (32 rows x 16 = 512 = 2 x 256)
  // one LDS arena: the two operand tiles (double buffered) while chunks are multiplied,
  // the four wavefronts' accumulators when they are summed at the end
  constexpr int TILES = 2 * 32 * (RT + CT) * PITCH, SUMS = 4 * 16 * RT * CT * 64;
  __shared__ __attribute__((aligned(16))) float arena[TILES > SUMS ? TILES : SUMS];
  float (*As)[32 * RT][PITCH] = reinterpret_cast<float (*)[32 * RT][PITCH]>(arena);
  float (*Bs)[32 * CT][PITCH] = reinterpret_cast<float (*)[32 * CT][PITCH]>(arena + 2 * 32 * RT * PITCH);
  const int tid = threadIdx.x, lane = tid & 63, li = lane & 31, lk = lane >> 5;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = blockIdx.z;
  const int N = p.N, H = p.H, Fg = p.Fg, cols = p.Cg * p.kk2;
  __amdgpu_buffer_rsrc_t r_img = __builtin_amdgcn_make_buffer_rsrc((void*)p.img, 0, (int)p.a_bytes, 0x00020000);
  __amdgpu_buffer_rsrc_t r_hid = __builtin_amdgcn_make_buffer_rsrc((void*)p.hid, 0, (int)p.b_bytes, 0x00020000);
  // lane's rows of the two tiles: row = tid/16 + 16*u, images 4*(tid%16) .. +3 of the chunk
  const int r16 = tid >> 4, n4 = (tid & 15) * 4;
  unsigned a_voff[NAV];      // hid(f, module, image) at image + N*(module + M*f)
#pragma unroll
  for (int u = 0; u < NAV; ++u) {
    const int f = r16 + 16 * u;
    a_voff[u] = f < Fg ? ((unsigned)(g * Fg + f) * (unsigned)p.M * (unsigned)N + (unsigned)n4) * 4u : FAR;
  }
  unsigned b_voff[NBV], b_yx[NBV];   // img(colour, y0 + ky, x0 + kx, image); bit ky | bit 16 + kx of the tap
#pragma unroll
  for (int u = 0; u < NBV; ++u) {
    const unsigned q = r16 + 16 * u;
    const unsigned c = fd_div(q, p.dkk2), r = q - c * (unsigned)p.kk2;
    const unsigned ky = fd_div(r, p.dk), kx = r - ky * (unsigned)p.k;
    const bool live = (int)q < cols;
    b_voff[u] = live ? ((((unsigned)(g * p.Cg) + c) * H + ky) * H + kx) * (unsigned)N * 4u + (unsigned)n4 * 4u : FAR;
    b_yx[u] = live ? (1u << ky) | (1u << (16 + kx)) : 0xffffffffu;
  }
  f32x16 acc[CT][RT];
#pragma unroll
  for (int j = 0; j < CT; ++j)
#pragma unroll
    for (int i = 0; i < RT; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[j][i][v] = 0.f;

  const int halves = N >> 6;                         // chunks of 64 images per module
  f32x4 ra[2][NAV], rb[2][NBV];   // two register sets: chunks are requested two ahead
  typedef std::integral_constant<int, 0> Set0;
  typedef std::integral_constant<int, 1> Set1;
  // chunk ci of this workgroup: module m_begin + (blockIdx.x + gridDim.x * (ci / halves)), images 64 * (ci % halves)
  auto fetch = [&](auto set_tag, int ci) __attribute__((always_inline)) {
    constexpr int SET = decltype(set_tag)::value;
    const int mi = blockIdx.x + gridDim.x * (ci / halves);
    const int m = p.m_begin + mi, n0 = (ci % halves) * 64;
    const int my = (int)fd_div((unsigned)m, p.dMx), mx = m - my * p.Mx;
    const int y0 = my * p.s + p.pad0, x0 = mx * p.s + p.pad0;
    const unsigned a_so = ((unsigned)m * (unsigned)N + (unsigned)n0) * 4u;
#pragma unroll
    for (int u = 0; u < NAV; ++u)
      ra[SET][u] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r_hid, (int)a_voff[u], (int)a_so, 0));
    const int ylo = y0 < 0 ? -y0 : 0, yhi = H - y0 < p.k ? H - y0 : p.k;
    const int xlo = x0 < 0 ? -x0 : 0, xhi = H - x0 < p.k ? H - x0 : p.k;
    const unsigned ym = yhi > ylo ? ((1u << yhi) - 1u) & ~((1u << ylo) - 1u) : 0u;
    const unsigned xm = xhi > xlo ? ((1u << xhi) - 1u) & ~((1u << xlo) - 1u) : 0u;
    const unsigned bad = ~(ym | (xm << 16));
    const unsigned b_add = (unsigned)(((y0 * H + x0) * N + n0) * 4);
#pragma unroll
    for (int u = 0; u < NBV; ++u) {
      const unsigned voff = (b_yx[u] & bad) ? FAR : b_voff[u] + b_add;
      rb[SET][u] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r_img, (int)voff, 0, 0));
    }
  };
  // The chunk held in LDS buffer `buf` is multiplied (steps 8*wv .. 8*wv + 7 of its 32)
  // while register set SET, if STASH, goes to the other buffer: its LDS writes are
  // issued between the MFMAs, and the second half of the operand reads under the
  // first half of the MFMAs.
  // `next`: chunk to request (into the other register set) once the first MFMAs are under
  // way, so that its scalar address arithmetic runs beside them; -1: none.
  auto multiply = [&](auto set_tag, auto stash_tag, int buf, int next) __attribute__((always_inline)) {
    constexpr int SET = decltype(set_tag)::value;
    constexpr bool STASH = decltype(stash_tag)::value;
    constexpr int NW = NAV + NBV;                       // 16-byte LDS writes of a lane per chunk
    constexpr int WPS = (NW + 7) / 8;                   // ... per step
    // Step t of this wavefront multiplies image 16*wv + 8*(t/4) + 4*lk + t%4 of the chunk (the
    // sum over images takes them in any order), so a lane's operands of four steps are
    // one 16-byte LDS read per row block.
    f32x4 av[2][RT], bv[2][CT];
    auto read = [&](int h) __attribute__((always_inline)) {
      const int kk = 16 * wv + 8 * h + 4 * lk;
#pragma unroll
      for (int i = 0; i < RT; ++i) av[h][i] = *reinterpret_cast<const f32x4*>(&As[buf][i * 32 + li][kk]);
#pragma unroll
      for (int j = 0; j < CT; ++j) bv[h][j] = *reinterpret_cast<const f32x4*>(&Bs[buf][j * 32 + li][kk]);
    };
    read(0);
    __builtin_amdgcn_sched_barrier(0);
    read(1);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < 8; ++t) {
#pragma unroll
      for (int j = 0; j < CT; ++j)
#pragma unroll
        for (int i = 0; i < RT; ++i)
          acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x2f32(bv[t >> 2][j][t & 3], av[t >> 2][i][t & 3], acc[j][i], 0, 0, 0);
      if (t == 0 && next >= 0) fetch(std::integral_constant<int, SET ^ 1>(), next);
      if (STASH) {
#pragma unroll
        for (int u = t * WPS; u < (t + 1) * WPS && u < NW; ++u) {
          if (u < NAV) *reinterpret_cast<f32x4*>(&As[buf ^ 1][r16 + 16 * u][n4]) = ra[SET][u];
          else *reinterpret_cast<f32x4*>(&Bs[buf ^ 1][r16 + 16 * (u - NAV)][n4]) = rb[SET][u - NAV];
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto stash = [&](auto set_tag, int buf) __attribute__((always_inline)) {
    constexpr int SET = decltype(set_tag)::value;
#pragma unroll
    for (int u = 0; u < NAV; ++u) *reinterpret_cast<f32x4*>(&As[buf][r16 + 16 * u][n4]) = ra[SET][u];
#pragma unroll
    for (int u = 0; u < NBV; ++u) *reinterpret_cast<f32x4*>(&Bs[buf][r16 + 16 * u][n4]) = rb[SET][u];
  };
  const int my_chunks = (int)blockIdx.x < p.m_count ? ((p.m_count - 1 - (int)blockIdx.x) / (int)gridDim.x + 1) * halves : 0;
  // While chunk i is multiplied, chunk i+1 (asked for one trip ago) is written to LDS and
  // chunk i+2 is requested; two chunks per trip so that the register sets swap statically.
  typedef std::true_type Yes;
  typedef std::false_type No;
  int ci = 0, buf = 0;
  if (my_chunks >= 2) {
    fetch(Set0(), 0);
    stash(Set0(), 0);
    fetch(Set0(), 1);
    __syncthreads();
    while (ci + 4 <= my_chunks) {
      multiply(Set0(), Yes(), buf, ci + 2);
      __syncthreads();
      buf ^= 1; ++ci;
      multiply(Set1(), Yes(), buf, ci + 2);
      __syncthreads();
      buf ^= 1; ++ci;
    }
    multiply(Set0(), Yes(), buf, -1);
    __syncthreads();
    buf ^= 1; ++ci;                  // LDS holds chunk ci, nothing is in flight
  } else {
    if (my_chunks > 0) {
      fetch(Set0(), 0);
      stash(Set0(), 0);
    }
    __syncthreads();
  }
  for (; ci < my_chunks; ++ci) {
    if (ci + 1 < my_chunks) {
      fetch(Set0(), ci + 1);
      multiply(Set0(), Yes(), buf, -1);
    } else {
      multiply(Set0(), No(), buf, -1);
    }
    __syncthreads();
    buf ^= 1;
  }
  // Sum the four wavefronts' accumulators in a fixed order: every wavefront leaves its
  // 16*RT*CT values per lane in LDS and then finishes a quarter of them.
  constexpr int NACC = 16 * RT * CT;
  float (*sums)[NACC][64] = reinterpret_cast<float (*)[NACC][64]>(arena);
#pragma unroll
  for (int j = 0; j < CT; ++j)
#pragma unroll
    for (int i = 0; i < RT; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) sums[wv][(j * RT + i) * 16 + v][lane] = acc[j][i][v];
  __syncthreads();
  // value e = (j*RT + i)*16 + v of lane (li, lk): column q = j*32 + 8*(v/4) + 4*lk + v%4, filter f = i*32 + li
  float* part = p.partial + (size_t)blockIdx.x * ((size_t)p.G * Fg * cols) + (size_t)g * Fg * cols;
#pragma unroll
  for (int x = 0; x < NACC / 4; ++x) {
    const int e = wv * (NACC / 4) + x;
    const float sum = (sums[0][e][lane] + sums[1][e][lane]) + (sums[2][e][lane] + sums[3][e][lane]);
    const int v = e & 15, ji = e >> 4, jt = ji / RT, it = ji - jt * RT;
    const int q = jt * 32 + 8 * (v >> 2) + 4 * lk + (v & 3), f = it * 32 + li;
    if (q < cols && f < Fg) part[(size_t)q * Fg + f] = sum;
  }
}

// The same gradients for at most 16*RB filters per group and 16*CB patch columns, without
// LDS tiles: on v_mfma_f32_16x16x4_f32 a lane holds one row (a filter, or a patch column) of
// an operand at four of sixteen reduction indices, and the reduction runs over the images,
// along which both arrays are contiguous.  So a lane's operands of four steps are ONE 16-byte
// load (images 4*kq .. 4*kq + 3 of a group of 16; the sum over images takes them in any
// order, as long as both operands take them alike), a wavefront's load covers 16 rows in
// 64-byte runs, and nothing is staged or synchronised: a wavefront owns a run of chunks
// (module, 16 images), keeps D chunks in flight and multiplies RB x CB blocks per step.
// Taps on the padding and chunks past the end are out-of-range loads (zeros); every trip
// issues the same number of loads, so that the waits the compiler places count alike on
// every path.  The four wavefronts are summed through LDS in a fixed order and every
// workgroup leaves one partial block for k_conv_outp_finish_*.
template <int RB, int CB, int D>
__global__ void __launch_bounds__(256, 1) k_conv_outp_regs(ConvArgs p) {
  constexpr unsigned FAR = 0x80000000u;  // beyond any buffer here: sizes are below 2^31 bytes
  constexpr int PF = 16 * RB + 4;
  __shared__ float sums[4][16 * CB * PF];
  const int tid = threadIdx.x, lane = tid & 63, li = lane & 15, kq = lane >> 4;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = blockIdx.z;
  const int N = p.N, H = p.H, Fg = p.Fg, cols = p.Cg * p.kk2;
  __amdgpu_buffer_rsrc_t r_img = __builtin_amdgcn_make_buffer_rsrc((void*)p.img, 0, (int)p.a_bytes, 0x00020000);
  __amdgpu_buffer_rsrc_t r_hid = __builtin_amdgcn_make_buffer_rsrc((void*)p.hid, 0, (int)p.b_bytes, 0x00020000);
  unsigned a_voff[RB];       // hid(f, module, image) at image + N*(module + M*f)
  const int f0 = 16 * RB * (int)blockIdx.y;         // (grid y: slices of 16*RB filters of the group)
#pragma unroll
  for (int i = 0; i < RB; ++i) {
    const int f = f0 + 16 * i + li;
    a_voff[i] = f < Fg ? ((unsigned)(g * Fg + f) * (unsigned)p.M * (unsigned)N + 4u * (unsigned)kq) * 4u : FAR;
  }
  unsigned b_voff[CB], b_yx[CB];   // img(colour, y0 + ky, x0 + kx, image); bit ky | bit 16 + kx of the tap
#pragma unroll
  for (int j = 0; j < CB; ++j) {
    const unsigned q = 16 * j + li;
    const unsigned c = fd_div(q, p.dkk2), r = q - c * (unsigned)p.kk2;
    const unsigned ky = fd_div(r, p.dk), kx = r - ky * (unsigned)p.k;
    const bool live = (int)q < cols;
    b_voff[j] = live ? ((((unsigned)(g * p.Cg) + c) * H + ky) * H + kx) * (unsigned)N * 4u + 16u * (unsigned)kq : FAR;
    b_yx[j] = live ? (1u << ky) | (1u << (16 + kx)) : 0xffffffffu;
  }
  f32x4 acc[CB][RB];
#pragma unroll
  for (int j = 0; j < CB; ++j)
#pragma unroll
    for (int i = 0; i < RB; ++i) acc[j][i] = (f32x4){0.f, 0.f, 0.f, 0.f};

  const int cpm = N >> 4;                               // chunks per module
  const int total = p.m_count * cpm;
  const int c0 = ((int)blockIdx.x * 4 + wv) * p.slabs_per_split;
  const int c1 = c0 + p.slabs_per_split < total ? c0 + p.slabs_per_split : total;
  int fm = c0 / cpm, fj = c0 - fm * cpm, fc = c0;       // the next chunk to ask for: module, group of 16 images, index
  f32x4 ra[D][RB], rb[D][CB];
  auto fetch = [&](auto set_tag) __attribute__((always_inline)) {
    constexpr int SET = decltype(set_tag)::value;
    const bool valid = fc < c1;
    const int m = p.m_begin + fm;
    const int my = (int)fd_div((unsigned)m, p.dMx), mx = m - my * p.Mx;
    const int y0 = my * p.s + p.pad0, x0 = mx * p.s + p.pad0;
    const unsigned a_so = ((unsigned)m * (unsigned)N + 16u * (unsigned)fj) * 4u;
    const unsigned gone = valid ? 0u : FAR;
#pragma unroll
    for (int i = 0; i < RB; ++i)
      ra[SET][i] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r_hid, (int)(a_voff[i] | gone), (int)a_so, 0));
    const int ylo = y0 < 0 ? -y0 : 0, yhi = H - y0 < p.k ? H - y0 : p.k;
    const int xlo = x0 < 0 ? -x0 : 0, xhi = H - x0 < p.k ? H - x0 : p.k;
    const unsigned ym = yhi > ylo ? ((1u << yhi) - 1u) & ~((1u << ylo) - 1u) : 0u;
    const unsigned xm = xhi > xlo ? ((1u << xhi) - 1u) & ~((1u << xlo) - 1u) : 0u;
    const unsigned bad = valid ? ~(ym | (xm << 16)) : 0xffffffffu;
    const unsigned b_add = (unsigned)(((y0 * H + x0) * N + 16 * fj) * 4);
#pragma unroll
    for (int j = 0; j < CB; ++j) {
      const unsigned voff = (b_yx[j] & bad) ? FAR : b_voff[j] + b_add;
      rb[SET][j] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r_img, (int)voff, 0, 0));
    }
    ++fc;
    if (++fj == cpm) { fj = 0; ++fm; }
  };
  auto multiply = [&](auto set_tag) __attribute__((always_inline)) {
    constexpr int SET = decltype(set_tag)::value;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int j = 0; j < CB; ++j)
#pragma unroll
        for (int i = 0; i < RB; ++i)
          acc[j][i] = __builtin_amdgcn_mfma_f32_16x16x4f32(rb[SET][j][t], ra[SET][i][t], acc[j][i], 0, 0, 0);
  };
  auto each_set = [&](auto&& fn) __attribute__((always_inline)) {
    fn(std::integral_constant<int, 0>());
    if constexpr (D > 1) fn(std::integral_constant<int, 1>());
    if constexpr (D > 2) fn(std::integral_constant<int, 2>());
    if constexpr (D > 3) fn(std::integral_constant<int, 3>());
  };
  // (the scheduling barriers keep the requests in the order of their use: the waits count on it)
  each_set([&](auto tag) __attribute__((always_inline)) { fetch(tag); __builtin_amdgcn_sched_barrier(0); });
  for (int c = c0; c < c1; c += D) {
    each_set([&](auto tag) __attribute__((always_inline)) {
      multiply(tag);               // (a chunk past the end multiplies zeros)
      __builtin_amdgcn_sched_barrier(0);
      fetch(tag);
      __builtin_amdgcn_sched_barrier(0);
    });
  }
  // acc[j][i][v] of lane (li, kq): filter 16*i + li, patch column 16*j + 4*kq + v.  LDS holds the
  // blocks as [column][filter] with a pitch of 16*RB + 4 (the four column groups of a write land
  // on different banks), so that a wavefront then reads, adds and stores one column of a
  // partial block as one run.
#pragma unroll
  for (int j = 0; j < CB; ++j)
#pragma unroll
    for (int i = 0; i < RB; ++i)
#pragma unroll
      for (int v = 0; v < 4; ++v) sums[wv][(16 * j + 4 * kq + v) * PF + 16 * i + li] = acc[j][i][v];
  __syncthreads();
  float* part = p.partial + (size_t)blockIdx.x * ((size_t)p.G * Fg * cols) + (size_t)g * Fg * cols;
  const bool f_ok = lane < 16 * RB && f0 + lane < Fg;
  const int fl = f_ok ? lane : 0;
#pragma unroll
  for (int u = 0; u < 4 * CB; ++u) {
    const int q = wv + 4 * u;
    const float sum = (sums[0][q * PF + fl] + sums[1][q * PF + fl]) + (sums[2][q * PF + fl] + sums[3][q * PF + fl]);
    if (f_ok && q < cols) part[(size_t)q * Fg + f0 + lane] = sum;
  }
}

// dW(f, q) = scale_t*dW + scale_o * sum over splits of partial[z][g][q][fl].
// 16 outputs per workgroup; 16 lane groups take every 16th split, eight loads in flight
// each, and meet in LDS (fixed order of additions).
__global__ void __launch_bounds__(256) k_conv_outp_finish(ConvArgs p) {
  __shared__ float sv[16][17];
  const int r = threadIdx.x & 15, grp = threadIdx.x >> 4;
  const int per_group = p.Fg * p.Cg * p.kk2;
  const int total = p.G * per_group;
  const int e = blockIdx.x * 16 + r;
  const float* part = p.partial + (size_t)blockIdx.y * p.splits * total;   // (grid y: chunk of modules)
  float acc = 0.f;
  if (e < total) {
    int z = grp;
    for (; z + 112 < p.splits; z += 128) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = part[(size_t)(z + 16 * u) * total + e];
#pragma unroll
      for (int u = 0; u < 8; ++u) acc += v[u];
    }
    for (; z < p.splits; z += 16) acc += part[(size_t)z * total + e];
  }
  sv[grp][r] = acc;
  __syncthreads();
  if (grp == 0 && e < total) {
    float sum = sv[0][r];
#pragma unroll
    for (int g2 = 1; g2 < 16; ++g2) sum += sv[g2][r];
    const int g = e / per_group, rem = e - g * per_group;
    const int q = rem / p.Fg, fl = rem - q * p.Fg;
    float* t = p.out + (size_t)blockIdx.y * total + (size_t)p.F * q + g * p.Fg + fl;
    *t = (p.scale_t == 0.f ? 0.f : p.scale_t * *t) + p.scale_o * sum;
  }
}

// The same sum for few partial blocks (fewer than 16 per chunk, e.g. the single block per module
// of a locally connected layer's gradient): one lane per output, the blocks added in order, so
// that a wavefront reads and writes whole 256-byte runs (with one lane group per 16th block the
// 2.4 million outputs of a 64-module layer took 53 us; this way 5 us).
__global__ void __launch_bounds__(256) k_conv_outp_finish_few(ConvArgs p) {
  const int per_group = p.Fg * p.Cg * p.kk2;
  const int total = p.G * per_group;
  const int e = blockIdx.x * 256 + threadIdx.x;
  if (e >= total) return;
  const float* part = p.partial + (size_t)blockIdx.y * p.splits * total;
  float sum = part[e];
  for (int z = 1; z < p.splits; ++z) sum += part[(size_t)z * total + e];
  const int g = e / per_group, rem = e - g * per_group;
  const int q = rem / p.Fg, fl = rem - q * p.Fg;
  float* t = p.out + (size_t)blockIdx.y * total + (size_t)p.F * q + g * p.Fg + fl;
  *t = (p.scale_t == 0.f ? 0.f : p.scale_t * *t) + p.scale_o * sum;
}

// The same sum for many partial blocks (the small-output kernel leaves one per workgroup, up to
// 256): 64 neighbouring outputs per workgroup, one per lane, so that a wavefront reads whole
// 256-byte runs; the 16 wavefronts take every 16th block with all their loads in flight and
// meet in LDS.  Fixed order of additions.
__global__ void __launch_bounds__(1024) k_conv_outp_finish_wide(ConvArgs p) {
  __shared__ float sv[16][64];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int per_group = p.Fg * p.Cg * p.kk2;
  const int total = p.G * per_group;
  const int e = blockIdx.x * 64 + lane;
  const float* part = p.partial + (size_t)blockIdx.y * p.splits * total;
  float acc = 0.f;
  if (e < total) {
    for (int z0 = wv; z0 < p.splits; z0 += 16 * 16) {
      float v[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        const int z = z0 + 16 * u;
        v[u] = z < p.splits ? part[(size_t)z * total + e] : 0.f;
      }
#pragma unroll
      for (int u = 0; u < 16; ++u) acc += v[u];
    }
  }
  sv[wv][lane] = acc;
  __syncthreads();
  if (wv == 0 && e < total) {
    float sum = sv[0][lane];
#pragma unroll
    for (int w = 1; w < 16; ++w) sum += sv[w][lane];
    const int g = e / per_group, rem = e - g * per_group;
    const int q = rem / p.Fg, fl = rem - q * p.Fg;
    float* t = p.out + (size_t)blockIdx.y * total + (size_t)p.F * q + g * p.Fg + fl;
    *t = (p.scale_t == 0.f ? 0.f : p.scale_t * *t) + p.scale_o * sum;
  }
}

// ------------------------------------------------------------------ convDown through a patch matrix
// With few colours per group the implicit GEMM above has only Cg useful columns
// in a 32-wide matrix-core block and re-reads the hidden activations once per
// filter tap.  Instead: P = hid (M*N x Fg, read once) * W (Fg x Cg*k*k) is a plain
// product on the buffers as they are (hid is column-major with leading dimension
// M*N), and every image pixel then gathers the <= ceil(k/s)^2 entries of P that
// land on it.  P(r, q) with r = module*N + image, q = (c*k + ky)*k + kx.
int dn_gemm(bool a_trans, bool b_trans, int M, int N, int K, float alpha, const float* A, int lda, const float* B,
            int ldb, float beta, float* C, int ldc);

// The patch product for layers with at most 2*KS filters per group and at most 32*CT
// patch columns, without LDS tiles: W of the group sits in registers as MFMA operands
// and a wavefront walks over tiles of 32 rows of hid (one module, 32 images), whose
// operands go from global memory straight into the operand registers (lane (image n,
// half h) loads filter 2*ks + h for step ks: 128-byte runs).  While tile i is
// multiplied, the loads of tile i+1 and the stores of tile i-1 are issued between its
// MFMAs.  Every path issues the same number of memory operations and nothing is in
// flight when the loop is entered, so that the compiler's wait counts (sized for the
// path with the fewest operations behind the awaited one) are those of the steady
// state.  P has pcols rounded up to 8 columns; the extra ones are written as zeros.
template <int KS, int CT>
__global__ void __launch_bounds__(256, 1)
k_conv_patch_regs(const float* hid, const float* flt, float* P, int prow, int Fg, int F, int pcols, int pcols8) {
  constexpr unsigned FAR = 0x80000000u;  // beyond any buffer here: sizes are below 2^31 bytes
  const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5, ln = lane & 31;
  __amdgpu_buffer_rsrc_t r_hid =
      __builtin_amdgcn_make_buffer_rsrc((void*)hid, 0, (int)((unsigned)prow * (unsigned)Fg * 4u), 0x00020000);
  __amdgpu_buffer_rsrc_t r_flt =
      __builtin_amdgcn_make_buffer_rsrc((void*)flt, 0, (int)((unsigned)F * (unsigned)pcols * 4u), 0x00020000);
  __amdgpu_buffer_rsrc_t r_out =
      __builtin_amdgcn_make_buffer_rsrc((void*)P, 0, (int)((unsigned)prow * (unsigned)pcols8 * 4u), 0x00020000);
  // W(f, q) of the group sits at f + F*q (flt already points at the group's first filter):
  // lanes of an operand run along q, so it is read along f (whole cache lines) into LDS
  // and picked up from there; rows of 32*CT + 1 floats keep both sides off bank conflicts.
  constexpr int QP = 32 * CT + 1;
  __shared__ float w_lds[2 * KS * QP];
  {
    constexpr int PER_LANE = 2 * KS * 32 * CT / 256;   // all requested before the first is written
    float w[PER_LANE];
#pragma unroll
    for (int it = 0; it < PER_LANE; ++it) {
      const int e = tid + it * 256, f = e % (2 * KS), q = e / (2 * KS);
      const unsigned off = q < pcols && f < Fg ? ((unsigned)f + (unsigned)F * (unsigned)q) * 4u : FAR;
      w[it] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r_flt, (int)off, 0, 0));
    }
#pragma unroll
    for (int it = 0; it < PER_LANE; ++it) {
      const int e = tid + it * 256, f = e % (2 * KS), q = e / (2 * KS);
      w_lds[f * QP + q] = w[it];
    }
  }
  __syncthreads();
  float b[KS][CT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) b[ks][ct] = w_lds[(2 * ks + half) * QP + ct * 32 + ln];
  const int T = prow >> 5;
  const int nwaves = gridDim.x * 4;
  const unsigned cstride = (unsigned)prow * 4u;                      // bytes between columns of hid and of P
  const unsigned in_lane = ln * 4u + (unsigned)half * cstride;       // a filter beyond the group is beyond the buffer
  const unsigned out_lane = ln * 4u + (unsigned)(4 * half) * cstride;

  // One tile step.  MULT: multiply tile `a` into `cur`.  Always: load tile tn into `an`
  // and store `prev` at row offset out_prev (FAR drops it).  acc[ct][v] of lane (n, half)
  // is patch column ct*32 + 8*(v/4) + 4*half + v%4.
  auto step = [&](auto mult_tag, const float (&a)[KS], float (&an)[KS], f32x16 (&cur)[CT], const f32x16 (&prev)[CT],
                  int tn, unsigned out_prev) __attribute__((always_inline)) {
    constexpr bool MULT = decltype(mult_tag)::value;
    const unsigned base = (unsigned)tn * 128u;
    unsigned octet[CT][4];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
      for (int q = 0; q < 4; ++q)
        octet[ct][q] = out_prev != FAR && ct * 32 + 8 * q < pcols8 ? out_prev + (unsigned)(ct * 32 + 8 * q) * cstride : FAR;
    if (MULT) {
#pragma unroll
      for (int ct = 0; ct < CT; ++ct)
#pragma unroll
        for (int v = 0; v < 16; ++v) cur[ct][v] = 0.f;
    }
    constexpr int SPS = (16 * CT + (KS - KS / 2) - 1) / (KS - KS / 2);  // stores per step
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if (ks < KS / 2) {
#pragma unroll
        for (int u = 0; u < 2; ++u)
          an[2 * ks + u] = __builtin_bit_cast(
              float, __builtin_amdgcn_raw_buffer_load_b32(r_hid, (int)in_lane, (int)(base + (unsigned)(4 * ks + 2 * u) * cstride), 0));
      } else {
#pragma unroll
        for (int u = 0; u < SPS; ++u) {
          const int si = (ks - KS / 2) * SPS + u;
          if (si < 16 * CT) {
            const float val = prev[si >> 4][si & 15];  // (a bit cast applied to the vector element itself reads element 0)
            __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(val), r_out, (int)out_lane,
                                                  (int)(octet[si >> 4][(si >> 2) & 3] + (si & 3) * cstride), 0);
          }
        }
      }
      if (MULT) {
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
          cur[ct] = __builtin_amdgcn_mfma_f32_32x32x2f32(b[ks][ct], a[ks], cur[ct], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  int t = blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(tid >> 6);
  if (t >= T) return;
  float a0[KS], a1[KS];
  f32x16 acc0[CT], acc1[CT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct)
#pragma unroll
    for (int v = 0; v < 16; ++v) { acc0[ct][v] = 0.f; acc1[ct][v] = 0.f; }
  step(std::false_type(), a1, a0, acc0, acc1, t, FAR);
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): nothing in flight when the loop is entered
  unsigned out_prev = FAR;
  while (true) {
    int tn = t + nwaves;
    step(std::true_type(), a0, a1, acc0, acc1, tn < T ? tn : t, out_prev);
    out_prev = (unsigned)t * 128u;
    if (tn >= T) { step(std::false_type(), a0, a0, acc1, acc0, t, out_prev); break; }
    t = tn;
    tn = t + nwaves;
    step(std::true_type(), a1, a0, acc1, acc0, tn < T ? tn : t, out_prev);
    out_prev = (unsigned)t * 128u;
    if (tn >= T) { step(std::false_type(), a1, a1, acc0, acc1, t, out_prev); break; }
    t = tn;
  }
}

// Stride 1 with a compile-time filter size: every pixel has exactly K x K candidate
// modules, the loops unroll and all K*K loads of a lane are in flight together (a tap
// whose module lies outside the grid re-reads module 0 and is weighted by zero).
template <int K>
__global__ void __launch_bounds__(256) k_conv_down_gather_s1(ConvArgs p, const float* P, int g) {
  const int NV = p.N >> 2;
  const uint32_t total = (uint32_t)NV * p.HH * p.Cg;
  const long long ldp = (long long)p.M * p.N;
  for (uint32_t e = blockIdx.x * 256u + threadIdx.x; e < total; e += gridDim.x * 256u) {
    const uint32_t nv = e % NV;
    const uint32_t pix = (e / NV) % p.HH;
    const int c = (int)(e / ((uint32_t)NV * p.HH));
    const int y = (int)(pix / p.H) - p.pad0, x = (int)(pix % p.H) - p.pad0;  // padded-frame coordinates
    const float* base = P + (long long)c * K * K * ldp + 4 * nv;
    float4 v[K * K];
    bool ok[K * K];
#pragma unroll
    for (int ky = 0; ky < K; ++ky)
#pragma unroll
      for (int kx = 0; kx < K; ++kx) {
        const int my = y - ky, mx = x - kx;
        const bool in = my >= 0 && my < p.Mx && mx >= 0 && mx < p.Mx;
        ok[ky * K + kx] = in;
        v[ky * K + kx] = *reinterpret_cast<const float4*>(base + (long long)(ky * K + kx) * ldp +
                                                          (long long)(in ? my * p.Mx + mx : 0) * p.N);
      }
    // same order of additions as the general kernel: my (and within it mx) descending
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
    for (int ky = 0; ky < K; ++ky)
#pragma unroll
      for (int kx = 0; kx < K; ++kx)
        if (ok[ky * K + kx]) {
          const float4 t = v[ky * K + kx];
          acc.x += t.x; acc.y += t.y; acc.z += t.z; acc.w += t.w;
        }
    float* t = p.out + (size_t)p.N * ((size_t)(g * p.Cg + c) * p.HH + pix) + 4 * nv;
    float4 r = acc;
    if (p.scale_t != 0.f || p.scale_o != 1.f) {
      const float4 o = p.scale_t == 0.f ? make_float4(0.f, 0.f, 0.f, 0.f) : *reinterpret_cast<const float4*>(t);
      r = make_float4(p.scale_t * o.x + p.scale_o * acc.x, p.scale_t * o.y + p.scale_o * acc.y,
                      p.scale_t * o.z + p.scale_o * acc.z, p.scale_t * o.w + p.scale_o * acc.w);
    }
    *reinterpret_cast<float4*>(t) = r;
  }
}

__global__ void __launch_bounds__(256) k_conv_down_gather(ConvArgs p, const float* P, int g) {
  // one lane: 4 neighbouring images of one (colour of the group, y, x)
  const int NV = p.N >> 2;
  const uint32_t total = (uint32_t)NV * p.HH * p.Cg;
  const long long ldp = (long long)p.M * p.N;
  for (uint32_t e = blockIdx.x * 256u + threadIdx.x; e < total; e += gridDim.x * 256u) {
    const uint32_t nv = e % NV;
    const uint32_t pix = (e / NV) % p.HH;
    const int c = (int)(e / ((uint32_t)NV * p.HH));
    const int y = (int)(pix / p.H) - p.pad0, x = (int)(pix % p.H) - p.pad0;  // padded-frame coordinates
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    // modules my with 0 <= y - my*s < k
    const int my_hi = y / p.s < p.Mx - 1 ? y / p.s : p.Mx - 1;
    const int mx_hi = x / p.s < p.Mx - 1 ? x / p.s : p.Mx - 1;
    for (int my = my_hi; my >= 0 && y - my * p.s < p.k; --my) {
      const int ky = y - my * p.s;
      for (int mx = mx_hi; mx >= 0 && x - mx * p.s < p.k; --mx) {
        const int kx = x - mx * p.s;
        const long long q = (long long)(c * p.k + ky) * p.k + kx;
        const float4 v = *reinterpret_cast<const float4*>(P + q * ldp + (long long)(my * p.Mx + mx) * p.N + 4 * nv);
        acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
      }
    }
    float* t = p.out + (size_t)p.N * ((size_t)(g * p.Cg + c) * p.HH + pix) + 4 * nv;
    float4 r = acc;
    if (p.scale_t != 0.f || p.scale_o != 1.f) {
      const float4 o = p.scale_t == 0.f ? make_float4(0.f, 0.f, 0.f, 0.f) : *reinterpret_cast<const float4*>(t);
      r = make_float4(p.scale_t * o.x + p.scale_o * acc.x, p.scale_t * o.y + p.scale_o * acc.y,
                      p.scale_t * o.z + p.scale_o * acc.z, p.scale_t * o.w + p.scale_o * acc.w);
    }
    *reinterpret_cast<float4*>(t) = r;
  }
}

// ------------------------------------------------------------------ convDown, stride 1, at most 4 colours
// One launch, every pixel written once, no intermediate (the counterpart of the reference's
// img_acts_color, cudamat_conv_kernels.cuh:419-554, dispatched at cudamat_conv.cu:375-405).
// The implicit GEMM of this pass has only Cg <= 4 output columns, which 32- and 16-wide
// matrix-core blocks waste; v_mfma_f32_4x4x1_16b_f32 runs at the same rate on 16
// independent 4 x 4 blocks of rank 1:
//   block rows    4 neighbouring images            (first operand: one hidden activation per lane,
//                                                   read from memory as it lies, 128-byte runs)
//   block columns the colours of the group (+ pad) (second operand: w[c, ky, kx, f] per lane)
//   blocks 0-7    images 0..31 with filter 2i, blocks 8-15 the same images with filter 2i + 1
// A wavefront owns a 4 x 4 tile of pixels for 32 images (16 accumulators of 4 registers, lane
// (block b, colour c), register v = image 4b + v) and one of NWV parts of the group's filters;
// per pair of filters it loads the (K + 3)^2 modules its pixels reach once (a module outside
// the grid is an out-of-range buffer offset and reads as zero) and issues 16 * K * K MFMAs,
// acc[pixel] += hid[module = pixel - tap] (x) w[tap], with the loads of the next pair and the
// LDS reads of its weights issued between them.  The wavefronts of a workgroup (the parts of
// the filters) and the two filter parities meet in LDS in a fixed order.
// Measured on the part: with 16 independent accumulators this MFMA form runs at the rate of the
// 32 x 32 x 2 form (149 against 155 TFLOP/s), but it occupies the pipe for 8 cycles only, and
// every other instruction of the same wavefront between two of them (LDS read, buffer load)
// costs about one such slot, where a 64-cycle MFMA hides a dozen; two wavefronts per SIMD halve
// that cost but need the operand sets in 256 registers, which spills.
template <int K, int FSC, int NWV>
__global__ void __launch_bounds__(64 * NWV, 1) k_conv_down_px(ConvArgs p) {
  constexpr int T = 4, HR = K + T - 1, KK = K * K, NA = HR * HR, NT = 64 * NWV;
  constexpr int CS = KK * FSC + 8;          // floats between the colours' weight blocks: their banks differ by 8
  constexpr int WSZ = 5 * CS;               // four colours and a block of zeros (lanes of the pad colours)
  constexpr int RED = NWV * (T * T * 2) * 64;   // the final sum reuses the weights' memory
  constexpr unsigned FAR_V = 0x40000000u, FAR_S = 0x20000000u;   // either one is beyond the buffer, and so is their sum
  __shared__ float lds[WSZ > RED ? WSZ : RED];
  const int tid = threadIdx.x, lane = tid & 63, par = lane >> 5, li = lane & 31, c = lane & 3;
  const int wq = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = blockIdx.z;
  // workgroup -> (image block, pixel tile); consecutive workgroups go round the 8 XCDs, so every XCD
  // is handed a contiguous run of tiles (neighbouring tiles share the modules between them in its L2)
  const int tiles_x = (p.H + T - 1) / T, tiles = tiles_x * tiles_x;
  const int total = (int)gridDim.x;
  int wid = (int)blockIdx.x;
  if ((total & 7) == 0) wid = (wid & 7) * (total >> 3) + (wid >> 3);
  const int nb = wid / tiles, tile = wid - nb * tiles;
  const int ty = tile / tiles_x, tx = tile - ty * tiles_x;
  const int y0 = ty * T, x0 = tx * T;
  const int my0 = y0 - p.pad0 - (K - 1), mx0 = x0 - p.pad0 - (K - 1);   // first module row / column of the halo
  const int Fq = p.Fg / NWV, nit = Fq >> 1;
  const int f0 = g * p.Fg + wq * Fq;                                     // first filter of this wavefront

  __amdgpu_buffer_rsrc_t r_hid = __builtin_amdgcn_make_buffer_rsrc((void*)p.hid, 0, (int)p.a_bytes, 0x00020000);
  __amdgpu_buffer_rsrc_t r_flt = __builtin_amdgcn_make_buffer_rsrc((void*)p.flt, 0, (int)p.b_bytes, 0x00020000);

  const unsigned plane = (unsigned)p.M * (unsigned)p.N * 4u;            // bytes between filters
  unsigned voff[HR], soff[HR], sstep[HR];
#pragma unroll
  for (int j = 0; j < HR; ++j) {
    const int mx = mx0 + j;
    voff[j] = mx >= 0 && mx < p.Mx ? (unsigned)li * 4u + (unsigned)par * plane + (unsigned)(mx * p.N) * 4u : FAR_V;
  }
#pragma unroll
  for (int r = 0; r < HR; ++r) {
    const int my = my0 + r;
    const bool ok = my >= 0 && my < p.Mx;
    soff[r] = ok ? (unsigned)f0 * plane + ((unsigned)(my * p.Mx) * (unsigned)p.N + (unsigned)(nb * 32)) * 4u : FAR_S;
    sstep[r] = ok ? 2u * plane : 0u;
  }
  float a0[NA], a1[NA];
  auto request = [&](float (&an)[NA], int idx) __attribute__((always_inline)) {
    an[idx] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r_hid, (int)voff[idx % HR], (int)soff[idx / HR], 0));
  };
#pragma unroll
  for (int i = 0; i < NA; ++i) request(a0, i);

  // weights of the group: w(f, q = c*KK + tap) at f + F*q, read along f, kept as [c][tap][f]
  {
    constexpr int PER = (4 * KK * FSC + NT - 1) / NT;
    float w[PER];
#pragma unroll
    for (int it = 0; it < PER; ++it) {
      const int e = tid + it * NT, f = e & (FSC - 1), q = e / FSC;
      const unsigned off = q < p.Cg * KK && f < p.Fg ? ((unsigned)(g * p.Fg + f) + (unsigned)p.F * (unsigned)q) * 4u : FAR_V;
      w[it] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r_flt, (int)off, 0, 0));
    }
#pragma unroll
    for (int it = 0; it < PER; ++it) {
      const int e = tid + it * NT, f = e & (FSC - 1), q = e / FSC;
      if (e < 4 * KK * FSC) lds[(q / KK) * CS + (q % KK) * FSC + f] = w[it];
    }
    for (int e = tid; e < KK * FSC; e += NT) lds[4 * CS + e] = 0.f;
  }
  __syncthreads();
  const float* wl = lds + (c < p.Cg ? c : 4) * CS + wq * Fq + par;   // + 2 per pair of filters, + FSC per tap

  f32x4 acc[T * T];
#pragma unroll
  for (int i = 0; i < T * T; ++i) acc[i] = (f32x4){0.f, 0.f, 0.f, 0.f};

  // One pair of filters: multiply (a, b) into the accumulators.  Between the MFMAs: one request
  // in GAP for the next pair's modules (into an; beyond the last pair the offsets are out of range
  // and nothing is fetched) and one LDS read per tap for the next pair's weights (into bn).
  // Taps run in descending order, so module rows are first used in ascending order.
  float b0[KK], b1[KK];
#pragma unroll
  for (int t = 0; t < KK; ++t) b0[t] = wl[t * FSC];
  auto step = [&](const float (&a)[NA], const float (&b)[KK], float (&an)[NA], float (&bn)[KK], const float* wn)
      __attribute__((always_inline)) {
    constexpr int NM = T * T * KK, GAP = NM / NA;
#pragma unroll
    for (int gi = 0; gi < KK; ++gi) {
      const int ky = K - 1 - gi / K, kx = K - 1 - gi % K;
#pragma unroll
      for (int yy = 0; yy < T; ++yy)
#pragma unroll
        for (int xx = 0; xx < T; ++xx) {
          const int m = (gi * T + yy) * T + xx;
          if (m % GAP == 0 && m / GAP < NA) {
            __builtin_amdgcn_sched_barrier(0);
            request(an, m / GAP);
            __builtin_amdgcn_sched_barrier(0);
          }
          if (m % (T * T) == T * T / 2) {
            __builtin_amdgcn_sched_barrier(0);
            bn[gi] = wn[gi * FSC];
            __builtin_amdgcn_sched_barrier(0);
          }
          acc[yy * T + xx] = __builtin_amdgcn_mfma_f32_4x4x1f32(a[(yy + K - 1 - ky) * HR + xx + K - 1 - kx], b[ky * K + kx],
                                                                acc[yy * T + xx], 0, 0, 0);
        }
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  int it = 0;
#define DOWN_PX_STEP(A, B, AN, BN)                                                      \
  _Pragma("unroll") for (int r = 0; r < HR; ++r) soff[r] = it + 1 < nit ? soff[r] + sstep[r] : FAR_S; \
  step(A, B, AN, BN, wl + 2 * (it + 1 < nit ? it + 1 : it));                            \
  if (++it >= nit) break;
  while (true) {
    DOWN_PX_STEP(a0, b0, a1, b1)
    DOWN_PX_STEP(a1, b1, a0, b0)
  }
#undef DOWN_PX_STEP

  // The two filter parities (lanes l and l + 32) are added inside the wavefront: v_permlane32_swap
  // on two accumulator registers leaves, in lanes 0-31, both parities of the first and, in lanes
  // 32-63, both parities of the second, so one addition finishes two registers.  The parts of the
  // filters (the wavefronts) then meet in LDS in a fixed order: red[wavefront][register pair][lane].
  __syncthreads();
#pragma unroll
  for (int j = 0; j < T * T * 2; ++j) {
    const float r0 = acc[j >> 1][(j & 1) * 2], r1 = acc[j >> 1][(j & 1) * 2 + 1];   // registers 2j and 2j + 1 of the tile
    const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(r0), __float_as_uint(r1), false, false);
    lds[(wq * (T * T * 2) + j) * 64 + lane] = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
  }
  __syncthreads();
  const int outs = T * T * p.Cg * 32;
  for (int o = tid; o < outs; o += NT) {
    const int img = o & 31, rest = o >> 5;
    const int pix = rest / p.Cg, cc = rest - pix * p.Cg;
    const int reg = pix * 4 + (img & 3), ln = 4 * (img >> 2) + cc + 32 * (reg & 1);
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < NWV; ++w) s += lds[(w * (T * T * 2) + (reg >> 1)) * 64 + ln];
    const int y = y0 + pix / T, x = x0 + pix % T;
    if (y < p.H && x < p.H) {
      float* t = p.out + ((size_t)(g * p.Cg + cc) * p.HH + (size_t)(y * p.H + x)) * p.N + nb * 32 + img;
      *t = (p.scale_t == 0.f ? 0.f : p.scale_t * *t) + p.scale_o * s;
    }
  }
}

// ------------------------------------------------------------------ host side

static char g_conv_err[256];
static bool g_conv_failed = false;

void conv_set_error(const char* where, const char* what) {
  snprintf(g_conv_err, sizeof(g_conv_err), "%s: %s", where, what);
  g_conv_failed = true;
}
void conv_clear_error() { g_conv_failed = false; }

#define CONV_REQUIRE(cond, where)        \
  do {                                   \
    if (!(cond)) {                       \
      conv_set_error(where, #cond);      \
      return;                            \
    }                                    \
  } while (0)

static int isqrt_exact(int v) {
  if (v < 0) return -1;
  int r = (int)(sqrt((double)v) + 0.5);
  return r * r == v ? r : -1;
}

// ------------------------------------------------------------------ convUp, short reductions
// Layers whose reduction (colours x k x k) has at most 2*KS terms and whose groups
// have at most 32*CT filters (a first layer over RGB is the usual case) do not need
// LDS tiles: the whole filter bank of a group lives in registers as MFMA operands
// and a wavefront walks over tiles of (one module, 32 images).  An image operand is
// used by this wavefront only, so it goes from global memory straight into the
// operand register: lane (image n, half h) loads tap k = 2*ks + h for step ks, a
// 128-byte run per half wavefront.  Interior modules need no vector ALU work at all
// (fixed lane offsets, module origin in a scalar register); modules that touch the
// padding mask taps by a bit test and send them out of the buffer's range, where
// loads return zero.  Output: 128-byte runs per filter.
// Schedule of a wavefront: while tile i is multiplied, the loads of tile i+1 and the
// stores of tile i-1 are issued between its MFMAs, so the matrix pipe is never idle
// behind memory instructions, and the arrival of tile i+1 is awaited at one place
// (the hand-over), where only the stores of tile i-1 are younger and may stay in flight.
template <int KS, int CT>
__global__ void __launch_bounds__(256, 1) k_conv_up_regs(ConvArgs p) {
  constexpr unsigned FAR = 0x80000000u;  // beyond any buffer here: sizes are below 2^31 bytes
  __shared__ unsigned yx_tab[2 * KS], tap_tab[2 * KS];
  const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5, ln = lane & 31;
  const int g = blockIdx.z;
  const int f_lo = blockIdx.y * (32 * CT);      // grid y: blocks of 32 * CT filters of the group
  const int K = p.Cg * p.kk2;
  for (int k = tid; k < 2 * KS; k += 256) {
    const unsigned c = fd_div((unsigned)k, p.dkk2), r = (unsigned)k - c * (unsigned)p.kk2;
    const unsigned ky = fd_div(r, p.dk), kx = r - ky * (unsigned)p.k;
    yx_tab[k] = k < K ? (1u << ky) | (1u << (16 + kx)) : 0xffffffffu;
    tap_tab[k] = k < K ? ((((unsigned)(g * p.Cg) + c) * p.H + ky) * p.H + kx) * (unsigned)p.N * 4u : FAR;
  }
  __amdgpu_buffer_rsrc_t r_img = __builtin_amdgcn_make_buffer_rsrc((void*)p.img, 0, (int)p.a_bytes, 0x00020000);
  __amdgpu_buffer_rsrc_t r_flt = __builtin_amdgcn_make_buffer_rsrc((void*)p.flt, 0, (int)p.b_bytes, 0x00020000);
  __amdgpu_buffer_rsrc_t r_out =
      __builtin_amdgcn_make_buffer_rsrc((void*)p.out, 0, (int)((unsigned)p.N * (unsigned)p.M * (unsigned)p.F * 4u), 0x00020000);

  // Filter operands of this lane: element (filter, tap k) sits at filter + F*k, so a
  // tap beyond the reduction is beyond the buffer and reads as zero.
  float b[KS][CT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const int fl = f_lo + ct * 32 + ln;                     // filter within the group
    const unsigned voff = fl < p.Fg ? ((unsigned)(g * p.Fg + fl) + (unsigned)(half * p.F)) * 4u : FAR;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      b[ks][ct] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r_flt, (int)voff, ks * 8 * p.F, 0));
  }
  __syncthreads();
  unsigned tap[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) tap[ks] = tap_tab[2 * ks + half] + ln * 4u;

  const int NB = p.N >> 5;
  const int T = p.M * NB;
  const int nwaves = gridDim.x * 4;
  const unsigned fstride = (unsigned)p.N * (unsigned)p.M * 4u;        // bytes between filters in the output
  const unsigned out_lane = ln * 4u + (unsigned)(4 * half) * fstride;

  // One tile step.  MULT: multiply tile `a` into `cur`.  Always: gather tile tn into
  // `an` and store `prev` (products of the tile whose output offset is out_prev; FAR
  // drops them).  acc[ct][v] of lane (n, half) is filter ct*32 + 8*(v/4) + 4*half + v%4.
  auto step = [&](auto mult_tag, const float (&a)[KS], float (&an)[KS], f32x16 (&cur)[CT], const f32x16 (&prev)[CT],
                  int tn, unsigned out_prev) __attribute__((always_inline)) {
    constexpr bool MULT = decltype(mult_tag)::value;
    const int m = (int)fd_div((unsigned)tn, p.dS), nb = tn - m * NB;  // (dS: divisor N/32 for this kernel)
    const int my = (int)fd_div((unsigned)m, p.dMx), mx = m - my * p.Mx;
    const int y0 = my * p.s + p.pad0, x0 = mx * p.s + p.pad0;
    const int base = ((y0 * p.H + x0) * p.N + nb * 32) * 4;
    const bool interior = y0 >= 0 && x0 >= 0 && y0 + p.k <= p.H && x0 + p.k <= p.H;
    // bit ky (kx) set: row y0 + ky (column x0 + kx) lies inside the image
    const int ylo = y0 < 0 ? -y0 : 0, yhi = p.H - y0 < p.k ? p.H - y0 : p.k;
    const int xlo = x0 < 0 ? -x0 : 0, xhi = p.H - x0 < p.k ? p.H - x0 : p.k;
    const unsigned ym = yhi > ylo ? ((1u << yhi) - 1u) & ~((1u << ylo) - 1u) : 0u;
    const unsigned xm = xhi > xlo ? ((1u << xhi) - 1u) & ~((1u << xlo) - 1u) : 0u;
    const unsigned bad = ~(ym | (xm << 16));
    unsigned octet[CT][4];  // filters per group are a multiple of 8: an octet is stored whole or dropped
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
      for (int q = 0; q < 4; ++q)
        octet[ct][q] = out_prev != FAR && f_lo + ct * 32 + 8 * q < p.Fg ? out_prev + (unsigned)(ct * 32 + 8 * q) * fstride : FAR;
    if (MULT) {
#pragma unroll
      for (int ct = 0; ct < CT; ++ct)
#pragma unroll
        for (int v = 0; v < 16; ++v) cur[ct][v] = 0.f;
    }
    // The gathers of the next tile go out in the first fifth of the steps, the stores of the
    // previous tile one at a time over the rest (every wavefront of the chip reaches the same
    // step at about the same time, so bunched stores arrive at the memory system as one burst;
    // spread out they cost the 3 -> 64 filters of 5 x 5 layer 18.6 us instead of 19.0).  The
    // loads come first so that waiting for them never waits for a store.
    constexpr int LKS = (KS + 4) / 5;                       // steps that issue loads
    constexpr int LPS = (KS + LKS - 1) / LKS;               // loads per such step
    constexpr int SPS = (16 * CT + (KS - LKS) - 1) / (KS - LKS);  // stores per later step
    auto rest = [&](int ks) __attribute__((always_inline)) {
      if (ks >= LKS) {
#pragma unroll
        for (int u = 0; u < SPS; ++u) {
          const int si = (ks - LKS) * SPS + u;
          if (si < 16 * CT) {
            const float val = prev[si >> 4][si & 15];  // (a bit cast applied to the vector element itself reads element 0)
            __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(val), r_out, (int)out_lane,
                                                  (int)(octet[si >> 4][(si >> 2) & 3] + (si & 3) * fstride), 0);
          }
        }
      }
      if (MULT) {
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
          cur[ct] = __builtin_amdgcn_mfma_f32_32x32x2f32(b[ks][ct], a[ks], cur[ct], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    if (interior) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        if (ks < LKS) {
#pragma unroll
          for (int u = 0; u < LPS; ++u) {
            const int idx = ks * LPS + u;
            if (idx < KS)
              an[idx] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r_img, (int)tap[idx], base, 0));
          }
        }
        rest(ks);
      }
    } else {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        if (ks < LKS) {
#pragma unroll
          for (int u = 0; u < LPS; ++u) {
            const int idx = ks * LPS + u;
            if (idx < KS) {
              const unsigned yx = yx_tab[2 * idx + half];
              const unsigned voff = (yx & bad) ? FAR : tap[idx] + (unsigned)base;
              an[idx] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r_img, (int)voff, 0, 0));
            }
          }
        }
        rest(ks);
      }
    }
  };
  auto out_of = [&](int t) {
    const int m = (int)fd_div((unsigned)t, p.dS), nb = t - m * NB;
    return ((unsigned)(nb * 32) + (unsigned)p.N * (unsigned)m) * 4u + (unsigned)(g * p.Fg + f_lo) * fstride;
  };
  // Round i hands tile i*nwaves + (wave + 12*i) mod nwaves to a wavefront: the shift keeps
  // a wavefront from meeting the same image column in every round (rounds are often a
  // whole number of module rows apart), which would give some all the tiles that touch
  // the padding and need the masked gather.
  const int wave = blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(tid >> 6);
  auto tile_of = [&](int round) {
    int w = wave + 12 * round;
    w -= (int)fd_div((unsigned)w, p.dSS) * nwaves;  // (dSS: divisor nwaves for this kernel)
    return round * nwaves + w;
  };
  int round = 0;
  int t = tile_of(0);
  if (t >= T) return;
  float a0[KS], a1[KS];
  f32x16 acc0[CT], acc1[CT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct)
#pragma unroll
    for (int v = 0; v < 16; ++v) { acc0[ct][v] = 0.f; acc1[ct][v] = 0.f; }
  step(std::false_type(), a1, a0, acc0, acc1, t, FAR);
  // Nothing is in flight when the loop is entered: the waits inside it are then those of
  // its own steady state (the compiler sizes a wait for the path with the fewest
  // operations behind the awaited one; a first trip with loads still in flight and no
  // stores behind them would make every later trip wait for its stores).
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
  unsigned out_prev = FAR;
  while (true) {
    int tn = tile_of(++round);
    step(std::true_type(), a0, a1, acc0, acc1, tn < T ? tn : t, out_prev);
    out_prev = out_of(t);
    if (tn >= T) { step(std::false_type(), a0, a0, acc1, acc0, t, out_prev); break; }
    t = tn;
    tn = tile_of(++round);
    step(std::true_type(), a1, a0, acc1, acc0, tn < T ? tn : t, out_prev);
    out_prev = out_of(t);
    if (tn >= T) { step(std::false_type(), a1, a1, acc0, acc1, t, out_prev); break; }
    t = tn;
  }
}

// ------------------------------------------------------------------ convUp, short reductions, one tile per wavefront
// The same layers as k_conv_up_regs (reductions of at most 80 taps, at most 64 filters per
// group) when the batch is a multiple of 64: a wavefront computes one (module, 64 images) tile
// for all filters of the group and ends; two such wavefronts share a SIMD.
//   v_mfma_f32_32x32x1_2b_f32: two 32 x 32 blocks of rank 1 per instruction.  Block rows are 32
//   filters (first operand, the same values in both halves of the wavefront: one LDS read of
//   the filter bank, kept as [tap][filter]); block columns are the images, block b the images
//   32b .. 32b + 31 (second operand: lane = image, so a tap of the whole tile is ONE 256-byte
//   run of the image tensor, its position a scalar: module origin + tap offset in an SGPR, a tap
//   in the padding an out-of-range offset that reads as zero -- no vector arithmetic, no masks).
// All taps of the tile are requested up front (in-order return: the MFMAs of tap k start when
// tap k has arrived), the reduction is exactly the taps (75, not 80), the first 32 filters are
// finished before the second 32 are started, so that their stores run under the second half's
// MFMAs.  Filter size and colours are compile-time, so a tap's offset is three scalar
// multiply-adds (with run-time sizes the 75 address computations were 3400 scalar instructions
// in front of the first MFMA: 28.9 us; with them 17.1 us; with non-temporal stores 15.0 us).
// Measured with the MFMAs replaced by plain arithmetic: 11.6 us (the 33.5 MB of stores and the
// loads); what remains exposed is the second half's stores, which no MFMA is left to cover.
typedef float f32x32 __attribute__((ext_vector_type(32)));
// cache policy of the output stores: non-temporal (the 33.5 MB of outputs of the 3 -> 64 filters layer are
// not read again by this kernel; measured 16.9 -> 15.0 us against the default policy)
#define ST_NT 2
template <int FB, int CG, int KF>   // FB: blocks of 32 filters of the group (1 or 2); CG colours per group, KF x KF filters
__global__ void __launch_bounds__(256, 2) k_conv_up_taps(ConvArgs p) {
  constexpr int K = CG * KF * KF, KMAX = K;
  constexpr unsigned FAR = 0x80000000u;
  __shared__ float w_lds[KMAX * 64];
  const int tid = threadIdx.x, lane = tid & 63, li = lane & 31, half = lane >> 5;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = blockIdx.z;
  const int NB = p.N >> 6;                                   // tiles of 64 images per module
  const int T = p.M * NB;
  const int t = blockIdx.x * 4 + wv;
  const bool live = t < T;
  const int m = live ? t / NB : 0, nb = live ? t - m * NB : 0;
  const int my = (int)fd_div((unsigned)m, p.dMx), mx = m - my * p.Mx;
  const int y0 = my * p.s + p.pad0, x0 = mx * p.s + p.pad0;
  __amdgpu_buffer_rsrc_t r_img = __builtin_amdgcn_make_buffer_rsrc((void*)p.img, 0, (int)p.a_bytes, 0x00020000);
  __amdgpu_buffer_rsrc_t r_flt = __builtin_amdgcn_make_buffer_rsrc((void*)p.flt, 0, (int)p.b_bytes, 0x00020000);
  __amdgpu_buffer_rsrc_t r_out =
      __builtin_amdgcn_make_buffer_rsrc((void*)p.out, 0, (int)((unsigned)p.N * (unsigned)p.M * (unsigned)p.F * 4u), 0x00020000);

  // the group's filter bank: w(f, k) at f + F*k, read along f, kept as [k][64].  Requested before
  // the tile's taps: waiting for it then leaves the (younger) tap loads in flight.
  constexpr int PER = (KMAX * 64 + 255) / 256;
  float w[PER];
#pragma unroll
  for (int it = 0; it < PER; ++it) {
    const int e = tid + it * 256, f = e & 63, k = e >> 6;
    const unsigned off = k < K && f < p.Fg ? ((unsigned)(g * p.Fg + f) + (unsigned)p.F * (unsigned)k) * 4u : FAR;
    w[it] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r_flt, (int)off, 0, 0));
  }
  // the tile's taps: lane = image; a tap's position is wave-uniform (scalar registers only)
  float a[KMAX];
  {
    const unsigned lane_off = (unsigned)lane * 4u;
    const unsigned sx = (unsigned)p.N * 4u, sy = (unsigned)p.H * sx, sc = (unsigned)p.H * sy;
    const unsigned base = (unsigned)(g * CG) * sc + (unsigned)y0 * sy + (unsigned)x0 * sx + (unsigned)(nb * 256);   // (wraps for y0, x0 < 0; taps inside the image come out right)
    bool yv[KF], xv[KF];
#pragma unroll
    for (int i = 0; i < KF; ++i) {
      yv[i] = live && (unsigned)(y0 + i) < (unsigned)p.H;
      xv[i] = (unsigned)(x0 + i) < (unsigned)p.H;
    }
#pragma unroll
    for (int c = 0; c < CG; ++c)
#pragma unroll
      for (int ky = 0; ky < KF; ++ky)
#pragma unroll
        for (int kx = 0; kx < KF; ++kx) {
          const unsigned so = yv[ky] && xv[kx] ? base + (unsigned)c * sc + (unsigned)ky * sy + (unsigned)kx * sx : FAR;
          a[(c * KF + ky) * KF + kx] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r_img, (int)lane_off, (int)so, 0));
        }
  }
#pragma unroll
  for (int it = 0; it < PER; ++it)
    if (tid + it * 256 < KMAX * 64) w_lds[tid + it * 256] = w[it];
  __syncthreads();
  if (!live) return;

  const unsigned fstride = (unsigned)p.N * (unsigned)p.M * 4u;          // bytes between filters in the output
  // register r of lane (li, half): filter 8*((r%16)/4) + 4*half + r%4 of the block, image 32*(r/16) + li
  const unsigned out_lane = ((unsigned)(nb * 64 + li) + (unsigned)p.N * (unsigned)m) * 4u + (unsigned)(4 * half) * fstride;
  f32x32 acc[FB];
  // filters are read RB - 1 taps ahead of their MFMA
  constexpr int RB = 6;
  auto run_block = [&](int fb, const f32x32* prev, int prev_fb) __attribute__((always_inline)) {
    const float* wl = w_lds + fb * 32 + li;
    float wq[RB];
#pragma unroll
    for (int i = 0; i < RB - 1; ++i) wq[i] = wl[i * 64];
    f32x32 c;
#pragma unroll
    for (int v = 0; v < 32; ++v) c[v] = 0.f;
#pragma unroll
    for (int k = 0; k < KMAX; ++k) {
      if (k < K) {
        if (k + RB - 1 < KMAX) wq[(k + RB - 1) % RB] = wl[(k + RB - 1) * 64];
        c = __builtin_amdgcn_mfma_f32_32x32x1f32(wq[k % RB], a[k], c, 0, 0, 0);
        // the previous block's outputs leave under these MFMAs, one store per tap
        if (prev && k < 32) {
          const float val = (*prev)[k];
          const int f_in_block = 8 * ((k & 15) >> 2) + (k & 3);
          const bool ok = prev_fb * 32 + f_in_block < p.Fg;   // (wave-uniform: filters per group are a multiple of 8, so lanes 32-63, four filters on, agree)
          const unsigned so = ok ? (unsigned)(g * p.Fg + prev_fb * 32 + f_in_block) * fstride + (unsigned)(k >> 4) * 128u : FAR;
          __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(val), r_out, (int)out_lane, (int)so, ST_NT);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    acc[fb] = c;
  };
  run_block(0, nullptr, 0);
  if (FB == 2) run_block(1, &acc[0], 0);
  // the last block's outputs
  {
    constexpr int last = FB - 1;
#pragma unroll
    for (int r = 0; r < 32; ++r) {
      const float val = acc[last][r];
      const int f_in_block = 8 * ((r & 15) >> 2) + (r & 3);
      const bool ok = last * 32 + f_in_block < p.Fg;
      const unsigned so = ok ? (unsigned)(g * p.Fg + last * 32 + f_in_block) * fstride + (unsigned)(r >> 4) * 128u : FAR;
      __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(val), r_out, (int)out_lane, (int)so, ST_NT);
    }
  }
  // (K < 32 taps: the first block's outputs that did not leave under the second block's MFMAs)
  if (FB == 2 && K < 32) {
#pragma unroll
    for (int r = 0; r < 32; ++r)
      if (r >= K) {
        const float val = acc[0][r];
        const int f_in_block = 8 * ((r & 15) >> 2) + (r & 3);
        const bool ok = f_in_block < p.Fg;
        const unsigned so = ok ? (unsigned)(g * p.Fg + f_in_block) * fstride + (unsigned)(r >> 4) * 128u : FAR;
        __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(val), r_out, (int)out_lane, (int)so, ST_NT);
      }
  }
}

static bool fast_ok(const ConvArgs& a) {
  // (the gathers use 32-bit byte offsets that include a margin for the padding / tap shift)
  const long long margin = (long long)a.N * ((long long)(a.k + (a.pad0 < 0 ? -a.pad0 : 0)) * (a.H + a.Mx) + a.k + a.H);
  return a.N % 16 == 0 && a.Fg % 16 == 0 && dn_aligned16(a.img) && dn_aligned16(a.flt) && dn_aligned16(a.hid) &&
         (long long)a.N * a.M * a.F + margin < (1ll << 30) && (long long)a.N * a.HH * a.C + margin < (1ll << 30);
}

static void fill_common(ConvArgs& a, int N, int C, int G, int H, int F, int k, int Mx, int s, int pad0) {
  a.N = N; a.C = C; a.G = G; a.Cg = C / G; a.H = H; a.F = F; a.Fg = F / G; a.k = k; a.Mx = Mx; a.s = s; a.pad0 = pad0;
  a.M = Mx * Mx; a.HH = H * H; a.kk2 = k * k;
  a.m_begin = 0; a.m_count = a.M; a.chunks = 1; a.splits = 1; a.slabs_per_split = 0; a.split_stride = 0; a.local = 0;
  a.scale_t = 0.f; a.scale_o = 1.f; a.partial = nullptr; a.a_bytes = 0; a.b_bytes = 0;
  a.dN = make_fastdiv((uint32_t)N); a.dMx = make_fastdiv((uint32_t)Mx);
  a.dk = make_fastdiv((uint32_t)k); a.dkk2 = make_fastdiv((uint32_t)(k * k));
  a.dS = make_fastdiv((uint32_t)s); a.dSS = make_fastdiv((uint32_t)(s * s)); a.yq = 0;
}

// Byte sizes of the two gathered arrays for the buffer-load kernels; 0 when one of them
// is too large for 32-bit buffer offsets (twice the size must not wrap).
static void set_buffer_ranges(ConvArgs& a, long long a_elems, long long b_elems) {
  const bool fits = a_elems * 4 < (1ll << 31) && b_elems * 4 < (1ll << 31);
  a.a_bytes = fits ? (unsigned)(a_elems * 4) : 0u;
  a.b_bytes = fits ? (unsigned)(b_elems * 4) : 0u;
}

// out = sum of the `splits` partial outputs of a convUp / convDown whose reduction was split.
__global__ void __launch_bounds__(256) k_conv_sum_splits(const float* partial, int splits, long long total4, float* out) {
  const long long stride = (long long)gridDim.x * 256;
  for (long long e = (long long)blockIdx.x * 256 + threadIdx.x; e < total4; e += stride) {
    float4 s = reinterpret_cast<const float4*>(partial)[e];
    for (int z = 1; z < splits; ++z) {
      const float4 v = reinterpret_cast<const float4*>(partial)[(long long)z * total4 + e];
      s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
    reinterpret_cast<float4*>(out)[e] = s;
  }
}

template <int MODE, bool LOCAL = false>
static void launch_rowmajor_tiles(const ConvArgs& a, long long rows, int cols, int gz);
template <int MODE, bool LOCAL = false>
static void launch_uniform_rows(const ConvArgs& a, long long rows, int cols, int gz);
template <int MODE>
static void launch_general_rows(const ConvArgs& a, long long rows, int cols, int gz);

// Layers on small maps (8 x 8, 16 x 16 modules at batch 128) have fewer tiles than the chip
// has CUs, and a lone workgroup per CU walks its reduction at the pace of the memory
// latency: split the reduction over up to 16 workgroups per tile (at least 8 slabs each)
// and sum the partial outputs with a second kernel.  (32 -> 64 filters of 5 x 5 on 8 x 8
// maps: convUp 51 -> 17 us.)
template <int MODE, bool LOCAL = false>
static void launch_rowmajor(const ConvArgs& a0, long long rows, int cols, int gz) {
  ConvArgs a = a0;
  const int cus = dn_num_cus();
  const long long tiles = (rows + 127) / 128 * (cols <= 96 ? 1 : (cols + 127) / 128) * gz;
  const int nslabs = MODE == CONV_UP ? (a.Cg * a.kk2 + CV_BK - 1) / CV_BK : a.kk2 * (a.Fg / CV_BK);
  const long long total = MODE == CONV_UP ? (long long)a.N * a.M * a.F : (long long)a.N * a.HH * a.C;
  long long want = 1;
  // (the sum of the partial outputs writes 16-byte groups)
  if ((MODE == CONV_UP || (MODE == CONV_DOWN && a.s == 1)) && a.scale_t == 0.f && a.scale_o == 1.f && dn_aligned16(a.out)) {
    if (tiles < cus && (2 * tiles < cus || nslabs < 40)) {
      want = (2ll * cus) / tiles;
      if (want > nslabs / 8) want = nslabs / 8;
      if (want > 16) want = 16;
    } else if (nslabs >= 40 && 10 * tiles <= (MODE == CONV_UP ? 25ll : 13ll) * cus) {
      // Long reductions on about one tile per CU: a lone workgroup per CU leaves every wait of its
      // slab loop exposed, so the reduction is cut until three to four workgroups share a CU, each
      // keeping at least 20 slabs (measured on 64 -> 64 colours of 5 x 5, batch 128: 16 x 16 maps
      // Up 98 -> 79 us and Down 74 -> 65 us, 18 x 18 maps Up 146 -> 96 us and Down 109 -> 89 us, 12 x 12
      // maps Up 61 -> 53 us; convDown stops gaining at 1.3 tiles per CU, convUp at 2.5; short
      // reductions lose to the extra pass over the output: 32 colours of 3 x 3, 22 -> 30 us)
      const long long target = (MODE == CONV_UP ? 4ll : 3ll) * cus;
      want = (target + tiles / 2) / tiles;
      if (want > 8) want = 8;
      while (want > 1 && nslabs / want < 20) --want;
    }
    if (want < 1) want = 1;
  }
  if (want > 1) {
    a.slabs_per_split = (int)((nslabs + want - 1) / want);
    a.splits = (nslabs + a.slabs_per_split - 1) / a.slabs_per_split;
  }
  if (a.splits > 1) {
    a.partial = (float*)dn_scratch((size_t)a.splits * total * sizeof(float));
    if (!a.partial) { a.splits = 1; a.slabs_per_split = 0; }
    else a.split_stride = total;
  }
  launch_rowmajor_tiles<MODE, LOCAL>(a, rows, cols, gz * a.splits);
  if (a.splits > 1) {
    const long long total4 = total / 4;            // (the batch is a multiple of 16)
    long long blocks = (total4 + 255) / 256;
    if (blocks > 8ll * cus) blocks = 8ll * cus;
    hipLaunchKernelGGL(k_conv_sum_splits, dim3((unsigned)blocks), dim3(256), 0, dn_stream(), (const float*)a.partial, a.splits, total4,
                       a.out);
  }
}

template <int MODE, bool LOCAL>
static void launch_rowmajor_tiles(const ConvArgs& a, long long rows, int cols, int gz) {
  if constexpr (LOCAL) {   // (the caller has checked what the uniform-row kernels need)
    launch_uniform_rows<MODE, true>(a, rows, cols, gz);
    return;
  }
  // Batches that are multiples of 128: tiles of 128 rows never straddle a module / pixel.
  // Measured on the benchmark layers: the buffer-load kernels win for long reductions
  // with up to 64 or more than 96 columns; 65-96 columns and short reductions are
  // faster on the 256-row tiles below.
  const int nslabs = MODE == CONV_UP ? (a.Cg * a.kk2 + CV_BK - 1) / CV_BK : a.kk2 * (a.Fg / CV_BK) / (a.s * a.s);
  if (a.N % 128 == 0 && a.a_bytes != 0 && a.b_bytes != 0 && nslabs >= 16 && (cols <= 64 || cols > 96)) {
    launch_uniform_rows<MODE>(a, rows, cols, gz);
    return;
  }
  launch_general_rows<MODE>(a, rows, cols, gz);
}

// The uniform-row kernels (batch a multiple of 128, both operands within 32-bit buffer ranges).
template <int MODE, bool LOCAL>
static void launch_uniform_rows(const ConvArgs& a, long long rows, int cols, int gz) {
  {
    const unsigned gx = (unsigned)(rows / 128);
    // (column counts that leave a 32-wide block half empty take 16-wide blocks)
    if (cols <= 16) hipLaunchKernelGGL((k_conv_mfma<MODE, 4, 1, 1, true, 1, false, LOCAL>), dim3(gx, 1, gz), dim3(256), 0, dn_stream(), a);
    else if (cols <= 32) hipLaunchKernelGGL((k_conv_mfma<MODE, 4, 1, 1, true, 0, false, LOCAL>), dim3(gx, (cols + 31) / 32, gz), dim3(256), 0, dn_stream(), a);
    else if (cols <= 48) hipLaunchKernelGGL((k_conv_mfma<MODE, 4, 1, 2, true, 3, false, LOCAL>), dim3(gx, 1, gz), dim3(256), 0, dn_stream(), a);
    else if (cols <= 64) hipLaunchKernelGGL((k_conv_mfma<MODE, 4, 1, 2, true, 0, false, LOCAL>), dim3(gx, (cols + 63) / 64, gz), dim3(256), 0, dn_stream(), a);
    else {
      // More than 96 columns: 128-wide tiles (64 x 64 per wavefront) or 64-wide ones (32 x 64).
      // What decides is how full the column tiles are and how evenly the tiles spread over the
      // CUs; at equal fill the wide tile is the faster one for convUp (the image gather is
      // repeated per column tile: measured rate 0.82 of the wide tile's), for convDown neither.
      // (384 filters in 2 groups on 13 x 13 maps: Up 449 -> 288 us, Down 330 -> 221 us.)
      const int cus = dn_num_cus();
      auto spread = [&](long long t) { return (double)t / (double)(((t + cus - 1) / cus) * cus); };
      const int c128 = (cols + 127) / 128, c64 = (cols + 63) / 64;
      const double s128 = (double)cols / (128.0 * c128) * spread((long long)gx * c128 * gz);
      const double s64 = (double)cols / (64.0 * c64) * spread((long long)gx * c64 * gz) * (MODE == CONV_UP ? 0.82 : 1.0);
      if (s64 > s128) hipLaunchKernelGGL((k_conv_mfma<MODE, 4, 1, 2, true, 0, false, LOCAL>), dim3(gx, c64, gz), dim3(256), 0, dn_stream(), a);
      else hipLaunchKernelGGL((k_conv_mfma<MODE, 2, 2, 2, true, 0, false, LOCAL>), dim3(gx, c128, gz), dim3(256), 0, dn_stream(), a);
    }
  }
}

template <int MODE>
static void launch_general_rows(const ConvArgs& a, long long rows, int cols, int gz) {
  // Up / Down: rows are plentiful, columns few: 4 wavefronts down the rows, WN blocks across.
  // With enough rows to keep every CU busy twice over, each wavefront takes two row
  // blocks (256-row tiles): twice the MFMAs per LDS read and per barrier.
  const long long tiles256 = (rows + 255) / 256 * ((cols + 127) / 128) * gz;
  if (tiles256 >= 2 * dn_num_cus() && cols <= 96) {  // (2 x 4 blocks per wavefront would leave one wavefront per SIMD)
    const unsigned gx = (unsigned)((rows + 255) / 256);
    if constexpr (MODE == CONV_UP) {
      if (a.pad0 == 0 && (a.Mx - 1) * a.s + a.k <= a.H && rows % 256 == 0) {  // nothing to mask in the image gather
        if (cols <= 32) hipLaunchKernelGGL((k_conv_mfma<MODE, 4, 2, 1, false, 0, true>), dim3(gx, (cols + 31) / 32, gz), dim3(256), 0, dn_stream(), a);
        else if (cols <= 64) hipLaunchKernelGGL((k_conv_mfma<MODE, 4, 2, 2, false, 0, true>), dim3(gx, (cols + 63) / 64, gz), dim3(256), 0, dn_stream(), a);
        else hipLaunchKernelGGL((k_conv_mfma<MODE, 4, 2, 3, false, 0, true>), dim3(gx, (cols + 95) / 96, gz), dim3(256), 0, dn_stream(), a);
        return;
      }
    }
    if (cols <= 32) hipLaunchKernelGGL((k_conv_mfma<MODE, 4, 2, 1>), dim3(gx, (cols + 31) / 32, gz), dim3(256), 0, dn_stream(), a);
    else if (cols <= 64) hipLaunchKernelGGL((k_conv_mfma<MODE, 4, 2, 2>), dim3(gx, (cols + 63) / 64, gz), dim3(256), 0, dn_stream(), a);
    else hipLaunchKernelGGL((k_conv_mfma<MODE, 4, 2, 3>), dim3(gx, (cols + 95) / 96, gz), dim3(256), 0, dn_stream(), a);
    return;
  }
  const unsigned gx = (unsigned)((rows + 127) / 128);
  if (cols <= 32) hipLaunchKernelGGL((k_conv_mfma<MODE, 4, 1, 1>), dim3(gx, (cols + 31) / 32, gz), dim3(256), 0, dn_stream(), a);
  else if (cols <= 64) hipLaunchKernelGGL((k_conv_mfma<MODE, 4, 1, 2>), dim3(gx, (cols + 63) / 64, gz), dim3(256), 0, dn_stream(), a);
  else if (cols <= 96) hipLaunchKernelGGL((k_conv_mfma<MODE, 4, 1, 3>), dim3(gx, (cols + 95) / 96, gz), dim3(256), 0, dn_stream(), a);
  else hipLaunchKernelGGL((k_conv_mfma<MODE, 2, 2, 2>), dim3(gx, (cols + 127) / 128, gz), dim3(256), 0, dn_stream(), a);  // 64 x 64 per wavefront
}

static void conv_up_impl(cudamat* images, cudamat* filters, cudamat* targets, int numModulesX, int paddingStart,
                         int moduleStride, int numImgColors, int numGroups, const char* where, bool local = false) {
  conv_clear_error();
  CONV_REQUIRE(images->on_device && filters->on_device && targets->on_device, where);
  CONV_REQUIRE(numGroups >= 1 && numImgColors > 0 && numImgColors % numGroups == 0, where);
  CONV_REQUIRE(moduleStride >= 1 && numModulesX >= 1, where);
  const int N = images->size[0], F = filters->size[0];
  CONV_REQUIRE(N > 0 && F > 0 && F % numGroups == 0, where);
  CONV_REQUIRE(images->size[1] % numImgColors == 0, where);
  const int H = isqrt_exact(images->size[1] / numImgColors);
  CONV_REQUIRE(H > 0, where);
  const int Cg = numImgColors / numGroups;
  const int M = numModulesX * numModulesX;
  const int fmm = local ? M : 1;  // filter banks
  CONV_REQUIRE(filters->size[1] % (Cg * fmm) == 0, where);
  const int k = isqrt_exact(filters->size[1] / (Cg * fmm));
  CONV_REQUIRE(k > 0, where);
  CONV_REQUIRE(paddingStart <= 0, where);
  CONV_REQUIRE(moduleStride <= k, where);
  CONV_REQUIRE(targets->size[0] == N && targets->size[1] == F * M, where);
  ConvArgs a;
  fill_common(a, N, numImgColors, numGroups, H, F, k, numModulesX, moduleStride, paddingStart);
  a.img = images->data_device; a.flt = filters->data_device; a.hid = nullptr; a.out = targets->data_device;
  a.local = local ? 1 : 0;
  set_buffer_ranges(a, (long long)N * numImgColors * H * H, (long long)F * filters->size[1]);
  const int K = a.Cg * a.kk2;
  if (!local && fast_ok(a) && K <= 80 && a.Fg <= 64 && N % 32 == 0 && a.a_bytes != 0 && a.b_bytes != 0 &&
      (long long)N * M * F * 4 < (1ll << 31)) {  // (32-bit offsets into the output, and an out-of-range offset beyond it)
    if (N % 64 == 0 && (k == 3 || k == 5) && (a.Cg == 1 || a.Cg == 3)) {
      // one (module, 64 images) tile per wavefront, two wavefronts per SIMD
      const long long tiles64 = (long long)M * (N / 64);
      const dim3 grid64((unsigned)((tiles64 + 3) / 4), 1, numGroups);
#define UP_TAPS(CG, KF) do { if (a.Fg <= 32) hipLaunchKernelGGL((k_conv_up_taps<1, CG, KF>), grid64, dim3(256), 0, dn_stream(), a); \
                             else hipLaunchKernelGGL((k_conv_up_taps<2, CG, KF>), grid64, dim3(256), 0, dn_stream(), a); } while (0)
      if (a.Cg == 3 && k == 5) UP_TAPS(3, 5); else if (a.Cg == 3) UP_TAPS(3, 3); else if (k == 5) UP_TAPS(1, 5); else UP_TAPS(1, 3);
#undef UP_TAPS
      if (dn_launch_status()) conv_set_error(where, hipGetErrorString(hipGetLastError()));
      return;
    }
    // short reduction, few filters per group: filter bank in registers
    const long long tiles = (long long)M * (N / 32);
    long long blocks = (tiles + 3) / 4;
    if (blocks > dn_num_cus()) blocks = dn_num_cus();  // one wavefront per SIMD, looping over tiles
    const dim3 grid((unsigned)blocks, 1, numGroups);
    a.dS = make_fastdiv((uint32_t)(N / 32));  // tile -> (module, image block)
    a.dSS = make_fastdiv((uint32_t)(blocks * 4)); // wavefronts of a group
    if (K <= 32) {
      if (a.Fg <= 32) hipLaunchKernelGGL((k_conv_up_regs<16, 1>), grid, dim3(256), 0, dn_stream(), a);
      else hipLaunchKernelGGL((k_conv_up_regs<16, 2>), grid, dim3(256), 0, dn_stream(), a);
    } else {
      // (33 to 64 filters as two blocks of 32 along grid y -- half the registers, two workgroups
      // per CU -- measured the same 19.4 us on the 3 -> 64 filters of 5 x 5 layer, and gathers the
      // images twice: one block of 64 it stays)
      if (a.Fg <= 32) hipLaunchKernelGGL((k_conv_up_regs<40, 1>), grid, dim3(256), 0, dn_stream(), a);
      else hipLaunchKernelGGL((k_conv_up_regs<40, 2>), grid, dim3(256), 0, dn_stream(), a);
    }
  } else if (!local && fast_ok(a)) {
    launch_rowmajor<CONV_UP>(a, (long long)M * N, a.Fg, numGroups);
  } else if (local && fast_ok(a) && N % 128 == 0 && a.a_bytes != 0 && a.b_bytes != 0) {
    // locally connected: a 128-row tile is one module, so the uniform-row kernels only add that
    // module's bank to the filter offset
    launch_rowmajor<CONV_UP, true>(a, (long long)M * N, a.Fg, numGroups);
  } else {
    const long long total = (long long)N * M * F;
    long long blocks = (total + 255) / 256;
    if (blocks > dn_num_cus() * 16ll) blocks = dn_num_cus() * 16ll;
    hipLaunchKernelGGL(k_conv_up_direct, dim3((unsigned)blocks), dim3(256), 0, dn_stream(), a);
  }
  if (dn_launch_status()) conv_set_error(where, hipGetErrorString(hipGetLastError()));
}

static void conv_down_impl(cudamat* hidActs, cudamat* filters, cudamat* targets, int imgSize, int paddingStart,
                           int moduleStride, int numImgColors, int numGroups, const char* where, bool local = false) {
  conv_clear_error();
  CONV_REQUIRE(hidActs->on_device && filters->on_device && targets->on_device, where);
  CONV_REQUIRE(numGroups >= 1 && numImgColors > 0 && numImgColors % numGroups == 0, where);
  CONV_REQUIRE(moduleStride >= 1 && imgSize >= 1, where);
  const int N = hidActs->size[0], F = filters->size[0];
  CONV_REQUIRE(N > 0 && F > 0 && F % numGroups == 0, where);
  CONV_REQUIRE(hidActs->size[1] % F == 0, where);
  const int M = hidActs->size[1] / F;
  const int Mx = isqrt_exact(M);
  CONV_REQUIRE(Mx > 0, where);
  const int Cg = numImgColors / numGroups;
  const int fmm = local ? M : 1;
  CONV_REQUIRE(filters->size[1] % (Cg * fmm) == 0, where);
  const int k = isqrt_exact(filters->size[1] / (Cg * fmm));
  CONV_REQUIRE(k > 0, where);
  CONV_REQUIRE(paddingStart <= 0 && moduleStride <= k, where);
  CONV_REQUIRE(targets->size[0] == N && targets->size[1] == numImgColors * imgSize * imgSize, where);
  ConvArgs a;
  fill_common(a, N, numImgColors, numGroups, imgSize, F, k, Mx, moduleStride, paddingStart);
  a.img = nullptr; a.flt = filters->data_device; a.hid = hidActs->data_device; a.out = targets->data_device;
  a.img = a.hid;  // alignment test only
  a.local = local ? 1 : 0;
  set_buffer_ranges(a, (long long)N * M * F, (long long)F * filters->size[1]);
  const bool local_uni = local && fast_ok(a) && dn_aligned16(a.out) && N % 128 == 0 && a.a_bytes != 0 && a.b_bytes != 0;
  if ((!local || local_uni) && fast_ok(a) && dn_aligned16(a.out) && a.Cg <= 16 && moduleStride > 1 && N % 128 == 0 &&
      a.a_bytes != 0 && a.b_bytes != 0) {
    // few colours, strided: the stride^2 pixel phases become columns of one implicit GEMM
    const int padw = paddingStart < 0 ? -paddingStart : 0;
    a.yq = (imgSize - 1 + padw) / moduleStride + 1;
    const int cols = a.Cg * moduleStride * moduleStride;
    const unsigned gx = (unsigned)((long long)a.yq * a.yq * N / 128);
    // column counts that leave a 32-wide block half empty take 16-wide blocks
    if (local) {
      if (cols <= 16) hipLaunchKernelGGL((k_conv_mfma<CONV_DOWNM, 4, 1, 1, true, 1, false, true>), dim3(gx, 1, numGroups), dim3(256), 0, dn_stream(), a);
      else if (cols <= 32) hipLaunchKernelGGL((k_conv_mfma<CONV_DOWNM, 4, 1, 1, true, 0, false, true>), dim3(gx, 1, numGroups), dim3(256), 0, dn_stream(), a);
      else if (cols <= 48) hipLaunchKernelGGL((k_conv_mfma<CONV_DOWNM, 4, 1, 2, true, 3, false, true>), dim3(gx, 1, numGroups), dim3(256), 0, dn_stream(), a);
      else if (cols <= 64) hipLaunchKernelGGL((k_conv_mfma<CONV_DOWNM, 4, 1, 2, true, 0, false, true>), dim3(gx, 1, numGroups), dim3(256), 0, dn_stream(), a);
      else if (cols <= 96) hipLaunchKernelGGL((k_conv_mfma<CONV_DOWNM, 4, 1, 3, true, 0, false, true>), dim3(gx, 1, numGroups), dim3(256), 0, dn_stream(), a);
      else hipLaunchKernelGGL((k_conv_mfma<CONV_DOWNM, 2, 2, 2, true, 0, false, true>), dim3(gx, (cols + 127) / 128, numGroups), dim3(256), 0, dn_stream(), a);
    } else {
      if (cols <= 16) hipLaunchKernelGGL((k_conv_mfma<CONV_DOWNM, 4, 1, 1, true, 1>), dim3(gx, 1, numGroups), dim3(256), 0, dn_stream(), a);
      else if (cols <= 32) hipLaunchKernelGGL((k_conv_mfma<CONV_DOWNM, 4, 1, 1, true>), dim3(gx, 1, numGroups), dim3(256), 0, dn_stream(), a);
      else if (cols <= 48) hipLaunchKernelGGL((k_conv_mfma<CONV_DOWNM, 4, 1, 2, true, 3>), dim3(gx, 1, numGroups), dim3(256), 0, dn_stream(), a);
      else if (cols <= 64) hipLaunchKernelGGL((k_conv_mfma<CONV_DOWNM, 4, 1, 2, true>), dim3(gx, 1, numGroups), dim3(256), 0, dn_stream(), a);
      else if (cols <= 96) hipLaunchKernelGGL((k_conv_mfma<CONV_DOWNM, 4, 1, 3, true>), dim3(gx, 1, numGroups), dim3(256), 0, dn_stream(), a);
      else hipLaunchKernelGGL((k_conv_mfma<CONV_DOWNM, 2, 2, 2, true>), dim3(gx, (cols + 127) / 128, numGroups), dim3(256), 0, dn_stream(), a);
    }
  } else if (!local && moduleStride == 1 && a.Cg <= 4 && (k == 3 || k == 5) && N % 32 == 0 && a.Fg % 8 == 0 &&
             a.Fg <= 128 && a.a_bytes != 0 && a.a_bytes <= 0x20000000u && a.b_bytes != 0 && a.b_bytes <= 0x20000000u &&
             (long long)N * a.HH * numImgColors * 4 < (1ll << 31)) {
    // at most four colours, stride 1: pixels accumulate in registers on 4 x 4 x 1 matrix-core blocks
    const int tiles_x = (imgSize + 3) / 4;
    const dim3 grid((unsigned)(tiles_x * tiles_x * (N / 32)), 1, numGroups);
#define DOWN_PX(KF, FS) hipLaunchKernelGGL((k_conv_down_px<KF, FS, 4>), grid, dim3(256), 0, dn_stream(), a)
    if (a.Fg <= 64) { if (k == 3) DOWN_PX(3, 64); else DOWN_PX(5, 64); }
    else { if (k == 3) DOWN_PX(3, 128); else DOWN_PX(5, 128); }
#undef DOWN_PX
  } else if (!local && fast_ok(a) && dn_aligned16(a.out) && a.Cg <= 16) {
    // few colours: patch-matrix form
    const long long prow = (long long)a.M * N;
    const int pcols = a.Cg * a.kk2, pcols8 = (pcols + 7) & ~7;
    float* P = (float*)dn_scratch((size_t)prow * pcols8 * sizeof(float), 1);
    if (!P) { conv_set_error(where, "out of device memory for the patch matrix"); return; }
    // short reductions over the filters: the register-resident product
    // (offsets are 32-bit: 96 columns of P, and the up to 64 filter rows the kernel asks for, must fit)
    const bool regs = a.Fg <= 64 && pcols <= 96 && prow % 32 == 0 && prow * 96 * 4 < (1ll << 31) &&
                      (long long)F * pcols * 4 < (1ll << 31);
    for (int g = 0; g < numGroups; ++g) {
      const float* hid_g = a.hid + (size_t)g * a.Fg * prow;
      const float* flt_g = a.flt + (size_t)g * a.Fg;
      if (regs) {
        long long blocks = (prow / 32 + 3) / 4;
        if (blocks > dn_num_cus()) blocks = dn_num_cus();  // one wavefront per SIMD, looping over tiles
        const dim3 grid((unsigned)blocks);
#define PATCH_REGS(KS, CT) hipLaunchKernelGGL((k_conv_patch_regs<KS, CT>), grid, dim3(256), 0, dn_stream(), hid_g, flt_g, P, (int)prow, a.Fg, F, pcols, pcols8)
        if (a.Fg <= 32) { if (pcols <= 32) PATCH_REGS(16, 1); else if (pcols <= 64) PATCH_REGS(16, 2); else PATCH_REGS(16, 3); }
        else { if (pcols <= 32) PATCH_REGS(32, 1); else if (pcols <= 64) PATCH_REGS(32, 2); else PATCH_REGS(32, 3); }
#undef PATCH_REGS
      } else if (dn_gemm(false, false, (int)prow, pcols, a.Fg, 1.f, hid_g, (int)prow, flt_g, F, 0.f, P, (int)prow)) {
        conv_set_error(where, "patch product failed");
        return;
      }
      const long long lanes = (long long)(N / 4) * a.HH * a.Cg;
      long long blocks = (lanes + 255) / 256;
      if (blocks > dn_num_cus() * 64ll) blocks = dn_num_cus() * 64ll;
      if (a.s == 1 && a.k == 3) hipLaunchKernelGGL((k_conv_down_gather_s1<3>), dim3((unsigned)blocks), dim3(256), 0, dn_stream(), a, (const float*)P, g);
      else if (a.s == 1 && a.k == 5) hipLaunchKernelGGL((k_conv_down_gather_s1<5>), dim3((unsigned)blocks), dim3(256), 0, dn_stream(), a, (const float*)P, g);
      else if (a.s == 1 && a.k == 7) hipLaunchKernelGGL((k_conv_down_gather_s1<7>), dim3((unsigned)blocks), dim3(256), 0, dn_stream(), a, (const float*)P, g);
      else hipLaunchKernelGGL(k_conv_down_gather, dim3((unsigned)blocks), dim3(256), 0, dn_stream(), a, (const float*)P, g);
    }
  } else if (!local && fast_ok(a) && dn_aligned16(a.out)) {
    const int q = (imgSize + moduleStride - 1) / moduleStride;
    launch_rowmajor<CONV_DOWN>(a, (long long)q * q * N, a.Cg, numGroups * moduleStride * moduleStride);
  } else if (local_uni) {
    // locally connected: a 128-row tile is one pixel; every slab adds the bank of the module its tap reaches
    const int q = (imgSize + moduleStride - 1) / moduleStride;
    launch_rowmajor<CONV_DOWN, true>(a, (long long)q * q * N, a.Cg, numGroups * moduleStride * moduleStride);
  } else {
    const long long total = (long long)N * a.HH * numImgColors;
    long long blocks = (total + 255) / 256;
    if (blocks > dn_num_cus() * 16ll) blocks = dn_num_cus() * 16ll;
    hipLaunchKernelGGL(k_conv_down_direct, dim3((unsigned)blocks), dim3(256), 0, dn_stream(), a);
  }
  if (dn_launch_status()) conv_set_error(where, hipGetErrorString(hipGetLastError()));
}

// Two chunks in flight per wavefront: with three or four, more of the first requests of the whole
// chip queue up in front of the first multiplication (measured 19.8 us against 21.3 on 128 images
// of 32 x 32 x 3 and 64 filters of 5 x 5).
#define OUTP_D 2
template <int RB>
static void launch_outp_regs_row(int cb, dim3 grid, const ConvArgs& a) {
  switch (cb) {
    case 1: hipLaunchKernelGGL((k_conv_outp_regs<RB, 1, OUTP_D>), grid, dim3(256), 0, dn_stream(), a); break;
    case 2: hipLaunchKernelGGL((k_conv_outp_regs<RB, 2, OUTP_D>), grid, dim3(256), 0, dn_stream(), a); break;
    case 3: hipLaunchKernelGGL((k_conv_outp_regs<RB, 3, OUTP_D>), grid, dim3(256), 0, dn_stream(), a); break;
    case 4: hipLaunchKernelGGL((k_conv_outp_regs<RB, 4, OUTP_D>), grid, dim3(256), 0, dn_stream(), a); break;
    default: hipLaunchKernelGGL((k_conv_outp_regs<RB, 5, OUTP_D>), grid, dim3(256), 0, dn_stream(), a); break;
  }
}
static void launch_outp_regs(int rb, int cb, dim3 grid, const ConvArgs& a) {
  switch (rb) {
    case 1: launch_outp_regs_row<1>(cb, grid, a); break;
    case 2: launch_outp_regs_row<2>(cb, grid, a); break;
    case 3: launch_outp_regs_row<3>(cb, grid, a); break;
    default: launch_outp_regs_row<4>(cb, grid, a); break;
  }
}

static void conv_outp_impl(cudamat* images, cudamat* hidActs, cudamat* targets, int numModulesX, int filterSize,
                           int paddingStart, int moduleStride, int numImgColors, int numGroups, int partialSum,
                           const char* where) {
  conv_clear_error();
  CONV_REQUIRE(images->on_device && hidActs->on_device && targets->on_device, where);
  CONV_REQUIRE(numGroups >= 1 && numImgColors > 0 && numImgColors % numGroups == 0, where);
  CONV_REQUIRE(moduleStride >= 1 && numModulesX >= 1 && filterSize >= 1, where);
  const int N = images->size[0];
  CONV_REQUIRE(N > 0 && hidActs->size[0] == N, where);
  CONV_REQUIRE(images->size[1] % numImgColors == 0, where);
  const int H = isqrt_exact(images->size[1] / numImgColors);
  CONV_REQUIRE(H > 0, where);
  const int M = numModulesX * numModulesX;
  CONV_REQUIRE(hidActs->size[1] % M == 0, where);
  const int F = hidActs->size[1] / M;
  CONV_REQUIRE(F > 0 && F % numGroups == 0, where);
  if (partialSum == 0) partialSum = M;
  CONV_REQUIRE(partialSum > 0 && M % partialSum == 0, where);
  CONV_REQUIRE(paddingStart <= 0 && moduleStride <= filterSize, where);
  const int Cg = numImgColors / numGroups;
  const int chunks = M / partialSum;
  CONV_REQUIRE(targets->size[0] == F && targets->size[1] == chunks * Cg * filterSize * filterSize, where);
  ConvArgs a;
  fill_common(a, N, numImgColors, numGroups, H, F, filterSize, numModulesX, moduleStride, paddingStart);
  a.img = images->data_device; a.hid = hidActs->data_device; a.flt = a.img;
  const int cols = Cg * a.kk2;
  const bool fast = fast_ok(a);
  // Several chunks (partial sums over groups of modules; one module each for a locally connected
  // layer): all of them in one launch of the general kernel, the chunk along grid z
  const bool batched = fast && chunks > 1 && (long long)chunks * numGroups <= 32767;   // (grid z: chunks x groups x splits)
  for (int ch = 0; ch < (batched ? 1 : chunks); ++ch) {
    a.m_begin = ch * partialSum; a.m_count = partialSum;
    a.chunks = batched ? chunks : 1;
    a.out = targets->data_device + (size_t)ch * cols * F;
    const bool few = fast && !batched && a.Fg <= 64 && cols <= 96 &&
                     (long long)N * numImgColors * H * H * 4 < (1ll << 31) && (long long)N * M * F * 4 < (1ll << 31);
    const bool small = few && N % 64 == 0;
    if (few && cols <= 80 && N % 16 == 0) {
      // operands straight into registers as 16 x 16 blocks: a wavefront owns a run of (module, 16 images) chunks
      // With an even number of filter blocks a workgroup takes half of them over twice the chunks:
      // half as many partial blocks to write and to sum (20.7 -> 19.8 us on the shape above; a
      // quarter of the filters per workgroup asks the vector caches for too many loads: 27 us)
      const int total_chunks = a.m_count * (N / 16);
      const int rb_all = (a.Fg + 15) / 16;
      const int ys = (rb_all % 2 == 0 && total_chunks >= 8 * dn_num_cus()) ? 2 : 1;
      const int cus = dn_num_cus() / ys;
      int nblocks = (total_chunks + 3) / 4 < cus ? (total_chunks + 3) / 4 : cus;
      a.slabs_per_split = (total_chunks + 4 * nblocks - 1) / (4 * nblocks);
      nblocks = (total_chunks + 4 * a.slabs_per_split - 1) / (4 * a.slabs_per_split);
      a.splits = nblocks;
      a.a_bytes = (unsigned)((long long)N * numImgColors * H * H * 4);
      a.b_bytes = (unsigned)((long long)N * M * F * 4);
      a.partial = (float*)dn_scratch((size_t)a.splits * F * cols * sizeof(float));
      if (!a.partial) { conv_set_error(where, "out of device memory for the split-K workspace"); return; }
      const dim3 grid((unsigned)nblocks, (unsigned)ys, numGroups);
      const int rb = rb_all / ys, cb = (cols + 15) / 16;
      launch_outp_regs(rb, cb, grid, a);
      const int total = F * cols;
      if (a.splits >= 64) hipLaunchKernelGGL(k_conv_outp_finish_wide, dim3((total + 63) / 64), dim3(1024), 0, dn_stream(), a);
      else if (a.splits < 16) hipLaunchKernelGGL(k_conv_outp_finish_few, dim3((total + 255) / 256), dim3(256), 0, dn_stream(), a);
      else hipLaunchKernelGGL(k_conv_outp_finish, dim3((total + 15) / 16), dim3(256), 0, dn_stream(), a);
    } else if (small) {
      // few filters and few patch columns: every wavefront holds the whole output block
      int nblocks = a.m_count < dn_num_cus() ? a.m_count : dn_num_cus();
      a.splits = nblocks;
      a.a_bytes = (unsigned)((long long)N * numImgColors * H * H * 4);
      a.b_bytes = (unsigned)((long long)N * M * F * 4);
      a.partial = (float*)dn_scratch((size_t)a.splits * F * cols * sizeof(float));
      if (!a.partial) { conv_set_error(where, "out of device memory for the split-K workspace"); return; }
      const dim3 grid((unsigned)nblocks, 1, numGroups);
      const int rt = a.Fg <= 32 ? 1 : 2, ct = cols <= 32 ? 1 : cols <= 64 ? 2 : 3;
#define OUTP_SMALL(RT, CT) hipLaunchKernelGGL((k_conv_outp_small<RT, CT>), grid, dim3(256), 0, dn_stream(), a)
      if (rt == 1) { if (ct == 1) OUTP_SMALL(1, 1); else if (ct == 2) OUTP_SMALL(1, 2); else OUTP_SMALL(1, 3); }
      else { if (ct == 1) OUTP_SMALL(2, 1); else if (ct == 2) OUTP_SMALL(2, 2); else OUTP_SMALL(2, 3); }
#undef OUTP_SMALL
      const int total = F * cols;
      if (a.splits >= 64) hipLaunchKernelGGL(k_conv_outp_finish_wide, dim3((total + 63) / 64), dim3(1024), 0, dn_stream(), a);
      else if (a.splits < 16) hipLaunchKernelGGL(k_conv_outp_finish_few, dim3((total + 255) / 256), dim3(256), 0, dn_stream(), a);
      else hipLaunchKernelGGL(k_conv_outp_finish, dim3((total + 15) / 16), dim3(256), 0, dn_stream(), a);
    } else if (fast) {
      // rows = filters of a group: pick the tile height that wastes least.
      const int Fg = a.Fg;
      int BMs = Fg <= 32 ? 32 : Fg <= 64 ? 64 : Fg <= 96 ? 96 : 128;
      if (Fg > 128 && (Fg + 95) / 96 * 96 < (Fg + 127) / 128 * 128) BMs = 96;   // e.g. 192 filters: 2 x 96, not 2 x 128
      const int gx = (Fg + BMs - 1) / BMs, gy = (cols + 127) / 128;
      const int nslabs = a.m_count * (N / CV_BK);
      // about two workgroups per CU (measured against one and three), at least 16 slabs (256 of the reduction) per split
      long long want = (2ll * dn_num_cus()) / ((long long)gx * gy * numGroups * a.chunks);
      if (want < 1) want = 1;
      if (want > nslabs / 16) want = nslabs / 16 > 0 ? nslabs / 16 : 1;
      if (want > 512) want = 512;
      a.slabs_per_split = (int)((nslabs + want - 1) / want);
      a.splits = (nslabs + a.slabs_per_split - 1) / a.slabs_per_split;
      CONV_REQUIRE((long long)numGroups * a.splits * a.chunks <= 65535, where);
      a.partial = (float*)dn_scratch((size_t)a.chunks * a.splits * F * cols * sizeof(float));
      if (!a.partial) { conv_set_error(where, "out of device memory for the split-K workspace"); return; }
      dim3 grid(gx, gy, numGroups * a.splits * a.chunks);
      if (paddingStart == 0 && (numModulesX - 1) * moduleStride + filterSize <= H) {  // nothing to mask in the image gather
        if (BMs == 32) hipLaunchKernelGGL((k_conv_mfma<CONV_OUTP, 1, 1, 1, false, 0, true>), grid, dim3(256), 0, dn_stream(), a);
        else if (BMs == 64) hipLaunchKernelGGL((k_conv_mfma<CONV_OUTP, 1, 2, 1, false, 0, true>), grid, dim3(256), 0, dn_stream(), a);
        else if (BMs == 96) hipLaunchKernelGGL((k_conv_mfma<CONV_OUTP, 1, 3, 1, false, 0, true>), grid, dim3(256), 0, dn_stream(), a);
        else hipLaunchKernelGGL((k_conv_mfma<CONV_OUTP, 2, 2, 2, false, 0, true>), grid, dim3(256), 0, dn_stream(), a);
      }
      else if (BMs == 32) hipLaunchKernelGGL((k_conv_mfma<CONV_OUTP, 1, 1, 1>), grid, dim3(256), 0, dn_stream(), a);
      else if (BMs == 64) hipLaunchKernelGGL((k_conv_mfma<CONV_OUTP, 1, 2, 1>), grid, dim3(256), 0, dn_stream(), a);
      else if (BMs == 96) hipLaunchKernelGGL((k_conv_mfma<CONV_OUTP, 1, 3, 1>), grid, dim3(256), 0, dn_stream(), a);
      else hipLaunchKernelGGL((k_conv_mfma<CONV_OUTP, 2, 2, 2>), grid, dim3(256), 0, dn_stream(), a);
      const int total = F * cols;
      if (a.splits < 16) hipLaunchKernelGGL(k_conv_outp_finish_few, dim3((total + 255) / 256, a.chunks), dim3(256), 0, dn_stream(), a);
      else hipLaunchKernelGGL(k_conv_outp_finish, dim3((total + 15) / 16, a.chunks), dim3(256), 0, dn_stream(), a);
    } else {
      hipLaunchKernelGGL(k_conv_outp_direct, dim3((unsigned)(F * cols)), dim3(256), 0, dn_stream(), a);
    }
  }
  if (dn_launch_status()) conv_set_error(where, hipGetErrorString(hipGetLastError()));
}

extern "C" {

const char* conv_last_error(void) { return g_conv_failed ? g_conv_err : nullptr; }

// Batches that are not a multiple of 16 images (deepnet's own examples train with 100): the
// matrix-core kernels need whole groups of images, so the batch-indexed operands are copied into
// a workspace with the batch rounded up (to a multiple of 128 when that costs at most 30 %
// more images, which also admits the uniform-row and register kernels; else of 32), the pad
// images zero, the pass runs on the copies, and a batch-indexed result is copied back.  Zero
// images add nothing to a weight gradient and their outputs are dropped, so results are the
// padded pass's exactly.  (64 -> 64 filters of 5 x 5 on 13 x 13 maps at batch 100: convUp
// 977 us on the one-lane-per-output kernel.)
static int padded_batch(int N) {
  if (N <= 16 || N % 16 == 0) return N;
  const int n128 = (N + 127) / 128 * 128;
  return (n128 - N) * 10 <= 3 * N ? n128 : (N + 31) / 32 * 32;
}

// dst (Np x cols) = src (N x cols) with zero rows N .. Np-1, or back (rows 0 .. N-1 only).
// One lane per group of four rows when VEC (both batch sizes are then multiples of 4); the
// column of a group comes from one multiply-high.
__global__ void __launch_bounds__(256) k_pad_batch(const float* src, float* dst, int N, int Np, unsigned total, FastDiv drows, int unpad,
                                                   int VEC) {
  const int W = VEC ? 4 : 1;
  const unsigned rows = drows.d;                     // row groups per column of the array being written
  for (unsigned e = blockIdx.x * 256u + threadIdx.x; e < total; e += gridDim.x * 256u) {
    const unsigned c = fd_div(e, drows);
    const unsigned r = (e - c * rows) * W;
    const float* s = src + (size_t)c * (unpad ? Np : N) + r;
    float* d = dst + (size_t)c * (unpad ? N : Np) + r;
    if (VEC) {
      const float4 v = (unpad || (int)r < N) ? *reinterpret_cast<const float4*>(s) : make_float4(0.f, 0.f, 0.f, 0.f);
      *reinterpret_cast<float4*>(d) = v;
    } else {
      *d = (unpad || (int)r < N) ? *s : 0.f;
    }
  }
}

static void pad_batch(const float* src, float* dst, int N, int Np, long long cols, bool unpad) {
  const bool vec = N % 4 == 0 && dn_aligned16(src) && dn_aligned16(dst);
  const int rows = (unpad ? N : Np) / (vec ? 4 : 1);
  const long long total = (long long)rows * cols;
  if (total <= 0) return;
  long long blocks = (total + 255) / 256;
  if (blocks > 16ll * dn_num_cus()) blocks = 16ll * dn_num_cus();
  const FastDiv fd = make_fastdiv((uint32_t)rows);
  hipLaunchKernelGGL(k_pad_batch, dim3((unsigned)blocks), dim3(256), 0, dn_stream(), src, dst, N, Np, (unsigned)total, fd, unpad ? 1 : 0,
                     vec ? 1 : 0);
}

// Padded stand-ins for up to three batch-indexed matrices in one workspace; null where the batch
// needs no padding or the workspace cannot be had (then the pass runs as it is).
struct PaddedBatch {
  cudamat m[3];
  int N, Np;
  bool on;
  // to128: round every batch of at least 32 images up to a multiple of 128 (locally connected
  // layers, whose matrix-core kernels need that)
  PaddedBatch(cudamat* a, cudamat* b, cudamat* c, bool to128 = false)
      : N(a->size[0]), Np(to128 && a->size[0] >= 32 ? (a->size[0] + 127) / 128 * 128 : padded_batch(a->size[0])), on(false) {
    cudamat* src[3] = {a, b, c};
    if (Np == N || !a->on_device || (b && (!b->on_device || b->size[0] != N)) || (c && (!c->on_device || c->size[0] != N))) return;
    size_t elems = 0;
    for (cudamat* x : src) if (x) elems += ((size_t)Np * x->size[1] + 3) / 4 * 4;
    // the copy kernel indexes with 32 bits: larger operands run unpadded
    for (cudamat* x : src) if (x && (long long)Np * x->size[1] >= (1ll << 32)) return;
    float* ws = (float*)dn_scratch(elems * sizeof(float), 2);
    if (!ws) return;
    for (int i = 0; i < 3; ++i) {
      if (!src[i]) continue;
      m[i] = *src[i];
      m[i].data_device = ws;
      m[i].size[0] = Np;
      m[i].owns_data = 0;
      ws += ((size_t)Np * src[i]->size[1] + 3) / 4 * 4;
    }
    on = true;
  }
  void fill(int i, const cudamat* from) { pad_batch(from->data_device, m[i].data_device, N, Np, from->size[1], false); }
  void drain(int i, cudamat* to) { pad_batch(m[i].data_device, to->data_device, N, Np, to->size[1], true); }
};

// Filter counts that are not a multiple of 16 (20 or 50 filters of a LeNet-like net), one group:
// the same remedy along the filter index.  Zero filters are appended to the filter bank, the
// hidden activations get zero maps for them (their columns come last in the (image, filter *
// modules) layout, so that is one contiguous copy and a zero tail), and the pass runs on the
// copies; the extra outputs of convUp and the extra rows of a weight gradient are dropped.
// (20 -> 50 filters of 5 x 5 at batch 128: convOutp 390 us on the one-lane-per-output kernel.)
static int padded_filters(int F, int numGroups) {
  return numGroups == 1 && F > 0 && F % 16 != 0 ? (F + 15) / 16 * 16 : F;
}

// Filter-major arrays (f + F*q): dst (Fp x Q) = src (F x Q) with zero rows F .. Fp-1, or back.
__global__ void __launch_bounds__(256) k_pad_filters(const float* src, float* dst, int F, int Fp, long long Q, int unpad) {
  const int rows = unpad ? F : Fp;
  const long long total = (long long)rows * Q;
  const long long stride = (long long)gridDim.x * 256;
  for (long long e = (long long)blockIdx.x * 256 + threadIdx.x; e < total; e += stride) {
    const long long q = e / rows;
    const int f = (int)(e - q * rows);
    if (unpad) dst[q * F + f] = src[q * Fp + f];
    else dst[e] = f < F ? src[q * F + f] : 0.f;
  }
}
// dst[0 .. n_total) = src[0 .. n_copy) followed by zeros.
__global__ void __launch_bounds__(256) k_copy_prefix(const float* src, float* dst, long long n_copy, long long n_total) {
  const long long stride = (long long)gridDim.x * 256;
  for (long long e = (long long)blockIdx.x * 256 + threadIdx.x; e < n_total; e += stride) dst[e] = e < n_copy ? src[e] : 0.f;
}
static unsigned pad_grid(long long total) {
  long long blocks = (total + 255) / 256;
  if (blocks > 16ll * dn_num_cus()) blocks = 16ll * dn_num_cus();
  return (unsigned)(blocks < 1 ? 1 : blocks);
}
// A stand-in of `rows x cols` floats for `like` at `*ws`, which is moved past it (16-byte steps).
static cudamat pad_standin(const cudamat* like, int rows, long long cols, float** ws) {
  cudamat m = *like;
  m.data_device = *ws;
  m.size[0] = rows; m.size[1] = (int)cols;
  m.owns_data = 0;
  *ws += ((size_t)rows * cols + 3) / 4 * 4;
  return m;
}

static void conv_up_filters(cudamat* images, cudamat* filters, cudamat* targets, int numModulesX, int paddingStart,
                            int moduleStride, int numImgColors, int numGroups) {
  const int F = filters->size[0], Fp = padded_filters(F, numGroups), N = images->size[0];
  const long long Q = filters->size[1], M = (long long)numModulesX * numModulesX;
  float* ws = nullptr;
  if (Fp != F && images->on_device && filters->on_device && targets->on_device && targets->size[0] == N &&
      targets->size[1] == F * M && (long long)N * Fp * M < (1ll << 31) && Fp * Q < (1ll << 31))
    ws = (float*)dn_scratch((((size_t)Fp * Q + 3) / 4 * 4 + ((size_t)N * Fp * M + 3) / 4 * 4) * sizeof(float), 3);
  if (!ws) {
    conv_up_impl(images, filters, targets, numModulesX, paddingStart, moduleStride, numImgColors, numGroups, "convUp");
    return;
  }
  cudamat fp = pad_standin(filters, Fp, Q, &ws), tp = pad_standin(targets, N, Fp * M, &ws);
  hipLaunchKernelGGL(k_pad_filters, dim3(pad_grid(Fp * Q)), dim3(256), 0, dn_stream(), (const float*)filters->data_device, fp.data_device, F, Fp, Q, 0);
  conv_up_impl(images, &fp, &tp, numModulesX, paddingStart, moduleStride, numImgColors, numGroups, "convUp");
  if (!conv_last_error())
    hipLaunchKernelGGL(k_copy_prefix, dim3(pad_grid((long long)N * F * M)), dim3(256), 0, dn_stream(), (const float*)tp.data_device,
                       targets->data_device, (long long)N * F * M, (long long)N * F * M);
}

static void conv_down_filters(cudamat* hidActs, cudamat* filters, cudamat* targets, int imgSize, int paddingStart,
                              int moduleStride, int numImgColors, int numGroups) {
  const int F = filters->size[0], Fp = padded_filters(F, numGroups), N = hidActs->size[0];
  const long long Q = filters->size[1];
  float* ws = nullptr;
  if (Fp != F && hidActs->on_device && filters->on_device && targets->on_device && hidActs->size[1] % F == 0 &&
      (long long)N * (hidActs->size[1] / F) * Fp < (1ll << 31) && Fp * Q < (1ll << 31))
    ws = (float*)dn_scratch((((size_t)Fp * Q + 3) / 4 * 4 + ((size_t)N * (hidActs->size[1] / F) * Fp + 3) / 4 * 4) * sizeof(float), 3);
  if (!ws) {
    conv_down_impl(hidActs, filters, targets, imgSize, paddingStart, moduleStride, numImgColors, numGroups, "convDown");
    return;
  }
  const long long M = hidActs->size[1] / F;
  cudamat fp = pad_standin(filters, Fp, Q, &ws), hp = pad_standin(hidActs, N, Fp * M, &ws);
  hipLaunchKernelGGL(k_pad_filters, dim3(pad_grid(Fp * Q)), dim3(256), 0, dn_stream(), (const float*)filters->data_device, fp.data_device, F, Fp, Q, 0);
  hipLaunchKernelGGL(k_copy_prefix, dim3(pad_grid((long long)N * Fp * M)), dim3(256), 0, dn_stream(), (const float*)hidActs->data_device,
                     hp.data_device, (long long)N * F * M, (long long)N * Fp * M);
  conv_down_impl(&hp, &fp, targets, imgSize, paddingStart, moduleStride, numImgColors, numGroups, "convDown");
}

static void conv_outp_filters(cudamat* images, cudamat* hidActs, cudamat* targets, int numModulesX, int filterSize,
                              int paddingStart, int moduleStride, int numImgColors, int numGroups, int partialSum) {
  const long long M = (long long)numModulesX * numModulesX;
  const int N = images->size[0];
  const int F = M > 0 && hidActs->size[1] % M == 0 ? (int)(hidActs->size[1] / M) : 0;
  const int Fp = padded_filters(F, numGroups);
  const long long Q = targets->size[1];
  float* ws = nullptr;
  if (Fp != F && images->on_device && hidActs->on_device && targets->on_device && hidActs->size[0] == N &&
      targets->size[0] == F && (long long)N * Fp * M < (1ll << 31) && Fp * Q < (1ll << 31))
    ws = (float*)dn_scratch((((size_t)Fp * Q + 3) / 4 * 4 + ((size_t)N * Fp * M + 3) / 4 * 4) * sizeof(float), 3);
  if (!ws) {
    conv_outp_impl(images, hidActs, targets, numModulesX, filterSize, paddingStart, moduleStride, numImgColors, numGroups,
                   partialSum, "convOutp");
    return;
  }
  cudamat tp = pad_standin(targets, Fp, Q, &ws), hp = pad_standin(hidActs, N, Fp * M, &ws);
  hipLaunchKernelGGL(k_copy_prefix, dim3(pad_grid((long long)N * Fp * M)), dim3(256), 0, dn_stream(), (const float*)hidActs->data_device,
                     hp.data_device, (long long)N * F * M, (long long)N * Fp * M);
  conv_outp_impl(images, &hp, &tp, numModulesX, filterSize, paddingStart, moduleStride, numImgColors, numGroups, partialSum,
                 "convOutp");
  if (!conv_last_error())
    hipLaunchKernelGGL(k_pad_filters, dim3(pad_grid((long long)F * Q)), dim3(256), 0, dn_stream(), (const float*)tp.data_device,
                       targets->data_device, F, Fp, Q, 1);
}

void convUp(cudamat* images, cudamat* filters, cudamat* targets, int numModulesX, int paddingStart, int moduleStride,
            int numImgColors, int numGroups) {
  PaddedBatch pb(images, targets, nullptr);
  if (pb.on) {
    pb.fill(0, images);
    conv_up_filters(&pb.m[0], filters, &pb.m[1], numModulesX, paddingStart, moduleStride, numImgColors, numGroups);
    if (!conv_last_error()) pb.drain(1, targets);
    return;
  }
  conv_up_filters(images, filters, targets, numModulesX, paddingStart, moduleStride, numImgColors, numGroups);
}

void convDown(cudamat* hidActs, cudamat* filters, cudamat* targets, int imgSize, int paddingStart, int moduleStride,
              int numImgColors, int numGroups) {
  PaddedBatch pb(hidActs, targets, nullptr);
  if (pb.on) {
    pb.fill(0, hidActs);
    conv_down_filters(&pb.m[0], filters, &pb.m[1], imgSize, paddingStart, moduleStride, numImgColors, numGroups);
    if (!conv_last_error()) pb.drain(1, targets);
    return;
  }
  conv_down_filters(hidActs, filters, targets, imgSize, paddingStart, moduleStride, numImgColors, numGroups);
}

void convOutp(cudamat* images, cudamat* hidActs, cudamat* targets, int numModulesX, int filterSize, int paddingStart,
              int moduleStride, int numImgColors, int numGroups, int partialSum) {
  PaddedBatch pb(images, hidActs, nullptr);
  if (pb.on) {
    pb.fill(0, images);
    pb.fill(1, hidActs);
    conv_outp_filters(&pb.m[0], &pb.m[1], targets, numModulesX, filterSize, paddingStart, moduleStride, numImgColors,
                      numGroups, partialSum);
    return;
  }
  conv_outp_filters(images, hidActs, targets, numModulesX, filterSize, paddingStart, moduleStride, numImgColors, numGroups,
                    partialSum);
}

// Locally connected layers: one filter bank per module, filters laid out
// (module, colour, ky, kx, filter) (cudamat_conv_kernels.cuh:66-67).  Batches that are a
// multiple of 128 run on the uniform-row matrix-core kernels, which add a module's bank to
// the filter offset (the reference switches its conv kernels the same way, with a template
// flag, cudamat_conv.cu:1415-1420); other batches are padded up to one when that is cheap,
// else take the one-lane-per-output kernels.  The weight gradient is convOutp with one
// module per chunk, which is how the reference computes it too (cudamat_conv.cu:1421-1423).
void localUp(cudamat* images, cudamat* filters, cudamat* targets, int numModulesX, int paddingStart, int moduleStride,
             int numImgColors, int numGroups) {
  PaddedBatch pb(images, targets, nullptr, true);
  if (pb.on) {
    pb.fill(0, images);
    conv_up_impl(&pb.m[0], filters, &pb.m[1], numModulesX, paddingStart, moduleStride, numImgColors, numGroups, "localUp",
                 true);
    if (!conv_last_error()) pb.drain(1, targets);
    return;
  }
  conv_up_impl(images, filters, targets, numModulesX, paddingStart, moduleStride, numImgColors, numGroups, "localUp",
               true);
}
void localDown(cudamat* hidActs, cudamat* filters, cudamat* targets, int imgSize, int paddingStart, int moduleStride,
               int numImgColors, int numGroups) {
  PaddedBatch pb(hidActs, targets, nullptr, true);
  if (pb.on) {
    pb.fill(0, hidActs);
    conv_down_impl(&pb.m[0], filters, &pb.m[1], imgSize, paddingStart, moduleStride, numImgColors, numGroups, "localDown",
                   true);
    if (!conv_last_error()) pb.drain(1, targets);
    return;
  }
  conv_down_impl(hidActs, filters, targets, imgSize, paddingStart, moduleStride, numImgColors, numGroups, "localDown",
                 true);
}
void localOutp(cudamat* images, cudamat* hidActs, cudamat* targets, int numModulesX, int filterSize, int paddingStart,
               int moduleStride, int numImgColors, int numGroups, int partialSum) {
  (void)partialSum;
  conv_outp_impl(images, hidActs, targets, numModulesX, filterSize, paddingStart, moduleStride, numImgColors,
                 numGroups, 1, "localOutp");
}

}  // extern "C"
