// Column gather / scatter by float-encoded indices, block replication, image
// translation crops, expansion and per-label column accumulation.
// Replaces cudamat/cudamat.cu:2120-2189, 2295-2321, 2348-2399 and the kernels
// cudamat_kernels.cu:720-817, 1090-1121.
//
// Every kernel walks columns with the lanes running down the rows, so both the
// gathered and the scattered side move in contiguous runs.  Indices that fall
// outside the matrix give NaN on a gather and are skipped on a scatter (the
// reference writes through them).
#include "common.h"
#include <math.h>

__device__ __forceinline__ int wrap_index(float f, int n) {
  int i = (int)f;
  if (i < 0) i += n;
  return (i < 0 || i >= n) ? -1 : i;
}

// W consecutive rows of a column per lane: 1, or 4 as one 16-byte access (row counts that are
// multiples of 4, aligned operands: 4096 x 4096 select_columns 53 -> 27 us).
template <int W>
__device__ __forceinline__ void rows_ld(const float* p, float (&v)[W]) {
  if constexpr (W == 4) { const float4 t = *reinterpret_cast<const float4*>(p); v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w; }
  else v[0] = *p;
}
template <int W>
__device__ __forceinline__ void rows_st(float* p, const float (&v)[W]) {
  if constexpr (W == 4) *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  else *p = v[0];
}

// target(:, c) = source(:, idx[c])
template <int W>
__global__ void k_select_cols(const float* source, float* target, const float* indices, int n_idx, int h, int src_w) {
  const int r = (blockIdx.x * blockDim.x + threadIdx.x) * W;
  if (r >= h) return;
  for (int c = blockIdx.y; c < n_idx; c += gridDim.y) {
    const int s = wrap_index(indices[c], src_w);
    float v[W];
    if (s < 0) { for (int k = 0; k < W; ++k) v[k] = NAN; }
    else rows_ld<W>(source + (size_t)s * h + r, v);
    rows_st<W>(target + (size_t)c * h + r, v);
  }
}

// target(:, idx[c]) = source(:, c)
template <int W>
__global__ void k_set_selected_cols(float* target, const float* source, const float* indices, int n_idx, int h,
                                    int tgt_w) {
  const int r = (blockIdx.x * blockDim.x + threadIdx.x) * W;
  if (r >= h) return;
  for (int c = blockIdx.y; c < n_idx; c += gridDim.y) {
    const int t = wrap_index(indices[c], tgt_w);
    if (t < 0) continue;
    float v[W];
    rows_ld<W>(source + (size_t)c * h + r, v);
    rows_st<W>(target + (size_t)t * h + r, v);
  }
}

// swap source(:, idx1[c]) with target(:, idx2[c])
template <int W>
__global__ void k_swap_cols(float* source, float* target, const float* idx1, const float* idx2, int cols, int src_w,
                            int tgt_w, int h) {
  const int r = (blockIdx.x * blockDim.x + threadIdx.x) * W;
  if (r >= h) return;
  for (int c = blockIdx.y; c < cols; c += gridDim.y) {
    const int s = (int)idx1[c], t = (int)idx2[c];
    if (s < 0 || s >= src_w || t < 0 || t >= tgt_w) continue;
    const size_t ps = (size_t)s * h + r, pt = (size_t)t * h + r;
    float a[W], b[W];
    rows_ld<W>(source + ps, a);
    rows_ld<W>(target + pt, b);
    rows_st<W>(source + ps, b);
    rows_st<W>(target + pt, a);
  }
}

// Within each column, every run of `blocksize` rows takes the value of its first row.
__global__ void k_blockify(const float* source, float* target, int numdims, int blocksize, FastDiv fd) {
  const size_t off = (size_t)blockIdx.x * numdims;
  for (int i = threadIdx.x; i < numdims; i += blockDim.x) {
    const int block = (int)fd_div((uint32_t)i, fd);
    target[off + i] = source[off + (size_t)block * blocksize];
  }
}

// One column = one image of source_w x source_w pixels with num_channels
// interleaved channels; crop a target_w x target_w window shifted by
// (off_x, off_y) from the centred position.  The source pixel is addressed the way
// the reference does it (cudamat_kernels.cu:795-817): a flat pixel index
// img*S*S + (pad + off_x + tx)*S + (pad + off_y + ty), so a window that leaves the image
// on the right continues in the next pixel row, and one that leaves it at the bottom in
// the next image -- deepnet's data cache relies on nothing else, but its offsets do reach
// there (datahandler.py:350-352 adds the centring shift that the kernel adds again).
// Only an index outside the whole source matrix reads 0 instead of foreign memory.
__global__ void k_translate(const float* source, float* target, const float* off_x_arr, const float* off_y_arr,
                            int source_w, int target_w, int num_channels, long long total) {
  const int img = blockIdx.x;
  const int pad = (source_w - target_w) / 2;
  const int tts = target_w * target_w, sts = source_w * source_w;
  const int off_x = (int)off_x_arr[img], off_y = (int)off_y_arr[img];
  const long long target_off = (long long)img * tts;
  const long long source_off = (long long)img * sts + (long long)(pad + off_x) * source_w + (pad + off_y);
  const int per_img = tts * num_channels;
  for (int e = threadIdx.x; e < per_img; e += blockDim.x) {
    const int pix = e / num_channels, ch = e - pix * num_channels;
    const int tx = pix / target_w, ty = pix - tx * target_w;
    const long long src = num_channels * (source_off + (long long)tx * source_w + ty) + ch;
    target[num_channels * (target_off + pix) + ch] = (src >= 0 && src < total) ? source[src] : 0.f;
  }
}

// target(:, c) = source(:, idx[c]) for every target column, NaN when outside.
template <int W>
__global__ void k_expand(const float* source, const float* indices, float* target, int h, int w, int tw) {
  const int r = (blockIdx.x * blockDim.x + threadIdx.x) * W;
  if (r >= h) return;
  for (int c = blockIdx.y; c < tw; c += gridDim.y) {
    const int s = (int)indices[c];
    float v[W];
    if (s >= 0 && s < w) rows_ld<W>(source + (size_t)s * h + r, v);
    else { for (int k = 0; k < W; ++k) v[k] = NAN; }
    rows_st<W>(target + (size_t)c * h + r, v);
  }
}

// target(:, c) = source(:, c) + mult * mat(:, idx[c])
template <int W>
__global__ void k_expand_and_add(const float* source, const float* mat, const float* indices, float* target, int w,
                                 int h, float mult, int w2) {
  const int r = (blockIdx.x * blockDim.x + threadIdx.x) * W;
  if (r >= h) return;
  for (int c = blockIdx.y; c < w; c += gridDim.y) {
    const int s = (int)indices[c];
    const size_t p = (size_t)c * h + r;
    float v[W];
    if (s >= 0 && s < w2) {
      float x[W], y[W];
      rows_ld<W>(source + p, x);
      rows_ld<W>(mat + (size_t)s * h + r, y);
      for (int k = 0; k < W; ++k) v[k] = x[k] + mult * y[k];
    } else {
      for (int k = 0; k < W; ++k) v[k] = NAN;
    }
    rows_st<W>(target + p, v);
  }
}

// target(:, c) = mult * sum of the columns i of mat with (int)idx[i] == c, divided
// by their count when avg is set and the count is not zero.
__global__ void k_accumulate_cols(const float* mat, const float* indices, float* target, int mat_w, int tgt_w, int h,
                                  float mult, int avg) {
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= h) return;
  for (int c = blockIdx.y; c < tgt_w; c += gridDim.y) {
    float sum = 0.f;
    unsigned count = 0;
    for (int i = 0; i < mat_w; ++i) {
      if ((int)indices[i] == c) {
        ++count;
        sum += mat[(size_t)i * h + r];
      }
    }
    target[(size_t)c * h + r] = mult * sum / (float)((avg == 1 && count > 0) ? count : 1u);
  }
}

static inline dim3 col_grid(int h, int cols, int rows_per_lane = 1) {
  const int lanes = (h + rows_per_lane - 1) / rows_per_lane;
  return dim3((lanes + 255) / 256, cols < 8192 ? (cols > 0 ? cols : 1) : 8192);
}
// 16-byte accesses down the rows: every column of these matrices then starts on a 16-byte boundary
static inline bool rows4(int h, const void* a, const void* b, const void* c = nullptr) {
  return h % 4 == 0 && dn_aligned16(a) && dn_aligned16(b) && (!c || dn_aligned16(c));
}

extern "C" {

int selectRows(cudamat* source, cudamat* target, cudamat* indices) {
  const int n = indices->size[1];
  if (!source->on_device || !target->on_device || !indices->on_device) return ERROR_NOT_ON_DEVICE;
  if (target->size[0] != source->size[0] || target->size[1] < n || indices->size[0] != 1)
    return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (n == 0 || source->size[0] == 0) return 0;
  if (rows4(source->size[0], source->data_device, target->data_device))
    hipLaunchKernelGGL(k_select_cols<4>, col_grid(source->size[0], n, 4), dim3(256), 0, dn_stream(), (const float*)source->data_device,
                       target->data_device, (const float*)indices->data_device, n, source->size[0], source->size[1]);
  else
    hipLaunchKernelGGL(k_select_cols<1>, col_grid(source->size[0], n), dim3(256), 0, dn_stream(), (const float*)source->data_device,
                       target->data_device, (const float*)indices->data_device, n, source->size[0], source->size[1]);
  return dn_launch_status();
}

int setSelectedRows(cudamat* target, cudamat* source, cudamat* indices) {
  const int n = indices->size[1];
  if (!source->on_device || !target->on_device || !indices->on_device) return ERROR_NOT_ON_DEVICE;
  if (target->size[0] != source->size[0] || source->size[1] < n || indices->size[0] != 1)
    return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (n == 0 || source->size[0] == 0) return 0;
  if (rows4(source->size[0], source->data_device, target->data_device))
    hipLaunchKernelGGL(k_set_selected_cols<4>, col_grid(source->size[0], n, 4), dim3(256), 0, dn_stream(), target->data_device,
                       (const float*)source->data_device, (const float*)indices->data_device, n, target->size[0],
                       target->size[1]);
  else
    hipLaunchKernelGGL(k_set_selected_cols<1>, col_grid(source->size[0], n), dim3(256), 0, dn_stream(), target->data_device,
                       (const float*)source->data_device, (const float*)indices->data_device, n, target->size[0],
                       target->size[1]);
  return dn_launch_status();
}

int swapColumns(cudamat* source, cudamat* target, cudamat* indices1, cudamat* indices2) {
  const int cols = indices1->size[1] * indices1->size[0];
  const int h = source->size[0];
  if (!source->on_device || !target->on_device || !indices1->on_device || !indices2->on_device)
    return ERROR_NOT_ON_DEVICE;
  if (target->size[0] != h || indices2->size[0] * indices2->size[1] != cols) return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (cols == 0 || h == 0) return 0;
  if (rows4(h, source->data_device, target->data_device))
    hipLaunchKernelGGL(k_swap_cols<4>, col_grid(h, cols, 4), dim3(256), 0, dn_stream(), source->data_device, target->data_device,
                       (const float*)indices1->data_device, (const float*)indices2->data_device, cols, source->size[1],
                       target->size[1], h);
  else
    hipLaunchKernelGGL(k_swap_cols<1>, col_grid(h, cols), dim3(256), 0, dn_stream(), source->data_device, target->data_device,
                       (const float*)indices1->data_device, (const float*)indices2->data_device, cols, source->size[1],
                       target->size[1], h);
  return dn_launch_status();
}

int generate_translations_big_var_off(cudamat* source, cudamat* target, cudamat* off_x, cudamat* off_y, int source_w,
                                      int target_w, int num_channels) {
  if (!source->on_device || !target->on_device || !off_x->on_device || !off_y->on_device) return ERROR_NOT_ON_DEVICE;
  const int imgs = source->size[1];
  if (target->size[1] != imgs || source->size[0] != source_w * source_w * num_channels ||
      target->size[0] != target_w * target_w * num_channels || off_x->size[0] * off_x->size[1] < imgs ||
      off_y->size[0] * off_y->size[1] < imgs || target_w > source_w)
    return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (imgs == 0) return 0;
  hipLaunchKernelGGL(k_translate, dim3(imgs), dim3(512), 0, dn_stream(), (const float*)source->data_device, target->data_device,
                     (const float*)off_x->data_device, (const float*)off_y->data_device, source_w, target_w,
                     num_channels, (long long)imgs * source->size[0]);
  return dn_launch_status();
}

int blockify(cudamat* source, cudamat* target, int blocksize) {
  if (!source->on_device || !target->on_device) return ERROR_NOT_ON_DEVICE;
  if (source->size[0] != target->size[0] || source->size[1] != target->size[1] || blocksize <= 0)
    return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (source->size[1] == 0 || source->size[0] == 0) return 0;
  hipLaunchKernelGGL(k_blockify, dim3(source->size[1]), dim3(512), 0, dn_stream(), (const float*)source->data_device,
                     target->data_device, source->size[0], blocksize, make_fastdiv((uint32_t)blocksize));
  return dn_launch_status();
}

int accumulate_columns(cudamat* mat, cudamat* indices, cudamat* target, float mult, int avg) {
  const int h = mat->size[0], w = mat->size[1], w2 = target->size[1];
  if (!mat->on_device || !indices->on_device || !target->on_device) return ERROR_NOT_ON_DEVICE;
  if (mat->is_trans) return ERROR_TRANSPOSED;
  if (target->size[0] != h) return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (indices->size[0] != 1 || indices->size[1] != w) return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (512 < w2) return ERROR_INCOMPATIBLE_DIMENSIONS;  // the reference's one-lane-per-target-column limit
  if (h == 0 || w2 == 0) return 0;
  hipLaunchKernelGGL(k_accumulate_cols, col_grid(h, w2), dim3(256), 0, dn_stream(), (const float*)mat->data_device,
                     (const float*)indices->data_device, target->data_device, w, w2, h, mult, avg);
  return dn_launch_status();
}

int expand(cudamat* source, cudamat* indices, cudamat* target) {
  const int h = source->size[0], w = source->size[1], w2 = target->size[1];
  if (!source->on_device || !indices->on_device || !target->on_device) return ERROR_NOT_ON_DEVICE;
  if (source->is_trans) return ERROR_TRANSPOSED;
  if (target->size[0] != h) return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (indices->size[0] != 1 || indices->size[1] != w2) return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (h == 0 || w2 == 0) return 0;
  if (rows4(h, source->data_device, target->data_device))
    hipLaunchKernelGGL(k_expand<4>, col_grid(h, w2, 4), dim3(256), 0, dn_stream(), (const float*)source->data_device,
                       (const float*)indices->data_device, target->data_device, h, w, w2);
  else
    hipLaunchKernelGGL(k_expand<1>, col_grid(h, w2), dim3(256), 0, dn_stream(), (const float*)source->data_device,
                       (const float*)indices->data_device, target->data_device, h, w, w2);
  return dn_launch_status();
}

int expand_and_add(cudamat* source, cudamat* mat, cudamat* indices, cudamat* target, float mult) {
  const int h = source->size[0], w = source->size[1], w2 = mat->size[1];
  if (!source->on_device || !mat->on_device || !indices->on_device || !target->on_device) return ERROR_NOT_ON_DEVICE;
  if (mat->is_trans) return ERROR_TRANSPOSED;
  if (target->size[0] != h || target->size[1] != w) return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (indices->size[0] != 1 || indices->size[1] != w) return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (mat->size[0] != h) return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (h == 0 || w == 0) return 0;
  if (rows4(h, source->data_device, target->data_device, mat->data_device))
    hipLaunchKernelGGL(k_expand_and_add<4>, col_grid(h, w, 4), dim3(256), 0, dn_stream(), (const float*)source->data_device,
                       (const float*)mat->data_device, (const float*)indices->data_device, target->data_device, w, h,
                       mult, w2);
  else
    hipLaunchKernelGGL(k_expand_and_add<1>, col_grid(h, w), dim3(256), 0, dn_stream(), (const float*)source->data_device,
                       (const float*)mat->data_device, (const float*)indices->data_device, target->data_device, w, h,
                       mult, w2);
  return dn_launch_status();
}

}  // extern "C"
