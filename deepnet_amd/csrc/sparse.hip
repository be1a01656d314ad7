// Compressed-sparse-row matrices: the handle type, its upload and the product with a
// dense matrix.  Replaces cudamat/cudamat.cu:125-153 (allocate_device_memory_sparse),
// :188-213 (copy_sparse_to_device), :407-418 (init_from_sparse_array), :1698-1727
// (sparse_dot) and the kernel cudamat_kernels.cu:370-384 (kSparseDot).
#include "common.h"

// target(row, col) = alpha * sum_i data[i] * dense(indices[i], col) + beta * target(row, col)
// over the non-zeros i of `row`; dense is k x n and target m x n, both column-major.
// Lanes run down 64 consecutive rows (target is written in 256-byte runs, and the
// non-zeros of a row are read once for CB columns); the four wavefronts of a workgroup
// take neighbouring groups of CB columns.  Each row is summed in index order in fp32,
// as the reference kernel does.  Indices and row pointers are clamped into range so
// that a malformed matrix cannot send an access outside its arrays.
template <int CB>
__global__ void __launch_bounds__(256)
k_sparse_dot(int m, int n, int k, int nnz, const float* data, const int* indptr, const int* indices,
             const float* dense, float* target, float beta, float alpha) {
  const int row = blockIdx.x * 64 + (threadIdx.x & 63);
  const int col0 = (blockIdx.y * 4 + (threadIdx.x >> 6)) * CB;
  if (row >= m || col0 >= n) return;
  int start = indptr[row], end = indptr[row + 1];
  if (start < 0) start = 0;
  if (end > nnz) end = nnz;
  const float* col[CB];
#pragma unroll
  for (int c = 0; c < CB; ++c) col[c] = dense + (size_t)(col0 + c < n ? col0 + c : n - 1) * k;
  float acc[CB];
#pragma unroll
  for (int c = 0; c < CB; ++c) acc[c] = 0.f;
  for (int i = start; i < end; ++i) {
    const float d = data[i];
    unsigned j = (unsigned)indices[i];
    if (j >= (unsigned)k) j = (unsigned)k - 1u;
#pragma unroll
    for (int c = 0; c < CB; ++c) acc[c] += d * col[c][j];
  }
#pragma unroll
  for (int c = 0; c < CB; ++c)
    if (col0 + c < n) {
      float* t = target + (size_t)(col0 + c) * m + row;
      *t = alpha * acc[c] + (beta == 0.f ? 0.f : beta * *t);
    }
}

static void release(cudamat_sparse* mat) {
  dn_flush();
  if (mat->data_device.data) hipFree(mat->data_device.data);
  if (mat->data_device.indices) hipFree(mat->data_device.indices);
  if (mat->data_device.indptr) hipFree(mat->data_device.indptr);
  mat->data_device.data = nullptr;
  mat->data_device.indices = nullptr;
  mat->data_device.indptr = nullptr;
  mat->on_device = 0;
}

extern "C" {

void init_from_sparse_array(cudamat_sparse* mat, float* data, int* indices, int* indptr, int m, int n, int nnz) {
  mat->data_host.data = data;
  mat->data_host.indices = indices;
  mat->data_host.indptr = indptr;
  mat->data_device.data = nullptr;
  mat->data_device.indices = nullptr;
  mat->data_device.indptr = nullptr;
  mat->size[0] = m;
  mat->size[1] = n;
  mat->on_device = 0;
  mat->on_host = 1;
  mat->is_trans = 0;
  mat->owns_data = 1;
  mat->nnz = nnz;
}

int allocate_device_memory_sparse(cudamat_sparse* mat) {
  const int nnz = mat->nnz, rows = mat->size[0];
  if (nnz < 0 || rows < 0) return ERROR_INCOMPATIBLE_DIMENSIONS;
  mat->data_device.data = nullptr;
  mat->data_device.indices = nullptr;
  mat->data_device.indptr = nullptr;
  // (an empty matrix still gets distinct, valid pointers)
  const size_t vals = (size_t)(nnz > 0 ? nnz : 1);
  if (dn_malloc((void**)&mat->data_device.data, vals * sizeof(float)) != hipSuccess ||
      dn_malloc((void**)&mat->data_device.indices, vals * sizeof(int)) != hipSuccess ||
      dn_malloc((void**)&mat->data_device.indptr, ((size_t)rows + 1) * sizeof(int)) != hipSuccess) {
    hipGetLastError();
    release(mat);
    return CUBLAS_ERROR;
  }
  mat->on_device = 1;
  return 0;
}

int copy_sparse_to_device(cudamat_sparse* mat) {
  if (!mat->on_device) {
    if (int err = allocate_device_memory_sparse(mat)) return err;
  }
  const size_t nnz = (size_t)mat->nnz, rows = (size_t)mat->size[0];
  dn_flush();
  if ((nnz && hipMemcpy(mat->data_device.data, mat->data_host.data, nnz * sizeof(float), hipMemcpyHostToDevice) != hipSuccess) ||
      (nnz && hipMemcpy(mat->data_device.indices, mat->data_host.indices, nnz * sizeof(int), hipMemcpyHostToDevice) != hipSuccess) ||
      hipMemcpy(mat->data_device.indptr, mat->data_host.indptr, (rows + 1) * sizeof(int), hipMemcpyHostToDevice) != hipSuccess)
    return CUBLAS_ERROR;
  return 0;
}

int free_device_memory_sparse(cudamat_sparse* mat) {
  if (mat->owns_data && mat->on_device) release(mat);
  return 0;
}

int sparse_dot(cudamat_sparse* mat1, cudamat* mat2, cudamat* target, float beta, float alpha) {
  if (!mat1->on_device || !mat2->on_device || !target->on_device) return ERROR_NOT_ON_DEVICE;
  const int m = mat1->size[0], k = mat1->size[1], k2 = mat2->size[0], n = mat2->size[1];
  if (k != k2) return ERROR_INCOMPATIBLE_DIMENSIONS;
  // (the reference does not look at the target's shape; a smaller one would be overrun)
  if (target->size[0] != m || target->size[1] != n) return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (m <= 0 || n <= 0) return 0;
  if (k <= 0) {  // no terms: target = beta * target
    cudamat t = *target;
    t.is_trans = 0;
    return beta == 0.f ? assign_scalar(&t, 0.f) : mult_by_scalar(&t, beta, &t);
  }
  const unsigned gx = (unsigned)((m + 63) / 64);
  if (n >= 16) {
    hipLaunchKernelGGL((k_sparse_dot<4>), dim3(gx, (unsigned)((n + 15) / 16)), dim3(256), 0, dn_stream(), m, n, k, mat1->nnz,
                       (const float*)mat1->data_device.data, (const int*)mat1->data_device.indptr,
                       (const int*)mat1->data_device.indices, (const float*)mat2->data_device, target->data_device, beta,
                       alpha);
  } else {
    hipLaunchKernelGGL((k_sparse_dot<1>), dim3(gx, (unsigned)((n + 3) / 4)), dim3(256), 0, dn_stream(), m, n, k, mat1->nnz,
                       (const float*)mat1->data_device.data, (const int*)mat1->data_device.indptr,
                       (const int*)mat1->data_device.indices, (const float*)mat2->data_device, target->data_device, beta,
                       alpha);
  }
  return dn_launch_status();
}

}  // extern "C"
