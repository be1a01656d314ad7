// Shared host/device helpers for the gfx950 matrix backend.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/cudamat_amd.h"

#define WAVE 64

// One CU count for launch sizing; MI355X has 256 CUs in 8 XCDs.  Queried once.
int dn_num_cus();

// hipMalloc that releases the library's cache of freed matrix blocks and retries when the device is full.
hipError_t dn_malloc(void** p, size_t bytes);

// Grow-only device workspaces (slot 0: partials and scalar results; slot 1: conv patch matrix).
void* dn_scratch(size_t bytes, int slot = 0);

// n 32-bit words that are zero between kernels (arrival counters); null when they cannot be had.
unsigned* dn_zero_words(int n);
// f is called when the last executable graph that this library made has been freed.
void dn_set_no_graphs_hook(void (*f)());

// Looks up (once per device) the fixed workspace of the entry points that allocate nothing.
int dn_noalloc_setup();

// The stream every kernel of the library is queued on: the NULL stream, or the stream a
// caller is capturing into a HIP graph (graph_capture_begin .. graph_capture_end).  Launches a
// held-back product first (dn_flush), so that work is queued in call order.
hipStream_t dn_stream();
// Deferred epilogues: dot() may hold its launch back (dn_defer_dot) so that the add_col_vec /
// activation / sample calls that follow it run in the product's epilogue; dn_flush() launches what
// is held back.  Called by everything that queues work, hands out workspaces, moves data or waits.
void dn_flush();
void dn_set_pending(bool on);
void dn_set_flush_hook(void (*f)());
void dn_set_ext_flush_hook(void (*f)());   // the conv library's held-back calls
void dn_set_ext_pending(bool on);
void dn_flush_ext();
bool dn_defer_enabled();                    // set_deferred_epilogues()
void dn_refresh_pending();                  // recomputes whether anything is held back
bool dn_softmax_held();                     // a softmax that waits for its loss and gradient (reduce.hip)
void dn_softmax_flush();
bool dn_defer_dot(cudamat* mat1, cudamat* mat2, cudamat* target, float beta, float alpha, int m, int n, int k, int* err);
bool dn_pending_sample(rnd_struct* rnd, cudamat* mat, cudamat* target, int* err);
// Sums along the rows, y = beta*y + alpha*rowsums(M) (M is h x w, leading dimension h), may be held back too
// and launched together (dn_row_sum_jobs), and a product into C may wait for a second one into the same C
// (dn_gemm_pair_sums, together with the sums; a product that stays alone takes the sums along where its kernel
// can, dn_gemm_sums); each with the bits of the separate launches.
// fill_with_rand may be held back as well: greater_than_scalar(mask, p) and mult_elementwise(state, mask)
// that follow it spell a dropout mask (deepnet/neuralnet.py:194-198) and run as one pass (dn_rng_dropmask).
bool dn_defer_fill_rand(rnd_struct* rnd, cudamat* mat, int* err);
int dn_rng_dropmask(rnd_struct* rnd, float* mask, float* state, size_t n, float p);
// ... and less_than(mask, probs, target = probs) behind it a Bernoulli sample that keeps its uniforms (dn_rng_bernoulli_keep).
int dn_rng_bernoulli_keep(rnd_struct* rnd, float* uni, float* probs, size_t n);
struct DnRowSumJob { const float* M; float* y; int h, w; float alpha, beta; int scalar; };   // scalar: dn_row_sum_job_kind() == 2
bool dn_defer_row_sum(const float* M, float* y, int h, int w, float alpha, float beta, int* err);
bool dn_row_sum_job_ok(const float* M, int h, int w);     // kind 1
int dn_row_sum_job_kind(const float* M, int h, int w);    // 0: not as a job, 1: 16-byte loads of four rows, 2: one row per lane
int dn_row_sum_jobs(const DnRowSumJob* jobs, int n);
int dn_gemm(bool a_trans, bool b_trans, int M, int N, int K, float alpha, const float* A, int lda, const float* B, int ldb,
            float beta, float* C, int ldc);
int dn_gemm_sums(bool a_trans, bool b_trans, int M, int N, int K, float alpha, const float* A, int lda, const float* B, int ldb,
                 float beta, float* C, int ldc, const DnRowSumJob* jobs, int njobs);
int dn_gemm_pair_sums(bool a_trans, bool b_trans, int M, int N, int K, float alpha, const float* A, int lda, const float* B,
                      int ldb, float beta, float alpha2, const float* A2, int lda2, const float* B2, int ldb2, float* C, int ldc,
                      const DnRowSumJob* jobs, int njobs);
bool dn_capturing();

// Records the launch status of the kernel just queued; returns CUDA_ERROR or 0.
static inline int dn_launch_status() {
  return hipPeekAtLastError() == hipSuccess ? 0 : CUDA_ERROR;
}

static inline bool dn_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

static inline long long dn_len(const cudamat* m) { return (long long)m->size[0] * (long long)m->size[1]; }

// Division of a 32-bit index by a run-time constant without the hardware-less
// integer divide: q = (n * magic) >> 32 >> shift for n < 2^31.
struct FastDiv {
  uint32_t magic;
  uint32_t sh1, sh2;   // min(ceil(log2 d), 1) and max(ceil(log2 d) - 1, 0)
  uint32_t d;
};

static inline FastDiv make_fastdiv(uint32_t d) {
  FastDiv f;
  f.d = d;
  if (d == 0) d = 1;
  uint32_t s = 0;
  while ((1ull << s) < d) ++s;            // s = ceil(log2 d)
  uint64_t m = ((1ull << 32) * ((1ull << s) - d)) / d + 1;
  f.magic = (uint32_t)m;
  f.sh1 = s < 1 ? s : 1;
  f.sh2 = s > 1 ? s - 1 : 0;
  return f;
}

// Exact for every 32-bit n and every divisor, without a branch
// (round-up method: q = (hi + ((n - hi) >> sh1)) >> sh2; d = 1 gives magic 1, no shifts).
__device__ __forceinline__ uint32_t fd_div(uint32_t n, const FastDiv& f) {
  const uint32_t hi = __umulhi(n, f.magic);
  return (hi + ((n - hi) >> f.sh1)) >> f.sh2;
}

// Wave-wide reductions through cross-lane shuffles (wave64).
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, WAVE));
  return v;
}
__device__ __forceinline__ double wave_sum_d(double v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
  return v;
}

// 16-byte global accesses.  STREAM marks data that is touched once (large
// operands): non-temporal loads and stores keep it from displacing the caches
// and measure about 12% faster on 64 MiB operands than plain ones.
typedef float dn_v4f __attribute__((ext_vector_type(4)));
template <bool STREAM>
__device__ __forceinline__ float4 dn_ld4(const float* p) {
  if (STREAM) {
    const dn_v4f v = __builtin_nontemporal_load(reinterpret_cast<const dn_v4f*>(p));
    return make_float4(v.x, v.y, v.z, v.w);
  }
  return *reinterpret_cast<const float4*>(p);
}
template <bool STREAM>
__device__ __forceinline__ void dn_st4(float* p, float4 r) {
  if (STREAM) {
    const dn_v4f v = {r.x, r.y, r.z, r.w};
    __builtin_nontemporal_store(v, reinterpret_cast<dn_v4f*>(p));
  } else {
    *reinterpret_cast<float4*>(p) = r;
  }
}
// Run-time selected variants (the flag is uniform across the launch).
__device__ __forceinline__ float4 dn_ld4_rt(const float* p, bool stream) {
  return stream ? dn_ld4<true>(p) : dn_ld4<false>(p);
}
__device__ __forceinline__ void dn_st4_rt(float* p, float4 r, bool stream) {
  if (stream) dn_st4<true>(p, r); else dn_st4<false>(p, r);
}
__device__ __forceinline__ float dn_ld1_rt(const float* p, bool stream) {
  return stream ? __builtin_nontemporal_load(p) : *p;
}
__device__ __forceinline__ void dn_st1_rt(float* p, float v, bool stream) {
  if (stream) __builtin_nontemporal_store(v, p); else *p = v;
}
// Operands of at least this many elements are streamed.
#define DN_STREAM_MIN_ELEMS (1ll << 22)
