// Multiply-with-carry RNG: 12288 independent streams, each a 64-bit word
// (carry << 32 | x) advanced by  word' = mult * lo32(word) + hi32(word).
// Replaces cudamat/cudamat.cu:55-83, 437-588 and cudamat_kernels.cu:96-239.
//
// Output contract (bit-exact for the integer stream and for everything that is
// a pure function of it): element i of a call is produced by stream i % 12288
// from that stream's draw number i / 12288 since the previous call, and each
// stream's word after the call is the word after its last draw.
//
// Two schedules produce that same sequence:
//   serial  - one lane per stream walks its draws in order (short calls);
//   split   - a stream's draws are cut into fixed chunks of RNG_CHUNK draws
//             dealt round-robin to RNG_SPLIT lanes; a lane reaches its next
//             chunk with one modular multiplication by a per-stream constant,
//             because one step is a multiplication by (2^32)^-1 modulo
//             m = mult * 2^32 - 1 (word' * 2^32 = m * lo + word).
#include "common.h"
#include <math.h>
#include <stdio.h>
#include <stdlib.h>

#define RNG_PI 3.1415926535897932f

__device__ __forceinline__ unsigned long long mwc_step(unsigned long long w, unsigned int mult) {
  return (unsigned long long)mult * (w & 0xffffffffull) + (w >> 32);
}

// (lo32 + 1) / 2^32 with the conversion rounded to nearest even: a value in (0, 1].
__device__ __forceinline__ float mwc_uniform(unsigned long long w) {
  return ((float)(unsigned int)(w & 0xffffffffull) + 1.0f) * 2.3283064365386963e-10f;
}

__global__ void k_seed(const unsigned int* mults, unsigned long long* words, unsigned int seed) {
  const unsigned int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= NUM_RND_STREAMS) return;
  unsigned long long w = ((unsigned long long)seed << 32) + 1ull;
  const unsigned int mult = mults[idx];
  for (int i = 0; i < NUM_RND_BURNIN; ++i) w = mwc_step(w, mult);
  words[idx] = w;
}

// ------------------------------------------------------------------ consumers
// One uniform per element.
struct OpUniform {
  float* out;
  __device__ __forceinline__ void operator()(size_t i, float u) const { out[i] = u; }
};
struct OpDropout {
  float* data;
  float p, val;
  __device__ __forceinline__ void operator()(size_t i, float u) const { data[i] = u > p ? data[i] : val; }
};
struct OpBernoulli {
  const float* in;
  float* out;
  __device__ __forceinline__ void operator()(size_t i, float u) const { out[i] = u < in[i] ? 1.f : 0.f; }
};
struct OpBernoulliTanh {
  const float* in;
  float* out;
  __device__ __forceinline__ void operator()(size_t i, float u) const {
    out[i] = (double)u < (1.0 + (double)in[i]) / 2.0 ? 1.f : 0.f;
  }
};
struct OpCopy {  // sample_poisson of the reference: draws are consumed, data copied
  const float* in;
  float* out;
  __device__ __forceinline__ void operator()(size_t i, float u) const { (void)u; out[i] = in[i]; }
};
struct OpPerturbEnergy {
  const float* in;
  float* out;
  __device__ __forceinline__ void operator()(size_t i, float u) const { out[i] = in[i] - logf(-logf(u)); }
};
struct OpPerturbProb {
  const float* in;
  float* out;
  __device__ __forceinline__ void operator()(size_t i, float u) const { out[i] = -in[i] / logf(u); }
};

#define RNG_BLOCK 64
#define RNG_BLOCKS (NUM_RND_STREAMS / RNG_BLOCK)

template <class Op>
__global__ void __launch_bounds__(RNG_BLOCK)
k_rng_serial(const unsigned int* mults, unsigned long long* words, size_t n, Op op) {
  const unsigned int idx = blockIdx.x * RNG_BLOCK + threadIdx.x;
  unsigned long long w = words[idx];
  const unsigned int mult = mults[idx];
  for (size_t i = idx; i < n; i += NUM_RND_STREAMS) {
    w = mwc_step(w, mult);
    op(i, mwc_uniform(w));
  }
  words[idx] = w;
}

// Box-Muller pairs: two draws give elements i and i + 12288 (cudamat_kernels.cu:125-143, 192-211).
__global__ void __launch_bounds__(RNG_BLOCK)
k_rng_gauss(const unsigned int* mults, unsigned long long* words, const float* in, float* out, size_t n, float mult_by) {
  const unsigned int idx = blockIdx.x * RNG_BLOCK + threadIdx.x;
  unsigned long long w = words[idx];
  const unsigned int mult = mults[idx];
  for (size_t i = idx; i < n; i += 2 * NUM_RND_STREAMS) {
    w = mwc_step(w, mult);
    const float r1 = mwc_uniform(w);
    w = mwc_step(w, mult);
    const float r2 = mwc_uniform(w);
    const float T = 2.f * RNG_PI * r2;
    const float R = sqrtf(-2.f * logf(r1));
    const float a = R * cosf(T), b = R * sinf(T);
    out[i] = in ? in[i] + mult_by * a : a;
    const size_t i2 = i + NUM_RND_STREAMS;
    if (i2 < n) out[i2] = in ? in[i2] + mult_by * b : b;
  }
  words[idx] = w;
}

template <class Op>
static int launch_rng(rnd_struct* st, size_t n, Op op) {
  hipLaunchKernelGGL((k_rng_serial<Op>), dim3(RNG_BLOCKS), dim3(RNG_BLOCK), 0, 0, st->dev_mults, st->dev_words, n, op);
  return dn_launch_status();
}

extern "C" {

int init_random(rnd_struct* rnd_state, int seed, char* cudamatpath) {
  FILE* f = cudamatpath ? fopen(cudamatpath, "r") : nullptr;
  if (!f) return ERROR_GENERIC;
  unsigned int* host_mults = (unsigned int*)malloc(NUM_RND_STREAMS * sizeof(unsigned int));
  int got = 0;
  for (; got < NUM_RND_STREAMS; ++got)
    if (fscanf(f, "%u", &host_mults[got]) != 1) break;
  fclose(f);
  if (got != NUM_RND_STREAMS) {
    free(host_mults);
    return ERROR_GENERIC;
  }
  void *dm = nullptr, *dw = nullptr;
  if (hipMalloc(&dm, NUM_RND_STREAMS * sizeof(unsigned int)) != hipSuccess ||
      hipMalloc(&dw, NUM_RND_STREAMS * sizeof(unsigned long long)) != hipSuccess ||
      hipMemcpy(dm, host_mults, NUM_RND_STREAMS * sizeof(unsigned int), hipMemcpyHostToDevice) != hipSuccess) {
    free(host_mults);
    return CUDA_ERROR;
  }
  free(host_mults);
  rnd_state->dev_mults = (unsigned int*)dm;
  rnd_state->dev_words = (unsigned long long*)dw;
  hipLaunchKernelGGL(k_seed, dim3(RNG_BLOCKS), dim3(RNG_BLOCK), 0, 0, rnd_state->dev_mults, rnd_state->dev_words,
                     (unsigned int)seed);
  return dn_launch_status();
}

int fill_with_rand(rnd_struct* rnd_state, cudamat* mat) {
  if (!mat->on_device) return ERROR_NOT_ON_DEVICE;
  return launch_rng(rnd_state, (size_t)dn_len(mat), OpUniform{mat->data_device});
}

int fill_with_randn(rnd_struct* rnd_state, cudamat* mat) {
  if (!mat->on_device) return ERROR_NOT_ON_DEVICE;
  hipLaunchKernelGGL(k_rng_gauss, dim3(RNG_BLOCKS), dim3(RNG_BLOCK), 0, 0, rnd_state->dev_mults, rnd_state->dev_words,
                     (const float*)nullptr, mat->data_device, (size_t)dn_len(mat), 1.f);
  return dn_launch_status();
}

// The sampling wrappers check dims before residency (cudamat.cu:469-572).
#define DN_SAMPLER(NAME, OP)                                                                           \
  int NAME(rnd_struct* rnd_state, cudamat* mat, cudamat* target) {                                     \
    if (mat->size[0] != target->size[0] || mat->size[1] != target->size[1])                            \
      return ERROR_INCOMPATIBLE_DIMENSIONS;                                                            \
    if (!mat->on_device || !target->on_device) return ERROR_NOT_ON_DEVICE;                             \
    return launch_rng(rnd_state, (size_t)dn_len(mat), OP{mat->data_device, target->data_device});      \
  }

DN_SAMPLER(sample_bernoulli, OpBernoulli)
DN_SAMPLER(sample_bernoulli_tanh, OpBernoulliTanh)
DN_SAMPLER(sample_poisson, OpCopy)
DN_SAMPLER(perturb_energy, OpPerturbEnergy)
DN_SAMPLER(perturb_prob, OpPerturbProb)

int sample_gaussian(rnd_struct* rnd_state, cudamat* mat, cudamat* target, float mult) {
  if (mat->size[0] != target->size[0] || mat->size[1] != target->size[1]) return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (!mat->on_device || !target->on_device) return ERROR_NOT_ON_DEVICE;
  hipLaunchKernelGGL(k_rng_gauss, dim3(RNG_BLOCKS), dim3(RNG_BLOCK), 0, 0, rnd_state->dev_mults, rnd_state->dev_words,
                     (const float*)mat->data_device, target->data_device, (size_t)dn_len(mat), mult);
  return dn_launch_status();
}

int dropout(rnd_struct* rnd_state, cudamat* mat, float dropprob, float val) {
  if (!mat->on_device) return ERROR_NOT_ON_DEVICE;
  return launch_rng(rnd_state, (size_t)dn_len(mat), OpDropout{mat->data_device, dropprob, val});
}

}  // extern "C"
