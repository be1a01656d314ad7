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
//   split   - a stream's draws are cut into parts of 2^c consecutive draws, one
//             lane per part.  One step is a multiplication by (2^32)^-1 modulo
//             m = mult * 2^32 - 1 (word' * 2^32 = m * lo + word), so a lane reaches
//             its first draw by multiplying the stream's word with per-stream
//             constants (2^32)^-(2^j) mod m, one per set bit of its part number.
#include "common.h"
#include "rng.h"
#include <vector>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>

#define RNG_PI 3.1415926535897932f

static inline const unsigned long long* rng_table(const unsigned long long* w) {
  return reinterpret_cast<const unsigned long long*>((reinterpret_cast<uintptr_t>(w) & ~(uintptr_t)(2 * RNG_BUF_BYTES - 1)) +
                                                     2 * RNG_BUF_BYTES);
}

// x * y * 2^-64 modulo m = mult * 2^32 - 1, in [0, m).  Dividing by 2^32 modulo m is
// the generator's own step (v -> mult * lo32(v) + (v >> 32)), applied twice to the
// 128-bit product; the result is below 2m + 2^32, so two subtractions suffice.
__device__ __forceinline__ unsigned long long mwc_montmul(unsigned long long x, unsigned long long y,
                                                          unsigned int mult) {
  const unsigned long long m = ((unsigned long long)mult << 32) - 1ull;
  unsigned __int128 v = (unsigned __int128)x * y;
  v = (v >> 32) + (unsigned __int128)mult * (unsigned int)v;
  v = (v >> 32) + (unsigned __int128)mult * (unsigned int)v;
  if (v >= m) v -= m;
  if (v >= m) v -= m;
  return (unsigned long long)v;
}

__global__ void k_seed(const unsigned int* mults, unsigned long long* words, unsigned long long* table,
                       unsigned int seed) {
  const unsigned int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= NUM_RND_STREAMS) return;
  unsigned long long w = ((unsigned long long)seed << 32) + 1ull;
  const unsigned int mult = mults[idx];
  for (int i = 0; i < NUM_RND_BURNIN; ++i) w = mwc_step(w, mult);
  words[idx] = w;
  // Jump table in the form t_j = (2^32)^(2 - 2^j) mod m, so that mwc_montmul(w, t_j)
  // = w * (2^32)^-(2^j): t_0 = 2^32, t_1 = 1, t_{j+1} = mwc_montmul(t_j, t_j).
  unsigned long long t = 1ull;
  table[idx] = 1ull << 32;
  for (int j = 1; j < RNG_JUMP_BITS; ++j) {
    table[(size_t)j * NUM_RND_STREAMS + idx] = t;
    t = mwc_montmul(t, t, mult);
  }
}

// ------------------------------------------------------------------ consumers
// One uniform per element.  An op names the array it reads (src, may be null), the
// array it writes (dst) and the pure function value(u, x) of the uniform u and the
// loaded x.  The loads do not depend on the draws, so a lane issues a batch of them
// before it walks the serial chain of its stream.
struct OpUniform {
  const float* src; float* dst;
  __device__ __forceinline__ float value(float u, float) const { return u; }
};
struct OpDropout {
  const float* src; float* dst;
  float p, val;
  __device__ __forceinline__ float value(float u, float x) const { return u > p ? x : val; }
};
struct OpBernoulli {
  const float* src; float* dst;
  __device__ __forceinline__ float value(float u, float x) const { return u < x ? 1.f : 0.f; }
};
struct OpBernoulliTanh {
  const float* src; float* dst;
  __device__ __forceinline__ float value(float u, float x) const {
    return (double)u < (1.0 + (double)x) / 2.0 ? 1.f : 0.f;
  }
};
struct OpCopy {  // sample_poisson of the reference: draws are consumed, data copied
  const float* src; float* dst;
  __device__ __forceinline__ float value(float, float x) const { return x; }
};
struct OpPerturbEnergy {
  const float* src; float* dst;
  __device__ __forceinline__ float value(float u, float x) const { return x - logf(-logf(u)); }
};
struct OpPerturbProb {
  const float* src; float* dst;
  __device__ __forceinline__ float value(float u, float x) const { return -x / logf(u); }
};
// fill_with_rand -> greater_than(p) -> mult by the mask (deepnet/neuralnet.py:194-198) in one pass:
// dst gets the mask (u > p ? 1 : 0), and where a second array is given (src, read and written in
// place) it is multiplied by the mask.
struct OpDropMask {
  const float* src; float* dst;
  float p;
  float* state;
  __device__ __forceinline__ float value(float u, float) const { return u > p ? 1.f : 0.f; }
};
// fill_with_rand(r) -> less_than(r, h, target = h) (the hidden sample of cudamat/examples/rbm_cudamat.py:63-65)
// in one pass: dst gets (u < src ? 1 : 0), uni the uniforms themselves.
struct OpBernoulliKeep {
  const float* src; float* dst;
  float* uni;
  __device__ __forceinline__ float value(float u, float x) const { return u < x ? 1.f : 0.f; }
};
// what an op stores besides dst[i] (u: the draw, v: the value stored in dst[i], x: what was loaded from src[i])
template <class Op>
__device__ __forceinline__ void rng_side(const Op&, size_t, float, float, float) {}
__device__ __forceinline__ void rng_side(const OpDropMask& op, size_t i, float, float v, float x) {
  if (op.state) op.state[i] = x * v;
}
__device__ __forceinline__ void rng_side(const OpBernoulliKeep& op, size_t i, float u, float, float) { op.uni[i] = u; }

// Draws [d0, d1) of one stream: element index of draw d is d * 12288 + idx.
// STREAM: the call is large, use non-temporal accesses.
#define RNG_BATCH 8
template <bool STREAM, class Op>
__device__ __forceinline__ unsigned long long rng_walk(unsigned long long w, unsigned int mult, unsigned int idx,
                                                       unsigned long long d0, unsigned long long d1, const Op& op) {
  size_t i = (size_t)d0 * NUM_RND_STREAMS + idx;
  unsigned long long d = d0;
  for (; d + RNG_BATCH <= d1; d += RNG_BATCH, i += (size_t)RNG_BATCH * NUM_RND_STREAMS) {
    float x[RNG_BATCH];
#pragma unroll
    for (int k = 0; k < RNG_BATCH; ++k)
      x[k] = op.src ? dn_ld1_rt(op.src + i + (size_t)k * NUM_RND_STREAMS, STREAM) : 0.f;
#pragma unroll
    for (int k = 0; k < RNG_BATCH; ++k) {
      w = mwc_step(w, mult);
      const float u = mwc_uniform(w), v = op.value(u, x[k]);
      dn_st1_rt(op.dst + i + (size_t)k * NUM_RND_STREAMS, v, STREAM);
      rng_side(op, i + (size_t)k * NUM_RND_STREAMS, u, v, x[k]);
    }
  }
  for (; d < d1; ++d, i += NUM_RND_STREAMS) {
    const float x = op.src ? op.src[i] : 0.f;
    w = mwc_step(w, mult);
    const float u = mwc_uniform(w), v = op.value(u, x);
    op.dst[i] = v;
    rng_side(op, i, u, v, x);
  }
  return w;
}

#define RNG_BLOCK 64
#define RNG_BLOCKS (NUM_RND_STREAMS / RNG_BLOCK)

template <class Op>
__global__ void __launch_bounds__(RNG_BLOCK)
k_rng_serial(const unsigned int* mults, unsigned long long* words, size_t n, Op op) {
  const unsigned int idx = blockIdx.x * RNG_BLOCK + threadIdx.x;
  const unsigned int mult = mults[idx];
  const unsigned long long draws = n > idx ? (n - idx + NUM_RND_STREAMS - 1) / NUM_RND_STREAMS : 0;
  words[idx] = rng_walk<false>(words[idx], mult, idx, 0, draws, op);
}

// Split schedule: lane (stream s, part p) produces draws [p << chbits, (p+1) << chbits)
// of its stream, reaching its first draw with one jump per set bit of p.  The lane
// that produces a stream's last draw writes the new word into the other buffer.
#define RNG_SPLIT_BLOCK 256
template <class Op, int B>
__global__ void __launch_bounds__(RNG_SPLIT_BLOCK)
k_rng_split(const unsigned int* mults, const unsigned long long* words, unsigned long long* next,
            const unsigned long long* table, size_t n, int chbits, Op op) {
  constexpr int blocks_per_part = NUM_RND_STREAMS / RNG_SPLIT_BLOCK;
  const unsigned int part = blockIdx.x / blocks_per_part;
  const unsigned int idx = (blockIdx.x % blocks_per_part) * RNG_SPLIT_BLOCK + threadIdx.x;
  if (idx >= n) {  // a stream without draws keeps its word
    if (part == 0) next[idx] = words[idx];
    return;
  }
  const unsigned long long draws = (n - idx + NUM_RND_STREAMS - 1) / NUM_RND_STREAMS;  // of this stream
  const unsigned long long d0 = (unsigned long long)part << chbits;
  if (d0 >= draws) return;
  const unsigned long long d1 = d0 + (1ull << chbits) < draws ? d0 + (1ull << chbits) : draws;
  size_t i = (size_t)d0 * NUM_RND_STREAMS + idx;
  unsigned long long d = d0;
  // The array reads do not depend on the generator: the first batch is requested
  // before the jump-ahead arithmetic, which then runs under the memory latency.
  float x[B];
  const bool full0 = d + B <= d1;
  if (full0) {
#pragma unroll
    for (int k = 0; k < B; ++k) x[k] = op.src ? __builtin_nontemporal_load(op.src + i + (size_t)k * NUM_RND_STREAMS) : 0.f;
  }
  const unsigned int mult = mults[idx];
  unsigned long long w = words[idx];
  for (unsigned int b = 0, pp = part; pp; ++b, pp >>= 1)
    if (pp & 1u) w = mwc_montmul(w, table[(size_t)(chbits + b) * NUM_RND_STREAMS + idx], mult);
  auto emit = [&](size_t at, float xv) {
    w = mwc_step(w, mult);
    const float u = mwc_uniform(w), v = op.value(u, xv);
    __builtin_nontemporal_store(v, op.dst + at);
    rng_side(op, at, u, v, xv);
  };
  if (full0) {
    for (;;) {
      const size_t inext = i + (size_t)B * NUM_RND_STREAMS;
      const bool more = d + 2 * B <= d1;
      float y[B];
#pragma unroll
      for (int k = 0; k < B; ++k) y[k] = x[k];
      if (more) {   // the next batch is requested before this one is consumed
#pragma unroll
        for (int k = 0; k < B; ++k) x[k] = op.src ? __builtin_nontemporal_load(op.src + inext + (size_t)k * NUM_RND_STREAMS) : 0.f;
      }
#pragma unroll
      for (int k = 0; k < B; ++k) emit(i + (size_t)k * NUM_RND_STREAMS, y[k]);
      d += B;
      i = inext;
      if (!more) break;
    }
  }
  for (; d < d1; ++d, i += NUM_RND_STREAMS) emit(i, op.src ? op.src[i] : 0.f);
  if (d1 == draws) next[idx] = w;
}

// Box-Muller pairs: two draws give elements i and i + 12288 (cudamat_kernels.cu:125-143, 192-211).
__device__ __forceinline__ void box_muller(float r1, float r2, float& a, float& b) {
  const float T = 2.f * RNG_PI * r2;
  const float R = sqrtf(-2.f * logf(r1));
  a = R * cosf(T);
  b = R * sinf(T);
}

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
    float a, b;
    box_muller(r1, r2, a, b);
    out[i] = in ? in[i] + mult_by * a : a;
    const size_t i2 = i + NUM_RND_STREAMS;
    if (i2 < n) out[i2] = in ? in[i2] + mult_by * b : b;
  }
  words[idx] = w;
}

// The same pairs on the split schedule.  A stream with an odd number of elements still
// takes both draws of its last pair, so its draw count is rounded up to even; parts are
// 2^chbits >= 16 draws, so no pair straddles two lanes.
#define RNG_GAUSS_PAIRS 4
__global__ void __launch_bounds__(RNG_SPLIT_BLOCK)
k_rng_gauss_split(const unsigned int* mults, const unsigned long long* words, unsigned long long* next,
                  const unsigned long long* table, const float* in, float* out, size_t n, int chbits, float mult_by) {
  constexpr int blocks_per_part = NUM_RND_STREAMS / RNG_SPLIT_BLOCK;
  constexpr int P = RNG_GAUSS_PAIRS;
  const unsigned int part = blockIdx.x / blocks_per_part;
  const unsigned int idx = (blockIdx.x % blocks_per_part) * RNG_SPLIT_BLOCK + threadIdx.x;
  if (idx >= n) {
    if (part == 0) next[idx] = words[idx];
    return;
  }
  const unsigned long long elems = (n - idx + NUM_RND_STREAMS - 1) / NUM_RND_STREAMS;  // of this stream
  const unsigned long long draws = (elems + 1) & ~1ull;
  const unsigned long long d0 = (unsigned long long)part << chbits;
  if (d0 >= draws) return;
  const unsigned long long d1 = d0 + (1ull << chbits) < draws ? d0 + (1ull << chbits) : draws;
  size_t i = (size_t)d0 * NUM_RND_STREAMS + idx;
  unsigned long long d = d0;
  // A batch of P pairs whose 2 P elements all exist; its reads are requested before the
  // jump-ahead arithmetic and before the previous batch is consumed.
  float x[2 * P];
  auto fetch = [&](size_t at) {
#pragma unroll
    for (int k = 0; k < 2 * P; ++k) x[k] = in ? __builtin_nontemporal_load(in + at + (size_t)k * NUM_RND_STREAMS) : 0.f;
  };
  const bool full0 = d + 2 * P <= d1 && d + 2 * P <= elems;
  if (full0) fetch(i);
  const unsigned int mult = mults[idx];
  unsigned long long w = words[idx];
  for (unsigned int b = 0, pp = part; pp; ++b, pp >>= 1)
    if (pp & 1u) w = mwc_montmul(w, table[(size_t)(chbits + b) * NUM_RND_STREAMS + idx], mult);
  auto pair = [&](float& a, float& b) {
    w = mwc_step(w, mult);
    const float r1 = mwc_uniform(w);
    w = mwc_step(w, mult);
    box_muller(r1, mwc_uniform(w), a, b);
  };
  if (full0) {
    for (;;) {
      const size_t inext = i + (size_t)(2 * P) * NUM_RND_STREAMS;
      const bool more = d + 4 * P <= d1 && d + 4 * P <= elems;
      float y[2 * P];
#pragma unroll
      for (int k = 0; k < 2 * P; ++k) y[k] = x[k];
      if (more) fetch(inext);
#pragma unroll
      for (int k = 0; k < P; ++k) {
        float a, b;
        pair(a, b);
        const size_t at = i + (size_t)(2 * k) * NUM_RND_STREAMS;
        __builtin_nontemporal_store(in ? y[2 * k] + mult_by * a : a, out + at);
        __builtin_nontemporal_store(in ? y[2 * k + 1] + mult_by * b : b, out + at + NUM_RND_STREAMS);
      }
      d += 2 * P;
      i = inext;
      if (!more) break;
    }
  }
  for (; d < d1; d += 2, i += 2 * (size_t)NUM_RND_STREAMS) {
    float a, b;
    pair(a, b);
    out[i] = in ? in[i] + mult_by * a : a;
    const size_t i2 = i + NUM_RND_STREAMS;
    if (d + 1 < elems) out[i2] = in ? in[i2] + mult_by * b : b;
  }
  if (d1 == draws) next[idx] = w;
}

// Calls with at least RNG_SPLIT_MIN_DRAWS draws per stream are cut into parts of 2^c
// draws.  A pure fill takes about RNG_SPLIT_PARTS parts per stream (c >= 4).  An op
// that also reads an array takes parts of 16 draws while that gives at most
// RNG_SPLIT_SRC_PARTS parts, all 16 reads of a lane in flight under its jump
// arithmetic; measured on 4096 x 4096 (sample_bernoulli): 25.0 us against 27-28 us
// for 64-draw parts and for four streams per lane with 16-byte accesses.  Part
// counts whose workgroups fill the chip's resident slots a little more than a whole
// number of times (43 parts of 32 draws: 2064 workgroups for 2048 slots) cost 2 us.
#define RNG_SPLIT_MIN_DRAWS 32
#define RNG_SPLIT_PARTS 24
#define RNG_SPLIT_SRC_PARTS 96

// Word buffers that a recorded graph refers to: its kernels carry the buffer's address, so
// from then on the generator's state has to stay in that buffer.
static std::vector<unsigned long long*>& rng_pinned() {
  static std::vector<unsigned long long*>* list = new std::vector<unsigned long long*>;   // never destroyed
  return *list;
}

static bool rng_is_pinned(const unsigned long long* w) {
  for (const unsigned long long* p : rng_pinned())
    if (p == w) return true;
  return false;
}

// (no graph is left: the state may move between the buffers again)
static void rng_unpin_all() { rng_pinned().clear(); }

bool rng_pin_if_recording(rnd_struct* st) {
  if (dn_capturing() && !rng_is_pinned(st->dev_words)) {
    rng_pinned().push_back(st->dev_words);
    dn_set_no_graphs_hook(rng_unpin_all);
  }
  return true;
}

__global__ void __launch_bounds__(256) k_rng_copy_words(const unsigned long long* from, unsigned long long* to) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < NUM_RND_STREAMS) to[i] = from[i];
}

void rng_publish(rnd_struct* st) {
  unsigned long long* next = rng_other(st->dev_words);
  if (rng_is_pinned(st->dev_words))
    hipLaunchKernelGGL(k_rng_copy_words, dim3(NUM_RND_STREAMS / 256), dim3(256), 0, dn_stream(), (const unsigned long long*)next,
                       st->dev_words);
  else
    st->dev_words = next;
}

template <class Op>
static int launch_rng(rnd_struct* st, size_t n, Op op) {
  if (n == 0) return 0;
  // Work that is held back may use this generator (a fill_with_rand that waits for its threshold)
  // and leave its next state in the other buffer: it is launched before the state is looked at.
  dn_flush();
  const size_t draws = (n + NUM_RND_STREAMS - 1) / NUM_RND_STREAMS;
  if (draws < RNG_SPLIT_MIN_DRAWS) {
    if (!rng_pin_if_recording(st)) return ERROR_UNSUPPORTED;
    hipLaunchKernelGGL((k_rng_serial<Op>), dim3(RNG_BLOCKS), dim3(RNG_BLOCK), 0, dn_stream(), st->dev_mults, st->dev_words, n,
                       op);
    return dn_launch_status();
  }
  int chbits = 4;
  while (((draws + (1ull << chbits) - 1) >> chbits) > (size_t)(op.src ? RNG_SPLIT_SRC_PARTS : RNG_SPLIT_PARTS)) ++chbits;
  const size_t parts = (draws + (1ull << chbits) - 1) >> chbits;
  // every jump exponent (chbits + bit of part) must be inside the table
  int top = 0;
  while ((parts - 1) >> top) ++top;
  if (chbits + top > RNG_JUMP_BITS) {
    if (!rng_pin_if_recording(st)) return ERROR_UNSUPPORTED;
    hipLaunchKernelGGL((k_rng_serial<Op>), dim3(RNG_BLOCKS), dim3(RNG_BLOCK), 0, dn_stream(), st->dev_mults, st->dev_words, n,
                       op);
    return dn_launch_status();
  }
  // (while a graph is recorded the buffer is pinned, and rng_publish() records the copy of the
  // new words back into it)
  if (!rng_pin_if_recording(st)) return ERROR_UNSUPPORTED;
  unsigned long long* next = rng_other(st->dev_words);
  const unsigned grid = (unsigned)(parts * (NUM_RND_STREAMS / RNG_SPLIT_BLOCK));
  if (op.src)
    hipLaunchKernelGGL((k_rng_split<Op, 16>), dim3(grid), dim3(RNG_SPLIT_BLOCK), 0, dn_stream(), st->dev_mults,
                       (const unsigned long long*)st->dev_words, next, rng_table(st->dev_words), n, chbits, op);
  else
    hipLaunchKernelGGL((k_rng_split<Op, 4>), dim3(grid), dim3(RNG_SPLIT_BLOCK), 0, dn_stream(), st->dev_mults,
                       (const unsigned long long*)st->dev_words, next, rng_table(st->dev_words), n, chbits, op);
  rng_publish(st);
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
  if (dn_malloc(&dm, NUM_RND_STREAMS * sizeof(unsigned int)) != hipSuccess ||
      dn_malloc(&dw, RNG_REGION_BYTES + 2 * RNG_BUF_BYTES) != hipSuccess ||
      hipMemcpy(dm, host_mults, NUM_RND_STREAMS * sizeof(unsigned int), hipMemcpyHostToDevice) != hipSuccess) {
    free(host_mults);
    return CUDA_ERROR;
  }
  free(host_mults);
  rnd_state->dev_mults = (unsigned int*)dm;
  // align the region to 256 KiB inside the (never freed, as in the reference) allocation
  const uintptr_t base = (reinterpret_cast<uintptr_t>(dw) + 2 * RNG_BUF_BYTES - 1) & ~(uintptr_t)(2 * RNG_BUF_BYTES - 1);
  rnd_state->dev_words = reinterpret_cast<unsigned long long*>(base);
  hipLaunchKernelGGL(k_seed, dim3(RNG_BLOCKS), dim3(RNG_BLOCK), 0, dn_stream(), rnd_state->dev_mults, rnd_state->dev_words,
                     const_cast<unsigned long long*>(rng_table(rnd_state->dev_words)), (unsigned int)seed);
  return dn_launch_status();
}

// Gaussian ops: parts of 16 draws (8 pairs, each a logf, sqrtf, sinf and cosf) while that
// gives at most RNG_GAUSS_PARTS parts per stream.
#define RNG_GAUSS_PARTS 256
static int launch_gauss(rnd_struct* st, const float* in, float* out, size_t n, float mult_by) {
  if (n == 0) return 0;
  dn_flush();          // (as in launch_rng)
  const size_t elems = (n + NUM_RND_STREAMS - 1) / NUM_RND_STREAMS;
  const size_t draws = (elems + 1) & ~(size_t)1;   // of the busiest stream
  int chbits = 4;
  while (((draws + (1ull << chbits) - 1) >> chbits) > (size_t)RNG_GAUSS_PARTS) ++chbits;
  const size_t parts = (draws + (1ull << chbits) - 1) >> chbits;
  int top = 0;
  while ((parts - 1) >> top) ++top;
  if (!rng_pin_if_recording(st)) return ERROR_UNSUPPORTED;
  if (draws < RNG_SPLIT_MIN_DRAWS || chbits + top > RNG_JUMP_BITS) {
    hipLaunchKernelGGL(k_rng_gauss, dim3(RNG_BLOCKS), dim3(RNG_BLOCK), 0, dn_stream(), st->dev_mults, st->dev_words, in, out, n,
                       mult_by);
    return dn_launch_status();
  }
  unsigned long long* next = rng_other(st->dev_words);
  const unsigned grid = (unsigned)(parts * (NUM_RND_STREAMS / RNG_SPLIT_BLOCK));
  hipLaunchKernelGGL(k_rng_gauss_split, dim3(grid), dim3(RNG_SPLIT_BLOCK), 0, dn_stream(), st->dev_mults,
                     (const unsigned long long*)st->dev_words, next, rng_table(st->dev_words), in, out, n, chbits, mult_by);
  rng_publish(st);
  return dn_launch_status();
}

// A generator that init_random() never set up (null handle or null state pointers): the
// reference would dereference it; here the call is refused.
static inline bool rng_ready(const rnd_struct* st) { return st && st->dev_mults && st->dev_words; }

int fill_with_rand(rnd_struct* rnd_state, cudamat* mat) {
  if (!mat->on_device) return ERROR_NOT_ON_DEVICE;
  if (!rng_ready(rnd_state)) return ERROR_GENERIC;
  // (held back: the threshold and the product of a dropout mask may follow)
  int held = 0;
  if (dn_defer_fill_rand(rnd_state, mat, &held)) return held;
  return launch_rng(rnd_state, (size_t)dn_len(mat), OpUniform{nullptr, mat->data_device});
}

int fill_with_randn(rnd_struct* rnd_state, cudamat* mat) {
  if (!mat->on_device) return ERROR_NOT_ON_DEVICE;
  if (!rng_ready(rnd_state)) return ERROR_GENERIC;
  return launch_gauss(rnd_state, nullptr, mat->data_device, (size_t)dn_len(mat), 1.f);
}

// The sampling wrappers check dims before residency (cudamat.cu:469-572).
#define DN_SAMPLER(NAME, OP)                                                                           \
  int NAME(rnd_struct* rnd_state, cudamat* mat, cudamat* target) {                                     \
    if (mat->size[0] != target->size[0] || mat->size[1] != target->size[1])                            \
      return ERROR_INCOMPATIBLE_DIMENSIONS;                                                            \
    if (!mat->on_device || !target->on_device) return ERROR_NOT_ON_DEVICE;                             \
    if (!rng_ready(rnd_state)) return ERROR_GENERIC;                                                   \
    return launch_rng(rnd_state, (size_t)dn_len(mat), OP{mat->data_device, target->data_device});      \
  }

int sample_bernoulli(rnd_struct* rnd_state, cudamat* mat, cudamat* target) {
  // (the sample of a product that is being held back with its sigmoid is drawn by the product's launch)
  int err = 0;
  if (dn_pending_sample(rnd_state, mat, target, &err)) return err;
  if (mat->size[0] != target->size[0] || mat->size[1] != target->size[1]) return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (!mat->on_device || !target->on_device) return ERROR_NOT_ON_DEVICE;
  if (!rng_ready(rnd_state)) return ERROR_GENERIC;
  return launch_rng(rnd_state, (size_t)dn_len(mat), OpBernoulli{mat->data_device, target->data_device});
}
DN_SAMPLER(sample_bernoulli_tanh, OpBernoulliTanh)
DN_SAMPLER(sample_poisson, OpCopy)
DN_SAMPLER(perturb_energy, OpPerturbEnergy)
DN_SAMPLER(perturb_prob, OpPerturbProb)

int sample_gaussian(rnd_struct* rnd_state, cudamat* mat, cudamat* target, float mult) {
  if (mat->size[0] != target->size[0] || mat->size[1] != target->size[1]) return ERROR_INCOMPATIBLE_DIMENSIONS;
  if (!mat->on_device || !target->on_device) return ERROR_NOT_ON_DEVICE;
  if (!rng_ready(rnd_state)) return ERROR_GENERIC;
  return launch_gauss(rnd_state, mat->data_device, target->data_device, (size_t)dn_len(mat), mult);
}

}  // extern "C"

// mask = (uniform draw > p) ? 1 : 0 over n elements, and state *= mask when state is given
// (fill_with_rand, greater_than_scalar and mult_elementwise in one pass, same draws, same values).
int dn_rng_dropmask(rnd_struct* rnd_state, float* mask, float* state, size_t n, float p) {
  if (!rng_ready(rnd_state)) return ERROR_GENERIC;
  return launch_rng(rnd_state, n, OpDropMask{state, mask, p, state});
}

int dn_rng_bernoulli_keep(rnd_struct* rnd_state, float* uni, float* probs, size_t n) {
  if (!rng_ready(rnd_state)) return ERROR_GENERIC;
  return launch_rng(rnd_state, n, OpBernoulliKeep{probs, probs, uni});
}

extern "C" {

int dropout(rnd_struct* rnd_state, cudamat* mat, float dropprob, float val) {
  if (!mat->on_device) return ERROR_NOT_ON_DEVICE;
  if (!rng_ready(rnd_state)) return ERROR_GENERIC;
  return launch_rng(rnd_state, (size_t)dn_len(mat), OpDropout{mat->data_device, mat->data_device, dropprob, val});
}

}  // extern "C"
