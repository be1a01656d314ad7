// Pieces of the multiply-with-carry generator that kernels outside rng.hip use (the product
// kernels that draw a Bernoulli sample of their own output).
#pragma once
#include "common.h"

__device__ __forceinline__ unsigned long long mwc_step(unsigned long long w, unsigned int mult) {
  return (unsigned long long)mult * (w & 0xffffffffull) + (w >> 32);
}

// (lo32 + 1) / 2^32 with the conversion rounded to nearest even: a value in (0, 1].
__device__ __forceinline__ float mwc_uniform(unsigned long long w) {
  return ((float)(unsigned int)(w & 0xffffffffull) + 1.0f) * 2.3283064365386963e-10f;
}

// Layout of the allocation behind rnd_struct::dev_words (N = 12288 words of 8 bytes):
// a region aligned to 256 KiB holds two word buffers A (offset 0) and B (offset
// 128 KiB) and, from offset 256 KiB, the jump table: entry j of stream t multiplies
// a word by (2^32)^-(2^j) modulo m_t, i.e. jumps 2^j draws ahead.  dev_words points
// at whichever of A / B holds the current words; the split schedule reads one
// buffer, writes the other and flips the pointer, so no lane can overwrite a word
// another lane still has to read.  Bit 17 of the pointer tells the two apart.
#define RNG_JUMP_BITS 21
#define RNG_BUF_BYTES (128u << 10)
#define RNG_REGION_BYTES ((size_t)2 * RNG_BUF_BYTES + (size_t)RNG_JUMP_BITS * NUM_RND_STREAMS * 8)

static inline unsigned long long* rng_other(unsigned long long* w) {
  return reinterpret_cast<unsigned long long*>(reinterpret_cast<uintptr_t>(w) ^ (uintptr_t)RNG_BUF_BYTES);
}

// A kernel has left the generator's next state in rng_other(st->dev_words): make it the
// current one.  Normally the pointer is flipped; once a recorded graph refers to the current
// buffer (rng.hip pins it until the last graph has been freed) the words are copied back into
// it instead, so that replays and eager calls keep drawing from one sequence.
void rng_publish(rnd_struct* st);
// To be called before a kernel that uses st->dev_words is launched: while a graph is being
// recorded it pins the buffer.  Always true (kept as a condition at the call sites).
bool rng_pin_if_recording(rnd_struct* st);

// What a product that also draws a Bernoulli sample of its output needs from the generator:
// the sample's buffer, the multipliers, the current words (read only) and the buffer that
// receives the words after the call.
struct DnGemmSample {
  float* sample;
  const unsigned int* mults;
  const unsigned long long* words;
  unsigned long long* next;
};
