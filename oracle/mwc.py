"""TEST INFRASTRUCTURE ONLY - CPU restatement of cudamat's multiply-with-carry RNG.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this; the product (deepnet_amd/) never does.

Follows cudamat/cudamat_kernels.cu:96-239 and cudamat/cudamat.cu:55-83:
  * 12288 streams; stream t owns multiplier mults[t] (first 12288 lines of
    rnd_multipliers_32bit.txt) and a 64-bit word;
  * seeding: word = (seed << 32) + 1, then 100 steps;
  * one step: word = mult * lo32(word) + hi32(word);
  * uniform: (float32(lo32(word)) + 1.0f) / 2^32, conversion rounded to nearest even;
  * a call over n elements gives element i the next draw of stream i % 12288
    (draw number i // 12288 of that call); streams keep their word between calls.

Two independent codings are kept on purpose - `*_py` on Python integers and the
vectorised numpy-uint64 class `MWC` - so the tests can play one against the
other; a third coding in C lives in host_backend.c.

Pins (tests/test_oracle_mwc.py): py == numpy == C on seeds 0, 1, 42 and a length
that is not a multiple of 12288; the step invariant word' * 2^32 == m * lo + word
(m = mult * 2^32 - 1), i.e. word' == word * (2^32)^-1 (mod m), checked with
Python's three-argument pow for every multiplier; jump-ahead against brute force.
"""
import numpy as np

NUM_RND_STREAMS = 96 * 128
NUM_RND_BURNIN = 100
MASK32 = 0xFFFFFFFF


def load_multipliers(path):
    """First 12288 unsigned integers of the multiplier table (cudamat.cu:60-65)."""
    vals = []
    with open(path) as f:
        for line in f:
            line = line.strip()
            if line:
                vals.append(int(line))
                if len(vals) == NUM_RND_STREAMS:
                    break
    if len(vals) != NUM_RND_STREAMS:
        raise ValueError("multiplier table too short: %d" % len(vals))
    return np.array(vals, dtype=np.uint32)


# ---------------------------------------------------------------- Python-int coding

def step_py(word, mult):
    """cudamat_kernels.cu:108 - one multiply-with-carry step on Python integers."""
    return mult * (word & MASK32) + (word >> 32)


def seed_word_py(seed, mult):
    """cudamat_kernels.cu:96-111."""
    word = ((seed & MASK32) << 32) + 1
    for _ in range(NUM_RND_BURNIN):
        word = step_py(word, mult)
    assert word < (1 << 64)
    return word


def uniform_py(word):
    """cudamat_kernels.cu:120 - float32 arithmetic throughout."""
    return (np.float32(np.uint32(word & MASK32)) + np.float32(1.0)) / np.float32(4294967296.0)


def jump_py(word, mult, k):
    """The word after k steps without taking them: word * (2^32)^-k modulo
    m = mult * 2^32 - 1, represented in [1, m - 1].  Valid for 0 < word < m."""
    m = (mult << 32) - 1
    r = (word * pow(1 << 32, -k, m)) % m
    return r


# ---------------------------------------------------------------- numpy coding

class MWC(object):
    """All 12288 streams at once on uint64 lanes."""

    def __init__(self, mults, seed):
        self.mults = np.asarray(mults, dtype=np.uint64)
        assert self.mults.shape == (NUM_RND_STREAMS,)
        words = np.full(NUM_RND_STREAMS, ((int(seed) & MASK32) << 32) + 1, dtype=np.uint64)
        for _ in range(NUM_RND_BURNIN):
            words = self._step(words, self.mults)
        self.words = words

    @staticmethod
    def _step(words, mults):
        return mults * (words & np.uint64(MASK32)) + (words >> np.uint64(32))

    @staticmethod
    def _to_uniform(words):
        lo = (words & np.uint64(MASK32)).astype(np.uint32)
        return (lo.astype(np.float32) + np.float32(1.0)) / np.float32(4294967296.0)

    def uniform(self, n):
        """The n float32 values fill_with_rand writes (cudamat_kernels.cu:113-123)."""
        out = np.empty(n, dtype=np.float32)
        done = 0
        while done < n:
            cnt = min(NUM_RND_STREAMS, n - done)
            self.words[:cnt] = self._step(self.words[:cnt], self.mults[:cnt])
            out[done:done + cnt] = self._to_uniform(self.words[:cnt])
            done += cnt
        return out

    def raw_lo32(self, n):
        """Same schedule as uniform(), returning the low 32 bits instead."""
        out = np.empty(n, dtype=np.uint32)
        done = 0
        while done < n:
            cnt = min(NUM_RND_STREAMS, n - done)
            self.words[:cnt] = self._step(self.words[:cnt], self.mults[:cnt])
            out[done:done + cnt] = (self.words[:cnt] & np.uint64(MASK32)).astype(np.uint32)
            done += cnt
        return out

    def bernoulli(self, p):
        """sample_bernoulli (cudamat_kernels.cu:157-167): 1 where u < p, flat column-major p."""
        p = np.asarray(p, dtype=np.float32).ravel(order='F')
        return (self.uniform(p.size) < p).astype(np.float32)

    def bernoulli_tanh(self, x):
        """cudamat_kernels.cu:168-178: the comparison is made in double precision."""
        x = np.asarray(x, dtype=np.float32).ravel(order='F')
        u = self.uniform(x.size).astype(np.float64)
        return (u < (1.0 + x.astype(np.float64)) / 2.0).astype(np.float32)

    def dropout(self, x, dropprob, val):
        """cudamat_kernels.cu:145-155: keep where u > dropprob, else val."""
        x = np.asarray(x, dtype=np.float32).ravel(order='F')
        u = self.uniform(x.size)
        return np.where(u > np.float32(dropprob), x, np.float32(val)).astype(np.float32)

    def gaussian_pairs(self, n):
        """The uniform pairs (r1, r2) behind fill_with_randn and which elements they
        feed (cudamat_kernels.cu:125-143): returns (r1, r2, idx_cos, idx_sin) where
        idx_sin is -1 when i + 12288 falls outside."""
        r1s, r2s, ic, isn = [], [], [], []
        base = 0
        while base < n:
            cnt = min(NUM_RND_STREAMS, n - base)
            self.words[:cnt] = self._step(self.words[:cnt], self.mults[:cnt])
            r1 = self._to_uniform(self.words[:cnt])
            self.words[:cnt] = self._step(self.words[:cnt], self.mults[:cnt])
            r2 = self._to_uniform(self.words[:cnt])
            i = base + np.arange(cnt)
            i2 = i + NUM_RND_STREAMS
            r1s.append(r1); r2s.append(r2); ic.append(i); isn.append(np.where(i2 < n, i2, -1))
            base += 2 * NUM_RND_STREAMS
        return (np.concatenate(r1s), np.concatenate(r2s), np.concatenate(ic), np.concatenate(isn))

    def randn(self, n):
        """fill_with_randn in float64 math on the exact uniforms: Box-Muller
        R = sqrt(-2 ln r1), T = 2 pi r2, (R cos T, R sin T).  The device uses float32
        log/cos/sin, so this is a tolerance target, not a bit pattern."""
        r1, r2, ic, isn = self.gaussian_pairs(n)
        T = np.float32(2.0) * np.float32(3.1415926535897932) * r2  # float32 product as in the kernel
        R = np.sqrt(-2.0 * np.log(r1.astype(np.float64)))
        out = np.empty(n, dtype=np.float64)
        out[ic] = R * np.cos(T.astype(np.float64))
        ok = isn >= 0
        out[isn[ok]] = (R * np.sin(T.astype(np.float64)))[ok]
        return out
