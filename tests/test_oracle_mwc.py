"""CPU-only pins of the RNG restatement: three independent codings (Python
integers, numpy uint64, C) agree with each other and with the committed known
answers; the algebra behind jump-ahead holds for every multiplier."""
import ctypes as ct
import hashlib
import json
import os

import numpy as np
import pytest

from oracle import mwc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
MULT_PATH = os.path.join(ROOT, 'deepnet_amd', 'rnd_multipliers_32bit.txt')
N = mwc.NUM_RND_STREAMS


@pytest.fixture(scope="module")
def mults():
    return mwc.load_multipliers(MULT_PATH)


@pytest.fixture(scope="module")
def kat():
    return json.load(open(os.path.join(ROOT, 'tests', 'golden', 'mwc_kat.json')))


@pytest.fixture(scope="module")
def clib():
    lib = ct.CDLL(os.path.join(ROOT, 'oracle', 'liboracle_host.so'))
    return lib


def _c_state(clib, mults, seed):
    words = np.empty(N, dtype=np.uint64)
    clib.mwc_seed(mults.ctypes.data_as(ct.POINTER(ct.c_uint32)), words.ctypes.data_as(ct.POINTER(ct.c_uint64)),
                  ct.c_uint32(seed))
    return words


def test_multiplier_table_is_the_reference_file(mults, kat):
    assert hashlib.md5(open(MULT_PATH, 'rb').read()).hexdigest() == kat['multipliers_md5'] \
        == '7f319b3a31c32456281d1f8d8e604202'
    assert mults[0] == 4294967118 and mults.dtype == np.uint32 and mults.shape == (N,)


@pytest.mark.parametrize("seed", [0, 1, 42])
def test_three_codings_agree_on_known_answers(mults, kat, clib, seed):
    host = mwc.MWC(mults, seed)
    cwords = _c_state(clib, mults, seed)
    assert np.array_equal(host.words, cwords)
    for stream in (0, 1, 12287):
        e = kat['streams']['%d:%d' % (seed, stream)]
        assert int(mults[stream]) == e['mult']
        assert mwc.seed_word_py(seed, e['mult']) == e['seeded_word'] == int(host.words[stream])
    # four whole rounds of draws
    raw = host.uniform(4 * N).reshape(4, N)
    cout = np.empty(4 * N, dtype=np.float32)
    clib.mwc_uniform(mults.ctypes.data_as(ct.POINTER(ct.c_uint32)), cwords.ctypes.data_as(ct.POINTER(ct.c_uint64)),
                     cout.ctypes.data_as(ct.POINTER(ct.c_float)), ct.c_size_t(4 * N))
    assert np.array_equal(raw.ravel().view(np.uint32), cout.view(np.uint32))
    assert np.array_equal(host.words, cwords)
    for stream in (0, 1, 12287):
        e = kat['streams']['%d:%d' % (seed, stream)]
        assert [int(v) for v in raw[:, stream].view(np.uint32)] == e['draw_uniform_bits']
        assert int(host.words[stream]) == e['draw_words'][3]


def test_whole_call_with_ragged_length_and_state_carry(mults, kat, clib):
    k = kat['fill_seed42']
    host = mwc.MWC(mults, 42)
    out = host.uniform(k['n'])
    assert hashlib.sha256(out.tobytes()).hexdigest() == k['sha256']
    assert [int(v) for v in out[:8].view(np.uint32)] == k['first8_bits']
    assert [int(v) for v in out[-8:].view(np.uint32)] == k['last8_bits']
    assert hashlib.sha256(host.words.tobytes()).hexdigest() == k['state_sha256']
    # streams 0..4 took four draws, the others three
    ref = mwc.MWC(mults, 42)
    for _ in range(3):
        ref.words = ref._step(ref.words, ref.mults)
    assert np.array_equal(host.words[5:], ref.words[5:])
    assert np.array_equal(host.words[:5], ref._step(ref.words, ref.mults)[:5])
    # two calls == one call of the summed length only when the first is a multiple of 12288
    a = mwc.MWC(mults, 42); b = mwc.MWC(mults, 42)
    x = np.concatenate([a.uniform(2 * N), a.uniform(100)])
    assert np.array_equal(x, b.uniform(2 * N + 100))
    # C coding, ragged length, then Bernoulli and dropout on the carried state
    cwords = _c_state(clib, mults, 42)
    cout = np.empty(k['n'], dtype=np.float32)
    u32 = mults.ctypes.data_as(ct.POINTER(ct.c_uint32)); u64 = cwords.ctypes.data_as(ct.POINTER(ct.c_uint64))
    clib.mwc_uniform(u32, u64, cout.ctypes.data_as(ct.POINTER(ct.c_float)), ct.c_size_t(k['n']))
    assert hashlib.sha256(cout.tobytes()).hexdigest() == k['sha256']
    p = np.random.default_rng(0).random(5000).astype(np.float32)
    cb = np.empty_like(p)
    clib.mwc_bernoulli(u32, u64, p.ctypes.data_as(ct.POINTER(ct.c_float)), cb.ctypes.data_as(ct.POINTER(ct.c_float)),
                       ct.c_size_t(p.size))
    assert np.array_equal(cb, host.bernoulli(p))
    d = p.copy()
    clib.mwc_dropout(u32, u64, d.ctypes.data_as(ct.POINTER(ct.c_float)), ct.c_size_t(d.size), ct.c_float(0.3),
                     ct.c_float(-1.0))
    assert np.array_equal(d, host.dropout(p, 0.3, -1.0))
    assert np.array_equal(host.words, cwords)


def test_uniform_map_edge_cases():
    # lo = 2^32 - 1 converts to 2^32 (round to nearest even), +1 is absorbed: exactly 1.0
    assert mwc.uniform_py(0xFFFFFFFF) == np.float32(1.0)
    assert mwc.uniform_py(0) == np.float32(2.0 ** -32)
    # 2^32 - 129 is 127 above 2^32 - 256 and 129 below 2^32 (float32 spacing there is 256)
    assert mwc.uniform_py(0x12345678FFFFFF7F) == np.float32(4294967040.0 / 4294967296.0)
    # conversion ties go to even: 2^24 + 1 -> 2^24, 2^24 + 3 -> 2^24 + 4
    assert mwc.uniform_py((1 << 24) + 1) == (np.float32(1 << 24) + np.float32(1)) / np.float32(2.0 ** 32)
    assert mwc.uniform_py((1 << 24) + 3) == (np.float32((1 << 24) + 4) + np.float32(1)) / np.float32(2.0 ** 32)


def test_step_is_division_by_2_32_modulo_m_for_every_multiplier(mults):
    rng = np.random.default_rng(5)
    for t in range(N):
        a = int(mults[t])
        m = (a << 32) - 1
        w = int(rng.integers(1, 1 << 62)) % m or 1
        w2 = mwc.step_py(w, a)
        assert (w2 << 32) == m * (w & 0xFFFFFFFF) + w          # exact identity
        assert w2 == (w * pow(1 << 32, -1, m)) % m and 0 < w2 < m


@pytest.mark.parametrize("k", [1, 2, 7, 64, 1366, 12345])
def test_jump_ahead_equals_k_steps(mults, k):
    for t in (0, 1, 777, 12287):
        a = int(mults[t])
        for seed in (0, 1, 42, 2 ** 31 - 1):
            w = mwc.seed_word_py(seed, a)
            s = w
            for _ in range(k):
                s = mwc.step_py(s, a)
            assert mwc.jump_py(w, a, k) == s


def test_statistics_like_the_reference_test(mults):
    # cudamat/test_cudamat.py:882-893: |mean(U) - 0.5| < 1e-2 and |mean(N)| < 1e-2 on 128 x 256 after init_random(1)
    host = mwc.MWC(mults, 1)
    assert abs(host.uniform(128 * 256).mean() - 0.5) < 1e-2
    z = host.randn(128 * 256)
    assert abs(z.mean()) < 1e-2 and abs(z.std() - 1) < 2e-2
