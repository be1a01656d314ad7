"""GPU parity of the multiply-with-carry RNG against the host restatement:
uniform, Bernoulli and dropout outputs and the carried state are bit-exact."""
import ctypes as ct

import numpy as np
import pytest

from oracle import mwc

pytestmark = pytest.mark.gpu

N = mwc.NUM_RND_STREAMS


@pytest.fixture(scope="module")
def mults(cm):
    return mwc.load_multipliers(cm.MULTIPLIERS_PATH)


def _device_words(cm):
    """Read the 12288 state words back through a float32 view of the same bytes."""
    st = cm.CUDAMatrix.rnd_state
    view = cm.cudamat()
    view.data_device = ct.cast(st.dev_rnd_words, ct.POINTER(ct.c_float))
    view.on_device, view.on_host, view.is_trans, view.owns_data = 1, 0, 0, 0
    view.size[0], view.size[1] = 2 * N, 1
    m = cm.CUDAMatrix(view)
    return m.asarray().ravel(order='F').view(np.uint64).copy()


@pytest.mark.parametrize("seed", [0, 1, 42, 2**31 - 1])
def test_seed_state_matches_host(cm, mults, seed):
    cm.CUDAMatrix.init_random(seed)
    host = mwc.MWC(mults, seed)
    assert np.array_equal(_device_words(cm), host.words)


@pytest.mark.parametrize("shape", [(1, 1), (100, 5), (96, 128), (500, 100), (3 * N + 5, 1), (1031, 257),
                                   (33 * N + 7, 1), (31 * N + 12287, 1), (32 * N, 1), (200 * N + 4097, 1), (2049, 1537)])
def test_fill_with_rand_bit_exact_and_state_carries_over(cm, mults, shape):
    cm.CUDAMatrix.init_random(42)
    host = mwc.MWC(mults, 42)
    a = cm.empty(shape)
    for _ in range(2):   # second call continues every stream where the first stopped
        a.fill_with_rand()
        got = a.asarray().ravel(order='F')
        want = host.uniform(got.size)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(_device_words(cm), host.words)
    a.free_device_memory()


def test_uniform_range_includes_one_excludes_zero(cm):
    cm.CUDAMatrix.init_random(7)
    a = cm.empty((4096, 1024))
    a.fill_with_rand()
    x = a.asarray()
    assert x.min() > 0.0 and x.max() <= 1.0
    assert abs(x.mean() - 0.5) < 1e-3          # test_cudamat.py:882-887 uses 1e-2 on 128x256
    a.free_device_memory()


def test_sample_bernoulli_bit_exact(cm, mults, rng):
    cm.CUDAMatrix.init_random(1)
    host = mwc.MWC(mults, 1)
    p = np.asarray(rng.random((500, 100)), dtype=np.float32, order='F')
    a, t = cm.CUDAMatrix(p), cm.empty(p.shape)
    r = a.sample_bernoulli(target=t)
    assert r is a                                   # returns self, not target (cudamat.py:481)
    want = host.bernoulli(p).reshape(p.shape, order='F')
    assert np.array_equal(t.asarray(), want)
    assert np.array_equal(a.asarray(), p)
    a.sample_bernoulli()                            # in place
    want2 = host.bernoulli(p).reshape(p.shape, order='F')
    assert np.array_equal(a.asarray(), want2)
    assert np.array_equal(_device_words(cm), host.words)


def test_dropout_and_bernoulli_tanh_bit_exact(cm, mults, rng):
    cm.CUDAMatrix.init_random(3)
    host = mwc.MWC(mults, 3)
    x = np.asarray(rng.uniform(-1, 1, (1024, 128)), dtype=np.float32, order='F')
    a = cm.CUDAMatrix(x)
    a.dropout(0.5, val=-7.0)
    assert np.array_equal(a.asarray(), host.dropout(x, 0.5, -7.0).reshape(x.shape, order='F'))
    b, t = cm.CUDAMatrix(x), cm.empty(x.shape)
    b.sample_bernoulli_tanh(target=t)
    assert np.array_equal(t.asarray(), host.bernoulli_tanh(x).reshape(x.shape, order='F'))
    b.sample_poisson(target=t)                      # placeholder op: copies, but consumes one draw each
    host.uniform(x.size)
    assert np.array_equal(t.asarray(), x)
    assert np.array_equal(_device_words(cm), host.words)


def test_deepnet_dropout_mask_sequence(cm, mults):
    """neuralnet.py:194-198 builds the mask as fill_with_rand -> greater_than(p) -> mult."""
    cm.CUDAMatrix.init_random(5)
    host = mwc.MWC(mults, 5)
    state = np.ones((1024, 128), dtype=np.float32, order='F')
    s, mask = cm.CUDAMatrix(state), cm.empty(state.shape)
    mask.fill_with_rand()
    mask.greater_than(0.5)
    s.mult(mask)
    want = (host.uniform(state.size) > np.float32(0.5)).astype(np.float32).reshape(state.shape, order='F')
    assert np.array_equal(s.asarray(), want)


# from 31 elements per stream on, lanes share a stream (parts of whole pairs); odd element
# counts leave a last pair with one element that still takes two draws
@pytest.mark.parametrize("n", [1, N, N + 1, 2 * N, 2 * N + 3, 5 * N + 17, 30 * N + 1, 31 * N + 7, 33 * N, 40 * N + 5,
                               257 * N + 4321])
def test_fill_with_randn_matches_box_muller_of_exact_uniforms(cm, mults, n):
    cm.CUDAMatrix.init_random(9)
    host = mwc.MWC(mults, 9)
    a = cm.empty((n, 1))
    a.fill_with_randn()
    got = a.asarray().ravel().astype(np.float64)
    want = host.randn(n)
    # float32 log/sqrt/cos/sin of exact uniforms: absolute error a few 1e-6 at |x| <= 6.7
    assert np.max(np.abs(got - want)) < 2e-5
    assert np.array_equal(_device_words(cm), host.words)


def test_randn_moments_and_sample_gaussian(cm, mults):
    cm.CUDAMatrix.init_random(11)
    host = mwc.MWC(mults, 11)
    a = cm.empty((2048, 512))
    a.fill_with_randn()
    x = a.asarray()
    assert abs(x.mean()) < 5e-3 and abs(x.std() - 1.0) < 5e-3
    host.randn(x.size)
    base = np.full((300, 70), 2.0, dtype=np.float32, order='F')
    b, t = cm.CUDAMatrix(base), cm.empty(base.shape)
    b.sample_gaussian(mult=0.5, target=t)
    want = 2.0 + 0.5 * host.randn(base.size).reshape(base.shape, order='F')
    assert np.max(np.abs(t.asarray() - want)) < 2e-5
    # the same on the schedule that shares a stream among lanes, ragged at the end
    big = np.asarray(np.arange(1031 * 613) % 17, dtype=np.float32).reshape((1031, 613), order='F')
    b, t = cm.CUDAMatrix(big), cm.empty(big.shape)
    b.sample_gaussian(mult=0.25, target=t)
    want = big + 0.25 * host.randn(big.size).reshape(big.shape, order='F')
    assert np.max(np.abs(t.asarray() - want)) < 2e-5
    assert np.array_equal(_device_words(cm), host.words)


def test_perturb_ops(cm, mults, rng):
    cm.CUDAMatrix.init_random(13)
    host = mwc.MWC(mults, 13)
    x = np.asarray(rng.uniform(0.1, 2, (200, 50)), dtype=np.float32, order='F')
    a, t = cm.CUDAMatrix(x), cm.empty(x.shape)
    a.perturb_energy_for_softmax_sampling(target=t)
    u = host.uniform(x.size).astype(np.float64).reshape(x.shape, order='F')
    with np.errstate(divide='ignore'):
        want = x - np.log(-np.log(u))
    ok = u < 1.0
    assert np.allclose(t.asarray()[ok], want[ok], rtol=2e-5, atol=2e-5)
    a.perturb_prob_for_softmax_sampling(target=t)
    u = host.uniform(x.size).astype(np.float64).reshape(x.shape, order='F')
    ok = u < 1.0
    assert np.allclose(t.asarray()[ok], (-x / np.log(u))[ok], rtol=2e-5)


def test_full_size_4096_uniform_and_bernoulli(cm, mults, rng):
    """The benchmark size: 1366 draws per stream.  Bit-exact against the host."""
    cm.CUDAMatrix.init_random(2)
    host = mwc.MWC(mults, 2)
    n = 4096
    a = cm.empty((n, n))
    a.fill_with_rand()
    got = a.asarray().ravel(order='F')
    assert np.array_equal(got.view(np.uint32), host.uniform(n * n).view(np.uint32))
    p = np.asarray(rng.random((n, n)), dtype=np.float32, order='F')
    b = cm.CUDAMatrix(p)
    b.sample_bernoulli(target=a)
    assert np.array_equal(a.asarray().ravel(order='F'), host.bernoulli(p))
    assert np.array_equal(_device_words(cm), host.words)
    a.free_device_memory(); b.free_device_memory()


@pytest.mark.parametrize("n,offset", [(40 * N + 4 * 777, 0), (33 * N + 8, 0), (64 * N, 0), (40 * N + 4 * 777, 1),
                                      (35 * N + 6, 0)])
def test_bernoulli_and_dropout_on_the_four_streams_per_lane_schedule(cm, mults, rng, n, offset):
    """Calls with a source array, a multiple of 4 elements and 16-byte alignment take the
    schedule with four streams per lane; element counts that leave the last draw ragged,
    a view that starts one float off alignment, and a count that is not a multiple of 4
    must all give the host's stream and state, call after call."""
    cm.CUDAMatrix.init_random(5)
    host = mwc.MWC(mults, 5)
    p = np.asarray(rng.random((n + offset, 1)), dtype=np.float32, order='F')
    P, T = cm.CUDAMatrix(p), cm.empty((n + offset, 1))
    src, dst = P.slice(offset, n + offset), T.slice(offset, n + offset)
    for _ in range(2):
        src.sample_bernoulli(target=dst)
        assert np.array_equal(dst.asarray().ravel(), host.bernoulli(p[offset:, 0]))
        assert np.array_equal(_device_words(cm), host.words)
    src.dropout(0.3, val=2.5)
    assert np.array_equal(src.asarray().ravel(), host.dropout(p[offset:, 0], 0.3, 2.5))
    assert np.array_equal(_device_words(cm), host.words)
    P.free_device_memory(); T.free_device_memory()


def test_sampler_error_codes(cm, rng):
    a = cm.CUDAMatrix(np.zeros((4, 4), dtype=np.float32))
    with pytest.raises(cm.CUDAMatException, match="Incompatible matrix dimensions"):
        a.sample_bernoulli(target=cm.empty((4, 5)))
    host_only = cm.CUDAMatrix(np.zeros((4, 4), dtype=np.float32), copy_to_device=False)
    with pytest.raises(cm.CUDAMatException, match="not in device memory"):
        host_only.fill_with_rand()


def test_recorded_draws_and_eager_calls_share_one_sequence(cm, mults):
    """A recorded graph carries the address of the state words it draws from.  Calls that
    move the state to the other buffer (large matrices, the sample of dot_bias_act) must
    leave it where the graph finds it: replays and eager calls interleave like eager calls."""
    cm.CUDAMatrix.init_random(21)
    host = mwc.MWC(mults, 21)
    small, big = cm.empty((300, 40)), cm.empty((1024, 512))
    small.fill_with_rand(); host.uniform(small.shape[0] * small.shape[1])
    with cm.Graph() as g:
        small.fill_with_rand()
    for step in range(3):
        g.launch()
        want = host.uniform(small.shape[0] * small.shape[1])
        assert np.array_equal(small.asarray().ravel(order='F').view(np.uint32), want.view(np.uint32)), step
        big.fill_with_rand()                                  # the split schedule
        want = host.uniform(big.shape[0] * big.shape[1])
        assert np.array_equal(big.asarray().ravel(order='F').view(np.uint32), want.view(np.uint32)), step
        # a product that draws the sample of its own output
        w = cm.CUDAMatrix(np.zeros((64, 96), dtype=np.float32)); v = cm.CUDAMatrix(np.ones((64, 100), dtype=np.float32))
        h, hs = cm.empty((96, 100)), cm.empty((96, 100))
        cm.dot_bias_act(w.T, v, None, target=h, act='sigmoid', sample=hs)
        u = host.uniform(96 * 100).reshape((96, 100), order='F')
        assert np.array_equal(hs.asarray(), (u < np.float32(0.5)).astype(np.float32)), step
        here = ct.cast(cm.CUDAMatrix.rnd_state.dev_rnd_words, ct.c_void_p).value
        big.fill_with_randn(); host.randn(big.shape[0] * big.shape[1])
        assert ct.cast(cm.CUDAMatrix.rnd_state.dev_rnd_words, ct.c_void_p).value == here      # the state stays put
    assert np.array_equal(_device_words(cm), host.words)
    g.free()
    # no graph is left: the next large call moves the state to the other buffer again
    here = ct.cast(cm.CUDAMatrix.rnd_state.dev_rnd_words, ct.c_void_p).value
    big.fill_with_rand()
    want = host.uniform(big.shape[0] * big.shape[1])
    assert np.array_equal(big.asarray().ravel(order='F').view(np.uint32), want.view(np.uint32))
    assert ct.cast(cm.CUDAMatrix.rnd_state.dev_rnd_words, ct.c_void_p).value != here
    assert np.array_equal(_device_words(cm), host.words)


def test_large_draws_are_recorded_too(cm, mults):
    """Matrices large enough for the schedule that shares a stream among lanes (and the sample
    of dot_bias_act) record like the small ones: every replay continues the host's sequence."""
    cm.CUDAMatrix.init_random(33)
    host = mwc.MWC(mults, 33)
    big, drop = cm.empty((1024, 512)), cm.CUDAMatrix(np.ones((700, 600), dtype=np.float32))
    gauss = cm.empty((512, 1024))
    w = cm.CUDAMatrix(np.zeros((64, 512), dtype=np.float32)); v = cm.CUDAMatrix(np.ones((64, 1024), dtype=np.float32))
    h, hs = cm.empty((512, 1024)), cm.empty((512, 1024))
    with cm.Graph() as g:
        big.fill_with_rand()
        drop.dropout(0.5)
        cm.dot_bias_act(w.T, v, None, target=h, act='sigmoid', sample=hs)
        gauss.fill_with_randn()
    keep = np.ones((700, 600), dtype=np.float32)
    for step in range(3):
        g.launch()
        want = host.uniform(big.shape[0] * big.shape[1])
        assert np.array_equal(big.asarray().ravel(order='F').view(np.uint32), want.view(np.uint32)), step
        keep *= (host.uniform(700 * 600) > np.float32(0.5)).astype(np.float32).reshape((700, 600), order='F')
        assert np.array_equal(drop.asarray(), keep), step
        u = host.uniform(512 * 1024).reshape((512, 1024), order='F')
        assert np.array_equal(hs.asarray(), (u < np.float32(0.5)).astype(np.float32)), step
        want = host.randn(512 * 1024)
        assert np.max(np.abs(gauss.asarray().ravel(order='F') - want)) < 2e-5, step
        if step == 1:
            big.fill_with_rand(); host.uniform(big.shape[0] * big.shape[1])      # an eager call in between
    assert np.array_equal(_device_words(cm), host.words)
    g.free()
