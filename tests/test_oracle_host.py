"""CPU-only: the C host restatement (the CPU baseline of the benchmark) against
numpy float64."""
import ctypes as ct
import os

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FP = ct.POINTER(ct.c_float)


@pytest.fixture(scope="module")
def lib():
    return ct.CDLL(os.path.join(ROOT, 'oracle', 'liboracle_host.so'))


def p(a):
    return a.ctypes.data_as(FP)


def f(rng, shape):
    return np.asarray(rng.standard_normal(shape), dtype=np.float32, order='F')


@pytest.mark.parametrize("threads", [1, 4])
@pytest.mark.parametrize("ta,tb", [(0, 0), (1, 0), (0, 1), (1, 1)])
def test_gemm(lib, rng, ta, tb, threads):
    m, n, k = 67, 45, 301
    A, B, C = f(rng, (m, k)), f(rng, (k, n)), f(rng, (m, n))
    As = np.asfortranarray(A.T) if ta else A
    Bs = np.asfortranarray(B.T) if tb else B
    want = -0.5 * C.astype(np.float64) + 1.5 * (A.astype(np.float64) @ B)
    lib.hb_set_threads(threads)
    lib.hb_gemm(ta, tb, m, n, k, ct.c_float(1.5), p(As), As.shape[0], p(Bs), Bs.shape[0], ct.c_float(-0.5), p(C), m)
    lib.hb_set_threads(1)
    assert np.allclose(C, want, rtol=1e-4, atol=1e-4)


def test_elementwise_and_reductions(lib, rng):
    h, w = 33, 21
    A, B = f(rng, (h, w)), f(rng, (h, w))
    T = np.empty_like(A)
    n = ct.c_size_t(A.size)
    lib.hb_sigmoid(p(A), p(T), n); assert np.allclose(T, 1 / (1 + np.exp(-A.astype(np.float64))), rtol=1e-6)
    lib.hb_exp(p(A), p(T), n); assert np.allclose(T, np.exp(A.astype(np.float64)), rtol=1e-6)
    lib.hb_mult(p(A), p(B), p(T), n); assert np.array_equal(T, A * B)
    A2 = A.copy(order='F'); lib.hb_add_mult(p(A2), p(B), ct.c_float(0.25), n); assert np.allclose(A2, A + 0.25 * B, rtol=1e-6, atol=1e-6)
    col, row = f(rng, (h,)), f(rng, (w,))
    lib.hb_add_col_vec(p(A), p(col), p(T), h, w); assert np.array_equal(T, A + col[:, None])
    lib.hb_mult_by_col(p(A), p(col), p(T), h, w); assert np.array_equal(T, A * col[:, None])
    lib.hb_add_row_vec(p(A), p(row), p(T), h, w); assert np.array_equal(T, A + row[None, :])
    r0, r1 = np.ones(w, np.float32), np.ones(h, np.float32)
    lib.hb_add_sums(p(A), p(r0), h, w, 0, ct.c_float(2.0), ct.c_float(-1.0))
    assert np.allclose(r0, 2 - A.astype(np.float64).sum(axis=0), rtol=1e-5, atol=1e-5)
    lib.hb_add_sums(p(A), p(r1), h, w, 1, ct.c_float(0.0), ct.c_float(1.0))
    assert np.allclose(r1, A.astype(np.float64).sum(axis=1), rtol=1e-5, atol=1e-5)
    lib.hb_max(p(A), p(r0), h, w, 0); assert np.array_equal(r0, A.max(axis=0))
    lib.hb_max(p(A), p(r1), h, w, 1); assert np.array_equal(r1, A.max(axis=1))
    lib.hb_softmax(p(A), p(T), h, w)
    e = np.exp(A.astype(np.float64) - A.max(axis=0)); assert np.allclose(T, e / e.sum(axis=0), rtol=1e-5)


def test_rbm_step_matches_a_numpy_evaluation(lib, rng):
    from oracle import mwc
    nv, nh, B, lr = 40, 24, 10, 0.1
    mults = mwc.load_multipliers(os.path.join(ROOT, 'deepnet_amd', 'rnd_multipliers_32bit.txt'))
    words = np.empty(mwc.NUM_RND_STREAMS, dtype=np.uint64)
    u32 = mults.ctypes.data_as(ct.POINTER(ct.c_uint32)); u64 = words.ctypes.data_as(ct.POINTER(ct.c_uint64))
    lib.mwc_seed(u32, u64, ct.c_uint32(1))
    host = mwc.MWC(mults, 1)
    v = np.asarray(rng.random((nv, B)) < 0.3, dtype=np.float32, order='F')
    W = f(rng, (nv, nh)) * np.float32(0.1)
    bv, bh = f(rng, (nv,)) * np.float32(0.1), f(rng, (nh,)) * np.float32(0.1)
    W0, bv0, bh0 = W.astype(np.float64), bv.astype(np.float64), bh.astype(np.float64)
    h, hs, h2 = (np.empty((nh, B), np.float32, order='F') for _ in range(3))
    v2 = np.empty((nv, B), np.float32, order='F')
    lib.hb_rbm_cd1_step(p(W), p(bv), p(bh), p(v), nv, nh, B, ct.c_float(lr), u32, u64, p(h), p(hs), p(v2), p(h2))
    sig = lambda z: 1 / (1 + np.exp(-z))
    hh = sig(W0.T @ v + bh0[:, None])
    assert np.allclose(h, hh, rtol=1e-5)
    s = host.bernoulli(h).reshape((nh, B), order='F')
    assert np.array_equal(hs, s)
    vv = sig(W0 @ s + bv0[:, None]); hh2 = sig(W0.T @ vv + bh0[:, None])
    eps = lr / B
    assert np.allclose(W, W0 + eps * (v @ hh.T - vv @ hh2.T), rtol=1e-4, atol=1e-6)
    assert np.allclose(bv, bv0 + eps * (v.sum(axis=1) - vv.sum(axis=1)), rtol=1e-4, atol=1e-6)
    assert np.allclose(bh, bh0 + eps * (hh.sum(axis=1) - hh2.sum(axis=1)), rtol=1e-4, atol=1e-6)


def test_mlp_step_matches_the_float64_net_oracle(lib, rng):
    """hb_mlp_step (the CPU baseline of the MLP benchmark step) against oracle/net_oracle.py,
    itself pinned by torch SGD, fed the dropout masks the C code drew; and the masks against
    the host generator."""
    import sys
    sys.path.insert(0, ROOT)
    from oracle import host_steps, mwc, net_oracle as no
    sizes, B, lr, mom = (20, 16, 12, 5), 8, 0.1, 0.9
    x = rng.random((sizes[0], B))
    labels = rng.integers(0, sizes[-1], B)
    W = [0.3 * rng.standard_normal((sizes[i], sizes[i + 1])) for i in range(3)]
    b = [0.1 * rng.standard_normal(sizes[i + 1]) for i in range(3)]
    m = host_steps.HostMLP(lib, sizes, B, x, labels, W, b, lr, mom, seed=5)
    hyp = lambda **kw: no.Hyper(base_epsilon=lr, initial_momentum=mom, final_momentum=mom, **kw)
    layers = [{'act': 'LINEAR', 'hyper': hyp()}]
    for i, act in enumerate(('RECTIFIED_LINEAR', 'RECTIFIED_LINEAR', 'SOFTMAX')):
        layers.append({'act': act, 'hyper': hyp(dropout=i < 2), 'bias': m.b[i].copy(),
                       'edge': {'w': m.W[i].copy(), 'hyper': hyp()}, 'loss': 'CROSS_ENTROPY'})
    onet = no.Net(layers)
    host = mwc.MWC(m.mults, 5)
    x32 = m.act[0].astype(np.float64)
    for step in range(3):
        m.step()
        for k in range(2):
            u = host.uniform(sizes[k + 1] * B).reshape((sizes[k + 1], B), order='F')
            assert np.array_equal(m.mask[k], (u > np.float32(0.5)).astype(np.float32))
        perf = onet.train_step(x32, labels.reshape(1, -1), step, masks=[None, m.mask[0], m.mask[1], None])
        assert abs(float(m.loss.sum()) - perf['cross_entropy']) <= 1e-5 * perf['cross_entropy']
        for i in range(3):
            L = onet.layers[i + 1]
            assert np.allclose(m.W[i], L['edge']['w'], rtol=1e-4, atol=1e-6)
            assert np.allclose(m.b[i], L['bias'].ravel(), rtol=1e-4, atol=1e-6)
