"""Matrices beyond 2^30 elements / 2^32 bytes and conv outputs beyond 2^31 and 2^32 bytes.

A float64 pass over such sizes would take minutes, so every check here is one the size does
not enter: an outer product v r^T has sums, maxima, transposes and products in closed form;
element-wise results are compared on probe columns (first, middle, last); the random streams
are checked by jumping the host streams ahead; conv outputs are checked one output at a time
against the definition.  What these sizes exercise is the 64-bit address arithmetic of the
kernels and the dispatch limits of the ones that use 32-bit offsets.
"""
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from oracle import conv_oracle as co   # noqa: E402
from oracle import mwc                 # noqa: E402

pytestmark = pytest.mark.gpu

H, W = 40960, 28001            # 1 146 920 960 elements, 4.59 GB: above 2^30 elements and 2^32 bytes
PROBES = (0, 1, W // 2, 16383, 26215, W - 2, W - 1)   # 26215 * H * 4 straddles 2^32 bytes


def _f(a):
    return np.asarray(a, dtype=np.float32, order='F')


def _cols(mat, cols=PROBES):
    """Host copies of single columns of a device matrix."""
    out = {}
    for c in cols:
        view = mat.slice(c, c + 1)
        out[c] = view.asarray().ravel().copy()
    return out


@pytest.fixture(scope="module")
def outer(cm):
    """a = v r^T on the device with positive v (H x 1) and r (1 x W), built by the
    broadcast kernels themselves."""
    r_ = np.random.default_rng(77)
    v = _f(r_.uniform(0.5, 1.5, (H, 1)))
    r = _f(r_.uniform(0.5, 1.5, (1, W)))
    a = cm.empty((H, W))
    a.assign(0.0)
    V, R = cm.CUDAMatrix(v), cm.CUDAMatrix(r)
    a.add_col_vec(V)
    a.mult_by_row(R)
    yield a, v.ravel(), r.ravel(), V, R
    for m in (a, V, R):
        m.free_device_memory()


def test_broadcasts_build_the_outer_product_exactly(cm, outer):
    a, v, r, V, R = outer
    for c, col in _cols(a).items():
        assert np.array_equal(col, v * r[c]), c


def test_sums_and_maxima_along_both_axes(cm, outer):
    a, v, r, V, R = outer
    v64, r64 = v.astype(np.float64), r.astype(np.float64)
    s0 = a.sum(axis=0).asarray().ravel()
    assert s0.shape == (W,)
    assert np.allclose(s0, r64 * v64.sum(), rtol=1e-5, atol=0)
    s1 = a.sum(axis=1).asarray().ravel()
    assert np.allclose(s1, v64 * r64.sum(), rtol=1e-5, atol=0)
    # fl(v * r) is monotone in each factor for positive factors: the maxima are exact
    m0 = a.max(axis=0).asarray().ravel()
    assert np.array_equal(m0, v.max() * r)
    m1 = a.max(axis=1).asarray().ravel()
    assert np.array_equal(m1, v * r.max())
    q0 = a.sqsum(axis=0).asarray().ravel()
    assert np.allclose(q0, (r64 ** 2) * (v64 ** 2).sum(), rtol=1e-5, atol=0)
    assert np.array_equal(a.argmax(axis=0).asarray().ravel(), np.full(W, float(np.argmax(v)), dtype=np.float32))
    # everything at once: (sum v)(sum r) through the flat dot product with ones is refused
    # above 2^18 elements by the reference's own sum(axis=None); the norm is not
    assert abs(a.euclid_norm() - np.sqrt((v64 ** 2).sum() * (r64 ** 2).sum())) < 1e-5 * np.sqrt((v64 ** 2).sum() * (r64 ** 2).sum())


def test_transpose_and_products_with_a_large_operand(cm, outer):
    a, v, r, V, R = outer
    v64, r64 = v.astype(np.float64), r.astype(np.float64)
    t = a.transpose()
    assert t.shape == (W, H)
    for c, col in _cols(t, (0, 1, H // 2, 38347, H - 1)).items():   # 38347 * W * 4 straddles 2^32 bytes
        assert np.array_equal(col, v[c] * r), c
    t.free_device_memory()
    g = np.random.default_rng(78)
    for n in (1, 8, 128):
        x = _f(g.standard_normal((H, n)))
        y = _f(g.standard_normal((W, n)))
        X, Y = cm.CUDAMatrix(x), cm.CUDAMatrix(y)
        # a^T x = r (v^T x): reduction over 40960, 28001 output rows taken from all of a
        got = cm.dot(a.T, X).asarray()
        want = np.outer(r64, v64 @ x.astype(np.float64))
        scale = np.outer(r64, np.abs(v64) @ np.abs(x).astype(np.float64))
        assert np.all(np.abs(got - want) <= 1e-4 * scale + 1e-30), n
        # a y = v (r^T y)
        got = cm.dot(a, Y).asarray()
        want = np.outer(v64, r64 @ y.astype(np.float64))
        scale = np.outer(v64, np.abs(r64) @ np.abs(y).astype(np.float64))
        assert np.all(np.abs(got - want) <= 1e-4 * scale + 1e-30), n
        X.free_device_memory(); Y.free_device_memory()
    # the weight-gradient shape: a large product written over all of a big target
    k = 16
    p = _f(g.standard_normal((H, k)))
    q = _f(g.standard_normal((k, W)))
    P, Q = cm.CUDAMatrix(p), cm.CUDAMatrix(q)
    big = cm.empty((H, W))
    cm.dot(P, Q, target=big)
    p64, q64 = p.astype(np.float64), q.astype(np.float64)
    for c, col in _cols(big).items():
        assert np.all(np.abs(col - p64 @ q64[:, c]) <= 1e-4 * (np.abs(p64) @ np.abs(q64[:, c])) + 1e-30), c
    big.add_dot(P, Q, mult=-1.0)           # beta = 1 path over the same target
    for c, col in _cols(big).items():
        assert np.all(np.abs(col) <= 2e-4 * (np.abs(p64) @ np.abs(q64[:, c])) + 1e-30), c
    for m in (P, Q, big):
        m.free_device_memory()


def test_elementwise_and_softmax_on_probe_columns(cm, outer):
    a, v, r, V, R = outer
    b = cm.empty((H, W))
    b.assign(a)
    before = _cols(b)
    for c in PROBES:
        assert np.array_equal(before[c], v * r[c])
    b.add_mult(a, -0.25)                       # b = a - 0.25 a
    b.mult(a)                                  # b = (0.75 a) a
    b.apply_sigmoid()
    got = _cols(b)
    for c in PROBES:
        s = (before[c] + np.float32(-0.25) * before[c]).astype(np.float32) * before[c]
        want = 1.0 / (1.0 + np.exp(-s.astype(np.float64)))
        assert np.allclose(got[c], want, rtol=2.5e-7, atol=0), c
    b.assign(a)
    b.apply_softmax()
    got = _cols(b)
    for c in PROBES:
        x = before[c].astype(np.float64)
        e = np.exp(x - x.max())
        assert np.allclose(got[c], e / e.sum(), rtol=2e-6, atol=0), c
    b.add_row_vec(R)
    got2 = _cols(b)
    for c in PROBES:
        assert np.array_equal(got2[c], got[c] + r[c]), c
    b.free_device_memory()


def test_random_streams_on_a_large_matrix_match_the_jumped_host_streams(cm):
    mults = mwc.load_multipliers(cm.MULTIPLIERS_PATH)
    seed = 9
    cm.CUDAMatrix.init_random(seed)
    host = mwc.MWC(mults, seed)
    start = [int(w) for w in host.words]
    n = H * W
    S = mwc.NUM_RND_STREAMS
    a = cm.empty((H, W))
    a.fill_with_rand()
    flat = a.reshape((n, 1))
    # first two rounds of draws
    head = flat.slice(0, 2 * S).asarray().ravel()
    assert np.array_equal(head.view(np.uint32), host.uniform(2 * S).view(np.uint32))
    # last rounds: jump every stream to two draws before its end, then step
    rounds = (n + S - 1) // S
    tail_from = (rounds - 3) * S
    words = np.array([mwc.jump_py(start[i], int(mults[i]), rounds - 3) for i in range(S)], dtype=np.uint64)
    host.words = words
    want = host.uniform(n - tail_from)
    tail = flat.slice(tail_from, n).asarray().ravel()
    assert np.array_equal(tail.view(np.uint32), want.view(np.uint32))
    a.reshape((H, W))
    # Bernoulli over the same size, against probabilities read back on probe ranges
    p = cm.empty((H, W))
    p.assign(0.5)
    p.sample_bernoulli(target=a)
    mean = a.sum(axis=0).asarray().ravel().astype(np.float64).sum() / n
    assert abs(mean - 0.5) < 1e-3
    a.free_device_memory(); p.free_device_memory()
    cm.CUDAMatrix.init_random(1)


@pytest.mark.parametrize("N", [8320, 16512])   # convUp output: 2.18 GB (32-bit offsets still fit) and 4.33 GB (they do not)
def test_conv_passes_with_outputs_beyond_32_bit_byte_offsets(cm, cc, N):
    C, Hh, F, k, s, p, G = 3, 32, 64, 5, 1, 2, 1
    Mx = co.n_modules(Hh, k, s, p)
    r = np.random.default_rng(N)
    x = _f(r.standard_normal((C * Hh * Hh, N), dtype=np.float32).T)
    w = _f(0.05 * r.standard_normal((F, C * k * k)))
    X, Wm = cm.CUDAMatrix(x), cm.CUDAMatrix(w)
    Y = cm.empty((N, F * Mx * Mx))
    Y.fill_with_randn()
    up, down, outp = cm.empty((N, F * Mx * Mx)), cm.empty((N, C * Hh * Hh)), cm.empty((F, C * k * k))
    cc.convUp(X, Wm, up, Mx, p, s, C, G)
    cc.convDown(Y, Wm, down, Mx, p, s, k, Hh, C, numGroups=G)
    cc.convOutp(X, Y, outp, Mx, p, k, s, C, numGroups=G)
    y = Y.asarray()
    u = up.asarray().reshape(N, F, Mx, Mx)
    d = down.asarray().reshape(N, C, Hh, Hh)
    o = outp.asarray().reshape(F, C, k, k)
    edge = lambda size: int(r.choice([0, size - 1, int(r.integers(size))]))
    for _ in range(200):
        n, f, my, mx = edge(N), edge(F), edge(Mx), edge(Mx)
        val, mag = co.conv_up_at(x, w, C, Mx, p, s, G, n, f, my, mx)
        assert abs(u[n, f, my, mx] - val) <= 1e-4 * mag + 1e-30
        c, yy, xx = int(r.integers(C)), edge(Hh), edge(Hh)
        val, mag = co.conv_down_at(y, w, C, Hh, p, s, G, n, c, yy, xx)
        assert abs(d[n, c, yy, xx] - val) <= 1e-4 * mag + 1e-6
    for _ in range(6):
        f, cl, ky, kx = int(r.integers(F)), int(r.integers(C)), edge(k), edge(k)
        val, mag = co.conv_outp_at(x, y, C, Mx, k, p, s, G, f, cl, ky, kx)
        assert abs(o[f, cl, ky, kx] - val) <= 1e-4 * mag
    for m in (X, Wm, Y, up, down, outp):
        m.free_device_memory()


def _rows(mat, N):
    """Host copy of a few images (rows) of a device matrix: first, middle (around the row
    whose first-filter offset passes 2^31 bytes) and last."""
    parts = []
    for lo in (0, N // 2 - 2, N - 4):
        parts.append(mat.get_row_slice(lo, lo + 4).asarray().copy())
    return _f(np.concatenate(parts, axis=0))


def test_pool_and_norm_on_maps_beyond_32_bit_byte_offsets(cm, cc):
    N, F, S = 16512, 64, 32                      # 16512 x 65536 floats: 4.33 GB per matrix
    subs, start, stride = 3, 0, 2
    O = (S - start - subs + stride - 1) // stride + 1
    X = cm.empty((N, F * S * S))
    X.fill_with_randn()
    x = _rows(X, N)
    T = cm.empty((N, F * O * O))
    cc.MaxPool(X, T, F, subs, start, stride, O)
    want = co.max_pool(x, F, subs, start, stride, O)
    assert np.array_equal(_rows(T, N), want.astype(np.float32))
    G = cm.empty((N, F * O * O))
    G.fill_with_randn()
    g = _rows(G, N)
    U = cm.empty((N, F * S * S))
    cc.MaxPoolUndo(X, U, G, T, subs, start, stride, O)
    assert np.allclose(_rows(U, N), co.max_pool_undo(x, g, want, subs, start, stride, O), rtol=1e-6, atol=1e-6)
    G.free_device_memory(); T.free_device_memory()
    # response normalisation over the same maps, then its gradient
    a, p, size = 0.001, 0.75, 5
    D, Tn = cm.empty((N, F * S * S)), cm.empty((N, F * S * S))
    cc.ResponseNorm(X, D, Tn, F, size, a, p)
    t_want, d_want = co.response_norm(x, F, size, a, p)
    assert np.allclose(_rows(D, N), d_want, rtol=2e-6)
    assert np.allclose(_rows(Tn, N), t_want, rtol=1e-5, atol=1e-7)
    U.fill_with_randn()                          # U now holds the incoming gradient
    og, d_got, t_got = _rows(U, N), _rows(D, N), _rows(Tn, N)
    R = cm.empty((N, F * S * S))
    cc.ResponseNormUndo(U, D, X, Tn, R, F, size, a, p)
    u_want, acts_want = co.response_norm_undo(og, d_got, x, t_got, F, size, a, p)
    assert np.allclose(_rows(Tn, N), acts_want, rtol=1e-5, atol=1e-9)
    assert np.allclose(_rows(R, N), u_want, rtol=1e-5, atol=1e-6)
    for m in (X, U, D, Tn, R):
        m.free_device_memory()
