"""GPU parity of reductions, softmax and the sum path (dot with ones):
1e-5 relative for sums / sums of squares / softmax, exact for max / argmax."""
import numpy as np
import pytest

from oracle import cudamat_oracle as orc

pytestmark = pytest.mark.gpu

REL = 1e-5
SHAPES = [(256, 128), (37, 53), (1, 7), (7, 1), (4100, 3), (3, 4100), (10, 128), (1000, 1000)]


def _rand(rng, shape, lo=-1.0, hi=1.0):
    return np.asarray(rng.uniform(lo, hi, shape), dtype=np.float32, order='F')


def _rel(got, want, scale=None):
    want = np.asarray(want, dtype=np.float64)
    scale = np.maximum(np.abs(want), 1e-30) if scale is None else scale
    return np.max(np.abs(np.asarray(got, np.float64) - want) / scale)


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("axis", [0, 1])
def test_sum(cm, rng, shape, axis):
    x = _rand(rng, shape)
    a = cm.CUDAMatrix(x)
    got = a.sum(axis=axis).asarray()
    want = x.astype(np.float64).sum(axis=axis, keepdims=True)
    # error relative to the sum of magnitudes (sums of signed values can cancel)
    assert _rel(got, want, np.abs(x).astype(np.float64).sum(axis=axis, keepdims=True) + 1e-30) < REL
    assert got.shape == want.shape


def test_sum_of_transposed_and_add_sums_and_total(cm, rng):
    x = _rand(rng, (300, 200), 0.0, 1.0)
    a = cm.CUDAMatrix(x)
    # test_cudamat.py:298-327: sums of a.T are the sums of the transpose
    assert _rel(cm.sum(a.T, axis=0).asarray(), x.T.astype(np.float64).sum(axis=0, keepdims=True)) < REL
    assert _rel(cm.sum(a.T, axis=1).asarray(), x.T.astype(np.float64).sum(axis=1, keepdims=True)) < REL
    t0 = _rand(rng, (300, 1)); t = cm.CUDAMatrix(t0)
    t.add_sums(a, axis=1, mult=-0.5)
    assert _rel(t.asarray(), t0 - 0.5 * x.astype(np.float64).sum(axis=1, keepdims=True)) < 2e-5
    t1 = _rand(rng, (1, 200)); t = cm.CUDAMatrix(t1)
    t.add_sums(a, axis=0, mult=2.0)
    assert _rel(t.asarray(), t1 + 2.0 * x.astype(np.float64).sum(axis=0, keepdims=True)) < REL
    assert abs(a.sum() - x.astype(np.float64).sum()) / x.astype(np.float64).sum() < REL


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("axis", [0, 1])
def test_max_argmax(cm, rng, shape, axis):
    x = _rand(rng, shape)
    a = cm.CUDAMatrix(x)
    assert np.array_equal(a.max(axis=axis).asarray(), orc.max_by_axis(x, axis).astype(np.float32))
    assert np.array_equal(a.argmax(axis=axis).asarray(), orc.argmax_by_axis(x, axis).astype(np.float32))


def test_argmax_ties_follow_the_reference_scan_order(cm):
    # equal maxima at rows 2 and 33: the reference's 32-lane scan reports 33
    # (lane 33 % 32 = 1 is visited before lane 2), cudamat_kernels.cu:1020-1050
    x = np.zeros((70, 3), dtype=np.float32, order='F')
    x[2, 0] = x[33, 0] = 5.0
    x[64, 1] = x[0, 1] = x[32, 1] = 1.0      # lane 0 holds rows 0, 32, 64 -> first of them
    x[:, 2] = -np.inf                          # nothing beats the start value: index 0, max -FLT_MAX
    a = cm.CUDAMatrix(x)
    assert a.argmax(axis=0).asarray().tolist() == [[33.0, 0.0, 0.0]]
    assert orc.argmax_by_axis(x, 0).tolist() == [[33.0, 0.0, 0.0]]
    m = a.max(axis=0).asarray()
    assert m[0, 0] == 5.0 and m[0, 2] == -np.finfo(np.float32).max
    # axis 1: first occurrence
    y = np.zeros((3, 70), dtype=np.float32, order='F'); y[1, 40] = y[1, 7] = 2.0
    assert cm.CUDAMatrix(y).argmax(axis=1).asarray().ravel().tolist() == [0.0, 7.0, 0.0]


@pytest.mark.parametrize("shape", [(256, 128), (37, 53), (5000, 2)])
@pytest.mark.parametrize("axis", [0, 1])
def test_sqsum_and_norm_limit_and_choose_max(cm, rng, shape, axis):
    x = _rand(rng, shape)
    a = cm.CUDAMatrix(x)
    got = a.sqsum(axis=axis).asarray()
    assert _rel(got, orc.sqsum_by_axis(x, None, axis, 1.0, 0.0)) < REL
    t0 = _rand(rng, got.shape); t = cm.CUDAMatrix(t0)
    t.add_sqsums(a, axis=axis, mult=0.25)
    want = orc.sqsum_by_axis(x, t0, axis, 0.25, 1.0)
    assert _rel(t.asarray(), want, np.abs(t0) + np.abs(want - t0)) < REL
    norm = float(np.median(np.sqrt((x.astype(np.float64) ** 2).sum(axis=axis))))
    lim = cm.empty(shape)
    a.norm_limit(norm, axis, target=lim)
    want = orc.normlimit_by_axis(x, axis, norm)
    assert np.allclose(lim.asarray(), want, rtol=1e-5, atol=1e-7)
    ch = cm.empty(shape)
    a.choose_max(axis, target=ch)
    assert np.array_equal(ch.asarray(), orc.choose_max_by_axis(x, axis).astype(np.float32))
    a.choose_max(axis)          # in place
    assert np.array_equal(a.asarray(), orc.choose_max_by_axis(x, axis).astype(np.float32))


@pytest.mark.parametrize("shape", [(4, 3), (512, 37), (516, 9), (784, 1024), (1024, 130), (1028, 64), (2048, 70), (2052, 33), (4096, 600),
                                   (4096, 12), (4100, 16), (1001, 40)])
def test_norm_limit_of_columns_held_in_registers(cm, rng, shape):
    """Columns of up to 4096 rows (a multiple of 4) are read once; taller or ragged ones take the
    general kernel.  Against the oracle (cudamat_kernels.cu:1100-1130), in place as well, and against
    the general kernel, which a view of the same column at an odd offset runs (other lanes add the
    squares there, so the norms agree to rounding)."""
    h, w = shape
    x = _rand(rng, shape)
    x[:, 0] *= 1e-3                     # a column under the limit stays as it is
    a = cm.CUDAMatrix(x)
    norm = float(np.median(np.sqrt((x.astype(np.float64) ** 2).sum(axis=0))))
    lim = cm.empty(shape)
    a.norm_limit(norm, 0, target=lim)
    want = orc.normlimit_by_axis(x, 0, norm)
    got = lim.asarray().copy()
    assert np.allclose(got, want, rtol=1e-5, atol=1e-7)
    assert np.array_equal(got[:, 0], x[:, 0])
    # one column at a time out of a taller matrix, starting one row down: unaligned, general kernel
    tall = np.zeros((h + 1, w), dtype=np.float32, order='F'); tall[1:, :] = x
    T = cm.CUDAMatrix(tall)
    for c in (0, w // 2, w - 1):
        part = T.slice(c, c + 1).reshape((1, h + 1)).slice(1, h + 1).reshape((h, 1))   # a view, 4 bytes off
        out = cm.empty((h, 1))
        part.norm_limit(norm, 0, target=out)
        assert np.allclose(out.asarray().ravel(), got[:, c], rtol=2e-6, atol=0), c
    a.norm_limit(norm, 0)
    assert np.array_equal(a.asarray(), got)


def test_choose_max_and_accumulate(cm, rng):
    x = _rand(rng, (10, 40))
    acc0 = np.ones((10, 40), dtype=np.float32, order='F')
    a, acc = cm.CUDAMatrix(x), cm.CUDAMatrix(acc0)
    a.choose_max_and_accumulate(acc)
    assert np.array_equal(acc.asarray(), acc0 + orc.choose_max_by_axis(x, 0).astype(np.float32))


# (columns of up to 4096, 8192 and 16384 rows have kernels of their own, longer ones three passes)
@pytest.mark.parametrize("shape", [(100, 10), (10, 128), (4096, 64), (1000, 33), (37, 53), (5, 1), (20000, 3), (4100, 37), (8192, 9),
                                   (10000, 5), (16384, 3), (16388, 2), (5001, 4)])
def test_softmax(cm, rng, shape):
    x = _rand(rng, shape, -8, 8)
    a, t = cm.CUDAMatrix(x), cm.empty(shape)
    a.apply_softmax(target=t)
    got = t.asarray()
    assert _rel(got, orc.softmax(x)) < REL
    assert np.max(np.abs(got.astype(np.float64).sum(axis=0) - 1.0)) < 1e-5
    # shift invariance: softmax(x + c) == softmax(x)
    b = cm.CUDAMatrix(x + np.float32(3.0))
    b.apply_softmax()
    assert np.allclose(b.asarray(), got, rtol=2e-5, atol=1e-9)
    a.apply_softmax()            # overwrite variant
    assert np.array_equal(a.asarray(), got)


@pytest.mark.parametrize("h", [64, 37])          # columns held in registers / the generic kernel
def test_softmax_over_wide_ranges_and_masked_entries(cm, rng, h):
    x = _rand(rng, (h, 40), -60, 60)
    x[3, :] = -np.inf                               # a masked logit: probability 0, the rest unaffected
    x[:, 7] *= 1.4                                  # differences down to -168: underflow to 0
    t = cm.CUDAMatrix(x).apply_softmax(target=cm.empty(x.shape)).asarray()
    want = orc.softmax(x)
    assert np.all(t[3, :] == 0) and np.all(np.isfinite(t))
    big = want > 1e-30
    assert np.max(np.abs(t[big] - want[big]) / want[big]) < REL
    assert np.all(t[~big] < 2e-30)
    assert np.max(np.abs(t.astype(np.float64).sum(axis=0) - 1.0)) < 1e-5
    x[5, 2] = np.nan                                # NaN is not swallowed
    t = cm.CUDAMatrix(x).apply_softmax(target=cm.empty(x.shape)).asarray()
    assert np.all(np.isnan(t[:, 2])) and np.all(np.isfinite(np.delete(t, 2, axis=1)))


def test_softmax_loss_helpers(cm, rng):
    x = _rand(rng, (10, 128), -3, 3)
    labels = np.asarray(rng.integers(0, 10, (1, 128)), dtype=np.float32, order='F')
    p = cm.CUDAMatrix(x); p.apply_softmax()
    pn = p.asarray().copy()
    lab = cm.CUDAMatrix(labels)
    t = cm.empty((1, 128))
    p.get_softmax_correct(lab, t)
    assert np.array_equal(t.asarray(), orc.get_softmax_correct(pn, labels).astype(np.float32))
    p.get_softmax_cross_entropy(lab, t, tiny=1e-10)
    assert _rel(t.asarray(), orc.get_softmax_cross_entropy(pn, labels, 1e-10)) < REL
    g = cm.empty((10, 128))
    p.apply_softmax_grad(lab, target=g)
    assert np.array_equal(g.asarray(), orc.apply_softmax_grad(pn, labels).astype(np.float32))


def test_vdot_and_euclid_norm(cm, rng):
    # one workgroup, the 4-byte path (< 1024 elements), 16-byte groups with a tail, many
    # workgroups with several trips each
    for shape in [(1, 1), (37, 53), (1023, 1), (1024, 1), (1000, 999), (2051, 2049)]:
        x, y = _rand(rng, shape), _rand(rng, shape)
        a, b = cm.CUDAMatrix(x), cm.CUDAMatrix(y)
        scale = np.abs(x.astype(np.float64) * y).sum()
        first = cm.vdot(a, b)
        assert abs(first - orc.vdot(x, y)) / scale < REL
        assert abs(a.euclid_norm() - orc.euclid_norm(x)) / orc.euclid_norm(x) < REL
        assert cm.vdot(a, b) == first          # the order of the sum is fixed
    # operands that start 20 bytes into an allocation
    x, y = _rand(rng, (5, 400)), _rand(rng, (5, 400))
    a, b = cm.CUDAMatrix(x).get_col_slice(1, 400), cm.CUDAMatrix(y).get_col_slice(1, 400)
    scale = np.abs(x[:, 1:].astype(np.float64) * y[:, 1:]).sum()
    assert abs(cm.vdot(a, b) - orc.vdot(x[:, 1:], y[:, 1:])) / scale < REL
    with pytest.raises(cm.CUDAMatException, match="Incompatible matrix dimensions"):
        cm.vdot(a, cm.CUDAMatrix(_rand(rng, (3, 3))))


def test_axis_error_codes(cm, rng):
    a = cm.CUDAMatrix(_rand(rng, (8, 6)))
    with pytest.raises(cm.CUDAMatException, match="Incompatible matrix dimensions"):
        a.max(axis=0, target=cm.empty((6, 1)))
    with pytest.raises(cm.CUDAMatException, match="transposed"):
        cm._check(cm._cudamat.max_by_axis(a.T.p_mat, cm.empty((1, 6)).p_mat, 0))
    with pytest.raises(cm.CUDAMatException, match="not supported"):
        cm._check(cm._cudamat.max_by_axis(a.p_mat, cm.empty((1, 6)).p_mat, 2))


@pytest.mark.parametrize("axis", [0, 1])
def test_full_size_4096_sum_max_softmax(cm, rng, axis):
    n = 4096
    x = np.asarray(rng.uniform(-1, 1, (n, n)), dtype=np.float32, order='F')
    a = cm.CUDAMatrix(x)
    x64 = x.astype(np.float64)
    got = a.sum(axis=axis).asarray()
    assert _rel(got, x64.sum(axis=axis, keepdims=True), np.abs(x64).sum(axis=axis, keepdims=True)) < REL
    assert np.array_equal(a.max(axis=axis).asarray(), x.max(axis=axis, keepdims=True))
    if axis == 0:
        a.apply_softmax()
        got = a.asarray()
        assert np.max(np.abs(got.astype(np.float64).sum(axis=0) - 1.0)) < 1e-5
        cols = np.arange(0, n, 97)
        assert _rel(got[:, cols], orc.softmax(x[:, cols])) < REL
    a.free_device_memory()


@pytest.mark.gpu
@pytest.mark.parametrize("h,w", [(10, 128), (1000, 64), (4096, 33), (7, 5), (256, 256), (2048, 2100), (4100, 40), (10000, 12), (16384, 2)])
def test_softmax_ce_grad_is_bit_identical_to_the_three_calls(cm, rng, h, w):
    # both softmax kernels (columns held in registers: h % 4 == 0; generic otherwise)
    x = np.asarray(3.0 * rng.standard_normal((h, w)), dtype=np.float32, order='F')
    lab = np.asarray(rng.integers(0, h, (1, w)), dtype=np.float32, order='F')
    X, L = cm.CUDAMatrix(x), cm.CUDAMatrix(lab)
    p1, l1, g1 = cm.empty((h, w)), cm.empty((1, w)), cm.empty((h, w))
    X.apply_softmax(target=p1)
    p1.get_softmax_cross_entropy(L, l1, tiny=1e-10)
    p1.apply_softmax_grad(L, target=g1)
    p2, l2, g2 = cm.empty((h, w)), cm.empty((1, w)), cm.empty((h, w))
    cm.softmax_ce_grad(X, L, probs=p2, loss=l2, grad=g2, tiny=1e-10)
    for a, b in ((p1, p2), (l1, l2), (g1, g2)):
        assert np.array_equal(a.asarray().view(np.uint32), b.asarray().view(np.uint32))
    # in place, without loss or gradient: plain softmax
    X2 = cm.CUDAMatrix(x)
    cm.softmax_ce_grad(X2, L)
    assert np.array_equal(X2.asarray().view(np.uint32), p1.asarray().view(np.uint32))
    # and against the float64 definitions
    e = np.exp(x.astype(np.float64) - x.max(axis=0, keepdims=True))
    p = e / e.sum(axis=0, keepdims=True)
    idx = lab.astype(int)[0]
    assert np.max(np.abs(p2.asarray() - p)) < 1e-6
    assert np.max(np.abs(l2.asarray()[0] + np.log(p[idx, np.arange(w)] + 1e-10)) / (1 + np.abs(np.log(p[idx, np.arange(w)] + 1e-10)))) < 1e-5
    onehot = np.zeros((h, w)); onehot[idx, np.arange(w)] = 1
    assert np.max(np.abs(g2.asarray() - (p - onehot))) < 1e-6


@pytest.mark.gpu
def test_softmax_ce_grad_errors(cm, rng):
    X = cm.CUDAMatrix(np.zeros((5, 4), dtype=np.float32))
    L = cm.CUDAMatrix(np.zeros((1, 4), dtype=np.float32))
    lib = cm._cudamat
    assert lib.softmax_ce_grad(X.p_mat, L.p_mat, cm.empty((4, 5)).p_mat, None, None, 0.0) == -1
    assert lib.softmax_ce_grad(X.p_mat, cm.empty((1, 3)).p_mat, X.p_mat, None, None, 0.0) == -1
    assert lib.softmax_ce_grad(X.p_mat, L.p_mat, X.p_mat, cm.empty((1, 3)).p_mat, None, 0.0) == -1
    assert lib.softmax_ce_grad(X.T.p_mat, L.p_mat, X.p_mat, None, None, 0.0) == -5
    host = cm.CUDAMatrix(np.zeros((1, 4), dtype=np.float32), copy_to_device=False)
    assert lib.softmax_ce_grad(X.p_mat, host.p_mat, X.p_mat, None, None, 0.0) == -8


@pytest.mark.parametrize("shape", [(1, 1), (37, 53), (500, 100), (784, 128), (10, 128), (1000, 999), (4096, 1100), (1100, 4096),
                                   (2048, 2048), (4096, 64)])
def test_sums_leave_the_bits_of_dot_with_a_vector_of_ones(cm, rng, shape):
    """sum / add_sums run the kernels that dot() with a vector of ones would run (the reference's
    spelling, cudamat.py:724-748 and 1546-1577) without reading the vector: the same bits, also
    for a transposed operand and with an accumulating target."""
    x = _rand(rng, shape)
    a = cm.CUDAMatrix(x)
    h, w = shape
    ones_h = cm.CUDAMatrix(np.ones((h, 1), dtype=np.float32)); ones_w = cm.CUDAMatrix(np.ones((w, 1), dtype=np.float32))
    assert np.array_equal(a.sum(axis=0).asarray(), cm.dot(ones_h.T, a).asarray())
    assert np.array_equal(a.sum(axis=1).asarray(), cm.dot(a, ones_w).asarray())
    assert np.array_equal(cm.sum(a.T, axis=0).asarray(), cm.dot(ones_w.T, a.T).asarray())
    assert np.array_equal(cm.sum(a.T, axis=1).asarray(), cm.dot(a.T, ones_h).asarray())
    base = _rand(rng, (h, 1))
    t1, t2 = cm.CUDAMatrix(base), cm.CUDAMatrix(base)
    t1.add_sums(a, axis=1, mult=0.25)
    t2.add_dot(a, ones_w, mult=0.25)
    assert np.array_equal(t1.asarray(), t2.asarray())
    with pytest.raises(cm.CUDAMatException, match="Incompatible matrix dimensions"):
        a.sum(axis=0, target=cm.empty((1, w + 1)))
    with pytest.raises(cm.CUDAMatException, match="Incompatible matrix dimensions"):
        cm.empty((h + 1, 1)).add_sums(a, axis=1)
    # the sum of everything: vdot() with as many ones (cudamat.py:719-720), without reading them
    ones_all = cm.CUDAMatrix(np.ones((h, w), dtype=np.float32))
    assert np.float32(a.sum()).tobytes() == np.float32(cm.vdot(a, ones_all)).tobytes()
    assert abs(a.sum() - x.astype(np.float64).sum()) <= 1e-5 * np.abs(x).astype(np.float64).sum()
