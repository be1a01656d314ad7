"""CPU-only pins of the numpy restatement: each formula against an independent
library routine or a hand-computed value, chosen so that a dropped term, a wrong
sign or a swapped operand fails."""
import numpy as np
import pytest
import scipy.special as sp

from oracle import cudamat_oracle as orc


@pytest.fixture
def x(rng):
    return rng.uniform(-6, 6, (37, 11))


def test_unary_closed_forms_against_library_routines(x):
    assert np.allclose(orc.apply_sigmoid(x), sp.expit(x), rtol=1e-14)
    assert np.allclose(orc.apply_tanh(x), np.tanh(x), rtol=1e-12, atol=1e-15)
    assert np.allclose(orc.apply_log_1_plus_exp(x), np.logaddexp(0, x), rtol=1e-14)
    assert np.allclose(orc.apply_abs(x), np.abs(x))
    assert np.allclose(orc.reciprocal(x), 1 / x)
    assert np.allclose(orc.apply_pow(np.abs(x), 2.5), np.abs(x) ** 2.5)
    assert np.allclose(orc.apply_log(np.abs(x).astype(np.float32), 0.0), np.log(np.abs(x).astype(np.float32).astype(np.float64)))
    assert orc.apply_sigmoid(np.array([0.0]))[0] == 0.5 and orc.apply_tanh(np.array([0.0]))[0] == 0.0
    assert np.array_equal(orc.sign(np.array([-3.0, -0.0, 0.0, 2.0])), [-1, 0, 0, 1])
    # the 'tiny' of apply_log is added in float32 before the log
    assert orc.apply_log(np.array([1.0], np.float32), 1e-10)[0] == 0.0


def test_binary_and_derivative_forms(rng):
    a, b = rng.uniform(-2, 2, (9, 7)), rng.uniform(0.05, 0.95, (9, 7))
    h = 1e-6
    # logistic: d/dz sigma(z) = y(1-y) with y = sigma(z)
    z = sp.logit(b)
    assert np.allclose(orc.apply_logistic_deriv(a, b), a * (sp.expit(z + h) - sp.expit(z - h)) / (2 * h), rtol=1e-6)
    # the tanh derivative of the reference carries a factor 1/2: a(1+y)(1-y)/2 (cudamat_kernels.cu:663-669)
    y = 2 * b - 1
    assert np.allclose(orc.apply_tanh_deriv(a, y), 0.5 * a * (1 - y ** 2))
    assert np.allclose(orc.apply_rectified_linear_deriv(a, a), a * (a > 0))
    assert np.allclose(orc.apply_rectified_linear_smooth_deriv(a, b), a * (1 - np.exp(-b)))
    assert np.allclose(orc.apply_cos_deriv(a, b), a * (np.cos(b + h) - np.cos(b - h)) / (2 * h), rtol=1e-5, atol=1e-8)
    assert np.allclose(orc.apply_sin_deriv(a, b), a * (np.sin(b + h) - np.sin(b - h)) / (2 * h), rtol=1e-5, atol=1e-8)
    assert np.array_equal(orc.upper_bound(np.array([1.0, 5.0]), np.array([3.0, 3.0])), [1, 3])
    assert np.array_equal(orc.lower_bound(np.array([1.0, 5.0]), np.array([3.0, 3.0])), [3, 5])
    assert np.array_equal(orc.less_than(np.array([1.0, 3.0]), np.array([3.0, 3.0])), [1, 0])
    assert np.array_equal(orc.greater_than_eq(np.array([1.0, 3.0]), np.array([3.0, 3.0])), [0, 1])
    assert np.allclose(orc.add_mult(a, b, 0.5), a + np.float32(0.5) * b)
    assert np.array_equal(orc.add_mult_sign(np.zeros(3), np.array([-2.0, 0.0, 4.0]), 0.5), [-0.5, 0, 0.5])
    t = (b > 0.5).astype(float)
    assert np.allclose(orc.compute_cross_entropy_bernoulli(t, b.astype(np.float32), 0.0),
                       -(t * np.log(b.astype(np.float32).astype(float)) + (1 - t) * np.log1p(-b.astype(np.float32).astype(float))),
                       rtol=1e-6)
    assert np.array_equal(orc.correct_preds(np.array([1.0, 0.0, 1.0]), np.array([0.7, 0.2, 0.1]), 0.5), [1, 1, 0])


def test_broadcasts_follow_column_major_indexing(rng):
    a = rng.standard_normal((5, 3))
    col, row = rng.standard_normal((5, 1)), rng.standard_normal((1, 3))
    flat = a.ravel(order='F')
    # kernel indexing: vec[i % h] for a column vector, vec[i / h] for a row vector
    want_c = np.array([flat[i] + col[i % 5, 0] for i in range(15)]).reshape((5, 3), order='F')
    want_r = np.array([flat[i] * row[0, i // 5] for i in range(15)]).reshape((5, 3), order='F')
    assert np.allclose(orc.add_col_vec(a, col), want_c)
    assert np.allclose(orc.mult_by_row_vec(a, row), want_r)
    assert np.allclose(orc.add_row_mult(a, row, 2.0), a + 2 * row)
    assert np.allclose(orc.div_by_col_vec(a, col), a / col)
    sq = rng.standard_normal((4, 4)); v = rng.standard_normal((4, 1))
    d = orc.diagonal_op(sq, v, 'add')
    assert np.allclose(np.diag(d), np.diag(sq) + v.ravel()) and np.allclose(d - np.diag(np.diag(d)), sq - np.diag(np.diag(sq)))


def test_dot_transposes_and_scalars(rng):
    A, B, C = rng.standard_normal((6, 4)), rng.standard_normal((4, 5)), rng.standard_normal((6, 5))
    assert np.allclose(orc.dot(A, B), A @ B)
    assert np.allclose(orc.dot(A.T.copy(), B, trans_a=True), A @ B)
    assert np.allclose(orc.dot(A, B.T.copy(), trans_b=True), A @ B)
    assert np.allclose(orc.dot(A, B, C, beta=-1.0, alpha=2.0), 2 * A @ B - C)


def test_reductions_softmax_and_losses(rng):
    x = rng.standard_normal((50, 20)).astype(np.float32)
    assert np.allclose(orc.softmax(x), sp.softmax(x.astype(np.float64), axis=0), rtol=1e-12)
    assert np.allclose(orc.softmax(x).sum(axis=0), 1)
    assert np.array_equal(orc.max_by_axis(x, 0), x.max(axis=0, keepdims=True))
    assert np.array_equal(orc.argmax_by_axis(x, 0).ravel(), x.argmax(axis=0))     # no ties: plain argmax
    assert np.array_equal(orc.argmax_by_axis(x, 1).ravel(), x.argmax(axis=1))
    assert orc.argmax_ref_order(np.array([0, 0, 5] + [0] * 30 + [5], dtype=np.float32)) == 33   # tie: lane 1 before lane 2
    assert orc.argmax_ref_order(np.full(40, -np.inf, dtype=np.float32)) == 0
    one = orc.choose_max_by_axis(x, 0)
    assert np.array_equal(one.sum(axis=0), np.ones(20)) and np.array_equal(one.argmax(axis=0), x.argmax(axis=0))
    assert np.allclose(orc.sqsum_by_axis(x, np.ones((1, 20)), 0, 2.0, 3.0), 3 + 2 * (x.astype(float) ** 2).sum(axis=0))
    lim = orc.normlimit_by_axis(x, 0, 5.0)
    norms = np.linalg.norm(lim, axis=0)
    assert np.all(norms <= 5.0 + 1e-9) and np.allclose(lim[:, np.linalg.norm(x, axis=0) < 5], x[:, np.linalg.norm(x, axis=0) < 5])
    p = orc.softmax(x[:10, :])
    labels = rng.integers(0, 10, (1, 20)).astype(np.float32)
    g = orc.apply_softmax_grad(p, labels)
    assert np.allclose(g.sum(axis=0), 0, atol=1e-12)            # p sums to 1, one-hot sums to 1
    ce = orc.get_softmax_cross_entropy(p.astype(np.float32), labels, 0.0)
    assert np.allclose(ce.ravel(), [-np.log(np.float32(p[int(l), j])) for j, l in enumerate(labels.ravel())], rtol=1e-6)
    assert np.array_equal(orc.get_softmax_correct(p, p.argmax(axis=0)[None, :].astype(np.float32)), np.ones((1, 20)))


def test_gather_scatter_semantics(rng):
    x = rng.standard_normal((4, 6))
    s = orc.select_columns(x, np.array([[0, -1, 7]]))
    assert np.array_equal(s[:, 0], x[:, 0]) and np.array_equal(s[:, 1], x[:, 5]) and np.all(np.isnan(s[:, 2]))
    assert np.array_equal(orc.blockify(np.arange(6.0).reshape(6, 1), 2).ravel(), [0, 0, 2, 2, 4, 4])
    acc = orc.accumulate_columns(x, np.array([[0, 1, 0, 2, 2, 2]]), 3, 1.0, True)
    assert np.allclose(acc[:, 0], x[:, [0, 2]].mean(axis=1)) and np.allclose(acc[:, 2], x[:, 3:].mean(axis=1))
    imgs = np.arange(2 * 4 * 4 * 1, dtype=float).reshape((16, 2), order='F')
    tr = orc.generate_translations(imgs, 4, 2, np.array([[0, 1]]), np.array([[0, -1]]), 1)
    assert np.array_equal(tr[:, 0], imgs[:, 0].reshape(4, 4)[1:3, 1:3].ravel())
    assert np.array_equal(tr[:, 1], imgs[:, 1].reshape(4, 4)[2:4, 0:2].ravel())
    # a window leaving the image: flat pixel addressing (cudamat_kernels.cu:807,814).  Image 0 is pixels
    # 0..15, image 1 pixels 16..31 of the matrix; pad = 1.  Offsets (1, 2): origin row 2, column 3, so the
    # second column of the window is column 4 = column 0 of the next row.
    tr = orc.generate_translations(imgs, 4, 2, np.array([[1, 2]]), np.array([[2, 2]]), 1)
    assert tr[:, 0].tolist() == [11.0, 12.0, 15.0, 16.0]          # pixel 16 already belongs to image 1
    # image 1, origin row 3: its second window row lies beyond the matrix -> 0 (foreign memory in the reference)
    assert tr[:, 1].tolist() == [16 + 15.0, 0.0, 0.0, 0.0]


def test_ulp_helper():
    one = np.float32(1.0)
    assert orc.ulp_diff(np.array([one]), np.array([1.0]))[0] == 0
    assert abs(orc.ulp_diff(np.array([np.nextafter(one, np.float32(2))]), np.array([1.0]))[0] - 1.0) < 1e-9
    assert orc.ulp_diff(np.array([np.float32(np.inf)]), np.array([np.inf]))[0] == 0
    assert orc.ulp_diff(np.array([np.float32(np.nan)]), np.array([np.nan]))[0] == 0
    assert np.isinf(orc.ulp_diff(np.array([np.float32(np.nan)]), np.array([1.0]))[0])


def test_fastdiv_magic_numbers_used_by_the_device_kernels():
    """The multiply-high division of deepnet_amd/csrc/common.h, restated, against // for
    awkward divisors and dividends up to 2^32 - 1."""
    def make(d):
        s = (d - 1).bit_length()
        return ((((1 << 32) * ((1 << s) - d)) // d + 1) & 0xFFFFFFFF, min(s, 1), max(s - 1, 0), d)

    def div(n, f):
        magic, sh1, sh2, d = f
        hi = (n * magic) >> 32
        return ((hi + ((n - hi) >> sh1)) & 0xFFFFFFFF) >> sh2

    rng = np.random.default_rng(0)
    for d in [1, 2, 3, 5, 7, 10, 37, 64, 100, 500, 784, 1023, 1024, 1025, 4096, 12288, 65537, 2 ** 31 - 1, 2 ** 31 + 3]:
        f = make(d)
        for n in [0, 1, d - 1, d, d + 1, 2 * d - 1, 2 ** 32 - 1, 2 ** 31, 123456789] + list(rng.integers(0, 2 ** 32, 200)):
            n = int(n)
            assert div(n, f) == n // d, (n, d)


def test_sparse_dot_against_scipy_and_a_dense_product(rng):
    # the loop restatement against two independent routines: scipy's CSR product and the
    # dense product of the densified matrix; a wrong index array (indices vs indptr), a
    # transposed dense operand or beta/alpha swapped would fail
    import scipy.sparse as sps
    m, k, n = 37, 29, 11
    S = sps.random(m, k, density=0.2, format='csr', random_state=3, dtype=np.float32)
    S = S.tolil()
    S[5, :] = 0          # an empty row
    S = S.tocsr()
    S.sort_indices()
    D = np.asarray(rng.standard_normal((k, n)), dtype=np.float32)
    T = np.asarray(rng.standard_normal((m, n)), dtype=np.float32)
    got = orc.sparse_dot(S.data, S.indices, S.indptr, D, T, beta=-0.5, alpha=2.0)
    want = 2.0 * (S.astype(np.float64) @ D.astype(np.float64)) - 0.5 * T.astype(np.float64)
    assert np.allclose(got, want, rtol=1e-12, atol=1e-12)
    dense = np.asarray(S.todense(), dtype=np.float64)
    assert np.allclose(orc.sparse_dot(S.data, S.indices, S.indptr, D), dense @ D.astype(np.float64), rtol=1e-12, atol=1e-12)
    # a hand-checked 2 x 3 case: rows [1 0 2], [0 3 0]
    got = orc.sparse_dot([1, 2, 3], [0, 2, 1], [0, 2, 3], np.array([[1., 10.], [2., 20.], [3., 30.]]))
    assert np.array_equal(got, np.array([[7., 70.], [6., 60.]]))
