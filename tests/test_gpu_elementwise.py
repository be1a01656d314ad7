"""GPU parity of the elementwise / scalar / compare / broadcast ops against the
float64 oracle: at most 2 float32 ulps (the bar for elementwise ops), exact for
comparisons, clamps, floor/ceil, sign and abs."""
import numpy as np
import pytest

from oracle import cudamat_oracle as orc

pytestmark = pytest.mark.gpu

ULP = 2.0
SHAPES = [(256, 128), (37, 53), (1, 1), (513, 7)]


def _check(got, want, tol=ULP, what=""):
    d = orc.ulp_diff(got, want)
    assert d.max() <= tol, "%s: %.2f ulp at %s" % (what, d.max(), np.unravel_index(np.argmax(d), d.shape))


def _rand(rng, shape, lo=-4.0, hi=4.0):
    return np.asarray(rng.uniform(lo, hi, shape), dtype=np.float32, order='F')


UNARY = [
    # (module fn or method name, oracle fn, input range, tolerance in ulp)
    ('sigmoid', orc.apply_sigmoid, (-30, 30), ULP),
    ('tanh', orc.apply_tanh, (-12, 12), ULP),
    ('exp', orc.apply_exp, (-80, 80), ULP),
    ('cos', orc.apply_cos, (-20, 20), ULP),
    ('sin', orc.apply_sin, (-20, 20), ULP),
    ('abs', orc.apply_abs, (-4, 4), 0),
    ('ceil', orc.apply_ceil, (-40, 40), 0),
    ('floor', orc.apply_floor, (-40, 40), 0),
    ('sqrt', orc.apply_sqrt, (0, 100), ULP),
    ('log_1_plus_exp', orc.apply_log_1_plus_exp, (-30, 30), ULP),
]


@pytest.mark.parametrize("name,ofn,rng_,tol", UNARY, ids=[u[0] for u in UNARY])
@pytest.mark.parametrize("shape", SHAPES)
def test_unary(cm, rng, name, ofn, rng_, tol, shape):
    x = _rand(rng, shape, *rng_)
    want = ofn(x)
    # with a separate target
    a, t = cm.CUDAMatrix(x), cm.empty(shape)
    r = getattr(cm, name)(a, target=t)
    assert r is t
    _check(t.asarray(), want, tol, name)
    assert np.array_equal(a.asarray(), x), "input modified"
    # in place
    getattr(cm, name)(a)
    _check(a.asarray(), want, tol, name + " in place")
    a.free_device_memory(); t.free_device_memory()


def test_tanh_and_softplus_keep_their_accuracy_near_zero(cm, rng):
    # 1 - 2/(exp(2x)+1) and log(1+exp(x)) cancel in float32 steps; the device
    # evaluates them so that the float64 value of the formula is met to 2 ulp.
    x = _rand(rng, (64, 64), -1e-3, 1e-3)
    a, t = cm.CUDAMatrix(x), cm.empty(x.shape)
    cm.tanh(a, target=t)
    _check(t.asarray(), np.tanh(x.astype(np.float64)), ULP, "tanh near 0")
    y = _rand(rng, (64, 64), -40, -5)
    b = cm.CUDAMatrix(y)
    cm.log_1_plus_exp(b)
    _check(b.asarray(), np.logaddexp(0.0, y.astype(np.float64)), ULP, "softplus, very negative")


def test_log_and_pow_and_reciprocal(cm, rng):
    x = _rand(rng, (256, 128), 0.01, 50)
    a, t = cm.CUDAMatrix(x), cm.empty(x.shape)
    cm.log(a, target=t)
    _check(t.asarray(), orc.apply_log(x), ULP, "log")
    cm.log(a, tiny=1e-3, target=t)
    _check(t.asarray(), orc.apply_log(x, 1e-3), ULP, "log tiny")
    cm.pow(a, 2.5, target=t)
    _check(t.asarray(), orc.apply_pow(x, 2.5), ULP, "pow")
    p = _rand(rng, x.shape, -2, 2)
    pm = cm.CUDAMatrix(p)
    cm.pow(a, pm, target=t)
    _check(t.asarray(), orc.apply_pow_matrix(x, p), ULP, "pow matrix")
    a.reciprocal(target=t)
    _check(t.asarray(), orc.reciprocal(x), 1, "reciprocal")


def test_sign_special_values(cm):
    x = np.array([[-2.5, -0.0, 0.0, 3.0, np.inf, -np.inf]], dtype=np.float32)
    a = cm.CUDAMatrix(x)
    s = a.sign()
    assert s is not a
    got = s.asarray()
    assert np.array_equal(got, np.array([[-1, 0, 0, 1, 1, -1]], dtype=np.float32))
    assert not np.signbit(got[0, 1])


def test_special_values_exp_sigmoid(cm):
    x = np.array([[-np.inf, -200.0, -0.0, 0.0, 200.0, np.inf, np.nan]], dtype=np.float32)
    a, t = cm.CUDAMatrix(x), cm.empty(x.shape)
    cm.exp(a, target=t)
    got = t.asarray()
    assert got[0, 0] == 0 and got[0, 1] == 0 and got[0, 2] == 1 and got[0, 3] == 1
    assert np.isinf(got[0, 4]) and np.isinf(got[0, 5]) and np.isnan(got[0, 6])
    cm.sigmoid(a, target=t)
    got = t.asarray()
    assert got[0, 0] == 0 and got[0, 2] == 0.5 and got[0, 4] == 1 and got[0, 5] == 1 and np.isnan(got[0, 6])


BINARY = [
    ('add', orc.add_elementwise, 1), ('subtract', orc.subtract_elementwise, 1),
    ('mult', orc.mult_elementwise, 1), ('divide', orc.divide_elementwise, 1),
    ('less_than', orc.less_than, 0), ('less_than_eq', orc.less_than_eq, 0),
    ('greater_than', orc.greater_than, 0), ('greater_than_eq', orc.greater_than_eq, 0),
    ('upper_bound', orc.upper_bound, 0), ('lower_bound', orc.lower_bound, 0),
    ('apply_logistic_deriv', orc.apply_logistic_deriv, ULP), ('apply_tanh_deriv', orc.apply_tanh_deriv, 1),
    ('apply_rectified_linear_deriv', orc.apply_rectified_linear_deriv, 0),
    ('apply_rectified_linear_smooth_deriv', orc.apply_rectified_linear_smooth_deriv, ULP),
    ('apply_cos_deriv', orc.apply_cos_deriv, ULP), ('apply_sin_deriv', orc.apply_sin_deriv, ULP),
]


@pytest.mark.parametrize("name,ofn,tol", BINARY, ids=[b[0] for b in BINARY])
@pytest.mark.parametrize("shape", SHAPES[:2])
def test_binary(cm, rng, name, ofn, tol, shape):
    x, y = _rand(rng, shape), _rand(rng, shape)
    y.flat[::7] = x.flat[::7]  # exercise equality for the comparisons
    want = ofn(x, y)
    a, b, t = cm.CUDAMatrix(x), cm.CUDAMatrix(y), cm.empty(shape)
    getattr(a, name)(b, target=t)
    _check(t.asarray(), want, tol, name)
    getattr(a, name)(b)
    _check(a.asarray(), want, tol, name + " in place")


SCALAR = [
    ('add', orc.add_scalar, 1), ('mult', orc.mult_by_scalar, 1), ('divide', orc.divide_by_scalar, 1),
    ('less_than', orc.less_than, 0), ('less_than_eq', orc.less_than_eq, 0),
    ('greater_than', orc.greater_than, 0), ('greater_than_eq', orc.greater_than_eq, 0),
    ('upper_bound', orc.upper_bound, 0), ('lower_bound', orc.lower_bound, 0),
]


@pytest.mark.parametrize("name,ofn,tol", SCALAR, ids=[s[0] for s in SCALAR])
def test_matrix_scalar(cm, rng, name, ofn, tol):
    x = _rand(rng, (256, 128))
    s = 0.37
    x.flat[::5] = np.float32(s)
    a, t = cm.CUDAMatrix(x), cm.empty(x.shape)
    getattr(a, name)(s, target=t)
    _check(t.asarray(), ofn(x, np.float32(s)), tol, name)


def test_subtract_scalar_and_assign(cm, rng):
    x = _rand(rng, (33, 9))
    a = cm.CUDAMatrix(x)
    a.subtract(1.5)
    _check(a.asarray(), x.astype(np.float64) - 1.5, 1)
    a.assign(2.25)
    assert np.all(a.asarray() == np.float32(2.25))
    b = cm.CUDAMatrix(x)
    a.assign(b)
    assert np.array_equal(a.asarray(), x)


def test_add_mult_family(cm, rng):
    x, y = _rand(rng, (256, 128)), _rand(rng, (256, 128))
    a, b = cm.CUDAMatrix(x), cm.CUDAMatrix(y)
    a.add_mult(b, 0.37)
    _check(a.asarray(), orc.add_mult(x, y, 0.37), 1, "add_mult")
    a = cm.CUDAMatrix(x)
    a.subtract_mult(b, 0.37)
    _check(a.asarray(), orc.add_mult(x, y, -0.37), 1, "subtract_mult")
    a = cm.CUDAMatrix(x)
    y2 = y.copy(); y2.flat[::3] = 0
    b2 = cm.CUDAMatrix(y2)
    a.add_mult_sign(b2, 0.5)
    _check(a.asarray(), orc.add_mult_sign(x, y2, 0.5), 1, "add_mult_sign")


def test_cross_entropy_family(cm, rng):
    t_ = np.asarray(rng.random((64, 32)) < 0.5, dtype=np.float32, order='F')
    p = _rand(rng, (64, 32), 0.001, 0.999)
    a, b, t = cm.CUDAMatrix(t_), cm.CUDAMatrix(p), cm.empty(p.shape)
    cm.cross_entropy(a, b, target=t)
    _check(t.asarray(), orc.compute_cross_entropy(t_, p, 1e-10), ULP, "cross_entropy")
    cm.cross_entropy_bernoulli(a, b, target=t, tiny=1e-6)
    _check(t.asarray(), orc.compute_cross_entropy_bernoulli(t_, p, 1e-6), 4, "cross_entropy_bernoulli")
    cm.correct_preds(a, b, target=t, cutoff=0.4)
    _check(t.asarray(), orc.correct_preds(t_, p, 0.4), 0, "correct_preds")


BCAST = [
    ('add_col_vec', orc.add_col_vec, 'col', None), ('add_col_mult', orc.add_col_mult, 'col', 0.7),
    ('add_row_vec', orc.add_row_vec, 'row', None), ('add_row_mult', orc.add_row_mult, 'row', -1.3),
    ('mult_by_col', orc.mult_by_col_vec, 'col', None), ('mult_by_row', orc.mult_by_row_vec, 'row', None),
    ('div_by_col', orc.div_by_col_vec, 'col', None), ('div_by_row', orc.div_by_row_vec, 'row', None),
]


@pytest.mark.parametrize("name,ofn,kind,mult", BCAST, ids=[b[0] for b in BCAST])
@pytest.mark.parametrize("shape", [(256, 128), (37, 53), (1, 9), (9, 1), (1030, 3)])
def test_broadcast(cm, rng, name, ofn, kind, mult, shape):
    x = _rand(rng, shape)
    v = _rand(rng, (shape[0], 1) if kind == 'col' else (1, shape[1]), 0.5, 2.0)
    a, vec, t = cm.CUDAMatrix(x), cm.CUDAMatrix(v), cm.empty(shape)
    args = (vec,) if mult is None else (vec, mult)
    want = ofn(x, v) if mult is None else ofn(x, v, mult)
    getattr(a, name)(*args, target=t)
    _check(t.asarray(), want, 1, name)
    getattr(a, name)(*args)
    _check(a.asarray(), want, 1, name + " in place")


def test_views_with_odd_offsets_take_the_unaligned_paths(cm, rng):
    # a column view of a 37-row matrix starts 37*k floats in: not 16-byte aligned
    x, y = _rand(rng, (37, 20)), _rand(rng, (37, 20))
    a, b = cm.CUDAMatrix(x), cm.CUDAMatrix(y)
    va, vb = a.slice(3, 11), b.slice(5, 13)       # different phases -> scalar kernel
    va.add(vb)
    want = x.copy(); want[:, 3:11] += y[:, 5:13]
    assert np.array_equal(a.asarray(), want)
    vc = b.slice(3, 11)                            # same phase as va -> peeled vector kernel
    va.mult(vc)
    want[:, 3:11] *= y[:, 3:11]
    assert np.array_equal(a.asarray(), want)
    v = _rand(rng, (37, 1))
    va.add_col_vec(cm.CUDAMatrix(v))
    want[:, 3:11] += v
    assert np.array_equal(a.asarray(), want)


def test_diagonal_ops(cm, rng):
    x = _rand(rng, (65, 65))
    v = _rand(rng, (65, 1))
    for name, op in (('add_diagonal', 'add'), ('mult_diagonal', 'mult')):
        a, t = cm.CUDAMatrix(x), cm.CUDAMatrix(x)
        getattr(a, name)(cm.CUDAMatrix(v), target=t)
        _check(t.asarray(), orc.diagonal_op(x, v, op), 1, name)
        t2 = cm.CUDAMatrix(x)
        getattr(a, name)(1.5, target=t2)
        _check(t2.asarray(), orc.diagonal_op(x, 1.5, op), 1, name + " scalar")


def test_error_codes_in_reference_order(cm, rng):
    x = _rand(rng, (8, 6))
    a, b = cm.CUDAMatrix(x), cm.CUDAMatrix(x)
    wrong = cm.CUDAMatrix(_rand(rng, (6, 8)))
    host_only = cm.CUDAMatrix(x, copy_to_device=False)
    with pytest.raises(cm.CUDAMatException, match="Incompatible matrix dimensions"):
        a.add(wrong)
    with pytest.raises(cm.CUDAMatException, match="not in device memory"):
        a.add(host_only)
    # binary ops: transposedness is checked before dims (cudamat.cu:1806-1812)
    with pytest.raises(cm.CUDAMatException, match="Incompatible transposedness"):
        cm._check(cm._cudamat.add_elementwise(a.p_mat, wrong.T.p_mat, b.p_mat))
    # broadcasts refuse a transposed matrix before looking at dims (cudamat.cu:596-604)
    with pytest.raises(cm.CUDAMatException, match="transposed"):
        cm._check(cm._cudamat.add_col_vec(a.T.p_mat, wrong.p_mat, b.p_mat))
    with pytest.raises(cm.CUDAMatException, match="Incompatible matrix dimensions"):
        a.add_col_vec(cm.CUDAMatrix(_rand(rng, (1, 6))))
    with pytest.raises(cm.CUDAMatException, match="Incompatible transposedness"):
        a.add_mult(cm.CUDAMatrix(_rand(rng, (6, 8))).T)
    with pytest.raises(ValueError):
        a.add("x")


@pytest.mark.parametrize("name", ['add_mult', 'mult', 'sigmoid', 'exp', 'mult_by_col', 'add_row_vec'])
def test_full_size_4096(cm, rng, name):
    """The benchmark's 4096 x 4096 operands: parity on a strided sample of the
    output plus a linearity / identity property over the whole of it."""
    n = 4096
    x = np.asarray(rng.uniform(-1, 1, (n, n)), dtype=np.float32, order='F')
    a = cm.CUDAMatrix(x)
    rows = np.arange(0, n, 61); cols = np.arange(0, n, 67)
    sub = np.ix_(rows, cols)
    if name == 'add_mult':
        y = np.asarray(rng.uniform(-1, 1, (n, n)), dtype=np.float32, order='F')
        b = cm.CUDAMatrix(y)
        a.add_mult(b, 0.5)
        got = a.asarray()
        _check(got[sub], orc.add_mult(x[sub], y[sub], 0.5), 1)
        a.add_mult(b, -0.5)   # exact inverse up to one rounding each way
        assert np.max(np.abs(a.asarray() - x)) <= 2.4e-7
    elif name == 'mult':
        b = cm.CUDAMatrix(x)
        a.mult(b)
        got = a.asarray()
        assert np.array_equal(got, x * x)
    elif name in ('sigmoid', 'exp'):
        getattr(cm, name)(a)
        got = a.asarray()
        ofn = orc.apply_sigmoid if name == 'sigmoid' else orc.apply_exp
        _check(got[sub], ofn(x[sub]), ULP)
        if name == 'sigmoid':   # sigma(x) + sigma(-x) = 1
            b = cm.CUDAMatrix(-x); cm.sigmoid(b)
            assert np.max(np.abs(got + b.asarray() - 1)) <= 2.4e-7
    elif name == 'mult_by_col':
        v = np.asarray(rng.uniform(-1, 1, (n, 1)), dtype=np.float32, order='F')
        a.mult_by_col(cm.CUDAMatrix(v))
        assert np.array_equal(a.asarray(), x * v)
    else:
        v = np.asarray(rng.uniform(-1, 1, (1, n)), dtype=np.float32, order='F')
        a.add_row_vec(cm.CUDAMatrix(v))
        assert np.array_equal(a.asarray(), x + v)
    a.free_device_memory()


def _log_uniform(rng, n, lo_exp, hi_exp, signed=True):
    x = np.exp2(rng.uniform(lo_exp, hi_exp, n))
    if signed:
        x *= rng.choice([-1.0, 1.0], n)
    return np.asarray(x, dtype=np.float32).reshape(-1, 1)


def test_transcendentals_over_their_whole_range(cm, rng):
    """2 ulp against the float64 value of each formula from denormal to overflow
    magnitudes, including the special values."""
    n = 200000
    specials = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1.0, -1.0, 1e-45, -1e-45, 3.4e38, -3.4e38,
                         88.72284, -87.33655, -103.97, 16.635532, -16.635532], dtype=np.float32).reshape(-1, 1)
    wide = np.vstack([_log_uniform(rng, n, -149, 128), specials])
    moderate = np.vstack([_log_uniform(rng, n, -30, 7), specials])          # up to +-128
    positive = np.vstack([_log_uniform(rng, n, -149, 128, signed=False), specials])
    trig = np.vstack([_log_uniform(rng, n, -30, 29), _log_uniform(rng, 1000, 29, 128), specials])
    cases = [('exp', orc.apply_exp, moderate), ('sigmoid', orc.apply_sigmoid, moderate),
             ('tanh', np.tanh, wide), ('log_1_plus_exp', lambda v: np.logaddexp(0.0, v.astype(np.float64)), moderate),
             ('sqrt', orc.apply_sqrt, positive), ('cos', orc.apply_cos, trig), ('sin', orc.apply_sin, trig)]
    for name, ofn, x in cases:
        a = cm.CUDAMatrix(x)
        getattr(cm, name)(a)
        with np.errstate(all='ignore'):
            want = ofn(x.astype(np.float64))
        d = orc.ulp_diff(a.asarray(), want)
        k = int(np.argmax(d))
        assert d.max() <= ULP, "%s: %.2f ulp at x=%r (got %r want %r)" % (name, d.max(), x.ravel()[k],
                                                                       a.asarray().ravel()[k], want.ravel()[k])
        a.free_device_memory()
    a = cm.CUDAMatrix(positive)
    cm.log(a)
    with np.errstate(all='ignore'):
        want = np.log(positive.astype(np.float64))
    d = orc.ulp_diff(a.asarray(), want)
    assert d.max() <= ULP, "log: %.2f ulp at %r" % (d.max(), positive.ravel()[int(np.argmax(d))])
    # pow: positive bases with any exponent, negative bases with integer exponents
    base = _log_uniform(rng, n, -40, 40, signed=False)
    expo = np.asarray(rng.uniform(-3, 3, (n, 1)), dtype=np.float32)
    a, p = cm.CUDAMatrix(base), cm.CUDAMatrix(expo)
    cm.pow(a, p)
    with np.errstate(all='ignore'):
        want = np.power(base.astype(np.float64), expo.astype(np.float64))
    d = orc.ulp_diff(a.asarray(), want)
    assert d.max() <= ULP, "pow: %.2f ulp" % d.max()
    nb = -_log_uniform(rng, 1000, -10, 10, signed=False)
    for e in (-3.0, -2.0, 0.0, 1.0, 2.0, 5.0):
        a = cm.CUDAMatrix(nb)
        cm.pow(a, e)
        d = orc.ulp_diff(a.asarray(), np.power(nb.astype(np.float64), e))
        assert d.max() <= ULP, "pow(neg, %g): %.2f ulp" % (e, d.max())
    a = cm.CUDAMatrix(np.array([[0.0, -2.0, 2.0, np.inf, np.nan]], dtype=np.float32))
    cm.pow(a, 0.5)
    got = a.asarray().ravel()
    assert got[0] == 0 and np.isnan(got[1]) and abs(got[2] - np.sqrt(2)) < 1e-7 and np.isinf(got[3]) and np.isnan(got[4])


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(784, 500), (1024, 1), (37, 13), (4096, 1024)])
@pytest.mark.parametrize("l2,l1,reset", [(None, None, True), (0.0005, None, True), (0.0005, 0.001, False), (None, 0.001, True)])
def test_momentum_update_is_bit_identical_to_the_calls_it_replaces(cm, rng, shape, l2, l1, reset):
    # the sequence of deepnet/parameter.py:80-106 against the one-pass extension; the oracle
    # pins the sequence's formula (float64, 2 ulp per step is too loose a bar for equality of
    # the two device paths, which is asserted bit for bit)
    w0 = np.asarray(rng.standard_normal(shape), dtype=np.float32, order='F')
    w0.flat[::7] = 0.0                                   # sign(0) = 0 in the l1 term
    d0 = np.asarray(0.1 * rng.standard_normal(shape), dtype=np.float32, order='F')
    g0 = np.asarray(rng.standard_normal(shape), dtype=np.float32, order='F')
    mom, eps = 0.9, 0.01
    w, d, g = cm.CUDAMatrix(w0), cm.CUDAMatrix(d0), cm.CUDAMatrix(g0)
    d.mult(mom)
    if l2 is not None:
        d.add_mult(w, l2)
    if l1 is not None:
        d.add_mult_sign(w, l1)
    d.add_mult(g)
    w.add_mult(d, -eps)
    if reset:
        g.assign(0)
    w2, d2, g2 = cm.CUDAMatrix(w0), cm.CUDAMatrix(d0), cm.CUDAMatrix(g0)
    cm.momentum_update(w2, d2, g2, mom, eps, l2_decay=l2, l1_decay=l1, reset_gradient=reset)
    assert np.array_equal(w.asarray().view(np.uint32), w2.asarray().view(np.uint32))
    assert np.array_equal(d.asarray().view(np.uint32), d2.asarray().view(np.uint32))
    assert np.array_equal(g.asarray(), g2.asarray())
    # and the formula itself, in float64
    want_d = np.float32(mom) * d0.astype(np.float64) + (np.float32(l2) * w0.astype(np.float64) if l2 is not None else 0) \
        + (np.float32(l1) * np.sign(w0).astype(np.float64) if l1 is not None else 0) + g0
    want_w = w0 - np.float32(eps) * want_d
    assert np.max(np.abs(d2.asarray() - want_d)) < 1e-5 and np.max(np.abs(w2.asarray() - want_w)) < 1e-5
    for x in (w, d, g, w2, d2, g2):
        x.free_device_memory()


@pytest.mark.gpu
def test_momentum_update_errors(cm, rng):
    a = cm.CUDAMatrix(np.zeros((4, 3), dtype=np.float32))
    b = cm.CUDAMatrix(np.zeros((3, 4), dtype=np.float32))
    host = cm.CUDAMatrix(np.zeros((4, 3), dtype=np.float32), copy_to_device=False)
    lib = cm._cudamat
    assert lib.momentum_update(a.p_mat, a.p_mat, host.p_mat, 0.9, 0.0, 0.0, 0.01, 0) == -8
    assert lib.momentum_update(a.p_mat, b.T.p_mat, a.p_mat, 0.9, 0.0, 0.0, 0.01, 0) == -7
    assert lib.momentum_update(a.p_mat, b.p_mat, a.p_mat, 0.9, 0.0, 0.0, 0.01, 0) == -1


def test_momentum_updates_of_many_parameters_in_one_launch(cm, rng):
    """MomentumUpdates gives the bits of one momentum_update per parameter: 11 parameters of
    assorted sizes (two launches), a view that starts 4 bytes into its parent, per-parameter
    and shared scalars, and the checks of the single call."""
    shapes = [(64, 48), (48, 1), (10, 1), (1, 1), (257, 33), (128, 128), (5, 7), (1024, 16), (3, 1), (100, 100), (31, 1)]
    def make():
        r = np.random.default_rng(5)
        ws = [cm.CUDAMatrix(np.asarray(r.uniform(-1, 1, s), dtype=np.float32, order='F')) for s in shapes]
        ds = [cm.CUDAMatrix(np.asarray(r.uniform(-1, 1, s), dtype=np.float32, order='F')) for s in shapes]
        gs = [cm.CUDAMatrix(np.asarray(r.uniform(-1, 1, s), dtype=np.float32, order='F')) for s in shapes]
        parent = cm.CUDAMatrix(np.asarray(r.uniform(-1, 1, (1, 41)), dtype=np.float32, order='F'))
        ws.append(parent.slice(1, 41)); ds.append(cm.CUDAMatrix(np.zeros((1, 40), dtype=np.float32))); gs.append(cm.CUDAMatrix(np.ones((1, 40), dtype=np.float32)))
        return ws, ds, gs, parent
    n = len(shapes) + 1
    moms = [0.5 + 0.03 * i for i in range(n)]
    l2s = [None if i % 3 == 0 else 0.001 * i for i in range(n)]
    l1s = [0.0005 * i if i % 4 == 1 else None for i in range(n)]
    for shared in (False, True):
        w1, d1, g1, p1 = make()
        w2, d2, g2, p2 = make()
        for step in range(2):
            for i in range(n):
                if shared:
                    cm.momentum_update(w1[i], d1[i], g1[i], 0.9, 0.01, l2_decay=0.002, reset_gradient=(step == 1))
                else:
                    cm.momentum_update(w1[i], d1[i], g1[i], moms[i], 0.01 + 0.001 * i, l2_decay=l2s[i], l1_decay=l1s[i], reset_gradient=(step == 1))
            upd = cm.MomentumUpdates(list(zip(w2, d2, g2)))
            if shared:
                upd.apply(0.9, 0.01, l2_decay=0.002, reset_gradient=(step == 1))
            else:
                upd.apply(moms, [0.01 + 0.001 * i for i in range(n)], l2_decay=l2s, l1_decay=l1s, reset_gradient=(step == 1))
        for i in range(n):
            assert np.array_equal(w1[i].asarray(), w2[i].asarray()), i
            assert np.array_equal(d1[i].asarray(), d2[i].asarray()), i
            assert np.array_equal(g1[i].asarray(), g2[i].asarray()), i
        assert np.array_equal(p1.asarray(), p2.asarray())
    a, b = cm.CUDAMatrix(np.zeros((4, 4), dtype=np.float32)), cm.CUDAMatrix(np.zeros((4, 5), dtype=np.float32))
    before = a.asarray().copy()
    with pytest.raises(cm.CUDAMatException):
        cm.MomentumUpdates([(a, a, a), (a, b, a)]).apply(0.9, 0.01)
    assert np.array_equal(a.asarray(), before)              # nothing ran
    with pytest.raises(ValueError):
        cm.MomentumUpdates([(a, a, a)]).apply([0.9, 0.8], 0.01)
