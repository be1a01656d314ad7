"""Deferred epilogues: dot() holds its launch back and the add_col_vec / activation / sample calls
that follow it on its own target run in the product's epilogue; an in-place mult_by_scalar is held
back likewise and the add_mult / add_mult_sign calls of a parameter update (deepnet/parameter.py:80-106)
are folded into one pass.  Every sequence here is run with
the deferral switched off (each call its own launch) and on, and must leave the same bits in every
matrix it touches and the same generator state; sequences that must NOT be folded (another
matrix in between, a second bias, operands that change between the calls, reads, frees) are
checked the same way."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _f(a):
    return np.asarray(a, dtype=np.float32, order='F')


def _bits(m):
    return m.asarray().view(np.uint32).copy()


SHAPES = [(500, 784, 100, True), (784, 500, 100, False), (1024, 784, 128, True), (10, 1024, 128, True), (33, 17, 5, False),
          (2048, 128, 2048, True), (64, 4096, 64, True), (3, 2, 2, False)]       # m, k, n, first operand transposed


def _run(cm, deferred, seq, shape, seed):
    m, k, n, ta = shape
    rng = np.random.default_rng(seed)
    cm.set_deferred_epilogues(deferred)
    cm.CUDAMatrix.init_random(7)
    A = cm.CUDAMatrix(_f(rng.standard_normal((k, m) if ta else (m, k)) * 0.1))
    B = cm.CUDAMatrix(_f(rng.standard_normal((k, n))))
    bias = cm.CUDAMatrix(_f(rng.standard_normal((m, 1))))
    other = cm.CUDAMatrix(_f(rng.standard_normal((m, n))))
    T, S = cm.empty((m, n)), cm.empty((m, n))
    T.assign(-3.0); S.assign(-4.0)
    a = A.T if ta else A
    out = seq(cm, a, B, bias, other, T, S)
    after = cm.empty((64, 48)); after.fill_with_rand()            # the generator's state shows in its next draws
    res = [_bits(x) for x in (T, S, other, bias, after)] + ([out] if out is not None else [])
    cm.set_deferred_epilogues(True)
    return res


def seq_sigmoid(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); T.add_col_vec(bias); T.apply_sigmoid()


def seq_sigmoid_sample(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); T.add_col_vec(bias); T.apply_sigmoid(); T.sample_bernoulli(target=S)


def seq_relu(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); T.add_col_vec(bias); T.lower_bound(0)


def seq_tanh(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); T.add_col_vec(bias); cm.tanh(T)


def seq_no_bias(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); T.apply_sigmoid(); T.sample_bernoulli(target=S)


def seq_bias_only_then_read(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); T.add_col_vec(bias)
    return T.asarray().view(np.uint32).copy()                   # the read launches what is held back


def seq_dot_alone_then_other_work(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); other.mult(T); T.apply_sigmoid()     # the sigmoid is an ordinary launch


def seq_bias_on_another_matrix(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); other.add_col_vec(bias); T.add_col_vec(bias); T.apply_sigmoid()


def seq_two_biases(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); T.add_col_vec(bias); T.add_col_vec(bias); T.apply_sigmoid(); T.apply_sigmoid()


def seq_bias_changes_in_between(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); T.add_col_vec(bias); bias.mult(2.0); T.apply_sigmoid(); bias.add(1.0); T.sample_bernoulli(target=S)


def seq_operand_changes_in_between(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); B.mult(0.5); T.add_col_vec(bias); cm.tanh(T)


def seq_sigmoid_into_another_target(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); T.add_col_vec(bias); T.apply_sigmoid(target=S); S.sample_bernoulli(target=other)


def seq_sample_in_place(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); T.add_col_vec(bias); T.apply_sigmoid(); T.sample_bernoulli()      # target = self: not folded


def seq_scaled_and_accumulating_products(cm, a, B, bias, other, T, S):
    cm.dot(a, B, mult=0.5, target=T); T.add_col_vec(bias); T.apply_sigmoid()             # alpha != 1: launched at once
    S.add_dot(a, B); S.add_col_vec(bias); S.lower_bound(0)


def seq_two_products_in_a_row(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); cm.dot(a, B, target=S); S.add_col_vec(bias); S.apply_sigmoid(); T.add_col_vec(bias); T.lower_bound(0)


def seq_free_while_held_back(cm, a, B, bias, other, T, S):
    tmp = cm.empty(T.shape)
    cm.dot(a, B, target=tmp); tmp.add_col_vec(bias)
    tmp.free_device_memory()                                     # launches (into memory that is then given back)
    again = cm.empty(T.shape); again.assign(1.5); T.add(again)


def seq_lower_bound_not_zero(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); T.add_col_vec(bias); T.lower_bound(0.25)


# ---- the parameter update of deepnet/parameter.py:80-106 (w = T, w_delta = S, gradient = other)

def _params(T, S, other):
    T.assign(0.25); S.assign(-0.5)                      # (the harness fills them with constants: make them vary)
    T.add(other); S.subtract(other)
    return T, S, other


def seq_update_plain(cm, a, B, bias, other, T, S):
    w, wd, g = _params(T, S, other)
    wd.mult(0.9); wd.add_mult(g); w.add_mult(wd, -0.01)


def seq_update_with_reset(cm, a, B, bias, other, T, S):
    w, wd, g = _params(T, S, other)
    wd.mult(0.9); wd.add_mult(g); w.add_mult(wd, -0.01); g.assign(0)


def seq_update_l2_l1_reset(cm, a, B, bias, other, T, S):
    w, wd, g = _params(T, S, other)
    wd.mult(0.5); wd.add_mult(w, 0.001); wd.add_mult_sign(w, 0.0005); wd.add_mult(g); w.add_mult(wd, -0.1); g.assign(0)


def seq_update_l2_only(cm, a, B, bias, other, T, S):
    w, wd, g = _params(T, S, other)
    wd.mult(0.5); wd.add_mult(w, 0.001); wd.add_mult(g); w.add_mult(wd, -0.1); g.assign(1.0)     # (not a reset)


def seq_update_l1_only_twice(cm, a, B, bias, other, T, S):
    w, wd, g = _params(T, S, other)
    for _ in range(2):
        wd.mult(0.5); wd.add_mult_sign(w, 0.0005); wd.add_mult(g); w.add_mult(wd, -0.1)


def seq_update_not_spelled_scaled_gradient(cm, a, B, bias, other, T, S):
    w, wd, g = _params(T, S, other)
    wd.mult(0.9); wd.add_mult(g, 0.5); w.add_mult(wd, -0.01); g.assign(0)


def seq_update_not_spelled_wrong_order(cm, a, B, bias, other, T, S):
    w, wd, g = _params(T, S, other)
    wd.mult(0.9); wd.add_mult(g); wd.add_mult(w, 0.001); w.add_mult(wd, -0.01)


def seq_update_not_spelled_no_gradient(cm, a, B, bias, other, T, S):
    w, wd, g = _params(T, S, other)
    wd.mult(0.9); wd.add_mult(w, 0.001); w.add_mult(wd, -0.01)


def seq_update_interrupted(cm, a, B, bias, other, T, S):
    w, wd, g = _params(T, S, other)
    wd.mult(0.9); g.mult(2.0); wd.add_mult(g); w.add_mult(wd, -0.01); wd.mult(0.5); bias.mult(3.0); wd.add_mult(g)


def seq_update_reads_another_matrix(cm, a, B, bias, other, T, S):
    w, wd, g = _params(T, S, other)
    wd.mult(0.9); wd.add_mult(g); w.add_mult(g, -0.01); w.add_mult(wd, -0.01)


def seq_update_too_many_terms(cm, a, B, bias, other, T, S):
    w, wd, g = _params(T, S, other)
    wd.mult(0.9); wd.add_mult(w, 0.001); wd.add_mult_sign(w, 0.0005); wd.add_mult(g); wd.add_mult(g); w.add_mult(wd, -0.01)


def seq_update_then_product(cm, a, B, bias, other, T, S):
    w, wd, g = _params(T, S, other)
    wd.mult(0.9); wd.add_mult(g); w.add_mult(wd, -0.01)
    cm.dot(a, B, target=g); g.add_col_vec(bias); g.apply_sigmoid(); wd.mult(0.5); wd.add_mult(g); w.add_mult(wd, 0.3); g.assign(0)


def seq_scale_alone_then_read(cm, a, B, bias, other, T, S):
    T.assign(2.0); T.add(other); T.mult(0.5)
    return T.asarray().view(np.uint32).copy()


SEQS = [seq_update_plain, seq_update_with_reset, seq_update_l2_l1_reset, seq_update_l2_only, seq_update_l1_only_twice,
        seq_update_not_spelled_scaled_gradient, seq_update_not_spelled_wrong_order, seq_update_not_spelled_no_gradient,
        seq_update_interrupted, seq_update_reads_another_matrix, seq_update_too_many_terms, seq_update_then_product,
        seq_scale_alone_then_read, seq_sigmoid, seq_sigmoid_sample, seq_relu, seq_tanh, seq_no_bias, seq_bias_only_then_read, seq_dot_alone_then_other_work,
        seq_bias_on_another_matrix, seq_two_biases, seq_bias_changes_in_between, seq_operand_changes_in_between,
        seq_sigmoid_into_another_target, seq_sample_in_place, seq_scaled_and_accumulating_products, seq_two_products_in_a_row,
        seq_free_while_held_back, seq_lower_bound_not_zero]


@pytest.mark.parametrize("seq", SEQS, ids=lambda f: f.__name__)
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "%dx%dx%d%s" % (s[0], s[1], s[2], 't' if s[3] else 'n'))
def test_same_bits_with_and_without_deferral(cm, seq, shape):
    want = _run(cm, False, seq, shape, 5)
    got = _run(cm, True, seq, shape, 5)
    for i, (g, w) in enumerate(zip(got, want)):
        assert np.array_equal(g, w), "matrix %d differs" % i
    cm.CUDAMatrix.init_random(1)


def test_the_folded_sequence_is_the_float64_definition(cm, rng):
    m, k, n = 500, 784, 100
    w, x, b = _f(0.05 * rng.standard_normal((k, m))), _f(rng.random((k, n))), _f(rng.standard_normal((m, 1)))
    W, X, Bv, T = cm.CUDAMatrix(w), cm.CUDAMatrix(x), cm.CUDAMatrix(b), cm.empty((m, n))
    cm.dot(W.T, X, target=T); T.add_col_vec(Bv); T.apply_sigmoid()
    want = 1.0 / (1.0 + np.exp(-(w.astype(np.float64).T @ x.astype(np.float64) + b)))
    assert np.allclose(T.asarray(), want, rtol=1e-5, atol=1e-6)


def test_training_steps_of_the_bench_keep_their_bits(cm):
    import bench
    for cls, seed, params in ((bench.RBM, 1, lambda o: [o.W, o.bv, o.bh, o.h, o.hs, o.v2, o.h2]),
                              (bench.MLP, 3, lambda o: o.W + o.b + o.dW + [o.loss] + o.mask)):
        res = []
        for deferred in (False, True):
            cm.set_deferred_epilogues(deferred)
            cm.CUDAMatrix.init_random(seed)
            obj = cls(cm)
            for _ in range(3):
                obj.step()
            res.append([_bits(p) for p in params(obj)])
        cm.set_deferred_epilogues(True)
        for a, b in zip(*res):
            assert np.array_equal(a, b)
    cm.CUDAMatrix.init_random(1)


def test_the_switch_reports_its_previous_setting(cm):
    assert cm.set_deferred_epilogues(False) is True
    assert cm.set_deferred_epilogues(True) is False
    assert cm.set_deferred_epilogues(True) is True
