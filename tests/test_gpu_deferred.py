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


# ---- the dropout mask of deepnet/neuralnet.py:194-198 (mask = S, state = T)

def seq_dropout(cm, a, B, bias, other, T, S):
    T.add(other); S.fill_with_rand(); S.greater_than(0.5); T.mult(S)


def seq_dropout_after_a_layer(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); T.add_col_vec(bias); T.lower_bound(0); S.fill_with_rand(); S.greater_than(0.3); T.mult(S)
    other.fill_with_rand(); other.greater_than(0.7); T.mult(other)


def seq_layer_mask_for_another_matrix(cm, a, B, bias, other, T, S):
    # the mask that follows the layer is meant for another matrix: the layer comes first, then the masking
    cm.dot(a, B, target=T); T.add_col_vec(bias); T.lower_bound(0); S.fill_with_rand(); S.greater_than(0.3); other.mult(S); other.add(T)


def seq_layer_mask_unfinished(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); T.lower_bound(0); S.fill_with_rand(); other.add(T); S.greater_than(0.5); T.mult(S)


def seq_layer_mask_is_an_operand(cm, a, B, bias, other, T, S):
    # the mask is drawn into the matrix the product reads: the product must see the old values
    cm.dot(a, B, target=T); T.lower_bound(0); B.fill_with_rand(); B.greater_than(0.5); cm.dot(a, B, target=S)


def seq_layer_mask_then_sample(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); T.add_col_vec(bias); T.lower_bound(0); S.fill_with_rand(); S.greater_than(0.5); T.mult(S)
    T.apply_sigmoid(); T.sample_bernoulli(target=other)


def seq_two_layers_with_masks(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); T.add_col_vec(bias); T.lower_bound(0); S.fill_with_rand(); S.greater_than(0.5); T.mult(S)
    cm.dot(a, B, target=other); other.lower_bound(0); S.fill_with_rand(); S.greater_than(0.25); other.mult(S)


def seq_layer_without_mask_then_draw(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); T.lower_bound(0); other.fill_with_randn(); S.fill_with_rand()


# the hidden sample as cudamat/examples/rbm_cudamat.py:63-65 spells it: r.fill_with_rand(); r.less_than(h, target=h)
def seq_sample_by_uniforms(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); T.add_col_vec(bias); T.apply_sigmoid(); S.fill_with_rand(); S.less_than(T, target=T)


def seq_sample_by_uniforms_into_another_target(cm, a, B, bias, other, T, S):
    T.apply_sigmoid(); S.fill_with_rand(); S.less_than(T, target=other); S.fill_with_rand(); T.less_than(S, target=S)


def seq_sample_by_uniforms_behind_a_relu_layer(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); T.lower_bound(0); S.fill_with_rand(); S.less_than(T, target=T); other.fill_with_rand()


def seq_sample_by_uniforms_of_itself(cm, a, B, bias, other, T, S):
    S.fill_with_rand(); S.less_than(S, target=S); T.fill_with_rand(); T.less_than(other)


def seq_dropout_mask_then_read(cm, a, B, bias, other, T, S):
    S.fill_with_rand(); S.greater_than(0.25)
    return S.asarray().view(np.uint32).copy()


def seq_dropout_into_another_target(cm, a, B, bias, other, T, S):
    T.add(other); S.fill_with_rand(); S.greater_than(0.5); T.mult(S, target=other)


def seq_dropout_threshold_into_another_target(cm, a, B, bias, other, T, S):
    T.add(other); S.fill_with_rand(); S.greater_than(0.5, target=other); T.mult(S)


def seq_dropout_mask_times_itself(cm, a, B, bias, other, T, S):
    S.fill_with_rand(); S.greater_than(0.5); S.mult(S); T.fill_with_rand(); T.mult(T)


def seq_dropout_roles_exchanged(cm, a, B, bias, other, T, S):
    T.add(other); S.fill_with_rand(); S.greater_than(0.5); S.mult(T)


def seq_fill_then_other_work(cm, a, B, bias, other, T, S):
    S.fill_with_rand(); T.add(S); S.greater_than(0.5); T.mult(S)


def seq_dropout_of_special_values(cm, a, B, bias, other, T, S):
    T.assign(-0.0); other.assign(float('inf')); T.add_mult(other, -1.0)        # -inf everywhere: times a zero of the mask is NaN
    S.fill_with_rand(); S.greater_than(0.5); T.mult(S)


def seq_fill_then_another_draw(cm, a, B, bias, other, T, S):
    # the generator's state moves to its other buffer in large calls: the second call must see the first one's
    S.fill_with_rand(); T.assign(0.5); T.sample_bernoulli(target=other); S.fill_with_rand(); T.fill_with_randn()
    S.fill_with_rand(); S.greater_than(0.5); other.sample_bernoulli()


# the backward pass of a layer of rectified linear units: deriv = dot(w, deriv_above);
# deriv.apply_rectified_linear_deriv(state)  (deepnet/neuralnet.py:203-222, layer.py:168-172)
def seq_relu_deriv(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); T.apply_rectified_linear_deriv(other)


def seq_masked_relu_deriv(cm, a, B, bias, other, T, S):
    # ... of a layer with dropout: deriv.mult(mask) in between (neuralnet.py:212-213)
    S.fill_with_rand(); S.greater_than(0.5); cm.dot(a, B, target=T); T.mult(S); T.apply_rectified_linear_deriv(other)


def seq_masked_deriv_without_activation(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); T.mult(other); S.add(T)


def seq_factor_then_bias(cm, a, B, bias, other, T, S):
    # a bias behind the factor is not the layer's sequence: nothing may be reordered
    cm.dot(a, B, target=T); T.mult(other); T.add_col_vec(bias); T.apply_sigmoid()


def seq_factor_twice(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); T.mult(other); T.mult(other); T.apply_rectified_linear_deriv(S)


def seq_factor_is_the_target(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); T.mult(T); T.apply_rectified_linear_deriv(other)


def seq_factor_into_another_target(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); T.mult(other, target=S); T.apply_rectified_linear_deriv(S)


def seq_factor_then_lower_bound(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); T.mult(other); T.lower_bound(0); S.fill_with_rand(); S.greater_than(0.5); T.mult(S)


def seq_relu_deriv_then_other_work(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); T.apply_rectified_linear_deriv(other); T.mult(0.5); other.add(T)


def seq_relu_deriv_into_another_target(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); T.apply_rectified_linear_deriv(other, target=S)


def seq_relu_deriv_by_itself(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); T.apply_rectified_linear_deriv(T)


def seq_relu_deriv_after_a_bias(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); T.add_col_vec(bias); T.apply_rectified_linear_deriv(other)


def seq_relu_deriv_of_another_matrix(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); S.apply_rectified_linear_deriv(T); other.apply_rectified_linear_deriv(S)


def seq_relu_deriv_with_special_values(cm, a, B, bias, other, T, S):
    other.assign(0.0); S.assign(-0.0); other.subtract(S)                  # zeros of both signs in the gate
    cm.dot(a, B, target=T); T.apply_rectified_linear_deriv(other)
    S.assign(np.inf); cm.dot(a, B, target=T); T.apply_rectified_linear_deriv(S)


# a softmax layer and its loss: state.apply_softmax(); state.get_softmax_cross_entropy(labels, loss);
# state.apply_softmax_grad(labels, target=deriv)  (deepnet/softmax_layer.py:25-62)
def _labels(cm, T, shift=0):
    m, n = T.shape
    return cm.CUDAMatrix(_f(((np.arange(n) * 7 + shift) % m).reshape(1, n))), cm.empty((1, n))


def seq_softmax_loss_grad(cm, a, B, bias, other, T, S):
    lab, loss = _labels(cm, T)
    cm.dot(a, B, target=T); T.add_col_vec(bias); T.apply_softmax(); T.get_softmax_cross_entropy(lab, loss); T.apply_softmax_grad(lab, target=S)
    return _bits(loss)


def seq_softmax_grad_only(cm, a, B, bias, other, T, S):
    lab, loss = _labels(cm, T)
    cm.dot(a, B, target=T); T.apply_softmax(); T.apply_softmax_grad(lab, target=S)


def seq_softmax_loss_only_then_read(cm, a, B, bias, other, T, S):
    lab, loss = _labels(cm, T)
    cm.dot(a, B, target=T); T.apply_softmax(); T.get_softmax_cross_entropy(lab, loss, tiny=1e-6)
    return _bits(loss)


def seq_softmax_alone_then_other_work(cm, a, B, bias, other, T, S):
    cm.dot(a, B, target=T); T.apply_softmax(); other.add(T)


def seq_softmax_grad_in_place(cm, a, B, bias, other, T, S):
    lab, loss = _labels(cm, T)
    cm.dot(a, B, target=T); T.apply_softmax(); T.get_softmax_cross_entropy(lab, loss); T.apply_softmax_grad(lab)
    return _bits(loss)


def seq_softmax_into_another_target(cm, a, B, bias, other, T, S):
    lab, loss = _labels(cm, T)
    cm.dot(a, B, target=T); T.apply_softmax(target=other); other.get_softmax_cross_entropy(lab, loss); other.apply_softmax_grad(lab, target=S)
    return _bits(loss)


def seq_softmax_loss_of_the_logits(cm, a, B, bias, other, T, S):
    # the loss and the gradient are asked of the matrix the softmax read, not of its result: nothing joins
    lab, loss = _labels(cm, T)
    cm.dot(a, B, target=T); T.apply_sigmoid(); T.apply_softmax(target=other); T.get_softmax_cross_entropy(lab, loss); T.apply_softmax_grad(lab, target=S)
    return _bits(loss)


def seq_softmax_two_label_vectors(cm, a, B, bias, other, T, S):
    lab, loss = _labels(cm, T)
    lab2, _ = _labels(cm, T, shift=1)
    cm.dot(a, B, target=T); T.apply_softmax(); T.get_softmax_cross_entropy(lab, loss); T.apply_softmax_grad(lab2, target=S)
    return _bits(loss)


def seq_softmax_correct_in_between(cm, a, B, bias, other, T, S):
    lab, loss = _labels(cm, T)
    hit = cm.empty(loss.shape)
    cm.dot(a, B, target=T); T.apply_softmax(); T.get_softmax_correct(lab, hit); T.get_softmax_cross_entropy(lab, loss); T.apply_softmax_grad(lab, target=S)
    return np.concatenate([_bits(loss).ravel(), _bits(hit).ravel()])


def seq_softmax_then_scale_in_place(cm, a, B, bias, other, T, S):
    # an in-place scale is held back itself and launches what waits before it
    cm.dot(a, B, target=T); T.apply_softmax(); T.mult(0.9); other.mult(0.5); other.add_mult(T)


def seq_softmax_gradient_over_the_logits_of_another(cm, a, B, bias, other, T, S):
    # the gradient's target is the matrix a second softmax reads
    lab, loss = _labels(cm, T)
    cm.dot(a, B, target=T); T.apply_softmax(target=other); other.apply_softmax_grad(lab, target=T); T.apply_softmax(target=S)
    S.get_softmax_cross_entropy(lab, loss)
    return _bits(loss)


SEQS = [seq_sample_by_uniforms, seq_sample_by_uniforms_into_another_target, seq_sample_by_uniforms_behind_a_relu_layer,
        seq_sample_by_uniforms_of_itself, seq_masked_relu_deriv, seq_masked_deriv_without_activation, seq_factor_then_bias, seq_factor_twice, seq_factor_is_the_target,
        seq_factor_into_another_target, seq_factor_then_lower_bound, seq_layer_mask_for_another_matrix, seq_layer_mask_unfinished, seq_layer_mask_is_an_operand, seq_layer_mask_then_sample,
        seq_two_layers_with_masks, seq_layer_without_mask_then_draw, seq_softmax_loss_grad, seq_softmax_grad_only, seq_softmax_loss_only_then_read, seq_softmax_alone_then_other_work,
        seq_softmax_grad_in_place, seq_softmax_into_another_target, seq_softmax_loss_of_the_logits, seq_softmax_two_label_vectors,
        seq_softmax_correct_in_between, seq_softmax_then_scale_in_place, seq_softmax_gradient_over_the_logits_of_another, seq_relu_deriv, seq_relu_deriv_then_other_work, seq_relu_deriv_into_another_target, seq_relu_deriv_by_itself,
        seq_relu_deriv_after_a_bias, seq_relu_deriv_of_another_matrix, seq_relu_deriv_with_special_values, seq_fill_then_another_draw, seq_dropout, seq_dropout_after_a_layer, seq_dropout_mask_then_read, seq_dropout_into_another_target,
        seq_dropout_threshold_into_another_target, seq_dropout_mask_times_itself, seq_dropout_roles_exchanged,
        seq_fill_then_other_work, seq_dropout_of_special_values, seq_update_plain, seq_update_with_reset, seq_update_l2_l1_reset, seq_update_l2_only, seq_update_l1_only_twice,
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


# ---- accumulating products and row sums (the statistics of a contrastive-divergence step,
# cudamat/examples/rbm_cudamat.py:73-86): W nv x nh, v / v2 nv x B, h / h2 nh x B, bv nv x 1, bh nh x 1

STAT_SHAPES = [(784, 500, 100), (500, 784, 100), (33, 17, 5), (1024, 1024, 128), (100, 60, 128), (2048, 64, 16), (256, 512, 200),
               (36, 40, 7), (4, 4, 2), (784, 1024, 128), (1024, 10, 128), (1280, 640, 64), (1022, 10, 128), (66, 130, 31)]          # nv, nh, batch


def stat_cd(cm, o):
    eps = 0.01
    o.W.add_dot(o.v, o.h.T, mult=eps); o.W.add_dot(o.v2, o.h2.T, mult=-eps)
    o.bv.add_sums(o.v, axis=1, mult=eps); o.bv.add_sums(o.v2, axis=1, mult=-eps)
    o.bh.add_sums(o.h, axis=1, mult=eps); o.bh.add_sums(o.h2, axis=1, mult=-eps)


def stat_cd_subtract_dot(cm, o):
    o.W.add_dot(o.v, o.h.T); o.W.subtract_dot(o.v2, o.h2.T)
    o.bh.add_sums(o.h, axis=1); o.bv.add_sums(o.v, axis=1, mult=0.5); o.bh.add_sums(o.h2, axis=1, mult=-1.0); o.bv.add_sums(o.v2, axis=1, mult=-0.5)


def stat_pair_then_read(cm, o):
    o.W.add_dot(o.v, o.h.T, mult=0.25); o.W.add_dot(o.v2, o.h2.T, mult=-0.75)
    return o.W.asarray().view(np.uint32).copy()


def stat_single_then_read(cm, o):
    o.W.add_dot(o.v, o.h.T, mult=0.25)
    return o.W.asarray().view(np.uint32).copy()


def stat_three_products(cm, o):
    o.W.add_dot(o.v, o.h.T, mult=0.25); o.W.add_dot(o.v2, o.h2.T, mult=-0.75); o.W.add_dot(o.v, o.h2.T, mult=0.125)


def stat_products_into_two_targets(cm, o):
    o.W.add_dot(o.v, o.h.T, mult=0.25); o.W2.add_dot(o.v2, o.h2.T, mult=-0.75); o.W.add_dot(o.v2, o.h.T); o.W2.add_dot(o.v, o.h2.T)


def stat_second_product_reads_the_target(cm, o):
    # the visible states are overwritten by a product of the weights, then used: nothing may be reordered
    o.W.add_dot(o.v, o.h.T, mult=0.25); cm.dot(o.W, o.h, target=o.v2); o.W.add_dot(o.v2, o.h2.T, mult=-0.75)


def stat_overwriting_product_after_accumulating(cm, o):
    o.W.add_dot(o.v, o.h.T, mult=0.25); cm.dot(o.v2, o.h2.T, target=o.W); o.W.add_dot(o.v, o.h2.T); o.W.add_dot(o.v2, o.h.T, mult=2.0)


def stat_transposed_operands(cm, o):
    # the same statistics with the roles exchanged: W2t is nh x nv
    o.W2t.add_dot(o.h, o.v.T, mult=0.5); o.W2t.add_dot(o.h2, o.v2.T, mult=-0.5)


def stat_three_sums_on_one_vector(cm, o):
    o.bv.add_sums(o.v, axis=1, mult=0.5); o.bv.add_sums(o.v2, axis=1, mult=-0.25); o.bv.add_sums(o.v, axis=1, mult=2.0)


def stat_sums_on_three_vectors(cm, o):
    o.bv.add_sums(o.v, axis=1); o.bh.add_sums(o.h, axis=1); o.bv2.add_sums(o.v2, axis=1); o.bv.add_sums(o.v2, axis=1, mult=-1.0)


def stat_sum_of_a_queued_result(cm, o):
    o.bv.add_sums(o.v, axis=1, mult=0.5); o.bv2.add_sums(o.bv, axis=1); o.bv.add_sums(o.v2, axis=1)


def stat_sum_into_a_queued_source(cm, o):
    col = o.v.slice(0, 1)                      # the first column of v as an nv x 1 vector
    o.bv.add_sums(o.v, axis=1, mult=0.5); col.add_sums(o.v2, axis=1); o.bv.add_sums(o.v, axis=1)


def stat_sums_other_axis_in_between(cm, o):
    o.bv.add_sums(o.v, axis=1, mult=0.5); o.row.add_sums(o.v, axis=0); o.bv.add_sums(o.v2, axis=1)


def stat_sums_then_read(cm, o):
    o.bh.add_sums(o.h, axis=1, mult=0.5); o.bh.add_sums(o.h2, axis=1, mult=-0.5)
    return o.bh.asarray().view(np.uint32).copy()


def stat_sum_with_assignment(cm, o):
    o.bv.assign(0); o.bv.add_sums(o.v, axis=1); o.bh.assign(1.0); o.bh.add_sums(o.h, axis=1, mult=3.0); o.bh.mult(0.5)


def stat_sums_of_transposed_views(cm, o):
    o.bh.add_sums(o.hT.T, axis=1, mult=0.5); o.bh.add_sums(o.h2, axis=1, mult=-0.5)      # hT is B x nh


# a weight gradient and the bias gradient of the same layer (deepnet/edge.py:236-242, layer.py:206-211): one
# product with the sums that follow it
def stat_gradient(cm, o):
    o.W.add_dot(o.v, o.h.T); o.bh.add_sums(o.h, axis=1)


def stat_gradient_two_sums(cm, o):
    o.W.add_dot(o.v, o.h.T, mult=0.5); o.bv.add_sums(o.v, axis=1); o.bh.add_sums(o.h, axis=1, mult=0.25)


def stat_gradient_sum_reads_the_target(cm, o):
    o.W.add_dot(o.v, o.h.T, mult=0.5); o.bv.add_sums(o.W, axis=1)


def stat_gradient_sum_into_an_operand(cm, o):
    col = o.v.slice(0, 1)
    o.W.add_dot(o.v, o.h.T, mult=0.5); col.add_sums(o.v2, axis=1); o.W.add_dot(o.v, o.h2.T)


def stat_gradient_then_second_product(cm, o):
    o.W.add_dot(o.v, o.h.T, mult=0.5); o.bh.add_sums(o.h, axis=1); o.W.add_dot(o.v2, o.h2.T, mult=-0.5); o.bh.add_sums(o.h2, axis=1)


def stat_gradients_of_two_layers(cm, o):
    o.W.add_dot(o.v, o.h.T); o.bh.add_sums(o.h, axis=1); o.W2t.add_dot(o.h2, o.v2.T); o.bv.add_sums(o.v2, axis=1)
    return o.bv.asarray().view(np.uint32).copy()


STATS = [stat_gradient, stat_gradient_two_sums, stat_gradient_sum_reads_the_target, stat_gradient_sum_into_an_operand,
         stat_gradient_then_second_product, stat_gradients_of_two_layers, stat_cd, stat_cd_subtract_dot, stat_pair_then_read, stat_single_then_read, stat_three_products, stat_products_into_two_targets,
         stat_second_product_reads_the_target, stat_overwriting_product_after_accumulating, stat_transposed_operands,
         stat_three_sums_on_one_vector, stat_sums_on_three_vectors, stat_sum_of_a_queued_result, stat_sum_into_a_queued_source,
         stat_sums_other_axis_in_between, stat_sums_then_read, stat_sum_with_assignment, stat_sums_of_transposed_views]


class _Stat(object):
    def __init__(self, cm, shape, seed):
        nv, nh, B = shape
        rng = np.random.default_rng(seed)
        g = lambda *d: cm.CUDAMatrix(_f(rng.standard_normal(d)))
        self.W, self.W2, self.W2t = g(nv, nh), g(nv, nh), g(nh, nv)
        self.v, self.v2, self.h, self.h2, self.hT = g(nv, B), g(nv, B), g(nh, B), g(nh, B), g(B, nh)
        self.bv, self.bv2, self.bh, self.row = g(nv, 1), g(nv, 1), g(nh, 1), g(1, B)

    def all(self):
        return [self.W, self.W2, self.W2t, self.v, self.v2, self.h, self.h2, self.bv, self.bv2, self.bh, self.row]


@pytest.mark.parametrize("seq", STATS, ids=lambda f: f.__name__)
@pytest.mark.parametrize("shape", STAT_SHAPES, ids=lambda s: "%dx%dx%d" % s)
def test_statistics_keep_their_bits(cm, seq, shape):
    res = []
    for deferred in (False, True):
        cm.set_deferred_epilogues(deferred)
        o = _Stat(cm, shape, 11)
        out = seq(cm, o)
        res.append([_bits(x) for x in o.all()] + ([out] if out is not None else []))
    cm.set_deferred_epilogues(True)
    for i, (w, g) in enumerate(zip(*res)):
        assert np.array_equal(g, w), "matrix %d differs" % i


def test_statistics_are_the_float64_definition(cm):
    o = _Stat(cm, (784, 500, 100), 12)
    w0, bv0, bh0 = o.W.asarray().astype(np.float64), o.bv.asarray().astype(np.float64), o.bh.asarray().astype(np.float64)
    v, v2, h, h2 = (x.asarray().astype(np.float64) for x in (o.v, o.v2, o.h, o.h2))
    stat_cd(cm, o)
    eps = np.float64(np.float32(0.01))
    assert np.allclose(o.W.asarray(), w0 + eps * (v @ h.T - v2 @ h2.T), rtol=1e-5, atol=1e-5)
    assert np.allclose(o.bv.asarray(), bv0 + eps * (v.sum(1, keepdims=True) - v2.sum(1, keepdims=True)), rtol=1e-5, atol=1e-5)
    assert np.allclose(o.bh.asarray(), bh0 + eps * (h.sum(1, keepdims=True) - h2.sum(1, keepdims=True)), rtol=1e-5, atol=1e-5)


# ---- consecutive parameter updates (deepnet updates every edge and layer of a net in turn, neuralnet.py:300-312)

def _upd(p, d, g, mom=0.9, lr=0.01, l2=None, l1=None, reset=True):
    d.mult(mom)
    if l2 is not None:
        d.add_mult(p, l2)
    if l1 is not None:
        d.add_mult_sign(p, l1)
    d.add_mult(g); p.add_mult(d, -lr)
    if reset:
        g.assign(0)


def upd_six_in_a_row(cm, P):
    for i in range(6):
        _upd(*P[i])


def upd_without_resets(cm, P):
    for i in range(4):
        _upd(*P[i], reset=False)


def upd_mixed_decays_and_resets(cm, P):
    _upd(*P[0], l2=0.001); _upd(*P[1], reset=False); _upd(*P[2], l1=0.002, l2=0.0005); _upd(*P[3], mom=0.5, lr=0.1, l1=0.01)


def upd_eleven(cm, P):
    for i in range(11):
        _upd(*P[i % 6], mom=0.9 - 0.05 * i)              # more than one launch holds; the same parameter again: in order


def upd_tied(cm, P):
    # the second update reads what the first wrote, the third writes what the second read (both are 1024 x 1)
    _upd(*P[1]); _upd(P[3][0], P[3][1], P[1][0], reset=False); _upd(P[1][0], P[1][1], P[3][2])


def upd_gradient_is_another_delta(cm, P):
    _upd(*P[0]); _upd(P[1][0], P[1][1], P[1][2]); _upd(P[0][0], P[0][2], P[0][1])     # roles exchanged on the same arrays


def upd_then_scale_that_is_no_update(cm, P):
    _upd(*P[0]); _upd(*P[1]); P[2][0].mult(0.5); P[2][0].add_mult(P[2][2], 2.0); P[2][1].add(P[2][0])


def upd_then_read(cm, P):
    _upd(*P[0]); _upd(*P[1], reset=False)
    return P[1][0].asarray().view(np.uint32).copy()


def upd_interleaved_with_a_product(cm, P):
    _upd(*P[0]); cm.dot(P[0][0], P[0][0].T, target=P[6]); _upd(*P[1]); _upd(*P[2])


def upd_reset_of_another_gradient(cm, P):
    P[0][1].mult(0.9); P[0][1].add_mult(P[0][2]); P[0][0].add_mult(P[0][1], -0.01); P[1][2].assign(0); _upd(*P[1])


UPDS = [upd_six_in_a_row, upd_without_resets, upd_mixed_decays_and_resets, upd_eleven, upd_tied, upd_gradient_is_another_delta,
        upd_then_scale_that_is_no_update, upd_then_read, upd_interleaved_with_a_product, upd_reset_of_another_gradient]


def _params_of_a_net(cm, seed):
    rng = np.random.default_rng(seed)
    g = lambda *d: cm.CUDAMatrix(_f(rng.standard_normal(d)))
    shapes = [(784, 1024), (1024, 1), (1024, 1024), (1024, 1), (37, 10), (10, 1)]
    P = [(g(*sh), g(*sh), g(*sh)) for sh in shapes]
    P.append(cm.empty((784, 784)))
    return P


@pytest.mark.parametrize("seq", UPDS, ids=lambda f: f.__name__)
def test_consecutive_updates_keep_their_bits(cm, seq):
    res = []
    for deferred in (False, True):
        cm.set_deferred_epilogues(deferred)
        P = _params_of_a_net(cm, 21)
        out = seq(cm, P)
        res.append([_bits(x) for t in P[:6] for x in t] + [_bits(P[6])] + ([out] if out is not None else []))
    cm.set_deferred_epilogues(True)
    for i, (w, g) in enumerate(zip(*res)):
        assert np.array_equal(g, w), "matrix %d differs" % i


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
                              (bench.MLP, 3, lambda o: o.W + o.b + o.dW + [o.loss] + o.mask),
                              (bench.RBMExample, 1, lambda o: [o.w_vh, o.w_v, o.w_h, o.wu_vh, o.wu_v, o.wu_h, o.v, o.h, o.r])):
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


def test_launch_deferred_queues_what_is_held_back(cm, rng):
    """A caller that goes on with its own work on the NULL stream (here: a plain hipMemcpy through the
    runtime, which the library does not see) finds the results of every call it has made."""
    import ctypes as ct
    hip = ct.CDLL('libamdhip64.so')
    hip.hipMemcpy.argtypes = [ct.c_void_p, ct.c_void_p, ct.c_size_t, ct.c_int]
    a, b = _f(rng.standard_normal((96, 64)) * 0.1), _f(rng.standard_normal((64, 40)))
    bias = _f(rng.standard_normal((96, 1)))
    A, B, bv = cm.CUDAMatrix(a), cm.CUDAMatrix(b), cm.CUDAMatrix(bias)
    T = cm.empty((96, 40)); T.assign(-3.0)
    cm.cuda_sync_threads()
    cm.dot(A, B, target=T)
    T.add_col_vec(bv)                         # both calls are held back now
    cm.launch_deferred()
    got = np.empty((96, 40), dtype=np.float32, order='F')
    assert hip.hipMemcpy(got.ctypes.data, ct.cast(T.p_mat.contents.data_device, ct.c_void_p), got.nbytes, 2) == 0
    want = a.astype(np.float64) @ b.astype(np.float64) + bias
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)
    T.apply_sigmoid()                         # and the library goes on from there
    np.testing.assert_allclose(T.asarray(), 1.0 / (1.0 + np.exp(-want)), rtol=1e-5, atol=1e-6)
    cm.launch_deferred()                      # nothing held back: no effect


# ---- random call sequences: whatever is held back, every matrix ends with the bits of the separate launches

def _random_sequence(cm, rng_ops, pool, vecs, rows, n_ops):
    """n_ops library calls on randomly chosen matrices of one shape family (m x n matrices, m x 1 and
    1 x n vectors, a k x m and a k x n operand pair per product): the operand choice includes every
    kind of aliasing the calls accept."""
    M = lambda: pool[rng_ops.integers(len(pool))]
    V = lambda: vecs[rng_ops.integers(len(vecs))]
    scal = lambda: float(np.float32(rng_ops.choice([0.0, 1.0, -1.0, 0.5, 0.9, -0.01, 2.0, 0.3])))
    m_, n_ = pool[0].shape
    lab, loss = cm.CUDAMatrix(_f(((np.arange(n_) * 5) % m_).reshape(1, n_))), cm.empty((1, n_))
    loss.assign(0)
    reads = []
    for _ in range(n_ops):
        op = rng_ops.integers(31)
        a, b, c = M(), M(), M()
        if op == 0: cm.dot(pool.A.T, pool.B, target=a)
        elif op == 1: a.add_dot(pool.A.T, pool.B, mult=scal())
        elif op == 2: a.add_dot(pool.A2.T, pool.B2, mult=scal())
        elif op == 3: a.subtract_dot(pool.A.T, pool.B2)
        elif op == 4: a.add_col_vec(V())
        elif op == 5: a.apply_sigmoid()
        elif op == 6: a.lower_bound(0)
        elif op == 7: a.sample_bernoulli(target=b)
        elif op == 8: a.mult(scal())
        elif op == 9: a.add_mult(b, scal())
        elif op == 10: a.add_mult_sign(b, scal())
        elif op == 11: a.assign(scal())
        elif op == 12: a.fill_with_rand()
        elif op == 13: a.greater_than(scal())
        elif op == 14: a.mult(b)
        elif op == 15: V().add_sums(a, axis=1, mult=scal())
        elif op == 16: rows[rng_ops.integers(len(rows))].add_sums(a, axis=0, mult=scal())
        elif op == 17: a.add(b, target=c)
        elif op == 18: cm.tanh(a)
        elif op == 19: reads.append(_bits(a))
        elif op == 20: a.add_mult(b)               # factor 1: the gradient of an update
        elif op == 22: a.apply_rectified_linear_deriv(b)
        elif op == 23: a.apply_rectified_linear_deriv(b, target=c)
        elif op == 24: a.apply_softmax() if rng_ops.integers(2) else a.apply_softmax(target=b)
        elif op == 25: a.get_softmax_cross_entropy(lab, loss)
        elif op == 26: a.apply_softmax_grad(lab, target=b)
        elif op == 27:      # a layer as deepnet spells it, with the variations that do and do not fold
            cm.dot(pool.A.T, pool.B, target=a)
            if rng_ops.integers(2): a.add_col_vec(V())
            kind = rng_ops.integers(4)
            if kind == 0: a.apply_sigmoid()
            elif kind == 1: a.lower_bound(0)
            elif kind == 2: cm.tanh(a)
            if rng_ops.integers(2):
                b.fill_with_rand()
                if rng_ops.integers(4): b.greater_than(scal())
                (a if rng_ops.integers(2) else c).mult(b)
            elif rng_ops.integers(2): a.sample_bernoulli(target=b)
        elif op == 29: a.less_than(b, target=b if rng_ops.integers(2) else c)
        elif op == 30: a.fill_with_rand(); a.less_than(b, target=b)
        elif op == 28:      # an output layer and its loss
            a.apply_softmax() if rng_ops.integers(2) else a.apply_softmax(target=b)
            src = a if rng_ops.integers(4) else b
            if rng_ops.integers(2): src.get_softmax_cross_entropy(lab, loss)
            if rng_ops.integers(4): src.apply_softmax_grad(lab, target=c)
        else: V().add_sums(a, axis=1)
    reads.append(_bits(loss))
    return reads


class _Pool(list):
    pass


@pytest.mark.parametrize("shape", [(500, 100, 784), (64, 128, 96), (33, 7, 20), (1024, 128, 128), (784, 500, 100)],
                         ids=lambda s: "%dx%dx%d" % s)
@pytest.mark.parametrize("seed", range(12))
def test_random_sequences_keep_their_bits(cm, shape, seed):
    m, n, k = shape
    res = []
    for deferred in (False, True):
        cm.set_deferred_epilogues(deferred)
        cm.CUDAMatrix.init_random(3 + seed)
        rng = np.random.default_rng(100 + seed)
        g = lambda *d: cm.CUDAMatrix(_f(rng.standard_normal(d) * 0.5))
        pool = _Pool(g(m, n) for _ in range(4))
        pool.A, pool.A2, pool.B, pool.B2 = g(k, m), g(k, m), g(k, n), g(k, n)
        vecs, rows = [g(m, 1) for _ in range(2)], [g(1, n) for _ in range(2)]
        reads = _random_sequence(cm, np.random.default_rng(5100 + seed), pool, vecs, rows, 60)
        after = cm.empty((64, 48)); after.fill_with_rand()
        res.append([_bits(x) for x in list(pool) + vecs + rows + [after]] + reads)
    cm.set_deferred_epilogues(True)
    cm.CUDAMatrix.init_random(1)
    assert len(res[0]) == len(res[1])
    for i, (w, gt) in enumerate(zip(*res)):
        assert np.array_equal(gt, w), "result %d differs" % i
