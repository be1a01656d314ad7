"""The conv stage of a deepnet edge (deepnet_amd/convolutions.py, mirroring the reference's
deepnet/convolutions.py:5-184) against its float64 restatement: forward state, gradient
w.r.t. the inputs and w.r.t. the weights, through the same buffers the reference reuses
(in-place MaxPoolUndo, ResponseNormUndo on a copy).  Tolerance: the conv bar, 1e-4 relative
(plus 2e-5 of the largest value where a sum cancels)."""
import os
import sys
import types

import numpy as np
import pytest

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from oracle import conv_oracle as co   # noqa: E402

pytestmark = pytest.mark.gpu


def _f(a):
    return np.asarray(a, dtype=np.float32, order='F')


def _close(got, want):
    want = np.asarray(want)
    return np.allclose(got, want, rtol=1e-4, atol=2e-5 * np.abs(want).max())


@pytest.fixture(scope="module")
def cv_mod(cm, cc):
    from deepnet_amd import convolutions
    return convolutions


STAGES = [  # N, C, H, F, k, stride, padding, pool (size, stride) or None, norm size or None, conv (False: local)
    (128, 3, 32, 64, 5, 1, 2, (3, 2), 5, True),      # benchmark config 4: conv -> pool -> rnorm
    (128, 3, 16, 32, 5, 1, 2, None, None, True),
    (64, 3, 16, 32, 5, 1, 2, (3, 2), None, True),
    (64, 4, 12, 16, 3, 1, 1, None, 3, True),
    (32, 16, 13, 32, 3, 2, 0, (2, 2), 5, True),      # strided modules, many colours
    (16, 2, 8, 16, 3, 1, 1, (2, 2), 3, False),       # locally connected
    (100, 1, 28, 64, 5, 1, 2, (3, 2), None, True),   # the first layer of deepnet's example convnet at its batch size of 100
]


@pytest.mark.parametrize("N,C,H,F,k,s,p,pool,norm,conv", STAGES)
def test_stage_forward_backward_and_weight_gradient(cm, cc, cv_mod, N, C, H, F, k, s, p, pool, norm, conv):
    r = np.random.default_rng(N + H + F)
    cv = cv_mod.ConvParams(size=k, stride=s, padding=p, num_filters=F, num_colors=C,
                           max_pool=pool is not None, pool_size=pool[0] if pool else 0,
                           pool_stride=pool[1] if pool else 0, rnorm=norm is not None, norm_size=norm or 0)
    n_locs = co.n_modules(H, k, s, p)
    n_out = (n_locs - cv.pool_size) // cv.pool_stride + 1 if pool else n_locs
    wcols = C * k * k * (1 if conv else n_locs * n_locs)
    inputs = _f(r.standard_normal((C * H * H, N)))
    w = _f(0.1 * r.standard_normal((F, wcols)))
    deriv = _f(r.standard_normal((F * n_out * n_out, N)))
    W = cm.CUDAMatrix(w)
    edge = cv_mod.ConvEdge(W, cv, inputs.shape, deriv.shape, conv=conv)
    state = cm.empty(deriv.shape)
    cv_mod.ConvolveUp(cm.CUDAMatrix(inputs), edge, state)
    fwd = co.stage_forward(inputs, w, cv, local=not conv)
    assert _close(state.asarray(), fwd['state'])
    if norm:
        assert np.allclose(edge.denoms.asarray(), fwd['denoms'], rtol=1e-5)

    layer = types.SimpleNamespace(dirty=False, is_input=False, deriv=cm.empty(inputs.shape))
    cv_mod.AccumulateConvDeriv(layer, edge, cm.CUDAMatrix(deriv))
    grad = cm.empty(w.shape)
    cv_mod.ConvOuter(edge, grad)
    d_in, d_w = co.stage_backward(fwd, w, cv, deriv, local=not conv)
    assert layer.dirty
    assert _close(layer.deriv.asarray(), d_in)
    assert _close(grad.asarray(), d_w)
    # the forward state survives the backward pass (the next step's loss reads it)
    assert _close(state.asarray(), fwd['state'])
    with pytest.raises(Exception):
        cv_mod.AccumulateConvDeriv(layer, edge, cm.CUDAMatrix(deriv))     # a second gradient: refused
    edge.free_device_memory()


def test_input_layer_gets_no_gradient_but_weights_do(cm, cc, cv_mod):
    N, C, H, F, k = 32, 3, 10, 16, 3
    r = np.random.default_rng(5)
    cv = cv_mod.ConvParams(size=k, stride=1, padding=1, num_filters=F, num_colors=C, max_pool=True, pool_size=2,
                           pool_stride=2)
    inputs = _f(r.standard_normal((C * H * H, N)))
    w = _f(0.1 * r.standard_normal((F, C * k * k)))
    deriv = _f(r.standard_normal((F * 25, N)))
    edge = cv_mod.ConvEdge(cm.CUDAMatrix(w), cv, inputs.shape, deriv.shape)
    state = cm.empty(deriv.shape)
    cv_mod.ConvolveUp(cm.CUDAMatrix(inputs), edge, state)
    sentinel = _f(np.full(inputs.shape, 7.0))
    layer = types.SimpleNamespace(dirty=False, is_input=True, deriv=cm.CUDAMatrix(sentinel))
    cv_mod.AccumulateConvDeriv(layer, edge, cm.CUDAMatrix(deriv))
    assert np.array_equal(layer.deriv.asarray(), sentinel)
    grad = cm.empty(w.shape)
    cv_mod.ConvOuter(edge, grad)
    fwd = co.stage_forward(inputs, w, cv)
    _, d_w = co.stage_backward(fwd, w, cv, deriv)
    assert _close(grad.asarray(), d_w)
    edge.free_device_memory()


def test_probabilistic_pooling_uses_minus_log_uniform_weights(cm, cc, cv_mod):
    N, C, H, F, k = 32, 2, 8, 16, 3
    r = np.random.default_rng(6)
    cv = cv_mod.ConvParams(size=k, stride=1, padding=1, num_filters=F, num_colors=C, max_pool=True, pool_size=2,
                           pool_stride=2, prob=True)
    inputs = _f(r.standard_normal((C * H * H, N)))
    w = _f(0.1 * r.standard_normal((F, C * k * k)))
    edge = cv_mod.ConvEdge(cm.CUDAMatrix(w), cv, inputs.shape, (F * 16, N))
    state = cm.empty((F * 16, N))
    cv_mod.ConvolveUp(cm.CUDAMatrix(inputs), edge, state)
    rnd = edge.rnd.asarray()
    assert np.all(rnd >= 0) and np.all(np.isfinite(rnd))                    # -log(u), u in (0, 1]
    assert abs(rnd.mean() - 1.0) < 0.05                                     # exponential variates
    want = co.prob_max_pool(edge.unpooled_layer.asarray(), rnd, F, 2, 0, 2, 4)
    assert np.array_equal(state.asarray(), want.T.astype(np.float32))
    with pytest.raises(Exception):
        cv_mod.AddConvolveUp(None, edge, state)
    edge.free_device_memory()
