"""Training steps of feed-forward nets through deepnet_amd/{layer,parameter,neuralnet}.py (the
step path of the reference's deepnet/neuralnet.py:138-337, its activation layers and
parameter.py:80-126) against the float64 restatement in oracle/net_oracle.py, which is itself
pinned against torch.optim.SGD.  The dropout masks the device drew are read back and fed to the
oracle, so both sides train on the same units.  Tolerances: parameters after k steps within 1e-4
relative (+1e-6 absolute: float32 parameters of size ~0.01-0.3), losses within 1e-5 relative."""
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from oracle import net_oracle as no   # noqa: E402

pytestmark = pytest.mark.gpu


def _f(a):
    return np.asarray(a, dtype=np.float32, order='F')


@pytest.fixture(scope="module")
def dn(cm, cc):
    import types
    from deepnet_amd import layer, neuralnet, parameter, convolutions
    return types.SimpleNamespace(layer=layer, nn=neuralnet, P=parameter, cv=convolutions)


def _hyp(dn, **kw):
    """The same hyper-parameters for the device classes and the oracle."""
    return dn.P.Hyperparams(**kw), no.Hyper(**{k: v for k, v in kw.items() if k != 'activation'})


def _build_chain(dn, spec, B, rng, fused=False):
    """spec: list of (activation, dims, layer kwargs for Hyperparams, edge dict or None).
    Returns (device net, oracle net)."""
    layers, edges, olayers = [], [], []
    for i, (act, dims, hkw, edge) in enumerate(spec):
        hd, ho = _hyp(dn, activation=act, **hkw)
        last = i == len(spec) - 1
        numlabels = dims if (last and act == dn.P.SOFTMAX) else 1
        bias = None if i == 0 else _f(0.1 * rng.standard_normal((dims, 1)))
        L = dn.layer.CreateLayer(act, 'layer%d' % i, 1 if numlabels > 1 else dims, B, hyperparams=hd,
                                 numlabels=numlabels, is_input=i == 0, is_output=last,
                                 loss_function=(edge or {}).get('loss', dn.P.CROSS_ENTROPY) if last else dn.P.SQUARED_LOSS,
                                 bias=bias)
        L.fused = fused
        layers.append(L)
        ol = {'act': act, 'hyper': ho}
        if i > 0:
            he_d, he_o = _hyp(dn, **edge.get('hyper', {}))
            E = dn.nn.Edge(layers[i - 1], L, edge['w'], hyperparams=he_d, conv_params=edge.get('cv'),
                           local=edge.get('local', False))
            E.fused = fused
            edges.append(E)
            ol.update(bias=bias, edge={'w': edge['w'], 'hyper': he_o, 'cv': edge.get('cv'), 'local': edge.get('local', False)},
                      loss=edge.get('loss', 'CROSS_ENTROPY'))
        olayers.append(ol)
    return dn.nn.NeuralNet(layers, edges), no.Net(olayers)


def _train_and_compare(cm, net, onet, batches, rtol=1e-4, atol=1e-6):
    for step, (x, t) in enumerate(batches):
        net.layer[0].data.assign(cm.CUDAMatrix(_f(x)))
        net.layer[-1].data.assign(cm.CUDAMatrix(_f(t)))
        losses = net.TrainOneBatch(step)
        masks = [L.mask.asarray().copy() if L.hyperparams.dropout else None for L in net.layer]
        perf = onet.train_step(x, t, step, masks=masks)
        assert len(losses) == 1
        for key, want in perf.items():
            assert abs(getattr(losses[0], key) - want) <= 1e-5 * max(1.0, abs(want)), (step, key)
        for i, E in enumerate(net.edge):
            assert np.allclose(E.params['weight'].asarray(), onet.layers[i + 1]['edge']['w'], rtol=rtol, atol=atol), (step, i)
            assert np.allclose(net.layer[i + 1].params['bias'].asarray(), onet.layers[i + 1]['bias'], rtol=rtol, atol=atol), (step, i)
            assert not E.gradient.asarray().any() and not net.layer[i + 1].gradient.asarray().any()   # reset after the update


def test_mlp_of_benchmark_config_3_trains_like_the_oracle(cm, dn):
    """784-1024-1024-10, ReLU, dropout 0.5 on the hidden layers, momentum 0.9, batch 128."""
    rng = np.random.default_rng(3)
    cm.CUDAMatrix.init_random(3)
    sizes, B = (784, 1024, 1024, 10), 128
    sgd = dict(base_epsilon=0.01, initial_momentum=0.9, final_momentum=0.9)
    w = [_f(0.01 * rng.standard_normal((sizes[i], sizes[i + 1]))) for i in range(3)]
    spec = [(dn.P.LINEAR, 784, sgd, None),
            (dn.P.RECTIFIED_LINEAR, 1024, dict(dropout=True, dropout_prob=0.5, **sgd), {'w': w[0], 'hyper': sgd}),
            (dn.P.RECTIFIED_LINEAR, 1024, dict(dropout=True, dropout_prob=0.5, **sgd), {'w': w[1], 'hyper': sgd}),
            (dn.P.SOFTMAX, 10, sgd, {'w': w[2], 'hyper': sgd})]
    net, onet = _build_chain(dn, spec, B, rng)
    batches = [(rng.random((784, B)), rng.integers(0, 10, (1, B)).astype(np.float64)) for _ in range(3)]
    _train_and_compare(cm, net, onet, batches)
    # evaluation: no sampling, hidden states scaled by 1 - dropout_prob
    x, t = batches[0]
    net.layer[0].data.assign(cm.CUDAMatrix(_f(x)))
    net.layer[-1].data.assign(cm.CUDAMatrix(_f(t)))
    losses = net.EvaluateOneBatch()
    probs = onet.forward(x, train=False)
    assert np.allclose(net.layer[-1].state.asarray(), probs, rtol=1e-4, atol=1e-7)
    perf, _ = onet.loss_and_deriv(t)
    assert abs(losses[0].cross_entropy - perf['cross_entropy']) <= 1e-5 * perf['cross_entropy']
    assert losses[0].correct_preds == perf['correct_preds']


@pytest.mark.parametrize("fused", [False, True])
def test_regularised_tanh_net_with_logistic_outputs(cm, dn, fused):
    """L2 and L1 decay, a column-norm limit, decaying learning rate, rising momentum, dropout on
    tanh units (the explicit mask in their derivative) and on the input layer; logistic outputs
    with cross-entropy.  `fused` routes the updates through the one-pass momentum_update."""
    rng = np.random.default_rng(11)
    cm.CUDAMatrix.init_random(11)
    sizes, B = (96, 160, 48), 64
    reg = dict(base_epsilon=0.1, initial_momentum=0.5, final_momentum=0.9, momentum_change_steps=3,
               epsilon_decay=dn.P.INVERSE_T, epsilon_decay_half_life=4, apply_l2_decay=True, l2_decay=0.001,
               apply_l1_decay=True, l1_decay=0.0005, apply_l1decay_after=1, apply_weight_norm=True, weight_norm=1.2)
    w = [_f(0.3 * rng.standard_normal((sizes[i], sizes[i + 1]))) for i in range(2)]
    spec = [(dn.P.LINEAR, 96, dict(dropout=True, dropout_prob=0.25), None),
            (dn.P.TANH, 160, dict(dropout=True, dropout_prob=0.5, base_epsilon=0.1), {'w': w[0], 'hyper': reg}),
            (dn.P.LOGISTIC, 48, dict(base_epsilon=0.1), {'w': w[1], 'hyper': reg, 'loss': 'CROSS_ENTROPY'})]
    net, onet = _build_chain(dn, spec, B, rng, fused=fused)
    batches = [(rng.standard_normal((96, B)), (rng.random((48, B)) < 0.3).astype(np.float64)) for _ in range(4)]
    _train_and_compare(cm, net, onet, batches, rtol=2e-4, atol=2e-6)
    norms = np.sqrt((net.edge[0].params['weight'].asarray().astype(np.float64) ** 2).sum(axis=0))
    assert np.all(norms <= 1.2 * (1 + 1e-5)) and np.any(norms > 1.19)      # the limit is active


def test_fused_updates_leave_the_same_bits(cm, dn):
    results = []
    for fused in (False, True):
        rng = np.random.default_rng(21)
        cm.CUDAMatrix.init_random(21)
        sgd = dict(base_epsilon=0.05, initial_momentum=0.9, final_momentum=0.9, apply_l2_decay=True, l2_decay=0.002)
        w = [_f(0.1 * rng.standard_normal(s)) for s in ((64, 128), (128, 8))]
        spec = [(dn.P.LINEAR, 64, {}, None),
                (dn.P.LOGISTIC, 128, dict(dropout=True, base_epsilon=0.05), {'w': w[0], 'hyper': sgd}),
                (dn.P.SOFTMAX, 8, dict(base_epsilon=0.05), {'w': w[1], 'hyper': sgd})]
        net, _ = _build_chain(dn, spec, 32, rng, fused=fused)
        for step in range(3):
            net.layer[0].data.assign(cm.CUDAMatrix(_f(rng.standard_normal((64, 32)))))
            net.layer[-1].data.assign(cm.CUDAMatrix(_f(rng.integers(0, 8, (1, 32)))))
            net.TrainOneBatch(step)
        results.append([E.params['weight'].asarray().copy() for E in net.edge] +
                       [L.params['bias'].asarray().copy() for L in net.layer[1:]])
    for a, b in zip(*results):
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_small_convnet_trains_like_the_oracle(cm, dn):
    """3x16x16 -> conv 5x5 pad 2 (16 filters) + pool 3/2 + rnorm 5 -> ReLU -> dense softmax(10)."""
    rng = np.random.default_rng(4)
    cm.CUDAMatrix.init_random(4)
    B, C, H, F, k = 64, 3, 16, 16, 5
    cvp = dn.cv.ConvParams(size=k, stride=1, padding=2, num_filters=F, num_colors=C, max_pool=True, pool_size=3,
                           pool_stride=2, rnorm=True, norm_size=5)
    O = (16 - 3) // 2 + 1
    sgd = dict(base_epsilon=0.05, initial_momentum=0.5, final_momentum=0.5)
    wc = _f(0.1 * rng.standard_normal((F, C * k * k)))
    wd = _f(0.05 * rng.standard_normal((F * O * O, 10)))
    spec = [(dn.P.LINEAR, C * H * H, {}, None),
            (dn.P.RECTIFIED_LINEAR, F * O * O, dict(base_epsilon=0.05), {'w': wc, 'hyper': sgd, 'cv': cvp}),
            (dn.P.SOFTMAX, 10, dict(base_epsilon=0.05), {'w': wd, 'hyper': sgd})]
    net, onet = _build_chain(dn, spec, B, rng)
    batches = [(rng.standard_normal((C * H * H, B)), rng.integers(0, 10, (1, B)).astype(np.float64)) for _ in range(3)]
    _train_and_compare(cm, net, onet, batches, rtol=2e-4, atol=2e-6)


def test_example_convnet_of_the_reference_at_its_batch_size(cm, dn):
    """deepnet/examples/convnet/model_conv.pbtxt: 784 -> conv 5x5 pad 2 (64 filters) + pool 3/2 ->
    10816 ReLU -> conv 5x5 pad 2 (64 -> 64) + pool 3/2 -> 2304 ReLU -> 1024 ReLU -> softmax(10),
    batch 100 (train.pbtxt), its learning rates, momentum schedules and L2 decay."""
    rng = np.random.default_rng(12)
    cm.CUDAMatrix.init_random(12)
    B = 100
    net_h = dict(base_epsilon=0.01, initial_momentum=0.5, final_momentum=0.9, momentum_change_steps=10000,
                 apply_l2_decay=True, l2_decay=0.001)
    bias_h = dict(net_h, apply_l2_decay=False)
    conv_h = dict(base_epsilon=0.001, initial_momentum=0.9, final_momentum=0.9, momentum_change_steps=20000)
    cv1 = dn.cv.ConvParams(size=5, stride=1, padding=2, num_filters=64, num_colors=1, max_pool=True, pool_size=3, pool_stride=2)
    cv2 = dn.cv.ConvParams(size=5, stride=1, padding=2, num_filters=64, num_colors=64, max_pool=True, pool_size=3, pool_stride=2)
    w1 = _f(0.1 * rng.standard_normal((64, 25)))
    w2 = _f(0.02 * rng.standard_normal((64, 64 * 25)))
    w3 = _f(0.02 * rng.standard_normal((2304, 1024)))
    w4 = _f(0.05 * rng.standard_normal((1024, 10)))
    spec = [(dn.P.LINEAR, 784, {}, None),
            (dn.P.RECTIFIED_LINEAR, 10816, bias_h, {'w': w1, 'hyper': conv_h, 'cv': cv1}),
            (dn.P.RECTIFIED_LINEAR, 2304, bias_h, {'w': w2, 'hyper': conv_h, 'cv': cv2}),
            (dn.P.RECTIFIED_LINEAR, 1024, bias_h, {'w': w3, 'hyper': net_h}),
            (dn.P.SOFTMAX, 10, bias_h, {'w': w4, 'hyper': net_h})]
    net, onet = _build_chain(dn, spec, B, rng)
    batches = [(rng.random((784, B)), rng.integers(0, 10, (1, B)).astype(np.float64)) for _ in range(2)]
    _train_and_compare(cm, net, onet, batches, rtol=2e-4, atol=2e-6)


def test_smooth_relu_hidden_units(cm, dn):
    """deepnet/smooth_relu_layer.py: softplus units whose derivative is taken from the output."""
    rng = np.random.default_rng(15)
    sizes, B = (24, 40, 6), 16
    sgd = dict(base_epsilon=0.05, initial_momentum=0.5, final_momentum=0.5)
    w = [_f(0.3 * rng.standard_normal((sizes[i], sizes[i + 1]))) for i in range(2)]
    spec = [(dn.P.LINEAR, 24, sgd, None),
            (dn.P.RECTIFIED_LINEAR_SMOOTH, 40, sgd, {'w': w[0], 'hyper': sgd}),
            (dn.P.SOFTMAX, 6, sgd, {'w': w[1], 'hyper': sgd})]
    net, onet = _build_chain(dn, spec, B, rng)
    assert type(net.layer[1]).__name__ == 'SmoothReluLayer'
    batches = [(3.0 * rng.standard_normal((24, B)), rng.integers(0, 6, (1, B)).astype(np.float64)) for _ in range(3)]
    _train_and_compare(cm, net, onet, batches)


def test_sin_and_cos_hidden_units(cm, dn):
    """deepnet/sin_layer.py, cos_layer.py: the pre-activation is kept and the derivative taken from it."""
    rng = np.random.default_rng(14)
    sizes, B = (24, 40, 32, 6), 16
    sgd = dict(base_epsilon=0.05, initial_momentum=0.5, final_momentum=0.5)
    w = [_f(0.3 * rng.standard_normal((sizes[i], sizes[i + 1]))) for i in range(3)]
    spec = [(dn.P.LINEAR, 24, sgd, None),
            (dn.P.SIN, 40, sgd, {'w': w[0], 'hyper': sgd}),
            (dn.P.COS, 32, sgd, {'w': w[1], 'hyper': sgd}),
            (dn.P.SOFTMAX, 6, sgd, {'w': w[2], 'hyper': sgd})]
    net, onet = _build_chain(dn, spec, B, rng)
    assert type(net.layer[1]).__name__ == 'SinLayer' and type(net.layer[2]).__name__ == 'CosLayer'
    batches = [(3.0 * rng.standard_normal((24, B)), rng.integers(0, 6, (1, B)).astype(np.float64)) for _ in range(3)]
    _train_and_compare(cm, net, onet, batches)
