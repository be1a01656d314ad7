"""The two step sequences bench.py times (RBM.step = cudamat/examples/rbm_cudamat.py:46-89 at
config 1, MLP.step = the op sequence of deepnet/neuralnet.py:138-291 + parameter.py:80-106 at
config 3), and their fused variants, against the float64 oracle fed the random draws the
device made.  Tolerance: parameters within 1e-4 relative + 1e-6 after each of three steps."""
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench                                  # noqa: E402
from oracle import mwc, net_oracle as no      # noqa: E402

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("fused", [False, True])
def test_rbm_step_of_the_benchmark_against_the_oracle(cm, fused):
    cm.CUDAMatrix.init_random(1)
    host = mwc.MWC(mwc.load_multipliers(cm.MULTIPLIERS_PATH), 1)
    rbm = bench.RBM(cm)                                   # 784 x 500, batch 100, lr 0.01, seed 1
    v = rbm.v.asarray().astype(np.float64)
    p = {'W': rbm.W.asarray().astype(np.float64), 'bv': rbm.bv.asarray().astype(np.float64),
         'bh': rbm.bh.asarray().astype(np.float64)}
    for k, s in (('dW', p['W']), ('dbv', p['bv']), ('dbh', p['bh'])):
        p[k] = np.zeros_like(s)
    plain = no.Hyper(base_epsilon=rbm.lr, initial_momentum=0.0, final_momentum=0.0)     # the example has no momentum
    hyper = {'edge': plain, 'vis': plain, 'hid': plain}
    for step in range(3):
        (rbm.step_fused if fused else rbm.step)()
        h, hs = rbm.h.asarray(), rbm.hs.asarray()
        # the sample is the host generator's Bernoulli draw on the device's probabilities, bit for bit
        assert np.array_equal(hs, host.bernoulli(h).reshape(h.shape, order='F'))
        h_want = no.activate('LOGISTIC', p['W'].T @ v + p['bh'])
        assert np.allclose(h, h_want, rtol=1e-5, atol=1e-6)
        err = no.rbm_cd_step(p, hyper, v, step, [hs])
        v2 = rbm.v2.asarray().astype(np.float64)
        assert abs(((v2 - v) ** 2).sum() - err) <= 1e-5 * err
        for got, want in ((rbm.W, p['W']), (rbm.bv, p['bv']), (rbm.bh, p['bh'])):
            assert np.allclose(got.asarray(), want, rtol=1e-4, atol=1e-6), step


@pytest.mark.parametrize("fused", [False, True])
def test_mlp_step_of_the_benchmark_against_the_oracle(cm, fused):
    cm.CUDAMatrix.init_random(3)
    mlp = bench.MLP(cm)                                   # 784-1024-1024-10, batch 128, lr 0.01, momentum 0.9
    x, labels = mlp.x.asarray().astype(np.float64), mlp.labels.asarray()
    hyp = lambda **kw: no.Hyper(base_epsilon=mlp.lr, initial_momentum=mlp.mom, final_momentum=mlp.mom, **kw)
    layers = [{'act': 'LINEAR', 'hyper': hyp()}]
    for i, act in enumerate(('RECTIFIED_LINEAR', 'RECTIFIED_LINEAR', 'SOFTMAX')):
        layers.append({'act': act, 'hyper': hyp(dropout=i < 2, dropout_prob=0.5), 'bias': mlp.b[i].asarray(),
                       'edge': {'w': mlp.W[i].asarray(), 'hyper': hyp()}, 'loss': 'CROSS_ENTROPY'})
    onet = no.Net(layers)
    twin_masks = []
    if fused:
        # the fused step draws its dropout decisions without writing masks: a twin run of the plain
        # step from the same seed makes the same draws and leaves them in its masks
        twin = bench.MLP(cm)
        for step in range(3):
            twin.step()
            twin_masks.append([twin.mask[0].asarray().copy(), twin.mask[1].asarray().copy()])
        cm.CUDAMatrix.init_random(3)
    for step in range(3):
        (mlp.step_fused if fused else mlp.step)()
        m01 = twin_masks[step] if fused else [mlp.mask[0].asarray(), mlp.mask[1].asarray()]
        masks = [None, m01[0], m01[1], None]
        for m in masks[1:3]:
            assert set(np.unique(m)) <= {0.0, 1.0} and 0.45 < m.mean() < 0.55
        perf = onet.train_step(x, labels, step, masks=masks)
        assert abs(float(mlp.loss.asarray().sum()) - perf['cross_entropy']) <= 1e-4 * perf['cross_entropy']
        for i in range(3):
            L = onet.layers[i + 1]
            assert np.allclose(mlp.W[i].asarray(), L['edge']['w'], rtol=1e-4, atol=1e-6), (step, i)
            assert np.allclose(mlp.b[i].asarray(), L['bias'], rtol=1e-4, atol=1e-6), (step, i)
            assert np.allclose(mlp.dW[i].asarray(), L['edge']['w_delta'], rtol=1e-4, atol=1e-6), (step, i)
