"""Contrastive-divergence steps through deepnet_amd/dbm.py (the step of the reference's
deepnet/dbm.py:64-282) against the float64 restatement oracle/net_oracle.rbm_cd_step, fed the
hidden samples the device drew (recorded as they are drawn).  Tolerance: parameters within 1e-4
relative + 1e-6 after every step, reconstruction error within 1e-5 relative."""
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from oracle import net_oracle as no   # noqa: E402

pytestmark = pytest.mark.gpu


def _f(a):
    return np.asarray(a, dtype=np.float32, order='F')


def _record_samples(layer):
    """Keep a host copy of every sample the layer draws, in order."""
    drawn = []
    original = layer.Sample

    def sample():
        original()
        drawn.append(layer.sample.asarray().copy())
    layer.Sample = sample
    return drawn


def _rbm(cm, nv, nh, B, rng, optimizer, gibbs_steps, hyp_kw):
    from deepnet_amd import dbm, layer as dl, neuralnet as dnn, parameter as dp
    hv = dp.Hyperparams(activation=dp.LOGISTIC, **hyp_kw)
    hh = dp.Hyperparams(activation=dp.LOGISTIC, **hyp_kw)
    he = dp.Hyperparams(**hyp_kw)
    w = _f(0.05 * rng.standard_normal((nv, nh)))
    bv, bh = _f(0.1 * rng.standard_normal((nv, 1))), _f(0.1 * rng.standard_normal((nh, 1)))
    vis = dl.LogisticLayer('visible', nv, B, hyperparams=hv, is_input=True, bias=bv)
    hid = dl.LogisticLayer('hidden', nh, B, hyperparams=hh, bias=bh)
    edge = dnn.Edge(vis, hid, w, hyperparams=he, directed=False)
    net = dbm.DBM([vis, hid], [edge], optimizer=optimizer, gibbs_steps=gibbs_steps)
    p = {'W': w.astype(np.float64), 'bv': bv.astype(np.float64), 'bh': bh.astype(np.float64),
         'dW': np.zeros((nv, nh)), 'dbv': np.zeros((nv, 1)), 'dbh': np.zeros((nh, 1))}
    oh = no.Hyper(**hyp_kw)
    return net, vis, hid, edge, p, {'edge': oh, 'vis': oh, 'hid': oh}


def _compare(vis, hid, edge, p, tag):
    for got, want in ((edge.params['weight'], p['W']), (vis.params['bias'], p['bv']), (hid.params['bias'], p['bh'])):
        assert np.allclose(got.asarray(), want, rtol=1e-4, atol=1e-6), tag


@pytest.mark.parametrize("gibbs_steps", [1, 3])
def test_rbm_of_benchmark_config_1_contrastive_divergence(cm, rng, gibbs_steps):
    """784 visible x 500 hidden logistic units, batch 100, momentum rising from 0.5 to 0.9."""
    cm.CUDAMatrix.init_random(1)
    nv, nh, B = 784, 500, 100
    kw = dict(base_epsilon=0.05, initial_momentum=0.5, final_momentum=0.9, momentum_change_steps=2)
    net, vis, hid, edge, p, oh = _rbm(cm, nv, nh, B, rng, 'CD', gibbs_steps, kw)
    drawn = _record_samples(hid)
    for step in range(3):
        v = (rng.random((nv, B)) < 0.13).astype(np.float64)
        vis.data.assign(cm.CUDAMatrix(_f(v)))
        del drawn[:]
        losses = net.TrainOneBatch(step)
        assert len(drawn) == gibbs_steps + 1                 # one before the sweeps, one after each
        err = no.rbm_cd_step(p, oh, v, step, drawn[:gibbs_steps])
        assert len(losses) == 1 and abs(losses[0].error - err) <= 1e-5 * err
        _compare(vis, hid, edge, p, step)
        assert not edge.gradient.asarray().any() and not vis.gradient.asarray().any()
        assert set(np.unique(drawn[0])) <= {0.0, 1.0}
    # evaluation: one up pass, the reconstruction from the hidden probabilities, its squared error
    v = (rng.random((nv, B)) < 0.13).astype(np.float64)
    vis.data.assign(cm.CUDAMatrix(_f(v)))
    losses = net.EvaluateOneBatch()
    h = no.activate('LOGISTIC', p['W'].T @ v + p['bh'])
    recon = no.activate('LOGISTIC', p['W'] @ h + p['bv'])
    want = float(((recon - v) ** 2).sum())
    assert len(losses) == 1 and abs(losses[0].error - want) <= 1e-4 * want


def test_rbm_with_persistent_chains(cm, rng):
    """PCD: the negative chain starts at the positive states once (step 0) and then carries
    over from step to step; the hidden sample that drives a sweep is the last one drawn."""
    cm.CUDAMatrix.init_random(2)
    nv, nh, B = 96, 64, 32
    kw = dict(base_epsilon=0.05, initial_momentum=0.5, final_momentum=0.5, apply_l2_decay=True, l2_decay=0.001)
    net, vis, hid, edge, p, oh = _rbm(cm, nv, nh, B, rng, 'PCD', 2, kw)
    drawn = _record_samples(hid)
    carried = None
    for step in range(3):
        v = (rng.random((nv, B)) < 0.3).astype(np.float64)
        vis.data.assign(cm.CUDAMatrix(_f(v)))
        del drawn[:]
        losses = net.TrainOneBatch(step)
        # step 0 draws once more, when the chains are initialised at the positive states
        assert len(drawn) == (3 if step == 0 else 2)
        used = ([drawn[0], drawn[1]] if step == 0 else [carried, drawn[0]])
        carried = drawn[-1]
        no.rbm_cd_step(p, oh, v, step, used)
        _compare(vis, hid, edge, p, step)
        # with persistent chains the loss is the reconstruction from the positive phase
        assert len(losses) == 1 and np.isfinite(losses[0].error)
        assert vis.state is vis.pos_state and hid.sample is hid.pos_sample      # back in the positive phase


def test_fused_route_leaves_the_same_bits(cm):
    """`fused = True` on layers and edges sends every up pass through dot_bias_act and every
    update through momentum_update: the parameters after two CD-1 steps are bit-identical."""
    results = []
    for fused in (False, True):
        r = np.random.default_rng(8)
        cm.CUDAMatrix.init_random(8)
        kw = dict(base_epsilon=0.05, initial_momentum=0.7, final_momentum=0.7, apply_l2_decay=True, l2_decay=0.002)
        net, vis, hid, edge, _, _ = _rbm(cm, 200, 120, 40, r, 'CD', 1, kw)
        for obj in (vis, hid, edge):
            obj.fused = fused
        for step in range(2):
            vis.data.assign(cm.CUDAMatrix(_f(r.random((200, 40)) < 0.2)))
            net.TrainOneBatch(step)
        results.append([m.asarray().copy() for m in (edge.params['weight'], vis.params['bias'], hid.params['bias'])])
    for a, b in zip(*results):
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_three_layer_machine_runs_mean_field_and_gibbs_sweeps(cm, rng):
    """A deep Boltzmann machine (visible - hidden1 - hidden2): no closed form to compare with,
    so only what must hold: the middle layer is computed from both neighbours, the updates are
    finite, move every parameter and reset the gradients."""
    from deepnet_amd import dbm, layer as dl, neuralnet as dnn, parameter as dp
    cm.CUDAMatrix.init_random(3)
    sizes, B = (48, 32, 16), 16
    kw = dict(base_epsilon=0.1)
    layers = [dl.LogisticLayer('l%d' % i, n, B, hyperparams=dp.Hyperparams(activation=dp.LOGISTIC, **kw), is_input=i == 0)
              for i, n in enumerate(sizes)]
    ws = [_f(0.1 * rng.standard_normal((sizes[i], sizes[i + 1]))) for i in range(2)]
    edges = [dnn.Edge(layers[i], layers[i + 1], ws[i], hyperparams=dp.Hyperparams(**kw), directed=False) for i in range(2)]
    net = dbm.DBM(layers, edges, optimizer='CD', mf_steps=3, gibbs_steps=2)
    assert [n.name for n in net.node_list] == ['l0', 'l1', 'l2'] and len(layers[1].incoming_edge) == 2
    layers[0].data.assign(cm.CUDAMatrix(_f(rng.random((sizes[0], B)) < 0.4)))
    losses = net.TrainOneBatch(0)
    assert len(losses) == 1 and np.isfinite(losses[0].error)
    for e, w0 in zip(edges, ws):
        w1 = e.params['weight'].asarray()
        assert np.all(np.isfinite(w1)) and np.any(w1 != w0) and not e.gradient.asarray().any()
    # mean field of the middle layer: sigmoid(W1^T v + W2 h2 + b) from the states at hand
    net.PositivePhase(train=False)
    v, h2 = layers[0].state.asarray().astype(np.float64), layers[2].state.asarray().astype(np.float64)
    w1, w2 = (e.params['weight'].asarray().astype(np.float64) for e in edges)
    b1 = layers[1].params['bias'].asarray().astype(np.float64)
    # the last mean-field sweep updated l1 before l2, so recompute l2 from l1 instead
    h1 = layers[1].state.asarray().astype(np.float64)
    b2 = layers[2].params['bias'].asarray().astype(np.float64)
    assert np.allclose(h2, no.activate('LOGISTIC', w2.T @ h1 + b2), rtol=1e-5, atol=1e-6)
    assert v.shape == (sizes[0], B) and b1.shape == (sizes[1], 1)
