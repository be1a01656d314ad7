#!/usr/bin/env python3
"""Benchmark of the MI355X matrix backend on synthetic data (one GPU).

A "step" is one pass over the elementwise / reduction / RNG op list of the
4096 x 4096 fp32 microbench, each op issued once on each of NSETS distinct
operand sets (so consecutive launches stream from HBM, not from the 256 MB
last-level cache).  `value` is the algorithmic bytes of a step divided by its
wall time (inputs resident in HBM, device synchronised on both sides).

Next to it, in the same JSON line:
  roofline      the axpy kernel (add_mult): algorithmic bytes per launch over the
                launch duration measured with HIP events on the NULL stream
  ops           per-op GB/s and fraction of the 8 TB/s HBM peak
  secondary     RBM CD-1 steps/s (784 x 500, batch 100), MLP steps/s, fp32 GEMM and
                conv TFLOP/s with their fraction of the 157.3 TFLOP/s MFMA peak
  cpu_baseline  the same op list timed through the C host restatement
                (oracle/host_backend.c) on this machine's cores
"""
import argparse
import ctypes as ct
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_FP32_PEAK_TFLOPS = 157.3
N = 4096
NSETS = 8


# ---------------------------------------------------------------- HIP events

class HipEvents(object):
    """hipEvent timing on the NULL stream (the stream the library launches on)."""

    def __init__(self, flush=None):
        self.flush = flush      # queues what the library holds back (cm.launch_deferred)
        self.hip = ct.CDLL('libamdhip64.so')
        self.hip.hipEventCreate.argtypes = [ct.POINTER(ct.c_void_p)]
        self.hip.hipEventRecord.argtypes = [ct.c_void_p, ct.c_void_p]
        self.hip.hipEventSynchronize.argtypes = [ct.c_void_p]
        self.hip.hipEventElapsedTime.argtypes = [ct.POINTER(ct.c_float), ct.c_void_p, ct.c_void_p]
        self.pool = []

    def new(self):
        ev = ct.c_void_p()
        assert self.hip.hipEventCreate(ct.byref(ev)) == 0
        self.pool.append(ev)
        return ev

    def record(self, ev):
        # (a call that the library holds back is not in the stream yet: it is queued first)
        if self.flush is not None:
            self.flush()
        assert self.hip.hipEventRecord(ev, None) == 0

    def elapsed_ms(self, a, b):
        assert self.hip.hipEventSynchronize(b) == 0
        ms = ct.c_float()
        assert self.hip.hipEventElapsedTime(ct.byref(ms), a, b) == 0
        return ms.value


# ---------------------------------------------------------------- workload

def build_c2(cm, seed=2):
    """Operand sets of the 4096^2 microbench (seeded, U(-1,1); probabilities U(0,1))."""
    rng = np.random.default_rng(seed)
    sets = []
    for _ in range(NSETS):
        s = {}
        s['A'] = cm.CUDAMatrix(np.asarray(rng.uniform(-1, 1, (N, N)), dtype=np.float32, order='F'))
        s['B'] = cm.CUDAMatrix(np.asarray(rng.uniform(-1, 1, (N, N)), dtype=np.float32, order='F'))
        s['P'] = cm.CUDAMatrix(np.asarray(rng.random((N, N)), dtype=np.float32, order='F'))
        s['T'] = cm.empty((N, N))
        s['col'] = cm.CUDAMatrix(np.asarray(rng.uniform(-1, 1, (N, 1)), dtype=np.float32, order='F'))
        s['row'] = cm.CUDAMatrix(np.asarray(rng.uniform(-1, 1, (1, N)), dtype=np.float32, order='F'))
        s['r0'] = cm.empty((1, N))
        s['r1'] = cm.empty((N, 1))
        sets.append(s)
    return sets


E = N * N
VEC = N * 4
# name -> (algorithmic bytes per launch, callable(set))
C2_OPS = [
    ('add_mult', 12 * E, lambda cm, s: s['A'].add_mult(s['B'], 0.5)),
    ('mult', 12 * E, lambda cm, s: s['A'].mult(s['B'], target=s['T'])),
    ('apply_sigmoid', 8 * E, lambda cm, s: s['A'].apply_sigmoid(target=s['T'])),
    ('apply_exp', 8 * E, lambda cm, s: cm.exp(s['A'], target=s['T'])),
    ('mult_by_col', 8 * E + VEC, lambda cm, s: s['A'].mult_by_col(s['col'], target=s['T'])),
    ('add_row_vec', 8 * E + VEC, lambda cm, s: s['A'].add_row_vec(s['row'], target=s['T'])),
    ('sum_axis0', 4 * E + VEC, lambda cm, s: s['A'].sum(axis=0, target=s['r0'])),
    ('sum_axis1', 4 * E + VEC, lambda cm, s: s['A'].sum(axis=1, target=s['r1'])),
    ('max_axis0', 4 * E + VEC, lambda cm, s: s['A'].max(axis=0, target=s['r0'])),
    ('max_axis1', 4 * E + VEC, lambda cm, s: s['A'].max(axis=1, target=s['r1'])),
    ('softmax', 8 * E, lambda cm, s: s['A'].apply_softmax(target=s['T'])),
    ('fill_with_rand', 4 * E, lambda cm, s: s['T'].fill_with_rand()),
    ('sample_bernoulli', 8 * E, lambda cm, s: s['P'].sample_bernoulli(target=s['T'])),
]
STEP_BYTES = NSETS * sum(b for _, b, _ in C2_OPS)


def run_c2_step(cm, sets, ev=None, marks=None):
    """One step.  With ev/marks, brackets the NSETS launches of every op that has a pair of events in marks."""
    for name, _, fn in C2_OPS:
        pair = marks.get(name) if ev is not None else None
        if pair:
            ev.record(pair[0])
        for s in sets:
            fn(cm, s)
        if pair:
            ev.record(pair[1])


# ---------------------------------------------------------------- secondary workloads

class RBM(object):
    """CD-1 step, 784 visible x 500 hidden, batch 100 (seed 1): dot -> sigmoid ->
    sample_bernoulli -> dot -> sigmoid -> dot -> sigmoid -> add_dot updates."""

    def __init__(self, cm, nv=784, nh=500, B=100, lr=0.01, seed=1):
        rng = np.random.default_rng(seed)
        self.cm, self.B, self.lr = cm, B, lr
        self.v = cm.CUDAMatrix(np.asarray(rng.random((nv, B)) < 0.13, dtype=np.float32, order='F'))
        self.W = cm.CUDAMatrix(np.asarray(0.01 * rng.standard_normal((nv, nh)), dtype=np.float32, order='F'))
        self.bv = cm.CUDAMatrix(np.zeros((nv, 1), dtype=np.float32))
        self.bh = cm.CUDAMatrix(np.zeros((nh, 1), dtype=np.float32))
        self.h, self.hs, self.h2 = cm.empty((nh, B)), cm.empty((nh, B)), cm.empty((nh, B))
        self.v2 = cm.empty((nv, B))
        self.flops = 5 * 2 * nv * nh * B

    def step_fused(self):
        """The same step through this backend's extensions: dot_bias_act with the hidden sample
        drawn by the product's own launch (states and samples bit-identical to step()) and the
        weight and bias statistics as one product (cd_update: equal to step() to rounding).
        4 launches instead of 16."""
        cm, eps = self.cm, self.lr / self.B
        W, v, h, hs, v2, h2 = self.W, self.v, self.h, self.hs, self.v2, self.h2
        cm.dot_bias_act(W.T, v, self.bh, target=h, act='sigmoid', sample=hs)
        cm.dot_bias_act(W, hs, self.bv, target=v2, act='sigmoid')
        cm.dot_bias_act(W.T, v2, self.bh, target=h2, act='sigmoid')
        cm.cd_update(W, self.bv, self.bh, v, h, v2, h2, eps)

    def step(self):
        cm, eps = self.cm, self.lr / self.B
        W, v, h, hs, v2, h2 = self.W, self.v, self.h, self.hs, self.v2, self.h2
        cm.dot(W.T, v, target=h); h.add_col_vec(self.bh); h.apply_sigmoid()
        h.sample_bernoulli(target=hs)
        cm.dot(W, hs, target=v2); v2.add_col_vec(self.bv); v2.apply_sigmoid()
        cm.dot(W.T, v2, target=h2); h2.add_col_vec(self.bh); h2.apply_sigmoid()
        W.add_dot(v, h.T, mult=eps); W.add_dot(v2, h2.T, mult=-eps)
        self.bv.add_sums(v, axis=1, mult=eps); self.bv.add_sums(v2, axis=1, mult=-eps)
        self.bh.add_sums(h, axis=1, mult=eps); self.bh.add_sums(h2, axis=1, mult=-eps)


class RBMExample(object):
    """The loop body of cudamat/examples/rbm_cudamat.py:46-89, call for call (28 library calls per
    minibatch: momentum on the three update buffers, positive phase with its statistics, the hidden sample
    spelled fill_with_rand -> less_than, negative phase with its statistics, three parameter updates and the
    reconstruction error, which the script reads back every step), on synthetic binary data."""

    def __init__(self, cm, num_vis=784, num_hid=500, batch_size=100, num_batches=20, seed=1):
        rng = np.random.default_rng(seed)
        f = lambda a: cm.CUDAMatrix(np.asarray(a, dtype=np.float32, order='F'))
        self.cm, self.bs, self.nb, self.nv = cm, batch_size, num_batches, num_vis
        self.epsilon, self.momentum = 0.1, 0.9
        self.dev_dat = f(rng.random((num_vis, batch_size * num_batches)) < 0.13)
        self.w_vh, self.w_v, self.w_h = f(0.1 * rng.standard_normal((num_vis, num_hid))), f(np.zeros((num_vis, 1))), \
            f(-4. * np.ones((num_hid, 1)))
        self.wu_vh, self.wu_v, self.wu_h = f(np.zeros((num_vis, num_hid))), f(np.zeros((num_vis, 1))), f(np.zeros((num_hid, 1)))
        self.v, self.h, self.r = cm.empty((num_vis, batch_size)), cm.empty((num_hid, batch_size)), cm.empty((num_hid, batch_size))
        self.batch = 0

    def step(self):
        cm, bs = self.cm, self.bs
        w_vh, w_v, w_h, wu_vh, wu_v, wu_h, v, h, r = (self.w_vh, self.w_v, self.w_h, self.wu_vh, self.wu_v, self.wu_h,
                                                      self.v, self.h, self.r)
        batch = self.batch
        self.batch = (batch + 1) % self.nb
        v_true = self.dev_dat.slice(batch * bs, (batch + 1) * bs)
        v.assign(v_true)
        wu_vh.mult(self.momentum); wu_v.mult(self.momentum); wu_h.mult(self.momentum)
        cm.dot(w_vh.T, v, target=h); h.add_col_vec(w_h); h.apply_sigmoid()
        wu_vh.add_dot(v, h.T); wu_v.add_sums(v, axis=1); wu_h.add_sums(h, axis=1)
        r.fill_with_rand(); r.less_than(h, target=h)
        cm.dot(w_vh, h, target=v); v.add_col_vec(w_v); v.apply_sigmoid()
        cm.dot(w_vh.T, v, target=h); h.add_col_vec(w_h); h.apply_sigmoid()
        wu_vh.subtract_dot(v, h.T); wu_v.add_sums(v, axis=1, mult=-1.); wu_h.add_sums(h, axis=1, mult=-1.)
        w_vh.add_mult(wu_vh, self.epsilon / bs); w_v.add_mult(wu_v, self.epsilon / bs); w_h.add_mult(wu_h, self.epsilon / bs)
        v.subtract(v_true)
        return v.euclid_norm() ** 2 / (self.nv * bs)


class MLP(object):
    """784-1024-1024-10 ReLU net, softmax cross-entropy, dropout 0.5 on the hidden
    layers (fill_with_rand -> greater_than -> mult), momentum SGD; batch 128, seed 3.
    Op sequence of deepnet/neuralnet.py:138-291 and parameter.py:80-106."""

    def __init__(self, cm, sizes=(784, 1024, 1024, 10), B=128, lr=0.01, mom=0.9, seed=3):
        rng = np.random.default_rng(seed)
        self.cm, self.B, self.lr, self.mom, self.sizes = cm, B, lr, mom, sizes
        f = lambda a: cm.CUDAMatrix(np.asarray(a, dtype=np.float32, order='F'))
        self.x = f(rng.random((sizes[0], B)))
        self.labels = f(rng.integers(0, sizes[-1], (1, B)))
        self.W = [f(0.01 * rng.standard_normal((sizes[i], sizes[i + 1]))) for i in range(3)]
        self.b = [f(np.zeros((sizes[i + 1], 1))) for i in range(3)]
        self.dW = [f(np.zeros((sizes[i], sizes[i + 1]))) for i in range(3)]
        self.db = [f(np.zeros((sizes[i + 1], 1))) for i in range(3)]
        # gradients accumulate and Update() leaves them at zero (neuralnet.py:269, 284, parameter.py:105)
        self.gW = [f(np.zeros((sizes[i], sizes[i + 1]))) for i in range(3)]
        self.gb = [f(np.zeros((sizes[i + 1], 1))) for i in range(3)]
        self.act = [self.x] + [cm.empty((sizes[i + 1], B)) for i in range(3)]
        self.mask = [cm.empty((sizes[i + 1], B)) for i in range(2)]
        self.delta = [cm.empty((sizes[i + 1], B)) for i in range(3)]
        self.loss = cm.empty((1, B))
        self.updates = None
        self.flops = 3 * 2 * B * (sizes[0] * sizes[1] + sizes[1] * sizes[2] + sizes[2] * sizes[3])

    def step(self):
        cm, B = self.cm, self.B
        act, W, b = self.act, self.W, self.b
        for i in range(3):
            cm.dot(W[i].T, act[i], target=act[i + 1])
            act[i + 1].add_col_vec(b[i])
            if i < 2:
                act[i + 1].lower_bound(0)
                self.mask[i].fill_with_rand(); self.mask[i].greater_than(0.5); act[i + 1].mult(self.mask[i])
            else:
                act[i + 1].apply_softmax()
        act[3].get_softmax_cross_entropy(self.labels, self.loss)
        act[3].apply_softmax_grad(self.labels, target=self.delta[2])
        for i in (2, 1, 0):
            self.gW[i].add_dot(act[i], self.delta[i].T, mult=1.0 / B)
            self.gb[i].add_sums(self.delta[i], axis=1, mult=1.0 / B)
            if i > 0:
                cm.dot(W[i], self.delta[i], target=self.delta[i - 1])
                self.delta[i - 1].mult(self.mask[i - 1])                      # the layer's dropout mask (neuralnet.py:212-213)
                self.delta[i - 1].apply_rectified_linear_deriv(act[i])
        for i in range(3):
            for p, d, g in ((W[i], self.dW[i], self.gW[i]), (b[i], self.db[i], self.gb[i])):
                d.mult(self.mom); d.add_mult(g); p.add_mult(d, -self.lr); g.assign(0)

    def step_fused(self):
        """The same step in 17 launches instead of 53 calls: this backend's extensions dot_bias_act,
        softmax_ce_grad and momentum_update (all six parameters in one launch), and the one-call forms that the reference's own
        API has for what deepnet spells out in several (dropout() for fill_with_rand ->
        greater_than -> mult, dot() into the gradient for assign(0) -> add_dot, dot() with a
        column of ones for assign(0) -> add_sums).  Every parameter, momentum buffer and loss
        gets the same bits as in step(); the dropout masks are not materialised."""
        cm, B = self.cm, self.B
        act, W, b = self.act, self.W, self.b
        if not hasattr(self, 'ones'):
            self.ones = cm.CUDAMatrix(np.ones((B, 1), dtype=np.float32))
        for i in range(3):
            if i < 2:
                cm.dot_bias_act(W[i].T, act[i], b[i], target=act[i + 1], act='relu')
                act[i + 1].dropout(0.5)
            else:
                cm.dot_bias_act(W[i].T, act[i], b[i], target=act[i + 1], act=None)
        cm.softmax_ce_grad(act[3], self.labels, loss=self.loss, grad=self.delta[2])
        for i in (2, 1, 0):
            cm.dot(act[i], self.delta[i].T, mult=1.0 / B, target=self.gW[i])
            cm.dot(self.delta[i], self.ones, mult=1.0 / B, target=self.gb[i])
            if i > 0:
                cm.dot(W[i], self.delta[i], target=self.delta[i - 1])
                self.delta[i - 1].apply_rectified_linear_deriv(act[i])
        if self.updates is None:
            self.updates = cm.MomentumUpdates([(W[i], self.dW[i], self.gW[i]) for i in range(3)] +
                                              [(b[i], self.db[i], self.gb[i]) for i in range(3)])
        self.updates.apply(self.mom, self.lr, reset_gradient=True)


def net_mlp(cm, sizes=(784, 1024, 1024, 10), B=128, seed=3, fused=False):
    """The MLP of config 3 as a deepnet net: Layer / Edge / NeuralNet objects of this package
    driven by TrainOneBatch, i.e. the reference's own control flow (neuralnet.py:138-337) with
    its per-step loss read-backs (two blocking sums per step in SoftmaxLayer.GetLoss)."""
    from deepnet_amd import layer as dl, neuralnet as dnn, parameter as dp
    rng = np.random.default_rng(seed)
    sgd = dict(base_epsilon=0.01, initial_momentum=0.9, final_momentum=0.9)
    layers = [dl.LinearLayer('input', sizes[0], B, hyperparams=dp.Hyperparams(), is_input=True)]
    for i in (1, 2):
        layers.append(dl.ReluLayer('hidden%d' % i, sizes[i], B,
                                   hyperparams=dp.Hyperparams(activation=dp.RECTIFIED_LINEAR, dropout=True, **sgd)))
    layers.append(dl.SoftmaxLayer('output', 1, B, hyperparams=dp.Hyperparams(activation=dp.SOFTMAX, **sgd),
                                  numlabels=sizes[3], is_output=True, loss_function=dp.CROSS_ENTROPY))
    edges = [dnn.Edge(layers[i], layers[i + 1], 0.01 * rng.standard_normal((sizes[i], sizes[i + 1])),
                      hyperparams=dp.Hyperparams(**sgd)) for i in range(3)]
    for obj in layers + edges:
        obj.fused = fused
    net = dnn.NeuralNet(layers, edges)
    layers[0].data.assign(cm.CUDAMatrix(np.asarray(rng.random((sizes[0], B)), dtype=np.float32, order='F')))
    layers[-1].data.assign(cm.CUDAMatrix(np.asarray(rng.integers(0, sizes[3], (1, B)), dtype=np.float32, order='F')))
    return net


def net_example_convnet(cm, B=100, seed=12):
    """The model of deepnet/examples/convnet (model_conv.pbtxt, batch 100 as in train.pbtxt):
    28 x 28 inputs -> conv 5 x 5 (64 filters) + pool 3/2 -> conv 5 x 5 (64 -> 64) + pool 3/2 -> 1024 ReLU
    -> softmax(10), as Layer / Edge / NeuralNet objects."""
    from deepnet_amd import layer as dl, neuralnet as dnn, parameter as dp, convolutions as dc
    rng = np.random.default_rng(seed)
    net_h = dict(base_epsilon=0.01, initial_momentum=0.5, final_momentum=0.9, momentum_change_steps=10000)
    conv_h = dict(base_epsilon=0.001, initial_momentum=0.9, final_momentum=0.9, momentum_change_steps=20000)
    hyp = lambda act, **kw: dp.Hyperparams(activation=act, **kw)
    L = [dl.LinearLayer('input_layer', 784, B, hyperparams=hyp(dp.LINEAR), is_input=True),
         dl.ReluLayer('hidden1', 10816, B, hyperparams=hyp(dp.RECTIFIED_LINEAR, **net_h)),
         dl.ReluLayer('hidden2', 2304, B, hyperparams=hyp(dp.RECTIFIED_LINEAR, **net_h)),
         dl.ReluLayer('hidden3', 1024, B, hyperparams=hyp(dp.RECTIFIED_LINEAR, **net_h)),
         dl.SoftmaxLayer('output_layer', 1, B, hyperparams=hyp(dp.SOFTMAX, **net_h), numlabels=10, is_output=True,
                         loss_function=dp.CROSS_ENTROPY)]
    cv = lambda colors: dc.ConvParams(size=5, stride=1, padding=2, num_filters=64, num_colors=colors, max_pool=True,
                                      pool_size=3, pool_stride=2)
    dense = dp.Hyperparams(apply_l2_decay=True, l2_decay=0.001, **net_h)
    E = [dnn.Edge(L[0], L[1], 0.1 * rng.standard_normal((64, 25)), hyperparams=dp.Hyperparams(**conv_h), conv_params=cv(1)),
         dnn.Edge(L[1], L[2], 0.02 * rng.standard_normal((64, 1600)), hyperparams=dp.Hyperparams(**conv_h), conv_params=cv(64)),
         dnn.Edge(L[2], L[3], 0.02 * rng.standard_normal((2304, 1024)), hyperparams=dense),
         dnn.Edge(L[3], L[4], 0.05 * rng.standard_normal((1024, 10)), hyperparams=dense)]
    L[0].data.assign(cm.CUDAMatrix(np.asarray(rng.random((784, B)), dtype=np.float32, order='F')))
    L[-1].data.assign(cm.CUDAMatrix(np.asarray(rng.integers(0, 10, (1, B)), dtype=np.float32, order='F')))
    return dnn.NeuralNet(L, E)


def time_loop(cm, fn, iters, warmup):
    for _ in range(warmup):
        fn()
    cm.cuda_sync_threads()
    t0 = time.perf_counter()
    for _ in range(iters):
        fn()
    cm.cuda_sync_threads()
    return (time.perf_counter() - t0) / iters


def gemm_probe(cm, ev, n=4096, iters=10, warm_s=0.03):
    rng = np.random.default_rng(6)
    a = cm.CUDAMatrix(np.asarray(rng.uniform(-1, 1, (n, n)), dtype=np.float32, order='F'))
    b = cm.CUDAMatrix(np.asarray(rng.uniform(-1, 1, (n, n)), dtype=np.float32, order='F'))
    c = cm.empty((n, n))
    out = {}
    for label, x, y in (('nn', a, b), ('tn', a.T, b), ('nt', a, b.T)):
        # untimed warm-up: the core clock under matrix-core load needs a few tens of ms to
        # settle (the first variant timed cold reads 10 % low)
        t0 = time.perf_counter()
        while (time.perf_counter() - t0) < warm_s:
            for _ in range(4):
                cm.dot(x, y, target=c)
            cm.cuda_sync_threads()
        e0, e1 = ev.new(), ev.new()
        ev.record(e0)
        for _ in range(iters):
            cm.dot(x, y, target=c)
        ev.record(e1)
        ms = ev.elapsed_ms(e0, e1) / iters
        tf = 2.0 * n ** 3 / (ms * 1e-3) / 1e12
        out[label] = {'ms': round(ms, 4), 'tflops': round(tf, 2), 'frac_mfma_fp32': round(tf / MFMA_FP32_PEAK_TFLOPS, 4)}
    for m in (a, b, c):
        m.free_device_memory()
    return out


def gemm_layer_shapes(cm, ev, iters=200):
    """The products of the RBM (config 1) and MLP (config 3) steps, one shape at a time: HIP
    events around `iters` back-to-back launches (an empty kernel takes 2.4 us that way)."""
    rng = np.random.default_rng(7)
    f = lambda *s: cm.CUDAMatrix(np.asarray(rng.standard_normal(s), dtype=np.float32, order='F'))
    out = {}

    def timed(label, fn, flops):
        for _ in range(20):
            fn()
        e0, e1 = ev.new(), ev.new()
        ev.record(e0)
        for _ in range(iters):
            fn()
        ev.record(e1)
        us = ev.elapsed_ms(e0, e1) / iters * 1e3
        tf = flops / (us * 1e-6) / 1e12
        out[label] = {'us': round(us, 2), 'tflops': round(tf, 2), 'frac_mfma_fp32': round(tf / MFMA_FP32_PEAK_TFLOPS, 4)}
    nv, nh, B = 784, 500, 100
    W, v, h, v2 = f(nv, nh), f(nv, B), f(nh, B), cm.empty((nv, B))
    hh = cm.empty((nh, B))
    timed('rbm_up_500x100x784', lambda: cm.dot(W.T, v, target=hh), 2.0 * nv * nh * B)
    timed('rbm_down_784x100x500', lambda: cm.dot(W, h, target=v2), 2.0 * nv * nh * B)
    timed('rbm_stats_784x500x100', lambda: W.add_dot(v, h.T, mult=1e-6), 2.0 * nv * nh * B)
    for m in (W, v, h, v2, hh):
        m.free_device_memory()
    for a, b in ((784, 1024), (1024, 1024), (1024, 10)):
        Wm, x, y, d = f(a, b), f(a, 128), cm.empty((b, 128)), f(b, 128)
        xb, g = cm.empty((a, 128)), cm.empty((a, b))
        timed('mlp_fwd_%dx128x%d' % (b, a), lambda: cm.dot(Wm.T, x, target=y), 2.0 * a * b * 128)
        timed('mlp_bwd_%dx128x%d' % (a, b), lambda: cm.dot(Wm, d, target=xb), 2.0 * a * b * 128)
        timed('mlp_grad_%dx%dx128' % (a, b), lambda: g.add_dot(x, d.T, mult=0.01), 2.0 * a * b * 128)
        for m in (Wm, x, y, d, xb, g):
            m.free_device_memory()
    return out


# ---------------------------------------------------------------- CPU baseline

def cpu_baseline_c2():
    """The same op list through the C host restatement, single thread, one pass over
    ONE operand set (4096^2) per op; RNG through the host MWC."""
    from oracle import mwc
    lib = ct.CDLL(os.path.join(ROOT, 'oracle', 'liboracle_host.so'))
    fp = ct.POINTER(ct.c_float)
    rng = np.random.default_rng(2)
    A = np.asarray(rng.uniform(-1, 1, (N, N)), dtype=np.float32, order='F')
    B = np.asarray(rng.uniform(-1, 1, (N, N)), dtype=np.float32, order='F')
    P = np.asarray(rng.random((N, N)), dtype=np.float32, order='F')
    T = np.empty((N, N), dtype=np.float32, order='F')
    col = np.asarray(rng.uniform(-1, 1, N), dtype=np.float32)
    r = np.empty(N, dtype=np.float32)
    mults = mwc.load_multipliers(os.path.join(ROOT, 'deepnet_amd', 'rnd_multipliers_32bit.txt'))
    words = np.empty(mwc.NUM_RND_STREAMS, dtype=np.uint64)
    p = lambda a: a.ctypes.data_as(fp)
    u32 = mults.ctypes.data_as(ct.POINTER(ct.c_uint32))
    u64 = words.ctypes.data_as(ct.POINTER(ct.c_uint64))
    lib.mwc_seed(u32, u64, ct.c_uint32(2))
    sz = ct.c_size_t(E)
    lib.hb_set_threads(1)
    ops = [
        ('add_mult', lambda: lib.hb_add_mult(p(A), p(B), ct.c_float(0.5), sz)),
        ('mult', lambda: lib.hb_mult(p(A), p(B), p(T), sz)),
        ('apply_sigmoid', lambda: lib.hb_sigmoid(p(A), p(T), sz)),
        ('apply_exp', lambda: lib.hb_exp(p(A), p(T), sz)),
        ('mult_by_col', lambda: lib.hb_mult_by_col(p(A), p(col), p(T), N, N)),
        ('add_row_vec', lambda: lib.hb_add_row_vec(p(A), p(col), p(T), N, N)),
        ('sum_axis0', lambda: lib.hb_add_sums(p(A), p(r), N, N, 0, ct.c_float(0), ct.c_float(1))),
        ('sum_axis1', lambda: lib.hb_add_sums(p(A), p(r), N, N, 1, ct.c_float(0), ct.c_float(1))),
        ('max_axis0', lambda: lib.hb_max(p(A), p(r), N, N, 0)),
        ('max_axis1', lambda: lib.hb_max(p(A), p(r), N, N, 1)),
        ('softmax', lambda: lib.hb_softmax(p(A), p(T), N, N)),
        ('fill_with_rand', lambda: lib.mwc_uniform(u32, u64, p(T), sz)),
        ('sample_bernoulli', lambda: lib.mwc_bernoulli(u32, u64, p(P), p(T), sz)),
    ]
    assert [o[0] for o in ops] == [o[0] for o in C2_OPS]
    for _, fn in ops:      # touch everything once
        fn()
    PASSES = 12                      # about 7 s of single-thread work
    t0 = time.perf_counter()
    per_op = {name: 0.0 for name, _ in ops}
    for _ in range(PASSES):
        for name, fn in ops:
            t1 = time.perf_counter()
            fn()
            per_op[name] += time.perf_counter() - t1
    total = (time.perf_counter() - t0) / PASSES
    per_op = {k: v / PASSES for k, v in per_op.items()}
    nbytes = sum(b for _, b, _ in C2_OPS)
    return {'value': round(nbytes / total / 1e9, 3), 'unit': 'GB/s', 'cores': 1, 'kind': 'port',
            'sample': '%d passes of the 13-op list over one 4096x4096 operand set (each pass = 1/%d of a GPU step), '
                      'oracle/host_backend.c, gcc -O3 x86-64-v3, 1 thread; host has %d cpus' % (PASSES, NSETS, os.cpu_count()),
            'seconds': round(total * PASSES, 3),
            'per_op_gbs': {n: round(b / per_op[n] / 1e9, 2) for n, b, _ in C2_OPS}}


def cpu_baseline_rbm(steps=100):
    from oracle import mwc
    lib = ct.CDLL(os.path.join(ROOT, 'oracle', 'liboracle_host.so'))
    fp = ct.POINTER(ct.c_float)
    nv, nh, B = 784, 500, 100
    rng = np.random.default_rng(1)
    v = np.asarray(rng.random((nv, B)) < 0.13, dtype=np.float32, order='F')
    W = np.asarray(0.01 * rng.standard_normal((nv, nh)), dtype=np.float32, order='F')
    bv, bh = np.zeros(nv, np.float32), np.zeros(nh, np.float32)
    h, hs, h2 = (np.empty((nh, B), np.float32, order='F') for _ in range(3))
    v2 = np.empty((nv, B), np.float32, order='F')
    mults = mwc.load_multipliers(os.path.join(ROOT, 'deepnet_amd', 'rnd_multipliers_32bit.txt'))
    words = np.empty(mwc.NUM_RND_STREAMS, dtype=np.uint64)
    u32 = mults.ctypes.data_as(ct.POINTER(ct.c_uint32))
    u64 = words.ctypes.data_as(ct.POINTER(ct.c_uint64))
    lib.mwc_seed(u32, u64, ct.c_uint32(1))
    p = lambda a: a.ctypes.data_as(fp)
    out = {}
    for threads in (1, os.cpu_count() or 1):
        lib.hb_set_threads(threads)
        call = lambda: lib.hb_rbm_cd1_step(p(W), p(bv), p(bh), p(v), nv, nh, B, ct.c_float(0.01), u32, u64,
                                           p(h), p(hs), p(v2), p(h2))
        call()
        t0 = time.perf_counter()
        for _ in range(steps):
            call()
        out[threads] = steps / (time.perf_counter() - t0)
    lib.hb_set_threads(1)
    return out


def cpu_baseline_mlp(steps=8):
    """The MLP step of config 3 (784-1024-1024-10, batch 128) through oracle/host_backend.c
    (hb_mlp_step: the same op sequence as MLP.step), on 1 thread and on all host threads."""
    from oracle import host_steps
    lib = host_steps.load()
    rng = np.random.default_rng(3)
    sizes, B = (784, 1024, 1024, 10), 128
    x = rng.random((sizes[0], B))
    labels = rng.integers(0, sizes[-1], (1, B))
    W = [0.01 * rng.standard_normal((sizes[i], sizes[i + 1])) for i in range(3)]
    b = [np.zeros(sizes[i + 1]) for i in range(3)]
    m = host_steps.HostMLP(lib, sizes, B, x, labels, W, b, 0.01, 0.9, seed=3)
    out = {}
    for threads in (1, os.cpu_count() or 1):
        lib.hb_set_threads(threads)
        m.step()
        t0 = time.perf_counter()
        for _ in range(steps):
            m.step()
        out[threads] = steps / (time.perf_counter() - t0)
    lib.hb_set_threads(1)
    return out


def cpu_baseline_conv():
    """The conv passes through the float64 numpy restatement (patch views + tensordot; numpy's
    own threading): the reference's CPU library has no convolution, so this is the only CPU
    figure there is to put beside the conv kernels.  Config 4 runs whole (one pass each);
    configs 5a / 5b take minutes per pass at batch 128, so they run on a sample of 8 of the 128
    images (same layer geometry, 1/16 of the work) and the time is reported for that sample."""
    from oracle import conv_oracle as co
    rng = np.random.default_rng(4)
    out = {}
    for name, (N, C, H, F, k, s, p, G) in (('c4', (128, 3, 32, 64, 5, 1, 2, 1)), ('c5a_8_of_128_images', (8, 3, 224, 96, 11, 4, 0, 1)),
                                           ('c5b_8_of_128_images', (8, 96, 27, 256, 5, 1, 2, 2))):
        Mx = (H + 2 * p - k) // s + 1
        x = rng.standard_normal((N, C * H * H)).astype(np.float32)
        w = (0.01 * rng.standard_normal((F, (C // G) * k * k))).astype(np.float32)
        y = rng.standard_normal((N, F * Mx * Mx)).astype(np.float32)
        res = {}
        for label, fn in (('convUp', lambda: co.conv_up(x, w, C, Mx, p, s, G)), ('convDown', lambda: co.conv_down(y, w, C, H, p, s, G)),
                          ('convOutp', lambda: co.conv_outp(x, y, C, Mx, k, p, s, G))):
            t0 = time.perf_counter()
            fn()
            res[label] = round((time.perf_counter() - t0) * 1e3, 1)
        out[name] = res
    return out


# ---------------------------------------------------------------- main

def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=10)
    ap.add_argument('--warmup', type=int, default=2)
    ap.add_argument('--no-cpu', action='store_true', help='skip the CPU baseline leg')
    ap.add_argument('--only-c2', action='store_true', help='skip the secondary workloads')
    ap.add_argument('--probe-mfma', action='store_true',
                    help='launch only the 4096^3 products and the conv layers a few times (for rocprofv3 --pmc runs)')
    ap.add_argument('--probe', action='store_true',
                    help='run only the roofline kernel (add_mult) and a copy-shaped calibration kernel '
                         '(mult by a scalar into a second matrix), for rocprofv3 --pmc runs')
    ap.add_argument('--no-graph', action='store_true',
                    help='skip the recorded-graph timings (rocprofv3 --kernel-trace crashes inside hipGraphLaunch)')
    ap.add_argument('--probe-c2', action='store_true',
                    help='launch every op of the 4096^2 list three times over the 8 operand sets, plus the copy-shaped '
                         'calibration kernel, and nothing else (for rocprofv3 --pmc runs)')
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this backend has no multi-GPU path (run with --gpus 1).")

    from deepnet_amd import cudamat as cm
    cm.cublas_init()
    cm.CUDAMatrix.init_random(2)
    ev = HipEvents(cm.launch_deferred)

    if args.probe_mfma:
        # the matrix-core kernels only, a few launches each and no clock warm-up: for counter runs
        import bench_conv
        bench_conv.WARM_MS = 0.0
        out = {'gemm_fp32_4096': gemm_probe(cm, ev, iters=3, warm_s=0.0)}
        out.update(bench_conv.run(cm, ev, iters=3))
        print(json.dumps({'probe_mfma': out}))
        return

    if args.probe:
        sets = build_c2(cm)
        for _ in range(3):
            for s in sets:
                s['A'].add_mult(s['B'], 0.5)          # k_ew<2, true, FAxpy>: reads 2 x 64 MiB, writes 64 MiB
            for s in sets:
                s['A'].mult(1.0, target=s['T'])       # k_ew<1, true, FMulS>: reads 64 MiB, writes 64 MiB
        cm.cuda_sync_threads()
        print(json.dumps({'probe': 'done', 'elements': E}))
        return

    if args.probe_c2:
        sets = build_c2(cm)
        for _ in range(3):
            for s in sets:
                s['A'].mult(1.0, target=s['T'])       # k_ew<1, true, FMulS>: reads 64 MiB, writes 64 MiB
            run_c2_step(cm, sets)
        cm.cuda_sync_threads()
        print(json.dumps({'probe_c2': 'done', 'elements': E, 'ops': [n for n, _, _ in C2_OPS]}))
        return

    sets = build_c2(cm)
    roof_op = 'add_mult'
    for _ in range(args.warmup):
        run_c2_step(cm, sets)
    # The timed steps: nothing waits inside them; the launches of the roofline's kernel have their own pair
    # of events in every step, read back after the last one.
    roof_marks = [{roof_op: (ev.new(), ev.new())} for _ in range(args.steps)]
    cm.cuda_sync_threads()
    t0 = time.perf_counter()
    for k in range(args.steps):
        run_c2_step(cm, sets, ev, roof_marks[k])
    cm.cuda_sync_threads()
    step_s = (time.perf_counter() - t0) / args.steps
    roof_ms = float(np.mean([ev.elapsed_ms(*m[roof_op]) / NSETS for m in roof_marks]))
    # The per-op figures: the same steps once more with events around every op, read back after each step.
    marks = {name: (ev.new(), ev.new()) for name, _, _ in C2_OPS}
    per_op_ms = {name: [] for name, _, _ in C2_OPS}
    for _ in range(args.steps):
        run_c2_step(cm, sets, ev, marks)
        for name, _, _ in C2_OPS:
            per_op_ms[name].append(ev.elapsed_ms(*marks[name]) / NSETS)
    cm.cuda_sync_threads()

    ops = {}
    for name, nbytes, _ in C2_OPS:
        ms = float(np.median(per_op_ms[name]))
        gbs = nbytes / (ms * 1e-3) / 1e9
        ops[name] = {'us': round(ms * 1e3, 2), 'gbs': round(gbs, 1), 'frac_hbm': round(gbs / HBM_PEAK_GBS, 4)}
    value = STEP_BYTES / step_s / 1e9

    traffic = None
    try:    # HBM bytes per launch from the committed rocprofv3 --pmc summary (FETCH_SIZE + WRITE_SIZE, calibrated)
        for ln in open(os.path.join(ROOT, 'profiles', 'k_ew_axpy_hbm_traffic.md')):
            if ln.startswith('traffic_bytes_per_launch:'):
                traffic = int(ln.split(':')[1])
    except OSError:
        pass
    roof_gbs = round(12 * E / (roof_ms * 1e-3) / 1e9, 1)
    roofline = {'kernel': 'k_ew<2, true, FAxpy> (add_mult, 4096x4096)', 'bound': 'hbm',
                'achieved': roof_gbs, 'peak': HBM_PEAK_GBS, 'unit': 'GB/s',
                'frac': round(roof_gbs / HBM_PEAK_GBS, 4), 'traffic': traffic,
                'traffic_source': 'profiles/k_ew_axpy_hbm_traffic.md (an earlier rocprofv3 --pmc run of bench.py --probe, '
                                  'not measured by this run)',
                'algorithmic_bytes_per_launch': 12 * E, 'avg_launch_us': round(roof_ms * 1e3, 2)}

    secondary = {}
    if not args.only_c2:
        for s in sets:
            for m in s.values():
                m.free_device_memory()
        cm.CUDAMatrix.init_random(1)
        rbm = RBM(cm)
        t = time_loop(cm, rbm.step, 200, 20)
        secondary['rbm_cd1'] = {'steps_per_sec': round(1.0 / t, 1), 'us_per_step': round(t * 1e6, 1),
                                'gemm_tflops': round(rbm.flops / t / 1e12, 3),
                                'config': '784 visible x 500 hidden, batch 100, fp32',
                                'note': 'the 16 calls of the reference API (cudamat/examples/rbm_cudamat.py:46-89); the library '
                                        'folds add_col_vec / apply_sigmoid / sample_bernoulli into the launch of the dot() they '
                                        'follow, and the two add_dot and four add_sums calls of the statistics into one launch '
                                        '(deferred epilogues, same bits): 4 launches',
                                'iters': 200, 'warmup': 20}
        cm.set_deferred_epilogues(False)
        t = time_loop(cm, rbm.step, 200, 20)
        cm.set_deferred_epilogues(True)
        secondary['rbm_cd1']['us_per_step_every_call_a_launch'] = round(t * 1e6, 1)
        t = time_loop(cm, rbm.step_fused, 200, 20)
        secondary['rbm_cd1_fused_extension'] = {
            'steps_per_sec': round(1.0 / t, 1), 'us_per_step': round(t * 1e6, 1),
            'note': 'same step with dot_bias_act, its sample, and the weight / bias statistics as one product (cd_update): extensions of this backend, not in the reference API; 4 launches instead of 16'}
        ex = RBMExample(cm)
        t = time_loop(cm, ex.step, 200, 20)
        secondary['rbm_example_script'] = {
            'steps_per_sec': round(1.0 / t, 1), 'us_per_step': round(t * 1e6, 1),
            'note': 'the loop body of cudamat/examples/rbm_cudamat.py:46-89 call for call (28 calls, the reconstruction error read '
                    'back every step as the script does): 15 launches'}
        cm.set_deferred_epilogues(False)
        t = time_loop(cm, ex.step, 200, 20)
        cm.set_deferred_epilogues(True)
        secondary['rbm_example_script']['us_per_step_every_call_a_launch'] = round(t * 1e6, 1)
        def recorded(step, iters, warm):
            # the step recorded once as a HIP graph (cm.Graph, an extension of this backend) and
            # replayed with one launch per step: same kernels, same results
            if args.no_graph:
                return None
            with cm.Graph() as g:
                step()
            tt = time_loop(cm, g.launch, iters, warm)
            g.free()
            return round(tt * 1e6, 1)
        secondary['rbm_cd1']['us_per_step_recorded_graph'] = recorded(rbm.step, 200, 20)
        secondary['rbm_cd1_fused_extension']['us_per_step_recorded_graph'] = recorded(rbm.step_fused, 200, 20)
        cm.CUDAMatrix.init_random(3)
        mlp = MLP(cm)
        t = time_loop(cm, mlp.step, 100, 10)
        secondary['mlp_784_1024_1024_10'] = {'steps_per_sec': round(1.0 / t, 1), 'us_per_step': round(t * 1e6, 1),
                                              'gemm_tflops': round(mlp.flops / t / 1e12, 3), 'batch': 128,
                                              'note': 'the 53 calls of the reference API; the library folds bias / activation calls into the '
                                                      'launch of the dot() they follow, the mult / add_mult calls of each parameter update '
                                                      'into one pass and fill_with_rand / greater_than / mult of a dropout mask into one pass '
                                                      '(same bits; behind a layer of rectified linear units in the layer\'s own launch), consecutive updates wait for each other and share a launch, a weight gradient takes the '
                                                      'bias gradient that follows it along a backward product the apply_rectified_linear_deriv behind it, and the softmax its loss and gradient: 10 launches',
                                              'iters': 100, 'warmup': 10}
        cm.set_deferred_epilogues(False)
        t = time_loop(cm, mlp.step, 100, 10)
        cm.set_deferred_epilogues(True)
        secondary['mlp_784_1024_1024_10']['us_per_step_every_call_a_launch'] = round(t * 1e6, 1)
        t = time_loop(cm, mlp.step_fused, 100, 10)
        secondary['mlp_fused_extensions'] = {
            'steps_per_sec': round(1.0 / t, 1), 'us_per_step': round(t * 1e6, 1),
            'note': 'same step with dot_bias_act, softmax_ce_grad and the momentum update of all six parameters in one launch (extensions of this backend, not in the reference API) and the one-call forms dropout / dot into the gradient of the reference API: 17 launches instead of 53 calls, same bits in every parameter'}
        secondary['mlp_784_1024_1024_10']['us_per_step_recorded_graph'] = recorded(mlp.step, 100, 10)
        secondary['mlp_fused_extensions']['us_per_step_recorded_graph'] = recorded(mlp.step_fused, 100, 10)
        net = net_mlp(cm)
        t = time_loop(cm, lambda: net.TrainOneBatch(0), 100, 10)
        secondary['mlp_through_neuralnet_classes'] = {
            'steps_per_sec': round(1.0 / t, 1), 'us_per_step': round(t * 1e6, 1),
            'note': 'same net as Layer / Edge / NeuralNet objects, TrainOneBatch with its two blocking loss read-backs per step'}
        for obj in net.layer + net.edge:
            obj.fused = True
        t = time_loop(cm, lambda: net.TrainOneBatch(0), 100, 10)
        secondary['mlp_through_neuralnet_classes']['us_per_step_fused_extensions'] = round(t * 1e6, 1)
        convnet = net_example_convnet(cm)
        t = time_loop(cm, lambda: convnet.TrainOneBatch(0), 50, 5)
        secondary['example_convnet_batch100'] = {
            'steps_per_sec': round(1.0 / t, 1), 'us_per_step': round(t * 1e6, 1),
            'note': 'deepnet/examples/convnet (two conv + pool stages, 1024 ReLU, softmax) at its batch size of 100: TrainOneBatch through the layer / edge classes'}
        for obj in convnet.layer + convnet.edge:
            obj.fused = True
        t = time_loop(cm, lambda: convnet.TrainOneBatch(0), 50, 5)
        secondary['example_convnet_batch100']['us_per_step_fused_extensions'] = round(t * 1e6, 1)
        secondary['gemm_fp32_4096'] = gemm_probe(cm, ev)
        secondary['gemm_layer_shapes'] = gemm_layer_shapes(cm, ev)
        try:
            import bench_conv
            secondary.update(bench_conv.run(cm, ev))
        except ImportError:
            pass

    line = {
        'metric': 'RBM CD-1 steps/sec; elementwise HBM GB/s; conv fp32 TFLOP/s vs roofline',
        'value': round(value, 1), 'unit': 'GB/s (elementwise/reduction/RNG microbench, algorithmic bytes)',
        'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup, 'ms_per_step': round(step_s * 1e3, 3),
        'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None, 'dtype': 'f32', 'data': 'synthetic',
        'config': {'workload': 'elementwise+reduction+RNG microbench, 4096x4096 fp32 column-major, 13 ops x %d '
                               'operand sets per step' % NSETS, 'step_bytes': STEP_BYTES},
        'roofline': roofline, 'ops': ops, 'secondary': secondary,
        'timing': {'value': 'wall time of the K = %d steps between two device synchronisations, after %d warm-up steps, one run'
                            % (args.steps, args.warmup),
                   'roofline': 'HIP events on the NULL stream around the %d add_mult launches of every timed step, read back after the '
                               'last step; mean over the K steps' % NSETS,
                   'ops': 'the K steps once more, outside the timed region, with HIP events around the %d launches of every op, '
                          'read back after each step; median over the K steps' % NSETS,
                   'steps_per_sec': 'wall time of `iters` steps after `warmup` steps, device synchronised on both sides, one run',
                   'gemm_conv': 'HIP events around 10 (4096^3, conv: median of 3 such groups) or 200 (layer shapes) back-to-back '
                                'launches after 30 ms of matrix-core warm-up',
                   'note': 'shorter than 100 iterations x 5 repeats; figures move by 1-3 % between runs and up to 5 % (host-bound '
                           'step loops: 20 %) between boxes'},
    }
    if not args.no_cpu:
        cb = cpu_baseline_c2()
        if not args.only_c2:
            r = cpu_baseline_rbm()
            cb['rbm_cd1_steps_per_sec'] = {'threads_%d' % k: round(v, 2) for k, v in r.items()}
            # what the port's products reach: 5 products of 78.4 MFLOP per step (eigenmat itself calls Eigen's
            # blocked product, eigenmat/eigenmat.cc:1059-1086, which this image does not have; the port's is a
            # plain blocked loop), so the ratios below say how far the GPU step is from THIS code, no more
            cb['rbm_cd1_gemm_gflops'] = {'threads_%d' % k: round(5 * 2 * 784 * 500 * 100 * v / 1e9, 1) for k, v in r.items()}
            cb['rbm_cd1_gemm_note'] = ('step rate x 392 MFLOP of products per step; the port multiplies with a blocked triple '
                                       'loop, eigenmat with Eigen (not in this image), so a tuned CPU GEMM would be several times faster')
            if 'rbm_cd1' in secondary:
                secondary['rbm_cd1']['vs_cpu_1thread'] = round(secondary['rbm_cd1']['steps_per_sec'] / r[1], 1)
                secondary['rbm_cd1']['vs_cpu_%dthreads' % max(r)] = round(secondary['rbm_cd1']['steps_per_sec'] / r[max(r)], 1)
            r = cpu_baseline_mlp()
            cb['mlp_784_1024_1024_10_steps_per_sec'] = {'threads_%d' % k: round(v, 2) for k, v in r.items()}
            if 'mlp_784_1024_1024_10' in secondary:
                secondary['mlp_784_1024_1024_10']['vs_cpu_1thread'] = round(
                    secondary['mlp_784_1024_1024_10']['steps_per_sec'] / r[1], 1)
                secondary['mlp_784_1024_1024_10']['vs_cpu_%dthreads' % max(r)] = round(
                    secondary['mlp_784_1024_1024_10']['steps_per_sec'] / r[max(r)], 1)
            cb['conv_numpy_f64_ms'] = cpu_baseline_conv()
        line['cpu_baseline'] = cb
    print(json.dumps(line))


if __name__ == '__main__':
    main()
