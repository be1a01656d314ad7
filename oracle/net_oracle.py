"""TEST INFRASTRUCTURE ONLY - float64 restatement of one training step of a deepnet
feed-forward net: deepnet/neuralnet.py:138-337 (ComputeUp, ComputeDown, AccumulateDeriv,
UpdateEdgeParams, UpdateLayerParams, TrainOneBatch), the activation layers
(logistic_layer.py, tanh_layer.py, relu_layer.py, linear_layer.py, softmax_layer.py) and the
update rule deepnet/parameter.py:80-126.  Only tests/ may import this.

The net is a chain: layer 0 is the input, every later layer has one incoming edge (dense,
or a conv stage as in oracle/conv_oracle.py).  Dropout masks are passed in, so that a test can
feed the masks the device drew.

Pinned by tests/test_oracle_net.py: for nets without response normalisation the gradients are
torch.autograd's and k steps equal k steps of torch.optim.SGD(momentum, weight_decay) on the
same model (tanh units with the slope halved in the backward pass, as the reference's kernel
does); norm-limited updates equal an explicit column renormalisation; the momentum and
learning-rate schedules are checked against their closed forms at hand-picked steps.
"""
import numpy as np

from . import conv_oracle as co
from . import cudamat_oracle as cmo

F64 = np.float64


class Hyper(object):
    """Defaults of Hyperparams in deepnet/protos/deepnet.proto:89-175 (the fields the step reads)."""

    def __init__(self, **kw):
        self.base_epsilon, self.epsilon_decay, self.epsilon_decay_half_life = 0.01, 'NONE', 1000
        self.initial_momentum, self.final_momentum, self.momentum_change_steps = 0.0, 0.0, 10
        self.apply_l2_decay, self.l2_decay, self.apply_l1_decay, self.l1_decay = False, 0.01, False, 0.01
        self.apply_l1decay_after, self.apply_weight_norm, self.weight_norm = 0, False, 10.0
        self.start_learning_after = 0
        self.dropout, self.dropout_prob = False, 0.5
        self.sparsity, self.sparsity_target, self.sparsity_cost, self.sparsity_damping = False, 0.1, 0.001, 0.9
        self.__dict__.update(kw)


def sparsity_gradient(h, act, means, state):
    """layer.py:138-155 with the divisors of logistic_layer.py:64-68 (mean * (1 - mean)) and
    layer.py:256-258 (1, rectified linear units): the running means after seeing ``state`` and
    cost * (mean - target) / divisor.  For logistic units this is cost * d/d(mean) of the
    Kullback-Leibler divergence between Bernoulli(target) and Bernoulli(mean), which is what
    tests/test_oracle_net.py checks it against by finite differences."""
    d = F64(np.float32(h.sparsity_damping))
    means = d * means + F64(np.float32((1 - h.sparsity_damping) / state.shape[1])) * state.sum(axis=1, keepdims=True)
    if act == 'LOGISTIC':
        div = means * (1.0 - means)
    elif act == 'RECTIFIED_LINEAR':
        div = 1.0
    else:
        raise ValueError('sparsity targets exist for logistic and rectified linear units')
    return means, F64(np.float32(h.sparsity_cost)) * (means - F64(np.float32(h.sparsity_target))) / div


def momentum_and_epsilon(h, step):
    """parameter.py:108-126."""
    momentum = h.final_momentum - (h.final_momentum - h.initial_momentum) * np.exp(-float(step) / h.momentum_change_steps)
    eps = h.base_epsilon
    if h.epsilon_decay == 'INVERSE_T':
        eps = h.base_epsilon / (1 + float(step) / h.epsilon_decay_half_life)
    elif h.epsilon_decay == 'EXPONENTIAL':
        eps = h.base_epsilon / np.power(2, float(step) / h.epsilon_decay_half_life)
    if step < h.start_learning_after:
        eps = 0.0
    # the device takes both as float32
    return F64(np.float32(momentum)), F64(np.float32(eps))


def update(h, w, w_delta, gradient, step, no_reg=False):
    """parameter.py:80-106; returns (w, w_delta) and leaves the gradient to the caller to clear."""
    momentum, eps = momentum_and_epsilon(h, step)
    w_delta = w_delta * momentum
    if not no_reg and h.apply_l2_decay:
        w_delta = w_delta + F64(np.float32(h.l2_decay)) * w
    if not no_reg and h.apply_l1_decay and step > h.apply_l1decay_after:
        w_delta = w_delta + F64(np.float32(h.l1_decay)) * np.sign(w)
    w_delta = w_delta + gradient
    w = w - eps * w_delta
    if not no_reg and h.apply_weight_norm:
        w = cmo.normlimit_by_axis(w, 0, h.weight_norm)               # per column of the weight matrix
    return w, w_delta


def activate(act, x):
    if act == 'LOGISTIC':
        return 1.0 / (1.0 + np.exp(-x))
    if act == 'TANH':
        return np.tanh(x)
    if act == 'RECTIFIED_LINEAR':
        return np.maximum(x, 0.0)
    if act == 'RECTIFIED_LINEAR_SMOOTH':           # smooth_relu_layer.py:11-16
        return cmo.apply_log_1_plus_exp(x)
    if act == 'SOFTMAX':
        e = np.exp(x - x.max(axis=0, keepdims=True))
        return e / e.sum(axis=0, keepdims=True)
    if act == 'SIN':
        return np.sin(x)
    if act == 'COS':
        return np.cos(x)
    assert act == 'LINEAR'
    return x


class Net(object):
    """layers: dicts with 'act', 'hyper' (Hyper), for non-input layers 'bias' (n, 1) and 'edge':
    {'w', 'hyper', optionally 'cv' and 'local'}; the last layer also 'loss' ('CROSS_ENTROPY' or
    'SQUARED_LOSS').  Arrays are float64 copies; velocities start at zero."""

    def __init__(self, layers):
        self.layers = layers
        for L in layers[1:]:
            L['bias'] = np.array(L['bias'], dtype=F64).reshape(-1, 1)
            L['bias_delta'] = np.zeros_like(L['bias'])
            L['edge']['w'] = np.array(L['edge']['w'], dtype=F64)
            L['edge']['w_delta'] = np.zeros_like(L['edge']['w'])

    def forward(self, x, masks=None, train=False):
        """ComputeUp over the chain; masks[i] multiplies the state of layer i when it has dropout
        and train is set, otherwise such a state is scaled by 1 - dropout_prob."""
        states, stages, pre = [], [], {}
        for i, L in enumerate(self.layers):
            if i == 0:
                s = np.array(x, dtype=F64)
                stages.append(None)
            else:
                e = L['edge']
                if e.get('cv') is not None:
                    fwd = co.stage_forward(states[-1], e['w'], e['cv'], local=e.get('local', False))
                    stages.append(fwd)
                    s = fwd['state']
                else:
                    stages.append(None)
                    s = e['w'].T @ states[-1]
                pre[i] = s + L['bias']
                s = activate(L['act'], pre[i])
            h = L['hyper']
            if h.dropout:
                s = s * np.asarray(masks[i], dtype=F64) if train else s * F64(np.float32(1.0 - h.dropout_prob))
            states.append(s)
        self.states, self.stages, self.pre = states, stages, pre
        return states[-1]

    def loss_and_deriv(self, targets):
        L, s = self.layers[-1], self.states[-1]
        B = s.shape[1]
        perf = {}
        if L['act'] == 'SOFTMAX':
            labels = np.asarray(targets).astype(int).ravel()
            onehot = np.zeros_like(s)
            onehot[labels, np.arange(B)] = 1.0
            perf['cross_entropy'] = float(-np.log(s[labels, np.arange(B)] + 1e-10).sum())
            perf['correct_preds'] = float((s.argmax(axis=0) == labels).sum())
            return perf, s - onehot
        t = np.asarray(targets, dtype=F64)
        if L['loss'] == 'CROSS_ENTROPY':          # logistic units, logistic_layer.py:37-48
            perf['cross_entropy'] = float(-(t * np.log(s + 1e-10) + (1 - t) * np.log(1 - s + 1e-10)).sum())
            perf['correct_preds'] = float(((s >= 0.5) == (t >= 0.5)).sum())
            return perf, s - t
        d = s - t
        perf['error'] = float((d * d).sum())
        return perf, self._through_activation(len(self.layers) - 1, d)

    def _through_activation(self, i, d):
        """ComputeDeriv of layer i on the gradient w.r.t. its outputs."""
        L, s = self.layers[i], self.states[i]
        act = L['act']
        if act == 'LOGISTIC':
            return d * s * (1.0 - s)
        if act == 'RECTIFIED_LINEAR':
            return d * (s > 0)
        if act == 'RECTIFIED_LINEAR_SMOOTH':        # smooth_relu_layer.py:18-20: from the output, not masked
            return cmo.apply_rectified_linear_smooth_deriv(d, s)
        if act == 'SIN':                            # sin_layer.py:15-17, cos_layer.py:15-17: from the kept input
            return d * np.cos(self.pre[i])
        if act == 'COS':
            return d * -np.sin(self.pre[i])
        if act == 'TANH':
            d = d * (1.0 + s) * (1.0 - s) * 0.5     # the reference's kTanhDeriv halves the slope (cudamat_kernels.cu:663-669)
        # tanh and linear units multiply by the mask explicitly (tanh_layer.py:19-21, linear_layer.py:28-30)
        if L['hyper'].dropout and self._masks is not None:
            d = d * np.asarray(self._masks[i], dtype=F64)
        return d

    def train_step(self, x, targets, step, masks=None):
        """TrainOneBatch: forward with dropout, then for each layer from the top: gradient
        through the activation, down the edge, weight and bias updates."""
        self._masks = masks
        self.forward(x, masks, train=True)
        perf, d = self.loss_and_deriv(targets)
        B = self.states[0].shape[1]
        for i in range(len(self.layers) - 1, 0, -1):
            L, e = self.layers[i], self.layers[i]['edge']
            if i < len(self.layers) - 1:
                if L['hyper'].sparsity:               # neuralnet.py:221-223
                    if 'means' not in L:
                        L['means'] = np.full((d.shape[0], 1), F64(np.float32(L['hyper'].sparsity_target)))
                    L['means'], grad = sparsity_gradient(L['hyper'], L['act'], L['means'], self.states[i])
                    d = d + grad
                d = self._through_activation(i, d)
            below = self.states[i - 1]
            if e.get('cv') is not None:
                d_in, d_w = co.stage_backward(self.stages[i], e['w'], e['cv'], d, local=e.get('local', False))
            else:
                d_in, d_w = e['w'] @ d, below @ d.T
            e['w'], e['w_delta'] = update(e['hyper'], e['w'], e['w_delta'], d_w / B, step)
            L['bias'], L['bias_delta'] = update(L['hyper'], L['bias'], L['bias_delta'],
                                                d.sum(axis=1, keepdims=True) / B, step, no_reg=True)
            d = d_in
        return perf


def rbm_cd_step(p, hyper, v_data, step, hid_samples, vis_act='LOGISTIC', hid_act='LOGISTIC'):
    """One contrastive-divergence step of a two-layer Boltzmann machine as deepnet/dbm.py runs it
    (PositivePhase :121-152, NegativePhase :186-236 with unsampled inputs, the updates :246-266,
    sufficient statistics layer.py:194-205 and edge.py:236-242).  p holds float64 'W' (visible x
    hidden), 'bv', 'bh' (column vectors) and the previous updates 'dW', 'dbv', 'dbh'; hyper the
    Hyper objects 'edge', 'vis', 'hid'.  hid_samples[i] is the hidden sample that drives Gibbs sweep
    i (the caller feeds the ones the device drew), so len(hid_samples) sweeps are made.  Returns
    the squared reconstruction error of the first sweep.  A sparsity target on the hidden layer
    moves the positive statistics by the sparsity gradient.

    Pinned by tests/test_oracle_net.py against the C coding of the CD-1 step in
    oracle/host_backend.c (hb_rbm_cd1_step, written from cudamat/examples/rbm_cudamat.py:46-89)
    fed the same samples, and by the fixed point W = 0 where every quantity has a closed form."""
    v = np.asarray(v_data, dtype=F64)
    B = v.shape[1]
    W, bv, bh = p['W'], p['bv'], p['bh']
    h = activate(hid_act, W.T @ v + bh)
    stats_W, stats_v, stats_h = v @ h.T, v.sum(axis=1, keepdims=True), h.sum(axis=1, keepdims=True)
    if hyper['hid'].sparsity:
        # hidden units with a sparsity target (layer.py:206-209, edge.py:230-240): p['means_h'] carries
        # the running means from step to step
        if 'means_h' not in p:
            p['means_h'] = np.full_like(bh, F64(np.float32(hyper['hid'].sparsity_target)))
        p['means_h'], grad = sparsity_gradient(hyper['hid'], hid_act, p['means_h'], h)
        stats_h = stats_h - B * grad
        stats_W = v @ (h - grad).T
    error = None
    for i, hs in enumerate(hid_samples):
        v_neg = activate(vis_act, W @ np.asarray(hs, dtype=F64) + bv)
        if i == 0:
            error = float(((v_neg - v) ** 2).sum())
        h_neg = activate(hid_act, W.T @ v_neg + bh)
    stats_W = stats_W - v_neg @ h_neg.T
    stats_v = stats_v - v_neg.sum(axis=1, keepdims=True)
    stats_h = stats_h - h_neg.sum(axis=1, keepdims=True)
    scale = F64(np.float32(-1.0 / B))
    p['W'], p['dW'] = update(hyper['edge'], W, p['dW'], scale * stats_W, step)
    p['bv'], p['dbv'] = update(hyper['vis'], bv, p['dbv'], scale * stats_v, step, no_reg=True)
    p['bh'], p['dbh'] = update(hyper['hid'], bh, p['dbh'], scale * stats_h, step, no_reg=True)
    return error
