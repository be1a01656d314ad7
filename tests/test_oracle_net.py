"""CPU-only pins of the training-step restatement (oracle/net_oracle.py): gradients and k
steps of momentum SGD against torch.autograd / torch.optim.SGD on the same model, the update
rule's optional terms against explicit formulas, the schedules against closed forms."""
import numpy as np
import pytest
import torch
import torch.nn.functional as TF

from oracle import conv_oracle as co
from oracle import net_oracle as no


class _Cv(object):
    def __init__(self, **kw):
        self.size = self.stride = self.padding = self.num_filters = self.num_colors = 0
        self.max_pool, self.pool_size, self.pool_stride, self.prob = False, 0, 0, False
        self.rnorm, self.norm_size, self.pow_scale, self.add_scale = False, 0, 0.75, 0.001
        self.__dict__.update(kw)


def _half_slope_tanh(x):
    """tanh whose backward pass has half the slope, like the reference's kTanhDeriv
    (cudamat_kernels.cu:663-669: a * (1 + b) * (1 - b) * 0.5)."""
    y = 0.5 * torch.tanh(x)
    return y + y.detach()


def _torch_act(act, x):
    return {'LOGISTIC': torch.sigmoid, 'TANH': _half_slope_tanh, 'RECTIFIED_LINEAR': torch.relu,
            'LINEAR': lambda t: t, 'SIN': torch.sin, 'COS': torch.cos,
            'RECTIFIED_LINEAR_SMOOTH': torch.nn.functional.softplus}[act](x)


@pytest.mark.parametrize("hidden,loss", [('RECTIFIED_LINEAR', 'softmax'), ('LOGISTIC', 'softmax'), ('TANH', 'logistic_ce'),
                                         ('RECTIFIED_LINEAR', 'linear_sq'), ('SIN', 'softmax'), ('COS', 'linear_sq'),
                                         ('RECTIFIED_LINEAR_SMOOTH', 'softmax')])
def test_dense_net_steps_equal_torch_sgd(rng, hidden, loss):
    sizes, B, steps = (12, 9, 7, 5), 6, 4
    mom, eps, l2 = 0.9, 0.05, 0.01
    # float32-representable hyper-parameters, so that both sides use the same numbers
    mom, eps, l2 = (float(np.float32(v)) for v in (mom, eps, l2))
    he = no.Hyper(base_epsilon=eps, initial_momentum=mom, final_momentum=mom, apply_l2_decay=True, l2_decay=l2)
    hl = no.Hyper(base_epsilon=eps, initial_momentum=mom, final_momentum=mom)
    hd = no.Hyper(base_epsilon=eps, initial_momentum=mom, final_momentum=mom, dropout=True, dropout_prob=0.5)
    if hidden in ('SIN', 'COS', 'RECTIFIED_LINEAR_SMOOTH'):
        hd = hl     # (sin_layer.py:15-17 does not mask its derivative, so with dropout it is not the gradient of anything)
    out_act = {'softmax': 'SOFTMAX', 'logistic_ce': 'LOGISTIC', 'linear_sq': 'LINEAR'}[loss]
    Ws = [0.3 * rng.standard_normal((sizes[i], sizes[i + 1])) for i in range(3)]
    bs = [0.1 * rng.standard_normal((sizes[i + 1], 1)) for i in range(3)]
    layers = [{'act': 'LINEAR', 'hyper': hl},
              {'act': hidden, 'hyper': hd, 'bias': bs[0], 'edge': {'w': Ws[0], 'hyper': he}},
              {'act': hidden, 'hyper': hl, 'bias': bs[1], 'edge': {'w': Ws[1], 'hyper': he}},
              {'act': out_act, 'hyper': hl, 'bias': bs[2], 'edge': {'w': Ws[2], 'hyper': he},
               'loss': 'SQUARED_LOSS' if loss == 'linear_sq' else 'CROSS_ENTROPY'}]
    net = no.Net(layers)
    tw = [torch.tensor(w, requires_grad=True) for w in Ws]
    tb = [torch.tensor(b, requires_grad=True) for b in bs]
    opt = torch.optim.SGD([{'params': tw, 'weight_decay': l2}, {'params': tb, 'weight_decay': 0.0}], lr=eps, momentum=mom)
    for step in range(steps):
        x = rng.standard_normal((sizes[0], B))
        mask = (rng.random((sizes[1], B)) > 0.5).astype(np.float64) if hd.dropout else np.ones((sizes[1], B))
        if loss == 'softmax':
            targets = rng.integers(0, sizes[-1], (1, B)).astype(np.float64)
        elif loss == 'logistic_ce':
            targets = (rng.random((sizes[-1], B)) < 0.5).astype(np.float64)
        else:
            targets = rng.standard_normal((sizes[-1], B))
        perf = net.train_step(x, targets, step, masks=[None, mask, None, None])
        # the same step in torch: mean loss over the batch gives deepnet's 1/B gradients
        opt.zero_grad()
        h = torch.tensor(x)
        h = _torch_act(hidden, tw[0].T @ h + tb[0]) * torch.tensor(mask)
        h = _torch_act(hidden, tw[1].T @ h + tb[1])
        z = tw[2].T @ h + tb[2]
        if loss == 'softmax':
            L = TF.cross_entropy(z.T, torch.tensor(targets.ravel()).long(), reduction='sum')
            assert abs(perf['cross_entropy'] - float(L.detach())) < 1e-6 * max(1.0, abs(float(L.detach())))
        elif loss == 'logistic_ce':
            L = TF.binary_cross_entropy_with_logits(z, torch.tensor(targets), reduction='sum')
            assert abs(perf['cross_entropy'] - float(L.detach())) < 1e-6 * max(1.0, abs(float(L.detach())))
        else:
            L = 0.5 * ((z - torch.tensor(targets)) ** 2).sum()
            assert abs(perf['error'] - 2 * float(L.detach())) < 1e-9 * max(1.0, float(L.detach()))
        (L / B).backward()
        opt.step()
        for i in range(3):
            assert np.allclose(net.layers[i + 1]['edge']['w'], tw[i].detach().numpy(), rtol=0, atol=1e-12), (step, i)
            assert np.allclose(net.layers[i + 1]['bias'], tb[i].detach().numpy(), rtol=0, atol=1e-12), (step, i)


def test_conv_net_steps_equal_torch_sgd(rng):
    """input 2x8x8 -> conv 3x3 pad 1 (8 filters) + pool 2/2 -> ReLU -> dense softmax."""
    N, C, H, F, k, classes = 5, 2, 8, 16, 3, 4
    cv = _Cv(size=k, stride=1, padding=1, num_filters=F, num_colors=C, max_pool=True, pool_size=2, pool_stride=2)
    mom, eps = float(np.float32(0.5)), float(np.float32(0.1))
    h = no.Hyper(base_epsilon=eps, initial_momentum=mom, final_momentum=mom)
    wc, bc = 0.3 * rng.standard_normal((F, C * k * k)), 0.1 * rng.standard_normal((F * 16, 1))
    wd, bd = 0.1 * rng.standard_normal((F * 16, classes)), np.zeros((classes, 1))
    net = no.Net([{'act': 'LINEAR', 'hyper': h},
                  {'act': 'RECTIFIED_LINEAR', 'hyper': h, 'bias': bc, 'edge': {'w': wc, 'hyper': h, 'cv': cv}},
                  {'act': 'SOFTMAX', 'hyper': h, 'bias': bd, 'edge': {'w': wd, 'hyper': h}, 'loss': 'CROSS_ENTROPY'}])
    t = [torch.tensor(a, requires_grad=True) for a in (wc, bc, wd, bd)]
    opt = torch.optim.SGD(t, lr=eps, momentum=mom)
    for step in range(3):
        x = rng.standard_normal((C * H * H, N))
        labels = rng.integers(0, classes, (1, N)).astype(np.float64)
        net.train_step(x, labels, step)
        opt.zero_grad()
        xt = torch.tensor(co.to_nchw(x.T, C, H))
        a = TF.max_pool2d(TF.conv2d(xt, t[0].reshape(F, C, k, k), padding=1), 2, 2)       # (N, F, 4, 4)
        a = torch.relu(a.reshape(N, -1).T + t[1])                                           # (F*16, N), deepnet's order
        z = t[2].T @ a + t[3]
        (TF.cross_entropy(z.T, torch.tensor(labels.ravel()).long(), reduction='sum') / N).backward()
        opt.step()
        got = [net.layers[1]['edge']['w'], net.layers[1]['bias'], net.layers[2]['edge']['w'], net.layers[2]['bias']]
        for g, want in zip(got, t):
            assert np.allclose(g, want.detach().numpy(), rtol=0, atol=1e-12), step


def test_update_rule_optional_terms_and_schedules(rng):
    w, v, g = rng.standard_normal((6, 4)), rng.standard_normal((6, 4)), rng.standard_normal((6, 4))
    h = no.Hyper(base_epsilon=0.5, initial_momentum=0.5, final_momentum=0.75, momentum_change_steps=10,
                 apply_l1_decay=True, l1_decay=0.25, apply_l1decay_after=3, apply_weight_norm=True, weight_norm=1.5,
                 epsilon_decay='INVERSE_T', epsilon_decay_half_life=8, start_learning_after=2)
    # schedules: momentum rises from initial to final with time constant momentum_change_steps
    m0, e0 = no.momentum_and_epsilon(h, 0)
    assert m0 == 0.5 and e0 == 0.0                              # no learning before start_learning_after
    m10, e8 = no.momentum_and_epsilon(h, 10)[0], no.momentum_and_epsilon(h, 8)[1]
    assert abs(m10 - (0.75 - 0.25 * np.exp(-1.0))) < 1e-7 and e8 == 0.25   # half life: epsilon halves at step 8
    h2 = no.Hyper(base_epsilon=0.5, epsilon_decay='EXPONENTIAL', epsilon_decay_half_life=8)
    assert no.momentum_and_epsilon(h2, 16)[1] == 0.125
    # step 3: the L1 term is not yet applied (step > apply_l1decay_after); step 4: it is
    for step, l1_on in ((3, False), (4, True)):
        m, e = no.momentum_and_epsilon(h, step)
        v2 = m * v + (0.25 * np.sign(w) if l1_on else 0.0) + g
        w2 = w - e * v2
        n = np.sqrt((w2 ** 2).sum(axis=0))
        w2 = w2 * np.where(n > 1.5, 1.5 / n, 1.0)
        gw, gv = no.update(h, w, v, g, step)
        assert np.allclose(gv, v2, atol=1e-14) and np.allclose(gw, w2, atol=1e-14)
        assert np.all(np.sqrt((gw ** 2).sum(axis=0)) <= 1.5 + 1e-12)
    # no_reg (the bias): neither decay nor the norm limit
    gw, gv = no.update(h, w, v, g, 9, no_reg=True)
    m, e = no.momentum_and_epsilon(h, 9)
    assert np.allclose(gv, m * v + g, atol=1e-14) and np.allclose(gw, w - e * (m * v + g), atol=1e-14)


def test_rbm_cd_step_against_the_c_coding_and_a_fixed_point(rng):
    import ctypes as ct
    import os
    from oracle import mwc
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    lib = ct.CDLL(os.path.join(root, 'oracle', 'liboracle_host.so'))
    nv, nh, B, lr = 60, 40, 20, 0.1
    v = np.asarray(rng.random((nv, B)) < 0.3, dtype=np.float32, order='F')
    W = np.asarray(0.1 * rng.standard_normal((nv, nh)), dtype=np.float32, order='F')
    bv = np.asarray(0.1 * rng.standard_normal(nv), dtype=np.float32)
    bh = np.asarray(0.1 * rng.standard_normal(nh), dtype=np.float32)
    p = {'W': W.astype(np.float64), 'bv': bv.astype(np.float64).reshape(-1, 1), 'bh': bh.astype(np.float64).reshape(-1, 1)}
    p.update(dW=np.zeros((nv, nh)), dbv=np.zeros((nv, 1)), dbh=np.zeros((nh, 1)))
    mults = mwc.load_multipliers(os.path.join(root, 'deepnet_amd', 'rnd_multipliers_32bit.txt'))
    words = np.empty(mwc.NUM_RND_STREAMS, dtype=np.uint64)
    fp = ct.POINTER(ct.c_float)
    u32, u64 = mults.ctypes.data_as(ct.POINTER(ct.c_uint32)), words.ctypes.data_as(ct.POINTER(ct.c_uint64))
    lib.mwc_seed(u32, u64, ct.c_uint32(5))
    h, hs, h2 = (np.empty((nh, B), np.float32, order='F') for _ in range(3))
    v2 = np.empty((nv, B), np.float32, order='F')
    q = lambda a: a.ctypes.data_as(fp)
    lib.hb_set_threads(1)
    lib.hb_rbm_cd1_step(q(W), q(bv), q(bh), q(v), nv, nh, B, ct.c_float(lr), u32, u64, q(h), q(hs), q(v2), q(h2))
    hyp = no.Hyper(base_epsilon=lr)                       # no momentum, no decay: the example's plain SGD
    err = no.rbm_cd_step(p, {'edge': hyp, 'vis': hyp, 'hid': hyp}, v, 0, [hs])
    assert np.allclose(p['W'], W, rtol=1e-5, atol=1e-7)
    assert np.allclose(p['bv'].ravel(), bv, rtol=1e-5, atol=1e-7) and np.allclose(p['bh'].ravel(), bh, rtol=1e-5, atol=1e-7)
    assert abs(err - float(((v2.astype(np.float64) - v) ** 2).sum())) < 1e-4 * err
    # W = 0, zero biases: h = 1/2 everywhere, the reconstruction is 1/2 whatever the samples, so
    # dW = eps/B * (v - 1/2) (1/2)^T summed over the batch, dbv = eps * (mean(v) - 1/2), dbh = 0
    z = {'W': np.zeros((nv, nh)), 'bv': np.zeros((nv, 1)), 'bh': np.zeros((nh, 1)),
         'dW': np.zeros((nv, nh)), 'dbv': np.zeros((nv, 1)), 'dbh': np.zeros((nh, 1))}
    err = no.rbm_cd_step(z, {'edge': hyp, 'vis': hyp, 'hid': hyp}, v, 0, [hs, 1 - hs])
    eps = float(np.float32(lr))
    rowsum = (v.astype(np.float64) - 0.5).sum(axis=1, keepdims=True)
    assert np.allclose(z['W'], eps / B * 0.5 * rowsum * np.ones((1, nh)), rtol=1e-6, atol=1e-12)
    assert np.allclose(z['bv'], eps / B * rowsum, rtol=1e-6, atol=1e-12) and np.allclose(z['bh'], 0.0, atol=1e-12)
    assert abs(err - 0.25 * nv * B) < 1e-9


def test_sparsity_term_is_the_kl_gradient_and_enters_both_kinds_of_step(rng):
    """layer.py:138-155.  (1) For logistic units cost * (mean - target) / (mean (1 - mean)) is the
    derivative of cost * KL(Bernoulli(target) || Bernoulli(mean)): checked by central differences,
    and the running mean by writing the recursion out.  (2) With damping 0 the mean is the batch
    mean, so a feed-forward step equals torch SGD on loss + B * cost * sum_i KL(target || mean_i).
    (3) An RBM at W = 0, b = 0 has every unit at 1/2, which gives the update in closed form."""
    h = no.Hyper(sparsity=True, sparsity_target=0.25, sparsity_cost=0.125, sparsity_damping=0.5)
    state1, state2 = rng.random((5, 4)), rng.random((5, 4))
    m0 = np.full((5, 1), 0.25)
    m1, g1 = no.sparsity_gradient(h, 'LOGISTIC', m0, state1)
    m2, g2 = no.sparsity_gradient(h, 'LOGISTIC', m1, state2)
    assert np.allclose(m2, 0.25 * 0.25 + 0.25 * state1.mean(axis=1, keepdims=True) + 0.5 * state2.mean(axis=1, keepdims=True),
                       rtol=0, atol=1e-15)
    kl = lambda m: 0.25 * np.log(0.25 / m) + 0.75 * np.log(0.75 / (1 - m))
    d = 1e-6
    assert np.allclose(g2, 0.125 * (kl(m2 + d) - kl(m2 - d)) / (2 * d), rtol=1e-7)
    _, g_relu = no.sparsity_gradient(h, 'RECTIFIED_LINEAR', m1, state2)
    assert np.allclose(g_relu, 0.125 * (m2 - 0.25), rtol=0, atol=1e-15)
    with pytest.raises(ValueError):
        no.sparsity_gradient(h, 'TANH', m0, state1)

    # (2) feed-forward, batch of 8 so that 1/B is the same number in float32 and float64
    sizes, B, steps = (12, 9, 7, 5), 8, 3
    eps, mom = float(np.float32(0.05)), float(np.float32(0.9))
    he = no.Hyper(base_epsilon=eps, initial_momentum=mom, final_momentum=mom)
    hs = no.Hyper(base_epsilon=eps, initial_momentum=mom, final_momentum=mom, sparsity=True, sparsity_target=0.25,
                  sparsity_cost=0.125, sparsity_damping=0.0)
    Ws = [0.3 * rng.standard_normal((sizes[i], sizes[i + 1])) for i in range(3)]
    bs = [0.1 * rng.standard_normal((sizes[i + 1], 1)) for i in range(3)]
    net = no.Net([{'act': 'LINEAR', 'hyper': he},
                  {'act': 'LOGISTIC', 'hyper': he, 'bias': bs[0], 'edge': {'w': Ws[0], 'hyper': he}},
                  {'act': 'LOGISTIC', 'hyper': hs, 'bias': bs[1], 'edge': {'w': Ws[1], 'hyper': he}},
                  {'act': 'SOFTMAX', 'hyper': he, 'bias': bs[2], 'edge': {'w': Ws[2], 'hyper': he}, 'loss': 'CROSS_ENTROPY'}])
    tw = [torch.tensor(w, requires_grad=True) for w in Ws]
    tb = [torch.tensor(b, requires_grad=True) for b in bs]
    opt = torch.optim.SGD(tw + tb, lr=eps, momentum=mom)
    for step in range(steps):
        x = rng.standard_normal((sizes[0], B))
        targets = rng.integers(0, sizes[-1], (1, B)).astype(np.float64)
        net.train_step(x, targets, step)
        opt.zero_grad()
        a1 = torch.sigmoid(tw[0].T @ torch.tensor(x) + tb[0])
        a2 = torch.sigmoid(tw[1].T @ a1 + tb[1])
        z = tw[2].T @ a2 + tb[2]
        m = a2.mean(dim=1)
        penalty = (0.25 * torch.log(0.25 / m) + 0.75 * torch.log(0.75 / (1 - m))).sum()
        L = TF.cross_entropy(z.T, torch.tensor(targets.ravel()).long(), reduction='sum') + B * 0.125 * penalty
        (L / B).backward()
        opt.step()
        for i in range(3):
            assert np.allclose(net.layers[i + 1]['edge']['w'], tw[i].detach().numpy(), rtol=0, atol=1e-12), (step, i)
            assert np.allclose(net.layers[i + 1]['bias'], tb[i].detach().numpy(), rtol=0, atol=1e-12), (step, i)

    # (3) RBM at the origin: all probabilities 1/2
    nv, nh = 6, 4
    hr = no.Hyper(base_epsilon=eps, sparsity=True, sparsity_target=0.25, sparsity_cost=0.125, sparsity_damping=0.5)
    plain = no.Hyper(base_epsilon=eps)
    p = {'W': np.zeros((nv, nh)), 'bv': np.zeros((nv, 1)), 'bh': np.zeros((nh, 1)),
         'dW': np.zeros((nv, nh)), 'dbv': np.zeros((nv, 1)), 'dbh': np.zeros((nh, 1))}
    v = (rng.random((nv, B)) < 0.5).astype(np.float64)
    no.rbm_cd_step(p, {'edge': plain, 'vis': plain, 'hid': hr}, v, 0, [np.zeros((nh, B))])
    mean = 0.5 * 0.25 + 0.5 * 0.5
    g = 0.125 * (mean - 0.25) / (mean * (1 - mean))
    assert np.allclose(p['means_h'], mean, rtol=0, atol=1e-15)
    assert np.allclose(p['bh'], -eps * g, rtol=0, atol=1e-15)
    assert np.allclose(p['W'], eps * (v.sum(axis=1, keepdims=True) * (0.5 - g) / B - 0.25) * np.ones((1, nh)), rtol=0, atol=1e-15)
    assert np.allclose(p['bv'], eps * (v.mean(axis=1, keepdims=True) - 0.5), rtol=0, atol=1e-15)
