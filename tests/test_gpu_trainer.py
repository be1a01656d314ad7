"""Nets built from deepnet's own model files (deepnet_amd/trainer.py: the role of
deepnet/trainer.py:34-46 + deepnet/neuralnet.py:70-109 + deepnet/parameter.py:21-71): the initial
parameters against the numpy draws the reference makes (same seed, same order), the merged
hyper-parameters, and training steps against the float64 restatement in oracle/net_oracle.py
(parameters within 1e-4 relative + 1e-6, losses within 1e-5 relative).  The model files under
tests/golden/ were written for these tests in the format of deepnet/examples/*/model*.pbtxt."""
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from oracle import net_oracle as no   # noqa: E402

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden')
TRAIN_OP = 'optimizer: %s\nstopcondition { steps: 100 }\ntrain: true\nbatchsize: 32\ndata_proto: "unused.pbtxt"\n'


def _f(a):
    return np.asarray(a, dtype=np.float32, order='F')


def _ohyper(h):
    return no.Hyper(**{k: getattr(h, k) for k in vars(no.Hyper()) if hasattr(h, k)})


def _oracle_chain(net, order):
    """The oracle's list-of-dicts form of a chain-shaped device net, from the device's parameters."""
    by_name = {l.name: l for l in net.layer}
    out = []
    for i, name in enumerate(order):
        L = by_name[name]
        d = {'act': L.activation, 'hyper': _ohyper(L.hyperparams)}
        if i:
            E = next(e for e in net.edge if e.node2 is L)
            assert E.node1 is by_name[order[i - 1]]
            d.update(bias=L.params['bias'].asarray().astype(np.float64), loss=L.loss_function,
                     edge={'w': E.params['weight'].asarray().astype(np.float64), 'hyper': _ohyper(E.hyperparams),
                           'cv': getattr(E, 'conv_params', None), 'local': E.local})
        out.append(d)
    return no.Net(out), [by_name[n] for n in order]


def _steps_match(cm, net, onet, chain, batches):
    for step, (x, t) in enumerate(batches):
        chain[0].data.assign(cm.CUDAMatrix(_f(x)))
        chain[-1].data.assign(cm.CUDAMatrix(_f(t)))
        losses = net.TrainOneBatch(step)
        masks = [L.mask.asarray().copy() if L.hyperparams.dropout else None for L in chain]
        perf = onet.train_step(x, t, step, masks=masks)
        # layers with a sparsity target report their mean activity first (neuralnet.py:176-181:
        # the per-unit sums over the batch, averaged over the units), then the output layer its loss
        sparse = [i for i, L in enumerate(chain) if L.hyperparams.sparsity and not L.is_input]
        assert len(losses) == len(sparse) + 1
        for rec, i in zip(losses, sparse):
            want = float(onet.states[i].sum(axis=1).mean())
            assert rec.count == chain[i].batchsize and abs(rec.sparsity - want) <= 1e-4 * max(1.0, abs(want)), (step, i)
        for key, want in perf.items():
            assert abs(getattr(losses[-1], key) - want) <= 1e-5 * max(1.0, abs(want)), (step, key)
        for i, L in enumerate(chain[1:], 1):
            E = next(e for e in net.edge if e.node2 is L)
            assert np.allclose(E.params['weight'].asarray(), onet.layers[i]['edge']['w'], rtol=1e-4, atol=1e-6), (step, i)
            assert np.allclose(L.params['bias'].asarray(), onet.layers[i]['bias'], rtol=1e-4, atol=1e-6), (step, i)


def test_convnet_from_a_model_file(cm, cc):
    from deepnet_amd import trainer, util, layer as dl, neuralnet as dnn
    model = util.ReadModel(os.path.join(GOLDEN, 'small_convnet.pbtxt'))
    net = trainer.CreateDeepnet(model, TRAIN_OP % 'GRADIENT_DESCENT')
    assert type(net) is dnn.NeuralNet and net.batchsize == 32 and net.train_stop_steps == 100
    by_name = {l.name: l for l in net.layer}
    assert [type(by_name[n]) for n in ('input_layer', 'output_layer', 'hidden1', 'hidden3')] == \
        [dl.LinearLayer, dl.SoftmaxLayer, dl.ReluLayer, dl.ReluLayer]
    assert [n.name for n in net.node_list] == ['input_layer', 'hidden1', 'hidden2', 'hidden3', 'output_layer']

    # parameter.py:43-71 on numpy's global generator, seeded with the model's seed: layers, then edges, as listed
    r = np.random.RandomState(17)
    want = {'output_layer': np.zeros((10, 1)), 'hidden1': np.zeros((400, 1)) + 0.1,
            'hidden2': 0.01 * r.randn(144, 1), 'hidden3': np.zeros((64, 1))}
    want_w = [0.1 * r.randn(16, 18), (1.0 / np.sqrt(16)) * r.randn(16, 9 * 9 * 16),
              (1.0 / np.sqrt(64)) * (2 * r.rand(144, 64) - 1), 0.1 * (2 * r.rand(64, 10) - 1)]
    for name, b in want.items():
        assert np.array_equal(by_name[name].params['bias'].asarray(), b.astype(np.float32)), name
    for E, w in zip(net.edge, want_w):
        assert np.array_equal(E.params['weight'].asarray(), w.astype(np.float32)), E.name
    assert net.edge[0].conv and net.edge[1].local and not (net.edge[2].conv or net.edge[2].local)

    # neuralnet.py:80-93: the model's hyper-parameters under those written for the layer / edge
    h1, h3, e0, e1 = by_name['hidden1'].hyperparams, by_name['hidden3'].hyperparams, net.edge[0].hyperparams, net.edge[1].hyperparams
    assert (h1.activation, h1.apply_l2_decay, h1.base_epsilon, h1.final_momentum) == ('RECTIFIED_LINEAR', False, 0.05, 0.9)
    assert (h3.dropout, h3.dropout_prob, h3.apply_l2_decay) == (True, 0.5, True)
    assert (e0.base_epsilon, e0.initial_momentum, e0.final_momentum, e0.momentum_change_steps, e0.apply_l2_decay) == \
        (0.01, 0.9, 0.9, 5, False)
    assert (e1.base_epsilon, e1.initial_momentum, e1.apply_l2_decay, e1.l2_decay) == (0.05, 0.5, True, 0.001)
    assert by_name['output_layer'].hyperparams.dropout is False and by_name['output_layer'].loss_function == 'CROSS_ENTROPY'

    order = ['input_layer', 'hidden1', 'hidden2', 'hidden3', 'output_layer']
    onet, chain = _oracle_chain(net, order)
    rng = np.random.default_rng(4)
    batches = [(rng.standard_normal((288, 32)), rng.integers(0, 10, (1, 32)).astype(np.float64)) for _ in range(3)]
    _steps_match(cm, net, onet, chain, batches)


DENSE_SPARSE = '''
name: "sparse_ff"  model_type: FEED_FORWARD_NET  seed: 3
hyperparams { base_epsilon: 0.1 initial_momentum: 0.5 final_momentum: 0.5 activation: LOGISTIC }
layer { name: "in" dimensions: 40 is_input: true hyperparams { activation: LINEAR } }
layer { name: "h1" dimensions: 48 param { name: "bias" initialization: CONSTANT }
        hyperparams { sparsity: true sparsity_target: 0.1 sparsity_cost: 0.5 sparsity_damping: 0.5 } }
layer { name: "h2" dimensions: 24 param { name: "bias" initialization: CONSTANT }
        hyperparams { activation: RECTIFIED_LINEAR sparsity: true sparsity_target: 0.05 sparsity_cost: 0.25 } }
layer { name: "out" dimensions: 8 is_output: true loss_function: CROSS_ENTROPY param { name: "bias" initialization: CONSTANT } }
edge { node1: "in" node2: "h1" param { name: "weight" initialization: DENSE_GAUSSIAN sigma: 0.3 } }
edge { node1: "h1" node2: "h2" param { name: "weight" initialization: DENSE_GAUSSIAN sigma: 0.3 } }
edge { node1: "h2" node2: "out" param { name: "weight" initialization: DENSE_GAUSSIAN sigma: 0.3 } }
'''


def test_sparsity_targets_on_hidden_layers_of_a_feed_forward_net(cm):
    """neuralnet.py:221-223 + layer.py:138-155: logistic units (divisor mean (1 - mean)) and
    rectified linear units (divisor 1), running means carried from step to step."""
    from deepnet_amd import trainer
    net = trainer.CreateDeepnet(DENSE_SPARSE, batchsize=16)
    onet, chain = _oracle_chain(net, ['in', 'h1', 'h2', 'out'])
    rng = np.random.default_rng(9)
    batches = [(rng.standard_normal((40, 16)), (rng.random((8, 16)) < 0.3).astype(np.float64)) for _ in range(4)]
    _steps_match(cm, net, onet, chain, batches)
    for i in (1, 2):
        assert np.allclose(chain[i].means.asarray(), onet.layers[i]['means'], rtol=1e-5)
    assert abs(float(onet.layers[1]['means'].mean()) - 0.1) > 0.05       # the means did move away from the target


@pytest.mark.parametrize("text,what", [
    ('name: "m" model_type: DBN', 'model_type'),
    ('name: "m" model_type: DBM', 'model_type'),
    ('name: "m" model_type: FEED_FORWARD_NET layer { name: "a" dimensions: 4 tied: true tied_to: "b" }', 'tied'),
    ('name: "m" model_type: FEED_FORWARD_NET layer { name: "a" dimensions: 4 hyperparams { activation: REPLICATED_SOFTMAX } }', 'activation'),
    ('name: "m" model_type: FEED_FORWARD_NET layer { name: "a" dimensions: 4 hyperparams { shared_prior: true adapt: ADAGRAD } }', 'shared_prior'),
    ('name: "m" model_type: FEED_FORWARD_NET layer { name: "a" dimensions: 4 hyperparams { adapt: ADAGRAD } }', 'adapt'),
    ('name: "m" model_type: FEED_FORWARD_NET hyperparams { learn_precision: true } layer { name: "a" dimensions: 4 }', 'learn_precision'),
    ('name: "m" model_type: FEED_FORWARD_NET layer { name: "a" dimensions: 4 param { name: "bias" initialization: PRETRAINED'
     ' pretrained_model: "binary_checkpoint.gz" } }', 'text-format'),
    ('name: "m" model_type: FEED_FORWARD_NET layer { name: "a" dimensions: 4 hyperparams { activation: TANH sparsity: true } is_input: true }'
     ' layer { name: "b" dimensions: 4 hyperparams { activation: TANH sparsity: true } }'
     ' layer { name: "c" dimensions: 2 is_output: true }'
     ' edge { node1: "a" node2: "b" param { name: "weight" } } edge { node1: "b" node2: "c" param { name: "weight" } }', None),
])
def test_what_the_builder_does_not_have_is_refused_by_name(cm, text, what):
    from deepnet_amd import trainer
    if what is None:
        # builds, and fails where the reference fails too: tanh units have no sparsity divisor (tanh_layer.py:45-50
        # reads a buffer that is never allocated)
        net = trainer.CreateDeepnet(text, batchsize=4)
        net.layer[0].data.assign(cm.CUDAMatrix(_f(np.ones((4, 4)))))
        net.layer[2].data.assign(cm.CUDAMatrix(_f(np.ones((2, 4)))))
        with pytest.raises(Exception, match='Sparsity not implemented'):
            net.TrainOneBatch(0)
        return
    with pytest.raises(NotImplementedError, match=what):
        trainer.CreateDeepnet(text, batchsize=4)


BLOBS = '''
name: "blobs"  model_type: FEED_FORWARD_NET  seed: 5
hyperparams { base_epsilon: 0.1 initial_momentum: 0.5 final_momentum: 0.9 momentum_change_steps: 50 activation: LOGISTIC }
layer { name: "in" dimensions: 20 is_input: true hyperparams { activation: LINEAR } }
layer { name: "h" dimensions: 32 param { name: "bias" initialization: CONSTANT } }
layer { name: "out" dimensions: 1 numlabels: 3 is_output: true loss_function: CROSS_ENTROPY
        hyperparams { activation: SOFTMAX } param { name: "bias" initialization: CONSTANT } }
edge { node1: "in" node2: "h" param { name: "weight" initialization: DENSE_GAUSSIAN_SQRT_FAN_IN sigma: 1.0 } }
edge { node1: "h" node2: "out" param { name: "weight" initialization: DENSE_GAUSSIAN_SQRT_FAN_IN sigma: 1.0 } }
'''


def test_training_loop_learns_from_a_device_resident_data_set(cm):
    """Model file -> net, arrays -> GPUCache (shuffled on the device), NeuralNet.Train with periodic
    evaluation (neuralnet.py:589-670): three Gaussian blobs are told apart after 300 steps, the
    accumulated counters add up, and the parameters equal those of stepping by hand over the
    same batches."""
    from deepnet_amd import trainer, datahandler as dh
    rng = np.random.default_rng(21)
    centres = 1.5 * rng.standard_normal((3, 20))

    def blobs(n):
        labels = rng.integers(0, 3, n)
        return (centres[labels] + rng.standard_normal((n, 20))).astype(np.float32), labels.reshape(-1, 1).astype(np.float32)
    train_x, train_y = blobs(600)
    test_x, test_y = blobs(200)
    op = 'optimizer: GRADIENT_DESCENT\nstopcondition { steps: 300 }\nbatchsize: 50\ndata_proto: "unused"\n'

    def run(by_hand):
        np.random.seed(77)                   # the shuffles of the cache
        net = trainer.CreateDeepnet(BLOBS, op)
        train = dh.GPUCache(dh.ArraySource([train_x, train_y]), 600, [20, 1], randomize=False)
        test = dh.GPUCache(dh.ArraySource([test_x, test_y]), 200, [20, 1])
        if by_hand:
            for step in range(300):
                net.GetBatch(train)
                net.TrainOneBatch(step)
            return net, None
        seen = []
        history = net.Train(train, eval_handler=test, eval_steps=4, eval_after=100, report=seen.append)
        assert history == seen
        return net, history
    net, history = run(False)
    assert [r['step'] for r in history] == [100, 200, 300]
    for r in history:
        assert len(r['train']) == 1 and r['train'][0].count == 100 * 50
        assert len(r['eval']) == 1 and r['eval'][0].count == 4 * 50
    first, last = history[0], history[-1]
    assert last['eval'][0].correct_preds / 200.0 > 0.95
    assert last['train'][0].cross_entropy < 0.5 * first['train'][0].cross_entropy
    # before training the net is at chance
    fresh = trainer.CreateDeepnet(BLOBS, op)
    chance = fresh.Evaluate(dh.GPUCache(dh.ArraySource([test_x, test_y]), 200, [20, 1]), 4)
    assert chance[0].correct_preds / 200.0 < 0.7
    by_hand, _ = run(True)
    for a, b in zip(net.edge, by_hand.edge):
        assert np.array_equal(a.params['weight'].asarray(), b.params['weight'].asarray())
    # a shuffled cache serves the same set in another order: still learns
    np.random.seed(1)
    net2 = trainer.CreateDeepnet(BLOBS, op)
    shuffled = dh.GPUCache(dh.ArraySource([train_x, train_y]), 600, [20, 1], randomize=True)
    h2 = net2.Train(shuffled, steps=300, eval_handler=dh.GPUCache(dh.ArraySource([test_x, test_y]), 200, [20, 1]), eval_steps=4)
    assert [r['step'] for r in h2] == [300] and h2[0]['eval'][0].correct_preds / 200.0 > 0.95


def test_model_written_with_its_parameters_loads_back_bit_for_bit(cm, cc, tmp_path):
    """parameter.py:17-19 / util.py:13-21, 79-81: train a few steps, store the parameters in the
    model message, write it as text, build a second net from the file: same parameters, same
    next step."""
    from deepnet_amd import trainer, util
    net = trainer.CreateDeepnet(os.path.join(GOLDEN, 'small_convnet.pbtxt'), TRAIN_OP % 'GRADIENT_DESCENT')
    by_name = {l.name: l for l in net.layer}
    rng = np.random.default_rng(6)
    x, t = _f(rng.standard_normal((288, 32))), _f(rng.integers(0, 10, (1, 32)))
    for step in range(2):
        by_name['input_layer'].data.assign(cm.CUDAMatrix(x))
        by_name['output_layer'].data.assign(cm.CUDAMatrix(t))
        net.TrainOneBatch(step)
    path = str(tmp_path / 'checkpoint.pbtxt')
    util.WritePbtxt(path, trainer.ModelWithParameters(net))
    again = trainer.CreateDeepnet(util.ReadModel(path), TRAIN_OP % 'GRADIENT_DESCENT')
    for a, b in zip(net.edge, again.edge):
        assert a.params['weight'].shape == b.params['weight'].shape
        assert np.array_equal(a.params['weight'].asarray().view(np.uint32), b.params['weight'].asarray().view(np.uint32))
    for a, b in zip(net.layer, again.layer):
        assert np.array_equal(a.params['bias'].asarray().view(np.uint32), b.params['bias'].asarray().view(np.uint32))
    # evaluation (no dropout, no momentum history involved) gives the same loss
    losses = []
    for n in (net, again):
        names = {l.name: l for l in n.layer}
        names['input_layer'].data.assign(cm.CUDAMatrix(x))
        names['output_layer'].data.assign(cm.CUDAMatrix(t))
        losses.append(n.EvaluateOneBatch()[0].cross_entropy)
    assert losses[0] == losses[1]
    with pytest.raises(ValueError, match='stored values'):
        bad = util.ReadModel(path)
        bad.all('layer')[2].param.set('dimensions', 3, 1)
        trainer.CreateDeepnet(bad, TRAIN_OP % 'GRADIENT_DESCENT')


def test_pretrained_parameters_come_from_other_model_files(cm, tmp_path):
    """layer.py:66-98, edge.py:165-215: a stack initialised from another model's file -- the
    weight as it is, its transpose times mult_factor for the decoder, biases from named nodes,
    the mean of two files, an .npy array."""
    from deepnet_amd import trainer, util
    rbm = trainer.CreateDeepnet("""
      name: "pre" model_type: FEED_FORWARD_NET hyperparams { activation: LOGISTIC }
      layer { name: "input_layer" dimensions: 96 is_input: true param { name: "bias" initialization: CONSTANT } }
      layer { name: "hidden1" dimensions: 64 is_output: true param { name: "bias" initialization: CONSTANT constant: -1.0 } }
      edge { node1: "input_layer" node2: "hidden1" param { name: "weight" initialization: DENSE_GAUSSIAN_SQRT_FAN_IN sigma: 1.0 } }
    """, batchsize=8)
    rng = np.random.default_rng(3)
    for obj, key in ((rbm.edge[0], 'weight'), (rbm.layer[0], 'bias'), (rbm.layer[1], 'bias')):
        obj.params[key].overwrite(_f(rng.standard_normal(obj.params[key].shape)))
    util.WritePbtxt(str(tmp_path / 'rbm_a.pbtxt'), trainer.ModelWithParameters(rbm))
    w_a = rbm.edge[0].params['weight'].asarray().copy()
    bv, bh = rbm.layer[0].params['bias'].asarray().copy(), rbm.layer[1].params['bias'].asarray().copy()
    rbm.edge[0].params['weight'].overwrite(_f(rng.standard_normal((96, 64))))
    util.WritePbtxt(str(tmp_path / 'rbm_b.pbtxt'), trainer.ModelWithParameters(rbm))
    w_b = rbm.edge[0].params['weight'].asarray().copy()
    out_bias = rng.standard_normal(96).astype(np.float32)
    np.save(str(tmp_path / 'out_bias.npy'), out_bias)
    text = """
      name: "ae" model_type: FEED_FORWARD_NET prefix: "%s"
      hyperparams { activation: LOGISTIC }
      layer { name: "x" dimensions: 96 is_input: true }
      layer { name: "code" dimensions: 64
              param { name: "bias" initialization: PRETRAINED pretrained_model: "rbm_a.pbtxt" pretrained_model_node1: "hidden1" } }
      layer { name: "y" dimensions: 96 is_output: true
              param { name: "bias" initialization: PRETRAINED pretrained_model: "out_bias.npy" } }
      edge { node1: "x" node2: "code"
             param { name: "weight" initialization: PRETRAINED pretrained_model: "rbm_a.pbtxt" pretrained_model: "rbm_b.pbtxt"
                     pretrained_model_node1: "input_layer" pretrained_model_node2: "hidden1" } }
      edge { node1: "code" node2: "y"
             param { name: "weight" initialization: PRETRAINED pretrained_model: "rbm_a.pbtxt" transpose_pretrained: true
                     mult_factor: 0.5 pretrained_model_node1: "hidden1" pretrained_model_node2: "input_layer" } }
    """ % str(tmp_path)
    net = trainer.CreateDeepnet(text, batchsize=8)
    by_name = {l.name: l for l in net.layer}
    assert np.array_equal(by_name['code'].params['bias'].asarray(), bh)
    assert np.array_equal(by_name['y'].params['bias'].asarray(), out_bias.reshape(-1, 1))
    mean_w = ((w_a.astype(np.float64) + w_b) / 2).astype(np.float32)
    assert np.array_equal(net.edge[0].params['weight'].asarray(), mean_w)
    assert np.array_equal(net.edge[1].params['weight'].asarray(), (0.5 * w_a.astype(np.float64)).T.astype(np.float32))
    assert bv.shape == (96, 1)
    with pytest.raises(LookupError, match='No edge found'):
        trainer.CreateDeepnet(text.replace('pretrained_model_node2: "hidden1"', 'pretrained_model_node2: "nowhere"'), batchsize=8)
