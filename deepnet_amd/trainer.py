"""Build a net on the device from deepnet's own model files.

``CreateDeepnet(model, train_op, eval_op)`` has the role of deepnet/trainer.py:34-46 followed
by ``LoadModelOnGPU`` (deepnet/neuralnet.py:70-109): the model-wide hyper-parameters are merged
under those of every layer and edge, parameters are initialised as deepnet/parameter.py:43-71
does (same numpy generator, seeded with the model's seed, same order: layers, then edges, as
listed), layers and edges are created and sorted.  ``model`` / ``train_op`` are the parsed
text files (``util.ReadModel`` / ``util.ReadOperation``), paths to them, or their text.
A field that would change the arithmetic of a step and has no counterpart here (tied
parameters, replicated softmax, adaptive learning rates, ...) raises
NotImplementedError by name instead of being dropped.
"""
import os

import numpy as np

from . import pbtxt
from .choose_matrix_library import cm
from .convolutions import ConvParams
from .layer import LAYER_TYPES
from .neuralnet import Edge, NeuralNet
from .parameter import Hyperparams

# Hyperparams fields that switch on behaviour this package does not have: refused when set.
# shared_prior / soft_shared_prior select other edge classes (transfer_edge.py:6, soft_transfer_edge.py:6);
# add_noise / shift / the windows are instructions to the data handler (datahandler.py:505-535), which the
# caller builds here.  The remaining unknown fields are read only by replicated-softmax layers
# (normalize, the priors) and fast-dropout nets, refused by activation / model type, or by nothing
# (decay_learning_rate_for_last), or concern display and model selection.  adapt other than NO_ADAPT
# raises 'Not implemented.' in the reference too (parameter.py:89-96); learn_precision selects the
# precision parameters of Gaussian units, which are not carried over.
_SWITCHES = ('shared_prior', 'soft_shared_prior', 'add_noise', 'shift', 'left_window', 'right_window', 'adapt',
             'learn_precision')
_OFF = (False, 0, 0.0, 'NO_ADAPT', None)

_CONV_FIELDS = ('size', 'stride', 'padding', 'num_filters', 'num_colors', 'max_pool', 'pool_size', 'pool_stride',
                'rnorm', 'norm_size', 'pow_scale', 'add_scale', 'prob')


def _as_message(x):
    if x is None or isinstance(x, pbtxt.Message):
        return x
    if isinstance(x, str) and '\n' not in x and (os.path.exists(x) or x.endswith('.pbtxt')):
        with open(x) as f:              # (a missing .pbtxt path raises FileNotFoundError, not a parse error)
            return pbtxt.parse(f.read())
    return pbtxt.parse(x)


def _hyperparams(model_hyp, own_hyp, where):
    """deepnet/neuralnet.py:80-93: the model's fields, overwritten by the fields written for
    this layer / edge; everything else at the defaults of the message."""
    fields = pbtxt.merged(model_hyp, own_hyp).scalars()
    for name in _SWITCHES:
        if fields.get(name) not in _OFF:
            raise NotImplementedError('%s: hyperparams.%s = %r is not supported' % (where, name, fields[name]))
    known = {k: v for k, v in fields.items() if k in Hyperparams._DEFAULTS}
    return Hyperparams(**known)


def _pretrained_array(param, model_file, find):
    """One file named by ``pretrained_model``: an .npy array, or a model file in which
    ``find(model)`` picks the layer / edge whose parameter of the same name is taken."""
    ext = os.path.splitext(model_file)[1]
    if ext == '.npy':
        return np.load(model_file), None
    if ext == '.npz':
        stats = np.load(model_file)
        if param.name != 'bias':
            raise NotImplementedError('parameter %s from an .npz file is not supported' % param.name)
        return np.nan_to_num(stats['mean'] / stats['std']), None
    from .util import ReadModel
    holder = find(ReadModel(model_file))
    stored = next(p for p in holder.all('param') if p.name == param.name)
    assert 'mat' in stored and stored.mat != '', 'Pretrained param %s of model %s is empty!!' % (stored.name, model_file)
    return _stored(stored, stored.all('dimensions')), stored.all('dimensions')


def LoadPretrained(param, dims, prefix, names):
    """deepnet/layer.py:66-98 (``names`` = (layer name,)) and deepnet/edge.py:165-215 (``names`` =
    (node1, node2)): the mean over the files listed in ``pretrained_model`` of the parameter of the
    same name found there, for edges times ``mult_factor`` and transposed when
    ``transpose_pretrained``."""
    files = param.all('pretrained_model')
    assert files, 'parameter %s: PRETRAINED without pretrained_model' % param.name
    transpose = param.get('transpose_pretrained', False)
    if len(names) == 1:
        want = (param.get('pretrained_model_node1', '') or names[0],)
        find = lambda model: next(n for n in model.all('layer') if n.name == want[0])
    else:
        want = (param.get('pretrained_model_node1', '') or names[0], param.get('pretrained_model_node2', '') or names[1])
        if transpose:
            want = want[::-1]

        def find(model):
            try:
                return next(e for e in model.all('edge') if (e.node1, e.node2) == want)
            except StopIteration:
                raise LookupError('No edge found between %s and %s.' % want)
    total = None
    for name in files:
        this_mat, stored_dims = _pretrained_array(param, os.path.join(prefix, name), find)
        if len(names) == 2:
            if stored_dims is not None:
                expect = list(stored_dims)[::-1] if transpose else list(stored_dims)
                assert list(dims) == expect, 'Param has shape %s but pretrained param has shape %s' % (list(dims), expect)
                this_mat = param.get('mult_factor', 1.0) * this_mat
            if transpose:
                this_mat = this_mat.T
        elif this_mat.ndim == 1:
            this_mat = this_mat.reshape(-1, 1)
        total = this_mat if total is None else total + this_mat
    return total / len(files)


def InitializeParameter(param, dims, prefix='', names=()):
    """deepnet/parameter.py:43-71 on the numpy global generator (seeded by the caller)."""
    kind = param.get('initialization', 'CONSTANT')
    sigma = param.get('sigma', 0.001)
    if kind == 'CONSTANT':
        return np.zeros(tuple(dims)) + param.get('constant', 0.0)
    if kind == 'DENSE_GAUSSIAN':
        return sigma * np.random.randn(*dims)
    if kind == 'DENSE_UNIFORM':
        return sigma * (2 * np.random.rand(*dims) - 1)
    if kind in ('DENSE_GAUSSIAN_SQRT_FAN_IN', 'DENSE_UNIFORM_SQRT_FAN_IN'):
        assert len(dims) > 1
        # (the reference takes dimensions[0], the filter count, as the fan-in of conv / local weights)
        fan_in = dims[0] if (param.get('conv', False) or param.get('local', False)) else dims[1]
        stddev = sigma / np.sqrt(fan_in)
        if kind == 'DENSE_GAUSSIAN_SQRT_FAN_IN':
            return stddev * np.random.randn(*dims)
        return stddev * (2 * np.random.rand(*dims) - 1)
    if kind == 'PRETRAINED':
        return LoadPretrained(param, dims, prefix, names)
    raise Exception('Unknown parameter initialization.')


def _stored(param, dims):
    """The array a parameter message carries in ``mat`` (deepnet/util.py:13-15: row-major float32)."""
    raw = param.mat
    raw = raw.encode('latin-1') if isinstance(raw, str) else raw
    a = np.frombuffer(raw, dtype=np.float32)
    if a.size != int(np.prod(dims)):
        raise ValueError('parameter %s: %d stored values for dimensions %s' % (param.get('name'), a.size, list(dims)))
    return a.reshape(tuple(dims)).copy()


def _refuse(msg, fields, where):
    for name in fields:
        if msg.get(name) not in _OFF and msg.get(name) != '':
            raise NotImplementedError('%s: %s is not supported' % (where, name))


def _layer(proto, model_hyp, batchsize, prefix=''):
    name = proto.name
    prefix = proto.get('prefix', '') or prefix
    _refuse(proto, ('tied', 'is_initialized'), 'layer ' + name)
    hyp = _hyperparams(model_hyp, proto.get('hyperparams'), 'layer ' + name)
    if hyp.activation not in LAYER_TYPES:
        raise NotImplementedError('layer %s: activation %s is not supported' % (name, hyp.activation))
    dims, numlabels = proto.dimensions, proto.get('numlabels', 1)
    bias = None
    for param in proto.all('param'):
        if param.name != 'bias':
            raise NotImplementedError('layer %s: parameter %s is not supported' % (name, param.name))
        pdims = param.all('dimensions') or [numlabels * dims, 1]
        if len(pdims) == 1:
            pdims = pdims + [1]
        # stored values win over the initialisation rule (parameter.py:36-39)
        bias = _stored(param, pdims) if 'mat' in param else InitializeParameter(param, pdims, prefix, (name,))
    return LAYER_TYPES[hyp.activation](
        name, dims, batchsize, hyperparams=hyp, numlabels=numlabels, is_input=proto.get('is_input', False),
        is_output=proto.get('is_output', False), loss_function=proto.get('loss_function', 'SQUARED_LOSS'),
        loss_weight=proto.get('loss_weight', 1.0), bias=bias)


def _edge(proto, model_hyp, layers, prefix=''):
    where = 'edge %s:%s' % (proto.node1, proto.node2)
    prefix = proto.get('prefix', '') or prefix
    _refuse(proto, ('tied', 'tied_transpose'), where)
    hyp = _hyperparams(model_hyp, proto.get('hyperparams'), where)
    by_name = {l.name: l for l in layers}
    node1, node2 = by_name[proto.node1], by_name[proto.node2]
    params = proto.all('param')
    if len(params) != 1 or params[0].name != 'weight':
        raise NotImplementedError('%s: exactly one parameter, "weight", is supported' % where)
    param = params[0]
    conv, local = param.get('conv', False), param.get('local', False)
    cv = None
    if conv or local:
        cvm = param.get('conv_params') or pbtxt.Message()
        cv = ConvParams(**{k: cvm.get(k) for k in _CONV_FIELDS if k in cvm})
    dims = param.all('dimensions')
    if not dims:
        if conv:
            dims = [cv.num_filters, cv.size ** 2 * cv.num_colors]
        elif local:
            side = int(round((node1.dimensions * node1.numlabels // cv.num_colors) ** 0.5))
            n_locs = (side + 2 * cv.padding - cv.size) // cv.stride + 1
            dims = [cv.num_filters, n_locs ** 2 * cv.size ** 2 * cv.num_colors]
        else:
            dims = [node1.numlabels * node1.dimensions, node2.numlabels * node2.dimensions]
    weight = _stored(param, dims) if 'mat' in param else InitializeParameter(param, dims, prefix, (proto.node1, proto.node2))
    return Edge(node1, node2, weight, hyperparams=hyp, conv_params=cv, local=bool(local),
                up_factor=proto.get('up_factor', 1.0), block_gradient=proto.get('block_gradient', False),
                down_factor=proto.get('down_factor', 1.0), directed=proto.get('directed', True))


def CreateDeepnet(model, train_op=None, eval_op=None, batchsize=None):
    """A NeuralNet (FEED_FORWARD_NET) with its parameters on the device; Boltzmann machines and
    belief nets (model_type DBM / DBN) are refused by name."""
    model, train_op, eval_op = _as_message(model), _as_message(train_op), _as_message(eval_op)
    op = train_op or eval_op
    if batchsize is None:
        if op is None:
            raise ValueError('a batch size or an operation that names one is needed')
        batchsize = op.get('batchsize', 1)
    seed = model.get('seed', 0)
    cm.CUDAMatrix.init_random(seed)          # deepnet/neuralnet.py:43-44
    np.random.seed(seed)
    model_hyp = model.get('hyperparams')
    prefix = model.get('prefix', '')
    layers = [_layer(p, model_hyp, batchsize, prefix) for p in model.all('layer')]
    edges = [_edge(p, model_hyp, layers, prefix) for p in model.all('edge')]
    by_name = {l.name: l for l in layers}
    kind = model.model_type
    if kind == 'FEED_FORWARD_NET':
        net = NeuralNet(layers, edges, verbose=bool(op and op.get('verbose', False)))
    else:
        raise NotImplementedError('model_type %s is not supported' % kind)
    net.net, net.t_op, net.e_op, net.batchsize = model, train_op, eval_op, batchsize
    if train_op and 'stopcondition' in train_op and train_op.stopcondition.get('steps', 0) > 0:
        net.train_stop_steps = train_op.stopcondition.steps
    return net


def ModelWithParameters(net):
    """The net's model message with the current device parameters stored in it (``dimensions``
    and ``mat`` of every parameter, as deepnet/parameter.py:17-19 stores them before a
    checkpoint is written): ``util.WritePbtxt(path, ModelWithParameters(net))`` writes a model
    file that ``CreateDeepnet`` loads back with the same parameters."""
    model = pbtxt.parse(pbtxt.dumps(net.net))            # a deep copy
    by_layer = {l.name: l for l in net.layer}
    by_edge = {(e.node1.name, e.node2.name): e for e in net.edge}
    for proto in model.all('layer'):
        for param in proto.all('param'):
            arr = by_layer[proto.name].params[param.name].asarray()
            param.set('dimensions', *arr.shape)
            param.set('mat', np.ascontiguousarray(arr, dtype=np.float32).tobytes())
    for proto in model.all('edge'):
        for param in proto.all('param'):
            arr = by_edge[(proto.node1, proto.node2)].params[param.name].asarray()
            param.set('dimensions', *arr.shape)
            param.set('mat', np.ascontiguousarray(arr, dtype=np.float32).tobytes())
    return model
