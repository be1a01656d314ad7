"""Feed-forward nets trained by back-propagation on the MI355X backend: the training-step
core of the reference's deepnet/neuralnet.py -- ``ComputeUp`` (:138-207), ``ComputeDown``
(:209-235), ``AccumulateDeriv`` (:237-255), ``UpdateEdgeParams`` (:257-275),
``UpdateLayerParams`` (:277-290), ``ForwardPropagate`` / ``BackwardPropagate`` /
``TrainOneBatch`` / ``EvaluateOneBatch`` (:292-337) -- and the part of deepnet/edge.py a
training step touches, issuing the same matrix and conv calls in the same order.

A net is built from Layer objects and Edge objects (dense or conv / locally connected)
instead of a protobuf model; data handlers, model files, evaluation loops over data sets,
tied parameters and replicated-softmax neighbours stay outside.
"""
import sys
import types

import numpy as np

from .choose_matrix_library import cm
from .convolutions import ConvolveUp, AccumulateConvDeriv, ConvOuter, AddConvolveUp, ConvEdge
from . import parameter as P
from .parameter import Parameter, Hyperparams


class Edge(Parameter):
    """A weight matrix between two layers (deepnet/edge.py:8-35, 83-92).  Dense: ``weight`` is
    (node1 dims, node2 dims).  With ``conv_params``: (num_filters, colours * size^2) shared
    filters, or one bank per module when ``local``; the conv buffers are those of ConvEdge.
    ``directed=False`` makes the edge incoming and outgoing at both ends."""

    def __init__(self, node1, node2, weight, hyperparams=None, conv_params=None, local=False, up_factor=1.0,
                 block_gradient=False, down_factor=1.0, directed=True):
        super(Edge, self).__init__()
        self.node1, self.node2 = node1, node2
        self.name = '%s:%s' % (node1.name, node2.name)
        self.hyperparams = hyperparams or Hyperparams()
        self.proto = _EdgeProto(up_factor, block_gradient, down_factor)
        self.tied_to = None
        self.marker = 0
        self.conv = conv_params is not None and not local
        self.local = conv_params is not None and local
        w = cm.CUDAMatrix(np.asarray(weight, dtype=np.float32, order='F'))
        self.params['weight'] = w
        if conv_params is not None:
            self.conv_params = conv_params
            buffers = ConvEdge(w, conv_params, node1.state.shape, node2.state.shape, conv=not local)
            for name in ('input_t', 'input_t2', 'output_t', 'output_t2', 'unpooled_layer', 'rnd',
                         'unrnormalized_layer', 'denoms', 'rnorm_temp1', 'rnorm_temp2'):
                if hasattr(buffers, name):
                    setattr(self, name, getattr(buffers, name))
        else:
            assert w.shape == (node1.state.shape[0], node2.state.shape[0])
        self.AllocateMemory()
        node1.AddOutgoingEdge(self)
        node2.AddIncomingEdge(self)
        if not directed:              # Boltzmann machines: either end is computed from the other (edge.py:30-38)
            node1.AddIncomingEdge(self)
            node2.AddOutgoingEdge(self)

    def AllocateMemory(self):
        shape = self.params['weight'].shape
        zeros = lambda: cm.CUDAMatrix(np.zeros(shape, dtype=np.float32, order='F'))
        self.temp, self.gradient, self.gradient_history = zeros(), zeros(), zeros()

    def CollectSufficientStatistics(self, neg=False):
        """edge.py:222-242 for ordinary units: node1.state node2.state^T, set in the positive
        phase and subtracted in the negative one."""
        if not hasattr(self, 'suff_stats'):
            self.suff_stats = cm.empty(self.params['weight'].shape)
        if not neg:
            # with sparsity targets the statistics are taken of state - sparsity gradient (:230-240)
            sparse = [n for n in (self.node1, self.node2) if n.hyperparams.sparsity]
            for n in sparse:
                n.state.add_col_mult(n.sparsity_gradient, -1)
            cm.dot(self.node1.state, self.node2.state.T, target=self.suff_stats)
            for n in sparse:
                n.state.add_col_vec(n.sparsity_gradient)
        else:
            self.suff_stats.add_dot(self.node1.state, self.node2.state.T, mult=-1.0)


# Activations the backend's dot_bias_act can apply in the product's epilogue (None: bias only).
_EPILOGUE = {P.LINEAR: None, P.LOGISTIC: 'sigmoid', P.RECTIFIED_LINEAR: 'relu', P.TANH: 'tanh', P.SOFTMAX: None}


def fused_up(layer, w, inputs):
    """state = activation(w . inputs + bias) in one launch where the layer asks for it
    (``layer.fused``) and its activation has an epilogue; the same bits as dot, add_col_vec,
    ApplyActivation.  Returns False when the three calls have to be made."""
    if not layer.fused or layer.activation not in _EPILOGUE or layer.replicated_neighbour is not None:
        return False
    cm.dot_bias_act(w, inputs, layer.params['bias'], target=layer.state, act=_EPILOGUE[layer.activation])
    if layer.activation == P.SOFTMAX:
        layer.ApplyActivation()
    return True


class _EdgeProto(object):
    def __init__(self, up_factor, block_gradient, down_factor=1.0):
        self.up_factor, self.block_gradient, self.down_factor = up_factor, block_gradient, down_factor


class NeuralNet(object):

    def __init__(self, layers, edges, verbose=False):
        self.layer, self.edge, self.verbose = list(layers), list(edges), verbose
        self.input_datalayer = [n for n in self.layer if n.is_input]
        self.output_datalayer = [n for n in self.layer if n.is_output]
        self.train_stop_steps = sys.maxsize
        self.batchsize = self.layer[0].batchsize if self.layer else 0
        self.node_list = self.Sort()

    def Sort(self):
        """Layers in an order in which every layer comes after all layers feeding it."""
        for e in self.edge:
            e.marker = 0
        order, ready = [], [n for n in self.layer if not n.incoming_neighbour]
        while ready:
            n = ready.pop()
            order.append(n)
            for e in n.outgoing_edge:
                if e.marker == 0:
                    e.marker = 1
                    if all(x.marker == 1 for x in e.node2.incoming_edge):
                        ready.append(e.node2)
        if not all(e.marker == 1 for e in self.edge):
            raise Exception('Invalid net for backprop. Cycle exists.')
        return order

    def ComputeUp(self, layer, train=False, step=0, maxsteps=0):
        """State of ``layer`` from the states of the layers feeding it; then dropout."""
        layer.dirty = False
        perf = None
        if layer.is_input or layer.is_initialized:
            layer.GetData()
        else:
            only = layer.incoming_edge[0] if len(layer.incoming_edge) == 1 else None
            done = (only is not None and not (only.conv or only.local) and only not in layer.outgoing_edge
                    and only.proto.up_factor == 1
                    and fused_up(layer, only.params['weight'].T, layer.incoming_neighbour[0].state))
            if not done:
                for i, edge in enumerate(layer.incoming_edge):
                    if edge in layer.outgoing_edge:
                        continue
                    inputs = layer.incoming_neighbour[i].state
                    if edge.conv or edge.local:
                        if i == 0:
                            ConvolveUp(inputs, edge, layer.state)
                        else:
                            AddConvolveUp(inputs, edge, layer.state)
                    else:
                        w = edge.params['weight']
                        factor = edge.proto.up_factor
                        if i == 0:
                            cm.dot(w.T, inputs, target=layer.state)
                            if factor != 1:
                                layer.state.mult(factor)
                        else:
                            layer.state.add_dot(w.T, inputs, mult=factor)
                layer.state.add_col_vec(layer.params['bias'])
                layer.ApplyActivation()
            if layer.hyperparams.sparsity:          # neuralnet.py:176-181: the mean activity, reported as a loss record
                layer.state.sum(axis=1, target=layer.dimsize)
                perf = types.SimpleNamespace(count=layer.batchsize,
                                             sparsity=layer.dimsize.sum() / layer.dimsize.shape[0])
        h = layer.hyperparams
        if h.dropout:
            if train and maxsteps - step >= h.stop_dropout_for_last:
                if h.mult_dropout:
                    layer.mask.fill_with_randn()
                    layer.mask.add(1)
                    layer.state.mult(layer.mask)
                else:
                    layer.mask.fill_with_rand()
                    layer.mask.greater_than(h.dropout_prob)
                    if h.blocksize > 1:
                        layer.mask.blockify(h.blocksize)
                    layer.state.mult(layer.mask)
            elif not h.mult_dropout:
                layer.state.mult(1.0 - h.dropout_prob)      # the expected output
        return perf

    def ComputeDown(self, layer, step):
        """Back-propagate through ``layer``: its deriv holds the gradient w.r.t. its outputs on
        entry and w.r.t. its inputs afterwards; send it down every incoming edge and update the
        parameters of those edges and of the layer."""
        if layer.is_input:
            return None
        if layer.is_output:
            loss = layer.GetLoss(get_deriv=True)
        else:
            loss = None
            if layer.hyperparams.sparsity:          # neuralnet.py:221-223
                layer.deriv.add_col_vec(layer.GetSparsityGradient())
            layer.ComputeDeriv()
        for edge in layer.incoming_edge:
            if edge.conv or edge.local:
                AccumulateConvDeriv(edge.node1, edge, layer.deriv)
            else:
                self.AccumulateDeriv(edge.node1, edge, layer.deriv)
            self.UpdateEdgeParams(edge, layer.deriv, step)
        self.UpdateLayerParams(layer, step)
        return loss

    def AccumulateDeriv(self, layer, edge, deriv):
        if layer.is_input or edge.proto.block_gradient:
            return
        if layer.dirty:
            layer.deriv.add_dot(edge.params['weight'], deriv)
        else:
            cm.dot(edge.params['weight'], deriv, target=layer.deriv)
            layer.dirty = True

    def UpdateEdgeParams(self, edge, deriv, step):
        numcases = edge.node1.batchsize
        if edge.conv or edge.local:
            ConvOuter(edge, edge.temp)
            edge.gradient.add_mult(edge.temp, mult=1.0 / numcases)
        else:
            edge.gradient.add_dot(edge.node1.state, deriv.T, mult=1.0 / numcases)
        edge.num_grads_received += 1
        if edge.num_grads_received == edge.num_shares:
            edge.Update('weight', step)

    def UpdateLayerParams(self, layer, step):
        layer.gradient.add_sums(layer.deriv, axis=1, mult=1.0 / layer.batchsize)
        layer.num_grads_received += 1
        if layer.num_grads_received == layer.num_shares:
            layer.Update('bias', step, no_reg=True)     # the bias is not regularised

    def ForwardPropagate(self, train=False, step=0):
        losses = []
        for node in self.node_list:
            loss = self.ComputeUp(node, train, step, self.train_stop_steps)
            if loss:
                losses.append(loss)
        return losses

    def BackwardPropagate(self, step):
        losses = []
        for node in reversed(self.node_list):
            loss = self.ComputeDown(node, step)
            if loss:
                losses.append(loss)
        return losses

    def TrainOneBatch(self, step):
        losses = self.ForwardPropagate(train=True)
        losses.extend(self.BackwardPropagate(step))
        return losses

    def EvaluateOneBatch(self):
        losses = self.ForwardPropagate()
        losses.extend([node.GetLoss() for node in self.output_datalayer])
        return losses

    # ---- the loop around the step (neuralnet.py:340-392, 510-530, 589-670)
    @property
    def datalayer(self):
        """Layers that read a data stream, in the order listed: stream i of a handler feeds datalayer[i]."""
        return [n for n in self.layer if n.is_input or n.is_output]

    def GetBatch(self, handler):
        """neuralnet.py:510-516: the next batch of every stream becomes the data of its layer
        (views into the handler's device-resident chunk, no copy)."""
        data_list = handler.Get(self.batchsize)
        layers = self.datalayer
        assert len(data_list) == len(layers), '%d streams for %d data layers' % (len(data_list), len(layers))
        for layer, data in zip(layers, data_list):
            assert data.shape[1] == layer.batchsize, 'batch of %d for layers of %d' % (data.shape[1], layer.batchsize)
            layer.SetData(data)

    def Evaluate(self, handler, steps):
        """``steps`` batches through EvaluateOneBatch, losses accumulated (neuralnet.py:340-392
        without collecting predictions)."""
        stats = []
        for _ in range(steps):
            self.GetBatch(handler)
            stats = Accumulate(stats, self.EvaluateOneBatch())
        return stats

    def Train(self, train_handler, steps=None, eval_handler=None, eval_steps=1, eval_after=0, start_step=0,
              report=None):
        """The training loop of neuralnet.py:589-670 without checkpoints, display and model
        selection: fetch a batch, TrainOneBatch, accumulate the losses; every ``eval_after``
        steps evaluate on ``eval_handler`` and start the accumulators afresh.  Returns the
        list of {'step', 'train', 'eval'} records (also handed to ``report`` as they are made);
        without ``eval_after`` one record at the end."""
        stop = self.train_stop_steps if steps is None else steps
        stats, history = [], []
        step = start_step
        while step < stop:
            self.GetBatch(train_handler)
            stats = Accumulate(stats, self.TrainOneBatch(step))
            step += 1
            if (eval_after and step % eval_after == 0) or step == stop:
                record = {'step': step, 'train': stats,
                          'eval': self.Evaluate(eval_handler, eval_steps) if eval_handler is not None else None}
                history.append(record)
                if report is not None:
                    report(record)
                stats = []
        return history


def Accumulate(stats, losses):
    """deepnet/util.py:137-142 over whatever counters the losses carry (count, cross_entropy,
    error, correct_preds, sparsity): the first batch starts the accumulators."""
    if not stats:
        return [types.SimpleNamespace(**vars(l)) for l in losses]
    for acc, loss in zip(stats, losses):
        for key, value in vars(loss).items():
            setattr(acc, key, getattr(acc, key, 0) + value)
    return stats
