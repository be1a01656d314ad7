"""Layers of units for feed-forward nets on the MI355X backend: the step-path part of the
reference's deepnet/layer.py and its activation subclasses (logistic_layer.py, tanh_layer.py,
relu_layer.py, linear_layer.py, softmax_layer.py, sin_layer.py, cos_layer.py) -- ``ApplyActivation``, ``ComputeDeriv``,
``Sample``, ``GetLoss``, ``GetData`` and the buffers of ``AllocateMemory`` -- issuing the same
matrix calls in the same order.  Configuration comes as plain arguments instead of protobuf
messages; tied layers, replicated softmax and display are not carried over.

States are (dimensions * numlabels, batchsize) matrices, one column per case.
"""
import types

import numpy as np

from .choose_matrix_library import cm
from . import parameter as P
from .parameter import Parameter, Hyperparams


def _zeros(shape):
    return cm.CUDAMatrix(np.zeros(shape, dtype=np.float32, order='F'))


def _metrics(count):
    """The fields of deepnet.proto's Metrics that the losses below fill."""
    return types.SimpleNamespace(count=count, cross_entropy=0.0, correct_preds=0.0, error=0.0)


class Layer(Parameter):
    """deepnet/layer.py:5-57 (construction) and :150-192 (buffers)."""

    activation = None

    def __init__(self, name, dimensions, batchsize, hyperparams=None, numlabels=1, is_input=False, is_output=False,
                 loss_function=P.SQUARED_LOSS, loss_weight=1.0, bias=None):
        super(Layer, self).__init__()
        self.name, self.dimensions, self.numlabels = name, dimensions, numlabels
        self.hyperparams = hyperparams or Hyperparams(activation=self.activation)
        self.is_input, self.is_output, self.is_initialized = is_input, is_output, False
        self.loss_function, self.loss_weight = loss_function, loss_weight
        self.incoming_edge, self.outgoing_edge = [], []
        self.incoming_neighbour, self.outgoing_neighbour = [], []
        self.replicated_neighbour = None
        self.tied_to = None
        self.tiny = 1e-10
        self.dirty = False
        self.data = None
        numdims = dimensions * numlabels
        self.params['bias'] = _zeros((numdims, 1)) if bias is None else cm.CUDAMatrix(
            np.asarray(bias, dtype=np.float32, order='F').reshape(numdims, 1))
        self.sample_input = self.hyperparams.sample_input
        self.AllocateMemory(batchsize)

    # ---- graph bookkeeping (layer.py:102-121)
    def AddIncomingEdge(self, edge):
        if edge not in self.incoming_edge:
            self.incoming_edge.append(edge)
            self.incoming_neighbour.append(edge.node2 if self is edge.node1 else edge.node1)

    def AddOutgoingEdge(self, edge):
        if edge not in self.outgoing_edge:
            self.outgoing_edge.append(edge)
            self.outgoing_neighbour.append(edge.node2 if self is edge.node1 else edge.node1)

    # ---- buffers
    def AllocateMemory(self, batchsize):
        self.AllocateBatchsizeDependentMemory(batchsize)
        numdims = self.dimensions * self.numlabels
        self.dimsize = _zeros((numdims, 1))
        if self.hyperparams.sparsity:
            self.means = cm.CUDAMatrix(np.full((numdims, 1), self.hyperparams.sparsity_target, dtype=np.float32, order='F'))
            self.sparsity_gradient = _zeros((numdims, 1))
            self.means_temp2 = _zeros((numdims, 1))
        self.gradient = _zeros((numdims, 1))
        self.gradient_history = _zeros((numdims, 1))

    def AllocateBatchsizeDependentMemory(self, batchsize):
        self.batchsize = batchsize
        numdims = self.dimensions * self.numlabels
        self.statesize = _zeros((numdims, batchsize))
        self.batchsize_temp = _zeros((1, batchsize))
        self.state = _zeros((numdims, batchsize))
        self.deriv = _zeros((numdims, batchsize))
        self.sample = _zeros((numdims, batchsize))
        if self.is_input or self.is_initialized or self.is_output:
            self.data = _zeros((self.dimensions, batchsize))
        if self.hyperparams.dropout:
            self.mask = _zeros(self.state.shape)

    def AllocateSamplingMemory(self, persistent):
        """What a layer of a Boltzmann machine holds besides its state (layer.py:176-186): the
        sufficient statistics, and with persistent chains separate positive / negative states and
        samples (``state`` / ``sample`` then point at the pair of the current phase)."""
        numdims = self.dimensions * self.numlabels
        self.suff_stats = cm.empty((numdims, 1))
        if persistent:
            self.pos_state, self.pos_sample = self.state, self.sample
            self.neg_state, self.neg_sample = _zeros(self.state.shape), _zeros(self.state.shape)

    def GetSparsityGradient(self):
        """layer.py:138-155: running mean activity of every unit (damped by sparsity_damping),
        and cost * (mean - target) / divisor as the extra gradient."""
        h = self.hyperparams
        self.means.mult(h.sparsity_damping)
        self.means.add_sums(self.state, axis=1, mult=(1 - h.sparsity_damping) / self.batchsize)
        self.means.subtract(h.sparsity_target, target=self.sparsity_gradient)
        self.sparsity_gradient.divide(self.GetSparsityDivisor())
        self.sparsity_gradient.mult(h.sparsity_cost)
        return self.sparsity_gradient

    def GetSparsityDivisor(self):
        """layer.py:256-258 (rectified linear units use it as it stands)."""
        self.means_temp2.assign(1)
        return self.means_temp2

    def CollectSufficientStatistics(self, neg=False):
        """layer.py:194-213: the row sums of the state, added with sign +1 in the positive and
        -1 in the negative phase; with a sparsity target the positive statistics are moved
        by -batchsize * sparsity gradient and the mean of the running means is returned."""
        h = self.hyperparams
        if not neg:
            self.state.sum(axis=1, target=self.suff_stats)
            if h.sparsity:
                self.suff_stats.add_mult(self.GetSparsityGradient(), -self.batchsize)
                return self.means.sum() / self.means.shape[0]
        else:
            self.suff_stats.add_sums(self.state, axis=1, mult=-1.0)
        return None

    def SetData(self, data):
        self.data = data

    def GetData(self):
        self.state.assign(self.data)

    def ResetState(self, rand=False):
        if rand:
            self.state.fill_with_randn()
            self.ApplyActivation()
        else:
            self.state.assign(0)

    # ---- what a subclass defines
    def ApplyActivation(self):
        pass

    def ComputeDeriv(self):
        pass

    def Sample(self):
        pass

    def GetLoss(self, get_deriv=False, **kwargs):
        pass

    def _squared_loss(self, perf, get_deriv, acc_deriv):
        """The SQUARED_LOSS branch shared by logistic and ReLU units (logistic_layer.py:50-60)."""
        target = self.statesize
        self.state.subtract(self.data, target=target)
        perf.error = target.euclid_norm() ** 2
        if acc_deriv:
            # (the reference passes the weight as `alpha=`, a keyword cudamat.py:1114 does not have)
            self.deriv.add_mult(target, mult=self.loss_weight)
        else:
            self.deriv.assign(target)
        if get_deriv:
            self.ComputeDeriv()


class LinearLayer(Layer):
    """deepnet/linear_layer.py (without a learnt precision)."""
    activation = P.LINEAR

    def GetSparsityDivisor(self):
        raise Exception('Sparsity not implemented for linear units.')

    def ComputeDeriv(self):
        if self.hyperparams.dropout:
            self.deriv.mult(self.mask)

    def GetLoss(self, get_deriv=False, **kwargs):
        perf = _metrics(self.batchsize)
        if self.loss_function != P.SQUARED_LOSS:
            raise Exception('Unknown loss function for linear units.')
        target = self.deriv if get_deriv else self.statesize
        self.state.subtract(self.data, target=target)
        perf.error = target.euclid_norm() ** 2
        if get_deriv:
            self.ComputeDeriv()
        return perf


class LogisticLayer(Layer):
    """deepnet/logistic_layer.py."""
    activation = P.LOGISTIC

    def ApplyActivation(self):
        cm.sigmoid(self.state)

    def Sample(self):
        self.state.sample_bernoulli(target=self.sample)

    def GetSparsityDivisor(self):
        """logistic_layer.py:64-68: mean * (1 - mean)."""
        self.means_temp2.assign(1)
        self.means_temp2.subtract(self.means)
        self.means_temp2.mult(self.means)
        return self.means_temp2

    def ComputeDeriv(self):
        self.deriv.apply_logistic_deriv(self.state)

    def GetLoss(self, get_deriv=False, acc_deriv=False, **kwargs):
        perf = _metrics(self.batchsize)
        if self.loss_function == P.CROSS_ENTROPY:
            temp1 = self.statesize
            cm.cross_entropy_bernoulli(self.data, self.state, target=temp1, tiny=self.tiny)
            perf.cross_entropy = temp1.sum()
            cm.correct_preds(self.data, self.state, target=temp1, cutoff=0.5)
            perf.correct_preds = temp1.sum()
            if get_deriv:
                self.state.subtract(self.data, target=self.deriv)
        elif self.loss_function == P.SQUARED_LOSS:
            self._squared_loss(perf, get_deriv, acc_deriv)
        else:
            raise Exception('Unknown loss function for logistic units.')
        return perf


class TanhLayer(Layer):
    """deepnet/tanh_layer.py."""
    activation = P.TANH

    def ApplyActivation(self):
        cm.tanh(self.state)

    def Sample(self):
        self.state.sample_bernoulli_tanh(target=self.sample)

    def GetSparsityDivisor(self):
        raise Exception('Sparsity not implemented for tanh units.')

    def ComputeDeriv(self):
        self.deriv.apply_tanh_deriv(self.state)
        if self.hyperparams.dropout:
            self.deriv.mult(self.mask)

    def GetLoss(self, get_deriv=False, **kwargs):
        perf = _metrics(self.batchsize)
        if self.loss_function != P.SQUARED_LOSS:
            raise Exception('Unknown loss function for tanh units.')
        self.state.subtract(self.data, target=self.deriv)
        perf.error = self.deriv.euclid_norm() ** 2
        if get_deriv:
            self.ComputeDeriv()
        return perf


class ReluLayer(Layer):
    """deepnet/relu_layer.py."""
    activation = P.RECTIFIED_LINEAR

    def ApplyActivation(self):
        self.state.lower_bound(0)

    def Sample(self):
        self.state.sample_gaussian(target=self.sample, mult=1.0)
        self.sample.lower_bound(0)

    def ComputeDeriv(self):
        self.deriv.apply_rectified_linear_deriv(self.state)

    def GetLoss(self, get_deriv=False, acc_deriv=False, **kwargs):
        perf = _metrics(self.batchsize)
        if self.loss_function != P.SQUARED_LOSS:
            raise Exception('Unknown loss function for ReLU units.')
        self._squared_loss(perf, get_deriv, acc_deriv)
        return perf


class SoftmaxLayer(Layer):
    """deepnet/softmax_layer.py: ``dimensions`` softmaxes of ``numlabels`` classes per case; the
    targets in ``data`` are class indices stored as floats."""
    activation = P.SOFTMAX

    def ApplyActivation(self):
        self.state.apply_softmax()

    def Sample(self):
        self.state.perturb_prob_for_softmax_sampling(target=self.sample)
        self.sample.choose_max(axis=0)

    def GetSparsityDivisor(self):
        raise Exception('Sparsity not implemented for softmax units.')

    def ComputeDeriv(self):
        raise Exception('Back prop through softmax not implemented.')

    def AllocateMemory(self, batchsize):
        super(SoftmaxLayer, self).AllocateMemory(batchsize)
        self.expansion_matrix = cm.CUDAMatrix(np.eye(self.numlabels, dtype=np.float32))

    def AllocateBatchsizeDependentMemory(self, batchsize):
        super(SoftmaxLayer, self).AllocateBatchsizeDependentMemory(batchsize)
        self.data = _zeros((self.dimensions, batchsize))
        self.batchsize_temp = _zeros((self.dimensions, batchsize))

    def GetData(self):
        self.expansion_matrix.select_columns(self.data, target=self.state)

    def GetLoss(self, get_deriv=False, **kwargs):
        perf = _metrics(self.batchsize)
        batchsize, dimensions, numlabels = self.batchsize, self.dimensions, self.numlabels
        state, data = self.state, self.data
        # one softmax per column while the loss kernels run
        state.reshape((numlabels, dimensions * batchsize))
        data.reshape((1, dimensions * batchsize))
        temp = self.batchsize_temp
        temp.reshape((1, dimensions * batchsize))
        self.deriv.reshape((numlabels, dimensions * batchsize))
        try:
            if self.loss_function == P.CROSS_ENTROPY:
                state.get_softmax_correct(data, target=temp)
                perf.correct_preds = temp.sum()
                state.get_softmax_cross_entropy(data, target=temp, tiny=self.tiny)
                perf.cross_entropy = temp.sum()
                if get_deriv:
                    state.apply_softmax_grad(data, target=self.deriv)
            elif self.loss_function == P.SQUARED_LOSS:
                state.apply_softmax_grad(data, target=self.deriv)
                perf.error = self.deriv.euclid_norm() ** 2
            else:
                raise Exception('Unknown loss function for Softmax units.')
        finally:
            state.reshape((numlabels * dimensions, batchsize))
            data.reshape((dimensions, batchsize))
            temp.reshape((dimensions, batchsize))
            self.deriv.reshape((numlabels * dimensions, batchsize))
        return perf


class SmoothReluLayer(ReluLayer):
    """deepnet/smooth_relu_layer.py: softplus units log(1 + exp(x)).  The derivative is taken from the
    output s as 1 - exp(-s), which equals sigmoid(x)."""
    activation = P.RECTIFIED_LINEAR_SMOOTH

    def ApplyActivation(self):
        cm.log_1_plus_exp(self.state)

    def ComputeDeriv(self):
        self.deriv.apply_rectified_linear_smooth_deriv(self.state)


class SinLayer(Layer):
    """deepnet/sin_layer.py: hidden units sin(x); the input is kept for the derivative."""
    activation = P.SIN

    def AllocateBatchsizeDependentMemory(self, batchsize):
        super(SinLayer, self).AllocateBatchsizeDependentMemory(batchsize)
        self.backup_state = _zeros(self.statesize.shape)

    def ApplyActivation(self):
        self.backup_state.assign(self.state)
        cm.sin(self.state)

    def ComputeDeriv(self):
        self.deriv.apply_sin_deriv(self.backup_state)


class CosLayer(SinLayer):
    """deepnet/cos_layer.py."""
    activation = P.COS

    def ApplyActivation(self):
        self.backup_state.assign(self.state)
        cm.cos(self.state)

    def ComputeDeriv(self):
        self.deriv.apply_cos_deriv(self.backup_state)


LAYER_TYPES = {cls.activation: cls for cls in (LinearLayer, LogisticLayer, TanhLayer, ReluLayer, SoftmaxLayer, SinLayer,
                                               CosLayer, SmoothReluLayer)}


def CreateLayer(activation, *args, **kwargs):
    """The layer class for an activation name (the role of deepnet/layer.py's IsLayerType dispatch)."""
    return LAYER_TYPES[activation](*args, **kwargs)
