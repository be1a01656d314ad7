"""Hyper-parameters and the parameter update of deepnet on the MI355X backend.

``Parameter.Update`` is the rule of the reference's deepnet/parameter.py:80-106 (momentum,
optional L2 / L1 decay, gradient step, optional column-norm limit, gradient reset) and
``GetMomentumAndEpsilon`` its schedule (:108-126), as the same sequence of matrix calls.
With ``fused=True`` the sequence runs as the backend's one-pass ``momentum_update``, which
leaves the same bits.  ``Hyperparams`` carries the fields of the protobuf message
(deepnet/protos/deepnet.proto:89-175) that the step path reads, with the proto's defaults,
for callers that have no protobuf classes.
"""
import math

from .choose_matrix_library import cm

# Hyperparams.Decay / Hyperparams.Activation / Layer.LossFunction values, by the proto's names
NONE, INVERSE_T, EXPONENTIAL = 'NONE', 'INVERSE_T', 'EXPONENTIAL'
LINEAR, LOGISTIC, TANH, RECTIFIED_LINEAR, SOFTMAX = 'LINEAR', 'LOGISTIC', 'TANH', 'RECTIFIED_LINEAR', 'SOFTMAX'
SIN, COS = 'SIN', 'COS'
RECTIFIED_LINEAR_SMOOTH = 'RECTIFIED_LINEAR_SMOOTH'
SQUARED_LOSS, CROSS_ENTROPY = 'SQUARED_LOSS', 'CROSS_ENTROPY'


class Hyperparams(object):
    _DEFAULTS = dict(
        base_epsilon=0.01, epsilon_decay=NONE, epsilon_decay_half_life=1000, initial_momentum=0.0,
        final_momentum=0.0, momentum_change_steps=10, dropout=False, dropout_prob=0.5, apply_weight_norm=False,
        weight_norm=10.0, apply_l2_decay=False, l2_decay=0.01, activation=LINEAR, stop_dropout_for_last=0,
        start_learning_after=0, apply_l1_decay=False, l1_decay=0.01, apply_l1decay_after=0, blocksize=1,
        mult_dropout=False, sparsity=False, mf_steps=1, gibbs_steps=1, step_up_cd_after=0, start_step_up_cd_after=0,
        sample_input=False, sample_input_after=0, sparsity_target=0.1, sparsity_cost=0.001, sparsity_damping=0.9)

    def __init__(self, **fields):
        unknown = set(fields) - set(self._DEFAULTS)
        if unknown:
            raise TypeError('not a field of the step path: %s' % ', '.join(sorted(unknown)))
        self.__dict__.update(self._DEFAULTS)
        self.__dict__.update(fields)


class Parameter(object):
    """Base of layers and edges: ``params`` (name -> CUDAMatrix), ``gradient`` (accumulated by
    the backward pass), ``gradient_history`` (the previous update) and ``hyperparams``."""

    fused = False      # True: one momentum_update call instead of the 3-6 calls of the reference

    def __init__(self):
        self.num_shares = 1
        self.num_grads_received = 0
        self.params = {}

    def ApplyL2Decay(self, w_delta, w, lambdaa, **kwargs):
        w_delta.add_mult(w, lambdaa)

    def GetMomentumAndEpsilon(self, step):
        h = self.hyperparams
        momentum = h.final_momentum - (h.final_momentum - h.initial_momentum) * math.exp(
            -float(step) / h.momentum_change_steps)
        epsilon = h.base_epsilon
        if h.epsilon_decay == INVERSE_T:
            epsilon = h.base_epsilon / (1 + float(step) / h.epsilon_decay_half_life)
        elif h.epsilon_decay == EXPONENTIAL:
            epsilon = h.base_epsilon / math.pow(2, float(step) / h.epsilon_decay_half_life)
        if step < h.start_learning_after:
            epsilon = 0.0
        return momentum, epsilon

    def Update(self, param_name, step, no_reg=False):
        h = self.hyperparams
        momentum, epsilon = self.GetMomentumAndEpsilon(step)
        w, w_delta, gradient = self.params[param_name], self.gradient_history, self.gradient
        l2 = h.l2_decay if (not no_reg and h.apply_l2_decay) else None
        l1 = h.l1_decay if (not no_reg and h.apply_l1_decay and step > h.apply_l1decay_after) else None
        fused = self.fused and type(self).ApplyL2Decay is Parameter.ApplyL2Decay
        if fused:
            cm.momentum_update(w, w_delta, gradient, momentum, epsilon, l2_decay=l2, l1_decay=l1, reset_gradient=True)
        else:
            w_delta.mult(momentum)
            if l2 is not None:
                self.ApplyL2Decay(w_delta, w, l2, step=step, eps=epsilon, mom=momentum)
            if l1 is not None:
                w_delta.add_mult_sign(w, l1)
            w_delta.add_mult(gradient)
            w.add_mult(w_delta, -epsilon)
        if not no_reg and h.apply_weight_norm:
            w.norm_limit(h.weight_norm, axis=0)
        self.num_grads_received = 0
        if not fused:
            gradient.assign(0)
