"""Boltzmann machines trained by contrastive divergence on the MI355X backend: the step of
the reference's deepnet/dbm.py -- ``ComputeUp`` (:64-118), ``PositivePhase`` (:121-170),
``InitializeNegPhase`` (:172-184), ``NegativePhase`` (:186-244), ``UpdateLayerParams`` /
``UpdateEdgeParams`` (:246-266), ``TrainOneBatch`` / ``EvaluateOneBatch`` (:273-282) -- with CD
(one set of states, chains restarted at the data) and PCD (persistent negative states), over the
layers and edges of this package.  An RBM is the two-layer case: one input layer, one hidden
layer, one edge.  Initialiser nets and replicated softmax are not carried over.
"""
import types

from .choose_matrix_library import cm
from .neuralnet import NeuralNet, fused_up

CD, PCD = 'CD', 'PCD'


class DBM(NeuralNet):

    def __init__(self, layers, edges, optimizer=CD, mf_steps=1, gibbs_steps=1, start_step_up_cd_after=0,
                 step_up_cd_after=0, positive_phase_order=None, negative_phase_order=None, verbose=False):
        self.optimizer = optimizer
        self.cd = optimizer == CD
        self.mf_steps, self.gibbs_steps = mf_steps, gibbs_steps
        self.start_step_up_cd_after, self.step_up_cd_after = start_step_up_cd_after, step_up_cd_after
        self._pos_order, self._neg_order = positive_phase_order, negative_phase_order
        for layer in layers:
            layer.AllocateSamplingMemory(persistent=not self.cd)
        super(DBM, self).__init__(layers, edges, verbose=verbose)

    def SetPhase(self, layer, pos=True):
        """With persistent chains: point state / sample at the buffers of the phase."""
        if pos:
            layer.state, layer.sample = layer.pos_state, layer.pos_sample
        else:
            layer.state, layer.sample = layer.neg_state, layer.neg_sample

    def Sort(self):
        """Input layers first; the positive phase updates the others, the negative phase all."""
        non_input = [n for n in self.layer if not n.is_input]
        node_list = list(self.input_datalayer) + non_input
        self.pos_phase_order = list(self._pos_order) if self._pos_order else non_input
        self.neg_phase_order = list(self._neg_order) if self._neg_order else node_list
        return node_list

    def ComputeUp(self, layer, train=False, compute_input=False, step=0, maxsteps=0, use_samples=False,
                  neg_phase=False):
        """State of ``layer`` from all its neighbours (edges are undirected here: the weight is
        used transposed when the layer is the edge's second node), from their samples when
        ``use_samples``.  The input layer reads its data unless ``compute_input``."""
        if layer.is_input and not compute_input:
            layer.GetData()
        else:
            fused = False
            if len(layer.incoming_edge) == 1:
                edge, neighbour = layer.incoming_edge[0], layer.incoming_neighbour[0]
                up = edge.node2 is layer
                if (edge.proto.up_factor if up else edge.proto.down_factor) == 1:
                    w = edge.params['weight']
                    fused = fused_up(layer, w.T if up else w, neighbour.sample if use_samples else neighbour.state)
            for i, edge in enumerate([] if fused else layer.incoming_edge):
                neighbour = layer.incoming_neighbour[i]
                inputs = neighbour.sample if use_samples else neighbour.state
                if edge.node2 is layer:
                    w, factor = edge.params['weight'].T, edge.proto.up_factor
                else:
                    w, factor = edge.params['weight'], edge.proto.down_factor
                if i == 0:
                    cm.dot(w, inputs, target=layer.state)
                    if factor != 1:
                        layer.state.mult(factor)
                else:
                    layer.state.add_dot(w, inputs, mult=factor)
            if not fused:
                layer.state.add_col_vec(layer.params['bias'])
                layer.ApplyActivation()
        h = layer.hyperparams
        if h.dropout:
            if train and maxsteps - step >= h.stop_dropout_for_last:
                if not neg_phase:                      # the negative phase reuses the mask of the positive one
                    layer.mask.fill_with_rand()
                    layer.mask.greater_than(h.dropout_prob)
                layer.state.mult(layer.mask)
            else:
                layer.state.mult(1.0 - h.dropout_prob)

    def PositivePhase(self, train=False, evaluate=False, step=0):
        """Sufficient statistics under the data: clamp the inputs, mean-field updates of the rest."""
        for node in self.node_list:
            if node.is_input:
                self.ComputeUp(node, train=train)
            else:
                node.ResetState(rand=False)
        for _ in range(self.mf_steps):
            for node in self.pos_phase_order:
                self.ComputeUp(node, train=train, step=step, maxsteps=self.train_stop_steps)
        losses = []
        if train:
            for node in self.layer:
                r = node.CollectSufficientStatistics()
                if r is not None:           # a layer with a sparsity target reports its mean activity (dbm.py:147-153)
                    losses.append(types.SimpleNamespace(count=1, sparsity=r))
            for edge in self.edge:
                edge.CollectSufficientStatistics()
        # With CD the reconstruction error is measured by the negative phase.
        if not self.cd or evaluate:
            for node in self.input_datalayer:
                self.ComputeUp(node, compute_input=True, step=step, maxsteps=self.train_stop_steps)
                losses.append(node.GetLoss())
        return losses

    def InitializeNegPhase(self, to_pos=False):
        """Start the persistent chains: at the positive states, or at random states."""
        for layer in self.layer:
            self.SetPhase(layer, pos=False)
            if to_pos:
                layer.state.assign(layer.pos_state)
            else:
                layer.ResetState(rand=True)
            layer.Sample()
            self.SetPhase(layer, pos=True)

    def NegativePhase(self, step=0, train=True, gibbs_steps=-1):
        """Sufficient statistics under the model: Gibbs sweeps from the data (CD) or from the
        persistent chains (PCD), then the parameter updates."""
        losses = []
        if self.cd:
            for node in self.node_list:
                if not node.is_input:
                    node.Sample()
        else:
            for node in self.layer:
                self.SetPhase(node, pos=False)
        if gibbs_steps < 0:
            start_after = self.start_step_up_cd_after
            if start_after > 0 and start_after < step:
                gibbs_steps = self.gibbs_steps + 1 + (step - start_after) // self.step_up_cd_after
            else:
                gibbs_steps = self.gibbs_steps
        for i in range(gibbs_steps):
            for node in self.neg_phase_order:
                self.ComputeUp(node, train=train, step=step, maxsteps=self.train_stop_steps, use_samples=True,
                               compute_input=True, neg_phase=True)
                if i == 0 and node.is_input and self.cd:
                    losses.append(node.GetLoss())
                if node.is_input:
                    if node.sample_input and node.hyperparams.sample_input_after <= step:
                        node.Sample()
                    else:
                        node.sample.assign(node.state)     # (not sampling the inputs usually learns faster)
                else:
                    node.Sample()
        if train:
            for node in self.layer:
                node.CollectSufficientStatistics(neg=True)
                self.UpdateLayerParams(node, step=step)
            for edge in self.edge:
                edge.CollectSufficientStatistics(neg=True)
                self.UpdateEdgeParams(edge, step=step)
        if not self.cd:
            for node in self.layer:
                self.SetPhase(node, pos=True)
        return losses

    def UpdateLayerParams(self, layer, step=0):
        layer.gradient.add_mult(layer.suff_stats, -1.0 / layer.batchsize)
        layer.num_grads_received += 1
        if layer.num_grads_received == layer.num_shares:
            layer.Update('bias', step, no_reg=True)

    def UpdateEdgeParams(self, edge, step):
        numcases = edge.node1.batchsize
        edge.gradient.add_mult(edge.suff_stats, -1.0 / numcases)
        edge.num_grads_received += 1
        if edge.num_grads_received == edge.num_shares:
            edge.Update('weight', step)

    def TrainOneBatch(self, step):
        losses = self.PositivePhase(train=True, step=step)
        if step == 0 and self.optimizer == PCD:
            self.InitializeNegPhase(to_pos=True)
        losses.extend(self.NegativePhase(step, train=True))
        return losses

    def EvaluateOneBatch(self):
        return self.PositivePhase(train=False, evaluate=True)
