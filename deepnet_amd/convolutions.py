"""The conv stage of a deepnet edge on the MI355X backend: the three functions of the
reference's deepnet/convolutions.py (ConvolveUp :5-67, AccumulateConvDeriv :69-146,
ConvOuter :148-184) with the same names, arguments and buffer usage, plus the buffer
allocation an edge does for them (deepnet/edge.py:94-142).

deepnet keeps layer states as (dims, batch); the conv library wants (batch, dims) with
the batch fastest, so a stage is: transpose in, convUp / localUp, optional max pooling,
optional response normalisation, transpose out.  The backward pass walks the same
buffers in reverse and deliberately reuses them the way the reference does:

  * MaxPoolUndo writes the un-pooled gradient over ``edge.unpooled_layer``, the very
    buffer it reads the un-pooled activations from (in place; convolutions.py:127-135);
    ConvOuter later reads the gradient from there (:166-167).
  * ResponseNormUndo is handed the *normalised* outputs as its ``inputs`` operand and a
    copy of the un-normalised layer as ``acts`` (convolutions.py:111-122).  That is the
    reverse of what the formula behind the library call expects, so with ``rnorm`` the
    reference back-propagates  y_k * sum(-2ab g x / d)  instead of  x_k * sum(-2ab g y / d);
    it is reproduced here as it stands, because a drop-in has to give the reference's
    numbers.

Any object with the attributes used below can play the edge; ``ConvEdge`` is a minimal one.
"""
import math

from .choose_matrix_library import cm, cc


class ConvParams(object):
    """The fields of Parameter.Convolution with their defaults (deepnet/protos/deepnet.proto:64-78)."""

    def __init__(self, size=0, stride=0, padding=0, num_filters=0, num_colors=0, max_pool=False, pool_size=0,
                 pool_stride=0, rnorm=False, norm_size=0, pow_scale=0.75, add_scale=0.001, prob=False):
        self.size, self.stride, self.padding = size, stride, padding
        self.num_filters, self.num_colors = num_filters, num_colors
        self.max_pool, self.pool_size, self.pool_stride, self.prob = max_pool, pool_size, pool_stride, prob
        self.rnorm, self.norm_size, self.pow_scale, self.add_scale = rnorm, norm_size, pow_scale, add_scale


def _sites(edge, numdims):
    """(image side, modules per side, pooled sites per side) for inputs of numdims values per image."""
    cv = edge.conv_params
    pixels, rest = divmod(numdims, cv.num_colors)
    side = math.isqrt(pixels)
    assert rest == 0 and side * side == pixels, '%d inputs are not %d square maps' % (numdims, cv.num_colors)
    n_locs = (side + 2 * cv.padding - cv.size) // cv.stride + 1
    n_pool = (n_locs - cv.pool_size) // cv.pool_stride + 1 if cv.max_pool else n_locs
    return side, n_locs, n_pool


def _check_filters(edge):
    cv = edge.conv_params
    f, numdims = edge.params['weight'].shape
    assert f == cv.num_filters, 'f is %d but num_filters is %d' % (f, cv.num_filters)
    if edge.conv:
        assert numdims == cv.size ** 2 * cv.num_colors


class ConvEdge(object):
    """What an edge holds for its conv stage (deepnet/edge.py:94-142): the transposed input and
    output and their gradient twins, the un-pooled layer when pooling, the un-normalised layer,
    the denominators and two temporaries when normalising.  ``node1_shape`` and ``node2_shape``
    are the (dims, batch) shapes of the two layer states."""

    def __init__(self, weight, conv_params, node1_shape, node2_shape, conv=True):
        self.params = {'weight': weight}
        self.conv_params = cv = conv_params
        self.conv, self.local = bool(conv), not conv
        numdims, numimages = node1_shape
        assert node2_shape[1] == numimages
        _, n_locs, n_pool = _sites(self, numdims)
        in_shape, out_shape = (numimages, numdims), (numimages, node2_shape[0])
        assert out_shape[1] == n_pool ** 2 * cv.num_filters, (
            'expected %d outputs, got %d' % (n_pool ** 2 * cv.num_filters, out_shape[1]))
        self.node1_shape = tuple(node1_shape)
        self.input_t, self.input_t2 = cm.empty(in_shape), cm.empty(in_shape)
        self.output_t, self.output_t2 = cm.empty(out_shape), cm.empty(out_shape)
        if cv.max_pool:
            self.unpooled_layer = cm.empty((numimages, n_locs ** 2 * cv.num_filters))
            if cv.prob:
                self.rnd = cm.empty(self.unpooled_layer.shape)
        if cv.rnorm:
            self.unrnormalized_layer, self.denoms = cm.empty(out_shape), cm.empty(out_shape)
            self.rnorm_temp1, self.rnorm_temp2 = cm.empty(out_shape), cm.empty(out_shape)

    def buffers(self):
        names = ('input_t', 'input_t2', 'output_t', 'output_t2', 'unpooled_layer', 'rnd', 'unrnormalized_layer',
                 'denoms', 'rnorm_temp1', 'rnorm_temp2')
        return [getattr(self, n) for n in names if hasattr(self, n)]

    def free_device_memory(self):
        for b in self.buffers():
            b.free_device_memory()


def ConvolveUp(inputs, edge, target):
    """target (dims_out, batch) = the conv stage of ``edge`` applied to inputs (dims_in, batch)."""
    cv = edge.conv_params
    _check_filters(edge)
    w = edge.params['weight']
    inputs.transpose(edge.input_t)
    numimages, numdims = edge.input_t.shape
    _, n_locs, n_pool = _sites(edge, numdims)

    # Where each step writes: the last one into output_t, earlier ones into the buffer the
    # backward pass will look for them in.
    after_conv = edge.unpooled_layer if cv.max_pool else (edge.unrnormalized_layer if cv.rnorm else edge.output_t)
    assert after_conv.shape[0] == numimages, '%d %d.' % (numimages, after_conv.shape[0])
    up = cc.convUp if edge.conv else cc.localUp
    up(edge.input_t, w, after_conv, n_locs, cv.padding, cv.stride, cv.num_colors)
    last = after_conv
    if cv.max_pool and cv.rnorm and not cv.prob and getattr(edge, 'fused', False):
        # this backend's one-launch form of the two calls below (same results)
        cc.MaxPoolResponseNorm(last, edge.unrnormalized_layer, edge.denoms, edge.output_t, cv.num_filters, cv.pool_size, 0,
                               cv.pool_stride, n_pool, cv.norm_size, cv.add_scale, cv.pow_scale)
        edge.output_t.transpose(target)
        return
    if cv.max_pool:
        pooled = edge.unrnormalized_layer if cv.rnorm else edge.output_t
        if cv.prob:
            # -log(u): the exponential variates ProbMaxPool weighs the candidates with
            edge.rnd.fill_with_rand()
            cm.log(edge.rnd)
            edge.rnd.mult(-1)
            cc.ProbMaxPool(last, edge.rnd, pooled, cv.num_filters, cv.pool_size, 0, cv.pool_stride, n_pool)
        else:
            cc.MaxPool(last, pooled, cv.num_filters, cv.pool_size, 0, cv.pool_stride, n_pool)
        last = pooled
    if cv.rnorm:
        cc.ResponseNorm(last, edge.denoms, edge.output_t, cv.num_filters, cv.norm_size, cv.add_scale, cv.pow_scale)
    edge.output_t.transpose(target)


def AccumulateConvDeriv(layer, edge, deriv):
    """layer.deriv (dims_in, batch) = gradient of the stage w.r.t. its inputs, given ``deriv``
    (dims_out, batch), the gradient w.r.t. its outputs.  Leaves the gradient w.r.t. the convUp
    outputs where ConvOuter expects it.  A second gradient into the same layer is refused, as in
    the reference."""
    if layer.dirty:
        raise Exception('Not implemented.')
    layer.dirty = True
    cv = edge.conv_params
    w = edge.params['weight']
    side, n_locs, n_pool = _sites(edge, edge.input_t.shape[1])

    deriv.transpose(edge.output_t2)
    grads, acts = edge.output_t2, edge.output_t
    if cv.rnorm and cv.max_pool and getattr(edge, 'fused', False):
        # this backend's one-launch form of the copy and the two calls below (same gradient in
        # unpooled_layer; rnorm_temp1 / rnorm_temp2 are not written)
        unpooled = edge.unpooled_layer
        cc.ResponseNormUndoMaxPoolUndo(grads, edge.denoms, acts, edge.unrnormalized_layer, unpooled, unpooled,
                                       cv.num_filters, cv.pool_size, 0, cv.pool_stride, n_pool, cv.norm_size,
                                       cv.add_scale, cv.pow_scale)
        grads = unpooled
    elif cv.rnorm:
        # ResponseNormUndo overwrites its `acts` operand: work on a copy of the un-normalised layer.
        edge.rnorm_temp1.assign(edge.unrnormalized_layer)
        cc.ResponseNormUndo(grads, edge.denoms, acts, edge.rnorm_temp1, edge.rnorm_temp2, cv.num_filters,
                            cv.norm_size, cv.add_scale, cv.pow_scale)
        grads, acts = edge.rnorm_temp2, edge.unrnormalized_layer
    if cv.max_pool and grads is not edge.unpooled_layer:
        # in place: the un-pooled activations are not needed once their gradient is known
        unpooled = edge.unpooled_layer
        cc.MaxPoolUndo(unpooled, unpooled, grads, acts, cv.pool_size, 0, cv.pool_stride, n_pool)
        grads = unpooled
    if layer.is_input:
        return
    down = cc.convDown if edge.conv else cc.localDown
    down(grads, w, edge.input_t2, n_locs, cv.padding, cv.stride, cv.size, side, cv.num_colors)
    edge.input_t2.transpose(layer.deriv)


def ConvOuter(edge, grad):
    """grad (filters, colours * size^2 [* modules]) = gradient w.r.t. the weights of ``edge``, from
    the inputs ConvolveUp saw and the gradient AccumulateConvDeriv left behind."""
    cv = edge.conv_params
    _check_filters(edge)
    if cv.max_pool:
        hid_grads = edge.unpooled_layer
    elif cv.rnorm:
        hid_grads = edge.rnorm_temp2
    else:
        hid_grads = edge.output_t2
    numdims = edge.node1.state.shape[0] if hasattr(edge, 'node1') else edge.node1_shape[0]
    _, n_locs, _ = _sites(edge, numdims)
    outp = cc.convOutp if edge.conv else cc.localOutp
    outp(edge.input_t, hid_grads, grad, n_locs, cv.padding, cv.size, cv.stride, cv.num_colors)


def AddConvolveUp(inputs, edge, target):
    """A second conv edge into one layer: not provided by the reference either (convolutions.py:186-187)."""
    raise Exception('Not implemented.')
