"""Python 3 bindings of the convolution / pooling / normalisation entry points:
the functions of the reference's cudamat/cudamat_conv.py:6-181 with the same names,
argument order and shape assertions, over ``libcudamat_conv.so`` built from ``csrc/``.

Operands are CUDAMatrix objects of shape (numImages, channels * size * size), i.e.
cuda-convnet's (channels, rows, cols, batch) layout with the batch fastest.  As in
the reference the wrappers negate ``paddingStart`` before the C call.  ``convDown``
and ``convOutp`` gain an optional ``numGroups`` (the reference hard-codes 1 there
although its C entry points take it).  A shape the reference would abort on
(C assert) raises ``CUDAMatException`` here.
"""
import ctypes as ct
import math
import os

from .cudamat import CUDAMatException, cudamat

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, 'libcudamat_conv.so')
if not os.path.exists(_LIB_PATH):
    raise ImportError("%s is missing: build it with `make -C %s`; this backend has no CPU fallback."
                      % (_LIB_PATH, os.path.join(_HERE, 'csrc')))
_ConvNet = ct.CDLL(_LIB_PATH)

_M = ct.c_void_p   # (see cudamat.py: void* handles convert faster than typed pointers)
_i, _f = ct.c_int, ct.c_float
_SIGNATURES = {
    'convUp': [_M, _M, _M, _i, _i, _i, _i, _i],
    'convDown': [_M, _M, _M, _i, _i, _i, _i, _i],
    'convOutp': [_M, _M, _M, _i, _i, _i, _i, _i, _i, _i],
    'localUp': [_M, _M, _M, _i, _i, _i, _i, _i],
    'localDown': [_M, _M, _M, _i, _i, _i, _i, _i],
    'localOutp': [_M, _M, _M, _i, _i, _i, _i, _i, _i, _i],
    'ResponseNorm': [_M, _M, _M, _i, _i, _f, _f],
    'ResponseNormUndo': [_M, _M, _M, _M, _M, _i, _i, _f, _f],
    'ContrastNorm': [_M, _M, _M, _M, _i, _i, _f, _f],
    'ContrastNormUndo': [_M, _M, _M, _M, _M, _i, _i, _f, _f],
    'MaxPool': [_M, _M, _i, _i, _i, _i, _i],
    'ProbMaxPool': [_M, _M, _M, _i, _i, _i, _i, _i],
    'MaxPoolUndo': [_M, _M, _M, _M, _i, _i, _i, _i],
    'MaxPoolResponseNorm': [_M, _M, _M, _M, _i, _i, _i, _i, _i, _i, _f, _f],
    'ResponseNormUndoMaxPoolUndo': [_M, _M, _M, _M, _M, _M, _i, _i, _i, _i, _i, _i, _f, _f],
}
for _n, _args in _SIGNATURES.items():
    _fn = getattr(_ConvNet, _n)
    _fn.restype = None
    _fn.argtypes = _args
_ConvNet.conv_last_error.restype = ct.c_char_p
_ConvNet.conv_last_error.argtypes = []


def _call(name, *args):
    getattr(_ConvNet, name)(*args)
    err = _ConvNet.conv_last_error()
    if err:
        raise CUDAMatException(err.decode())


def convUp(images, filters, targets, numModulesX, paddingStart, moduleStride, numImgColors, numGroups=1):
    """
    images - (n_images, img_w**2 * n_chans)
    filters - (n_filters, filter_w**2 * n_chans)
    targets - (n_images, n_locs**2 * n_filters)
    numModulesX - number of filter locations along an axis (n_locs)
    paddingStart - k for a k-pixel border of zeros
    moduleStride - stride of the filter locations
    numImgColors - n_chans
    """
    numImages = images.shape[0]
    numFilters = filters.shape[0]
    assert targets.shape == (numImages, numFilters * numModulesX * numModulesX), '%s %d %d-%d-%d' % (
        targets.shape.__str__(), numImages, numFilters, numModulesX, numModulesX)
    _call('convUp', images.p_mat, filters.p_mat, targets.p_mat, numModulesX, -paddingStart, moduleStride,
          numImgColors, numGroups)


def convDown(hidSums, filters, targets, numModulesX, paddingStart, moduleStride, filterSizeX, imSizeX, numImgColors,
             numGroups=1):
    """
    hidSums - (n_images, n_locs**2 * n_filters)
    filters - (n_filters, filter_w**2 * n_chans)
    targets - (n_images, img_w**2 * n_chans)
    """
    numImages = hidSums.shape[0]
    assert paddingStart >= 0
    assert targets.shape == (numImages, numImgColors * imSizeX * imSizeX)
    _call('convDown', hidSums.p_mat, filters.p_mat, targets.p_mat, imSizeX, -paddingStart, moduleStride, numImgColors,
          numGroups)


def convOutp(images, hidSums, targets, numModulesX, paddingStart, filterSizeX, moduleStride, numImgColors,
             numGroups=1, partialSum=0):
    """
    images - (n_images, img_w**2 * n_chans)
    hidSums - (n_images, n_locs**2 * n_filters)
    targets - (n_filters, filter_w**2 * n_chans)
    """
    numFilters = hidSums.shape[1] // (numModulesX ** 2)
    chunks = 1 if partialSum == 0 else (numModulesX ** 2) // partialSum
    assert targets.shape == (numFilters, chunks * (numImgColors // numGroups) * filterSizeX * filterSizeX), \
        '%s %d %d-%d-%d' % (targets.shape.__str__(), numFilters, numImgColors, filterSizeX, filterSizeX)
    _call('convOutp', images.p_mat, hidSums.p_mat, targets.p_mat, numModulesX, filterSizeX, -paddingStart,
          moduleStride, numImgColors, numGroups, partialSum)


def localUp(images, filters, targets, numModulesX, paddingStart, moduleStride, numImgColors, numGroups=1):
    numImages = images.shape[0]
    numFilters = filters.shape[0]
    assert targets.shape == (numImages, numFilters * numModulesX * numModulesX)
    _call('localUp', images.p_mat, filters.p_mat, targets.p_mat, numModulesX, -paddingStart, moduleStride,
          numImgColors, numGroups)


def localDown(hidSums, filters, targets, numModulesX, paddingStart, moduleStride, filterSizeX, imSizeX, numImgColors,
              numGroups=1):
    numImages = hidSums.shape[0]
    assert paddingStart >= 0
    assert targets.shape == (numImages, numImgColors * imSizeX * imSizeX)
    _call('localDown', hidSums.p_mat, filters.p_mat, targets.p_mat, imSizeX, -paddingStart, moduleStride,
          numImgColors, numGroups)


def localOutp(images, hidSums, targets, numModulesX, paddingStart, filterSizeX, moduleStride, numImgColors,
              numGroups=1):
    numFilters = hidSums.shape[1] // (numModulesX ** 2)
    assert targets.shape == (numFilters, numModulesX ** 2 * (numImgColors // numGroups) * filterSizeX ** 2)
    _call('localOutp', images.p_mat, hidSums.p_mat, targets.p_mat, numModulesX, filterSizeX, -paddingStart,
          moduleStride, numImgColors, numGroups, 0)


def MaxPool(images, targets, numChannels, subsX, startX, strideX, outputsX):
    """
    images - (n_images, img_w**2 * n_chans)
    numChannels - number of filter/color channels
    subsX - width of pooling area
    startX - pixel where pooling starts
    strideX - stride
    outputsX - number of pooling sites
    """
    numImages = images.shape[0]
    assert targets.shape == (numImages, numChannels * outputsX * outputsX)
    _call('MaxPool', images.p_mat, targets.p_mat, numChannels, subsX, startX, strideX, outputsX)


def ProbMaxPool(images, rnd, targets, numChannels, subsX, startX, strideX, outputsX):
    numImages = images.shape[0]
    assert targets.shape == (numImages, numChannels * outputsX * outputsX)
    assert rnd.shape == images.shape
    _call('ProbMaxPool', images.p_mat, rnd.p_mat, targets.p_mat, numChannels, subsX, startX, strideX, outputsX)


def MaxPoolUndo(images, targets, grad, maxes, subsX, startX, strideX, outputsX):
    """
    images - (n_images, img_w**2 * n_chans)
    grad - (n_images, outputsX**2 * n_chans) gradients w.r.t. the pooled outputs
    maxes - (n_images, outputsX**2 * n_chans) the pooled outputs
    """
    assert targets.shape == images.shape
    _call('MaxPoolUndo', images.p_mat, grad.p_mat, maxes.p_mat, targets.p_mat, subsX, startX, strideX, outputsX)


def ResponseNorm(images, denoms, targets, numChannels, sizeX, addScale, powScale):
    assert targets.shape == images.shape
    assert targets.shape == denoms.shape
    _call('ResponseNorm', images.p_mat, denoms.p_mat, targets.p_mat, numChannels, sizeX, float(addScale),
          float(powScale))


def ResponseNormUndo(outGrad, denoms, inGrad, acts, targets, numChannels, sizeX, addScale, powScale):
    """Overwrites ``acts`` (as the reference does) with -2*addScale*powScale*outGrad*acts/denoms."""
    assert targets.shape == outGrad.shape
    assert targets.shape == denoms.shape
    assert targets.shape == inGrad.shape
    assert targets.shape == acts.shape
    _call('ResponseNormUndo', outGrad.p_mat, denoms.p_mat, inGrad.p_mat, acts.p_mat, targets.p_mat, numChannels,
          sizeX, float(addScale), float(powScale))


def ContrastNorm(images, meanDiffs, denoms, targets, numChannels, sizeX, addScale, powScale):
    assert targets.shape == images.shape == meanDiffs.shape == denoms.shape
    _call('ContrastNorm', images.p_mat, meanDiffs.p_mat, denoms.p_mat, targets.p_mat, numChannels, sizeX,
          float(addScale), float(powScale))


def ContrastNormUndo(outGrad, denoms, meanDiffs, acts, targets, numChannels, sizeX, addScale, powScale):
    assert targets.shape == outGrad.shape == denoms.shape == meanDiffs.shape == acts.shape
    _call('ContrastNormUndo', outGrad.p_mat, denoms.p_mat, meanDiffs.p_mat, acts.p_mat, targets.p_mat, numChannels,
          sizeX, float(addScale), float(powScale))


def MaxPoolResponseNorm(images, pooled, denoms, targets, numChannels, subsX, startX, strideX, outputsX, sizeX, addScale,
                        powScale):
    """Extension of this backend (not in the reference): MaxPool(images -> pooled) followed by
    ResponseNorm(pooled -> denoms, targets), the pair deepnet/convolutions.py:58-66 always issues
    together, in one launch (the pooled map stays in LDS between the two stages); same results."""
    numImages = images.shape[0]
    assert pooled.shape == (numImages, numChannels * outputsX * outputsX)
    assert targets.shape == pooled.shape == denoms.shape
    _call('MaxPoolResponseNorm', images.p_mat, pooled.p_mat, denoms.p_mat, targets.p_mat, numChannels, subsX, startX,
          strideX, outputsX, sizeX, float(addScale), float(powScale))


def ResponseNormUndoMaxPoolUndo(outGrad, denoms, inGrad, acts, images, targets, numChannels, subsX, startX, strideX,
                                outputsX, sizeX, addScale, powScale):
    """Extension of this backend (not in the reference): ResponseNormUndo(outGrad, denoms, inGrad, acts)
    followed by MaxPoolUndo(images, its result, acts -> targets), the pair of
    deepnet/convolutions.py:120-134, in one launch.  ``acts`` are the pooled activations and are left
    unchanged (ResponseNormUndo alone overwrites its ``acts``); ``targets`` may be ``images``."""
    assert targets.shape == images.shape
    assert outGrad.shape == denoms.shape == inGrad.shape == acts.shape
    _call('ResponseNormUndoMaxPoolUndo', outGrad.p_mat, denoms.p_mat, inGrad.p_mat, acts.p_mat, images.p_mat,
          targets.p_mat, numChannels, subsX, startX, strideX, outputsX, sizeX, float(addScale), float(powScale))
