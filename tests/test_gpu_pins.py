"""The enumerations of tests/test_oracle_pins.py (every arg-max tie pattern, every ProbMaxPool
sequence over a set of ordinary and overflowing values, every 0/1 image under MaxPoolUndo) run
on the device and compared with the oracle bit for bit."""
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import test_oracle_pins as pins                                  # noqa: E402
from oracle import conv_oracle as co, cudamat_oracle as orc      # noqa: E402

pytestmark = pytest.mark.gpu


def _f(a):
    return np.asarray(a, dtype=np.float32, order='F')


def test_argmax_family_on_every_tie_pattern(cm):
    x = _f(pins.tie_columns(40))
    want = orc.argmax_by_axis(x, 0)
    a = cm.CUDAMatrix(x)
    assert np.array_equal(a.argmax(axis=0).asarray(), want)
    onehot = cm.empty(x.shape)
    a.choose_max(axis=0, target=onehot)
    got = onehot.asarray()
    assert np.array_equal(got, orc.choose_max_by_axis(x, 0))
    labels = _f(want)
    correct = cm.empty((1, x.shape[1]))
    a.get_softmax_correct(cm.CUDAMatrix(labels), correct)
    assert np.all(correct.asarray() == 1.0)
    labels[0, ::2] += 1.0
    a.get_softmax_correct(cm.CUDAMatrix(labels), correct)
    assert np.array_equal(correct.asarray()[0], np.tile([0.0, 1.0], x.shape[1] // 2 + 1)[:x.shape[1]])
    # tall columns take the 256-lane kernel: the same rule over 4 wavefronts
    tall = np.zeros((5000, 6), dtype=np.float32)
    for j, rows in enumerate([(4999, 31), (32, 1), (4097, 4064), (70, 38, 6), (0,), (4999,)]):
        tall[list(rows), j] = 3.0
    assert np.array_equal(cm.CUDAMatrix(_f(tall)).argmax(axis=0).asarray(), orc.argmax_by_axis(tall, 0))


def test_prob_max_pool_on_every_sequence(cm, cc):
    seqs, x, r = pins.prob_inputs()
    T = cm.empty((x.shape[0], 1))
    cc.ProbMaxPool(cm.CUDAMatrix(_f(x)), cm.CUDAMatrix(_f(r)), T, 1, 2, 0, 2, 1)
    want = co.prob_max_pool(x, r, 1, 2, 0, 2, 1).astype(np.float32)
    assert np.array_equal(T.asarray(), want, equal_nan=True)


@pytest.mark.parametrize("S,subs,start,stride", pins.POOL_UNDO_CASES)
def test_max_pool_undo_on_every_binary_image(cm, cc, S, subs, start, stride):
    O, imgs, grads = pins.pool_undo_inputs(S, subs, start, stride)
    X, T = cm.CUDAMatrix(_f(imgs)), cm.empty((imgs.shape[0], O * O))
    cc.MaxPool(X, T, 1, subs, start, stride, O)
    acts = co.max_pool(imgs, 1, subs, start, stride, O)
    assert np.array_equal(T.asarray(), acts.astype(np.float32))
    U = cm.empty(imgs.shape)
    cc.MaxPoolUndo(X, U, cm.CUDAMatrix(_f(grads)), T, subs, start, stride, O)
    # gradients are multiples of 0.25 below 2^10: every sum is exact in fp32
    assert np.array_equal(U.asarray(), co.max_pool_undo(imgs, grads, acts, subs, start, stride, O).astype(np.float32))
