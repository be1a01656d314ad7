"""The entry point that allocates nothing (max_by_axis_noalloc) against max_by_axis,
called through the C ABI: two calls in a row on the fixed workspace, the second with a
smaller input, then shapes that take its other paths."""
import ctypes as ct

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _both(cm, x, axis):
    lib = cm._cudamat
    a = cm.CUDAMatrix(x)
    shape = (1, x.shape[1]) if axis == 0 else (x.shape[0], 1)
    want, got = cm.empty(shape), cm.empty(shape)
    got.assign(-7.0)
    assert lib.max_by_axis(a.p_mat, want.p_mat, ct.c_int(axis)) == 0
    assert lib.max_by_axis_noalloc(a.p_mat, got.p_mat, ct.c_int(axis)) == 0
    w, g = want.asarray(), got.asarray()
    for m in (a, want, got):
        m.free_device_memory()
    return w, g


def test_two_calls_in_a_row_second_one_smaller(cm):
    rng = np.random.default_rng(77)
    # 4096 x 4096: 4 column slices, 16384 partials and 64 counters of the workspace in use;
    # then 2048 x 1024 (4 slices of 256 columns) on the same workspace, and the first again
    for shape in [(4096, 4096), (2048, 1024), (4096, 4096)]:
        x = np.asarray(rng.uniform(-1, 1, shape), dtype=np.float32, order='F')
        want, got = _both(cm, x, 1)
        assert np.array_equal(got, want)                          # bit-identical to max_by_axis
        assert np.array_equal(got[:, 0], x.max(axis=1))           # and exact against numpy


@pytest.mark.parametrize("shape", [(64, 512), (1000, 37), (1024, 4096), (37, 53), (8192, 600), (20000, 300), (4, 1)])
@pytest.mark.parametrize("axis", [0, 1])
def test_other_shapes_and_axis0(cm, shape, axis):
    rng = np.random.default_rng(78)
    x = np.asarray(rng.uniform(-1, 1, shape), dtype=np.float32, order='F')
    want, got = _both(cm, x, axis)
    assert np.array_equal(got, want)
    assert np.array_equal(got.ravel(), x.max(axis=axis))


def test_unaligned_view_and_errors(cm):
    rng = np.random.default_rng(79)
    x = np.asarray(rng.uniform(-1, 1, (1001, 300)), dtype=np.float32, order='F')
    a = cm.CUDAMatrix(x)
    v = a.get_col_slice(1, 300) if hasattr(a, 'get_col_slice') else a.slice(1, 300)   # starts 4004 bytes in
    t = cm.empty((1001, 1))
    assert cm._cudamat.max_by_axis_noalloc(v.p_mat, t.p_mat, ct.c_int(1)) == 0
    assert np.array_equal(t.asarray()[:, 0], x[:, 1:].max(axis=1))
    bad = cm.empty((5, 1))
    assert cm._cudamat.max_by_axis_noalloc(a.p_mat, bad.p_mat, ct.c_int(1)) == -1
    assert cm._cudamat.max_by_axis_noalloc(a.p_mat, t.p_mat, ct.c_int(2)) == -9
    with pytest.raises(cm.CUDAMatException):
        a.max_noalloc(1, bad)
    assert np.array_equal(a.max_noalloc(1, t).asarray()[:, 0], x.max(axis=1))
