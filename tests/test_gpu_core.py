"""GPU tests of handles, transfers, views, row slices, transpose and the column
gather / scatter ops (modelled on cudamat/test_cudamat.py:12-290, 596-794)."""
import ctypes as ct

import numpy as np
import pytest

from oracle import cudamat_oracle as orc

pytestmark = pytest.mark.gpu


def _rand(rng, shape):
    return np.asarray(rng.standard_normal(shape), dtype=np.float32, order='F')


def test_roundtrip_reshape_and_T_field(cm, rng):
    x = _rand(rng, (256, 128))
    a = cm.CUDAMatrix(x)
    assert a.shape == (256, 128)
    assert np.array_equal(a.asarray(), x)
    a.reshape((128, 256))
    assert np.array_equal(a.asarray().ravel(order='F'), x.ravel(order='F'))   # test_cudamat.py:12-28
    a.reshape((-1, 64)); assert a.shape == (512, 64)
    a.reshape((256, -1)); assert a.shape == (256, 128)
    with pytest.raises(cm.CUDAMatException):
        a.reshape((7, 7))
    b = cm.CUDAMatrix(_rand(rng, (256, 10)))
    t = cm.dot(a.T, b)                                                        # test_cudamat.py:30-44
    assert np.allclose(t.asarray(), x.T.astype(np.float64) @ b.asarray(), atol=1e-3)


def test_empty_matrices_are_harmless(cm):
    e = cm.empty((0, 5))
    assert e.shape == (0, 5)
    e.add(1.0); cm.exp(e); e.assign(3.0)
    assert e.asarray().shape == (0, 5)
    z = cm.CUDAMatrix(np.zeros((4, 0), dtype=np.float32))
    z.mult(2.0)
    assert z.asarray().shape == (4, 0)


def test_copy_transpose(cm, rng):
    for shape in [(256, 128), (37, 53), (1, 9), (9, 1), (3072, 128), (65, 64), (128, 14400), (14400, 128), (68, 132),
                  (4, 4), (132, 4), (60, 200)]:        # (multiples of 4 take the 16-byte kernel, ragged tiles included)
        x = _rand(rng, shape)
        a = cm.CUDAMatrix(x)
        t = a.transpose()
        assert np.array_equal(t.asarray(), x.T)
        t2 = cm.empty((shape[1], shape[0]))
        a.transpose(target=t2)
        assert np.array_equal(t2.asarray(), x.T)
    with pytest.raises(cm.CUDAMatException):
        a.transpose(target=cm.empty((5, 5)))
    # a source view that starts off a 16-byte boundary (column 1 of a 3-row parent) takes the scalar kernel
    x = _rand(rng, (3, 17))
    view = cm.CUDAMatrix(x).slice(1, 17).reshape((4, 12))
    assert np.array_equal(view.transpose().asarray(), x[:, 1:].reshape((4, 12), order='F').T)


def test_column_slices_alias_the_parent(cm, rng):
    x = _rand(rng, (37, 20))
    a = cm.CUDAMatrix(x)
    v = a.slice(3, 11)
    assert v.shape == (37, 8) and v.mat.owns_data == 0
    assert np.array_equal(v.asarray(), x[:, 3:11])
    v.assign(0.0)
    want = x.copy(); want[:, 3:11] = 0
    assert np.array_equal(a.asarray(), want)
    v.free_device_memory()                   # a view frees nothing
    assert np.array_equal(a.asarray(), want)
    y = _rand(rng, (37, 5))
    a.set_col_slice(0, 5, cm.CUDAMatrix(y))
    want[:, 0:5] = y
    assert np.array_equal(a.asarray(), want)
    t = cm.empty((37, 4))
    a.get_col_slice(2, 6, target=t)
    assert np.array_equal(t.asarray(), want[:, 2:6])
    with pytest.raises(cm.CUDAMatException):
        a.slice(5, 21)
    with pytest.raises(cm.CUDAMatException, match="transposed"):
        cm._check(cm._cudamat.get_slice(a.T.p_mat, ct.byref(cm.cudamat()), 0, 1))
    row = cm.CUDAMatrix(_rand(rng, (1, 30)))
    assert np.array_equal(row.slice(4, 9).asarray(), row.asarray()[:, 4:9])


def test_row_slices(cm, rng):
    for shape, (s, e) in [((256, 128), (10, 120)), ((37, 53), (0, 37)), ((300, 3), (299, 300)), ((70, 1), (3, 40))]:
        x = _rand(rng, shape)
        a = cm.CUDAMatrix(x)
        r = a.get_row_slice(s, e)
        assert np.array_equal(r.asarray(), x[s:e, :])
        y = _rand(rng, (e - s, shape[1]))
        a.set_row_slice(s, e, cm.CUDAMatrix(y))
        want = x.copy(); want[s:e, :] = y
        assert np.array_equal(a.asarray(), want)
    with pytest.raises(cm.CUDAMatException):
        a.get_row_slice(5, 500)


@pytest.mark.parametrize("h", [37, 40, 1028])          # one row per lane, and four (row counts that are multiples of 4)
def test_select_set_swap_columns(cm, rng, h):
    x = _rand(rng, (h, 20))
    a = cm.CUDAMatrix(x)
    idx = np.array([[0, 19, -1, 5, 5, 25, -21]], dtype=np.float32)
    t = cm.empty((h, idx.size))
    a.select_columns(cm.CUDAMatrix(idx), t)
    want = orc.select_columns(x, idx)
    got = t.asarray()
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.array_equal(got[~np.isnan(want)], want[~np.isnan(want)].astype(np.float32))
    src = _rand(rng, (h, 3))
    sidx = np.array([[4, -1, 7]], dtype=np.float32)
    a.set_selected_columns(cm.CUDAMatrix(sidx), cm.CUDAMatrix(src))
    assert np.array_equal(a.asarray(), orc.set_selected_columns(x, src, sidx).astype(np.float32))
    # swap: disjoint index sets within one matrix = an in-place shuffle (cudamat.py:1496-1512)
    b = cm.CUDAMatrix(x)
    i1 = np.array([[0, 1, 2]], dtype=np.float32); i2 = np.array([[10, 11, 12]], dtype=np.float32)
    b.swap_columns(cm.CUDAMatrix(i1), cm.CUDAMatrix(i2), b)
    want = x.copy(); want[:, [0, 1, 2]] = x[:, [10, 11, 12]]; want[:, [10, 11, 12]] = x[:, [0, 1, 2]]
    assert np.array_equal(b.asarray(), want)


def test_blockify_expand_accumulate_translations(cm, rng):
    x = _rand(rng, (24, 7))
    a, t = cm.CUDAMatrix(x), cm.empty((24, 7))
    a.blockify(4, target=t)
    assert np.array_equal(t.asarray(), orc.blockify(x, 4).astype(np.float32))
    idx = np.array([[0, 6, 3, 3, 9, 1, 0, 2, 5]], dtype=np.float32)
    e = cm.empty((24, 9))
    a.expand(cm.CUDAMatrix(idx), e)
    want = orc.expand(x, idx)
    assert np.array_equal(np.isnan(e.asarray()), np.isnan(want))
    assert np.array_equal(e.asarray()[~np.isnan(want)], want[~np.isnan(want)].astype(np.float32))
    m = _rand(rng, (24, 4))
    idx2 = np.asarray(rng.integers(0, 4, (1, 7)), dtype=np.float32)
    r = cm.empty((24, 7))
    a.expand_and_add(cm.CUDAMatrix(m), cm.CUDAMatrix(idx2), target=r, mult=0.5)
    assert np.allclose(r.asarray(), orc.expand_and_add(x, m, idx2, 0.5), rtol=1e-6)
    lab = np.asarray(rng.integers(0, 3, (1, 7)), dtype=np.float32)
    acc = cm.empty((24, 3))
    a.accumulate_columns(cm.CUDAMatrix(lab), acc, mult=2.0, avg=True)
    assert np.allclose(acc.asarray(), orc.accumulate_columns(x, lab, 3, 2.0, True), rtol=1e-5, atol=1e-6)
    a.accumulate_columns(cm.CUDAMatrix(lab), acc, mult=1.0, avg=False)
    assert np.allclose(acc.asarray(), orc.accumulate_columns(x, lab, 3, 1.0, False), rtol=1e-5, atol=1e-6)
    # translations: 3-channel 8x8 images cropped to 6x6 with per-image offsets
    imgs = _rand(rng, (8 * 8 * 3, 5))
    ox = np.array([[0, 1, -1, 1, 0]], dtype=np.float32); oy = np.array([[0, -1, 1, 1, -1]], dtype=np.float32)
    tr = cm.CUDAMatrix(imgs).generate_translations(8, 6, cm.CUDAMatrix(ox), cm.CUDAMatrix(oy))
    assert np.array_equal(tr.asarray(), orc.generate_translations(imgs, 8, 6, ox, oy, 3).astype(np.float32))
    # offsets that push the window out of the image: the next pixel row / next image, 0 past the matrix
    ox = np.array([[2, 3, -2, 0, 3]], dtype=np.float32); oy = np.array([[3, 0, -3, 2, 3]], dtype=np.float32)
    tr = cm.CUDAMatrix(imgs).generate_translations(8, 6, cm.CUDAMatrix(ox), cm.CUDAMatrix(oy))
    want = orc.generate_translations(imgs, 8, 6, ox, oy, 3).astype(np.float32)
    assert np.array_equal(tr.asarray(), want) and (want[:, 4] == 0).any() and (want[:, 0] != 0).all()


@pytest.mark.parametrize("n", [1, 3, 1023, 4096, 16384, 16385])
def test_small_results_reach_the_host_after_the_work_queued_before_them(cm, n):
    """Matrices of up to 16384 elements are read back through a pinned block that a kernel
    fills and tags; every read must show the values of the kernel queued just before it."""
    a = cm.empty((n, 1))
    b = cm.CUDAMatrix(np.arange(n, dtype=np.float32).reshape(n, 1))
    for i in range(300):
        a.assign(float(i))
        a.add(b)
        got = a.asarray()
        assert got[0, 0] == i and got[-1, 0] == i + n - 1 and np.array_equal(got[:, 0], np.arange(n, dtype=np.float32) + i), i


def test_freed_blocks_are_reused_without_disturbing_queued_work(cm, rng):
    """free_device_memory keeps a block for the next matrix of its size; work queued on the old
    owner finishes before the new owner's first kernel, so results do not change."""
    x = np.asarray(rng.uniform(-1, 1, (257, 129)), dtype=np.float32, order='F')
    a = cm.CUDAMatrix(x)
    total = np.zeros_like(x)
    for i in range(50):
        t = cm.empty(x.shape)
        a.mult(float(i), target=t)
        u = cm.empty(x.shape)
        t.add(a, target=u)
        t.free_device_memory()                   # its block goes to the next empty() of this size
        v = cm.empty(x.shape)
        v.assign(1.0)
        assert np.array_equal(u.asarray(), x * np.float32(i) + x)
        assert np.array_equal(v.asarray(), np.ones_like(x))
        u.free_device_memory(); v.free_device_memory()
    # other sizes, empty matrices and a shape changed after allocation
    w = cm.empty((64, 64)); w.reshape((32, 128)); w.free_device_memory()
    z = cm.empty((0, 5)); z.free_device_memory()
    big = cm.empty((2048, 2048)); big.assign(2.0)
    assert float(big.sum()) == 2.0 * 2048 * 2048
    big.free_device_memory()
