"""The device-resident data cache (deepnet_amd/datahandler.py, mirroring the reference's
GPUCache, datahandler.py:259-415) and the checkpoint byte format (deepnet_amd/util.py,
util.py:13-21) against numpy restatements of the same steps.  Data movement is bit-exact;
normalisation is one subtraction and one division per element (2 ulp)."""
import os
import random
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from oracle import cudamat_oracle as orc   # noqa: E402

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dh(cm):
    from deepnet_amd import datahandler
    return datahandler


def _set(n, rng):
    images = rng.random((n, 3072)).astype(np.float32)         # 32 x 32 pixels x 3 interleaved channels
    labels = rng.integers(0, 10, (n, 1)).astype(np.float32)
    return images, labels


def test_batches_normalised_and_in_order(cm, dh, rng):
    images, labels = _set(1000, rng)
    mean, std = images.mean(axis=0), images.std(axis=0)
    cache = dh.GPUCache(dh.ArraySource([images, labels]), capacity=1000, numdim_list=[3072, 1])
    cache.SetDataStats(0, mean, std)
    want = orc.div_by_col_vec(orc.add_col_mult(images.T, mean, -1.0), (1e-10 + std.astype(np.float64)).astype(np.float32))
    seen = 0
    for k in range(9):                                          # 7 batches of 128, the remainder of 104 skipped, 2 more
        x, y = cache.Get(128)
        assert x.shape == (3072, 128) and y.shape == (1, 128)
        lo = (k % 7) * 128
        assert np.allclose(x.asarray(), want[:, lo:lo + 128], rtol=3e-7, atol=1e-7)
        assert np.array_equal(y.asarray(), labels.T[:, lo:lo + 128])
        seen += 128
    cache2 = dh.GPUCache(dh.ArraySource([images, labels]), capacity=1000, numdim_list=[3072, 1])
    sizes = [cache2.Get(300, get_last_piece=True)[0].shape[1] for _ in range(5)]
    assert sizes == [300, 300, 300, 100, 300]


def test_chunks_smaller_than_the_set_reuse_the_allocation(cm, dh, rng):
    images, labels = _set(700, rng)
    cache = dh.GPUCache(dh.ArraySource([images, labels]), capacity=300, numdim_list=[3072, 1], randomize=True)
    got = []
    for _ in range(7):                                          # chunks of 300, 300, 100 rows: 3 + 3 + 1 batches
        x, y = cache.Get(100)
        got.append((x.asarray().copy(), y.asarray().copy()))
    for k, (x, y) in enumerate(got):                            # never shuffled: the parent holds more than the cache
        assert np.array_equal(x, images.T[:, 100 * k:100 * k + 100]) and np.array_equal(y, labels.T[:, 100 * k:100 * k + 100])
    assert cache.allocated_memory_size == [3072 * 300, 300]


def test_shuffle_is_the_pairwise_swap_of_a_permutation(cm, dh, rng):
    images, labels = _set(501, rng)                             # odd: one column stays where it is
    cache = dh.GPUCache(dh.ArraySource([images, labels]), capacity=501, numdim_list=[3072, 1], randomize=True)
    np.random.seed(7)
    x, y = cache.Get(501)
    np.random.seed(7)
    idx = np.arange(501)
    np.random.shuffle(idx)
    a, b = idx[:250], idx[250:500]
    perm = np.arange(501)
    perm[a], perm[b] = b, a
    assert np.array_equal(x.asarray(), images.T[:, perm]) and np.array_equal(y.asarray(), labels.T[:, perm])
    assert sorted(y.asarray().ravel().tolist()) == sorted(labels.ravel().tolist())


def test_random_crops_and_noise(cm, dh, rng):
    images, labels = _set(256, rng)
    cache = dh.GPUCache(dh.ArraySource([images, labels]), capacity=256, numdim_list=[3072, 1], shift=[True, False],
                        shift_amt_x=4, shift_amt_y=3)
    random.seed(3)
    x, y = cache.Get(64)
    random.seed(3)
    shift = (32 - 24) // 2
    ox = [random.choice(range(-4, 5)) + shift for _ in range(64)]
    oy = [random.choice(range(-3, 4)) + shift for _ in range(64)]
    assert x.shape == (24 * 24 * 3, 64)
    # The cache adds the centring shift to the offsets and the library adds it again
    # (datahandler.py:350-352, cudamat_kernels.cu:800-807): origins run from 4 to 12, so windows
    # do leave the 32 x 32 image; both sides address the pixels flat, like the reference.
    assert max(ox) + shift + 24 > 32
    assert np.array_equal(x.asarray(), orc.generate_translations(images.T[:, :64], 32, 24, ox, oy, 3))
    assert np.array_equal(y.asarray(), labels.T[:, :64])
    # the centre crop for test data
    centre = dh.GPUCache(dh.ArraySource([images, labels]), capacity=256, numdim_list=[3072, 1], shift=[True, False],
                         shift_amt_x=4, shift_amt_y=4, center_only=True)
    xc, _ = centre.Get(32)
    off = [4] * 32                                              # (origin 8: rows and columns 8..31)
    assert np.array_equal(xc.asarray(), orc.generate_translations(images.T[:, :32], 32, 24, off, off, 3))
    # Gaussian noise of the configured width on the stream that asks for it
    noisy = dh.GPUCache(dh.ArraySource([images, labels]), capacity=256, numdim_list=[3072, 1], add_noise=[True, False], sigma=0.05)
    xn, yn = noisy.Get(256)
    diff = xn.asarray().astype(np.float64) - images.T
    assert abs(diff.std() - 0.05) < 0.002 and abs(diff.mean()) < 0.001
    assert np.array_equal(yn.asarray(), labels.T)


def test_checkpoint_byte_format_round_trip(cm, rng):
    from deepnet_amd import util
    w = np.asarray(rng.standard_normal((5, 7)), dtype=np.float32, order='F')
    holder = type('Edge', (), {})()
    holder.params = {'weight': cm.CUDAMatrix(w)}
    rec = util.ParamRecord('weight')
    util.SaveParameters(holder, [rec])
    assert rec.dimensions == [5, 7] and rec.mat == np.ascontiguousarray(w).tobytes()      # row-major bytes
    assert np.array_equal(util.ParameterAsNumpy(rec), w)
    holder.params['weight'].assign(0)
    util.LoadParameters(holder, [rec])
    assert np.array_equal(holder.params['weight'].asarray(), w)
    fresh = type('Edge', (), {})()
    fresh.params = {}
    util.LoadParameters(fresh, [rec])
    assert np.array_equal(fresh.params['weight'].asarray(), w)
