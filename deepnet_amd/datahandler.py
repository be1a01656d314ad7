"""The device-resident stage of deepnet's data pipeline on the MI355X backend: ``GPUCache``
of the reference's deepnet/datahandler.py:259-415 -- a chunk of the data set kept in HBM as
(dims, datapoints) matrices, normalised (add_col_mult / div_by_col), shuffled in place
(swap_columns), served as column-slice views, optionally with Gaussian noise
(sample_gaussian) or random crops (generate_translations) applied to each batch -- with the
reference's method names and the same matrix calls.

The stages above it (disk readers, the host-memory cache, the protobuf data configuration)
are not part of this package: the parent is any object with ``Get(n)`` returning a list of
(datapoints, dims) arrays and a ``_maxpos`` attribute, e.g. ``ArraySource`` below.
"""
import random

import numpy as np

from .choose_matrix_library import cm


class ArraySource(object):
    """A parent cache over arrays already in host memory: hands out at most ``n`` rows of each
    array per call, in order, wrapping around at the end (the contract of Cache.Get,
    datahandler.py:238-256, without its shuffling)."""

    def __init__(self, arrays):
        self.data = [np.asarray(a) for a in arrays]
        self._maxpos = self.data[0].shape[0]
        self._pos = 0

    def Get(self, n):
        if self._pos == self._maxpos:
            self._pos = 0
        start, end = self._pos, min(self._pos + n, self._maxpos)
        self._pos = end
        return [d[start:end] for d in self.data]


class GPUCache(object):
    """``capacity`` is in data points (the reference derives it from a byte budget,
    datahandler.py:200-203); ``numdim_list`` gives the width of each data stream."""

    def __init__(self, parent, capacity, numdim_list, randomize=False, add_noise=None, shift=None, shift_amt_x=0,
                 shift_amt_y=0, center_only=False, image_size=32, num_channels=3, sigma=0.01):
        self.parent = parent
        self.num_data = len(numdim_list)
        self.numdim_list = list(numdim_list)
        self._maxpos = int(capacity)
        self._pos = 0
        self.datasize = 0
        self.randomize = randomize
        self.data = [None] * self.num_data
        self.empty = True
        self.allocated_memory_size = [0] * self.num_data
        self.normalize = [False] * self.num_data
        self.means = [None] * self.num_data
        self.stds = [None] * self.num_data
        self.add_noise = list(add_noise) if add_noise is not None else [False] * self.num_data
        self.translate = list(shift) if shift is not None else [False] * self.num_data
        shift_amt = max(shift_amt_x, shift_amt_y)
        self.sizeX = image_size                 # (32 and 3 channels are hard-wired in the reference, :289-291)
        self.sizex = image_size - 2 * shift_amt
        self.num_channels = num_channels
        if center_only:                         # test data: the centre crop, no noise
            self.translate_range_x, self.translate_range_y, self.sigma = [0], [0], 0
        else:
            self.translate_range_x = list(range(-shift_amt_x, shift_amt_x + 1))
            self.translate_range_y = list(range(-shift_amt_y, shift_amt_y + 1))
            self.sigma = sigma
        self.translated_d = self.offset_x = self.offset_y = None

    def SetDataStats(self, i, mean, std):
        """Per-dimension mean and standard deviation for stream i (the reference reads them
        from an .npz file, :385-391)."""
        self.normalize[i] = True
        self.means[i] = cm.CUDAMatrix(np.asarray(mean, dtype=np.float32).reshape(-1, 1))
        self.stds[i] = cm.CUDAMatrix((1e-10 + np.asarray(std, dtype=np.float64)).astype(np.float32).reshape(-1, 1))

    def Normalize(self):
        for i, batch in enumerate(self.data):
            if self.normalize[i]:
                batch.add_col_mult(self.means[i], mult=-1.0)
                batch.div_by_col(self.stds[i])

    def LoadData(self):
        data_cpu = self.parent.Get(self._maxpos)
        datasize = data_cpu[0].shape[0]
        assert datasize <= self._maxpos, "GPU cache can only store %d datapoints, but parent gave it %d." % (
            self._maxpos, datasize)
        self.datasize = datasize
        for i, d in enumerate(data_cpu):
            mat = (d.toarray() if hasattr(d, 'toarray') else np.asarray(d)).T
            size = mat.shape[0] * mat.shape[1]
            if size > self.allocated_memory_size[i]:
                if self.data[i] is not None:
                    self.data[i].free_device_memory()      # (the reference leaks the smaller buffer)
                self.data[i] = cm.CUDAMatrix(mat)
                self.allocated_memory_size[i] = size
            else:
                self.data[i].overwrite(mat)                # a smaller chunk reuses the allocation
        self.Normalize()

    def AddNoise(self, batch, i):
        batch[i].sample_gaussian(mult=self.sigma)

    def TranslateData(self, batch, i):
        """Replace batch[i] by random crops of sizex x sizex pixels out of its sizeX x sizeX images."""
        d = batch[i]
        batchsize = d.shape[1]
        shift = (self.sizeX - self.sizex) // 2
        offset_x = np.array([random.choice(self.translate_range_x) + shift for _ in range(batchsize)]).reshape(1, -1)
        offset_y = np.array([random.choice(self.translate_range_y) + shift for _ in range(batchsize)]).reshape(1, -1)
        if self.offset_x is None or self.offset_x.shape != offset_x.shape:
            self.offset_x, self.offset_y = cm.CUDAMatrix(offset_x), cm.CUDAMatrix(offset_y)
        else:
            self.offset_x.overwrite(offset_x)
            self.offset_y.overwrite(offset_y)
        if self.translated_d is None or self.translated_d.shape[1] != batchsize:
            self.translated_d = cm.empty((self.sizex ** 2 * self.num_channels, batchsize))
        d.generate_translations(self.sizeX, self.sizex, self.offset_x, self.offset_y, target=self.translated_d)
        batch[i] = self.translated_d

    def ShuffleData(self):
        """In-place shuffle: one half of a random permutation swaps columns with the other half,
        the same pairs in every stream."""
        indices = np.arange(self.datasize)
        np.random.shuffle(indices)
        half = self.datasize // 2
        indices1_gpu = cm.CUDAMatrix(indices[:half].reshape(1, -1))
        indices2_gpu = cm.CUDAMatrix(indices[half:2 * half].reshape(1, -1))
        for d in self.data:
            d.swap_columns(indices1_gpu, indices2_gpu, target=d)
        indices1_gpu.free_device_memory()
        indices2_gpu.free_device_memory()

    def Get(self, batchsize, get_last_piece=False):
        """The next ``batchsize`` data points of every stream as (dims, batchsize) views; a
        shorter remainder at the end of the chunk is skipped unless ``get_last_piece``."""
        if self._pos == self.datasize:
            self._pos = 0
        if self._pos == 0:
            if self.empty or self._maxpos < self.parent._maxpos:
                self.LoadData()
                self.empty = False
            if self.randomize and self._maxpos == self.parent._maxpos:
                self.ShuffleData()          # the whole set is resident: nobody above has shuffled it
        start, end = self._pos, self._pos + batchsize
        skip = False
        if end > self.datasize:
            end = self.datasize
            skip = not get_last_piece
        self._pos = end
        if skip:
            return self.Get(batchsize, get_last_piece=get_last_piece)
        batch = [d.slice(start, end) for d in self.data]
        for i in range(self.num_data):
            if self.add_noise[i]:
                self.AddNoise(batch, i)
            if self.translate[i]:
                self.TranslateData(batch, i)
        return batch
