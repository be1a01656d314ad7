"""TEST INFRASTRUCTURE ONLY - ctypes drivers for the step functions of oracle/host_backend.c
(the CPU baseline of the benchmark).  Only tests/ and bench.py's cpu_baseline leg use this."""
import ctypes as ct
import os

import numpy as np

from . import mwc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FP = ct.POINTER(ct.c_float)


def load():
    return ct.CDLL(os.path.join(ROOT, 'oracle', 'liboracle_host.so'))


class HostMLP(object):
    """The buffers of hb_mlp_step (op sequence of deepnet/neuralnet.py:138-291 and
    parameter.py:80-106) as numpy arrays: W[i] (sizes[i], sizes[i+1]), b[i], their velocities
    dW / db and gradients gW / gb, activations act[i] (sizes[i], B) with act[0] = the inputs,
    dropout masks mask[i] and back-propagated gradients delta[i]; all float32, column-major."""

    def __init__(self, lib, sizes, B, x, labels, W, b, lr, mom, seed):
        self.lib, self.sizes, self.B, self.lr, self.mom = lib, list(sizes), B, lr, mom
        nl = self.nl = len(sizes) - 1
        f = lambda a: np.array(a, dtype=np.float32, order='F')
        self.W, self.b = [f(w) for w in W], [f(np.asarray(v).reshape(-1)) for v in b]
        self.dW, self.db = [np.zeros_like(w) for w in self.W], [np.zeros_like(v) for v in self.b]
        self.gW, self.gb = [np.zeros_like(w) for w in self.W], [np.zeros_like(v) for v in self.b]
        self.act = [f(x)] + [np.zeros((sizes[i + 1], B), np.float32, order='F') for i in range(nl)]
        self.mask = [np.zeros((sizes[i + 1], B), np.float32, order='F') for i in range(nl - 1)]
        self.delta = [np.zeros((sizes[i + 1], B), np.float32, order='F') for i in range(nl)]
        self.labels, self.loss = f(np.asarray(labels).reshape(-1)), np.zeros(B, np.float32)
        self.mults = mwc.load_multipliers(os.path.join(ROOT, 'deepnet_amd', 'rnd_multipliers_32bit.txt'))
        self.words = np.empty(mwc.NUM_RND_STREAMS, dtype=np.uint64)
        self._u32 = self.mults.ctypes.data_as(ct.POINTER(ct.c_uint32))
        self._u64 = self.words.ctypes.data_as(ct.POINTER(ct.c_uint64))
        lib.mwc_seed(self._u32, self._u64, ct.c_uint32(seed))
        arr = lambda lst: (FP * len(lst))(*[a.ctypes.data_as(FP) for a in lst])
        self._sizes = (ct.c_int * len(sizes))(*sizes)
        self._args = [arr(self.W), arr(self.b), arr(self.dW), arr(self.db), arr(self.gW), arr(self.gb), arr(self.act),
                      arr(self.mask), arr(self.delta)]

    def step(self):
        self.lib.hb_mlp_step(self.nl, self._sizes, self.B, ct.c_float(self.lr), ct.c_float(self.mom), *self._args,
                             self.labels.ctypes.data_as(FP), self.loss.ctypes.data_as(FP), self._u32, self._u64)
