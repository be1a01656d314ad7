"""Run-to-run determinism of the kernels whose workgroups meet inside one launch.

The one-launch reductions (`sum / max / sqsum` along axis 1, `vdot`, `max_by_axis_noalloc`), the
split reductions of the conv passes and the last-arriver finishes publish partial results with
agent-scope atomic stores, count themselves in on a counter and let the workgroup that arrives
last add the partials in a fixed order.  A partial that the last arriver missed would show up
as a rare wrong result in the last bits, so each of them is launched 200 times back to back on
one input, interleaved with an unrelated streaming kernel (which keeps the caches and the
memory system busy with other traffic), and every result must have the bits of the first."""
import ctypes as ct

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

REPEATS = 200


def _f(a):
    return np.asarray(a, dtype=np.float32, order='F')


class _Noise:
    """An unrelated streaming kernel between the launches under test."""

    def __init__(self, cm, rng):
        self.a = cm.CUDAMatrix(_f(rng.uniform(-1, 1, (2048, 2048))))
        self.b = cm.CUDAMatrix(_f(rng.uniform(-1, 1, (2048, 2048))))

    def __call__(self, i):
        if i % 3 == 0:
            self.a.add_mult(self.b, 1e-3)
        elif i % 3 == 1:
            self.b.mult(0.999)


def _soak(cm, launch, read, noise):
    """launch() queues the kernel under test into result buffer i % 4; results are read back in
    batches of four so that launches really run back to back."""
    first = None
    for start in range(0, REPEATS, 4):
        for i in range(start, start + 4):
            launch(i % 4)
            noise(i)
        for j in range(4):
            got = read(j)
            if first is None:
                first = got.copy()
            elif not np.array_equal(got.view(np.uint32), first.view(np.uint32)):
                bad = np.flatnonzero(got.view(np.uint32).ravel() != first.view(np.uint32).ravel())
                pytest.fail("launch %d differs from launch 0 in %d elements (first at %d: %r vs %r)"
                            % (start + j, bad.size, bad[0], got.ravel()[bad[0]], first.ravel()[bad[0]]))
    return first


@pytest.mark.parametrize("shape", [(4096, 4096), (4100, 4092)])
@pytest.mark.parametrize("op", ["sum", "max", "sqsum"])
def test_axis1_reductions_repeat_bit_for_bit(cm, shape, op):
    rng = np.random.default_rng(91)
    x = _f(rng.uniform(-1, 1, shape))
    X = cm.CUDAMatrix(x)
    outs = [cm.empty((shape[0], 1)) for _ in range(4)]
    noise = _Noise(cm, rng)
    lib = cm._cudamat

    def launch(slot):
        if op == "sum":
            assert lib.sum_by_axis(X.p_mat, outs[slot].p_mat, ct.c_int(1)) == 0
        elif op == "max":
            assert lib.max_by_axis(X.p_mat, outs[slot].p_mat, ct.c_int(1)) == 0
        else:
            assert lib.sqsum_by_axis(X.p_mat, outs[slot].p_mat, ct.c_int(1), ct.c_float(1.0), ct.c_float(0.0)) == 0

    first = _soak(cm, launch, lambda slot: outs[slot].asarray(), noise)
    want = {"sum": x.astype(np.float64).sum(axis=1), "max": x.max(axis=1).astype(np.float64),
            "sqsum": (x.astype(np.float64) ** 2).sum(axis=1)}[op]
    assert np.allclose(first[:, 0], want, rtol=1e-5, atol=1e-5)


def test_vdot_repeats_bit_for_bit(cm):
    rng = np.random.default_rng(92)
    a, b = _f(rng.uniform(-1, 1, (4096, 4096))), _f(rng.uniform(-1, 1, (4096, 4096)))
    A, B = cm.CUDAMatrix(a), cm.CUDAMatrix(b)
    noise = _Noise(cm, rng)
    first = None
    for i in range(REPEATS):
        got = np.float32(cm.vdot(A, B))
        noise(i)
        if first is None:
            first = got
        assert got.view(np.uint32) == first.view(np.uint32), "call %d: %r, call 0: %r" % (i, got, first)
    assert abs(float(first) - float(np.vdot(a.astype(np.float64), b.astype(np.float64)))) < 1e-5 * 4096 * 4096 / 3


def test_max_noalloc_repeats_bit_for_bit(cm):
    rng = np.random.default_rng(93)
    x = _f(rng.uniform(-1, 1, (4096, 4096)))
    X = cm.CUDAMatrix(x)
    outs = [cm.empty((4096, 1)) for _ in range(4)]
    noise = _Noise(cm, rng)

    def launch(slot):
        assert cm._cudamat.max_by_axis_noalloc(X.p_mat, outs[slot].p_mat, ct.c_int(1)) == 0

    first = _soak(cm, launch, lambda slot: outs[slot].asarray(), noise)
    assert np.array_equal(first[:, 0], x.max(axis=1))


CONV_SOAKS = [  # pass, N, C, H, F, k, stride, padding
    ("up", 128, 32, 8, 64, 5, 1, 2),       # few tiles: the reduction of convUp is split over workgroups and summed by a second kernel
    ("down", 128, 32, 8, 64, 5, 1, 2),     # the same for convDown
    ("outp", 128, 3, 32, 64, 5, 1, 2),     # config 4: one partial block per workgroup and a finishing kernel
    ("down", 128, 3, 32, 64, 5, 1, 2),     # config 4: wavefronts of a workgroup meet in LDS
    ("outp", 128, 32, 8, 64, 5, 1, 2),     # the general split-K kernel
]


@pytest.mark.parametrize("which,N,C,H,F,k,s,p", CONV_SOAKS)
def test_conv_passes_repeat_bit_for_bit(cm, cc, which, N, C, H, F, k, s, p):
    from oracle import conv_oracle as co
    rng = np.random.default_rng(94)
    Mx = co.n_modules(H, k, s, p)
    X = cm.CUDAMatrix(_f(rng.standard_normal((N, C * H * H))))
    W = cm.CUDAMatrix(_f(0.1 * rng.standard_normal((F, C * k * k))))
    Y = cm.CUDAMatrix(_f(rng.standard_normal((N, F * Mx * Mx))))
    shape = {"up": (N, F * Mx * Mx), "down": (N, C * H * H), "outp": (F, C * k * k)}[which]
    outs = [cm.empty(shape) for _ in range(4)]
    noise = _Noise(cm, rng)

    def launch(slot):
        if which == "up":
            cc.convUp(X, W, outs[slot], Mx, p, s, C)
        elif which == "down":
            cc.convDown(Y, W, outs[slot], Mx, p, s, k, H, C)
        else:
            cc.convOutp(X, Y, outs[slot], Mx, p, k, s, C)

    _soak(cm, launch, lambda slot: outs[slot].asarray(), noise)
