"""Recorded step sequences (cm.Graph: graph_capture_begin / _end / graph_launch of the C ABI)
against the same steps run call by call: every replay is compared bit for bit, with eager
work and synchronisations between the replays."""
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench          # noqa: E402

pytestmark = pytest.mark.gpu


def _bits(m):
    return m.asarray().view(np.uint32).copy()


def _eager_between(cm, rng):
    """Unrelated work and a synchronisation, as a program would do between two replays."""
    a = cm.CUDAMatrix(np.asarray(rng.standard_normal((300, 70)), dtype=np.float32, order='F'))
    b = cm.empty((300, 70))
    a.apply_sigmoid(target=b)
    s = b.sum(axis=1)
    total = float(s.asarray().sum())
    for m in (a, b, s):
        m.free_device_memory()
    return total


@pytest.mark.parametrize("kind,fused", [('rbm', False), ('rbm', True), ('mlp', False), ('mlp', True)])
def test_replays_equal_eager_steps(cm, kind, fused):
    rng = np.random.default_rng(5)
    make = (lambda: bench.RBM(cm)) if kind == 'rbm' else (lambda: bench.MLP(cm))
    # (the fused MLP step does not materialise its dropout masks)
    params = (lambda o: [o.W, o.bv, o.bh, o.h, o.v2]) if kind == 'rbm' else (lambda o: o.W + o.b + o.dW + [o.loss] + ([] if fused else o.mask))
    # reference: five steps call by call
    cm.CUDAMatrix.init_random(11)
    ref = make()
    want = []
    for _ in range(5):
        (ref.step_fused if fused else ref.step)()
        want.append([_bits(m) for m in params(ref)])
    # same start: one eager step (workspaces reach their sizes), then the step is recorded once
    # (recording runs nothing) and replayed four times
    cm.CUDAMatrix.init_random(11)
    obj = make()
    step = obj.step_fused if fused else obj.step
    step()
    for got, w in zip([_bits(m) for m in params(obj)], want[0]):
        assert np.array_equal(got, w)
    with cm.Graph() as g:
        step()
    for got, w in zip([_bits(m) for m in params(obj)], want[0]):
        assert np.array_equal(got, w)                   # recording changed nothing
    for i in range(1, 5):
        g.launch()
        got = [_bits(m) for m in params(obj)]            # (reading back waits for the replay)
        for a, w in zip(got, want[i]):
            assert np.array_equal(a, w), (kind, fused, i)
        _eager_between(cm, rng)
    g.free()


def test_conv_stage_is_recorded_with_the_matrix_ops(cm, cc):
    rng = np.random.default_rng(6)
    N, C, H, F, k, p = 128, 3, 16, 32, 5, 2
    f = lambda a: cm.CUDAMatrix(np.asarray(a, dtype=np.float32, order='F'))
    x, w = f(rng.standard_normal((N, C * H * H))), f(0.1 * rng.standard_normal((F, C * k * k)))
    up, pooled = cm.empty((N, F * H * H)), cm.empty((N, F * 7 * 7))
    den, normed = cm.empty(pooled.shape), cm.empty(pooled.shape)

    def stage():
        cc.convUp(x, w, up, H, p, 1, C)
        up.lower_bound(0)
        cc.MaxPool(up, pooled, F, 3, 0, 2, 7)
        cc.ResponseNorm(pooled, den, normed, F, 5, 0.001, 0.75)
    stage()
    want = _bits(normed)
    with cm.Graph() as g:
        stage()
    for i in range(3):
        normed.assign(0)
        x.mult(1.0)
        g.launch()
        assert np.array_equal(_bits(normed), want)
    # new inputs in the same buffers: the replay works on what the buffers hold now
    x.assign(f(rng.standard_normal((N, C * H * H))))
    g.launch()
    got = _bits(normed)
    stage()
    assert np.array_equal(got, _bits(normed)) and not np.array_equal(got, want)
    g.free()


def test_split_conv_layer_records_with_and_without_its_workspace(cm, cc):
    """A conv layer whose reduction is split over workgroups (partial outputs in the grow-only
    workspace): recorded after an eager call it replays the split form; recorded in a fresh
    process state, where the workspace would have to grow, it records the unsplit form.  Both
    give the eager result to rounding."""
    rng = np.random.default_rng(9)
    N, C, H, F, k, p = 128, 64, 16, 64, 5, 2
    f = lambda a: cm.CUDAMatrix(np.asarray(a, dtype=np.float32, order='F'))
    x, w = f(rng.standard_normal((N, C * H * H))), f(0.05 * rng.standard_normal((F, C * k * k)))
    up1, up2, up3 = cm.empty((N, F * H * H)), cm.empty((N, F * H * H)), cm.empty((N, F * H * H))
    with cm.Graph() as g_first:                       # whatever workspace earlier tests left: may or may not suffice
        cc.convUp(x, w, up1, H, p, 1, C)
    g_first.launch()
    cc.convUp(x, w, up2, H, p, 1, C)                  # eager: the workspace has its size now
    with cm.Graph() as g_second:
        cc.convUp(x, w, up3, H, p, 1, C)
    g_second.launch()
    a, b, c = up1.asarray(), up2.asarray(), up3.asarray()
    assert np.array_equal(b.view(np.uint32), c.view(np.uint32))
    scale = np.abs(b).max()
    assert np.max(np.abs(a - b)) <= 1e-5 * scale
    g_first.free(); g_second.free()


def test_what_cannot_be_recorded_raises(cm):
    a = cm.CUDAMatrix(np.ones((8, 8), dtype=np.float32))
    with pytest.raises(cm.CUDAMatException):
        with cm.Graph():
            a.asarray()
    with pytest.raises(cm.CUDAMatException):
        with cm.Graph():
            cm.empty((4, 4))
    with pytest.raises(cm.CUDAMatException):
        with cm.Graph():
            a.euclid_norm()
    # the library is back on the NULL stream and works as before
    a.add(1.0)
    assert np.array_equal(a.asarray(), np.full((8, 8), 2.0, dtype=np.float32))
    with cm.Graph() as g:
        a.add(1.0)
    assert np.array_equal(a.asarray(), np.full((8, 8), 2.0, dtype=np.float32))
    g.launch(); g.launch()
    assert np.array_equal(a.asarray(), np.full((8, 8), 4.0, dtype=np.float32))
    g.free()


def test_replays_survive_growth_of_the_library_workspaces(cm):
    """A recorded reduction carries the addresses of the workspace, the arrival counters and
    the vector of ones it used.  Later eager calls that outgrow them get new ones; the old
    blocks stay allocated, and the replay still gives the recorded result."""
    rng = np.random.default_rng(3)
    x = np.asarray(rng.uniform(-1, 1, (64, 8192)), dtype=np.float32, order='F')
    a, r1, r0 = cm.CUDAMatrix(x), cm.empty((64, 1)), cm.empty((1, 8192))
    a.sum(axis=1, target=r1); a.sum(axis=0, target=r0)            # eagerly once: the workspaces reach their sizes
    want1, want0 = r1.asarray().copy(), r0.asarray().copy()
    with cm.Graph() as g:
        a.sum(axis=1, target=r1)
        a.sum(axis=0, target=r0)
    # a product whose split reduction needs a larger workspace, a sum that needs a longer vector of ones
    p = cm.CUDAMatrix(np.asarray(rng.uniform(-1, 1, (256, 32768)), dtype=np.float32, order='F'))
    q = cm.CUDAMatrix(np.asarray(rng.uniform(-1, 1, (32768, 256)), dtype=np.float32, order='F'))
    pq = cm.dot(p, q)
    ref = p.asarray().astype(np.float64) @ q.asarray().astype(np.float64)
    assert np.max(np.abs(pq.asarray() - ref)) <= 1e-4 * np.max(np.abs(p.asarray()).astype(np.float64) @ np.abs(q.asarray()))
    long = cm.CUDAMatrix(np.ones((cm.MAX_ONES + 4096, 2), dtype=np.float32))
    assert np.array_equal(long.sum(axis=0).asarray(), np.full((1, 2), cm.MAX_ONES + 4096, dtype=np.float32))
    for _ in range(2):
        r1.assign(0); r0.assign(0)
        g.launch()
        assert np.array_equal(r1.asarray(), want1) and np.array_equal(r0.asarray(), want0)
    g.free()


def test_the_entry_point_that_allocates_nothing_is_recorded(cm):
    """max_by_axis_noalloc is meant for callers under graph capture: recorded along axis 1 on a
    matrix wide enough for column slices (partials and arrival counters of the fixed workspace in
    use), replayed with eager work in between on inputs that change between the replays, every
    replay compared bit for bit with the eager call on the same input."""
    rng = np.random.default_rng(17)
    x = cm.CUDAMatrix(np.asarray(rng.uniform(-1, 1, (2048, 4096)), dtype=np.float32, order='F'))
    got, want = cm.empty((2048, 1)), cm.empty((2048, 1))
    x.max_noalloc(1, got)                   # once eagerly: the workspace's address is looked up here
    with cm.Graph() as g:
        x.mult(-0.75)                       # the input changes from replay to replay
        x.max_noalloc(1, got)
    for _ in range(4):
        g.launch()
        x.max(1, want)
        assert np.array_equal(_bits(got), _bits(want))
        assert np.array_equal(got.asarray()[:, 0], x.asarray().max(axis=1))
        _eager_between(cm, rng)
    g.free()
