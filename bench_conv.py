"""Convolution leg of bench.py: the three conv passes, local max-pool and response
norm at the benchmark's layer shapes, timed with HIP events on the NULL stream.

  C4   3x32x32 -> 64 @ 5x5, stride 1, padding 2, batch 128; pool 3x3/2 -> 15x15; rnorm 5
  C5a  3x224x224 -> 96 @ 11x11, stride 4, no padding, batch 128
  C5b  96x27x27 -> 256 @ 5x5, padding 2, 2 groups, batch 128
"""
import numpy as np

MFMA_FP32_PEAK_TFLOPS = 157.3
HBM_PEAK_GBS = 8000.0

LAYERS = {
    'c4_3x32x32_64f5': dict(N=128, C=3, H=32, F=64, k=5, s=1, p=2, G=1),
    'c5a_3x224x224_96f11s4': dict(N=128, C=3, H=224, F=96, k=11, s=4, p=0, G=1),
    'c5b_96x27x27_256f5g2': dict(N=128, C=96, H=27, F=256, k=5, s=1, p=2, G=2),
}


WARM_MS = 30.0   # the core clock under matrix-core load needs a few tens of ms to settle


def _time(ev, fn, iters, sync):
    import time
    fn()
    sync()
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < WARM_MS:
        for _ in range(5):
            fn()
        sync()
    e0, e1 = ev.new(), ev.new()
    reps = []
    for _ in range(3):      # median of three groups of `iters` back-to-back launches
        ev.record(e0)
        for _ in range(iters):
            fn()
        ev.record(e1)
        reps.append(ev.elapsed_ms(e0, e1) / iters)
    return sorted(reps)[1]


def run(cm, ev, iters=10):
    from deepnet_amd import cudamat_conv as cc
    rng = np.random.default_rng(5)
    f = lambda a: cm.CUDAMatrix(np.asarray(a, dtype=np.float32, order='F'))
    out = {}
    for name, L in LAYERS.items():
        N, C, H, F, k, s, p, G = (L[x] for x in ('N', 'C', 'H', 'F', 'k', 's', 'p', 'G'))
        Mx = (H + 2 * p - k) // s + 1
        X = f(rng.standard_normal((N, C * H * H)))
        W = f(0.01 * rng.standard_normal((F, (C // G) * k * k)))
        Y = f(rng.standard_normal((N, F * Mx * Mx)))
        up, down, dw = cm.empty((N, F * Mx * Mx)), cm.empty((N, C * H * H)), cm.empty((F, (C // G) * k * k))
        flops = 2.0 * N * F * Mx * Mx * (C // G) * k * k
        res = {'gflop_per_pass': round(flops / 1e9, 3)}
        for label, fn in (('convUp', lambda: cc.convUp(X, W, up, Mx, p, s, C, G)),
                          ('convDown', lambda: cc.convDown(Y, W, down, Mx, p, s, k, H, C, numGroups=G)),
                          ('convOutp', lambda: cc.convOutp(X, Y, dw, Mx, p, k, s, C, numGroups=G))):
            ms = _time(ev, fn, iters, cm.cuda_sync_threads)
            tf = flops / (ms * 1e-3) / 1e12
            res[label] = {'ms': round(ms, 4), 'tflops': round(tf, 2),
                          'frac_mfma_fp32': round(tf / MFMA_FP32_PEAK_TFLOPS, 4)}
        if name.startswith('c4'):
            O = 15
            pooled, grad = cm.empty((N, F * O * O)), f(rng.standard_normal((N, F * O * O)))
            undo = cm.empty((N, F * Mx * Mx))
            den, normed, nundo = cm.empty((N, F * O * O)), cm.empty((N, F * O * O)), cm.empty((N, F * O * O))
            acts = cm.empty((N, F * O * O))
            e_in, e_out = 4.0 * N * F * Mx * Mx, 4.0 * N * F * O * O
            for label, fn, nbytes in (
                    ('MaxPool', lambda: cc.MaxPool(up, pooled, F, 3, 0, 2, O), e_in + e_out),
                    ('MaxPoolUndo', lambda: cc.MaxPoolUndo(up, undo, grad, pooled, 3, 0, 2, O), 2 * e_in + 2 * e_out),
                    ('ResponseNorm', lambda: cc.ResponseNorm(pooled, den, normed, F, 5, 0.001, 0.75), 3 * e_out),
                    ('ResponseNormUndo', lambda: (acts.assign(normed),
                                                  cc.ResponseNormUndo(grad, den, pooled, acts, nundo, F, 5, 0.001, 0.75)),
                     (2 + 7) * e_out)):
                ms = _time(ev, fn, iters, cm.cuda_sync_threads)
                gbs = nbytes / (ms * 1e-3) / 1e9
                res[label] = {'us': round(ms * 1e3, 2), 'gbs': round(gbs, 1), 'frac_hbm': round(gbs / HBM_PEAK_GBS, 4)}
            # the two pairs deepnet issues back to back, each as one launch (extensions of this backend):
            # algorithmic bytes = the un-pooled map in + three pooled-size arrays out; four pooled-size arrays and the
            # un-pooled map in + the un-pooled gradient out
            p2, d2, n2 = cm.empty((N, F * O * O)), cm.empty((N, F * O * O)), cm.empty((N, F * O * O))
            for label, fn, nbytes in (
                    ('MaxPoolResponseNorm', lambda: cc.MaxPoolResponseNorm(up, p2, d2, n2, F, 3, 0, 2, O, 5, 0.001, 0.75),
                     e_in + 3 * e_out),
                    ('ResponseNormUndoMaxPoolUndo', lambda: cc.ResponseNormUndoMaxPoolUndo(grad, d2, n2, p2, up, undo, F, 3, 0, 2, O,
                                                                                          5, 0.001, 0.75), 2 * e_in + 4 * e_out)):
                ms = _time(ev, fn, iters, cm.cuda_sync_threads)
                gbs = nbytes / (ms * 1e-3) / 1e9
                res[label] = {'us': round(ms * 1e3, 2), 'gbs': round(gbs, 1), 'frac_hbm': round(gbs / HBM_PEAK_GBS, 4)}
            res['stage_fwd_bwd'] = _stage(cm, ev, iters, L, W, rng)
            res['stage_fwd_bwd_fused_pool_norm'] = _stage(cm, ev, iters, L, W, rng, fused=True)
        out[name] = res
        for m in (X, W, Y, up, down, dw):
            m.free_device_memory()
    out['local_64x8x8_64f3'] = _local(cm, cc, ev, iters, rng)
    return {'conv': out}


def _local(cm, cc, ev, iters, rng):
    """A locally connected layer (unshared filters: one bank per module) at batch 128:
    64 colours on 8 x 8 maps, 64 filters of 3 x 3, padding 1 (64 modules)."""
    N, C, H, F, k, s, p = 128, 64, 8, 64, 3, 1, 1
    Mx = (H + 2 * p - k) // s + 1
    M = Mx * Mx
    f = lambda a: cm.CUDAMatrix(np.asarray(a, dtype=np.float32, order='F'))
    X, W, Y = f(rng.standard_normal((N, C * H * H))), f(0.01 * rng.standard_normal((F, M * C * k * k))), f(rng.standard_normal((N, F * M)))
    up, down, dw = cm.empty((N, F * M)), cm.empty((N, C * H * H)), cm.empty((F, M * C * k * k))
    flops = 2.0 * N * F * M * C * k * k
    res = {'gflop_per_pass': round(flops / 1e9, 3)}
    for label, fn in (('localUp', lambda: cc.localUp(X, W, up, Mx, p, s, C)),
                      ('localDown', lambda: cc.localDown(Y, W, down, Mx, p, s, k, H, C)),
                      ('localOutp', lambda: cc.localOutp(X, Y, dw, Mx, p, k, s, C))):
        ms = _time(ev, fn, iters, cm.cuda_sync_threads)
        tf = flops / (ms * 1e-3) / 1e12
        res[label] = {'ms': round(ms, 4), 'tflops': round(tf, 2), 'frac_mfma_fp32': round(tf / MFMA_FP32_PEAK_TFLOPS, 4)}
    for m in (X, W, Y, up, down, dw):
        m.free_device_memory()
    return res


def _stage(cm, ev, iters, L, W, rng, fused=False):
    """The whole conv stage of a deepnet edge at this layer (transpose, convUp, pool 3x3/2,
    rnorm 5, transpose; then the backward pass and the weight gradient) through
    deepnet_amd/convolutions.py: twelve library calls per step."""
    import types
    from deepnet_amd import convolutions as cv_mod
    N, C, H, F, k, s, p = (L[x] for x in ('N', 'C', 'H', 'F', 'k', 's', 'p'))
    cv = cv_mod.ConvParams(size=k, stride=s, padding=p, num_filters=F, num_colors=C, max_pool=True, pool_size=3,
                           pool_stride=2, rnorm=True, norm_size=5)
    O = ((H + 2 * p - k) // s + 1 - 3) // 2 + 1
    f = lambda a: cm.CUDAMatrix(np.asarray(a, dtype=np.float32, order='F'))
    inputs, deriv = f(rng.standard_normal((C * H * H, N))), f(rng.standard_normal((F * O * O, N)))
    edge = cv_mod.ConvEdge(W, cv, inputs.shape, deriv.shape)
    edge.fused = fused
    state, grad = cm.empty(deriv.shape), cm.empty(W.shape)
    layer = types.SimpleNamespace(dirty=False, is_input=False, deriv=cm.empty(inputs.shape))

    def step():
        layer.dirty = False
        cv_mod.ConvolveUp(inputs, edge, state)
        cv_mod.AccumulateConvDeriv(layer, edge, deriv)
        cv_mod.ConvOuter(edge, grad)
    ms = _time(ev, step, iters, cm.cuda_sync_threads)
    edge.free_device_memory()
    return {'us': round(ms * 1e3, 1), 'steps_per_sec': round(1e3 / ms, 1)}
