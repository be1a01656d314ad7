"""Brute-force pins for the edge rules the reference has no test of its own for: the scan order
that decides arg-max ties, the scan of ProbMaxPool, and the rule that every tied pixel receives
the gradient in MaxPoolUndo.  Each oracle function is compared, on inputs small enough to
enumerate every tie pattern, with a second formulation written from the other end (a closed
form of the tie order; a scalar per-thread walk; a per-pixel gather instead of a per-window
scatter).  CPU only; tests/test_gpu_pins.py runs the same enumerations on the device."""
import itertools

import numpy as np

from oracle import conv_oracle as co, cudamat_oracle as orc

FLT_MAX = float(np.finfo(np.float32).max)


# ------------------------------------------------------------------ arg-max tie order

def argmax_closed_form(col):
    """What the 32-lane scan of cudamat_kernels.cu:1020-1050 amounts to: among the rows holding
    the column's maximum, the one in the lowest lane (row % 32), and the first row of that lane;
    row 0 when nothing is greater than -FLT_MAX (NaN never compares greater)."""
    col = np.asarray(col, dtype=np.float32)
    cand = [i for i, v in enumerate(col) if v > -np.float32(FLT_MAX)]
    if not cand:
        return 0
    m = max(col[i] for i in cand)
    return min((i for i in cand if col[i] == m), key=lambda i: (i % 32, i))


def tie_columns(h):
    """Every column of height h with one, two or three rows at the maximum (the rest lower, at
    two different levels so that 'lower but not lowest' rows exist too)."""
    cols = []
    for k in (1, 2, 3):
        for pos in itertools.combinations(range(h), k):
            c = np.where(np.arange(h) % 3 == 0, -1.0, 0.0).astype(np.float32)
            c[list(pos)] = 2.0
            cols.append(c)
    return np.stack(cols, axis=1)


def test_argmax_scan_equals_the_closed_form_on_every_tie_pattern():
    x = tie_columns(40)                          # 40 + 780 + 9880 columns; rows 32..39 share lanes 0..7
    for j in range(x.shape[1]):
        assert orc.argmax_ref_order(x[:, j]) == argmax_closed_form(x[:, j])
    # heights around the lane count, all two-row ties
    for h in (1, 2, 31, 32, 33, 64, 65, 70):
        for pos in itertools.combinations(range(h), min(2, h)):
            c = np.full(h, -3.0, dtype=np.float32)
            c[list(pos)] = 7.0
            assert orc.argmax_ref_order(c) == argmax_closed_form(c)
    # nothing beats the start value
    for fill in (-FLT_MAX, -np.inf, np.nan):
        c = np.full(50, fill, dtype=np.float32)
        assert orc.argmax_ref_order(c) == argmax_closed_form(c) == 0
    c = np.full(50, np.nan, dtype=np.float32); c[37] = -5.0; c[5] = -5.0
    assert orc.argmax_ref_order(c) == argmax_closed_form(c) == 5
    rng = np.random.default_rng(0)
    for _ in range(300):
        c = rng.integers(0, 4, rng.integers(1, 200)).astype(np.float32)     # many ties
        assert orc.argmax_ref_order(c) == argmax_closed_form(c)
    assert orc.get_softmax_correct(x[:, :5], [orc.argmax_ref_order(x[:, j]) for j in range(5)]).tolist() == [[1.0] * 5]


# ------------------------------------------------------------------ ProbMaxPool scan

PROB_VALUES = [(1.0, 0.5), (-1.0, 0.5), (3e38, 3e38), (-3e38, 3e38), (np.inf, 1.0), (np.nan, 1.0), (2.0, 0.0), (1e30, 1e30)]


def prob_pool_scalar(window):
    """One thread of kLocalProbPool (cudamat_conv_kernels.cuh:1594-1608) over its window, value
    by value in float32: agg() returns 0 (keep) when prod * rnd_used > img * rnd."""
    prod, used = np.float32(-2e38), np.float32(-2e38)
    with np.errstate(over='ignore', invalid='ignore'):
        for img, r in window:
            img, r = np.float32(img), np.float32(r)
            res = 0 if prod * used > img * r else 1
            if res:
                prod, used = img, r
    return prod


def prob_inputs():
    """All 8^4 assignments of PROB_VALUES to the four pixels of a 2x2 map, as the images of one
    batch: one 2x2 window covers the map, pixel order (0,0), (0,1), (1,0), (1,1)."""
    seqs = list(itertools.product(range(len(PROB_VALUES)), repeat=4))
    x = np.array([[PROB_VALUES[i][0] for i in s] for s in seqs], dtype=np.float32)
    r = np.array([[PROB_VALUES[i][1] for i in s] for s in seqs], dtype=np.float32)
    return seqs, x, r


def test_prob_max_pool_scan_equals_a_scalar_walk_on_every_sequence():
    seqs, x, r = prob_inputs()
    got = co.prob_max_pool(x, r, 1, 2, 0, 2, 1)
    want = np.array([prob_pool_scalar([PROB_VALUES[i] for i in s]) for s in seqs], dtype=np.float64)
    assert np.array_equal(got[:, 0], want, equal_nan=True)
    # the start value's product overflows to +inf, so only a candidate whose own product is +inf
    # or NaN can ever replace it: finite inputs leave -2e38
    finite = [k for k, s in enumerate(seqs) if all(i in (0, 1, 6) for i in s)]
    assert np.all(got[finite, 0] == np.float64(np.float32(-2e38)))
    assert np.any(got[:, 0] != np.float64(np.float32(-2e38)))


# ------------------------------------------------------------------ MaxPoolUndo: tied pixels

def pool_undo_gather(img, grads, acts, S, subs, start, stride, O):
    """One pixel at a time, as kLocalMaxUndo walks (cudamat_conv_kernels.cuh:1455-1502): the
    outputs whose window holds the pixel, from the bounds the kernel computes, adding the
    gradient of every output whose maximum equals the pixel."""
    out = np.zeros(S * S)
    for py in range(S):
        for px in range(S):
            lo, hi = start, start + stride * (O - 1) + subs
            if not (lo <= px < hi and lo <= py < hi):
                continue
            oy0 = 0 if py - start < subs else 1 + (py - start - subs) // stride
            oy1 = min(O, 1 + (py - start) // stride)
            ox0 = 0 if px - start < subs else 1 + (px - start - subs) // stride
            ox1 = min(O, 1 + (px - start) // stride)
            for my in range(oy0, oy1):
                for mx in range(ox0, ox1):
                    o = my * O + mx
                    out[py * S + px] += (img[py * S + px] == acts[o]) * grads[o]
    return out


POOL_UNDO_CASES = [(3, 2, 0, 1), (3, 2, 0, 2), (3, 3, -1, 2), (4, 2, 0, 2), (4, 3, 0, 1)]      # S, subs, start, stride


def pool_undo_inputs(S, subs, start, stride):
    O = (S - start - subs + stride - 1) // stride + 1
    n = min(2 ** (S * S), 4096)
    bits = np.arange(n) if n == 2 ** (S * S) else np.random.default_rng(S).integers(0, 2 ** (S * S), n)
    imgs = ((bits[:, None] >> np.arange(S * S)) & 1).astype(np.float32)      # every 0/1 image: every tie pattern
    grads = (1.0 + np.arange(O * O) * 0.25)[None, :].repeat(n, axis=0).astype(np.float32)
    return O, imgs, grads


def test_max_pool_undo_gives_every_tied_pixel_the_gradient():
    for S, subs, start, stride in POOL_UNDO_CASES:
        O, imgs, grads = pool_undo_inputs(S, subs, start, stride)
        acts = co.max_pool(imgs, 1, subs, start, stride, O)
        got = co.max_pool_undo(imgs, grads, acts, subs, start, stride, O)
        for n in range(0, imgs.shape[0], 7):
            want = pool_undo_gather(imgs[n], grads[n].astype(np.float64), acts[n], S, subs, start, stride, O)
            assert np.array_equal(got[n], want), (S, subs, start, stride, n)
        # the gradient of an output goes, whole, to each pixel of its window at the maximum
        total = np.zeros(imgs.shape[0])
        x = imgs.reshape(-1, S, S)
        for oy in range(O):
            for ox in range(O):
                y0, x0 = max(0, start + oy * stride), max(0, start + ox * stride)
                y1, x1 = min(S, start + oy * stride + subs), min(S, start + ox * stride + subs)
                win = x[:, y0:y1, x0:x1].reshape(len(x), -1)
                total += (win == win.max(axis=1, keepdims=True)).sum(axis=1) * grads[:, oy * O + ox]
        assert np.allclose(got.sum(axis=1), total)
