"""GPU parity of convUp / convDown / convOutp, MaxPool(+Undo), ResponseNorm(+Undo)
against the float64 restatement: 1e-4 relative for the convolutions (error measured
against the sum of magnitudes, as for dot), exact for pooling, 2e-6 relative for the
normalisation's denominators and 1e-5 for its outputs (x^-p through the hardware log2 / exp2,
as the reference's __powf).  Shapes with a batch that is not a multiple of 16 run the
one-lane-per-output kernels; the others the matrix-core kernel."""
import numpy as np
import pytest

from oracle import conv_oracle as co

pytestmark = pytest.mark.gpu

REL = 1e-4

CASES = [  # N, C, H, F, k, stride, padding, groups
    (2, 3, 6, 16, 3, 1, 1, 1),       # direct kernels (batch 2)
    (3, 4, 7, 8, 3, 2, 1, 2),
    (16, 3, 6, 16, 3, 1, 1, 1),      # matrix-core kernels from here on
    (16, 3, 8, 16, 5, 1, 2, 1),
    (32, 1, 9, 32, 3, 1, 0, 1),
    (16, 3, 12, 16, 5, 4, 0, 1),     # strided; last module stops short of the edge
    (16, 3, 13, 48, 4, 3, 2, 1),     # stride 3, 48 filters (3 column blocks)
    (32, 8, 7, 32, 3, 1, 1, 2),      # 2 groups of 4 colours / 16 filters
    (16, 32, 6, 64, 3, 2, 1, 2),
    (128, 3, 32, 64, 5, 1, 2, 1),    # the CIFAR layer of the benchmark
    (16, 48, 9, 160, 3, 1, 1, 1),    # more than 128 filters: two column tiles
    (128, 48, 6, 32, 3, 1, 1, 2),    # batch 128: the uniform-row (buffer load) kernels, 24 colours per group
    (128, 40, 7, 48, 3, 2, 1, 1),    # the same with stride 2 (four phases in convDown), 40 colours
    (256, 20, 5, 144, 4, 1, 2, 1),   # batch 256, 144 filters (two column tiles), padding 2 > k/2
    (128, 3, 12, 16, 5, 4, 0, 1),    # few colours, strided, batch 128: convDown with the phases merged into columns
    (128, 3, 13, 32, 4, 3, 2, 1),    # the same: stride 3 does not divide k = 4, padding 2
    (128, 4, 9, 32, 3, 2, 1, 2),     # the same: 2 groups of 2 colours
    (256, 8, 8, 16, 5, 2, 2, 1),     # the same: 8 colours x 4 phases = 32 columns, batch 256
    (128, 16, 7, 16, 3, 3, 0, 1),    # the same: 16 colours x 9 phases = 144 columns (two column tiles), stride == k
    (64, 3, 10, 48, 5, 1, 2, 1),     # convUp with the filter bank in registers: 48 filters (a half-used column block)
    (96, 1, 11, 64, 5, 2, 1, 1),     # the same: 3 image blocks per module, 25 taps, stride 2
    (32, 5, 6, 16, 4, 1, 3, 1),      # the same: exactly 80 taps, padding 3 (every module touches the padding)
    (32, 2, 9, 128, 3, 1, 1, 2),     # the same: 2 groups of 64 filters
    (128, 48, 7, 32, 5, 1, 2, 1),    # uniform-row kernels with 16-wide column blocks: convDown onto 48 colours
    (128, 16, 8, 48, 5, 1, 2, 1),    # the same: convUp onto 48 filters, convDown onto 16 colours (one block of 16)
    (128, 96, 6, 64, 5, 1, 2, 2),    # the same in 2 groups of 48 colours / 32 filters (the shape of config 5b)
    (128, 32, 6, 160, 3, 1, 1, 1),   # uniform-row kernels, more than 96 columns on few tiles: 64-wide column tiles (convUp: 64 + 64 + 32 filters)
    (128, 160, 6, 32, 3, 1, 1, 1),   # the same for convDown onto 160 colours
    (128, 64, 5, 224, 3, 1, 1, 2),   # the same in 2 groups: 112 filters per group (64 + 48)
    (128, 224, 5, 64, 3, 1, 1, 2),   # ... and 112 colours per group in convDown
    (128, 32, 14, 256, 3, 1, 1, 1),  # full 128-wide column tiles and enough of them: the wide kernel stays
    (32, 16, 6, 192, 3, 1, 1, 1),    # convOutp with 192 filters: two 96-row tiles instead of two 128-row ones
    (32, 32, 5, 320, 3, 1, 1, 2),    # the same in 2 groups of 160 filters (96 + 64)
    (128, 32, 8, 64, 5, 1, 2, 1),    # a small map with a long reduction: convUp / convDown split their reduction over workgroups
    (128, 64, 4, 96, 3, 1, 1, 2),    # the same in 2 groups of 32 colours / 48 filters (three 16-wide column blocks in convUp)
    (100, 1, 12, 64, 5, 1, 2, 1),    # batch 100 (deepnet's examples): operands padded to 128 images, register / uniform-row kernels
    (100, 32, 7, 32, 3, 1, 1, 1),    # the same with many colours
    (50, 4, 7, 32, 3, 2, 1, 2),      # batch 50 -> 64, strided, 2 groups
    (20, 3, 6, 16, 5, 1, 2, 1),      # batch 20 -> 32
    (200, 16, 5, 48, 3, 1, 1, 1),    # batch 200 -> 256
    (36, 2, 6, 16, 3, 1, 0, 1),      # batch 36 -> 64 with a batch-indexed result that must not spill into its neighbours
    (128, 1, 12, 20, 5, 1, 0, 1),    # 20 filters (a LeNet-like first layer): filter bank and hidden maps padded to 32 filters
    (128, 20, 8, 50, 5, 1, 0, 1),    # 20 colours -> 50 filters (padded to 64)
    (100, 3, 8, 10, 3, 1, 1, 1),     # batch 100 and 10 filters: both paddings at once
    (64, 4, 9, 24, 3, 2, 1, 1),      # 24 filters, strided
    # convDown of stride-1 layers with at most 4 colours (4 x 4 x 1 matrix-core blocks, pixels in registers):
    (32, 4, 7, 8, 3, 1, 2, 1),       # 4 colours, 8 filters (one pair per wavefront), map not a multiple of the 4 x 4 tile
    (96, 3, 13, 24, 5, 1, 4, 1),     # padding k - 1: the module grid is larger than the image
    (64, 8, 6, 144, 3, 1, 0, 2),     # 2 groups of 4 colours / 72 filters, no padding
    (32, 2, 9, 128, 5, 1, 1, 1),     # 128 filters in one group
    (160, 1, 5, 40, 5, 1, 3, 1),     # one colour, 5 image blocks, a single tile row
    # convUp with one (module, 64 images) tile per wavefront (1 or 3 colours, 3 x 3 or 5 x 5 filters, batch a multiple of 64):
    (64, 3, 9, 16, 3, 2, 1, 1),      # stride 2, 16 filters (one block of 32, half used)
    (192, 1, 7, 64, 3, 1, 2, 1),     # one colour, padding wider than half the filter, three image tiles per module
    (64, 6, 8, 128, 5, 1, 2, 2),     # 2 groups of 3 colours / 64 filters
    (128, 3, 6, 8, 5, 1, 4, 1),      # 8 filters, every module touches the padding
    (64, 3, 11, 40, 5, 3, 0, 1),     # 40 filters (second block of 32 a quarter used), stride 3, last module short of the edge
    # convOutp with at most 64 x 80 outputs (operands straight into 16 x 16 x 4 blocks, a wavefront per run of (module, 16 images) chunks):
    (48, 2, 7, 8, 3, 1, 1, 1),       # 3 chunks per module (an odd number for two register sets), 8 filters, 18 columns
    (16, 5, 6, 56, 4, 2, 3, 1),      # exactly 80 columns, 56 filters (last block half used), stride 2, padding 3
    (80, 3, 5, 24, 3, 1, 1, 1),      # 5 chunks per module, fewer chunks than wavefronts
    (64, 3, 40, 32, 3, 1, 1, 1),     # enough chunks for two filter slices per module range (grid y)
    (32, 8, 9, 96, 3, 1, 1, 2),      # 2 groups of 4 colours / 48 filters
    # convOutp with 81 to 96 patch columns and at most 64 filters ([row][image] LDS tiles, 32-wide column blocks):
    (64, 6, 8, 32, 4, 1, 1, 1),      # 96 columns, 32 filters
    (128, 9, 7, 64, 3, 1, 1, 1),     # 81 columns, 64 filters, two chunks of 64 images per module
]


def _f(a):
    return np.asarray(a, dtype=np.float32, order='F')


def _relerr(got, want, bound):
    """The larger of two measures: every element against the bound |x| * |w| of its own sum
    (robust to cancellation), and the whole result against its own size (Frobenius norms, ten
    times stricter: REL / 10 = 1e-5 relative to the result itself)."""
    got = np.asarray(got, np.float64)
    elementwise = np.max(np.abs(got - want) / (bound + 1e-30))
    whole = np.linalg.norm(got - want) / (np.linalg.norm(want) + 1e-30)
    return max(elementwise, 10.0 * whole)


@pytest.mark.parametrize("N,C,H,F,k,s,p,G", CASES)
def test_three_conv_passes(cm, cc, rng, N, C, H, F, k, s, p, G):
    Mx = co.n_modules(H, k, s, p)
    x = _f(rng.standard_normal((N, C * H * H)))
    w = _f(0.1 * rng.standard_normal((F, (C // G) * k * k)))
    y = _f(rng.standard_normal((N, F * Mx * Mx)))
    X, W, Y = cm.CUDAMatrix(x), cm.CUDAMatrix(w), cm.CUDAMatrix(y)
    up = cm.CUDAMatrix(np.full((N, F * Mx * Mx), np.nan, dtype=np.float32))     # must be overwritten, not accumulated
    cc.convUp(X, W, up, Mx, p, s, C, G)
    assert _relerr(up.asarray(), co.conv_up(x, w, C, Mx, p, s, G), co.conv_up(np.abs(x), np.abs(w), C, Mx, p, s, G)) < REL
    down = cm.CUDAMatrix(np.full((N, C * H * H), np.nan, dtype=np.float32))
    cc.convDown(Y, W, down, Mx, p, s, k, H, C, numGroups=G)
    assert _relerr(down.asarray(), co.conv_down(y, w, C, H, p, s, G),
                   co.conv_down(np.abs(y), np.abs(w), C, H, p, s, G) + 1e-6) < REL
    outp = cm.CUDAMatrix(np.full((F, (C // G) * k * k), np.nan, dtype=np.float32))
    cc.convOutp(X, Y, outp, Mx, p, k, s, C, numGroups=G)
    assert _relerr(outp.asarray(), co.conv_outp(x, y, C, Mx, k, p, s, G),
                   co.conv_outp(np.abs(x), np.abs(y), C, Mx, k, p, s, G)) < REL
    # adjoint identities on the device results themselves
    a = float((up.asarray().astype(np.float64) * y).sum())
    b = float((down.asarray().astype(np.float64) * x).sum())
    c = float((outp.asarray().astype(np.float64) * w).sum())
    scale = float((np.abs(up.asarray()).astype(np.float64) * np.abs(y)).sum())
    assert abs(a - b) / scale < 1e-5 and abs(a - c) / scale < 1e-5
    for m in (X, W, Y, up, down, outp):
        m.free_device_memory()


def test_outp_with_partial_sums(cm, cc, rng):
    N, C, H, F, k, s, p = 16, 3, 8, 16, 3, 1, 1
    Mx = co.n_modules(H, k, s, p)
    x, y = _f(rng.standard_normal((N, C * H * H))), _f(rng.standard_normal((N, F * Mx * Mx)))
    t = cm.empty((F, Mx * C * k * k))
    cc.convOutp(cm.CUDAMatrix(x), cm.CUDAMatrix(y), t, Mx, p, k, s, C, partialSum=Mx)
    want = co.conv_outp(x, y, C, Mx, k, p, s, partial_sum=Mx)
    assert np.max(np.abs(t.asarray() - want)) < 1e-3


def test_fast_and_direct_kernels_agree(cm, cc, rng):
    """The same problem through both code paths: batch 16 (matrix cores) and the same 16
    images split as 2 batches of 8 (one lane per output)."""
    C, H, F, k, s, p = 3, 10, 16, 5, 2, 2
    Mx = co.n_modules(H, k, s, p)
    x = _f(rng.standard_normal((16, C * H * H)))
    w = _f(0.1 * rng.standard_normal((F, C * k * k)))
    W = cm.CUDAMatrix(w)
    full = cm.empty((16, F * Mx * Mx))
    cc.convUp(cm.CUDAMatrix(x), W, full, Mx, p, s, C)
    halves = []
    for part in (x[:8], x[8:]):
        t = cm.empty((8, F * Mx * Mx))
        cc.convUp(cm.CUDAMatrix(_f(part)), W, t, Mx, p, s, C)
        halves.append(t.asarray())
    assert np.allclose(full.asarray(), np.vstack(halves), rtol=1e-5, atol=1e-5)


def test_bad_shapes_raise_instead_of_aborting(cm, cc, rng):
    X = cm.CUDAMatrix(_f(rng.standard_normal((16, 3 * 36))))
    W = cm.CUDAMatrix(_f(rng.standard_normal((16, 27))))
    with pytest.raises(AssertionError):
        cc.convUp(X, W, cm.empty((16, 5)), 6, 1, 1, 3)
    with pytest.raises(cm.CUDAMatException, match="convUp"):
        cc._call('convUp', X.p_mat, W.p_mat, cm.empty((16, 16 * 36)).p_mat, 6, -1, 1, 4, 1)   # 108 % 4 colours
    host_only = cm.CUDAMatrix(_f(rng.standard_normal((16, 108))), copy_to_device=False)
    with pytest.raises(cm.CUDAMatException, match="on_device"):
        cc.MaxPool(host_only, cm.empty((16, 3 * 9)), 3, 2, 0, 2, 3)


POOLS = [  # N, F, S, subs, start, stride
    (2, 3, 8, 2, 0, 2), (5, 4, 9, 3, 0, 2), (16, 16, 32, 3, 0, 2), (16, 8, 7, 3, -1, 2), (128, 64, 32, 3, 0, 2),
    (4, 2, 6, 2, 0, 1),
    (8, 3, 9, 2, 0, 2), (12, 2, 10, 2, -1, 2), (8, 4, 11, 3, -2, 2), (4, 3, 5, 3, 0, 2), (16, 2, 8, 3, 1, 2),   # vector kernels with fixed window shapes
    (8, 2, 9, 3, 0, 3), (4, 2, 12, 4, -1, 3),    # other shapes: the general kernels
    # windows of 6 and 7, strides 1 and 2, with and without a negative start: the regime where
    # the reference changes kernels (kLocalPool2, cudamat_conv.cu:1040-1089)
    (8, 4, 12, 6, 0, 1), (8, 4, 12, 6, 0, 2), (16, 2, 13, 7, 0, 1), (16, 2, 13, 7, -3, 2), (4, 3, 14, 6, -2, 2),
    (128, 16, 16, 7, -3, 1),
    # larger maps with stride 2 from 0 (the gradient kernel that takes 2 x 2 pixels per lane: odd and
    # even sizes, windows of 3 and 2, outputs that stop short of the last rows)
    (8, 3, 55, 3, 0, 2), (4, 2, 40, 3, 0, 2), (4, 2, 41, 2, 0, 2), (8, 2, 44, 2, 0, 2), (4, 3, 47, 3, 0, 2),
]


@pytest.mark.parametrize("N,F,S,subs,start,stride", POOLS)
def test_max_pool_and_undo(cm, cc, rng, N, F, S, subs, start, stride):
    O = (S - start - subs + stride - 1) // stride + 1
    x = _f(rng.standard_normal((N, F * S * S)))
    X, T = cm.CUDAMatrix(x), cm.empty((N, F * O * O))
    cc.MaxPool(X, T, F, subs, start, stride, O)
    want = co.max_pool(x, F, subs, start, stride, O)
    assert np.array_equal(T.asarray(), want.astype(np.float32))
    g = _f(rng.standard_normal((N, F * O * O)))
    U = cm.empty((N, F * S * S))
    cc.MaxPoolUndo(X, U, cm.CUDAMatrix(g), T, subs, start, stride, O)
    # a pixel adds up to ceil(subs/stride)^2 gradients in fp32; the oracle adds them in float64
    terms = (-(-subs // stride)) ** 2
    tol = 1e-6 if terms <= 4 else 1e-5
    assert np.allclose(U.asarray(), co.max_pool_undo(x, g, want, subs, start, stride, O), rtol=tol, atol=tol)
    # ties: a constant image routes every output's gradient to all pixels of its window
    ones = cm.CUDAMatrix(np.ones((N, F * S * S), dtype=np.float32))
    cc.MaxPool(ones, T, F, subs, start, stride, O)
    cc.MaxPoolUndo(ones, U, cm.CUDAMatrix(g), T, subs, start, stride, O)
    one_np = np.ones((N, F * S * S))
    assert np.allclose(U.asarray(), co.max_pool_undo(one_np, g, co.max_pool(one_np, F, subs, start, stride, O), subs, start,
                                                     stride, O), rtol=1e-5, atol=1e-5)


def test_prob_max_pool_follows_the_reference_scan(cm, cc, rng):
    N, F, S = 16, 4, 6
    x, r = _f(rng.standard_normal((N, F * S * S))), _f(rng.random((N, F * S * S)))
    T = cm.empty((N, F * 9))
    cc.ProbMaxPool(cm.CUDAMatrix(x), cm.CUDAMatrix(r), T, F, 2, 0, 2, 3)
    assert np.array_equal(T.asarray(), co.prob_max_pool(x, r, F, 2, 0, 2, 3).astype(np.float32))


@pytest.mark.parametrize("N,F,S,size", [(2, 3, 7, 3), (16, 16, 15, 5), (5, 4, 6, 4), (128, 64, 15, 5),
                                      (8, 4, 9, 3), (8, 2, 5, 7), (12, 3, 8, 4), (4, 2, 3, 9),
                                      # sizes 6 and 8 (kCNorm2 / kRNormUndo2 in the reference,
                                      # cudamat_conv_kernels.cu:303-441); a batch that is not a multiple of
                                      # the image block; maps of 32 and 48 pixels a side (smaller image
                                      # blocks, and past what fits in LDS)
                                      (16, 4, 12, 6), (32, 2, 10, 8), (100, 8, 15, 5), (44, 3, 13, 7),
                                      (16, 4, 32, 5), (8, 2, 48, 3), (16, 2, 22, 6), (4, 2, 45, 5),
                                      (32, 2, 16, 5), (64, 3, 16, 7)])      # 16 x 16 maps of 32 images: LDS tiles of exactly 64 KiB
def test_response_norm_and_undo(cm, cc, rng, N, F, S, size):
    a, p = 0.001, 0.75
    x = _f(rng.standard_normal((N, F * S * S)) * 3)
    X, D, T = cm.CUDAMatrix(x), cm.empty(x.shape), cm.empty(x.shape)
    cc.ResponseNorm(X, D, T, F, size, a, p)
    t_want, d_want = co.response_norm(x, F, size, a, p)
    assert np.allclose(D.asarray(), d_want, rtol=2e-6)
    assert np.allclose(T.asarray(), t_want, rtol=1e-5, atol=1e-7)    # hardware log2/exp2 pow, like the reference's __powf
    g = _f(rng.standard_normal(x.shape))
    acts = cm.CUDAMatrix(T.asarray().copy(order='F'))
    U = cm.empty(x.shape)
    cc.ResponseNormUndo(cm.CUDAMatrix(g), D, X, acts, U, F, size, a, p)
    u_want, acts_want = co.response_norm_undo(g, D.asarray(), x, T.asarray(), F, size, a, p)
    assert np.allclose(acts.asarray(), acts_want, rtol=1e-5, atol=1e-9)      # acts is overwritten, as in the reference
    assert np.allclose(U.asarray(), u_want, rtol=1e-5, atol=1e-6)
    # contrast norm with separate mean differences
    md = _f(rng.standard_normal(x.shape))
    cc.ContrastNorm(X, cm.CUDAMatrix(md), D, T, F, size, a, p)
    t2, d2 = co.contrast_norm(x, md, F, size, a, p)
    assert np.allclose(D.asarray(), d2, rtol=2e-6) and np.allclose(T.asarray(), t2, rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("N,F,S,size", [(16, 4, 9, 3), (32, 8, 15, 5), (8, 2, 12, 6), (6, 3, 7, 4), (8, 2, 48, 5)])
def test_contrast_norm_undo_by_name(cm, cc, rng, N, F, S, size):
    """ContrastNormUndo (cudamat_conv.cu:1436-1439) is ResponseNormUndo with the mean differences
    in the place of the inputs; called here under its own name, in place over outGrads as
    convolutions.py may, and against the definition."""
    a, p = 0.002, 0.75
    x = _f(rng.standard_normal((N, F * S * S)) * 2)
    md = _f(rng.standard_normal(x.shape))
    X, MD, D, T = cm.CUDAMatrix(x), cm.CUDAMatrix(md), cm.empty(x.shape), cm.empty(x.shape)
    cc.ContrastNorm(X, MD, D, T, F, size, a, p)
    g = _f(rng.standard_normal(x.shape))
    acts = cm.CUDAMatrix(T.asarray().copy(order='F'))
    U = cm.empty(x.shape)
    cc.ContrastNormUndo(cm.CUDAMatrix(g), D, MD, acts, U, F, size, a, p)
    u_want, acts_want = co.response_norm_undo(g, D.asarray(), md, T.asarray(), F, size, a, p)
    assert np.allclose(acts.asarray(), acts_want, rtol=1e-5, atol=1e-9)
    assert np.allclose(U.asarray(), u_want, rtol=1e-5, atol=1e-6)
    # the target may be the gradient array itself
    G = cm.CUDAMatrix(g)
    acts2 = cm.CUDAMatrix(T.asarray().copy(order='F'))
    cc.ContrastNormUndo(G, D, MD, acts2, G, F, size, a, p)
    assert np.array_equal(G.asarray(), U.asarray())


def test_conv_layer_chain_like_deepnet(cm, cc, rng):
    """convolutions.py:5-67 order: transpose -> convUp -> MaxPool -> ResponseNorm -> transpose."""
    N, C, H, F, k, p = 128, 3, 32, 64, 5, 2
    Mx = co.n_modules(H, k, 1, p)
    inputs = _f(rng.standard_normal((C * H * H, N)))            # deepnet keeps (dims, batch)
    w = _f(0.01 * rng.standard_normal((F, C * k * k)))
    inp = cm.CUDAMatrix(inputs)
    xt = cm.empty((N, C * H * H))
    inp.transpose(xt)
    conv = cm.empty((N, F * Mx * Mx)); cc.convUp(xt, cm.CUDAMatrix(w), conv, Mx, p, 1, C)
    O = 15
    pooled = cm.empty((N, F * O * O)); cc.MaxPool(conv, pooled, F, 3, 0, 2, O)
    den, normed = cm.empty((N, F * O * O)), cm.empty((N, F * O * O))
    cc.ResponseNorm(pooled, den, normed, F, 5, 0.001, 0.75)
    out = cm.empty((F * O * O, N)); normed.transpose(out)
    want = co.conv_up(inputs.T, w, C, Mx, p, 1)
    want = co.max_pool(want, F, 3, 0, 2, O)
    want, _ = co.response_norm(want, F, 5, 0.001, 0.75)
    assert np.allclose(out.asarray(), want.T, rtol=2e-4, atol=2e-5)


@pytest.mark.parametrize("N,C,H,F,k,s,p", [
    (4, 2, 6, 16, 3, 1, 1), (16, 3, 8, 16, 3, 2, 0),           # one lane per output
    # batches of 128: the matrix-core kernels with one filter bank per module.  Stride 1 and
    # strided with few colours (phases merged into columns) or many; 16 to 96 filters; padding
    (128, 3, 8, 32, 3, 1, 1), (128, 3, 9, 16, 3, 2, 0), (128, 20, 6, 48, 3, 1, 0), (256, 4, 7, 64, 5, 1, 2),
    (128, 32, 6, 96, 3, 2, 1), (128, 1, 10, 16, 4, 2, 0), (128, 3, 12, 64, 5, 1, 2),
    # batches that are padded up to 128 (100 images, 40 images), and one too small for that
    (100, 3, 8, 32, 3, 1, 1), (40, 2, 7, 16, 3, 2, 1), (24, 2, 7, 16, 3, 2, 1)])
def test_locally_connected_layers(cm, cc, rng, N, C, H, F, k, s, p):
    Mx = co.n_modules(H, k, s, p)
    M = Mx * Mx
    x = _f(rng.standard_normal((N, C * H * H)))
    w = _f(0.1 * rng.standard_normal((F, M * C * k * k)))
    y = _f(rng.standard_normal((N, F * M)))
    X, W, Y = cm.CUDAMatrix(x), cm.CUDAMatrix(w), cm.CUDAMatrix(y)
    up, down, outp = cm.empty((N, F * M)), cm.empty((N, C * H * H)), cm.empty((F, M * C * k * k))
    cc.localUp(X, W, up, Mx, p, s, C)
    assert np.allclose(up.asarray(), co.local_up(x, w, C, Mx, p, s), rtol=1e-4, atol=1e-5)
    cc.localDown(Y, W, down, Mx, p, s, k, H, C)
    assert np.allclose(down.asarray(), co.local_down(y, w, C, H, p, s), rtol=1e-4, atol=1e-5)
    cc.localOutp(X, Y, outp, Mx, p, k, s, C)
    assert np.allclose(outp.asarray(), co.local_outp(x, y, C, Mx, k, p, s), rtol=1e-4, atol=1e-4)


def test_locally_connected_layers_with_groups(cm, cc, rng):
    """Two groups at batch 128: each group of filters sees its own half of the colours, which is
    the ungrouped layer applied to the two halves."""
    N, C, H, F, k, s, p, G = 128, 8, 7, 64, 3, 1, 1, 2
    Mx = co.n_modules(H, k, s, p)
    M, Cg, Fg = Mx * Mx, C // G, F // G
    x = _f(rng.standard_normal((N, C * H * H)))
    w = _f(0.1 * rng.standard_normal((F, M * Cg * k * k)))
    y = _f(rng.standard_normal((N, F * M)))
    X, W, Y = cm.CUDAMatrix(x), cm.CUDAMatrix(w), cm.CUDAMatrix(y)
    up, down, outp = cm.empty((N, F * M)), cm.empty((N, C * H * H)), cm.empty((F, M * Cg * k * k))
    cc.localUp(X, W, up, Mx, p, s, C, G)
    cc.localDown(Y, W, down, Mx, p, s, k, H, C, numGroups=G)
    cc.localOutp(X, Y, outp, Mx, p, k, s, C, numGroups=G)
    for g in range(G):
        xs = x[:, g * Cg * H * H:(g + 1) * Cg * H * H]
        ws = w[g * Fg:(g + 1) * Fg]
        ys = y[:, g * Fg * M:(g + 1) * Fg * M]
        assert np.allclose(up.asarray()[:, g * Fg * M:(g + 1) * Fg * M], co.local_up(xs, ws, Cg, Mx, p, s), rtol=1e-4, atol=1e-5)
        assert np.allclose(down.asarray()[:, g * Cg * H * H:(g + 1) * Cg * H * H], co.local_down(ys, ws, Cg, H, p, s),
                           rtol=1e-4, atol=1e-5)
        assert np.allclose(outp.asarray()[g * Fg:(g + 1) * Fg], co.local_outp(xs, ys, Cg, Mx, k, p, s), rtol=1e-4, atol=1e-4)


def _random_conv_cases(seed, count):
    """Seeded layer geometries that reach every convolution code path: batch 128/256 for the
    buffer-load kernels (few or many colours, strided or not), batch 16/48 for the general
    matrix-core kernels, odd batches for the one-lane-per-output kernels."""
    r = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        N = int(r.choice([128, 128, 256, 16, 48, 6]))
        G = int(r.choice([1, 1, 2]))
        Cg = int(r.choice([1, 2, 3, 4, 16, 20, 24]))
        Fg = int(r.choice([16, 32, 48]))
        k = int(r.integers(2, 6))
        s = int(r.integers(1, k + 1))
        p = int(r.integers(0, k))
        H = int(r.integers(k, 12))
        if co.n_modules(H, k, s, p) < 1 or N * Cg * G * H * H > 3_000_000:
            continue
        out.append((N, Cg * G, H, Fg * G, k, s, p, G))
    return out


@pytest.mark.parametrize("N,C,H,F,k,s,p,G", _random_conv_cases(20240607, 24))
def test_three_conv_passes_on_random_geometries(cm, cc, rng, N, C, H, F, k, s, p, G):
    test_three_conv_passes(cm, cc, rng, N, C, H, F, k, s, p, G)


def _random_small_layer_cases(seed, count):
    """Seeded first-layer-like geometries (few colours, few filters, short reductions) for
    the register-resident convUp / patch-product convDown kernels and the small-output
    convOutp kernel: batches of 32..160 (one to five image blocks per module; 64-image
    chunks with and without a remainder), reductions up to and beyond the 80 / 96 term
    limits, filter groups that are not a multiple of 32, every stride and padding."""
    r = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        N = int(r.choice([32, 64, 96, 128, 160]))
        G = int(r.choice([1, 1, 2]))
        Cg = int(r.choice([1, 2, 3, 4, 5]))
        Fg = int(r.choice([16, 32, 48, 64]))
        k = int(r.integers(2, 7))
        s = int(r.integers(1, k + 1))
        p = int(r.integers(0, k))
        H = int(r.integers(k, 15))
        if co.n_modules(H, k, s, p) < 1 or Cg * k * k > 110:
            continue
        out.append((N, Cg * G, H, Fg * G, k, s, p, G))
    return out


@pytest.mark.parametrize("N,C,H,F,k,s,p,G", _random_small_layer_cases(20240611, 30))
def test_three_conv_passes_on_random_small_layers(cm, cc, rng, N, C, H, F, k, s, p, G):
    test_three_conv_passes(cm, cc, rng, N, C, H, F, k, s, p, G)


FULL_LAYERS = [  # the conv layers of benchmark config 5 at full size: N, C, H, F, k, stride, padding, groups
    (128, 3, 224, 96, 11, 4, 0, 1),
    (128, 96, 27, 256, 5, 1, 2, 2),
]


@pytest.mark.parametrize("N,C,H,F,k,s,p,G", FULL_LAYERS)
def test_benchmark_layers_at_full_size_on_sampled_outputs(cm, cc, N, C, H, F, k, s, p, G):
    """The kernels these shapes select (256-row tiles with the unmasked gather, uniform-row
    tiles, 16-wide column blocks, split-K convOutp) only come into play at sizes where the
    float64 passes would take minutes: random outputs of each pass are checked against the
    definition evaluated for that single output, and the three results against each other
    through the adjoint identities."""
    r = np.random.default_rng(55)
    Mx = co.n_modules(H, k, s, p)
    Cg = C // G
    x = _f(r.standard_normal((N, C * H * H)))
    w = _f(0.05 * r.standard_normal((F, Cg * k * k)))
    y = _f(r.standard_normal((N, F * Mx * Mx)))
    X, W, Y = cm.CUDAMatrix(x), cm.CUDAMatrix(w), cm.CUDAMatrix(y)
    up, down, outp = cm.empty((N, F * Mx * Mx)), cm.empty((N, C * H * H)), cm.empty((F, Cg * k * k))
    cc.convUp(X, W, up, Mx, p, s, C, G)
    cc.convDown(Y, W, down, Mx, p, s, k, H, C, numGroups=G)
    cc.convOutp(X, Y, outp, Mx, p, k, s, C, numGroups=G)
    u, d, o = up.asarray().reshape(N, F, Mx, Mx), down.asarray().reshape(N, C, H, H), outp.asarray().reshape(F, Cg, k, k)
    edge = lambda size: int(r.choice([0, size - 1, int(r.integers(size))]))      # borders twice as often as the interior
    for _ in range(300):
        n, f, my, mx = int(r.integers(N)), int(r.integers(F)), edge(Mx), edge(Mx)
        val, mag = co.conv_up_at(x, w, C, Mx, p, s, G, n, f, my, mx)
        assert abs(u[n, f, my, mx] - val) <= REL * mag + 1e-30
        c, yy, xx = int(r.integers(C)), edge(H), edge(H)
        val, mag = co.conv_down_at(y, w, C, H, p, s, G, n, c, yy, xx)
        assert abs(d[n, c, yy, xx] - val) <= REL * mag + 1e-6
    for _ in range(12):
        f, cl, ky, kx = int(r.integers(F)), int(r.integers(Cg)), edge(k), edge(k)
        val, mag = co.conv_outp_at(x, y, C, Mx, k, p, s, G, f, cl, ky, kx)
        assert abs(o[f, cl, ky, kx] - val) <= REL * mag
    a = float((up.asarray().astype(np.float64) * y).sum())
    b = float((down.asarray().astype(np.float64) * x).sum())
    c_ = float((outp.asarray().astype(np.float64) * w).sum())
    scale = float((np.abs(up.asarray()).astype(np.float64) * np.abs(y)).sum())
    assert abs(a - b) / scale < 1e-5 and abs(a - c_) / scale < 1e-5
    for m in (X, W, Y, up, down, outp):
        m.free_device_memory()


@pytest.mark.parametrize("S,subs,O", [(55, 3, 27), (40, 3, 20), (41, 2, 21), (48, 2, 24), (46, 3, 20), (5, 3, 2), (8, 2, 4), (9, 3, 4), (32, 3, 16)])
def test_pool_gradient_in_blocks_has_the_bits_of_the_general_kernel(cm, cc, rng, S, subs, O):
    """Windows of 2 or 3 with stride 2 from 0 take a kernel that handles 2 x 2 pixels per lane; it adds the same
    terms in the same order as the general kernel, which the same images reach in a batch that is
    not a multiple of 4."""
    N, F = 8, 3
    x = _f(rng.integers(-3, 4, (N, F * S * S)))          # small integers: plenty of ties
    g = _f(rng.standard_normal((N, F * O * O)))
    X, T = cm.CUDAMatrix(x), cm.empty((N, F * O * O))
    cc.MaxPool(X, T, F, subs, 0, 2, O)
    U = cm.empty((N, F * S * S))
    cc.MaxPoolUndo(X, U, cm.CUDAMatrix(g), T, subs, 0, 2, O)
    want = co.max_pool_undo(x, g, T.asarray(), subs, 0, 2, O)
    assert np.allclose(U.asarray(), want, rtol=1e-6, atol=1e-6)
    # one image more in front: N = 9 is not a multiple of 4, so the general kernel runs; its columns 1..8 are the same problem
    x9 = np.vstack([x[:1], x]); g9 = np.vstack([g[:1], g])
    X9, T9, U9 = cm.CUDAMatrix(_f(x9)), cm.empty((N + 1, F * O * O)), cm.empty((N + 1, F * S * S))
    cc.MaxPool(X9, T9, F, subs, 0, 2, O)
    cc.MaxPoolUndo(X9, U9, cm.CUDAMatrix(_f(g9)), T9, subs, 0, 2, O)
    assert np.array_equal(U9.asarray()[1:], U.asarray())


FUSED_POOL_NORM = [  # N, F, S (un-pooled side), subs, start, stride, norm size
    (128, 64, 32, 3, 0, 2, 5),      # config 4
    (32, 8, 32, 3, 0, 2, 5), (64, 4, 24, 3, 0, 2, 3), (32, 3, 13, 2, 0, 2, 3), (16, 4, 20, 2, 0, 2, 7), (100, 6, 27, 3, 0, 2, 5),
    (32, 2, 9, 3, -1, 2, 3), (36, 3, 11, 3, 0, 2, 7),
    # shapes the one-launch kernels do not take (other strides / windows / norm sizes, odd batches, large
    # pooled maps): the entry points run the separate kernels
    (8, 3, 9, 3, 0, 3, 3), (16, 2, 12, 4, -1, 3, 5), (6, 3, 8, 2, 0, 2, 4), (5, 2, 9, 3, 0, 2, 3), (16, 2, 60, 3, 0, 2, 5),
]


@pytest.mark.parametrize("N,F,S,subs,start,stride,size", FUSED_POOL_NORM)
def test_pool_and_norm_in_one_launch_equal_the_separate_calls(cm, cc, rng, N, F, S, subs, start, stride, size):
    """MaxPoolResponseNorm / ResponseNormUndoMaxPoolUndo against MaxPool -> ResponseNorm and
    ResponseNormUndo (on a copy of the pooled layer) -> MaxPoolUndo: pooled values bit for bit, the
    rest to 1e-5 (the one-launch kernels repeat the arithmetic of the separate ones; shapes that take
    other separate kernels may differ in the order of additions), and against the definition."""
    a, p = 0.001, 0.75
    O = (S - start - subs + stride - 1) // stride + 1
    x = _f(rng.standard_normal((N, F * S * S)) * 2)
    X = cm.CUDAMatrix(x)
    shape = (N, F * O * O)
    pooled1, den1, out1 = cm.empty(shape), cm.empty(shape), cm.empty(shape)
    cm.set_deferred_epilogues(False)          # (each call its own launch: a held-back MaxPool would join the ResponseNorm)
    cc.MaxPool(X, pooled1, F, subs, start, stride, O)
    cc.ResponseNorm(pooled1, den1, out1, F, size, a, p)
    cm.set_deferred_epilogues(True)
    pooled2, den2, out2 = cm.empty(shape), cm.empty(shape), cm.empty(shape)
    for m in (pooled2, den2, out2):
        m.assign(np.nan)
    cc.MaxPoolResponseNorm(X, pooled2, den2, out2, F, subs, start, stride, O, size, a, p)
    assert np.array_equal(pooled2.asarray(), pooled1.asarray())
    assert np.allclose(den2.asarray(), den1.asarray(), rtol=1e-6) and np.allclose(out2.asarray(), out1.asarray(), rtol=1e-5, atol=1e-7)
    want_pool = co.max_pool(x, F, subs, start, stride, O)
    want_out, want_den = co.response_norm(want_pool.astype(np.float32), F, size, a, p)
    assert np.array_equal(pooled2.asarray(), want_pool.astype(np.float32))
    assert np.allclose(den2.asarray(), want_den, rtol=2e-6) and np.allclose(out2.asarray(), want_out, rtol=1e-5, atol=1e-7)
    # backward, with deepnet's operand order (the normalised outputs as `inputs`, convolutions.py:111-122)
    g = _f(rng.standard_normal(shape))
    G = cm.CUDAMatrix(g)
    tmp_acts, tmp_grad, undo1 = cm.empty(shape), cm.empty(shape), cm.empty(x.shape)
    tmp_acts.assign(pooled1)
    cc.ResponseNormUndo(G, den1, out1, tmp_acts, tmp_grad, F, size, a, p)
    cc.MaxPoolUndo(X, undo1, tmp_grad, pooled1, subs, start, stride, O)
    undo2 = cm.empty(x.shape)
    undo2.assign(np.nan)
    before = pooled2.asarray().copy()
    cc.ResponseNormUndoMaxPoolUndo(G, den2, out2, pooled2, X, undo2, F, subs, start, stride, O, size, a, p)
    assert np.array_equal(pooled2.asarray(), before)                  # the pooled layer is only read
    assert np.allclose(undo2.asarray(), undo1.asarray(), rtol=1e-5, atol=1e-6)
    ng, _ = co.response_norm_undo(g, den1.asarray(), out1.asarray(), pooled1.asarray(), F, size, a, p)
    want_undo = co.max_pool_undo(x, ng.astype(np.float32), pooled1.asarray(), subs, start, stride, O)
    assert np.allclose(undo2.asarray(), want_undo, rtol=1e-5, atol=1e-5)
    # in place over the un-pooled layer, as convolutions.py uses it
    X2 = cm.CUDAMatrix(x)
    cc.ResponseNormUndoMaxPoolUndo(G, den2, out2, pooled2, X2, X2, F, subs, start, stride, O, size, a, p)
    assert np.array_equal(X2.asarray().view(np.uint32), undo2.asarray().view(np.uint32))


def test_pool_and_norm_in_one_launch_keep_the_bits_at_the_benchmark_layer(cm, cc, rng):
    """At config 4 (64 maps of 32 x 32 -> 15 x 15, batch 128, norm size 5) the separate calls run the
    kernels whose arithmetic the one-launch kernels repeat: every output has the same bits."""
    N, F, S, O = 128, 64, 32, 15
    x = _f(rng.standard_normal((N, F * S * S)))
    X = cm.CUDAMatrix(x)
    shape = (N, F * O * O)
    pooled1, den1, out1, pooled2, den2, out2 = (cm.empty(shape) for _ in range(6))
    cc.MaxPool(X, pooled1, F, 3, 0, 2, O); cc.ResponseNorm(pooled1, den1, out1, F, 5, 0.001, 0.75)
    cc.MaxPoolResponseNorm(X, pooled2, den2, out2, F, 3, 0, 2, O, 5, 0.001, 0.75)
    for a, b in ((pooled1, pooled2), (den1, den2), (out1, out2)):
        assert np.array_equal(a.asarray().view(np.uint32), b.asarray().view(np.uint32))
    G = cm.CUDAMatrix(_f(rng.standard_normal(shape)))
    tmp_acts, tmp_grad, undo1, undo2 = cm.empty(shape), cm.empty(shape), cm.empty(x.shape), cm.empty(x.shape)
    tmp_acts.assign(pooled1)
    cc.ResponseNormUndo(G, den1, out1, tmp_acts, tmp_grad, F, 5, 0.001, 0.75)
    cc.MaxPoolUndo(X, undo1, tmp_grad, pooled1, 3, 0, 2, O)
    cc.ResponseNormUndoMaxPoolUndo(G, den2, out2, pooled2, X, undo2, F, 3, 0, 2, O, 5, 0.001, 0.75)
    assert np.array_equal(undo1.asarray().view(np.uint32), undo2.asarray().view(np.uint32))


@pytest.mark.parametrize("N,F,S,subs,start,stride,size", FUSED_POOL_NORM)
def test_a_held_back_max_pool_joins_the_response_norm_that_follows(cm, cc, rng, N, F, S, subs, start, stride, size):
    """deepnet/convolutions.py:58-66 calls MaxPool and then ResponseNorm on the pooled map: the library
    holds the MaxPool back and runs both as one launch where its LDS kernel applies.  With the
    deferral off and on: the same bits in the pooled map, the denominators and the result, whatever
    comes between or after the two calls."""
    a, p = 0.001, 0.75
    O = (S - start - subs + stride - 1) // stride + 1
    x = _f(rng.standard_normal((N, F * S * S)) * 2)
    shape = (N, F * O * O)
    res = []
    for deferred in (False, True):
        cm.set_deferred_epilogues(deferred)
        X = cm.CUDAMatrix(x)
        pooled, den, out, other, den2, out2 = (cm.empty(shape) for _ in range(6))
        for m in (pooled, den, out, other, den2, out2):
            m.assign(np.nan)
        cc.MaxPool(X, pooled, F, subs, start, stride, O); cc.ResponseNorm(pooled, den, out, F, size, a, p)   # the pair
        cc.MaxPool(X, other, F, subs, start, stride, O)                                                     # held back, then read
        first = other.asarray().copy()
        cc.MaxPool(X, other, F, subs, start, stride, O); other.mult(2.0)                  # ... then used by the matrix library
        cc.MaxPool(X, other, F, subs, start, stride, O); cc.ResponseNorm(pooled, den2, out2, F, size, a, p)  # ... then a norm of another map
        cc.MaxPool(X, other, F, subs, start, stride, O); cc.MaxPool(X, pooled, F, subs, start, stride, O)    # two in a row
        res.append([m.asarray().view(np.uint32).copy() for m in (pooled, den, out, other, den2, out2)] + [first.view(np.uint32)])
    cm.set_deferred_epilogues(True)
    for i, (w, g) in enumerate(zip(*res)):
        assert np.array_equal(w, g), "result %d differs" % i
