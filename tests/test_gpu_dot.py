"""GPU parity of dot / add_dot / subtract_dot (fp32 MFMA kernel and the
matrix-vector paths) against np.dot in float64: 1e-4 relative."""
import numpy as np
import pytest

from oracle import cudamat_oracle as orc

pytestmark = pytest.mark.gpu

REL = 1e-4


def _rand(rng, shape):
    return np.asarray(rng.standard_normal(shape), dtype=np.float32, order='F')


def _relerr(got, want, A, B):
    """The larger of two measures: every element against the bound |A|.|B| of its own sum (robust
    to cancellation), and the whole product against its own size (Frobenius norms, ten times
    stricter: 1e-5 relative to the result itself)."""
    bound = np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64)
    got = np.asarray(got, np.float64)
    elementwise = np.max(np.abs(got - want) / (bound + 1e-30))
    whole = np.linalg.norm(got - want) / (np.linalg.norm(want) + 1e-30)
    return max(elementwise, 10.0 * whole)


# (m, k, n): test_cudamat.py:796-880 uses 128x256x64-like shapes, eigenmat/test.py:23-47
# 500x1000x600; the rest are the benchmark's step shapes and ragged edges.
SHAPES = [(64, 128, 32), (128, 256, 64), (500, 1000, 600), (500, 784, 100), (784, 500, 100),
          (784, 100, 500), (1024, 784, 128), (10, 1024, 128), (1024, 128, 1024), (1, 5, 1),
          (33, 17, 65), (130, 1, 70), (129, 257, 131), (1, 300, 40), (300, 40, 1), (5, 7, 3)]


@pytest.mark.parametrize("m,k,n", SHAPES)
@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True), (True, True)])
def test_dot_all_transpose_combinations(cm, rng, m, k, n, ta, tb):
    A, B = _rand(rng, (m, k)), _rand(rng, (k, n))
    a = cm.CUDAMatrix(np.asfortranarray(A.T)) if ta else cm.CUDAMatrix(A)
    b = cm.CUDAMatrix(np.asfortranarray(B.T)) if tb else cm.CUDAMatrix(B)
    t = cm.dot(a.T if ta else a, b.T if tb else b)
    assert t.shape == (m, n)
    want = A.astype(np.float64) @ B.astype(np.float64)
    assert _relerr(t.asarray(), want, A, B) < REL
    for h in (a, b, t):
        h.free_device_memory()


@pytest.mark.parametrize("alpha,beta", [(1.0, 0.0), (1.0, 1.0), (-1.0, 1.0), (np.pi, -1.0), (0.0, 1.0)])
def test_alpha_beta(cm, rng, alpha, beta):
    A, B, C = _rand(rng, (128, 256)), _rand(rng, (256, 64)), _rand(rng, (128, 64))
    a, b, c = cm.CUDAMatrix(A), cm.CUDAMatrix(B), cm.CUDAMatrix(C)
    cm._check(cm._cudamat.dot(a.p_mat, b.p_mat, c.p_mat, beta, alpha))
    want = orc.dot(A, B, C, beta=beta, alpha=alpha)
    bound = abs(alpha) * (np.abs(A).astype(np.float64) @ np.abs(B)) + abs(beta) * np.abs(C) + 1e-30
    assert np.max(np.abs(c.asarray() - want) / bound) < REL


def test_beta_zero_ignores_garbage_in_target(cm, rng):
    A, B = _rand(rng, (70, 30)), _rand(rng, (30, 50))
    t = cm.CUDAMatrix(np.full((70, 50), np.nan, dtype=np.float32))
    cm.dot(cm.CUDAMatrix(A), cm.CUDAMatrix(B), target=t)
    assert np.all(np.isfinite(t.asarray()))


def test_add_dot_subtract_dot_and_mult(cm, rng):
    A, B, C = _rand(rng, (784, 100)), _rand(rng, (500, 100)), _rand(rng, (784, 500))
    a, b, c = cm.CUDAMatrix(A), cm.CUDAMatrix(B), cm.CUDAMatrix(C)
    c.add_dot(a, b.T, mult=0.01)
    want = C + 0.01 * (A.astype(np.float64) @ B.T)
    assert np.max(np.abs(c.asarray() - want)) < 1e-4
    c.subtract_dot(a, b.T)
    want = want - A.astype(np.float64) @ B.T
    assert np.max(np.abs(c.asarray() - want) / (np.abs(A).astype(np.float64) @ np.abs(B.T) + 1)) < REL
    d = a.dot(b.T, mult=2.0)
    assert _relerr(d.asarray(), 2.0 * (A.astype(np.float64) @ B.T), 2 * A, B.T) < REL


def test_dot_on_column_views(cm, rng):
    # operands that start 37*k floats into a buffer: unaligned loads inside the tile loader
    A, B = _rand(rng, (37, 90)), _rand(rng, (37, 50))
    a, b = cm.CUDAMatrix(A), cm.CUDAMatrix(B)
    va, vb = a.slice(5, 85), b.slice(3, 47)
    t = cm.dot(va.T, vb)
    want = A[:, 5:85].astype(np.float64).T @ B[:, 3:47]
    assert _relerr(t.asarray(), want, A[:, 5:85].T, B[:, 3:47]) < REL


def test_dot_error_codes(cm, rng):
    a, b = cm.CUDAMatrix(_rand(rng, (8, 6))), cm.CUDAMatrix(_rand(rng, (5, 4)))
    with pytest.raises(cm.CUDAMatException, match="Incompatible matrix dimensions"):
        cm.dot(a, b)
    with pytest.raises(cm.CUDAMatException, match="Incompatible matrix dimensions"):
        cm.dot(a, cm.CUDAMatrix(_rand(rng, (6, 4))), target=cm.empty((8, 5)))
    host_only = cm.CUDAMatrix(_rand(rng, (6, 4)), copy_to_device=False)
    with pytest.raises(cm.CUDAMatException, match="not in device memory"):
        cm.dot(a, host_only, target=cm.empty((8, 4)))


@pytest.mark.parametrize("n", [2048, 4096])
def test_large_square_products(cm, rng, n):
    """Checked on sampled rows/columns against float64 and through the identity
    (A B) x = A (B x) on the whole product."""
    A = np.asarray(rng.uniform(-1, 1, (n, n)), dtype=np.float32, order='F')
    B = np.asarray(rng.uniform(-1, 1, (n, n)), dtype=np.float32, order='F')
    a, b = cm.CUDAMatrix(A), cm.CUDAMatrix(B)
    c = cm.dot(a, b)
    got = c.asarray()
    rows = np.arange(0, n, 211); cols = np.arange(0, n, 173)
    want = A[rows, :].astype(np.float64) @ B[:, cols].astype(np.float64)
    bound = np.abs(A[rows, :]).astype(np.float64) @ np.abs(B[:, cols]).astype(np.float64)
    assert np.max(np.abs(got[np.ix_(rows, cols)] - want) / bound) < REL
    x = rng.uniform(-1, 1, (n,))
    lhs = got.astype(np.float64) @ x
    rhs = A.astype(np.float64) @ (B.astype(np.float64) @ x)
    assert np.max(np.abs(lhs - rhs)) / np.max(np.abs(rhs)) < 1e-4
    ct_ = cm.dot(a.T, b.T)
    want_t = A[:, rows].astype(np.float64).T @ B[cols, :].astype(np.float64).T
    bound_t = np.abs(A[:, rows]).astype(np.float64).T @ np.abs(B[cols, :]).astype(np.float64).T
    assert np.max(np.abs(ct_.asarray()[np.ix_(rows, cols)] - want_t) / bound_t) < REL
    for h in (a, b, c, ct_):
        h.free_device_memory()


@pytest.mark.parametrize("m,k,n", [(1000, 1001, 1000), (1001, 1000, 1000), (1000, 1000, 1001), (1003, 999, 1005), (1088, 50, 1088),
                                   (1100, 48, 1000), (1100, 47, 1000), (2000, 130, 1300), (1004, 1030, 996)])
@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True)])
def test_products_on_the_tile_loop_with_any_alignment(cm, rng, m, k, n, ta, tb):
    """More 64 x 64 tiles than the single-launch kernels take: the loop over 16-deep slabs whose
    loads are unconditional 16-byte requests.  Leading dimensions that are not multiples of four
    floats, operands that start at an odd float of a parent buffer, tiles that hang over the edge,
    reductions of exactly three slabs (the shortest that enter the loop) and of one float less."""
    A = np.asarray(rng.uniform(-1, 1, (k, m) if ta else (m, k)), dtype=np.float32, order='F')
    B = np.asarray(rng.uniform(-1, 1, (n, k) if tb else (k, n)), dtype=np.float32, order='F')
    C = np.asarray(rng.uniform(-1, 1, (m, n)), dtype=np.float32, order='F')
    opa = (A.T if ta else A).astype(np.float64); opb = (B.T if tb else B).astype(np.float64)
    want = 0.5 * C.astype(np.float64) + 1.25 * (opa @ opb)
    bound = 0.5 * np.abs(C).astype(np.float64) + 1.25 * (np.abs(opa) @ np.abs(opb))
    # whole matrices, then the same operands as views one column into a parent with one more column
    # (the view starts rows-of-the-parent floats into the buffer: any 4-byte alignment)
    pa = np.asfortranarray(np.concatenate([np.zeros((A.shape[0], 1), np.float32), A], axis=1))
    pb = np.asfortranarray(np.concatenate([np.zeros((B.shape[0], 1), np.float32), B], axis=1))
    for view in (False, True):
        if view:
            ha, hb = cm.CUDAMatrix(pa), cm.CUDAMatrix(pb)
            a, b = ha.slice(1, pa.shape[1]), hb.slice(1, pb.shape[1])
        else:
            ha, hb = cm.CUDAMatrix(A), cm.CUDAMatrix(B)
            a, b = ha, hb
        c = cm.CUDAMatrix(C)
        cm._check(cm._cudamat.dot((a.T if ta else a).p_mat, (b.T if tb else b).p_mat, c.p_mat, 0.5, 1.25))
        assert np.max(np.abs(c.asarray() - want) / bound) < REL, view
        for h in (ha, hb, c):
            h.free_device_memory()


@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True), (True, True)])
def test_split_k_products(cm, rng, ta, tb):
    """About one 64 x 64 tile per CU and K >= 2048: the reduction is split over two workgroups
    per tile and summed by a second kernel, with alpha and beta applied there."""
    m, n, k = 1024, 1040, 2500
    A = np.asarray(rng.uniform(-1, 1, (k, m) if ta else (m, k)), dtype=np.float32, order='F')
    B = np.asarray(rng.uniform(-1, 1, (n, k) if tb else (k, n)), dtype=np.float32, order='F')
    C = np.asarray(rng.uniform(-1, 1, (m, n)), dtype=np.float32, order='F')
    a, b, c = cm.CUDAMatrix(A), cm.CUDAMatrix(B), cm.CUDAMatrix(C)
    c.add_dot(a.T if ta else a, b.T if tb else b, mult=-0.75)
    opa = (A.T if ta else A).astype(np.float64); opb = (B.T if tb else B).astype(np.float64)
    want = C.astype(np.float64) - 0.75 * (opa @ opb)
    bound = np.abs(C).astype(np.float64) + 0.75 * (np.abs(opa) @ np.abs(opb))
    assert np.max(np.abs(c.asarray() - want) / bound) < REL
    for h in (a, b, c):
        h.free_device_memory()


# ---- the fused extension: dot -> add_col_vec -> activation in one call

@pytest.mark.parametrize("m,n,k,ta,tb", [
    (500, 100, 784, True, False),      # RBM up pass (single-launch kernel)
    (784, 100, 500, False, False),     # RBM down pass
    (1024, 128, 784, True, False),     # MLP layer
    (10, 128, 1024, True, False),      # MLP output layer (fewer rows than a tile)
    (300, 700, 96, False, True),       # mid-sized: the single-launch kernel
    (1024, 1024, 2304, True, False),   # one 64 x 64 tile per CU and a long K: split-K, falls back to separate launches
    (2048, 2048, 64, False, False),    # big tiles, fused epilogue
    (37, 1, 50, False, False),         # one output column: matrix-vector kernel
])
@pytest.mark.parametrize("act", [None, 'sigmoid', 'relu', 'tanh'])
def test_dot_bias_act_is_bit_identical_to_the_three_calls(cm, rng, m, n, k, ta, tb, act):
    a = np.asarray(rng.standard_normal((k, m) if ta else (m, k)), dtype=np.float32, order='F')
    b = np.asarray(rng.standard_normal((n, k) if tb else (k, n)), dtype=np.float32, order='F')
    bias = np.asarray(rng.standard_normal((m, 1)), dtype=np.float32, order='F')
    A, B, V = cm.CUDAMatrix(a), cm.CUDAMatrix(b), cm.CUDAMatrix(bias)
    opa, opb = (A.T if ta else A), (B.T if tb else B)
    want = cm.empty((m, n))
    cm.dot(opa, opb, target=want)
    want.add_col_vec(V)
    if act == 'sigmoid':
        want.apply_sigmoid()
    elif act == 'relu':
        want.lower_bound(0)
    elif act == 'tanh':
        cm.tanh(want)
    got = cm.CUDAMatrix(np.full((m, n), np.nan, dtype=np.float32))
    r = cm.dot_bias_act(opa, opb, V, target=got, act=act)
    assert r is got
    assert np.array_equal(got.asarray().view(np.uint32), want.asarray().view(np.uint32))
    # without a bias, and allocating its own target
    got2 = cm.dot_bias_act(opa, opb, None, act=act)
    want2 = cm.dot(opa, opb)
    if act == 'sigmoid':
        want2.apply_sigmoid()
    elif act == 'relu':
        want2.lower_bound(0)
    elif act == 'tanh':
        cm.tanh(want2)
    assert np.array_equal(got2.asarray().view(np.uint32), want2.asarray().view(np.uint32))
    for x in (A, B, V, want, got, got2, want2):
        x.free_device_memory()


@pytest.mark.gpu
@pytest.mark.parametrize("m,n,k,ta,act", [
    (500, 100, 784, True, 'sigmoid'),      # the RBM's up-pass: 16 x 16 blocks, 5 draws per stream
    (37, 19, 50, False, 'sigmoid'),        # fewer outputs than streams: the idle streams keep their words
    (1024, 128, 784, True, 'sigmoid'),     # 16 x 16 blocks on 512 workgroups, 11 draws per stream
    (768, 192, 300, True, 'sigmoid'),      # 32 x 32 blocks (144 of them), 12 draws per stream
    (1024, 128, 512, True, 'relu'),        # 32 x 32 blocks: both operands K-contiguous, rows 2 KiB apart
    (96, 128, 64, False, 'tanh'),          # exactly 12288 outputs
    (1024, 200, 300, True, 'sigmoid'),     # more than 16 draws per stream: separate kernels
    (2048, 2048, 64, False, 'sigmoid'),    # a product on the big tiles: separate sample kernel
    (300, 1, 40, False, 'sigmoid'),        # one column: the vector kernels
])
def test_dot_bias_act_sample_is_bit_identical_to_the_separate_calls(cm, rng, m, n, k, ta, act):
    A = _rand(rng, (k, m) if ta else (m, k))
    a, b = cm.CUDAMatrix(A), cm.CUDAMatrix(_rand(rng, (k, n)))
    bias = cm.CUDAMatrix(_rand(rng, (m, 1)))
    opa = a.T if ta else a
    want, want_s, want_next = cm.empty((m, n)), cm.empty((m, n)), cm.empty((300, 77))
    got, got_s, got_next = cm.empty((m, n)), cm.empty((m, n)), cm.empty((300, 77))
    for i in range(2):                       # twice: the second call starts from the words the first one left
        cm.CUDAMatrix.init_random(40 + i)
        want_next.fill_with_rand()           # (moves the generator off its seed state)
        cm.dot_bias_act(opa, b, bias, target=want, act=act)
        want.sample_bernoulli(target=want_s)
        want.sample_bernoulli(target=want_s)
        want_next.fill_with_rand()
        cm.CUDAMatrix.init_random(40 + i)
        got_next.fill_with_rand()
        cm.dot_bias_act(opa, b, bias, target=got, act=act, sample=got_s)
        r = cm.dot_bias_act(opa, b, bias, target=got, act=act, sample=got_s)
        assert r is got
        got_next.fill_with_rand()
        for x, y in ((want, got), (want_s, got_s), (want_next, got_next)):
            assert np.array_equal(x.asarray().view(np.uint32), y.asarray().view(np.uint32))
    smp = got_s.asarray()
    assert set(np.unique(smp)) <= {0.0, 1.0}
    if act == 'sigmoid' and m * n > 1000:
        assert abs(smp.mean() - got.asarray().mean()) < 0.05
    cm.CUDAMatrix.init_random(1)


@pytest.mark.gpu
def test_dot_bias_act_sample_errors_and_recording(cm, rng):
    a, b = cm.CUDAMatrix(_rand(rng, (64, 32))), cm.CUDAMatrix(_rand(rng, (32, 48)))
    t, s = cm.empty((64, 48)), cm.empty((64, 48))
    with pytest.raises(cm.CUDAMatException):
        cm.dot_bias_act(a, b, None, target=t, sample=cm.empty((64, 47)))
    with pytest.raises(cm.CUDAMatException):
        cm.dot_bias_act(a, b, None, target=t, sample=t)              # the sample needs a buffer of its own
    assert cm._cudamat.dot_bias_act_sample(cm.CUDAMatrix.rnd_state_p, a.p_mat, b.p_mat, None, t.p_mat, None, 1) != 0
    # recorded, the call keeps the generator's state in one word buffer; every replay draws on
    # from where the last one stopped
    cm.CUDAMatrix.init_random(9)
    want = []
    for _ in range(3):
        cm.dot_bias_act(a, b, None, target=t, sample=s)
        want.append(s.asarray().copy())
    cm.CUDAMatrix.init_random(9)
    cm.dot_bias_act(a, b, None, target=t, sample=s)
    with cm.Graph() as g:
        cm.dot_bias_act(a, b, None, target=t, sample=s)
    for i in (1, 2):
        g.launch()
        assert np.array_equal(s.asarray(), want[i])
    g.free()
    cm.CUDAMatrix.init_random(1)


def test_dot_bias_act_errors(cm, rng):
    A = cm.CUDAMatrix(np.zeros((8, 5), dtype=np.float32))
    B = cm.CUDAMatrix(np.zeros((5, 3), dtype=np.float32))
    T = cm.empty((8, 3))
    with pytest.raises(cm.CUDAMatException):
        cm.dot_bias_act(A, B, cm.CUDAMatrix(np.zeros((3, 1), dtype=np.float32)), target=T)     # bias of the wrong length
    with pytest.raises(cm.CUDAMatException):
        cm.dot_bias_act(A, B, None, target=cm.empty((8, 4)))
    with pytest.raises(ValueError):
        cm.dot_bias_act(A, B, None, target=T, act='softsign')
    host_only = cm.CUDAMatrix(np.zeros((8, 1), dtype=np.float32), copy_to_device=False)
    with pytest.raises(cm.CUDAMatException):
        cm.dot_bias_act(A, B, host_only, target=T)


@pytest.mark.gpu
@pytest.mark.parametrize("m,k,n,density", [(37, 29, 11, 0.2), (64, 64, 16, 0.1), (1000, 4096, 128, 0.01),
                                           (5, 7, 1, 0.5), (300, 50, 19, 0.0)])
def test_sparse_dot(cm, rng, m, k, n, density):
    # CSR x dense against the loop restatement (itself pinned against scipy); rows are
    # summed in fp32 in index order on the device: tolerance 1e-5 of sum |terms|
    import scipy.sparse as sps
    S = sps.random(m, k, density=density, format='csr', random_state=7, dtype=np.float32)
    S.sort_indices()
    D = np.asarray(rng.standard_normal((k, n)), dtype=np.float32, order='F')
    T = np.asarray(rng.standard_normal((m, n)), dtype=np.float32, order='F')
    sp_ = cm.SparseCUDAMatrix(S.data, S.indices, S.indptr, (m, k))
    d, t = cm.CUDAMatrix(D), cm.CUDAMatrix(T)
    bound = np.abs(S).astype(np.float64) @ np.abs(D).astype(np.float64)
    for beta, alpha in ((0.0, 1.0), (-0.5, 2.0)):
        t2 = cm.CUDAMatrix(T)
        cm.sparse_dot(sp_, d, target=t2, beta=beta, alpha=alpha)
        want = orc.sparse_dot(S.data, S.indices, S.indptr, D, T, beta=beta, alpha=alpha)
        assert np.max(np.abs(t2.asarray() - want) / (abs(alpha) * bound + abs(beta) * np.abs(T) + 1e-6)) < 1e-5
        t2.free_device_memory()
    # beta = 0 must overwrite, not scale, what the target held (NaN * 0 would stay NaN)
    t3 = cm.CUDAMatrix(np.full((m, n), np.nan, dtype=np.float32))
    cm.sparse_dot(sp_, d, target=t3)
    assert np.all(np.isfinite(t3.asarray()))
    out = cm.sparse_dot(sp_, d)                      # allocates its own m x n target
    assert out.shape == (m, n) and np.array_equal(out.asarray(), t3.asarray())
    sp_.free_device_memory()
    for x in (d, t, t3, out):
        x.free_device_memory()


@pytest.mark.gpu
def test_sparse_dot_errors(cm, rng):
    import scipy.sparse as sps
    S = sps.random(8, 6, density=0.5, format='csr', random_state=1, dtype=np.float32)
    sp_ = cm.SparseCUDAMatrix(S.data, S.indices, S.indptr, (8, 6))
    host_only = cm.SparseCUDAMatrix(S.data, S.indices, S.indptr, (8, 6), copy_to_device=False)
    d = cm.CUDAMatrix(np.zeros((6, 3), dtype=np.float32))
    with pytest.raises(cm.CUDAMatException):         # not on the device (-8)
        cm.sparse_dot(host_only, d)
    with pytest.raises(cm.CUDAMatException):         # inner dimensions differ (-1)
        cm.sparse_dot(sp_, cm.CUDAMatrix(np.zeros((5, 3), dtype=np.float32)))
    with pytest.raises(cm.CUDAMatException):         # target of the wrong shape (-1; the reference would overrun it)
        cm.sparse_dot(sp_, d, target=cm.empty((8, 2)))
    assert cm._cudamat.sparse_dot(host_only.p_mat, d.p_mat, d.p_mat, 0.0, 1.0) == -8


@pytest.mark.gpu
def test_fused_training_steps_of_the_bench_match_the_reference_sequences(cm):
    # bench.py's MLP step through the extensions leaves the same bits in every parameter as the
    # reference call sequence (same seed, three steps).  The RBM step's layer states and samples
    # have the same bits too; its parameters come from cd_update, which forms the statistics in one
    # accumulation where the six reference calls round twice: equal to rounding, step after step.
    import bench
    def run(cls, seed, fused, params, steps):
        cm.CUDAMatrix.init_random(seed)
        model = cls(cm)
        for _ in range(steps):
            (model.step_fused if fused else model.step)()
        return [p.asarray().copy() for p in params(model)]
    mlp = lambda m: m.W + m.b + m.dW + [m.loss]
    for a, b in zip(run(bench.MLP, 3, False, mlp, 3), run(bench.MLP, 3, True, mlp, 3)):
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    states = lambda m: [m.h, m.hs, m.v2, m.h2]
    for a, b in zip(run(bench.RBM, 1, False, states, 1), run(bench.RBM, 1, True, states, 1)):
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    rbm = lambda m: [m.W, m.bv, m.bh]
    for steps in (1, 3):
        for a, b in zip(run(bench.RBM, 1, False, rbm, steps), run(bench.RBM, 1, True, rbm, steps)):
            assert np.allclose(a, b, rtol=2e-6, atol=2e-8)
    cm.CUDAMatrix.init_random(1)


@pytest.mark.gpu
@pytest.mark.parametrize("nv,nh,B", [(784, 500, 100), (33, 65, 7), (64, 32, 1), (5, 3, 2), (100, 257, 33), (31, 31, 128)])
def test_cd_update_equals_the_six_reference_calls(cm, rng, nv, nh, B):
    f = lambda a: np.asarray(a, dtype=np.float32, order='F')
    w, bv, bh = f(0.1 * rng.standard_normal((nv, nh))), f(rng.standard_normal((nv, 1))), f(rng.standard_normal((nh, 1)))
    v, v2 = f(rng.random((nv, B)) < 0.3), f(rng.random((nv, B)))
    h, h2 = f(rng.random((nh, B))), f(rng.random((nh, B)))
    eps = 0.01 / B
    V, H, V2, H2 = (cm.CUDAMatrix(a) for a in (v, h, v2, h2))
    W1, BV1, BH1 = cm.CUDAMatrix(w), cm.CUDAMatrix(bv), cm.CUDAMatrix(bh)
    W1.add_dot(V, H.T, mult=eps); W1.add_dot(V2, H2.T, mult=-eps)
    BV1.add_sums(V, axis=1, mult=eps); BV1.add_sums(V2, axis=1, mult=-eps)
    BH1.add_sums(H, axis=1, mult=eps); BH1.add_sums(H2, axis=1, mult=-eps)
    W2, BV2, BH2 = cm.CUDAMatrix(w), cm.CUDAMatrix(bv), cm.CUDAMatrix(bh)
    cm.cd_update(W2, BV2, BH2, V, H, V2, H2, eps)
    d = np.float64
    want_w = w.astype(d) + eps * (v.astype(d) @ h.astype(d).T - v2.astype(d) @ h2.astype(d).T)
    want_bv = bv.astype(d) + eps * (v.astype(d).sum(1, keepdims=True) - v2.astype(d).sum(1, keepdims=True))
    want_bh = bh.astype(d) + eps * (h.astype(d).sum(1, keepdims=True) - h2.astype(d).sum(1, keepdims=True))
    for got, ref, want in ((W2, W1, want_w), (BV2, BV1, want_bv), (BH2, BH1, want_bh)):
        assert np.allclose(got.asarray(), want, rtol=1e-6, atol=1e-7)          # against float64
        assert np.allclose(got.asarray(), ref.asarray(), rtol=2e-6, atol=2e-7)  # against the six calls
        if (nv, nh, B) == (784, 500, 100):      # (the shape of the benchmark runs the six calls' own kernels: same bits)
            assert np.array_equal(got.asarray().view(np.uint32), ref.asarray().view(np.uint32))
    # without the bias vectors; a second call continues from the first
    W3 = cm.CUDAMatrix(w)
    cm.cd_update(W3, None, None, V, H, V2, H2, eps)
    assert np.array_equal(W3.asarray().view(np.uint32), W2.asarray().view(np.uint32))
    cm.cd_update(W3, None, None, V, H, V2, H2, eps)
    assert np.allclose(W3.asarray(), 2 * want_w - w.astype(d), rtol=1e-6, atol=2e-7)
    # shape and flag errors
    assert cm._cudamat.cd_update(W3.p_mat, None, None, V.p_mat, H.p_mat, V2.p_mat, V2.p_mat, 0.1) == (0 if nv == nh else -1)
    assert cm._cudamat.cd_update(W3.p_mat, None, None, V.T.p_mat, H.p_mat, V2.p_mat, H2.p_mat, 0.1) == -5


def _random_small_products(seed, count):
    r = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        m, n = int(r.integers(1, 300)), int(r.integers(1, 300))
        k = int(r.choice([int(r.integers(1, 40)), int(r.integers(40, 1100)), 4 * int(r.integers(8, 260))]))
        out.append((m, k, n, bool(r.integers(0, 2)), bool(r.integers(0, 2)), float(r.choice([0.0, 1.0, -0.5]))))
    return out


@pytest.mark.parametrize("m,k,n,ta,tb,beta", _random_small_products(20240612, 40))
def test_small_products_on_random_shapes(cm, rng, m, k, n, ta, tb, beta):
    # the one-launch kernel for products that cannot fill the chip: ragged tiles, ragged and
    # whole chunks of the reduction, leading dimensions that are and are not multiples of 4
    A, B, C = _rand(rng, (m, k)), _rand(rng, (k, n)), _rand(rng, (m, n))
    a = cm.CUDAMatrix(np.asfortranarray(A.T)) if ta else cm.CUDAMatrix(A)
    b = cm.CUDAMatrix(np.asfortranarray(B.T)) if tb else cm.CUDAMatrix(B)
    c = cm.CUDAMatrix(C) if beta != 0.0 else cm.CUDAMatrix(np.full((m, n), np.nan, dtype=np.float32))
    cm._check(cm._cudamat.dot((a.T if ta else a).p_mat, (b.T if tb else b).p_mat, c.p_mat, beta, 1.5))
    want = 1.5 * (A.astype(np.float64) @ B.astype(np.float64)) + (beta * C.astype(np.float64) if beta != 0.0 else 0.0)
    bound = 1.5 * (np.abs(A).astype(np.float64) @ np.abs(B)) + abs(beta) * np.abs(C) + 1e-30
    assert np.max(np.abs(c.asarray() - want) / bound) < REL
    for h in (a, b, c):
        h.free_device_memory()


@pytest.mark.parametrize("m,k,n", [(1024, 128, 1024), (1000, 100, 1000), (1001, 97, 999), (777, 128, 1100), (784, 1, 1024),
                                   (1022, 7, 1026), (650, 60, 1300)])
@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True), (True, True)])
def test_short_reductions_on_about_one_tile_per_cu(cm, rng, m, k, n, ta, tb):
    """Products with K <= 128 and 128 to 512 tiles of 64 x 64 (on 256 CUs) take the kernel that loads
    the whole K extent at once: whole and ragged tiles, K a multiple of 4 and not (16-byte groups
    or single elements), row counts that are and are not multiples of 4; alpha and a beta that
    reads the target, and the bias / activation epilogue of dot_bias_act."""
    A, B, C = _rand(rng, (m, k)), _rand(rng, (k, n)), _rand(rng, (m, n))
    a = cm.CUDAMatrix(np.asfortranarray(A.T)) if ta else cm.CUDAMatrix(A)
    b = cm.CUDAMatrix(np.asfortranarray(B.T)) if tb else cm.CUDAMatrix(B)
    c = cm.CUDAMatrix(C)
    opa, opb = (a.T if ta else a), (b.T if tb else b)
    cm._check(cm._cudamat.dot(opa.p_mat, opb.p_mat, c.p_mat, -0.5, 2.0))
    prod = A.astype(np.float64) @ B.astype(np.float64)
    want = 2.0 * prod - 0.5 * C
    bound = 2.0 * (np.abs(A).astype(np.float64) @ np.abs(B)) + 0.5 * np.abs(C) + 1e-30
    assert np.max(np.abs(c.asarray() - want) / bound) < REL
    # beta = 0 must not read the target
    c.assign(np.nan)
    cm.dot(opa, opb, target=c)
    assert _relerr(c.asarray(), prod, A, B) < REL
    # the epilogue: bit-identical to the separate calls
    bias = cm.CUDAMatrix(_rand(rng, (m, 1)))
    t1, t2 = cm.empty((m, n)), cm.empty((m, n))
    cm.dot(opa, opb, target=t1); t1.add_col_vec(bias); cm.tanh(t1)
    cm.dot_bias_act(opa, opb, bias, target=t2, act='tanh')
    assert np.array_equal(t1.asarray().view(np.uint32), t2.asarray().view(np.uint32))
    for h in (a, b, c, bias, t1, t2):
        h.free_device_memory()


@pytest.mark.parametrize("m,k,n", [(15, 31, 17), (16, 32, 16), (17, 33, 15), (48, 64, 80), (31, 65, 33), (100, 1029, 20),
                                   (3, 2000, 5), (250, 96, 250)])
@pytest.mark.parametrize("ta,tb", [(False, False), (True, False), (False, True), (True, True)])
def test_small_products_around_the_16_wide_blocks(cm, rng, m, k, n, ta, tb):
    """Shapes that take the 16 x 16 block kernel: edges at 15 / 16 / 17, a reduction that ends
    inside, at and just past a 32-deep chunk, long reductions over few outputs; with alpha and
    a beta that reads the target."""
    A, B, C = _rand(rng, (m, k)), _rand(rng, (k, n)), _rand(rng, (m, n))
    a = cm.CUDAMatrix(np.asfortranarray(A.T)) if ta else cm.CUDAMatrix(A)
    b = cm.CUDAMatrix(np.asfortranarray(B.T)) if tb else cm.CUDAMatrix(B)
    c = cm.CUDAMatrix(C)
    cm._check(cm._cudamat.dot((a.T if ta else a).p_mat, (b.T if tb else b).p_mat, c.p_mat, -0.5, 2.0))
    want = 2.0 * (A.astype(np.float64) @ B.astype(np.float64)) - 0.5 * C
    bound = 2.0 * (np.abs(A).astype(np.float64) @ np.abs(B)) + 0.5 * np.abs(C) + 1e-30
    assert np.max(np.abs(c.asarray() - want) / bound) < REL
    for h in (a, b, c):
        h.free_device_memory()
