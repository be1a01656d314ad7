"""CPU-only pins of the conv / pool / norm restatement: literal loops, torch's
library routines after layout permutes, adjoint identities and finite differences."""
import numpy as np
import pytest
import torch
import torch.nn.functional as TF

from oracle import conv_oracle as co

CASES = [  # N, C, H, F, k, stride, padding, groups
    (2, 3, 6, 16, 3, 1, 0, 1),
    (2, 3, 6, 16, 3, 1, 1, 1),
    (3, 1, 8, 4, 5, 1, 2, 1),
    (2, 4, 7, 4, 3, 2, 1, 2),
    (2, 3, 12, 8, 5, 4, 0, 1),     # the last module stops short of the image edge (as 224/11/4 does)
    (2, 8, 5, 8, 3, 1, 1, 4),
    (1, 2, 9, 6, 3, 3, 0, 2),
]


def _data(rng, N, C, H, F, k, G):
    return rng.standard_normal((N, C * H * H)), rng.standard_normal((F, (C // G) * k * k))


@pytest.mark.parametrize("N,C,H,F,k,s,p,G", CASES)
def test_conv_up_against_loops_and_torch(rng, N, C, H, F, k, s, p, G):
    x, w = _data(rng, N, C, H, F, k, G)
    Mx = co.n_modules(H, k, s, p)
    got = co.conv_up(x, w, C, Mx, p, s, G)
    assert np.allclose(got, co.conv_up_loops(x, w, C, Mx, p, s, G), atol=1e-12)
    # cross-correlation without flip == torch conv2d
    t = TF.conv2d(torch.from_numpy(co.to_nchw(x, C, H)), torch.from_numpy(co.filters_to_fckk(w, C // G, k)),
                  stride=s, padding=p, groups=G).numpy()
    assert t.shape[-1] == Mx
    assert np.allclose(got, t.reshape(N, -1), atol=1e-12)


@pytest.mark.parametrize("N,C,H,F,k,s,p,G", CASES)
def test_conv_down_and_outp_are_the_adjoints(rng, N, C, H, F, k, s, p, G):
    x, w = _data(rng, N, C, H, F, k, G)
    Mx = co.n_modules(H, k, s, p)
    y = rng.standard_normal((N, F * Mx * Mx))
    d = co.conv_down(y, w, C, H, p, s, G)
    assert np.allclose(d, co.conv_down_loops(y, w, C, H, p, s, G), atol=1e-12)
    o = co.conv_outp(x, y, C, Mx, k, p, s, G)
    up = co.conv_up(x, w, C, Mx, p, s, G)
    assert np.isclose((up * y).sum(), (x * d).sum()) and np.isclose((up * y).sum(), (w * o).sum())
    # torch autograd of the forward pass
    xt = torch.from_numpy(co.to_nchw(x, C, H)).requires_grad_()
    wt = torch.from_numpy(co.filters_to_fckk(w, C // G, k)).requires_grad_()
    out = TF.conv2d(xt, wt, stride=s, padding=p, groups=G)
    out.backward(torch.from_numpy(y.reshape(out.shape)))
    assert np.allclose(d, xt.grad.numpy().reshape(N, -1), atol=1e-12)
    assert np.allclose(o, wt.grad.numpy().reshape(F, -1), atol=1e-12)


def test_outp_partial_sums_add_up(rng):
    N, C, H, F, k, s, p = 2, 3, 6, 4, 3, 1, 1
    x, _ = _data(rng, N, C, H, F, k, 1)
    Mx = co.n_modules(H, k, s, p)
    y = rng.standard_normal((N, F * Mx * Mx))
    whole = co.conv_outp(x, y, C, Mx, k, p, s)
    parts = co.conv_outp(x, y, C, Mx, k, p, s, partial_sum=Mx)       # one chunk per module row
    assert parts.shape == (F, Mx * C * k * k)
    assert np.allclose(parts.reshape(F, Mx, C * k * k).sum(axis=1), whole)


@pytest.mark.parametrize("S,subs,start,stride", [(8, 2, 0, 2), (9, 3, 0, 2), (32, 3, 0, 2), (7, 3, -1, 2), (6, 2, 0, 1)])
def test_max_pool_and_undo(rng, S, subs, start, stride):
    N, F = 3, 4
    O = (S - start - subs + stride - 1) // stride + 1            # windows may hang over the far edge
    x = rng.standard_normal((N, F * S * S))
    got = co.max_pool(x, F, subs, start, stride, O)
    if start == 0 and (S - subs) % stride == 0:                   # no clipped window: torch defines the same thing
        t = TF.max_pool2d(torch.from_numpy(co.to_nchw(x, F, S)), subs, stride).numpy()
        assert np.allclose(got, t.reshape(N, -1))
    # brute force
    x4 = co.to_nchw(x, F, S)
    for oy in range(O):
        for ox in range(O):
            win = x4[:, :, max(0, start + oy * stride):start + oy * stride + subs, max(0, start + ox * stride):start + ox * stride + subs]
            assert np.allclose(got.reshape(N, F, O, O)[:, :, oy, ox], win.max(axis=(2, 3)))
    g = rng.standard_normal(got.shape)
    u = co.max_pool_undo(x, g, got, subs, start, stride, O)
    # without ties the undo is the gradient of the pooling
    xt = torch.from_numpy(x4).requires_grad_()
    if start == 0 and (S - subs) % stride == 0:
        TF.max_pool2d(xt, subs, stride).backward(torch.from_numpy(g.reshape(N, F, O, O)))
        assert np.allclose(u, xt.grad.numpy().reshape(N, -1))
    assert np.isclose(u.sum(), g.sum())                           # every output routes its gradient to exactly one pixel


def test_max_pool_undo_gives_the_gradient_to_every_tied_pixel():
    x = np.zeros((1, 16)); x[0, [0, 1]] = 5.0                      # 4x4 image, two equal maxima in the first 2x2 window
    pooled = co.max_pool(x, 1, 2, 0, 2, 2)
    g = np.array([[1.0, 10.0, 100.0, 1000.0]])
    u = co.max_pool_undo(x, g, pooled, 2, 0, 2, 2).reshape(4, 4)
    assert u[0, 0] == 1.0 and u[0, 1] == 1.0                       # both tied pixels (cudamat_conv_kernels.cuh:1502)
    assert u[0, 2] == 10.0 and u[0, 3] == 10.0                     # an all-zero window ties everywhere


def test_prob_max_pool_start_value_overflows(rng):
    x = rng.standard_normal((2, 2 * 36)); r = rng.random((2, 2 * 36))
    out = co.prob_max_pool(x, r, 2, 2, 0, 2, 3)
    assert np.all(out == np.float32(-2e38))                        # (-2e38)^2 = +inf beats every candidate


@pytest.mark.parametrize("size", [3, 5, 4])
def test_response_norm_closed_form_and_gradient(rng, size):
    N, F, S = 2, 3, 7
    a, p = 0.01, 0.75
    x = rng.standard_normal((N, F * S * S))
    t, den = co.response_norm(x, F, size, a, p)
    x4 = torch.from_numpy(co.to_nchw(x, F, S))
    if size % 2 == 1:   # symmetric window: size^2 * avg_pool(x^2) with zero padding
        ap = TF.avg_pool2d(x4 * x4, size, stride=1, padding=size // 2, count_include_pad=True).numpy() * size * size
        assert np.allclose(den, (1 + np.float32(a).astype(np.float64) * ap).reshape(N, -1))
    assert np.allclose(t, x * den ** -np.float64(np.float32(p)))
    # undo == gradient of the forward map, by autograd on the same closed form and by finite differences
    a64, p64 = float(np.float32(a)), float(np.float32(p))

    def fwd(xt):
        S_ = xt.shape[-1]
        sq = xt * xt
        acc = torch.zeros_like(xt)
        lo = -(size // 2)
        for dy in range(lo, lo + size):
            for dx in range(lo, lo + size):
                ys, xs = slice(max(0, -dy), min(S_, S_ - dy)), slice(max(0, -dx), min(S_, S_ - dx))
                yd, xd = slice(max(0, dy), min(S_, S_ + dy)), slice(max(0, dx), min(S_, S_ + dx))
                acc[..., ys, xs] = acc[..., ys, xs] + sq[..., yd, xd]
        return xt * (1 + a64 * acc) ** (-p64)

    xt = x4.clone().requires_grad_()
    g = rng.standard_normal(t.shape)
    fwd(xt).backward(torch.from_numpy(g.reshape(N, F, S, S)))
    undo, acts2 = co.response_norm_undo(g, den, x, t, F, size, a, p)
    assert np.allclose(undo, xt.grad.numpy().reshape(N, -1), atol=1e-10)
    assert np.allclose(acts2, -2 * np.float64(np.float32(-2.0) * np.float32(a) * np.float32(p)) / -2 * g * t / den)
    e = np.zeros_like(x); e[0, 5] = 1e-6
    fd = ((co.response_norm(x + e, F, size, a, p)[0] - co.response_norm(x - e, F, size, a, p)[0]) / 2e-6 * g).sum()
    assert np.isclose(fd, undo[0, 5], rtol=1e-5)


def test_local_layers_reduce_to_conv_with_shared_filters_and_are_adjoint(rng):
    N, C, H, F, k, s, p = 2, 2, 6, 4, 3, 1, 1
    Mx = co.n_modules(H, k, s, p)
    M = Mx * Mx
    x = rng.standard_normal((N, C * H * H))
    w = rng.standard_normal((F, C * k * k))
    w_local = np.tile(w.reshape(F, 1, C * k * k), (1, M, 1)).reshape(F, -1)     # the same bank at every module
    assert np.allclose(co.local_up(x, w_local, C, Mx, p, s), co.conv_up(x, w, C, Mx, p, s))
    wl = rng.standard_normal((F, M * C * k * k))
    y = rng.standard_normal((N, F * M))
    up, down, outp = co.local_up(x, wl, C, Mx, p, s), co.local_down(y, wl, C, H, p, s), co.local_outp(x, y, C, Mx, k, p, s)
    assert np.isclose((up * y).sum(), (x * down).sum()) and np.isclose((up * y).sum(), (wl * outp).sum())


@pytest.mark.parametrize("N,C,H,F,k,s,p,G", [(3, 4, 7, 6, 3, 2, 1, 2), (2, 3, 9, 4, 4, 3, 2, 1), (4, 2, 6, 2, 5, 1, 4, 1)])
def test_single_output_evaluators_agree_with_the_full_passes(rng, N, C, H, F, k, s, p, G):
    # the sampled forms used for full-size device checks, against the vectorised passes
    # (themselves pinned against the literal loops, torch and the adjoint identities)
    Mx = co.n_modules(H, k, s, p)
    x = rng.standard_normal((N, C * H * H))
    w = rng.standard_normal((F, (C // G) * k * k))
    y = rng.standard_normal((N, F * Mx * Mx))
    up = co.conv_up(x, w, C, Mx, p, s, G).reshape(N, F, Mx, Mx)
    down = co.conv_down(y, w, C, H, p, s, G).reshape(N, C, H, H)
    outp = co.conv_outp(x, y, C, Mx, k, p, s, G).reshape(F, C // G, k, k)
    for _ in range(40):
        n, f, my, mx = rng.integers(N), rng.integers(F), rng.integers(Mx), rng.integers(Mx)
        assert abs(co.conv_up_at(x, w, C, Mx, p, s, G, n, f, my, mx)[0] - up[n, f, my, mx]) < 1e-10
        c, yy, xx = rng.integers(C), rng.integers(H), rng.integers(H)
        assert abs(co.conv_down_at(y, w, C, H, p, s, G, n, c, yy, xx)[0] - down[n, c, yy, xx]) < 1e-10
        cl, ky, kx = rng.integers(C // G), rng.integers(k), rng.integers(k)
        assert abs(co.conv_outp_at(x, y, C, Mx, k, p, s, G, f, cl, ky, kx)[0] - outp[f, cl, ky, kx]) < 1e-10


class _Cv(object):
    """Parameter.Convolution with the proto's defaults (deepnet.proto:64-78)."""

    def __init__(self, **kw):
        self.size = self.stride = self.padding = self.num_filters = self.num_colors = 0
        self.max_pool, self.pool_size, self.pool_stride, self.prob = False, 0, 0, False
        self.rnorm, self.norm_size, self.pow_scale, self.add_scale = False, 0, 0.75, 0.001
        self.__dict__.update(kw)


def _torch_stage(x, w, cv, side):
    """The stage in torch on (N, C, H, W) tensors: conv2d -> max_pool2d -> LRN by avg_pool2d."""
    t = TF.conv2d(x, w, stride=cv.stride, padding=cv.padding)
    if cv.max_pool:
        t = TF.max_pool2d(t, cv.pool_size, cv.pool_stride)
    unnorm, den = t, None
    if cv.rnorm:
        den = 1.0 + cv.add_scale_f * cv.norm_size ** 2 * TF.avg_pool2d(t * t, cv.norm_size, 1, cv.norm_size // 2,
                                                                      count_include_pad=True)
        t = t * den ** (-cv.pow_scale_f)
    return t, unnorm, den


@pytest.mark.parametrize("pool,rnorm", [(False, False), (True, False), (False, True), (True, True)])
def test_conv_stage_forward_and_backward_against_torch(rng, pool, rnorm):
    """Forward: the chain in torch.  Backward without normalisation: torch.autograd's gradient of
    that chain (pooling windows that fit the map, no ties).  With normalisation the reference
    feeds ResponseNormUndo its operands in the other order, which is not the true gradient: its
    result is pinned against the same expression written with torch's pooling routines."""
    N, C, H, F, k = 3, 2, 9, 16, 3
    cv = _Cv(size=k, stride=1, padding=1, num_filters=F, num_colors=C, max_pool=pool, pool_size=3, pool_stride=2,
             rnorm=rnorm, norm_size=3)
    cv.add_scale_f, cv.pow_scale_f = float(np.float32(cv.add_scale)), float(np.float32(cv.pow_scale))
    inputs = rng.standard_normal((C * H * H, N))                       # deepnet's (dims, batch)
    w = rng.standard_normal((F, C * k * k))
    fwd = co.stage_forward(inputs, w, cv)
    xt = torch.from_numpy(co.to_nchw(inputs.T, C, H)).requires_grad_(True)
    wt = torch.from_numpy(co.filters_to_fckk(w, C, k)).requires_grad_(True)
    out, unnorm, den = _torch_stage(xt, wt, cv, H)
    assert np.allclose(fwd['state'].T, out.detach().numpy().reshape(N, -1), atol=1e-12)
    deriv = rng.standard_normal(fwd['state'].shape)
    g = torch.from_numpy(deriv.T.reshape(out.shape).copy())
    if rnorm:
        # deepnet's operand order: y_k * window_sum(-2ab * g * x / d) + g * d^-b, then the true
        # gradient of the rest of the chain
        ab = float(np.float32(-2.0) * np.float32(cv.add_scale) * np.float32(cv.pow_scale))
        inner = ab * g * unnorm.detach() / den.detach()
        win = cv.norm_size ** 2 * TF.avg_pool2d(inner, cv.norm_size, 1, cv.norm_size // 2, count_include_pad=True)
        g = out.detach() * win + g * den.detach() ** (-cv.pow_scale_f)
        unnorm.backward(g)
    else:
        out.backward(g)
    d_in, d_w = co.stage_backward(fwd, w, cv, deriv)
    assert np.allclose(d_in.T, xt.grad.numpy().reshape(N, -1), atol=1e-10)
    assert np.allclose(d_w, wt.grad.numpy().reshape(F, -1), atol=1e-10)
