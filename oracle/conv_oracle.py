"""TEST INFRASTRUCTURE ONLY - numpy restatement of cudamat_conv's convolution,
pooling and normalisation.  Only tests/, __graft_entry__.smoke() and bench.py's
cpu_baseline leg may import this; the product (deepnet_amd/) never does.

Tensors are given in the device layout: 2-D arrays of shape (numImages, C*S*S)
whose column index is (c*S + y)*S + x  (cudamat/cudamat_conv.cu:9-13); filters are
(numFilters, Cg*k*k) with column (c*k + ky)*k + kx.  All arithmetic is float64.

Two codings of each convolution pass are kept: `*_loops`, a literal nest of Python
loops over the definition (tiny shapes only), and the vectorised one used on real
sizes.  The reference has no tests for these entry points (nothing under
/root/reference references convUp ... outside convolutions.py), so parity is
pinned here by: loops == vectorised; == torch.nn.functional.conv2d / max_pool2d /
avg_pool2d after layout permutes where those define the same thing; the adjoint
identities <convUp(x,w),y> = <x,convDown(y,w)> = <w,convOutp(x,y)>; and float64
finite differences for the normalisation gradient (tests/test_oracle_conv.py).
The tie rule of MaxPoolUndo (every tied position receives the gradient,
cudamat_conv_kernels.cuh:1502) is pinned by a hand-made case only.
"""
import numpy as np

F64 = np.float64


def to_nchw(mat, C, S):
    """(N, C*S*S) device layout -> (N, C, S, S)."""
    mat = np.asarray(mat, dtype=F64)
    return mat.reshape(mat.shape[0], C, S, S)


def from_nchw(t):
    return np.asarray(t, dtype=F64).reshape(t.shape[0], -1)


def filters_to_fckk(flt, Cg, k):
    """(F, Cg*k*k) -> (F, Cg, k, k)."""
    flt = np.asarray(flt, dtype=F64)
    return flt.reshape(flt.shape[0], Cg, k, k)


def n_modules(H, k, stride, padding):
    """deepnet/convolutions.py:35: n_locs = (x + 2p - size) / stride + 1 (floor)."""
    return (H + 2 * padding - k) // stride + 1


# ---- filterActs: cudamat_conv.cu:15-257, cudamat_conv_kernels.cuh:82-394 ----------

def conv_up_loops(images, filters, C, Mx, padding, stride, groups=1):
    """out[n, f, my, mx] = sum_{c,ky,kx} img[n, g*Cg+c, my*s+ky-p, mx*s+kx-p] * w[f, c, ky, kx]; zero outside."""
    images = np.asarray(images, dtype=F64)
    filters = np.asarray(filters, dtype=F64)
    N = images.shape[0]
    H = int(round(np.sqrt(images.shape[1] // C)))
    F = filters.shape[0]
    Cg = C // groups
    k = int(round(np.sqrt(filters.shape[1] // Cg)))
    Fg = F // groups
    out = np.zeros((N, F * Mx * Mx))
    for n in range(N):
        for f in range(F):
            g = f // Fg
            for my in range(Mx):
                for mx in range(Mx):
                    acc = 0.0
                    for c in range(Cg):
                        for ky in range(k):
                            for kx in range(k):
                                y, x = my * stride + ky - padding, mx * stride + kx - padding
                                if 0 <= y < H and 0 <= x < H:
                                    acc += images[n, ((g * Cg + c) * H + y) * H + x] * filters[f, (c * k + ky) * k + kx]
                    out[n, (f * Mx + my) * Mx + mx] = acc
    return out


def _geom(images, filters, C, groups):
    N = images.shape[0]
    H = int(round(np.sqrt(images.shape[1] // C)))
    F = filters.shape[0]
    Cg = C // groups
    k = int(round(np.sqrt(filters.shape[1] // Cg)))
    return N, H, F, Cg, k, F // groups


def _patch_view(xp, ky, kx, Mx, stride):
    """xp: padded (N, C, Hp, Hp) -> (N, C, Mx, Mx) samples at module origin + (ky, kx)."""
    return xp[:, :, ky:ky + (Mx - 1) * stride + 1:stride, kx:kx + (Mx - 1) * stride + 1:stride]


def _pad_for(H, k, Mx, padding, stride):
    """Zero border wide enough for every module, including ones reaching past the far edge."""
    far = max(0, (Mx - 1) * stride + k - padding - H)
    return padding, far


def conv_up(images, filters, C, Mx, padding, stride, groups=1):
    images = np.asarray(images, dtype=F64)
    filters = np.asarray(filters, dtype=F64)
    N, H, F, Cg, k, Fg = _geom(images, filters, C, groups)
    x = to_nchw(images, C, H)
    w = filters_to_fckk(filters, Cg, k)
    lo, hi = _pad_for(H, k, Mx, padding, stride)
    xp = np.pad(x, ((0, 0), (0, 0), (lo, hi), (lo, hi)))
    out = np.zeros((N, F, Mx, Mx))
    for g in range(groups):
        xs = xp[:, g * Cg:(g + 1) * Cg]
        ws = w[g * Fg:(g + 1) * Fg]
        for ky in range(k):
            for kx in range(k):
                out[:, g * Fg:(g + 1) * Fg] += np.einsum('ncyx,fc->nfyx', _patch_view(xs, ky, kx, Mx, stride), ws[:, :, ky, kx])
    return from_nchw(out)


# ---- imgActs: cudamat_conv.cu:265-640 ------------------------------------------------

def conv_down(hid, filters, C, H, padding, stride, groups=1):
    """Adjoint of conv_up w.r.t. the images."""
    hid = np.asarray(hid, dtype=F64)
    filters = np.asarray(filters, dtype=F64)
    N, F = hid.shape[0], filters.shape[0]
    Cg = C // groups
    k = int(round(np.sqrt(filters.shape[1] // Cg)))
    Fg = F // groups
    Mx = int(round(np.sqrt(hid.shape[1] // F)))
    h = hid.reshape(N, F, Mx, Mx)
    w = filters_to_fckk(filters, Cg, k)
    lo, hi = _pad_for(H, k, Mx, padding, stride)
    gp = np.zeros((N, C, H + lo + hi, H + lo + hi))
    for g in range(groups):
        hs = h[:, g * Fg:(g + 1) * Fg]
        ws = w[g * Fg:(g + 1) * Fg]
        for ky in range(k):
            for kx in range(k):
                _patch_view(gp[:, g * Cg:(g + 1) * Cg], ky, kx, Mx, stride)[...] += np.einsum('nfyx,fc->ncyx', hs, ws[:, :, ky, kx])
    return from_nchw(gp[:, :, lo:lo + H, lo:lo + H])


def conv_down_loops(hid, filters, C, H, padding, stride, groups=1):
    hid = np.asarray(hid, dtype=F64)
    filters = np.asarray(filters, dtype=F64)
    N, F = hid.shape[0], filters.shape[0]
    Cg = C // groups
    k = int(round(np.sqrt(filters.shape[1] // Cg)))
    Fg = F // groups
    Mx = int(round(np.sqrt(hid.shape[1] // F)))
    out = np.zeros((N, C * H * H))
    for n in range(N):
        for f in range(F):
            g = f // Fg
            for my in range(Mx):
                for mx in range(Mx):
                    hv = hid[n, (f * Mx + my) * Mx + mx]
                    for c in range(Cg):
                        for ky in range(k):
                            for kx in range(k):
                                y, x = my * stride + ky - padding, mx * stride + kx - padding
                                if 0 <= y < H and 0 <= x < H:
                                    out[n, ((g * Cg + c) * H + y) * H + x] += hv * filters[f, (c * k + ky) * k + kx]
    return out


# ---- weightActs: cudamat_conv.cu:642-1015 ----------------------------------------------

def conv_outp(images, hid, C, Mx, k, padding, stride, groups=1, partial_sum=0):
    """dw[f, c, ky, kx] = sum_{n, my, mx} img[n, g*Cg+c, my*s+ky-p, mx*s+kx-p] * hid[n, f, my, mx].
    With partial_sum the modules are summed in consecutive chunks of that many and the
    result is (F, chunks*Cg*k*k), chunk-major."""
    images = np.asarray(images, dtype=F64)
    hid = np.asarray(hid, dtype=F64)
    N = images.shape[0]
    H = int(round(np.sqrt(images.shape[1] // C)))
    F = hid.shape[1] // (Mx * Mx)
    Cg, Fg = C // groups, F // groups
    x = to_nchw(images, C, H)
    h = hid.reshape(N, F, Mx, Mx)
    lo, hi = _pad_for(H, k, Mx, padding, stride)
    xp = np.pad(x, ((0, 0), (0, 0), (lo, hi), (lo, hi)))
    M = Mx * Mx
    ps = M if partial_sum == 0 else partial_sum
    chunks = M // ps
    out = np.zeros((chunks, F, Cg, k, k))
    for g in range(groups):
        xs = xp[:, g * Cg:(g + 1) * Cg]
        hs = h[:, g * Fg:(g + 1) * Fg].reshape(N, Fg, M)
        for ky in range(k):
            for kx in range(k):
                pv = _patch_view(xs, ky, kx, Mx, stride).reshape(N, Cg, M)
                for ch in range(chunks):
                    sl = slice(ch * ps, (ch + 1) * ps)
                    out[ch, g * Fg:(g + 1) * Fg, :, ky, kx] = np.einsum('ncm,nfm->fc', pv[:, :, sl], hs[:, :, sl])
    return np.concatenate([out[ch].reshape(F, -1) for ch in range(chunks)], axis=1)


# ---- locally connected layers: cudamat_conv.cu:1415-1423, filters (module, colour, ky, kx, filter) ----

# ---- single outputs of the three passes: for checks at sizes where the full float64
# ---- convolution would take minutes.  Each returns (value, sum of |terms|).

def conv_up_at(images, filters, C, Mx, padding, stride, groups, n, f, my, mx):
    """targets[n, (f, my, mx)] of convUp, straight from the definition
    (cudamat_conv_kernels.cuh:82-257: out = sum_{c,ky,kx} img(g*Cg+c, my*s-pad+ky, mx*s-pad+kx) * w(f, c, ky, kx))."""
    N, H, F, Cg, k, Fg = _geom(images, filters, C, groups)
    g = f // Fg
    w = np.asarray(filters[f], dtype=F64).reshape(Cg, k, k)
    x = np.asarray(images[n], dtype=F64).reshape(C, H, H)[g * Cg:(g + 1) * Cg]
    val = mag = 0.0
    for ky in range(k):
        y = my * stride - padding + ky
        if not 0 <= y < H:
            continue
        for kx in range(k):
            xx = mx * stride - padding + kx
            if 0 <= xx < H:
                t = x[:, y, xx] * w[:, ky, kx]
                val += t.sum(); mag += np.abs(t).sum()
    return val, mag


def conv_down_at(hid, filters, C, H, padding, stride, groups, n, c, y, x):
    """targets[n, (c, y, x)] of convDown: the sum over the group's filters and over the
    modules (my, mx) whose tap (y + pad - my*s, x + pad - mx*s) exists
    (cudamat_conv_kernels.cuh:265-640)."""
    hid = np.asarray(hid)
    F = filters.shape[0]
    Cg = C // groups
    Fg = F // groups
    k = int(round((filters.shape[1] // Cg) ** 0.5))
    M = hid.shape[1] // F
    Mx = int(round(M ** 0.5))
    g, cl = c // Cg, c % Cg
    w = np.asarray(filters[g * Fg:(g + 1) * Fg], dtype=F64).reshape(Fg, Cg, k, k)[:, cl]
    h = np.asarray(hid[n], dtype=F64).reshape(F, Mx, Mx)[g * Fg:(g + 1) * Fg]
    val = mag = 0.0
    for my in range(Mx):
        ky = y + padding - my * stride
        if not 0 <= ky < k:
            continue
        for mx in range(Mx):
            kx = x + padding - mx * stride
            if 0 <= kx < k:
                t = h[:, my, mx] * w[:, ky, kx]
                val += t.sum(); mag += np.abs(t).sum()
    return val, mag


def conv_outp_at(images, hid, C, Mx, k, padding, stride, groups, f, c, ky, kx):
    """targets[f, (c, ky, kx)] of convOutp with one module group (c counts colours of
    f's group): the sum over all modules and images (cudamat_conv_kernels.cuh:642-1015)."""
    images, hid = np.asarray(images), np.asarray(hid)
    N = images.shape[0]
    H = int(round((images.shape[1] // C) ** 0.5))
    F = hid.shape[1] // (Mx * Mx)
    Cg, Fg = C // groups, F // groups
    g = f // Fg
    x = images.reshape(N, C, H, H)[:, g * Cg + c]
    h = hid.reshape(N, F, Mx, Mx)[:, f]
    val = mag = 0.0
    for my in range(Mx):
        y = my * stride - padding + ky
        if not 0 <= y < H:
            continue
        xs = np.arange(Mx) * stride - padding + kx
        ok = (xs >= 0) & (xs < H)
        t = x[:, y, xs[ok]].astype(F64) * h[:, my, ok].astype(F64)
        val += t.sum(); mag += np.abs(t).sum()
    return val, mag


def local_up(images, filters, C, Mx, padding, stride):
    """Like conv_up with a separate filter bank per module: filters is (F, M*C*k*k) with
    column ((m*C + c)*k + ky)*k + kx."""
    images = np.asarray(images, dtype=F64)
    filters = np.asarray(filters, dtype=F64)
    N = images.shape[0]
    H = int(round(np.sqrt(images.shape[1] // C)))
    F = filters.shape[0]
    M = Mx * Mx
    k = int(round(np.sqrt(filters.shape[1] // (M * C))))
    w = filters.reshape(F, M, C, k, k)
    lo, hi = _pad_for(H, k, Mx, padding, stride)
    xp = np.pad(to_nchw(images, C, H), ((0, 0), (0, 0), (lo, hi), (lo, hi)))
    out = np.zeros((N, F, Mx, Mx))
    for my in range(Mx):
        for mx in range(Mx):
            patch = xp[:, :, my * stride:my * stride + k, mx * stride:mx * stride + k]
            out[:, :, my, mx] = np.einsum('ncyx,fcyx->nf', patch, w[:, my * Mx + mx])
    return from_nchw(out)


def local_down(hid, filters, C, H, padding, stride):
    hid = np.asarray(hid, dtype=F64)
    filters = np.asarray(filters, dtype=F64)
    N, F = hid.shape[0], filters.shape[0]
    Mx = int(round(np.sqrt(hid.shape[1] // F)))
    M = Mx * Mx
    k = int(round(np.sqrt(filters.shape[1] // (M * C))))
    w = filters.reshape(F, M, C, k, k)
    h = hid.reshape(N, F, Mx, Mx)
    lo, hi = _pad_for(H, k, Mx, padding, stride)
    gp = np.zeros((N, C, H + lo + hi, H + lo + hi))
    for my in range(Mx):
        for mx in range(Mx):
            gp[:, :, my * stride:my * stride + k, mx * stride:mx * stride + k] += np.einsum(
                'nf,fcyx->ncyx', h[:, :, my, mx], w[:, my * Mx + mx])
    return from_nchw(gp[:, :, lo:lo + H, lo:lo + H])


def local_outp(images, hid, C, Mx, k, padding, stride):
    """(F, M*C*k*k): per-module weight gradient == conv_outp with one module per chunk."""
    return conv_outp(images, hid, C, Mx, k, padding, stride, partial_sum=1)


# ---- pooling: cudamat_conv.cu:1021-1182, cudamat_conv_kernels.cuh:1355-1530 -------------

def max_pool(images, F, subs, start, stride, O):
    images = np.asarray(images, dtype=F64)
    N = images.shape[0]
    S = int(round(np.sqrt(images.shape[1] // F)))
    x = to_nchw(images, F, S)
    out = np.full((N, F, O, O), -2e38)
    for oy in range(O):
        for ox in range(O):
            y0, x0 = max(0, start + oy * stride), max(0, start + ox * stride)
            y1, x1 = min(S, start + oy * stride + subs), min(S, start + ox * stride + subs)
            if y1 > y0 and x1 > x0:
                out[:, :, oy, ox] = np.maximum(x[:, :, y0:y1, x0:x1].max(axis=(2, 3)), -2e38)
    return from_nchw(out)


def max_pool_undo(images, max_grads, max_acts, subs, start, stride, O):
    """target[px] = sum over outputs whose window holds px of (img[px] == maxAct[o]) * maxGrad[o]."""
    images = np.asarray(images, dtype=F64)
    N = images.shape[0]
    F = max_grads.shape[1] // (O * O)
    S = int(round(np.sqrt(images.shape[1] // F)))
    x = to_nchw(images, F, S)
    mg = np.asarray(max_grads, dtype=F64).reshape(N, F, O, O)
    ma = np.asarray(max_acts, dtype=F64).reshape(N, F, O, O)
    out = np.zeros((N, F, S, S))
    for oy in range(O):
        for ox in range(O):
            y0, x0 = max(0, start + oy * stride), max(0, start + ox * stride)
            y1, x1 = min(S, start + oy * stride + subs), min(S, start + ox * stride + subs)
            if y1 > y0 and x1 > x0:
                hit = x[:, :, y0:y1, x0:x1] == ma[:, :, oy, ox][:, :, None, None]
                out[:, :, y0:y1, x0:x1] += hit * mg[:, :, oy, ox][:, :, None, None]
    return from_nchw(out)


def prob_max_pool(images, rnd, F, subs, start, stride, O):
    """The reference's scan (cudamat_conv_kernels.cuh:44-55, 1594-1608) in float32: the
    candidate replaces the running value unless running*r_running > candidate*r_candidate,
    starting from (-2e38, -2e38), whose product overflows to +inf."""
    images = np.asarray(images, dtype=np.float32)
    rnd = np.asarray(rnd, dtype=np.float32)
    N = images.shape[0]
    S = int(round(np.sqrt(images.shape[1] // F)))
    x = images.reshape(N, F, S, S)
    r = rnd.reshape(N, F, S, S)
    out = np.empty((N, F, O, O), dtype=np.float32)
    with np.errstate(over='ignore', invalid='ignore'):
        for oy in range(O):
            for ox in range(O):
                acc = np.full((N, F), -2e38, dtype=np.float32)
                racc = np.full((N, F), -2e38, dtype=np.float32)
                for y in range(max(0, start + oy * stride), min(S, start + oy * stride + subs)):
                    for xx in range(max(0, start + ox * stride), min(S, start + ox * stride + subs)):
                        keep = acc * racc > x[:, :, y, xx] * r[:, :, y, xx]
                        acc = np.where(keep, acc, x[:, :, y, xx])
                        racc = np.where(keep, racc, r[:, :, y, xx])
                out[:, :, oy, ox] = acc
    return out.reshape(N, -1).astype(F64)


# ---- normalisation: cudamat_conv_kernels.cu:112-176, cudamat_conv_kernels.cuh:1920-2023 ----

def _window_sum(t, size, lo_off):
    """Sum over the clipped window [p + lo_off, p + lo_off + size) along the last two axes."""
    S = t.shape[-1]
    out = np.zeros_like(t)
    for dy in range(lo_off, lo_off + size):
        for dx in range(lo_off, lo_off + size):
            if abs(dy) >= S or abs(dx) >= S:
                continue            # this shift moves the whole map out of the window
            ys, xs = slice(max(0, -dy), min(S, S - dy)), slice(max(0, -dx), min(S, S - dx))
            yd, xd = slice(max(0, dy), min(S, S + dy)), slice(max(0, dx), min(S, S + dx))
            out[..., ys, xs] += t[..., yd, xd]
    return out


def contrast_norm(images, mean_diffs, F, size, add_scale, pow_scale):
    """denoms = 1 + addScale * sum_{window at -size/2} meanDiffs^2; target = images * denoms^-powScale."""
    images = np.asarray(images, dtype=F64)
    S = int(round(np.sqrt(images.shape[1] // F)))
    x = to_nchw(images, F, S)
    md = to_nchw(mean_diffs, F, S)
    den = 1.0 + F64(np.float32(add_scale)) * _window_sum(md * md, size, -(size // 2))
    return from_nchw(x * den ** (-F64(np.float32(pow_scale)))), from_nchw(den)


def response_norm(images, F, size, add_scale, pow_scale):
    return contrast_norm(images, images, F, size, add_scale, pow_scale)


def response_norm_undo(out_grads, denoms, inputs, acts, F, size, add_scale, pow_scale):
    """Returns (target, acts_after): acts' = -2*addScale*powScale*outGrads*acts/denoms;
    target = inputs * sum_{mirrored window} acts' + outGrads * denoms^-powScale."""
    og = np.asarray(out_grads, dtype=F64)
    S = int(round(np.sqrt(og.shape[1] // F)))
    a, p = F64(np.float32(add_scale)), F64(np.float32(pow_scale))
    og4, den4, in4, act4 = (to_nchw(t, F, S) for t in (out_grads, denoms, inputs, acts))
    act2 = F64(np.float32(-2.0) * np.float32(add_scale) * np.float32(pow_scale)) * og4 * act4 / den4
    win = _window_sum(act2, size, size // 2 - size + 1)
    return from_nchw(in4 * win + og4 * den4 ** (-p)), from_nchw(act2)


# ---- the conv stage of an edge: deepnet/convolutions.py:5-184 -------------------------------
# cv is any object with the fields of Parameter.Convolution (deepnet.proto:64-78).  Layer
# states are (dims, batch) as in deepnet; everything in between is in the device layout.

def _stage_sites(cv, numdims):
    side = int(round(np.sqrt(numdims // cv.num_colors)))
    n_locs = n_modules(side, cv.size, cv.stride, cv.padding)                       # convolutions.py:35
    n_pool = (n_locs - cv.pool_size) // cv.pool_stride + 1 if cv.max_pool else n_locs   # :48
    return side, n_locs, n_pool


def stage_forward(inputs, w, cv, local=False):
    """ConvolveUp (convolutions.py:5-67) without probabilistic pooling.  Returns a dict with
    the state (dims_out, batch) and every intermediate the backward pass reads."""
    x_t = np.asarray(inputs, dtype=F64).T
    side, n_locs, n_pool = _stage_sites(cv, x_t.shape[1])
    up = local_up if local else conv_up
    keep = {'input_t': x_t}
    cur = up(x_t, w, cv.num_colors, n_locs, cv.padding, cv.stride)
    if cv.max_pool:
        keep['unpooled'] = cur
        cur = max_pool(cur, cv.num_filters, cv.pool_size, 0, cv.pool_stride, n_pool)
    if cv.rnorm:
        keep['unnormalized'] = cur
        cur, keep['denoms'] = response_norm(cur, cv.num_filters, cv.norm_size, cv.add_scale, cv.pow_scale)
    keep['output_t'] = cur
    keep['state'] = cur.T
    return keep


def stage_backward(fwd, w, cv, deriv, local=False):
    """AccumulateConvDeriv + ConvOuter (convolutions.py:69-184) on what stage_forward kept:
    returns (gradient w.r.t. the inputs as (dims_in, batch), gradient w.r.t. the weights).
    The normalisation step is given the operands in deepnet's order (:120-122): the normalised
    outputs where the library call names `inputs`, the un-normalised layer where it names `acts`."""
    grads = np.asarray(deriv, dtype=F64).T
    acts = fwd['output_t']
    side, n_locs, n_pool = _stage_sites(cv, fwd['input_t'].shape[1])
    if cv.rnorm:
        grads, _ = response_norm_undo(grads, fwd['denoms'], acts, fwd['unnormalized'], cv.num_filters,
                                      cv.norm_size, cv.add_scale, cv.pow_scale)
        acts = fwd['unnormalized']
    if cv.max_pool:
        grads = max_pool_undo(fwd['unpooled'], grads, acts, cv.pool_size, 0, cv.pool_stride, n_pool)
    if local:
        d_in = local_down(grads, w, cv.num_colors, side, cv.padding, cv.stride)
        d_w = local_outp(fwd['input_t'], grads, cv.num_colors, n_locs, cv.size, cv.padding, cv.stride)
    else:
        d_in = conv_down(grads, w, cv.num_colors, side, cv.padding, cv.stride)
        d_w = conv_outp(fwd['input_t'], grads, cv.num_colors, n_locs, cv.size, cv.padding, cv.stride)
    return d_in.T, d_w
