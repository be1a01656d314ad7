"""TEST INFRASTRUCTURE ONLY - numpy restatement of the matrix ops of cudamat.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this; the product (deepnet_amd/) never does.

Every function takes numpy arrays (any float dtype, logical shape = the
CUDAMatrix shape) and evaluates the reference's formula in float64; callers
round to float32 and compare within the stated tolerance.  Each function cites
the kernel or wrapper it restates (paths relative to the reference tree).

How the restatement is pinned (the reference ships no golden vectors and cannot
be built here - no nvcc, no Eigen, Python 2 sources):
  * elementwise / broadcast / compare: closed forms; tests compare against
    independent library routines (scipy.special.expit, np.tanh, np.logaddexp ...)
    and special values, so a dropped term or a swapped operand fails.
  * reductions, softmax: numpy/scipy library routines of the same definition.
  * dot: np.dot in float64 for the four transpose combinations.
  * conv / pool / norm: conv_oracle.py (brute force + torch cross-checks).
The arg-max tie rule, choose_max and the NaN conventions of the gather ops
follow the device kernels' text and are pinned only by hand-written cases:
"parity unpinned" beyond those.
"""
import numpy as np

F64 = np.float64


def _a(x):
    return np.asarray(x, dtype=F64)


# ---- unary: cudamat_kernels.cu:386-506 -------------------------------------

def sign(x):
    x = _a(x)
    out = np.where(x != 0, np.copysign(1.0, x), 0.0)  # NaN is "truthy" in C: copysign(1, NaN)
    return out


def apply_cos(x): return np.cos(_a(x))
def apply_sin(x): return np.sin(_a(x))


def apply_sigmoid(x):
    with np.errstate(over='ignore'):
        return 1.0 / (1.0 + np.exp(-_a(x)))


def apply_tanh(x):
    # 1 - 2 / (exp(2x) + 1)   (cudamat_kernels.cu:410-419)
    with np.errstate(over='ignore'):
        return 1.0 - 2.0 / (np.exp(2.0 * _a(x)) + 1.0)


def apply_abs(x):
    x = _a(x)
    return x * ((x > 0).astype(F64) - (x < 0).astype(F64))


def apply_log_1_plus_exp(x):
    # log(1 + exp(x)), branches as in cudamat_kernels.cu:427-438; log1p keeps the
    # float64 evaluation faithful to the formula when exp(.) is far below 1
    x = _a(x)
    with np.errstate(over='ignore'):
        return np.where(x > 0, np.log1p(np.exp(-x)) + x, np.log1p(np.exp(x)))


def apply_log(x, tiny=0.0):
    # the sum x + tiny is formed in float32 on the device
    with np.errstate(divide='ignore', invalid='ignore'):
        return np.log((np.asarray(x, np.float32) + np.float32(tiny)).astype(F64))


def apply_exp(x):
    with np.errstate(over='ignore'):
        return np.exp(_a(x))


def apply_ceil(x): return np.ceil(_a(x))
def apply_floor(x): return np.floor(_a(x))


def apply_sqrt(x):
    with np.errstate(invalid='ignore'):
        return np.sqrt(_a(x))


def apply_pow(x, p):
    with np.errstate(all='ignore'):
        return np.power(_a(x), F64(np.float32(p)))


def apply_pow_matrix(x, p):
    with np.errstate(all='ignore'):
        return np.power(_a(x), _a(p))


def reciprocal(x):
    with np.errstate(divide='ignore'):
        return 1.0 / _a(x)


# ---- binary: cudamat_kernels.cu:298-364, 600-685 ----------------------------

def less_than(a, b): return (_a(a) < _a(b)).astype(F64)
def less_than_eq(a, b): return (_a(a) <= _a(b)).astype(F64)
def greater_than(a, b): return (_a(a) > _a(b)).astype(F64)
def greater_than_eq(a, b): return (_a(a) >= _a(b)).astype(F64)
def upper_bound(a, b): return np.where(_a(a) > _a(b), _a(b), _a(a))
def lower_bound(a, b): return np.where(_a(a) < _a(b), _a(b), _a(a))
def add_elementwise(a, b): return _a(a) + _a(b)
def subtract_elementwise(a, b): return _a(a) - _a(b)
def mult_elementwise(a, b): return _a(a) * _a(b)


def divide_elementwise(a, b):
    with np.errstate(all='ignore'):
        return _a(a) / _a(b)


def apply_cos_deriv(a, b): return -_a(a) * np.sin(_a(b))
def apply_sin_deriv(a, b): return _a(a) * np.cos(_a(b))
def apply_logistic_deriv(a, b): return _a(a) * _a(b) * (1.0 - _a(b))
def apply_tanh_deriv(a, b): return _a(a) * (1.0 + _a(b)) * (1.0 - _a(b)) * 0.5
def apply_rectified_linear_deriv(a, b): return _a(a) * (_a(b) > 0)
def apply_rectified_linear_smooth_deriv(a, b): return _a(a) * -np.expm1(-_a(b))  # a*(1 - exp(-b))
def add_mult(a, b, alpha): return _a(a) + F64(np.float32(alpha)) * _a(b)


def add_mult_sign(a, b, mult):
    b = _a(b)
    m = F64(np.float32(mult))
    return _a(a) + np.where(b > 0, m, np.where(b < 0, -m, 0.0))


def compute_cross_entropy(t, p, tiny):
    with np.errstate(all='ignore'):
        return -_a(t) * np.log((np.asarray(p, np.float32) + np.float32(tiny)).astype(F64))


def compute_cross_entropy_bernoulli(t, p, tiny):
    p32 = np.asarray(p, np.float32)
    with np.errstate(all='ignore'):
        return (-_a(t) * np.log((p32 + np.float32(tiny)).astype(F64))
                - (1.0 - _a(t)) * np.log((np.float32(1) - p32 + np.float32(tiny)).astype(F64)))


def correct_preds(t, p, cutoff):
    c = F64(np.float32(cutoff))
    return _a(t) * (_a(p) >= c) + (1.0 - _a(t)) * (_a(p) < c)


# ---- scalar: cudamat_kernels.cu:310-364, 687-716 ----------------------------

def mult_by_scalar(a, s): return F64(np.float32(s)) * _a(a)
def add_scalar(a, s): return _a(a) + F64(np.float32(s))


def divide_by_scalar(a, s):
    with np.errstate(all='ignore'):
        return _a(a) / F64(np.float32(s))


# ---- broadcasts: cudamat_kernels.cu:508-598 --------------------------------

def add_col_vec(a, v): return _a(a) + _a(v).reshape(-1, 1)
def add_col_mult(a, v, m): return _a(a) + F64(np.float32(m)) * _a(v).reshape(-1, 1)
def add_row_vec(a, v): return _a(a) + _a(v).reshape(1, -1)
def add_row_mult(a, v, m): return _a(a) + F64(np.float32(m)) * _a(v).reshape(1, -1)
def mult_by_col_vec(a, v): return _a(a) * _a(v).reshape(-1, 1)
def mult_by_row_vec(a, v): return _a(a) * _a(v).reshape(1, -1)


def div_by_col_vec(a, v):
    with np.errstate(all='ignore'):
        return _a(a) / _a(v).reshape(-1, 1)


def div_by_row_vec(a, v):
    with np.errstate(all='ignore'):
        return _a(a) / _a(v).reshape(1, -1)


def diagonal_op(a, val, op):
    """add_diagonal / mult_diagonal (+ _scalar): only the diagonal changes
    (cudamat_kernels.cu:515-545)."""
    out = _a(a).copy()
    idx = np.arange(out.shape[1])
    v = _a(val).ravel() if np.ndim(val) else F64(np.float32(val))
    out[idx, idx] = out[idx, idx] + v if op == 'add' else out[idx, idx] * v
    return out


# ---- contraction: cudamat.cu:1671-1696 --------------------------------------

def dot(a, b, c=None, beta=0.0, alpha=1.0, trans_a=False, trans_b=False):
    """beta*c + alpha*op(a).op(b); a, b given as stored (before op)."""
    A = _a(a).T if trans_a else _a(a)
    B = _a(b).T if trans_b else _a(b)
    out = F64(np.float32(alpha)) * (A @ B)
    if beta != 0.0:
        out = out + F64(np.float32(beta)) * _a(c)
    return out


def sparse_dot(data, indices, indptr, dense, target=None, beta=0.0, alpha=1.0):
    """CSR (m x k) times dense (k x n): the loop of kSparseDot (cudamat_kernels.cu:370-384),
    target[row, col] = alpha * sum_i data[i] * dense[indices[i], col] + beta * target[row, col]
    over i in [indptr[row], indptr[row+1]), summed in float64 here.  The launcher
    (cudamat.cu:1698-1727) reads dense and target as plain column-major arrays."""
    dense = _a(dense)
    m, n = len(indptr) - 1, dense.shape[1]
    out = np.zeros((m, n), dtype=F64)
    for row in range(m):
        for i in range(int(indptr[row]), int(indptr[row + 1])):
            out[row, :] += F64(np.float32(data[i])) * dense[int(indices[i]), :]
    out = F64(np.float32(alpha)) * out
    if beta != 0.0:
        out = out + F64(np.float32(beta)) * _a(target)
    return out


# ---- reductions: cudamat.cu:1148-1315, cudamat_kernels.cu:936-1088 ----------

FLT_MAX = float(np.finfo(np.float32).max)


def max_by_axis(x, axis):
    """axis 0: start value -FLT_MAX and strict '>' (cudamat_kernels.cu:1002-1018).
    axis 1: first element start, as eigenmat/eigenmat.cc:617-639."""
    x = _a(x)
    if axis == 0:
        return np.maximum(np.max(x, axis=0, keepdims=True), -FLT_MAX)
    return np.max(x, axis=1, keepdims=True)


def argmax_ref_order(col):
    """Arg-max of one column in the reference's scan order (cudamat_kernels.cu:1020-1050):
    32 lanes, lane t scans rows t, t+32, ... keeping the first strictly larger value;
    then lanes are scanned in order, again strictly larger.  Start (-FLT_MAX, 0)."""
    col = np.asarray(col, dtype=np.float32)
    lane_max = np.full(32, -np.float32(FLT_MAX), dtype=np.float32)
    lane_arg = np.zeros(32, dtype=np.int64)
    for i, v in enumerate(col):
        t = i % 32
        if v > lane_max[t]:
            lane_max[t] = v
            lane_arg[t] = i
    cur_max, cur_arg = -np.float32(FLT_MAX), 0
    for t in range(32):
        if lane_max[t] > cur_max:
            cur_max, cur_arg = lane_max[t], lane_arg[t]
    return int(cur_arg)


def argmax_by_axis(x, axis):
    x = np.asarray(x, dtype=np.float32)
    if axis == 0:
        return np.array([[argmax_ref_order(x[:, j]) for j in range(x.shape[1])]], dtype=F64)
    return np.argmax(x, axis=1).reshape(-1, 1).astype(F64)  # first occurrence (eigenmat.cc:700-709)


def choose_max_by_axis(x, axis):
    """One-hot of the arg-max (the intended result; the reference kernel clears the
    wrong column, cudamat_kernels.cu:980)."""
    x = np.asarray(x, dtype=np.float32)
    out = np.zeros(x.shape, dtype=F64)
    am = argmax_by_axis(x, axis).astype(int)
    if axis == 0:
        out[am.ravel(), np.arange(x.shape[1])] = 1.0
    else:
        out[np.arange(x.shape[0]), am.ravel()] = 1.0
    return out


def sqsum_by_axis(x, target, axis, mult, p):
    """target = p*target + mult*sum(x^2) (cudamat_kernels.cu:1052-1066)."""
    s = np.sum(_a(x) ** 2, axis=axis, keepdims=True)
    out = F64(np.float32(mult)) * s
    if p != 0.0:
        out = out + F64(np.float32(p)) * _a(target)
    return out


def normlimit_by_axis(x, axis, norm):
    """cudamat_kernels.cu:1068-1088: scale = norm_of_line < norm ? 1 : norm / norm_of_line."""
    x = _a(x)
    n = np.sqrt(np.sum(x ** 2, axis=axis, keepdims=True))
    with np.errstate(all='ignore'):
        scale = np.where(n < norm, 1.0, norm / n)
    return x * scale


def softmax(x):
    """Per column: exp(x - max) / sum (cudamat_kernels.cu:868-934)."""
    x = _a(x)
    e = np.exp(x - np.max(x, axis=0, keepdims=True))
    return e / np.sum(e, axis=0, keepdims=True)


def apply_softmax_grad(p, labels):
    """p - onehot(int(label)) (cudamat_kernels.cu:819-825)."""
    out = _a(p).copy()
    lab = np.asarray(labels).ravel().astype(int)
    for j, l in enumerate(lab):
        if 0 <= l < out.shape[0]:
            out[l, j] -= 1.0
    return out


def get_softmax_cross_entropy(p, labels, tiny):
    """-log(p[label] + tiny), the sum in float32 (cudamat_kernels.cu:827-833)."""
    p32 = np.asarray(p, np.float32)
    lab = np.asarray(labels).ravel().astype(int)
    v = p32[lab, np.arange(p32.shape[1])] + np.float32(tiny)
    return -np.log(v.astype(F64)).reshape(1, -1)


def get_softmax_correct(p, labels):
    am = argmax_by_axis(p, 0).ravel().astype(int)
    return (am == np.asarray(labels).ravel().astype(int)).astype(F64).reshape(1, -1)


def vdot(a, b): return float(np.dot(_a(a).ravel(), _a(b).ravel()))
def euclid_norm(a): return float(np.sqrt(np.sum(_a(a) ** 2)))


# ---- gather / scatter: cudamat_kernels.cu:720-817, 1090-1121 ----------------

def select_columns(src, indices):
    src = _a(src)
    idx = np.asarray(indices).ravel().astype(int)
    out = np.empty((src.shape[0], idx.size), dtype=F64)
    for c, i in enumerate(idx):
        if i < 0:
            i += src.shape[1]
        out[:, c] = src[:, i] if 0 <= i < src.shape[1] else np.nan
    return out


def set_selected_columns(tgt, src, indices):
    out = _a(tgt).copy()
    idx = np.asarray(indices).ravel().astype(int)
    for c, i in enumerate(idx):
        if i < 0:
            i += out.shape[1]
        if 0 <= i < out.shape[1]:
            out[:, i] = _a(src)[:, c]
    return out


def blockify(src, blocksize):
    src = _a(src)
    rows = (np.arange(src.shape[0]) // blocksize) * blocksize
    return src[rows, :]


def expand(src, indices):
    src = _a(src)
    idx = np.asarray(indices).ravel().astype(int)
    out = np.full((src.shape[0], idx.size), np.nan)
    ok = (idx >= 0) & (idx < src.shape[1])
    out[:, ok] = src[:, idx[ok]]
    return out


def expand_and_add(src, mat, indices, mult):
    src, mat = _a(src), _a(mat)
    idx = np.asarray(indices).ravel().astype(int)
    out = np.full(src.shape, np.nan)
    ok = (idx >= 0) & (idx < mat.shape[1])
    out[:, ok] = src[:, ok] + F64(np.float32(mult)) * mat[:, idx[ok]]
    return out


def accumulate_columns(mat, indices, target_width, mult, avg):
    mat = _a(mat)
    idx = np.asarray(indices).ravel().astype(int)
    out = np.zeros((mat.shape[0], target_width))
    for c in range(target_width):
        sel = idx == c
        s = mat[:, sel].sum(axis=1)
        cnt = int(sel.sum())
        out[:, c] = F64(np.float32(mult)) * s / (cnt if (avg and cnt > 0) else 1)
    return out


def generate_translations(src, source_w, target_w, off_x, off_y, num_channels):
    """cudamat_kernels.cu:795-817: column = image, pixels row-major with channels interleaved;
    target pixel (tx, ty) of image b comes from the flat pixel index
    b*S*S + (pad + off_x + tx)*S + (pad + off_y + ty) of the whole source matrix, so a window
    leaving the image continues in the next pixel row / the next image.  An index outside the
    matrix (the reference reads foreign memory there) gives 0."""
    src = _a(src)
    n = src.shape[1]
    flat = src.ravel(order='F')
    pad = (source_w - target_w) // 2
    tx, ty = np.meshgrid(np.arange(target_w), np.arange(target_w), indexing='ij')
    out = np.zeros((target_w * target_w * num_channels, n))
    for b in range(n):
        ox, oy = int(np.asarray(off_x).ravel()[b]), int(np.asarray(off_y).ravel()[b])
        pix = b * source_w * source_w + (pad + ox + tx) * source_w + (pad + oy + ty)          # (target_w, target_w)
        idx = (num_channels * pix[..., None] + np.arange(num_channels)).ravel()
        ok = (idx >= 0) & (idx < flat.size)
        out[:, b] = np.where(ok, flat[np.clip(idx, 0, flat.size - 1)], 0.0)
    return out


# ---- ulp helper used by the parity tests --------------------------------------

def ulp_diff(got32, want64):
    """|got - float32(want)| in units of float32 ulps of the float64 value (0 where
    both are the same inf / both NaN)."""
    got = np.asarray(got32, dtype=np.float32)
    want = np.asarray(want64, dtype=F64)
    want32 = want.astype(np.float32)
    same_special = (np.isnan(got) & np.isnan(want32)) | (np.isinf(got) & (got == want32))
    with np.errstate(all='ignore'):
        spacing = np.spacing(np.abs(want32).astype(np.float32)).astype(F64)
        spacing = np.where(np.isfinite(spacing) & (spacing > 0), spacing, np.finfo(np.float32).tiny)
        d = np.abs(got.astype(F64) - want) / spacing
    d = np.where(same_special, 0.0, d)
    d = np.where(np.isnan(d), np.inf, d)
    return d
