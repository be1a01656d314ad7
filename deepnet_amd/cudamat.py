"""Python 3 matrix API over the MI355X backend: the ``CUDAMatrix`` surface of the
reference's cudamat/cudamat.py (class ``CUDAMatrix`` :146, module functions
:1533-1858, lifetime :1860-1897), bound through ctypes to ``libcudamat.so`` built
from ``csrc/``.

Method names, argument order, defaults (which ops write in place and which
allocate), return values and the error-code -> ``CUDAMatException`` mapping follow
the reference; the bodies are generated from small tables instead of being
spelled out one by one.  Matrices are fp32, column-major on the device and
Fortran-ordered on the host.

The library is required: importing this module without a built
``libcudamat.so`` raises ``ImportError`` (there is no CPU fallback).
"""
import ctypes as ct
import os
import warnings

import numpy as np

MAX_ONES = 1024 * 256

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, 'libcudamat.so')
MULTIPLIERS_PATH = os.path.join(_HERE, 'rnd_multipliers_32bit.txt')


def _load_library():
    if not os.path.exists(_LIB_PATH):
        raise ImportError(
            "%s is missing: build it with `make -C %s` (or __graft_entry__.build()); "
            "this backend has no CPU fallback." % (_LIB_PATH, os.path.join(_HERE, 'csrc')))
    return ct.CDLL(_LIB_PATH)


_cudamat = _load_library()


class cudamat(ct.Structure):
    """Mirror of struct cudamat (cudamat/cudamat.cuh:21-29)."""
    _fields_ = [('data_host', ct.POINTER(ct.c_float)),
                ('data_device', ct.POINTER(ct.c_float)),
                ('on_device', ct.c_int),
                ('on_host', ct.c_int),
                ('size', ct.c_int * 2),
                ('is_trans', ct.c_int),
                ('owns_data', ct.c_int)]


class rnd_struct(ct.Structure):
    """Mirror of struct rnd_struct (cudamat/cudamat.cuh:31-34)."""
    _fields_ = [('dev_rnd_mults', ct.POINTER(ct.c_uint)),
                ('dev_rnd_words', ct.POINTER(ct.c_longlong))]


class sparse_data(ct.Structure):
    """Mirror of struct sparse_data (cudamat/cudamat.cuh:36-39)."""
    _fields_ = [('indices', ct.POINTER(ct.c_int)),
                ('indptr', ct.POINTER(ct.c_int)),
                ('data', ct.POINTER(ct.c_float))]


class cudamat_sparse(ct.Structure):
    """Mirror of struct cudamat_sparse (cudamat/cudamat.cuh:41-50)."""
    _fields_ = [('data_host', sparse_data),
                ('data_device', sparse_data),
                ('on_device', ct.c_int),
                ('on_host', ct.c_int),
                ('size', ct.c_int * 2),
                ('is_trans', ct.c_int),
                ('owns_data', ct.c_int),
                ('nnz', ct.c_int)]


# Handles are declared as void*: ctypes converts a pointer object (CUDAMatrix.p_mat) to a
# void* argument markedly faster than it type-checks a POINTER(cudamat) one, and the steps
# of small models are bound by exactly this per-call host cost.
_M = ct.c_void_p
_S = ct.c_void_p
_R = ct.c_void_p
_f, _i, _u = ct.c_float, ct.c_int, ct.c_uint

# name -> (restype, argtypes): the prototypes of include/cudamat_amd.h.
_SIGNATURES = {
    'get_last_cuda_error': (ct.c_char_p, []),
    'cublas_init': (_i, []), 'cublas_shutdown': (_i, []),
    'cuda_set_device': (_i, [_i]), 'cuda_sync_threads': (None, []),
    'get_leading_dimension': (_i, [_M]), 'get_nonleading_dimension': (_i, [_M]),
    'set_transpose': (None, [_M, _i]),
    'set_shape': (_i, [_M, _u, _u]), 'reshape': (_i, [_M, _u, _u]),
    'get_slice': (_i, [_M, _M, _u, _u]), 'get_vector_slice': (_i, [_M, _M, _u, _u]),
    'init_from_array': (None, [_M, ct.POINTER(ct.c_float), _i, _i]),
    'set_on_device': (None, [_M]), 'init_empty': (_i, [_M, _i, _i]),
    'allocate_device_memory': (_i, [_M]),
    'copy_to_host': (_i, [_M]), 'copy_to_device': (_i, [_M]),
    'copy_on_device': (_i, [_M, _M]), 'free_device_memory': (_i, [_M]),
    'get_row_slice': (_i, [_M, _M, _u, _u]), 'set_row_slice': (_i, [_M, _M, _u, _u]),
    'copy_transpose': (_i, [_M, _M]),
    'init_random': (_i, [_R, _i, ct.c_char_p]),
    'fill_with_rand': (_i, [_R, _M]), 'fill_with_randn': (_i, [_R, _M]),
    'sample_bernoulli': (_i, [_R, _M, _M]), 'sample_bernoulli_tanh': (_i, [_R, _M, _M]),
    'sample_poisson': (_i, [_R, _M, _M]), 'sample_gaussian': (_i, [_R, _M, _M, _f]),
    'perturb_energy': (_i, [_R, _M, _M]), 'perturb_prob': (_i, [_R, _M, _M]),
    'dropout': (_i, [_R, _M, _f, _f]),
    'add_col_mult': (_i, [_M, _M, _M, _f]), 'add_row_mult': (_i, [_M, _M, _M, _f]),
    'mult_diagonal_scalar': (_i, [_M, _f, _M]), 'add_diagonal_scalar': (_i, [_M, _f, _M]),
    'graph_capture_begin': (ct.c_void_p, []), 'graph_capture_end': (ct.c_void_p, []),
    'graph_launch': (_i, [ct.c_void_p]), 'graph_free': (_i, [ct.c_void_p]), 'graph_set_stream': (_i, [ct.c_void_p, _i]),
    'max_by_axis': (_i, [_M, _M, _i]), 'max_by_axis_noalloc': (_i, [_M, _M, _i]), 'argmax_by_axis': (_i, [_M, _M, _i]),
    'choose_max_by_axis': (_i, [_M, _M, _i]), 'choose_max_and_accumulate': (_i, [_M, _M]),
    'sum_by_axis': (_i, [_M, _M, _i]), 'add_sum_by_axis': (_i, [_M, _M, _i, _f]),
    'sqsum_by_axis': (_i, [_M, _M, _i, _f, _f]), 'normlimit_by_axis': (_i, [_M, _M, _i, _f]),
    'apply_log': (_i, [_M, _M, _f]), 'apply_pow': (_i, [_M, _f, _M]),
    'compute_cross_entropy': (_i, [_M, _M, _M, _f]),
    'compute_cross_entropy_bernoulli': (_i, [_M, _M, _M, _f]),
    'correct_preds': (_i, [_M, _M, _M, _f]),
    'dot': (_i, [_M, _M, _M, _f, _f]),
    'dot_bias_act': (_i, [_M, _M, _M, _M, ct.c_int]),
    'cd_update': (_i, [_M, _M, _M, _M, _M, _M, _M, _f]), 'set_deferred_epilogues': (_i, [_i]), 'launch_deferred': (_i, []),
    'dot_bias_act_sample': (_i, [ct.c_void_p, _M, _M, _M, _M, _M, ct.c_int]),
    'momentum_update': (_i, [_M, _M, _M, _f, _f, _f, _f, ct.c_int]),
    'momentum_update_many': (_i, [ct.c_int, ct.c_void_p, ct.c_void_p, ct.c_void_p, ct.c_void_p, ct.c_void_p, ct.c_void_p,
                                  ct.c_void_p, ct.c_void_p]),
    'softmax_ce_grad': (_i, [_M, _M, _M, _M, _M, _f]),
    'init_from_sparse_array': (None, [_S, ct.POINTER(ct.c_float), ct.POINTER(ct.c_int), ct.POINTER(ct.c_int),
                                      _i, _i, _i]),
    'allocate_device_memory_sparse': (_i, [_S]), 'copy_sparse_to_device': (_i, [_S]),
    'free_device_memory_sparse': (_i, [_S]),
    'sparse_dot': (_i, [_S, _M, _M, _f, _f]),
    'vdot': (_f, [_M, _M, ct.POINTER(_i)]), 'euclid_norm': (_f, [_M, ct.POINTER(_i)]), 'sum_all': (_f, [_M, ct.POINTER(_i)]),
    'add_mult': (_i, [_M, _M, _f]), 'add_mult_sign': (_i, [_M, _M, _f]),
    'assign_scalar': (_i, [_M, _f]),
    'selectRows': (_i, [_M, _M, _M]), 'setSelectedRows': (_i, [_M, _M, _M]),
    'swapColumns': (_i, [_M, _M, _M, _M]),
    'generate_translations_big_var_off': (_i, [_M, _M, _M, _M, _i, _i, _i]),
    'blockify': (_i, [_M, _M, _i]),
    'accumulate_columns': (_i, [_M, _M, _M, _f, _i]),
    'expand': (_i, [_M, _M, _M]), 'expand_and_add': (_i, [_M, _M, _M, _M, _f]),
    'softmax': (_i, [_M, _M]), 'softmax_overwrite': (_i, [_M]),
    'apply_softmax_grad': (_i, [_M, _M, _M]), 'get_softmax_correct': (_i, [_M, _M, _M]),
    'get_softmax_cross_entropy': (_i, [_M, _M, _M, _f]),
}
# families that share one prototype
for _n in ('add_col_vec', 'add_row_vec', 'mult_by_col_vec', 'mult_by_row_vec', 'div_by_col_vec',
           'div_by_row_vec', 'mult_diagonal', 'add_diagonal', 'less_than_eq', 'less_than',
           'greater_than_eq', 'greater_than', 'upper_bound', 'lower_bound', 'apply_pow_matrix',
           'add_elementwise', 'subtract_elementwise', 'divide_elementwise', 'mult_elementwise',
           'apply_sin_deriv', 'apply_cos_deriv', 'apply_logistic_deriv', 'apply_tanh_deriv',
           'apply_rectified_linear_deriv', 'apply_rectified_linear_smooth_deriv'):
    _SIGNATURES[_n] = (_i, [_M, _M, _M])
for _n in ('less_than_eq_scalar', 'less_than_scalar', 'greater_than_eq_scalar', 'greater_than_scalar',
           'upper_bound_scalar', 'lower_bound_scalar', 'mult_by_scalar', 'divide_by_scalar', 'add_scalar'):
    _SIGNATURES[_n] = (_i, [_M, _f, _M])
for _n in ('sign', 'apply_cos', 'apply_sin', 'apply_sigmoid', 'apply_tanh', 'apply_abs',
           'apply_log_1_plus_exp', 'apply_exp', 'apply_ceil', 'apply_floor', 'apply_sqrt', 'reciprocal'):
    _SIGNATURES[_n] = (_i, [_M, _M])

for _n, (_res, _args) in _SIGNATURES.items():
    _fn = getattr(_cudamat, _n)  # AttributeError here = the library does not export the ABI
    _fn.restype = _res
    _fn.argtypes = _args


def deprecated(func):
    """Decorator that emits a DeprecationWarning when func is called."""
    def newFunc(*args, **kwargs):
        warnings.warn("Call to deprecated function %s." % func.__name__, category=DeprecationWarning)
        return func(*args, **kwargs)
    newFunc.__name__ = func.__name__
    newFunc.__doc__ = func.__doc__
    newFunc.__dict__.update(func.__dict__)
    return newFunc


class CUDAMatException(Exception):
    pass


def get_last_cuda_error():
    return _cudamat.get_last_cuda_error().decode()


_ERROR_TEXT = {
    -1: "Incompatible matrix dimensions.",
    -2: "CUBLAS error.",
    -4: "Operation not supported on views.",
    -5: "Operation not supported on transposed matrices.",
    -6: "",
    -7: "Incompatible transposedness.",
    -8: "Matrix is not in device memory.",
    -9: "Operation not supported.",
}


def generate_exception(err_code):
    """Return a CUDAMatException for err_code (cudamat.py:101-123)."""
    if err_code == -3:
        return CUDAMatException("CUDA error: " + get_last_cuda_error())
    return CUDAMatException(_ERROR_TEXT.get(err_code, "Unknown error %d." % err_code))


def _check(err_code):
    if err_code:
        raise generate_exception(err_code)


def _is_scalar(val):
    return isinstance(val, (int, float, np.integer, np.floating))


class TransposedCUDAMatrix(object):
    """A struct copy with is_trans set, sharing the device pointer (cudamat.py:139-144)."""

    def __init__(self, mat):
        self.mat = cudamat()
        ct.memmove(ct.pointer(self.mat), ct.pointer(mat), ct.sizeof(self.mat))
        self.mat.is_trans = 1
        self.p_mat = ct.pointer(self.mat)


class CUDAMatrix(object):
    """A matrix of single precision floating point numbers on the GPU."""

    rndInitialized = 0
    rnd_state = None
    rnd_state_p = None
    ones = None

    def __init__(self, array, copy_to_device=True):
        """From a numpy ndarray (converted to float32, Fortran order, and copied to the
        device unless copy_to_device is False), or from an existing cudamat struct."""
        if isinstance(array, np.ndarray):
            array = reformat(array)
            self.mat = cudamat()
            self.size = self.mat.size
            self.p_mat = ct.pointer(self.mat)
            self.numpy_array = array
            _cudamat.init_from_array(self.p_mat, array.ctypes.data_as(ct.POINTER(ct.c_float)),
                                     array.shape[0], array.shape[1])
            if copy_to_device:
                _check(_cudamat.copy_to_device(self.p_mat))
        else:
            self.mat = array
            self.p_mat = ct.pointer(self.mat)
        self.T = TransposedCUDAMatrix(self.mat)

    def overwrite(self, array, copy_to_device=True):
        """Re-point self at a new host array (no larger than the original)."""
        assert isinstance(array, np.ndarray), 'array must be a np.ndarray.'
        array = reformat(array)
        self.numpy_array = array
        _cudamat.init_from_array(self.p_mat, array.ctypes.data_as(ct.POINTER(ct.c_float)),
                                 array.shape[0], array.shape[1])
        _cudamat.set_on_device(self.p_mat)
        if copy_to_device:
            _check(_cudamat.copy_to_device(self.p_mat))

    @staticmethod
    def init_random(seed=0):
        """Initialize and seed the 12288-stream random number generator."""
        CUDAMatrix.rndInitialized = 1
        CUDAMatrix.rnd_state = rnd_struct()
        CUDAMatrix.rnd_state_p = ct.pointer(CUDAMatrix.rnd_state)
        _check(_cudamat.init_random(CUDAMatrix.rnd_state_p, int(seed), MULTIPLIERS_PATH.encode()))

    @property
    def shape(self):
        return (self.mat.size[0], self.mat.size[1])

    def set_shape(self, shape):
        """Set the shape without any checking."""
        _check(_cudamat.set_shape(self.p_mat, int(shape[0]), int(shape[1])))
        return self

    def reshape(self, shape):
        """Reinterpret the contents with a new shape of the same element count; one
        entry may be -1."""
        m, n = shape
        mlen = self.shape[0] * self.shape[1]
        if m == -1:
            assert n > 0 and mlen % n == 0
            m = mlen // n
        elif n == -1:
            assert m > 0 and mlen % m == 0
            n = mlen // m
        _check(_cudamat.reshape(self.p_mat, int(m), int(n)))
        return self

    def blockify(source, blocksize, target=None):
        if target is None:
            target = source
        _check(_cudamat.blockify(source.p_mat, target.p_mat, int(blocksize)))
        return target

    def generate_translations(source, source_w, target_w, off_x, off_y, target=None):
        num_channels = source.shape[0] // (source_w ** 2)
        if target is None:
            target = empty((target_w ** 2 * num_channels, source.shape[1]))
        _check(_cudamat.generate_translations_big_var_off(
            source.p_mat, target.p_mat, off_x.p_mat, off_y.p_mat, int(source_w), int(target_w), int(num_channels)))
        return target

    def asarray(self):
        """Copy the matrix to an ndarray on the CPU and return it."""
        self.copy_to_host()
        return self.numpy_array

    def copy_to_device(self):
        _check(_cudamat.copy_to_device(self.p_mat))

    def copy_to_host(self):
        if not self.mat.on_host:
            m, n = self.mat.size[0], self.mat.size[1]
            self.numpy_array = np.empty((m, n), dtype=np.float32, order='F')
            self.mat.data_host = self.numpy_array.ctypes.data_as(ct.POINTER(ct.c_float))
            self.mat.on_host = 1
        _check(_cudamat.copy_to_host(self.p_mat))

    def assign(self, val):
        """Assign a scalar or a CUDAMatrix of the same dimensions to self."""
        if isinstance(val, CUDAMatrix):
            _check(_cudamat.copy_on_device(val.p_mat, self.p_mat))
        elif _is_scalar(val):
            _check(_cudamat.assign_scalar(self.p_mat, float(val)))
        else:
            raise ValueError("Assigned value must be of type CUDAMatrix, int, or float.")
        return self

    def free_device_memory(self):
        _check(_cudamat.free_device_memory(self.p_mat))

    def set_trans(self, is_trans):
        _cudamat.set_transpose(self.p_mat, 1 * is_trans)

    def slice(self, first_col, last_col):
        """A view of columns [first_col, last_col) (elements, for a vector)."""
        mat = cudamat()
        if self.mat.size[0] == 1 or self.mat.size[1] == 1:
            err = _cudamat.get_vector_slice(self.p_mat, ct.pointer(mat), int(first_col), int(last_col))
        else:
            err = _cudamat.get_slice(self.p_mat, ct.pointer(mat), int(first_col), int(last_col))
        _check(err)
        new_mat = CUDAMatrix(mat)
        new_mat.sliceof = getattr(self, 'sliceof', self)
        return new_mat

    def get_col_slice(self, first_col, last_col, target=None):
        col_slice = self.slice(first_col, last_col)
        if target is not None:
            target.assign(col_slice)
            return target
        return col_slice

    def set_col_slice(self, first_col, last_col, mat):
        self.slice(first_col, last_col).assign(mat)
        return self

    def get_row_slice(self, start, end, target=None):
        if target is None:
            target = empty((end - start, self.shape[1]))
        _check(_cudamat.get_row_slice(self.p_mat, target.p_mat, int(start), int(end)))
        return target

    def set_row_slice(self, start, end, mat):
        _check(_cudamat.set_row_slice(mat.p_mat, self.p_mat, int(start), int(end)))
        return self

    def transpose(self, target=None):
        """Return a transposed copy of the matrix."""
        if target is None:
            target = empty((self.shape[1], self.shape[0]))
        _check(_cudamat.copy_transpose(self.p_mat, target.p_mat))
        return target

    # ---- random numbers -------------------------------------------------
    def fill_with_rand(self):
        _check(_cudamat.fill_with_rand(CUDAMatrix.rnd_state_p, self.p_mat))
        return self

    def fill_with_randn(self):
        _check(_cudamat.fill_with_randn(CUDAMatrix.rnd_state_p, self.p_mat))
        return self

    def dropout(self, dropprob, val=0.0):
        """Set entries to val with probability dropprob."""
        _check(_cudamat.dropout(CUDAMatrix.rnd_state_p, self.p_mat, float(dropprob), float(val)))
        return self

    def sample_gaussian(self, mult=1.0, target=None):
        if target is None:
            target = self
        _check(_cudamat.sample_gaussian(CUDAMatrix.rnd_state_p, self.p_mat, target.p_mat, float(mult)))
        return self

    # ---- sums ---------------------------------------------------------
    def sum(self, axis=None, target=None):
        """Sum along axis (0 = leading dimension, 1 = non-leading); None sums everything
        and returns a Python float."""
        if axis is None:
            # (the reference takes vdot() with a vector of ones, cudamat.py:719-720; sum_all is that
            # kernel without the reads of the vector and leaves the same bits)
            err_code = ct.c_int(0)
            res = _cudamat.sum_all(self.p_mat, ct.byref(err_code))
            _check(err_code.value)
            return res
        return sum(self, axis, target)

    def add_sums(self, mat, axis, mult=1.):
        """self += mult * (sums of mat along axis)."""
        if axis not in (0, 1):
            raise ValueError("axis must be 0 or 1.")
        # (the reference multiplies by a vector of ones, cudamat.py:724-748; add_sum_by_axis runs
        # the same kernels without reading the vector and leaves the same bits)
        _check(_cudamat.add_sum_by_axis(mat.p_mat, self.p_mat, int(axis), float(mult)))
        return self

    def cumsum(self, axis, temp=None, target=None):
        """Not provided by the device library (the reference declares the kernel but
        never defines it: cudamat_kernels.cuh:70, cudamat.py:874)."""
        raise CUDAMatException("Operation not supported.")

    def choose_max_and_accumulate(self, acc):
        _check(_cudamat.choose_max_and_accumulate(self.p_mat, acc.p_mat))
        return acc

    def choose_max(self, axis, target=None):
        """Set the argmax along axis to 1 and the rest to 0."""
        if target is None:
            target = self
        _check(_cudamat.choose_max_by_axis(self.p_mat, target.p_mat, int(axis)))
        return target

    def _axis_target(self, axis, target):
        m, n = self.shape
        if target is None:
            target = empty((1, n)) if axis == 0 else empty((m, 1))
        return target

    def max(self, axis, target=None):
        target = self._axis_target(axis, target)
        _check(_cudamat.max_by_axis(self.p_mat, target.p_mat, int(axis)))
        return target

    def max_noalloc(self, axis, target):
        """max(axis) into an existing target through the entry point that allocates no
        device memory (an extension of this backend; the target is not optional)."""
        _check(_cudamat.max_by_axis_noalloc(self.p_mat, target.p_mat, int(axis)))
        return target

    def argmax(self, axis, target=None):
        target = self._axis_target(axis, target)
        _check(_cudamat.argmax_by_axis(self.p_mat, target.p_mat, int(axis)))
        return target

    def add_sqsums(self, mat, axis, mult=1.):
        """self += mult * (sums of squares of mat along axis)."""
        m, n = mat.shape
        if axis == 0:
            assert self.shape == (1, n), 'Self has shape %s but mat has shape %s' % (self.shape, mat.shape)
        elif axis == 1:
            assert self.shape == (m, 1)
        _check(_cudamat.sqsum_by_axis(mat.p_mat, self.p_mat, int(axis), float(mult), 1.0))

    def sqsum(self, axis, target=None):
        target = self._axis_target(axis, target)
        _check(_cudamat.sqsum_by_axis(self.p_mat, target.p_mat, int(axis), 1.0, 0.0))
        return target

    def norm_limit(self, norm, axis, target=None):
        """Scale every column (axis 0) or row (axis 1) whose norm exceeds `norm` down to it."""
        if target is None:
            target = self
        _check(_cudamat.normlimit_by_axis(self.p_mat, target.p_mat, int(axis), float(norm)))
        return target

    def apply_softmax(self, target=None):
        return softmax(self, target)

    def sign(self, target=None):
        if target is None:
            target = empty((self.mat.size[0], self.mat.size[1]))
        _check(_cudamat.sign(self.p_mat, target.p_mat))
        return target

    def apply_cos(self, target=None):
        return cos(self, target)

    def apply_sin(self, target=None):
        return sin(self, target)

    def apply_sigmoid(self, target=None):
        return sigmoid(self, target)

    # ---- contraction -------------------------------------------------
    def dot(self, mat2, mult=1.0, target=None):
        return dot(self, mat2, mult, target)

    def add_dot(self, m1, m2, mult=1.0):
        """self += mult * m1 . m2"""
        _check(_cudamat.dot(m1.p_mat, m2.p_mat, self.p_mat, 1., float(mult)))
        return self

    def subtract_dot(self, m1, m2):
        _check(_cudamat.dot(m1.p_mat, m2.p_mat, self.p_mat, 1., -1.))
        return self

    def add_mult_sign(self, mat2, mult=1.):
        _check(_cudamat.add_mult_sign(self.p_mat, mat2.p_mat, float(mult)))
        return self

    def add_mult(self, mat2, mult=1.):
        """self += mult * mat2"""
        _check(_cudamat.add_mult(self.p_mat, mat2.p_mat, float(mult)))
        return self

    def subtract_mult(self, mat2, mult=1.):
        _check(_cudamat.add_mult(self.p_mat, mat2.p_mat, float(-1. * mult)))
        return self

    def subtract(self, val, target=None):
        """Subtract a scalar or a CUDAMatrix of the same dimensions."""
        if target is None:
            target = self
        if isinstance(val, CUDAMatrix):
            _check(_cudamat.subtract_elementwise(self.p_mat, val.p_mat, target.p_mat))
        elif _is_scalar(val):
            _check(_cudamat.add_scalar(self.p_mat, float(-1 * val), target.p_mat))
        else:
            raise ValueError("Value must be of type CUDAMatrix, int, or float.")
        return target

    # ---- gather / scatter -------------------------------------------
    def accumulate_columns(self, indices, target, mult=1.0, avg=False):
        if target is None:
            target = self
        _check(_cudamat.accumulate_columns(self.p_mat, indices.p_mat, target.p_mat, float(mult), 1 if avg else 0))
        return target

    def expand(self, expansion_indices, target):
        _check(_cudamat.expand(self.p_mat, expansion_indices.p_mat, target.p_mat))
        return target

    def expand_and_add(self, val, expansion_indices, target=None, mult=1.0):
        if target is None:
            target = self
        if isinstance(val, CUDAMatrix) and isinstance(expansion_indices, CUDAMatrix):
            _check(_cudamat.expand_and_add(self.p_mat, val.p_mat, expansion_indices.p_mat, target.p_mat, float(mult)))
        else:
            raise ValueError("Value must be of type CUDAMatrix, int, or float.")
        return target

    def select_columns(self, indices, target):
        """target[:, c] = self[:, indices[c]]; indices are float-encoded integers, negative
        ones count from the end, out-of-range ones give NaN columns."""
        _check(_cudamat.selectRows(self.p_mat, target.p_mat, indices.p_mat))
        return target

    def swap_columns(self, indices1, indices2, target):
        """Swap self[:, indices1[c]] with target[:, indices2[c]]."""
        assert indices1.shape == indices2.shape
        _check(_cudamat.swapColumns(self.p_mat, target.p_mat, indices1.p_mat, indices2.p_mat))
        return target

    def set_selected_columns(self, indices, source):
        """self[:, indices[c]] = source[:, c]"""
        _check(_cudamat.setSelectedRows(self.p_mat, source.p_mat, indices.p_mat))
        return self

    # ---- softmax losses ----------------------------------------------
    def get_softmax_correct(self, labels, target):
        """target[i] = 1 iff the argmax of column i equals labels[i]."""
        assert labels.shape == (1, self.shape[1])
        assert target.shape == labels.shape
        if not isinstance(labels, CUDAMatrix):
            raise ValueError("labels must be of type CUDAMatrix.")
        _check(_cudamat.get_softmax_correct(self.p_mat, labels.p_mat, target.p_mat))
        return target

    def get_softmax_cross_entropy(self, labels, target, tiny=1e-10):
        """target[i] = -log(self[labels[i], i] + tiny)."""
        assert labels.shape == (1, self.shape[1])
        assert target.shape == labels.shape
        if not isinstance(labels, CUDAMatrix):
            raise ValueError("labels must be of type CUDAMatrix.")
        _check(_cudamat.get_softmax_cross_entropy(self.p_mat, labels.p_mat, target.p_mat, float(tiny)))
        return target

    def apply_softmax_grad(self, labels, target=None):
        """target = self - onehot(labels)."""
        if target is None:
            target = self
        assert labels.shape == (1, self.shape[1])
        assert target.shape == self.shape
        if not isinstance(labels, CUDAMatrix):
            raise ValueError("labels must be of type CUDAMatrix.")
        _check(_cudamat.apply_softmax_grad(self.p_mat, labels.p_mat, target.p_mat))
        return target

    def euclid_norm(self):
        err_code = ct.c_int(0)
        res = _cudamat.euclid_norm(self.p_mat, ct.byref(err_code))
        _check(err_code.value)
        return res


# ---- generated methods ------------------------------------------------------

def _method_vec(cname, doc, with_mult=False):
    """(self, vec[, mult], target=None) -> target; default target is self."""
    fn = getattr(_cudamat, cname)
    if with_mult:
        def method(self, vec, mult, target=None):
            if target is None:
                target = self
            _check(fn(self.p_mat, vec.p_mat, target.p_mat, float(mult)))
            return target
    else:
        def method(self, vec, target=None):
            if target is None:
                target = self
            _check(fn(self.p_mat, vec.p_mat, target.p_mat))
            return target
    method.__doc__ = doc
    return method


def _method_mat_or_scalar(mat_cname, scalar_cname, doc, what="Value"):
    """(self, val, target=None): val a CUDAMatrix (mat_cname) or a number (scalar_cname)."""
    mat_fn = getattr(_cudamat, mat_cname)
    scalar_fn = getattr(_cudamat, scalar_cname) if scalar_cname else None

    def method(self, val, target=None):
        if target is None:
            target = self
        if isinstance(val, CUDAMatrix):
            _check(mat_fn(self.p_mat, val.p_mat, target.p_mat))
        elif scalar_fn is not None and _is_scalar(val):
            _check(scalar_fn(self.p_mat, float(val), target.p_mat))
        elif scalar_fn is not None:
            raise ValueError("%s must be of type CUDAMatrix, int, or float." % what)
        else:
            raise ValueError("%s must be of type CUDAMatrix." % what)
        return target
    method.__doc__ = doc
    return method


def _method_sampler(cname, doc):
    """(self, target=None) -> self; draws from the global RNG state."""
    fn = getattr(_cudamat, cname)

    def method(self, target=None):
        if target is None:
            target = self
        _check(fn(CUDAMatrix.rnd_state_p, self.p_mat, target.p_mat))
        return self
    method.__doc__ = doc
    return method


def _method_scalar_deprecated(cname, doc):
    fn = getattr(_cudamat, cname)

    def method(self, alpha, target=None):
        if target is None:
            target = self
        _check(fn(self.p_mat, float(alpha), target.p_mat))
        return target
    method.__doc__ = doc
    return method


for _py, _c, _doc, _mult in (
        ('add_col_vec', 'add_col_vec', "Add vector vec to every column of the matrix.", False),
        ('add_col_mult', 'add_col_mult', "Add mult * vec to every column of the matrix.", True),
        ('add_row_vec', 'add_row_vec', "Add vector vec to every row of the matrix.", False),
        ('add_row_mult', 'add_row_mult', "Add mult * vec to every row of the matrix.", True),
        ('mult_by_col', 'mult_by_col_vec', "Multiply vector vec into every column of the matrix.", False),
        ('mult_by_row', 'mult_by_row_vec', "Multiply vector vec into every row of the matrix.", False),
        ('div_by_col', 'div_by_col_vec', "Divide every column of the matrix by vector vec.", False),
        ('div_by_row', 'div_by_row_vec', "Divide every row of the matrix by vector vec.", False)):
    setattr(CUDAMatrix, _py, _method_vec(_c, _doc, _mult))

for _py, _cm, _cs, _doc in (
        ('less_than_eq', 'less_than_eq', 'less_than_eq_scalar', "target = 1. * (self <= val)"),
        ('less_than', 'less_than', 'less_than_scalar', "target = 1. * (self < val)"),
        ('greater_than_eq', 'greater_than_eq', 'greater_than_eq_scalar', "target = 1. * (self >= val)"),
        ('greater_than', 'greater_than', 'greater_than_scalar', "target = 1. * (self > val)"),
        ('upper_bound', 'upper_bound', 'upper_bound_scalar', "target = (self > val) ? val : self"),
        ('lower_bound', 'lower_bound', 'lower_bound_scalar', "target = (self < val) ? val : self"),
        ('add', 'add_elementwise', 'add_scalar', "target = self + val"),
        ('divide', 'divide_elementwise', 'divide_by_scalar', "target = self / val"),
        ('mult', 'mult_elementwise', 'mult_by_scalar', "target = self * val"),
        ('apply_cos_deriv', 'apply_cos_deriv', None, "target = -self * sin(val)"),
        ('apply_sin_deriv', 'apply_sin_deriv', None, "target = self * cos(val)"),
        ('apply_logistic_deriv', 'apply_logistic_deriv', None, "target = self * val * (1 - val)"),
        ('apply_tanh_deriv', 'apply_tanh_deriv', None, "target = self * (1 + val) * (1 - val) * 0.5"),
        ('apply_rectified_linear_deriv', 'apply_rectified_linear_deriv', None, "target = self * (val > 0)"),
        ('apply_rectified_linear_smooth_deriv', 'apply_rectified_linear_smooth_deriv', None,
         "target = self * (1 - exp(-val))")):
    setattr(CUDAMatrix, _py, _method_mat_or_scalar(_cm, _cs, _doc))


def _method_diag(mat_cname, scalar_cname, doc):
    inner = _method_mat_or_scalar(mat_cname, scalar_cname, doc)

    def method(self, val, target=None):
        assert self.shape[0] == self.shape[1], 'self must be a square matrix'
        return inner(self, val, target)
    method.__doc__ = doc
    return method


CUDAMatrix.mult_diagonal = _method_diag('mult_diagonal', 'mult_diagonal_scalar', "Multiply the diagonal by val.")
CUDAMatrix.add_diagonal = _method_diag('add_diagonal', 'add_diagonal_scalar', "Add val to the diagonal.")

for _py, _c, _doc in (
        ('sample_bernoulli', 'sample_bernoulli', "target = 1 with probability self, else 0."),
        ('sample_bernoulli_tanh', 'sample_bernoulli_tanh', "target = 1 with probability (1+self)/2, else 0."),
        ('sample_poisson', 'sample_poisson', "Placeholder of the reference: consumes draws, copies self."),
        ('perturb_energy_for_softmax_sampling', 'perturb_energy', "target = self - log(-log(rand))."),
        ('perturb_prob_for_softmax_sampling', 'perturb_prob', "target = -self / log(rand).")):
    setattr(CUDAMatrix, _py, _method_sampler(_c, _doc))

CUDAMatrix.mult_by_scalar = deprecated(_method_scalar_deprecated('mult_by_scalar', "Multiply the matrix by a scalar."))
CUDAMatrix.div_by_scalar = deprecated(_method_scalar_deprecated('divide_by_scalar', "Divide the matrix by a scalar."))
CUDAMatrix.add_scalar = deprecated(_method_scalar_deprecated('add_scalar', "Increment the matrix by a scalar."))


def _assign_scalar(self, alpha):
    """Assign scalar alpha to every element of the matrix."""
    _check(_cudamat.assign_scalar(self.p_mat, float(alpha)))
    return self


CUDAMatrix.assign_scalar = deprecated(_assign_scalar)


def _reciprocal(self, target=None):
    """Find the reciprocal of each element of the matrix."""
    if target is None:
        target = self
    _check(_cudamat.reciprocal(self.p_mat, target.p_mat))
    return target


CUDAMatrix.reciprocal = _reciprocal


# ---- module-level functions (cudamat.py:1533-1858) -------------------------

def empty(shape):
    """Create a new CUDAMatrix with the given shape (uninitialised device memory)."""
    mat = cudamat()
    _check(_cudamat.init_empty(ct.pointer(mat), int(shape[0]), int(shape[1])))
    return CUDAMatrix(mat)


_ones_views = {}


_ones_retired = []


def _ones(n, trans=False):
    """View of the first n entries of the device vector of ones (grown on demand), as a
    column or, with trans, as a row.  Views are kept per (n, trans): the sums call this
    on every step with the same few sizes."""
    if not isinstance(CUDAMatrix.ones, CUDAMatrix):
        raise CUDAMatException("cublas_init() has not been called.")
    if n > CUDAMatrix.ones.shape[0]:
        # (a recorded graph may still sum with the old vector: it is kept, and the vector at
        # least doubles, so all the kept ones together are smaller than the current one)
        _ones_retired.append(CUDAMatrix.ones)
        CUDAMatrix.ones = CUDAMatrix(np.ones((max(n, 2 * CUDAMatrix.ones.shape[0]), 1), dtype=np.float32, order='F'))
        _ones_views.clear()
    key = (n, trans)
    view = _ones_views.get(key)
    if view is None or view._ones_parent is not CUDAMatrix.ones:
        view = CUDAMatrix.ones.slice(0, n)
        if trans:
            view.set_trans(True)
        view._ones_parent = CUDAMatrix.ones
        if len(_ones_views) > 256:
            _ones_views.clear()
        _ones_views[key] = view
    return view


def sum(mat, axis, target=None):
    """Sum along axis: 0 = leading dimension, 1 = non-leading, of the matrix as it is seen (a
    transposed operand is honoured).  The reference multiplies by a vector of ones
    (cudamat.py:1546-1577); sum_by_axis runs the same kernels without reading the vector and
    leaves the same bits."""
    m = _cudamat.get_leading_dimension(mat.p_mat)
    n = _cudamat.get_nonleading_dimension(mat.p_mat)
    if axis == 0:
        if target is None:
            target = empty((1, n))
    elif axis == 1:
        if target is None:
            target = empty((m, 1))
    else:
        raise ValueError("axis must be 0 or 1.")
    _check(_cudamat.sum_by_axis(mat.p_mat, target.p_mat, int(axis)))
    return target


def dot(m1, m2, mult=1.0, target=None):
    """target = mult * m1 . m2"""
    if target is None:
        m = _cudamat.get_leading_dimension(m1.p_mat)
        n = _cudamat.get_nonleading_dimension(m2.p_mat)
        target = empty((m, n))
    _check(_cudamat.dot(m1.p_mat, m2.p_mat, target.p_mat, 0., float(mult)))
    return target


_ACTS = {None: 0, 'none': 0, 'linear': 0, 'sigmoid': 1, 'logistic': 1, 'relu': 2, 'rectified_linear': 2, 'tanh': 3}


class Graph(object):
    """A recorded sequence of library calls (an extension of this backend: a HIP graph).

        step()                                  # once, eagerly: workspaces reach their sizes
        with cm.Graph() as g:
            step()                              # recorded, not run
        for _ in range(n):
            g.launch()                          # one launch replays the whole sequence

    The calls are recorded with the matrices and scalars they were given; the random generator's
    state lives on the device, so every replay draws fresh numbers.  Calls that wait for the
    device (asarray, copy_to_host, vdot, euclid_norm) and allocations (empty, CUDAMatrix(...))
    raise CUDAMatException while recording."""

    def __init__(self):
        self._exec = None

    def __enter__(self):
        stream = _cudamat.graph_capture_begin()
        if not stream:
            raise CUDAMatException("could not start recording a graph")
        # (the conv library links against this one and queues on the same stream)
        return self

    def __exit__(self, exc_type, exc, tb):
        handle = _cudamat.graph_capture_end()
        if exc_type is not None:
            if handle:                              # a recording that was given up is not kept
                _cudamat.graph_free(handle)
            return False
        if not handle:
            raise CUDAMatException("recording the graph failed")
        self._exec = handle
        return False

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass

    def launch(self):
        if not self._exec:
            raise CUDAMatException("no recorded graph to launch")
        _check(_cudamat.graph_launch(self._exec))

    def free(self):
        if self._exec:
            _cudamat.graph_free(self._exec)
            self._exec = None


def dot_bias_act(m1, m2, bias=None, target=None, act='sigmoid', sample=None):
    """Extension of this backend (not in the reference): target = act(m1 . m2 + bias) in
    one launch, bit-identical to
        cm.dot(m1, m2, target=target); target.add_col_vec(bias); target.apply_sigmoid()
    (act: None, 'sigmoid', 'relu' = lower_bound(0), 'tanh'; bias: rows x 1 or None).
    With `sample` (a matrix of target's shape) the same launch also does
        target.sample_bernoulli(target=sample)
    with the same draws and the same generator state afterwards."""
    if act not in _ACTS:
        raise ValueError("act must be one of %s" % sorted(k for k in _ACTS if k))
    if target is None:
        m = _cudamat.get_leading_dimension(m1.p_mat)
        n = _cudamat.get_nonleading_dimension(m2.p_mat)
        target = empty((m, n))
    b = bias.p_mat if bias is not None else None
    if sample is None:
        _check(_cudamat.dot_bias_act(m1.p_mat, m2.p_mat, b, target.p_mat, _ACTS[act]))
    else:
        _check(_cudamat.dot_bias_act_sample(CUDAMatrix.rnd_state_p, m1.p_mat, m2.p_mat, b, target.p_mat, sample.p_mat,
                                            _ACTS[act]))
    return target


def set_deferred_epilogues(on):
    """Extension of this backend: `dot` holds its launch back so that an `add_col_vec`, an activation
    (`apply_sigmoid`, `lower_bound(0)`, `apply_tanh`) and a `sample_bernoulli` that follow it on its
    own target run in the product's epilogue - one launch for the three or four calls of a layer's
    up-pass, same bits, same order of work; `apply_rectified_linear_deriv(state)` of the product's target
    directly behind it (a layer's backward pass) runs there too, and so does the dropout mask of a layer of
    rectified linear units (`mask.fill_with_rand(); mask.greater_than(p); state.mult(mask)`).  Likewise the calls of a parameter update
    (deepnet/parameter.py:80-106) run as one pass, two `add_dot` calls of the same shape into one
    target as one launch, and up to four `add_sums(.., axis=1)` calls onto two vectors as one launch
    (the statistics of cudamat/examples/rbm_cudamat.py:73-86); an `add_dot` that stays alone takes the
    `add_sums` calls that follow it along in its launch (the gradients of a layer, deepnet/edge.py:236-242,
    layer.py:206-211), and `apply_softmax` waits for the `get_softmax_cross_entropy` and `apply_softmax_grad`
    of its result (deepnet/softmax_layer.py:25-62).  On by default; returns the previous setting."""
    return bool(_cudamat.set_deferred_epilogues(1 if on else 0))


def launch_deferred():
    """Extension of this backend: queues the calls that are held back (see `set_deferred_epilogues`)
    and waits for nothing.  For a caller that records its own events on the NULL stream, or queues
    other work behind the library's, and must have every call made so far in the stream."""
    _check(_cudamat.launch_deferred())


def cd_update(W, bv, bh, v, h, v2, h2, eps):
    """Extension of this backend (not in the reference): the contrastive-divergence update
        W.add_dot(v, h.T, mult=eps); W.add_dot(v2, h2.T, mult=-eps)
        bv.add_sums(v, axis=1, mult=eps); bv.add_sums(v2, axis=1, mult=-eps)
        bh.add_sums(h, axis=1, mult=eps); bh.add_sums(h2, axis=1, mult=-eps)
    (cudamat/examples/rbm_cudamat.py:57-85) as one product over the concatenated reduction
    [v | v2] . [h | -h2]^T with a row of ones appended to each operand, one launch.  The sums are
    formed in one accumulation instead of two rounded updates, so the result equals the six calls
    to rounding (about 1e-7 relative), not bit for bit; for batches of up to 128 the library runs
    the two products and four sums of the six calls themselves in one launch, with their bits.
    bv / bh may be None."""
    _check(_cudamat.cd_update(W.p_mat, bv.p_mat if bv is not None else None, bh.p_mat if bh is not None else None,
                              v.p_mat, h.p_mat, v2.p_mat, h2.p_mat, float(eps)))
    return W


def softmax_ce_grad(mat, labels, probs=None, loss=None, grad=None, tiny=1e-10):
    """Extension of this backend (not in the reference): one launch for
        mat.apply_softmax(target=probs); probs.get_softmax_cross_entropy(labels, target=loss, tiny=tiny)
        probs.apply_softmax_grad(labels, target=grad)
    with the same bits; probs defaults to mat (in place), loss and grad are skipped when None."""
    if probs is None:
        probs = mat
    _check(_cudamat.softmax_ce_grad(mat.p_mat, labels.p_mat, probs.p_mat, loss.p_mat if loss is not None else None,
                                    grad.p_mat if grad is not None else None, ct.c_float(tiny)))
    return probs


def momentum_update(w, w_delta, gradient, momentum, epsilon, l2_decay=None, l1_decay=None, reset_gradient=True):
    """Extension of this backend (not in the reference): the update of
    deepnet/parameter.py:80-106 in one pass over the parameter, the same bits as
        w_delta.mult(momentum); w_delta.add_mult(w, l2_decay); w_delta.add_mult_sign(w, l1_decay)
        w_delta.add_mult(gradient); w.add_mult(w_delta, -epsilon); gradient.assign(0)
    (the l2 / l1 terms only when a decay is given, the last call only with reset_gradient)."""
    flags = (1 if l2_decay is not None else 0) | (2 if l1_decay is not None else 0) | (4 if reset_gradient else 0)
    _check(_cudamat.momentum_update(w.p_mat, w_delta.p_mat, gradient.p_mat, ct.c_float(momentum),
                                    ct.c_float(l2_decay or 0.0), ct.c_float(l1_decay or 0.0), ct.c_float(epsilon), flags))
    return w


class MomentumUpdates(object):
    """Extension of this backend: momentum_update for a fixed list of parameters in one launch
    per 8 of them.  updates: a list of (w, w_delta, gradient) triples; the argument arrays are
    built once, each step passes the scalars:

        upd = cm.MomentumUpdates([(W1, dW1, gW1), (b1, db1, gb1), ...])
        upd.apply(momentum, epsilon)                 # the same bits as one momentum_update each

    momentum, epsilon, l2_decay, l1_decay: one number for all parameters or a sequence with one
    entry per parameter (l2_decay / l1_decay None: no such term)."""

    def __init__(self, updates):
        self._keep = [tuple(u) for u in updates]
        n = len(self._keep)
        ptrs = ct.POINTER(cudamat) * n
        self._w = ptrs(*[u[0].p_mat for u in self._keep])
        self._wd = ptrs(*[u[1].p_mat for u in self._keep])
        self._g = ptrs(*[u[2].p_mat for u in self._keep])
        self._n = n
        self._cache = {}

    def _floats(self, v):
        seq = [0.0 if x is None else float(x) for x in (v if isinstance(v, (list, tuple)) else [v] * self._n)]
        if len(seq) != self._n:
            raise ValueError("one value per parameter expected")
        return (ct.c_float * self._n)(*seq)

    def apply(self, momentum, epsilon, l2_decay=None, l1_decay=None, reset_gradient=True):
        key = (repr(momentum), repr(epsilon), repr(l2_decay), repr(l1_decay), bool(reset_gradient))
        args = self._cache.get(key)
        if args is None:
            per = lambda v: list(v) if isinstance(v, (list, tuple)) else [v] * self._n
            flags = [(1 if a is not None else 0) | (2 if b is not None else 0) | (4 if reset_gradient else 0)
                     for a, b in zip(per(l2_decay), per(l1_decay))]
            args = (self._floats(momentum), self._floats(l2_decay), self._floats(l1_decay), self._floats(epsilon),
                    (ct.c_int * self._n)(*flags))
            if len(self._cache) > 64:
                self._cache.clear()
            self._cache[key] = args
        _check(_cudamat.momentum_update_many(self._n, self._w, self._wd, self._g, args[0], args[1], args[2], args[3], args[4]))


class SparseCUDAMatrix(object):
    """A compressed-sparse-row matrix on the device.  The reference exports the C entry
    points (cudamat.cu:125-213, 407-418, 1698-1727) but has no Python class for them; this
    one only packs the three CSR arrays (data, indices, indptr as scipy.sparse.csr_matrix
    holds them) into the C handle and uploads them."""

    def __init__(self, data, indices, indptr, shape, copy_to_device=True):
        self.data = np.ascontiguousarray(data, dtype=np.float32)
        self.indices = np.ascontiguousarray(indices, dtype=np.int32)
        self.indptr = np.ascontiguousarray(indptr, dtype=np.int32)
        m, n = int(shape[0]), int(shape[1])
        if self.indptr.size != m + 1 or self.data.size != self.indices.size:
            raise ValueError("CSR arrays do not fit the shape")
        self.shape = (m, n)
        self.mat = cudamat_sparse()
        self.p_mat = ct.pointer(self.mat)
        _cudamat.init_from_sparse_array(self.p_mat, self.data.ctypes.data_as(ct.POINTER(ct.c_float)),
                                        self.indices.ctypes.data_as(ct.POINTER(ct.c_int)),
                                        self.indptr.ctypes.data_as(ct.POINTER(ct.c_int)), m, n, int(self.data.size))
        if copy_to_device:
            self.copy_to_device()

    def copy_to_device(self):
        _check(_cudamat.copy_sparse_to_device(self.p_mat))

    def free_device_memory(self):
        _check(_cudamat.free_device_memory_sparse(self.p_mat))


def sparse_dot(sparse, dense, target=None, beta=0.0, alpha=1.0):
    """target = beta * target + alpha * sparse . dense (cudamat.cu:1698-1727; dense and
    target are taken as plain column-major arrays)."""
    if target is None:
        target = empty((sparse.shape[0], dense.mat.size[1]))
    _check(_cudamat.sparse_dot(sparse.p_mat, dense.p_mat, target.p_mat, ct.c_float(beta), ct.c_float(alpha)))
    return target


def vdot(m1, m2):
    """Dot product of m1 and m2 taken as flat vectors."""
    err_code = ct.c_int(0)
    res = _cudamat.vdot(m1.p_mat, m2.p_mat, ct.byref(err_code))
    _check(err_code.value)
    return res


def softmax(mat, target=None):
    """Softmax of every column."""
    if target is not None:
        _check(_cudamat.softmax(mat.p_mat, target.p_mat))
    else:
        _check(_cudamat.softmax_overwrite(mat.p_mat))
        target = mat
    return target


def _unary_function(cname, doc):
    fn = getattr(_cudamat, cname)

    def function(mat, target=None):
        if target is None:
            target = mat
        _check(fn(mat.p_mat, target.p_mat))
        return target
    function.__doc__ = doc
    return function


cos = _unary_function('apply_cos', "cos of each element.")
sin = _unary_function('apply_sin', "sin of each element.")
sigmoid = _unary_function('apply_sigmoid', "Logistic sigmoid of each element.")
tanh = _unary_function('apply_tanh', "tanh of each element.")
abs = _unary_function('apply_abs', "Absolute value of each element.")
exp = _unary_function('apply_exp', "exp of each element.")
ceil = _unary_function('apply_ceil', "ceil of each element.")
floor = _unary_function('apply_floor', "floor of each element.")
sqrt = _unary_function('apply_sqrt', "Square root of each element.")


def log_1_plus_exp(mat, target=None, exact=False):
    """log(1 + exp(x)) of each element.  `exact` is accepted for compatibility: the
    device code always uses the accurate exp and log."""
    if target is None:
        target = mat
    _check(_cudamat.apply_log_1_plus_exp(mat.p_mat, target.p_mat))
    return target


def log(mat, tiny=0.0, target=None):
    """log(x + tiny) of each element."""
    if target is None:
        target = mat
    _check(_cudamat.apply_log(mat.p_mat, target.p_mat, float(tiny)))
    return target


def _binary_param(fn, mat, p, target, value):
    if target is None:
        target = mat
    if not isinstance(p, CUDAMatrix):
        raise ValueError("Value must be of type CUDAMatrix.")
    _check(fn(mat.p_mat, p.p_mat, target.p_mat, float(value)))
    return target


def cross_entropy_bernoulli(mat, p, target=None, tiny=1e-10):
    """-mat*log(p + tiny) - (1-mat)*log(1 - p + tiny)"""
    return _binary_param(_cudamat.compute_cross_entropy_bernoulli, mat, p, target, tiny)


def cross_entropy(mat, p, target=None, tiny=1e-10):
    """-mat*log(p + tiny)"""
    return _binary_param(_cudamat.compute_cross_entropy, mat, p, target, tiny)


def correct_preds(mat, p, target=None, cutoff=0.5):
    """mat*(p >= cutoff) + (1-mat)*(p < cutoff)"""
    return _binary_param(_cudamat.correct_preds, mat, p, target, cutoff)


def pow(mat, p, target=None):
    """mat ** p elementwise; p is a scalar or a CUDAMatrix of the same shape."""
    if target is None:
        target = mat
    if isinstance(p, CUDAMatrix):
        _check(_cudamat.apply_pow_matrix(mat.p_mat, p.p_mat, target.p_mat))
    elif _is_scalar(p):
        _check(_cudamat.apply_pow(mat.p_mat, float(p), target.p_mat))
    else:
        raise ValueError("Value must be of type CUDAMatrix, int, or float.")
    return target


def cuda_sync_threads():
    _cudamat.cuda_sync_threads()


def reformat(array):
    """Return array as a float32 array in FORTRAN order."""
    return np.array(array, dtype=np.float32, order='F')


def cuda_set_device(dev_id):
    _check(_cudamat.cuda_set_device(int(dev_id)))


def cublas_init():
    """Initialise the library and the device vector of ones used by the sums."""
    _check(_cudamat.cublas_init())
    CUDAMatrix.ones = CUDAMatrix(np.ones((MAX_ONES, 1), dtype=np.float32, order='F'))


init = cublas_init


def cublas_shutdown():
    CUDAMatrix.ones = 0
    _ones_views.clear()
    del _ones_retired[:]
    _cudamat.cublas_shutdown()


shutdown = cublas_shutdown
