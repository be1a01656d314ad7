"""CPU-only: the shared libraries load and export every symbol the headers under
include/ declare; the ctypes mirrors have the C layout; argument errors that are
detected before any device work come back with the reference's codes."""
import ctypes as ct
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header):
    text = open(os.path.join(ROOT, 'include', header)).read()
    text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
    names = re.findall(r'^\s*(?:const\s+)?(?:int|float|void|char\s*\*|const char\s*\*)\s*\*?\s*(\w+)\s*\(', text, flags=re.M)
    return sorted(set(names))


@pytest.mark.parametrize("header,lib", [('cudamat_amd.h', 'libcudamat.so'), ('cudamat_conv_amd.h', 'libcudamat_conv.so')])
def test_every_declared_symbol_is_exported(header, lib):
    names = _declared(header)
    assert len(names) > 10, names
    dll = ct.CDLL(os.path.join(ROOT, 'deepnet_amd', lib))
    missing = [n for n in names if not hasattr(dll, n)]
    assert not missing, missing


def test_conv_library_exports_its_entry_points_and_nothing_else():
    """The reference's conv library exports its 13 entry points (cudamat_conv.cu:1402-1456); this one
    adds conv_last_error and the two fused pooling + normalisation calls, and takes stream, workspaces and contraction kernels from libcudamat.so, so a
    program that links both gets one copy of that state and no second `dot`."""
    import subprocess
    lib = os.path.join(ROOT, 'deepnet_amd', 'libcudamat_conv.so')
    out = subprocess.run(['nm', '-D', '--defined-only', lib], check=True, capture_output=True, text=True).stdout
    exported = sorted(line.split()[-1] for line in out.splitlines() if line.strip())
    want = sorted("""convUp convDown convOutp localUp localDown localOutp ResponseNorm ResponseNormUndo ContrastNorm
    ContrastNormUndo MaxPool ProbMaxPool MaxPoolUndo conv_last_error MaxPoolResponseNorm
    ResponseNormUndoMaxPoolUndo""".split())
    assert exported == want
    needed = subprocess.run(['readelf', '-d', lib], check=True, capture_output=True, text=True).stdout
    assert 'libcudamat.so' in needed and '$ORIGIN' in needed


def test_matrix_header_covers_what_the_reference_binds_at_import():
    # the ~60 symbols cudamat/cudamat.py:12-79 touches while importing
    needed = """get_last_cuda_error cublas_init cublas_shutdown cuda_set_device init_random init_empty reshape
    copy_to_host copy_to_device copy_on_device free_device_memory get_slice get_row_slice set_row_slice
    copy_transpose get_vector_slice fill_with_rand fill_with_randn add_col_vec add_col_mult add_row_mult
    add_row_vec mult_by_col_vec mult_by_row_vec div_by_col_vec div_by_row_vec less_than less_than_scalar
    greater_than greater_than_scalar max_by_axis argmax_by_axis sqsum_by_axis normlimit_by_axis sign
    apply_sigmoid apply_tanh apply_abs apply_log_1_plus_exp apply_log apply_floor apply_ceil apply_exp
    apply_sqrt apply_pow apply_pow_matrix reciprocal add_elementwise subtract_elementwise divide_elementwise
    mult_elementwise apply_logistic_deriv assign_scalar mult_by_scalar divide_by_scalar add_scalar euclid_norm
    selectRows setSelectedRows vdot dot""".split()
    declared = set(_declared('cudamat_amd.h'))
    assert not [n for n in needed if n not in declared]


def test_struct_layout_matches_the_c_struct():
    from deepnet_amd import cudamat as cm
    assert ct.sizeof(cm.cudamat) == 40            # 2 pointers + 6 ints on LP64 (cudamat.cuh:21-29)
    assert cm.cudamat.size.offset == 24 and cm.cudamat.is_trans.offset == 32 and cm.cudamat.owns_data.offset == 36
    assert ct.sizeof(cm.rnd_struct) == 16


def test_host_side_argument_errors_need_no_device():
    from deepnet_amd import cudamat as cm
    x = np.arange(12, dtype=np.float32).reshape(3, 4)
    a = cm.CUDAMatrix(x, copy_to_device=False)
    b = cm.CUDAMatrix(x, copy_to_device=False)
    assert a.shape == (3, 4) and a.mat.on_host == 1 and a.mat.on_device == 0 and a.mat.owns_data == 1
    assert a.numpy_array.flags['F_CONTIGUOUS'] and a.numpy_array.dtype == np.float32      # reformat()
    lib = cm._cudamat
    assert lib.get_leading_dimension(a.p_mat) == 3 and lib.get_nonleading_dimension(a.p_mat) == 4
    assert lib.get_leading_dimension(a.T.p_mat) == 4 and a.T.mat.is_trans == 1 and a.mat.is_trans == 0
    # not on device -> -8, for every family
    assert lib.add_elementwise(a.p_mat, b.p_mat, a.p_mat) == -8
    assert lib.apply_sigmoid(a.p_mat, a.p_mat) == -8
    assert lib.add_col_vec(a.p_mat, b.p_mat, a.p_mat) == -8
    assert lib.dot(a.p_mat, b.p_mat, a.p_mat, 0.0, 1.0) == -8
    assert lib.max_by_axis(a.p_mat, b.p_mat, 0) == -8
    assert lib.copy_to_host(a.p_mat) == -8
    assert lib.fill_with_rand(None, a.p_mat) == -8
    assert lib.get_slice(a.p_mat, ct.byref(cm.cudamat()), 0, 1) == -8
    assert lib.get_slice(a.T.p_mat, ct.byref(cm.cudamat()), 0, 1) == -5        # transposed first (cudamat.cu:332-336)
    assert lib.sample_bernoulli(None, a.p_mat, cm.CUDAMatrix(np.zeros((2, 2), np.float32), False).p_mat) == -1
    # a generator that init_random() never set up is refused (-6) instead of dereferenced
    fake = cm.cudamat()
    fake.on_device, fake.size[0], fake.size[1] = 1, 2, 2        # claims to be on the device; never touched
    empty_state = cm.rnd_struct()
    for st in (None, ct.byref(empty_state)):
        assert lib.fill_with_rand(st, ct.byref(fake)) == -6 and lib.fill_with_randn(st, ct.byref(fake)) == -6
        assert lib.sample_bernoulli(st, ct.byref(fake), ct.byref(fake)) == -6
        assert lib.sample_gaussian(st, ct.byref(fake), ct.byref(fake), ct.c_float(1.0)) == -6
        assert lib.dropout(st, ct.byref(fake), ct.c_float(0.5), ct.c_float(0.0)) == -6
    with pytest.raises(cm.CUDAMatException, match="not in device memory"):
        a.add(b)
    # reshape is pure bookkeeping
    a.reshape((4, 3)); assert a.shape == (4, 3)
    a.reshape((-1, 6)); assert a.shape == (2, 6)
    with pytest.raises(cm.CUDAMatException, match="Incompatible matrix dimensions"):
        a.reshape((5, 5))
    a.set_shape((1, 12)); assert a.shape == (1, 12)
    assert lib.free_device_memory(a.p_mat) == 0                     # nothing on the device: a no-op
    assert isinstance(cm.generate_exception(-7), cm.CUDAMatException)
    assert "transposedness" in str(cm.generate_exception(-7))
    with pytest.raises(ValueError):
        a.assign("nope")


def test_missing_library_is_loud(tmp_path, monkeypatch):
    import importlib.util
    src = os.path.join(ROOT, 'deepnet_amd', 'cudamat.py')
    dst = tmp_path / 'cudamat_copy.py'
    dst.write_text(open(src).read())
    spec = importlib.util.spec_from_file_location('cudamat_copy', str(dst))
    mod = importlib.util.module_from_spec(spec)
    with pytest.raises(ImportError, match="no CPU fallback"):
        spec.loader.exec_module(mod)


def test_sparse_struct_layout_and_host_side_init():
    from deepnet_amd import cudamat as cm
    # three pointers; two of them + 7 ints, padded to pointer alignment (cudamat.cuh:36-50)
    assert ct.sizeof(cm.sparse_data) == 24 and ct.sizeof(cm.cudamat_sparse) == 80
    assert cm.cudamat_sparse.size.offset == 56 and cm.cudamat_sparse.nnz.offset == 72
    sp = cm.SparseCUDAMatrix([1.0, 2.0, 3.0], [0, 2, 1], [0, 2, 3], (2, 3), copy_to_device=False)
    assert (sp.mat.size[0], sp.mat.size[1], sp.mat.nnz) == (2, 3, 3)
    assert sp.mat.on_host == 1 and sp.mat.on_device == 0 and sp.mat.owns_data == 1 and sp.mat.is_trans == 0
    assert sp.mat.data_host.indptr[2] == 3 and sp.mat.data_host.data[1] == 2.0
    with pytest.raises(ValueError):
        cm.SparseCUDAMatrix([1.0], [0], [0, 1], (2, 3), copy_to_device=False)
