"""Parameter (de)serialisation of deepnet checkpoints: the raw float32 byte strings the
reference keeps in ``Parameter.mat`` with the shape in ``Parameter.dimensions``
(deepnet/util.py:13-21, deepnet/parameter.py:17-19).  Works on any object with ``name``, ``mat``
and ``dimensions`` attributes, e.g. a message of the reference's deepnet_pb2 or ``ParamRecord``."""
import os

import numpy as np


class ParamRecord(object):
    """Stand-in for the protobuf Parameter message: name, mat (bytes), dimensions (list of int)."""

    def __init__(self, name, mat=b'', dimensions=()):
        self.name, self.mat, self.dimensions = name, mat, list(dimensions)


def ParameterAsNumpy(param):
    """The array stored in a parameter record: row-major float32 of shape ``dimensions``."""
    return np.frombuffer(param.mat, dtype='float32').reshape(*tuple(param.dimensions)).copy()


def NumpyAsParameter(numpy_array):
    """The byte string to store for an array (row-major, whatever the array's memory order)."""
    assert numpy_array.dtype == 'float32', 'Saved arrays should be float32.'
    return numpy_array.tobytes()


def SaveParameters(obj, records):
    """Write the device parameters of a layer or edge into its records (parameter.py:17-19)."""
    for rec in records:
        arr = obj.params[rec.name].asarray()
        rec.mat = NumpyAsParameter(arr)
        rec.dimensions[:] = list(arr.shape)


def LoadParameters(obj, records):
    """Upload the arrays held by the records into the device parameters of a layer or edge,
    reusing the device buffers (the shapes must match)."""
    from .choose_matrix_library import cm
    for rec in records:
        mat = ParameterAsNumpy(rec)
        if rec.name in obj.params:
            assert obj.params[rec.name].shape == mat.shape
            obj.params[rec.name].overwrite(mat)
        else:
            obj.params[rec.name] = cm.CUDAMatrix(mat)


def _read_text_message(path):
    from . import pbtxt
    if os.path.splitext(path)[1] != '.pbtxt':
        raise NotImplementedError('%s: only text-format (.pbtxt) files are read; binary protocol '
                                  'buffers need the generated message classes' % path)
    with open(path) as f:
        return pbtxt.parse(f.read())


def ReadModel(proto_file):
    """deepnet/util.py:67-77 for text-format files: the Model message as a pbtxt.Message tree."""
    return _read_text_message(proto_file)


def ReadOperation(proto_file):
    """deepnet/util.py:55-65 for text-format files."""
    return _read_text_message(proto_file)


def WritePbtxt(output_file, pb):
    """deepnet/util.py:79-81: a message tree as a text-format file."""
    from . import pbtxt
    with open(output_file, 'w') as f:
        f.write(pbtxt.dumps(pb))
