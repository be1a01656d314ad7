"""Backend selector with the names deepnet modules import (`cm`, `cc`): the
counterpart of deepnet/choose_matrix_library.py:1-16.  There is one backend here,
the MI355X one; USE_GPU=no is refused instead of silently switching to a CPU
library."""
import os

use_gpu = os.environ.get('USE_GPU', 'auto')
assert use_gpu in ['auto', 'yes', 'no'], "environment variable USE_GPU, should be one of 'auto', 'yes', 'no'."
if use_gpu == 'no':
    raise ImportError("USE_GPU=no: this package only provides the GPU matrix backend.")

from . import cudamat as cm  # noqa: E402
from . import cudamat_conv as cc  # noqa: E402

__all__ = ['cm', 'cc']
