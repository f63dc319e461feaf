"""addmm.dtype on the MI355X HIP kernels (directory-backend entry point)."""

import os
import sys

_ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
if _ROOT not in sys.path:
    sys.path.insert(0, _ROOT)

from backendbench_amd.ops import SLOTS as _SLOTS  # noqa: E402

_op = _SLOTS["addmm__dtype"]


def addmm__dtype_kernel_impl(*args, **kwargs):
    return _op(*args, **kwargs)
