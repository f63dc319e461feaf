"""Writes the directory-backend tree for this operator set.

    python -m backendbench_amd.scripts.create_kernel_directory [ops_dir]

creates ``<ops_dir>/<folder>/<folder>_implementation_v1.py`` for every slot in
backendbench_amd.ops.SLOTS, each exporting ``<folder>_kernel_impl`` — the layout
BackendBench/backends/directory.py:25-100 scans (and
BackendBench/scripts/create_simple_test_ops.py:20-109 exemplifies).  The files are
executed by path, outside any package, so each one puts the repository root on
sys.path itself before importing the wrappers.
"""

import os
import sys

TEMPLATE = '''"""{op_name} on the MI355X HIP kernels (directory-backend entry point)."""

import os
import sys

_ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
if _ROOT not in sys.path:
    sys.path.insert(0, _ROOT)

from backendbench_amd.ops import SLOTS as _SLOTS  # noqa: E402

_op = _SLOTS["{folder}"]


def {folder}_kernel_impl(*args, **kwargs):
    return _op(*args, **kwargs)
'''


def create(ops_dir="generated_kernels"):
    from backendbench_amd.ops import SLOTS
    from backendbench_amd.utils import folder_name_to_op_name

    os.makedirs(ops_dir, exist_ok=True)
    for folder in SLOTS:
        d = os.path.join(ops_dir, folder)
        os.makedirs(d, exist_ok=True)
        with open(os.path.join(d, f"{folder}_implementation_v1.py"), "w") as f:
            f.write(TEMPLATE.format(folder=folder, op_name=folder_name_to_op_name(folder)))
    return sorted(SLOTS)


if __name__ == "__main__":
    target = sys.argv[1] if len(sys.argv) > 1 else "generated_kernels"
    names = create(target)
    print(f"wrote {len(names)} operator folders under {target}/")
