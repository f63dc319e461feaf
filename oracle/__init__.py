"""TEST INFRASTRUCTURE — not part of the product.

The checker the HIP kernels are compared against.  Only tests/, __graft_entry__.smoke()
and bench.py's cpu_baseline leg may import this package; backendbench_amd never does.

What the oracle is
------------------
The reference (meta-pytorch/BackendBench) defines the correct result of an operator as
`torch.ops.aten.<op>(*args, **kwargs)` (BackendBench/eval.py:100, BackendBench/backends/
aten.py:14-15): the arithmetic lives in the third-party dependency `torch`
(pyproject.toml:19, unpinned there; this image pins torch 2.10.0+rocm7.0), not under the
reference tree.  `aten_cpu.reference()` runs exactly that on CPU copies of the arguments.
`numpy_ref` restates the published definition of every operator in numpy float64 / exact
integer arithmetic; tests/test_oracle.py pins the first against the second, against the
literal expectations the reference's own tests hold
(test/test_monkey_patch.py:100,135,188; test/test_directory_backend.py:35-94), against
closed forms and brute force, and against the committed digests in
tests/golden/aten_cpu_golden.json (drift of the torch build).

Parity status: every function of `aten_cpu` is pinned by those checks; none is
"parity unpinned".
"""
