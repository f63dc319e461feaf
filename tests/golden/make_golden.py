"""Writes tests/golden/aten_cpu_golden.json: a digest of the oracle's output for every edge
case of the suite (inputs are seeded, so only outputs need recording).

    python tests/golden/make_golden.py

Made with torch's ATen CPU kernels (the oracle, oracle/aten_cpu.py) — the reference package
itself is not imported.  The file pins the oracle against drift of the torch build: a
different torch that changes any result changes a digest.  Per output tensor it stores
shape and dtype, plus a SHA-256 of the bytes (integer outputs) or special-value counts, norms
and the first values (floating outputs).
"""

import hashlib
import json
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from backendbench_amd.suite import edge_cases  # noqa: E402
from oracle import aten_cpu  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "aten_cpu_golden.json")


def digest(t):
    """Integer/bool outputs: SHA-256 of the bytes (exact).  Floating outputs: counts of NaN,
    +inf, -inf, the fp64 L1 norm and signed sum of the finite values, and the first values —
    compared with a small tolerance so that a different host CPU (thread count, vector width:
    summation order) does not trip it while a changed formula does."""
    t = t.detach().cpu().contiguous().reshape(-1)
    d = {"shape": None, "dtype": str(t.dtype)}
    if t.dtype.is_floating_point:
        x = t.double()
        finite = torch.isfinite(x)
        d.update(nan=int((x != x).sum()), pinf=int((x == float("inf")).sum()), ninf=int((x == float("-inf")).sum()),
                 l1=float(x[finite].abs().sum()), total=float(x[finite].sum()),
                 head=[v if v == v and abs(v) != float("inf") else str(v) for v in x[:6].tolist()])
    else:
        raw = t.view(torch.uint8).numpy().tobytes() if t.numel() else b""
        d.update(sha256=hashlib.sha256(raw).hexdigest(), head=[int(v) for v in t[:6].tolist()])
    return d


def record(case):
    args, kwargs = case.make("cpu")
    out = aten_cpu.reference(case.op, args, kwargs)
    outs = out if isinstance(out, (tuple, list)) else [out]
    ds = [digest(o) for o in outs]
    for d, o in zip(ds, outs):
        d["shape"] = list(o.shape)
    return ds


def main():
    table = {"torch": torch.__version__, "cases": {c.key: record(c) for c in edge_cases()}}
    with open(OUT, "w") as f:
        json.dump(table, f, indent=0, sort_keys=True)
    print(f"wrote {len(table['cases'])} cases to {OUT} ({os.path.getsize(OUT) // 1024} KiB)")


if __name__ == "__main__":
    main()
