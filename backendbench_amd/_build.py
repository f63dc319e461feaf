"""Builds libmi355_aten.so (hand-written HIP, gfx950 only) in-tree with hipcc.

The library lands in backendbench_amd/lib/ so that it travels with the source tree to
the machine that has the GPU; nothing is compiled at import time.  Run as
``python -m backendbench_amd._build`` or through ``__graft_entry__.build()``.
"""

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_DIR = PKG_DIR / "lib"
LIB_PATH = LIB_DIR / "libmi355_aten.so"
OBJ_DIR = LIB_DIR / "obj"

SOURCES = [
    "common.hip",
    "elementwise.hip",
    "reduce.hip",
    "softmax.hip",
    "layernorm.hip",
    "index.hip",
    "gemm.hip",
    "gemm_x16.hip",
    "gemm_f64.hip",
    "calib.hip",
]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# Packed-FP32 VALU forms are switched off for device code (the host pass does not know
# the feature and says so; that is harmless).
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _fresh(src: str, obj: Path) -> bool:
    """True when `obj` is newer than its source and every header beside it."""
    if not obj.exists():
        return False
    deps = [CSRC / src, *CSRC.glob("*.h"), PKG_DIR.parent / "include" / "mi355_aten.h", Path(__file__)]
    return obj.stat().st_mtime > max(d.stat().st_mtime for d in deps)


def _compile(src: str, incremental: bool = False) -> Path:
    obj = OBJ_DIR / (Path(src).stem + ".o")
    if incremental and _fresh(src, obj):
        return obj
    cmd = [HIPCC, *FLAGS, "-c", str(CSRC / src), "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{proc.stdout}\n{proc.stderr}")
    return obj


TRACE_LIB_PATH = LIB_DIR / "libmi355_gemm_trace.so"


def build_trace(verbose: bool = True) -> Path:
    """The GEMM sources once more with -DMI355_GEMM_TRACE: the four-wave kernels then stamp the
    shader clock (s_memtime) around the phases of every tile and of every step of the K loop and
    leave the sums in the caller's workspace (layout beside the stamps in csrc/gemm.hip).  A
    diagnostic build of its own, read by `bench.py --only-op C3.mm_down --trace`; the product
    library carries no stamps."""
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    objs = []
    for src, extra in (("gemm.hip", ["-DMI355_GEMM_TRACE"]), ("gemm_x16.hip", ["-DMI355_GEMM_TRACE"]), ("gemm_f64.hip", []), ("common.hip", ["-DMI355_GEMM_ONLY"])):
        obj = OBJ_DIR / (Path(src).stem + ".trace.o")
        proc = subprocess.run([HIPCC, *FLAGS, *extra, "-c", str(CSRC / src), "-o", str(obj)], capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed for {src} (trace build):\n{proc.stdout}\n{proc.stderr}")
        objs.append(obj)
    tmp = TRACE_LIB_PATH.with_suffix(".so.tmp")
    proc = subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *map(str, objs), "-o", str(tmp)],
                          capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed (trace build):\n{proc.stdout}\n{proc.stderr}")
    os.replace(tmp, TRACE_LIB_PATH)
    if verbose:
        print(f"built {TRACE_LIB_PATH} ({TRACE_LIB_PATH.stat().st_size // 1024} KiB)")
    return TRACE_LIB_PATH


def ablate_lib_path(bits: int) -> Path:
    return LIB_DIR / f"libmi355_gemm_ablate_{bits}.so"


def build_ablate(bits: int, verbose: bool = True) -> Path:
    """A measurement build of the GEMM sources with -DMI355_X16_ABLATE=<bits>: parts of the 16x16x32
    kernel's K loop or epilogue left out (bit list beside the macro in csrc/gemm_x16.hip).  Its results
    are wrong; `bench.py --only-op C3.mm_down --ablate <bits>` times it to show what each part costs."""
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    objs = []
    for src, extra in (("gemm.hip", []), ("gemm_x16.hip", [f"-DMI355_X16_ABLATE={bits}"]), ("gemm_f64.hip", []), ("common.hip", ["-DMI355_GEMM_ONLY"])):
        obj = OBJ_DIR / (Path(src).stem + f".ablate{bits}.o")
        proc = subprocess.run([HIPCC, *FLAGS, *extra, "-c", str(CSRC / src), "-o", str(obj)], capture_output=True, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed for {src} (ablation build):\n{proc.stdout}\n{proc.stderr}")
        objs.append(obj)
    out = ablate_lib_path(bits)
    tmp = out.with_suffix(".so.tmp")
    proc = subprocess.run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *map(str, objs), "-o", str(tmp)],
                          capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed (ablation build):\n{proc.stdout}\n{proc.stderr}")
    os.replace(tmp, out)
    if verbose:
        print(f"built {out} ({out.stat().st_size // 1024} KiB)")
    return out


def build(verbose: bool = True, jobs: int = 8, incremental: bool = False) -> Path:
    """Compile every kernel source for gfx950 and link the shared library.  `incremental`
    (developer convenience, `--incremental` on the command line) keeps objects that are newer
    than their source and the headers; the default recompiles everything."""
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(lambda s: _compile(s, incremental), SOURCES))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *map(str, objs), "-o", str(tmp)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stdout}\n{proc.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"built {LIB_PATH} ({LIB_PATH.stat().st_size // 1024} KiB)")
    return LIB_PATH


if __name__ == "__main__":
    if "--trace" in sys.argv[1:]:
        build_trace()
    elif "--ablate" in sys.argv[1:]:
        build_ablate(int(sys.argv[sys.argv.index("--ablate") + 1]))
    else:
        build(incremental="--incremental" in sys.argv[1:])
    sys.exit(0)
