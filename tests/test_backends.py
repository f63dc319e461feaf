"""The drop-in boundary on the host: directory scan, naming, symbol lookup, the torch.library
override and the CLI.  Techniques follow the reference's tests: pass-through and watermarked
implementations generated on the fly (test/test_directory_backend.py:35-120,
test/test_monkey_patch.py:100-229, test/test_backend_evaluation.py:64-115); the watermark is
the closed form 42 + int(md5(folder)[:8], 16) % 100
(BackendBench/scripts/create_watermarked_operators.py:24-29)."""

import hashlib
import os
import subprocess
import sys

import pytest
import torch

import backendbench_amd
from backendbench_amd import eval as ev
from backendbench_amd.backends import AtenBackend, Backend, DirectoryBackend
from backendbench_amd.suite import SmokeTestSuite
from backendbench_amd.suite.base import Test as Case

PASS_THROUGH = '''import torch

def {folder}_kernel_impl(*args, **kwargs):
    return torch.ops.aten.{op}(*args, **kwargs)
'''

WATERMARK = '''import torch

def {folder}_kernel_impl(*args, **kwargs):
    for a in args:
        if isinstance(a, torch.Tensor):
            return torch.full_like(a, {value})
    return torch.tensor({value})
'''


def watermark(folder):
    return 42.0 + int(hashlib.md5(folder.encode()).hexdigest()[:8], 16) % 100


def write_ops(base, template, folders, **extra):
    for folder, op in folders.items():
        d = base / folder
        d.mkdir(parents=True, exist_ok=True)
        (d / f"{folder}_implementation_v1.py").write_text(template.format(folder=folder, op=op, value=watermark(folder), **extra))


FIVE = {"relu__default": "relu.default", "add__Tensor": "add.Tensor", "mul__Tensor": "mul.Tensor",
        "abs__default": "abs.default", "sum__default": "sum.default"}


def test_watermark_closed_form():
    assert watermark("relu__default") == 42.0 + int(hashlib.md5(b"relu__default").hexdigest()[:8], 16) % 100
    assert 42.0 <= watermark("add__Tensor") < 142.0 and watermark("add__Tensor") != watermark("relu__default")


def test_backend_protocol():
    a = AtenBackend()
    assert isinstance(a, Backend) and a.name == "aten"
    for op in (torch.ops.aten.relu.default, torch.ops.aten.add.Tensor, "anything"):
        assert op in a and a[op] is op


def test_directory_backend_loads_pass_through_ops(tmp_path):
    write_ops(tmp_path, PASS_THROUGH, FIVE)
    (tmp_path / "README.md").write_text("not a folder")
    (tmp_path / "empty_folder").mkdir()
    (tmp_path / "no_such_op__default").mkdir()
    (tmp_path / "no_such_op__default" / "no_such_op__default_implementation_v1.py").write_text(
        "def no_such_op__default_kernel_impl(*a, **k):\n    return None\n")
    b = DirectoryBackend(str(tmp_path))
    assert b.name == "directory" and len(b.compiled_kernels) == 5
    x, y = torch.tensor([-1.0, 0.0, 1.0, 2.5]), torch.tensor([1.0, 2.0, 3.0, -4.0])
    assert torch.equal(b[torch.ops.aten.relu.default](x), torch.tensor([0.0, 0.0, 1.0, 2.5]))
    assert torch.equal(b[torch.ops.aten.add.Tensor](x, y), x + y)
    assert torch.equal(b[torch.ops.aten.mul.Tensor](x, y), x * y)
    assert torch.equal(b[torch.ops.aten.abs.default](x), x.abs())
    assert torch.equal(b[torch.ops.aten.sum.default](x), x.sum())
    assert torch.ops.aten.add.Scalar not in b      # only the exact overload is registered
    with pytest.raises(KeyError, match="not implemented in DirectoryBackend"):
        b[torch.ops.aten.add.Scalar]


def test_directory_backend_picks_first_file_and_survives_broken_folders(tmp_path):
    d = tmp_path / "relu__default"
    d.mkdir()
    (d / "relu__default_implementation_v2.py").write_text("def relu__default_kernel_impl(x):\n    return x * 0 + 2\n")
    (d / "relu__default_implementation_v1.py").write_text("def relu__default_kernel_impl(x):\n    return x * 0 + 1\n")
    (d / "other.py").write_text("raise RuntimeError('never imported')\n")
    bad = tmp_path / "mul__Tensor"
    bad.mkdir()
    (bad / "mul__Tensor_implementation_v1.py").write_text("def wrong_name(*a):\n    pass\n")
    worse = tmp_path / "add__Tensor"
    worse.mkdir()
    (worse / "add__Tensor_implementation_v1.py").write_text("raise ImportError('broken on import')\n")
    b = DirectoryBackend(str(tmp_path))
    assert list(b.compiled_kernels) == [torch.ops.aten.relu.default]
    assert b[torch.ops.aten.relu.default](torch.zeros(2)).tolist() == [1.0, 1.0]
    assert len(DirectoryBackend(str(tmp_path / "missing")).compiled_kernels) == 0


def test_inplace_folder_maps_to_inplace_overload(tmp_path):
    write_ops(tmp_path, PASS_THROUGH, {"add___Tensor": "add_.Tensor"})
    b = DirectoryBackend(str(tmp_path))
    assert torch.ops.aten.add_.Tensor in b and torch.ops.aten.add.Tensor not in b


def test_repo_kernel_directory_layout(repo_root):
    base = os.path.join(repo_root, "generated_kernels")
    from backendbench_amd.ops import SLOTS

    assert sorted(os.listdir(base)) == sorted(SLOTS)
    for folder in SLOTS:
        assert os.path.isfile(os.path.join(base, folder, f"{folder}_implementation_v1.py"))
    b = DirectoryBackend(base)
    assert len(b.compiled_kernels) == len(SLOTS) == 68
    expected = {"add.Tensor", "mul.Tensor", "maximum.default", "relu.default", "clamp.default", "where.self",
                "sum.dim_IntList", "sum.default", "mean.dim", "mean.default", "amax.default", "argmax.default",
                "_softmax.default", "native_layer_norm.default", "mm.default", "addmm.default",
                "index_select.default", "embedding.default", "gather.default"}
    from backendbench_amd.ops import CORE_SLOTS

    assert len(CORE_SLOTS) == 19 and expected <= {op.__name__ for op in b.compiled_kernels}
    assert {"add_.Tensor", "relu_.default", "clamp.Tensor", "_log_softmax.default", "mm.out", "sum.IntList_out"} <= {op.__name__ for op in b.compiled_kernels}


@pytest.mark.skipif(torch.cuda.is_available(), reason="host-only behaviour")
def test_wrappers_fail_loudly_without_a_gpu(repo_root):
    """No CPU fallback: on a machine without a GPU every slot raises instead of computing."""
    b = DirectoryBackend(os.path.join(repo_root, "generated_kernels"))
    with pytest.raises(RuntimeError, match="no GPU visible"):
        b[torch.ops.aten.relu.default](torch.randn(4))
    with pytest.raises(RuntimeError, match="no GPU visible"):
        b[torch.ops.aten.mm.default](torch.randn(4, 4), torch.randn(4, 4))
    c, p, cr, _ = ev.eval_one_op(torch.ops.aten.relu.default, b[torch.ops.aten.relu.default],
                                 [Case(lambda: torch.randn(2))], [])
    assert c == 0.0 and "no GPU visible" in cr[0].error_msg


def test_watermarked_ops_fail_correctness(tmp_path):
    write_ops(tmp_path, WATERMARK, {"relu__default": "relu.default"})
    b = DirectoryBackend(str(tmp_path))
    for t in SmokeTestSuite:
        c, p, cr, pr = ev.eval_one_op(t.op, b[t.op], t.correctness_tests, t.performance_tests)
        assert c == 0.0 and not cr[0].is_correct and float(p) == pytest.approx(1.0)


# ---- torch.library override (CPU key: runs everywhere) --------------------------------
def test_enable_disable_cpu_key(tmp_path):
    write_ops(tmp_path, WATERMARK, {"relu__default": "relu.default", "add__Tensor": "add.Tensor"})
    x = torch.tensor([-1.0, 0.0, 1.0])
    assert torch.relu(x).tolist() == [0.0, 0.0, 1.0]
    backendbench_amd.enable(kernel_dir=str(tmp_path), dispatch_key="CPU")
    try:
        assert torch.relu(x).tolist() == [watermark("relu__default")] * 3
        assert torch.add(x, x).tolist() == [watermark("add__Tensor")] * 3
        assert torch.mul(x, 2).tolist() == [-2.0, 0.0, 2.0]                  # ops without a folder untouched
        assert torch.nn.functional.leaky_relu(x, 0.01).tolist() == pytest.approx([-0.01, 0.0, 1.0])
    finally:
        backendbench_amd.disable()
    assert torch.relu(x).tolist() == [0.0, 0.0, 1.0]
    backendbench_amd.disable()  # a second disable only warns


def test_context_manager_restores_and_is_exception_safe(tmp_path):
    write_ops(tmp_path, WATERMARK, {"relu__default": "relu.default"})
    x = torch.tensor([-1.0, 0.0, 1.0])
    with backendbench_amd.BackendBench.enable(kernel_dir=str(tmp_path), dispatch_key="CPU"):
        assert torch.relu(x).tolist() == [watermark("relu__default")] * 3
    assert torch.relu(x).tolist() == [0.0, 0.0, 1.0]
    with pytest.raises(ValueError):
        with backendbench_amd.BackendBench.enable(kernel_dir=str(tmp_path), dispatch_key="CPU"):
            assert torch.relu(x)[0].item() == watermark("relu__default")
            raise ValueError("inside")
    assert torch.relu(x).tolist() == [0.0, 0.0, 1.0]


def test_enable_rejects_other_dispatch_keys(tmp_path, caplog):
    write_ops(tmp_path, WATERMARK, {"relu__default": "relu.default"})
    backendbench_amd.enable(kernel_dir=str(tmp_path / "missing"))  # missing directory: warning, no-op
    assert torch.relu(torch.tensor([-1.0])).item() == 0.0


# ---- CLI -------------------------------------------------------------------------------
def run_cli(repo_root, *argv):
    env = dict(os.environ, PYTHONPATH=repo_root)
    return subprocess.run([sys.executable, "-m", "backendbench_amd.scripts.main", *argv], cwd=repo_root, env=env,
                          capture_output=True, text=True, timeout=300)


def test_cli_smoke_directory_backend(tmp_path, repo_root):
    write_ops(tmp_path / "ops", PASS_THROUGH, {"relu__default": "relu.default"})
    r = run_cli(repo_root, "--suite", "smoke", "--backend", "directory", "--ops-directory", str(tmp_path / "ops"))
    assert r.returncode == 0, r.stderr
    assert "correctness score (mean pass rate over all operators): 1.00" in r.stdout
    for name in ("full_results.json", "operator_summary.csv", "failed_tests.json", "OVERALL_SUMMARY.md"):
        assert (tmp_path / "ops" / name).is_file()          # default log dir = the ops directory


def test_cli_aten_backend_and_flag_checks(tmp_path, repo_root):
    r = run_cli(repo_root, "--suite", "smoke", "--backend", "aten", "--log-dir", str(tmp_path / "out"))
    assert r.returncode == 0 and (tmp_path / "out" / "OVERALL_SUMMARY.md").is_file()
    r = run_cli(repo_root, "--suite", "smoke", "--topn-inputs", "3", "--disable-output-logs")
    assert r.returncode != 0 and "topn-inputs" in (r.stderr + r.stdout)
