"""GPU tests of the overloads and callers next to the core slots:

  * out= overloads write their result into `out` itself when it has the result's shape, dtype and a
    dense layout (no temporary, no copy kernel), and fall back to compute-then-copy otherwise;
  * mm.dtype / addmm.dtype (BackendBench/scripts/op_map.py:740,271): bf16 / f16 operands, fp32 result;
  * a training step under the dispatcher override (BackendBench/__init__.py:70-143; the reference's
    docs/correctness.md:21 trains nanoGPT this way): forward on this backend's kernels, backward on
    ATen's, gradients compared with the stock run and with the CPU oracle;
  * the in-launch split-K's bounded wait giving up (forced from the host, every kernel runs to its end);
  * the allocation-free reduction under HIP graph capture and replay.

Through the drop-in boundary and the C ABI like every other GPU test; same bars as tests/test_parity_gpu.py.
"""

import ctypes
import os
import sys

import pytest
import torch

from backendbench_amd import _lib
from backendbench_amd import eval as ev
from backendbench_amd.backends import DirectoryBackend
from oracle import aten_cpu

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
aten = torch.ops.aten


@pytest.fixture(scope="module")
def backend():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return DirectoryBackend(os.path.join(ROOT, "generated_kernels"))


def announce(what):
    print(f"\n[gpu-case] {what}", flush=True)
    sys.stdout.flush()


def _t(shape, dtype=torch.float32, seed=0, scale=1.0):
    return (torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * scale).to(dtype)


class _LaunchSpy:
    """Records the C entry points the wrappers call (they all go through ops._common.launch)."""

    def __init__(self):
        import backendbench_amd.ops._common as c
        import backendbench_amd.ops.elementwise as e
        import backendbench_amd.ops.index as i
        import backendbench_amd.ops.matmul as m
        import backendbench_amd.ops.reduce as r

        self.mods, self.orig, self.calls = (c, e, r, m, i), c.launch, []

    def __enter__(self):
        def spy(name, *a):
            self.calls.append(name)
            return self.orig(name, *a)

        for mod in self.mods:
            mod.launch = spy
        return self

    def __exit__(self, *exc):
        for mod in self.mods:
            mod.launch = self.orig


# ---------------------------------------------------------------- out= in place
def _direct_out_cases():
    f32, bf16, i64 = torch.float32, torch.bfloat16, torch.int64
    idx = torch.tensor([4, 0, 4, 2, 7])
    gidx = torch.randint(0, 40, (9, 40), generator=torch.Generator().manual_seed(5))
    return [
        ("add.out", aten.add.out, [_t((64, 300)), _t((64, 300), seed=1)], {"alpha": 2}, ((64, 300), f32)),
        ("add.out_broadcast", aten.add.out, [_t((64, 300)), _t((300,), seed=1)], {}, ((64, 300), f32)),
        ("mul.out", aten.mul.out, [_t((64, 300), bf16), _t((64, 300), bf16, seed=1)], {}, ((64, 300), bf16)),
        ("maximum.out", aten.maximum.out, [_t((64, 300)), _t((64, 300), seed=1)], {}, ((64, 300), f32)),
        ("relu.out", aten.relu.out, [_t((64, 300))], {}, ((64, 300), f32)),
        ("clamp.out", aten.clamp.out, [_t((64, 300)), -0.1, 0.3], {}, ((64, 300), f32)),
        ("where.self_out", aten.where.self_out, [_t((64, 300), seed=9) > 0, _t((64, 300)), _t((64, 300), seed=1)], {}, ((64, 300), f32)),
        ("sum.IntList_out", aten.sum.IntList_out, [_t((6, 300, 4)), [1]], {"keepdim": True}, ((6, 1, 4), f32)),
        ("mean.out", aten.mean.out, [_t((64, 300)), [0]], {}, ((300,), f32)),
        ("amax.out", aten.amax.out, [_t((64, 300)), [-1]], {}, ((64,), f32)),
        ("argmax.out", aten.argmax.out, [_t((64, 300)), 1], {}, ((64,), i64)),
        ("_softmax.out", aten._softmax.out, [_t((64, 300)), -1, False], {}, ((64, 300), f32)),
        ("_log_softmax.out", aten._log_softmax.out, [_t((64, 300), bf16), -1, False], {}, ((64, 300), bf16)),
        ("mm.out", aten.mm.out, [_t((64, 96), bf16), _t((96, 32), bf16, seed=1)], {}, ((64, 32), bf16)),
        ("addmm.out", aten.addmm.out, [_t((32,)), _t((64, 96)), _t((96, 32), seed=1)], {"beta": 0.5, "alpha": 2.0}, ((64, 32), f32)),
        ("index_select.out", aten.index_select.out, [_t((9, 50)), 0, idx], {}, ((5, 50), f32)),
        ("embedding.out", aten.embedding.out, [_t((9, 50)), idx], {}, ((5, 50), f32)),
        ("gather.out", aten.gather.out, [_t((9, 40)), 1, gidx], {}, ((9, 40), f32)),
        ("sum.out", aten.sum.out, [_t((64, 300))], {}, ((), f32)),
    ]


@pytest.mark.parametrize("case", _direct_out_cases(), ids=[c[0] for c in _direct_out_cases()])
def test_out_overloads_write_into_out_without_a_copy(backend, case):
    """An `out` of the result's shape and dtype receives the kernel's stores directly: the wrapper launches
    the same entry points as the functional overload, no mi355_copy behind them, and returns `out` itself
    holding what ATen's out= overload writes on the CPU."""
    key, op, args, kwargs, (oshape, odtype) = case
    announce(key)
    out = torch.full(oshape, 7, dtype=odtype).cuda()
    gpu_args = [a.cuda() if isinstance(a, torch.Tensor) else a for a in args]
    with _LaunchSpy() as spy:
        res = backend[op](*gpu_args, out=out, **kwargs)
    torch.cuda.synchronize()
    from backendbench_amd.ops import check_index_errors

    check_index_errors()
    assert res is out
    assert "mi355_copy" not in spy.calls, f"{key}: the result went through a temporary ({spy.calls})"
    assert len(spy.calls) >= 1
    ref = op(*args, out=torch.full(oshape, 7, dtype=odtype), **kwargs)
    exact = not ref.dtype.is_floating_point or key in ("where.self_out", "index_select.out", "gather.out", "embedding.out")
    assert ev.allclose(ref, res.cpu(), exact=exact), key


def test_out_overloads_keep_permuted_layouts_and_refuse_aliases(backend):
    """A transposed `out` next to transposed operands is written in place (one flat pass over the shared
    layout); an `out` that shares memory with an operand, or differs in layout, dtype or shape, takes the
    compute-then-copy path.  Results equal ATen's in every case."""
    announce("out= layouts and aliasing")
    a, b = _t((300, 64)), _t((300, 64), seed=1)
    ag, bg = a.cuda().t(), b.cuda().t()                      # [64, 300] views, stride (1, 64)
    out = torch.empty(300, 64, device="cuda").t()
    with _LaunchSpy() as spy:
        res = backend[aten.add.out](ag, bg, out=out)
    assert res is out and spy.calls == ["mi355_binary"]
    assert ev.allclose(aten.add.Tensor(a.t(), b.t()), res.cpu())
    # row-major out, transposed operands: layouts differ, the result is copied into `out`
    out2 = torch.empty(64, 300, device="cuda")
    with _LaunchSpy() as spy:
        res = backend[aten.add.out](ag, bg, out=out2)
    assert res is out2 and "mi355_copy" in spy.calls
    assert ev.allclose(aten.add.Tensor(a.t(), b.t()), res.cpu())
    # out is one of the operands: never written while it is read
    x, y = _t((128, 96), torch.bfloat16).cuda(), _t((96, 96), torch.bfloat16, seed=2).cuda()
    want = aten_cpu.reference(aten.mm.default, [x, y])
    sq = y.clone()
    with _LaunchSpy() as spy:
        res = backend[aten.mm.out](sq, sq, out=sq)
    assert res is sq and "mi355_copy" in spy.calls
    assert ev.allclose(aten_cpu.reference(aten.mm.default, [y, y]), res.cpu())
    z = x.clone()
    res = backend[aten.relu.out](z, out=z)
    assert res is z and ev.allclose(aten_cpu.reference(aten.relu.default, [x]), z.cpu())
    assert ev.allclose(want, backend[aten.mm.default](x, y).cpu())


def test_native_layer_norm_out_writes_three_tensors_in_place(backend):
    announce("native_layer_norm.out in place")
    x, w, b = _t((6, 5, 256), torch.bfloat16, seed=3), _t((256,), torch.bfloat16, seed=4), _t((256,), torch.bfloat16, seed=5)
    outs = [torch.empty(6, 5, 256, dtype=torch.bfloat16, device="cuda"), torch.empty(6, 5, 1, device="cuda"), torch.empty(6, 5, 1, device="cuda")]
    with _LaunchSpy() as spy:
        res = backend[aten.native_layer_norm.out](x.cuda(), [256], w.cuda(), b.cuda(), 1e-5, out0=outs[0], out1=outs[1], out2=outs[2])
    assert spy.calls == ["mi355_layer_norm"] and all(r is o for r, o in zip(res, outs))
    ref = aten_cpu.reference(aten.native_layer_norm.default, [x, [256], w, b, 1e-5])
    for r, want in zip(res, ref):
        assert r.shape == want.shape and r.dtype == want.dtype and ev.allclose(want, r.cpu())


# ---------------------------------------------------------------- mm.dtype / addmm.dtype
def _f32_reference(a, b, c=None, alpha=1, beta=1):
    """What mm.dtype / addmm.dtype with out_dtype=float32 define (ATen has no CPU kernel for them): the fp32
    product of the exactly widened operands."""
    prod = aten_cpu.reference(aten.mm.default, [a.float(), b.float()])
    if c is None:
        return prod
    return beta * c.float().cpu() + alpha * prod if beta != 0 else alpha * prod


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_mm_dtype_returns_the_fp32_accumulators(backend, dtype):
    """bf16 / f16 operands, fp32 result: aligned shapes run on the MFMA kernels' fp32 store, everything else
    (odd K or N, strided views, K = 0, empty outputs) on the widened fp32 product; both are held to 1e-5 of the
    terms' scale against float64 - a result rounded to the operand dtype on the way would miss that by 100x."""
    from tight import tight_check

    announce(f"mm.dtype / addmm.dtype {dtype}")

    class Case:
        def __init__(self, op):
            self.op = op

    g = torch.Generator().manual_seed(11)
    shapes = [(256, 512, 384), (300, 256, 260), (129, 96, 64), (64, 100, 48), (77, 64, 50), (5, 8, 3), (128, 0, 64), (0, 64, 32), (1024, 2048, 1024)]
    for M, K, N in shapes:
        a = torch.randn(M, K, generator=g).to(dtype)
        b = (torch.randn(K, N, generator=g) * 0.1).to(dtype)
        bias = torch.randn(N, generator=g).to(dtype)
        for layout in ("nn", "nt"):
            bg = b.cuda() if layout == "nn" else b.t().contiguous().cuda().t()
            with _LaunchSpy() as spy:
                got = backend[aten.mm.dtype](a.cuda(), bg, torch.float32)
            assert got.dtype == torch.float32 and got.shape == (M, N)
            ref = _f32_reference(a, b)
            assert ev.allclose(ref, got.cpu()), (M, K, N, layout)
            if M and N and K:
                assert tight_check(Case(aten.mm.default), [a, b], {}, got.cpu()) is None, (M, K, N, layout)
            if K and K % 32 == 0 and N % 8 == 0 and M and N:
                assert spy.calls == [], f"{(M, K, N, layout)}: expected the direct fp32 store, saw {spy.calls}"
            got = backend[aten.addmm.dtype](bias.cuda(), a.cuda(), bg, torch.float32, beta=0.5, alpha=2)
            assert got.dtype == torch.float32
            ref = _f32_reference(a, b, bias, alpha=2, beta=0.5)
            assert ev.allclose(ref, got.cpu()), (M, K, N, layout, "addmm")
            if M and N and K:
                assert tight_check(Case(aten.addmm.default), [bias, a, b], {"beta": 0.5, "alpha": 2}, got.cpu()) is None
    # out_dtype equal to the operands' dtype is plain mm; anything else is refused as ATen's GPU kernels do
    a, b = torch.randn(64, 64, generator=g).to(dtype).cuda(), torch.randn(64, 64, generator=g).to(dtype).cuda()
    same = backend[aten.mm.dtype](a, b, dtype)
    assert same.dtype == dtype and ev.bit_equal(same.cpu(), backend[aten.mm.default](a, b).cpu())
    with pytest.raises(RuntimeError, match="out_dtype"):
        backend[aten.mm.dtype](a, b, torch.float64)
    with pytest.raises(RuntimeError, match="out_dtype"):
        backend[aten.mm.dtype](a.float(), b.float(), torch.bfloat16)
    # out= forms: in place when `out` is fp32 of the right shape, resized otherwise
    out = torch.empty(64, 64, device="cuda")
    assert backend[aten.mm.dtype_out](a, b, torch.float32, out=out) is out
    assert ev.allclose(_f32_reference(a.cpu(), b.cpu()), out.cpu())
    out = torch.empty(3, device="cuda")
    res = backend[aten.addmm.dtype_out](a[0], a, b, torch.float32, out=out)
    assert res is out and out.shape == (64, 64) and ev.allclose(_f32_reference(a.cpu(), b.cpu(), a[0].cpu()), out.cpu())


@pytest.mark.parametrize("which", ["up", "down"])
def test_mm_dtype_at_the_mlp_shapes(backend, which):
    """The two 7B-MLP products with fp32 output, sampled rows and columns against float64."""
    announce(f"mm.dtype C3 {which}")
    M, K, N = (4096, 4096, 11008) if which == "up" else (4096, 11008, 4096)
    g = torch.Generator().manual_seed(7)
    a = torch.randn(M, K, generator=g).bfloat16()
    b = (torch.randn(K, N, generator=g) * 0.02).bfloat16()
    got = backend[aten.mm.dtype](a.cuda(), b.cuda(), torch.float32)
    assert got.dtype == torch.float32 and got.shape == (M, N)
    rows = torch.tensor([0, 1, 127, 128, 255, 256, 2047, 2048, 4095])
    cols = torch.tensor([0, 1, 127, 128, 129, 255, 256, 4095, N - 129, N - 1])
    exact = a[rows].double() @ b.double()
    err = (got[rows.cuda()].cpu().double() - exact).abs()
    scale = torch.sqrt((a[rows].double() ** 2) @ (b.double() ** 2))
    assert bool((err <= 1e-5 * (K ** 0.5) * scale).all()), float((err / scale).max())
    exact_c = a.double() @ b[:, cols].double()
    err = (got[:, cols.cuda()].cpu().double() - exact_c).abs()
    scale = torch.sqrt((a.double() ** 2) @ (b[:, cols].double() ** 2))
    assert bool((err <= 1e-5 * (K ** 0.5) * scale).all()), float((err / scale).max())


# ---------------------------------------------------------------- training step under the override
def _tiny_transformer(dtype):
    torch.manual_seed(0)
    V, D, H, T = 503, 128, 256, 48

    class Block(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.emb = torch.nn.Embedding(V, D)
            self.ln1 = torch.nn.LayerNorm(D)
            self.qkv = torch.nn.Linear(D, 3 * D)
            self.proj = torch.nn.Linear(D, D)
            self.ln2 = torch.nn.LayerNorm(D)
            self.fc1 = torch.nn.Linear(D, H)
            self.fc2 = torch.nn.Linear(H, D)
            self.head = torch.nn.Linear(D, V, bias=False)

        def forward(self, tok):
            x = self.emb(tok)                                   # embedding
            h = self.ln1(x)                                     # native_layer_norm
            q, k, v = self.qkv(h).split(D, dim=-1)              # addmm
            att = torch.softmax((q @ k.transpose(-1, -2)) / D ** 0.5, dim=-1)   # mm, _softmax
            x = x + self.proj(att @ v)                          # add
            x = x + self.fc2(torch.relu(self.fc1(self.ln2(x))))  # relu
            return self.head(x)

    return Block().to(dtype), V, T


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_training_step_under_the_dispatcher_override(backend, dtype):
    """Forward on this backend's kernels, backward on ATen's own: the statistics native_layer_norm returns
    (fp32 mean / rstd), the probabilities of _softmax and the rows of embedding are what
    native_layer_norm_backward, _softmax_backward_data and embedding_dense_backward
    (BackendBench/scripts/op_map.py:775,192,445) expect.  The loss and every parameter's gradient agree with
    the stock run on the GPU, and in fp32 with autograd on the CPU (the oracle)."""
    import backendbench_amd

    announce(f"training step under enable(), {dtype}")
    model, V, T = _tiny_transformer(dtype)
    tok = torch.randint(0, V, (T,), generator=torch.Generator().manual_seed(1))
    target = torch.randint(0, V, (T,), generator=torch.Generator().manual_seed(2))

    def step(m, tok, target):
        m.zero_grad(set_to_none=True)
        logits = m(tok)
        loss = torch.nn.functional.cross_entropy(logits.float(), target)
        loss.backward()
        return loss.detach().float().cpu(), {n: p.grad.detach().float().cpu() for n, p in m.named_parameters()}

    cpu_loss, cpu_grads = step(model, tok, target) if dtype == torch.float32 else (None, None)
    gm = model.cuda()
    stock_loss, stock_grads = step(gm, tok.cuda(), target.cuda())
    with _LaunchSpy() as spy:
        with backendbench_amd.BackendBench.enable(kernel_dir=os.path.join(ROOT, "generated_kernels"), dispatch_key="CUDA"):
            ours_loss, ours_grads = step(gm, tok.cuda(), target.cuda())
            torch.cuda.synchronize()
    for name in ("mi355_index_select", "mi355_layer_norm", "mi355_gemm", "mi355_softmax", "mi355_unary", "mi355_binary"):
        assert name in spy.calls, f"{name} never ran in the training step ({sorted(set(spy.calls))})"
    tol = 2e-3 if dtype == torch.float32 else 5e-2

    def close(a, b, what):
        scale = max(float(b.abs().max()), 1e-6)
        err = float((a - b).abs().max())
        assert err <= tol * scale, f"{dtype} {what}: max abs diff {err:.3e} at scale {scale:.3e}"

    close(ours_loss, stock_loss, "loss vs stock")
    assert set(ours_grads) == set(stock_grads) and all(torch.isfinite(g).all() for g in ours_grads.values())
    for n in stock_grads:
        close(ours_grads[n], stock_grads[n], f"grad {n} vs stock")
    if cpu_grads is not None:
        close(ours_loss, cpu_loss, "loss vs CPU oracle")
        for n in cpu_grads:
            close(ours_grads[n], cpu_grads[n], f"grad {n} vs CPU oracle")


def test_gpt2_training_step_under_the_dispatcher_override(backend):
    """A randomly initialised 2-layer GPT-2 (transformers config, nothing downloaded): one forward + backward
    with the override on gives the loss and gradients of the stock run, in fp32 and in bf16."""
    transformers = pytest.importorskip("transformers")
    import backendbench_amd

    announce("GPT-2 training step under enable()")
    torch.manual_seed(0)
    cfg = transformers.GPT2Config(n_layer=2, n_head=4, n_embd=256, n_positions=128, vocab_size=1003,
                                  resid_pdrop=0.0, embd_pdrop=0.0, attn_pdrop=0.0)
    cfg._attn_implementation = "eager"
    model = transformers.GPT2LMHeadModel(cfg)
    ids = torch.randint(0, 1003, (4, 96), generator=torch.Generator().manual_seed(1)).cuda()
    for dtype in (torch.float32, torch.bfloat16):
        m = model.to(device="cuda", dtype=dtype).train()

        def step():
            m.zero_grad(set_to_none=True)
            loss = m(ids, labels=ids).loss
            loss.backward()
            return float(loss), {n: p.grad.detach().float().clone() for n, p in m.named_parameters() if p.grad is not None}

        stock_loss, stock = step()
        with backendbench_amd.BackendBench.enable(kernel_dir=os.path.join(ROOT, "generated_kernels"), dispatch_key="CUDA"):
            ours_loss, ours = step()
            torch.cuda.synchronize()
        tol = 2e-3 if dtype == torch.float32 else 6e-2
        assert abs(ours_loss - stock_loss) <= tol * max(abs(stock_loss), 1.0), (dtype, ours_loss, stock_loss)
        assert set(ours) == set(stock)
        for n in stock:
            scale = max(float(stock[n].abs().max()), 1e-6)
            err = float((ours[n] - stock[n]).abs().max())
            assert err <= tol * scale, f"{dtype} grad {n}: max abs diff {err:.3e} at scale {scale:.3e}"


# ---------------------------------------------------------------- split-K give-up path
def test_split_k_gives_up_cleanly_and_the_next_launch_is_unharmed(gemm_knobs):
    """The summing workgroup of the in-launch split-K waits for its partner a bounded number of polls.  With
    the limit set to 0 from the host it gives up at once: its tile is filled with NaNs, the library's status
    word reports it (mi355_gemm itself has long returned success), every kernel still runs to its end, and the
    producer's flag - raised after the give-up, in the same workspace - does not satisfy the next launch,
    which has a flag value of its own and gives the exact result."""
    announce("split-K bounded wait: give-up and recovery")
    lib = _lib.load()
    g = torch.Generator().manual_seed(31)
    M, K, N = 2048, 3072, 2304
    dtype = torch.bfloat16
    code = _lib.dtype_code(dtype)
    need = lib.mi355_gemm_workspace_bytes(M, N, K, code)
    assert need > 0
    a = (torch.randint(-1, 2, (M, K), generator=g) * (torch.randint(0, 4, (M, K), generator=g) == 0)).to(dtype).cuda()
    b = torch.randint(-1, 2, (N, K), generator=g).to(dtype).cuda().t()
    ref = aten_cpu.reference(aten.mm.default, [a.float(), b.float()]).to(dtype)
    ws = torch.zeros(need, dtype=torch.uint8, device="cuda")   # one workspace for every launch of this test
    out = torch.empty(M, N, dtype=dtype, device="cuda")

    def launch():
        _lib.check(lib.mi355_gemm(a.data_ptr(), a.stride(0), a.stride(1), b.data_ptr(), b.stride(0), b.stride(1), None, 0, 0,
                                  out.data_ptr(), M, N, K, 1.0, 0.0, code, ws.data_ptr(), need, _lib.current_stream_handle()))
        torch.cuda.synchronize()

    gemm_knobs.tile("x16split")
    launch()
    assert lib.mi355_gemm_status() == 0 and ev.bit_equal(ref, out.cpu())
    gemm_knobs.spin_limit(0)
    launch()                                                   # returns success; the kernels ran to their end
    gave_up = bool(torch.isnan(out).any())
    rc = lib.mi355_gemm_status()
    assert (rc != 0) == gave_up, "the status word must tell exactly when a tile was given up"
    if gave_up:
        assert b"gave up" in lib.mi355_last_error()
        assert lib.mi355_gemm_status() == 0, "reading the word clears it"
        clean = ~torch.isnan(out)
        assert ev.bit_equal(ref[clean.cpu()], out[clean].cpu()), "tiles that were not given up are exact"
    gemm_knobs.spin_limit(None)
    for _ in range(3):                                          # the same workspace, flags of the give-up run still in it
        out.fill_(5)
        launch()
        assert lib.mi355_gemm_status() == 0 and ev.bit_equal(ref, out.cpu())


def test_split_k_inside_the_launch_gives_up_and_recovers_on_128x128_tiles(gemm_knobs):
    """The same bounded wait on the 128x128-tile kernels' in-launch split (four parts here): with a poll limit of
    0 a summing workgroup whose producers are not done yet writes NaNs and sets the status word; every kernel
    still runs to its end, tiles that were not given up are exact, and later launches on the same workspace -
    late flags of the abandoned tiles still in it - are exact again."""
    print("\n[gpu-case] in-launch split K on 128x128 tiles: give-up path", flush=True)
    sys.stdout.flush()
    lib = _lib.load()
    g = torch.Generator().manual_seed(12)
    M, K, N = 1024, 8192, 2048
    dtype = torch.bfloat16
    code = _lib.dtype_code(dtype)
    gemm_knobs.split("inlaunch")
    need = lib.mi355_gemm_workspace_bytes(M, N, K, code)
    assert need > 0
    a = (torch.randint(-1, 2, (M, K), generator=g) * (torch.randint(0, 8, (M, K), generator=g) == 0)).to(dtype).cuda()
    b = torch.randint(-1, 2, (N, K), generator=g).to(dtype).cuda().t()
    ref = aten_cpu.reference(aten.mm.default, [a.float(), b.float()]).to(dtype)
    ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
    out = torch.empty(M, N, dtype=dtype, device="cuda")

    def launch():
        _lib.check(lib.mi355_gemm(a.data_ptr(), a.stride(0), a.stride(1), b.data_ptr(), b.stride(0), b.stride(1), None, 0, 0,
                                  out.data_ptr(), M, N, K, 1.0, 0.0, code, ws.data_ptr(), need, _lib.current_stream_handle()))
        torch.cuda.synchronize()

    launch()
    assert lib.mi355_gemm_status() == 0 and ev.bit_equal(ref, out.cpu())
    gemm_knobs.spin_limit(0)
    launch()
    gave_up = bool(torch.isnan(out).any())
    rc = lib.mi355_gemm_status()
    assert (rc != 0) == gave_up, "the status word must tell exactly when a tile was given up"
    if gave_up:
        assert b"gave up" in lib.mi355_last_error()
        assert lib.mi355_gemm_status() == 0, "reading the word clears it"
        clean = ~torch.isnan(out)
        assert ev.bit_equal(ref[clean.cpu()], out[clean].cpu()), "tiles that were not given up are exact"
    gemm_knobs.spin_limit(None)
    for _ in range(3):
        out.fill_(5)
        launch()
        assert lib.mi355_gemm_status() == 0 and ev.bit_equal(ref, out.cpu())


def test_set_knob_rejects_unknown_names():
    lib = _lib.load()
    assert lib.mi355_set_knob(b"no_such_knob", b"1") == -1 and b"unknown knob" in lib.mi355_last_error()
    assert lib.mi355_set_knob(b"x16_spin_limit", b"-5") == -1
    assert lib.mi355_set_knob(b"x16_spin_limit", None) == 0
