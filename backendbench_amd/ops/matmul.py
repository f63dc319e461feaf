"""mm / addmm on the bf16/f16/f32 MFMA kernels (fp32 accumulate) with a generic fallback."""

import torch

from .. import _lib
from ._common import cast, copy_into, dense, device_managed, launch, new_dense, new_result

_GEMM_DTYPES = (torch.bfloat16, torch.float16, torch.float32, torch.float64)
_SPLITK_MAX_OUT = 256 * 256 * 128 + 1  # the planner never splits problems with more than 128 tiles of 256x256
_ws_fn = None


def _workspace_bytes():
    global _ws_fn
    if _ws_fn is None:
        _ws_fn = _lib.load().mi355_gemm_workspace_bytes
    return _ws_fn


def _gemm(a, b, c, alpha, beta):
    if a.dim() != 2 or b.dim() != 2:
        raise RuntimeError(f"mat1 and mat2 must be matrices, got {a.dim()}-D and {b.dim()}-D tensors")
    if a.shape[1] != b.shape[0]:
        raise RuntimeError(f"mat1 and mat2 shapes cannot be multiplied ({a.shape[0]}x{a.shape[1]} and "
                           f"{b.shape[0]}x{b.shape[1]})")
    if a.dtype != b.dtype:
        raise RuntimeError(f"expected m1 and m2 to have the same dtype, but got: {a.dtype} != {b.dtype}")
    if a.dtype not in _GEMM_DTYPES:
        raise NotImplementedError(f"mi355 backend: matmul on {a.dtype} is not supported")
    M, K = a.shape
    N = b.shape[1]
    out = new_result((M, N), a.dtype, a.device)
    if M == 0 or N == 0:
        return out
    if c is not None:
        if c.dtype != a.dtype:
            raise RuntimeError(f"self and mat2 must have the same dtype, but got {c.dtype} and {a.dtype}")
        c = c.expand(M, N)  # raises like ATen when self cannot broadcast to [M, N]
        c_ptr, c_rs, c_cs = c.data_ptr(), c.stride(0), c.stride(1)
    else:
        c_ptr, c_rs, c_cs = None, 0, 0
    code = _lib.dtype_code(a.dtype)
    # The MFMA kernels want K-contiguous rows of A and a row-major or K-contiguous B.  Any other
    # layout (a transposed left operand, sliced views) is densified once with the copy kernel: one
    # pass over the operand, instead of the whole product on the FMA fallback.
    if M * N >= 64 * 64 and K >= 16 and a.dtype != torch.float64:
        V = 16 // a.element_size()
        if K % V:
            # rows of K elements would not start on 16-byte boundaries: both operands are copied
            # once into K-contiguous buffers padded with zeros to a multiple of 64 (exact: the pad
            # adds 0 * 0 terms), instead of running the whole product on the FMA fallback
            Kp = (K + 63) // 64 * 64
            both = torch.zeros((M + N, Kp), dtype=a.dtype, device=a.device)  # one fill for both operands
            ap, btp = both[:M], both[M:]
            copy_into(ap[:, :K], a)
            copy_into(btp[:, :K], b.t())
            a, b, K = ap, btp.t(), Kp
        elif b.stride(1) == 1 and N > 1 and (N % V or b.stride(0) % V or b.data_ptr() % 16):
            # a row-major right operand whose rows are misaligned (N = 1001): its transpose is
            # K-contiguous, which the kernels take for any N
            b = dense(b.t()).t()
        if a.stride(1) != 1 and M > 1 and K > 1:
            # a transposed left operand (x.t() @ dy) goes in as it is when the MFMA kernels take it
            direct = (a.stride(0) == 1 and a.element_size() == 2 and K % 64 == 0 and M % 8 == 0
                      and a.stride(1) % 8 == 0 and a.data_ptr() % 16 == 0 and M * N >= 128 * 128)
            if not direct:
                a = dense(a)
        if b.stride(1) != 1 and b.stride(0) != 1 and K > 1 and N > 1:
            b = dense(b)
    ws, ws_bytes = None, 0
    if M * N < _SPLITK_MAX_OUT:  # only skinny / small outputs are ever split along K
        ws_bytes = _workspace_bytes()(M, N, K, code)
        if ws_bytes:
            ws = new_dense((ws_bytes,), torch.uint8, a.device)
    launch("mi355_gemm", a.data_ptr(), a.stride(0), a.stride(1), b.data_ptr(), b.stride(0), b.stride(1), c_ptr,
           c_rs, c_cs, out.data_ptr(), M, N, K, float(alpha), float(beta), code,
           ws.data_ptr() if ws is not None else None, ws_bytes)
    return out


_HALF = (torch.bfloat16, torch.float16)
_UNSUPPORTED = -2  # MI355_ERR_UNSUPPORTED
_f32out_fn = None


def _check_out_dtype(a, out_dtype):
    """ATen's rule for the .dtype overloads: the operands' own dtype, or fp32 for f16 / bf16 operands."""
    if not (out_dtype == a.dtype or (out_dtype == torch.float32 and a.dtype in _HALF)):
        raise RuntimeError("out_dtype must be the same as input dtype or fp32 for fp16/bf16 inputs")


def _gemm_f32out(a, b, c, alpha, beta):
    """bf16 / f16 operands, fp32 result (mm.dtype / addmm.dtype with out_dtype=float32): the MFMA kernels
    store their fp32 accumulators unrounded (mi355_gemm_f32out).  Layouts that entry point does not take
    (odd K or N, misaligned views) run as an fp32 product of the widened operands instead: the products of
    two bf16 / f16 values are exact in fp32, so both paths add up the same terms in fp32."""
    global _f32out_fn
    if a.dim() != 2 or b.dim() != 2:
        raise RuntimeError(f"mat1 and mat2 must be matrices, got {a.dim()}-D and {b.dim()}-D tensors")
    if a.shape[1] != b.shape[0]:
        raise RuntimeError(f"mat1 and mat2 shapes cannot be multiplied ({a.shape[0]}x{a.shape[1]} and "
                           f"{b.shape[0]}x{b.shape[1]})")
    if a.dtype != b.dtype:
        raise RuntimeError(f"expected m1 and m2 to have the same dtype, but got: {a.dtype} != {b.dtype}")
    M, K = a.shape
    N = b.shape[1]
    if c is not None:
        if c.dtype != a.dtype:
            raise RuntimeError(f"self and mat2 must have the same dtype, but got {c.dtype} and {a.dtype}")
        c = c.expand(M, N)
    if M and N and K:
        if a.stride(1) != 1:
            a = dense(a)
        if b.stride(1) != 1 and b.stride(0) != 1:
            b = dense(b)
        out = new_result((M, N), torch.float32, a.device)
        if _f32out_fn is None:
            _f32out_fn = _lib.load().mi355_gemm_f32out
        c_args = (c.data_ptr(), c.stride(0), c.stride(1)) if c is not None else (None, 0, 0)
        rc = _f32out_fn(a.data_ptr(), a.stride(0), a.stride(1), b.data_ptr(), b.stride(0), b.stride(1), *c_args,
                        out.data_ptr(), M, N, K, float(alpha), float(beta), _lib.dtype_code(a.dtype),
                        _lib.current_stream_handle())
        if rc == 0:
            return out
        if rc != _UNSUPPORTED:
            _lib.check(rc)
    wide_c = cast(c, torch.float32) if c is not None else None
    return _gemm(cast(a, torch.float32), cast(b, torch.float32), wide_c, alpha, beta)


@device_managed
def mm_dtype(self, mat2, out_dtype):
    """aten.mm.dtype: mm with the result in `out_dtype` (fp32 from bf16 / f16 operands, or the operands' dtype)."""
    _check_out_dtype(self, out_dtype)
    if out_dtype == self.dtype:
        return _gemm(self, mat2, None, 1.0, 0.0)
    return _gemm_f32out(self, mat2, None, 1.0, 0.0)


@device_managed
def addmm_dtype(self, mat1, mat2, out_dtype, *, beta=1, alpha=1):
    """aten.addmm.dtype: beta * self + alpha * (mat1 @ mat2) in `out_dtype`; self has the operands' dtype."""
    _check_out_dtype(mat1, out_dtype)
    if out_dtype == mat1.dtype:
        return _gemm(mat1, mat2, self, alpha, beta)
    return _gemm_f32out(mat1, mat2, self, alpha, beta)


@device_managed
def mm(self, mat2):
    """aten.mm.default"""
    return _gemm(self, mat2, None, 1.0, 0.0)


@device_managed
def addmm(self, mat1, mat2, *, beta=1, alpha=1):
    """aten.addmm.default: beta * self + alpha * (mat1 @ mat2); beta == 0 never reads self."""
    return _gemm(mat1, mat2, self, alpha, beta)
