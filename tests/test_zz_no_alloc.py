"""The entry point that allocates nothing: crl_gemm_static_scratch (K-sliced GEMM whose partial sums live in a fixed
array of the library's device image) against crl_gemm with tile 4 (the same kernels on the per-stream workspace the
library allocates), through the C ABI. Bit-exact, on two calls in a row, the second with a smaller input; then the size
limit's error path."""
import ctypes as C

import pytest
import torch

from chessrl_amd import _lib
from chessrl_amd._lib import check, lib

pytestmark = pytest.mark.gpu

TORCH_DT = {_lib.F32: torch.float32, _lib.BF16: torch.bfloat16, _lib.F16: torch.float16}


def p(t):
    return C.c_void_p(t.data_ptr()) if t is not None else None


def both(A, W, bias, res, out_dt, act, alpha):
    M, K = A.shape
    N = W.shape[0]
    in_dt = {torch.bfloat16: _lib.BF16, torch.float16: _lib.F16, torch.uint8: _lib.FP8}[A.dtype]
    ldc = (N + 7) // 8 * 8
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    outs = []
    for static in (False, True):
        out = torch.full((M, ldc), -7.0, dtype=TORCH_DT[out_dt], device=A.device)
        amax = torch.zeros(1, device=A.device)
        args = [p(A), A.stride(0), p(W), W.stride(0), p(out), ldc, M, N, K, in_dt, out_dt, p(bias), act, 0.5, alpha,
                p(res), res.stride(0) if res is not None else 0, _lib.BF16, 1.0, p(amax)]
        if static:
            check(lib().crl_gemm_static_scratch(*args, st), "crl_gemm_static_scratch")
        else:
            check(lib().crl_gemm(*args, 4, st), "crl_gemm")
        torch.cuda.synchronize()
        outs.append((out, amax))
    return outs


def test_static_scratch_gemm_equals_allocating_gemm(cuda):
    torch.manual_seed(0)
    # two calls in a row on the same scratch array, the second smaller (stale partial sums of the first stay behind it)
    for (M, N, K, dt, out_dt, act) in [(128, 768, 3072, torch.bfloat16, _lib.F32, 1), (37, 250, 1024, torch.bfloat16, _lib.BF16, 0),
                                       (64, 128, 8192, torch.float16, _lib.F16, 2), (100, 1929, 256, torch.uint8, _lib.F32, 0)]:
        if dt == torch.uint8:
            A = (torch.randn(M, K, device=cuda) * 20).to(torch.float8_e4m3fn).view(torch.uint8)
            W = (torch.randn(N, K, device=cuda) * 20).to(torch.float8_e4m3fn).view(torch.uint8)
        else:
            A = torch.randn(M, K, device=cuda).to(dt)
            W = (torch.randn(N, K, device=cuda) * 0.05).to(dt)
        bias = torch.randn(N, device=cuda)
        ldr = (N + 7) // 8 * 8
        res = torch.randn(M, ldr, device=cuda).bfloat16()
        (o1, a1), (o2, a2) = both(A, W, bias, res, out_dt, act, 0.7)
        assert torch.equal(o1, o2), (M, N, K)
        assert torch.equal(a1, a2) and a1.item() > 0
        # and it is the product: against torch on the same operands
        Af = A.view(torch.float8_e4m3fn).float() if dt == torch.uint8 else A.float()
        Wf = W.view(torch.float8_e4m3fn).float() if dt == torch.uint8 else W.float()
        v = 0.5 * (Af @ Wf.t()) + bias
        v = [lambda t: t, torch.nn.functional.gelu, torch.nn.functional.mish][act](v)
        ref = res[:, :N].float() + 0.7 * v
        tol = 2e-2 if out_dt != _lib.F32 else 2e-3
        assert torch.allclose(o2[:, :N].float(), ref, rtol=tol, atol=tol * max(1.0, ref.abs().max().item() / 50)), (o2[:, :N].float() - ref).abs().max()
    # the library allocated nothing through torch, and the size limit is an error, not an overflow
    assert lib().crl_gemm_static_scratch_bytes() == 8 << 20
    A = torch.randn(4096, 8192, device=cuda).bfloat16()        # 2 slices x 4096 x 512 fp32 partial sums = 16 MB
    W = torch.randn(512, 8192, device=cuda).bfloat16()
    out = torch.zeros(4096, 512, device=cuda)
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib().crl_gemm_static_scratch(p(A), 8192, p(W), 8192, p(out), 512, 4096, 512, 8192, _lib.BF16, _lib.F32, None, 0, 1.0, 1.0,
                                       None, 0, _lib.BF16, 1.0, None, st)
    assert rc == -1 and b"fixed scratch array holds" in lib().crl_last_error()
    assert bool((out == 0).all())
    # the largest product that fits (exactly 8 MB of partial sums) runs
    rc = lib().crl_gemm_static_scratch(p(A), 8192, p(W), 8192, p(out), 512, 2048, 512, 8192, _lib.BF16, _lib.F32, None, 0, 1.0, 1.0,
                                       None, 0, _lib.BF16, 1.0, None, st)
    torch.cuda.synchronize()
    assert rc == 0
    ref = A[:2048].float() @ W.float().t()
    assert torch.allclose(out[:2048], ref, rtol=1e-3, atol=0.5)
