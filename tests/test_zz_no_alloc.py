"""The entry point that allocates nothing (csrc/no_alloc.h), called through ctypes as a caller
without this package would: the product cut along K with its partial products in the library's
own fixed array. Checked against the existing entry points (mllm_gemm_split + mllm_pending_sum bit
for bit, mllm_gemm and float64 within rounding) on two calls in a row, the second with a smaller
input (the array then still holds the first call's partial products beyond what the second
writes), and for its refusals. torch only brings the inputs' and outputs' memory."""

import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

F32, BF16 = 0, 1
P = ctypes.c_void_p


@pytest.fixture(scope="module")
def lib():
    from mini_llm_amd.csrc import build

    lib = ctypes.CDLL(str(build.ensure_built()))
    lib.mllm_linear_split_static.argtypes = [P, P, ctypes.c_int, P, P, P] + [ctypes.c_int] * 5 + [P]
    lib.mllm_linear_split_static.restype = ctypes.c_int
    lib.mllm_gemm_split.argtypes = [P, P, ctypes.c_int, P] + [ctypes.c_int] * 6 + [P]
    lib.mllm_gemm_split.restype = ctypes.c_int
    lib.mllm_pending_sum.argtypes = [P, P, P, ctypes.c_int, P, ctypes.c_int, ctypes.c_int, P]
    lib.mllm_pending_sum.restype = ctypes.c_int
    lib.mllm_gemm.argtypes = [P, P, ctypes.c_int, P, P, P] + [ctypes.c_int] * 8 + [P]
    lib.mllm_gemm.restype = ctypes.c_int
    lib.mllm_static_scratch_bytes.restype = ctypes.c_longlong
    lib.mllm_static_scratch_prepare.restype = ctypes.c_int
    lib.mllm_last_error.restype = ctypes.c_char_p
    return lib


def operands(seed, m, n, k, dtype):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((m, k), generator=g).to(dtype).cuda()
    w = (torch.randn((n, k), generator=g) * 0.1).to(dtype).cuda()
    bias = torch.randn((n,), generator=g).cuda()
    residual = torch.randn((m, n), generator=g).cuda()
    return x, w, bias, residual


def existing(lib, x, w, bias, residual, k_blocks, code):
    """The same product through the entry points that take their scratch memory from the caller."""
    m, k = x.shape
    n = w.shape[0]
    partials = torch.empty((k_blocks, m, n), dtype=torch.float32, device="cuda")
    assert lib.mllm_gemm_split(x.data_ptr(), w.data_ptr(), 0, partials.data_ptr(), m, n, k, code, k_blocks, 0, None) == 0, lib.mllm_last_error()
    out = torch.empty((m, n), dtype=torch.float32, device="cuda")
    assert lib.mllm_pending_sum(residual.data_ptr(), partials.data_ptr(), bias.data_ptr(), k_blocks, out.data_ptr(), m, n, None) == 0, lib.mllm_last_error()
    whole = torch.empty((m, n), dtype=torch.float32, device="cuda")
    assert lib.mllm_gemm(x.data_ptr(), w.data_ptr(), 0, bias.data_ptr(), residual.data_ptr(), whole.data_ptr(), m, n, k, code, F32, 0, 0, 0, None) == 0, lib.mllm_last_error()
    torch.cuda.synchronize()
    return out.cpu().numpy(), whole.cpu().numpy()


@pytest.mark.parametrize("dtype,code", [(torch.bfloat16, BF16), (torch.float32, F32)])
def test_two_calls_in_a_row_the_second_smaller(lib, dtype, code):
    assert lib.mllm_static_scratch_bytes() == 4 << 20
    assert lib.mllm_static_scratch_prepare() == 0, lib.mllm_last_error()
    # (rows, columns, K, partial products): few rows (the kernel for few rows), then fewer rows and
    # columns and fewer partial products; then many rows (the tiled kernel), then fewer again
    for calls in (((48, 776, 3072, 8), (5, 200, 1024, 4)), ((300, 320, 2048, 4), (130, 96, 512, 2))):
        for call, (m, n, k, k_blocks) in enumerate(calls):
            x, w, bias, residual = operands(10 * call + m, m, n, k, dtype)
            out = torch.full((m + 1, n), float("nan"), dtype=torch.float32, device="cuda")   # a guard row behind the output
            status = lib.mllm_linear_split_static(x.data_ptr(), w.data_ptr(), 0, bias.data_ptr(), residual.data_ptr(), out.data_ptr(),
                                                  m, n, k, code, k_blocks, None)
            assert status == 0, lib.mllm_last_error()
            torch.cuda.synchronize()
            got = out.cpu().numpy()
            assert np.isnan(got[m]).all(), "the call wrote beyond its output"
            split, whole = existing(lib, x, w, bias, residual, k_blocks, code)
            np.testing.assert_array_equal(got[:m], split)                     # the same kernels, the same order of sums
            exact = x.double().cpu().numpy() @ w.double().cpu().numpy().T + bias.cpu().numpy() + residual.cpu().numpy()
            np.testing.assert_allclose(got[:m], exact, rtol=2e-5, atol=2e-4)
            np.testing.assert_allclose(got[:m], whole, rtol=2e-5, atol=2e-4)  # the product left whole
    # without bias and residual
    x, w, _, _ = operands(3, 7, 64, 256, dtype)
    out = torch.empty((7, 64), dtype=torch.float32, device="cuda")
    assert lib.mllm_linear_split_static(x.data_ptr(), w.data_ptr(), 0, None, None, out.data_ptr(), 7, 64, 256, code, 2, None) == 0, lib.mllm_last_error()
    torch.cuda.synchronize()
    np.testing.assert_allclose(out.cpu().numpy(), x.double().cpu().numpy() @ w.double().cpu().numpy().T, rtol=2e-5, atol=2e-4)


def test_what_does_not_fit_is_refused(lib):
    x, w, bias, residual = operands(1, 4, 64, 64, torch.float32)
    out = torch.zeros((4, 64), dtype=torch.float32, device="cuda")
    args = (x.data_ptr(), w.data_ptr(), 0, bias.data_ptr(), residual.data_ptr(), out.data_ptr())
    # 16 x 1024 x 128 floats are 8 MiB: beyond the array (no kernel runs: the operands here are far smaller)
    assert lib.mllm_linear_split_static(*args, 1024, 128, 64, F32, 16, None) != 0
    assert b"do not fit" in lib.mllm_last_error()
    assert lib.mllm_linear_split_static(*args, 4, 64, 64, F32, 17, None) != 0 and b"1..16" in lib.mllm_last_error()
    assert lib.mllm_linear_split_static(*args, 4, 64, 62, F32, 2, None) != 0          # K is no whole number of 16-byte pieces
    assert lib.mllm_linear_split_static(None, w.data_ptr(), 0, None, None, out.data_ptr(), 4, 64, 64, F32, 2, None) != 0
    torch.cuda.synchronize()
    assert (out == 0).all()
