"""ntg_gemm_relu_dev = ntg_gemm_dev followed by the reference's relu_ (clamp_(x, 0): activation_functions.cpp:141-143,
min_max.cpp:45-63, :115-121 -- max(x, 0) that returns 0 for NaN and for -0).  The clamp commutes with the one rounding of
the result, so whatever kernel serves the product -- epilogue of the DMA-fed kernels, split-K reduction, or a second pass
over C behind the streaming / register-staged / padded forms -- the bits must be those of clamping what ntg_gemm_dev
stores.  The expected values are built that way, from ntg_gemm_dev itself (checked against the oracle elsewhere)."""
import ctypes

import numpy as np
import pytest
import torch

from neurotensor_amd import _lib
from neurotensor_amd import functional as F

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32, "f64": torch.float64}
TRANS = [(False, False), (False, True), (True, False), (True, True)]


def setup_module(module):
    assert torch.cuda.is_available(), "GPU tests need a visible MI355X"
    _lib.load()


def bits(t):
    return t.contiguous().view({2: torch.int16, 4: torch.int32, 8: torch.int64}[t.element_size()])


def clamp0(t):
    """relu_ of the reference: x > 0 ? x : +0 (NaN and -0 give +0)."""
    return torch.where(t > 0, t, torch.zeros_like(t))


def run_pair(lib, st, dt, m, k, n, ta, tb, mode, batch=1, ldc=None, workspace=False, poison=False):
    gen = torch.Generator(device=DEV).manual_seed(1000 * m + 10 * k + n + 7 * batch)
    mk = lambda *shape: (torch.randn(*shape, device=DEV, generator=gen) * 0.5).to(dt)
    a = mk(batch, k, m) if ta else mk(batch, m, k)
    b = mk(batch, n, k) if tb else mk(batch, k, n)
    ldc = ldc or n
    c0 = mk(batch, m, ldc)
    bias = mk(n)
    if poison:
        bias[0] = float("nan")          # a NaN column: relu_ gives 0
        bias[1] = -0.0
        a[:, :, :] = 0 if poison == "zero" else a       # with zero products, column 1 is -0 + 0 ... exactly the bias
    d = _lib.GemmDesc()
    d.dtype, d.transpose_a, d.transpose_b, d.c_mode = F.ntg_dtype(a), int(ta), int(tb), mode
    d.m, d.k, d.n, d.batches, d.ldc = m, k, n, batch, ldc
    d.stride_a, d.stride_b, d.stride_c = m * k, k * n, m * ldc
    if mode == _lib.C_BIAS:
        d.bias, d.bias_col_stride = bias.data_ptr(), 1
    ws = None
    if workspace:
        need = lib.ntg_gemm_workspace_bytes(ctypes.byref(d))
        assert need > 0, (m, k, n)
        ws = torch.empty(need, dtype=torch.uint8, device=DEV)
        d.workspace, d.workspace_bytes = ws.data_ptr(), need
    plain, fused = c0.clone(), c0.clone()
    _lib.check(lib.ntg_gemm_dev(ctypes.byref(d), a.data_ptr(), b.data_ptr(), plain.data_ptr(), st))
    _lib.check(lib.ntg_gemm_relu_dev(ctypes.byref(d), a.data_ptr(), b.data_ptr(), fused.data_ptr(), st))
    torch.cuda.synchronize()
    want = plain.clone()
    want[:, :, :n] = clamp0(plain[:, :, :n])
    assert torch.equal(bits(fused), bits(want)), (dt, m, k, n, ta, tb, mode, batch, ldc, workspace)
    assert bool((fused[:, :, :n] >= 0).all()) and float((fused[:, :, :n] > 0).double().mean()) > 0.2
    return fused


@pytest.mark.parametrize("name", list(DTYPES))
def test_relu_epilogue_equals_clamped_product(name):
    dt = DTYPES[name]
    lib = _lib.load()
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    modes = (_lib.C_OVERWRITE, _lib.C_ACCUMULATE, _lib.C_BIAS)
    i = 0
    # DMA-fed kernels (aligned rows, ragged tiles), register-staged kernels (odd sizes), streaming kernels (few rows)
    for (m, k, n) in [(200, 256, 264), (129, 203, 205), (8, 512, 384), (33, 64, 72), (256, 96, 1024)]:
        for ta, tb in TRANS:
            run_pair(lib, st, dt, m, k, n, ta, tb, modes[i % 3])
            i += 1
    # batches, padded rows of C (the padding keeps its contents)
    run_pair(lib, st, dt, 96, 128, 80, False, False, _lib.C_BIAS, batch=5, ldc=88)
    run_pair(lib, st, dt, 70, 45, 50, False, True, _lib.C_ACCUMULATE, batch=3, ldc=54)
    # NaN and -0: both become +0
    out = run_pair(lib, st, dt, 64, 32, 64, False, False, _lib.C_BIAS, poison="zero")
    assert bool((bits(out[:, :, :2]) == 0).all())
    out = run_pair(lib, st, dt, 7, 32, 64, False, False, _lib.C_BIAS, poison="zero")        # streaming kernel + second pass
    assert bool((bits(out[:, :, :2]) == 0).all())


@pytest.mark.parametrize("name", list(DTYPES))
def test_relu_epilogue_with_workspace_forms(name):
    """split along k (the reduction clamps) and, for the 16-bit types, padded copies of operands with odd rows"""
    dt = DTYPES[name]
    lib = _lib.load()
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    shapes = [(256, 4096, 2048), (64, 8192, 1024)] if dt in (torch.float16, torch.bfloat16) else [(256, 1024, 256)]
    for (m, k, n) in shapes:
        for mode in (_lib.C_OVERWRITE, _lib.C_BIAS, _lib.C_ACCUMULATE):
            run_pair(lib, st, dt, m, k, n, False, False, mode, workspace=True)
    if dt in (torch.float16, torch.bfloat16):
        run_pair(lib, st, dt, 2048, 1001, 2048, False, False, _lib.C_BIAS, workspace=True)
        run_pair(lib, st, dt, 2048, 1024, 2044, False, True, _lib.C_ACCUMULATE, workspace=True)


def test_relu_epilogue_argument_errors():
    lib = _lib.load()
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    x = torch.zeros(16, 16, dtype=torch.int32, device=DEV)
    d = _lib.GemmDesc()
    d.dtype, d.m, d.k, d.n, d.batches = _lib.INT32, 16, 16, 16, 1
    assert lib.ntg_gemm_relu_dev(ctypes.byref(d), x.data_ptr(), x.data_ptr(), x.data_ptr(), st) == 2      # unsupported dtype
    assert b"Float16" in lib.ntg_last_error()
    d.dtype = _lib.COMPLEX64
    assert lib.ntg_gemm_relu_dev(ctypes.byref(d), x.data_ptr(), x.data_ptr(), x.data_ptr(), st) == 2
    d.dtype = _lib.FLOAT32
    assert lib.ntg_gemm_relu_dev(ctypes.byref(d), None, x.data_ptr(), x.data_ptr(), st) == 1
