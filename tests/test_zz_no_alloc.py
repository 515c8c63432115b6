"""ntg_gemm_noalloc_dev (the entry point that allocates nothing: its split-K partial sums and integer byte planes live
in a fixed array inside the library's device code) against ntg_gemm_dev with a caller-owned workspace, through the C ABI.

Both run the same kernels in the same order, so every result must be bit-identical -- for the floating dtypes too.
Calls follow each other on one stream, a smaller product after a larger one, so stale contents of the shared array
from the previous call would show."""
import ctypes

import numpy as np
import pytest
import torch

from neurotensor_amd import _lib
from neurotensor_amd import functional as F
from util import randn, to_torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


UNSIGNED = {"u16": (np.int16, _lib.UINT16), "u32": (np.int32, _lib.UINT32), "u64": (np.int64, _lib.UINT64)}   # same bit patterns


def _desc(t, m, k, n, ta, tb, mode, batches=1, code=None):
    d = _lib.GemmDesc()
    d.dtype, d.transpose_a, d.transpose_b, d.c_mode = (code if code is not None else F.ntg_dtype(t)), int(ta), int(tb), mode
    d.m, d.k, d.n, d.batches = m, k, n, batches
    if batches > 1:
        d.stride_a, d.stride_b, d.stride_c = m * k, k * n, m * n
    return d


def _operands(rng, dtype, m, k, n, ta, tb, batches=1):
    bf = dtype == "bf16"
    lead = (batches,) if batches > 1 else ()
    if dtype in ("bf16", np.float16, np.float32, np.float64):
        a = randn(rng, lead + ((k, m) if ta else (m, k)), dtype, 0.25)
        b = randn(rng, lead + ((n, k) if tb else (k, n)), dtype, 0.25)
        c0 = randn(rng, lead + (m, n), dtype)
        bias = randn(rng, (n,), dtype)
    else:
        info = np.iinfo(dtype)
        a = rng.integers(info.min, info.max, lead + ((k, m) if ta else (m, k)), dtype=dtype, endpoint=True)
        b = rng.integers(info.min, info.max, lead + ((n, k) if tb else (k, n)), dtype=dtype, endpoint=True)
        c0 = rng.integers(info.min, info.max, lead + (m, n), dtype=dtype, endpoint=True)
        bias = rng.integers(info.min, info.max, (n,), dtype=dtype, endpoint=True)
    return [to_torch(x, DEV, bf) for x in (a, b, c0, bias)]


def _both(lib, rng, dtype, m, k, n, ta, tb, mode, batches=1, expect_workspace=True):
    """Runs one product through both entry points; returns the workspace size the product asks for."""
    npdt, code = UNSIGNED.get(dtype, (dtype, None)) if isinstance(dtype, str) else (dtype, None)
    a, b, c0, bias = _operands(rng, npdt, m, k, n, ta, tb, batches)
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    d = _desc(a, m, k, n, ta, tb, mode, batches, code)
    if mode == _lib.C_BIAS:
        d.bias, d.bias_col_stride = bias.data_ptr(), 1
    need = lib.ntg_gemm_workspace_bytes(ctypes.byref(d))
    assert need <= _lib.NOALLOC_SCRATCH_BYTES, (dtype, m, k, n, need)
    assert (need > 0) == expect_workspace, (dtype, m, k, n, need)
    # the existing entry point, workspace owned by the caller (torch)
    ws = torch.empty(max(need, 256), dtype=torch.uint8, device=DEV)
    want = c0.clone()
    d.workspace, d.workspace_bytes = ws.data_ptr(), need
    _lib.check(lib.ntg_gemm_dev(ctypes.byref(d), a.data_ptr(), b.data_ptr(), want.data_ptr(), st))
    # the entry point under test: descriptor without a workspace
    got = c0.clone()
    d.workspace, d.workspace_bytes = None, 0
    _lib.check(lib.ntg_gemm_noalloc_dev(ctypes.byref(d), a.data_ptr(), b.data_ptr(), got.data_ptr(), st))
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.uint8), want.view(torch.uint8)), (dtype, m, k, n, ta, tb, mode, batches)
    if mode == _lib.C_OVERWRITE:
        assert not torch.equal(got.view(torch.uint8), c0.view(torch.uint8))
    return need


def test_noalloc_entry_point_matches_the_workspace_entry_point():
    lib = _lib.load()
    rng = np.random.default_rng(2718)
    OV, ACC, BIAS = _lib.C_OVERWRITE, _lib.C_ACCUMULATE, _lib.C_BIAS
    # (dtype, m, k, n, ta, tb, mode): each larger product is followed by a smaller one of the same family
    calls = [
        ("bf16", 256, 4096, 2048, False, False, OV), ("bf16", 64, 8192, 512, False, True, ACC),
        (np.float16, 520, 4096, 1032, True, False, BIAS), (np.float16, 128, 2048, 512, False, False, OV),
        (np.float32, 256, 4096, 2048, False, True, ACC), (np.float32, 64, 4096, 256, True, True, OV),
        (np.float64, 256, 4096, 1024, False, False, OV), (np.float64, 64, 2048, 256, False, True, BIAS),
        (np.int16, 640, 520, 712, False, False, ACC), (np.int16, 256, 200, 264, True, False, OV),
        (np.int32, 512, 512, 512, False, True, OV), ("u32", 320, 392, 328, False, False, BIAS),
        (np.int64, 768, 520, 776, True, True, ACC), ("u64", 512, 512, 520, False, False, OV),
    ]
    sizes = []
    for (dtype, m, k, n, ta, tb, mode) in calls:
        sizes.append(_both(lib, rng, dtype, m, k, n, ta, tb, mode))
    assert all(b < a for a, b in zip(sizes[0::2], sizes[1::2])), sizes      # the second call of each pair is the smaller one
    # the first product once more after all the others: same bits as a fresh caller-owned workspace gives
    _both(lib, rng, "bf16", 256, 4096, 2048, False, False, OV)
    # a batch of integer products (planes of every item in the array)
    _both(lib, rng, np.int16, 256, 256, 256, False, False, ACC, batches=3)
    # products that have no workspace form run on the plain kernels
    _both(lib, rng, np.float32, 512, 512, 512, False, False, ACC, expect_workspace=False)
    _both(lib, rng, "bf16", 100, 72, 48, False, True, OV, expect_workspace=False)


def test_noalloc_entry_point_rejects_what_does_not_fit():
    lib = _lib.load()
    # Int32 batch 8 x 1024^3 as byte planes needs 192 MiB
    a = torch.zeros((8, 1024, 1024), dtype=torch.int32, device=DEV)
    c = torch.zeros((8, 1024, 1024), dtype=torch.int32, device=DEV)
    d = _desc(a, 1024, 1024, 1024, False, False, _lib.C_ACCUMULATE, 8)
    need = lib.ntg_gemm_workspace_bytes(ctypes.byref(d))
    assert need > _lib.NOALLOC_SCRATCH_BYTES
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.ntg_gemm_noalloc_dev(ctypes.byref(d), a.data_ptr(), a.data_ptr(), c.data_ptr(), st)
    assert rc == 1
    msg = lib.ntg_last_error().decode()
    assert str(need) in msg and str(_lib.NOALLOC_SCRATCH_BYTES) in msg, msg
    torch.cuda.synchronize()
    assert int(c.abs().max()) == 0                                            # nothing was launched
    # argument errors as in ntg_gemm_dev
    assert lib.ntg_gemm_noalloc_dev(ctypes.byref(d), None, a.data_ptr(), c.data_ptr(), st) == 1
    d.stride_c = 0
    assert lib.ntg_gemm_noalloc_dev(ctypes.byref(d), a.data_ptr(), a.data_ptr(), c.data_ptr(), st) == 1
