"""ntg_gemm_noalloc_dev (the entry point that allocates nothing: its split-K partial sums, integer byte planes and padded
copies live in a fixed array inside the library's device code) against ntg_gemm_dev with a caller-owned workspace, through the C ABI.

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
    # padded copies (rows that are not 16-byte multiples: A, B and C copied into the array, the bias written as the padded
    # C's starting value, the result copied back), a larger product before a smaller one, then the 8-bit form
    big = _both(lib, rng, "bf16", 2048, 1001, 2044, False, False, BIAS)
    small = _both(lib, rng, "bf16", 1032, 2001, 1048, False, True, ACC)
    assert small < big, (small, big)
    _both(lib, rng, np.float16, 2048, 1001, 2044, True, False, ACC)
    _both(lib, rng, np.int8, 520, 1001, 530, False, False, ACC)
    # a batch whose items are split along k (the partial sums of every item and k range in the array)
    _both(lib, rng, "bf16", 256, 4096, 512, False, False, ACC, batches=3)
    _both(lib, rng, np.float32, 64, 4096, 256, False, True, BIAS, batches=5)
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
    assert "ntg_gemm_dev" in msg and "without a workspace" in msg, msg         # (the message names the allocation-free fallback)
    torch.cuda.synchronize()
    assert int(c.abs().max()) == 0                                            # nothing was launched
    # argument errors as in ntg_gemm_dev
    assert lib.ntg_gemm_noalloc_dev(ctypes.byref(d), None, a.data_ptr(), c.data_ptr(), st) == 1
    d.stride_c = 0
    assert lib.ntg_gemm_noalloc_dev(ctypes.byref(d), a.data_ptr(), a.data_ptr(), c.data_ptr(), st) == 1


def test_noalloc_calls_on_two_streams_are_ordered_by_the_library():
    """Two streams use the one array without any synchronisation by the caller: a long split product on one stream, a short
    one on the other right behind it, several rounds.  The library orders them (an event behind each user's last kernel),
    so both results are those of caller-owned workspaces."""
    lib = _lib.load()
    rng = np.random.default_rng(99)
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    a1, b1, c1, _ = _operands(rng, "bf16", 256, 8192, 2048, False, False)
    a2, b2, c2, _ = _operands(rng, "bf16", 64, 4096, 512, False, True)
    d1 = _desc(a1, 256, 8192, 2048, False, False, _lib.C_OVERWRITE)
    d2 = _desc(a2, 64, 4096, 512, False, True, _lib.C_OVERWRITE)
    want = []
    for (d, a, b, c) in ((d1, a1, b1, c1), (d2, a2, b2, c2)):
        need = lib.ntg_gemm_workspace_bytes(ctypes.byref(d))
        assert 0 < need <= _lib.NOALLOC_SCRATCH_BYTES
        ws = torch.empty(need, dtype=torch.uint8, device=DEV)
        w = torch.empty_like(c)
        d.workspace, d.workspace_bytes = ws.data_ptr(), need
        _lib.check(lib.ntg_gemm_dev(ctypes.byref(d), a.data_ptr(), b.data_ptr(), w.data_ptr(), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
        d.workspace, d.workspace_bytes = None, 0
        want.append(w)
    torch.cuda.synchronize()
    for rnd in range(6):
        g1, g2 = torch.zeros_like(c1), torch.zeros_like(c2)
        torch.cuda.synchronize()
        _lib.check(lib.ntg_gemm_noalloc_dev(ctypes.byref(d1), a1.data_ptr(), b1.data_ptr(), g1.data_ptr(), ctypes.c_void_p(s1.cuda_stream)))
        _lib.check(lib.ntg_gemm_noalloc_dev(ctypes.byref(d2), a2.data_ptr(), b2.data_ptr(), g2.data_ptr(), ctypes.c_void_p(s2.cuda_stream)))
        _lib.check(lib.ntg_gemm_noalloc_dev(ctypes.byref(d1), a1.data_ptr(), b1.data_ptr(), g1.data_ptr(), ctypes.c_void_p(s1.cuda_stream)))
        torch.cuda.synchronize()
        assert torch.equal(g1.view(torch.int16), want[0].view(torch.int16)), rnd
        assert torch.equal(g2.view(torch.int16), want[1].view(torch.int16)), rnd
