"""GPU parity of the matmult path against the CPU oracle, through the C ABI.

Integer dtypes must be bit-exact; fp32/fp64 within max|d| <= 1e-5*K*max|A|*max|B|;
fp16/bf16 within 2e-2 of max|C_ref| (fp32 accumulate on the GPU; the fp16 oracle rounds
to half every 16 k like the reference's AVX2 build, the bf16 oracle is this build's own
definition -- "parity unpinned" by the reference, which has no BFloat16 DType).
"""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from neurotensor_amd import _lib
from neurotensor_amd import functional as F
from util import HALF_REL, float_tol, from_torch, randn, to_f64, to_torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
TRANS = [(False, False), (False, True), (True, False), (True, True)]
FLOATS = [np.float32, np.float64, np.float16, "bf16"]
INTS = [np.int8, np.int16, np.int32, np.int64, np.uint8, np.uint16, np.uint32, np.uint64]


def setup_module(module):
    assert torch.cuda.is_available(), "GPU tests need a visible MI355X"
    _lib.load()


def code_of(dtype):
    return oracle.BF16 if dtype == "bf16" else oracle._NP_TO_DT[np.dtype(dtype)]


def make_inputs(rng, m, k, n, dtype, ta, tb, scale=1.0, int_range=None):
    if dtype in FLOATS or dtype == "bf16":
        a = randn(rng, (m, k), dtype, scale)
        b = randn(rng, (k, n), dtype, scale)
        c0 = randn(rng, (m, n), dtype, scale)
    else:
        info = np.iinfo(dtype)
        lo, hi = int_range if int_range else (info.min, info.max)
        a = rng.integers(lo, hi, (m, k), dtype=dtype, endpoint=True)
        b = rng.integers(lo, hi, (k, n), dtype=dtype, endpoint=True)
        c0 = rng.integers(lo, hi, (m, n), dtype=dtype, endpoint=True)
    sa = np.ascontiguousarray(a.T) if ta else a
    sb = np.ascontiguousarray(b.T) if tb else b
    return a, b, sa, sb, c0


def assert_close(got, ref, a, b, k, dtype, what=""):
    bf = dtype == "bf16"
    if dtype in (np.float32, np.float64):
        tol = float_tol(k, a, b)
        err = np.abs(got.astype(np.float64) - ref.astype(np.float64)).max(initial=0.0)
        assert err <= tol, f"{what}: max|d|={err} > {tol}"
    elif dtype in (np.float16, "bf16"):
        g, r = to_f64(got, bf), to_f64(ref, bf)
        scale = max(np.abs(r).max(initial=0.0), 1e-30)
        err = np.abs(g - r).max(initial=0.0) / scale
        assert err <= HALF_REL, f"{what}: rel err {err} > {HALF_REL}"
    else:
        assert got.tobytes() == ref.tobytes(), f"{what}: integer result not bit-exact"


def host_matmult(sa, sb, c, m, k, n, ta, tb, dt):
    lib = _lib.load()
    p = lambda x: x.ctypes.data_as(ctypes.c_void_p)
    _lib.check(lib.ntg_matmult(dt, p(sa), p(sb), p(c), m, k, k, n, int(ta), int(tb)))
    return c


def dev_matmult(sa, sb, c0, m, k, n, ta, tb, dtype, mode=_lib.C_ACCUMULATE, flags=0):
    bf = dtype == "bf16"
    ta_, tb_ = to_torch(sa, DEV, bf), to_torch(sb, DEV, bf)
    tc = to_torch(c0.copy(), DEV, bf)
    lib = _lib.load()
    d = _lib.GemmDesc()
    d.dtype = code_of(dtype)
    d.transpose_a, d.transpose_b, d.c_mode = int(ta), int(tb), mode
    d.m, d.k, d.n, d.batches = m, k, n, 1
    d.flags = flags
    _lib.check(lib.ntg_gemm_dev(ctypes.byref(d), ta_.data_ptr(), tb_.data_ptr(), tc.data_ptr(),
                                ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
    torch.cuda.synchronize()
    return from_torch(tc)


@pytest.mark.parametrize("dtype", FLOATS + INTS, ids=lambda d: d if isinstance(d, str) else np.dtype(d).name)
@pytest.mark.parametrize("ta,tb", TRANS)
def test_host_entry_point_every_dtype(dtype, ta, tb):
    """ntg_matmult == nt_matmult<T>: host pointers, C += op(A).op(B), ragged sizes."""
    rng = np.random.default_rng(100)
    m, k, n = 37, 53, 29
    a, b, sa, sb, c0 = make_inputs(rng, m, k, n, dtype, ta, tb)
    dt = code_of(dtype)
    ref = oracle.matmult2d(sa, sb, c0.copy(), ta, tb, dt=dt)
    got = host_matmult(sa, sb, c0.copy(), m, k, n, ta, tb, dt)
    af = to_f64(a, dtype == "bf16") if dtype in FLOATS else a
    bfm = to_f64(b, dtype == "bf16") if dtype in FLOATS else b
    assert_close(got, ref, af, bfm, k, dtype, f"host {dtype} ta={ta} tb={tb}")


SHAPES = [(1, 1, 1), (1, 64, 1), (5, 1, 7), (33, 70, 65), (64, 64, 64), (128, 128, 128), (129, 131, 127),
          (256, 64, 256), (300, 200, 500), (17, 1000, 19), (512, 96, 384), (100, 333, 40)]


@pytest.mark.parametrize("dtype", FLOATS, ids=lambda d: d if isinstance(d, str) else np.dtype(d).name)
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_device_entry_point_shapes(dtype, shape):
    """Edge and ragged sizes on device buffers, all four flag pairs, accumulate into C0 != 0."""
    m, k, n = shape
    rng = np.random.default_rng(200 + m + k + n)
    for ta, tb in TRANS:
        a, b, sa, sb, c0 = make_inputs(rng, m, k, n, dtype, ta, tb)
        ref = oracle.matmult2d(sa, sb, c0.copy(), ta, tb, dt=code_of(dtype))
        got = dev_matmult(sa, sb, c0, m, k, n, ta, tb, dtype)
        bf = dtype == "bf16"
        assert_close(got, ref, to_f64(a, bf), to_f64(b, bf), k, dtype, f"dev {dtype} {shape} ta={ta} tb={tb}")


@pytest.mark.parametrize("dtype", [np.int32, np.int64, np.int8, np.int16])
@pytest.mark.parametrize("shape", [(1, 1, 1), (65, 130, 67), (128, 64, 128), (200, 17, 3)])
def test_device_integers_bit_exact(dtype, shape):
    m, k, n = shape
    rng = np.random.default_rng(300 + m)
    for ta, tb in TRANS:
        a, b, sa, sb, c0 = make_inputs(rng, m, k, n, dtype, ta, tb)
        ref = oracle.matmult2d(sa, sb, c0.copy(), ta, tb)
        got = dev_matmult(sa, sb, c0, m, k, n, ta, tb, dtype)
        assert got.tobytes() == ref.tobytes()


@pytest.mark.parametrize("dtype", [np.int8, np.uint8], ids=["int8", "uint8"])
@pytest.mark.parametrize("shape", [(128, 64, 128), (256, 192, 256), (272, 80, 144), (1040, 528, 2064), (4096, 1024, 4096), (48, 16, 16),
                                   (3056, 528, 4080), (2032, 1040, 4080)],
                         ids=lambda s: "x".join(map(str, s)))
def test_int8_matrix_pipe_bit_exact(dtype, shape):
    """Int8 / UInt8 with 16-byte rows (sizes multiples of 16) run on v_mfma_i32_32x32x32_i8: every result byte must equal the
    reference's wrapping arithmetic over the full value range, in all four transpose forms (both LDS layouts, the
    transposing 8-bit reads), on 64-, 128- and 256-wide tiles and the 192 x 256 (3056 x 4080, A stored [m][k]) and 128 x 256
    (2032 x 4080) ones, ragged edges and k tails, all three C modes, batches; and
    must equal the vector-ALU kernel (the same product with rows that are not 16-byte multiples takes that path)."""
    m, k, n = shape
    rng = np.random.default_rng(3100 + m)

    def exact(x, y):      # |sum| < 2^27: exact in float64, and BLAS-fast (numpy has no fast integer matmul)
        return (x.astype(np.float64) @ y.astype(np.float64)).astype(np.int64)

    info = np.iinfo(dtype)
    big = m >= 4096
    for ta, tb in TRANS:
        a = rng.integers(info.min, info.max, (m, k), dtype=dtype, endpoint=True)
        b = rng.integers(info.min, info.max, (k, n), dtype=dtype, endpoint=True)
        c0 = rng.integers(info.min, info.max, (m, n), dtype=dtype, endpoint=True)
        sa = np.ascontiguousarray(a.T) if ta else a
        sb = np.ascontiguousarray(b.T) if tb else b
        # exact reference, then wrap to 8 bits
        ref = (exact(a, b) + c0.astype(np.int64)).astype(dtype)
        got = dev_matmult(sa, sb, c0, m, k, n, ta, tb, dtype)
        assert got.tobytes() == ref.tobytes(), (shape, ta, tb)
        if m < 2000:
            assert oracle.matmult2d(sa, sb, c0.copy(), ta, tb).tobytes() == ref.tobytes()
        got0 = dev_matmult(sa, sb, c0, m, k, n, ta, tb, dtype, mode=_lib.C_OVERWRITE)
        assert got0.tobytes() == (exact(a, b)).astype(dtype).tobytes()
        if big:
            break
    # bias mode and a batch with a broadcast operand, through the dispatcher mirror
    ta_, tb_ = to_torch(a, DEV, False), to_torch(b, DEV, False)
    bias = rng.integers(info.min, info.max, (n,), dtype=dtype, endpoint=True)
    y = F.linear(ta_, tb_, to_torch(bias, DEV, False))
    refy = (exact(a, b) + bias.astype(np.int64)).astype(dtype)
    assert from_torch(y).tobytes() == refy.tobytes()
    if not big:
        a3 = rng.integers(info.min, info.max, (3, m, k), dtype=dtype, endpoint=True)
        out = F.matmult(to_torch(a3, DEV, False), tb_)
        ref3 = np.stack([exact(a3[i], b).astype(dtype) for i in range(3)])
        assert from_torch(out).tobytes() == ref3.tobytes()
        # the same values through the vector-ALU kernel: drop one column of B (rows are no longer 16-byte multiples)
        outv = F.matmult(ta_, to_torch(np.ascontiguousarray(b[:, :n - 1]), DEV, False))
        assert from_torch(outv).tobytes() == exact(a, b[:, :n - 1]).astype(dtype).tobytes()


@pytest.mark.parametrize("dtype", [np.float32, np.float16, "bf16", np.float64])
def test_c_modes(dtype):
    """overwrite ignores the incoming C (even NaN); accumulate adds to it."""
    rng = np.random.default_rng(400)
    m, k, n = 70, 90, 50
    a, b, sa, sb, c0 = make_inputs(rng, m, k, n, dtype, False, False)
    zeros = np.zeros_like(c0)
    ref0 = oracle.matmult2d(sa, sb, zeros.copy(), dt=code_of(dtype))
    junk = c0.copy()
    if dtype == "bf16":
        junk[:] = 0x7FC0
    else:
        junk[:] = np.nan
    got = dev_matmult(sa, sb, junk, m, k, n, False, False, dtype, mode=_lib.C_OVERWRITE)
    bf = dtype == "bf16"
    assert_close(got, ref0, to_f64(a, bf), to_f64(b, bf), k, dtype, "overwrite")


@pytest.mark.parametrize("tdtype", [torch.float32, torch.float64, torch.bfloat16, torch.float16, torch.int32, torch.int8],
                         ids=["fp32", "fp64", "bf16", "fp16", "int32", "int8"])
def test_empty_k_is_an_empty_sum(tdtype):
    """k = 0: C += nothing leaves C alone, overwrite gives zeros, bias mode gives the broadcast bias -- for a strided
    batch, without touching A or B (the product kernels themselves assume at least one k)."""
    lib = _lib.load()
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    batch, m, n = 3, 48, 80
    c0 = (torch.arange(batch * m * n, device=DEV) % 13 - 6).to(tdtype).reshape(batch, m, n)
    bias = (torch.arange(batch * n, device=DEV) % 7 - 3).to(tdtype).reshape(batch, 1, n)
    dummy = torch.zeros(16, dtype=tdtype, device=DEV)
    for mode, want in ((_lib.C_ACCUMULATE, c0), (_lib.C_OVERWRITE, torch.zeros_like(c0)), (_lib.C_BIAS, bias.expand(batch, m, n))):
        c = c0.clone()
        d = _lib.GemmDesc()
        d.dtype = F.ntg_dtype(c)
        d.c_mode = mode
        d.m, d.k, d.n, d.batches = m, 0, n, batch
        d.stride_c = m * n
        if mode == _lib.C_BIAS:
            d.bias = bias.data_ptr()
            d.bias_batch_stride, d.bias_row_stride, d.bias_col_stride = n, 0, 1
        _lib.check(lib.ntg_gemm_dev(ctypes.byref(d), dummy.data_ptr(), dummy.data_ptr(), c.data_ptr(), st))
        torch.cuda.synchronize()
        assert torch.equal(c, want), mode


@pytest.mark.parametrize("code,npdt", [(_lib.INT16, np.int16), (_lib.UINT16, np.int16), (_lib.INT32, np.int32), (_lib.UINT32, np.int32),
                                       (_lib.INT64, np.int64), (_lib.UINT64, np.int64)],
                         ids=["int16", "uint16", "int32", "uint32", "int64", "uint64"])
def test_wide_integers_on_the_8bit_matrix_pipe_bit_exact(code, npdt):
    """Large 16-, 32- and 64-bit integer products run as 3 / 10 / 36 products of balanced byte planes on
    v_mfma_i32_32x32x32_i8 when the caller gives the workspace: every result must equal the wrapping arithmetic of the
    reference in the element type over the FULL value range -- checked against the vector-ALU kernel (same call without
    workspace) on all elements and against exact integer arithmetic on sampled rows -- in all four transpose forms, the
    three C modes, ragged sizes (k and n not multiples of 16), a broadcast operand."""
    lib = _lib.load()
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rng = np.random.default_rng(4200)
    batch, m, k, n = 4, 520, 2057, 522
    full = lambda shape: rng.integers(0, 2**64, shape, dtype=np.uint64).astype(npdt)      # (keeps the low bits)
    for (ta, tb), mode, bcast_b in zip(TRANS, (_lib.C_OVERWRITE, _lib.C_ACCUMULATE, _lib.C_BIAS, _lib.C_ACCUMULATE), (False, True, False, False)):
        nb = 1 if bcast_b else batch
        a, b, c0, bias = full((batch, m, k)), full((nb, k, n)), full((batch, m, n)), full((n,))
        sa = np.ascontiguousarray(a.transpose(0, 2, 1)) if ta else a
        sb = np.ascontiguousarray(b.transpose(0, 2, 1)) if tb else b
        ta_, tb_, tbias = (torch.from_numpy(x).to(DEV) for x in (sa, sb, bias))      # (signed and unsigned share their bit patterns)
        results = []
        for use_ws in (True, False):
            c = torch.from_numpy(c0.copy()).to(DEV)
            d = _lib.GemmDesc()
            d.dtype = code
            d.transpose_a, d.transpose_b, d.c_mode = int(ta), int(tb), mode
            d.m, d.k, d.n, d.batches = m, k, n, batch
            d.stride_a, d.stride_b, d.stride_c = m * k, (0 if bcast_b else k * n), m * n
            if mode == _lib.C_BIAS:
                d.bias = tbias.data_ptr()
                d.bias_col_stride = 1
            wsb = lib.ntg_gemm_workspace_bytes(ctypes.byref(d))
            assert wsb > 0
            if use_ws:
                ws = torch.empty(wsb, dtype=torch.uint8, device=DEV)
                d.workspace, d.workspace_bytes = ws.data_ptr(), wsb
            _lib.check(lib.ntg_gemm_dev(ctypes.byref(d), ta_.data_ptr(), tb_.data_ptr(), c.data_ptr(), st))
            torch.cuda.synchronize()
            results.append(c.cpu().numpy())
        assert np.array_equal(results[0], results[1]), (ta, tb, mode)
        # exact arithmetic (uint64 wraps modulo 2^64, which keeps the low bits of every width) on a few rows of two items
        for bi in (0, batch - 1):
            rows = np.r_[0:3, m - 3:m]
            exact = a[bi, rows].astype(np.uint64) @ b[0 if bcast_b else bi].astype(np.uint64)
            init = c0[bi, rows].astype(np.uint64) if mode == _lib.C_ACCUMULATE else bias.astype(np.uint64)[None, :] if mode == _lib.C_BIAS else np.uint64(0)
            assert np.array_equal(results[0][bi, rows], (exact + init).astype(npdt)), (ta, tb, mode, bi)


def test_host_batch_with_repeated_pointers():
    """nt_matmult_batch: uniform shape, entries of A/B may repeat (broadcast by handle)."""
    rng = np.random.default_rng(500)
    m, k, n = 40, 33, 21
    As = [rng.standard_normal((m, k)).astype(np.float32) for _ in range(3)]
    Bsh = rng.standard_normal((n, k)).astype(np.float32)          # stored [n,k] -> transpose_b
    Alist = [As[0], As[1], As[2], As[0], As[1]]
    Blist = [Bsh] * 5
    C0 = [rng.standard_normal((m, n)).astype(np.float32) for _ in range(5)]
    ref = [c.copy() for c in C0]
    oracle.matmult_batch_ptrs(Alist, Blist, ref, False, True)
    got = [c.copy() for c in C0]
    arr = ctypes.c_void_p * 5
    lib = _lib.load()
    _lib.check(lib.ntg_matmult_batch(_lib.FLOAT32, arr(*[x.ctypes.data for x in Alist]), arr(*[x.ctypes.data for x in Blist]),
                                     arr(*[x.ctypes.data for x in got]), 5, m, k, k, n, 0, 1))
    for g, r, a_ in zip(got, ref, Alist):
        assert np.abs(g - r).max() <= float_tol(k, a_, Bsh)
    # same pointers -> bit-identical results (the reference's batched == per-item invariant)
    assert got[0].tobytes() != got[3].tobytes() or np.array_equal(C0[0], C0[3])
    single = host_matmult(As[0], Bsh, C0[0].copy(), m, k, n, False, True, _lib.FLOAT32)
    assert single.tobytes() == got[0].tobytes()


@pytest.mark.parametrize("pattern", ["distinct", "shared_b", "shared_a", "mixed"])
def test_host_batch_int32_full_range_every_pointer_pattern(pattern):
    """nt_matmult_batch on host pointers, Int32 wrapping modulo 2^32 with full-range entries: items that are all new
    matrices or all one matrix take the strided kernels (large enough here for the byte-plane form), any other pattern
    of repeated pointers the pointer tables; every pattern equals exact integer arithmetic, item by item."""
    rng = np.random.default_rng(77)
    nb, m, k, n = 4, 256, 1024, 2304
    full = lambda shape: rng.integers(-2**31, 2**31, shape, dtype=np.int64).astype(np.int32)
    As = [full((m, k)) for _ in range(nb)]
    Bs = [full((k, n)) for _ in range(nb)]
    if pattern == "shared_b":
        Bs = [Bs[0]] * nb
    elif pattern == "shared_a":
        As = [As[0]] * nb
    elif pattern == "mixed":
        As = [As[0], As[1], As[0], As[1]]
    C0 = [full((m, n)) for _ in range(nb)]
    got = [c.copy() for c in C0]
    arr = ctypes.c_void_p * nb
    lib = _lib.load()
    _lib.check(lib.ntg_matmult_batch(_lib.INT32, arr(*[x.ctypes.data for x in As]), arr(*[x.ctypes.data for x in Bs]),
                                     arr(*[x.ctypes.data for x in got]), nb, m, k, k, n, 0, 0))
    rows = np.array([0, 1, 127, 128, 255])
    for i in range(nb):
        # exact: 64-bit wrapping sums of 32 x 32 -> 64-bit products keep the low 32 bits intact
        exact = As[i][rows].astype(np.int64) @ Bs[i].astype(np.int64) + C0[i][rows].astype(np.int64)
        assert np.array_equal(got[i][rows], exact.astype(np.int32)), (pattern, i)


def test_functional_batch_rules_and_views():
    """N-D x K-D: trailing batch dims must match; lower-rank operand is reused; a transposed
    view is consumed by flipping the flag (no copy); results equal the oracle's."""
    rng = np.random.default_rng(600)
    a = rng.standard_normal((2, 3, 10, 7)).astype(np.float32)
    b = rng.standard_normal((3, 7, 6)).astype(np.float32)
    ta_, tb_ = torch.from_numpy(a).to(DEV), torch.from_numpy(b).to(DEV)
    out = F.matmult(ta_, tb_)
    ref = oracle.matmult(a, b)
    assert tuple(out.shape) == ref.shape
    assert np.abs(out.cpu().numpy() - ref).max() <= float_tol(7, a, b)
    # single-matrix B broadcasts with stride 0
    b2 = rng.standard_normal((7, 5)).astype(np.float32)
    out2 = F.matmult(ta_, torch.from_numpy(b2).to(DEV))
    assert np.abs(out2.cpu().numpy() - oracle.matmult(a, b2)).max() <= float_tol(7, a, b2)
    # lower-rank A with both flags
    a3 = rng.standard_normal((7, 10)).astype(np.float32)
    b3 = rng.standard_normal((4, 6, 7)).astype(np.float32)
    out3 = F.matmult(torch.from_numpy(a3).to(DEV), torch.from_numpy(b3).to(DEV), None, True, True)
    assert np.abs(out3.cpu().numpy() - oracle.matmult(a3, b3, None, True, True)).max() <= float_tol(7, a3, b3)
    # transposed view == explicit flag
    v = tb_.transpose(-1, -2)                       # shape (3, 6, 7), non-contiguous
    out4 = F.matmult(ta_, v, None, False, True)
    assert torch.equal(out4, out)
    # out= accumulates
    acc = out.clone()
    F.matmult(ta_, tb_, acc)
    assert torch.allclose(acc, 2 * out, rtol=1e-6, atol=1e-6)
    with pytest.raises(ValueError):
        F.matmult(ta_, torch.from_numpy(np.zeros((2, 7, 6), np.float32)).to(DEV))   # batch dims do not line up
    with pytest.raises(ValueError):
        F.matmult(ta_, tb_, None, True, False)                                       # inner sizes differ
    with pytest.raises(ValueError):
        F.matmult(ta_, tb_.double())                                                 # dtype mismatch


# ---------------------------------------------------------------------------------------
# BASELINE configurations
# ---------------------------------------------------------------------------------------

def test_config1_fp32_512_cube():
    rng = np.random.default_rng(1001)
    a = rng.standard_normal((512, 512)).astype(np.float32)
    b = rng.standard_normal((512, 512)).astype(np.float32)
    ref = oracle.matmult2d(a, b)
    got = dev_matmult(a, b, np.zeros((512, 512), np.float32), 512, 512, 512, False, False, np.float32)
    err = np.abs(got - ref).max()
    assert err <= float_tol(512, a, b)
    # far inside the stated bound in practice: a few ulps of sqrt(K)
    assert err <= 1e-3
    host = host_matmult(a, b, np.zeros((512, 512), np.float32), 512, 512, 512, False, False, _lib.FLOAT32)
    assert host.tobytes() == got.tobytes()


def test_config2_batched_fp32_and_transpose_b():
    rng = np.random.default_rng(1002)
    a = rng.standard_normal((32, 1024, 768)).astype(np.float32)
    b = rng.standard_normal((32, 768, 1024)).astype(np.float32)
    bt = np.ascontiguousarray(b.transpose(0, 2, 1))                 # stored [32,1024,768]
    ta_, tb_, tbt = (torch.from_numpy(x).to(DEV) for x in (a, b, bt))
    out_a = F.matmult(ta_, tb_)
    out_b = F.matmult(ta_, tbt, None, False, True)
    tol = float_tol(768, a, b)
    assert (out_a - out_b).abs().max().item() <= tol
    ref64 = torch.bmm(ta_.double(), tb_.double())
    assert (out_a.double() - ref64).abs().max().item() <= tol
    # oracle on a few whole items (the tiled restatement is bit-equal to the closed form)
    got = out_a.cpu().numpy()
    for i in (0, 13, 31):
        ref = oracle.matmult2d(a[i], b[i], kind="tiled")
        assert np.abs(got[i] - ref).max() <= tol
        ref_t = oracle.matmult2d(a[i], bt[i], tb=True, kind="tiled")
        assert ref_t.tobytes() == ref.tobytes()


def test_config2_int32_bit_exact():
    rng = np.random.default_rng(1003)
    a = rng.integers(-8, 9, (8, 1024, 1024)).astype(np.int32)
    b = rng.integers(-8, 9, (8, 1024, 1024)).astype(np.int32)
    out = F.matmult(torch.from_numpy(a).to(DEV), torch.from_numpy(b).to(DEV)).cpu().numpy()
    for i in range(8):
        ref = oracle.matmult2d(a[i], b[i], kind="tiled")
        assert out[i].tobytes() == ref.tobytes()


def _sampled_oracle_check(a_np, b_np, got_t, ta, tb, dtype, rows, cols, k):
    """Oracle parity on a sub-block of a large product: op(A)[rows,:] . op(B)[:,cols]."""
    bf = dtype == "bf16"
    A = a_np.T if ta else a_np
    B = b_np.T if tb else b_np
    sa = np.ascontiguousarray(A[rows, :])
    sb = np.ascontiguousarray(B[:, cols])
    ref = oracle.matmult2d(sa, sb, dt=code_of(dtype))
    got = from_torch(got_t[rows][:, cols].contiguous())
    assert_close(got, ref, to_f64(sa, bf), to_f64(sb, bf), k, dtype, "sampled block")


@pytest.mark.parametrize("dtype,scale", [("bf16", 0.02), (np.float16, 0.02), (np.float32, 1.0), (np.float64, 1.0)],
                         ids=["bf16", "fp16", "fp32", "fp64"])
def test_config3_4096_cube(dtype, scale):
    n = 4096
    rng = np.random.default_rng(1004)
    a = randn(rng, (n, n), dtype, scale)
    b = randn(rng, (n, n), dtype, scale)
    bf = dtype == "bf16"
    ta_, tb_ = to_torch(a, DEV, bf), to_torch(b, DEV, bf)
    out = F.matmult(ta_, tb_)
    torch.cuda.synchronize()
    rows = np.r_[0:32, 2040:2072, 4064:4096]
    cols = np.r_[0:16, 1000:1016, 4080:4096]
    _sampled_oracle_check(a, b, out, False, False, dtype, rows, cols, n)
    # whole-matrix cross-check against an independent library GEMM in higher precision
    if dtype in (np.float32, np.float64):
        ref = torch.matmul(ta_.double(), tb_.double())
        tol = 1e-5 * n * ta_.abs().max().item() * tb_.abs().max().item()
        assert (out.double() - ref).abs().max().item() <= tol
    else:
        ref = torch.matmul(ta_.float(), tb_.float())
        assert ((out.float() - ref).abs().max() / ref.abs().max()).item() <= HALF_REL
        # 384 whole rows (from the first, a middle and the last tile row, each crossing a block boundary of the tile) against the
        # exact result: every element is the once-rounded float64 product wherever that is clear of a rounding boundary
        from util import assert_one_rounding
        fmt = "bf16" if bf else "f16"
        rsel = torch.as_tensor(np.r_[0:128, 1984:2112, 3968:4096], device=DEV)
        ar, bd = ta_[rsel].double(), tb_.double()
        ref64 = ar @ bd
        spread = ((ar * ar) @ (bd * bd)).sqrt()
        assert_one_rounding(out[rsel].double().cpu().numpy(), ref64.cpu().numpy(), spread.cpu().numpy(), n, fmt, f"{fmt} 4096^3 overwrite",
                            min_exact=0.75 if bf else 0.2)
        c0r = to_torch(randn(rng, (n, n), dtype, 0.5), DEV, bf)
        accr = c0r.clone()
        F.matmult(ta_, tb_, accr)                                    # the headline's own mode: C += A.B
        assert_one_rounding(accr[rsel].double().cpu().numpy(), (ref64 + c0r[rsel].double()).cpu().numpy(),
                            (spread + c0r[rsel].double().abs()).cpu().numpy(), n, fmt, f"{fmt} 4096^3 accumulate", min_exact=0.75 if bf else 0.2)
        del ar, bd, ref64, spread, c0r, accr
    # linearity, a size-independent property: (2A).B == 2(A.B) exactly in binary floating point
    out2 = F.matmult(ta_ * 2, tb_)
    if dtype is np.float16:      # half subnormals (|c| < 6.1e-5) round on a fixed 2^-24 grid
        assert (out2.float() - 2 * out.float()).abs().max().item() <= 2.0 ** -23
    else:
        assert torch.equal(out2, out * 2)
    # accumulate contract at full size: C0 + A.B
    acc = out.clone()
    F.matmult(ta_, tb_, acc)
    if dtype in (np.float32, np.float64):
        # (Float32 starts every chain from C0, as the reference does: C0 + A.B is not the rounded sum of two rounded terms)
        assert (acc.double() - 2 * out.double()).abs().max().item() <= 1e-5 * n * float(ta_.abs().max() * tb_.abs().max())
    else:
        assert ((acc.float() - 2 * out.float()).abs().max() / out.float().abs().max()).item() <= HALF_REL


@pytest.mark.parametrize("dtype", ["bf16", np.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("shape", [(2056, 1000, 2312), (1800, 1016, 3080), (2304, 992, 1928), (3000, 40, 2056), (2056, 8, 2056),
                                   (3848, 1000, 4088), (4104, 40, 2056), (1024, 512, 1536), (128, 96, 128), (136, 72, 8),
                                   (3000, 1016, 4000)],
                         ids=lambda s: "x".join(map(str, s)))
def test_ragged_16bit_dma_kernel(dtype, shape):
    """M, N, K that are not multiples of the tile (but keep 16-byte rows) stay on the DMA-fed kernel: edge
    rows/columns, the k tail (8, 24, none, 8-only) and all three C modes.  The tile follows the kernel's cost
    estimate: 3848 x 4088 (16 x 16 large tiles, one per CU) and 4104 x 2056 run on 256 x 256 tiles, 2056 x 2312,
    1800 x 3080 and 2304 x 1928 on the 128 x 256 tile (one round over the CUs), 3000 x 4000 on the 192 x 256 tile
    (16 x 16 tiles), 3000 x 2056 with k = 40 on 128 x 128, the others (short k,
    or few tiles) on 64 x 64; two shapes are tile-aligned."""
    m, k, n = shape
    bf = dtype == "bf16"
    rng = np.random.default_rng(1100 + k)
    for ta, tb in TRANS:
        a = randn(rng, (m, k), dtype, 0.25)
        b = randn(rng, (k, n), dtype, 0.25)
        sa = np.ascontiguousarray(a.T) if ta else a
        sb = np.ascontiguousarray(b.T) if tb else b
        ta_, tb_ = to_torch(sa, DEV, bf), to_torch(sb, DEV, bf)
        ref = torch.matmul(to_torch(a, DEV, bf).float(), to_torch(b, DEV, bf).float())
        scale = ref.abs().max().item()
        # C sits inside a larger buffer of sentinels: nothing outside [m, n] may be written
        guard = torch.full((m + 2, n), 7.0, device=DEV).to(ta_.dtype)
        c = guard[1:m + 1]
        c.zero_()
        out = F.matmult(ta_, tb_, c, ta, tb, accumulate=False)
        assert ((out.float() - ref).abs().max() / scale).item() <= HALF_REL, (shape, ta, tb)
        assert torch.all(guard[0] == 7.0) and torch.all(guard[m + 1] == 7.0)
        F.matmult(ta_, tb_, c, ta, tb)                                   # accumulate: 2 * A.B
        assert ((c.float() - 2 * ref).abs().max() / scale).item() <= 2 * HALF_REL
        # oracle on the last rows / columns and on an interior block
        rows = np.r_[0:8, m - 8:m]
        cols = np.r_[0:8, n - 8:n]
        _sampled_oracle_check(sa, sb, out := F.matmult(ta_, tb_, None, ta, tb), ta, tb, dtype, rows, cols, k)
    # bias mode on a ragged shape
    bias = randn(rng, (n,), dtype)
    y = F.linear(to_torch(a, DEV, bf), to_torch(b, DEV, bf), to_torch(bias, DEV, bf))
    refy = ref + to_torch(bias, DEV, bf).float()
    assert ((y.float() - refy).abs().max() / refy.abs().max()).item() <= HALF_REL


@pytest.mark.parametrize("dtype", ["bf16", np.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("shape", [(33, 128, 512, 1000), (70, 250, 512, 256), (270, 128, 1032, 264)], ids=lambda s: "x".join(map(str, s)))
def test_batched_16bit_two_launch_plan(dtype, shape):
    """Batches whose tiles fill the CUs a whole number of times plus a small rest go out as two launches (the first items
    on the chosen tile, the rest on a smaller one): 33 -> 32 + 1, 70 -> 64 + 6, 270 -> 256 + 14 items.  Every item must
    come out the same whichever launch computed it: all three C modes, broadcast A, ragged edges."""
    batch, m, k, n = shape
    bf = dtype == "bf16"
    rng = np.random.default_rng(2100 + batch)
    a = to_torch(randn(rng, (batch, m, k), dtype, 0.25), DEV, bf)
    b = to_torch(randn(rng, (batch, k, n), dtype, 0.25), DEV, bf)
    ref = torch.matmul(a.float(), b.float())
    scale = ref.abs().max().item()
    guard = torch.full((batch + 2, m, n), 7.0, device=DEV).to(a.dtype)
    c = guard[1:batch + 1]
    c.zero_()
    out = F.matmult(a, b, c, accumulate=False)
    assert ((out.float() - ref).abs().max() / scale).item() <= HALF_REL
    assert torch.all(guard[0] == 7.0) and torch.all(guard[batch + 1] == 7.0)
    # identical operands in the first and the last item: the two launches must agree bit for bit
    a2, b2 = a.clone(), b.clone()
    a2[batch - 1], b2[batch - 1] = a2[0], b2[0]
    out2 = F.matmult(a2, b2)
    assert torch.equal(out2[0], out2[batch - 1])
    F.matmult(a, b, c)                                               # accumulate: 2 * A.B
    assert ((c.float() - 2 * ref).abs().max() / scale).item() <= 2 * HALF_REL
    # one A for every item (stride 0), B stored [n, k], bias broadcast over the batch
    w = to_torch(randn(rng, (n, k), dtype, 0.25), DEV, bf)
    bias = to_torch(randn(rng, (n,), dtype), DEV, bf)
    y = F.linear(a, w, bias, False, True)
    refy = torch.matmul(a.float(), w.float().T) + bias.float()
    assert ((y.float() - refy).abs().max() / refy.abs().max()).item() <= HALF_REL


@pytest.mark.parametrize("dtype", ["bf16", np.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("shape", [(2048, 1024, 4096), (2040, 1000, 2312), (1000, 1016, 1720), (1800, 1016, 3080), (3000, 1016, 4000)],
                         ids=lambda s: "x".join(map(str, s)))
def test_16bit_product_is_the_same_in_every_batch_size(dtype, shape):
    """A product alone, as every item of a batch of 3 and of a batch of 5: the kernel's cost estimate gives these different
    tiles (128 x 256 for the single 2048 x 4096 output and for 3 x 1000 x 1720, 192 x 256 for 3000 x 4000 and for batches of
    1800 x 3080, 256 x 256 or 128 x 128 for the others),
    and the bits must not depend on that (the reference's batched == per-item rule, tests/src/matmult_test.cpp:108-189).
    All four transpose forms; the single product also against torch in float."""
    m, k, n = shape
    bf = dtype == "bf16"
    rng = np.random.default_rng(3100 + m)
    a = to_torch(randn(rng, (m, k), dtype, 0.25), DEV, bf)
    b = to_torch(randn(rng, (k, n), dtype, 0.25), DEV, bf)
    ref = torch.matmul(a.float(), b.float())
    for ta, tb in TRANS:
        sa = a.t().contiguous() if ta else a
        sb = b.t().contiguous() if tb else b
        one = F.matmult(sa, sb, None, ta, tb)
        assert ((one.float() - ref).abs().max() / ref.abs().max()).item() <= HALF_REL, (shape, ta, tb)
        for batch in (3, 5):
            out = F.matmult(sa.expand(batch, *sa.shape).contiguous(), sb.expand(batch, *sb.shape).contiguous(), None, ta, tb)
            for i in range(batch):
                assert torch.equal(out[i].view(torch.int16), one.view(torch.int16)), (shape, ta, tb, batch, i)


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["fp32", "fp64"])
@pytest.mark.parametrize("shape", [(1860, 260, 1860), (2052, 1000, 2308), (1028, 132, 516), (68, 20, 4), (132, 16, 260), (130, 22, 66)],
                         ids=lambda s: "x".join(map(str, s)))
def test_ragged_fp32_fp64_ring_kernels(dtype, shape):
    """Float32 / Float64 with 16-byte rows (sizes multiples of 4 / 2) stay on the DMA-fed kernels: 1860 x 1860 runs on
    128 x 128 tiles, the others on 64 x 64; edge rows / columns, a last 16-byte chunk of C of which only the first half
    exists (fp32, n % 8 == 4), k tails (fp32: 4, 8, 4, none; fp64: 4, none, 4, 4, none, 6), all three C modes, nothing
    written outside [m, n].  130 x 22 x 66 has 8-byte but not 16-byte rows in fp32: the register-staged kernel."""
    m, k, n = shape
    rng = np.random.default_rng(1300 + k)
    for ta, tb in TRANS:
        a = randn(rng, (m, k), dtype)
        b = randn(rng, (k, n), dtype)
        sa = np.ascontiguousarray(a.T) if ta else a
        sb = np.ascontiguousarray(b.T) if tb else b
        ta_, tb_ = to_torch(sa, DEV, False), to_torch(sb, DEV, False)
        ref = torch.matmul(to_torch(a, DEV, False).double(), to_torch(b, DEV, False).double())
        tol = 1e-5 * k * float(np.abs(a).max() * np.abs(b).max())
        guard = torch.full((m + 2, n), 7.0, device=DEV, dtype=ta_.dtype)
        c = guard[1:m + 1]
        c.zero_()
        out = F.matmult(ta_, tb_, c, ta, tb, accumulate=False)
        assert (out.double() - ref).abs().max().item() <= tol, (shape, ta, tb)
        assert torch.all(guard[0] == 7.0) and torch.all(guard[m + 1] == 7.0)
        F.matmult(ta_, tb_, c, ta, tb)                                   # accumulate: 2 * A.B
        assert (c.double() - 2 * ref).abs().max().item() <= 2 * tol
        assert torch.all(guard[0] == 7.0) and torch.all(guard[m + 1] == 7.0)
        rows = np.r_[0:4, m - 4:m]
        cols = np.r_[0:4, n - 4:n]
        _sampled_oracle_check(sa, sb, F.matmult(ta_, tb_, None, ta, tb), ta, tb, dtype, rows, cols, k)
    bias = randn(rng, (n,), dtype)
    y = F.linear(to_torch(a, DEV, False), to_torch(b, DEV, False), to_torch(bias, DEV, False))
    assert (y.double() - (ref + to_torch(bias, DEV, False).double())).abs().max().item() <= tol


@pytest.mark.parametrize("dtype", ["bf16", np.float32, np.int32], ids=["bf16", "fp32", "int32"])
def test_operands_beyond_2_31_elements(dtype):
    """A holds more than 2^31 elements (4.4 - 9.6 GB): every row offset in the loaders and the stores is 64-bit.
    The rows past the 2^31-element mark are checked against torch on that slice."""
    bf = dtype == "bf16"
    if bf:
        m, k, n, td = 66000, 33000, 256, torch.bfloat16
    elif dtype == np.float32:
        m, k, n, td = 40000, 60000, 128, torch.float32
    else:
        m, k, n, td = 50000, 45000, 8, torch.int32
    assert m * k > 2 ** 31
    torch.manual_seed(5)
    if dtype == np.int32:
        a = torch.randint(-8, 9, (m, k), device=DEV, dtype=td)
        b = torch.randint(-8, 9, (k, n), device=DEV, dtype=td)
    else:
        a = torch.empty((m, k), device=DEV, dtype=td).normal_(0, 0.05 if bf else 1.0)
        b = torch.empty((k, n), device=DEV, dtype=td).normal_(0, 0.05 if bf else 1.0)
    c = F.matmult(a, b)
    for lo in (0, m - 300):
        rows = slice(lo, lo + 300)
        if dtype == np.int32:
            ref = (a[rows].double() @ b.double())                       # |sum| < 2^53: exact
            assert torch.equal(c[rows].double(), ref)
        else:
            ref = a[rows].double() @ b.double()
            err = (c[rows].double() - ref).abs().max().item()
            tol = HALF_REL * ref.abs().max().item() if bf else 1e-5 * k * float(a[rows].abs().max().item() * b.abs().max().item())
            assert err <= tol, (lo, err, tol)
    # transpose_a: A stored [k, m] with the same footprint
    if not bf:
        return
    at = torch.empty((k, m), device=DEV, dtype=td).normal_(0, 0.05)
    ct = F.matmult(at, b, None, True, False)
    ref = at[:, m - 256:].double().t() @ b.double()
    assert (ct[m - 256:].double() - ref).abs().max().item() <= HALF_REL * ref.abs().max().item()


@pytest.mark.parametrize("dtype", ["bf16", np.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("m", [1, 7, 16, 17, 32])
def test_skinny_16bit(dtype, m):
    """m <= 32 in Float16 / BFloat16 streams B once through the HBM-bound kernel: every transpose pair, strip widths of
    2, 4 and 8 columns per lane, the guarded (ragged / unaligned) instantiation, all three C modes, batches."""
    bf = dtype == "bf16"
    rng = np.random.default_rng(1800 + m)
    for (k, n, batch) in [(4096, 8192, 1), (1024, 2048, 1), (512, 256, 3), (1000, 520, 2), (136, 24, 1), (2048, 1030, 1)]:
        for ta, tb in TRANS:
            a = randn(rng, (batch, m, k), dtype, 0.25)
            b = randn(rng, (batch, k, n), dtype, 0.25)
            sa = np.ascontiguousarray(a.transpose(0, 2, 1)) if ta else a
            sb = np.ascontiguousarray(b.transpose(0, 2, 1)) if tb else b
            ta_, tb_ = to_torch(sa, DEV, bf), to_torch(sb, DEV, bf)
            ref = torch.matmul(to_torch(a, DEV, bf).double(), to_torch(b, DEV, bf).double())
            scale = ref.abs().max().item()
            out = F.matmult(ta_, tb_, None, ta, tb)
            assert tuple(out.shape) == (batch, m, n)
            assert ((out.double() - ref).abs().max() / scale).item() <= HALF_REL, (m, k, n, batch, ta, tb)
            c0 = to_torch(randn(rng, (batch, m, n), dtype), DEV, bf)
            c = c0.clone()
            F.matmult(ta_, tb_, c, ta, tb)                                        # C += A.B
            assert ((c.double() - (ref + c0.double())).abs().max() / scale).item() <= HALF_REL
    # deterministic: two launches give identical bits; the oracle agrees on a small case
    a = randn(rng, (m, 512), dtype)
    b = randn(rng, (512, 64), dtype)
    ta_, tb_ = to_torch(a, DEV, bf), to_torch(b, DEV, bf)
    o1, o2 = F.matmult(ta_, tb_), F.matmult(ta_, tb_)
    assert torch.equal(o1, o2)
    want = to_f64(oracle.matmult2d(a, b, dt=code_of(dtype)), bf)
    got = o1.double().cpu().numpy()
    assert np.abs(got - want).max() <= HALF_REL * np.abs(want).max()
    # bias mode (linear with a small batch)
    bias = randn(rng, (64,), dtype)
    y = F.linear(ta_, tb_, to_torch(bias, DEV, bf))
    refy = ta_.double() @ tb_.double() + to_torch(bias, DEV, bf).double()
    assert ((y.double() - refy).abs().max() / refy.abs().max()).item() <= HALF_REL


@pytest.mark.parametrize("dtype", ["bf16", np.float16, np.float32, np.float64], ids=["bf16", "fp16", "fp32", "fp64"])
def test_split_k_medium_rows(dtype):
    """Few output tiles and a deep k: ntg_gemm_workspace_bytes offers a workspace and the product is split along k
    (fp32 partial sums for the 16-bit dtypes, ordered reduction).  Every transpose pair and C mode; the result must also
    equal the unsplit run to rounding, and two runs must be bit-identical."""
    bf = dtype == "bf16"
    half = bf or dtype == np.float16
    rng = np.random.default_rng(1900)
    lib = _lib.load()
    for (m, k, n) in [(256, 4096, 2048), (520, 4096, 1032), (64, 8192, 1024), (768, 6144, 1024)]:
        for ta, tb in TRANS:
            a = randn(rng, (m, k), dtype, 0.25)
            b = randn(rng, (k, n), dtype, 0.25)
            sa = np.ascontiguousarray(a.T) if ta else a
            sb = np.ascontiguousarray(b.T) if tb else b
            ta_, tb_ = to_torch(sa, DEV, bf), to_torch(sb, DEV, bf)
            d = _lib.GemmDesc()
            d.dtype, d.transpose_a, d.transpose_b, d.c_mode = F.ntg_dtype(ta_), int(ta), int(tb), _lib.C_OVERWRITE
            d.m, d.k, d.n, d.batches = m, k, n, 1
            ws_bytes = lib.ntg_gemm_workspace_bytes(ctypes.byref(d))
            assert ws_bytes > 0, (m, k, n)
            assert ws_bytes % (m * n * (4 if half else a.itemsize)) == 0
            ref = to_torch(a, DEV, bf).double() @ to_torch(b, DEV, bf).double()
            scale = ref.abs().max().item()
            tol = HALF_REL * scale if half else 1e-5 * k * float(np.abs(to_f64(a, bf)).max() * np.abs(to_f64(b, bf)).max())
            out = F.matmult(ta_, tb_, None, ta, tb)                                # functional passes the workspace
            assert (out.double() - ref).abs().max().item() <= tol
            assert torch.equal(out, F.matmult(ta_, tb_, None, ta, tb))
            # the same product without a workspace (one pass over k)
            st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
            plain = torch.empty_like(out)
            _lib.check(lib.ntg_gemm_dev(ctypes.byref(d), ta_.data_ptr(), tb_.data_ptr(), plain.data_ptr(), st))
            assert (plain.double() - ref).abs().max().item() <= tol
            assert (plain.double() - out.double()).abs().max().item() <= (2 * HALF_REL * scale / 8 if half else tol)
            # C += and bias
            c0 = to_torch(randn(rng, (m, n), dtype), DEV, bf)
            c = c0.clone()
            F.matmult(ta_, tb_, c, ta, tb)
            assert (c.double() - (ref + c0.double())).abs().max().item() <= tol + (HALF_REL * scale if half else 0)
        bias = to_torch(randn(rng, (n,), dtype), DEV, bf)
        y = F.linear(to_torch(a, DEV, bf), to_torch(b, DEV, bf), bias)
        refy = to_torch(a, DEV, bf).double() @ to_torch(b, DEV, bf).double() + bias.double()
        assert (y.double() - refy).abs().max().item() <= tol + (HALF_REL * scale if half else 0)
    # no split where it does not apply: many tiles, shallow k (a batch is offered what its item is offered)
    for (m, k, n, bt) in [(4096, 4096, 4096, 1), (256, 128, 256, 1), (4096, 4096, 4096, 2)]:
        d = _lib.GemmDesc()
        d.dtype, d.m, d.k, d.n, d.batches = F.ntg_dtype(ta_), m, k, n, bt
        d.stride_a, d.stride_b, d.stride_c = m * k, k * n, m * n
        assert lib.ntg_gemm_workspace_bytes(ctypes.byref(d)) == 0


def test_skinny_fp32_config5b():
    rng = np.random.default_rng(1005)
    a = rng.standard_normal((16, 8192)).astype(np.float32)
    b = rng.standard_normal((8192, 8192)).astype(np.float32)
    ta_, tb_ = torch.from_numpy(a).to(DEV), torch.from_numpy(b).to(DEV)
    out = F.matmult(ta_, tb_)
    ref = oracle.matmult2d(a, b, kind="tiled")
    tol = float_tol(8192, a, b)
    assert np.abs(out.cpu().numpy() - ref).max() <= tol
    # deterministic: two runs are bit-identical
    assert torch.equal(F.matmult(ta_, tb_), out)
    # other flag pairs of the skinny path, ragged sizes, m in (1, 16, 17, 32)
    for m, k, n, ta, tb in [(1, 300, 1000, False, False), (16, 257, 513, False, True), (17, 1024, 96, True, False),
                            (32, 640, 2048, True, True), (3, 64, 5, False, False)]:
        A, B, sa, sb, c0 = make_inputs(rng, m, k, n, np.float32, ta, tb)
        ref = oracle.matmult2d(sa, sb, c0.copy(), ta, tb)
        got = dev_matmult(sa, sb, c0, m, k, n, ta, tb, np.float32)
        assert np.abs(got - ref).max() <= float_tol(k, A, B), (m, k, n, ta, tb)


def test_host_entry_staging_large_transfers_threads_and_release():
    """The host-pointer seam stages through a grow-only device arena and a ring of 8 MiB pinned chunks: operands of
    several chunks (and not a whole number of them), a smaller call after a larger one, a larger one after that (the
    arena grows), two threads calling at once, and a call after ntg_release_host_buffers -- every result bit-identical
    to the device entry point on the same operands."""
    import threading
    lib = _lib.load()
    rng = np.random.default_rng(515)

    def case(m, k, n, dtype, ta=False, tb=False):
        a, b, sa, sb, c0 = make_inputs(rng, m, k, n, dtype, ta, tb, int_range=(-1000, 1000))
        want = dev_matmult(sa, sb, c0, m, k, n, ta, tb, dtype)
        return (sa, sb, c0, m, k, n, ta, tb, dtype, want)

    def check_case(cs):
        sa, sb, c0, m, k, n, ta, tb, dtype, want = cs
        got = host_matmult(sa, sb, c0.copy(), m, k, n, ta, tb, code_of(dtype))
        assert got.tobytes() == want.tobytes(), (m, k, n, dtype)

    big = case(2500, 1100, 2300, np.float32)           # A 10.5 MiB, B 9.7 MiB, C 21.9 MiB
    small = case(70, 90, 50, np.float32, True, True)
    bigger = case(3000, 2100, 2600, np.int32, False, True)
    half = case(1111, 1000, 2224, "bf16")
    for cs in (big, small, bigger, half, big):
        check_case(cs)
    errors = []

    def worker(cs):
        try:
            for _ in range(3):
                check_case(cs)
        except Exception as e:          # noqa: BLE001 (reported below)
            errors.append(e)

    ts = [threading.Thread(target=worker, args=(cs,)) for cs in (big, half, small)]
    for t in ts:
        t.start()
    for t in ts:
        t.join()
    assert not errors, errors
    assert lib.ntg_release_host_buffers() == 0
    check_case(small)
    check_case(big)
    # batch entry point with repeated inputs, several chunks in total
    m, k, n = 600, 700, 800
    As = [rng.standard_normal((m, k)).astype(np.float32) for _ in range(3)]
    Bm = rng.standard_normal((k, n)).astype(np.float32)
    Cs = [rng.standard_normal((m, n)).astype(np.float32) for _ in range(5)]
    want = [c + 0 for c in Cs]
    idx = [0, 1, 2, 1, 0]
    for i, c in enumerate(want):
        host_matmult(As[idx[i]], Bm, c, m, k, n, False, False, _lib.FLOAT32)
    arr = lambda xs: (ctypes.c_void_p * len(xs))(*[x.ctypes.data for x in xs])
    _lib.check(lib.ntg_matmult_batch(_lib.FLOAT32, arr([As[i] for i in idx]), arr([Bm] * 5), arr(Cs), 5, m, k, k, n, 0, 0))
    for i in range(5):
        assert np.abs(Cs[i] - want[i]).max() <= float_tol(k, As[idx[i]], Bm)


@pytest.mark.parametrize("kind", ["bf16", "int8"])
def test_single_large_products_split_into_two_launches(kind):
    """A single product whose tiles make whole rounds over the CUs plus a rest goes out as two launches on sub-matrices
    (leading tile columns or rows on the chosen tile, the remaining strip on another): the seam must not show -- bias
    and C0 follow the strip, both transpose layouts, ragged edges.  Checked whole against float64 products on the GPU:
    Int8 bit-exact (wrapping), BFloat16 within one ulp of the correctly rounded result and equal to it almost everywhere."""
    lib = _lib.load()
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    gen = torch.Generator(device=DEV).manual_seed(77)
    cases = [(8192, 1024, 11008, False, True, _lib.C_BIAS), (11008, 1024, 4096, True, False, _lib.C_ACCUMULATE),
             (5000, 1024, 5000, False, False, _lib.C_ACCUMULATE), (8192, 1024, 11008, False, False, _lib.C_OVERWRITE)]
    for (m, k, n, ta, tb, mode) in cases:
        if kind == "bf16":
            mk = lambda *shape: (torch.randn(*shape, device=DEV, generator=gen) * 0.25).bfloat16()
        else:
            mk = lambda *shape: torch.randint(-128, 128, shape, device=DEV, generator=gen, dtype=torch.int8)
        a, b, c0, bias = mk(m, k), mk(k, n), mk(m, n), mk(n)
        sa = a.t().contiguous() if ta else a
        sb = b.t().contiguous() if tb else b
        c = c0.clone()
        d = _lib.GemmDesc()
        d.dtype, d.transpose_a, d.transpose_b, d.c_mode = F.ntg_dtype(a), int(ta), int(tb), mode
        d.m, d.k, d.n, d.batches = m, k, n, 1
        if mode == _lib.C_BIAS:
            d.bias, d.bias_col_stride = bias.data_ptr(), 1
        _lib.check(lib.ntg_gemm_dev(ctypes.byref(d), sa.data_ptr(), sb.data_ptr(), c.data_ptr(), st))
        torch.cuda.synchronize()
        ref = a.double() @ b.double()
        if mode == _lib.C_ACCUMULATE:
            ref += c0.double()
        elif mode == _lib.C_BIAS:
            ref += bias.double()
        if kind == "int8":
            want = (ref.to(torch.int64) & 0xff).to(torch.uint8)
            assert torch.equal(c.view(torch.uint8), want), (m, k, n, ta, tb, mode)
        else:
            want = ref.to(torch.bfloat16)                      # correctly rounded (float64 holds the sum exactly enough)
            ulp = torch.maximum(ref.abs(), torch.tensor(1e-30, device=DEV, dtype=torch.float64)).log2().floor().exp2() * 2.0 ** -7
            err = (c.double() - want.double()).abs()
            assert bool((err <= 1.5 * ulp + 1e-4).all()), (m, k, n, ta, tb, mode, float((err / ulp).max()))
            assert float((c == want).double().mean()) > 0.97, (m, k, n, ta, tb, mode)
        del ref


def test_small_fp32_products_on_32_wide_tiles():
    """Float32 products with too few output elements for 64 x 64 tiles (config 1 is one of them): every transpose pair and C
    mode, ragged edges in m, n and k, padded rows, batches, against float64 products within the stated bound; two runs are
    bit-identical.  Rows that keep the 16-byte rule (pitches +4 / +8 / +4, sizes that are multiples of 4) take the 32 x 32-tile
    kernel on v_mfma_f32_16x16x4 -- k tails that are not whole 128-k stages, one to nine stages, edge tiles whose loads are
    clamped -- the odd pitches the register-staged kernel."""
    lib = _lib.load()
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    gen = torch.Generator(device=DEV).manual_seed(4242)
    modes = (_lib.C_OVERWRITE, _lib.C_ACCUMULATE, _lib.C_BIAS)
    i = 0
    cases = [(512, 512, 512, 1, (3, 5, 2)), (100, 300, 70, 1, (3, 5, 2)), (33, 64, 33, 1, (3, 5, 2)), (40, 1003, 50, 2, (3, 5, 2)),
             (256, 130, 250, 3, (3, 5, 2)), (65, 77, 129, 4, (3, 5, 2)),
             (512, 512, 512, 1, (4, 8, 4)), (100, 300, 72, 1, (4, 8, 4)), (36, 64, 36, 1, (0, 0, 0)), (40, 1004, 52, 2, (4, 8, 4)),
             (256, 132, 248, 3, (0, 4, 8)), (68, 76, 128, 4, (4, 8, 4)), (132, 1156, 60, 1, (0, 0, 0)), (48, 640, 36, 5, (8, 4, 4))]
    for (m, k, n, batch, pads) in cases:
        for ta, tb in TRANS:
            mode = modes[i % 3]
            i += 1
            lda, ldb, ldc = (m if ta else k) + pads[0], (k if tb else n) + pads[1], n + pads[2]
            a = torch.randn(batch, k if ta else m, lda, device=DEV, generator=gen)
            b = torch.randn(batch, n if tb else k, ldb, device=DEV, generator=gen)
            c0 = torch.randn(batch, m, ldc, device=DEV, generator=gen)
            bias = torch.randn(n, device=DEV, generator=gen)
            la = a[:, :, :m].transpose(1, 2) if ta else a[:, :, :k]
            lb = b[:, :, :k].transpose(1, 2) if tb else b[:, :, :n]
            d = _lib.GemmDesc()
            d.dtype, d.transpose_a, d.transpose_b, d.c_mode = _lib.FLOAT32, int(ta), int(tb), mode
            d.m, d.k, d.n, d.batches = m, k, n, batch
            d.lda, d.ldb, d.ldc = lda, ldb, ldc
            d.stride_a, d.stride_b, d.stride_c = a.shape[1] * lda, b.shape[1] * ldb, m * ldc
            if mode == _lib.C_BIAS:
                d.bias, d.bias_col_stride = bias.data_ptr(), 1
            # (a deep k on few tiles may be offered a split along k; no workspace is passed here, so the plain kernels run)
            outs = []
            for rep in range(2):
                c = c0.clone()
                _lib.check(lib.ntg_gemm_dev(ctypes.byref(d), a.data_ptr(), b.data_ptr(), c.data_ptr(), st))
                torch.cuda.synchronize()
                outs.append(c)
            assert torch.equal(outs[0], outs[1])
            ref = la.double() @ lb.double()
            if mode == _lib.C_ACCUMULATE:
                ref += c0[:, :, :n].double()
            elif mode == _lib.C_BIAS:
                ref += bias.double()
            tol = 1e-5 * k * float(la.abs().max() * lb.abs().max())
            assert (outs[0][:, :, :n].double() - ref).abs().max().item() <= tol, (m, k, n, batch, ta, tb, mode)
            assert torch.equal(outs[0][:, :, n:], c0[:, :, n:])                 # padding of C untouched
            # relu_ in the same launch == clamp of the plain result
            c = c0.clone()
            _lib.check(lib.ntg_gemm_relu_dev(ctypes.byref(d), a.data_ptr(), b.data_ptr(), c.data_ptr(), st))
            torch.cuda.synchronize()
            want = outs[0].clone()
            want[:, :, :n] = torch.where(outs[0][:, :, :n] > 0, outs[0][:, :, :n], torch.zeros_like(outs[0][:, :, :n]))
            assert torch.equal(c, want)


@pytest.mark.parametrize("dtype", ["bf16", np.float16], ids=["bf16", "fp16"])
def test_batched_16bit_products_split_along_the_columns(dtype):
    """A batch whose 256-wide tiles make whole rounds over the CUs plus a fraction (64 x [256 x 2304] outputs: 576 tiles)
    goes out as two launches, the leading 2048 columns of every item and the last 256 on other tiles.  Items must equal
    the same product computed alone, bit for bit (bias and C0 follow the columns), for both layouts of B."""
    bf = dtype == "bf16"
    lib = _lib.load()
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rng = np.random.default_rng(5151)
    batch, m, k, n = 64, 256, 1024, 2304
    a = to_torch(randn(rng, (batch, m, k), dtype, 0.25), DEV, bf)
    c0 = to_torch(randn(rng, (batch, m, n), dtype), DEV, bf)
    bias = to_torch(randn(rng, (n,), dtype), DEV, bf)
    for tb, mode in ((False, _lib.C_BIAS), (True, _lib.C_ACCUMULATE)):
        b = to_torch(randn(rng, (batch, n, k) if tb else (batch, k, n), dtype, 0.25), DEV, bf)
        d = _lib.GemmDesc()
        d.dtype, d.transpose_b, d.c_mode = F.ntg_dtype(a), int(tb), mode
        d.m, d.k, d.n, d.batches = m, k, n, batch
        d.stride_a, d.stride_b, d.stride_c = m * k, k * n, m * n
        if mode == _lib.C_BIAS:
            d.bias, d.bias_col_stride = bias.data_ptr(), 1
        c = c0.clone()
        _lib.check(lib.ntg_gemm_dev(ctypes.byref(d), a.data_ptr(), b.data_ptr(), c.data_ptr(), st))
        for i in (0, 17, 63):
            one = c0[i].clone()
            d1 = _lib.GemmDesc()
            d1.dtype, d1.transpose_b, d1.c_mode = d.dtype, int(tb), mode
            d1.m, d1.k, d1.n, d1.batches = m, k, n, 1
            if mode == _lib.C_BIAS:
                d1.bias, d1.bias_col_stride = bias.data_ptr(), 1
            _lib.check(lib.ntg_gemm_dev(ctypes.byref(d1), a[i].data_ptr(), b[i].data_ptr(), one.data_ptr(), st))
            torch.cuda.synchronize()
            assert torch.equal(c[i].view(torch.int16), one.view(torch.int16)), (tb, mode, i)
            bi = b[i].t() if tb else b[i]
            ref = a[i].double() @ bi.double() + (c0[i].double() if mode == _lib.C_ACCUMULATE else bias.double())
            assert (one.double() - ref).abs().max().item() <= HALF_REL * ref.abs().max().item()


@pytest.mark.parametrize("dtype", ["bf16", np.float16], ids=["bf16", "fp16"])
def test_16bit_products_on_deep_k_steps(dtype):
    """Mid-sized 16-bit products (128 x 128 and 128 x 256 tiles) run on the kernels whose K-step is 128 bytes of
    k per row.  All four storage forms, edges that are not multiples of the tile, k that is not a multiple of the 64-element
    K-step (tails of 8 and 40), overwrite / accumulate / bias: every element is the once-rounded exact result (within the
    float32 accumulation bound), and a strip of 64 columns computed as a product of its own -- on 64 x 64 tiles, 64-byte
    K-steps -- has the same bits: the order of summation over k does not depend on the kernel."""
    from util import assert_one_rounding
    bf = dtype == "bf16"
    fmt = "bf16" if bf else "f16"
    lib = _lib.load()
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rng = np.random.default_rng(6464)
    # (the last two take 128 x 256 tiles: three stages of 48 KiB)
    cases = [(1536, 4136, 1528, _lib.C_ACCUMULATE), (776, 3080, 4040, _lib.C_BIAS), (2048, 2048, 2048, _lib.C_OVERWRITE),
             (264, 4104, 5000, _lib.C_ACCUMULATE), (2304, 2312, 2296, _lib.C_BIAS), (520, 4104, 11000, _lib.C_ACCUMULATE)]
    for m, k, n, mode in cases:
        for ta in (False, True):
            for tb in (False, True):
                a = to_torch(randn(rng, (k, m) if ta else (m, k), dtype, 0.25), DEV, bf)
                b = to_torch(randn(rng, (n, k) if tb else (k, n), dtype, 0.25), DEV, bf)
                c0 = to_torch(randn(rng, (m, n), dtype), DEV, bf)
                bias = to_torch(randn(rng, (n,), dtype), DEV, bf)

                def run(ncols, out, ldc):
                    d = _lib.GemmDesc()
                    d.dtype, d.transpose_a, d.transpose_b, d.c_mode = F.ntg_dtype(a), int(ta), int(tb), mode
                    d.m, d.k, d.n, d.batches = m, k, ncols, 1
                    d.lda, d.ldb, d.ldc = (m if ta else k), (k if tb else n), ldc
                    if mode == _lib.C_BIAS:
                        d.bias, d.bias_col_stride = bias.data_ptr(), 1
                    _lib.check(lib.ntg_gemm_dev(ctypes.byref(d), a.data_ptr(), b.data_ptr(), out.data_ptr(), st))

                c = c0.clone()
                run(n, c, n)
                strip = c0[:, :64].contiguous()
                run(64, strip, 64)
                torch.cuda.synchronize()
                what = f"{fmt} {m}x{k}x{n} ta={ta} tb={tb} mode={mode}"
                assert torch.equal(c[:, :64].contiguous().view(torch.int16), strip.view(torch.int16)), what
                al = (a.t() if ta else a).double()
                bl = (b.t() if tb else b).double()
                add = c0.double() if mode == _lib.C_ACCUMULATE else bias.double().expand(m, n) if mode == _lib.C_BIAS else torch.zeros(m, n, device=DEV, dtype=torch.float64)
                ref = al @ bl + add
                spread = add.abs() + ((al * al) @ (bl * bl)).sqrt()
                # (Float16 at k = 4000: the float32 accumulation bound is a good part of an ulp, so fewer elements are clear of a boundary)
                assert_one_rounding(c.double().cpu().numpy(), ref.cpu().numpy(), spread.cpu().numpy(), k, fmt, what, min_exact=0.75 if bf else 0.2)


def test_deep_k_steps_at_their_shortest_k():
    """The tile choice puts products on the 128-byte K-step kernels from k = 304 on (128 x 256 tiles, a batch of two
    2112 x 3840 outputs) and k = 536 (128 x 128 tiles): five to nine K-steps, so the loops end inside their first rounds
    over the stages, with a k tail (304 = 4 x 64 + 48, 536 = 8 x 64 + 24).  BFloat16 against the once-rounded exact result
    and, bit for bit, against a strip of 64 columns computed on 64 x 64 tiles; Int8 (k = 304 is two K-steps of 128 and a tail
    of 48) against exact integer arithmetic."""
    from util import assert_one_rounding
    lib = _lib.load()
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rng = np.random.default_rng(304)
    for batch, m, k, n in ((2, 2112, 304, 3840), (1, 576, 536, 3648)):
        for ta, tb in ((False, False), (False, True), (True, False)):
            a = to_torch(randn(rng, (batch, k, m) if ta else (batch, m, k), "bf16", 0.25), DEV, True)
            b = to_torch(randn(rng, (batch, n, k) if tb else (batch, k, n), "bf16", 0.25), DEV, True)
            c0 = to_torch(randn(rng, (batch, m, n), "bf16"), DEV, True)

            def run(ncols, out, ldc):
                d = _lib.GemmDesc()
                d.dtype, d.transpose_a, d.transpose_b, d.c_mode = F.ntg_dtype(a), int(ta), int(tb), _lib.C_ACCUMULATE
                d.m, d.k, d.n, d.batches = m, k, ncols, batch
                d.lda, d.ldb, d.ldc = (m if ta else k), (k if tb else n), ldc
                d.stride_a, d.stride_b, d.stride_c = m * k, k * n, m * ldc
                _lib.check(lib.ntg_gemm_dev(ctypes.byref(d), a.data_ptr(), b.data_ptr(), out.data_ptr(), st))

            c = c0.clone()
            run(n, c, n)
            strip = c0[:, :, :64].contiguous()
            run(64, strip, 64)
            torch.cuda.synchronize()
            what = f"bf16 {batch}x{m}x{k}x{n} ta={ta} tb={tb}"
            assert torch.equal(c[:, :, :64].contiguous().view(torch.int16), strip.view(torch.int16)), what
            al = (a.transpose(1, 2) if ta else a).double()
            bl = (b.transpose(1, 2) if tb else b).double()
            ref = al @ bl + c0.double()
            spread = c0.double().abs() + ((al * al) @ (bl * bl)).sqrt()
            assert_one_rounding(c.double().cpu().numpy(), ref.cpu().numpy(), spread.cpu().numpy(), k, "bf16", what)
    # Int8: the same batch, every value of the range, wrapping sums
    batch, m, k, n = 2, 2112, 304, 3840
    for tb in (False, True):
        a = torch.randint(-128, 128, (batch, m, k), device=DEV, dtype=torch.int8)
        b = torch.randint(-128, 128, (batch, n, k) if tb else (batch, k, n), device=DEV, dtype=torch.int8)
        c0 = torch.randint(-128, 128, (batch, m, n), device=DEV, dtype=torch.int8)
        c = c0.clone()
        d = _lib.GemmDesc()
        d.dtype, d.transpose_b, d.c_mode = F.ntg_dtype(a), int(tb), _lib.C_ACCUMULATE
        d.m, d.k, d.n, d.batches = m, k, n, batch
        d.stride_a, d.stride_b, d.stride_c = m * k, k * n, m * n
        _lib.check(lib.ntg_gemm_dev(ctypes.byref(d), a.data_ptr(), b.data_ptr(), c.data_ptr(), st))
        torch.cuda.synchronize()
        bl = (b.transpose(1, 2) if tb else b).double()
        exact = (a.double() @ bl + c0.double()).to(torch.int64)          # |sum| < 2^23: exact in float64
        want = ((exact + 128) % 256 - 128).to(torch.int8)
        assert torch.equal(c, want), ("int8", tb)


def test_host_batch_bf16_pointer_tables_on_deep_k_steps():
    """nt_matmult_batch with a mixed pattern of repeated pointers (pointer tables) at a size that takes the 128-byte
    K-step kernels: every item has the bits of the same product run alone through nt_matmult (the reference's
    batched == per-item invariant), and is the once-rounded exact result on a sample of rows."""
    from util import assert_one_rounding
    rng = np.random.default_rng(4242)
    nb, m, k, n = 3, 1536, 4104, 1528
    a = [randn(rng, (m, k), "bf16", 0.25) for _ in range(2)]
    b = [randn(rng, (k, n), "bf16", 0.25) for _ in range(2)]
    As, Bs = [a[0], a[1], a[0]], [b[0], b[0], b[1]]
    C0 = [randn(rng, (m, n), "bf16") for _ in range(nb)]
    got = [c.copy() for c in C0]
    arr = ctypes.c_void_p * nb
    lib = _lib.load()
    _lib.check(lib.ntg_matmult_batch(_lib.BFLOAT16, arr(*[x.ctypes.data for x in As]), arr(*[x.ctypes.data for x in Bs]),
                                     arr(*[x.ctypes.data for x in got]), nb, m, k, k, n, 0, 0))
    rows = np.arange(0, m, 37)
    for i in range(nb):
        single = host_matmult(As[i], Bs[i], C0[i].copy(), m, k, n, False, False, _lib.BFLOAT16)
        assert single.tobytes() == got[i].tobytes(), i
        al, bl, cl = to_f64(As[i][rows], True), to_f64(Bs[i], True), to_f64(C0[i][rows], True)
        assert_one_rounding(to_f64(got[i][rows], True), al @ bl + cl, np.abs(cl) + np.sqrt((al * al) @ (bl * bl)), k, "bf16", f"item {i}")


@pytest.mark.parametrize("dtype", [np.float32, np.float64, "bf16", np.float16], ids=["fp32", "fp64", "bf16", "fp16"])
@pytest.mark.parametrize("shape", [(256, 256, 256), (64, 8192, 64), (48, 300, 100), (16, 512, 256), (256, 1024, 256), (256, 8192, 512),
                                   (512, 512, 512)], ids=lambda s: "x".join(map(str, s)))
def test_item_is_the_same_alone_and_in_every_batch_form(dtype, shape):
    """The reference's batched == per-item rule (tests/src/matmult_test.cpp:108-189: every item of a list product equals the
    product of the pair alone, element for element) at sizes where this library has kernels that sum over k in different
    orders: products with few output tiles and a deep k are split along k when a workspace is offered (64 x 8192 x 64,
    256 x 1024 x 256, 256 x 8192 x 512), 16 rows take the streaming kernel, the others the tile kernels.  Which order an item
    gets may depend on the item's own sizes only: alone, as every item of strided batches of 3 and 8 (distinct items), in a
    device pointer table (with and without the caller's vouch for the entries' alignment), through the host entry points
    with distinct and with repeated pointers -- the bits are the same."""
    m, k, n = shape
    bf = dtype == "bf16"
    rng = np.random.default_rng(9100 + m + k)
    nb = 8
    a = to_torch(randn(rng, (nb, m, k), dtype, 0.5), DEV, bf)
    b = to_torch(randn(rng, (nb, k, n), dtype, 0.5), DEV, bf)
    bits = lambda t: t.contiguous().view(torch.int16 if t.element_size() == 2 else torch.int32 if t.element_size() == 4 else torch.int64)
    lib = _lib.load()
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for ta, tb in ((False, False), (False, True), (True, False)):
        sa = a.transpose(1, 2).contiguous() if ta else a
        sb = b.transpose(1, 2).contiguous() if tb else b
        alone = [F.matmult(sa[i], sb[i], None, ta, tb) for i in range(nb)]
        ref = torch.matmul(a[0].double(), b[0].double())
        tol = 1e-5 * k * float(a[0].abs().max() * b[0].abs().max()) if dtype in (np.float32, np.float64) else HALF_REL * float(ref.abs().max())
        assert (alone[0].double() - ref).abs().max().item() <= tol
        for batch in (3, 8):
            out = F.matmult(sa[:batch].contiguous(), sb[:batch].contiguous(), None, ta, tb)
            for i in range(batch):
                assert torch.equal(bits(out[i]), bits(alone[i])), (shape, ta, tb, "strided batch", batch, i)
        # one matrix against every item (stride 0 on B): still the item's own result
        out = F.matmult(sa[:3].contiguous(), sb[1], None, ta, tb)
        assert torch.equal(bits(out[1]), bits(alone[1])), (shape, ta, tb, "broadcast b")
        # device pointer tables: never split along k, so they stand for the items only where an item alone is not split either
        d = _lib.GemmDesc()
        d.dtype = code_of(dtype)
        d.transpose_a, d.transpose_b, d.c_mode = int(ta), int(tb), _lib.C_OVERWRITE
        d.m, d.k, d.n, d.batches = m, k, n, 1
        if lib.ntg_gemm_workspace_bytes(ctypes.byref(d)) == 0:
            d.batches = 5
            order = [4, 0, 2, 2, 7]
            for flags in (_lib.GEMM_PTRS_ALIGNED16, 0):
                d.flags = flags
                c = torch.zeros((5, m, n), dtype=a.dtype, device=DEV)
                tab = torch.tensor([sa[i].data_ptr() for i in order] + [sb[i].data_ptr() for i in order] + [c[j].data_ptr() for j in range(5)],
                                   dtype=torch.int64, device=DEV)
                _lib.check(lib.ntg_gemm_ptrs_dev(ctypes.byref(d), tab.data_ptr(), tab.data_ptr() + 40, tab.data_ptr() + 80, st))
                torch.cuda.synchronize()
                for j, i in enumerate(order):
                    assert torch.equal(bits(c[j]), bits(alone[i])), (shape, ta, tb, "pointer table", flags, j)
    # the host entry points (the drop-in seam): nt_matmult against nt_matmult_batch with distinct and with repeated pointers
    if dtype == "bf16":
        return
    ha = [a[i].cpu().numpy() for i in range(4)]
    hb = [b[i].cpu().numpy() for i in range(4)]
    code = code_of(dtype)
    single = []
    for i in range(4):
        c = np.zeros((m, n), ha[0].dtype)
        host_matmult(ha[i], hb[i], c, m, k, n, False, False, code)
        single.append(c)
        # (Float32: the seam keeps the reference's order of summation -- NTG_GEMM_KEEP_K_ORDER -- so it stands beside the device
        #  entry under the same flag; the other dtypes beside the functional face, workspace forms included)
        dev_alone = dev_matmult(ha[i], hb[i], np.zeros((m, n), ha[0].dtype), m, k, n, False, False, dtype, mode=_lib.C_OVERWRITE,
                                flags=_lib.GEMM_KEEP_K_ORDER) if dtype is np.float32 else alone_np(a[i], b[i])
        assert np.array_equal(c.view(np.uint8), dev_alone.view(np.uint8)), (shape, "host alone == device alone", i)
    arr = ctypes.c_void_p * 4
    for name, ia, ib in (("distinct", [0, 1, 2, 3], [0, 1, 2, 3]), ("shared b", [0, 1, 2, 3], [1, 1, 1, 1]), ("mixed", [0, 1, 0, 1], [2, 2, 3, 3])):
        got = [np.zeros((m, n), ha[0].dtype) for _ in range(4)]
        _lib.check(lib.ntg_matmult_batch(code, arr(*[ha[i].ctypes.data for i in ia]), arr(*[hb[i].ctypes.data for i in ib]),
                                         arr(*[g.ctypes.data for g in got]), 4, m, k, k, n, 0, 0))
        for j in range(4):
            want = single[ia[j]] if ia[j] == ib[j] else None
            if want is None:
                want = np.zeros((m, n), ha[0].dtype)
                host_matmult(ha[ia[j]], hb[ib[j]], want, m, k, n, False, False, code)
            assert np.array_equal(got[j].view(np.uint8), want.view(np.uint8)), (shape, "host batch", name, j)


def alone_np(a, b):
    """one product on device tensors through the functional face, as a numpy array"""
    return from_torch(F.matmult(a, b))


def test_host_entry_pipelined_panels_and_groups_bit_identical_to_the_device_entry():
    """Host-pointer calls of 48 MiB and more cross the link in panels (rows of one product, groups of items of a batch):
    uploads on one stream, the panels' products on a second, downloads on a third.  Every storage form, a C that is
    zeros (not uploaded: the products overwrite) and one that is not (uploaded, accumulated), 16-bit operands, a last panel
    that is not whole, a batch with distinct matrices and one with a shared B -- each bit-identical to the device entry
    point on the whole product / batch."""
    lib = _lib.load()
    rng = np.random.default_rng(616)
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for (m, k, n, dtype, ta, tb) in [(3100, 2000, 2600, np.float32, False, False), (2900, 2100, 2500, np.float32, True, False),
                                      (3000, 2056, 2504, np.float32, False, True), (5000, 3000, 4104, "bf16", False, False),
                                      (2600, 1500, 2200, np.float64, True, True)]:
        a, b, sa, sb, c0 = make_inputs(rng, m, k, n, dtype, ta, tb)
        for zero in (False, True):
            start = np.zeros_like(c0) if zero else c0
            want = dev_matmult(sa, sb, start, m, k, n, ta, tb, dtype)
            got = host_matmult(sa, sb, start.copy(), m, k, n, ta, tb, code_of(dtype))
            assert got.tobytes() == want.tobytes(), (m, k, n, dtype, ta, tb, zero)
    # batches: 9 items of 1000 x 1100 x 1200 (groups of two; the last group has one), distinct and with one B for all
    nb, m, k, n = 9, 1000, 1100, 1200
    As = [rng.standard_normal((m, k)).astype(np.float32) for _ in range(nb)]
    Bs = [rng.standard_normal((k, n)).astype(np.float32) for _ in range(nb)]
    arr = lambda xs: (ctypes.c_void_p * len(xs))(*[x.ctypes.data for x in xs])
    for shared_b in (False, True):
        for zero in (False, True):
            C0 = [np.zeros((m, n), np.float32) if zero else rng.standard_normal((m, n)).astype(np.float32) for _ in range(nb)]
            Bl = [Bs[0]] * nb if shared_b else Bs
            got = [c.copy() for c in C0]
            _lib.check(lib.ntg_matmult_batch(_lib.FLOAT32, arr(As), arr(Bl), arr(got), nb, m, k, k, n, 0, 0))
            # the device entry on the whole batch
            da = torch.from_numpy(np.stack(As)).to(DEV)
            db = torch.from_numpy(Bs[0] if shared_b else np.stack(Bs)).to(DEV)
            dc = torch.from_numpy(np.stack(C0)).to(DEV)
            d = _lib.GemmDesc()
            d.dtype, d.c_mode = _lib.FLOAT32, _lib.C_ACCUMULATE
            d.m, d.k, d.n, d.batches = m, k, n, nb
            d.stride_a, d.stride_b, d.stride_c = m * k, 0 if shared_b else k * n, m * n
            _lib.check(lib.ntg_gemm_dev(ctypes.byref(d), da.data_ptr(), db.data_ptr(), dc.data_ptr(), st))
            torch.cuda.synchronize()
            want = dc.cpu().numpy()
            for i in range(nb):
                assert got[i].tobytes() == want[i].tobytes(), ("batch", shared_b, zero, i)
    assert lib.ntg_release_host_buffers() == 0


@pytest.mark.parametrize("shape", [(128, 256, 128), (512, 512, 512), (300, 1000, 260), (130, 22, 66), (33, 77, 35), (1860, 36, 132), (96, 4100, 64)],
                         ids=lambda s: "x".join(map(str, s)))
def test_fp32_product_is_the_reference_chain_bit_for_bit(shape):
    """Float32 on the matrix pipe, bit for bit the reference's own sum: every output element is c = 0; for k ascending:
    c = fma(a[i, k], b[k, j], c) (the closed form of the oracle, which the reference's k-outer loop nest computes).  Holds
    because one v_mfma_f32_32x32x2 is two fused multiply-adds in a row per element and the kernels feed it k in ascending
    order.  All four storage forms; shapes on 128- and 64-wide tiles of the DMA-fed kernel, with k tails and ragged edges, and
    shapes whose rows are not 16-byte multiples (the register-staged kernel); no workspace, so nothing is split along k."""
    m, k, n = shape
    rng = np.random.default_rng(4242 + m + k + n)
    a = randn(rng, (m, k), np.float32)
    b = randn(rng, (k, n), np.float32)
    if k >= 64:       # wide dynamic range: rounding differences could not hide
        a[:, ::7] *= 1000.0
        b[5::11, :] *= 1e-3
    for ta, tb in TRANS:
        sa = np.ascontiguousarray(a.T) if ta else a
        sb = np.ascontiguousarray(b.T) if tb else b
        want = oracle.matmult2d(sa, sb, None, ta, tb)
        got = dev_matmult(sa, sb, np.zeros((m, n), np.float32), m, k, n, ta, tb, np.float32, mode=_lib.C_OVERWRITE)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (shape, ta, tb, int((got != want).sum()))
        # the accumulate contract: the chain starts from what C holds (nt_matmult's C += ...)
        c0 = randn(rng, (m, n), np.float32) * 50.0
        want = oracle.matmult2d(sa, sb, c0.copy(), ta, tb)
        got = dev_matmult(sa, sb, c0, m, k, n, ta, tb, np.float32, mode=_lib.C_ACCUMULATE)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (shape, ta, tb, "accumulate", int((got != want).sum()))
    # cpu::linear: the bias row is the starting value of every row's chains (matmult_cpu.cpp:1637-1647)
    bias = randn(rng, (n,), np.float32) * 20.0
    w_nk = np.ascontiguousarray(b.T)
    want = oracle.linear(a, w_nk, bias, False, True)
    tx, tw, tbias = to_torch(a, DEV, False), to_torch(w_nk, DEV, False), to_torch(bias, DEV, False)
    ty = torch.empty((m, n), dtype=torch.float32, device=DEV)
    d = _lib.GemmDesc()
    d.dtype, d.transpose_b, d.c_mode = _lib.FLOAT32, 1, _lib.C_BIAS
    d.m, d.k, d.n, d.batches = m, k, n, 1
    d.bias, d.bias_col_stride = tbias.data_ptr(), 1
    _lib.check(_lib.load().ntg_gemm_dev(ctypes.byref(d), tx.data_ptr(), tw.data_ptr(), ty.data_ptr(),
                                        ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
    torch.cuda.synchronize()
    got = ty.cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (shape, "linear", int((got != want).sum()))


@pytest.mark.parametrize("shape", [(16, 1024, 640), (64, 8192, 64), (300, 257, 123), (2048, 3000, 2048)], ids=lambda s: "x".join(map(str, s)))
def test_host_entry_points_fp32_are_the_reference_chain_bit_for_bit(shape):
    """The drop-in seam in Float32: nt_matmult / nt_matmult_batch / linear on host memory give the bits of the reference's
    own loop nest (the oracle's tiled restatement == its closed form): 16 rows (the streaming kernel is bypassed), few tiles
    with a deep k (no split along k at the seam), ragged sizes on the register-staged kernel, and a product large enough to
    cross the link in panels; C0 random (the accumulate contract), two storage forms."""
    m, k, n = shape
    rng = np.random.default_rng(777 + m)
    lib = _lib.load()
    a = randn(rng, (m, k), np.float32)
    b = randn(rng, (k, n), np.float32)
    for ta, tb in ((False, False), (True, True)) if m < 2048 else ((False, True),):
        sa = np.ascontiguousarray(a.T) if ta else a
        sb = np.ascontiguousarray(b.T) if tb else b
        c0 = randn(rng, (m, n), np.float32) * 10.0
        want = oracle.matmult2d(sa, sb, c0.copy(), ta, tb, kind="tiled", threads=8)
        got = host_matmult(sa, sb, c0.copy(), m, k, n, ta, tb, _lib.FLOAT32)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (shape, ta, tb, int((got != want).sum()))
    if m >= 2048:
        return
    # a batch with a repeated operand, and linear with its bias row
    items = 3
    As = [randn(rng, (m, k), np.float32) for _ in range(items)]
    Cs = [randn(rng, (m, n), np.float32) for _ in range(items)]
    want = [oracle.matmult2d(As[i], b, Cs[i].copy(), False, False, kind="tiled", threads=8) for i in range(items)]
    pa = (ctypes.c_void_p * items)(*[x.ctypes.data for x in As])
    pb = (ctypes.c_void_p * items)(*[b.ctypes.data] * items)
    pc = (ctypes.c_void_p * items)(*[x.ctypes.data for x in Cs])
    _lib.check(lib.ntg_matmult_batch(_lib.FLOAT32, pa, pb, pc, items, m, k, k, n, 0, 0))
    for i in range(items):
        assert np.array_equal(Cs[i].view(np.uint32), want[i].view(np.uint32)), (shape, "batch item", i)
    bias = randn(rng, (n,), np.float32) * 5.0
    w_nk = np.ascontiguousarray(b.T)
    want = oracle.linear(a, w_nk, bias, False, True)
    y = np.empty((m, n), np.float32)
    vp = lambda x: x.ctypes.data_as(ctypes.c_void_p)
    _lib.check(lib.ntg_linear(_lib.FLOAT32, vp(a), vp(w_nk), vp(bias), vp(y), m, k, n, 0, 1, 1, n))
    assert np.array_equal(y.view(np.uint32), want.view(np.uint32)), (shape, "linear")


@pytest.mark.parametrize("dtype", ["bf16", np.float32, np.int8, np.float64], ids=["bf16", "fp32", "int8", "fp64"])
def test_pointer_tables_without_a_vouch_find_their_alignment_on_the_device(dtype):
    """ntg_gemm_ptrs_dev without NTG_GEMM_PTRS_ALIGNED16 on products large enough to pay for it: a small kernel looks at the
    tables' entries, and the product runs on the DMA-fed kernel when all of them are 16-byte multiples, on the register-staged
    one otherwise (8-bit integers: the vector ALU's; both are launched, one of them returns at once).  Aligned tables, then
    tables with one entry moved by one element: in both cases every item has the bits of the item alone."""
    bf = dtype == "bf16"
    m, k, n, nb = (2048, 1024, 2048, 5) if dtype in (np.float32, np.float64) else (1024, 1024, 1024, 6)
    rng = np.random.default_rng(60606)
    lib = _lib.load()
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    # operands inside larger buffers, so that an entry can be moved by one element without leaving its allocation
    if dtype == np.int8:
        abuf = to_torch(rng.integers(-128, 127, (nb, m * k + 8), dtype=np.int8, endpoint=True), DEV)
        bbuf = to_torch(rng.integers(-128, 127, (nb, k * n + 8), dtype=np.int8, endpoint=True), DEV)
    else:
        abuf = to_torch(randn(rng, (nb, m * k + 8), dtype, 0.5), DEV, bf)
        bbuf = to_torch(randn(rng, (nb, k * n + 8), dtype, 0.5), DEV, bf)
    bits = lambda t: t.contiguous().view({1: torch.int8, 2: torch.int16, 4: torch.int32, 8: torch.int64}[t.element_size()])
    for shift in (0, 1):
        offs = [0] * nb
        offs[2] = shift                                   # one misaligned A, and below one misaligned B
        a = [abuf[i, offs[i]:offs[i] + m * k].view(m, k) for i in range(nb)]
        b = [bbuf[i, (shift if i == 4 else 0):(shift if i == 4 else 0) + k * n].view(k, n) for i in range(nb)]
        alone = [F.matmult(a[i].clone(), b[i].clone()) for i in range(nb)]
        c = torch.zeros((nb, m, n), dtype=abuf.dtype, device=DEV)
        d = _lib.GemmDesc()
        d.dtype = code_of(dtype)
        d.c_mode = _lib.C_OVERWRITE
        d.m, d.k, d.n, d.batches = m, k, n, nb
        tab = torch.tensor([x.data_ptr() for x in a] + [x.data_ptr() for x in b] + [c[j].data_ptr() for j in range(nb)], dtype=torch.int64, device=DEV)
        _lib.check(lib.ntg_gemm_ptrs_dev(ctypes.byref(d), tab.data_ptr(), tab.data_ptr() + 8 * nb, tab.data_ptr() + 16 * nb, st))
        torch.cuda.synchronize()
        for i in range(nb):
            assert torch.equal(bits(c[i]), bits(alone[i])), (dtype, "shift", shift, "item", i)
