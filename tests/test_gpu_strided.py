"""ntg_gemm_desc's lda / ldb / ldc and batch strides with data: A, B and C are sub-matrices of larger padded buffers
(row pitch above the row length, items further apart than a matrix, base pointers inside the buffer), compared with the
CPU oracle on contiguous copies of the same sub-views; everything in the buffers outside C's sub-views must keep its
bytes.  16-byte pitches keep the DMA-fed kernels (ring, ring64, 8-bit ring), odd pitches take the register-staged,
streaming and vector-ALU kernels; both also through the workspace forms (split along k, integer byte planes).

16-bit floating results are also held to ONE rounding: within one ulp of RNE(float64 GEMM) and bit-equal to it away
from rounding boundaries, on k that is not a multiple of any tile step -- a dropped or clamped k tail cannot pass."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from neurotensor_amd import _lib
from util import HALF_REL, assert_one_rounding, float_tol

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
TRANS = [(False, False), (False, True), (True, False), (True, True)]
# name -> (numpy dtype of the bit patterns, ntg dtype code, oracle dtype code or None)
DTYPES = {
    "f32": (np.float32, _lib.FLOAT32, None), "f64": (np.float64, _lib.FLOAT64, None), "f16": (np.float16, _lib.FLOAT16, None),
    "bf16": (np.uint16, _lib.BFLOAT16, oracle.BF16),
    "i8": (np.int8, _lib.INT8, None), "u8": (np.uint8, _lib.UINT8, None), "i16": (np.int16, _lib.INT16, None), "u16": (np.uint16, _lib.UINT16, None),
    "i32": (np.int32, _lib.INT32, None), "u32": (np.uint32, _lib.UINT32, None), "i64": (np.int64, _lib.INT64, None), "u64": (np.uint64, _lib.UINT64, None),
}
FLOATS = ("f32", "f64", "f16", "bf16")


def setup_module(module):
    assert torch.cuda.is_available(), "GPU tests need a visible MI355X"
    _lib.load()


def fill(rng, name, count, scale=1.0):
    npdt = DTYPES[name][0]
    if name == "bf16":
        return oracle.to_bf16_bits((rng.standard_normal(count) * scale).astype(np.float32))
    if name in FLOATS:
        return (rng.standard_normal(count) * scale).astype(npdt)
    info = np.iinfo(npdt)
    return rng.integers(info.min, info.max, count, dtype=npdt, endpoint=True)


def widen(name, arr):
    return oracle.from_bf16_bits(arr).astype(np.float64) if name == "bf16" else arr.astype(np.float64)


def upload(arr):
    return torch.from_numpy(arr.view(np.uint8).copy()).to(DEV)


def sub(buf, off, rows, cols, ld):
    """rows x cols view with row pitch ld starting at element off of a flat buffer"""
    return np.lib.stride_tricks.as_strided(buf[off:], (rows, cols), (ld * buf.itemsize, buf.itemsize))


def run_case(rng, name, m, k, n, ta, tb, pads, mode, batches=1, gap=0, base=0, bcast_b=False, workspace=False, one_rounding=False, flags=0, f32_bits=False):
    npdt, code, ocode = DTYPES[name]
    es = np.dtype(npdt).itemsize
    ra, ca = (k, m) if ta else (m, k)
    rb, cb = (n, k) if tb else (k, n)
    lda, ldb, ldc = ca + pads[0], cb + pads[1], n + pads[2]
    sA, sB, sC = ra * lda + gap, (0 if bcast_b else rb * ldb + gap), m * ldc + gap
    bufA = fill(rng, name, base + batches * (ra * lda + gap) + 8, 0.5)
    bufB = fill(rng, name, base + batches * (rb * ldb + gap) + 8, 0.5)
    bufC = fill(rng, name, base + batches * sC + 8)
    bias = fill(rng, name, n)
    dA, dB, dC, dbias = upload(bufA), upload(bufB), upload(bufC), upload(bias)
    d = _lib.GemmDesc()
    d.dtype, d.transpose_a, d.transpose_b, d.c_mode = code, int(ta), int(tb), mode
    d.m, d.k, d.n, d.batches = m, k, n, batches
    d.lda, d.ldb, d.ldc = lda, ldb, ldc
    d.stride_a, d.stride_b, d.stride_c = sA, sB, sC
    if mode == _lib.C_BIAS:
        d.bias, d.bias_col_stride = dbias.data_ptr(), 1
    lib = _lib.load()
    ws = None
    d.flags = flags
    if workspace == "offered":                        # whatever form the query offers for this descriptor, if any
        workspace = lib.ntg_gemm_workspace_bytes(ctypes.byref(d)) > 0
    if workspace:
        need = lib.ntg_gemm_workspace_bytes(ctypes.byref(d))
        if workspace is not True:
            need = max(need, int(workspace))          # explicit size: the query knows sizes and pitches, not the base pointers
        assert need > 0, (name, m, k, n, "expected a workspace form")
        ws = torch.empty(need, dtype=torch.uint8, device=DEV)
        d.workspace, d.workspace_bytes = ws.data_ptr(), need
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    _lib.check(lib.ntg_gemm_dev(ctypes.byref(d), dA.data_ptr() + base * es, dB.data_ptr() + base * es, dC.data_ptr() + base * es, st))
    torch.cuda.synchronize()
    got = dC.cpu().numpy().view(npdt)
    want = bufC.copy()                     # bytes outside the C sub-views must survive
    what = f"{name} {m}x{k}x{n} ta={ta} tb={tb} pads={pads} mode={mode} batches={batches} gap={gap} base={base} bcast_b={bcast_b} ws={workspace} flags={flags}"
    for bi in range(batches):
        sa = np.ascontiguousarray(sub(bufA, base + bi * sA, ra, ca, lda))
        sb = np.ascontiguousarray(sub(bufB, base + bi * sB, rb, cb, ldb))
        cview = sub(bufC, base + bi * sC, m, n, ldc)
        if mode == _lib.C_ACCUMULATE:
            c_init = np.ascontiguousarray(cview)
        elif mode == _lib.C_BIAS:
            c_init = np.ascontiguousarray(np.broadcast_to(bias, (m, n)))
        else:
            c_init = np.zeros((m, n), npdt)
        ref = oracle.matmult2d(sa, sb, c_init.copy(), ta, tb, dt=ocode) if ocode is not None else oracle.matmult2d(sa, sb, c_init.copy(), ta, tb)
        g = np.ascontiguousarray(sub(got, base + bi * sC, m, n, ldc))
        if name in FLOATS:
            al = widen(name, sa.T if ta else sa)
            bl = widen(name, sb.T if tb else sb)
            if name in ("f32", "f64"):
                err = np.abs(g.astype(np.float64) - ref.astype(np.float64)).max()
                assert err <= float_tol(k, al, bl), f"{what} item {bi}: max|d| = {err}"
                if f32_bits:       # the reference's chain of fused multiply-adds in ascending k, starting from C0: the same bits
                    assert np.array_equal(g.view(np.uint32), ref.view(np.uint32)), f"{what} item {bi}: {int((g != ref).sum())} elements differ from the chain"
            else:
                r64 = widen(name, ref)
                assert np.abs(widen(name, g) - r64).max() <= HALF_REL * max(np.abs(r64).max(), 1e-30), f"{what} item {bi}"
                if one_rounding:
                    c64 = widen(name, c_init)
                    assert_one_rounding(widen(name, g), c64 + al @ bl, np.abs(c64) + np.sqrt((al * al) @ (bl * bl)), k, name, f"{what} item {bi}",
                                        min_exact=0.75 if name == "bf16" else 0.35)    # (half has 8 x finer ulps: fewer elements clear the bound)
        else:
            assert g.tobytes() == ref.tobytes(), f"{what} item {bi}: integer result is not bit-exact"
        sub(want, base + bi * sC, m, n, ldc)[...] = g            # the computed part is checked above
    assert got.tobytes() == want.tobytes(), f"{what}: bytes outside the C sub-views changed"


# pads (lda, ldb, ldc beyond the row length): multiples of 16 elements keep 16-byte pitches for every element size
ALIGNED = (16, 32, 48)
ODD = (3, 5, 7)


@pytest.mark.parametrize("name", list(DTYPES))
def test_leading_dimensions_and_batch_strides(name):
    """general shapes: every dtype x four flag pairs x {16-byte pitches, odd pitches} x the three C modes, batches of 3
    whose items lie further apart than a matrix"""
    rng = np.random.default_rng(7700 + list(DTYPES).index(name))
    modes = (_lib.C_ACCUMULATE, _lib.C_BIAS, _lib.C_OVERWRITE)
    i = 0
    for ta, tb in TRANS:
        for pads, gap, base in ((ALIGNED, 64, 0), (ALIGNED, 0, 32), (ODD, 11, 0), (ODD, 0, 3), ((0, 0, 16), 0, 0), ((16, 0, 1), 5, 1)):
            run_case(rng, name, 144, 208, 176, ta, tb, pads, modes[i % 3], batches=3 if i % 2 == 0 else 1, gap=gap, base=base)
            i += 1
    # a broadcast B (stride 0) beside padded A and C, and ragged sizes inside padded rows
    run_case(rng, name, 70, 136, 90, False, False, (8, 16, 24), _lib.C_ACCUMULATE, batches=4, gap=40, bcast_b=True)
    run_case(rng, name, 37, 53, 29, True, True, ODD, _lib.C_BIAS, batches=2, gap=1)


@pytest.mark.parametrize("name", FLOATS)
def test_leading_dimensions_on_the_streaming_kernels(name):
    """m <= 32: the kernels that stream B once (Float32 and the 16-bit types) and whatever serves Float64"""
    rng = np.random.default_rng(7800 + FLOATS.index(name))
    for ta, tb in TRANS:
        run_case(rng, name, 16, 520, 264, ta, tb, ALIGNED, _lib.C_ACCUMULATE)
        run_case(rng, name, 7, 333, 130, ta, tb, ODD, _lib.C_BIAS, batches=2, gap=9, base=1)
        run_case(rng, name, 32, 256, 512, ta, tb, (0, 8, 8), _lib.C_OVERWRITE, batches=2, gap=0)


@pytest.mark.parametrize("name", ["bf16", "f16", "f32", "f64", "i16", "u32", "i64"])
def test_leading_dimensions_through_the_workspace_forms(name):
    """split along k (floating dtypes, few tiles and a deep k) and byte planes (wide integers) with padded operands"""
    rng = np.random.default_rng(7900 + list(DTYPES).index(name))
    if name in FLOATS:
        for (ta, tb), mode in zip(TRANS, (_lib.C_OVERWRITE, _lib.C_ACCUMULATE, _lib.C_BIAS, _lib.C_ACCUMULATE)):
            run_case(rng, name, 128, 2048, 256, ta, tb, ALIGNED, mode, workspace=True)
    else:
        for (ta, tb), mode in zip(TRANS, (_lib.C_OVERWRITE, _lib.C_ACCUMULATE, _lib.C_BIAS, _lib.C_ACCUMULATE)):
            run_case(rng, name, 512, 520, 520, ta, tb, ODD, mode, batches=2, gap=13, base=1, workspace=True)


@pytest.mark.parametrize("name", ["bf16", "f16"])
def test_16bit_results_are_rounded_once_on_ragged_k(name):
    """k = 1001, 1000, 1016, 40, 8: not multiples of the 32-wide K-step (nor, for 1001, of a 16-byte chunk: the
    register-staged kernel), in every flag pair and kernel family (ring tiles of every size via the batch count and the
    shape, streaming kernel, split along k); one rounding of the exact sum, C0 included."""
    rng = np.random.default_rng(8000 + FLOATS.index(name))
    for ta, tb in TRANS:
        run_case(rng, name, 136, 1001, 152, ta, tb, (0, 0, 0), _lib.C_ACCUMULATE, one_rounding=True)        # odd rows: register-staged
        run_case(rng, name, 136, 1000, 152, ta, tb, (0, 0, 0), _lib.C_ACCUMULATE, one_rounding=True)        # 16-byte rows: ring, ragged
        run_case(rng, name, 264, 1016, 520, ta, tb, (8, 8, 8), _lib.C_BIAS, one_rounding=True)
        run_case(rng, name, 64, 40, 72, ta, tb, (0, 0, 0), _lib.C_OVERWRITE, batches=5, one_rounding=True)
        run_case(rng, name, 16, 1000, 136, ta, tb, (0, 0, 0), _lib.C_ACCUMULATE, one_rounding=True)         # streaming kernel
        run_case(rng, name, 8, 8, 8, ta, tb, (0, 0, 0), _lib.C_ACCUMULATE, one_rounding=True)
    run_case(rng, name, 128, 2080, 264, False, True, (0, 0, 0), _lib.C_ACCUMULATE, workspace=True, one_rounding=True)
    run_case(rng, name, 520, 1544, 776, False, False, (0, 0, 0), _lib.C_ACCUMULATE, one_rounding=True)      # 256-wide tiles, ragged everywhere


@pytest.mark.parametrize("name", ["bf16", "f16", "i8", "u8", "f32", "f64"])
def test_rows_that_are_not_16_byte_multiples_through_padded_copies(name):
    """Large 8-bit, 16-bit, Float32 and Float64 products whose pitches, sizes or base pointers miss the 16-byte rule are offered
    a workspace (ntg_gemm_workspace_bytes) with which the operands are copied into zero-padded rows and the DMA-fed kernel runs:
    every flag pair, the three C modes, batches with a broadcast operand, odd k / n / m and odd base pointers;
    integers bit-exact against the oracle, 16-bit floats held to one rounding, Float32 / Float64 within their bound."""
    rng = np.random.default_rng(8100 + list(DTYPES).index(name))
    half = name in ("bf16", "f16")
    m, k, n = (1304, 1001, 1702) if half else (1700, 1501, 1702) if name == "f32" else (2100, 2001, 2053) if name == "f64" else (520, 1001, 530)
    modes = (_lib.C_ACCUMULATE, _lib.C_BIAS, _lib.C_OVERWRITE, _lib.C_ACCUMULATE)
    for (ta, tb), mode in zip(TRANS, modes):
        run_case(rng, name, m, k, n, ta, tb, (0, 0, 0), mode, workspace=True, one_rounding=half)             # odd k: A and B padded, C as it lies
    run_case(rng, name, m + 3, k + 7, n + 1, True, False, ODD, _lib.C_BIAS, base=1, workspace=True, one_rounding=half)   # everything odd, C padded too
    run_case(rng, name, m, k + 7, n - 6, False, True, (0, 8, 5), _lib.C_ACCUMULATE, batches=2, gap=3, workspace=True, one_rounding=half)
    run_case(rng, name, m, 1008, n - 6, False, False, (0, 0, 0), _lib.C_OVERWRITE, batches=2, bcast_b=True, base=3, workspace=64 << 20, one_rounding=half)   # only the base pointers are odd
    if True:
        # only k misses the chunk and an operand stored [k][m] / [k][n] keeps the 16-byte rule: it is read where it lies and only
        # its last k-rows are copied (several k tails, among them one whose padded size is a whole K-step); Float32 must be
        # the reference's bits
        f32 = name == "f32"
        m2, n2 = (1700, 1704) if f32 else (1304, 1712) if half else (2100, 2056) if name == "f64" else (528, 544)
        ks = (1501, 1502, 1503, 1535) if f32 else (1001, 1003, 1017, 1087) if half else (2001, 2003, 2005, 2047) if name == "f64" else (1001, 1009, 1023, 1090)
        for (ta, tb), mode, k2 in zip(TRANS, modes, ks):
            run_case(rng, name, m2, k2, n2, ta, tb, (0, 0, 0), mode, workspace=True, one_rounding=half,
                     flags=_lib.GEMM_KEEP_K_ORDER if f32 else 0, f32_bits=f32)
        run_case(rng, name, m2, ks[0], n2, False, False, (0, 16, 16), _lib.C_ACCUMULATE, batches=2, gap=16, workspace=True, one_rounding=half)
        run_case(rng, name, m2, ks[1] + 8, n2, True, False, (16, 0, 0), _lib.C_BIAS, batches=3, bcast_b=True, workspace=True, one_rounding=half)
        if f32:
            run_case(rng, name, 520, 16385, 512, False, False, (0, 0, 0), _lib.C_OVERWRITE, workspace=True)          # few tiles, a deep k
        if half:
            # products that go out as two launches with shifted operand pointers (rows / columns split, a batch in two parts)
            run_case(rng, name, 2056, 1001, 2320, False, False, (0, 0, 0), _lib.C_ACCUMULATE, workspace=True, one_rounding=True)
            run_case(rng, name, 2320, 1001, 2056, True, False, (0, 0, 0), _lib.C_OVERWRITE, workspace=True, one_rounding=True)
            run_case(rng, name, 264, 1001, 2304, False, False, (0, 0, 0), _lib.C_ACCUMULATE, batches=33, workspace=True, one_rounding=True)

def _random_dim(rng, hi):
    """sizes that sit on, just below and just above the tile edges, tiny ones, multiples of 8 and anything else"""
    kind = int(rng.integers(0, 4))
    if kind == 0:
        return int(rng.integers(1, 40))
    if kind == 1:
        d = int(rng.choice([32, 64, 128, 256, 512])) * int(rng.integers(1, 4)) + int(rng.choice([-8, -1, 0, 0, 1, 4, 8]))
        return max(1, min(d, hi))
    if kind == 2:
        return 8 * int(rng.integers(1, hi // 8 + 1))
    return int(rng.integers(1, hi + 1))


@pytest.mark.parametrize("name", list(DTYPES))
def test_seeded_random_shapes(name):
    """A seeded sweep over what the fixed cases above pick by hand: sizes around every tile edge, the four storage forms, the
    three C modes, pitches that keep or miss the 16-byte rule, batches with gaps, odd base pointers and a broadcast B, with
    and without the workspace form that the query offers.  Integers bit-exact, 16-bit floats within 2e-2 of max|C|,
    Float32 / Float64 within 1e-5 K max|A| max|B|; Float32 without a split along k (no workspace, or NTG_GEMM_KEEP_K_ORDER)
    and above the streaming kernel's 32 rows, or with the flag at any size, must be the reference's chain bit for bit."""
    import os
    rounds = int(os.environ.get("NTG_TEST_SWEEP_ROUNDS", "1"))     # (more of the same from further seeds, for a longer run by hand)
    rng = np.random.default_rng(9100 + list(DTYPES).index(name))
    modes = (_lib.C_ACCUMULATE, _lib.C_BIAS, _lib.C_OVERWRITE)
    done = 0
    while done < 40 * rounds:
        m, k, n = _random_dim(rng, 700), _random_dim(rng, 1400), _random_dim(rng, 700)
        batches = int(rng.choice([1, 1, 1, 2, 5]))
        if m * k * n * batches > 1.2e8:
            continue
        ta, tb = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        pads = ALIGNED if rng.integers(0, 3) == 0 else ODD if rng.integers(0, 2) == 0 else (0, 0, 0)
        gap = int(rng.choice([0, 0, 16, 7])) if batches > 1 else 0
        base = int(rng.choice([0, 0, 0, 16, 3]))
        bcast_b = batches > 1 and bool(rng.integers(0, 3) == 0)
        keep = name == "f32" and bool(rng.integers(0, 2))
        ws = "offered" if rng.integers(0, 2) else False
        # (the chain is kept by the flag; without it only where neither a split along k nor the streaming kernel is in reach)
        bits = name == "f32" and (keep or (ws is False and m > 32))
        run_case(rng, name, m, k, n, ta, tb, pads, modes[int(rng.integers(0, 3))], batches=batches, gap=gap, base=base, bcast_b=bcast_b,
                 workspace=ws, flags=_lib.GEMM_KEEP_K_ORDER if keep else 0, f32_bits=bits)
        done += 1
