"""Pins the CPU oracle's GEMM arithmetic without the reference binary.

Each check is chosen so that a plausible restatement mistake (dropped term,
transposed operand, wrong index form, wrong rounding point) fails it:
  * float64 numpy GEMM on the same inputs (value-level),
  * identity / permutation operands (exact),
  * all four transpose flag combinations == explicit transposes (bitwise),
  * accumulate contract C0 != 0,
  * tiled k-outer restatement == closed form == literal triple loop (bitwise),
  * integer wraparound vs Python big-int arithmetic (exact),
  * Float16: software half conversion vs numpy for all 65536 patterns, and the
    16-wide k-tile rounding schedule vs an independent numpy restatement.
"""
import numpy as np
import pytest

import oracle


def rng(seed):
    return np.random.default_rng(seed)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("ta,tb", [(False, False), (False, True), (True, False), (True, True)])
def test_float_vs_numpy_and_transposes(dtype, ta, tb):
    r = rng(1)
    m, k, n = 37, 53, 29
    a = r.standard_normal((m, k)).astype(dtype)
    b = r.standard_normal((k, n)).astype(dtype)
    base = oracle.matmult2d(a, b)
    sa = np.ascontiguousarray(a.T) if ta else a
    sb = np.ascontiguousarray(b.T) if tb else b
    got = oracle.matmult2d(sa, sb, ta=ta, tb=tb)
    assert got.tobytes() == base.tobytes()          # flags only change addressing
    ref = a.astype(np.float64) @ b.astype(np.float64)
    tol = (1e-6 if dtype == np.float32 else 1e-14) * k * np.abs(a).max() * np.abs(b).max()
    assert np.abs(got - ref).max() <= tol


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.float16, np.int32, np.int64, np.int16, np.int8, np.uint8, np.uint32])
def test_closed_equals_naive_bitwise(dtype):
    r = rng(2)
    m, k, n = 9, 35, 11
    if np.issubdtype(dtype, np.floating):
        a = r.standard_normal((m, k)).astype(dtype)
        b = r.standard_normal((k, n)).astype(dtype)
        c0 = r.standard_normal((m, n)).astype(dtype)
    else:
        info = np.iinfo(dtype)
        a = r.integers(info.min, info.max, (m, k), dtype=dtype, endpoint=True)
        b = r.integers(info.min, info.max, (k, n), dtype=dtype, endpoint=True)
        c0 = r.integers(info.min, info.max, (m, n), dtype=dtype, endpoint=True)
    for ta in (False, True):
        for tb in (False, True):
            sa = np.ascontiguousarray(a.T) if ta else a
            sb = np.ascontiguousarray(b.T) if tb else b
            c1 = oracle.matmult2d(sa, sb, c0.copy(), ta, tb, kind="closed")
            c2 = oracle.matmult2d(sa, sb, c0.copy(), ta, tb, kind="naive")
            assert c1.tobytes() == c2.tobytes()


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.float16, np.int32, np.int64])
@pytest.mark.parametrize("shape", [(16, 16, 16), (33, 50, 17), (1, 7, 1), (70, 19, 130), (5, 16, 5)])
def test_tiled_equals_closed_bitwise(dtype, shape):
    """The k-tile-outermost packed loop nest is per element the same ascending-k chain."""
    r = rng(3)
    m, k, n = shape
    if np.issubdtype(dtype, np.floating):
        a = r.standard_normal((m, k)).astype(dtype)
        b = r.standard_normal((k, n)).astype(dtype)
        c0 = r.standard_normal((m, n)).astype(dtype)
    else:
        a = r.integers(-2**31, 2**31 - 1, (m, k)).astype(dtype)
        b = r.integers(-2**31, 2**31 - 1, (k, n)).astype(dtype)
        c0 = r.integers(-100, 100, (m, n)).astype(dtype)
    for ta in (False, True):
        for tb in (False, True):
            sa = np.ascontiguousarray(a.T) if ta else a
            sb = np.ascontiguousarray(b.T) if tb else b
            c1 = oracle.matmult2d(sa, sb, c0.copy(), ta, tb, kind="closed")
            c2 = oracle.matmult2d(sa, sb, c0.copy(), ta, tb, kind="tiled", threads=3)
            assert c1.tobytes() == c2.tobytes(), (dtype, shape, ta, tb)


def test_tiled_crosses_pack_block_boundary():
    """n > 7056 (=16*21*21) exercises the second j block of the fp32 packed path."""
    r = rng(4)
    m, k, n = 3, 20, 7056 + 21
    a = r.standard_normal((m, k)).astype(np.float32)
    b = r.standard_normal((k, n)).astype(np.float32)
    c1 = oracle.matmult2d(a, b, kind="closed")
    c2 = oracle.matmult2d(a, b, kind="tiled", threads=2)
    assert c1.tobytes() == c2.tobytes()
    bt = np.ascontiguousarray(b.T)
    c3 = oracle.matmult2d(a, bt, tb=True, kind="tiled", threads=2)
    assert c1.tobytes() == c3.tobytes()


def test_identity_permutation_and_accumulate():
    r = rng(5)
    n = 24
    x = r.standard_normal((n, n)).astype(np.float32)
    eye = np.eye(n, dtype=np.float32)
    assert np.array_equal(oracle.matmult2d(x, eye), x)
    assert np.array_equal(oracle.matmult2d(eye, x), x)
    perm = r.permutation(n)
    P = eye[perm]
    assert np.array_equal(oracle.matmult2d(P, x), x[perm])
    assert np.array_equal(oracle.matmult2d(x, P, tb=True), x[:, perm])   # x . P^T
    c0 = r.standard_normal((n, n)).astype(np.float32)
    got = oracle.matmult2d(x, eye, c0.copy())
    assert np.array_equal(got, c0 + x)               # one fused step per element: fma(x,1,c0)


@pytest.mark.parametrize("dtype,bits", [(np.int8, 8), (np.int16, 16), (np.int32, 32), (np.int64, 64), (np.uint8, 8), (np.uint32, 32), (np.uint64, 64)])
def test_integer_wraparound_exact(dtype, bits):
    r = rng(6)
    m, k, n = 5, 9, 4
    info = np.iinfo(dtype)
    a = r.integers(info.min, info.max, (m, k), dtype=dtype, endpoint=True)
    b = r.integers(info.min, info.max, (k, n), dtype=dtype, endpoint=True)
    c0 = r.integers(info.min, info.max, (m, n), dtype=dtype, endpoint=True)
    got = oracle.matmult2d(a, b, c0.copy())
    mod = 1 << bits
    for i in range(m):
        for j in range(n):
            v = int(c0[i, j]) + sum(int(a[i, t]) * int(b[t, j]) for t in range(k))
            v %= mod
            if info.min < 0 and v >= mod // 2:
                v -= mod
            assert int(got[i, j]) == v


def test_config_int32_no_overflow_matches_numpy():
    r = rng(7)
    a = r.integers(-8, 9, (64, 80)).astype(np.int32)
    b = r.integers(-8, 9, (80, 48)).astype(np.int32)
    assert np.array_equal(oracle.matmult2d(a, b), a.astype(np.int64) @ b.astype(np.int64))


def test_half_conversions_all_patterns():
    L = oracle.lib()
    pats = np.arange(65536, dtype=np.uint16)
    as_f32 = pats.view(np.float16).astype(np.float32)
    for p in range(0, 65536, 1):
        f = L.oracle_f16_to_f32(p)
        e = as_f32[p]
        assert (np.isnan(f) and np.isnan(e)) or np.float32(f).tobytes() == e.tobytes(), p
    r = rng(8)
    xs = np.concatenate([
        r.standard_normal(4000).astype(np.float32) * 10.0 ** r.integers(-9, 6, 4000),
        np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 1e-8, 2.0 ** -24, 2.0 ** -25, 3 * 2.0 ** -25,
                  np.inf, -np.inf, 6.1e-5, 6.097e-5], dtype=np.float32),
        (pats.view(np.float16).astype(np.float32)[::37]),
    ]).astype(np.float32)
    with np.errstate(over="ignore"):
        exp = xs.astype(np.float16).view(np.uint16)
    for x, e in zip(xs, exp):
        if np.isnan(x):
            continue
        assert L.oracle_f32_to_f16(float(x)) == int(e), float(x)


def test_bf16_conversion_rne():
    import torch
    r = rng(9)
    xs = (r.standard_normal(5000) * 10.0 ** r.integers(-20, 20, 5000)).astype(np.float32)
    exp = torch.from_numpy(xs).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = oracle.to_bf16_bits(xs)
    assert np.array_equal(got, exp)
    L = oracle.lib()
    for x, e in zip(xs[:500], exp[:500]):
        assert L.oracle_f32_to_bf16(float(x)) == int(e)
    assert np.array_equal(oracle.from_bf16_bits(exp), torch.from_numpy(exp.view(np.int16)).view(torch.bfloat16).float().numpy())


def test_f16_ktile_rounding_schedule():
    """Independent numpy restatement: per 16-wide k tile, widen C, accumulate the 16
    products one fused step at a time in float32, round to half."""
    r = rng(10)
    m, k, n = 6, 70, 5
    a = r.standard_normal((m, k)).astype(np.float16)
    b = r.standard_normal((k, n)).astype(np.float16)
    c0 = r.standard_normal((m, n)).astype(np.float16)
    got = oracle.matmult2d(a, b, c0.copy())
    exp = c0.copy()
    for i in range(m):
        for j in range(n):
            c = exp[i, j]
            for k0 in range(0, k, 16):
                acc = np.float64(np.float32(c))
                for t in range(k0, min(k0 + 16, k)):
                    # float32 fma == round_f32(exact(a*b) + acc); the product of two halves
                    # is exact in float64 and the sum of it with a float32 is exact enough
                    # in float64 (<= 48 significant bits) that one rounding to f32 is the fma
                    acc = np.float64(np.float32(np.float64(a[i, t]) * np.float64(b[t, j]) + acc))
                c = np.float16(np.float32(acc))
            exp[i, j] = c
    assert got.tobytes() == exp.tobytes()
    # and it is NOT the same as a single rounding at the end (guards the chunking)
    single = (c0.astype(np.float32) + a.astype(np.float32) @ b.astype(np.float32)).astype(np.float16)
    assert np.abs(got.astype(np.float32) - single.astype(np.float32)).max() <= 2e-2 * np.abs(single).max()


def test_bf16_definition():
    """BFloat16 has no counterpart in the reference; this build defines it as: bf16 operands, one float32 fma chain over
    all of K starting from C0, ONE round-to-nearest-even at the end.  Pinned against RNE_bf16(float64 GEMM): products of
    two bf16 values are exact in float32, so the chain's only error is the float32 accumulation, and the result must be
    bit-equal to RNE(exact) wherever the exact value is further from a rounding boundary than that error, and within one
    bf16 ulp everywhere.  A wrong rounding point (truncation, rounding per k-tile, double rounding through another
    format) fails this."""
    from util import assert_one_rounding
    r = rng(11)
    for (m, k, n, with_c0, ta, tb) in [(7, 100, 9, False, False, False), (33, 257, 40, True, False, True), (16, 1001, 24, True, True, False),
                                       (5, 8, 3, True, True, True), (64, 515, 17, False, False, False)]:
        a = oracle.to_bf16_bits(r.standard_normal((m, k)).astype(np.float32))
        b = oracle.to_bf16_bits(r.standard_normal((k, n)).astype(np.float32))
        c0 = oracle.to_bf16_bits((r.standard_normal((m, n)) * (4.0 if with_c0 else 0.0)).astype(np.float32))
        sa = np.ascontiguousarray(a.T) if ta else a
        sb = np.ascontiguousarray(b.T) if tb else b
        got = oracle.matmult2d(sa, sb, c0.copy(), ta, tb, dt=oracle.BF16)
        a64, b64, c64 = (oracle.from_bf16_bits(x).astype(np.float64) for x in (a, b, c0))
        ref = c64 + a64 @ b64
        mag = np.abs(c64) + np.sqrt((a64 * a64) @ (b64 * b64))
        assert_one_rounding(oracle.from_bf16_bits(got).astype(np.float64), ref, mag, k, "bf16", f"bf16 oracle {m}x{k}x{n}")
        got_n = oracle.matmult2d(sa, sb, c0.copy(), ta, tb, dt=oracle.BF16, kind="naive")
        assert got.tobytes() == got_n.tobytes()
    # the check has teeth: truncating instead of rounding, or rounding every 16 k, fails it
    a64, b64 = oracle.from_bf16_bits(a).astype(np.float64), oracle.from_bf16_bits(b).astype(np.float64)
    ref = a64 @ b64
    mag = np.sqrt((a64 * a64) @ (b64 * b64))
    trunc = ((ref.astype(np.float32).view(np.uint32) >> 16).astype(np.uint16))
    with pytest.raises(AssertionError):
        assert_one_rounding(oracle.from_bf16_bits(trunc).astype(np.float64), ref, mag, k, "bf16")
    acc = np.zeros((m, n), np.float64)
    for k0 in range(0, k, 16):
        acc = oracle.from_bf16_bits(oracle.to_bf16_bits((acc + a64[:, k0:k0 + 16] @ b64[k0:k0 + 16]).astype(np.float32))).astype(np.float64)
    with pytest.raises(AssertionError):
        assert_one_rounding(acc, ref, mag, k, "bf16")


def test_batched_equals_per_item_and_broadcast():
    """The reference's own invariant (tests/src/matmult_test.cpp:108-189): the batched
    call is bit-equal to per-item calls; broadcast == explicit repeat."""
    r = rng(12)
    a = r.standard_normal((2, 3, 10, 7)).astype(np.float32)
    b = r.standard_normal((3, 7, 6)).astype(np.float32)
    out = oracle.matmult(a, b)
    assert out.shape == (2, 3, 10, 6)
    for i in range(2):
        for j in range(3):
            assert out[i, j].tobytes() == oracle.matmult2d(a[i, j], b[j]).tobytes()
    rep = np.ascontiguousarray(np.broadcast_to(b, (2, 3, 7, 6)))
    assert oracle.matmult(a, rep).tobytes() == out.tobytes()
    # lower-rank A, higher-rank B with transposes
    a2 = r.standard_normal((7, 10)).astype(np.float32)       # stored [k, m] -> ta
    b2 = r.standard_normal((4, 6, 7)).astype(np.float32)     # stored [n, k] -> tb
    o2 = oracle.matmult(a2, b2, ta=True, tb=True)
    assert o2.shape == (4, 10, 6)
    for i in range(4):
        assert np.allclose(o2[i], a2.T @ b2[i].T, atol=1e-5)
    As = [a[0, 0], a[0, 1], a[0, 0]]
    Bs = [b[0], b[0], b[0]]
    Cs = [np.zeros((10, 6), np.float32) for _ in range(3)]
    oracle.matmult_batch_ptrs(As, Bs, Cs)
    assert Cs[0].tobytes() == Cs[2].tobytes() == oracle.matmult2d(a[0, 0], b[0]).tobytes()
