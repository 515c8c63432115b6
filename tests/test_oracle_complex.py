"""Pins the oracle's restatement of the reference's complex matmult (CPU only).

No fixture or test of the reference holds a complex matmult value, so this is "parity unpinned by any reference
fixture"; what pins the restatement is the reference's code itself, walked literally:
  * the generic micro kernel (nt_matmult_simde.hpp:301-350) on vectors of interleaved (re, im) lanes with
    broadcast = set1 = (a.re, a.im, a.re, a.im, ...) and lane-wise fmadd (simde_traits_avx2.h:928-937, :996-1002), on
    operands of small integers where every step is exact -- a transposed lane, a swapped re / im or a true complex
    product fails it;
  * its reduction to two real products (real parts, imaginary parts), bit for bit against the real oracle, which is
    pinned by tests/test_oracle_gemm.py -- this carries the rounding behaviour;
  * complex_32: float lanes inside k tiles of 2 * pack_size = 8 (simde_traits_avx2.h:1275), rounded to half between
    tiles, against an independent numpy restatement."""
import numpy as np
import pytest

import oracle

CODES = {oracle.C32: np.float16, oracle.C64: np.float32, oracle.C128: np.float64}
PACK = {oracle.C32: 4, oracle.C64: 4, oracle.C128: 2}          # complex elements per 256-bit vector
TRANS = [(False, False), (False, True), (True, False), (True, True)]


def stored(x, t):
    return np.ascontiguousarray(x.transpose(1, 0, 2)) if t else x


@pytest.mark.parametrize("dt", list(CODES))
def test_vector_lane_walk_of_the_micro_kernel(dt):
    """k tile outermost; per C tile row two vectors of `pack` complex = 2 pack real lanes; per kk: aVec = the (re, im)
    pair of A(i, kk) repeated, C0 = aVec * B0 + C0, C1 = aVec * B1 + C1 lane by lane."""
    rng = np.random.default_rng(31)
    real = CODES[dt]
    pack, tile = PACK[dt], 2 * PACK[dt]
    m, k, n = 5, 2 * tile + 3, tile + 3                      # ragged in every direction
    a = rng.integers(-3, 4, (m, k, 2)).astype(real)
    b = rng.integers(-3, 4, (k, n, 2)).astype(real)
    c0 = rng.integers(-3, 4, (m, n, 2)).astype(real)
    want = c0.astype(np.float64)
    npad = (n + tile - 1) // tile * tile
    bp = np.zeros((k, npad, 2))
    bp[:, :n] = b
    cp = np.zeros((m, npad, 2))
    cp[:, :n] = want
    for k0 in range(0, k, tile):
        for j0 in range(0, npad, tile):
            for i in range(m):
                vec = [cp[i, j0:j0 + pack].reshape(-1).copy(), cp[i, j0 + pack:j0 + tile].reshape(-1).copy()]   # lanes re, im, re, im ...
                for kk in range(k0, min(k0 + tile, k)):
                    avec = np.tile(a[i, kk].astype(np.float64), pack)                                           # set1
                    rows = [bp[kk, j0:j0 + pack].reshape(-1), bp[kk, j0 + pack:j0 + tile].reshape(-1)]
                    vec = [avec * rows[0] + vec[0], avec * rows[1] + vec[1]]
                cp[i, j0:j0 + pack] = vec[0].reshape(pack, 2)
                cp[i, j0 + pack:j0 + tile] = vec[1].reshape(pack, 2)
    want = cp[:, :n]
    assert np.abs(want).max() < 2000                           # exact in every format, half included
    for ta, tb in TRANS:
        got = oracle.matmult2d_complex(stored(a, ta), stored(b, tb), c0.copy(), ta, tb, dt)
        assert np.array_equal(got.astype(np.float64), want), (ta, tb)
        gotn = oracle.matmult2d_complex(stored(a, ta), stored(b, tb), c0.copy(), ta, tb, dt, kind="naive")
        assert gotn.tobytes() == got.tobytes()
    # and it is not the complex product
    true = (c0[..., 0] + 1j * c0[..., 1]) + (a[..., 0] + 1j * a[..., 1]).astype(np.complex128) @ (b[..., 0] + 1j * b[..., 1]).astype(np.complex128)
    assert not np.array_equal(want[..., 0], true.real)


@pytest.mark.parametrize("dt", [oracle.C64, oracle.C128])
def test_complex_is_two_real_products_bit_for_bit(dt):
    rng = np.random.default_rng(32)
    real = CODES[dt]
    for (m, k, n) in [(7, 50, 9), (33, 129, 20), (1, 1, 1), (16, 16, 16)]:
        a = rng.standard_normal((m, k, 2)).astype(real)
        b = rng.standard_normal((k, n, 2)).astype(real)
        c0 = rng.standard_normal((m, n, 2)).astype(real)
        for ta, tb in TRANS:
            got = oracle.matmult2d_complex(stored(a, ta), stored(b, tb), c0.copy(), ta, tb, dt)
            for part in (0, 1):
                plane = oracle.matmult2d(np.ascontiguousarray(a[..., part]), np.ascontiguousarray(b[..., part]), c0[..., part].copy())
                assert got[..., part].tobytes() == plane.tobytes(), (m, k, n, ta, tb, part)
            assert oracle.matmult2d_complex(stored(a, ta), stored(b, tb), c0.copy(), ta, tb, dt, kind="naive").tobytes() == got.tobytes()


def test_complex32_rounds_to_half_every_8_k():
    rng = np.random.default_rng(33)
    m, k, n = 6, 43, 5
    a = rng.standard_normal((m, k, 2)).astype(np.float16)
    b = rng.standard_normal((k, n, 2)).astype(np.float16)
    c0 = rng.standard_normal((m, n, 2)).astype(np.float16)
    got = oracle.matmult2d_complex(a, b, c0.copy(), dt=oracle.C32)
    exp = c0.copy()
    for i in range(m):
        for j in range(n):
            for part in (0, 1):
                c = exp[i, j, part]
                for k0 in range(0, k, 8):
                    acc = np.float64(np.float32(c))
                    for t in range(k0, min(k0 + 8, k)):
                        # product of two halves: exact in float64; adding a float32 keeps <= 48 significant bits, so the
                        # one rounding to float32 is the fused step's
                        acc = np.float64(np.float32(np.float64(a[i, t, part]) * np.float64(b[t, j, part]) + acc))
                    c = np.float16(np.float32(acc))
                exp[i, j, part] = c
    assert got.tobytes() == exp.tobytes()
    # the 16-wide tiles of the real Float16 path would give other bits somewhere
    plane16 = np.stack([oracle.matmult2d(np.ascontiguousarray(a[..., p]), np.ascontiguousarray(b[..., p]), c0[..., p].copy()) for p in (0, 1)], axis=-1)
    assert plane16.tobytes() != got.tobytes()
    assert np.abs(plane16.astype(np.float32) - got.astype(np.float32)).max() <= 2e-2 * np.abs(got.astype(np.float32)).max()
    for ta, tb in TRANS:
        g = oracle.matmult2d_complex(stored(a, ta), stored(b, tb), c0.copy(), ta, tb, oracle.C32)
        assert g.tobytes() == got.tobytes()
        assert oracle.matmult2d_complex(stored(a, ta), stored(b, tb), c0.copy(), ta, tb, oracle.C32, kind="naive").tobytes() == got.tobytes()


def test_one_lane_of_a_complex32_product_is_the_half_product_with_k_tiles_of_8():
    """F16_LANE8 (half values, float chains rounded to half every 8 k) on the plane of real parts and on the plane of
    imaginary parts == the two lanes of the Complex32 product, bit for bit, with C0 and every flag pair: what lets the
    complex convolutions be restated plane by plane (oracle.complex_lanes)."""
    rng = np.random.default_rng(77)
    for (m, k, n) in [(3, 5, 4), (9, 8, 7), (17, 41, 12), (6, 64, 10)]:
        for ta, tb in TRANS:
            a = rng.standard_normal((m, k, 2)).astype(np.float16)
            b = rng.standard_normal((k, n, 2)).astype(np.float16)
            c0 = rng.standard_normal((m, n, 2)).astype(np.float16)
            sa, sb = stored(a, ta), stored(b, tb)
            want = oracle.matmult2d_complex(sa, sb, c0.copy(), ta, tb, oracle.C32)
            for lane in (0, 1):
                got = oracle.matmult2d(np.ascontiguousarray(sa[..., lane]), np.ascontiguousarray(sb[..., lane]),
                                       np.ascontiguousarray(c0[..., lane]), ta, tb, dt=oracle.F16_LANE8)
                assert got.tobytes() == np.ascontiguousarray(want[..., lane]).tobytes(), (m, k, n, ta, tb, lane)
            # ... and it is not Float16's own schedule (tiles of 16) once k passes 8
            if k > 8:
                f16 = oracle.matmult2d(np.ascontiguousarray(sa[..., 0]), np.ascontiguousarray(sb[..., 0]), np.ascontiguousarray(c0[..., 0]), ta, tb)
                assert f16.tobytes() != np.ascontiguousarray(want[..., 0]).tobytes() or k <= 16


@pytest.mark.parametrize("dt", list(CODES))
def test_complex_convolutions_plane_by_plane_equal_unfold_then_complex_matmult(dt):
    """oracle.complex_lanes(oracle.conv2d / convnd) against the direct statement of the reference's lowering: unfold the
    complex image (whole elements move), then the complex matmult per group (conv.cpp:69-118, :134-174)."""
    real = CODES[dt]
    rng = np.random.default_rng(5)
    for (B, C, H, W, O, kr, kc, s, p, dil, groups) in [(2, 4, 7, 6, 6, 3, 2, 1, 1, 1, 2), (1, 3, 9, 9, 4, 3, 3, 2, 1, 1, 1)]:
        x = (rng.standard_normal((B, C, H, W, 2)) * 0.5).astype(real)
        w = (rng.standard_normal((O, C // groups, kr, kc, 2)) * 0.5).astype(real)
        got = oracle.complex_lanes(oracle.conv2d, dt, x, w, stride=s, padding=p, dilation=dil, groups=groups)
        col = np.stack([oracle.unfold2d(np.ascontiguousarray(x[..., q]), (kr, kc), dilation=dil, padding=p, stride=s) for q in (0, 1)], axis=-1)
        cg, og, taps = C // groups, O // groups, kr * kc
        want = np.empty((B, O, col.shape[2], 2), real)
        for bi in range(B):
            for g in range(groups):
                w2d = np.ascontiguousarray(w[g * og:(g + 1) * og].reshape(og, cg * taps, 2))
                want[bi, g * og:(g + 1) * og] = oracle.matmult2d_complex(w2d, np.ascontiguousarray(col[bi, g * cg * taps:(g + 1) * cg * taps]), dt=dt)
        assert got.reshape(want.shape).tobytes() == want.tobytes(), (dt, B, C, H, W)
    # three spatial axes
    x = (rng.standard_normal((2, 4, 4, 5, 6, 2)) * 0.5).astype(real)
    w = (rng.standard_normal((6, 2, 2, 3, 2, 2)) * 0.5).astype(real)
    got = oracle.complex_lanes(oracle.convnd, dt, x, w, stride=(1, 2, 1), padding=(1, 0, 1), dilation=1, groups=2)
    cols = [oracle.unfoldnd(np.ascontiguousarray(x[..., q]), (2, 3, 2), 1, (1, 0, 1), (1, 2, 1))[0] for q in (0, 1)]
    col = np.stack(cols, axis=-1)
    want = np.empty((2, 6, col.shape[2], 2), real)
    for bi in range(2):
        for g in range(2):
            w2d = np.ascontiguousarray(w[g * 3:(g + 1) * 3].reshape(3, 24, 2))
            want[bi, g * 3:(g + 1) * 3] = oracle.matmult2d_complex(w2d, np.ascontiguousarray(col[bi, g * 24:(g + 1) * 24]), dt=dt)
    assert got.reshape(want.shape).tobytes() == want.tobytes()


def test_batch_ordered_sum_rounds_after_every_addition_in_half():
    """the weight gradient adds the per-image products item by item in the element type (sum_exp_log.cpp:112-124)"""
    per = np.array([[2048.0], [1.0], [1.0], [1.0]], np.float16)        # 2048 + 1 rounds back to 2048 in half, three times over
    assert float(oracle._batch_ordered_sum(per)[0]) == 2048.0
    assert float(per.astype(np.float32).sum()) == 2051.0
