"""Complex32 / Complex64 / Complex128 through the C ABI against the oracle's restatement of the reference's complex
matmult (lane-wise on interleaved re / im: one real product of the real parts, one of the imaginary parts; Complex32
rounded to half every 8 k).  The GPU kernel runs the same fused chains in the same order, so every result -- Complex32
included -- must be bit-identical.  Parity is unpinned by any reference fixture (none holds a complex matmult value); the
oracle is pinned in tests/test_oracle_complex.py."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from neurotensor_amd import _lib

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
TRANS = [(False, False), (False, True), (True, False), (True, True)]
KINDS = {"c32": (np.float16, _lib.COMPLEX32, oracle.C32), "c64": (np.float32, _lib.COMPLEX64, oracle.C64), "c128": (np.float64, _lib.COMPLEX128, oracle.C128)}


def setup_module(module):
    assert torch.cuda.is_available(), "GPU tests need a visible MI355X"
    _lib.load()


def rnd(rng, shape, real, scale=1.0):
    return (rng.standard_normal(shape + (2,)) * scale).astype(real)


def stored(x, t):
    return np.ascontiguousarray(x.transpose(1, 0, 2)) if t else x


def up(x):
    return torch.from_numpy(np.ascontiguousarray(x).view(np.uint8).reshape(-1).copy()).to(DEV)


def down(t, real, shape):
    return t.cpu().numpy().view(real).reshape(shape)


@pytest.mark.parametrize("kind", list(KINDS))
def test_complex_product_bit_exact(kind):
    real, code, ocode = KINDS[kind]
    lib = _lib.load()
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rng = np.random.default_rng(9100 + code)
    modes = (_lib.C_ACCUMULATE, _lib.C_OVERWRITE, _lib.C_BIAS)
    i = 0
    for (m, k, n) in [(1, 1, 1), (5, 3, 7), (64, 16, 64), (70, 45, 130), (129, 100, 65), (200, 257, 31)]:
        for ta, tb in TRANS:
            mode = modes[i % 3]
            i += 1
            a, b, c0, bias = rnd(rng, (m, k), real, 0.5), rnd(rng, (k, n), real, 0.5), rnd(rng, (m, n), real), rnd(rng, (n,), real)
            sa, sb = stored(a, ta), stored(b, tb)
            init = c0.copy() if mode == _lib.C_ACCUMULATE else np.ascontiguousarray(np.broadcast_to(bias, (m, n, 2))).copy() if mode == _lib.C_BIAS else np.zeros_like(c0)
            want = oracle.matmult2d_complex(sa, sb, init, ta, tb, ocode)
            da, db, dc, dbias = up(sa), up(sb), up(c0), up(bias)
            d = _lib.GemmDesc()
            d.dtype, d.transpose_a, d.transpose_b, d.c_mode = code, int(ta), int(tb), mode
            d.m, d.k, d.n, d.batches = m, k, n, 1
            if mode == _lib.C_BIAS:
                d.bias, d.bias_col_stride = dbias.data_ptr(), 1
            assert lib.ntg_gemm_workspace_bytes(ctypes.byref(d)) == 0
            _lib.check(lib.ntg_gemm_dev(ctypes.byref(d), da.data_ptr(), db.data_ptr(), dc.data_ptr(), st))
            torch.cuda.synchronize()
            got = down(dc, real, (m, n, 2))
            assert got.tobytes() == want.tobytes(), (kind, m, k, n, ta, tb, mode)
            # the host-pointer drop-in (nt_matmult<complex_64> and friends: C += ...)
            hc = c0.copy()
            vp = lambda x: x.ctypes.data_as(ctypes.c_void_p)
            _lib.check(lib.ntg_matmult(code, vp(sa), vp(sb), vp(hc), m, k, k, n, int(ta), int(tb)))
            assert hc.tobytes() == oracle.matmult2d_complex(sa, sb, c0.copy(), ta, tb, ocode).tobytes()
    # it is not the complex product
    a, b = rnd(rng, (8, 8), np.float64), rnd(rng, (8, 8), np.float64)
    lanes = oracle.matmult2d_complex(a, b, dt=oracle.C128)
    true = (a[..., 0] + 1j * a[..., 1]) @ (b[..., 0] + 1j * b[..., 1])
    assert np.abs(lanes[..., 0] - true.real).max() > 1e-3


@pytest.mark.parametrize("kind", list(KINDS))
def test_complex_batches_strides_and_pointer_tables(kind):
    real, code, ocode = KINDS[kind]
    lib = _lib.load()
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rng = np.random.default_rng(9200 + code)
    batch, m, k, n = 3, 40, 50, 36
    lda, ldb, ldc = k + 3, n + 5, n + 2                       # padded rows (in complex elements)
    A = rnd(rng, (batch, m, lda), real, 0.5)
    B = rnd(rng, (k, ldb), real, 0.5)                         # broadcast over the batch
    C = rnd(rng, (batch, m, ldc), real)
    dA, dB, dC = up(A), up(B), up(C)
    d = _lib.GemmDesc()
    d.dtype, d.c_mode = code, _lib.C_ACCUMULATE
    d.m, d.k, d.n, d.batches = m, k, n, batch
    d.lda, d.ldb, d.ldc = lda, ldb, ldc
    d.stride_a, d.stride_b, d.stride_c = m * lda, 0, m * ldc
    _lib.check(lib.ntg_gemm_dev(ctypes.byref(d), dA.data_ptr(), dB.data_ptr(), dC.data_ptr(), st))
    torch.cuda.synchronize()
    got = down(dC, real, (batch, m, ldc, 2))
    want = C.copy()
    for bi in range(batch):
        want[bi, :, :n] = oracle.matmult2d_complex(np.ascontiguousarray(A[bi, :, :k]), np.ascontiguousarray(B[:, :n]), np.ascontiguousarray(C[bi, :, :n]), dt=ocode)
    assert got.tobytes() == want.tobytes()                    # products exact, padding untouched
    # pointer tables (nt_matmult_batch with the tables in device memory), repeated entries
    items = [rnd(rng, (m, k), real, 0.5) for _ in range(2)]
    bm = rnd(rng, (k, n), real, 0.5)
    idx = [0, 1, 0, 1, 1]
    cs = [rnd(rng, (m, n), real) for _ in idx]
    d_items, d_b, d_cs = [up(x) for x in items], up(bm), [up(x) for x in cs]
    tab = torch.tensor([d_items[i].data_ptr() for i in idx] + [d_b.data_ptr()] * len(idx) + [x.data_ptr() for x in d_cs], dtype=torch.int64, device=DEV)
    d = _lib.GemmDesc()
    d.dtype, d.c_mode = code, _lib.C_ACCUMULATE
    d.m, d.k, d.n, d.batches = m, k, n, len(idx)
    es = tab.element_size()
    _lib.check(lib.ntg_gemm_ptrs_dev(ctypes.byref(d), tab.data_ptr(), tab.data_ptr() + len(idx) * es, tab.data_ptr() + 2 * len(idx) * es, st))
    torch.cuda.synchronize()
    for j, i in enumerate(idx):
        assert down(d_cs[j], real, (m, n, 2)).tobytes() == oracle.matmult2d_complex(items[i], bm, cs[j].copy(), dt=ocode).tobytes()
    # host batch entry point with the same pattern, and linear with a bias row
    hcs = [x.copy() for x in cs]
    arr = lambda xs: (ctypes.c_void_p * len(xs))(*[x.ctypes.data for x in xs])
    _lib.check(lib.ntg_matmult_batch(code, arr([items[i] for i in idx]), arr([bm] * len(idx)), arr(hcs), len(idx), m, k, k, n, 0, 0))
    for j, i in enumerate(idx):
        assert hcs[j].tobytes() == oracle.matmult2d_complex(items[i], bm, cs[j].copy(), dt=ocode).tobytes()
    bias = rnd(rng, (n,), real)
    y = np.empty((m, n, 2), real)
    vp = lambda x: x.ctypes.data_as(ctypes.c_void_p)
    _lib.check(lib.ntg_linear(code, vp(items[0]), vp(bm), vp(bias), vp(y), m, k, n, 0, 0, 1, n))
    assert y.tobytes() == oracle.matmult2d_complex(items[0], bm, np.ascontiguousarray(np.broadcast_to(bias, (m, n, 2))).copy(), dt=ocode).tobytes()
    # k = 0: C += nothing; overwrite gives zeros
    hc = cs[0].copy()
    _lib.check(lib.ntg_matmult(code, vp(items[0]), vp(bm), vp(hc), m, 0, 0, n, 0, 0))
    assert hc.tobytes() == cs[0].tobytes()


@pytest.mark.parametrize("kind", list(KINDS))
def test_complex_conv2d_forward_and_unfold(kind):
    """the reference's conv2d smoke test sweeps every complex dtype (tests/src/conv_test.cpp:192-213: [1,3,16,16] (*)
    [4,3,3,3], stride 1, padding 1); conv2d = unfold + the matmult above (conv.cpp:69-96), also grouped and 1x1"""
    real, code, ocode = KINDS[kind]
    lib = _lib.load()
    rng = np.random.default_rng(9300 + code)
    vp = lambda x: x.ctypes.data_as(ctypes.c_void_p)
    for (B, C, H, W, O, kr, kc, s, p, dil, groups) in [(1, 3, 16, 16, 4, 3, 3, 1, 1, 1, 1), (2, 4, 9, 11, 6, 3, 2, 2, 1, 1, 2), (2, 5, 7, 7, 3, 1, 1, 1, 0, 1, 1)]:
        x = rnd(rng, (B, C, H, W), real, 0.5)
        w = rnd(rng, (O, C // groups, kr, kc), real, 0.5)
        planes = [oracle.unfold2d(np.ascontiguousarray(x[..., q]), (kr, kc), dilation=dil, padding=p, stride=s) for q in (0, 1)]
        col = np.stack(planes, axis=-1)                                   # [B, C kr kc, L, 2]: im2col moves whole elements
        Ho = (H + 2 * p - dil * (kr - 1) - 1) // s + 1
        Wo = (W + 2 * p - dil * (kc - 1) - 1) // s + 1
        got_col = np.empty_like(col)
        _lib.check(lib.ntg_unfold2d(code, vp(x), vp(got_col), B, C, H, W, kr, kc, s, s, p, p, dil, dil))
        assert got_col.tobytes() == np.ascontiguousarray(col).tobytes()
        cg, og, taps = C // groups, O // groups, kr * kc
        want = np.empty((B, O, Ho * Wo, 2), real)
        for bi in range(B):
            for g in range(groups):
                w2d = np.ascontiguousarray(w[g * og:(g + 1) * og].reshape(og, cg * taps, 2))
                want[bi, g * og:(g + 1) * og] = oracle.matmult2d_complex(w2d, np.ascontiguousarray(col[bi, g * cg * taps:(g + 1) * cg * taps]), dt=ocode)
        out = np.empty((B, O, Ho, Wo, 2), real)
        _lib.check(lib.ntg_conv2d(code, vp(x), vp(w), vp(out), B, C, H, W, O, kr, kc, s, s, p, p, dil, dil, groups))
        assert out.tobytes() == want.tobytes(), (kind, B, C, H, W, O, kr, kc, s, p, groups)


def _arr64(*v):
    return (ctypes.c_int64 * len(v))(*v)


@pytest.mark.parametrize("kind", list(KINDS))
def test_complex_conv2d_gradients_bit_exact(kind):
    """conv_dimage / conv_dkernel for the complex dtypes (the reference lowers them like the real ones, conv.cpp:318-346,
    :444-471): d_col = W_g^T . dY with the lane-wise product, then the unfold adjoint adding taps in ascending order in the
    element type; dW = the per-image products dY_b . col_b^T, each from zero, added up in batch order in the element type and
    added to d_kernel last.  Bit for bit against the oracle's plane-by-plane restatement (oracle.complex_lanes), overwrite
    and accumulate; also unfold2d_backward on its own.  No reference fixture holds a complex value: parity unpinned by the
    reference, the restatement is pinned in tests/test_oracle_complex.py."""
    real, code, ocode = KINDS[kind]
    lib = _lib.load()
    rng = np.random.default_rng(9400 + code)
    vp = lambda x: x.ctypes.data_as(ctypes.c_void_p)
    for (B, C, H, W, O, kr, kc, s, p, dil, groups) in [(1, 3, 16, 16, 4, 3, 3, 1, 1, 1, 1), (3, 4, 9, 11, 6, 3, 2, 2, 1, 1, 2), (2, 6, 8, 8, 4, 2, 2, 1, 0, 2, 1)]:
        x = rnd(rng, (B, C, H, W), real, 0.5)
        w = rnd(rng, (O, C // groups, kr, kc), real, 0.5)
        Ho = (H + 2 * p - dil * (kr - 1) - 1) // s + 1
        Wo = (W + 2 * p - dil * (kc - 1) - 1) // s + 1
        gy = rnd(rng, (B, O, Ho, Wo), real, 0.5)
        wdx, wdw = oracle.complex_lanes(oracle.conv2d_backward, ocode, x, w, gy, stride=s, padding=p, dilation=dil, groups=groups)
        dx, dw = np.empty_like(x), np.empty_like(w)
        _lib.check(lib.ntg_conv2d_backward(code, vp(x), vp(w), vp(gy), vp(dx), vp(dw), B, C, H, W, O, kr, kc, s, s, p, p, dil, dil, groups, 0))
        assert dx.tobytes() == np.ascontiguousarray(wdx).tobytes(), (kind, "dX", B, C, H, W, groups)
        assert dw.tobytes() == np.ascontiguousarray(wdw).tobytes(), (kind, "dW", B, C, H, W, groups)
        # accumulate: the gradients are added to what d_image / d_kernel hold (the scatter lands on d_image element by element,
        # the summed products on d_kernel in one addition)
        dx0, dw0 = rnd(rng, x.shape[:-1], real), rnd(rng, w.shape[:-1], real)
        dx, dw = dx0.copy(), dw0.copy()
        _lib.check(lib.ntg_conv2d_backward(code, vp(x), vp(w), vp(gy), vp(dx), vp(dw), B, C, H, W, O, kr, kc, s, s, p, p, dil, dil, groups, 1))
        assert dw.tobytes() == (dw0 + np.ascontiguousarray(wdw)).astype(real).tobytes(), (kind, "dW accumulate")
        # dX accumulate: d_image + taps in order, element type -- restated directly
        dcol = np.stack([_dcol_plane(oracle, w[..., q], gy[..., q], B, C, O, kr, kc, groups, ocode) for q in (0, 1)], axis=-1)
        want = dx0.copy()
        for q in (0, 1):
            want[..., q] = _col2im_onto(dx0[..., q], dcol[..., q], (H, W), (kr, kc), dil, p, s)
        assert dx.tobytes() == want.tobytes(), (kind, "dX accumulate")
        # the unfold adjoint alone
        col = rnd(rng, (B, C * kr * kc, Ho * Wo), real)
        im = np.empty((B, C, H, W, 2), real)
        _lib.check(lib.ntg_unfold2d_backward(code, vp(col), vp(im), B, C, H, W, kr, kc, s, s, p, p, dil, dil, 0))
        want = np.stack([oracle.unfoldnd_backward(np.ascontiguousarray(col[..., q]), (H, W), (kr, kc), dil, p, s) for q in (0, 1)], axis=-1)
        assert im.tobytes() == np.ascontiguousarray(want).tobytes(), (kind, "unfold2d_backward")


def _dcol_plane(oracle, w, gy, B, C, O, kr, kc, groups, ocode):
    """d_col of one lane: per group W_g^T . dY_g in the lane's arithmetic"""
    og, add = O // groups, (C // groups) * kr * kc
    g3 = np.ascontiguousarray(gy).reshape(B, O, -1)
    dcol = np.zeros((B, C * kr * kc, g3.shape[2]), g3.dtype)
    prev = oracle._HALF_AS_COMPLEX32_LANE[0]
    oracle._HALF_AS_COMPLEX32_LANE[0] = ocode == oracle.C32
    try:
        for g in range(groups):
            wg = np.ascontiguousarray(w[g * og:(g + 1) * og].reshape(og, -1))
            dcol[:, g * add:(g + 1) * add, :] = oracle.matmult(wg, np.ascontiguousarray(g3[:, g * og:(g + 1) * og, :]), None, True, False)
    finally:
        oracle._HALF_AS_COMPLEX32_LANE[0] = prev
    return dcol


def _col2im_onto(start, col, size, k, dil, p, s):
    """start + the taps of col in ascending order, every addition in the array's own type"""
    B, C = start.shape[:2]
    kr, kc = k
    Ho = (size[0] + 2 * p - dil * (kr - 1) - 1) // s + 1
    Wo = (size[1] + 2 * p - dil * (kc - 1) - 1) // s + 1
    c6 = col.reshape(B, C, kr, kc, Ho, Wo)
    xp = np.zeros((B, C, size[0] + 2 * p, size[1] + 2 * p), start.dtype)
    xp[:, :, p:p + size[0], p:p + size[1]] = start
    for i in range(kr):
        for j in range(kc):
            xp[:, :, i * dil:i * dil + (Ho - 1) * s + 1:s, j * dil:j * dil + (Wo - 1) * s + 1:s] += c6[:, :, i, j]
    return xp[:, :, p:p + size[0], p:p + size[1]]


@pytest.mark.parametrize("kind", list(KINDS))
def test_complex_conv3d_forward_and_gradients_bit_exact(kind):
    """conv3d and its gradients for the complex dtypes (tests/src/conv_test.cpp:216-235 sweeps them; conv.cpp:122-175, :347,
    :472): unfold -> lane-wise product, bit for bit against the plane-by-plane oracle; grouped, strided, padded."""
    real, code, ocode = KINDS[kind]
    lib = _lib.load()
    rng = np.random.default_rng(9500 + code)
    vp = lambda x: x.ctypes.data_as(ctypes.c_void_p)
    for (B, C, size, O, k, s, p, d, groups) in [(1, 3, (6, 6, 6), 4, (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), 1),
                                                 (2, 4, (4, 5, 6), 6, (2, 3, 2), (1, 2, 1), (1, 0, 1), (1, 1, 2), 2)]:
        x = rnd(rng, (B, C) + size, real, 0.5)
        w = rnd(rng, (O, C // groups) + k, real, 0.5)
        want = oracle.complex_lanes(oracle.convnd, ocode, x, w, stride=s, padding=p, dilation=d, groups=groups)
        out = np.empty(want.shape, real)
        _lib.check(lib.ntg_convnd(code, vp(x), vp(w), vp(out), B, C, O, 3, _arr64(*size), _arr64(*k), _arr64(*s), _arr64(*p), _arr64(*d), groups))
        assert out.tobytes() == np.ascontiguousarray(want).tobytes(), (kind, "conv3d", size)
        gy = rnd(rng, want.shape[:-1], real, 0.5)
        wdx, wdw = oracle.complex_lanes(oracle.convnd_backward, ocode, x, w, gy, stride=s, padding=p, dilation=d, groups=groups)
        dx, dw = np.empty_like(x), np.empty_like(w)
        _lib.check(lib.ntg_convnd_backward(code, vp(x), vp(w), vp(gy), vp(dx), vp(dw), B, C, O, 3, _arr64(*size), _arr64(*k), _arr64(*s), _arr64(*p),
                                           _arr64(*d), groups, 0))
        assert dx.tobytes() == np.ascontiguousarray(wdx).tobytes(), (kind, "conv3d dX", size)
        assert dw.tobytes() == np.ascontiguousarray(wdw).tobytes(), (kind, "conv3d dW", size)


@pytest.mark.parametrize("kind", list(KINDS))
def test_complex_transposed_convolutions(kind):
    """conv_transpose1d / 2d / 3d for the complex dtypes (tests/src/conv_test.cpp:237-279).  This library computes a
    transposed convolution as the image gradient of the matching convolution: per tap a product over the input channels,
    then the taps added -- the same terms as the reference's dilate -> pad -> unfold -> one product over (channel, tap)
    (conv.cpp:538-745), summed in another order.  So, as for the real floating dtypes, the result is held to the floating
    tolerance of its lane type (1e-5 K max|x| max|w| per lane; 2e-2 of the largest result for the half lanes), not bit for bit."""
    real, code, ocode = KINDS[kind]
    lib = _lib.load()
    rng = np.random.default_rng(9600 + code)
    vp = lambda x: x.ctypes.data_as(ctypes.c_void_p)

    def close(got, want, kdepth, x, w, what):
        g, r = got.astype(np.float64), np.asarray(want, np.float64)
        tol = 2e-2 * max(np.abs(r).max(), 1e-30) if real == np.float16 else 1e-5 * kdepth * float(np.abs(x).max()) * float(np.abs(w).max())
        assert np.abs(g - r).max() <= tol, (kind, what, float(np.abs(g - r).max()), tol)

    for (B, Cin, H, W, Cog, kr, kc, s, p, op, dil, groups) in [(1, 3, 8, 8, 4, 3, 3, 1, 1, 0, 1, 1), (2, 4, 5, 6, 3, 3, 2, 2, 1, 1, 1, 2)]:
        x = rnd(rng, (B, Cin, H, W), real, 0.5)
        w = rnd(rng, (Cin, Cog, kr, kc), real, 0.5)
        want = oracle.complex_lanes(oracle.conv_transpose2d, ocode, x, w, stride=s, padding=p, output_padding=op, dilation=dil, groups=groups)
        out = np.empty(want.shape, real)
        _lib.check(lib.ntg_conv_transpose2d(code, vp(x), vp(w), vp(out), B, Cin, H, W, Cog * groups, kr, kc, s, s, p, p, dil, dil, op, op, groups))
        close(out, want, (Cin // groups) * kr * kc, x, w, "conv_transpose2d")
    # one axis (conv_transpose1d = the one-row case) and three axes
    x = rnd(rng, (2, 4, 9), real, 0.5)
    w = rnd(rng, (4, 3, 4), real, 0.5)
    want = oracle.complex_lanes(oracle.conv_transpose1d, ocode, x, w, stride=2, padding=1, output_padding=1, dilation=1, groups=2)
    out = np.empty(want.shape, real)
    _lib.check(lib.ntg_conv_transposend(code, vp(x), vp(w), vp(out), 2, 4, 6, 1, _arr64(9), _arr64(4), _arr64(2), _arr64(1), _arr64(1), _arr64(1), 2))
    close(out, want, 2 * 4, x, w, "conv_transpose1d")
    x = rnd(rng, (1, 4, 3, 4, 5), real, 0.5)
    w = rnd(rng, (4, 2, 2, 3, 3), real, 0.5)
    want = oracle.complex_lanes(oracle.conv_transposend, ocode, x, w, stride=(2, 1, 2), padding=(0, 1, 1), output_padding=(1, 0, 1), dilation=1, groups=2)
    out = np.empty(want.shape, real)
    _lib.check(lib.ntg_conv_transposend(code, vp(x), vp(w), vp(out), 1, 4, 4, 3, _arr64(3, 4, 5), _arr64(2, 3, 3), _arr64(2, 1, 2), _arr64(0, 1, 1),
                                        _arr64(1, 1, 1), _arr64(1, 0, 1), 2))
    close(out, want, 2 * 18, x, w, "conv_transpose3d")
