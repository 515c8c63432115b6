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
