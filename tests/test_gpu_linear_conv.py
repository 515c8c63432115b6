"""GPU parity of the layers above the GEMM: linear (bias-initialised GEMM + gradient GEMMs),
unfold2d and conv2d, against the reference's golden vectors and the CPU oracle."""
import ctypes
import os

import numpy as np
import pytest
import torch

import oracle
from neurotensor_amd import _lib
from neurotensor_amd import functional as F
from util import HALF_REL, assert_one_rounding, float_tol, from_torch, randn, to_f64, to_torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def setup_module(module):
    assert torch.cuda.is_available(), "GPU tests need a visible MI355X"
    _lib.load()


def load(golden_dir, name):
    return np.load(os.path.join(golden_dir, name + ".npy"), allow_pickle=False)


def nt_allclose(a, b, rtol=1e-5, atol=1e-6):
    return bool(np.all(np.abs(a - b) <= atol + rtol * np.abs(b)))


def dev(x):
    return torch.from_numpy(np.ascontiguousarray(x)).to(DEV)


def linear_backward_gpu(x, w, grad, ta, tb):
    """The gradient GEMMs of TensorGrad linear (nn/functional/matmult.cpp:253-275), flags only."""
    dx = F.matmult(w, grad, None, tb, True) if ta else F.matmult(grad, w, None, False, not tb)
    dw = F.matmult(grad, x, None, True, ta) if tb else F.matmult(x, grad, None, not ta, False)
    return dx, dw


def test_linear_golden_grads(golden_dir):
    """tests/src/linear_autograd_test.cpp:126-148 replayed on the GPU path."""
    x, w, b, g = (load(golden_dir, "linear_" + n) for n in ("input", "weight", "bias", "grad"))
    out = F.linear(dev(x), dev(w), dev(b), False, True)
    assert tuple(out.shape) == (3, 4, 3)
    assert np.allclose(out.cpu().numpy(), oracle.linear(x, w, b, False, True), rtol=1e-5, atol=1e-6)
    dx, dw = linear_backward_gpu(dev(x), dev(w), dev(g), False, True)
    dw = dw.sum(0)                                   # accumulate_gradient's broadcast reduction
    db = dev(g).reshape(-1, 3).sum(0)
    assert nt_allclose(dx.cpu().numpy(), load(golden_dir, "linear_xgrad"))
    assert nt_allclose(dw.cpu().numpy(), load(golden_dir, "linear_wgrad"))
    assert nt_allclose(db.cpu().numpy(), load(golden_dir, "linear_bgrad"))


def test_linear_host_entry_and_bias_shapes():
    rng = np.random.default_rng(700)
    m, k, n = 45, 70, 33
    x = rng.standard_normal((m, k)).astype(np.float32)
    w = rng.standard_normal((n, k)).astype(np.float32)       # transpose_w
    lib = _lib.load()
    p = lambda a: a.ctypes.data_as(ctypes.c_void_p)
    for br, bc in [(1, n), (m, 1), (m, n), (1, 1)]:
        bias = rng.standard_normal((br, bc)).astype(np.float32)
        y = np.full((m, n), np.nan, np.float32)
        _lib.check(lib.ntg_linear(_lib.FLOAT32, p(x), p(w), p(bias), p(y), m, k, n, 0, 1, br, bc))
        ref = oracle.linear(x, w, bias, False, True)
        assert np.abs(y - ref).max() <= float_tol(k, x, w) + 1e-6
        yd = F.linear(dev(x), dev(w), dev(bias), False, True)
        assert np.array_equal(yd.cpu().numpy(), y)
    with pytest.raises(ValueError):
        F.linear(dev(x), dev(w), dev(np.zeros((2, n), np.float32)), False, True)


@pytest.mark.parametrize("dtype", [np.float32, "bf16"], ids=["fp32", "bf16"])
def test_config4_linear_training_step(dtype):
    """X[8192,4096], W[11008,4096] (transpose_b), b zeros; Y = X.W^T + b, dX = dY.W, dW = dY^T.X."""
    M, K, N = 8192, 4096, 11008
    bf = dtype == "bf16"
    rng = np.random.default_rng(1006)
    x = randn(rng, (M, K), dtype)
    w = randn(rng, (N, K), dtype, 0.02)
    gy = randn(rng, (M, N), dtype)
    bias = np.zeros((N,), np.uint16 if bf else np.float32)
    tx, tw, tg, tb_ = (to_torch(v, DEV, bf) for v in (x, w, gy, bias))
    y = F.linear(tx, tw, tb_, False, True)
    dx, dw = linear_backward_gpu(tx, tw, tg, False, True)
    torch.cuda.synchronize()
    assert tuple(y.shape) == (M, N) and tuple(dx.shape) == (M, K) and tuple(dw.shape) == (N, K)
    code = oracle.BF16 if bf else oracle.F32
    rows = np.r_[0:24, 5000:5024]
    cols = np.r_[0:24, 11000:11008]

    def check(got_t, A, B, ta, tb, r, c, kk):
        Al = A.T if ta else A
        Bl = B.T if tb else B
        sa, sb = np.ascontiguousarray(Al[r, :]), np.ascontiguousarray(Bl[:, c])
        ref = oracle.matmult2d(sa, sb, dt=code)
        got = from_torch(got_t[r][:, c].contiguous())
        if bf:
            rr, gg = to_f64(ref, True), to_f64(got, True)
            assert np.abs(rr - gg).max() / np.abs(rr).max() <= HALF_REL
        else:
            assert np.abs(ref - got).max() <= float_tol(kk, sa, sb)

    check(y, x, w, False, True, rows, cols, K)                    # Y  = X . W^T
    check(dx, gy, w, False, False, rows, np.r_[0:24, 4072:4096], N)   # dX = dY . W
    check(dw, gy, x, True, False, np.r_[0:24, 10984:11008], np.r_[0:24, 4072:4096], M)   # dW = dY^T . X
    # whole-matrix cross-check of all three products with an independent GEMM (double for Float32, float for BFloat16)
    def whole(got, lhs, rhs, kk):
        if not bf:
            ref = torch.matmul(lhs.double(), rhs.double())
            assert (got.double() - ref).abs().max().item() <= 1e-5 * kk * lhs.abs().max().item() * rhs.abs().max().item()
        else:
            ref = torch.matmul(lhs.float(), rhs.float())
            assert ((got.float() - ref).abs().max() / ref.abs().max()).item() <= HALF_REL
        del ref

    whole(y, tx, tw.t(), K)            # Y  = X . W^T
    whole(dx, tg, tw, N)               # dX = dY . W
    whole(dw, tg.t(), tx, M)           # dW = dY^T . X


def test_unfold_golden_and_random(golden_dir):
    x = load(golden_dir, "unfold_input")
    exp = load(golden_dir, "unfold_output")
    col = F.unfold2d(dev(x), (3, 2), dilation=(1, 2), padding=1, stride=(2, 2))
    assert np.array_equal(col.cpu().numpy(), exp)
    rng = np.random.default_rng(800)
    for dtype in (np.float32, np.float64, np.float16, np.int32):
        xi = (rng.standard_normal((3, 5, 13, 17)) * 10).astype(dtype)
        for k, d, p, s in [((3, 3), 1, 1, 1), ((2, 4), (2, 1), (0, 3), (1, 2)), ((1, 1), 1, 0, 3), ((5, 5), 1, 2, 2)]:
            got = F.unfold2d(dev(xi), k, dilation=d, padding=p, stride=s).cpu().numpy()
            assert np.array_equal(got, oracle.unfold2d(xi, k, dilation=d, padding=p, stride=s))
    # host entry point
    lib = _lib.load()
    xi = rng.standard_normal((2, 3, 9, 8)).astype(np.float32)
    col = np.full((2, 27, 72), np.nan, np.float32)
    _lib.check(lib.ntg_unfold2d(_lib.FLOAT32, xi.ctypes.data_as(ctypes.c_void_p), col.ctypes.data_as(ctypes.c_void_p),
                                2, 3, 9, 8, 3, 3, 1, 1, 1, 1, 1, 1))
    assert np.array_equal(col, oracle.unfold2d(xi, 3, padding=1))
    with pytest.raises(ValueError):
        F.unfold2d(dev(xi), 20)


CONV_CASES = [("", 1, 1), ("_batched", 1, 1), ("_grouped", 0, 2), ("_grouped_batched", 0, 2)]


@pytest.mark.parametrize("sfx,pad,groups", CONV_CASES)
def test_conv2d_golden(golden_dir, sfx, pad, groups):
    """tests/src/conv_autograd_test.cpp:250-371 forward outputs on the GPU path."""
    x = load(golden_dir, "conv2d_input" + sfx)
    w = load(golden_dir, "conv2d_weight" + sfx)
    exp = load(golden_dir, "conv2d_output" + sfx)
    out = F.conv2d(dev(x), dev(w), stride=1, padding=pad, dilation=1, groups=groups).cpu().numpy()
    assert out.shape == exp.shape
    assert np.abs(out - exp).max() <= 1e-4
    assert np.abs(out - oracle.conv2d(x, w, 1, pad, 1, groups)).max() <= 1e-5
    # host entry point
    lib = _lib.load()
    B, C, H, W = x.shape
    O, _, kh, kw = w.shape
    y = np.full(exp.shape, np.nan, np.float32)
    p = lambda a: np.ascontiguousarray(a).ctypes.data_as(ctypes.c_void_p)
    _lib.check(lib.ntg_conv2d(_lib.FLOAT32, p(x), p(w), y.ctypes.data_as(ctypes.c_void_p), B, C, H, W, O, kh, kw,
                              1, 1, pad, pad, 1, 1, groups))
    # (Float32 at the host seam runs the gathering kernels: unfold + matmult bit for bit; the functional face above may take the
    #  channels-last kernels, which sum the same products in another order)
    assert np.array_equal(y.view(np.uint32), oracle.conv2d(x, w, 1, pad, 1, groups).view(np.uint32))
    assert np.abs(y - out).max() <= 1e-5


@pytest.mark.parametrize("sfx,pad,groups", CONV_CASES)
def test_conv2d_backward_golden(golden_dir, sfx, pad, groups):
    """conv_dimage / conv_dkernel (conv.cpp:318-346, 444-471) against the xgrad / wgrad fixtures of
    tests/src/conv_autograd_test.cpp:250-371, device and host entry points."""
    x = load(golden_dir, "conv2d_input" + sfx)
    w = load(golden_dir, "conv2d_weight" + sfx)
    g = load(golden_dir, "conv2d_grad" + sfx)
    xg = load(golden_dir, "conv2d_xgrad" + sfx)
    wg = load(golden_dir, "conv2d_wgrad" + sfx)
    dx, dw = F.conv2d_backward(dev(x), dev(w), dev(g), stride=1, padding=pad, dilation=1, groups=groups)
    dx, dw = dx.cpu().numpy(), dw.cpu().numpy()
    assert dx.shape == xg.shape and dw.shape == wg.shape
    assert np.abs(dx - xg).max() <= 1e-4 * max(1.0, np.abs(xg).max())
    assert np.abs(dw - wg).max() <= 1e-4 * max(1.0, np.abs(wg).max())
    odx, odw = oracle.conv2d_backward(x, w, g, 1, pad, 1, groups)
    assert np.abs(dx - odx).max() <= 1e-5 and np.abs(dw - odw).max() <= 1e-4
    lib = _lib.load()
    B, C, H, W = x.shape
    O, _, kh, kw = w.shape
    hx = np.full(x.shape, np.nan, np.float32)
    hw = np.full(w.shape, np.nan, np.float32)
    p = lambda a: np.ascontiguousarray(a).ctypes.data_as(ctypes.c_void_p)
    _lib.check(lib.ntg_conv2d_backward(_lib.FLOAT32, p(x), p(w), p(g), hx.ctypes.data_as(ctypes.c_void_p),
                                       hw.ctypes.data_as(ctypes.c_void_p), B, C, H, W, O, kh, kw, 1, 1, pad, pad, 1, 1, groups, 0))
    # (Float32 at the host seam: the reference's own two algorithms, the oracle's bits; the functional face above may take the
    #  implicit and channels-last forms, which sum the same products in another order)
    assert np.array_equal(hx.view(np.uint32), odx.view(np.uint32)) and np.array_equal(hw.view(np.uint32), odw.view(np.uint32))
    assert np.abs(hx - dx).max() <= 1e-5 * max(1.0, np.abs(dx).max()) and np.abs(hw - dw).max() <= 1e-4 * max(1.0, np.abs(dw).max())
    # accumulate != 0 adds to the incoming gradients, like the reference's += (conv.cpp:466-469)
    hx2, hw2 = hx.copy(), hw.copy()
    _lib.check(lib.ntg_conv2d_backward(_lib.FLOAT32, p(x), p(w), p(g), hx2.ctypes.data_as(ctypes.c_void_p),
                                       hw2.ctypes.data_as(ctypes.c_void_p), B, C, H, W, O, kh, kw, 1, 1, pad, pad, 1, 1, groups, 1))
    assert np.allclose(hx2, 2 * hx, rtol=1e-5, atol=1e-5) and np.allclose(hw2, 2 * hw, rtol=1e-5, atol=1e-4)


def test_unfold_backward_golden_and_random(golden_dir):
    g = load(golden_dir, "unfold_grad")
    want = load(golden_dir, "unfold_input_grad")
    got = F.unfold2d_backward(dev(g), (8, 8), (3, 2), dilation=(1, 2), padding=1, stride=(2, 2)).cpu().numpy()
    assert np.allclose(got, want, rtol=1e-6, atol=1e-6)
    rng = np.random.default_rng(950)
    for dtype in (np.float32, np.float64):
        for (H, W), k, d, p, s in [((13, 17), (3, 3), 1, 1, 1), ((9, 12), (2, 4), (2, 1), (0, 3), (1, 2)), ((10, 10), (5, 5), 1, 2, 2)]:
            x = rng.standard_normal((2, 3, H, W)).astype(dtype)
            col = oracle.unfold2d(x, k, dilation=d, padding=p, stride=s)
            gcol = rng.standard_normal(col.shape).astype(dtype)
            ref = oracle.unfold2d_backward(gcol, (H, W), k, dilation=d, padding=p, stride=s)
            got = F.unfold2d_backward(dev(gcol), (H, W), k, dilation=d, padding=p, stride=s).cpu().numpy()
            # same tap order as the scatter loop: bit-identical sums
            assert np.array_equal(got, ref)


def test_conv2d_backward_random_vs_oracle():
    rng = np.random.default_rng(960)
    x = rng.standard_normal((3, 6, 14, 11)).astype(np.float32)
    w = rng.standard_normal((8, 3, 3, 2)).astype(np.float32)
    kw = dict(stride=(2, 1), padding=(1, 2), dilation=(1, 2), groups=2)
    out = oracle.conv2d(x, w, kw["stride"], kw["padding"], kw["dilation"], kw["groups"])
    g = rng.standard_normal(out.shape).astype(np.float32)
    dx, dw = F.conv2d_backward(dev(x), dev(w), dev(g), **kw)
    odx, odw = oracle.conv2d_backward(x, w, g, kw["stride"], kw["padding"], kw["dilation"], kw["groups"])
    assert np.abs(dx.cpu().numpy() - odx).max() <= 1e-4
    assert np.abs(dw.cpu().numpy() - odw).max() <= 1e-3
    # gradient check against torch autograd in float64 (independent of both implementations)
    tx = torch.from_numpy(x).double().requires_grad_(True)
    tw = torch.from_numpy(w).double().requires_grad_(True)
    torch.nn.functional.conv2d(tx, tw, None, kw["stride"], kw["padding"], kw["dilation"], kw["groups"]).backward(torch.from_numpy(g).double())
    assert np.abs(dx.cpu().numpy() - tx.grad.numpy()).max() <= 1e-4
    assert np.abs(dw.cpu().numpy() - tw.grad.numpy()).max() <= 1e-3


BACKWARD_GEOMS = [
    # (B, C, H, W, O, kh, kw, stride, padding, dilation, groups)
    (2, 8, 20, 23, 16, 3, 3, 1, 1, 1, 1),                  # stride 1: both gradients as implicit GEMMs
    (3, 6, 17, 9, 9, 2, 4, 1, (0, 3), (2, 1), 3),          # groups, asymmetric taps / padding / dilation
    (2, 4, 11, 12, 6, 3, 3, 1, (3, 4), 1, 2),              # padding beyond the kernel reach (negative padding of the dX conv)
    (1, 3, 7, 31, 4, 1, 1, 1, 0, 1, 1),
    (2, 5, 12, 12, 7, 5, 5, 2, 2, 1, 1),                   # stride 2: dX through the stored col matrix + col2im
    (4, 32, 30, 28, 64, 3, 3, 1, 1, 1, 1),
    (8, 64, 28, 28, 128, 3, 3, 1, 1, 1, 1),                # enough tiles for the large-tile kernels
    (3, 48, 15, 13, 64, 3, 3, 1, 1, 1, 2),                 # channels-last dX with image planes of odd size (195), two groups
    (2, 16, 9, 11, 96, 3, 2, 1, (2, 0), (2, 1), 1),
    (2, 16, 12, 16, 24, 3, 3, (2, 1), (1, 2), (1, 2), 2),  # channels-last dW with stride, dilation and groups (L = 96)
    (64, 256, 6, 6, 128, 3, 3, 1, 1, 1, 1),                # dW with two images per K loop (36 pixels each: the seam falls inside a K-step)
    (8, 512, 5, 7, 512, 3, 3, 1, 1, 1, 1),                 # 35 pixels per image, two images per K loop, four tile rows
    (12, 128, 7, 7, 64, 3, 3, 1, 1, 1, 4),                 # groups; 49 pixels per image (rows of dY not 16-byte multiples)
    (6, 32, 8, 12, 48, 1, 1, 1, 0, 1, 2),                  # 1x1: both gradients are plain batched products
    # strides > 1: dX as one stride-1 convolution per phase of the image
    (4, 32, 17, 19, 64, 3, 3, 2, 1, 1, 1),
    (2, 16, 20, 14, 32, 5, 4, (2, 3), (2, 1), 1, 2),       # different strides per axis, groups
    (3, 8, 9, 9, 16, 2, 2, 4, 0, 1, 1),                    # stride beyond the kernel: phases without taps stay zero
    (2, 8, 23, 23, 16, 7, 7, 2, 3, 1, 1),
    (2, 16, 11, 12, 32, 3, 3, (1, 2), (0, 2), 1, 1),       # stride on one axis only, rows left over by the stride
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.float16, "bf16"], ids=["fp32", "fp64", "fp16", "bf16"])
@pytest.mark.parametrize("geom", BACKWARD_GEOMS, ids=lambda g: "-".join(str(v).replace(" ", "") for v in g))
def test_conv2d_backward_geometries(dtype, geom):
    """conv_dimage / conv_dkernel against torch autograd in double (and the oracle on the small cases),
    with and without accumulation into existing gradients."""
    B, C, H, W, O, kh, kw, s, p, d, groups = geom
    bf = dtype == "bf16"
    rng = np.random.default_rng(1400 + C + H)
    x = randn(rng, (B, C, H, W), dtype)
    w = randn(rng, (O, C // groups, kh, kw), dtype, 1.0 / np.sqrt(C // groups * kh * kw))
    tx, tw = to_torch(x, DEV, bf), to_torch(w, DEV, bf)
    rx = tx.double().requires_grad_(True)
    rw = tw.double().requires_grad_(True)
    ry = torch.nn.functional.conv2d(rx, rw, None, s, p, d, groups)
    g = randn(rng, tuple(ry.shape), dtype)
    tg = to_torch(g, DEV, bf)
    ry.backward(tg.double())
    dx, dw = F.conv2d_backward(tx, tw, tg, stride=s, padding=p, dilation=d, groups=groups)
    assert dx.shape == tx.shape and dw.shape == tw.shape
    sx, sw = rx.grad.abs().max().item(), rw.grad.abs().max().item()
    if dtype in (np.float32, np.float64):
        kx = O // groups * kh * kw
        kw_ = B * ry.shape[2] * ry.shape[3]
        tolx = 1e-5 * kx * float(tg.abs().max().item() * tw.abs().max().item())
        tolw = 1e-5 * kw_ * float(tg.abs().max().item() * tx.abs().max().item())
    else:
        tolx, tolw = HALF_REL * sx, HALF_REL * sw
    assert (dx.double() - rx.grad).abs().max().item() <= tolx
    assert (dw.double() - rw.grad).abs().max().item() <= tolw
    if B * C * H * W <= 20000 and dtype in (np.float32, np.float64):      # the oracle's col2im is fp32 / fp64 only
        odx, odw = oracle.conv2d_backward(x, w, g, s, p, d, groups)
        assert np.abs(dx.cpu().numpy().astype(np.float64) - odx.astype(np.float64)).max() <= tolx
        assert np.abs(dw.cpu().numpy().astype(np.float64) - odw.astype(np.float64)).max() <= tolw
    # accumulate: the gradients are added to what the buffers hold
    dx2, dw2 = dx.clone(), dw.clone()
    lib = _lib.load()
    ws_bytes = lib.ntg_conv2d_backward_workspace_bytes(F.ntg_dtype(tx), B, C, H, W, O, kh, kw, *F._pair(s), *F._pair(p), *F._pair(d), groups)
    assert ws_bytes > 0
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=DEV)
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    _lib.check(lib.ntg_conv2d_backward_dev(F.ntg_dtype(tx), tx.data_ptr(), tw.data_ptr(), tg.data_ptr(), dx2.data_ptr(), dw2.data_ptr(),
                                           ws.data_ptr(), ws_bytes, B, C, H, W, O, kh, kw, *F._pair(s), *F._pair(p), *F._pair(d),
                                           groups, 1, st))
    assert (dx2.double() - 2 * rx.grad).abs().max().item() <= 2 * tolx + (0 if dtype in (np.float32, np.float64) else HALF_REL * sx)
    assert (dw2.double() - 2 * rw.grad).abs().max().item() <= 2 * tolw + (0 if dtype in (np.float32, np.float64) else HALF_REL * sw)


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.float16, np.int32])
def test_conv2d_random_vs_oracle(dtype):
    rng = np.random.default_rng(900)
    x = (rng.standard_normal((3, 6, 14, 11)) * (4 if dtype == np.int32 else 1)).astype(dtype)
    w = (rng.standard_normal((8, 3, 3, 2)) * (4 if dtype == np.int32 else 1)).astype(dtype)
    out = F.conv2d(dev(x), dev(w), stride=(2, 1), padding=(1, 2), dilation=(1, 2), groups=2).cpu().numpy()
    ref = oracle.conv2d(x, w, (2, 1), (1, 2), (1, 2), 2)
    if dtype == np.int32:
        assert np.array_equal(out, ref)
    elif dtype == np.float16:
        assert np.abs(out.astype(np.float64) - ref.astype(np.float64)).max() <= HALF_REL * np.abs(ref.astype(np.float64)).max()
    else:
        assert np.abs(out - ref).max() <= 1e-5 * 18 * np.abs(x).max() * np.abs(w).max()
    with pytest.raises(ValueError):
        F.conv2d(dev(x), dev(w), groups=4)


IMPLICIT_GEOMS = [
    # (B, C, H, W, O, kh, kw, stride, padding, dilation, groups)
    (2, 8, 20, 23, 16, 3, 3, 1, 1, 1, 1),
    (3, 6, 17, 9, 9, 2, 4, (2, 1), (0, 3), (2, 1), 3),
    (2, 5, 12, 12, 7, 5, 5, 2, 2, 1, 1),
    (1, 3, 7, 31, 4, 1, 1, 1, 0, 1, 1),
    (2, 4, 9, 9, 6, 3, 3, 3, (4, 0), (1, 2), 2),          # padding wider than the kernel reach
    (16, 64, 28, 28, 128, 3, 3, 1, 1, 1, 1),               # enough tiles for the large-tile kernels
    (24, 32, 33, 35, 96, 3, 3, 2, 1, 1, 2),
    # channel counts that fill whole 64-byte runs (the channels-last gather) with output planes of odd size
    (4, 64, 15, 15, 40, 3, 3, 1, 1, 1, 1),                 # Ho*Wo = 225
    (3, 64, 14, 14, 48, 3, 3, 2, 1, 1, 2),                 # Ho*Wo = 49, two groups of 32 channels
    (2, 128, 19, 11, 72, 3, 2, 1, (2, 0), (2, 1), 1),               # Ho*Wo = 190
    (2, 64, 1, 50, 48, 1, 5, 1, (0, 2), 1, 1),                      # one image row: what conv1d lowers to
    (1, 32, 40, 6, 8, 4, 1, (3, 1), 0, (2, 1), 1),                  # fewer filters than one tile row, one tap column
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.float16, "bf16"], ids=["fp32", "fp64", "fp16", "bf16"])
@pytest.mark.parametrize("geom", IMPLICIT_GEOMS, ids=lambda g: "-".join(str(v).replace(" ", "") for v in g))
def test_conv2d_implicit_gather(dtype, geom):
    """The floating dtypes never store the unfolded matrix: the GEMM gathers it.  It must equal
    W_g . unfold2d(x) formed explicitly (bit for bit where both use the same kernel), the oracle on
    the small cases and torch's conv2d in double on all."""
    B, C, H, W, O, kh, kw, s, p, d, groups = geom
    bf = dtype == "bf16"
    rng = np.random.default_rng(1300 + C + H)
    x = randn(rng, (B, C, H, W), dtype)
    w = randn(rng, (O, C // groups, kh, kw), dtype, 1.0 / np.sqrt(C // groups * kh * kw))
    tx, tw = to_torch(x, DEV, bf), to_torch(w, DEV, bf)
    lib = _lib.load()
    assert lib.ntg_conv2d_forward_workspace_bytes(F.ntg_dtype(tx), B, C, H, W, kh, kw, 1, 1, 0, 0, 1, 1) == 0
    out = F.conv2d(tx, tw, stride=s, padding=p, dilation=d, groups=groups)
    ref = torch.nn.functional.conv2d(tx.double(), tw.double(), None, s, p, d, groups)
    assert out.shape == ref.shape
    K = C // groups * kh * kw
    scale = ref.abs().max().item()
    if dtype in (np.float32, np.float64):
        tol = 1e-5 * K * float(tx.abs().max() * tw.abs().max())
        assert (out.double() - ref).abs().max().item() <= tol
        # explicit form with the same GEMM: unfold2d, then W_g . col_b per group
        col = F.unfold2d(tx, (kh, kw), dilation=d, padding=p, stride=s)                    # [B, C*kh*kw, L]
        og = O // groups
        for g in range(groups):
            wg = tw[g * og:(g + 1) * og].reshape(og, K).contiguous()
            cg = col[:, g * K:(g + 1) * K].contiguous()
            exp = F.matmult(wg.expand(B, og, K).contiguous(), cg)
            got = out[:, g * og:(g + 1) * og].reshape(B, og, -1)
            assert (got.double() - exp.double()).abs().max().item() <= tol * 1e-1
    else:
        assert ((out.double() - ref).abs().max().item()) <= HALF_REL * scale
    if B * C * H * W <= 20000 and not bf:
        oref = oracle.conv2d(x, w, s, p, d, groups)
        err = np.abs(out.cpu().numpy().astype(np.float64) - oref.astype(np.float64)).max()
        assert err <= (HALF_REL * scale if dtype == np.float16 else 1e-5 * K * np.abs(x).max() * np.abs(w).max())


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.float16, "bf16", np.int32, np.int8], ids=["fp32", "fp64", "fp16", "bf16", "int32", "int8"])
def test_conv2d_pointwise_is_a_product_on_the_image(dtype):
    """1x1 kernel, stride 1, no padding: unfold2d is the identity (conv.cpp:94 multiplies by the image itself), so the
    library runs W_g . x_b in place without a col buffer -- every dtype, grouped, aligned rows or not.  Integers bit-exact
    against the oracle's conv2d, floats against torch in double."""
    bf = dtype == "bf16"
    integer = dtype in (np.int32, np.int8)
    rng = np.random.default_rng(1900)
    lib = _lib.load()
    for (B, C, H, W, O, groups) in [(3, 64, 8, 12, 40, 1), (2, 96, 7, 7, 64, 2), (5, 24, 9, 5, 18, 3)]:
        if integer:
            x = rng.integers(-100, 100, (B, C, H, W)).astype(dtype)
            w = rng.integers(-100, 100, (O, C // groups, 1, 1)).astype(dtype)
        else:
            x = randn(rng, (B, C, H, W), dtype)
            w = randn(rng, (O, C // groups, 1, 1), dtype, 1.0 / np.sqrt(C // groups))
        tx, tw = to_torch(x, DEV, bf), to_torch(w, DEV, bf)
        assert lib.ntg_conv2d_forward_workspace_bytes(F.ntg_dtype(tx), B, C, H, W, 1, 1, 1, 1, 0, 0, 1, 1) == 0
        out = F.conv2d(tx, tw, groups=groups)
        assert tuple(out.shape) == (B, O, H, W)
        if integer:
            assert np.array_equal(out.cpu().numpy(), oracle.conv2d(x, w, 1, 0, 1, groups))
            continue
        ref = torch.nn.functional.conv2d(tx.double(), tw.double(), None, 1, 0, 1, groups)
        err = (out.double() - ref).abs().max().item()
        if dtype in (np.float32, np.float64):
            assert err <= 1e-5 * (C // groups) * float(tx.abs().max() * tw.abs().max())
        else:
            assert err <= HALF_REL * ref.abs().max().item()


@pytest.mark.parametrize("seed,big", [(11, False), (12, False), (13, True)], ids=["small-a", "small-b", "large"])
def test_conv2d_random_geometries_forward_and_gradients(seed, big):
    """Seeded random geometries (channels per group from 3 to 256, kernels up to 5x5, strides up to 3, dilation, padding,
    groups, batches up to 64, Float32 / BFloat16 / Float16) through conv2d and both gradients against torch in double:
    whichever of the kernels a geometry selects -- channels-last with or without padded channels, phases, several images
    per K loop, pointwise products, element-wise gathers, GEMM + col2im -- the result must be the convolution."""
    rng = np.random.default_rng(seed)
    for it in range(24 if big else 60):
        dt = [torch.float32, torch.bfloat16, torch.float16][int(rng.integers(0, 3))]
        groups = int(rng.choice([1, 1, 1, 2, 4]))
        cg = int(rng.choice([16, 32, 64, 128, 256] if big else [3, 8, 12, 16, 24, 32, 48, 64]))
        og = int(rng.choice([16, 32, 64, 128, 256] if big else [4, 8, 16, 24, 32, 40, 64, 96]))
        kh, kw = int(rng.integers(1, 6)), int(rng.integers(1, 6))
        s = (int(rng.integers(1, 4)), int(rng.integers(1, 4))) if rng.random() < 0.5 else (1, 1)
        d = (int(rng.integers(1, 3)), int(rng.integers(1, 3))) if rng.random() < 0.3 else (1, 1)
        p = (int(rng.integers(0, 4)), int(rng.integers(0, 4)))
        H, W = int(rng.integers(1, 50 if big else 30)), int(rng.integers(1, 50 if big else 30))
        B = int(rng.choice([1, 2, 16, 64, 24] if big else [1, 2, 3, 8, 33]))
        if H + 2 * p[0] - d[0] * (kh - 1) - 1 < 0 or W + 2 * p[1] - d[1] * (kw - 1) - 1 < 0:
            continue
        case = f"dt={dt} B={B} C={cg * groups} H={H} W={W} O={og * groups} k=({kh},{kw}) s={s} p={p} d={d} groups={groups}"
        print(case, flush=True)
        x = torch.randn(B, cg * groups, H, W, device=DEV).to(dt)
        w = (torch.randn(og * groups, cg, kh, kw, device=DEV) / (cg * kh * kw) ** 0.5).to(dt)
        xr, wr = x.double().requires_grad_(True), w.double().requires_grad_(True)
        yr = torch.nn.functional.conv2d(xr, wr, None, s, p, d, groups)
        g = torch.randn_like(yr).to(dt)
        yr.backward(g.double())
        y = F.conv2d(x, w, stride=s, padding=p, dilation=d, groups=groups)
        dx, dw = F.conv2d_backward(x, w, g, stride=s, padding=p, dilation=d, groups=groups)
        if dt == torch.float32:
            L = yr.shape[2] * yr.shape[3]
            tols = (1e-5 * cg * kh * kw * float(x.abs().max() * w.abs().max()), 1e-5 * og * kh * kw * float(g.abs().max() * w.abs().max()),
                    1e-5 * B * L * float(g.abs().max() * x.abs().max()))
        else:
            tols = tuple(HALF_REL * max(r.abs().max().item(), 1e-30) for r in (yr, xr.grad, wr.grad))
        for got, ref, tol, what in ((y, yr.detach(), tols[0], "y"), (dx, xr.grad, tols[1], "dx"), (dw, wr.grad, tols[2], "dw")):
            assert (got.double() - ref).abs().max().item() <= tol, (case, what)


def _gpu_family(golden_dir, name, sfx, fwd, bwd, ofwd, obwd, kw):
    x, w, exp, g, xg, wg = (load(golden_dir, f"{name}_{part}{sfx}") for part in ("input", "weight", "output", "grad", "xgrad", "wgrad"))
    out = fwd(dev(x), dev(w), **kw).cpu().numpy()
    assert out.shape == exp.shape
    assert np.abs(out - exp).max() <= 1e-4 * max(1.0, np.abs(exp).max())
    assert np.abs(out - ofwd(x, w, **kw)).max() <= 1e-5 * max(1.0, np.abs(exp).max())
    dx, dw = bwd(dev(x), dev(w), dev(g), **kw)
    dx, dw = dx.cpu().numpy(), dw.cpu().numpy()
    assert dx.shape == xg.shape and dw.shape == wg.shape
    assert np.abs(dx - xg).max() <= 1e-4 * max(1.0, np.abs(xg).max())
    assert np.abs(dw - wg).max() <= 1e-4 * max(1.0, np.abs(wg).max())
    odx, odw = obwd(x, w, g, **kw)
    assert np.abs(dx - odx).max() <= 1e-5 * max(1.0, np.abs(xg).max())
    assert np.abs(dw - odw).max() <= 1e-5 * max(1.0, np.abs(wg).max())


@pytest.mark.parametrize("sfx,kw", [("", dict(stride=1, padding=1)), ("_grouped", dict(stride=1, groups=2)),
                                    ("_batched", dict(stride=1, padding=1)), ("_grouped_batched", dict(stride=1, groups=2))])
def test_conv1d_golden(golden_dir, sfx, kw):
    """tests/src/conv_autograd_test.cpp:125-247 (conv1d outputs and gradients) on the GPU path."""
    _gpu_family(golden_dir, "conv1d", sfx, F.conv1d, F.conv1d_backward, oracle.conv1d, oracle.conv1d_backward, kw)


@pytest.mark.parametrize("sfx,kw", [("", dict(stride=2, output_padding=1)), ("_grouped", dict(stride=1, groups=2, padding=1)),
                                    ("_grouped_bigger", dict(stride=1, groups=5, padding=1)),
                                    ("_batched", dict(stride=2, output_padding=1, padding=1)),
                                    ("_grouped_batched", dict(stride=1, groups=2, padding=1))])
def test_conv_transpose1d_golden(golden_dir, sfx, kw):
    """tests/src/conv_autograd_test.cpp:555-716 on the GPU path."""
    _gpu_family(golden_dir, "conv_transpose1d", sfx, F.conv_transpose1d, F.conv_transpose1d_backward,
                oracle.conv_transpose1d, oracle.conv_transpose1d_backward, kw)


@pytest.mark.parametrize("sfx,kw", [("", dict(stride=2, output_padding=1)), ("_grouped", dict(stride=1, groups=5, padding=1)),
                                    ("_batched", dict(stride=2, output_padding=1, padding=1)),
                                    ("_grouped_batched", dict(stride=1, groups=2, padding=1))])
def test_conv_transpose2d_golden(golden_dir, sfx, kw):
    """tests/src/conv_autograd_test.cpp:720-846 on the GPU path, device and host entry points."""
    _gpu_family(golden_dir, "conv_transpose2d", sfx, F.conv_transpose2d, F.conv_transpose2d_backward,
                oracle.conv_transpose2d, oracle.conv_transpose2d_backward, kw)
    x = load(golden_dir, "conv_transpose2d_input" + sfx)
    w = load(golden_dir, "conv_transpose2d_weight" + sfx)
    exp = load(golden_dir, "conv_transpose2d_output" + sfx)
    lib = _lib.load()
    B, Cin, H, W = x.shape
    _, Cog, kh, kw_ = w.shape
    groups = kw.get("groups", 1)
    s, p, op = kw.get("stride", 1), kw.get("padding", 0), kw.get("output_padding", 0)
    y = np.full(exp.shape, np.nan, np.float32)
    ptr = lambda a: np.ascontiguousarray(a).ctypes.data_as(ctypes.c_void_p)
    _lib.check(lib.ntg_conv_transpose2d(_lib.FLOAT32, ptr(x), ptr(w), y.ctypes.data_as(ctypes.c_void_p), B, Cin, H, W, Cog * groups,
                                        kh, kw_, s, s, p, p, 1, 1, op, op, groups))
    assert np.array_equal(y, F.conv_transpose2d(dev(x), dev(w), **kw).cpu().numpy())


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.float16, "bf16", np.int32], ids=["fp32", "fp64", "fp16", "bf16", "int32"])
def test_conv_transpose2d_random_vs_torch(dtype):
    """Strides, dilations, groups and output_padding against torch's conv_transpose2d in double; integers bit-exact."""
    bf = dtype == "bf16"
    rng = np.random.default_rng(1500)
    for (B, Cin, H, W, Cout, kh, kw_, s, p, op, d, groups) in [
            (2, 6, 9, 11, 8, 3, 3, 1, 1, 0, 1, 2), (3, 4, 7, 6, 6, 2, 4, (2, 3), (1, 0), (1, 2), (2, 1), 1),
            (2, 8, 13, 12, 4, 5, 3, 2, 2, 1, 1, 4), (4, 32, 20, 20, 48, 3, 3, 1, 1, 0, 1, 1)]:
        if dtype == np.int32:
            x = rng.integers(-4, 5, (B, Cin, H, W)).astype(np.int32)
            w = rng.integers(-4, 5, (Cin, Cout // groups, kh, kw_)).astype(np.int32)
        else:
            x = randn(rng, (B, Cin, H, W), dtype)
            w = randn(rng, (Cin, Cout // groups, kh, kw_), dtype, 1.0 / np.sqrt(Cin // groups * kh * kw_))
        tx, tw = to_torch(x, DEV, bf), to_torch(w, DEV, bf)
        out = F.conv_transpose2d(tx, tw, stride=s, padding=p, output_padding=op, dilation=d, groups=groups)
        ref = torch.nn.functional.conv_transpose2d(tx.double().cpu(), tw.double().cpu(), None, s, p, op, groups, d)
        assert tuple(out.shape) == tuple(ref.shape)
        got = out.double().cpu()
        if dtype == np.int32:
            assert torch.equal(got, ref)
        elif dtype in (np.float32, np.float64):
            K = Cin // groups * kh * kw_
            assert (got - ref).abs().max().item() <= 1e-5 * K * float(tx.abs().max().item() * tw.abs().max().item())
        else:
            assert (got - ref).abs().max().item() <= HALF_REL * ref.abs().max().item()
    with pytest.raises(ValueError):
        F.conv_transpose2d(tx, tw[:-1])
    with pytest.raises((ValueError, _lib.NtgError)):
        F.conv_transpose2d(tx, tw, stride=1, output_padding=1)


@pytest.mark.parametrize("sfx,kw", [("", dict(stride=1, padding=1)), ("_grouped", dict(stride=1, groups=2)),
                                    ("_batched", dict(stride=1, padding=1)), ("_grouped_batched", dict(stride=1, groups=2))])
def test_conv3d_golden(golden_dir, sfx, kw):
    """tests/src/conv_autograd_test.cpp:375-497 on the GPU path."""
    _gpu_family(golden_dir, "conv3d", sfx, F.conv3d, F.conv3d_backward, oracle.convnd, oracle.convnd_backward, kw)


@pytest.mark.parametrize("sfx,kw", [("", dict(stride=2, output_padding=1)), ("_grouped_batched", dict(stride=1, groups=2, padding=1))])
def test_conv_transpose3d_golden(golden_dir, sfx, kw):
    """tests/src/conv_autograd_test.cpp:847-971 on the GPU path."""
    _gpu_family(golden_dir, "conv_transpose3d", sfx, F.conv_transpose3d, F.conv_transposend_backward,
                oracle.conv_transposend, oracle.conv_transposend_backward, kw)


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.float16, "bf16", np.int32], ids=["fp32", "fp64", "fp16", "bf16", "int32"])
def test_conv3d_and_transpose_random_vs_torch(dtype):
    """conv3d / conv_transpose3d forward and gradients with strides, dilations, padding and groups against torch in double;
    the unfold itself bit-exact against the oracle; 4 spatial axes against the oracle."""
    bf = dtype == "bf16"
    ints = dtype == np.int32
    rng = np.random.default_rng(1600)
    for (B, C, size, O, k, s, p, d, groups) in [(2, 4, (6, 7, 8), 6, (2, 3, 2), (1, 2, 1), (1, 0, 2), (2, 1, 1), 2),
                                                (3, 3, (9, 8, 7), 5, (3, 3, 3), 1, 1, 1, 1), (2, 8, (5, 10, 6), 4, (1, 2, 3), 2, (0, 1, 1), 1, 4)]:
        if ints:
            x = rng.integers(-4, 5, (B, C) + size).astype(np.int32)
            w = rng.integers(-4, 5, (O, C // groups) + k).astype(np.int32)
        else:
            x = randn(rng, (B, C) + size, dtype)
            w = randn(rng, (O, C // groups) + k, dtype, 1.0 / np.sqrt(C // groups * np.prod(k)))
        tx, tw = to_torch(x, DEV, bf), to_torch(w, DEV, bf)
        y = F.conv3d(tx, tw, stride=s, padding=p, dilation=d, groups=groups)
        rx = tx.double().cpu().requires_grad_(not ints)
        rw = tw.double().cpu().requires_grad_(not ints)
        ry = torch.nn.functional.conv3d(rx, rw, None, s, p, d, groups)
        assert tuple(y.shape) == tuple(ry.shape)
        K = C // groups * int(np.prod(k))
        if ints:
            assert torch.equal(y.double().cpu(), ry)
            continue
        tol = (1e-5 * K * float(tx.abs().max().item() * tw.abs().max().item())) if dtype in (np.float32, np.float64) else HALF_REL * ry.abs().max().item()
        assert (y.double().cpu() - ry.detach()).abs().max().item() <= tol
        g = randn(rng, tuple(ry.shape), dtype)
        tg = to_torch(g, DEV, bf)
        ry.backward(tg.double().cpu())
        dx, dw = F.conv3d_backward(tx, tw, tg, stride=s, padding=p, dilation=d, groups=groups)
        rel = 1e-4 if dtype in (np.float32, np.float64) else HALF_REL
        assert (dx.double().cpu() - rx.grad).abs().max().item() <= rel * max(1.0, rx.grad.abs().max().item())
        assert (dw.double().cpu() - rw.grad).abs().max().item() <= rel * max(1.0, rw.grad.abs().max().item())
        # transposed: the same kernel tensor read as [Cin = O, Cout/groups = C/groups, *k]
        xt = to_torch(randn(rng, tuple(ry.shape), dtype), DEV, bf)
        yt = F.conv_transpose3d(xt, tw, stride=s, padding=p, dilation=d, groups=groups)
        rt = torch.nn.functional.conv_transpose3d(xt.double().cpu(), tw.double().cpu(), None, s, p, 0, groups, d)
        assert tuple(yt.shape) == tuple(rt.shape)
        assert (yt.double().cpu() - rt).abs().max().item() <= rel * max(1.0, rt.abs().max().item()) * (10 if dtype in (np.float32, np.float64) else 1)
    # 4 spatial axes, and the unfold alone
    x4 = randn(rng, (2, 3, 4, 5, 4, 6), np.float32)
    w4 = randn(rng, (4, 3, 2, 2, 1, 3), np.float32, 0.3)
    y4 = F.convnd(dev(x4), dev(w4), stride=(1, 2, 1, 1), padding=(1, 0, 0, 1), dilation=1)
    assert np.abs(y4.cpu().numpy() - oracle.convnd(x4, w4, (1, 2, 1, 1), (1, 0, 0, 1), 1)).max() <= 1e-4
    lib = _lib.load()
    x3 = randn(rng, (2, 3, 6, 5, 7), np.float32)
    ref_col, out = oracle.unfoldnd(x3, (2, 3, 2), (2, 1, 1), (1, 0, 2), (1, 2, 1))
    col = torch.empty(ref_col.shape, dtype=torch.float32, device=DEV)
    arr = lambda v: (ctypes.c_int64 * 3)(*v)
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    _lib.check(lib.ntg_unfoldnd_dev(_lib.FLOAT32, dev(x3).data_ptr(), col.data_ptr(), 2, 3, 3, arr((6, 5, 7)), arr((2, 3, 2)), arr((1, 2, 1)),
                                    arr((1, 0, 2)), arr((2, 1, 1)), st))
    assert np.array_equal(col.cpu().numpy(), ref_col)
    gcol = randn(rng, ref_col.shape, np.float32)
    back = torch.empty((2, 3, 6, 5, 7), dtype=torch.float32, device=DEV)
    _lib.check(lib.ntg_unfoldnd_backward_dev(_lib.FLOAT32, dev(gcol).data_ptr(), back.data_ptr(), 2, 3, 3, arr((6, 5, 7)), arr((2, 3, 2)),
                                             arr((1, 2, 1)), arr((1, 0, 2)), arr((2, 1, 1)), 0, st))
    assert np.array_equal(back.cpu().numpy(), oracle.unfoldnd_backward(gcol, (6, 5, 7), (2, 3, 2), (2, 1, 1), (1, 0, 2), (1, 2, 1)))


@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["fp32", "fp16"])
def test_conv2d_wide_kernels_and_empty_inputs(dtype):
    """Kernels wider than 8 taps on an axis leave the implicit-GEMM path (one byte of tap mask per pixel) for the stored
    im2col matrix; zero-sized batches and channels return without touching memory; bad geometry is an error."""
    rng = np.random.default_rng(1700)
    lib = _lib.load()
    for (B, C, H, W, O, kh, kw_, s, p, d, groups) in [(2, 4, 20, 15, 6, 9, 3, 1, (4, 1), 1, 2), (3, 2, 8, 30, 4, 2, 11, (1, 2), (0, 5), 1, 1)]:
        x = randn(rng, (B, C, H, W), dtype)
        w = randn(rng, (O, C // groups, kh, kw_), dtype, 1.0 / np.sqrt(C // groups * kh * kw_))
        tx, tw = dev(x), dev(w)
        assert lib.ntg_conv2d_forward_workspace_bytes(F.ntg_dtype(tx), B, C, H, W, kh, kw_, *F._pair(s), *F._pair(p), *F._pair(d)) > 0
        rx, rw = tx.double().cpu().requires_grad_(True), tw.double().cpu().requires_grad_(True)
        ry = torch.nn.functional.conv2d(rx, rw, None, s, p, d, groups)
        y = F.conv2d(tx, tw, stride=s, padding=p, dilation=d, groups=groups)
        tol = 1e-4 if dtype == np.float32 else HALF_REL * ry.abs().max().item()
        assert (y.double().cpu() - ry.detach()).abs().max().item() <= tol
        g = dev(randn(rng, tuple(ry.shape), dtype))
        ry.backward(g.double().cpu())
        dx, dw = F.conv2d_backward(tx, tw, g, stride=s, padding=p, dilation=d, groups=groups)
        assert (dx.double().cpu() - rx.grad).abs().max().item() <= (1e-4 if dtype == np.float32 else HALF_REL * rx.grad.abs().max().item())
        assert (dw.double().cpu() - rw.grad).abs().max().item() <= (1e-3 if dtype == np.float32 else HALF_REL * rw.grad.abs().max().item())
    # empty batch / no filters: nothing to do, no error
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    dt = F.ntg_dtype(tx)
    _lib.check(lib.ntg_conv2d_dev(dt, None, None, None, None, 0, 0, 3, 8, 8, 4, 3, 3, 1, 1, 1, 1, 1, 1, 1, st))
    _lib.check(lib.ntg_conv2d_dev(dt, tx.data_ptr(), tw.data_ptr(), None, None, 0, 2, 3, 8, 8, 0, 3, 3, 1, 1, 1, 1, 1, 1, 1, st))
    _lib.check(lib.ntg_conv2d_backward_dev(dt, None, None, None, None, None, None, 0, 0, 3, 8, 8, 4, 3, 3, 1, 1, 1, 1, 1, 1, 1, 0, st))
    # kernel larger than the padded image, channels not divisible by groups
    assert lib.ntg_conv2d_dev(dt, tx.data_ptr(), tw.data_ptr(), tx.data_ptr(), None, 0, 1, 3, 4, 4, 4, 7, 7, 1, 1, 1, 1, 1, 1, 1, st) == 1
    assert lib.ntg_conv2d_dev(dt, tx.data_ptr(), tw.data_ptr(), tx.data_ptr(), None, 0, 1, 3, 8, 8, 4, 3, 3, 1, 1, 1, 1, 1, 1, 2, st) == 1
    assert b"groups" in lib.ntg_last_error()


def test_config5a_conv2d_resnet_block():
    """image [64,256,56,56], weight [256,256,3,3], stride 1, pad 1 (GEMM M=200704, K=2304, N=256)."""
    rng = np.random.default_rng(1007)
    x = rng.standard_normal((64, 256, 56, 56)).astype(np.float32)
    w = (rng.standard_normal((256, 256, 3, 3)) / np.sqrt(2304.0)).astype(np.float32)
    tx, tw = dev(x), dev(w)
    out = F.conv2d(tx, tw, stride=1, padding=1)
    torch.cuda.synchronize()
    assert tuple(out.shape) == (64, 256, 56, 56)
    tol = float_tol(2304, x, w)
    for b in (0, 63):                                            # two whole images through the oracle
        ref = oracle.conv2d(x[b:b + 1], w, 1, 1, 1, 1, kind="tiled")
        assert np.abs(out[b:b + 1].cpu().numpy() - ref).max() <= tol
    ref_all = torch.nn.functional.conv2d(tx.double(), tw.double(), padding=1)
    assert (out.double() - ref_all).abs().max().item() <= tol
    # the same block in BFloat16: output pixels 0 .. 3071 of every image (12 tiles of 256) and pixels 3072 .. 3135 come from
    # two launches on different tiles, both gathering from a channels-last copy that carries the padding as a zero border
    xh, wh = tx.bfloat16(), tw.bfloat16()
    outh = F.conv2d(xh, wh, stride=1, padding=1)
    refh = torch.nn.functional.conv2d(xh.double(), wh.double(), padding=1)
    scale = refh.abs().max().item()
    flat, flat_ref = outh.double().reshape(64, 256, 3136), refh.reshape(64, 256, 3136)
    for lo, hi in ((0, 3072), (3072, 3136)):
        assert (flat[:, :, lo:hi] - flat_ref[:, :, lo:hi]).abs().max().item() <= HALF_REL * scale
    # and one rounding of the exact sum: two whole images, element by element
    for b in (0, 63):
        spread = torch.nn.functional.conv2d(xh[b:b + 1].double() ** 2, wh.double() ** 2, padding=1).sqrt()
        assert_one_rounding(outh[b:b + 1].double().cpu().numpy(), refh[b:b + 1].cpu().numpy(), spread.cpu().numpy(), 2304, "bf16", f"conv image {b}")
    del ref_all, refh


def test_config5a_conv2d_gradients_full_size():
    """Both gradients of the config-5a block at full size (channels-last kernels), Float32 against the stated bound
    and BFloat16 against 2e-2 of the largest gradient; references from torch autograd in double."""
    rng = np.random.default_rng(1008)
    x = dev(rng.standard_normal((64, 256, 56, 56)).astype(np.float32))
    w = dev((rng.standard_normal((256, 256, 3, 3)) / np.sqrt(2304.0)).astype(np.float32))
    g = dev(rng.standard_normal((64, 256, 56, 56)).astype(np.float32))
    for half in (False, True):
        tx, tw, tg = (t.bfloat16() if half else t for t in (x, w, g))
        rx = tx.double().requires_grad_(True)
        rw = tw.double().requires_grad_(True)
        torch.nn.functional.conv2d(rx, rw, padding=1).backward(tg.double())
        dx, dw = F.conv2d_backward(tx, tw, tg, stride=1, padding=1)
        ex = (dx.double() - rx.grad).abs().max().item()
        ew = (dw.double() - rw.grad).abs().max().item()
        if half:
            assert ex <= HALF_REL * rx.grad.abs().max().item()
            assert ew <= HALF_REL * rw.grad.abs().max().item()
            # dX is one rounding of the exact sum (whole tile columns and the narrow rest come from two launches)
            for b in (0, 63):
                spread = torch.nn.functional.conv_transpose2d(tg[b:b + 1].double() ** 2, tw.double() ** 2, padding=1).sqrt()
                assert_one_rounding(dx[b:b + 1].double().cpu().numpy(), rx.grad[b:b + 1].cpu().numpy(), spread.cpu().numpy(), 2304, "bf16", f"dX image {b}")
        else:
            assert ex <= 1e-5 * 2304 * float(tg.abs().max() * tw.abs().max())
            assert ew <= 1e-5 * 200704 * float(tg.abs().max() * tx.abs().max())
        del rx, rw, dx, dw


@pytest.mark.parametrize("ranges", [1, 3, 4, 6])
def test_conv2d_weight_gradient_k_ranges_across_images(ranges, monkeypatch):
    """The 16-bit weight gradient with the output pixels of all images cut into k ranges (forced through the library's
    NTG_DW_RANGES knob): ranges that end inside an image (4 ranges over 6 images), pairs of images (3), whole images (6) and
    everything in one (1), against torch autograd in double and against the per-image form; grouped as well."""
    rng = np.random.default_rng(77 + ranges)
    for groups, dt in ((1, torch.bfloat16), (2, torch.float16)):
        x = dev(rng.standard_normal((6, 16, 32, 32)).astype(np.float32)).to(dt)
        w = dev((rng.standard_normal((32, 16 // groups, 3, 3)) / 12.0).astype(np.float32)).to(dt)
        g = dev(rng.standard_normal((6, 32, 32, 32)).astype(np.float32)).to(dt)
        rx = x.double().requires_grad_(True)
        rw = w.double().requires_grad_(True)
        torch.nn.functional.conv2d(rx, rw, padding=1, groups=groups).backward(g.double())
        monkeypatch.setenv("NTG_DW_RANGES", "0")
        _, dw_images = F.conv2d_backward(x, w, g, stride=1, padding=1, groups=groups)
        monkeypatch.setenv("NTG_DW_RANGES", str(ranges))
        _, dw = F.conv2d_backward(x, w, g, stride=1, padding=1, groups=groups)
        monkeypatch.delenv("NTG_DW_RANGES")
        tol = HALF_REL * rw.grad.abs().max().item()
        assert (dw.double() - rw.grad).abs().max().item() <= tol, (groups, ranges)
        assert (dw.double() - dw_images.double()).abs().max().item() <= tol, (groups, ranges)
        if ranges == 6:
            # whole images per range: the same products and the same order of adding them up
            assert torch.equal(dw, dw_images)


@pytest.mark.parametrize("geom", [
    # (B, C, H, W, O, kh, kw, stride, padding, dilation, groups)
    (2, 8, 18, 18, 16, 3, 3, 1, 1, 1, 1),       # rows of the weights and of the output plane are 16-byte multiples: the DMA-fed gather
    (3, 16, 20, 12, 24, 3, 3, 2, 1, 1, 2),      # grouped, strided
    (2, 5, 9, 11, 7, 3, 2, 1, 0, 1, 1),         # nothing aligned: the register-staged gather
    (1, 12, 15, 15, 8, 5, 5, 1, 2, 2, 1),       # dilated
], ids=lambda g: "x".join(map(str, g)))
def test_conv2d_fp32_without_workspace_is_the_reference_chain_bit_for_bit(geom):
    """Float32 conv2d on the gathering kernels (no workspace): the k axis is the reference's own (channel, tap row, tap column)
    order of im2col, every output element is the chain c = 0; c = fma(w[o, kk], col[kk, l], c) in ascending kk -- the bits of
    unfold + matmult (conv.cpp:86-95), which the oracle restates."""
    B, C, H, W, O, kh, kw, st, pd, dl, groups = geom
    rng = np.random.default_rng(31 + B + C + O)
    x = rng.standard_normal((B, C, H, W)).astype(np.float32)
    w = (rng.standard_normal((O, C // groups, kh, kw)) * 3.0).astype(np.float32)
    want = oracle.conv2d(x, w, st, pd, dl, groups)
    tx, tw = dev(x), dev(w)
    out = torch.empty(want.shape, dtype=torch.float32, device=DEV)
    lib = _lib.load()
    need = lib.ntg_conv2d_forward_workspace_bytes(_lib.FLOAT32, B, C, H, W, kh, kw, st, st, pd, pd, dl, dl)
    assert need == 0
    _lib.check(lib.ntg_conv2d_dev(_lib.FLOAT32, tx.data_ptr(), tw.data_ptr(), out.data_ptr(), None, 0, B, C, H, W, O, kh, kw,
                                  st, st, pd, pd, dl, dl, groups, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (geom, int((got != want).sum()))
    # the host-pointer entry point (functional::conv2d's seam) takes the same kernels for Float32
    host = np.empty_like(want)
    vp = lambda a: a.ctypes.data_as(ctypes.c_void_p)
    _lib.check(lib.ntg_conv2d(_lib.FLOAT32, vp(x), vp(w), vp(host), B, C, H, W, O, kh, kw, st, st, pd, pd, dl, dl, groups))
    assert np.array_equal(host.view(np.uint32), want.view(np.uint32)), (geom, "host entry")


@pytest.mark.parametrize("geom", [
    (2, 8, 18, 18, 16, 3, 3, 1, 1, 1, 1),
    (3, 16, 20, 12, 24, 3, 3, 2, 1, 1, 2),
    (2, 5, 9, 11, 7, 3, 2, 1, 0, 1, 1),
    (1, 12, 15, 15, 8, 5, 5, 1, 2, 2, 1),
    (4, 6, 10, 10, 6, 1, 1, 1, 0, 1, 1),        # 1 x 1: products on the tensors where they lie
], ids=lambda g: "x".join(map(str, g)))
def test_conv2d_backward_fp32_host_entry_is_the_reference_bit_for_bit(geom):
    """ntg_conv2d_backward on host memory in Float32 runs the reference's own two algorithms -- conv_dimage as W^T . dY into the
    col matrix + col2im (conv.cpp:318-346), conv_dkernel as one product per image over the output pixels + the sum over the batch
    (conv.cpp:444-471) -- and returns the oracle's bits, also when it adds to gradients that are already there (square geometries here: one stride,
    padding and dilation for both axes)."""
    B, C, H, W, O, kh, kw, st, pd, dl, groups = geom
    rng = np.random.default_rng(97 + B + C + O)
    x = rng.standard_normal((B, C, H, W)).astype(np.float32)
    w = (rng.standard_normal((O, C // groups, kh, kw)) * 2.0).astype(np.float32)
    Ho = (H + 2 * pd - dl * (kh - 1) - 1) // st + 1
    Wo = (W + 2 * pd - dl * (kw - 1) - 1) // st + 1
    g = rng.standard_normal((B, O, Ho, Wo)).astype(np.float32)
    odx, odw = oracle.conv2d_backward(x, w, g, st, pd, dl, groups)
    lib = _lib.load()
    vp = lambda a: a.ctypes.data_as(ctypes.c_void_p)
    dx = np.full(x.shape, np.nan, np.float32)
    dw = np.full(w.shape, np.nan, np.float32)
    _lib.check(lib.ntg_conv2d_backward(_lib.FLOAT32, vp(x), vp(w), vp(g), vp(dx), vp(dw), B, C, H, W, O, kh, kw, st, st, pd, pd, dl, dl, groups, 0))
    assert np.array_equal(dx.view(np.uint32), odx.view(np.uint32)), (geom, "d_image", int((dx != odx).sum()))
    assert np.array_equal(dw.view(np.uint32), odw.view(np.uint32)), (geom, "d_kernel", int((dw != odw).sum()))
    dx0 = rng.standard_normal(x.shape).astype(np.float32)
    dw0 = rng.standard_normal(w.shape).astype(np.float32)
    dx, dw = dx0.copy(), dw0.copy()
    _lib.check(lib.ntg_conv2d_backward(_lib.FLOAT32, vp(x), vp(w), vp(g), vp(dx), vp(dw), B, C, H, W, O, kh, kw, st, st, pd, pd, dl, dl, groups, 1))
    # d_kernel: the summed per-image products are added in one addition (sum(0), then +=); d_image: unfold2d_backward scatters
    # onto the tensor it is handed, so the taps land on the old values one by one (conv.cpp:343-345)
    assert np.array_equal(dw.view(np.uint32), (dw0 + odw).view(np.uint32)), (geom, "d_kernel +=")
    from test_gpu_complex import _col2im_onto, _dcol_plane
    dcol = _dcol_plane(oracle, w, g, B, C, O, kh, kw, groups, None)
    want = _col2im_onto(dx0, dcol, (H, W), (kh, kw), dl, pd, st)
    assert np.array_equal(dx.view(np.uint32), np.ascontiguousarray(want).view(np.uint32)), (geom, "d_image +=")
