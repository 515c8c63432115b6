"""CPU oracle for NeuroTensor's dense matmult path -- TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this package; the shipped library never does.  The arithmetic lives in
``nt_oracle.c`` (built by ``oracle/Makefile`` into ``libnt_oracle.so``); this
module is the numpy face of it plus restatements of the Tensor-level functions
that sit above the GEMM in the reference:

  matmult / matmult_batch   nt/functional/cpu/matmult_cpu.cpp:97-153, 654-861
  linear                    nt/functional/cpu/matmult_cpu.cpp:1624-1714
  linear_backward           nt/nn/functional/matmult.cpp:253-275
  matmult_backward          nt/nn/functional/matmult.cpp:37-62
  unfold2d                  nt/functional/tensor_files/colim_transform.cpp:565-588
  conv2d                    nt/functional/tensor_files/conv.cpp:69-119
  conv2d_backward           nt/functional/tensor_files/conv.cpp:318-346, 444-471
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libnt_oracle.so")

# numeric values of nt::DType (nt/dtype/DType_enum.h:14-20); BF16/U64 are this build's extensions
F16, F32, F64 = 0, 1, 2
I8, I16, I32, I64 = 7, 8, 9, 10
U8, U16, U32 = 12, 13, 14
BF16, U64 = 100, 101
C32, C64, C128 = 4, 5, 6          # interleaved (re, im) pairs; numpy carries them as real arrays with a trailing axis of 2
F16_LANE8 = 200                   # closed form only: float16 values with k tiles of 8 -- one lane of a Complex32 product
_COMPLEX_REAL = {C32: np.dtype(np.float16), C64: np.dtype(np.float32), C128: np.dtype(np.float64)}

_NP_TO_DT = {
    np.dtype(np.float16): F16, np.dtype(np.float32): F32, np.dtype(np.float64): F64,
    np.dtype(np.int8): I8, np.dtype(np.int16): I16, np.dtype(np.int32): I32, np.dtype(np.int64): I64,
    np.dtype(np.uint8): U8, np.dtype(np.uint16): U16, np.dtype(np.uint32): U32, np.dtype(np.uint64): U64,
}


def build(force=False):
    """Compile libnt_oracle.so with the committed Makefile."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "libnt_oracle.so"])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        i64, vp, ci = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int
        L.oracle_matmult.argtypes = [ci, vp, vp, vp, i64, i64, i64, ci, ci]
        L.oracle_matmult_naive.argtypes = [ci, vp, vp, vp, i64, i64, i64, ci, ci]
        L.oracle_tiled_matmult.argtypes = [ci, vp, vp, vp, i64, i64, i64, ci, ci, ci]
        pp = ctypes.POINTER(ctypes.c_void_p)
        L.oracle_matmult_batch.argtypes = [ci, pp, pp, pp, i64, i64, i64, i64, ci, ci]
        L.oracle_tiled_matmult_batch.argtypes = [ci, pp, pp, pp, i64, i64, i64, i64, ci, ci, ci]
        L.oracle_tiled_threads.argtypes = [ci]
        L.oracle_unfold2d.argtypes = [i64, vp, vp] + [i64] * 12
        L.oracle_unfold2d_backward.argtypes = [ci, vp, vp] + [i64] * 12
        L.oracle_f32_to_f16.argtypes = [ctypes.c_float]
        L.oracle_f32_to_f16.restype = ctypes.c_uint16
        L.oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.oracle_f16_to_f32.restype = ctypes.c_float
        L.oracle_f32_to_bf16.argtypes = [ctypes.c_float]
        L.oracle_f32_to_bf16.restype = ctypes.c_uint16
        L.oracle_bf16_to_f32.argtypes = [ctypes.c_uint16]
        L.oracle_bf16_to_f32.restype = ctypes.c_float
        _lib = L
    return _lib


# --------------------------------------------------------------------------
# bfloat16 travels through numpy as uint16 bit patterns
# --------------------------------------------------------------------------

def to_bf16_bits(x):
    """float32 array -> uint16 bfloat16 bit patterns, round to nearest even."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    r[nan] = ((u[nan] >> 16) | 0x40).astype(np.uint16)
    return r


def from_bf16_bits(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


_HALF_AS_COMPLEX32_LANE = [False]


def dtype_code(arr, dt=None):
    if dt is not None:
        return dt
    if _HALF_AS_COMPLEX32_LANE[0] and arr.dtype == np.float16:
        return F16_LANE8
    return _NP_TO_DT[arr.dtype]


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _mkn(a_shape, b_shape, ta, tb):
    """Logical sizes after the flags (matmult_cpu.cpp:97-107)."""
    m, k = (a_shape[-1], a_shape[-2]) if ta else (a_shape[-2], a_shape[-1])
    kb, n = (b_shape[-1], b_shape[-2]) if tb else (b_shape[-2], b_shape[-1])
    if k != kb:
        raise ValueError(f"inner sizes differ: {k} vs {kb}")
    return m, k, n


def matmult2d(a, b, c=None, ta=False, tb=False, dt=None, kind="closed", threads=0):
    """C[m,n] (+)= op(a).op(b) on 2-D contiguous arrays. kind: closed | naive | tiled."""
    a = np.ascontiguousarray(a)
    b = np.ascontiguousarray(b)
    code = dtype_code(a, dt)
    m, k, n = _mkn(a.shape, b.shape, ta, tb)
    if c is None:
        c = np.zeros((m, n), dtype=a.dtype)      # matmult_cpu.cpp:110
    assert c.flags["C_CONTIGUOUS"] and c.shape == (m, n) and c.dtype == a.dtype
    L = lib()
    if kind == "closed":
        rc = L.oracle_matmult(code, _ptr(a), _ptr(b), _ptr(c), m, k, n, int(ta), int(tb))
    elif kind == "naive":
        rc = L.oracle_matmult_naive(code, _ptr(a), _ptr(b), _ptr(c), m, k, n, int(ta), int(tb))
    elif kind == "tiled":
        rc = L.oracle_tiled_matmult(code, _ptr(a), _ptr(b), _ptr(c), m, k, n, int(ta), int(tb), threads)
    else:
        raise ValueError(kind)
    if rc:
        raise RuntimeError(f"oracle matmult failed rc={rc}")
    return c


def matmult2d_complex(a, b, c=None, ta=False, tb=False, dt=C64, kind="closed"):
    """The reference's complex matmult (lane-wise on interleaved re / im, see closed_c64 in nt_oracle.c) on arrays
    [rows, cols, 2] of the real type (float16 for C32, float32 for C64, float64 for C128)."""
    real = _COMPLEX_REAL[dt]
    a = np.ascontiguousarray(a, dtype=real)
    b = np.ascontiguousarray(b, dtype=real)
    assert a.ndim == 3 and b.ndim == 3 and a.shape[2] == 2 and b.shape[2] == 2
    m, k, n = _mkn(a.shape[:2], b.shape[:2], ta, tb)
    if c is None:
        c = np.zeros((m, n, 2), dtype=real)
    assert c.flags["C_CONTIGUOUS"] and c.shape == (m, n, 2) and c.dtype == real
    L = lib()
    fn = L.oracle_matmult if kind == "closed" else L.oracle_matmult_naive
    rc = fn(dt, _ptr(a), _ptr(b), _ptr(c), m, k, n, int(ta), int(tb))
    if rc:
        raise RuntimeError(f"oracle complex matmult failed rc={rc}")
    return c


def matmult(a, b, c=None, ta=False, tb=False, dt=None, kind="closed", threads=0):
    """N-D x K-D matmult with the reference's batch rule: the leading batch dims of
    the lower-rank operand must equal the trailing batch dims of the higher-rank
    one; the lower-rank operand is reused cyclically (matmult_cpu.cpp:863-1005)."""
    a = np.ascontiguousarray(a)
    b = np.ascontiguousarray(b)
    if a.ndim < 2 or b.ndim < 2:
        raise ValueError("matmult needs >=2 dims")
    m, k, n = _mkn(a.shape, b.shape, ta, tb)
    if a.ndim == 2 and b.ndim == 2:
        return matmult2d(a, b, c, ta, tb, dt, kind, threads)
    abatch, bbatch = a.shape[:-2], b.shape[:-2]
    if len(abatch) >= len(bbatch):
        big, small = abatch, bbatch
    else:
        big, small = bbatch, abatch
    if len(small) and tuple(big[len(big) - len(small):]) != tuple(small):
        raise ValueError(f"batch dims do not line up: {abatch} vs {bbatch}")
    nb = int(np.prod(big)) if len(big) else 1
    na = int(np.prod(abatch)) if len(abatch) else 1
    nbb = int(np.prod(bbatch)) if len(bbatch) else 1
    a3 = a.reshape(na, *a.shape[-2:])
    b3 = b.reshape(nbb, *b.shape[-2:])
    out_shape = tuple(big) + (m, n)
    if c is None:
        c = np.zeros(out_shape, dtype=a.dtype)    # matmult_cpu.cpp:707
    assert c.flags["C_CONTIGUOUS"] and c.size == nb * m * n
    c3 = c.reshape(nb, m, n)
    for i in range(nb):
        matmult2d(a3[i % na], b3[i % nbb], c3[i], ta, tb, dt, kind, threads)
    return c


def matmult_batch_ptrs(As, Bs, Cs, ta=False, tb=False, dt=None, tiled=False, threads=0):
    """nt_matmult_batch on lists of 2-D arrays (entries may repeat)."""
    code = dtype_code(As[0], dt)
    m, k, n = _mkn(As[0].shape, Bs[0].shape, ta, tb)
    nb = len(As)
    arr = ctypes.c_void_p * nb
    pa = arr(*[x.ctypes.data for x in As])
    pb = arr(*[x.ctypes.data for x in Bs])
    pc = arr(*[x.ctypes.data for x in Cs])
    L = lib()
    if tiled:
        rc = L.oracle_tiled_matmult_batch(code, pa, pb, pc, nb, m, k, n, int(ta), int(tb), threads)
    else:
        rc = L.oracle_matmult_batch(code, pa, pb, pc, nb, m, k, n, int(ta), int(tb))
    if rc:
        raise RuntimeError(f"oracle batch failed rc={rc}")
    return Cs


def linear(x, w, bias, ta=False, tb=False, dt=None, kind="closed"):
    """bias broadcast to the output shape is the INITIAL ACCUMULATOR of the
    accumulating GEMM (matmult_cpu.cpp:1637-1647, 1667-1673)."""
    x = np.ascontiguousarray(x)
    w = np.ascontiguousarray(w)
    m, k, n = _mkn(x.shape, w.shape, ta, tb)
    big = x.shape[:-2] if x.ndim >= w.ndim else w.shape[:-2]
    out_shape = tuple(big) + (m, n)
    bias = np.asarray(bias)
    if bias.ndim == 1:
        bias = bias.reshape(1, -1)
    c = np.ascontiguousarray(np.broadcast_to(bias, out_shape)).copy()
    return matmult(x, w, c, ta, tb, dt, kind)


def matmult_backward(a, b, grad, ta=False, tb=False, dt=None, kind="closed"):
    """dA, dB of C = op(a).op(b) using only transpose flags (nn/functional/matmult.cpp:37-62)."""
    if ta:
        da = matmult(b, grad, None, tb, True, dt, kind)
    else:
        da = matmult(grad, b, None, False, not tb, dt, kind)
    if tb:
        db = matmult(grad, a, None, True, ta, dt, kind)
    else:
        db = matmult(a, grad, None, not ta, False, dt, kind)
    return da, db


def _sum_to(arr, shape):
    """grad += in_grad with broadcasting reduced back by sum_as (operators.cpp:175-187)."""
    arr = np.asarray(arr)
    while arr.ndim > len(shape):
        arr = arr.sum(axis=0)
    for ax, s in enumerate(shape):
        if s == 1 and arr.shape[ax] != 1:
            arr = arr.sum(axis=ax, keepdims=True)
    return arr


def linear_backward(x, w, bias_shape, grad, ta=False, tb=False, dt=None, kind="closed"):
    """dX, dW, db of linear (nn/functional/matmult.cpp:253-275); batch dims of dW/db are
    reduced by accumulate_gradient's broadcasting += (AutoGrad.cpp:7-25)."""
    dx, dw = matmult_backward(x, w, grad, ta, tb, dt, kind)
    dx = _sum_to(dx, x.shape)
    dw = _sum_to(dw, w.shape)
    db = _sum_to(grad, tuple(bias_shape)) if len(bias_shape) == grad.ndim else \
        grad.reshape(-1, grad.shape[-1]).sum(axis=0).reshape(bias_shape)
    return dx, dw, db


def _batch_ordered_sum(per_item):
    """sum(0) as the reference forms it (tensor_files/sum_exp_log.cpp:112-124): item 0, then += item 1, ... in the element
    type (float16 sums round after every addition)."""
    acc = per_item[0].copy()
    for b in range(1, per_item.shape[0]):
        acc = acc + per_item[b]
    return acc


def complex_lanes(fn, dt, *arrays, **kw):
    """A convolution of the complex dtypes, restated plane by plane.  The reference's complex matmult works lane-wise on
    interleaved (re, im) pairs -- one real product of the real parts, one of the imaginary parts, see matmult2d_complex --
    and unfold / its adjoint / element-wise sums move or add whole elements lane by lane, so the whole unfold -> matmult
    pipeline on complex tensors is the same pipeline on the plane of real parts and on the plane of imaginary parts, each in
    the lane's real type: float32 chains for Complex64, float64 for Complex128, and for Complex32 half values with float
    chains rounded to half every 8 k (the complex_32 tile, not Float16's 16).  `arrays`: complex tensors as real arrays with
    a trailing axis of 2; fn(*planes, **kw) is one of this module's real convolution functions; its result (an array or a
    tuple of arrays) comes back with the lanes stacked on a new trailing axis."""
    real = _COMPLEX_REAL[dt]
    outs = []
    prev = _HALF_AS_COMPLEX32_LANE[0]
    _HALF_AS_COMPLEX32_LANE[0] = dt == C32
    try:
        for lane in (0, 1):
            planes = [np.ascontiguousarray(np.asarray(a, dtype=real)[..., lane]) for a in arrays]
            outs.append(fn(*planes, **kw))
    finally:
        _HALF_AS_COMPLEX32_LANE[0] = prev
    if isinstance(outs[0], tuple):
        return tuple(np.stack([outs[0][i], outs[1][i]], axis=-1) for i in range(len(outs[0])))
    return np.stack(outs, axis=-1)


def out_hw(h, w, k, s, p, d):
    return ((h + 2 * p[0] - d[0] * (k[0] - 1) - 1) // s[0] + 1,
            (w + 2 * p[1] - d[1] * (k[1] - 1) - 1) // s[1] + 1)


def _pair(v):
    return (v, v) if np.isscalar(v) else tuple(v)


def unfold2d(x, kernel_size, dilation=1, padding=0, stride=1, transpose_out=True):
    """[B,C,H,W] -> col [B, C*kh*kw, Ho*Wo] (transpose_out=True, the layout conv2d uses)."""
    x = np.ascontiguousarray(x)
    k, d, p, s = _pair(kernel_size), _pair(dilation), _pair(padding), _pair(stride)
    x4 = x.reshape((-1,) + x.shape[-3:]) if x.ndim != 3 else x.reshape((1,) + x.shape)
    B, C, H, W = x4.shape
    Ho, Wo = out_hw(H, W, k, s, p, d)
    if Ho * Wo <= 0:
        raise ValueError("sliding blocks must be at least one")
    col = np.zeros((B, C * k[0] * k[1], Ho * Wo), dtype=x.dtype)
    rc = lib().oracle_unfold2d(x.dtype.itemsize, _ptr(x4), _ptr(col), B, C, H, W,
                               k[0], k[1], s[0], s[1], p[0], p[1], d[0], d[1])
    if rc:
        raise RuntimeError("oracle unfold2d failed")
    return col if transpose_out else np.ascontiguousarray(col.transpose(0, 2, 1))


def unfold2d_backward(col, output_size, kernel_size, dilation=1, padding=0, stride=1, channels=None):
    col = np.ascontiguousarray(col)
    k, d, p, s = _pair(kernel_size), _pair(dilation), _pair(padding), _pair(stride)
    B = col.shape[0]
    C = col.shape[1] // (k[0] * k[1]) if channels is None else channels
    H, W = output_size
    if col.dtype not in (np.float32, np.float64):
        # the same scatter-add, taps in ascending order, in the element type (float16 sums round after every addition)
        return unfoldnd_backward(col.reshape(B, -1, col.shape[-1]), (H, W), k, d, p, s)
    im = np.zeros((B, C, H, W), dtype=col.dtype)
    rc = lib().oracle_unfold2d_backward(_NP_TO_DT[col.dtype], _ptr(col), _ptr(im), B, C, H, W,
                                        k[0], k[1], s[0], s[1], p[0], p[1], d[0], d[1])
    if rc:
        raise RuntimeError("oracle unfold2d_backward failed")
    return im


def conv2d(image, kernel, stride=1, padding=0, dilation=1, groups=1, kind="closed"):
    """unfold2d(transpose_out) -> matmult(col, W2d, true, true) -> RowColSwap -> [B,O,Ho,Wo]
    (conv.cpp:69-96); groups>1 splits channels/filters per group (conv.cpp:97-118)."""
    image = np.ascontiguousarray(image)
    kernel = np.ascontiguousarray(kernel)
    s, p, d = _pair(stride), _pair(padding), _pair(dilation)
    x = image.reshape((1,) + image.shape) if image.ndim == 3 else image.reshape((-1,) + image.shape[-3:])
    w = kernel.reshape((1,) + kernel.shape) if kernel.ndim == 3 else kernel
    B, C, H, W = x.shape
    O, Cg, kh, kw = w.shape
    Ho, Wo = out_hw(H, W, (kh, kw), s, p, d)
    col = unfold2d(x, (kh, kw), d, p, s, True)                     # [B, C*kh*kw, L]
    if groups == 1:
        out = matmult(col, w.reshape(O, -1), None, True, True, kind=kind)   # [B, L, O]
        return np.ascontiguousarray(out.transpose(0, 2, 1)).reshape(B, O, Ho, Wo)
    assert C % groups == 0 and Cg * groups == C and O % groups == 0
    add = (C // groups) * kh * kw
    og = O // groups
    out = np.zeros((B, O, Ho * Wo), dtype=image.dtype)
    for g in range(groups):
        colg = np.ascontiguousarray(col[:, g * add:(g + 1) * add, :])
        wg = np.ascontiguousarray(w[g * og:(g + 1) * og].reshape(og, -1))
        o = matmult(colg, wg, None, True, True, kind=kind)          # [B, L, og]
        out[:, g * og:(g + 1) * og, :] = o.transpose(0, 2, 1)
    return out.reshape(B, O, Ho, Wo)


def conv2d_backward(image, kernel, grad, stride=1, padding=0, dilation=1, groups=1, kind="closed"):
    """d_image: d_col = matmult(W2d, dY, true, false) then col2im (conv.cpp:318-346);
    d_kernel = sum_b matmult(dY_b, col_b, false, true) (conv.cpp:444-471)."""
    image = np.ascontiguousarray(image)
    kernel = np.ascontiguousarray(kernel)
    s, p, d = _pair(stride), _pair(padding), _pair(dilation)
    B, C, H, W = image.shape
    O, Cg, kh, kw = kernel.shape
    Ho, Wo = out_hw(H, W, (kh, kw), s, p, d)
    g3 = np.ascontiguousarray(grad).reshape(B, O, Ho * Wo)
    col = unfold2d(image, (kh, kw), d, p, s, True)
    add = (C // groups) * kh * kw
    og = O // groups
    dcol = np.zeros_like(col)
    dk = np.zeros((O, Cg * kh * kw), dtype=image.dtype)
    for g in range(groups):
        wg = np.ascontiguousarray(kernel[g * og:(g + 1) * og].reshape(og, -1))
        gg = np.ascontiguousarray(g3[:, g * og:(g + 1) * og, :])
        dcol[:, g * add:(g + 1) * add, :] = matmult(wg, gg, None, True, False, kind=kind)
        colg = np.ascontiguousarray(col[:, g * add:(g + 1) * add, :])
        per_item = matmult(gg, colg, None, False, True, kind=kind)   # [B, og, add]
        dk[g * og:(g + 1) * og] = _batch_ordered_sum(per_item)
    dimg = unfold2d_backward(dcol, (H, W), (kh, kw), d, p, s, channels=C)
    return dimg, dk.reshape(kernel.shape)


def conv1d(image, kernel, stride=1, padding=0, dilation=1, groups=1, kind="closed"):
    """functional::conv1d (conv.cpp:13-67): unfold1d (window index c*k + j, the one-row case of the
    2-d unfold) then the same matmult / group split as conv2d."""
    x = image.reshape((1,) + image.shape) if image.ndim == 2 else image.reshape((-1,) + image.shape[-2:])
    w = kernel.reshape((1,) + kernel.shape) if kernel.ndim == 2 else kernel
    out = conv2d(x[:, :, None, :], w[:, :, None, :], (1, stride), (0, padding), (1, dilation), groups, kind)
    return out[:, :, 0, :]


def conv1d_backward(image, kernel, grad, stride=1, padding=0, dilation=1, groups=1, kind="closed"):
    x = image.reshape((1,) + image.shape) if image.ndim == 2 else image.reshape((-1,) + image.shape[-2:])
    w = kernel.reshape((1,) + kernel.shape) if kernel.ndim == 2 else kernel
    g = np.ascontiguousarray(grad).reshape(x.shape[0], w.shape[0], 1, -1)
    dx, dw = conv2d_backward(np.ascontiguousarray(x[:, :, None, :]), np.ascontiguousarray(w[:, :, None, :]), g,
                             (1, stride), (0, padding), (1, dilation), groups, kind)
    return dx[:, :, 0, :].reshape(image.shape), dw[:, :, 0, :].reshape(kernel.shape)


def conv_transpose2d(image, kernel, stride=1, padding=0, output_padding=0, dilation=1, groups=1, kind="closed"):
    """functional::conv_transpose2d (conv.cpp:614-676): zero-dilate the input by the stride (:632-634), pad bottom/right
    by output_padding (:635-637), unfold2d with padding d*(k-1) - p and stride 1 (:639-641), then per group
    matmult(w.transpose(0,1).flip(-1,-2) viewed [Cout/g, Cin/g*kh*kw], col) (:645-675)."""
    x = image.reshape((1,) + image.shape) if image.ndim == 3 else image.reshape((-1,) + image.shape[-3:])
    w = kernel.reshape((1,) + kernel.shape) if kernel.ndim == 3 else kernel
    s, p, op, d = _pair(stride), _pair(padding), _pair(output_padding), _pair(dilation)
    B, Cin, H, W = x.shape
    _, Cog, kh, kw = w.shape
    assert w.shape[0] == Cin and Cin % groups == 0
    xd = np.zeros((B, Cin, (H - 1) * s[0] + 1 + op[0], (W - 1) * s[1] + 1 + op[1]), dtype=x.dtype)
    xd[:, :, 0:(H - 1) * s[0] + 1:s[0], 0:(W - 1) * s[1] + 1:s[1]] = x
    ph, pw = (kh - 1) * d[0] - p[0], (kw - 1) * d[1] - p[1]
    assert ph >= 0 and pw >= 0, "padding wider than the kernel reach is not representable by unfold2d"
    col = unfold2d(xd, (kh, kw), d, (ph, pw), 1, True)                               # [B, Cin*kh*kw, R*C]
    R = (H - 1) * s[0] - 2 * p[0] + d[0] * (kh - 1) + 1 + op[0]
    Cc = (W - 1) * s[1] - 2 * p[1] + d[1] * (kw - 1) + 1 + op[1]
    wt = np.ascontiguousarray(w.transpose(1, 0, 2, 3)[:, :, ::-1, ::-1])              # [Cout/g, Cin, kh, kw]
    cig = Cin // groups
    add = cig * kh * kw
    out = np.zeros((B, Cog * groups, R * Cc), dtype=x.dtype)
    for g in range(groups):
        kg = np.ascontiguousarray(wt[:, g * cig:(g + 1) * cig].reshape(Cog, -1))
        colg = np.ascontiguousarray(col[:, g * add:(g + 1) * add, :])
        out[:, g * Cog:(g + 1) * Cog, :] = matmult(kg, colg, None, False, False, kind=kind)
    return out.reshape(B, Cog * groups, R, Cc)


def conv_transpose2d_backward(image, kernel, grad, stride=1, padding=0, output_padding=0, dilation=1, groups=1, kind="closed"):
    """The transposed convolution is the adjoint of conv2d with the same kernel, so its image gradient is conv2d(grad, kernel)
    and its kernel gradient is conv_dkernel with image and output gradient exchanged.  (The reference reaches the same sums
    through the saved unfolded input and flipped kernel; pinned by the conv_transpose*_{xgrad,wgrad} fixtures.)"""
    x = image.reshape((1,) + image.shape) if image.ndim == 3 else image.reshape((-1,) + image.shape[-3:])
    w = kernel.reshape((1,) + kernel.shape) if kernel.ndim == 3 else kernel
    g = np.ascontiguousarray(grad).reshape((x.shape[0], w.shape[1] * groups) + grad.shape[-2:])
    dx = conv2d(g, w, stride, padding, dilation, groups, kind)
    _, dw = conv2d_backward(g, w, np.ascontiguousarray(x), stride, padding, dilation, groups, kind)
    return dx.reshape(image.shape), dw.reshape(kernel.shape)


def conv_transpose1d(image, kernel, stride=1, padding=0, output_padding=0, dilation=1, groups=1, kind="closed"):
    """functional::conv_transpose1d (conv.cpp:538-612), the one-row case of conv_transpose2d."""
    x = image.reshape((1,) + image.shape) if image.ndim == 2 else image.reshape((-1,) + image.shape[-2:])
    w = kernel.reshape((1,) + kernel.shape) if kernel.ndim == 2 else kernel
    out = conv_transpose2d(x[:, :, None, :], w[:, :, None, :], (1, stride), (0, padding), (0, output_padding), (1, dilation), groups, kind)
    return out[:, :, 0, :]


def conv_transpose1d_backward(image, kernel, grad, stride=1, padding=0, output_padding=0, dilation=1, groups=1, kind="closed"):
    x = image.reshape((1,) + image.shape) if image.ndim == 2 else image.reshape((-1,) + image.shape[-2:])
    w = kernel.reshape((1,) + kernel.shape) if kernel.ndim == 2 else kernel
    dx, dw = conv_transpose2d_backward(np.ascontiguousarray(x[:, :, None, :]), np.ascontiguousarray(w[:, :, None, :]),
                                       np.ascontiguousarray(grad)[..., None, :], (1, stride), (0, padding), (0, output_padding),
                                       (1, dilation), groups, kind)
    return dx[:, :, 0, :].reshape(image.shape), dw[:, :, 0, :].reshape(kernel.shape)


# ---- convolutions over N spatial axes (conv3d conv.cpp:122-175, convnd :177-316, conv_transpose3d :678-745) ----
def _ntuple(v, n):
    return tuple(int(x) for x in v) if isinstance(v, (tuple, list)) else (int(v),) * n


def unfoldnd(x, kernel_size, dilation=1, padding=0, stride=1):
    """functional::unfold3d / unfoldnd with transpose_out=true: x [B, C, *size] -> col [B, C*prod(k), prod(out)];
    row index ((c*k0 + t0)*k1 + t1)..., column index (o0*out1 + o1)... (nt/functional/cpu/unfold3d.cpp:9-80).
    Pure data movement, written with numpy slicing (one strided copy per tap)."""
    x = np.ascontiguousarray(x)
    nd = x.ndim - 2
    k, d, p, s = _ntuple(kernel_size, nd), _ntuple(dilation, nd), _ntuple(padding, nd), _ntuple(stride, nd)
    B, C = x.shape[:2]
    size = x.shape[2:]
    out = tuple((size[a] + 2 * p[a] - d[a] * (k[a] - 1) - 1) // s[a] + 1 for a in range(nd))
    if min(out) <= 0:
        raise ValueError("the array of sliding blocks would be empty")
    xp = np.zeros((B, C) + tuple(size[a] + 2 * p[a] for a in range(nd)), dtype=x.dtype)
    xp[(slice(None), slice(None)) + tuple(slice(p[a], p[a] + size[a]) for a in range(nd))] = x
    col = np.zeros((B, C) + k + out, dtype=x.dtype)
    for tap in np.ndindex(*k):
        src = tuple(slice(tap[a] * d[a], tap[a] * d[a] + (out[a] - 1) * s[a] + 1, s[a]) for a in range(nd))
        col[(slice(None), slice(None)) + tap] = xp[(slice(None), slice(None)) + src]
    return col.reshape(B, C * int(np.prod(k)), int(np.prod(out))), out


def unfoldnd_backward(col, size, kernel_size, dilation=1, padding=0, stride=1):
    """The adjoint of unfoldnd (unfold3d_backward.cpp / unfoldnd_backward.cpp): taps are added in ascending order."""
    nd = len(size)
    k, d, p, s = _ntuple(kernel_size, nd), _ntuple(dilation, nd), _ntuple(padding, nd), _ntuple(stride, nd)
    out = tuple((size[a] + 2 * p[a] - d[a] * (k[a] - 1) - 1) // s[a] + 1 for a in range(nd))
    B = col.shape[0]
    C = col.shape[1] // int(np.prod(k))
    c6 = col.reshape((B, C) + k + out)
    xp = np.zeros((B, C) + tuple(size[a] + 2 * p[a] for a in range(nd)), dtype=col.dtype)
    for tap in np.ndindex(*k):
        dst = tuple(slice(tap[a] * d[a], tap[a] * d[a] + (out[a] - 1) * s[a] + 1, s[a]) for a in range(nd))
        xp[(slice(None), slice(None)) + dst] += c6[(slice(None), slice(None)) + tap]
    return np.ascontiguousarray(xp[(slice(None), slice(None)) + tuple(slice(p[a], p[a] + size[a]) for a in range(nd))])


def convnd(image, kernel, stride=1, padding=0, dilation=1, groups=1, kind="closed"):
    """conv3d / convnd: unfold, then per group matmult(col_g, W_g, true, true) transposed back (conv.cpp:134-174)."""
    x = np.ascontiguousarray(image)
    w = np.ascontiguousarray(kernel)
    nd = w.ndim - 2
    B, C = x.shape[:2]
    O = w.shape[0]
    col, out = unfoldnd(x, w.shape[2:], dilation, padding, stride)
    add = (C // groups) * int(np.prod(w.shape[2:]))
    og = O // groups
    res = np.zeros((B, O, col.shape[2]), dtype=x.dtype)
    for g in range(groups):
        colg = np.ascontiguousarray(col[:, g * add:(g + 1) * add, :])
        wg = np.ascontiguousarray(w[g * og:(g + 1) * og].reshape(og, -1))
        res[:, g * og:(g + 1) * og, :] = matmult(colg, wg, None, True, True, kind=kind).transpose(0, 2, 1)
    return res.reshape((B, O) + out)


def convnd_backward(image, kernel, grad, stride=1, padding=0, dilation=1, groups=1, kind="closed"):
    """conv_dimage / conv_dkernel for any number of axes (conv.cpp:318-535): d_col = W_g^T . dY then the unfold adjoint;
    d_kernel = sum over the batch of dY_b . col_b^T."""
    x = np.ascontiguousarray(image)
    w = np.ascontiguousarray(kernel)
    B, C = x.shape[:2]
    O = w.shape[0]
    col, out = unfoldnd(x, w.shape[2:], dilation, padding, stride)
    g3 = np.ascontiguousarray(grad).reshape(B, O, -1)
    add = (C // groups) * int(np.prod(w.shape[2:]))
    og = O // groups
    dcol = np.zeros_like(col)
    dk = np.zeros((O, add), dtype=x.dtype)
    for g in range(groups):
        wg = np.ascontiguousarray(w[g * og:(g + 1) * og].reshape(og, -1))
        gg = np.ascontiguousarray(g3[:, g * og:(g + 1) * og, :])
        dcol[:, g * add:(g + 1) * add, :] = matmult(wg, gg, None, True, False, kind=kind)
        colg = np.ascontiguousarray(col[:, g * add:(g + 1) * add, :])
        dk[g * og:(g + 1) * og] = _batch_ordered_sum(matmult(gg, colg, None, False, True, kind=kind))
    dimg = unfoldnd_backward(dcol, x.shape[2:], w.shape[2:], dilation, padding, stride)
    return dimg, dk.reshape(w.shape)


def conv_transposend(image, kernel, stride=1, padding=0, output_padding=0, dilation=1, groups=1, kind="closed"):
    """conv_transpose3d / conv_transposend (conv.cpp:678-905): zero-dilate by the stride, pad the far side by output_padding,
    unfold with padding d*(k-1) - p and stride 1, matmult with the channel-swapped, tap-reversed kernel per group."""
    x = np.ascontiguousarray(image)
    w = np.ascontiguousarray(kernel)
    nd = w.ndim - 2
    s, p, op, d = _ntuple(stride, nd), _ntuple(padding, nd), _ntuple(output_padding, nd), _ntuple(dilation, nd)
    B, Cin = x.shape[:2]
    size = x.shape[2:]
    k = w.shape[2:]
    Cog = w.shape[1]
    xd = np.zeros((B, Cin) + tuple((size[a] - 1) * s[a] + 1 + op[a] for a in range(nd)), dtype=x.dtype)
    xd[(slice(None), slice(None)) + tuple(slice(0, (size[a] - 1) * s[a] + 1, s[a]) for a in range(nd))] = x
    pad = tuple((k[a] - 1) * d[a] - p[a] for a in range(nd))
    assert min(pad) >= 0
    col, out = unfoldnd(xd, k, d, pad, 1)
    flip = (slice(None), slice(None)) + (slice(None, None, -1),) * nd
    wt = np.ascontiguousarray(np.swapaxes(w, 0, 1)[flip])                      # [Cout/g, Cin, *k]
    cig = Cin // groups
    add = cig * int(np.prod(k))
    res = np.zeros((B, Cog * groups, col.shape[2]), dtype=x.dtype)
    for g in range(groups):
        kg = np.ascontiguousarray(wt[:, g * cig:(g + 1) * cig].reshape(Cog, -1))
        colg = np.ascontiguousarray(col[:, g * add:(g + 1) * add, :])
        res[:, g * Cog:(g + 1) * Cog, :] = matmult(kg, colg, None, False, False, kind=kind)
    return res.reshape((B, Cog * groups) + out)


def conv_transposend_backward(image, kernel, grad, stride=1, padding=0, output_padding=0, dilation=1, groups=1, kind="closed"):
    """Adjoint relations as for conv_transpose2d_backward."""
    x = np.ascontiguousarray(image)
    w = np.ascontiguousarray(kernel)
    g = np.ascontiguousarray(grad)
    dx = convnd(g, w, stride, padding, dilation, groups, kind)
    _, dw = convnd_backward(g, w, x, stride, padding, dilation, groups, kind)
    return dx.reshape(x.shape), dw
