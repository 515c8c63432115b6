"""nt::functional::{matmult, linear, matmult_cT, unfold2d, conv2d} on torch tensors in HBM.

A Python restatement of the reference's Tensor-level dispatcher
(nt/functional/cpu/matmult_cpu.cpp) whose every arithmetic step is an entry point of
libntgemm.so; torch only owns the device memory and the stream.  Shape rules and error
conditions follow the reference (lines cited at each check); errors surface as
ValueError where the reference throws from utils::throw_exception.
"""
import ctypes

import torch

from . import _lib
from ._lib import GemmDesc, check, load

_TORCH_TO_NTG = {
    torch.float16: _lib.FLOAT16, torch.bfloat16: _lib.BFLOAT16,
    torch.float32: _lib.FLOAT32, torch.float64: _lib.FLOAT64,
    torch.int8: _lib.INT8, torch.int16: _lib.INT16, torch.int32: _lib.INT32, torch.int64: _lib.INT64,
    torch.uint8: _lib.UINT8,
}


def ntg_dtype(t):
    try:
        return _TORCH_TO_NTG[t.dtype]
    except KeyError:
        raise ValueError(f"dtype {t.dtype} has no matmult on this backend")


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _require_device(*ts):
    for t in ts:
        if not t.is_cuda:
            raise ValueError("neurotensor_amd.functional works on tensors in device memory (cuda)")


def _as_matrix_view(t, trans):
    """(storage tensor, transpose flag): a contiguous tensor is used as is; a view whose last
    two dims are a transposed contiguous matrix flips the flag instead of copying
    (was_transposed_back, matmult_cpu.cpp:204-250, 268-274); anything else is cloned
    (matmult_cpu.cpp:277-279, 471-473)."""
    if t.is_contiguous():
        return t, trans
    tt = t.transpose(-1, -2)
    if tt.is_contiguous():
        return tt, not trans
    return t.contiguous(), trans


def _logical(a_shape, b_shape, ta, tb):
    m, k = (a_shape[-1], a_shape[-2]) if ta else (a_shape[-2], a_shape[-1])
    kb, n = (b_shape[-1], b_shape[-2]) if tb else (b_shape[-2], b_shape[-1])
    if k != kb:
        # determine_transposes, matmult_cpu.cpp:73-90
        raise ValueError(f"Expected dimensions -2 and -1 of shapes ({tuple(a_shape)},{tuple(b_shape)}) "
                         "to be equal for matrix multiplication")
    return m, k, n


def _launch(a, b, c, m, k, n, ta, tb, batches, sa, sb, sc, c_mode, bias=None, bias_strides=(0, 0, 0),
            a_off=0, b_off=0, c_off=0, bias_off=0, relu=False):
    es = a.element_size()
    d = GemmDesc()
    d.dtype = ntg_dtype(a)
    d.transpose_a, d.transpose_b, d.c_mode = int(ta), int(tb), c_mode
    d.m, d.k, d.n = m, k, n
    d.batches = batches
    d.stride_a, d.stride_b, d.stride_c = sa, sb, sc
    if bias is not None:
        d.bias = bias.data_ptr() + bias_off * es
        d.bias_batch_stride, d.bias_row_stride, d.bias_col_stride = bias_strides
    L = load()
    ws_bytes = L.ntg_gemm_workspace_bytes(ctypes.byref(d))      # > 0: few output tiles, deep k -> split along k
    ws = None
    if ws_bytes > 0:
        ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=a.device)
        d.workspace, d.workspace_bytes = ws.data_ptr(), ws_bytes
    entry = L.ntg_gemm_relu_dev if relu else L.ntg_gemm_dev
    check(entry(ctypes.byref(d), a.data_ptr() + a_off * es, b.data_ptr() + b_off * es, c.data_ptr() + c_off * es, _stream()))


def matmult(a, b, out=None, transpose_a=False, transpose_b=False, accumulate=None):
    """functional::matmult (tensor_files/matmult.cpp:14-25 -> cpu::matmult, matmult_cpu.cpp:1616-1622).

    Without `out`: returns op(a).op(b) (the reference allocates zeros and accumulates,
    matmult_cpu.cpp:110, :707; here the kernel overwrites, which is the same result).
    With `out`: out += op(a).op(b) -- the accumulate contract (matmult_cpu.cpp:123-153)."""
    _require_device(a, b)
    if a.dim() < 2 or b.dim() < 2:
        raise ValueError(f"Expected tensors to have dims greater than 1, but instead had dims of {a.dim()} and {b.dim()}")
    if a.dtype != b.dtype:
        raise ValueError(f"Expected both tensors to have the same dtype but got {a.dtype} and {b.dtype}")   # :868
    a_st, ta = _as_matrix_view(a, bool(transpose_a))
    b_st, tb = _as_matrix_view(b, bool(transpose_b))
    m, k, n = _logical(a_st.shape, b_st.shape, ta, tb)
    abatch, bbatch = tuple(a_st.shape[:-2]), tuple(b_st.shape[:-2])
    big, small = (abatch, bbatch) if len(abatch) >= len(bbatch) else (bbatch, abatch)
    if len(small) and big[len(big) - len(small):] != small:
        # matmult_cpu.cpp:870-872, 919-921, 970-973
        raise ValueError(f"Cannot multiply tensors of shapes {tuple(a.shape)} and {tuple(b.shape)}, outter dimensions do not match")
    out_shape = big + (m, n)
    nbig = 1
    for s in big:
        nbig *= s
    nsmall = 1
    for s in small:
        nsmall *= s
    if out is None:
        c = torch.empty(out_shape, dtype=a.dtype, device=a.device)
        c_mode = _lib.C_OVERWRITE
    else:
        _require_device(out)
        # matmult_cpu.cpp:137-143, 807-816
        if out.dtype != a.dtype:
            raise ValueError(f"Expected dtype {a.dtype} for output matrix multiplication, C dtype inputted was {out.dtype}")
        if not out.is_contiguous():
            raise ValueError("Expected output tensor for matrix multiplication to be contiguous")
        if tuple(out.shape) != out_shape and not (out.numel() == nbig * m * n and tuple(out.shape[-2:]) == (m, n)):
            raise ValueError(f"Got invalid shape for output tensor {tuple(out.shape)} expected {out_shape}")
        if len(bbatch) > len(abatch) and (ta or tb):
            # handle_dim_k_n_matmult_std out-variant, matmult_cpu.cpp:952
            raise ValueError("Transposing a and b are not currently supported for tensors of tensors")
        c = out
        c_mode = _lib.C_ACCUMULATE if accumulate in (None, True) else _lib.C_OVERWRITE
    if nbig == 0 or m == 0 or n == 0:
        return c
    a_items = nbig if abatch == big else nsmall
    b_items = nbig if bbatch == big else nsmall
    amat, bmat, cmat = m * k, k * n, m * n
    if a_items == nbig and b_items == nbig:
        _launch(a_st, b_st, c, m, k, n, ta, tb, nbig, amat, bmat, cmat, c_mode)
    elif nsmall == 1:
        # the lower-rank operand is one matrix: stride 0 broadcasts it (repeat_ of the handle, :883)
        sa = amat if a_items == nbig else 0
        sb = bmat if b_items == nbig else 0
        _launch(a_st, b_st, c, m, k, n, ta, tb, nbig, sa, sb, cmat, c_mode)
    else:
        # item i of the big operand pairs with item i mod nsmall of the small one
        outer = nbig // nsmall
        for o in range(outer):
            a_off = o * nsmall * amat if a_items == nbig else 0
            b_off = o * nsmall * bmat if b_items == nbig else 0
            _launch(a_st, b_st, c, m, k, n, ta, tb, nsmall, amat, bmat, cmat, c_mode,
                    a_off=a_off, b_off=b_off, c_off=o * nsmall * cmat)
    return c


def matmult_cT(a, b):
    """matmult(a, b, false, true) (tensor_files/matmult.cpp:38)."""
    return matmult(a, b, None, False, True)


def linear_relu(x, w, bias, transpose_a=False, transpose_b=False):
    """relu_(linear(x, w, bias)) in one launch (activation_functions.cpp:141-143: relu = clamp(x, 0)); the clamp runs in
    the product's epilogue and gives the bits of the two calls in a row."""
    return linear(x, w, bias, transpose_a, transpose_b, _relu=True)


def relu_(x):
    """relu_ on a contiguous floating tensor in HBM: the product entry point with an empty k (C = max(C, 0))."""
    _require_device(x)
    if not x.is_contiguous():
        raise ValueError("relu_ expects a contiguous tensor")
    if x.numel():
        cols = x.shape[-1] if x.dim() else 1
        _launch(x, x, x, x.numel() // cols, 0, cols, False, False, 1, 0, 0, 0, _lib.C_ACCUMULATE, relu=True)
    return x


def linear(x, w, bias, transpose_a=False, transpose_b=False, _relu=False):
    """functional::linear -> cpu::linear (matmult_cpu.cpp:1624-1714): the bias, broadcast to the
    output shape, is the initial accumulator of the GEMM.  Done here in one pass (C_BIAS)."""
    _require_device(x, w, bias)
    if not (x.dtype == w.dtype == bias.dtype):
        raise ValueError("linear expects input, weight and bias of one dtype")
    nd = max(x.dim(), w.dim(), bias.dim())
    if nd < 2:
        raise ValueError(f"Cannot perform matrix multiplication with dimensions less than 2 got {nd} for tensor dimensions")

    def unsq(t):      # unsqueeze_as, matmult_cpu.cpp:1712-1713
        return t.reshape((1,) * (nd - t.dim()) + tuple(t.shape))

    x, w, bias = unsq(x), unsq(w), unsq(bias)
    x_st, ta = _as_matrix_view(x, bool(transpose_a))
    w_st, tb = _as_matrix_view(w, bool(transpose_b))
    m, k, n = _logical(x_st.shape, w_st.shape, ta, tb)
    if bias.shape[-2] not in (1, m):
        raise ValueError(f"Got invalid shape for bias ({tuple(bias.shape)}) to linear function expected rows to be 1 or {m}")
    if bias.shape[-1] not in (1, n):
        raise ValueError(f"Got invalid shape for bias ({tuple(bias.shape)}) to linear function expected cols to be 1 or {n}")
    xb, wb, bb = tuple(x_st.shape[:-2]), tuple(w_st.shape[:-2]), tuple(bias.shape[:-2])

    def strip(s):
        s = list(s)
        while s and s[0] == 1:
            s.pop(0)
        return tuple(s)

    xs, ws, bs = strip(xb), strip(wb), strip(bb)
    big = xs if len(xs) >= len(ws) else ws
    for small in (xs, ws, bs):
        if len(small) and big[len(big) - len(small):] != small:
            raise ValueError(f"Error, invalid batch shapes for linear: ({tuple(x.shape)}, {tuple(w.shape)}, {tuple(bias.shape)})")
    nbig = 1
    for s in big:
        nbig *= s
    out = torch.empty(big + (m, n), dtype=x.dtype, device=x.device)
    if nbig == 0 or m == 0 or n == 0:
        return out
    bias_c = bias.contiguous()
    brs = 0 if bias.shape[-2] == 1 else bias.shape[-1]
    bcs = 0 if bias.shape[-1] == 1 else 1
    bmat = bias.shape[-2] * bias.shape[-1]

    def count(s):
        c = 1
        for v in s:
            c *= v
        return c

    nx, nw, nb = count(xs), count(ws), count(bs)
    if all(v in (1, nbig) for v in (nx, nw, nb)):
        _launch(x_st, w_st, out, m, k, n, ta, tb, nbig,
                m * k if nx == nbig else 0, k * n if nw == nbig else 0, m * n, _lib.C_BIAS,
                bias=bias_c, bias_strides=(bmat if nb == nbig else 0, brs, bcs), relu=_relu)
    else:
        # mixed ranks: item i uses item i mod count of each lower-rank operand
        for i in range(nbig):
            _launch(x_st, w_st, out, m, k, n, ta, tb, 1, 0, 0, 0, _lib.C_BIAS,
                    bias=bias_c, bias_strides=(0, brs, bcs),
                    a_off=(i % nx) * m * k, b_off=(i % nw) * k * n, c_off=i * m * n, bias_off=(i % nb) * bmat, relu=_relu)
    return out


def _pair(v):
    if isinstance(v, (tuple, list)):
        if len(v) != 2:
            raise ValueError("expected a pair")
        return int(v[0]), int(v[1])
    return int(v), int(v)


def unfold2d(x, kernel_size, dilation=1, padding=0, stride=1, transpose_out=True):
    """functional::unfold2d (tensor_files/colim_transform.cpp:565-588): [..,C,H,W] -> [B, C*kh*kw, L]."""
    _require_device(x)
    if x.dim() < 3:
        raise ValueError(f"Expected input tensot to unfold to have dims greater than or equal to 3 but got {x.dim()}D")
    k, d, p, s = _pair(kernel_size), _pair(dilation), _pair(padding), _pair(stride)
    im = x.reshape((1,) + tuple(x.shape)) if x.dim() == 3 else x.reshape((-1,) + tuple(x.shape[-3:]))
    im = im.contiguous()
    B, C, H, W = im.shape
    Ho = (H + 2 * p[0] - d[0] * (k[0] - 1) - 1) // s[0] + 1
    Wo = (W + 2 * p[1] - d[1] * (k[1] - 1) - 1) // s[1] + 1
    if Ho * Wo <= 0 or Ho <= 0:
        raise ValueError(f"calculated shape of the array of sliding blocks as ({Ho}, {Wo}), but its components must be at least one.")
    col = torch.empty((B, C * k[0] * k[1], Ho * Wo), dtype=x.dtype, device=x.device)
    check(load().ntg_unfold2d_dev(ntg_dtype(x), im.data_ptr(), col.data_ptr(), B, C, H, W,
                                  k[0], k[1], s[0], s[1], p[0], p[1], d[0], d[1], _stream()))
    return col if transpose_out else col.transpose(-1, -2)


def conv2d(image, kernel, stride=1, padding=0, dilation=1, groups=1):
    """functional::conv2d (tensor_files/conv.cpp:69-119): unfold2d then matmult; out [B,O,Ho,Wo]."""
    _require_device(image, kernel)
    if image.dim() < 3:
        raise ValueError(f"Expected to get a 3D or greater tensor as the input for a 2d convolution, but got {image.dim()}D")
    if kernel.dim() not in (3, 4):
        raise ValueError(f"Expected to get a 4D or 3D tensor as the kernel for a 2d convolution, but got {kernel.dim()}D")
    if image.dtype != kernel.dtype:
        raise ValueError(f"Expected both kernel and image to have the same dtype for conv2d but got {kernel.dtype} and {image.dtype}")
    s, p, d = _pair(stride), _pair(padding), _pair(dilation)
    if min(s) < 1:
        raise ValueError(f"Conv2d stride cannot be less than 1 but got {s}")
    if min(d) < 1:
        raise ValueError(f"Conv2d dilation cannot be less than 1 but got {d}")
    if min(p) < 0:
        raise ValueError(f"Conv2d padding cannot be less than 1 but got {p}")
    x = image.reshape((1,) + tuple(image.shape)) if image.dim() == 3 else image.reshape((-1,) + tuple(image.shape[-3:]))
    w = kernel.reshape((1,) + tuple(kernel.shape)) if kernel.dim() == 3 else kernel
    x, w = x.contiguous(), w.contiguous()
    B, C, H, W = x.shape
    O, Cg, kh, kw = w.shape
    if C % groups != 0:
        raise ValueError(f"Expected image channels to be divisible by groups in Conv2d but got {C} % {groups} != 0")
    if Cg * groups != C:
        raise ValueError(f"Expected kernel rows times groups to be equal to rows of image Conv2d but got {Cg} * {groups} != {C}")
    L = load()
    dt = ntg_dtype(x)
    ws_bytes = L.ntg_conv2d_fast_workspace_bytes(dt, B, C, H, W, O, kh, kw, s[0], s[1], p[0], p[1], d[0], d[1], groups)
    if ws_bytes < 0:
        raise ValueError("the array of sliding blocks would be empty")
    Ho = (H + 2 * p[0] - d[0] * (kh - 1) - 1) // s[0] + 1
    Wo = (W + 2 * p[1] - d[1] * (kw - 1) - 1) // s[1] + 1
    out = torch.empty((B, O, Ho, Wo), dtype=x.dtype, device=x.device)
    ws = torch.empty((max(ws_bytes, 1),), dtype=torch.uint8, device=x.device)
    check(L.ntg_conv2d_dev(dt, x.data_ptr(), w.data_ptr(), out.data_ptr(), ws.data_ptr(), ws_bytes,
                           B, C, H, W, O, kh, kw, s[0], s[1], p[0], p[1], d[0], d[1], groups, _stream()))
    return out


def unfold2d_backward(col, output_size, kernel_size, dilation=1, padding=0, stride=1):
    """functional::unfold2d_backward with transpose_out=true (colim_transform.cpp:592-653):
    col [B, C*kh*kw, L] -> image gradient [B, C, H, W]."""
    _require_device(col)
    k, d, p, s = _pair(kernel_size), _pair(dilation), _pair(padding), _pair(stride)
    H, W = _pair(output_size)
    if col.dim() not in (2, 3):
        raise ValueError(f"Expected to get a shape with a dimensionality of 3D or 2D, but got {col.dim()} dimensions")
    c3 = col.reshape((1,) + tuple(col.shape)) if col.dim() == 2 else col
    c3 = c3.contiguous()
    B = c3.shape[0]
    if c3.shape[1] % (k[0] * k[1]) != 0:
        raise ValueError("col rows are not a multiple of the kernel size")
    C = c3.shape[1] // (k[0] * k[1])
    Ho = (H + 2 * p[0] - d[0] * (k[0] - 1) - 1) // s[0] + 1
    Wo = (W + 2 * p[1] - d[1] * (k[1] - 1) - 1) // s[1] + 1
    if Ho * Wo != c3.shape[2]:
        raise ValueError(f"col has {c3.shape[2]} sliding blocks, the geometry gives {Ho * Wo}")
    im = torch.empty((B, C, H, W), dtype=col.dtype, device=col.device)
    check(load().ntg_unfold2d_backward_dev(ntg_dtype(col), c3.data_ptr(), im.data_ptr(), B, C, H, W,
                                           k[0], k[1], s[0], s[1], p[0], p[1], d[0], d[1], 0, _stream()))
    return im


def conv2d_backward(image, kernel, grad, stride=1, padding=0, dilation=1, groups=1):
    """conv_dimage + conv_dkernel for dim == 2 (conv.cpp:318-346, 444-471): returns (d_image, d_kernel)."""
    _require_device(image, kernel, grad)
    s, p, d = _pair(stride), _pair(padding), _pair(dilation)
    x = image.reshape((1,) + tuple(image.shape)) if image.dim() == 3 else image.reshape((-1,) + tuple(image.shape[-3:]))
    w = kernel.reshape((1,) + tuple(kernel.shape)) if kernel.dim() == 3 else kernel
    x, w, g = x.contiguous(), w.contiguous(), grad.contiguous()
    B, C, H, W = x.shape
    O, Cg, kh, kw = w.shape
    if C % groups != 0 or Cg * groups != C or O % groups != 0:
        raise ValueError(f"channels {C}, kernel channels {Cg} and filters {O} do not fit groups={groups}")
    L = load()
    dt = ntg_dtype(x)
    ws_bytes = L.ntg_conv2d_backward_workspace_bytes(dt, B, C, H, W, O, kh, kw, s[0], s[1], p[0], p[1], d[0], d[1], groups)
    if ws_bytes < 0:
        raise ValueError("the array of sliding blocks would be empty")
    Ho = (H + 2 * p[0] - d[0] * (kh - 1) - 1) // s[0] + 1
    Wo = (W + 2 * p[1] - d[1] * (kw - 1) - 1) // s[1] + 1
    if g.numel() != B * O * Ho * Wo:
        raise ValueError(f"grad has {g.numel()} elements, expected {(B, O, Ho, Wo)}")
    dx = torch.empty_like(x)
    dw = torch.empty_like(w)
    ws = torch.empty((max(ws_bytes, 1),), dtype=torch.uint8, device=x.device)
    check(L.ntg_conv2d_backward_dev(dt, x.data_ptr(), w.data_ptr(), g.data_ptr(), dx.data_ptr(), dw.data_ptr(), ws.data_ptr(), ws_bytes,
                                    B, C, H, W, O, kh, kw, s[0], s[1], p[0], p[1], d[0], d[1], groups, 0, _stream()))
    return dx.reshape(image.shape), dw.reshape(kernel.shape)


def conv1d(image, kernel, stride=1, padding=0, dilation=1, groups=1):
    """functional::conv1d (tensor_files/conv.cpp:13-67): unfold1d then matmult; image [.., C, W], kernel [O, C/groups, k]
    -> [B, O, Wo].  A convolution over one axis is the two-axis one with a single image row and a single tap row."""
    _require_device(image, kernel)
    if image.dim() < 2:
        raise ValueError(f"Expected to get a 2D or greater tensor as the input for a 1d convolution, but got {image.dim()}D")
    if kernel.dim() not in (2, 3):
        raise ValueError(f"Expected to get a 3D or 2D tensor as the kernel for a 1d convolution, but got {kernel.dim()}D")
    if stride < 1:
        raise ValueError(f"Conv1d stride cannot be less than 1 but got {stride}")
    if dilation < 1:
        raise ValueError(f"Conv1d dilation cannot be less than 1 but got {dilation}")
    if padding < 0:
        raise ValueError(f"Conv1d padding cannot be less than 1 but got {padding}")
    x = image.reshape((1,) + tuple(image.shape)) if image.dim() == 2 else image.reshape((-1,) + tuple(image.shape[-2:]))
    w = kernel.reshape((1,) + tuple(kernel.shape)) if kernel.dim() == 2 else kernel
    out = conv2d(x.unsqueeze(2), w.unsqueeze(2), (1, stride), (0, padding), (1, dilation), groups)
    return out.squeeze(2)


def conv1d_backward(image, kernel, grad, stride=1, padding=0, dilation=1, groups=1):
    """Gradients of conv1d with respect to image and kernel (conv_dimage / conv_dkernel with dim == 1)."""
    x = image.reshape((1,) + tuple(image.shape)) if image.dim() == 2 else image.reshape((-1,) + tuple(image.shape[-2:]))
    w = kernel.reshape((1,) + tuple(kernel.shape)) if kernel.dim() == 2 else kernel
    dx, dw = conv2d_backward(x.unsqueeze(2), w.unsqueeze(2), grad.reshape(x.shape[0], w.shape[0], 1, -1),
                             (1, stride), (0, padding), (1, dilation), groups)
    return dx.squeeze(2).reshape(image.shape), dw.squeeze(2).reshape(kernel.shape)


def conv_transpose2d(image, kernel, stride=1, padding=0, output_padding=0, dilation=1, groups=1):
    """functional::conv_transpose2d (tensor_files/conv.cpp:614-676): image [.., Cin, H, W], kernel [Cin, Cout/groups, kh, kw]
    -> [B, Cout, (H-1)*s - 2p + d(kh-1) + 1 + output_padding, ...]."""
    _require_device(image, kernel)
    if image.dim() < 3:
        raise ValueError(f"Expected to get a 3D or greater tensor as the input for a conv2d transpose, but got {image.dim()}D")
    if kernel.dim() not in (3, 4):
        raise ValueError(f"Expected to get a 4D or 3D tensor as the kernel for a conv2d transpose, but got {kernel.dim()}D")
    if image.dtype != kernel.dtype:
        raise ValueError(f"Expected both kernel and image to have the same dtype for conv2d transpose but got {kernel.dtype} and {image.dtype}")
    s, p, op, d = _pair(stride), _pair(padding), _pair(output_padding), _pair(dilation)
    if min(s) < 1:
        raise ValueError(f"Conv2d Transpose stride cannot be less than 1 but got {s}")
    if min(d) < 1:
        raise ValueError(f"Conv2d Transpose dilation cannot be less than 1 but got {d}")
    if min(op) < 0:
        raise ValueError(f"Conv2d Transpose output_padding cannot be less than 1 but got {op}")
    if min(p) < 0:
        raise ValueError(f"Conv2d Transpose padding cannot be less than 1 but got {p}")
    if groups < 1:
        raise ValueError(f"Expected groups for a convolution to be greater than 0 but got {groups}")
    x = image.reshape((1,) + tuple(image.shape)) if image.dim() == 3 else image.reshape((-1,) + tuple(image.shape[-3:]))
    w = kernel.reshape((1,) + tuple(kernel.shape)) if kernel.dim() == 3 else kernel
    x, w = x.contiguous(), w.contiguous()
    B, Cin, H, W = x.shape
    if w.shape[0] != Cin:
        raise ValueError(f"Expected image channels to be the same as the kernel batches for conv_transpose2d but got {tuple(x.shape)} and {tuple(w.shape)}")
    if Cin % groups != 0:
        raise ValueError(f"Expected image channels to be divisible by groups in Conv2d Transpose but got {Cin} % {groups} != 0")
    _, Cog, kh, kw = w.shape
    Cout = Cog * groups
    L = load()
    dt = ntg_dtype(x)
    args = (B, Cin, H, W, Cout, kh, kw, s[0], s[1], p[0], p[1], d[0], d[1], op[0], op[1], groups)
    ws_bytes = L.ntg_conv_transpose2d_workspace_bytes(dt, *args)
    if ws_bytes < 0:
        raise ValueError("conv_transpose2d: " + L.ntg_last_error().decode() if L.ntg_last_error() else "invalid geometry")
    R = (H - 1) * s[0] - 2 * p[0] + d[0] * (kh - 1) + 1 + op[0]
    Cc = (W - 1) * s[1] - 2 * p[1] + d[1] * (kw - 1) + 1 + op[1]
    out = torch.empty((B, Cout, R, Cc), dtype=x.dtype, device=x.device)
    ws = torch.empty((max(ws_bytes, 1),), dtype=torch.uint8, device=x.device)
    check(L.ntg_conv_transpose2d_dev(dt, x.data_ptr(), w.data_ptr(), out.data_ptr(), ws.data_ptr(), ws_bytes, *args, _stream()))
    return out


def conv_transpose2d_backward(image, kernel, grad, stride=1, padding=0, output_padding=0, dilation=1, groups=1):
    """Gradients of conv_transpose2d: d_image = conv2d(grad, kernel) and d_kernel = conv_dkernel with the roles of image
    and output gradient exchanged (the transposed convolution is the adjoint of that convolution)."""
    s, p, d = _pair(stride), _pair(padding), _pair(dilation)
    x = image.reshape((1,) + tuple(image.shape)) if image.dim() == 3 else image.reshape((-1,) + tuple(image.shape[-3:]))
    w = kernel.reshape((1,) + tuple(kernel.shape)) if kernel.dim() == 3 else kernel
    g = grad.reshape((x.shape[0], w.shape[1] * groups) + tuple(grad.shape[-2:])).contiguous()
    dx = conv2d(g, w, s, p, d, groups)
    _, dw = conv2d_backward(g, w, x.contiguous(), s, p, d, groups)
    return dx.reshape(image.shape), dw.reshape(kernel.shape)


def conv_transpose1d(image, kernel, stride=1, padding=0, output_padding=0, dilation=1, groups=1):
    """functional::conv_transpose1d (tensor_files/conv.cpp:538-612): image [.., Cin, W], kernel [Cin, Cout/groups, k]."""
    x = image.reshape((1,) + tuple(image.shape)) if image.dim() == 2 else image.reshape((-1,) + tuple(image.shape[-2:]))
    w = kernel.reshape((1,) + tuple(kernel.shape)) if kernel.dim() == 2 else kernel
    out = conv_transpose2d(x.unsqueeze(2), w.unsqueeze(2), (1, stride), (0, padding), (0, output_padding), (1, dilation), groups)
    return out.squeeze(2)


def conv_transpose1d_backward(image, kernel, grad, stride=1, padding=0, output_padding=0, dilation=1, groups=1):
    x = image.reshape((1,) + tuple(image.shape)) if image.dim() == 2 else image.reshape((-1,) + tuple(image.shape[-2:]))
    w = kernel.reshape((1,) + tuple(kernel.shape)) if kernel.dim() == 2 else kernel
    dx, dw = conv_transpose2d_backward(x.unsqueeze(2), w.unsqueeze(2), grad.unsqueeze(-2), (1, stride), (0, padding),
                                       (0, output_padding), (1, dilation), groups)
    return dx.squeeze(2).reshape(image.shape), dw.squeeze(2).reshape(kernel.shape)


# ---- convolutions over N spatial axes: conv3d / convnd / conv_transpose3d (tensor_files/conv.cpp:122-316, 678-905) ----
def _ntuple(v, n):
    return tuple(int(x) for x in v) if isinstance(v, (tuple, list)) else (int(v),) * n


def _i64arr(vals):
    return (ctypes.c_int64 * len(vals))(*vals)


def convnd(image, kernel, stride=1, padding=0, dilation=1, groups=1):
    """functional::conv3d / convnd: image [B, C, *size], kernel [O, C/groups, *k] with 1..4 spatial axes -> [B, O, *out]."""
    _require_device(image, kernel)
    nd = kernel.dim() - 2
    if nd < 1 or nd > 4:
        raise ValueError(f"Expected a kernel with 1 to 4 spatial dimensions but got {nd}")
    if image.dim() != nd + 2:
        raise ValueError(f"Expected to get a {nd + 2}D tensor as the input for a {nd}d convolution, but got {image.dim()}D")
    if image.dtype != kernel.dtype:
        raise ValueError(f"Expected both kernel and image to have the same dtype for conv{nd}d but got {kernel.dtype} and {image.dtype}")
    s, p, d = _ntuple(stride, nd), _ntuple(padding, nd), _ntuple(dilation, nd)
    if min(s) < 1:
        raise ValueError(f"Conv{nd}d stride cannot be less than 1 but got {s}")
    if min(d) < 1:
        raise ValueError(f"Conv{nd}d dilation cannot be less than 1 but got {d}")
    if min(p) < 0:
        raise ValueError(f"Conv{nd}d padding cannot be less than 1 but got {p}")
    x, w = image.contiguous(), kernel.contiguous()
    B, C = x.shape[:2]
    O, Cg = w.shape[:2]
    size, k = tuple(x.shape[2:]), tuple(w.shape[2:])
    if groups < 1 or C % groups != 0 or Cg * groups != C or O % groups != 0:
        raise ValueError(f"Expected kernel rows times groups to be equal to rows of image Conv{nd}d but got {Cg} * {groups} != {C}")
    out = tuple((size[a] + 2 * p[a] - d[a] * (k[a] - 1) - 1) // s[a] + 1 for a in range(nd))
    if min(out) <= 0:
        raise ValueError("the array of sliding blocks would be empty")
    L = load()
    dt = ntg_dtype(x)
    geo = (_i64arr(size), _i64arr(k), _i64arr(s), _i64arr(p), _i64arr(d))
    ws_bytes = L.ntg_convnd_workspace_bytes(dt, B, C, O, nd, *geo, groups, 0)
    if ws_bytes < 0:
        raise ValueError("invalid convolution geometry")
    y = torch.empty((B, O) + out, dtype=x.dtype, device=x.device)
    ws = torch.empty((max(ws_bytes, 1),), dtype=torch.uint8, device=x.device)
    check(L.ntg_convnd_dev(dt, x.data_ptr(), w.data_ptr(), y.data_ptr(), ws.data_ptr(), ws_bytes, B, C, O, nd, *geo, groups, _stream()))
    return y


def convnd_backward(image, kernel, grad, stride=1, padding=0, dilation=1, groups=1):
    """conv_dimage + conv_dkernel for 1..4 spatial axes (conv.cpp:318-535): returns (d_image, d_kernel)."""
    _require_device(image, kernel, grad)
    nd = kernel.dim() - 2
    s, p, d = _ntuple(stride, nd), _ntuple(padding, nd), _ntuple(dilation, nd)
    x, w, g = image.contiguous(), kernel.contiguous(), grad.contiguous()
    B, C = x.shape[:2]
    O = w.shape[0]
    size, k = tuple(x.shape[2:]), tuple(w.shape[2:])
    L = load()
    dt = ntg_dtype(x)
    geo = (_i64arr(size), _i64arr(k), _i64arr(s), _i64arr(p), _i64arr(d))
    ws_bytes = L.ntg_convnd_workspace_bytes(dt, B, C, O, nd, *geo, groups, 1)
    if ws_bytes < 0:
        raise ValueError("invalid convolution geometry")
    dx, dw = torch.empty_like(x), torch.empty_like(w)
    ws = torch.empty((max(ws_bytes, 1),), dtype=torch.uint8, device=x.device)
    check(L.ntg_convnd_backward_dev(dt, x.data_ptr(), w.data_ptr(), g.data_ptr(), dx.data_ptr(), dw.data_ptr(), ws.data_ptr(), ws_bytes,
                                    B, C, O, nd, *geo, groups, 0, _stream()))
    return dx, dw


def conv3d(image, kernel, stride=1, padding=0, dilation=1, groups=1):
    """functional::conv3d (conv.cpp:122-175): image [.., C, D, H, W], kernel [O, C/groups, kd, kh, kw]."""
    if image.dim() < 4:
        raise ValueError(f"Expected to get a 4D or greater tensor as the input for a 3d convolution, but got {image.dim()}D")
    if kernel.dim() not in (4, 5):
        raise ValueError(f"Expected to get a 5D or 4D tensor as the kernel for a 3d convolution, but got {kernel.dim()}D")
    x = image.reshape((1,) + tuple(image.shape)) if image.dim() == 4 else image.reshape((-1,) + tuple(image.shape[-4:]))
    w = kernel.reshape((1,) + tuple(kernel.shape)) if kernel.dim() == 4 else kernel
    return convnd(x, w, stride, padding, dilation, groups)


def conv3d_backward(image, kernel, grad, stride=1, padding=0, dilation=1, groups=1):
    x = image.reshape((1,) + tuple(image.shape)) if image.dim() == 4 else image.reshape((-1,) + tuple(image.shape[-4:]))
    w = kernel.reshape((1,) + tuple(kernel.shape)) if kernel.dim() == 4 else kernel
    dx, dw = convnd_backward(x, w, grad, stride, padding, dilation, groups)
    return dx.reshape(image.shape), dw.reshape(kernel.shape)


def conv_transposend(image, kernel, stride=1, padding=0, output_padding=0, dilation=1, groups=1):
    """functional::conv_transpose3d / conv_transposend (conv.cpp:678-905): image [B, Cin, *size], kernel [Cin, Cout/groups, *k]."""
    _require_device(image, kernel)
    nd = kernel.dim() - 2
    if image.dim() != nd + 2:
        raise ValueError(f"Expected to get a {nd + 2}D tensor as the input for a conv{nd}d transpose, but got {image.dim()}D")
    s, p, op, d = _ntuple(stride, nd), _ntuple(padding, nd), _ntuple(output_padding, nd), _ntuple(dilation, nd)
    x, w = image.contiguous(), kernel.contiguous()
    B, Cin = x.shape[:2]
    if w.shape[0] != Cin:
        raise ValueError(f"Expected image channels to be the same as the kernel batches for conv_transpose{nd}d but got {tuple(x.shape)} and {tuple(w.shape)}")
    if groups < 1 or Cin % groups != 0:
        raise ValueError(f"Expected image channels to be divisible by groups in Conv{nd}d Transpose but got {Cin} % {groups} != 0")
    Cout = w.shape[1] * groups
    size, k = tuple(x.shape[2:]), tuple(w.shape[2:])
    out = tuple((size[a] - 1) * s[a] - 2 * p[a] + d[a] * (k[a] - 1) + 1 + op[a] for a in range(nd))
    L = load()
    dt = ntg_dtype(x)
    geo = (_i64arr(size), _i64arr(k), _i64arr(s), _i64arr(p), _i64arr(d), _i64arr(op))
    ws_bytes = L.ntg_conv_transposend_workspace_bytes(dt, B, Cin, Cout, nd, *geo, groups)
    if ws_bytes < 0:
        raise ValueError("invalid transposed-convolution geometry: " + L.ntg_last_error().decode())
    y = torch.empty((B, Cout) + out, dtype=x.dtype, device=x.device)
    ws = torch.empty((max(ws_bytes, 1),), dtype=torch.uint8, device=x.device)
    check(L.ntg_conv_transposend_dev(dt, x.data_ptr(), w.data_ptr(), y.data_ptr(), ws.data_ptr(), ws_bytes, B, Cin, Cout, nd, *geo, groups,
                                     _stream()))
    return y


def conv_transposend_backward(image, kernel, grad, stride=1, padding=0, output_padding=0, dilation=1, groups=1):
    """Gradients of the transposed convolution through its adjoint: d_image = convnd(grad, kernel), d_kernel = conv_dkernel
    with image and output gradient exchanged."""
    g = grad.contiguous()
    dx = convnd(g, kernel, stride, padding, dilation, groups)
    _, dw = convnd_backward(g, kernel, image.contiguous(), stride, padding, dilation, groups)
    return dx.reshape(image.shape), dw


def conv_transpose3d(image, kernel, stride=1, padding=0, output_padding=0, dilation=1, groups=1):
    if image.dim() < 4:
        raise ValueError(f"Expected to get a 4D or greater tensor as the input for a conv3d transpose, but got {image.dim()}D")
    if kernel.dim() not in (4, 5):
        raise ValueError(f"Expected to get a 5D or 4D tensor as the kernel for a conv3d transpose, but got {kernel.dim()}D")
    x = image.reshape((1,) + tuple(image.shape)) if image.dim() == 4 else image.reshape((-1,) + tuple(image.shape[-4:]))
    w = kernel.reshape((1,) + tuple(kernel.shape)) if kernel.dim() == 4 else kernel
    return conv_transposend(x, w, stride, padding, output_padding, dilation, groups)
