"""CPU-side checks of the drop-in boundary: libntgemm.so loads, exports every symbol
include/ntgemm.h declares, and rejects bad arguments before touching a device."""
import ctypes
import os
import re

import numpy as np
import pytest

from neurotensor_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "ntgemm.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ntg_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_all_exported_and_bound():
    lib = _lib.load()
    names = declared_symbols()
    assert len(names) >= 14
    for n in names:
        assert hasattr(lib, n), f"{n} declared in ntgemm.h but not exported"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes signature"
    assert set(_lib.SIGNATURES) == set(names)


def test_dtype_sizes_follow_nt_dtype_values():
    lib = _lib.load()
    sizes = {_lib.FLOAT16: 2, _lib.FLOAT32: 4, _lib.FLOAT64: 8, _lib.INT8: 1, _lib.INT16: 2, _lib.INT32: 4,
             _lib.INT64: 8, _lib.UINT8: 1, _lib.UINT16: 2, _lib.UINT32: 4, _lib.BFLOAT16: 2, _lib.UINT64: 8,
             _lib.COMPLEX32: 4, _lib.COMPLEX64: 8, _lib.COMPLEX128: 16}
    for dt, sz in sizes.items():
        assert lib.ntg_dtype_size(dt) == sz
    # Float128=3, int128=11, uint128=15, Bool=16, TensorObj=17 are not served
    for dt in (3, 11, 15, 16, 17, 55):
        assert lib.ntg_dtype_size(dt) == 0
    assert lib.ntg_version() >= 100


def test_desc_struct_layout():
    assert ctypes.sizeof(_lib.GemmDesc) == 16 + 8 * 3 + 8 * 3 + 8 + 8 * 3 + 8 + 8 * 3 + 8 + 8 + 8
    assert _lib.GemmDesc.flags.offset == ctypes.sizeof(_lib.GemmDesc) - 8 and _lib.GemmDesc.workspace_bytes.offset == _lib.GemmDesc.flags.offset - 8


def test_argument_errors_do_not_need_a_device():
    lib = _lib.load()
    a = np.zeros((4, 4), np.float32)
    p = a.ctypes.data_as(ctypes.c_void_p)
    # inner sizes differ
    rc = lib.ntg_matmult(_lib.FLOAT32, p, p, p, 4, 4, 3, 4, 0, 0)
    assert rc == 1 and b"inner sizes" in lib.ntg_last_error()
    # unsupported dtype (Float128 = 3)
    rc = lib.ntg_matmult(3, p, p, p, 4, 4, 4, 4, 0, 0)
    assert rc == 2
    # the complex dtypes have their workspace sized like the integers' (stored col matrix) plus the per-image weight gradients
    assert lib.ntg_conv2d_backward_workspace_bytes(_lib.COMPLEX64, 2, 3, 5, 5, 4, 3, 3, 1, 1, 1, 1, 1, 1, 1) == 11008 + 2 * 4 * 27 * 8   # col 2*27*25*8 = 10800 -> 11008 (256-byte aligned)
    assert lib.ntg_conv2d_backward_workspace_bytes(_lib.INT64, 2, 3, 5, 5, 4, 3, 3, 1, 1, 1, 1, 1, 1, 1) == 10800
    # negative size
    rc = lib.ntg_matmult(_lib.FLOAT32, p, p, p, -1, 4, 4, 4, 0, 0)
    assert rc == 1
    # empty product is a no-op
    assert lib.ntg_matmult(_lib.FLOAT32, p, p, p, 0, 4, 4, 4, 0, 0) == 0
    # bias that does not broadcast
    rc = lib.ntg_linear(_lib.FLOAT32, p, p, p, p, 4, 4, 4, 0, 0, 2, 4)
    assert rc == 1 and b"bias" in lib.ntg_last_error()
    # empty sliding-block array
    rc = lib.ntg_unfold2d(_lib.FLOAT32, p, p, 1, 1, 2, 2, 5, 5, 1, 1, 0, 0, 1, 1)
    assert rc == 1
    assert lib.ntg_conv2d_workspace_bytes(_lib.FLOAT32, 1, 3, 8, 8, 3, 3, 1, 1, 1, 1, 1, 1) == 27 * 64 * 4
    # implicit-GEMM convolutions need no workspace; integers and kernels wider than 8 taps unfold
    assert lib.ntg_conv2d_forward_workspace_bytes(_lib.FLOAT32, 1, 3, 8, 8, 3, 3, 1, 1, 1, 1, 1, 1) == 0
    assert lib.ntg_conv2d_forward_workspace_bytes(_lib.INT32, 1, 3, 8, 8, 3, 3, 1, 1, 1, 1, 1, 1) == 27 * 64 * 4
    assert lib.ntg_conv2d_forward_workspace_bytes(_lib.FLOAT32, 1, 3, 16, 16, 9, 3, 1, 1, 4, 1, 1, 1) == 27 * 3 * 256 * 4
    # a 1x1 kernel with unit stride and no padding is a product on the image where it lies: no buffer for any dtype
    assert lib.ntg_conv2d_forward_workspace_bytes(_lib.INT32, 2, 3, 8, 8, 1, 1, 1, 1, 0, 0, 1, 1) == 0
    assert lib.ntg_conv2d_forward_workspace_bytes(_lib.INT32, 2, 3, 8, 8, 1, 1, 2, 1, 0, 0, 1, 1) == 2 * 3 * 4 * 8 * 4
    # the faster forward form: channels-last copy of the image with its zero border (the padding made real: 7x7 -> 9x9;
    # 256-byte aligned) + permuted weights, when the channels of a group fill whole 64-byte runs; else what the plain query says
    fast = lib.ntg_conv2d_fast_workspace_bytes
    assert fast(_lib.BFLOAT16, 2, 64, 7, 7, 48, 3, 3, 1, 1, 1, 1, 1, 1, 2) == 20736 + 48 * 32 * 9 * 2    # 2*64*81*2 = 20736
    assert fast(_lib.FLOAT32, 1, 16, 5, 5, 8, 3, 3, 1, 1, 1, 1, 1, 1, 1) == 3328 + 8 * 16 * 9 * 4        # 16*49*4 = 3136 -> 3328
    # 16-bit: channels per group are padded to whole 64-byte runs in the copy (up to 4x); Float32 takes whole runs only
    assert fast(_lib.BFLOAT16, 2, 40, 5, 5, 8, 3, 3, 1, 1, 1, 1, 1, 1, 1) == 12544 + 8 * 64 * 9 * 2       # 40 -> 64 channels, 5x5 -> 7x7
    assert fast(_lib.BFLOAT16, 2, 64, 5, 5, 8, 3, 3, 2, 2, 0, 0, 1, 1, 1) == 6400 + 8 * 64 * 9 * 2        # no padding: no border
    assert fast(_lib.FLOAT32, 1, 24, 8, 8, 4, 3, 3, 1, 1, 1, 1, 1, 1, 1) == 0                             # 24 is not a multiple of 16
    # up to 32 bytes of channels per group: pixels of 16 or 32 bytes, 4 or 2 taps of a tap row per K-step (rows padded to that)
    assert fast(_lib.BFLOAT16, 1, 16, 5, 5, 8, 3, 3, 1, 1, 1, 1, 1, 1, 1) == 1024 + 8 * 3 * 4 * 16 * 2   # 16 channels, rows of 3 -> 4 taps
    assert fast(_lib.FLOAT16, 2, 24, 5, 5, 8, 3, 3, 1, 1, 1, 1, 1, 1, 2) == 3328 + 8 * 3 * 4 * 16 * 2     # 2 groups of 12 -> 16
    assert fast(_lib.BFLOAT16, 1, 3, 8, 8, 4, 3, 3, 1, 1, 1, 1, 1, 1, 1) == 1024 + 4 * 3 * 4 * 8 * 2      # RGB: 3 -> 8 channels
    assert fast(_lib.FLOAT32, 1, 3, 8, 8, 4, 3, 3, 1, 1, 1, 1, 1, 1, 1) == 1024 + 4 * 3 * 4 * 4 * 4       # RGB: 3 -> 4 channels
    assert fast(_lib.FLOAT64, 1, 16, 5, 5, 8, 3, 3, 1, 1, 1, 1, 1, 1, 1) == 0
    assert fast(_lib.INT32, 1, 16, 5, 5, 8, 3, 3, 1, 1, 1, 1, 1, 1, 1) == 16 * 9 * 25 * 4
    assert fast(_lib.FLOAT32, 4, 64, 8, 8, 32, 1, 1, 1, 1, 0, 0, 1, 1, 1) == 0                            # 1x1: product in place
    assert fast(_lib.FLOAT32, 4, 64, 7, 7, 32, 1, 1, 1, 1, 0, 0, 1, 1, 1) == 50176 + 32 * 64 * 4   # rows of 196 bytes
    assert fast(_lib.FLOAT32, 1, 16, 2, 2, 8, 3, 3, 1, 1, 0, 0, 1, 1, 1) == -1                            # kernel larger than the image
    # per-image weight gradients [B, O, C/g * taps] instead of the im2col matrix
    # (the larger figure: channels-last copy of the image with the 2 channels of each group padded to 4, per-image results)
    assert lib.ntg_conv2d_backward_workspace_bytes(_lib.FLOAT32, 2, 4, 8, 8, 6, 3, 3, 1, 1, 1, 1, 1, 1, 2) == 2 * 2 * 4 * 64 * 4 + 2 * 6 * 4 * 9 * 4
    assert lib.ntg_conv2d_backward_workspace_bytes(_lib.FLOAT64, 2, 4, 8, 8, 6, 3, 3, 1, 1, 1, 1, 1, 1, 2) == 2 * 6 * 2 * 9 * 8
    assert lib.ntg_conv2d_backward_workspace_bytes(_lib.FLOAT32, 2, 4, 8, 8, 6, 3, 3, 1, 1, 1, 1, 1, 1, 3) == -1
    # transposed convolution: output_padding must stay below the stride; sizes follow (in-1)*s - 2p + d(k-1) + 1 + op
    assert lib.ntg_conv_transpose2d_workspace_bytes(_lib.FLOAT32, 1, 3, 9, 7, 8, 3, 3, 2, 2, 0, 0, 1, 1, 2, 1, 1) == -1
    assert lib.ntg_conv_transpose2d_workspace_bytes(_lib.FLOAT32, 1, 3, 9, 7, 8, 3, 3, 2, 2, 0, 0, 1, 1, 1, 1, 1) > 0
    assert lib.ntg_conv_transpose2d(_lib.FLOAT32, p, p, p, 1, 3, 9, 7, 8, 3, 3, 2, 2, 0, 0, 1, 1, 2, 1, 1) == 1
    assert b"output_padding" in lib.ntg_last_error()
    assert lib.ntg_conv_transpose2d(_lib.FLOAT32, p, p, p, 1, 3, 9, 7, 8, 3, 3, 2, 2, 0, 0, 1, 1, 1, 1, 2) == 1    # 3 % 2 groups
    # N-d geometry arrays
    arr = lambda *v: (ctypes.c_int64 * len(v))(*v)
    # three spatial axes: floats gather the operand inside the product, integers unfold [B, C*taps, L] first
    assert lib.ntg_convnd_workspace_bytes(_lib.FLOAT32, 2, 3, 4, 3, arr(5, 6, 7), arr(2, 3, 2), arr(1, 2, 1), arr(1, 0, 2), arr(2, 1, 1), 1, 0) == 0
    assert lib.ntg_convnd_workspace_bytes(_lib.INT32, 2, 3, 4, 3, arr(5, 6, 7), arr(2, 3, 2), arr(1, 2, 1), arr(1, 0, 2), arr(2, 1, 1), 1, 0) \
        == 2 * 3 * 12 * (5 * 2 * 10) * 4
    assert lib.ntg_convnd_workspace_bytes(_lib.FLOAT32, 2, 3, 4, 5, arr(5, 6, 7), arr(2, 3, 2), arr(1, 2, 1), arr(1, 0, 2), arr(2, 1, 1), 1, 0) == -1
    assert lib.ntg_convnd(_lib.FLOAT32, p, p, p, 1, 3, 4, 3, arr(5, 6, 7), arr(2, 3, 9), arr(1, 1, 1), arr(0, 0, 0), arr(1, 1, 1), 1) == 1
    assert b"sliding blocks" in lib.ntg_last_error()
    assert lib.ntg_convnd(_lib.FLOAT32, p, p, p, 0, 3, 4, 3, arr(5, 6, 7), arr(2, 3, 2), arr(1, 1, 1), arr(0, 0, 0), arr(1, 1, 1), 1) == 0
    assert lib.ntg_conv_transposend(_lib.FLOAT32, p, p, p, 1, 3, 4, 3, arr(5, 6, 7), arr(2, 3, 2), arr(1, 1, 1), arr(0, 0, 0), arr(1, 1, 1),
                                    arr(0, 1, 0), 1) == 1
    d = _lib.GemmDesc()
    d.dtype, d.m, d.k, d.n, d.batches, d.c_mode = _lib.FLOAT32, 4, 4, 4, 1, 7
    assert lib.ntg_gemm_dev(ctypes.byref(d), p, p, p, None) == 1


def test_split_k_planner_needs_no_device():
    """ntg_gemm_workspace_bytes is host arithmetic: which products are offered a split along k, and into how many ranges
    (bytes = ranges x m x n x 4 for the 16-bit dtypes, whose partial sums are fp32; x element size otherwise)."""
    lib = _lib.load()

    def ws(dtype, m, k, n, batches=1, ta=0, tb=0, lda=0):
        d = _lib.GemmDesc()
        d.dtype, d.transpose_a, d.transpose_b, d.c_mode = dtype, ta, tb, _lib.C_OVERWRITE
        d.m, d.k, d.n, d.batches, d.lda = m, k, n, batches, lda
        return lib.ntg_gemm_workspace_bytes(ctypes.byref(d))

    def ranges(dtype, m, k, n, es):
        b = ws(dtype, m, k, n)
        assert b % (m * n * es) == 0
        return b // (m * n * es)

    # full-chip products are never split; integers and the streaming (m <= 32) shapes neither.  The plan looks at one item
    # only -- a split changes the order of summation over k, and an item must come out the same alone and in a batch -- so a
    # batch is offered its item's split, with the partial sums of every item
    for dt in (_lib.BFLOAT16, _lib.FLOAT16, _lib.FLOAT32, _lib.FLOAT64):
        assert ws(dt, 4096, 4096, 4096) == 0
        assert ws(dt, 4096, 4096, 4096, batches=3) == 0
        one = ws(dt, 256, 8192, 2048)
        assert one > 0 and ws(dt, 256, 8192, 2048, batches=2) == 2 * one and ws(dt, 256, 8192, 2048, batches=7) == 7 * one
    assert ws(_lib.INT32, 64, 8192, 64) == 0
    assert ws(_lib.FLOAT32, 16, 8192, 8192) == 0 and ws(_lib.BFLOAT16, 32, 8192, 8192) == 0
    # 16-bit, 128 x 128 tiles: 64 tiles and k = 8192 -> four ranges; one tile and k = 16384 -> sixteen
    assert ranges(_lib.BFLOAT16, 128, 8192, 8192, 4) == 4
    assert ranges(_lib.FLOAT16, 128, 16384, 128, 4) == 16
    # a short k does not pay for the second pass; a product that already has a tile for most CUs does not either
    assert ws(_lib.BFLOAT16, 1024, 1024, 1024) == 0
    assert ws(_lib.BFLOAT16, 1536, 4096, 1536) == 0
    # rows that are not 16-byte multiples cannot use the kernel that writes fp32 partial sums; products this large are
    # offered padded copies of the operands that need them instead (B and C for n = 8190, A for a pitch of 8196)
    assert ws(_lib.BFLOAT16, 128, 8192, 8190) == 8192 * 8192 * 2 + 128 * 8192 * 2 and ws(_lib.BFLOAT16, 128, 8192, 8192, lda=8196) == 128 * 8192 * 2
    assert ws(_lib.BFLOAT16, 128, 1024, 1022) == 0 and ws(_lib.BFLOAT16, 128, 1024, 1024, lda=1028) == 0      # too small to repay the copies
    # 8-bit integers: the alternative is the vector ALU, so the padded form starts earlier
    # (k 1001 -> 1008, n 530 -> 544; the copies of A and B have rows of whole 128-byte lines: 1024 and 640 bytes)
    assert ws(_lib.INT8, 520, 1001, 530) == 520 * 1024 + 1008 * 640 + 520 * 544 + (256 - 520 * 1024 % 256) % 256 + (256 - 1008 * 640 % 256) % 256 + (256 - 520 * 544 % 256) % 256
    assert ws(_lib.INT8, 100, 101, 103) == 0 and ws(_lib.INT32, 100, 101, 103) == 0
    # fp32 / fp64, 64 x 64 tiles: 16 tiles and k = 1024 -> eight ranges of 128; 256 or more tiles -> none
    assert ranges(_lib.FLOAT32, 256, 1024, 256, 4) == 8
    assert ranges(_lib.FLOAT64, 256, 1024, 256, 8) == 8
    assert ws(_lib.FLOAT32, 1024, 4096, 1024) == 0 and ws(_lib.FLOAT64, 1024, 4096, 1024) == 0
    assert ws(_lib.FLOAT32, 768, 768, 768) == 0
    # NTG_GEMM_KEEP_K_ORDER: no split along k is offered (padded copies and byte planes keep the order and stay on offer)
    d = _lib.GemmDesc()
    d.dtype, d.c_mode, d.flags = _lib.FLOAT32, _lib.C_OVERWRITE, _lib.GEMM_KEEP_K_ORDER
    d.m, d.k, d.n, d.batches = 256, 1024, 256, 1
    assert lib.ntg_gemm_workspace_bytes(ctypes.byref(d)) == 0
    d.dtype, d.m, d.k, d.n = _lib.BFLOAT16, 128, 8192, 8190
    assert lib.ntg_gemm_workspace_bytes(ctypes.byref(d)) == 8192 * 8192 * 2 + 128 * 8192 * 2


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libntgemm.so"))
    with pytest.raises(RuntimeError, match="not built"):
        _lib.load()
