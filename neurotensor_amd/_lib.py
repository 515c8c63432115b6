"""ctypes binding of libntgemm.so (the C ABI declared in include/ntgemm.h).

There is no fallback: if the HIP library has not been built, loading raises.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# NTG_LIB_PATH points the loader at another build of the same library (the host-sanitizer build, lib/asan/libntgemm.so)
LIB_PATH = os.environ.get("NTG_LIB_PATH") or os.path.join(_HERE, "lib", "libntgemm.so")

# ntg_dtype (== nt::DType values; BF16/U64 are extensions)
FLOAT16, FLOAT32, FLOAT64 = 0, 1, 2
COMPLEX32, COMPLEX64, COMPLEX128 = 4, 5, 6      # interleaved (re, im) pairs of half / float / double
INT8, INT16, INT32, INT64 = 7, 8, 9, 10
UINT8, UINT16, UINT32 = 12, 13, 14
BFLOAT16, UINT64 = 100, 101

C_OVERWRITE, C_ACCUMULATE, C_BIAS = 0, 1, 2
GEMM_PTRS_ALIGNED16 = 1               # NTG_GEMM_PTRS_ALIGNED16
GEMM_KEEP_K_ORDER = 2                 # NTG_GEMM_KEEP_K_ORDER
NOALLOC_SCRATCH_BYTES = 64 << 20      # NTG_NOALLOC_SCRATCH_BYTES
DIAG_MFMA_OPERAND_BYTES = 128 << 10   # NTG_DIAG_MFMA_OPERAND_BYTES
DIAG_MFMA_FLOPS_PER_PASS = 8388608    # NTG_DIAG_MFMA_FLOPS_PER_PASS

STATUS_NAMES = {0: "NTG_OK", 1: "NTG_ERR_INVALID_ARGUMENT", 2: "NTG_ERR_UNSUPPORTED_DTYPE",
                3: "NTG_ERR_DEVICE", 4: "NTG_ERR_OUT_OF_MEMORY", 5: "NTG_ERR_NO_DEVICE"}


class GemmDesc(ctypes.Structure):
    _fields_ = [
        ("dtype", ctypes.c_int32), ("transpose_a", ctypes.c_int32), ("transpose_b", ctypes.c_int32), ("c_mode", ctypes.c_int32),
        ("m", ctypes.c_int64), ("k", ctypes.c_int64), ("n", ctypes.c_int64),
        ("lda", ctypes.c_int64), ("ldb", ctypes.c_int64), ("ldc", ctypes.c_int64),
        ("batches", ctypes.c_int64),
        ("stride_a", ctypes.c_int64), ("stride_b", ctypes.c_int64), ("stride_c", ctypes.c_int64),
        ("bias", ctypes.c_void_p),
        ("bias_batch_stride", ctypes.c_int64), ("bias_row_stride", ctypes.c_int64), ("bias_col_stride", ctypes.c_int64),
        ("workspace", ctypes.c_void_p), ("workspace_bytes", ctypes.c_int64),
        ("flags", ctypes.c_int64),
    ]


class NtgError(RuntimeError):
    """Raised when an entry point of libntgemm.so returns a non-zero ntg_status."""

    def __init__(self, status, message):
        super().__init__(f"{STATUS_NAMES.get(status, status)}: {message}")
        self.status = status


# every symbol include/ntgemm.h declares, with its ctypes signature
_i64, _vp, _ci = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int
_pi64 = ctypes.POINTER(ctypes.c_int64)
_pp = ctypes.POINTER(ctypes.c_void_p)
SIGNATURES = {
    "ntg_last_error": (ctypes.c_char_p, []),
    "ntg_version": (_ci, []),
    "ntg_dtype_size": (_i64, [_ci]),
    "ntg_device_count": (_ci, []),
    "ntg_release_host_buffers": (_ci, []),
    "ntg_matmult": (_ci, [_ci, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _ci, _ci]),
    "ntg_matmult_batch": (_ci, [_ci, _pp, _pp, _pp, _i64, _i64, _i64, _i64, _i64, _ci, _ci]),
    "ntg_linear": (_ci, [_ci, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _ci, _ci, _i64, _i64]),
    "ntg_unfold2d": (_ci, [_ci, _vp, _vp] + [_i64] * 12),
    "ntg_conv2d": (_ci, [_ci, _vp, _vp, _vp] + [_i64] * 14),
    "ntg_matmult_dev": (_ci, [_ci, _vp, _vp, _vp, _i64, _i64, _i64, _ci, _ci, _vp]),
    "ntg_gemm_dev": (_ci, [ctypes.POINTER(GemmDesc), _vp, _vp, _vp, _vp]),
    "ntg_gemm_relu_dev": (_ci, [ctypes.POINTER(GemmDesc), _vp, _vp, _vp, _vp]),
    "ntg_gemm_noalloc_dev": (_ci, [ctypes.POINTER(GemmDesc), _vp, _vp, _vp, _vp]),
    "ntg_gemm_workspace_bytes": (_i64, [ctypes.POINTER(GemmDesc)]),
    "ntg_gemm_ptrs_dev": (_ci, [ctypes.POINTER(GemmDesc), _vp, _vp, _vp, _vp]),
    "ntg_diag_mfma_rate_dev": (_ci, [_ci, _vp, _i64, _i64, _vp, _vp]),
    "ntg_unfold2d_dev": (_ci, [_ci, _vp, _vp] + [_i64] * 12 + [_vp]),
    "ntg_conv2d_workspace_bytes": (_i64, [_ci] + [_i64] * 12),
    "ntg_conv2d_forward_workspace_bytes": (_i64, [_ci] + [_i64] * 12),
    "ntg_conv2d_fast_workspace_bytes": (_i64, [_ci] + [_i64] * 14),
    "ntg_conv2d_backward_workspace_bytes": (_i64, [_ci] + [_i64] * 14),
    "ntg_conv_transpose2d_workspace_bytes": (_i64, [_ci] + [_i64] * 16),
    "ntg_conv_transpose2d_dev": (_ci, [_ci, _vp, _vp, _vp, _vp, _i64] + [_i64] * 16 + [_vp]),
    "ntg_conv_transpose2d": (_ci, [_ci, _vp, _vp, _vp] + [_i64] * 16),
    "ntg_unfoldnd_dev": (_ci, [_ci, _vp, _vp, _i64, _i64, _ci] + [_pi64] * 5 + [_vp]),
    "ntg_unfoldnd_backward_dev": (_ci, [_ci, _vp, _vp, _i64, _i64, _ci] + [_pi64] * 5 + [_ci, _vp]),
    "ntg_convnd_workspace_bytes": (_i64, [_ci, _i64, _i64, _i64, _ci] + [_pi64] * 5 + [_i64, _ci]),
    "ntg_convnd_dev": (_ci, [_ci, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _ci] + [_pi64] * 5 + [_i64, _vp]),
    "ntg_convnd_backward_dev": (_ci, [_ci, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _ci] + [_pi64] * 5 + [_i64, _ci, _vp]),
    "ntg_conv_transposend_workspace_bytes": (_i64, [_ci, _i64, _i64, _i64, _ci] + [_pi64] * 6 + [_i64]),
    "ntg_conv_transposend_dev": (_ci, [_ci, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _ci] + [_pi64] * 6 + [_i64, _vp]),
    "ntg_convnd": (_ci, [_ci, _vp, _vp, _vp, _i64, _i64, _i64, _ci] + [_pi64] * 5 + [_i64]),
    "ntg_convnd_backward": (_ci, [_ci, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _ci] + [_pi64] * 5 + [_i64, _ci]),
    "ntg_conv_transposend": (_ci, [_ci, _vp, _vp, _vp, _i64, _i64, _i64, _ci] + [_pi64] * 6 + [_i64]),
    "ntg_conv2d_dev": (_ci, [_ci, _vp, _vp, _vp, _vp, _i64] + [_i64] * 14 + [_vp]),
    "ntg_unfold2d_backward": (_ci, [_ci, _vp, _vp] + [_i64] * 12 + [_ci]),
    "ntg_unfold2d_backward_dev": (_ci, [_ci, _vp, _vp] + [_i64] * 12 + [_ci, _vp]),
    "ntg_conv2d_backward": (_ci, [_ci, _vp, _vp, _vp, _vp, _vp] + [_i64] * 14 + [_ci]),
    "ntg_conv2d_backward_dev": (_ci, [_ci, _vp, _vp, _vp, _vp, _vp, _vp, _i64] + [_i64] * 14 + [_ci, _vp]),
}

_lib = None


def load():
    """Load libntgemm.so once; raise if it is missing (no CPU fallback exists)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: the HIP extension is not built. "
            "Run `python -c 'import __graft_entry__ as g; g.build()'` (or `make -C neurotensor_amd/csrc`).")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)          # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(status):
    if status != 0:
        raise NtgError(status, load().ntg_last_error().decode("utf-8", "replace"))
