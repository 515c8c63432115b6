// C ABI of the gfx950 matmult backend (declared in include/ntgemm.h): argument checks,
// dtype dispatch, host<->device staging for the host-pointer entry points, and the
// conv2d lowering.  No entry point throws; failures are reported as ntg_status plus a
// thread-local message.
#include "../../include/ntgemm.h"
#include "ntg_common.h"
#include "host_stage.h"

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <algorithm>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <vector>

namespace ntg {
hipError_t launch_gemm_mfma_f32(bool ta, bool tb, const GemmParams& p, hipStream_t s);
hipError_t launch_gemm_mfma_f64(bool ta, bool tb, const GemmParams& p, hipStream_t s);
hipError_t launch_gemm_mfma_f16(bool ta, bool tb, const GemmParams& p, hipStream_t s);
hipError_t launch_gemm_mfma_bf16(bool ta, bool tb, const GemmParams& p, hipStream_t s);
hipError_t launch_gemm_skinny(int dtype, bool ta, bool tb, const GemmParams& p, hipStream_t s, bool* handled);
hipError_t launch_gemm_ring_only_f32(bool ta, bool tb, const GemmParams& p, hipStream_t s, bool* taken);
hipError_t launch_gemm_ring_only_f16(bool ta, bool tb, const GemmParams& p, hipStream_t s, bool* taken);
hipError_t launch_gemm_ring_only_bf16(bool ta, bool tb, const GemmParams& p, hipStream_t s, bool* taken);
hipError_t launch_gemm_ring_only_i8(int dtype, bool ta, bool tb, const GemmParams& p, hipStream_t s, bool* taken);
hipError_t launch_gemm_ring_only_f64(bool ta, bool tb, const GemmParams& p, hipStream_t s, bool* taken);
hipError_t launch_gemm_ring_only(int dtype, bool ta, bool tb, const GemmParams& p, hipStream_t s, bool* taken) {
    *taken = false;
    switch (dtype) {
    case DT_I8: case DT_U8: return launch_gemm_ring_only_i8(dtype, ta, tb, p, s, taken);
    case DT_F32: return launch_gemm_ring_only_f32(ta, tb, p, s, taken);
    case DT_F64: return launch_gemm_ring_only_f64(ta, tb, p, s, taken);
    case DT_F16: return launch_gemm_ring_only_f16(ta, tb, p, s, taken);
    case DT_BF16: return launch_gemm_ring_only_bf16(ta, tb, p, s, taken);
    default: return hipSuccess;
    }
}
hipError_t launch_conv_mfma_f32(bool tb, int nd, const GemmParams& p, hipStream_t s);
hipError_t launch_conv_mfma_f64(bool tb, int nd, const GemmParams& p, hipStream_t s);
hipError_t launch_conv_mfma_f16(bool tb, int nd, const GemmParams& p, hipStream_t s);
hipError_t launch_conv_mfma_bf16(bool tb, int nd, const GemmParams& p, hipStream_t s);

hipError_t launch_conv_nhwc_f32(const GemmParams& p, hipStream_t s);
hipError_t launch_conv_nhwc_f16(const GemmParams& p, hipStream_t s);
hipError_t launch_conv_nhwc_bf16(const GemmParams& p, hipStream_t s);
hipError_t launch_conv_nhwc(int dtype, const GemmParams& p, hipStream_t s) {
    switch (dtype) {
    case DT_F32: return launch_conv_nhwc_f32(p, s);
    case DT_F16: return launch_conv_nhwc_f16(p, s);
    case DT_BF16: return launch_conv_nhwc_bf16(p, s);
    default: return hipErrorInvalidValue;
    }
}

hipError_t launch_conv_nhwc_dw_f32(bool ta, const GemmParams& p, hipStream_t s);
hipError_t launch_conv_nhwc_dw_f16(bool ta, const GemmParams& p, hipStream_t s);
hipError_t launch_conv_nhwc_dw_bf16(bool ta, const GemmParams& p, hipStream_t s);
hipError_t launch_conv_nhwc_dw(int dtype, bool ta, const GemmParams& p, hipStream_t s) {
    switch (dtype) {
    case DT_F32: return launch_conv_nhwc_dw_f32(ta, p, s);
    case DT_F16: return launch_conv_nhwc_dw_f16(ta, p, s);
    case DT_BF16: return launch_conv_nhwc_dw_bf16(ta, p, s);
    default: return hipErrorInvalidValue;
    }
}

hipError_t launch_conv_mfma(int dtype, bool tb, int nd, const GemmParams& p, hipStream_t s) {
    switch (dtype) {
    case DT_F32: return launch_conv_mfma_f32(tb, nd, p, s);
    case DT_F64: return launch_conv_mfma_f64(tb, nd, p, s);
    case DT_F16: return launch_conv_mfma_f16(tb, nd, p, s);
    case DT_BF16: return launch_conv_mfma_bf16(tb, nd, p, s);
    default: return hipErrorInvalidValue;
    }
}
}  // namespace ntg

// Scratch memory of ntg_gemm_noalloc_dev: a fixed array in every GPU's copy of this code object, so that the entry point
// needs no allocator.  Host code never uses the array's name as an address: ntg::noalloc_scratch_of_current_device() asks the runtime
// for the address of the current device's copy once and keeps it.
static __device__ __align__(256) unsigned char scratch[NTG_NOALLOC_SCRATCH_BYTES];

// Flags of ntg_gemm_ptrs_dev's alignment check (one word per call, handed out round-robin), in the same kind of array and
// for the same reason: the device entry points allocate nothing.
#define NTG_GATE_SLOTS 1024
static __device__ __align__(256) int gate_flags[NTG_GATE_SLOTS];
namespace ntg {
// *flag = 1 when every entry of the three pointer tables is a multiple of 16 bytes, else 0
__global__ void __launch_bounds__(256) ptr_tables_aligned_kernel(const void* const* a, const void* const* b, void* const* c, const int batch, int* flag) {
    __shared__ unsigned bits;
    if (threadIdx.x == 0) bits = 0u;
    __syncthreads();
    unsigned mine = 0u;
    for (int i = threadIdx.x; i < batch; i += 256)
        mine |= (unsigned)(reinterpret_cast<uintptr_t>(a[i]) | reinterpret_cast<uintptr_t>(b[i]) | reinterpret_cast<uintptr_t>(c[i])) & 15u;
    if (mine) atomicOr(&bits, mine);
    __syncthreads();
    if (threadIdx.x == 0) *flag = bits == 0u ? 1 : 0;
}
}  // namespace ntg

namespace {

thread_local std::string g_last_error;

int fail(int status, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return status;
}

int hip_fail(hipError_t e, const char* what) {
    if (e == hipErrorOutOfMemory) return fail(NTG_ERR_OUT_OF_MEMORY, "%s: %s", what, hipGetErrorString(e));
    if (e == hipErrorNoDevice || e == hipErrorInvalidDevice) return fail(NTG_ERR_NO_DEVICE, "%s: %s", what, hipGetErrorString(e));
    return fail(NTG_ERR_DEVICE, "%s: %s", what, hipGetErrorString(e));
}

#define HIP_TRY(expr)                                   \
    do {                                                \
        hipError_t e__ = (expr);                        \
        if (e__ != hipSuccess) return hip_fail(e__, #expr); \
    } while (0)


inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

bool is_int_dtype(int dt) {
    switch (dt) {
    case ntg::DT_I8: case ntg::DT_I16: case ntg::DT_I32: case ntg::DT_I64:
    case ntg::DT_U8: case ntg::DT_U16: case ntg::DT_U32: case ntg::DT_U64: return true;
    default: return false;
    }
}

bool is_complex_dtype(int dt) { return dt == ntg::DT_C32 || dt == ntg::DT_C64 || dt == ntg::DT_C128; }
// integers and the complex types: computed lane by lane on the vector ALU, bit-exact; no matrix-pipe or gathering forms
bool is_valu_dtype(int dt) { return is_int_dtype(dt) || is_complex_dtype(dt); }

// Fills the derived fields and launches the kernel family for the dtype.
int launch_gemm(ntg::GemmParams p, int dtype, bool ta, bool tb, hipStream_t s) {
    const int64_t es = ntg::elem_size(dtype);
    const int64_t ve = 16 / es;
    p.vecA_ok = (p.lda % ve == 0) && (p.Aptr || p.sA % ve == 0) && (p.krange_items == 0 || p.sAk % ve == 0);
    p.vecB_ok = (p.ldb % ve == 0) && (p.Bptr || p.sB % ve == 0) && (p.krange_items == 0 || p.sBk % ve == 0);
    hipError_t e;
    // relu_ on the result: inside the DMA-fed kernel's epilogue where that kernel serves the product (more than 32 rows: the
    // streaming kernels take the others), else as a pass over C after whichever kernel runs
    const int act = p.act;
    p.act = ntg::ACT_NONE;
    if (act != ntg::ACT_NONE) {
        if (p.Cptr || !(dtype == ntg::DT_F32 || dtype == ntg::DT_F64 || dtype == ntg::DT_F16 || dtype == ntg::DT_BF16))
            return fail(NTG_ERR_INVALID_ARGUMENT, "the relu epilogue takes strided floating-point results");
        if (p.M > 32 && p.cmode != ntg::C_PARTIAL) {
            ntg::GemmParams q = p;
            q.act = act;
            bool taken = false;
            e = ntg::launch_gemm_ring_only(dtype, ta, tb, q, s, &taken);
            if (e != hipSuccess) return hip_fail(e, "gemm launch");
            if (taken) return NTG_OK;
        }
    }
    const auto finish = [&]() -> int {
        if (act == ntg::ACT_NONE) return NTG_OK;
        const hipError_t ea = ntg::launch_relu_inplace(dtype, p.C, p.ldc, p.sC, p.M, p.N, p.batch, s);
        return ea == hipSuccess ? NTG_OK : hip_fail(ea, "relu launch");
    };
    if (dtype == ntg::DT_I8 || dtype == ntg::DT_U8) {
        e = ntg::launch_gemm_mfma_i8(dtype, ta, tb, p, s);
    } else if (is_int_dtype(dtype)) {
        e = ntg::launch_gemm_valu(dtype, ta, tb, p, s);
    } else if (is_complex_dtype(dtype)) {
        e = ntg::launch_gemm_complex(dtype, ta, tb, p, s);
    } else {
        bool handled = false;
        // (the streaming kernels for up to 32 rows split k over their wavefronts: not for a caller who wants the one chain)
        if (!(p.keep_k_order && dtype == ntg::DT_F32)) e = ntg::launch_gemm_skinny(dtype, ta, tb, p, s, &handled);
        if (e != hipSuccess) return hip_fail(e, "skinny gemm launch");
        if (handled) return finish();
        switch (dtype) {
        case ntg::DT_F32: e = ntg::launch_gemm_mfma_f32(ta, tb, p, s); break;
        case ntg::DT_F64: e = ntg::launch_gemm_mfma_f64(ta, tb, p, s); break;
        case ntg::DT_F16: e = ntg::launch_gemm_mfma_f16(ta, tb, p, s); break;
        case ntg::DT_BF16: e = ntg::launch_gemm_mfma_bf16(ta, tb, p, s); break;
        default: return fail(NTG_ERR_UNSUPPORTED_DTYPE, "dtype %d is not supported", dtype);
        }
    }
    if (e != hipSuccess) return hip_fail(e, "gemm launch");
    return finish();
}

// Split-K.  A product whose output tiles cannot occupy the 256 CUs but whose K is deep (a Linear layer on a few
// hundred rows) is cut into `splits` equal k ranges, computed as one batched launch of the ordinary kernels into a
// workspace [splits][M][N] (fp32 sums for the 16-bit dtypes, so nothing is rounded early), and added up in ascending
// range order by a second kernel.  Deterministic; applied only when the caller supplies the workspace.
// The plan is a function of ONE item's M, N, K (and dtype, flags, alignment) only, never of the batch count: a split
// changes the order of summation over k, and an item must come out bit for bit the same alone and inside a batch
// (the reference's batched == per-item rule, tests/src/matmult_test.cpp:108-189).  A batch whose items are split runs one
// batched launch per k range into [splits][batch][M][N] and one reduction over all items.
struct SplitPlan { int splits; int64_t kc; int64_t bytes; };

// 16-, 32- and 64-bit integers on the 8-bit matrix pipe (byte planes, gemm_mfma_i8.hip): P (P + 1) / 2 8-bit products
// (P bytes per element) instead of the vector ALU's multiply-adds, plus the passes that split the operands and
// recombine the partial sums.  Taken when the caller supplies the workspace and an estimate of both times favours it.
// Measured on MI355X: the vector-ALU kernel spends about 0.07 us (16- and 32-bit; 0.13 us 64-bit) per k on each round of
// 64 x 64 tiles over the 256 CUs, plus as much once; the plane form costs its P + 3 launches (17 / 30 / 55 us for
// P = 2 / 4 / 8), the 8-bit products at about 10^9 multiply-adds per us, and the partial sums written and read at 4 TB/s.
struct IntPlanesPlan {
    bool ok; int planes, Kp, Np; int64_t a_bytes, b_bytes, p_bytes;
    int64_t bytes() const { return a_bytes + b_bytes + p_bytes; }
};
static int int_planes_of(int dtype) {
    switch (dtype) {
    case ntg::DT_I16: case ntg::DT_U16: return 2;
    case ntg::DT_I32: case ntg::DT_U32: return 4;
    case ntg::DT_I64: case ntg::DT_U64: return 8;
    default: return 0;
    }
}
static IntPlanesPlan plan_int_planes(const ntg::GemmParams& p, int dtype) {
    IntPlanesPlan pl;
    std::memset(&pl, 0, sizeof pl);
    const int P = int_planes_of(dtype);
    if (P == 0 || p.Aptr || p.Bptr || p.Cptr) return pl;
    if (p.M < 128 || p.N < 128 || p.K < 64) return pl;
    pl.planes = P;
    pl.Kp = (p.K + 15) / 16 * 16;
    pl.Np = (p.N + 15) / 16 * 16;
    {
        const double macs = (double)p.M * p.N * p.K * p.batch;
        const double rounds = (double)(((int64_t)((p.M + 63) / 64) * ((p.N + 63) / 64) * p.batch + 255) / 256);
        const double valu_us = (double)p.K * (P == 8 ? 0.13 : P == 4 ? 0.07 : 0.055) * (rounds + 1.0);
        const double planes_us = (P == 8 ? 55.0 : P == 4 ? 30.0 : 17.0) + macs * (P * (P + 1) / 2) / 1.0e9 +
                                 8.0 * P * p.batch * (double)p.M * pl.Np / 4.0e6;
        if (planes_us > 0.8 * valu_us) return pl;
    }
    if ((int64_t)P * pl.Kp >= (1 << 17) || pl.Np >= (1 << 23)) return pl;     // 32-bit partial sums: P K 2^14 < 2^31
    pl.a_bytes = (int64_t)align_up((size_t)((p.sA == 0 ? 1 : p.batch) * (int64_t)p.M * P * pl.Kp), 256);
    pl.b_bytes = (int64_t)align_up((size_t)((p.sB == 0 ? 1 : p.batch) * (int64_t)P * pl.Kp * pl.Np), 256);
    pl.p_bytes = (int64_t)P * p.batch * p.M * pl.Np * 4;
    pl.ok = true;
    return pl;
}
static int run_int_planes(const ntg::GemmParams& p, const IntPlanesPlan& pl, bool ta, bool tb, void* ws, hipStream_t s) {
    const int P = pl.planes;
    char* a_pl = static_cast<char*>(ws);
    char* b_pl = a_pl + pl.a_bytes;
    char* parts = b_pl + pl.b_bytes;
    ntg::IntPlanesParams q;
    q.M = p.M; q.N = p.N; q.K = p.K; q.Kp = pl.Kp; q.Np = pl.Np; q.batch = p.batch;
    q.lda = p.lda; q.ldb = p.ldb; q.sA = p.sA; q.sB = p.sB; q.ta = ta; q.tb = tb;
    hipError_t e = ntg::launch_int_split_planes(P, p.A, p.B, a_pl, b_pl, q, s);
    if (e != hipSuccess) return hip_fail(e, "byte-plane split launch");
    const int64_t per = (int64_t)p.M * pl.Np;
    for (int sh = 0; sh < P; ++sh) {
        ntg::GemmParams g;
        std::memset(&g, 0, sizeof g);
        g.M = p.M; g.N = pl.Np; g.K = (sh + 1) * pl.Kp; g.batch = p.batch;
        g.A = a_pl;
        g.B = b_pl + (int64_t)(P - 1 - sh) * pl.Kp * pl.Np;
        g.C = parts + (int64_t)sh * p.batch * per * 4;
        g.lda = (int64_t)P * pl.Kp; g.ldb = pl.Np; g.ldc = pl.Np;
        g.sA = p.sA == 0 ? 0 : (int64_t)p.M * P * pl.Kp;
        g.sB = p.sB == 0 ? 0 : (int64_t)P * pl.Kp * pl.Np;
        g.sC = per;
        g.cmode = ntg::C_PARTIAL;
        g.vecA_ok = 1; g.vecB_ok = 1;
        e = ntg::launch_gemm_mfma_i8(ntg::DT_I8, false, false, g, s);
        if (e != hipSuccess) return hip_fail(e, "byte-plane product launch");
    }
    e = ntg::launch_int_combine(P, parts, p, pl.Np, s);
    if (e != hipSuccess) return hip_fail(e, "byte-plane combine launch");
    return NTG_OK;
}

// Padded copies.  The DMA-fed kernels need 16-byte rows (leading dimensions, batch strides, base pointers, and K, N -- M
// under transpose_a -- multiples of one 16-byte chunk); a product that misses this falls to the vector ALU
// (8-bit: 40 x slower) or the register-staged kernel (16-bit: half the rate; Float32 / Float64: 0.8 - 0.85 of it).  With a workspace the operands that need it
// are copied into rows padded with zeros to whole chunks (zero products add nothing: bit-identical integers, the same
// single rounding for the 16-bit floats), the product runs on the DMA-fed kernel, and a result whose own rows are not
// 16-byte multiples is computed into a padded copy and copied back.  Taken for products large enough to repay the copies.
struct PadPlan {
    bool ok, padA, padB, padC;
    bool stripA, stripB;            // the operand stays where it is, only its last k-rows are copied (and continued with zeros)
    int strip_k0, strip_rows;
    int Mp, Kp, Np;
    int64_t lda2, ldb2, rowsA2, rowsB2, a_bytes, b_bytes, c_bytes;
    int64_t bytes() const { return a_bytes + b_bytes + c_bytes; }
};
static PadPlan plan_pad(const ntg::GemmParams& p, int dtype, bool ta, bool tb) {
    PadPlan pl;
    std::memset(&pl, 0, sizeof pl);
    const bool half = dtype == ntg::DT_F16 || dtype == ntg::DT_BF16, byte = dtype == ntg::DT_I8 || dtype == ntg::DT_U8;
    const bool wide = dtype == ntg::DT_F32 || dtype == ntg::DT_F64;
    if ((!half && !byte && !wide) || p.Aptr || p.Bptr || p.Cptr || p.M <= 32) return pl;
    const int64_t es = ntg::elem_size(dtype), ve = 16 / es;
    // from where the faster kernel repays the copies: 8-bit against the vector ALU (40 x), 16-bit against the register-staged
    // kernel at half the rate, Float32 / Float64 against the register-staged kernel at 0.8 - 0.85 of the DMA-fed one
    const double macs = (double)p.M * p.N * p.K * p.batch;
    if (macs < (byte ? 268435456.0 : half ? 2147483648.0 : dtype == ntg::DT_F32 ? 4294967296.0 : 8589934592.0)) return pl;
    auto up = [&](int64_t v) { return (v + ve - 1) / ve * ve; };
    pl.Kp = (int)up(p.K); pl.Np = (int)up(p.N); pl.Mp = ta ? (int)up(p.M) : p.M;
    auto misaligned = [&](const void* ptr, int64_t ld, int64_t stride) {
        return ld % ve != 0 || (p.batch > 1 && stride % ve != 0) || (reinterpret_cast<uintptr_t>(ptr) & 15) != 0;
    };
    pl.padA = misaligned(p.A, p.lda, p.sA) || pl.Kp != p.K || pl.Mp != p.M;
    pl.padB = misaligned(p.B, p.ldb, p.sB) || pl.Kp != p.K || pl.Np != p.N;
    pl.padC = misaligned(p.C, p.ldc, p.sC) || pl.Np != p.N || pl.Mp != p.M;
    if (!pl.padA && !pl.padB && !pl.padC) return pl;                       // nothing that padding would fix
    // (the copies' rows start on 128-byte boundaries: a pitch that is only a multiple of 16 bytes splits the cache lines that the
    //  kernel fetches, which costs it 3 - 13 %)
    auto line_pitch = [&](int64_t elems) { return (elems * es + 127) / 128 * 128 / es; };
    pl.lda2 = line_pitch(ta ? pl.Mp : pl.Kp); pl.rowsA2 = ta ? pl.Kp : p.M;
    pl.ldb2 = line_pitch(tb ? pl.Kp : pl.Np); pl.rowsB2 = tb ? pl.Np : pl.Kp;
    const int64_t ldmax = (int64_t)(1 << 23) / es;                         // (the kernels' 32-bit lane offsets)
    if ((pl.padA ? pl.lda2 : p.lda) >= ldmax || (pl.padB ? pl.ldb2 : p.ldb) >= ldmax) return pl;
    // An operand stored [k][m] / [k][n] that only lacks k-rows up to a whole chunk: its rows keep the 16-byte rule, so the kernel
    // reads it in place and takes its last k-rows (from a multiple of 128, which every kernel's K-step divides) from a copy of at
    // most 128 rows that continues with rows of zeros, instead of a copy of everything.
    if (pl.Kp != p.K && p.K > 128) {
        pl.strip_k0 = (pl.Kp - 1) / 128 * 128;
        pl.strip_rows = pl.Kp - pl.strip_k0;
        pl.stripA = pl.padA && ta && !misaligned(p.A, p.lda, p.sA) && pl.Mp == p.M;
        pl.stripB = pl.padB && !tb && !misaligned(p.B, p.ldb, p.sB) && pl.Np == p.N;
        if (pl.stripA) { pl.padA = false; pl.a_bytes = (int64_t)align_up((size_t)((p.sA == 0 ? 1 : p.batch) * pl.strip_rows * p.lda * es), 256); }
        if (pl.stripB) { pl.padB = false; pl.b_bytes = (int64_t)align_up((size_t)((p.sB == 0 ? 1 : p.batch) * pl.strip_rows * p.ldb * es), 256); }
    }
    if (pl.padA) pl.a_bytes = (int64_t)align_up((size_t)((p.sA == 0 ? 1 : p.batch) * pl.rowsA2 * pl.lda2 * es), 256);
    if (pl.padB) pl.b_bytes = (int64_t)align_up((size_t)((p.sB == 0 ? 1 : p.batch) * pl.rowsB2 * pl.ldb2 * es), 256);
    if (pl.padC) pl.c_bytes = (int64_t)align_up((size_t)((int64_t)p.batch * pl.Mp * pl.Np * es), 256);
    pl.ok = true;
    return pl;
}
static int run_padded(const ntg::GemmParams& p, const PadPlan& pl, int dtype, bool ta, bool tb, void* ws, hipStream_t s) {
    const int64_t es = ntg::elem_size(dtype);
    char* a2 = static_cast<char*>(ws);
    char* b2 = a2 + pl.a_bytes;
    char* c2 = b2 + pl.b_bytes;
    ntg::GemmParams q = p;
    q.M = pl.Mp; q.K = pl.Kp; q.N = pl.Np;
    hipError_t e;
    if (pl.padA) {
        e = ntg::launch_pad_copy(es, p.A, p.lda, p.sA, a2, pl.lda2, pl.rowsA2 * pl.lda2, ta ? p.K : p.M, ta ? p.M : p.K, pl.rowsA2, p.sA == 0 ? 1 : p.batch, s);
        if (e != hipSuccess) return hip_fail(e, "padded copy of A");
        q.A = a2; q.lda = pl.lda2; q.sA = p.sA == 0 ? 0 : pl.rowsA2 * pl.lda2;
    }
    if (pl.padB) {
        e = ntg::launch_pad_copy(es, p.B, p.ldb, p.sB, b2, pl.ldb2, pl.rowsB2 * pl.ldb2, tb ? p.N : p.K, tb ? p.K : p.N, pl.rowsB2, p.sB == 0 ? 1 : p.batch, s);
        if (e != hipSuccess) return hip_fail(e, "padded copy of B");
        q.B = b2; q.ldb = pl.ldb2; q.sB = p.sB == 0 ? 0 : pl.rowsB2 * pl.ldb2;
    }
    if (pl.stripA) {
        e = ntg::launch_pad_copy(es, static_cast<const char*>(p.A) + (int64_t)pl.strip_k0 * p.lda * es, p.lda, p.sA, a2, p.lda, (int64_t)pl.strip_rows * p.lda,
                                 p.K - pl.strip_k0, p.M, pl.strip_rows, p.sA == 0 ? 1 : p.batch, s);
        if (e != hipSuccess) return hip_fail(e, "copy of A's last k-rows");
        q.tailA = a2; q.s_tailA = p.sA == 0 ? 0 : (int64_t)pl.strip_rows * p.lda; q.tail_k0 = pl.strip_k0;
    }
    if (pl.stripB) {
        e = ntg::launch_pad_copy(es, static_cast<const char*>(p.B) + (int64_t)pl.strip_k0 * p.ldb * es, p.ldb, p.sB, b2, p.ldb, (int64_t)pl.strip_rows * p.ldb,
                                 p.K - pl.strip_k0, p.N, pl.strip_rows, p.sB == 0 ? 1 : p.batch, s);
        if (e != hipSuccess) return hip_fail(e, "copy of B's last k-rows");
        q.tailB = b2; q.s_tailB = p.sB == 0 ? 0 : (int64_t)pl.strip_rows * p.ldb; q.tail_k0 = pl.strip_k0;
    }
    if (pl.padC) {
        const int64_t sc2 = (int64_t)pl.Mp * pl.Np;
        if (p.cmode == ntg::C_ACCUMULATE) {
            e = ntg::launch_pad_copy(es, p.C, p.ldc, p.sC, c2, pl.Np, sc2, p.M, p.N, pl.Mp, p.batch, s);
            if (e != hipSuccess) return hip_fail(e, "padded copy of C");
        } else if (p.cmode == ntg::C_BIAS) {
            // the bias becomes the initial accumulator in the padded layout (reading it at padded indices would leave its array)
            e = ntg::launch_bias_fill(es, p.bias, p.bias_bs, p.bias_rs, p.bias_cs, c2, pl.Np, sc2, p.M, p.N, pl.Mp, p.batch, s);
            if (e != hipSuccess) return hip_fail(e, "bias fill");
            q.cmode = ntg::C_ACCUMULATE;
            q.bias = nullptr;
        }
        q.C = c2; q.ldc = pl.Np; q.sC = sc2;
    }
    const int rc = launch_gemm(q, dtype, ta, tb, s);
    if (rc) return rc;
    if (pl.padC) {
        e = ntg::launch_unpad_copy(es, c2, pl.Np, (int64_t)pl.Mp * pl.Np, p.C, p.ldc, p.sC, p.M, p.N, p.batch, s);
        if (e != hipSuccess) return hip_fail(e, "copy of the padded result");
    }
    return NTG_OK;
}

SplitPlan plan_splitk(const ntg::GemmParams& p, int dtype, bool ta) {
    SplitPlan none{1, p.K, 0};
    const int64_t es = ntg::elem_size(dtype);
    if (is_valu_dtype(dtype) || es == 0 || p.batch < 1 || p.batch > 65535 || p.Aptr || p.Bptr || p.Cptr || p.keep_k_order) return none;
    if (p.M <= 32 && dtype != ntg::DT_F64) return none;                       // the streaming kernels take these
    const bool half = dtype == ntg::DT_F16 || dtype == ntg::DT_BF16;
    if (half) {
        // only the DMA-fed kernel writes fp32 partial sums: 16-byte rows everywhere
        if (p.K % 8 || p.N % 8 || (ta && p.M % 8) || p.lda % 8 || p.ldb % 8 || p.lda >= (1 << 22) || p.ldb >= (1 << 22)) return none;
        if ((reinterpret_cast<uintptr_t>(p.A) & 15) || (reinterpret_cast<uintptr_t>(p.B) & 15)) return none;
        if (p.batch > 1 && (p.sA % 8 || p.sB % 8)) return none;
        // Both sides from the tile estimate of the 16-bit kernels (ring16_cost_us): the product as it is, against S batched
        // products over K / S (the tiles that the batched launch picks) plus the second pass, measured at about 4 us + the
        // fp32 partial sums written and read (8 S M N bytes) at 4 TB/s.  A split has to win by 5 %.  On a sweep of 23
        // shapes (64 .. 1024 rows, k 2048 .. 16384) the choice is the best measured S in 20 and within 5 % in two more
        // (1024 x 4096 x 1024: no split, 20.9 us against 24.5; 64 x 8192 x 8192: two ranges, 26.9 us against 38.3).
        const int rect = ntg::RECT_128 | ntg::RECT_192;
        const int edge1 = ntg::ring16_tile_edge(p.M, p.N, p.K, 1, rect);
        if (edge1 == 256) return none;                                // (larger problems fill the chip by themselves)
        const double whole_us = ntg::ring16_cost_us(edge1, ntg::ring16_tiles(edge1, p.M, p.N, 1), p.K);
        int64_t best = 1;
        double best_us = whole_us;
        for (int64_t sp = 2; sp <= 16; ++sp) {
            if (p.K % (sp * 32) != 0 || p.K / sp < 256) continue;
            const int edge = ntg::ring16_tile_edge(p.M, p.N, p.K / sp, sp, rect);
            const double us = ntg::ring16_cost_us(edge, ntg::ring16_tiles(edge, p.M, p.N, sp), p.K / sp) + 4.0 +
                              8.0 * (double)sp * (double)p.M * (double)p.N / 4.0e6;
            if (us < 0.95 * whole_us && us < best_us) { best = sp; best_us = us; }
        }
        if (best == 1) return none;
        return SplitPlan{(int)best, p.K / best, best * (int64_t)p.batch * p.M * p.N * 4};
    }
    // fp32 / fp64: their kernels go down to 64 x 64 tiles by themselves; a split pays only when those leave CUs without a
    // tile.  Same kind of estimate: a CU spends about 14.4 ns (fp32) / 28.8 ns (fp64) per k on each 64 x 64 tile it is
    // handed; the second pass costs about 5 us + the partial sums written and read at 4 TB/s.
    const int64_t tiles = ((p.M + 63) / 64) * ((p.N + 63) / 64);
    if (tiles > 255) return none;
    const double per_k = dtype == ntg::DT_F32 ? 0.0144 : 0.0288;
    auto estimate_us = [&](int64_t sp) {
        const double rounds = (double)((tiles * sp + 255) / 256);
        const double second_pass = sp == 1 ? 0.0 : 5.0 + 2.0 * (double)sp * (double)p.M * (double)p.N * (double)es / 4.0e6;
        return rounds * (double)(p.K / sp) * per_k + second_pass;
    };
    int64_t best = 1;
    double best_us = estimate_us(1);
    for (int64_t sp = 2; sp <= 16; ++sp) {
        if (p.K % (sp * 32) != 0 || p.K / sp < 64) continue;
        const double us = estimate_us(sp);
        if (us < 0.9 * best_us) { best = sp; best_us = us; }
    }
    if (best > 1) return SplitPlan{(int)best, p.K / best, best * (int64_t)p.batch * p.M * p.N * es};
    return none;
}

int run_gemm(ntg::GemmParams p, int dtype, bool ta, bool tb, hipStream_t s, void* workspace = nullptr, int64_t workspace_bytes = 0) {
    const int64_t es = ntg::elem_size(dtype);
    if (es == 0) return fail(NTG_ERR_UNSUPPORTED_DTYPE, "dtype %d is not supported by the gfx950 matmult backend", dtype);
    if (p.M == 0 || p.N == 0 || p.batch == 0) return NTG_OK;
    if (p.K == 0) {
        // empty sum: C keeps what it holds, or becomes the bias / zero.  The product kernels assume at least one k.
        if (p.cmode == ntg::C_ACCUMULATE && p.act == ntg::ACT_NONE) return NTG_OK;      // (with relu: C = relu_(C), below)
        if (p.Cptr) return fail(NTG_ERR_INVALID_ARGUMENT, "k = 0 with a C mode other than accumulate needs strided operands");
        hipError_t e = hipSuccess;
        if (is_int_dtype(dtype)) {
            e = ntg::launch_gemm_valu(dtype, ta, tb, p, s);                 // its k loop runs zero times
        } else if (is_complex_dtype(dtype)) {
            e = ntg::launch_gemm_complex(dtype, ta, tb, p, s);              // likewise
        } else {
            for (int b = 0; b < p.batch && e == hipSuccess; ++b) {
                ntg::GemmParams q = p;
                q.batch = 1;
                q.C = static_cast<char*>(p.C) + (int64_t)b * p.sC * es;
                if (p.bias) q.bias = static_cast<const char*>(p.bias) + (int64_t)b * p.bias_bs * es;
                e = ntg::launch_splitk_reduce(dtype, nullptr, 0, q, s);     // C0 plus no partial sums
            }
        }
        if (e != hipSuccess) return hip_fail(e, "empty-k launch");
        return NTG_OK;
    }
    if (int_planes_of(dtype)) {
        const IntPlanesPlan ip = plan_int_planes(p, dtype);
        if (ip.ok && workspace && workspace_bytes >= ip.bytes() && (reinterpret_cast<uintptr_t>(workspace) & 255) == 0)
            return run_int_planes(p, ip, ta, tb, workspace, s);
    }
    {
        const PadPlan pp = plan_pad(p, dtype, ta, tb);
        if (pp.ok && workspace && workspace_bytes >= pp.bytes() && (reinterpret_cast<uintptr_t>(workspace) & 255) == 0)
            return run_padded(p, pp, dtype, ta, tb, workspace, s);
    }
    const SplitPlan plan = plan_splitk(p, dtype, ta);
    if (plan.splits > 1 && workspace && workspace_bytes >= plan.bytes && (reinterpret_cast<uintptr_t>(workspace) & 15) == 0) {
        ntg::GemmParams q = p;
        q.K = (int)plan.kc;
        q.ldc = p.N;
        q.sC = (int64_t)p.M * p.N;
        q.cmode = (dtype == ntg::DT_F16 || dtype == ntg::DT_BF16) ? ntg::C_PARTIAL : ntg::C_OVERWRITE;
        q.bias = nullptr;
        q.act = ntg::ACT_NONE;                     // (the reduction applies it, after the last k range)
        const int64_t step_a = (ta ? plan.kc * p.lda : plan.kc), step_b = (tb ? plan.kc : plan.kc * p.ldb);   // elements from one k range to the next
        q.C = workspace;
        q.batch = plan.splits * p.batch;
        if (p.batch == 1) {
            // the k ranges are the items of one batched launch
            q.sA = step_a;
            q.sB = step_b;
        } else {
            // ... range r of item i is launch index r * batch + i
            q.krange_items = p.batch;
            q.sAk = step_a;
            q.sBk = step_b;
        }
        {
            int rc = launch_gemm(q, dtype, ta, tb, s);
            if (rc) return rc;
        }
        hipError_t e = ntg::launch_splitk_reduce(dtype, workspace, plan.splits, p, s);
        if (e != hipSuccess) return hip_fail(e, "split-K reduction launch");
        return NTG_OK;
    }
    return launch_gemm(p, dtype, ta, tb, s);
}

int check_sizes(int64_t m, int64_t k, int64_t n, int64_t batches) {
    if (m < 0 || k < 0 || n < 0 || batches < 0) return fail(NTG_ERR_INVALID_ARGUMENT, "negative size (m=%lld k=%lld n=%lld batches=%lld)", (long long)m, (long long)k, (long long)n, (long long)batches);
    if (m > 0x7fffffffLL || k > 0x7fffffffLL || n > 0x7fffffffLL || batches > 0x7fffffffLL)
        return fail(NTG_ERR_INVALID_ARGUMENT, "a size exceeds 2^31-1");
    return NTG_OK;
}

int desc_to_params(const ntg_gemm_desc* d, ntg::GemmParams& p) {
    if (!d) return fail(NTG_ERR_INVALID_ARGUMENT, "null descriptor");
    if (ntg::elem_size(d->dtype) == 0) return fail(NTG_ERR_UNSUPPORTED_DTYPE, "dtype %d is not supported", d->dtype);
    int rc = check_sizes(d->m, d->k, d->n, d->batches);
    if (rc) return rc;
    if (d->c_mode < 0 || d->c_mode > 2) return fail(NTG_ERR_INVALID_ARGUMENT, "c_mode %d is not one of overwrite/accumulate/bias", d->c_mode);
    std::memset(&p, 0, sizeof p);
    p.M = (int)d->m; p.K = (int)d->k; p.N = (int)d->n; p.batch = (int)d->batches;
    p.lda = d->lda ? d->lda : (d->transpose_a ? d->m : d->k);
    p.ldb = d->ldb ? d->ldb : (d->transpose_b ? d->k : d->n);
    p.ldc = d->ldc ? d->ldc : d->n;
    if (p.lda < (d->transpose_a ? d->m : d->k) || p.ldb < (d->transpose_b ? d->k : d->n) || p.ldc < d->n)
        return fail(NTG_ERR_INVALID_ARGUMENT, "leading dimension smaller than the stored row length");
    p.sA = d->stride_a; p.sB = d->stride_b; p.sC = d->stride_c;
    p.cmode = d->c_mode;
    p.bias = d->bias;
    p.bias_bs = d->bias_batch_stride; p.bias_rs = d->bias_row_stride; p.bias_cs = d->bias_col_stride;
    if (p.cmode == NTG_C_BIAS && !p.bias) return fail(NTG_ERR_INVALID_ARGUMENT, "c_mode is bias but bias is null");
    p.keep_k_order = (d->flags & NTG_GEMM_KEEP_K_ORDER) != 0;
    return NTG_OK;
}

}  // namespace

// Device address of `scratch` on the current device (each GPU holds its own copy at its own address), looked up on the
// first call per device.  The function has external linkage on purpose: the compiler gives a file-scope static device
// variable a symbol the runtime can look up only when a host function with external linkage refers to it.
namespace ntg {
// One per GPU: the address of its copy of `scratch`, and what orders the users of that copy.  Calls that use the array are
// enqueued one at a time (the mutex spans a call's whole sequence of launches); a call on another stream than the previous
// user's first makes its stream wait for the event recorded behind that user's last kernel.  Streams under capture take no
// part in this (an event recorded inside a capture cannot be waited for from outside): their callers order such calls themselves.
struct NoallocState {
    std::mutex mutex;
    void* ptr = nullptr;
    hipEvent_t done = nullptr;
    hipStream_t last_stream = nullptr;
    bool used = false;
};
int noalloc_state_of_current_device(NoallocState** out) {
    constexpr int kMaxDevices = 64;
    static std::mutex setup_mutex;
    static NoallocState states[kMaxDevices];
    int dev = -1;
    HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return fail(NTG_ERR_DEVICE, "device ordinal %d outside 0..%d", dev, kMaxDevices - 1);
    NoallocState& st = states[dev];
    std::lock_guard<std::mutex> lock(setup_mutex);
    if (!st.ptr) {
        void* ptr = nullptr;
        HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        if (!ptr) return fail(NTG_ERR_DEVICE, "hipGetSymbolAddress returned a null address for the static scratch");
        HIP_TRY(hipEventCreateWithFlags(&st.done, hipEventDisableTiming));
        st.ptr = ptr;
    }
    *out = &st;
    return NTG_OK;
}
}  // namespace ntg

extern "C" {

const char* ntg_last_error(void) { return g_last_error.c_str(); }
int ntg_version(void) { return 100; }
int64_t ntg_dtype_size(int dtype) { return ntg::elem_size(dtype); }

int ntg_release_host_buffers(void) {
    ntg::HostSession::release_all();
    return NTG_OK;
}

int ntg_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) return 0;
    return n;
}

int ntg_gemm_dev(const ntg_gemm_desc* d, const void* dA, const void* dB, void* dC, void* stream) {
    ntg::GemmParams p;
    int rc = desc_to_params(d, p);
    if (rc) return rc;
    if (p.M == 0 || p.N == 0 || p.batch == 0) return NTG_OK;
    if (!dA || !dB || !dC) return fail(NTG_ERR_INVALID_ARGUMENT, "null matrix pointer");
    if (p.batch > 1 && p.sC == 0) return fail(NTG_ERR_INVALID_ARGUMENT, "stride_c must be non-zero for a batch (outputs may not alias)");
    p.A = dA; p.B = dB; p.C = dC;
    return run_gemm(p, d->dtype, d->transpose_a != 0, d->transpose_b != 0, static_cast<hipStream_t>(stream), d->workspace, d->workspace_bytes);
}

int ntg_gemm_relu_dev(const ntg_gemm_desc* d, const void* dA, const void* dB, void* dC, void* stream) {
    ntg::GemmParams p;
    int rc = desc_to_params(d, p);
    if (rc) return rc;
    if (!(d->dtype == ntg::DT_F32 || d->dtype == ntg::DT_F64 || d->dtype == ntg::DT_F16 || d->dtype == ntg::DT_BF16))
        return fail(NTG_ERR_UNSUPPORTED_DTYPE, "ntg_gemm_relu_dev takes Float16, BFloat16, Float32 and Float64 (dtype %d)", d->dtype);
    if (p.M == 0 || p.N == 0 || p.batch == 0) return NTG_OK;
    if (!dC || (p.K > 0 && (!dA || !dB))) return fail(NTG_ERR_INVALID_ARGUMENT, "null matrix pointer");      // (k = 0: C = relu_(C0), no operands)
    if (p.batch > 1 && p.sC == 0) return fail(NTG_ERR_INVALID_ARGUMENT, "stride_c must be non-zero for a batch (outputs may not alias)");
    p.A = dA; p.B = dB; p.C = dC;
    p.act = ntg::ACT_RELU;
    return run_gemm(p, d->dtype, d->transpose_a != 0, d->transpose_b != 0, static_cast<hipStream_t>(stream), d->workspace, d->workspace_bytes);
}

int64_t ntg_gemm_workspace_bytes(const ntg_gemm_desc* d) {
    ntg::GemmParams p;
    if (desc_to_params(d, p)) return -1;
    if (p.M == 0 || p.N == 0 || p.batch == 0) return 0;
    if (int_planes_of(d->dtype)) {
        const IntPlanesPlan ip = plan_int_planes(p, d->dtype);
        return ip.ok ? ip.bytes() : 0;
    }
    {
        const PadPlan pp = plan_pad(p, d->dtype, d->transpose_a != 0, d->transpose_b != 0);      // pointers taken as 16-byte aligned
        if (pp.ok) return pp.bytes();
    }
    return plan_splitk(p, d->dtype, d->transpose_a != 0).bytes;      // pointers taken as 16-byte aligned
}

int ntg_gemm_noalloc_dev(const ntg_gemm_desc* d, const void* dA, const void* dB, void* dC, void* stream) {
    ntg::GemmParams p;
    int rc = desc_to_params(d, p);
    if (rc) return rc;
    if (p.M == 0 || p.N == 0 || p.batch == 0) return NTG_OK;
    if (!dA || !dB || !dC) return fail(NTG_ERR_INVALID_ARGUMENT, "null matrix pointer");
    if (p.batch > 1 && p.sC == 0) return fail(NTG_ERR_INVALID_ARGUMENT, "stride_c must be non-zero for a batch (outputs may not alias)");
    const int64_t need = ntg_gemm_workspace_bytes(d);
    if (need < 0) return fail(NTG_ERR_INVALID_ARGUMENT, "bad descriptor");
    if (need > (int64_t)NTG_NOALLOC_SCRATCH_BYTES)
        return fail(NTG_ERR_INVALID_ARGUMENT, "this product's workspace form needs %lld bytes, the static scratch of ntg_gemm_noalloc_dev holds %lld: "
                    "call ntg_gemm_dev with a workspace of the caller's, or ntg_gemm_dev without a workspace (the plain kernels: they allocate "
                    "nothing either, but a split along k is then not taken and floating-point sums may differ in their last bits)",
                    (long long)need, (long long)NTG_NOALLOC_SCRATCH_BYTES);
    p.A = dA; p.B = dB; p.C = dC;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (need == 0) return run_gemm(p, d->dtype, d->transpose_a != 0, d->transpose_b != 0, s);      // the plain kernels: the array is not used
    ntg::NoallocState* st = nullptr;
    rc = ntg::noalloc_state_of_current_device(&st);
    if (rc) return rc;
    std::lock_guard<std::mutex> lock(st->mutex);
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &capture) != hipSuccess) {      // (e.g. the default stream while another stream captures)
        (void)hipGetLastError();
        capture = hipStreamCaptureStatusActive;
    }
    const bool ordered = capture == hipStreamCaptureStatusNone;
    if (ordered && st->used && st->last_stream != s) HIP_TRY(hipStreamWaitEvent(s, st->done, 0));     // the previous user of the array finishes first
    rc = run_gemm(p, d->dtype, d->transpose_a != 0, d->transpose_b != 0, s, st->ptr, need);
    if (ordered) {
        HIP_TRY(hipEventRecord(st->done, s));
        st->last_stream = s;
        st->used = true;
    }
    return rc;
}

// Address of the current device's copy of gate_flags (looked up once per device) and the next slot of it.
static int next_gate_slot(int** out) {
    constexpr int kMaxDevices = 64;
    static std::mutex mutex;
    static int* base[kMaxDevices];
    static unsigned next[kMaxDevices];
    int dev = -1;
    HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return fail(NTG_ERR_DEVICE, "device ordinal %d outside 0..%d", dev, kMaxDevices - 1);
    std::lock_guard<std::mutex> lock(mutex);
    if (!base[dev]) {
        void* ptr = nullptr;
        HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(gate_flags)));
        if (!ptr) return fail(NTG_ERR_DEVICE, "hipGetSymbolAddress returned a null address for the gate flags");
        base[dev] = static_cast<int*>(ptr);
    }
    *out = base[dev] + (next[dev]++ % NTG_GATE_SLOTS);
    return NTG_OK;
}

// Pointer tables without the caller's vouch: the entries' alignment is a fact of device memory, so it is found out there.  A
// one-workgroup kernel ORs the low bits of all entries into a flag; then the product is launched twice, on the DMA-fed
// kernel (which needs 16-byte entries) and on the register-staged one (which does not), each returning at once unless the
// flag names it.  The two kernels give the same bits, so nothing depends on which one runs.  Worth two extra launches
// (about 4 us) only for products that take a few times that; the floating types that have both kernels, more than 32 rows.
static bool gated_tables_pay(const ntg::GemmParams& p, int dtype) {
    const bool byte = dtype == ntg::DT_I8 || dtype == ntg::DT_U8;
    if (dtype != ntg::DT_F32 && dtype != ntg::DT_F64 && dtype != ntg::DT_F16 && dtype != ntg::DT_BF16 && !byte) return false;
    if (p.M <= 32 || p.K <= 0 || p.act != ntg::ACT_NONE) return false;
    const double flops = 2.0 * (double)p.M * (double)p.N * (double)p.K * (double)p.batch;
    // (8-bit: the kernel that needs no alignment is the vector ALU's, 40 x slower: the check pays almost at once)
    return flops >= (byte ? 1.0e9 : dtype == ntg::DT_F32 || dtype == ntg::DT_F64 ? 3.2e10 : 8.0e9);
}
static int launch_gemm_tables_gated(ntg::GemmParams p, int dtype, bool ta, bool tb, hipStream_t s) {
    int* flag = nullptr;
    int rc = next_gate_slot(&flag);
    if (rc) return rc;
    hipLaunchKernelGGL(ntg::ptr_tables_aligned_kernel, dim3(1), dim3(256), 0, s, p.Aptr, p.Bptr, p.Cptr, p.batch, flag);
    HIP_TRY(hipGetLastError());
    const int64_t ve = 16 / ntg::elem_size(dtype);
    ntg::GemmParams q = p;
    q.vecA_ok = p.lda % ve == 0;
    q.vecB_ok = p.ldb % ve == 0;
    q.ptrs_aligned = 1; q.gate = flag; q.gate_want = 1;
    bool taken = false;
    hipError_t e = ntg::launch_gemm_ring_only(dtype, ta, tb, q, s, &taken);
    if (e != hipSuccess) return hip_fail(e, "gemm launch");
    p.ptrs_aligned = 0;
    if (taken) { p.gate = flag; p.gate_want = 0; }        // (not taken: sizes or pitches rule the DMA-fed kernel out anyway)
    return launch_gemm(p, dtype, ta, tb, s);
}

// aligned: the caller vouches that every table entry is a multiple of 16 bytes (true for the host entry points' own arena)
static int gemm_ptrs(const ntg_gemm_desc* d, const void* const* dA, const void* const* dB, void* const* dC, void* stream, bool aligned) {
    ntg::GemmParams p;
    int rc = desc_to_params(d, p);
    if (rc) return rc;
    if (p.M == 0 || p.N == 0 || p.batch == 0) return NTG_OK;
    if (!dA || !dB || !dC) return fail(NTG_ERR_INVALID_ARGUMENT, "null pointer table");
    p.Aptr = dA; p.Bptr = dB; p.Cptr = dC;
    p.ptrs_aligned = aligned ? 1 : 0;
    if (!aligned && gated_tables_pay(p, d->dtype))
        return launch_gemm_tables_gated(p, d->dtype, d->transpose_a != 0, d->transpose_b != 0, static_cast<hipStream_t>(stream));
    return run_gemm(p, d->dtype, d->transpose_a != 0, d->transpose_b != 0, static_cast<hipStream_t>(stream));
}

int ntg_gemm_ptrs_dev(const ntg_gemm_desc* d, const void* const* dA, const void* const* dB, void* const* dC, void* stream) {
    // (the tables are in device memory: their entries' alignment is what the caller says it is)
    return gemm_ptrs(d, dA, dB, dC, stream, d && (d->flags & NTG_GEMM_PTRS_ALIGNED16) != 0);
}

// The host-pointer entry points are the reference's own seam (nt_matmult / nt_matmult_batch / cpu::linear on host memory): there a
// Float32 product keeps the reference's order of summation -- no split along k, whose gain the transfers would hide anyway.
static int64_t host_entry_flags(int dtype) { return dtype == ntg::DT_F32 ? NTG_GEMM_KEEP_K_ORDER : 0; }

int ntg_matmult_dev(int dtype, const void* dA, const void* dB, void* dC, int64_t m, int64_t k, int64_t n,
                    int transpose_a, int transpose_b, void* stream) {
    ntg_gemm_desc d;
    std::memset(&d, 0, sizeof d);
    d.dtype = dtype; d.transpose_a = transpose_a; d.transpose_b = transpose_b; d.c_mode = NTG_C_ACCUMULATE;
    d.m = m; d.k = k; d.n = n; d.batches = 1;
    return ntg_gemm_dev(&d, dA, dB, dC, stream);
}

int ntg_matmult(int dtype, const void* A, const void* B, void* C,
                int64_t a_rows, int64_t a_cols, int64_t b_rows, int64_t b_cols,
                int transpose_a, int transpose_b) {
    const void* As[1] = {A};
    const void* Bs[1] = {B};
    void* Cs[1] = {C};
    return ntg_matmult_batch(dtype, As, Bs, Cs, 1, a_rows, a_cols, b_rows, b_cols, transpose_a, transpose_b);
}

// The host-pointer seam, pipelined: large operands cross the link in panels so that uploads, products and downloads
// overlap (the link is full duplex and the kernel is short beside the transfers).
//   one product:  B first (and A whole when it is stored [k][m]), then panels of rows: A's rows and C's rows up, the
//                 panel's product on a second stream, its rows of C down on a third while the next panels go up;
//   a batch of distinct matrices (or one shared A or B): the same with groups of items as panels.
// A C that is all zeros in the caller's memory (what functional::matmult hands over: zeros, then accumulate,
// matmult_cpu.cpp:110, :707) is not uploaded; the products overwrite instead, which gives the same bits (the sums start
// from +0 either way).  Panels are products of their own, so this form is taken only where that cannot change a bit: no
// workspace form exists for the whole product (a split along k would depend on the panel's rows), more than 32 rows.
// Returns -1 when the call is not one for this form (nothing has been done then).
static int matmult_host_pipelined(int dtype, const void* const* A, const void* const* B, void* const* C, int64_t batches,
                                  int64_t m, int64_t k, int64_t n, int ta, int tb) {
    const int64_t es = ntg::elem_size(dtype);
    const size_t a_bytes = (size_t)(m * k * es), b_bytes = (size_t)(k * n * es), c_bytes = (size_t)(m * n * es);
    if ((a_bytes + b_bytes + c_bytes) * (size_t)batches < ((size_t)48 << 20)) return -1;
    ntg_gemm_desc d;
    std::memset(&d, 0, sizeof d);
    d.dtype = dtype; d.transpose_a = ta; d.transpose_b = tb;
    d.m = m; d.k = k; d.n = n; d.batches = 1;
    d.flags = host_entry_flags(dtype);
    const size_t a_slot = align_up(a_bytes, 256), b_slot = align_up(b_bytes, 256), c_slot = align_up(c_bytes, 256);
    std::vector<ntg::HostSession::Range> up;
    if (batches == 1) {
        if (m < 1024 || ntg_gemm_workspace_bytes(&d) != 0) return -1;
        // rows per panel: multiples of 256, about 16 MiB of A and C rows together, at least four panels
        int64_t rows = (int64_t)(((size_t)16 << 20) / (size_t)((k + n) * es)) / 256 * 256;
        rows = std::max<int64_t>(256, std::min<int64_t>(rows, (m / 4) / 256 * 256));
        // (the rows that are left over join the last panel: a panel of 32 rows or fewer would run on the streaming kernel,
        //  whose sums over k have another order)
        const int panels = (int)std::max<int64_t>(1, m / rows);
        auto panel_rows = [&](int p) { return p == panels - 1 ? m - (int64_t)p * rows : rows; };
        ntg::HostSession mem;
        HIP_TRY(mem.reserve(a_slot + b_slot + c_slot));

        const size_t oa = 0, ob = a_slot, oc = a_slot + b_slot;
        // B (and an A stored [k][m]: a panel of rows of op(A) is a column block of the stored matrix) go first; C is looked
        // at while the stagers are busy with them
        up.push_back({ob, B[0], b_bytes, 0});
        if (ta) up.push_back({oa, A[0], a_bytes, 0});
        HIP_TRY(mem.begin_uploads(up.data(), up.size(), 1));
        const bool zero = ntg::HostSession::all_zero(C[0], c_bytes);
        HIP_TRY(mem.end_uploads());
        up.clear();
        for (int p = 0; p < panels; ++p) {
            const int64_t m0 = p * rows, mr = panel_rows(p);
            if (!ta) up.push_back({oa + (size_t)(m0 * k * es), static_cast<const char*>(A[0]) + m0 * k * es, (size_t)(mr * k * es), p});
            if (!zero) up.push_back({oc + (size_t)(m0 * n * es), static_cast<const char*>(C[0]) + m0 * n * es, (size_t)(mr * n * es), p});
        }
        HIP_TRY(mem.begin_uploads(up.data(), up.size(), panels));
        d.lda = ta ? m : k;
        d.c_mode = zero ? NTG_C_OVERWRITE : NTG_C_ACCUMULATE;
        for (int p = 0; p < panels; ++p) {
            const int64_t m0 = p * rows, mr = panel_rows(p);
            const size_t c_off = (size_t)(m0 * n * es);
            HIP_TRY(mem.uploaded_through(p));
            d.m = mr;
            const int rc = ntg_gemm_dev(&d, mem.at(oa + (size_t)((ta ? m0 : m0 * k) * es)), mem.at(ob), mem.at(oc + c_off), mem.compute_stream());
            if (rc) return rc;
            HIP_TRY(mem.download_async(static_cast<char*>(C[0]) + c_off, oc + c_off, (size_t)(mr * n * es), mem.compute_stream()));
        }
        HIP_TRY(mem.end_uploads());
        HIP_TRY(mem.finish_downloads());
        return NTG_OK;
    }
    // a batch: distinct A, B, C per item, or one B (or one A) for all
    if (m <= 32) return -1;
    bool a_same = true, b_same = true;
    for (int64_t i = 1; i < batches; ++i) { a_same = a_same && A[i] == A[0]; b_same = b_same && B[i] == B[0]; }
    {
        std::map<const void*, int64_t> seen;
        for (int64_t i = 0; i < batches && !a_same; ++i)
            if (!seen.emplace(A[i], i).second) return -1;
        seen.clear();
        for (int64_t i = 0; i < batches && !b_same; ++i)
            if (!seen.emplace(B[i], i).second) return -1;
        seen.clear();
        for (int64_t i = 0; i < batches; ++i)
            if (!seen.emplace(C[i], i).second) return -1;          // (aliasing outputs: the general path reports it)
    }
    const size_t per_item = (a_same ? 0 : a_bytes) + (b_same ? 0 : b_bytes) + c_bytes;
    int64_t group = std::max<int64_t>(1, (int64_t)(((size_t)24 << 20) / per_item));
    group = std::min(group, std::max<int64_t>(1, batches / 4));
    const int panels = (int)((batches + group - 1) / group);
    d.batches = group;
    d.stride_a = a_same ? 0 : (int64_t)(a_slot / (size_t)es);
    d.stride_b = b_same ? 0 : (int64_t)(b_slot / (size_t)es);
    d.stride_c = (int64_t)(c_slot / (size_t)es);
    if (a_slot % (size_t)es || b_slot % (size_t)es || c_slot % (size_t)es) return -1;
    const int64_t ws_bytes = ntg_gemm_workspace_bytes(&d);          // (planned per item: the same form for any group size)
    if (ws_bytes < 0) return -1;
    const size_t na = a_same ? 1 : (size_t)batches, nb = b_same ? 1 : (size_t)batches;
    const size_t oa = 0, ob = na * a_slot, oc = ob + nb * b_slot, ow = oc + (size_t)batches * c_slot;
    ntg::HostSession mem;
    HIP_TRY(mem.reserve(ow + (size_t)ws_bytes));
    // the shared operand and the first group's A and B go first; the outputs are looked at while the stagers are busy with them
    if (a_same) up.push_back({oa, A[0], a_bytes, 0});
    if (b_same) up.push_back({ob, B[0], b_bytes, 0});
    for (int64_t i = 0; i < std::min(group, batches); ++i) {
        if (!a_same) up.push_back({oa + (size_t)i * a_slot, A[i], a_bytes, 0});
        if (!b_same) up.push_back({ob + (size_t)i * b_slot, B[i], b_bytes, 0});
    }
    HIP_TRY(mem.begin_uploads(up.data(), up.size(), 1));
    bool zero = true;
    for (int64_t i = 0; i < batches && zero; ++i) zero = ntg::HostSession::all_zero(C[i], c_bytes);
    HIP_TRY(mem.end_uploads());
    up.clear();
    for (int64_t i = 0; i < batches; ++i) {
        const int p = (int)(i / group);
        if (!a_same && p > 0) up.push_back({oa + (size_t)i * a_slot, A[i], a_bytes, p});
        if (!b_same && p > 0) up.push_back({ob + (size_t)i * b_slot, B[i], b_bytes, p});
        if (!zero) up.push_back({oc + (size_t)i * c_slot, C[i], c_bytes, p});
    }
    HIP_TRY(mem.begin_uploads(up.data(), up.size(), panels));
    if (ws_bytes > 0) { d.workspace = mem.at(ow); d.workspace_bytes = ws_bytes; }
    d.c_mode = zero ? NTG_C_OVERWRITE : NTG_C_ACCUMULATE;
    for (int p = 0; p < panels; ++p) {
        const int64_t i0 = p * group, cnt = std::min(group, batches - i0);
        HIP_TRY(mem.uploaded_through(p));
        d.batches = cnt;
        const int rc = ntg_gemm_dev(&d, mem.at(oa + (a_same ? 0 : (size_t)i0 * a_slot)), mem.at(ob + (b_same ? 0 : (size_t)i0 * b_slot)),
                                    mem.at(oc + (size_t)i0 * c_slot), mem.compute_stream());
        if (rc) return rc;
        for (int64_t i = i0; i < i0 + cnt; ++i) HIP_TRY(mem.download_async(C[i], oc + (size_t)i * c_slot, c_bytes, mem.compute_stream()));
    }
    HIP_TRY(mem.end_uploads());
    HIP_TRY(mem.finish_downloads());
    return NTG_OK;
}

int ntg_matmult_batch(int dtype, const void* const* A, const void* const* B, void* const* C,
                      int64_t batches, int64_t a_rows, int64_t a_cols, int64_t b_rows, int64_t b_cols,
                      int transpose_a, int transpose_b) {
    const int64_t es = ntg::elem_size(dtype);
    if (es == 0) return fail(NTG_ERR_UNSUPPORTED_DTYPE, "dtype %d is not supported by the gfx950 matmult backend", dtype);
    if (a_cols != b_rows) return fail(NTG_ERR_INVALID_ARGUMENT, "inner sizes differ: a_cols=%lld b_rows=%lld", (long long)a_cols, (long long)b_rows);
    const int64_t m = a_rows, k = a_cols, n = b_cols;
    int rc = check_sizes(m, k, n, batches);
    if (rc) return rc;
    if (batches == 0 || m == 0 || n == 0 || k == 0) return NTG_OK;   // C += empty sum
    if (!A || !B || !C) return fail(NTG_ERR_INVALID_ARGUMENT, "null pointer array");
    for (int64_t i = 0; i < batches; ++i)
        if (!A[i] || !B[i] || !C[i]) return fail(NTG_ERR_INVALID_ARGUMENT, "null matrix pointer in item %lld", (long long)i);
    rc = matmult_host_pipelined(dtype, A, B, C, batches, m, k, n, transpose_a, transpose_b);
    if (rc >= 0) return rc;
    rc = NTG_OK;

    const size_t a_bytes = (size_t)(m * k * es), b_bytes = (size_t)(k * n * es), c_bytes = (size_t)(m * n * es);
    // every distinct input matrix gets one slot in a single device arena
    std::map<const void*, size_t> slotA, slotB;
    size_t off = 0;
    for (int64_t i = 0; i < batches; ++i)
        if (slotA.emplace(A[i], off).second) off += align_up(a_bytes, 256);
    for (int64_t i = 0; i < batches; ++i)
        if (slotB.emplace(B[i], off).second) off += align_up(b_bytes, 256);
    const size_t c_off = off;
    off += align_up(c_bytes, 256) * (size_t)batches;
    const size_t tab_off = off;
    off += align_up(3 * sizeof(void*) * (size_t)batches, 256);
    ntg_gemm_desc d;
    std::memset(&d, 0, sizeof d);
    d.dtype = dtype; d.transpose_a = transpose_a; d.transpose_b = transpose_b; d.c_mode = NTG_C_ACCUMULATE;
    d.m = m; d.k = k; d.n = n; d.batches = batches;
    d.flags = host_entry_flags(dtype);
    // The arena is this function's own: when every item's A (and B) is a new matrix, or all items share one, the slots
    // lie at a constant stride and the strided kernels (and their workspace forms) serve the batch; any other pattern of
    // repeated pointers goes through the pointer tables.
    auto constant_stride = [&](const std::map<const void*, size_t>& slot, const void* const* P, size_t bytes, int64_t& stride) {
        const size_t step = slot.size() == 1 ? 0 : align_up(bytes, 256);
        for (int64_t i = 0; i < batches; ++i)
            if (slot.at(P[i]) != slot.at(P[0]) + (size_t)i * step) return false;
        stride = (int64_t)(step / (size_t)es);
        return true;
    };
    const bool strided = constant_stride(slotA, A, a_bytes, d.stride_a) && constant_stride(slotB, B, b_bytes, d.stride_b);
    if (strided) d.stride_c = (int64_t)(align_up(c_bytes, 256) / (size_t)es);
    else d.stride_a = d.stride_b = 0;
    const size_t ws_off = off;
    int64_t ws_bytes = strided ? ntg_gemm_workspace_bytes(&d) : 0;
    // A pattern of repeated pointers runs as ONE table batch, which has no workspace form.  Where an item on its own would
    // be given one that changes the order of summation over k (a split), the items go out one by one in that form instead,
    // so that an item comes out bit for bit the same alone and in any batch (tests/src/matmult_test.cpp:108-189).
    bool per_item = false;
    if (!strided) {
        ntg_gemm_desc one = d;
        one.batches = 1;
        const int64_t wb = ntg_gemm_workspace_bytes(&one);
        if (wb > 0) { per_item = true; ws_bytes = wb; }
    }
    if (ws_bytes > 0) off += (size_t)ws_bytes;

    ntg::HostSession mem;
    HIP_TRY(mem.reserve(off));
    for (auto& kv : slotA) HIP_TRY(mem.upload(kv.second, kv.first, a_bytes));
    for (auto& kv : slotB) HIP_TRY(mem.upload(kv.second, kv.first, b_bytes));
    std::vector<void*> tab(3 * (size_t)batches);
    std::map<const void*, int64_t> seenC;
    for (int64_t i = 0; i < batches; ++i) {
        const auto ins = seenC.emplace(C[i], i);
        if (!ins.second) return fail(NTG_ERR_INVALID_ARGUMENT, "output pointers of items %lld and %lld alias", (long long)ins.first->second, (long long)i);
        const size_t dc_off = c_off + (size_t)i * align_up(c_bytes, 256);
        HIP_TRY(mem.upload(dc_off, C[i], c_bytes));   // accumulate contract: C is an input too
        tab[(size_t)i] = mem.at(slotA[A[i]]);
        tab[(size_t)(batches + i)] = mem.at(slotB[B[i]]);
        tab[(size_t)(2 * batches + i)] = mem.at(dc_off);
    }
    void** dtab = reinterpret_cast<void**>(mem.at(tab_off));
    if (ws_bytes > 0) { d.workspace = mem.at(ws_off); d.workspace_bytes = ws_bytes; }
    if (strided) {
        rc = ntg_gemm_dev(&d, tab[0], tab[(size_t)batches], tab[(size_t)(2 * batches)], mem.stream());
    } else if (per_item) {
        d.batches = 1;
        for (int64_t i = 0; i < batches && rc == NTG_OK; ++i)
            rc = ntg_gemm_dev(&d, tab[(size_t)i], tab[(size_t)(batches + i)], tab[(size_t)(2 * batches + i)], mem.stream());
    } else {
        HIP_TRY(mem.upload(tab_off, tab.data(), tab.size() * sizeof(void*)));
        rc = gemm_ptrs(&d, dtab, dtab + batches, dtab + 2 * batches, mem.stream(), true);     // (every slot of the arena is 256-byte aligned)
    }
    if (rc) return rc;
    for (int64_t i = 0; i < batches; ++i)
        HIP_TRY(mem.download(C[i], c_off + (size_t)i * align_up(c_bytes, 256), c_bytes));
    return NTG_OK;
}

int ntg_linear(int dtype, const void* X, const void* W, const void* bias, void* Y,
               int64_t m, int64_t k, int64_t n, int transpose_x, int transpose_w,
               int64_t bias_rows, int64_t bias_cols) {
    const int64_t es = ntg::elem_size(dtype);
    if (es == 0) return fail(NTG_ERR_UNSUPPORTED_DTYPE, "dtype %d is not supported by the gfx950 matmult backend", dtype);
    int rc = check_sizes(m, k, n, 1);
    if (rc) return rc;
    if ((bias_rows != 1 && bias_rows != m) || (bias_cols != 1 && bias_cols != n))
        return fail(NTG_ERR_INVALID_ARGUMENT, "bias shape [%lld, %lld] does not broadcast to [%lld, %lld]",
                    (long long)bias_rows, (long long)bias_cols, (long long)m, (long long)n);
    if (m == 0 || n == 0) return NTG_OK;
    if (!X || !W || !bias || !Y) return fail(NTG_ERR_INVALID_ARGUMENT, "null pointer");
    const size_t x_bytes = (size_t)(m * k * es), w_bytes = (size_t)(k * n * es), y_bytes = (size_t)(m * n * es);
    const size_t bias_bytes = (size_t)(bias_rows * bias_cols * es);
    ntg::HostSession mem;
    const size_t ox = 0, ow = align_up(x_bytes, 256), ob = ow + align_up(w_bytes, 256), oy = ob + align_up(bias_bytes, 256);
    HIP_TRY(mem.reserve(oy + y_bytes));
    if (x_bytes) HIP_TRY(mem.upload(ox, X, x_bytes));
    if (w_bytes) HIP_TRY(mem.upload(ow, W, w_bytes));
    HIP_TRY(mem.upload(ob, bias, bias_bytes));
    ntg_gemm_desc d;
    std::memset(&d, 0, sizeof d);
    d.dtype = dtype; d.transpose_a = transpose_x; d.transpose_b = transpose_w; d.c_mode = NTG_C_BIAS;
    d.m = m; d.k = k; d.n = n; d.batches = 1;
    d.flags = host_entry_flags(dtype);
    d.bias = mem.at(ob);
    d.bias_row_stride = (bias_rows == 1) ? 0 : bias_cols;
    d.bias_col_stride = (bias_cols == 1) ? 0 : 1;
    rc = ntg_gemm_dev(&d, mem.at(ox), mem.at(ow), mem.at(oy), mem.stream());
    if (rc) return rc;
    HIP_TRY(mem.download(Y, oy, y_bytes));
    return NTG_OK;
}

static int unfold_out(int64_t height, int64_t width, int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c,
                      int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c, int64_t& Ho, int64_t& Wo) {
    if (k_r < 1 || k_c < 1 || s_r < 1 || s_c < 1 || d_r < 1 || d_c < 1 || p_r < 0 || p_c < 0)
        return fail(NTG_ERR_INVALID_ARGUMENT, "kernel/stride/dilation must be >= 1 and padding >= 0");
    Ho = (height + 2 * p_r - d_r * (k_r - 1) - 1) / s_r + 1;
    Wo = (width + 2 * p_c - d_c * (k_c - 1) - 1) / s_c + 1;
    if (height + 2 * p_r - d_r * (k_r - 1) - 1 < 0 || width + 2 * p_c - d_c * (k_c - 1) - 1 < 0 || Ho <= 0 || Wo <= 0)
        return fail(NTG_ERR_INVALID_ARGUMENT, "the array of sliding blocks would be empty (Ho=%lld, Wo=%lld)", (long long)Ho, (long long)Wo);
    return NTG_OK;
}

int ntg_unfold2d_dev(int dtype, const void* image, void* col,
                     int64_t batch, int64_t channels, int64_t height, int64_t width,
                     int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c,
                     int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c, void* stream) {
    const int64_t es = ntg::elem_size(dtype);
    if (es == 0) return fail(NTG_ERR_UNSUPPORTED_DTYPE, "dtype %d is not supported", dtype);
    if (batch < 0 || channels < 0 || height < 0 || width < 0) return fail(NTG_ERR_INVALID_ARGUMENT, "negative size");
    int64_t Ho, Wo;
    int rc = unfold_out(height, width, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, Ho, Wo);
    if (rc) return rc;
    if (batch == 0 || channels == 0) return NTG_OK;
    if (!image || !col) return fail(NTG_ERR_INVALID_ARGUMENT, "null pointer");
    hipError_t e = ntg::launch_unfold2d(es, image, col, batch, channels, height, width, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c,
                                        static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(e, "unfold2d launch");
    return NTG_OK;
}

int ntg_unfold2d(int dtype, const void* image, void* col,
                 int64_t batch, int64_t channels, int64_t height, int64_t width,
                 int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c,
                 int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c) {
    const int64_t es = ntg::elem_size(dtype);
    if (es == 0) return fail(NTG_ERR_UNSUPPORTED_DTYPE, "dtype %d is not supported", dtype);
    int64_t Ho, Wo;
    int rc = unfold_out(height, width, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, Ho, Wo);
    if (rc) return rc;
    if (batch <= 0 || channels <= 0) return batch < 0 || channels < 0 ? fail(NTG_ERR_INVALID_ARGUMENT, "negative size") : NTG_OK;
    if (!image || !col) return fail(NTG_ERR_INVALID_ARGUMENT, "null pointer");
    const size_t im_bytes = (size_t)(batch * channels * height * width * es);
    const size_t col_bytes = (size_t)(batch * channels * k_r * k_c * Ho * Wo * es);
    ntg::HostSession mem;
    const size_t oc = align_up(im_bytes, 256);
    HIP_TRY(mem.reserve(oc + col_bytes));
    HIP_TRY(mem.upload(0, image, im_bytes));
    rc = ntg_unfold2d_dev(dtype, mem.at(0), mem.at(oc), batch, channels, height, width, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, mem.stream());
    if (rc) return rc;
    HIP_TRY(mem.download(col, oc, col_bytes));
    return NTG_OK;
}

// Geometry of a convolution over two or three spatial axes; axis 0 is the depth (size 1, one tap for two axes).
struct Geo3 {
    int nd;
    int64_t sz[3], k[3], s[3], p[3], d[3], o[3];
    int64_t vol() const { return sz[0] * sz[1] * sz[2]; }
    int64_t taps() const { return k[0] * k[1] * k[2]; }
    int64_t L() const { return o[0] * o[1] * o[2]; }
};

static Geo3 geo2(int64_t height, int64_t width, int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c, int64_t p_r, int64_t p_c,
                 int64_t d_r, int64_t d_c, int64_t Ho, int64_t Wo) {
    return Geo3{2, {1, height, width}, {1, k_r, k_c}, {1, s_r, s_c}, {0, p_r, p_c}, {1, d_r, d_c}, {1, Ho, Wo}};
}

// The geometry of the convolution that maps the output gradient back to the image (all strides 1): its "image" is the
// gradient, its outputs are the image elements, its padding is d*(k-1) - p (negative = the image is cropped).
static Geo3 geo_dimage(const Geo3& g) {
    Geo3 t = g;
    for (int a = 0; a < 3; ++a) {
        t.sz[a] = g.o[a]; t.o[a] = g.sz[a]; t.s[a] = 1;
        t.p[a] = g.d[a] * (g.k[a] - 1) - g.p[a];
    }
    return t;
}

// The floating dtypes gather the im2col operand inside the GEMM (no col buffer) when every index the kernel forms fits
// 32 bits with room for its out-of-range sentinels and the kernel has at most 8 taps per axis (one byte of tap mask).
static bool conv_implicit_g(int dtype, int64_t channels, const Geo3& g) {
    if (is_valu_dtype(dtype)) return false;
    const int64_t lim = 1 << 24;
    for (int a = 0; a < 3; ++a) {
        if (g.k[a] > 8) return false;
        if (g.sz[a] >= lim || g.s[a] >= lim || g.p[a] >= lim || g.p[a] <= -lim) return false;
        if (g.k[a] * g.d[a] >= lim || g.o[a] * g.s[a] >= lim) return false;
    }
    if (channels >= lim || g.taps() >= lim) return false;
    // byte offsets inside one image are formed in 32 bits
    if (channels * g.vol() * ntg::elem_size(dtype) >= 0x7fffffffLL || channels * g.taps() >= 0x7fffffffLL || g.L() >= 0x7fffffffLL) return false;
    return channels * g.vol() > 0;
}

static bool conv_implicit(int dtype, int64_t channels, int64_t height, int64_t width, int64_t k_r, int64_t k_c,
                          int64_t s_r, int64_t s_c, int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c, int64_t Ho, int64_t Wo) {
    return conv_implicit_g(dtype, channels, geo2(height, width, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, Ho, Wo));
}

static void fill_conv_geom(ntg::ConvGeom& c, int64_t slice_channels, const Geo3& g) {
    c.D = (int)g.sz[0]; c.H = (int)g.sz[1]; c.W = (int)g.sz[2]; c.chan = (int)g.vol();
    c.s_d = (int)g.s[0]; c.s_r = (int)g.s[1]; c.s_c = (int)g.s[2];
    c.p_d = (int)g.p[0]; c.p_r = (int)g.p[1]; c.p_c = (int)g.p[2];
    c.d_d = (int)g.d[0]; c.d_r = (int)g.d[1]; c.d_c = (int)g.d[2];
    c.k_d = (int)g.k[0]; c.k_r = (int)g.k[1]; c.k_c = (int)g.k[2];
    c.k_rc = (int)(g.k[1] * g.k[2]); c.k_drc = (int)g.taps();
    c.Wo = (int)g.o[2]; c.HoWo = (int)(g.o[1] * g.o[2]);
    c.last = (int)(slice_channels * g.vol() - 1);
    c.div_kdrc = ntg::make_fastdiv((uint32_t)c.k_drc);
    c.div_krc = ntg::make_fastdiv((uint32_t)c.k_rc);
    c.div_kc = ntg::make_fastdiv((uint32_t)c.k_c);
    c.div_wo = ntg::make_fastdiv((uint32_t)c.Wo);
    c.div_howo = ntg::make_fastdiv((uint32_t)c.HoWo);
}

// out_b[g*og:(g+1)*og, L] = W_g[og, add] . col_b[g*add:(g+1)*add, L] with col_b gathered from the image by the B loader.
// The reference forms (col_b^T . W_g^T) and swaps rows/columns afterwards (conv.cpp:94, :143); each output element is the
// same ascending-k sum of the same products.
static int conv_forward_gather(int dtype, const void* image, const void* kernel, void* out, int64_t batch, int64_t channels,
                               int64_t out_channels, const Geo3& g, int64_t groups, hipStream_t hs) {
    const int64_t es = ntg::elem_size(dtype), cg = channels / groups, og = out_channels / groups;
    const int64_t L = g.L(), add = cg * g.taps(), vol = g.vol();
    for (int64_t gi = 0; gi < groups; ++gi) {
        ntg::GemmParams p;
        std::memset(&p, 0, sizeof p);
        p.M = (int)og; p.K = (int)add; p.N = (int)L; p.batch = (int)batch;
        p.A = static_cast<const char*>(kernel) + gi * og * add * es;
        p.B = static_cast<const char*>(image) + gi * cg * vol * es;
        p.C = static_cast<char*>(out) + gi * og * L * es;
        p.lda = add; p.ldb = L; p.ldc = L;
        p.sA = 0; p.sB = channels * vol; p.sC = out_channels * L;
        p.cmode = ntg::C_OVERWRITE;
        p.vecA_ok = (add * es) % 16 == 0;
        fill_conv_geom(p.conv, cg, g);
        hipError_t e = ntg::launch_conv_mfma(dtype, false, g.nd, p, hs);
        if (e != hipSuccess) return hip_fail(e, "implicit convolution launch");
    }
    return NTG_OK;
}

// A 1x1 kernel with unit stride and no padding unfolds the image onto itself (col_b == x_b as a [C, H*W] matrix), so the
// convolution is the batched product W_g . x_b on the image where it lies.  Integer dtypes always take it; the floating
// ones when rows of the image and of W are 16-byte multiples (what the DMA-fed kernels need), else they gather.
static bool conv_pointwise(const Geo3& g) {
    for (int a = 0; a < 3; ++a)
        if (g.k[a] != 1 || g.s[a] != 1 || g.p[a] != 0) return false;
    return true;
}
static bool conv_pointwise_ok(int dtype, int64_t channels, int64_t groups, const Geo3& g) {
    if (!conv_pointwise(g)) return false;
    if (is_valu_dtype(dtype)) return true;
    const int64_t es = ntg::elem_size(dtype);
    return (g.L() * es) % 16 == 0 && (channels / groups * es) % 16 == 0;
}
static int conv_forward_pointwise(int dtype, const void* image, const void* kernel, void* out, int64_t batch, int64_t channels,
                                  int64_t out_channels, const Geo3& g, int64_t groups, void* stream) {
    const int64_t es = ntg::elem_size(dtype), cg = channels / groups, og = out_channels / groups, L = g.L();
    for (int64_t gi = 0; gi < groups; ++gi) {
        ntg_gemm_desc d;
        std::memset(&d, 0, sizeof d);
        d.dtype = dtype; d.c_mode = NTG_C_OVERWRITE;
        d.m = og; d.k = cg; d.n = L;
        d.lda = cg; d.ldb = L; d.ldc = L;
        d.batches = batch;
        d.stride_a = 0; d.stride_b = channels * L; d.stride_c = out_channels * L;
        int rc = ntg_gemm_dev(&d, static_cast<const char*>(kernel) + gi * og * cg * es, static_cast<const char*>(image) + gi * cg * L * es,
                              static_cast<char*>(out) + gi * og * L * es, stream);
        if (rc) return rc;
    }
    return NTG_OK;
}

// Channels-last form of the same convolution, for the floating dtypes up to 32 bits: the image is first copied to
// [B][pixel][C] and the weights to [O][(taps, c)] in the workspace; then one K-step of the product is 64 bytes of consecutive
// channels of one tap, and the kernel's DMA gathers the operand in 16-byte pieces instead of element by element.

// Byte offsets inside a channels-last image are formed in 32 bits from two terms (the pixel of the window origin, and the
// tap reach with the padding taken off): both must stay below 2^30
static bool conv_nhwc_offsets_fit(int64_t channels, int64_t es, const Geo3& g) {
    const int64_t pr = g.p[1] < 0 ? -g.p[1] : g.p[1], pc = g.p[2] < 0 ? -g.p[2] : g.p[2];
    const int64_t reach = ((pr + g.k[1] * g.d[1]) * g.sz[2] + pc + g.k[2] * g.d[2]) * channels * es;
    return channels * g.vol() * es < (1LL << 30) && reach < (1LL << 30);
}
// A K-step of the channels-last kernel is 64 bytes of channels of one tap, so the copy pads the channels of each group
// with zeros to the next multiple of 64 bytes (and the permuted weights likewise).  The padding is arithmetic spent on
// zeros: accepted up to 4x for the 16-bit types, whose element-wise gather is bound by the vector ALU (beyond that --
// RGB input layers -- the gathering kernels are the better choice); Float32 takes whole runs only: its element-wise
// DMA gather was measured faster than a padded copy (24 -> 32 channels: 48 against 60 us).  0: not accepted.
static int64_t nhwc_padded_channels(int64_t es, int64_t cg) {
    const int64_t step = 64 / es, cgp = (cg + step - 1) / step * step;
    return cg > 0 && cgp <= (es == 2 ? 4 : 1) * cg ? cgp : 0;
}
// The channels-last copy carries the convolution's padding as a border of zero pixels (two axes, non-negative padding):
// the padded image is as large as the windows reach, every tap of every window then exists, and the kernel's gather needs
// neither a validity test nor a per-lane address select -- its DMA is that of a stored operand.  gp describes the padded
// image with padding 0 (what the kernel is told); hm where the copy puts the pixels.
struct HaloPlan { bool on; ntg::HaloMap hm; Geo3 gp; int64_t vol; };
static HaloPlan conv_halo(const Geo3& g) {
    HaloPlan h;
    std::memset(&h.hm, 0, sizeof h.hm);
    h.on = false; h.gp = g; h.vol = g.vol();
    if (g.nd != 2 || g.p[1] < 0 || g.p[2] < 0) return h;
    const int64_t need_h = (g.o[1] - 1) * g.s[1] + (g.k[1] - 1) * g.d[1] + 1, need_w = (g.o[2] - 1) * g.s[2] + (g.k[2] - 1) * g.d[2] + 1;
    const int64_t Hp = std::max(need_h, g.p[1] + g.sz[1]), Wp = std::max(need_w, g.p[2] + g.sz[2]);
    if (Hp * Wp > 2 * g.sz[1] * g.sz[2] + 64) return h;               // (a border larger than the image: not worth the copy)
    h.hm.W = g.sz[2]; h.hm.H = g.sz[1]; h.hm.Wp = Wp; h.hm.Hp = Hp; h.hm.top = g.p[1]; h.hm.left = g.p[2];
    h.gp.sz[1] = Hp; h.gp.sz[2] = Wp; h.gp.p[1] = 0; h.gp.p[2] = 0;
    h.vol = Hp * Wp;
    h.on = true;
    return h;
}

// Few channels per group (up to 32 bytes of them): a pixel of the copy holds 16 or 32 bytes and a K-step covers 4 or 2
// consecutive taps of a tap row, the row padded to a multiple of that with zero weights -- an RGB 7 x 7 input layer in
// BFloat16 runs on K = 7 * 8 * 8 instead of 49 * 32.  Forward only.
struct MergedTaps { int64_t cgp, T, kq_pad; };
static bool conv_nhwc_merged(int dtype, int64_t channels, int64_t out_channels, int64_t groups, const Geo3& g, MergedTaps& mt) {
    if (dtype != ntg::DT_F32 && dtype != ntg::DT_F16 && dtype != ntg::DT_BF16) return false;
    if (g.nd != 2 || !conv_implicit_g(dtype, channels, g) || out_channels <= 0) return false;
    const int64_t es = ntg::elem_size(dtype), cg = channels / groups;
    if (cg <= 0 || cg * es > 32) return false;
    const int64_t cb = cg * es <= 16 ? 16 : 32;
    mt.cgp = cb / es; mt.T = 64 / cb; mt.kq_pad = (g.k[2] + mt.T - 1) / mt.T * mt.T;
    if (mt.kq_pad > 8 || mt.kq_pad * mt.cgp > 4 * g.k[2] * cg) return false;          // (padding: at most 4x the arithmetic)
    return conv_nhwc_offsets_fit(groups * mt.cgp, es, g);
}
static int64_t conv_nhwc_merged_workspace(int dtype, int64_t batch, int64_t out_channels, int64_t groups, const Geo3& g, const MergedTaps& mt) {
    const int64_t es = ntg::elem_size(dtype);
    return (int64_t)align_up((size_t)(batch * groups * mt.cgp * g.vol() * es), 256) + out_channels * g.k[1] * mt.kq_pad * mt.cgp * es;
}
static bool conv_nhwc_ok(int dtype, int64_t channels, int64_t out_channels, int64_t groups, const Geo3& g) {
    if (dtype != ntg::DT_F32 && dtype != ntg::DT_F16 && dtype != ntg::DT_BF16) return false;
    if (g.nd != 2 || !conv_implicit_g(dtype, channels, g)) return false;
    const int64_t es = ntg::elem_size(dtype), cgp = nhwc_padded_channels(es, channels / groups);
    return cgp > 0 && out_channels > 0 && conv_nhwc_offsets_fit(groups * cgp, es, g) && conv_nhwc_offsets_fit(groups * cgp, es, conv_halo(g).gp);
}
static int64_t conv_nhwc_workspace(int dtype, int64_t batch, int64_t channels, int64_t out_channels, int64_t groups, const Geo3& g) {
    const int64_t es = ntg::elem_size(dtype), cgp = nhwc_padded_channels(es, channels / groups);
    return (int64_t)align_up((size_t)(batch * groups * cgp * conv_halo(g).vol * es), 256) + out_channels * cgp * g.taps() * es;
}
static int conv_forward_nhwc(int dtype, const void* image, const void* kernel, void* out, void* ws, int64_t batch, int64_t channels,
                             int64_t out_channels, const Geo3& g, int64_t groups, hipStream_t hs, const MergedTaps* mt = nullptr) {
    const int64_t es = ntg::elem_size(dtype), cg = channels / groups, og = out_channels / groups;
    const int64_t cgp = mt ? mt->cgp : nhwc_padded_channels(es, cg), chp = groups * cgp;      // channels per group / per pixel in the copy
    const int64_t L = g.L(), taps = g.taps(), vol = g.vol(), K = mt ? g.k[1] * mt->kq_pad * cgp : taps * cgp;
    HaloPlan halo = conv_halo(g);
    if (mt) { halo.on = false; halo.vol = vol; halo.gp = g; }                    // (the merged-tap form keeps its validity bits)
    const int64_t volp = halo.vol;                                               // pixels per image of the copy
    const bool tap_inner = halo.on && g.s[1] == 1 && g.s[2] == 1;                // (neighbouring taps share pixels only at unit strides)
    char* ws_img = static_cast<char*>(ws);
    char* ws_w = ws_img + align_up((size_t)(batch * chp * volp * es), 256);
    const ntg::HaloMap* hm = halo.on ? &halo.hm : nullptr;
    // (the 16-byte copy kernel zeroes the border and permutes the weights in the same launch)
    const int64_t wchunk = tap_inner ? 64 / es : 0;                              // (taps inside a 64-byte run of channels)
    const ntg::WeightsJob wjob = {mt ? 0 : 1, kernel, ws_w, out_channels, 0, 0, cg, cgp, taps, wchunk};
    bool took_along = false;
    hipError_t e = cgp == cg ? ntg::launch_nchw_to_nhwc(es, image, ws_img, batch, channels, vol, hs, hm, &wjob, &took_along)
                             : ntg::launch_nchw_to_nhwc_padded(es, image, ws_img, batch, groups, cg, cgp, vol, hs, hm);
    if (e != hipSuccess) return hip_fail(e, "channels-last copy launch");
    if (halo.on && volp != vol && !took_along) {
        e = ntg::launch_halo_zero(es, ws_img, batch, chp, halo.hm, hs);
        if (e != hipSuccess) return hip_fail(e, "border fill launch");
    }
    if (mt) e = ntg::launch_weights_channels_last_rows(es, kernel, ws_w, out_channels, cg, cgp, g.k[1], g.k[2], mt->kq_pad, hs);
    else if (!took_along) e = ntg::launch_weights_channels_last(es, kernel, ws_w, out_channels, cg, cgp, taps, hs, wchunk);
    if (e != hipSuccess) return hip_fail(e, "weight permutation launch");
    for (int64_t gi = 0; gi < groups; ++gi) {
        ntg::GemmParams p;
        std::memset(&p, 0, sizeof p);
        p.M = (int)og; p.K = (int)K; p.N = (int)L; p.batch = (int)batch;
        p.A = ws_w + gi * og * K * es;
        p.B = ws_img + gi * cgp * es;
        p.C = static_cast<char*>(out) + gi * og * L * es;
        p.lda = K; p.ldb = chp; p.ldc = L;
        p.sA = 0; p.sB = chp * volp; p.sC = out_channels * L;
        p.cmode = ntg::C_OVERWRITE;
        p.vecA_ok = 1; p.vecB_ok = 1;
        fill_conv_geom(p.conv, cgp, halo.gp);
        p.conv.chan = (int)chp;                    // elements from one pixel to the next
        p.conv.halo = halo.on ? 1 : 0;
        p.conv.tap_inner = tap_inner ? 1 : 0;
        if (mt) { p.conv.tap_step = (int)mt->T; p.conv.kq_pad = (int)mt->kq_pad; }
        e = ntg::launch_conv_nhwc(dtype, p, hs);
        if (e != hipSuccess) return hip_fail(e, "channels-last convolution launch");
    }
    return NTG_OK;
}

// dW: one batched GEMM  P_{b,g} [og, add] = dY_{b,g} [og, L] . col_{b,g}^T  with col gathered from the image, into
// ws [B][O][add]; then the per-image results are summed in batch order (the same additions, in the same order, as
// accumulating one GEMM per image into dW, conv.cpp:466-469).
static int conv_dkernel_gather(int dtype, const void* image, const void* grad_out, void* d_kernel, void* ws, int64_t batch,
                               int64_t channels, int64_t out_channels, const Geo3& g, int64_t groups, int accumulate, hipStream_t hs) {
    const int64_t es = ntg::elem_size(dtype), cg = channels / groups, og = out_channels / groups;
    const int64_t L = g.L(), add = cg * g.taps(), vol = g.vol();
    for (int64_t gi = 0; gi < groups; ++gi) {
        ntg::GemmParams p;
        std::memset(&p, 0, sizeof p);
        p.M = (int)og; p.K = (int)L; p.N = (int)add; p.batch = (int)batch;
        p.A = static_cast<const char*>(grad_out) + gi * og * L * es;
        p.B = static_cast<const char*>(image) + gi * cg * vol * es;
        p.C = static_cast<char*>(ws) + gi * og * add * es;
        p.lda = L; p.ldb = L; p.ldc = add;
        p.sA = out_channels * L; p.sB = channels * vol; p.sC = out_channels * add;
        p.cmode = ntg::C_OVERWRITE;
        p.vecA_ok = (L * es) % 16 == 0 && (p.sA * es) % 16 == 0;
        fill_conv_geom(p.conv, cg, g);
        hipError_t e = ntg::launch_conv_mfma(dtype, true, g.nd, p, hs);
        if (e != hipSuccess) return hip_fail(e, "implicit conv_dkernel launch");
    }
    hipError_t e = ntg::launch_reduce_batch(dtype, ws, d_kernel, batch, out_channels * add, accumulate, hs);
    if (e != hipSuccess) return hip_fail(e, "weight gradient reduction launch");
    return NTG_OK;
}

// dX (all strides 1): the convolution of dY with the channel-swapped, tap-reversed kernel (written to ws) and padding
// d*(k-1) - p, again as an implicit GEMM; one sum over (oc, taps) per element instead of the reference's GEMM over oc
// followed by col2im over the taps -- same terms, different rounding order, inside the stated tolerance.
static int conv_dimage_gather(int dtype, const void* kernel, const void* grad_out, void* d_image, void* ws, int64_t batch,
                              int64_t channels, int64_t out_channels, const Geo3& g, int64_t groups, int accumulate, hipStream_t hs) {
    const int64_t es = ntg::elem_size(dtype), cg = channels / groups, og = out_channels / groups;
    const int64_t L = g.L(), taps = g.taps(), vol = g.vol();
    hipError_t e = ntg::launch_flip_weights(es, kernel, ws, groups, og, cg, taps, hs);
    if (e != hipSuccess) return hip_fail(e, "weight flip launch");
    const Geo3 t = geo_dimage(g);
    for (int64_t gi = 0; gi < groups; ++gi) {
        ntg::GemmParams p;
        std::memset(&p, 0, sizeof p);
        p.M = (int)cg; p.K = (int)(og * taps); p.N = (int)vol; p.batch = (int)batch;
        p.A = static_cast<const char*>(ws) + gi * cg * og * taps * es;
        p.B = static_cast<const char*>(grad_out) + gi * og * L * es;
        p.C = static_cast<char*>(d_image) + gi * cg * vol * es;
        p.lda = og * taps; p.ldb = vol; p.ldc = vol;
        p.sA = 0; p.sB = out_channels * L; p.sC = channels * vol;
        p.cmode = accumulate ? ntg::C_ACCUMULATE : ntg::C_OVERWRITE;
        p.vecA_ok = (og * taps * es) % 16 == 0;
        fill_conv_geom(p.conv, og, t);
        e = ntg::launch_conv_mfma(dtype, false, g.nd, p, hs);
        if (e != hipSuccess) return hip_fail(e, "implicit conv_dimage launch");
    }
    return NTG_OK;
}

// The same gradient through the channels-last kernel: dY is copied to [B][pixel][O] and the flipped weights to
// [C][(taps, oc)] in the workspace (out channels of a group in whole 64-byte runs, padded like the forward copy).
static bool conv_dimage_nhwc_ok(int dtype, int64_t channels, int64_t out_channels, int64_t groups, const Geo3& g) {
    return conv_nhwc_ok(dtype, out_channels, channels, groups, geo_dimage(g));
}
static int64_t conv_dimage_nhwc_workspace(int dtype, int64_t batch, int64_t channels, int64_t out_channels, int64_t groups, const Geo3& g) {
    return conv_nhwc_workspace(dtype, batch, out_channels, channels, groups, geo_dimage(g));
}
static int conv_dimage_nhwc(int dtype, const void* kernel, const void* grad_out, void* d_image, void* ws, int64_t batch,
                            int64_t channels, int64_t out_channels, const Geo3& g, int64_t groups, int accumulate, hipStream_t hs) {
    const int64_t es = ntg::elem_size(dtype), cg = channels / groups, og = out_channels / groups;
    const int64_t ogp = nhwc_padded_channels(es, og), ochp = groups * ogp;      // out channels per group / per pixel in the copy
    const int64_t L = g.L(), taps = g.taps(), vol = g.vol(), K = taps * ogp;
    const Geo3 t = geo_dimage(g);
    const HaloPlan halo = conv_halo(t);                                         // (the "image" of this convolution is dY)
    const int64_t Lp = halo.vol;
    const bool tap_inner = halo.on && t.s[1] == 1 && t.s[2] == 1;
    char* ws_gy = static_cast<char*>(ws);
    char* ws_w = ws_gy + align_up((size_t)(batch * ochp * Lp * es), 256);
    const ntg::HaloMap* hm = halo.on ? &halo.hm : nullptr;
    const int64_t wchunk = tap_inner ? 64 / es : 0;
    const ntg::WeightsJob wjob = {2, kernel, ws_w, groups, og, ogp, cg, 0, taps, wchunk};
    bool took_along = false;                                                    // (border and weight flip inside the copy's launch)
    hipError_t e = ogp == og ? ntg::launch_nchw_to_nhwc(es, grad_out, ws_gy, batch, out_channels, L, hs, hm, &wjob, &took_along)
                             : ntg::launch_nchw_to_nhwc_padded(es, grad_out, ws_gy, batch, groups, og, ogp, L, hs, hm);
    if (e != hipSuccess) return hip_fail(e, "channels-last copy launch");
    if (halo.on && Lp != L && !took_along) {
        e = ntg::launch_halo_zero(es, ws_gy, batch, ochp, halo.hm, hs);
        if (e != hipSuccess) return hip_fail(e, "border fill launch");
    }
    if (!took_along) e = ntg::launch_flip_weights_channels_last(es, kernel, ws_w, groups, og, ogp, cg, taps, hs, wchunk);
    if (e != hipSuccess) return hip_fail(e, "weight flip launch");
    for (int64_t gi = 0; gi < groups; ++gi) {
        ntg::GemmParams p;
        std::memset(&p, 0, sizeof p);
        p.M = (int)cg; p.K = (int)K; p.N = (int)vol; p.batch = (int)batch;
        p.A = ws_w + gi * cg * K * es;
        p.B = ws_gy + gi * ogp * es;
        p.C = static_cast<char*>(d_image) + gi * cg * vol * es;
        p.lda = K; p.ldb = ochp; p.ldc = vol;
        p.sA = 0; p.sB = ochp * Lp; p.sC = channels * vol;
        p.cmode = accumulate ? ntg::C_ACCUMULATE : ntg::C_OVERWRITE;
        p.vecA_ok = 1; p.vecB_ok = 1;
        fill_conv_geom(p.conv, ogp, halo.gp);
        p.conv.chan = (int)ochp;
        p.conv.halo = halo.on ? 1 : 0;
        p.conv.tap_inner = tap_inner ? 1 : 0;
        e = ntg::launch_conv_nhwc(dtype, p, hs);
        if (e != hipSuccess) return hip_fail(e, "channels-last conv_dimage launch");
    }
    return NTG_OK;
}

// dX of a convolution with strides > 1 (dilation 1), without the col matrix: the image rows y with (y + p) mod s = e
// form one phase; they receive only the taps i = e + s m (m = 0 .. M_e - 1), and, with a = (y + p) / s,
//   dX[y] = sum_m dY[a - m] W[e + s m],
// a stride-1 convolution of dY with the M_e reversed taps.  So every phase (er, ec) is one channels-last convolution
// (the forward kernel) of the shared channels-last copy of dY with its own small kernel, written to a plane of the
// phase's rows and columns in the workspace; a last pass interleaves the planes into dX.  Exactly the products of the
// reference's GEMM + col2im, none wasted on the zeros a dilated gradient would hold.
struct PhasePlan {
    bool ok;
    int64_t Mr[4], Mc[4], a0r[4], a0c[4], hp[4], wp[4];
    int64_t ogp, gy_bytes, w_bytes, tmp_bytes;
};
static Geo3 phase_geo(const Geo3& g, const PhasePlan& pp, int er, int ec) {
    // image = the dY plane, kernel Mr x Mc, stride 1, padding (M - 1) - a0 (first row of the plane is a0), outputs hp x wp
    return Geo3{2, {1, g.o[1], g.o[2]}, {1, pp.Mr[er], pp.Mc[ec]}, {1, 1, 1}, {0, pp.Mr[er] - 1 - pp.a0r[er], pp.Mc[ec] - 1 - pp.a0c[ec]},
                {1, 1, 1}, {1, pp.hp[er], pp.wp[ec]}};
}
static PhasePlan plan_dimage_phases(int dtype, int64_t batch, int64_t channels, int64_t out_channels, int64_t groups, const Geo3& g) {
    PhasePlan pp;
    std::memset(&pp, 0, sizeof pp);
    if (dtype != ntg::DT_F32 && dtype != ntg::DT_F16 && dtype != ntg::DT_BF16) return pp;
    if (g.nd != 2 || g.d[1] != 1 || g.d[2] != 1 || (g.s[1] == 1 && g.s[2] == 1) || g.s[1] > 4 || g.s[2] > 4 || g.p[1] < 0 || g.p[2] < 0) return pp;
    if (g.k[1] > 8 * g.s[1] || g.k[2] > 8 * g.s[2]) return pp;
    const int64_t es = ntg::elem_size(dtype), og = out_channels / groups;
    pp.ogp = nhwc_padded_channels(es, og);
    if (pp.ogp == 0 || batch * channels * g.vol() >= 0x7fffffffLL) return pp;
    // the image channels of a group are the rows of these products: with a handful of them (an RGB input layer) a 64-row
    // tile is mostly padding, and the GEMM over (channel, tap) rows followed by col2im is the better form
    if (channels / groups < 16) return pp;
    for (int ax = 1; ax <= 2; ++ax) {
        int64_t* M = ax == 1 ? pp.Mr : pp.Mc;
        int64_t* a0 = ax == 1 ? pp.a0r : pp.a0c;
        int64_t* n = ax == 1 ? pp.hp : pp.wp;
        for (int64_t e = 0; e < g.s[ax]; ++e) {
            M[e] = e < g.k[ax] ? (g.k[ax] - e + g.s[ax] - 1) / g.s[ax] : 0;
            // image positions y = s a + e - p in [0, size): a from a0
            a0[e] = g.p[ax] > e ? (g.p[ax] - e + g.s[ax] - 1) / g.s[ax] : 0;
            const int64_t last = g.sz[ax] - 1 + g.p[ax] - e;                      // largest s a
            n[e] = last >= 0 && last / g.s[ax] >= a0[e] ? last / g.s[ax] - a0[e] + 1 : 0;
        }
    }
    int64_t wmax = 0, tmp = 0;
    for (int64_t er = 0; er < g.s[1]; ++er)
        for (int64_t ec = 0; ec < g.s[2]; ++ec) {
            if (pp.Mr[er] == 0 || pp.Mc[ec] == 0 || pp.hp[er] == 0 || pp.wp[ec] == 0) continue;
            if (!conv_nhwc_ok(dtype, out_channels, channels, groups, phase_geo(g, pp, (int)er, (int)ec))) return pp;
            wmax += (int64_t)align_up((size_t)(channels * pp.Mr[er] * pp.Mc[ec] * pp.ogp * es), 256);
            tmp += (int64_t)align_up((size_t)(batch * channels * pp.hp[er] * pp.wp[ec] * es), 256);
        }
    pp.gy_bytes = (int64_t)align_up((size_t)(batch * groups * pp.ogp * g.L() * es), 256);
    pp.w_bytes = wmax;
    pp.tmp_bytes = tmp;
    pp.ok = true;
    return pp;
}
static int conv_dimage_phases(int dtype, const PhasePlan& pp, const void* kernel, const void* grad_out, void* d_image, void* ws, int64_t batch,
                              int64_t channels, int64_t out_channels, const Geo3& g, int64_t groups, int accumulate, hipStream_t hs) {
    const int64_t es = ntg::elem_size(dtype), cg = channels / groups, og = out_channels / groups;
    const int64_t ogp = pp.ogp, ochp = groups * ogp, L = g.L();
    char* ws_gy = static_cast<char*>(ws);
    char* ws_w = ws_gy + pp.gy_bytes;
    char* ws_tmp = ws_w + pp.w_bytes;
    hipError_t e = ogp == og ? ntg::launch_nchw_to_nhwc(es, grad_out, ws_gy, batch, out_channels, L, hs)
                             : ntg::launch_nchw_to_nhwc_padded(es, grad_out, ws_gy, batch, groups, og, ogp, L, hs);
    if (e != hipSuccess) return hip_fail(e, "channels-last copy launch");
    ntg::PhaseLayout lay;
    std::memset(&lay, 0, sizeof lay);
    lay.H = (int)g.sz[1]; lay.W = (int)g.sz[2]; lay.p_r = (int)g.p[1]; lay.p_c = (int)g.p[2]; lay.s_r = (int)g.s[1]; lay.s_c = (int)g.s[2];
    lay.total = (uint32_t)(batch * channels * g.vol());
    lay.div_w = ntg::make_fastdiv((uint32_t)lay.W); lay.div_h = ntg::make_fastdiv((uint32_t)lay.H);
    lay.div_sr = ntg::make_fastdiv((uint32_t)lay.s_r); lay.div_sc = ntg::make_fastdiv((uint32_t)lay.s_c);
    for (int i = 0; i < 4; ++i) { lay.a0r[i] = (int)pp.a0r[i]; lay.a0c[i] = (int)pp.a0c[i]; lay.hp[i] = (int)pp.hp[i]; lay.wp[i] = (int)pp.wp[i]; }
    for (int i = 0; i < 16; ++i) lay.off[i] = -1;
    int64_t w_off = 0, t_off = 0;
    for (int64_t er = 0; er < g.s[1]; ++er)
        for (int64_t ec = 0; ec < g.s[2]; ++ec) {
            if (pp.Mr[er] == 0 || pp.Mc[ec] == 0 || pp.hp[er] == 0 || pp.wp[ec] == 0) continue;
            const Geo3 t = phase_geo(g, pp, (int)er, (int)ec);
            const int64_t taps = pp.Mr[er] * pp.Mc[ec], K = taps * ogp, plane = pp.hp[er] * pp.wp[ec];
            char* wph = ws_w + w_off;
            char* tph = ws_tmp + t_off;
            e = ntg::launch_phase_weights(es, kernel, wph, groups, og, ogp, cg, g.k[1], g.k[2], er, ec, g.s[1], g.s[2], pp.Mr[er], pp.Mc[ec], hs);
            if (e != hipSuccess) return hip_fail(e, "phase weight launch");
            for (int64_t gi = 0; gi < groups; ++gi) {
                ntg::GemmParams p;
                std::memset(&p, 0, sizeof p);
                p.M = (int)cg; p.K = (int)K; p.N = (int)plane; p.batch = (int)batch;
                p.A = wph + gi * cg * K * es;
                p.B = ws_gy + gi * ogp * es;
                p.C = tph + gi * cg * plane * es;
                p.lda = K; p.ldb = ochp; p.ldc = plane;
                p.sA = 0; p.sB = ochp * L; p.sC = channels * plane;
                p.cmode = ntg::C_OVERWRITE;
                p.vecA_ok = 1; p.vecB_ok = 1;
                fill_conv_geom(p.conv, ogp, t);
                p.conv.chan = (int)ochp;
                e = ntg::launch_conv_nhwc(dtype, p, hs);
                if (e != hipSuccess) return hip_fail(e, "phase convolution launch");
            }
            lay.off[er * g.s[2] + ec] = t_off / es;
            w_off += (int64_t)align_up((size_t)(channels * taps * ogp * es), 256);
            t_off += (int64_t)align_up((size_t)(batch * channels * plane * es), 256);
        }
    e = ntg::launch_phase_interleave(dtype, ws_tmp, d_image, lay, accumulate, hs);
    if (e != hipSuccess) return hip_fail(e, "phase interleave launch");
    return NTG_OK;
}

// dW through the channels-last kernel: the image is copied to [B][pixel][C]; per image and group
// P_{b,g} [og][(taps, c)] = dY_{b,g} [og, L] . col^T gathered 16 bytes of channels at a time; the per-image results are
// summed in batch order into the kernel's [O][c][taps] layout.  The copy pads the channels of a group to whole 16-byte
// runs; dY is read where it lies or from a channels-last copy of its own (below).
// Large output planes with 16-byte rows: dY is read where it lies, one image per K loop (measured faster from about 512
// pixels: no copy, one LDS read per block instead of the transposing ones).  Otherwise, when the out channels of a group
// are a 16-byte multiple, dY goes through its own channels-last copy: as a [pixel][out channel] matrix the images follow
// each other, so several of them can share one K loop.
static bool conv_dkernel_nhwc_copies_dy(int dtype, int64_t out_channels, int64_t groups, const Geo3& g) {
    const int64_t es = ntg::elem_size(dtype);
    if ((g.L() * es) % 16 == 0 && g.L() >= 512) return false;
    return ((out_channels / groups) * es) % 16 == 0;
}
// Images per K loop: the largest divisor of the batch that still leaves two workgroups per CU (128 x 128 tiles), so that
// fewer per-image results are written and summed (64 images of a 3 x 3 x 256 x 256 layer: 16 partial sums instead of 64;
// 7 x 7 maps: K = 784 instead of 49).
static int64_t conv_dkernel_fold(int64_t batch, int64_t og, int64_t n, int64_t groups, int64_t L) {
    const int64_t tiles = ((og + 127) / 128) * ((n + 127) / 128) * groups;
    int64_t best = 1;
    for (int64_t f = 2; f <= batch; ++f) {
        if (batch % f) continue;
        if ((batch / f) * tiles < 512 || f * L >= (1LL << 30)) break;
        best = f;
    }
    return best;
}
// 16-bit, dY read where it lies: instead of one product per image, the output pixels of all images counted through are cut
// into `ranges` equal k ranges (whole K-steps; an image is whole K-steps too) so that tiles x ranges fill whole rounds
// over the CUs: 64 images of a 3 x 3 x 256 x 256 layer on 56 x 56 maps are 9 tiles x 28 ranges = 252 tiles of 7168 pixels
// in one round (235 us + 10 us for adding 28 partial sums), against 512 + 256 tiles in three rounds (217 + 46 us, + 18 us
// for 64 partial sums).  Returns the number of ranges, 0: one product per image.
// The estimate prices the gathering kernel as measured on that layer: 0.41 of a CU's MFMA peak on 256 x 256 tiles, 0.35 on
// 128 x 128 tiles when two workgroups share a CU and 0.245 when one has it alone; it has to be 5 % ahead.
static double dkernel16_cost_us(int edge, int64_t tiles, int64_t K) {
    const double cu_flops_per_us = 9.77e6, area = (double)edge * edge;
    if (edge == 256) return (double)((tiles + 255) / 256) * (2.0 * area * (double)K / (cu_flops_per_us * 0.41) + 6.0);
    if (edge == 128) {
        if (tiles <= 256) return 2.0 * area * (double)K / (cu_flops_per_us * 0.245) + 3.0;
        return (double)((tiles + 511) / 512) * (4.0 * area * (double)K / (cu_flops_per_us * 0.35) + 3.0);
    }
    return (double)((tiles + 1023) / 1024) * (8.0 * area * (double)K / (cu_flops_per_us * 0.2) + 2.0);
}
static double dkernel16_plan_cost_us(int64_t M, int64_t N, int64_t K, int64_t batch) {
    const ntg::Ring16Plan pl = ntg::ring16_plan(M, N, K, batch);
    if (pl.head >= batch) return dkernel16_cost_us(pl.edge, ntg::ring16_tiles(pl.edge, M, N, batch), K);
    return dkernel16_cost_us(pl.edge, ntg::ring16_tiles(pl.edge, M, N, pl.head), K) +
           dkernel16_cost_us(pl.tail_edge, ntg::ring16_tiles(pl.tail_edge, M, N, batch - pl.head), K) + 2.0;
}
static int64_t conv_dkernel_ranges(int dtype, int64_t batch, int64_t og, int64_t out_channels, int64_t N, int64_t L) {
    const int64_t es = ntg::elem_size(dtype), bk = 64 / es;
    if (es != 2 || batch < 2 || L % bk != 0 || batch * L >= (1LL << 30)) return 0;
    auto reduce_us = [&](int64_t items) { return 3.0 + (double)items * (double)(out_channels * N * es) / 4.0e6; };
    const int64_t hc = ntg::ring16_column_split(og, N, L, batch);
    const double cur = (hc ? dkernel16_plan_cost_us(og, hc, L, batch) + dkernel16_plan_cost_us(og, N - hc, L, batch) + 2.0
                           : dkernel16_plan_cost_us(og, N, L, batch)) + reduce_us(batch);
    const int64_t steps = batch * L / bk;
    // measurement and test knob: NTG_DW_RANGES=r forces r ranges where r is admissible, 0 forces one product per image
    if (const char* env = std::getenv("NTG_DW_RANGES")) {
        const int64_t r = std::atoll(env);
        return r > 0 && r <= batch && steps % r == 0 ? r : 0;
    }
    int64_t best = 0;
    double best_us = 0.95 * cur;
    for (int64_t r = 1; r <= batch; ++r) {
        if (steps % r != 0 || steps / r < 16) continue;
        const int64_t kr = steps / r * bk;
        const int edge = ntg::ring16_tile_edge(og, N, kr, r);
        const double us = dkernel16_cost_us(edge, ntg::ring16_tiles(edge, og, N, r), kr) + reduce_us(r);
        if (us < best_us) { best_us = us; best = r; }
    }
    return best;
}
static int64_t dkernel_padded_channels(int64_t es, int64_t cg) { const int64_t v = 16 / es; return (cg + v - 1) / v * v; }
// The copy of the image carries the padding as a border of zero pixels where the plain 16-byte copy serves it (whole
// 16-byte runs of channels): the gather then needs no validity test, and keeps the window origins in a table.
static HaloPlan dkernel_halo(int64_t es, int64_t cg, int64_t groups, const Geo3& g) {
    HaloPlan h = conv_halo(g);
    if (h.on && (dkernel_padded_channels(es, cg) != cg || !conv_nhwc_offsets_fit(groups * cg, es, h.gp))) {
        h.on = false; h.gp = g; h.vol = g.vol();
    }
    return h;
}
static bool conv_dkernel_nhwc_ok(int dtype, int64_t channels, int64_t out_channels, int64_t groups, const Geo3& g) {
    if (dtype != ntg::DT_F32 && dtype != ntg::DT_F16 && dtype != ntg::DT_BF16) return false;
    if (g.nd != 2 || !conv_implicit_g(dtype, channels, g)) return false;
    const int64_t es = ntg::elem_size(dtype), cg = channels / groups;
    if (g.k[1] * g.d[1] >= 32768 || g.k[2] * g.d[2] >= 32768) return false;      // tap reach packed in 16 bits
    // rows of dY that are 16-byte multiples are read where they lie; otherwise dY is copied channels-last too and read
    // as a [pixel][out channel] operand, which needs the out channels of a group to be a 16-byte multiple
    const bool a_ok = (g.L() * es) % 16 == 0 || conv_dkernel_nhwc_copies_dy(dtype, out_channels, groups, g);
    // the channels of a group are gathered in 16-byte runs: the copy pads them to whole runs (RGB: 3 -> 8 or 4)
    const int64_t cgp = dkernel_padded_channels(es, cg);
    return a_ok && cgp <= 4 * cg && out_channels > 0 && cgp * g.taps() < 0x7fffffffLL && conv_nhwc_offsets_fit(groups * cgp, es, g);
}
static int64_t conv_dkernel_nhwc_workspace(int dtype, int64_t batch, int64_t channels, int64_t out_channels, int64_t groups, const Geo3& g) {
    const int64_t es = ntg::elem_size(dtype);
    const int64_t gy = conv_dkernel_nhwc_copies_dy(dtype, out_channels, groups, g) ? (int64_t)align_up((size_t)(batch * out_channels * g.L() * es), 256) : 0;
    const int64_t cgp = dkernel_padded_channels(es, channels / groups);
    return (int64_t)align_up((size_t)(batch * groups * cgp * dkernel_halo(es, channels / groups, groups, g).vol * es), 256) + gy +
           batch * out_channels * cgp * g.taps() * es;
}
static int conv_dkernel_nhwc(int dtype, const void* image, const void* grad_out, void* d_kernel, void* ws, int64_t batch,
                             int64_t channels, int64_t out_channels, const Geo3& g, int64_t groups, int accumulate, hipStream_t hs) {
    const int64_t es = ntg::elem_size(dtype), cg = channels / groups, og = out_channels / groups;
    const int64_t cgp = dkernel_padded_channels(es, cg), chp = groups * cgp;      // channels per group / per pixel in the copy
    const int64_t L = g.L(), taps = g.taps(), vol = g.vol(), N = taps * cgp;
    const HaloPlan halo = dkernel_halo(es, cg, groups, g);
    const int64_t volp = halo.vol;                                                         // pixels per image of the copy
    const bool copy_dy = conv_dkernel_nhwc_copies_dy(dtype, out_channels, groups, g);      // dY read as [pixel][out channel] from its own copy
    const int64_t ranges = copy_dy ? 0 : conv_dkernel_ranges(dtype, batch, og, out_channels, N, L);
    const int64_t fold = copy_dy ? conv_dkernel_fold(batch, og, N, groups, L) : 1, items = ranges ? ranges : batch / fold;
    char* ws_img = static_cast<char*>(ws);
    char* ws_gy = ws_img + align_up((size_t)(batch * chp * volp * es), 256);
    char* ws_part = ws_gy + (copy_dy ? align_up((size_t)(batch * out_channels * L * es), 256) : 0);
    bool took_along = false;
    hipError_t e = cgp == cg ? ntg::launch_nchw_to_nhwc(es, image, ws_img, batch, channels, vol, hs, halo.on ? &halo.hm : nullptr, nullptr, &took_along)
                             : ntg::launch_nchw_to_nhwc_padded(es, image, ws_img, batch, groups, cg, cgp, vol, hs);
    if (e == hipSuccess && halo.on && volp != vol && !took_along) e = ntg::launch_halo_zero(es, ws_img, batch, chp, halo.hm, hs);
    if (e == hipSuccess && copy_dy) e = ntg::launch_nchw_to_nhwc(es, grad_out, ws_gy, batch, out_channels, L, hs);
    if (e != hipSuccess) return hip_fail(e, "channels-last copy launch");
    for (int64_t gi = 0; gi < groups; ++gi) {
        ntg::GemmParams p;
        std::memset(&p, 0, sizeof p);
        p.M = (int)og; p.K = (int)(fold * L); p.N = (int)N; p.batch = (int)items;
        if (copy_dy) {
            p.A = ws_gy + gi * og * es;
            p.lda = out_channels;
        } else {
            p.A = static_cast<const char*>(grad_out) + gi * og * L * es;
            p.lda = L;
        }
        p.B = ws_img + gi * cgp * es;
        p.C = ws_part + gi * og * N * es;
        p.ldb = chp; p.ldc = N;
        p.sA = fold * out_channels * L; p.sB = fold * chp * volp; p.sC = out_channels * N;
        p.cmode = ntg::C_OVERWRITE;
        p.vecA_ok = 1; p.vecB_ok = 1;
        fill_conv_geom(p.conv, cgp, halo.gp);
        p.conv.chan = (int)chp;                    // elements from one pixel to the next
        if (fold > 1 || ranges) {
            p.conv.fold_L = (int)L;
            p.conv.div_fold = ntg::make_fastdiv((uint32_t)L);
            p.conv.fold_stride = chp * volp;
        }
        if (halo.on && fold == 1 && L < (1 << 20)) p.conv.pix_table = (int)L;     // (a K-step inside one image: see the kernel)
        if (ranges) {
            const int64_t bk = 64 / es;
            p.K = (int)(batch * L / ranges);
            p.sA = 0; p.sB = 0;
            p.conv.k_ranges = 1;
            p.conv.a_steps = (int)(L / bk);
            p.conv.div_a_steps = ntg::make_fastdiv((uint32_t)(L / bk));
            p.conv.a_image_stride = out_channels * L;
        }
        e = ntg::launch_conv_nhwc_dw(dtype, copy_dy, p, hs);
        if (e != hipSuccess) return hip_fail(e, "channels-last conv_dkernel launch");
    }
    // (groups are consecutive row blocks of both layouts, so one pass covers them all)
    e = ntg::launch_reduce_batch_taps_last(dtype, ws_part, d_kernel, items, out_channels, cg, cgp, taps, accumulate, hs);
    if (e != hipSuccess) return hip_fail(e, "weight gradient reduction launch");
    return NTG_OK;
}

// The weight gradient from a stored col matrix (integers, complex types, four spatial axes): per group g
//   dW_g [og, add] (+)= sum over the images b of dY_{b,g} [og, L] . col_{b,g}^T   (col_{b,g} stored [add, L]).
// Integers: one accumulating product per (group, image) straight into dW (exact in any order).  Complex types: the
// reference's order, which the results are checked against bit for bit -- every image's product on its own from zero, the
// products added up in batch order in the element type, that sum added to dW last (conv.cpp:444-471: matmult(grad, image,
// false, true).sum(0), then d_kernel +=); the per-image products [B][O][add] lie behind the col matrix in the workspace.
static int64_t complex_dkernel_extra(int dtype, int64_t batch, int64_t out_channels, int64_t add, int64_t col_bytes) {
    if (!is_complex_dtype(dtype)) return 0;
    return (int64_t)(align_up((size_t)col_bytes, 256) - (size_t)col_bytes) + batch * out_channels * add * ntg::elem_size(dtype);
}
static int conv_dkernel_from_col(int dtype, const char* gy, char* col, void* d_kernel, int64_t batch, int64_t out_channels, int64_t ccol,
                                 int64_t groups, int64_t L, int accumulate, void* stream) {
    const int64_t es = ntg::elem_size(dtype), add = ccol / groups, og = out_channels / groups;
    ntg_gemm_desc d;
    int rc = NTG_OK;
    if (is_complex_dtype(dtype)) {
        char* per = col + align_up((size_t)(batch * ccol * L * es), 256);
        for (int64_t g = 0; g < groups && rc == NTG_OK; ++g) {
            std::memset(&d, 0, sizeof d);
            d.dtype = dtype; d.transpose_b = 1; d.c_mode = NTG_C_OVERWRITE;
            d.m = og; d.k = L; d.n = add;
            d.lda = L; d.ldb = L; d.ldc = add; d.batches = batch;
            d.stride_a = out_channels * L; d.stride_b = ccol * L; d.stride_c = out_channels * add;
            rc = ntg_gemm_dev(&d, gy + g * og * L * es, col + g * add * L * es, per + g * og * add * es, stream);
        }
        if (rc) return rc;
        hipError_t e = ntg::launch_reduce_batch(dtype, per, d_kernel, batch, out_channels * add, accumulate, static_cast<hipStream_t>(stream));
        if (e != hipSuccess) return hip_fail(e, "weight gradient reduction launch");
        return NTG_OK;
    }
    for (int64_t g = 0; g < groups; ++g)
        for (int64_t b = 0; b < batch; ++b) {
            std::memset(&d, 0, sizeof d);
            d.dtype = dtype; d.transpose_b = 1;
            d.c_mode = (b == 0 && !accumulate) ? NTG_C_OVERWRITE : NTG_C_ACCUMULATE;
            d.m = og; d.k = L; d.n = add;
            d.lda = L; d.ldb = L; d.ldc = add; d.batches = 1;
            rc = ntg_gemm_dev(&d, gy + ((b * out_channels + g * og) * L) * es, col + ((b * ccol + g * add) * L) * es,
                              static_cast<char*>(d_kernel) + g * og * add * es, stream);
            if (rc) return rc;
        }
    return NTG_OK;
}

// Which backward gradients run as implicit GEMMs, and the workspace the call needs.
struct ConvBackwardPlan { bool gather_dw, gather_dx, nhwc_dx, nhwc_dw, phase_dx; int64_t need, need_nhwc_dx, need_nhwc_dw, need_phase_dx; PhasePlan phases; };
// reference_order (Float32 through the host entry points): the forms whose sums are the reference's own, bit for bit -- the
// image gradient as W^T . dY into the col matrix + col2im (conv.cpp:318-346; the implicit forms run one chain over out
// channels and taps where the reference rounds in between), the weight gradient per image with k = the output pixels +
// the sum over the batch (conv.cpp:444-471; not the channels-last kernels, whose partial sums may span images).
static ConvBackwardPlan plan_conv_backward_g(int dtype, bool want_dx, bool want_dw, int64_t batch, int64_t channels, int64_t out_channels,
                                             const Geo3& g, int64_t groups, bool reference_order = false) {
    const int64_t es = ntg::elem_size(dtype);
    const int64_t cg = channels / groups, taps = g.taps();
    ConvBackwardPlan pl;
    pl.gather_dw = want_dw && conv_implicit_g(dtype, channels, g);
    pl.gather_dx = want_dx && !reference_order && g.s[0] == 1 && g.s[1] == 1 && g.s[2] == 1 && conv_implicit_g(dtype, out_channels, geo_dimage(g));
    const int64_t col = batch * channels * taps * g.L() * es;
    int64_t need = 0;
    if (want_dw) need = std::max(need, pl.gather_dw ? batch * out_channels * cg * taps * es : col + complex_dkernel_extra(dtype, batch, out_channels, cg * taps, col));
    if (want_dx) need = std::max(need, pl.gather_dx ? out_channels * cg * taps * es : col);
    pl.need = need;
    // the channels-last form of dX is taken when the caller's workspace also holds the copy of dY
    pl.nhwc_dx = pl.gather_dx && g.nd == 2 && conv_dimage_nhwc_ok(dtype, channels, out_channels, groups, g);
    pl.need_nhwc_dx = pl.nhwc_dx ? conv_dimage_nhwc_workspace(dtype, batch, channels, out_channels, groups, g) : 0;
    pl.nhwc_dw = pl.gather_dw && !reference_order && conv_dkernel_nhwc_ok(dtype, channels, out_channels, groups, g);
    pl.need_nhwc_dw = pl.nhwc_dw ? conv_dkernel_nhwc_workspace(dtype, batch, channels, out_channels, groups, g) : 0;
    // strides > 1: dX phase by phase instead of GEMM + col2im, again when the workspace allows
    std::memset(&pl.phases, 0, sizeof pl.phases);
    if (want_dx && !pl.gather_dx && !reference_order && conv_implicit_g(dtype, out_channels, geo_dimage(g)))
        pl.phases = plan_dimage_phases(dtype, batch, channels, out_channels, groups, g);
    pl.phase_dx = pl.phases.ok;
    pl.need_phase_dx = pl.phase_dx ? pl.phases.gy_bytes + pl.phases.w_bytes + pl.phases.tmp_bytes : 0;
    return pl;
}

int64_t ntg_conv2d_fast_workspace_bytes(int dtype, int64_t batch, int64_t channels, int64_t height, int64_t width,
                                        int64_t out_channels, int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c,
                                        int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c, int64_t groups) {
    const int64_t es = ntg::elem_size(dtype);
    int64_t Ho, Wo;
    if (es == 0 || unfold_out(height, width, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, Ho, Wo)) return -1;
    const Geo3 g = geo2(height, width, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, Ho, Wo);
    const bool groups_ok = groups >= 1 && channels % groups == 0 && out_channels % groups == 0;      // (the call itself reports bad groups)
    if (groups_ok && conv_pointwise_ok(dtype, channels, groups, g)) return 0;
    MergedTaps mt;
    if (groups_ok && conv_nhwc_merged(dtype, channels, out_channels, groups, g, mt)) return conv_nhwc_merged_workspace(dtype, batch, out_channels, groups, g, mt);
    if (groups_ok && conv_nhwc_ok(dtype, channels, out_channels, groups, g)) return conv_nhwc_workspace(dtype, batch, channels, out_channels, groups, g);
    return ntg_conv2d_forward_workspace_bytes(dtype, batch, channels, height, width, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c);
}

int64_t ntg_conv2d_forward_workspace_bytes(int dtype, int64_t batch, int64_t channels, int64_t height, int64_t width,
                                           int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c,
                                           int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c) {
    const int64_t es = ntg::elem_size(dtype);
    int64_t Ho, Wo;
    if (es == 0 || unfold_out(height, width, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, Ho, Wo)) return -1;
    if (conv_implicit(dtype, channels, height, width, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, Ho, Wo)) return 0;
    if (conv_pointwise(geo2(height, width, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, Ho, Wo))) return 0;
    return batch * channels * k_r * k_c * Ho * Wo * es;
}

int64_t ntg_conv2d_workspace_bytes(int dtype, int64_t batch, int64_t channels, int64_t height, int64_t width,
                                   int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c,
                                   int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c) {
    const int64_t es = ntg::elem_size(dtype);
    int64_t Ho, Wo;
    if (es == 0 || unfold_out(height, width, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, Ho, Wo)) return -1;
    return batch * channels * k_r * k_c * Ho * Wo * es;
}

int ntg_conv2d_dev(int dtype, const void* image, const void* kernel, void* out,
                   void* workspace, int64_t workspace_bytes,
                   int64_t batch, int64_t channels, int64_t height, int64_t width,
                   int64_t out_channels, int64_t k_r, int64_t k_c,
                   int64_t s_r, int64_t s_c, int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c,
                   int64_t groups, void* stream) {
    const int64_t es = ntg::elem_size(dtype);
    if (es == 0) return fail(NTG_ERR_UNSUPPORTED_DTYPE, "dtype %d is not supported", dtype);
    if (batch < 0 || channels < 0 || out_channels < 0 || height < 0 || width < 0) return fail(NTG_ERR_INVALID_ARGUMENT, "negative size");
    if (groups < 1) return fail(NTG_ERR_INVALID_ARGUMENT, "groups must be >= 1");
    // conv.cpp:97-98
    if (channels % groups != 0) return fail(NTG_ERR_INVALID_ARGUMENT, "image channels (%lld) not divisible by groups (%lld)", (long long)channels, (long long)groups);
    if (out_channels % groups != 0) return fail(NTG_ERR_INVALID_ARGUMENT, "out channels (%lld) not divisible by groups (%lld)", (long long)out_channels, (long long)groups);
    int64_t Ho, Wo;
    int rc = unfold_out(height, width, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, Ho, Wo);
    if (rc) return rc;
    if (batch == 0 || out_channels == 0) return NTG_OK;
    if (!image || !kernel || !out) return fail(NTG_ERR_INVALID_ARGUMENT, "null pointer");
    const int64_t L = Ho * Wo, ckk = channels * k_r * k_c;
    const int64_t add = (channels / groups) * k_r * k_c, og = out_channels / groups;
    {
        const Geo3 g = geo2(height, width, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, Ho, Wo);
        if (conv_pointwise_ok(dtype, channels, groups, g) &&
            (is_valu_dtype(dtype) || ((reinterpret_cast<uintptr_t>(image) | reinterpret_cast<uintptr_t>(kernel) | reinterpret_cast<uintptr_t>(out)) & 15) == 0))
            return conv_forward_pointwise(dtype, image, kernel, out, batch, channels, out_channels, g, groups, stream);
        // with the workspace of ntg_conv2d_fast_workspace_bytes: channels-last copy of the image, 16-byte gathers
        MergedTaps mt;
        if (conv_nhwc_merged(dtype, channels, out_channels, groups, g, mt) && workspace && (reinterpret_cast<uintptr_t>(workspace) & 15) == 0 &&
            workspace_bytes >= conv_nhwc_merged_workspace(dtype, batch, out_channels, groups, g, mt))
            return conv_forward_nhwc(dtype, image, kernel, out, workspace, batch, channels, out_channels, g, groups, static_cast<hipStream_t>(stream), &mt);
        if (conv_nhwc_ok(dtype, channels, out_channels, groups, g) && workspace && (reinterpret_cast<uintptr_t>(workspace) & 15) == 0 &&
            workspace_bytes >= conv_nhwc_workspace(dtype, batch, channels, out_channels, groups, g))
            return conv_forward_nhwc(dtype, image, kernel, out, workspace, batch, channels, out_channels, g, groups, static_cast<hipStream_t>(stream));
        if (conv_implicit_g(dtype, channels, g))      // col_b is never stored: the GEMM's B loader gathers it from the image
            return conv_forward_gather(dtype, image, kernel, out, batch, channels, out_channels, g, groups, static_cast<hipStream_t>(stream));
    }
    const int64_t need = batch * channels * k_r * k_c * Ho * Wo * es;
    if (need > 0 && (!workspace || workspace_bytes < need))
        return fail(NTG_ERR_INVALID_ARGUMENT, "workspace of %lld bytes needed, %lld given", (long long)need, (long long)workspace_bytes);
    rc = ntg_unfold2d_dev(dtype, image, workspace, batch, channels, height, width, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, stream);
    if (rc) return rc;
    for (int64_t g = 0; g < groups; ++g) {
        ntg_gemm_desc d;
        std::memset(&d, 0, sizeof d);
        d.dtype = dtype; d.c_mode = NTG_C_OVERWRITE;
        d.m = og; d.k = add; d.n = L;
        d.lda = add; d.ldb = L; d.ldc = L;
        d.batches = batch;
        d.stride_a = 0; d.stride_b = ckk * L; d.stride_c = out_channels * L;
        rc = ntg_gemm_dev(&d, static_cast<const char*>(kernel) + g * og * add * es,
                          static_cast<const char*>(workspace) + g * add * L * es,
                          static_cast<char*>(out) + g * og * L * es, stream);
        if (rc) return rc;
    }
    return NTG_OK;
}

int ntg_conv2d(int dtype, const void* image, const void* kernel, void* out,
               int64_t batch, int64_t channels, int64_t height, int64_t width,
               int64_t out_channels, int64_t k_r, int64_t k_c,
               int64_t s_r, int64_t s_c, int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c,
               int64_t groups) {
    const int64_t es = ntg::elem_size(dtype);
    if (es == 0) return fail(NTG_ERR_UNSUPPORTED_DTYPE, "dtype %d is not supported", dtype);
    if (batch < 0 || channels < 0 || out_channels < 0 || height < 0 || width < 0) return fail(NTG_ERR_INVALID_ARGUMENT, "negative size");
    if (groups < 1 || channels % groups != 0 || out_channels % groups != 0)
        return fail(NTG_ERR_INVALID_ARGUMENT, "channels (%lld) and out channels (%lld) must be divisible by groups (%lld)",
                    (long long)channels, (long long)out_channels, (long long)groups);
    int64_t Ho, Wo;
    int rc = unfold_out(height, width, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, Ho, Wo);
    if (rc) return rc;
    if (batch == 0 || out_channels == 0) return NTG_OK;
    if (!image || !kernel || !out) return fail(NTG_ERR_INVALID_ARGUMENT, "null pointer");
    const size_t im_bytes = (size_t)(batch * channels * height * width * es);
    const size_t k_bytes = (size_t)(out_channels * (channels / groups) * k_r * k_c * es);
    const size_t o_bytes = (size_t)(batch * out_channels * Ho * Wo * es);
    // Float32 at the reference's seam: the gathering kernels (no workspace), whose k axis is im2col's own -- the result is
    // unfold + matmult bit for bit (conv.cpp:86-95); the channels-last kernels sum the same products taps-outermost, and what
    // they would gain is small beside the transfers of this call.  The other dtypes take the faster form.
    const int64_t ws = dtype == ntg::DT_F32
        ? ntg_conv2d_forward_workspace_bytes(dtype, batch, channels, height, width, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c)
        : ntg_conv2d_fast_workspace_bytes(dtype, batch, channels, height, width, out_channels, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, groups);
    if (ws < 0) return fail(NTG_ERR_INVALID_ARGUMENT, "the array of sliding blocks would be empty");
    ntg::HostSession mem;
    const size_t ok_ = align_up(im_bytes, 256), oo = ok_ + align_up(k_bytes, 256), ow = oo + align_up(o_bytes, 256);
    HIP_TRY(mem.reserve(ow + (size_t)ws));
    if (im_bytes) HIP_TRY(mem.upload(0, image, im_bytes));
    if (k_bytes) HIP_TRY(mem.upload(ok_, kernel, k_bytes));
    rc = ntg_conv2d_dev(dtype, mem.at(0), mem.at(ok_), mem.at(oo), mem.at(ow), ws, batch, channels, height, width,
                        out_channels, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, groups, mem.stream());
    if (rc) return rc;
    HIP_TRY(mem.download(out, oo, o_bytes));
    return NTG_OK;
}

int ntg_unfold2d_backward_dev(int dtype, const void* col, void* image,
                              int64_t batch, int64_t channels, int64_t height, int64_t width,
                              int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c,
                              int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c, int accumulate, void* stream) {
    const int64_t es = ntg::elem_size(dtype);
    if (es == 0) return fail(NTG_ERR_UNSUPPORTED_DTYPE, "dtype %d is not supported", dtype);
    if (batch < 0 || channels < 0 || height < 0 || width < 0) return fail(NTG_ERR_INVALID_ARGUMENT, "negative size");
    int64_t Ho, Wo;
    int rc = unfold_out(height, width, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, Ho, Wo);
    if (rc) return rc;
    if (batch == 0 || channels == 0) return NTG_OK;
    if (!col || !image) return fail(NTG_ERR_INVALID_ARGUMENT, "null pointer");
    hipError_t e = ntg::launch_col2im(dtype, col, image, batch, channels, height, width, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c,
                                      accumulate, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(e, "col2im launch");
    return NTG_OK;
}

int ntg_unfold2d_backward(int dtype, const void* col, void* image,
                          int64_t batch, int64_t channels, int64_t height, int64_t width,
                          int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c,
                          int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c, int accumulate) {
    const int64_t es = ntg::elem_size(dtype);
    if (es == 0) return fail(NTG_ERR_UNSUPPORTED_DTYPE, "dtype %d is not supported", dtype);
    if (batch < 0 || channels < 0 || height < 0 || width < 0) return fail(NTG_ERR_INVALID_ARGUMENT, "negative size");
    int64_t Ho, Wo;
    int rc = unfold_out(height, width, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, Ho, Wo);
    if (rc) return rc;
    if (batch == 0 || channels == 0) return NTG_OK;
    if (!col || !image) return fail(NTG_ERR_INVALID_ARGUMENT, "null pointer");
    const size_t im_bytes = (size_t)(batch * channels * height * width * es);
    const size_t col_bytes = (size_t)(batch * channels * k_r * k_c * Ho * Wo * es);
    ntg::HostSession mem;
    const size_t oc = align_up(im_bytes, 256);
    HIP_TRY(mem.reserve(oc + col_bytes));
    if (accumulate) HIP_TRY(mem.upload(0, image, im_bytes));
    HIP_TRY(mem.upload(oc, col, col_bytes));
    rc = ntg_unfold2d_backward_dev(dtype, mem.at(oc), mem.at(0), batch, channels, height, width, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c,
                                   accumulate, mem.stream());
    if (rc) return rc;
    HIP_TRY(mem.download(image, 0, im_bytes));
    return NTG_OK;
}

static ConvBackwardPlan plan_conv_backward(int dtype, bool want_dx, bool want_dw, int64_t batch, int64_t channels, int64_t height, int64_t width,
                                           int64_t out_channels, int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c, int64_t p_r, int64_t p_c,
                                           int64_t d_r, int64_t d_c, int64_t groups, int64_t Ho, int64_t Wo, bool reference_order = false) {
    return plan_conv_backward_g(dtype, want_dx, want_dw, batch, channels, out_channels,
                                geo2(height, width, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, Ho, Wo), groups, reference_order);
}

int64_t ntg_conv2d_backward_workspace_bytes(int dtype, int64_t batch, int64_t channels, int64_t height, int64_t width,
                                            int64_t out_channels, int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c,
                                            int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c, int64_t groups) {
    int64_t Ho, Wo;
    if (ntg::elem_size(dtype) == 0 || groups < 1 || channels % groups != 0 || out_channels % groups != 0 ||
        unfold_out(height, width, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, Ho, Wo)) return -1;
    // the larger of what the call needs at least and what lets dX take its channels-last form (copy of dY + flipped weights)
    const ConvBackwardPlan pl = plan_conv_backward(dtype, true, true, batch, channels, height, width, out_channels, k_r, k_c, s_r, s_c, p_r, p_c,
                                                   d_r, d_c, groups, Ho, Wo);
    return std::max(std::max(pl.need, pl.need_phase_dx), std::max(pl.need_nhwc_dx, pl.need_nhwc_dw));
}

static int conv2d_backward_dev_impl(int dtype, const void* image, const void* kernel, const void* grad_out,
                                    void* d_image, void* d_kernel, void* workspace, int64_t workspace_bytes,
                                    int64_t batch, int64_t channels, int64_t height, int64_t width,
                                    int64_t out_channels, int64_t k_r, int64_t k_c,
                                    int64_t s_r, int64_t s_c, int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c,
                                    int64_t groups, int accumulate, void* stream, bool reference_order) {
    const int64_t es = ntg::elem_size(dtype);
    if (es == 0) return fail(NTG_ERR_UNSUPPORTED_DTYPE, "dtype %d is not supported", dtype);
    if (batch < 0 || channels < 0 || out_channels < 0 || height < 0 || width < 0) return fail(NTG_ERR_INVALID_ARGUMENT, "negative size");
    if (groups < 1 || channels % groups != 0 || out_channels % groups != 0)
        return fail(NTG_ERR_INVALID_ARGUMENT, "channels (%lld) and out channels (%lld) must be divisible by groups (%lld)",
                    (long long)channels, (long long)out_channels, (long long)groups);
    int64_t Ho, Wo;
    int rc = unfold_out(height, width, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, Ho, Wo);
    if (rc) return rc;
    if (batch == 0 || out_channels == 0 || channels == 0) return NTG_OK;
    if (!kernel || !grad_out || (d_kernel && !image)) return fail(NTG_ERR_INVALID_ARGUMENT, "null pointer");
    const int64_t L = Ho * Wo, ckk = channels * k_r * k_c;
    const int64_t add = (channels / groups) * k_r * k_c, og = out_channels / groups;
    const ConvBackwardPlan plan = plan_conv_backward(dtype, d_image != nullptr, d_kernel != nullptr, batch, channels, height, width,
                                                     out_channels, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, groups, Ho, Wo, reference_order);
    if (plan.need > 0 && (!workspace || workspace_bytes < plan.need))
        return fail(NTG_ERR_INVALID_ARGUMENT, "workspace of %lld bytes needed, %lld given", (long long)plan.need, (long long)workspace_bytes);
    const char* kern = static_cast<const char*>(kernel);
    const char* gy = static_cast<const char*>(grad_out);
    char* ws = static_cast<char*>(workspace);
    hipStream_t hs = static_cast<hipStream_t>(stream);
    ntg_gemm_desc d;
    // Floating dtypes: neither gradient needs the stored im2col matrix (conv_dkernel_gather, conv_dimage_gather).
    bool gather_dw = plan.gather_dw, gather_dx = plan.gather_dx;
    const Geo3 geo = geo2(height, width, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, Ho, Wo);
    // 1x1 kernel, unit stride, no padding (floating dtypes, 16-byte rows): col is the image itself, so both gradients are
    // products on the tensors where they lie: dX_b = W_g^T . dY_b, and dW_g = sum_b dY_b . X_b^T through per-image results
    // in the workspace (the amount the gathering form needs), summed in batch order.
    if (!is_valu_dtype(dtype) && !(reference_order && accumulate) && conv_pointwise_ok(dtype, channels, groups, geo) && (og * es) % 16 == 0 &&
        ((reinterpret_cast<uintptr_t>(image) | reinterpret_cast<uintptr_t>(kernel) | reinterpret_cast<uintptr_t>(grad_out) |
          reinterpret_cast<uintptr_t>(d_image) | reinterpret_cast<uintptr_t>(d_kernel) | reinterpret_cast<uintptr_t>(ws)) & 15) == 0) {
        const int64_t cg = channels / groups;
        for (int64_t g = 0; g < groups && d_image; ++g) {
            std::memset(&d, 0, sizeof d);
            d.dtype = dtype; d.transpose_a = 1; d.c_mode = accumulate ? NTG_C_ACCUMULATE : NTG_C_OVERWRITE;
            d.m = cg; d.k = og; d.n = L; d.batches = batch;
            d.stride_a = 0; d.stride_b = out_channels * L; d.stride_c = channels * L;
            rc = ntg_gemm_dev(&d, kern + g * og * cg * es, gy + g * og * L * es, static_cast<char*>(d_image) + g * cg * L * es, stream);
            if (rc) return rc;
        }
        for (int64_t g = 0; g < groups && d_kernel; ++g) {
            std::memset(&d, 0, sizeof d);
            d.dtype = dtype; d.transpose_b = 1; d.c_mode = NTG_C_OVERWRITE;
            d.m = og; d.k = L; d.n = cg; d.batches = batch;
            d.stride_a = out_channels * L; d.stride_b = channels * L; d.stride_c = out_channels * cg;
            rc = ntg_gemm_dev(&d, gy + g * og * L * es, static_cast<const char*>(image) + g * cg * L * es, ws + g * og * cg * es, stream);
            if (rc) return rc;
        }
        if (d_kernel) {
            hipError_t e = ntg::launch_reduce_batch(dtype, ws, d_kernel, batch, out_channels * cg, accumulate, hs);
            if (e != hipSuccess) return hip_fail(e, "weight gradient reduction launch");
        }
        return NTG_OK;
    }
    if (gather_dw) {
        if (plan.nhwc_dw && workspace_bytes >= plan.need_nhwc_dw && ((reinterpret_cast<uintptr_t>(ws) | reinterpret_cast<uintptr_t>(grad_out)) & 15) == 0)
            rc = conv_dkernel_nhwc(dtype, image, grad_out, d_kernel, ws, batch, channels, out_channels, geo, groups, accumulate, hs);
        else
            rc = conv_dkernel_gather(dtype, image, grad_out, d_kernel, ws, batch, channels, out_channels, geo, groups, accumulate, hs);
        if (rc) return rc;
    }
    if (gather_dx) {
        if (plan.nhwc_dx && workspace_bytes >= plan.need_nhwc_dx && (reinterpret_cast<uintptr_t>(ws) & 15) == 0)
            rc = conv_dimage_nhwc(dtype, kernel, grad_out, d_image, ws, batch, channels, out_channels, geo, groups, accumulate, hs);
        else
            rc = conv_dimage_gather(dtype, kernel, grad_out, d_image, ws, batch, channels, out_channels, geo, groups, accumulate, hs);
        if (rc) return rc;
    }
    if (gather_dw) d_kernel = nullptr;    // done
    if (gather_dx) d_image = nullptr;
    if (d_image && plan.phase_dx && workspace_bytes >= plan.need_phase_dx && (reinterpret_cast<uintptr_t>(ws) & 15) == 0) {
        rc = conv_dimage_phases(dtype, plan.phases, kernel, grad_out, d_image, ws, batch, channels, out_channels, geo, groups, accumulate, hs);
        if (rc) return rc;
        d_image = nullptr;
    }
    if (d_kernel) {
        // col = im2col(image); per group g:  dW_g [og, add] (+)= sum_b dY_{b,g} [og, L] . col_{b,g}^T  (col_{b,g} stored [add, L])
        rc = ntg_unfold2d_dev(dtype, image, ws, batch, channels, height, width, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, stream);
        if (rc) return rc;
        rc = conv_dkernel_from_col(dtype, gy, ws, d_kernel, batch, out_channels, ckk, groups, L, accumulate, stream);
        if (rc) return rc;
    }
    if (d_image) {
        // d_col_{b,g} [add, L] = W_g^T . dY_{b,g}   (W_g stored [og, add] -> transpose_a), then col2im
        for (int64_t g = 0; g < groups; ++g) {
            std::memset(&d, 0, sizeof d);
            d.dtype = dtype; d.transpose_a = 1; d.c_mode = NTG_C_OVERWRITE;
            d.m = add; d.k = og; d.n = L;
            d.lda = add; d.ldb = L; d.ldc = L; d.batches = batch;
            d.stride_a = 0; d.stride_b = out_channels * L; d.stride_c = ckk * L;
            rc = ntg_gemm_dev(&d, kern + g * og * add * es, gy + g * og * L * es, ws + g * add * L * es, stream);
            if (rc) return rc;
        }
        rc = ntg_unfold2d_backward_dev(dtype, ws, d_image, batch, channels, height, width, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c,
                                       accumulate, stream);
        if (rc) return rc;
    }
    return NTG_OK;
}

int ntg_conv2d_backward_dev(int dtype, const void* image, const void* kernel, const void* grad_out,
                            void* d_image, void* d_kernel, void* workspace, int64_t workspace_bytes,
                            int64_t batch, int64_t channels, int64_t height, int64_t width,
                            int64_t out_channels, int64_t k_r, int64_t k_c,
                            int64_t s_r, int64_t s_c, int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c,
                            int64_t groups, int accumulate, void* stream) {
    return conv2d_backward_dev_impl(dtype, image, kernel, grad_out, d_image, d_kernel, workspace, workspace_bytes, batch, channels, height, width,
                                    out_channels, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, groups, accumulate, stream, false);
}

// conv_transpose2d = the image gradient of the convolution whose output is `input`: per group
// out_g [cog, Rout*Cout] = flipped, channel-swapped kernel . unfold(zero-dilated input), which is what
// the reference forms explicitly (conv.cpp:614-676: dilate by stride, pad by output_padding, unfold2d
// with padding d*(k-1) - p and stride 1, matmult with w.transpose(0,1).flip).  Here it is the
// conv_dimage path of ntg_conv2d_backward_dev with the roles renamed; kernel is [in_channels,
// out_channels/groups, k_r, k_c] as in the reference.
static int conv_transpose_out(int64_t in_h, int64_t in_w, int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c, int64_t p_r, int64_t p_c,
                              int64_t d_r, int64_t d_c, int64_t op_r, int64_t op_c, int64_t& out_h, int64_t& out_w) {
    if (k_r < 1 || k_c < 1) return fail(NTG_ERR_INVALID_ARGUMENT, "kernel size must be >= 1");
    if (s_r < 1 || s_c < 1) return fail(NTG_ERR_INVALID_ARGUMENT, "Conv2d Transpose stride cannot be less than 1 but got (%lld, %lld)", (long long)s_r, (long long)s_c);
    if (d_r < 1 || d_c < 1) return fail(NTG_ERR_INVALID_ARGUMENT, "Conv2d Transpose dilation cannot be less than 1 but got (%lld, %lld)", (long long)d_r, (long long)d_c);
    if (p_r < 0 || p_c < 0) return fail(NTG_ERR_INVALID_ARGUMENT, "Conv2d Transpose padding cannot be less than 0 but got (%lld, %lld)", (long long)p_r, (long long)p_c);
    if (op_r < 0 || op_c < 0) return fail(NTG_ERR_INVALID_ARGUMENT, "Conv2d Transpose output_padding cannot be less than 0 but got (%lld, %lld)", (long long)op_r, (long long)op_c);
    // the reference accepts any output_padding; rows past the reach of the kernel would be zero.  This backend needs the
    // forward convolution of the result to reproduce the input size, which holds for output_padding < stride.
    if (op_r >= s_r || op_c >= s_c) return fail(NTG_ERR_INVALID_ARGUMENT, "output_padding (%lld, %lld) must be smaller than stride (%lld, %lld)",
                                                (long long)op_r, (long long)op_c, (long long)s_r, (long long)s_c);
    if (in_h < 1 || in_w < 1) return fail(NTG_ERR_INVALID_ARGUMENT, "empty input");
    out_h = (in_h - 1) * s_r - 2 * p_r + d_r * (k_r - 1) + 1 + op_r;
    out_w = (in_w - 1) * s_c - 2 * p_c + d_c * (k_c - 1) + 1 + op_c;
    if (out_h < 1 || out_w < 1) return fail(NTG_ERR_INVALID_ARGUMENT, "the output of the transposed convolution would be empty");
    // a padding wider than the kernel reach would make the matching convolution read fewer input rows than exist
    if ((out_h + 2 * p_r - d_r * (k_r - 1) - 1) / s_r + 1 != in_h || (out_w + 2 * p_c - d_c * (k_c - 1) - 1) / s_c + 1 != in_w)
        return fail(NTG_ERR_INVALID_ARGUMENT, "geometry is not the transpose of a convolution");
    return NTG_OK;
}

int64_t ntg_conv_transpose2d_workspace_bytes(int dtype, int64_t batch, int64_t in_channels, int64_t in_h, int64_t in_w,
                                             int64_t out_channels, int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c,
                                             int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c, int64_t op_r, int64_t op_c, int64_t groups) {
    int64_t oh, ow, Ho, Wo;
    if (ntg::elem_size(dtype) == 0 || groups < 1 || in_channels % groups != 0 || out_channels % groups != 0 ||
        conv_transpose_out(in_h, in_w, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, op_r, op_c, oh, ow) ||
        unfold_out(oh, ow, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, Ho, Wo)) return -1;
    const ConvBackwardPlan pl = plan_conv_backward(dtype, true, false, batch, out_channels, oh, ow, in_channels, k_r, k_c, s_r, s_c, p_r, p_c,
                                                   d_r, d_c, groups, Ho, Wo);
    return std::max(pl.need, std::max(pl.need_nhwc_dx, pl.need_phase_dx));      // (the larger amount lets it run channels-last)
}

int ntg_conv_transpose2d_dev(int dtype, const void* input, const void* kernel, void* out, void* workspace, int64_t workspace_bytes,
                             int64_t batch, int64_t in_channels, int64_t in_h, int64_t in_w, int64_t out_channels,
                             int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c, int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c,
                             int64_t op_r, int64_t op_c, int64_t groups, void* stream) {
    if (ntg::elem_size(dtype) == 0) return fail(NTG_ERR_UNSUPPORTED_DTYPE, "dtype %d is not supported", dtype);
    if (batch < 0 || in_channels < 0 || out_channels < 0) return fail(NTG_ERR_INVALID_ARGUMENT, "negative size");
    if (groups < 1) return fail(NTG_ERR_INVALID_ARGUMENT, "groups must be >= 1");
    if (in_channels % groups != 0)
        return fail(NTG_ERR_INVALID_ARGUMENT, "Expected image channels to be divisible by groups in Conv2d Transpose but got %lld %% %lld != 0",
                    (long long)in_channels, (long long)groups);
    if (out_channels % groups != 0) return fail(NTG_ERR_INVALID_ARGUMENT, "out channels (%lld) not divisible by groups (%lld)", (long long)out_channels, (long long)groups);
    int64_t oh, ow;
    int rc = conv_transpose_out(in_h, in_w, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, op_r, op_c, oh, ow);
    if (rc) return rc;
    if (batch == 0 || out_channels == 0) return NTG_OK;
    if (in_channels == 0) {
        hipError_t e = ntg::launch_col2im(dtype, nullptr, out, batch, out_channels, oh, ow, 0, 0, 1, 1, 0, 0, 1, 1, 0, static_cast<hipStream_t>(stream));
        if (e != hipSuccess) return hip_fail(e, "zero fill");
        return NTG_OK;
    }
    return ntg_conv2d_backward_dev(dtype, nullptr, kernel, input, out, nullptr, workspace, workspace_bytes, batch, out_channels, oh, ow,
                                   in_channels, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, groups, 0, stream);
}

int ntg_conv_transpose2d(int dtype, const void* input, const void* kernel, void* out,
                         int64_t batch, int64_t in_channels, int64_t in_h, int64_t in_w, int64_t out_channels,
                         int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c, int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c,
                         int64_t op_r, int64_t op_c, int64_t groups) {
    const int64_t es = ntg::elem_size(dtype);
    if (es == 0) return fail(NTG_ERR_UNSUPPORTED_DTYPE, "dtype %d is not supported", dtype);
    if (batch < 0 || in_channels < 0 || out_channels < 0) return fail(NTG_ERR_INVALID_ARGUMENT, "negative size");
    if (groups < 1 || in_channels % groups != 0 || out_channels % groups != 0)
        return fail(NTG_ERR_INVALID_ARGUMENT, "channels (%lld) and out channels (%lld) must be divisible by groups (%lld)",
                    (long long)in_channels, (long long)out_channels, (long long)groups);
    int64_t oh, ow;
    int rc = conv_transpose_out(in_h, in_w, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, op_r, op_c, oh, ow);
    if (rc) return rc;
    if (batch == 0 || out_channels == 0) return NTG_OK;
    if (!input || !kernel || !out) return fail(NTG_ERR_INVALID_ARGUMENT, "null pointer");
    const size_t in_bytes = (size_t)(batch * in_channels * in_h * in_w * es);
    const size_t k_bytes = (size_t)(in_channels * (out_channels / groups) * k_r * k_c * es);
    const size_t o_bytes = (size_t)(batch * out_channels * oh * ow * es);
    const int64_t wsb = ntg_conv_transpose2d_workspace_bytes(dtype, batch, in_channels, in_h, in_w, out_channels, k_r, k_c, s_r, s_c,
                                                             p_r, p_c, d_r, d_c, op_r, op_c, groups);
    if (wsb < 0) return fail(NTG_ERR_INVALID_ARGUMENT, "invalid geometry");
    ntg::HostSession mem;
    const size_t o_k = align_up(in_bytes, 256), o_o = o_k + align_up(k_bytes, 256), o_ws = o_o + align_up(o_bytes, 256);
    HIP_TRY(mem.reserve(o_ws + (size_t)wsb));
    if (in_bytes) HIP_TRY(mem.upload(0, input, in_bytes));
    if (k_bytes) HIP_TRY(mem.upload(o_k, kernel, k_bytes));
    rc = ntg_conv_transpose2d_dev(dtype, mem.at(0), mem.at(o_k), mem.at(o_o), mem.at(o_ws), wsb, batch, in_channels, in_h, in_w, out_channels,
                                  k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, op_r, op_c, groups, mem.stream());
    if (rc) return rc;
    HIP_TRY(mem.download(out, o_o, o_bytes));
    return NTG_OK;
}

int ntg_conv2d_backward(int dtype, const void* image, const void* kernel, const void* grad_out,
                        void* d_image, void* d_kernel,
                        int64_t batch, int64_t channels, int64_t height, int64_t width,
                        int64_t out_channels, int64_t k_r, int64_t k_c,
                        int64_t s_r, int64_t s_c, int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c,
                        int64_t groups, int accumulate) {
    const int64_t es = ntg::elem_size(dtype);
    if (es == 0) return fail(NTG_ERR_UNSUPPORTED_DTYPE, "dtype %d is not supported", dtype);
    if (batch < 0 || channels < 0 || out_channels < 0 || height < 0 || width < 0) return fail(NTG_ERR_INVALID_ARGUMENT, "negative size");
    if (groups < 1 || channels % groups != 0 || out_channels % groups != 0)
        return fail(NTG_ERR_INVALID_ARGUMENT, "channels (%lld) and out channels (%lld) must be divisible by groups (%lld)",
                    (long long)channels, (long long)out_channels, (long long)groups);
    int64_t Ho, Wo;
    int rc = unfold_out(height, width, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, Ho, Wo);
    if (rc) return rc;
    if (batch == 0 || out_channels == 0 || channels == 0) return NTG_OK;
    if (!image || !kernel || !grad_out) return fail(NTG_ERR_INVALID_ARGUMENT, "null pointer");
    const size_t im_bytes = (size_t)(batch * channels * height * width * es);
    const size_t k_bytes = (size_t)(out_channels * (channels / groups) * k_r * k_c * es);
    const size_t g_bytes = (size_t)(batch * out_channels * Ho * Wo * es);
    // Float32 at the reference's seam: its own two algorithms (see plan_conv_backward_g), whose results are conv_dimage's and
    // conv_dkernel's bit for bit; what the faster forms would gain is small beside the transfers of this call
    const bool reference_order = dtype == ntg::DT_F32;
    const int64_t wsb = reference_order
        ? plan_conv_backward(dtype, d_image != nullptr, d_kernel != nullptr, batch, channels, height, width, out_channels, k_r, k_c, s_r, s_c,
                             p_r, p_c, d_r, d_c, groups, Ho, Wo, true).need
        : ntg_conv2d_backward_workspace_bytes(dtype, batch, channels, height, width, out_channels, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, groups);
    ntg::HostSession mem;
    const size_t o_k = align_up(im_bytes, 256), o_g = o_k + align_up(k_bytes, 256), o_di = o_g + align_up(g_bytes, 256);
    const size_t o_dk = o_di + align_up(im_bytes, 256), o_ws = o_dk + align_up(k_bytes, 256);
    HIP_TRY(mem.reserve(o_ws + (size_t)wsb));
    HIP_TRY(mem.upload(0, image, im_bytes));
    HIP_TRY(mem.upload(o_k, kernel, k_bytes));
    HIP_TRY(mem.upload(o_g, grad_out, g_bytes));
    if (accumulate && d_image) HIP_TRY(mem.upload(o_di, d_image, im_bytes));
    if (accumulate && d_kernel) HIP_TRY(mem.upload(o_dk, d_kernel, k_bytes));
    rc = conv2d_backward_dev_impl(dtype, mem.at(0), mem.at(o_k), mem.at(o_g), d_image ? mem.at(o_di) : nullptr,
                                  d_kernel ? mem.at(o_dk) : nullptr, mem.at(o_ws), wsb, batch, channels, height, width, out_channels,
                                  k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, groups, accumulate, mem.stream(), reference_order);
    if (rc) return rc;
    if (d_image) HIP_TRY(mem.download(d_image, o_di, im_bytes));
    if (d_kernel) HIP_TRY(mem.download(d_kernel, o_dk, k_bytes));
    return NTG_OK;
}

// ---------------------------------------------------------------------------------------------------
// Convolutions over 1..4 spatial axes (conv3d conv.cpp:122-175, convnd :177-316, their gradients :347, :472 and
// conv_transpose3d / conv_transposend :678-905): unfold -> matmult like the reference.  One and two axes go to
// the 2-d entry points above (implicit GEMM); three and four axes store the unfolded matrix.
// Geometry arrays hold `ndim` entries, slowest axis first (depth, rows, columns).
static int fill_nd(ntg::UnfoldNdParams& u, int64_t batch, int64_t channels, int ndim, const int64_t* size, const int64_t* k,
                   const int64_t* s, const int64_t* p, const int64_t* d) {
    if (ndim < 1 || ndim > NTG_MAX_SPATIAL) return fail(NTG_ERR_INVALID_ARGUMENT, "ndim must be 1..%d but got %d", NTG_MAX_SPATIAL, ndim);
    if (!size || !k || !s || !p || !d) return fail(NTG_ERR_INVALID_ARGUMENT, "null geometry array");
    if (batch < 0 || channels < 0) return fail(NTG_ERR_INVALID_ARGUMENT, "negative size");
    std::memset(&u, 0, sizeof u);
    u.nd = ndim; u.batch = batch; u.channels = channels;
    u.taps = 1; u.L = 1; u.vol = 1;
    for (int a = 0; a < ndim; ++a) {
        if (size[a] < 0) return fail(NTG_ERR_INVALID_ARGUMENT, "negative size");
        if (k[a] < 1 || s[a] < 1 || d[a] < 1 || p[a] < 0) return fail(NTG_ERR_INVALID_ARGUMENT, "kernel/stride/dilation must be >= 1 and padding >= 0");
        const int64_t span = size[a] + 2 * p[a] - d[a] * (k[a] - 1) - 1;
        const int64_t o = span / s[a] + 1;
        if (span < 0 || o <= 0) return fail(NTG_ERR_INVALID_ARGUMENT, "the array of sliding blocks would be empty (axis %d)", a);
        u.size[a] = size[a]; u.k[a] = k[a]; u.s[a] = s[a]; u.p[a] = p[a]; u.d[a] = d[a]; u.out[a] = o;
        u.taps *= k[a]; u.L *= o; u.vol *= size[a];
    }
    u.ccol = channels * u.taps;
    u.total = batch * u.ccol * u.L;
    return NTG_OK;
}

// trailing two axes of a 1- or 2-axis geometry as (rows, columns) for the 2-d entry points
struct Geo2 { int64_t h, w, kr, kc, sr, sc, pr, pc, dr, dc; };
static Geo2 as_2d(int ndim, const int64_t* size, const int64_t* k, const int64_t* s, const int64_t* p, const int64_t* d) {
    if (ndim == 1) return {1, size[0], 1, k[0], 1, s[0], 0, p[0], 1, d[0]};
    return {size[0], size[1], k[0], k[1], s[0], s[1], p[0], p[1], d[0], d[1]};
}

static Geo3 geo_from(const ntg::UnfoldNdParams& u) {
    Geo3 g{3, {1, 1, 1}, {1, 1, 1}, {1, 1, 1}, {0, 0, 0}, {1, 1, 1}, {1, 1, 1}};
    for (int a = 0; a < 3; ++a) { g.sz[a] = u.size[a]; g.k[a] = u.k[a]; g.s[a] = u.s[a]; g.p[a] = u.p[a]; g.d[a] = u.d[a]; g.o[a] = u.out[a]; }
    return g;
}

int ntg_unfoldnd_dev(int dtype, const void* image, void* col, int64_t batch, int64_t channels, int ndim, const int64_t* size,
                     const int64_t* kernel_size, const int64_t* stride, const int64_t* padding, const int64_t* dilation, void* stream) {
    const int64_t es = ntg::elem_size(dtype);
    if (es == 0) return fail(NTG_ERR_UNSUPPORTED_DTYPE, "dtype %d is not supported", dtype);
    ntg::UnfoldNdParams u;
    int rc = fill_nd(u, batch, channels, ndim, size, kernel_size, stride, padding, dilation);
    if (rc) return rc;
    if (u.total == 0) return NTG_OK;
    if (!image || !col) return fail(NTG_ERR_INVALID_ARGUMENT, "null pointer");
    hipError_t e = ntg::launch_unfoldnd(es, image, col, u, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(e, "unfoldnd launch");
    return NTG_OK;
}

int ntg_unfoldnd_backward_dev(int dtype, const void* col, void* image, int64_t batch, int64_t channels, int ndim, const int64_t* size,
                              const int64_t* kernel_size, const int64_t* stride, const int64_t* padding, const int64_t* dilation,
                              int accumulate, void* stream) {
    if (ntg::elem_size(dtype) == 0) return fail(NTG_ERR_UNSUPPORTED_DTYPE, "dtype %d is not supported", dtype);
    ntg::UnfoldNdParams u;
    int rc = fill_nd(u, batch, channels, ndim, size, kernel_size, stride, padding, dilation);
    if (rc) return rc;
    if (batch * channels * u.vol == 0) return NTG_OK;
    if (!image || !col) return fail(NTG_ERR_INVALID_ARGUMENT, "null pointer");
    hipError_t e = ntg::launch_col2imnd(dtype, col, image, u, accumulate, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(e, "col2imnd launch");
    return NTG_OK;
}

static int check_groups(int64_t channels, int64_t out_channels, int64_t groups) {
    if (channels < 0 || out_channels < 0) return fail(NTG_ERR_INVALID_ARGUMENT, "negative size");
    if (groups < 1) return fail(NTG_ERR_INVALID_ARGUMENT, "groups must be >= 1");
    if (channels % groups != 0) return fail(NTG_ERR_INVALID_ARGUMENT, "image channels (%lld) not divisible by groups (%lld)", (long long)channels, (long long)groups);
    if (out_channels % groups != 0) return fail(NTG_ERR_INVALID_ARGUMENT, "out channels (%lld) not divisible by groups (%lld)", (long long)out_channels, (long long)groups);
    return NTG_OK;
}

int64_t ntg_convnd_workspace_bytes(int dtype, int64_t batch, int64_t channels, int64_t out_channels, int ndim, const int64_t* size,
                                   const int64_t* kernel_size, const int64_t* stride, const int64_t* padding, const int64_t* dilation,
                                   int64_t groups, int backward) {
    const int64_t es = ntg::elem_size(dtype);
    ntg::UnfoldNdParams u;
    if (es == 0 || check_groups(channels, out_channels, groups) || fill_nd(u, batch, channels, ndim, size, kernel_size, stride, padding, dilation)) return -1;
    if (ndim <= 2) {
        const Geo2 g = as_2d(ndim, size, kernel_size, stride, padding, dilation);
        return backward ? ntg_conv2d_backward_workspace_bytes(dtype, batch, channels, g.h, g.w, out_channels, g.kr, g.kc, g.sr, g.sc, g.pr, g.pc, g.dr, g.dc, groups)
                        : ntg_conv2d_forward_workspace_bytes(dtype, batch, channels, g.h, g.w, g.kr, g.kc, g.sr, g.sc, g.pr, g.pc, g.dr, g.dc);
    }
    if (ndim == 3) {
        const Geo3 g = geo_from(u);
        if (backward) return plan_conv_backward_g(dtype, true, true, batch, channels, out_channels, g, groups).need;
        if (conv_implicit_g(dtype, channels, g)) return 0;
    }
    return u.total * es + (backward ? complex_dkernel_extra(dtype, batch, out_channels, (channels / groups) * u.taps, u.total * es) : 0);
}

int ntg_convnd_dev(int dtype, const void* image, const void* kernel, void* out, void* workspace, int64_t workspace_bytes,
                   int64_t batch, int64_t channels, int64_t out_channels, int ndim, const int64_t* size, const int64_t* kernel_size,
                   const int64_t* stride, const int64_t* padding, const int64_t* dilation, int64_t groups, void* stream) {
    const int64_t es = ntg::elem_size(dtype);
    if (es == 0) return fail(NTG_ERR_UNSUPPORTED_DTYPE, "dtype %d is not supported", dtype);
    int rc = check_groups(channels, out_channels, groups);
    if (rc) return rc;
    ntg::UnfoldNdParams u;
    rc = fill_nd(u, batch, channels, ndim, size, kernel_size, stride, padding, dilation);
    if (rc) return rc;
    if (ndim <= 2) {
        const Geo2 g = as_2d(ndim, size, kernel_size, stride, padding, dilation);
        return ntg_conv2d_dev(dtype, image, kernel, out, workspace, workspace_bytes, batch, channels, g.h, g.w, out_channels, g.kr, g.kc,
                              g.sr, g.sc, g.pr, g.pc, g.dr, g.dc, groups, stream);
    }
    if (batch == 0 || out_channels == 0) return NTG_OK;
    if (!image || !kernel || !out) return fail(NTG_ERR_INVALID_ARGUMENT, "null pointer");
    if (ndim == 3) {
        const Geo3 g = geo_from(u);
        if (conv_implicit_g(dtype, channels, g))      // three axes, floating dtype: gathered inside the GEMM, no col buffer
            return conv_forward_gather(dtype, image, kernel, out, batch, channels, out_channels, g, groups, static_cast<hipStream_t>(stream));
    }
    const int64_t need = u.total * es;
    if (need > 0 && (!workspace || workspace_bytes < need))
        return fail(NTG_ERR_INVALID_ARGUMENT, "workspace of %lld bytes needed, %lld given", (long long)need, (long long)workspace_bytes);
    hipError_t e = ntg::launch_unfoldnd(es, image, workspace, u, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(e, "unfoldnd launch");
    // out_b[g*og:(g+1)*og, L] = W_g[og, add] . col_b[g*add:(g+1)*add, L]   (the reference's (col^T . W^T)^T, conv.cpp:143, :171)
    const int64_t add = (channels / groups) * u.taps, og = out_channels / groups;
    for (int64_t g = 0; g < groups; ++g) {
        ntg_gemm_desc d;
        std::memset(&d, 0, sizeof d);
        d.dtype = dtype; d.c_mode = NTG_C_OVERWRITE;
        d.m = og; d.k = add; d.n = u.L;
        d.lda = add; d.ldb = u.L; d.ldc = u.L;
        d.batches = batch;
        d.stride_a = 0; d.stride_b = u.ccol * u.L; d.stride_c = out_channels * u.L;
        rc = ntg_gemm_dev(&d, static_cast<const char*>(kernel) + g * og * add * es, static_cast<const char*>(workspace) + g * add * u.L * es,
                          static_cast<char*>(out) + g * og * u.L * es, stream);
        if (rc) return rc;
    }
    return NTG_OK;
}

int ntg_convnd_backward_dev(int dtype, const void* image, const void* kernel, const void* grad_out, void* d_image, void* d_kernel,
                            void* workspace, int64_t workspace_bytes, int64_t batch, int64_t channels, int64_t out_channels, int ndim,
                            const int64_t* size, const int64_t* kernel_size, const int64_t* stride, const int64_t* padding,
                            const int64_t* dilation, int64_t groups, int accumulate, void* stream) {
    const int64_t es = ntg::elem_size(dtype);
    if (es == 0) return fail(NTG_ERR_UNSUPPORTED_DTYPE, "dtype %d is not supported", dtype);
    int rc = check_groups(channels, out_channels, groups);
    if (rc) return rc;
    ntg::UnfoldNdParams u;
    rc = fill_nd(u, batch, channels, ndim, size, kernel_size, stride, padding, dilation);
    if (rc) return rc;
    if (ndim <= 2) {
        const Geo2 g = as_2d(ndim, size, kernel_size, stride, padding, dilation);
        return ntg_conv2d_backward_dev(dtype, image, kernel, grad_out, d_image, d_kernel, workspace, workspace_bytes, batch, channels, g.h, g.w,
                                       out_channels, g.kr, g.kc, g.sr, g.sc, g.pr, g.pc, g.dr, g.dc, groups, accumulate, stream);
    }
    if (batch == 0 || out_channels == 0 || channels == 0) return NTG_OK;
    if (!kernel || !grad_out || (d_kernel && !image)) return fail(NTG_ERR_INVALID_ARGUMENT, "null pointer");
    int64_t need = u.total * es + (d_kernel ? complex_dkernel_extra(dtype, batch, out_channels, (channels / groups) * u.taps, u.total * es) : 0);
    if (ndim == 3) {
        const Geo3 g = geo_from(u);
        const ConvBackwardPlan plan = plan_conv_backward_g(dtype, d_image != nullptr, d_kernel != nullptr, batch, channels, out_channels, g, groups);
        need = plan.need;
        if (need > 0 && (!workspace || workspace_bytes < need))
            return fail(NTG_ERR_INVALID_ARGUMENT, "workspace of %lld bytes needed, %lld given", (long long)need, (long long)workspace_bytes);
        if (plan.gather_dw) {
            rc = conv_dkernel_gather(dtype, image, grad_out, d_kernel, workspace, batch, channels, out_channels, g, groups, accumulate,
                                     static_cast<hipStream_t>(stream));
            if (rc) return rc;
            d_kernel = nullptr;
        }
        if (plan.gather_dx) {
            rc = conv_dimage_gather(dtype, kernel, grad_out, d_image, workspace, batch, channels, out_channels, g, groups, accumulate,
                                    static_cast<hipStream_t>(stream));
            if (rc) return rc;
            d_image = nullptr;
        }
        if (!d_kernel && !d_image) return NTG_OK;
    }
    if (!workspace || workspace_bytes < need)
        return fail(NTG_ERR_INVALID_ARGUMENT, "workspace of %lld bytes needed, %lld given", (long long)need, (long long)workspace_bytes);
    const int64_t L = u.L, add = (channels / groups) * u.taps, og = out_channels / groups;
    const char* kern = static_cast<const char*>(kernel);
    const char* gy = static_cast<const char*>(grad_out);
    char* ws = static_cast<char*>(workspace);
    ntg_gemm_desc d;
    if (d_kernel) {
        hipError_t e = ntg::launch_unfoldnd(es, image, ws, u, static_cast<hipStream_t>(stream));
        if (e != hipSuccess) return hip_fail(e, "unfoldnd launch");
        rc = conv_dkernel_from_col(dtype, gy, ws, d_kernel, batch, out_channels, u.ccol, groups, L, accumulate, stream);
        if (rc) return rc;
    }
    if (d_image) {
        for (int64_t g = 0; g < groups; ++g) {
            std::memset(&d, 0, sizeof d);
            d.dtype = dtype; d.transpose_a = 1; d.c_mode = NTG_C_OVERWRITE;
            d.m = add; d.k = og; d.n = L;
            d.lda = add; d.ldb = L; d.ldc = L; d.batches = batch;
            d.stride_a = 0; d.stride_b = out_channels * L; d.stride_c = u.ccol * L;
            rc = ntg_gemm_dev(&d, kern + g * og * add * es, gy + g * og * L * es, ws + g * add * L * es, stream);
            if (rc) return rc;
        }
        hipError_t e = ntg::launch_col2imnd(dtype, ws, d_image, u, accumulate, static_cast<hipStream_t>(stream));
        if (e != hipSuccess) return hip_fail(e, "col2imnd launch");
    }
    return NTG_OK;
}

// output size of the transposed convolution per axis; the geometry of the convolution it is the adjoint of
static int transpose_nd_out(int ndim, const int64_t* in_size, const int64_t* k, const int64_t* s, const int64_t* p, const int64_t* d,
                            const int64_t* op, int64_t* out_size) {
    if (ndim < 1 || ndim > NTG_MAX_SPATIAL) return fail(NTG_ERR_INVALID_ARGUMENT, "ndim must be 1..%d but got %d", NTG_MAX_SPATIAL, ndim);
    if (!in_size || !k || !s || !p || !d || !op) return fail(NTG_ERR_INVALID_ARGUMENT, "null geometry array");
    for (int a = 0; a < ndim; ++a) {
        if (k[a] < 1 || s[a] < 1 || d[a] < 1 || p[a] < 0 || op[a] < 0)
            return fail(NTG_ERR_INVALID_ARGUMENT, "kernel/stride/dilation must be >= 1 and padding/output_padding >= 0");
        if (op[a] >= s[a]) return fail(NTG_ERR_INVALID_ARGUMENT, "output_padding (%lld) must be smaller than stride (%lld)", (long long)op[a], (long long)s[a]);
        if (in_size[a] < 1) return fail(NTG_ERR_INVALID_ARGUMENT, "empty input");
        out_size[a] = (in_size[a] - 1) * s[a] - 2 * p[a] + d[a] * (k[a] - 1) + 1 + op[a];
        if (out_size[a] < 1) return fail(NTG_ERR_INVALID_ARGUMENT, "the output of the transposed convolution would be empty");
    }
    return NTG_OK;
}

int64_t ntg_conv_transposend_workspace_bytes(int dtype, int64_t batch, int64_t in_channels, int64_t out_channels, int ndim,
                                             const int64_t* in_size, const int64_t* kernel_size, const int64_t* stride,
                                             const int64_t* padding, const int64_t* dilation, const int64_t* output_padding, int64_t groups) {
    int64_t os[NTG_MAX_SPATIAL];
    if (ntg::elem_size(dtype) == 0 || check_groups(in_channels, out_channels, groups) ||
        transpose_nd_out(ndim, in_size, kernel_size, stride, padding, dilation, output_padding, os)) return -1;
    if (ndim <= 2) {
        const Geo2 g = as_2d(ndim, in_size, kernel_size, stride, padding, dilation);
        return ntg_conv_transpose2d_workspace_bytes(dtype, batch, in_channels, g.h, g.w, out_channels, g.kr, g.kc, g.sr, g.sc, g.pr, g.pc, g.dr, g.dc,
                                                    ndim == 1 ? 0 : output_padding[0], output_padding[ndim - 1], groups);
    }
    return ntg_convnd_workspace_bytes(dtype, batch, out_channels, in_channels, ndim, os, kernel_size, stride, padding, dilation, groups, 1);
}

int ntg_conv_transposend_dev(int dtype, const void* input, const void* kernel, void* out, void* workspace, int64_t workspace_bytes,
                             int64_t batch, int64_t in_channels, int64_t out_channels, int ndim, const int64_t* in_size,
                             const int64_t* kernel_size, const int64_t* stride, const int64_t* padding, const int64_t* dilation,
                             const int64_t* output_padding, int64_t groups, void* stream) {
    if (ntg::elem_size(dtype) == 0) return fail(NTG_ERR_UNSUPPORTED_DTYPE, "dtype %d is not supported", dtype);
    int rc = check_groups(in_channels, out_channels, groups);
    if (rc) return rc;
    int64_t os[NTG_MAX_SPATIAL];
    rc = transpose_nd_out(ndim, in_size, kernel_size, stride, padding, dilation, output_padding, os);
    if (rc) return rc;
    if (ndim <= 2) {
        const Geo2 g = as_2d(ndim, in_size, kernel_size, stride, padding, dilation);
        return ntg_conv_transpose2d_dev(dtype, input, kernel, out, workspace, workspace_bytes, batch, in_channels, g.h, g.w, out_channels, g.kr, g.kc,
                                        g.sr, g.sc, g.pr, g.pc, g.dr, g.dc, ndim == 1 ? 0 : output_padding[0], output_padding[ndim - 1], groups, stream);
    }
    if (batch == 0 || out_channels == 0) return NTG_OK;
    if (in_channels == 0) return fail(NTG_ERR_INVALID_ARGUMENT, "empty input");
    // the image gradient of the convolution [out_channels -> in_channels] over an image of the output's size
    return ntg_convnd_backward_dev(dtype, nullptr, kernel, input, out, nullptr, workspace, workspace_bytes, batch, out_channels, in_channels, ndim,
                                   os, kernel_size, stride, padding, dilation, groups, 0, stream);
}

// host-pointer forms (synchronous)
int ntg_convnd(int dtype, const void* image, const void* kernel, void* out, int64_t batch, int64_t channels, int64_t out_channels, int ndim,
               const int64_t* size, const int64_t* kernel_size, const int64_t* stride, const int64_t* padding, const int64_t* dilation, int64_t groups) {
    const int64_t es = ntg::elem_size(dtype);
    if (es == 0) return fail(NTG_ERR_UNSUPPORTED_DTYPE, "dtype %d is not supported", dtype);
    int rc = check_groups(channels, out_channels, groups);
    if (rc) return rc;
    ntg::UnfoldNdParams u;
    rc = fill_nd(u, batch, channels, ndim, size, kernel_size, stride, padding, dilation);
    if (rc) return rc;
    if (batch == 0 || out_channels == 0) return NTG_OK;
    if (!image || !kernel || !out) return fail(NTG_ERR_INVALID_ARGUMENT, "null pointer");
    const size_t im_bytes = (size_t)(batch * channels * u.vol * es), k_bytes = (size_t)(out_channels * (channels / groups) * u.taps * es);
    const size_t o_bytes = (size_t)(batch * out_channels * u.L * es);
    const int64_t wsb = ntg_convnd_workspace_bytes(dtype, batch, channels, out_channels, ndim, size, kernel_size, stride, padding, dilation, groups, 0);
    ntg::HostSession mem;
    const size_t o_k = align_up(im_bytes, 256), o_o = o_k + align_up(k_bytes, 256), o_ws = o_o + align_up(o_bytes, 256);
    HIP_TRY(mem.reserve(o_ws + (size_t)wsb));
    if (im_bytes) HIP_TRY(mem.upload(0, image, im_bytes));
    if (k_bytes) HIP_TRY(mem.upload(o_k, kernel, k_bytes));
    rc = ntg_convnd_dev(dtype, mem.at(0), mem.at(o_k), mem.at(o_o), mem.at(o_ws), wsb, batch, channels, out_channels, ndim, size, kernel_size,
                        stride, padding, dilation, groups, mem.stream());
    if (rc) return rc;
    HIP_TRY(mem.download(out, o_o, o_bytes));
    return NTG_OK;
}

int ntg_convnd_backward(int dtype, const void* image, const void* kernel, const void* grad_out, void* d_image, void* d_kernel,
                        int64_t batch, int64_t channels, int64_t out_channels, int ndim, const int64_t* size, const int64_t* kernel_size,
                        const int64_t* stride, const int64_t* padding, const int64_t* dilation, int64_t groups, int accumulate) {
    const int64_t es = ntg::elem_size(dtype);
    if (es == 0) return fail(NTG_ERR_UNSUPPORTED_DTYPE, "dtype %d is not supported", dtype);
    int rc = check_groups(channels, out_channels, groups);
    if (rc) return rc;
    ntg::UnfoldNdParams u;
    rc = fill_nd(u, batch, channels, ndim, size, kernel_size, stride, padding, dilation);
    if (rc) return rc;
    if (batch == 0 || out_channels == 0 || channels == 0) return NTG_OK;
    if (!image || !kernel || !grad_out) return fail(NTG_ERR_INVALID_ARGUMENT, "null pointer");
    if (ndim <= 2) {        // (the two-axis host entry point: it keeps the reference's order of summation for Float32)
        const Geo2 g = as_2d(ndim, size, kernel_size, stride, padding, dilation);
        return ntg_conv2d_backward(dtype, image, kernel, grad_out, d_image, d_kernel, batch, channels, g.h, g.w, out_channels, g.kr, g.kc,
                                   g.sr, g.sc, g.pr, g.pc, g.dr, g.dc, groups, accumulate);
    }
    const size_t im_bytes = (size_t)(batch * channels * u.vol * es), k_bytes = (size_t)(out_channels * (channels / groups) * u.taps * es);
    const size_t g_bytes = (size_t)(batch * out_channels * u.L * es);
    const int64_t wsb = ntg_convnd_workspace_bytes(dtype, batch, channels, out_channels, ndim, size, kernel_size, stride, padding, dilation, groups, 1);
    ntg::HostSession mem;
    const size_t o_k = align_up(im_bytes, 256), o_g = o_k + align_up(k_bytes, 256), o_di = o_g + align_up(g_bytes, 256);
    const size_t o_dk = o_di + align_up(im_bytes, 256), o_ws = o_dk + align_up(k_bytes, 256);
    HIP_TRY(mem.reserve(o_ws + (size_t)wsb));
    HIP_TRY(mem.upload(0, image, im_bytes));
    HIP_TRY(mem.upload(o_k, kernel, k_bytes));
    HIP_TRY(mem.upload(o_g, grad_out, g_bytes));
    if (accumulate && d_image) HIP_TRY(mem.upload(o_di, d_image, im_bytes));
    if (accumulate && d_kernel) HIP_TRY(mem.upload(o_dk, d_kernel, k_bytes));
    rc = ntg_convnd_backward_dev(dtype, mem.at(0), mem.at(o_k), mem.at(o_g), d_image ? mem.at(o_di) : nullptr, d_kernel ? mem.at(o_dk) : nullptr,
                                 mem.at(o_ws), wsb, batch, channels, out_channels, ndim, size, kernel_size, stride, padding, dilation, groups,
                                 accumulate, mem.stream());
    if (rc) return rc;
    if (d_image) HIP_TRY(mem.download(d_image, o_di, im_bytes));
    if (d_kernel) HIP_TRY(mem.download(d_kernel, o_dk, k_bytes));
    return NTG_OK;
}

int ntg_conv_transposend(int dtype, const void* input, const void* kernel, void* out, int64_t batch, int64_t in_channels, int64_t out_channels,
                         int ndim, const int64_t* in_size, const int64_t* kernel_size, const int64_t* stride, const int64_t* padding,
                         const int64_t* dilation, const int64_t* output_padding, int64_t groups) {
    const int64_t es = ntg::elem_size(dtype);
    if (es == 0) return fail(NTG_ERR_UNSUPPORTED_DTYPE, "dtype %d is not supported", dtype);
    int rc = check_groups(in_channels, out_channels, groups);
    if (rc) return rc;
    int64_t os[NTG_MAX_SPATIAL];
    rc = transpose_nd_out(ndim, in_size, kernel_size, stride, padding, dilation, output_padding, os);
    if (rc) return rc;
    if (batch == 0 || out_channels == 0) return NTG_OK;
    if (!input || !kernel || !out) return fail(NTG_ERR_INVALID_ARGUMENT, "null pointer");
    int64_t in_vol = 1, out_vol = 1, taps = 1;
    for (int a = 0; a < ndim; ++a) { in_vol *= in_size[a]; out_vol *= os[a]; taps *= kernel_size[a]; }
    const size_t in_bytes = (size_t)(batch * in_channels * in_vol * es), k_bytes = (size_t)(in_channels * (out_channels / groups) * taps * es);
    const size_t o_bytes = (size_t)(batch * out_channels * out_vol * es);
    const int64_t wsb = ntg_conv_transposend_workspace_bytes(dtype, batch, in_channels, out_channels, ndim, in_size, kernel_size, stride, padding,
                                                             dilation, output_padding, groups);
    if (wsb < 0) return fail(NTG_ERR_INVALID_ARGUMENT, "invalid geometry");
    ntg::HostSession mem;
    const size_t o_k = align_up(in_bytes, 256), o_o = o_k + align_up(k_bytes, 256), o_ws = o_o + align_up(o_bytes, 256);
    HIP_TRY(mem.reserve(o_ws + (size_t)wsb));
    if (in_bytes) HIP_TRY(mem.upload(0, input, in_bytes));
    if (k_bytes) HIP_TRY(mem.upload(o_k, kernel, k_bytes));
    rc = ntg_conv_transposend_dev(dtype, mem.at(0), mem.at(o_k), mem.at(o_o), mem.at(o_ws), wsb, batch, in_channels, out_channels, ndim, in_size,
                                  kernel_size, stride, padding, dilation, output_padding, groups, mem.stream());
    if (rc) return rc;
    HIP_TRY(mem.download(out, o_o, o_bytes));
    return NTG_OK;
}

}  // extern "C"
