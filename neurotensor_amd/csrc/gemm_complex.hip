// Complex32 / Complex64 / Complex128 matmult as the reference computes it:  C (+)= op(A) (.) op(B)  where the product of
// two elements multiplies the real parts and the imaginary parts SEPARATELY.  The reference sends its complex types
// through the generic micro kernel (nt/functional/cpu/matmult/nt_matmult_simde.hpp:301-350) on vectors of interleaved
// (re, im) lanes; broadcast(A + kk) fills a vector with (a.re, a.im, a.re, a.im, ...) and fmadd is the plain lane-wise
// fused multiply-add (nt/mp/simde_traits/simde_traits_avx2.h:928-937, :996-1002 complex_64; :1037-1044, :1106-1112
// complex_128; :1285-1294, :1365-1373 complex_32), so per element
//     c.re = fma(a.re, b.re, c.re),  c.im = fma(a.im, b.im, c.im)      for k ascending, starting from the incoming C.
// This kernel runs exactly those chains on the vector ALU -- one lane per 4 x 4 block of outputs, every output's chain in
// ascending k from its initial value (C, the bias, or zero) -- so Complex64 / Complex128 results are bit-identical to the
// reference's.  Complex32 keeps float lanes inside a k tile of 2 * pack_size = 8 and converts half <-> float at the tile's
// load and store (simde_traits_avx2.h:1275-1303): the chain is rounded to half (nearest even) after every 8 k.
// LDS-tiled like the integer kernel: 64 x 64 outputs per workgroup, operand tiles stored k-major.
#include "ntg_common.h"

namespace ntg {

template <class R> struct alignas(2 * sizeof(R)) Cx { R re, im; };

template <class R, class L> struct CxLane {
    static __device__ __forceinline__ L up(R v) { return (L)v; }
    static __device__ __forceinline__ R down(L v) { return (R)v; }          // _Float16 <- float: round to nearest even
};
__device__ __forceinline__ float cx_fma(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ __forceinline__ double cx_fma(double a, double b, double c) { return __builtin_fma(a, b, c); }

// R: stored real type, L: lane type, KT: k between two roundings of the chain to R (0: never -- R == L)
template <class R, class L, int KT>
__global__ void __launch_bounds__(256) gemm_complex_kernel(const GemmParams p, const int ta, const int tb) {
    using E = Cx<R>;
    constexpr int BM = 64, BN = 64, BK = 16, PAD = sizeof(E) >= 16 ? 1 : 2;
    static_assert(KT == 0 || BK % KT == 0, "rounding points fall on tile-internal k");
    __shared__ E sA[BK][BM + PAD];
    __shared__ E sB[BK][BN + PAD];

    const int tid = threadIdx.x;
    const int lid = xcd_contiguous_id(blockIdx.x, gridDim.x);
    const int tiles = p.tiles_m * p.tiles_n;
    const int b = lid / tiles;
    int tm, tn;
    tile_coords(lid - b * tiles, p.tiles_m, p.tiles_n, 16, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;

    const E* A = p.Aptr ? static_cast<const E*>(p.Aptr[b]) : static_cast<const E*>(p.A) + (int64_t)b * p.sA;
    const E* B = p.Bptr ? static_cast<const E*>(p.Bptr[b]) : static_cast<const E*>(p.B) + (int64_t)b * p.sB;
    E* C = p.Cptr ? static_cast<E*>(p.Cptr[b]) : static_cast<E*>(p.C) + (int64_t)b * p.sC;
    const E* bias = static_cast<const E*>(p.bias);

    const int tx = tid & 15, ty = tid >> 4;   // 16 x 16 lanes, 4 x 4 outputs each
    // every chain starts from its initial value
    L are[4][4], aim[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            E v;
            v.re = (R)0; v.im = (R)0;
            if (m < p.M && n < p.N) {
                if (p.cmode == C_ACCUMULATE) v = C[(int64_t)m * p.ldc + n];
                else if (p.cmode == C_BIAS) v = bias[(int64_t)b * p.bias_bs + (int64_t)m * p.bias_rs + (int64_t)n * p.bias_cs];
            }
            are[i][j] = CxLane<R, L>::up(v.re);
            aim[i][j] = CxLane<R, L>::up(v.im);
        }
    }

    for (int k0 = 0; k0 < p.K; k0 += BK) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int e = tid + q * 256;
            int mn, kk;
            if (ta) { mn = e & 63; kk = e >> 6; } else { kk = e & 15; mn = e >> 4; }
            const int m = m0 + mn, k = k0 + kk;
            E v;
            v.re = (R)0; v.im = (R)0;
            if (m < p.M && k < p.K) v = ta ? A[(int64_t)k * p.lda + m] : A[(int64_t)m * p.lda + k];
            sA[kk][mn] = v;
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int e = tid + q * 256;
            int mn, kk;
            if (tb) { kk = e & 15; mn = e >> 4; } else { mn = e & 63; kk = e >> 6; }
            const int n = n0 + mn, k = k0 + kk;
            E v;
            v.re = (R)0; v.im = (R)0;
            if (n < p.N && k < p.K) v = tb ? B[(int64_t)n * p.ldb + k] : B[(int64_t)k * p.ldb + n];
            sB[kk][mn] = v;
        }
        __syncthreads();
        const int kmax = p.K - k0 < BK ? p.K - k0 : BK;      // (steps past K would be fma(0, 0, c) = c, but -0 + 0 is not -0)
        for (int kk = 0; kk < kmax; ++kk) {
            E a[4], bb[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = sA[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) bb[j] = sB[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    are[i][j] = cx_fma(CxLane<R, L>::up(a[i].re), CxLane<R, L>::up(bb[j].re), are[i][j]);
                    aim[i][j] = cx_fma(CxLane<R, L>::up(a[i].im), CxLane<R, L>::up(bb[j].im), aim[i][j]);
                }
            if constexpr (KT != 0) {
                if ((kk + 1) % KT == 0 || kk + 1 == kmax) {           // end of a k tile of the reference: store + reload in R
#pragma unroll
                    for (int i = 0; i < 4; ++i)
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            are[i][j] = CxLane<R, L>::up(CxLane<R, L>::down(are[i][j]));
                            aim[i][j] = CxLane<R, L>::up(CxLane<R, L>::down(aim[i][j]));
                        }
                }
            }
        }
        __syncthreads();
    }

#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= p.M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= p.N) continue;
            E v;
            v.re = CxLane<R, L>::down(are[i][j]);
            v.im = CxLane<R, L>::down(aim[i][j]);
            C[(int64_t)m * p.ldc + n] = v;
        }
    }
}

template <class R, class L, int KT>
static hipError_t launch_complex_t(bool ta, bool tb, const GemmParams& pin, hipStream_t s) {
    GemmParams p = pin;
    p.tiles_m = (p.M + 63) / 64;
    p.tiles_n = (p.N + 63) / 64;
    const int64_t blocks = (int64_t)p.tiles_m * p.tiles_n * p.batch;
    if (blocks <= 0) return hipSuccess;
    if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
    hipLaunchKernelGGL((gemm_complex_kernel<R, L, KT>), dim3((unsigned)blocks), dim3(256), 0, s, p, (int)ta, (int)tb);
    return hipGetLastError();
}

hipError_t launch_gemm_complex(int dtype, bool ta, bool tb, const GemmParams& p, hipStream_t s) {
    switch (dtype) {
    case DT_C32: return launch_complex_t<_Float16, float, 8>(ta, tb, p, s);
    case DT_C64: return launch_complex_t<float, float, 0>(ta, tb, p, s);
    case DT_C128: return launch_complex_t<double, double, 0>(ta, tb, p, s);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace ntg
