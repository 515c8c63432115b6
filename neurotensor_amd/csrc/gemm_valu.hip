// Integer GEMM on the vector ALU:  C (+)= op(A) . op(B)  with multiply and add that wrap
// in the element type, so results are bit-identical to the reference's integer lanes
// (nt/mp/simde_traits/simde_traits_avx2.h:444-446 int32 mullo+add, :523-540 int64,
// :668-670 int8, :810-812 int16).  gfx950 has no 32/64-bit integer MFMA, so this is a
// classic LDS-tiled outer-product kernel: a 64x64 tile of C per workgroup, 4x4 outputs
// per lane, both operand tiles stored k-major in LDS so the inner loop reads one vector
// of A rows and one of B columns per k.  The accumulator type is the element type
// (unsigned of the same width: same residues, no signed-overflow UB).
#include "ntg_common.h"

namespace ntg {

template <class T>
__global__ void __launch_bounds__(256) gemm_valu_kernel(const GemmParams p, const int ta, const int tb) {
    constexpr int BM = 64, BN = 64, BK = 16, PAD = 4;
    __shared__ T sA[BK][BM + PAD];
    __shared__ T sB[BK][BN + PAD];

    if (p.gate && *p.gate != p.gate_want) return;       // (uniform: the other kernel of a gated pair does this product)
    const int tid = threadIdx.x;
    const int lid = xcd_contiguous_id(blockIdx.x, gridDim.x);
    const int tiles = p.tiles_m * p.tiles_n;
    const int b = lid / tiles;
    int tm, tn;
    tile_coords(lid - b * tiles, p.tiles_m, p.tiles_n, 16, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;

    const T* A = p.Aptr ? static_cast<const T*>(p.Aptr[b]) : static_cast<const T*>(p.A) + (int64_t)b * p.sA;
    const T* B = p.Bptr ? static_cast<const T*>(p.Bptr[b]) : static_cast<const T*>(p.B) + (int64_t)b * p.sB;
    T* C = p.Cptr ? static_cast<T*>(p.Cptr[b]) : static_cast<T*>(p.C) + (int64_t)b * p.sC;

    const int tx = tid & 15, ty = tid >> 4;   // 16 x 16 lanes, 4 x 4 outputs each
    T acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0;

    for (int k0 = 0; k0 < p.K; k0 += BK) {
        // each lane moves 4 elements per operand; the fast index follows the
        // operand's contiguous direction in global memory
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int e = tid + q * 256;
            int mn, kk;
            if (ta) { mn = e & 63; kk = e >> 6; } else { kk = e & 15; mn = e >> 4; }
            const int m = m0 + mn, k = k0 + kk;
            T v = 0;
            if (m < p.M && k < p.K) v = ta ? A[(int64_t)k * p.lda + m] : A[(int64_t)m * p.lda + k];
            sA[kk][mn] = v;
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int e = tid + q * 256;
            int mn, kk;
            if (tb) { kk = e & 15; mn = e >> 4; } else { mn = e & 63; kk = e >> 6; }
            const int n = n0 + mn, k = k0 + kk;
            T v = 0;
            if (n < p.N && k < p.K) v = tb ? B[(int64_t)n * p.ldb + k] : B[(int64_t)k * p.ldb + n];
            sB[kk][mn] = v;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < BK; ++kk) {
            T a[4], bb[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = sA[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) bb[j] = sB[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = (T)(acc[i][j] + (T)(a[i] * bb[j]));
        }
        __syncthreads();
    }

    const T* bias = static_cast<const T*>(p.bias);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= p.M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= p.N) continue;
            T* cp = C + (int64_t)m * p.ldc + n;
            T v = acc[i][j];
            if (p.cmode == C_ACCUMULATE) v = (T)(v + *cp);
            else if (p.cmode == C_BIAS) v = (T)(v + bias[(int64_t)b * p.bias_bs + (int64_t)m * p.bias_rs + (int64_t)n * p.bias_cs]);
            *cp = v;
        }
    }
}

template <class T>
static hipError_t launch_valu_t(bool ta, bool tb, const GemmParams& pin, hipStream_t s) {
    GemmParams p = pin;
    p.tiles_m = (p.M + 63) / 64;
    p.tiles_n = (p.N + 63) / 64;
    const int64_t blocks = (int64_t)p.tiles_m * p.tiles_n * p.batch;
    if (blocks <= 0) return hipSuccess;
    if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
    hipLaunchKernelGGL(gemm_valu_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, s, p, (int)ta, (int)tb);
    return hipGetLastError();
}

hipError_t launch_gemm_valu(int dtype, bool ta, bool tb, const GemmParams& p, hipStream_t s) {
    switch (dtype) {
    case DT_I8: case DT_U8: return launch_valu_t<uint8_t>(ta, tb, p, s);
    case DT_I16: case DT_U16: return launch_valu_t<uint16_t>(ta, tb, p, s);
    case DT_I32: case DT_U32: return launch_valu_t<uint32_t>(ta, tb, p, s);
    case DT_I64: case DT_U64: return launch_valu_t<uint64_t>(ta, tb, p, s);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace ntg
