// Float32 products too small to give every CU a 64 x 64 tile (config 1, 512 x 512 x 512: 64 such tiles on 256 CUs).
//
// One workgroup per 32 x 32 tile of C, NW = four or eight wavefronts that split k between them: wavefront w takes the 16-wide
// k steps w, w + NW, w + 2 NW, ... and keeps one 32 x 32 accumulator block (v_mfma_f32_32x32x2f32, eight per step).  No LDS in the
// loop: a lane's operand values are exactly what it can load by itself -- lane (r = lane % 32, h = lane / 32) feeds row r
// of A and column r of B for the eight k 8 h .. 8 h + 7 of a step, so a K-contiguous operand is two 16-byte loads per
// lane and step (any alignment: global memory takes unaligned vector loads) and an M/N-contiguous one eight 4-byte loads
// that the 32 lanes of a half coalesce; MFMA j of a step multiplies k = j (lower half) and k = 8 + j (upper half).
// The loads of four steps are in flight while the four before them are multiplied.  At the end the NW accumulator
// blocks meet in LDS and are added in wavefront order (fixed: deterministic), C0 / bias are added, the optional clamp is
// applied and each wavefront stores a quarter of the tile.
// Rows and columns past the edge load from the last valid row / column and are not stored; a k tail is loaded
// element-wise with zeros.
#include "ntg_common.h"

namespace ntg {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// the lane's eight values of a K-contiguous operand: row `row` (ld elements long), k = k0 .. k0 + 7
__device__ __forceinline__ void load_kc(const float* __restrict__ base, int64_t ld, int row, int k0, int K, float (&v)[8]) {
    const float* ptr = base + (int64_t)row * ld + k0;
    if (k0 + 8 <= K) {
        f32x4 lo, hi;
        __builtin_memcpy(&lo, ptr, 16);
        __builtin_memcpy(&hi, ptr + 4, 16);
#pragma unroll
        for (int e = 0; e < 4; ++e) { v[e] = lo[e]; v[4 + e] = hi[e]; }
    } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = k0 + e < K ? ptr[e] : 0.0f;
    }
}
// ... of an operand stored [k][mn]: column `col`, k = k0 .. k0 + 7
__device__ __forceinline__ void load_mc(const float* __restrict__ base, int64_t ld, int col, int k0, int K, float (&v)[8]) {
    const float* ptr = base + (int64_t)k0 * ld + col;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = k0 + e < K ? ptr[(int64_t)e * ld] : 0.0f;
}

template <bool TA, bool TB, int NW>
__global__ void __launch_bounds__(64 * NW) gemm_small32_f32_kernel(const GemmParams p) {
    __shared__ float red[NW][16][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 31, h = lane >> 5;
    const int tiles = p.tiles_m * p.tiles_n;
    const int b = blockIdx.x / tiles, t = blockIdx.x - b * tiles;
    const int tm = t / p.tiles_n, tn = t - tm * p.tiles_n;
    const int m0 = tm * 32, n0 = tn * 32;
    const float* A = static_cast<const float*>(p.A) + (int64_t)b * p.sA;
    const float* B = static_cast<const float*>(p.B) + (int64_t)b * p.sB;
    const int arow = m0 + r < p.M ? m0 + r : p.M - 1;      // (rows / columns past the edge: valid loads, results dropped)
    const int bcol = n0 + r < p.N ? n0 + r : p.N - 1;
    const int KT = (p.K + 15) / 16;

    auto load = [&](int kt, float (&a)[8], float (&bv)[8]) {
        const int k0 = 16 * kt + 8 * h;
        if (TA) load_mc(A, p.lda, arow, k0, p.K, a); else load_kc(A, p.lda, arow, k0, p.K, a);
        if (TB) load_kc(B, p.ldb, bcol, k0, p.K, bv); else load_mc(B, p.ldb, bcol, k0, p.K, bv);
    };
    f32x16 acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
    // this wavefront's steps are wave, wave + NW, ...: nsteps of them, taken in chunks of four; the loads of one chunk (64
    // registers) are in flight while the 32 MFMAs of the chunk before run (about a microsecond: the memory latency)
    const int nsteps = wave < KT ? (KT - wave + NW - 1) / NW : 0, nc = (nsteps + 3) / 4;      // (uniform per wavefront)
    auto load_chunk = [&](int c, float (&a)[4][8], float (&bv)[4][8]) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
            if (4 * c + q < nsteps) load(wave + NW * (4 * c + q), a[q], bv[q]);
    };
    auto mma_chunk = [&](int c, const float (&a)[4][8], const float (&bv)[4][8]) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
            if (4 * c + q < nsteps) {
#pragma unroll
                for (int j = 0; j < 8; ++j) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[q][j], bv[q][j], acc, 0, 0, 0);
            }
    };
    float a_even[4][8], b_even[4][8], a_odd[4][8], b_odd[4][8];
    if (nc > 0) load_chunk(0, a_even, b_even);
    for (int c = 0; c < nc; c += 2) {
        if (c + 1 < nc) load_chunk(c + 1, a_odd, b_odd);
        mma_chunk(c, a_even, b_even);
        if (c + 1 < nc) {
            if (c + 2 < nc) load_chunk(c + 2, a_even, b_even);
            mma_chunk(c + 1, a_odd, b_odd);
        }
    }
    // the block of D: lane holds column lane % 32, rows 8 (v / 4) + 4 (lane / 32) + v % 4 for v = 0 .. 15
#pragma unroll
    for (int v = 0; v < 16; ++v) red[wave][v][lane] = acc[v];
    __syncthreads();
    float* C = static_cast<float*>(p.C) + (int64_t)b * p.sC;
    const float* bias = static_cast<const float*>(p.bias);
    const int n = n0 + r;
#pragma unroll
    for (int q = 0; q < 16 / NW; ++q) {
        const int v = (16 / NW) * wave + q;
        const int m = m0 + 8 * (v >> 2) + 4 * h + (v & 3);
        float sum = red[0][v][lane];
#pragma unroll
        for (int w = 1; w < NW; ++w) sum += red[w][v][lane];
        if (m >= p.M || n >= p.N) continue;
        float* cp = C + (int64_t)m * p.ldc + n;
        if (p.cmode == C_ACCUMULATE) sum += *cp;
        else if (p.cmode == C_BIAS) sum += bias[(int64_t)b * p.bias_bs + (int64_t)m * p.bias_rs + (int64_t)n * p.bias_cs];
        if (p.act == ACT_RELU) sum = sum > 0.0f ? sum : 0.0f;
        *cp = sum;
    }
}

}  // namespace

// true when the product is one for this kernel: strided Float32 operands, so few output elements that 64 x 64 tiles
// would leave more than half of the CUs without one, and a k worth splitting four ways
bool small32_f32_wins(const GemmParams& p) {
    if (p.Aptr || p.Bptr || p.Cptr || p.cmode == C_PARTIAL || p.K < 64 || p.M < 1 || p.N < 1) return false;
    const int64_t t64 = (int64_t)((p.M + 63) / 64) * ((p.N + 63) / 64) * p.batch;
    const int64_t t32 = (int64_t)((p.M + 31) / 32) * ((p.N + 31) / 32) * p.batch;
    return t64 < 128 && t32 <= 1024;
}

hipError_t launch_gemm_small32_f32(bool ta, bool tb, const GemmParams& pin, hipStream_t s) {
    GemmParams p = pin;
    p.tiles_m = (p.M + 31) / 32;
    p.tiles_n = (p.N + 31) / 32;
    const int64_t blocks = (int64_t)p.tiles_m * p.tiles_n * p.batch;
    if (blocks <= 0) return hipSuccess;
    if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
    const dim3 g((unsigned)blocks);
    // eight wavefronts (k split eight ways) from 16 steps on: the first loads' latency is paid once either way, the
    // multiplies behind it take half as long
    const bool wide = p.K >= 256;
#define NTG_SMALL32(TA_, TB_)                                                                                              \
    do {                                                                                                                   \
        if (wide) hipLaunchKernelGGL((gemm_small32_f32_kernel<TA_, TB_, 8>), g, dim3(512), 0, s, p);                       \
        else hipLaunchKernelGGL((gemm_small32_f32_kernel<TA_, TB_, 4>), g, dim3(256), 0, s, p);                            \
    } while (0)
    if (ta) {
        if (tb) NTG_SMALL32(true, true); else NTG_SMALL32(true, false);
    } else {
        if (tb) NTG_SMALL32(false, true); else NTG_SMALL32(false, false);
    }
#undef NTG_SMALL32
    return hipGetLastError();
}

}  // namespace ntg
