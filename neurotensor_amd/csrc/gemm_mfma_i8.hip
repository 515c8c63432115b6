// Int8 / UInt8 on the matrix pipe: v_mfma_i32_32x32x32_i8 in the DMA-fed LDS ring kernel.  The reference multiplies and
// adds 8-bit integers with wrap-around in the element type (nt/mp/simde_traits/simde_traits_avx2.h:668-670); the low 8 bits
// of the exact products' 32-bit sum are that result for either signedness, so the outputs are bit-identical.  Rows that are
// not 16-byte multiples, and pointer-table batches, stay on the vector-ALU kernel.  Int32 / UInt32 products run on the
// same instruction as ten products of byte planes (second half of this file).
#include "gemm_ring_impl.h"
namespace ntg {
hipError_t launch_gemm_mfma_i8(int dtype, bool ta, bool tb, const GemmParams& p, hipStream_t s) {
    if (!ring_eligible(p, ta, 1)) {
        if (p.cmode == C_PARTIAL) return hipErrorInvalidValue;      // (only the DMA-fed kernel writes 32-bit sums)
        return launch_gemm_valu(dtype, ta, tb, p, s);
    }
    const int te = ring16_tile_edge(p.M, p.N, p.K, p.batch);
    if (te == 256) return launch_ring_wb<DT_I8, 4>(ta, tb, p, s);
    if (te == 64) return launch_ring_wb<DT_I8, 1>(ta, tb, p, s);
    return launch_ring_wb<DT_I8, 2>(ta, tb, p, s);
}

// ---- Int32 / UInt32 products on the same pipe ------------------------------------------------------------------
// The reference's 32-bit integer product wraps in the element type, i.e. it is the exact product modulo 2^32.  Write every
// operand as four balanced signed bytes, a = sum_i a_i 2^(8 i) (mod 2^32) with a_i in [-128, 127]; then
//   sum_k a b = sum_{i + j <= 3} 2^(8 (i + j)) sum_k a_i b_j   (mod 2^32),
// the terms with i + j >= 4 being multiples of 2^32: ten 8-bit products.  With the planes of A laid side by side in a row,
// [A_0 | A_1 | A_2 | A_3], and those of B stacked in reverse, [B_3; B_2; B_1; B_0], the products of one shift s = i + j are
// ONE product of depth (s + 1) K: the first s + 1 planes of A's rows against the last s + 1 planes of B.  Four launches
// of the 8-bit kernel write their 32-bit sums P_s; a last pass forms C0 + sum_s P_s << 8 s.  Every partial sum stays below
// 2^31 in magnitude (4 K 2^14, K < 32768), so nothing depends on how the accumulators overflow.
// four balanced signed bytes of a 32-bit pattern, least significant first
__device__ __forceinline__ void balanced_bytes(uint32_t v, uint32_t (&d)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int8_t b = (int8_t)(v & 0xffu);
        d[i] = (uint32_t)(uint8_t)b;
        v = (v - (uint32_t)(int32_t)b) >> 8;
    }
}
// One thread splits four consecutive elements (along k for A, along n for B: the contiguous axis of the planes) and writes
// one 4-byte word per plane.
template <bool TRANS>
__global__ void __launch_bounds__(256) i32_split_a_kernel(const uint32_t* __restrict__ A, uint32_t* __restrict__ pl, const I32PlanesParams q) {
    // pl[b][m][i * Kp + k] = digit i of A(m, k); k >= K: zero
    const int64_t kq = q.Kp / 4, total = (int64_t)q.M * kq;
    const int b = blockIdx.y;
    const uint32_t* Ab = A + (int64_t)b * q.sA;
    uint32_t* pb = pl + (int64_t)b * q.M * q.Kp;             // (in words: a row holds 4 planes of Kp / 4 words)
    for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * 256) {
        const int64_t m = idx / kq, k = (idx - m * kq) * 4;
        uint32_t w[4] = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const uint32_t v = k + e < q.K ? (TRANS ? Ab[(k + e) * q.lda + m] : Ab[m * q.lda + k + e]) : 0u;
            uint32_t d[4];
            balanced_bytes(v, d);
#pragma unroll
            for (int i = 0; i < 4; ++i) w[i] |= d[i] << (8 * e);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) pb[m * q.Kp + (int64_t)i * kq + k / 4] = w[i];
    }
}
template <bool TRANS>
__global__ void __launch_bounds__(256) i32_split_b_kernel(const uint32_t* __restrict__ B, uint32_t* __restrict__ pl, const I32PlanesParams q) {
    // pl[b][(3 - j) * Kp + k][n] = digit j of B(k, n); k >= K or n >= N: zero
    const int64_t nq = q.Np / 4, total = (int64_t)q.Kp * nq;
    const int b = blockIdx.y;
    const uint32_t* Bb = B + (int64_t)b * q.sB;
    uint32_t* pb = pl + (int64_t)b * q.Kp * q.Np;            // (in words)
    for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * 256) {
        const int64_t k = idx / nq, n = (idx - k * nq) * 4;
        uint32_t w[4] = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const uint32_t v = (k < q.K && n + e < q.N) ? (TRANS ? Bb[(n + e) * q.ldb + k] : Bb[k * q.ldb + n + e]) : 0u;
            uint32_t d[4];
            balanced_bytes(v, d);
#pragma unroll
            for (int j = 0; j < 4; ++j) w[j] |= d[j] << (8 * e);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) pb[((int64_t)(3 - j) * q.Kp + k) * nq + n / 4] = w[j];
    }
}
hipError_t launch_i32_split_planes(const void* A, const void* B, void* a_planes, void* b_planes, const I32PlanesParams& q, hipStream_t s) {
    const int na = q.sA == 0 ? 1 : q.batch, nb = q.sB == 0 ? 1 : q.batch;       // a broadcast operand is split once
    const dim3 ga((unsigned)grid_for((int64_t)q.M * q.Kp / 4), (unsigned)na), gb((unsigned)grid_for((int64_t)q.Kp * q.Np / 4), (unsigned)nb), t(256);
    if (q.ta) hipLaunchKernelGGL(i32_split_a_kernel<true>, ga, t, 0, s, (const uint32_t*)A, (uint32_t*)a_planes, q);
    else hipLaunchKernelGGL(i32_split_a_kernel<false>, ga, t, 0, s, (const uint32_t*)A, (uint32_t*)a_planes, q);
    if (q.tb) hipLaunchKernelGGL(i32_split_b_kernel<true>, gb, t, 0, s, (const uint32_t*)B, (uint32_t*)b_planes, q);
    else hipLaunchKernelGGL(i32_split_b_kernel<false>, gb, t, 0, s, (const uint32_t*)B, (uint32_t*)b_planes, q);
    return hipGetLastError();
}

// C = C0 + sum_s P_s << 8 s  (mod 2^32); parts[s][b][m][Np]
__global__ void __launch_bounds__(256) i32_combine_kernel(const uint32_t* __restrict__ parts, const GemmParams p, const int Np) {
    const int64_t per = (int64_t)p.M * Np, all = per * p.batch, total = (int64_t)p.batch * p.M * p.N;
    uint32_t* C = static_cast<uint32_t*>(p.C);
    const uint32_t* bias = static_cast<const uint32_t*>(p.bias);
    for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * 256) {
        const int64_t n = idx % p.N, m = (idx / p.N) % p.M, b = idx / ((int64_t)p.N * p.M);
        const int64_t src = b * per + m * Np + n;
        uint32_t* cp = C + b * p.sC + m * p.ldc + n;
        uint32_t acc = 0u;
        if (p.cmode == C_ACCUMULATE) acc = *cp;
        else if (p.cmode == C_BIAS) acc = bias[b * p.bias_bs + m * p.bias_rs + n * p.bias_cs];
#pragma unroll
        for (int s = 0; s < 4; ++s) acc += parts[(int64_t)s * all + src] << (8 * s);
        *cp = acc;
    }
}
// the same, four consecutive columns per thread with 16-byte accesses (N, ldc, sC multiples of 4, C 16-byte aligned)
__global__ void __launch_bounds__(256) i32_combine_vec_kernel(const uint32_t* __restrict__ parts, const GemmParams p, const int Np) {
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    const int64_t per = (int64_t)p.M * Np, all = per * p.batch, nq = p.N / 4, total = (int64_t)p.batch * p.M * nq;
    uint32_t* C = static_cast<uint32_t*>(p.C);
    const uint32_t* bias = static_cast<const uint32_t*>(p.bias);
    for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * 256) {
        const int64_t n = (idx % nq) * 4, m = (idx / nq) % p.M, b = idx / (nq * p.M);
        const int64_t src = b * per + m * Np + n;
        u4* cp = reinterpret_cast<u4*>(C + b * p.sC + m * p.ldc + n);
        u4 acc = {0u, 0u, 0u, 0u};
        if (p.cmode == C_ACCUMULATE) acc = *cp;
        else if (p.cmode == C_BIAS) {
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[e] = bias[b * p.bias_bs + m * p.bias_rs + (n + e) * p.bias_cs];
        }
        u4 x[4];
#pragma unroll
        for (int s = 0; s < 4; ++s) x[s] = *reinterpret_cast<const u4*>(parts + (int64_t)s * all + src);
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[e] += x[s][e] << (8 * s);
        *cp = acc;
    }
}
hipError_t launch_i32_combine(const void* parts, const GemmParams& p, int Np, hipStream_t s) {
    const int64_t total = (int64_t)p.batch * p.M * p.N;
    if (total == 0) return hipSuccess;
    if (p.N % 4 == 0 && p.ldc % 4 == 0 && p.sC % 4 == 0 && (reinterpret_cast<uintptr_t>(p.C) & 15) == 0) {
        hipLaunchKernelGGL(i32_combine_vec_kernel, dim3((unsigned)grid_for(total / 4)), dim3(256), 0, s, (const uint32_t*)parts, p, Np);
        return hipGetLastError();
    }
    hipLaunchKernelGGL(i32_combine_kernel, dim3((unsigned)grid_for(total)), dim3(256), 0, s, (const uint32_t*)parts, p, Np);
    return hipGetLastError();
}
}  // namespace ntg
