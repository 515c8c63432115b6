// Int8 / UInt8 on the matrix pipe: v_mfma_i32_32x32x32_i8 in the DMA-fed LDS ring kernel.  The reference multiplies and
// adds 8-bit integers with wrap-around in the element type (nt/mp/simde_traits/simde_traits_avx2.h:668-670); the low 8 bits
// of the exact products' 32-bit sum are that result for either signedness, so the outputs are bit-identical.  Rows that are
// not 16-byte multiples, and pointer-table batches, stay on the vector-ALU kernel.  16-, 32- and 64-bit integer products
// run on the same instruction as products of byte planes (second half of this file).
#include "gemm_ring_impl.h"
namespace ntg {
hipError_t launch_gemm_mfma_i8(int dtype, bool ta, bool tb, const GemmParams& p, hipStream_t s) {
    if ((p.tailA || p.tailB) && !ring_eligible(p, ta, 1)) return hipErrorInvalidValue;     // (only the DMA-fed kernel reads copied tail rows)
    if (!ring_eligible(p, ta, 1)) {
        if (p.cmode == C_PARTIAL) return hipErrorInvalidValue;      // (only the DMA-fed kernel writes 32-bit sums)
        return launch_gemm_valu(dtype, ta, tb, p, s);
    }
    // (an MN-major 192-row tile of bytes has 12 chunks per k-row, which the chunk swizzle of the transposing reads does not fit)
    const int rect = ta ? RECT_128 : RECT_128 | RECT_192;
    auto launch = [&](int te, const GemmParams& q) {
        if (te == 256) return launch_ring_wb<DT_I8, 4>(ta, tb, q, s);
        if (te == 224) return tb ? launch_ring_cfg<DT_I8, false, true, 3, 4>(q, s) : launch_ring_cfg<DT_I8, false, false, 3, 4>(q, s);
        if (te == 192) return launch_ring_wb<DT_I8, 2, 4, 2>(ta, tb, q, s);     // (128-byte K-steps, as for the 16-bit products)
        if (te == 64) return launch_ring_wb<DT_I8, 1>(ta, tb, q, s);
        // (k in 16-bit elements: the same number of K-steps)
        if (ring16_deep128(ring16_tiles(128, q.M, q.N, q.batch), q.K / 2)) return launch_ring_wb<DT_I8, 2, 0, 2>(ta, tb, q, s);
        return launch_ring_wb<DT_I8, 2>(ta, tb, q, s);
    };
    if (p.batch == 1 && p.cmode != C_PARTIAL) {
        // (the estimate of the 16-bit kernel: a K-step of 64 bytes per row is 64 k here, so the same tile takes half the steps)
        const Ring16Split sp = ring16_split(p.M, p.N, p.K, rect);
        if (sp.axis) {
            GemmParams head, tail;
            ring_split_params(p, ta, tb, 1, sp, head, tail);
            const hipError_t e = launch(sp.head_edge, head);
            if (e != hipSuccess) return e;
            return launch(sp.tail_edge, tail);
        }
    }
    return launch(ring16_tile_edge(p.M, p.N, p.K, p.batch, rect), p);
}
// the DMA-fed kernel or nothing (the gated pair of an unvouched pointer-table batch)
hipError_t launch_gemm_ring_only_i8(int dtype, bool ta, bool tb, const GemmParams& p, hipStream_t s, bool* taken) {
    *taken = ring_eligible(p, ta, 1);
    return *taken ? launch_gemm_mfma_i8(dtype, ta, tb, p, s) : hipSuccess;
}

// ---- 16-, 32- and 64-bit integer products on the same pipe --------------------------------------------------------
// The reference's integer product wraps in the element type (nt/mp/simde_traits/simde_traits_avx2.h:810-812 16-bit,
// :444-446 32-bit, :523-540 64-bit), i.e. it is the exact product modulo 2^W, W = 8 P.  Write every operand as P balanced
// signed bytes, a = sum_i a_i 2^(8 i) (mod 2^W) with a_i in [-128, 127]; then
//   sum_k a b = sum_{i + j < P} 2^(8 (i + j)) sum_k a_i b_j   (mod 2^W),
// the terms with i + j >= P being multiples of 2^W: 3, 10 or 36 8-bit products.  With the planes of A laid side by side in
// a row, [A_0 | A_1 | .. | A_{P-1}], and those of B stacked in reverse, [B_{P-1}; ..; B_1; B_0], the products of one shift
// s = i + j are ONE product of depth (s + 1) K: the first s + 1 planes of A's rows against the last s + 1 planes of B.
// P launches of the 8-bit kernel write their 32-bit sums P_s; a last pass forms C0 + sum_s P_s << 8 s in the element
// type.  Every partial sum stays below 2^31 in magnitude (P K 2^14 with P K < 2^17), so nothing depends on how the
// accumulators overflow.
template <int P> struct PlaneElem;
template <> struct PlaneElem<2> { typedef uint16_t U; typedef uint32_t X; };
template <> struct PlaneElem<4> { typedef uint32_t U; typedef uint32_t X; };
template <> struct PlaneElem<8> { typedef uint64_t U; typedef uint64_t X; };
// P balanced signed bytes of a W-bit pattern, least significant first (computed in X, at least W bits wide: what is
// carried out of the top byte is a multiple of 2^W)
template <int P>
__device__ __forceinline__ void balanced_bytes(typename PlaneElem<P>::X v, uint32_t (&d)[P]) {
    typedef typename PlaneElem<P>::X X;
#pragma unroll
    for (int i = 0; i < P; ++i) {
        const int8_t b = (int8_t)(v & 0xffu);
        d[i] = (uint32_t)(uint8_t)b;
        v = (v - (X)(int64_t)b) >> 8;
    }
}
// One thread splits four consecutive elements (along k for A, along n for B: the contiguous axis of the planes) and writes
// one 4-byte word per plane.
template <int P, bool TRANS>
__global__ void __launch_bounds__(256) int_split_a_kernel(const typename PlaneElem<P>::U* __restrict__ A, uint32_t* __restrict__ pl, const IntPlanesParams q) {
    // pl[b][m][i * Kp + k] = digit i of A(m, k); k >= K: zero
    const int64_t kq = q.Kp / 4, total = (int64_t)q.M * kq;
    const int b = blockIdx.y;
    const typename PlaneElem<P>::U* Ab = A + (int64_t)b * q.sA;
    uint32_t* pb = pl + (int64_t)b * q.M * P * kq;           // (in words: a row holds P planes of Kp / 4 words)
    for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * 256) {
        const int64_t m = idx / kq, k = (idx - m * kq) * 4;
        uint32_t w[P];
#pragma unroll
        for (int i = 0; i < P; ++i) w[i] = 0u;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const typename PlaneElem<P>::X v = k + e < q.K ? (TRANS ? Ab[(k + e) * q.lda + m] : Ab[m * q.lda + k + e]) : 0;
            uint32_t d[P];
            balanced_bytes<P>(v, d);
#pragma unroll
            for (int i = 0; i < P; ++i) w[i] |= d[i] << (8 * e);
        }
#pragma unroll
        for (int i = 0; i < P; ++i) pb[m * P * kq + (int64_t)i * kq + k / 4] = w[i];
    }
}
template <int P, bool TRANS>
__global__ void __launch_bounds__(256) int_split_b_kernel(const typename PlaneElem<P>::U* __restrict__ B, uint32_t* __restrict__ pl, const IntPlanesParams q) {
    // pl[b][(P - 1 - j) * Kp + k][n] = digit j of B(k, n); k >= K or n >= N: zero
    const int64_t nq = q.Np / 4, total = (int64_t)q.Kp * nq;
    const int b = blockIdx.y;
    const typename PlaneElem<P>::U* Bb = B + (int64_t)b * q.sB;
    uint32_t* pb = pl + (int64_t)b * P * q.Kp * nq;          // (in words)
    for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * 256) {
        const int64_t k = idx / nq, n = (idx - k * nq) * 4;
        uint32_t w[P];
#pragma unroll
        for (int j = 0; j < P; ++j) w[j] = 0u;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const typename PlaneElem<P>::X v = (k < q.K && n + e < q.N) ? (TRANS ? Bb[(n + e) * q.ldb + k] : Bb[k * q.ldb + n + e]) : 0;
            uint32_t d[P];
            balanced_bytes<P>(v, d);
#pragma unroll
            for (int j = 0; j < P; ++j) w[j] |= d[j] << (8 * e);
        }
#pragma unroll
        for (int j = 0; j < P; ++j) pb[((int64_t)(P - 1 - j) * q.Kp + k) * nq + n / 4] = w[j];
    }
}
template <int P>
static hipError_t launch_split_planes(const void* A, const void* B, void* a_planes, void* b_planes, const IntPlanesParams& q, hipStream_t s) {
    typedef typename PlaneElem<P>::U U;
    const int na = q.sA == 0 ? 1 : q.batch, nb = q.sB == 0 ? 1 : q.batch;       // a broadcast operand is split once
    const dim3 ga((unsigned)grid_for((int64_t)q.M * q.Kp / 4), (unsigned)na), gb((unsigned)grid_for((int64_t)q.Kp * q.Np / 4), (unsigned)nb), t(256);
    if (q.ta) hipLaunchKernelGGL((int_split_a_kernel<P, true>), ga, t, 0, s, (const U*)A, (uint32_t*)a_planes, q);
    else hipLaunchKernelGGL((int_split_a_kernel<P, false>), ga, t, 0, s, (const U*)A, (uint32_t*)a_planes, q);
    if (q.tb) hipLaunchKernelGGL((int_split_b_kernel<P, true>), gb, t, 0, s, (const U*)B, (uint32_t*)b_planes, q);
    else hipLaunchKernelGGL((int_split_b_kernel<P, false>), gb, t, 0, s, (const U*)B, (uint32_t*)b_planes, q);
    return hipGetLastError();
}
hipError_t launch_int_split_planes(int planes, const void* A, const void* B, void* a_planes, void* b_planes, const IntPlanesParams& q, hipStream_t s) {
    if (planes == 2) return launch_split_planes<2>(A, B, a_planes, b_planes, q, s);
    if (planes == 4) return launch_split_planes<4>(A, B, a_planes, b_planes, q, s);
    if (planes == 8) return launch_split_planes<8>(A, B, a_planes, b_planes, q, s);
    return hipErrorInvalidValue;
}

// C = C0 + sum_s P_s << 8 s  (mod 2^W); parts[s][b][m][Np], signed 32-bit sums
template <int P>
__global__ void __launch_bounds__(256) int_combine_kernel(const int32_t* __restrict__ parts, const GemmParams p, const int Np) {
    typedef typename PlaneElem<P>::U U;
    typedef typename PlaneElem<P>::X X;
    const int64_t per = (int64_t)p.M * Np, all = per * p.batch, total = (int64_t)p.batch * p.M * p.N;
    U* C = static_cast<U*>(p.C);
    const U* bias = static_cast<const U*>(p.bias);
    for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * 256) {
        const int64_t n = idx % p.N, m = (idx / p.N) % p.M, b = idx / ((int64_t)p.N * p.M);
        const int64_t src = b * per + m * Np + n;
        U* cp = C + b * p.sC + m * p.ldc + n;
        X acc = 0;
        if (p.cmode == C_ACCUMULATE) acc = *cp;
        else if (p.cmode == C_BIAS) acc = bias[b * p.bias_bs + m * p.bias_rs + n * p.bias_cs];
#pragma unroll
        for (int s = 0; s < P; ++s) acc += (X)(int64_t)parts[(int64_t)s * all + src] << (8 * s);
        *cp = (U)acc;
    }
}
// the same, four consecutive columns per thread with 16-byte accesses (N, ldc, sC multiples of 4, C 16-byte aligned)
template <int P>
__global__ void __launch_bounds__(256) int_combine_vec_kernel(const int32_t* __restrict__ parts, const GemmParams p, const int Np) {
    typedef typename PlaneElem<P>::U U;
    typedef typename PlaneElem<P>::X X;
    typedef int32_t i4 __attribute__((ext_vector_type(4)));
    struct alignas(sizeof(U) * 4 < 16 ? sizeof(U) * 4 : 16) CVec { U v[4]; };
    const int64_t per = (int64_t)p.M * Np, all = per * p.batch, nq = p.N / 4, total = (int64_t)p.batch * p.M * nq;
    U* C = static_cast<U*>(p.C);
    const U* bias = static_cast<const U*>(p.bias);
    for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * 256) {
        const int64_t n = (idx % nq) * 4, m = (idx / nq) % p.M, b = idx / (nq * p.M);
        const int64_t src = b * per + m * Np + n;
        CVec* cp = reinterpret_cast<CVec*>(C + b * p.sC + m * p.ldc + n);
        X acc[4] = {0, 0, 0, 0};
        if (p.cmode == C_ACCUMULATE) {
            const CVec c0 = *cp;
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[e] = c0.v[e];
        } else if (p.cmode == C_BIAS) {
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[e] = bias[b * p.bias_bs + m * p.bias_rs + (n + e) * p.bias_cs];
        }
        i4 x[P];
#pragma unroll
        for (int s = 0; s < P; ++s) x[s] = *reinterpret_cast<const i4*>(parts + (int64_t)s * all + src);
#pragma unroll
        for (int s = 0; s < P; ++s)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[e] += (X)(int64_t)x[s][e] << (8 * s);
        CVec out;
#pragma unroll
        for (int e = 0; e < 4; ++e) out.v[e] = (U)acc[e];
        *cp = out;
    }
}
template <int P>
static hipError_t launch_combine(const void* parts, const GemmParams& p, int Np, hipStream_t s) {
    const int64_t total = (int64_t)p.batch * p.M * p.N;
    if (total == 0) return hipSuccess;
    if (p.N % 4 == 0 && p.ldc % 4 == 0 && p.sC % 4 == 0 && (reinterpret_cast<uintptr_t>(p.C) & 15) == 0)
        hipLaunchKernelGGL(int_combine_vec_kernel<P>, dim3((unsigned)grid_for(total / 4)), dim3(256), 0, s, (const int32_t*)parts, p, Np);
    else
        hipLaunchKernelGGL(int_combine_kernel<P>, dim3((unsigned)grid_for(total)), dim3(256), 0, s, (const int32_t*)parts, p, Np);
    return hipGetLastError();
}
hipError_t launch_int_combine(int planes, const void* parts, const GemmParams& p, int Np, hipStream_t s) {
    if (planes == 2) return launch_combine<2>(parts, p, Np, s);
    if (planes == 4) return launch_combine<4>(parts, p, Np, s);
    if (planes == 8) return launch_combine<8>(parts, p, Np, s);
    return hipErrorInvalidValue;
}
}  // namespace ntg
