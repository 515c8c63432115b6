// Skinny GEMM (m <= 32): C[m, n] (+)= op(A)[m, k] . op(B)[k, n]   (Float32 first, Float16 / BFloat16 below)
//
// With so few rows the product streams B exactly once and is bound by HBM bandwidth,
// not by the matrix cores, so the tiling is chosen for the memory system: a workgroup of
// 8 wavefronts owns a strip of SW columns of C and all of K; the wavefronts take k-steps
// of 16 round-robin, feed v_mfma_f32_16x16x4_f32 straight from global memory (B is used
// once, so staging it in LDS would only add traffic), and their partial sums are added in
// a fixed order through LDS, which keeps the result deterministic (no atomics).
//
// Lane (c = lane%16, g = lane/16) holds, per k-step, A[row c][k0+4g .. k0+4g+3] and
// B[k0+4g+e][n0 + CPL*c .. +CPL-1] for e = 0..3: MFMA e uses k = k0+4g+e for lane group g
// on both operands, and MFMA column c stands for strip column CPL*c + j.
#include "ntg_common.h"

namespace ntg {

typedef float floatx4 __attribute__((ext_vector_type(4)));

template <int MB, int CPL, bool TA, bool TB, bool FAST>
__global__ void __launch_bounds__(512) gemm_skinny_f32_kernel(const GemmParams p) {
    constexpr int NW = 8;
    constexpr int SW = 16 * CPL;
    __shared__ float part[NW][MB * CPL * 4][64];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int c = lane & 15, g = lane >> 4;
    const int b = blockIdx.y;
    const int n0 = blockIdx.x * SW;

    // (global pointers: the waits of the register ring below are per k-step only if the loads are not FLAT instructions)
    const NTG_GLOBAL float* A = (const NTG_GLOBAL float*)(p.Aptr ? static_cast<const float*>(p.Aptr[b]) : static_cast<const float*>(p.A) + (int64_t)b * p.sA);
    const NTG_GLOBAL float* B = (const NTG_GLOBAL float*)(p.Bptr ? static_cast<const float*>(p.Bptr[b]) : static_cast<const float*>(p.B) + (int64_t)b * p.sB);
    NTG_GLOBAL float* C = (NTG_GLOBAL float*)(p.Cptr ? static_cast<float*>(p.Cptr[b]) : static_cast<float*>(p.C) + (int64_t)b * p.sC);

    floatx4 acc[MB][CPL];
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
        for (int j = 0; j < CPL; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

    const int steps = (p.K + 15) / 16;
    // D k-steps of loads are kept in flight per wavefront (a register ring), so that
    // 8 wavefronts per CU cover the HBM latency-bandwidth product.
    constexpr int D = 4;
    float a[D][MB][4];
    float bv[D][4][CPL];

    auto load_step = [&](int d, int s) {
        const int kl = s * 16 + 4 * g;          // this lane's first k
#pragma unroll
        for (int i = 0; i < MB; ++i) {
            const int row = i * 16 + c;
            if constexpr (FAST && !TA) {
                const floatx4 t = (row < p.M) ? *(const NTG_GLOBAL floatx4*)(A + (int64_t)row * p.lda + kl) : floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int e = 0; e < 4; ++e) a[d][i][e] = t[e];
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int k = kl + e;
                    float v = 0.f;
                    if (row < p.M && k < p.K) v = TA ? A[(int64_t)k * p.lda + row] : A[(int64_t)row * p.lda + k];
                    a[d][i][e] = v;
                }
            }
        }
        if constexpr (!TB) {
            typedef float fv __attribute__((ext_vector_type(CPL)));
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int k = kl + e;
                if constexpr (FAST) {
                    const fv t = *(const NTG_GLOBAL fv*)(B + (int64_t)k * p.ldb + n0 + CPL * c);
#pragma unroll
                    for (int j = 0; j < CPL; ++j) bv[d][e][j] = t[j];
                } else {
#pragma unroll
                    for (int j = 0; j < CPL; ++j) {
                        const int n = n0 + CPL * c + j;
                        bv[d][e][j] = (k < p.K && n < p.N) ? B[(int64_t)k * p.ldb + n] : 0.f;
                    }
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < CPL; ++j) {
                const int n = n0 + CPL * c + j;
                if constexpr (FAST) {
                    const floatx4 t = *(const NTG_GLOBAL floatx4*)(B + (int64_t)n * p.ldb + kl);
#pragma unroll
                    for (int e = 0; e < 4; ++e) bv[d][e][j] = t[e];
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int k = kl + e;
                        bv[d][e][j] = (k < p.K && n < p.N) ? B[(int64_t)n * p.ldb + k] : 0.f;
                    }
                }
            }
        }
    };

    auto compute = [&](int d) __attribute__((always_inline)) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
#pragma unroll
            for (int i = 0; i < MB; ++i)
#pragma unroll
                for (int j = 0; j < CPL; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[d][i][e], bv[d][e][j], acc[i][j], 0, 0, 0);
    };
    // Rounds of D k-steps.  While a whole further round exists, a round runs without a branch (multiply step d, request the
    // step that takes its registers): the number of loads in flight is then the same at every wait, and the compiler waits
    // for one step's loads and leaves the other D - 1 steps in flight.  (Where paths with different counts meet it waits
    // for everything; the guarded rounds at the end, and the whole loop for a short k, are of that kind.)
    int base = wave;
    if (wave + (2 * D - 1) * NW < steps) {               // (uniform per wavefront)
#pragma unroll
        for (int d = 0; d < D; ++d) load_step(d, wave + d * NW);
        for (; base + (2 * D - 1) * NW < steps; base += D * NW) {
#pragma unroll
            for (int d = 0; d < D; ++d) {
                compute(d);
                load_step(d, base + (d + D) * NW);
            }
        }
    } else {
#pragma unroll
        for (int d = 0; d < D; ++d)
            if (wave + d * NW < steps) load_step(d, wave + d * NW);
    }
    for (; base < steps; base += D * NW) {
#pragma unroll
        for (int d = 0; d < D; ++d) {
            const int s = base + d * NW;
            if (s < steps) {
                compute(d);
                if (s + D * NW < steps) load_step(d, s + D * NW);
            }
        }
    }

#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
        for (int j = 0; j < CPL; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) part[wave][(i * CPL + j) * 4 + r][lane] = acc[i][j][r];
    __syncthreads();

    constexpr int TOTAL = MB * CPL * 4 * 64;
    const NTG_GLOBAL float* bias = (const NTG_GLOBAL float*)static_cast<const float*>(p.bias);
    for (int idx = tid; idx < TOTAL; idx += 512) {
        const int l = idx & 63, q = idx >> 6;
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) sum += part[w][q][l];     // fixed order: deterministic
        const int r = q & 3, j = (q >> 2) % CPL, i = (q >> 2) / CPL;
        const int m = i * 16 + 4 * (l >> 4) + r;
        const int n = n0 + CPL * (l & 15) + j;
        if (m < p.M && n < p.N) {
            NTG_GLOBAL float* cp = C + (int64_t)m * p.ldc + n;
            if (p.cmode == C_ACCUMULATE) sum += *cp;
            else if (p.cmode == C_BIAS) sum += bias[(int64_t)b * p.bias_bs + (int64_t)m * p.bias_rs + (int64_t)n * p.bias_cs];
            *cp = sum;
        }
    }
}

template <int MB, int CPL, bool TA, bool TB>
static hipError_t launch_skinny_cfg(const GemmParams& p, hipStream_t s) {
    constexpr int SW = 16 * CPL;
    const bool a_fast = TA || ((p.lda % 4 == 0) && !p.Aptr && ((reinterpret_cast<uintptr_t>(p.A) & 15) == 0) && (p.sA % 4 == 0));
    const int bw = TB ? 4 : CPL;    // floats per vector load of B
    const bool b_fast = (p.ldb % bw == 0) && !p.Bptr && ((reinterpret_cast<uintptr_t>(p.B) & 15) == 0) && (p.sB % 4 == 0);
    const bool fast = a_fast && b_fast && (p.K % 16 == 0) && (p.N % SW == 0);
    dim3 grid((unsigned)((p.N + SW - 1) / SW), (unsigned)p.batch);
    if (fast) hipLaunchKernelGGL((gemm_skinny_f32_kernel<MB, CPL, TA, TB, true>), grid, dim3(512), 0, s, p);
    else hipLaunchKernelGGL((gemm_skinny_f32_kernel<MB, CPL, TA, TB, false>), grid, dim3(512), 0, s, p);
    return hipGetLastError();
}

template <int MB, int CPL>
static hipError_t launch_skinny_t(bool ta, bool tb, const GemmParams& p, hipStream_t s) {
    if (ta) return tb ? launch_skinny_cfg<MB, CPL, true, true>(p, s) : launch_skinny_cfg<MB, CPL, true, false>(p, s);
    return tb ? launch_skinny_cfg<MB, CPL, false, true>(p, s) : launch_skinny_cfg<MB, CPL, false, false>(p, s);
}

// ---- Float16 / BFloat16, m <= 32 -----------------------------------------------------------------
// Same plan with v_mfma_f32_16x16x32: lane (c = lane%16, g = lane/16) feeds 8 consecutive k
// (k0 + 8g ..) of row c of A and of one column of B.  Per k-step of 32:
//   TB  (B stored [n][k]): the 8 k of column c + 16 j are one 16-byte load; MFMA j covers column c + 16 j.
//   !TB (B stored [k][n]): the lane loads CPL consecutive columns (n0 + CPL c ..) of each of its 8 k rows
//       (coalesced along n) and transposes the 8 x CPL block in registers (v_perm_b32); MFMA j covers
//       column CPL c + j.
// fp32 accumulation over all of K, one rounding at the end (C0 added in fp32).
typedef uint32_t su32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 sbf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 shalfx8 __attribute__((ext_vector_type(8)));

template <int DT> struct Skinny16;
template <> struct Skinny16<DT_F16> {
    using T = _Float16;
    static __device__ __forceinline__ floatx4 mma(su32x4 a, su32x4 b, floatx4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(shalfx8, a), __builtin_bit_cast(shalfx8, b), c, 0, 0, 0);
    }
};
template <> struct Skinny16<DT_BF16> {
    using T = __bf16;
    static __device__ __forceinline__ floatx4 mma(su32x4 a, su32x4 b, floatx4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(sbf16x8, a), __builtin_bit_cast(sbf16x8, b), c, 0, 0, 0);
    }
};

template <int DT, int MB, int CPL, bool TA, bool TB, bool FAST>
__global__ void __launch_bounds__(512) gemm_skinny16_kernel(const GemmParams p) {
    using S = Skinny16<DT>;
    using T = typename S::T;
    constexpr int NW = 8;
    constexpr int SW = 16 * CPL;
    constexpr int BW = TB ? 4 : (CPL + 1) / 2;          // dwords per B load
    constexpr int NB = TB ? CPL : 8;                    // B loads per k-step
    __shared__ float part[NW][MB * CPL * 4][64];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int c = lane & 15, g = lane >> 4;
    const int b = blockIdx.y;
    const int n0 = blockIdx.x * SW;

    const NTG_GLOBAL T* A = (const NTG_GLOBAL T*)(p.Aptr ? static_cast<const T*>(p.Aptr[b]) : static_cast<const T*>(p.A) + (int64_t)b * p.sA);
    const NTG_GLOBAL T* B = (const NTG_GLOBAL T*)(p.Bptr ? static_cast<const T*>(p.Bptr[b]) : static_cast<const T*>(p.B) + (int64_t)b * p.sB);
    NTG_GLOBAL T* C = (NTG_GLOBAL T*)(p.Cptr ? static_cast<T*>(p.Cptr[b]) : static_cast<T*>(p.C) + (int64_t)b * p.sC);

    floatx4 acc[MB][CPL];
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
        for (int j = 0; j < CPL; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

    const int steps = (p.K + 31) / 32;
    constexpr int D = (NB * BW >= 32 || MB * CPL >= 8) ? 2 : 4;   // k-steps of loads in flight per wavefront (register budget)
    su32x4 a[D][MB];
    uint32_t bv[D][NB][BW];

    auto gather8 = [&](auto&& elem) -> su32x4 {          // 8 elements -> 4 packed dwords
        T tmp[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) tmp[e] = elem(e);
        su32x4 r;
        __builtin_memcpy(&r, tmp, 16);
        return r;
    };

    auto load_step = [&](int d, int s) {
        const int kl = s * 32 + 8 * g;                   // this lane's first k
#pragma unroll
        for (int i = 0; i < MB; ++i) {
            const int row = i * 16 + c;
            if constexpr (FAST && !TA) {
                a[d][i] = (row < p.M) ? *(const NTG_GLOBAL su32x4*)(A + (int64_t)row * p.lda + kl) : su32x4{0u, 0u, 0u, 0u};
            } else {
                a[d][i] = gather8([&](int e) -> T {
                    const int k = kl + e;
                    if (row >= p.M || k >= p.K) return (T)0.0f;
                    return TA ? A[(int64_t)k * p.lda + row] : A[(int64_t)row * p.lda + k];
                });
            }
        }
        if constexpr (TB) {
#pragma unroll
            for (int j = 0; j < CPL; ++j) {
                const int n = n0 + c + 16 * j;
                su32x4 t;
                if constexpr (FAST) {
                    t = *(const NTG_GLOBAL su32x4*)(B + (int64_t)n * p.ldb + kl);
                } else {
                    t = gather8([&](int e) -> T { return (n < p.N && kl + e < p.K) ? B[(int64_t)n * p.ldb + kl + e] : (T)0.0f; });
                }
#pragma unroll
                for (int w = 0; w < 4; ++w) bv[d][j][w] = t[w];
            }
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int k = kl + e;
                const int n = n0 + CPL * c;
                if constexpr (FAST) {
                    if constexpr (CPL == 8) {
                        const su32x4 t = *(const NTG_GLOBAL su32x4*)(B + (int64_t)k * p.ldb + n);
#pragma unroll
                        for (int w = 0; w < 4; ++w) bv[d][e][w] = t[w];
                    } else if constexpr (CPL == 4) {
                        typedef uint32_t u2 __attribute__((ext_vector_type(2)));
                        const u2 t = *(const NTG_GLOBAL u2*)(B + (int64_t)k * p.ldb + n);
                        bv[d][e][0] = t[0];
                        bv[d][e][1] = t[1];
                    } else {
                        bv[d][e][0] = *(const NTG_GLOBAL uint32_t*)(B + (int64_t)k * p.ldb + n);
                    }
                } else {
                    T tmp[2 * BW];
#pragma unroll
                    for (int j = 0; j < 2 * BW; ++j) tmp[j] = (j < CPL && k < p.K && n + j < p.N) ? B[(int64_t)k * p.ldb + n + j] : (T)0.0f;
                    __builtin_memcpy(&bv[d][e][0], tmp, 4 * BW);
                }
            }
        }
    };

    auto compute = [&](int d) {
#pragma unroll
        for (int j = 0; j < CPL; ++j) {
            su32x4 bt;
            if constexpr (TB) {
#pragma unroll
                for (int w = 0; w < 4; ++w) bt[w] = bv[d][j][w];
            } else {
                // column j of the 8 x CPL block: dword w packs k rows 2w, 2w+1
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const uint32_t lo = bv[d][2 * w][j >> 1], hi = bv[d][2 * w + 1][j >> 1];
                    bt[w] = (j & 1) ? __builtin_amdgcn_perm(hi, lo, 0x07060302u) : __builtin_amdgcn_perm(hi, lo, 0x05040100u);
                }
            }
#pragma unroll
            for (int i = 0; i < MB; ++i) acc[i][j] = S::mma(a[d][i], bt, acc[i][j]);
        }
    };

    // (rounds without a branch while a whole further round exists: see the Float32 kernel above)
    int base = wave;
    if (wave + (2 * D - 1) * NW < steps) {               // (uniform per wavefront)
#pragma unroll
        for (int d = 0; d < D; ++d) load_step(d, wave + d * NW);
        for (; base + (2 * D - 1) * NW < steps; base += D * NW) {
#pragma unroll
            for (int d = 0; d < D; ++d) {
                compute(d);
                load_step(d, base + (d + D) * NW);
            }
        }
    } else {
#pragma unroll
        for (int d = 0; d < D; ++d)
            if (wave + d * NW < steps) load_step(d, wave + d * NW);
    }
    for (; base < steps; base += D * NW) {
#pragma unroll
        for (int d = 0; d < D; ++d) {
            const int s = base + d * NW;
            if (s < steps) {
                compute(d);
                if (s + D * NW < steps) load_step(d, s + D * NW);
            }
        }
    }

#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
        for (int j = 0; j < CPL; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) part[wave][(i * CPL + j) * 4 + r][lane] = acc[i][j][r];
    __syncthreads();

    constexpr int TOTAL = MB * CPL * 4 * 64;
    const NTG_GLOBAL T* bias = (const NTG_GLOBAL T*)static_cast<const T*>(p.bias);
    for (int idx = tid; idx < TOTAL; idx += 512) {
        const int l = idx & 63, q = idx >> 6;
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) sum += part[w][q][l];     // fixed order: deterministic
        const int r = q & 3, j = (q >> 2) % CPL, i = (q >> 2) / CPL;
        const int m = i * 16 + 4 * (l >> 4) + r;
        const int n = n0 + (TB ? (l & 15) + 16 * j : CPL * (l & 15) + j);
        if (m < p.M && n < p.N) {
            NTG_GLOBAL T* cp = C + (int64_t)m * p.ldc + n;
            if (p.cmode == C_ACCUMULATE) sum += (float)*cp;
            else if (p.cmode == C_BIAS) sum += (float)bias[(int64_t)b * p.bias_bs + (int64_t)m * p.bias_rs + (int64_t)n * p.bias_cs];
            *cp = (T)sum;
        }
    }
}

template <int DT, int MB, int CPL, bool TA, bool TB>
static hipError_t launch_skinny16_cfg(const GemmParams& p, hipStream_t s) {
    constexpr int SW = 16 * CPL;
    const bool a_fast = TA || ((p.lda % 8 == 0) && !p.Aptr && ((reinterpret_cast<uintptr_t>(p.A) & 15) == 0) && (p.sA % 8 == 0));
    const int bw = TB ? 8 : CPL;    // elements per vector load of B
    const bool b_fast = (p.ldb % bw == 0) && !p.Bptr && ((reinterpret_cast<uintptr_t>(p.B) & 15) == 0) && (p.sB % 8 == 0);
    const bool fast = a_fast && b_fast && (p.K % 32 == 0) && (p.N % SW == 0);
    dim3 grid((unsigned)((p.N + SW - 1) / SW), (unsigned)p.batch);
    if (fast) hipLaunchKernelGGL((gemm_skinny16_kernel<DT, MB, CPL, TA, TB, true>), grid, dim3(512), 0, s, p);
    else hipLaunchKernelGGL((gemm_skinny16_kernel<DT, MB, CPL, TA, TB, false>), grid, dim3(512), 0, s, p);
    return hipGetLastError();
}

template <int DT, int MB, int CPL>
static hipError_t launch_skinny16_t(bool ta, bool tb, const GemmParams& p, hipStream_t s) {
    if (ta) return tb ? launch_skinny16_cfg<DT, MB, CPL, true, true>(p, s) : launch_skinny16_cfg<DT, MB, CPL, true, false>(p, s);
    return tb ? launch_skinny16_cfg<DT, MB, CPL, false, true>(p, s) : launch_skinny16_cfg<DT, MB, CPL, false, false>(p, s);
}

template <int DT>
static hipError_t launch_skinny16(bool ta, bool tb, const GemmParams& p, hipStream_t s) {
    // Columns per lane (strip = 16 x that): as many workgroups as possible without exceeding one per CU -- a second
    // round of workgroups costs more than narrower strips gain.  B stored [k][n] is loaded with (2 x columns)-byte
    // accesses, so 2 columns per lane (4-byte loads) is never worth it there.
    const int widest = p.M > 16 ? 4 : 8, narrowest = tb ? 2 : 4;
    int cpl = widest;
    for (int cand = widest; cand >= narrowest; cand >>= 1) {
        const int64_t wgs = ((p.N + 16 * cand - 1) / (16 * cand)) * (int64_t)p.batch;
        if (wgs <= 256) cpl = cand;
    }
    if (p.M <= 16) {
        if (cpl == 8) return launch_skinny16_t<DT, 1, 8>(ta, tb, p, s);
        if (cpl == 4) return launch_skinny16_t<DT, 1, 4>(ta, tb, p, s);
        return launch_skinny16_t<DT, 1, 2>(ta, tb, p, s);
    }
    if (cpl == 4) return launch_skinny16_t<DT, 2, 4>(ta, tb, p, s);
    return launch_skinny16_t<DT, 2, 2>(ta, tb, p, s);
}

hipError_t launch_gemm_skinny(int dtype, bool ta, bool tb, const GemmParams& p, hipStream_t s, bool* handled) {
    *handled = false;
    if (p.M > 32 || p.batch > 65535) return hipSuccess;
    if ((dtype == DT_F16 || dtype == DT_BF16) && p.K >= 128) {
        *handled = true;
        return dtype == DT_F16 ? launch_skinny16<DT_F16>(ta, tb, p, s) : launch_skinny16<DT_BF16>(ta, tb, p, s);
    }
    if (dtype != DT_F32 || p.K < 64) return hipSuccess;
    *handled = true;
    // widest strip that still gives every CU a workgroup
    const int64_t want = 256;
    int cpl = 4;
    if (p.M > 16) cpl = 2;
    while (cpl > 1 && ((p.N + 16 * cpl - 1) / (16 * cpl)) * (int64_t)p.batch < want) cpl >>= 1;
    if (p.M <= 16) {
        if (cpl == 4) return launch_skinny_t<1, 4>(ta, tb, p, s);
        if (cpl == 2) return launch_skinny_t<1, 2>(ta, tb, p, s);
        return launch_skinny_t<1, 1>(ta, tb, p, s);
    }
    if (cpl == 2) return launch_skinny_t<2, 2>(ta, tb, p, s);
    return launch_skinny_t<2, 1>(ta, tb, p, s);
}

}  // namespace ntg
