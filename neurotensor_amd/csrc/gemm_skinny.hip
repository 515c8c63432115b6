// Skinny Float32 GEMM (m <= 32): C[m, n] (+)= op(A)[m, k] . op(B)[k, n]
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

    const float* A = p.Aptr ? static_cast<const float*>(p.Aptr[b]) : static_cast<const float*>(p.A) + (int64_t)b * p.sA;
    const float* B = p.Bptr ? static_cast<const float*>(p.Bptr[b]) : static_cast<const float*>(p.B) + (int64_t)b * p.sB;
    float* C = p.Cptr ? static_cast<float*>(p.Cptr[b]) : static_cast<float*>(p.C) + (int64_t)b * p.sC;

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
                const floatx4 t = (row < p.M) ? *reinterpret_cast<const floatx4*>(A + (int64_t)row * p.lda + kl) : floatx4{0.f, 0.f, 0.f, 0.f};
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
                    const fv t = *reinterpret_cast<const fv*>(B + (int64_t)k * p.ldb + n0 + CPL * c);
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
                    const floatx4 t = *reinterpret_cast<const floatx4*>(B + (int64_t)n * p.ldb + kl);
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

#pragma unroll
    for (int d = 0; d < D; ++d)
        if (wave + d * NW < steps) load_step(d, wave + d * NW);

    for (int base = wave; base < steps; base += D * NW) {
#pragma unroll
        for (int d = 0; d < D; ++d) {
            const int s = base + d * NW;
            if (s < steps) {
#pragma unroll
                for (int e = 0; e < 4; ++e)
#pragma unroll
                    for (int i = 0; i < MB; ++i)
#pragma unroll
                        for (int j = 0; j < CPL; ++j)
                            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[d][i][e], bv[d][e][j], acc[i][j], 0, 0, 0);
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
    const float* bias = static_cast<const float*>(p.bias);
    for (int idx = tid; idx < TOTAL; idx += 512) {
        const int l = idx & 63, q = idx >> 6;
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) sum += part[w][q][l];     // fixed order: deterministic
        const int r = q & 3, j = (q >> 2) % CPL, i = (q >> 2) / CPL;
        const int m = i * 16 + 4 * (l >> 4) + r;
        const int n = n0 + CPL * (l & 15) + j;
        if (m < p.M && n < p.N) {
            float* cp = C + (int64_t)m * p.ldc + n;
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

hipError_t launch_gemm_skinny(int dtype, bool ta, bool tb, const GemmParams& p, hipStream_t s, bool* handled) {
    *handled = false;
    if (dtype != DT_F32 || p.M > 32 || p.K < 64 || p.batch > 65535) return hipSuccess;
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
