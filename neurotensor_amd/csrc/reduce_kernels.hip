// Small reductions and permutations around the GEMM kernels: the ordered sum of the split-K partial products, the
// ordered sum of per-image weight gradients, and the channel-swapped, tap-reversed copy of a convolution kernel.
// All are HBM bound, deterministic (fixed summation order, no atomics) and launched on the caller's stream.
#include "ntg_common.h"

#include <algorithm>
#include <cstring>

namespace ntg {

// out[i] (+)= sum over b of part[b*n + i], b ascending: the order in which per-image weight
// gradients are added up by the reference's batch loop (conv.cpp:466-469).
template <class T, class Acc>
__global__ void __launch_bounds__(256) reduce_batch_kernel(const T* __restrict__ part, T* __restrict__ out, const int64_t batch,
                                                           const int64_t n, const int accumulate) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        Acc acc = accumulate ? (Acc)out[i] : (Acc)0;
        for (int64_t b = 0; b < batch; ++b) acc += (Acc)part[b * n + i];
        out[i] = (T)acc;
    }
}


// The reference's own order for the element types whose sums are checked bit for bit (Float32, Float64, the complex types):
// conv_dkernel forms sum(0) of the per-image products first -- item 0, then += item 1, ... in the element type
// (tensor_files/sum_exp_log.cpp:112-124) -- and adds that sum to d_kernel last (conv.cpp:466-469).
template <class T>
__global__ void __launch_bounds__(256) reduce_batch_sum_first_kernel(const T* __restrict__ part, T* __restrict__ out, const int64_t batch,
                                                                     const int64_t n, const int accumulate) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        T acc = part[i];
        for (int64_t b = 1; b < batch; ++b) acc += part[b * n + i];
        if (accumulate) {
            T o = out[i];
            o += acc;
            acc = o;
        }
        out[i] = acc;
    }
}

// The same ordered sum for per-image weight gradients held channels-last, part[b][o][t][c], into the kernel's own layout
// out[o][c][t]: threads follow the partial sums (coalesced reads of the large side), the small result is written scattered.
template <class T, class Acc>
__global__ void __launch_bounds__(256) reduce_batch_taps_last_kernel(const T* __restrict__ part, T* __restrict__ out, const int64_t batch,
                                                                     const int64_t rows, const int64_t cg, const int64_t cgp, const int64_t taps,
                                                                     const int accumulate) {
    const int64_t n = rows * cgp * taps;                  // (the partial sums hold cgp >= cg channels per tap, the rest padding)
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        const int64_t c = i % cgp, t = (i / cgp) % taps, o = i / (cgp * taps);
        if (c >= cg) continue;
        T* dst = out + (o * cg + c) * taps + t;
        Acc acc = accumulate ? (Acc)*dst : (Acc)0;
        for (int64_t b = 0; b < batch; ++b) acc += (Acc)part[b * n + i];
        *dst = (T)acc;
    }
}

// The same with 16-byte loads: a thread owns VEC consecutive channels of one (row, tap) and keeps four partial-sum
// loads in flight; the order of the additions per element is unchanged.  Needs cg % VEC == 0 and aligned partial sums.
template <class T, class Acc>
__global__ void __launch_bounds__(256) reduce_batch_taps_last_vec_kernel(const T* __restrict__ part, T* __restrict__ out, const int64_t batch,
                                                                         const int64_t rows, const int64_t cg, const int64_t taps, const int accumulate) {
    constexpr int VEC = 16 / (int)sizeof(T);
    typedef T TV __attribute__((ext_vector_type(VEC)));
    const int64_t n = rows * cg * taps, nv = n / VEC;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; v < nv; v += stride) {
        const int64_t i = v * VEC;
        const int64_t c = i % cg, t = (i / cg) % taps, o = i / (cg * taps);
        T* dst = out + (o * cg + c) * taps + t;
        Acc acc[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] = accumulate ? (Acc)dst[(int64_t)e * taps] : (Acc)0;
        const T* pp = part + i;
        int64_t b = 0;
        for (; b + 4 <= batch; b += 4) {
            TV x[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) x[u] = *reinterpret_cast<const TV*>(pp + (b + u) * n);
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int e = 0; e < VEC; ++e) acc[e] += (Acc)x[u][e];
        }
        for (; b < batch; ++b) {
            const TV x = *reinterpret_cast<const TV*>(pp + b * n);
#pragma unroll
            for (int e = 0; e < VEC; ++e) acc[e] += (Acc)x[e];
        }
#pragma unroll
        for (int e = 0; e < VEC; ++e) dst[(int64_t)e * taps] = (T)acc[e];
    }
}

// Split-K epilogue: C (+)= sum over the k ranges of part[s][m][n], s ascending, starting from C0 (the incoming C, the
// broadcast bias, or zero).  One rounding to T at the end.
template <class T, class P, class Acc>
__global__ void __launch_bounds__(256) splitk_reduce_kernel(const P* __restrict__ part, const int splits, const int64_t split_stride, const GemmParams p) {
    const int64_t total = (int64_t)p.M * p.N;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const int64_t b = blockIdx.y;                                      // item of the batch: its partial sums follow the previous item's
    T* C = static_cast<T*>(p.C) + b * p.sC;
    const T* bias = static_cast<const T*>(p.bias) + b * p.bias_bs;
    part += b * total;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
        const int64_t m = idx / p.N, n = idx - m * p.N;
        T* cp = C + m * p.ldc + n;
        Acc acc = (Acc)0;
        if (p.cmode == C_ACCUMULATE) acc = (Acc)*cp;
        else if (p.cmode == C_BIAS) acc = (Acc)bias[m * p.bias_rs + n * p.bias_cs];
        for (int s = 0; s < splits; ++s) acc += (Acc)part[(int64_t)s * split_stride + idx];
        if (p.act == ACT_RELU) acc = acc > (Acc)0 ? acc : (Acc)0;
        *cp = (T)acc;
    }
}

// The same sum, four consecutive columns per thread with 16-byte accesses to the partial sums (rows of C and of the
// partial matrices must start on a multiple of four elements); the partial loads of four k ranges are in flight together.
template <class T, class P, class Acc>
__global__ void __launch_bounds__(256) splitk_reduce_vec_kernel(const P* __restrict__ part, const int splits, const int64_t split_stride, const GemmParams p) {
    typedef T TV __attribute__((ext_vector_type(4)));
    typedef P PV __attribute__((ext_vector_type(4)));
    const int64_t nq = p.N / 4, total = (int64_t)p.M * p.N, quads = (int64_t)p.M * nq;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const int64_t b = blockIdx.y;
    T* C = static_cast<T*>(p.C) + b * p.sC;
    const T* bias = static_cast<const T*>(p.bias) + b * p.bias_bs;
    part += b * total;
    for (int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; q < quads; q += stride) {
        const int64_t m = q / nq, n = (q - m * nq) * 4;
        TV* cp = reinterpret_cast<TV*>(C + m * p.ldc + n);
        Acc acc[4] = {(Acc)0, (Acc)0, (Acc)0, (Acc)0};
        if (p.cmode == C_ACCUMULATE) {
            const TV c0 = *cp;
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[e] = (Acc)c0[e];
        } else if (p.cmode == C_BIAS) {
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[e] = (Acc)bias[m * p.bias_rs + (n + e) * p.bias_cs];
        }
        const P* pp = part + q * 4;
        int s = 0;
        for (; s + 4 <= splits; s += 4) {
            PV v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = *reinterpret_cast<const PV*>(pp + (int64_t)(s + u) * split_stride);
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[e] += (Acc)v[u][e];
        }
        for (; s < splits; ++s) {
            const PV v = *reinterpret_cast<const PV*>(pp + (int64_t)s * split_stride);
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[e] += (Acc)v[e];
        }
        TV o;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = (T)((p.act == ACT_RELU && !(acc[e] > (Acc)0)) ? (Acc)0 : acc[e]);
        *cp = o;
    }
}

// p.batch items (at most 65535 per call): item b's partial sums start b * M * N elements into every k range's block, the
// ranges' blocks lie p.batch * M * N elements apart
template <class T, class P, class Acc>
static void launch_splitk_reduce_t(const void* part, int splits, const GemmParams& p, hipStream_t s) {
    const int64_t total = (int64_t)p.M * p.N, split_stride = total * p.batch;
    const bool vec = p.N % 4 == 0 && p.ldc % 4 == 0 && p.sC % 4 == 0 && (reinterpret_cast<uintptr_t>(p.C) % (4 * sizeof(T))) == 0 &&
                     (reinterpret_cast<uintptr_t>(part) % (4 * sizeof(P))) == 0;
    if (vec) hipLaunchKernelGGL((splitk_reduce_vec_kernel<T, P, Acc>), dim3(grid_for(total / 4), (unsigned)p.batch), dim3(256), 0, s, (const P*)part, splits, split_stride, p);
    else hipLaunchKernelGGL((splitk_reduce_kernel<T, P, Acc>), dim3(grid_for(total), (unsigned)p.batch), dim3(256), 0, s, (const P*)part, splits, split_stride, p);
}

// C[b][m][n] = C[b][m][n] > 0 ? C[b][m][n] : 0 -- relu_ = clamp_(x, 0) of the reference (activation_functions.cpp:143,
// min_max.cpp:115-121: max(x, 0) with the second operand returned for NaN and for -0)
template <class T>
__global__ void __launch_bounds__(256) relu_inplace_kernel(T* __restrict__ C, const int64_t ldc, const int64_t sC, const int64_t M, const int64_t N,
                                                           const int64_t batch) {
    const int64_t total = batch * M * N;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int64_t n = i % N, m = (i / N) % M, b = i / (N * M);
        T* cp = C + b * sC + m * ldc + n;
        const T v = *cp;
        if (!((float)v > 0.0f) || v != v) *cp = (T)0.0f;
    }
}
template <>
__global__ void __launch_bounds__(256) relu_inplace_kernel<double>(double* __restrict__ C, const int64_t ldc, const int64_t sC, const int64_t M,
                                                                   const int64_t N, const int64_t batch) {
    const int64_t total = batch * M * N;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int64_t n = i % N, m = (i / N) % M, b = i / (N * M);
        double* cp = C + b * sC + m * ldc + n;
        if (!(*cp > 0.0)) *cp = 0.0;
    }
}
hipError_t launch_relu_inplace(int dtype, void* C, int64_t ldc, int64_t sC, int64_t M, int64_t N, int64_t batch, hipStream_t s) {
    const int64_t total = batch * M * N;
    if (total <= 0) return hipSuccess;
    const dim3 g(grid_for(total)), t(256);
    switch (dtype) {
    case DT_F32: hipLaunchKernelGGL(relu_inplace_kernel<float>, g, t, 0, s, (float*)C, ldc, sC, M, N, batch); break;
    case DT_F64: hipLaunchKernelGGL(relu_inplace_kernel<double>, g, t, 0, s, (double*)C, ldc, sC, M, N, batch); break;
    case DT_F16: hipLaunchKernelGGL(relu_inplace_kernel<_Float16>, g, t, 0, s, (_Float16*)C, ldc, sC, M, N, batch); break;
    case DT_BF16: hipLaunchKernelGGL(relu_inplace_kernel<__bf16>, g, t, 0, s, (__bf16*)C, ldc, sC, M, N, batch); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_splitk_reduce(int dtype, const void* part, int splits, const GemmParams& p, hipStream_t s) {
    const int64_t total = (int64_t)p.M * p.N;
    if (total == 0 || p.batch < 1) return hipSuccess;
    if (p.batch > 65535) return hipErrorInvalidValue;
    switch (dtype) {
    case DT_F32: launch_splitk_reduce_t<float, float, float>(part, splits, p, s); break;
    case DT_F64: launch_splitk_reduce_t<double, double, double>(part, splits, p, s); break;
    case DT_F16: launch_splitk_reduce_t<_Float16, float, float>(part, splits, p, s); break;
    case DT_BF16: launch_splitk_reduce_t<__bf16, float, float>(part, splits, p, s); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}


// wt[g][c][oc][t] = w[g*og + oc][c][taps-1-t]: the kernel with input/output channels swapped
// inside each group and both tap axes reversed, i.e. the weights of the convolution that maps
// the output gradient back to the image.
template <class T>
__global__ void __launch_bounds__(256) flip_weights_kernel(const T* __restrict__ w, T* __restrict__ wt, const int64_t groups,
                                                           const int64_t og, const int64_t cg, const int64_t taps) {
    const int64_t total = groups * og * cg * taps;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
        const int64_t t = idx % taps;
        int64_t r = idx / taps;
        const int64_t oc = r % og;
        r /= og;
        const int64_t c = r % cg;
        const int64_t g = r / cg;
        wt[idx] = w[((g * og + oc) * cg + c) * taps + (taps - 1 - t)];
    }
}


hipError_t launch_reduce_batch(int dtype, const void* part, void* out, int64_t batch, int64_t n, int accumulate, hipStream_t s) {
    if (n == 0) return hipSuccess;
    const dim3 g(grid_for(n)), b(256);
    switch (dtype) {
    case DT_F32: hipLaunchKernelGGL((reduce_batch_sum_first_kernel<float>), g, b, 0, s, (const float*)part, (float*)out, batch, n, accumulate); break;
    case DT_F64: hipLaunchKernelGGL((reduce_batch_sum_first_kernel<double>), g, b, 0, s, (const double*)part, (double*)out, batch, n, accumulate); break;
    case DT_F16: hipLaunchKernelGGL((reduce_batch_kernel<_Float16, float>), g, b, 0, s, (const _Float16*)part, (_Float16*)out, batch, n, accumulate); break;
    case DT_BF16: hipLaunchKernelGGL((reduce_batch_kernel<__bf16, float>), g, b, 0, s, (const __bf16*)part, (__bf16*)out, batch, n, accumulate); break;
    case DT_C32: hipLaunchKernelGGL((reduce_batch_sum_first_kernel<LanePair<_Float16>>), g, b, 0, s, (const LanePair<_Float16>*)part, (LanePair<_Float16>*)out, batch, n, accumulate); break;
    case DT_C64: hipLaunchKernelGGL((reduce_batch_sum_first_kernel<LanePair<float>>), g, b, 0, s, (const LanePair<float>*)part, (LanePair<float>*)out, batch, n, accumulate); break;
    case DT_C128: hipLaunchKernelGGL((reduce_batch_sum_first_kernel<LanePair<double>>), g, b, 0, s, (const LanePair<double>*)part, (LanePair<double>*)out, batch, n, accumulate); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_reduce_batch_taps_last(int dtype, const void* part, void* out, int64_t batch, int64_t rows, int64_t cg, int64_t cgp,
                                         int64_t taps, int accumulate, hipStream_t s) {
    const int64_t n = rows * cgp * taps;
    if (n == 0) return hipSuccess;
    const int64_t vec = 16 / elem_size(dtype);
    if (cgp == cg && cg % vec == 0 && (reinterpret_cast<uintptr_t>(part) & 15) == 0) {
        const dim3 g(grid_for(n / vec)), b(256);
        switch (dtype) {
        case DT_F32: hipLaunchKernelGGL((reduce_batch_taps_last_vec_kernel<float, float>), g, b, 0, s, (const float*)part, (float*)out, batch, rows, cg, taps, accumulate); break;
        case DT_F16: hipLaunchKernelGGL((reduce_batch_taps_last_vec_kernel<_Float16, float>), g, b, 0, s, (const _Float16*)part, (_Float16*)out, batch, rows, cg, taps, accumulate); break;
        case DT_BF16: hipLaunchKernelGGL((reduce_batch_taps_last_vec_kernel<__bf16, float>), g, b, 0, s, (const __bf16*)part, (__bf16*)out, batch, rows, cg, taps, accumulate); break;
        default: return hipErrorInvalidValue;
        }
        return hipGetLastError();
    }
    const dim3 g(grid_for(n)), b(256);
    switch (dtype) {
    case DT_F32: hipLaunchKernelGGL((reduce_batch_taps_last_kernel<float, float>), g, b, 0, s, (const float*)part, (float*)out, batch, rows, cg, cgp, taps, accumulate); break;
    case DT_F16: hipLaunchKernelGGL((reduce_batch_taps_last_kernel<_Float16, float>), g, b, 0, s, (const _Float16*)part, (_Float16*)out, batch, rows, cg, cgp, taps, accumulate); break;
    case DT_BF16: hipLaunchKernelGGL((reduce_batch_taps_last_kernel<__bf16, float>), g, b, 0, s, (const __bf16*)part, (__bf16*)out, batch, rows, cg, cgp, taps, accumulate); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_flip_weights(int64_t es, const void* w, void* wt, int64_t groups, int64_t og, int64_t cg, int64_t taps, hipStream_t s) {
    const int64_t total = groups * og * cg * taps;
    if (total == 0) return hipSuccess;
    const dim3 g(grid_for(total)), b(256);
    switch (es) {
    case 2: hipLaunchKernelGGL(flip_weights_kernel<uint16_t>, g, b, 0, s, (const uint16_t*)w, (uint16_t*)wt, groups, og, cg, taps); break;
    case 4: hipLaunchKernelGGL(flip_weights_kernel<uint32_t>, g, b, 0, s, (const uint32_t*)w, (uint32_t*)wt, groups, og, cg, taps); break;
    case 8: hipLaunchKernelGGL(flip_weights_kernel<uint64_t>, g, b, 0, s, (const uint64_t*)w, (uint64_t*)wt, groups, og, cg, taps); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// out[b][p][c] = in[b][c][p]: an image batch from channel planes to channels-last, 64 x 64 tiles through LDS so that
// both the loads (along p) and the stores (along c) are coalesced.
// Where pixel p of the source image goes in a copy that carries a border of zero pixels (Wp == 0: no border, Pp == P)
struct PixRemap { int64_t Pp; uint32_t W, Wp, off0; };
__device__ __forceinline__ int64_t remap_pixel(const PixRemap& r, int64_t p) {
    return r.Wp ? p + (int64_t)((uint32_t)p / r.W) * (r.Wp - r.W) + r.off0 : p;
}
static PixRemap make_remap(const HaloMap* h, int64_t P) {
    PixRemap r;
    r.Pp = P; r.W = 1; r.Wp = 0; r.off0 = 0;
    if (h && h->Wp) { r.Pp = h->Hp * h->Wp; r.W = (uint32_t)h->W; r.Wp = (uint32_t)h->Wp; r.off0 = (uint32_t)(h->top * h->Wp + h->left); }
    return r;
}

// zeros the border pixels of a channels-last copy [B][Hp * Wp][C] (16-byte pieces; C * sizeof(T) a multiple of 16).
// Only the border is visited: its pixels are numbered top rows, bottom rows, then the left and right pieces of the
// image's rows.
// (vectors first, first + step, ... of the per_image 16-byte vectors of one image's border)
__device__ __forceinline__ void zero_border_vectors(uint4* __restrict__ img, const uint32_t per_image, const uint32_t vec_per_pixel, const HaloMap& h,
                                                    const uint32_t first, const uint32_t step) {
    const uint32_t top_n = (uint32_t)(h.top * h.Wp), bot_n = (uint32_t)((h.Hp - h.top - h.H) * h.Wp), side = (uint32_t)(h.Wp - h.W);
    for (uint32_t i = first; i < per_image; i += step) {
        uint32_t j = i / vec_per_pixel, pix;
        const uint32_t v = i - j * vec_per_pixel;
        if (j < top_n) pix = j;
        else if (j < top_n + bot_n) pix = (uint32_t)((h.top + h.H) * h.Wp) + (j - top_n);
        else {
            j -= top_n + bot_n;
            const uint32_t row = j / side, c = j - row * side;
            pix = (uint32_t)((h.top + row) * h.Wp) + (c < (uint32_t)h.left ? c : (uint32_t)h.W + c);
        }
        img[(int64_t)pix * vec_per_pixel + v] = make_uint4(0u, 0u, 0u, 0u);
    }
}
__global__ void __launch_bounds__(256) halo_zero_kernel(uint4* __restrict__ out, const uint32_t per_image, const uint32_t vec_per_pixel, const HaloMap h) {
    zero_border_vectors(out + (int64_t)blockIdx.y * (h.Hp * h.Wp) * vec_per_pixel, per_image, vec_per_pixel, h, blockIdx.x * 256u + threadIdx.x, gridDim.x * 256u);
}
hipError_t launch_halo_zero(int64_t es, void* out, int64_t batch, int64_t C, const HaloMap& h, hipStream_t s) {
    if ((C * es) % 16 != 0 || (reinterpret_cast<uintptr_t>(out) & 15) != 0) return hipErrorInvalidValue;
    const int64_t vpp = C * es / 16, border = h.Hp * h.Wp - h.H * h.W, per_image = border * vpp;
    if (batch <= 0 || per_image <= 0) return hipSuccess;
    if (per_image > 0x7fffffffLL || h.Hp * h.Wp > 0x7fffffffLL) return hipErrorInvalidValue;
    const int64_t gx = std::min<int64_t>((per_image + 255) / 256, 64);
    for (int64_t b0 = 0; b0 < batch; b0 += 65535) {
        const int64_t nb = std::min<int64_t>(batch - b0, 65535);
        hipLaunchKernelGGL(halo_zero_kernel, dim3((unsigned)gx, (unsigned)nb), dim3(256), 0, s,
                           (uint4*)out + b0 * h.Hp * h.Wp * vpp, (uint32_t)per_image, (uint32_t)vpp, h);
    }
    return hipGetLastError();
}

template <class T>
__global__ void __launch_bounds__(256) nchw_to_nhwc_kernel(const T* __restrict__ in, T* __restrict__ out, const int64_t C, const int64_t P, const PixRemap r) {
    __shared__ T tile[64][65];
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    const int64_t p0 = (int64_t)blockIdx.x * 64, c0 = (int64_t)blockIdx.y * 64, b = blockIdx.z;
    const T* src = in + b * C * P;
    T* dst = out + b * C * r.Pp;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int64_t c = c0 + ty + 4 * i, pp = p0 + tx;
        if (c < C && pp < P) tile[ty + 4 * i][tx] = src[c * P + pp];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int64_t pp = p0 + ty + 4 * i, c = c0 + tx;
        if (c < C && pp < P) dst[remap_pixel(r, pp) * C + c] = tile[tx][ty + 4 * i];
    }
}

// element idx of the two weight permutations (see weights_channels_last_kernel, flip_weights_channels_last_kernel)
template <class T>
__device__ __forceinline__ void weights_channels_last_elem(const T* __restrict__ w, T* __restrict__ wp, const int64_t idx, const int64_t cg, const int64_t cgp,
                                                           const int64_t taps, const int64_t chunk) {
    const int64_t c = idx % cgp;
    const int64_t t = (idx / cgp) % taps;
    const int64_t o = idx / (cgp * taps);
    // chunk != 0: the k order (run of `chunk` channels, tap, channel inside the run) instead of (tap, channel)
    const int64_t dst = chunk ? o * taps * cgp + ((c / chunk) * taps + t) * chunk + c % chunk : idx;
    wp[dst] = c < cg ? w[(o * cg + c) * taps + t] : (T)0;
}
template <class T>
__device__ __forceinline__ void flip_weights_channels_last_elem(const T* __restrict__ w, T* __restrict__ wt, const int64_t idx, const int64_t og, const int64_t ogp,
                                                                const int64_t cg, const int64_t taps, const int64_t chunk) {
    const int64_t oc = idx % ogp;
    int64_t r = idx / ogp;
    const int64_t t = r % taps;
    r /= taps;
    const int64_t c = r % cg;
    const int64_t g = r / cg;
    // chunk != 0: the k order (run of `chunk` out channels, tap, out channel inside the run) instead of (tap, out channel)
    const int64_t dst = chunk ? r * taps * ogp + ((oc / chunk) * taps + t) * chunk + oc % chunk : idx;
    wt[dst] = oc < og ? w[((g * og + oc) * cg + c) * taps + (taps - 1 - t)] : (T)0;
}
// what a channels-last copy takes along: the border of zero pixels of its own output and a weight permutation
struct CopyExtras { HaloMap h; uint32_t border_vecs, vpp; WeightsJob job; int64_t job_total; };

// The same copy with 16-byte accesses on both sides (C and P multiples of one 16-byte vector, aligned pointers): a
// thread loads VEC pixels of one channel, the tile goes through LDS as single elements (row pitch chosen so that the
// column-wise read-back spreads over the banks), and a thread stores VEC channels of one pixel.
template <class T>
__global__ void __launch_bounds__(256) nchw_to_nhwc_vec_kernel(const T* __restrict__ in, T* __restrict__ out, const int64_t C, const int64_t P, const PixRemap r,
                                                               const CopyExtras ex) {
    constexpr int VEC = 16 / (int)sizeof(T), VPR = 64 / VEC;            // elements per vector, vectors per tile row
    constexpr int PITCH = sizeof(T) == 2 ? 66 : 65;                     // elements: 33 / 65 words
    typedef T TV __attribute__((ext_vector_type(VEC)));
    __shared__ T tile[64 * PITCH];
    const int64_t p0 = (int64_t)blockIdx.x * 64, c0 = (int64_t)blockIdx.y * 64, b = blockIdx.z;
    const T* src = in + b * C * P;
    T* dst = out + b * C * r.Pp;
#pragma unroll
    for (int i = 0; i < 64 * VPR / 256; ++i) {
        const int v = threadIdx.x + 256 * i, c = v / VPR, pv = v % VPR;
        if (c0 + c < C && p0 + pv * VEC < P) {
            const TV x = *reinterpret_cast<const TV*>(src + (c0 + c) * P + p0 + pv * VEC);
#pragma unroll
            for (int e = 0; e < VEC; ++e) tile[c * PITCH + pv * VEC + e] = x[e];
        }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 64 * VPR / 256; ++i) {
        const int v = threadIdx.x + 256 * i, pp = v / VPR, cv = v % VPR;
        if (c0 + cv * VEC < C && p0 + pp < P) {
            TV x;
#pragma unroll
            for (int e = 0; e < VEC; ++e) x[e] = tile[(cv * VEC + e) * PITCH + pp];
            *reinterpret_cast<TV*>(dst + remap_pixel(r, p0 + pp) * C + c0 + cv * VEC) = x;
        }
    }
    // the blocks of an image share its border, all blocks of the launch the weight permutation (a few elements each)
    const uint32_t per_image = gridDim.x * gridDim.y, bid = blockIdx.y * gridDim.x + blockIdx.x;
    if (ex.border_vecs)
        zero_border_vectors(reinterpret_cast<uint4*>(dst), ex.border_vecs, ex.vpp, ex.h, bid * 256u + threadIdx.x, per_image * 256u);
    if (ex.job.kind) {
        const int64_t step = (int64_t)gridDim.z * per_image * 256;
        for (int64_t idx = ((int64_t)blockIdx.z * per_image + bid) * 256 + threadIdx.x; idx < ex.job_total; idx += step) {
            if (ex.job.kind == 1) weights_channels_last_elem<T>((const T*)ex.job.w, (T*)ex.job.wp, idx, ex.job.cg, ex.job.cgp, ex.job.taps, ex.job.chunk);
            else flip_weights_channels_last_elem<T>((const T*)ex.job.w, (T*)ex.job.wp, idx, ex.job.og, ex.job.ogp, ex.job.cg, ex.job.taps, ex.job.chunk);
        }
    }
}

hipError_t launch_nchw_to_nhwc(int64_t es, const void* in, void* out, int64_t batch, int64_t C, int64_t P, hipStream_t s, const HaloMap* halo,
                               const WeightsJob* job, bool* took_along) {
    if (took_along) *took_along = false;
    if (batch * C * P == 0) return hipSuccess;
    const PixRemap r = make_remap(halo, P);
    const int64_t gx = (P + 63) / 64, gy = (C + 63) / 64;
    if (gx > 0x7fffffffLL || gy > 65535) return hipErrorInvalidValue;
    const int64_t vec = 16 / es;
    const bool vec_ok = C % vec == 0 && P % vec == 0 && ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
    CopyExtras ex;
    std::memset(&ex, 0, sizeof ex);
    if (vec_ok && (es == 2 || es == 4) && took_along) {
        // (the caller acts on *took_along: without it the copy stays what it was)
        const int64_t vpp = C * es / 16, border = halo && halo->Wp ? halo->Hp * halo->Wp - halo->H * halo->W : 0;
        if (border * vpp <= 0x7fffffffLL && (!halo || halo->Hp * halo->Wp <= 0x7fffffffLL)) {
            if (border > 0) { ex.h = *halo; ex.border_vecs = (uint32_t)(border * vpp); ex.vpp = (uint32_t)vpp; }
            if (job && job->kind) {
                ex.job = *job;
                ex.job_total = job->kind == 1 ? job->a * job->cgp * job->taps : job->a * job->ogp * job->cg * job->taps;
            }
            *took_along = true;
        }
    }
    for (int64_t b0 = 0; b0 < batch; b0 += 65535) {                    // (grid z limit)
        const int64_t nb = batch - b0 < 65535 ? batch - b0 : 65535;
        const dim3 g((unsigned)gx, (unsigned)gy, (unsigned)nb), t(256);
        const char* src = static_cast<const char*>(in) + b0 * C * P * es;
        char* dst = static_cast<char*>(out) + b0 * C * r.Pp * es;
        if (es == 2 && vec_ok) hipLaunchKernelGGL(nchw_to_nhwc_vec_kernel<uint16_t>, g, t, 0, s, (const uint16_t*)src, (uint16_t*)dst, C, P, r, ex);
        else if (es == 4 && vec_ok) hipLaunchKernelGGL(nchw_to_nhwc_vec_kernel<uint32_t>, g, t, 0, s, (const uint32_t*)src, (uint32_t*)dst, C, P, r, ex);
        else if (es == 2) hipLaunchKernelGGL(nchw_to_nhwc_kernel<uint16_t>, g, t, 0, s, (const uint16_t*)src, (uint16_t*)dst, C, P, r);
        else if (es == 4) hipLaunchKernelGGL(nchw_to_nhwc_kernel<uint32_t>, g, t, 0, s, (const uint32_t*)src, (uint32_t*)dst, C, P, r);
        else return hipErrorInvalidValue;
        ex.job.kind = 0;                                               // (the first launch has done the weights)
    }
    return hipGetLastError();
}

// wt[g][c][t][oc] = w[g*og + oc][c][taps-1-t]: the weights of the convolution that maps the output gradient back to the
// image (channel axes swapped inside each group, taps reversed), with the out channels of one tap consecutive and
// padded with zeros from og to ogp per tap.
template <class T>
__global__ void __launch_bounds__(256) flip_weights_channels_last_kernel(const T* __restrict__ w, T* __restrict__ wt, const int64_t groups,
                                                                         const int64_t og, const int64_t ogp, const int64_t cg, const int64_t taps,
                                                                         const int64_t chunk) {
    const int64_t total = groups * ogp * cg * taps;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride)
        flip_weights_channels_last_elem<T>(w, wt, idx, og, ogp, cg, taps, chunk);
}

hipError_t launch_flip_weights_channels_last(int64_t es, const void* w, void* wt, int64_t groups, int64_t og, int64_t ogp, int64_t cg, int64_t taps, hipStream_t s,
                                             int64_t chunk) {
    const int64_t total = groups * ogp * cg * taps;
    if (total == 0) return hipSuccess;
    const dim3 g(grid_for(total)), t(256);
    switch (es) {
    case 2: hipLaunchKernelGGL(flip_weights_channels_last_kernel<uint16_t>, g, t, 0, s, (const uint16_t*)w, (uint16_t*)wt, groups, og, ogp, cg, taps, chunk); break;
    case 4: hipLaunchKernelGGL(flip_weights_channels_last_kernel<uint32_t>, g, t, 0, s, (const uint32_t*)w, (uint32_t*)wt, groups, og, ogp, cg, taps, chunk); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// Weights of one phase of a strided convolution's image gradient: the taps i = er + s_r (Mr-1-mr), j = ec + s_c (Mc-1-mc)
// of w [g*og + oc][c][k_r][k_c], as wt[g][c][(mr, mc)][oc] with the out channels padded with zeros from og to ogp.
struct PhaseWeights { int64_t groups, og, ogp, cg, k_r, k_c, er, ec, s_r, s_c, Mr, Mc; };
template <class T>
__global__ void __launch_bounds__(256) phase_weights_kernel(const T* __restrict__ w, T* __restrict__ wt, const PhaseWeights q) {
    const int64_t total = q.groups * q.cg * q.Mr * q.Mc * q.ogp;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
        const int64_t oc = idx % q.ogp;
        int64_t r = idx / q.ogp;
        const int64_t mc = r % q.Mc;
        r /= q.Mc;
        const int64_t mr = r % q.Mr;
        r /= q.Mr;
        const int64_t c = r % q.cg, g = r / q.cg;
        const int64_t i = q.er + q.s_r * (q.Mr - 1 - mr), j = q.ec + q.s_c * (q.Mc - 1 - mc);
        wt[idx] = oc < q.og ? w[(((g * q.og + oc) * q.cg + c) * q.k_r + i) * q.k_c + j] : (T)0;
    }
}

hipError_t launch_phase_weights(int64_t es, const void* w, void* wt, int64_t groups, int64_t og, int64_t ogp, int64_t cg, int64_t k_r, int64_t k_c,
                                int64_t er, int64_t ec, int64_t s_r, int64_t s_c, int64_t Mr, int64_t Mc, hipStream_t s) {
    const PhaseWeights q{groups, og, ogp, cg, k_r, k_c, er, ec, s_r, s_c, Mr, Mc};
    const int64_t total = groups * cg * Mr * Mc * ogp;
    if (total == 0) return hipSuccess;
    const dim3 g(grid_for(total)), t(256);
    switch (es) {
    case 2: hipLaunchKernelGGL(phase_weights_kernel<uint16_t>, g, t, 0, s, (const uint16_t*)w, (uint16_t*)wt, q); break;
    case 4: hipLaunchKernelGGL(phase_weights_kernel<uint32_t>, g, t, 0, s, (const uint32_t*)w, (uint32_t*)wt, q); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// im[b][c][y][x] (+)= the element of the phase plane that holds it: phase (er, ec) = ((y + p_r) % s_r, (x + p_c) % s_c)
// stores the image rows y = s_r (a0 + a) + er - p_r as its rows a (columns likewise); phases without taps contribute zero.
template <class T, class Acc>
__global__ void __launch_bounds__(256) phase_interleave_kernel(const T* __restrict__ tmp, T* __restrict__ im, const PhaseLayout q, const int accumulate) {
    const uint32_t idx = blockIdx.x * 256u + threadIdx.x;
    if (idx >= q.total) return;
    const uint32_t t = fast_div(idx, q.div_w), x = idx - t * (uint32_t)q.W;
    const uint32_t bc = fast_div(t, q.div_h), y = t - bc * (uint32_t)q.H;
    const uint32_t Y = y + (uint32_t)q.p_r, X = x + (uint32_t)q.p_c;
    const uint32_t ar = fast_div(Y, q.div_sr), er = Y - ar * (uint32_t)q.s_r;
    const uint32_t ac = fast_div(X, q.div_sc), ec = X - ac * (uint32_t)q.s_c;
    Acc v = accumulate ? (Acc)im[idx] : (Acc)0;
    const int ph = (int)(er * (uint32_t)q.s_c + ec);
    if (q.off[ph] >= 0) {
        const int a = (int)ar - q.a0r[er], b = (int)ac - q.a0c[ec];      // inside the plane by construction
        v += (Acc)tmp[q.off[ph] + ((int64_t)bc * q.hp[er] + a) * q.wp[ec] + b];
    }
    im[idx] = (T)v;
}

hipError_t launch_phase_interleave(int dtype, const void* tmp, void* im, const PhaseLayout& q, int accumulate, hipStream_t s) {
    if (q.total == 0) return hipSuccess;
    const dim3 g((q.total + 255u) / 256u), t(256);
    switch (dtype) {
    case DT_F32: hipLaunchKernelGGL((phase_interleave_kernel<float, float>), g, t, 0, s, (const float*)tmp, (float*)im, q, accumulate); break;
    case DT_F16: hipLaunchKernelGGL((phase_interleave_kernel<_Float16, float>), g, t, 0, s, (const _Float16*)tmp, (_Float16*)im, q, accumulate); break;
    case DT_BF16: hipLaunchKernelGGL((phase_interleave_kernel<__bf16, float>), g, t, 0, s, (const __bf16*)tmp, (__bf16*)im, q, accumulate); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// wp[o][t][c] = w[o][c][t]: convolution weights with the channel index fastest (the k order of the channels-last gather),
// the channels of one tap padded with zeros from cg to cgp
template <class T>
__global__ void __launch_bounds__(256) weights_channels_last_kernel(const T* __restrict__ w, T* __restrict__ wp, const int64_t rows,
                                                                    const int64_t cg, const int64_t cgp, const int64_t taps, const int64_t chunk) {
    const int64_t total = rows * cgp * taps;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride)
        weights_channels_last_elem<T>(w, wp, idx, cg, cgp, taps, chunk);
}

hipError_t launch_weights_channels_last(int64_t es, const void* w, void* wp, int64_t rows, int64_t cg, int64_t cgp, int64_t taps, hipStream_t s, int64_t chunk) {
    const int64_t total = rows * cgp * taps;
    if (total == 0) return hipSuccess;
    const dim3 g(grid_for(total)), t(256);
    switch (es) {
    case 2: hipLaunchKernelGGL(weights_channels_last_kernel<uint16_t>, g, t, 0, s, (const uint16_t*)w, (uint16_t*)wp, rows, cg, cgp, taps, chunk); break;
    case 4: hipLaunchKernelGGL(weights_channels_last_kernel<uint32_t>, g, t, 0, s, (const uint32_t*)w, (uint32_t*)wp, rows, cg, cgp, taps, chunk); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// wp[o][r][q][c] = w[o][c][r][q] with every tap row padded with zeros from k_c to kq_pad taps and the channels from cg to cgp
template <class T>
__global__ void __launch_bounds__(256) weights_channels_last_rows_kernel(const T* __restrict__ w, T* __restrict__ wp, const int64_t rows, const int64_t cg,
                                                                         const int64_t cgp, const int64_t k_r, const int64_t k_c, const int64_t kq_pad) {
    const int64_t total = rows * k_r * kq_pad * cgp;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
        const int64_t c = idx % cgp;
        int64_t t = idx / cgp;
        const int64_t q = t % kq_pad;
        t /= kq_pad;
        const int64_t r = t % k_r, o = t / k_r;
        wp[idx] = (c < cg && q < k_c) ? w[((o * cg + c) * k_r + r) * k_c + q] : (T)0;
    }
}

hipError_t launch_weights_channels_last_rows(int64_t es, const void* w, void* wp, int64_t rows, int64_t cg, int64_t cgp, int64_t k_r, int64_t k_c,
                                             int64_t kq_pad, hipStream_t s) {
    const int64_t total = rows * k_r * kq_pad * cgp;
    if (total == 0) return hipSuccess;
    const dim3 g(grid_for(total)), t(256);
    switch (es) {
    case 2: hipLaunchKernelGGL(weights_channels_last_rows_kernel<uint16_t>, g, t, 0, s, (const uint16_t*)w, (uint16_t*)wp, rows, cg, cgp, k_r, k_c, kq_pad); break;
    case 4: hipLaunchKernelGGL(weights_channels_last_rows_kernel<uint32_t>, g, t, 0, s, (const uint32_t*)w, (uint32_t*)wp, rows, cg, cgp, k_r, k_c, kq_pad); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// out[b][p][g*cgp + c] = in[b][g*cg + c][p] for c < cg, 0 for cg <= c < cgp: the channels-last copy with the channels of
// every group padded to cgp.  64 x 64 tiles of (channel inside the group, pixel) through LDS, like the plain copy.
template <class T>
__global__ void __launch_bounds__(256) nchw_to_nhwc_pad_kernel(const T* __restrict__ in, T* __restrict__ out, const int64_t groups,
                                                               const int64_t cg, const int64_t cgp, const int64_t P, const int cblocks, const PixRemap r) {
    __shared__ T tile[64][65];
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    const int64_t g = blockIdx.y / cblocks, c0 = (int64_t)(blockIdx.y % cblocks) * 64;
    const int64_t p0 = (int64_t)blockIdx.x * 64, b = blockIdx.z;
    const T* src = in + (b * groups + g) * cg * P;
    T* dst = out + b * r.Pp * groups * cgp + g * cgp;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int64_t c = c0 + ty + 4 * i, pp = p0 + tx;
        tile[ty + 4 * i][tx] = (c < cg && pp < P) ? src[c * P + pp] : (T)0;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int64_t pp = p0 + ty + 4 * i, c = c0 + tx;
        if (c < cgp && pp < P) dst[remap_pixel(r, pp) * groups * cgp + c] = tile[tx][ty + 4 * i];
    }
}

// The same for groups of at most 32 bytes of channels (padded to 16 or 32 bytes): one thread per pixel and group reads its
// cg channels (each a coalesced stream over the pixels) and stores the padded run with 16-byte stores.
template <class T, int CP>
__global__ void __launch_bounds__(256) nchw_to_nhwc_few_kernel(const T* __restrict__ in, T* __restrict__ out, const int64_t total, const int64_t groups,
                                                               const int64_t cg, const int64_t P, const PixRemap r) {
    constexpr int VEC = 16 / (int)sizeof(T);
    typedef T TV __attribute__((ext_vector_type(VEC)));
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const int64_t pp = idx % P, bg = idx / P, b = bg / groups, g = bg - b * groups;
    const T* src = in + bg * cg * P + pp;
    TV* dst = reinterpret_cast<TV*>(out + ((b * r.Pp + remap_pixel(r, pp)) * groups + g) * CP);
#pragma unroll
    for (int v = 0; v < CP / VEC; ++v) {
        TV x;
#pragma unroll
        for (int e = 0; e < VEC; ++e) x[e] = (v * VEC + e) < cg ? src[(int64_t)(v * VEC + e) * P] : (T)0;
        dst[v] = x;
    }
}

hipError_t launch_nchw_to_nhwc_padded(int64_t es, const void* in, void* out, int64_t batch, int64_t groups, int64_t cg, int64_t cgp, int64_t P, hipStream_t s,
                                      const HaloMap* halo) {
    if (batch * groups * cgp * P == 0) return hipSuccess;
    const PixRemap r = make_remap(halo, P);
    if (cgp * es <= 32 && (cgp * es) % 16 == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0) {
        const int64_t total = batch * groups * P, blocks = (total + 255) / 256;
        if (blocks <= 0x7fffffffLL) {
            const dim3 g((unsigned)blocks), t(256);
            if (es == 2 && cgp == 8) hipLaunchKernelGGL((nchw_to_nhwc_few_kernel<uint16_t, 8>), g, t, 0, s, (const uint16_t*)in, (uint16_t*)out, total, groups, cg, P, r);
            else if (es == 2) hipLaunchKernelGGL((nchw_to_nhwc_few_kernel<uint16_t, 16>), g, t, 0, s, (const uint16_t*)in, (uint16_t*)out, total, groups, cg, P, r);
            else if (es == 4 && cgp == 4) hipLaunchKernelGGL((nchw_to_nhwc_few_kernel<uint32_t, 4>), g, t, 0, s, (const uint32_t*)in, (uint32_t*)out, total, groups, cg, P, r);
            else if (es == 4) hipLaunchKernelGGL((nchw_to_nhwc_few_kernel<uint32_t, 8>), g, t, 0, s, (const uint32_t*)in, (uint32_t*)out, total, groups, cg, P, r);
            else return hipErrorInvalidValue;
            return hipGetLastError();
        }
    }
    const int64_t cblocks = (cgp + 63) / 64, gx = (P + 63) / 64, gy = cblocks * groups;
    if (gx > 0x7fffffffLL || gy > 65535) return hipErrorInvalidValue;
    for (int64_t b0 = 0; b0 < batch; b0 += 65535) {                    // (grid z limit)
        const int64_t nb = batch - b0 < 65535 ? batch - b0 : 65535;
        const dim3 g((unsigned)gx, (unsigned)gy, (unsigned)nb), t(256);
        const char* src = static_cast<const char*>(in) + b0 * groups * cg * P * es;
        char* dst = static_cast<char*>(out) + b0 * groups * cgp * r.Pp * es;
        if (es == 2) hipLaunchKernelGGL(nchw_to_nhwc_pad_kernel<uint16_t>, g, t, 0, s, (const uint16_t*)src, (uint16_t*)dst, groups, cg, cgp, P, (int)cblocks, r);
        else if (es == 4) hipLaunchKernelGGL(nchw_to_nhwc_pad_kernel<uint32_t>, g, t, 0, s, (const uint32_t*)src, (uint32_t*)dst, groups, cg, cgp, P, (int)cblocks, r);
        else return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace ntg
