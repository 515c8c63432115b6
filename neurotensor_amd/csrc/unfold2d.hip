// im2col on the GPU: col[b, c*kh*kw + i*kw + j, h*Wo + w] = im[b, c, h*s_r - p_r + i*d_r, w*s_c - p_c + j*d_c]
// (zero where the tap falls in the padding).  Same layout as the reference's im2col_cpu
// (nt/functional/cpu/unfold2d.cpp:12-112) behind functional::unfold2d(..., transpose_out=true)
// (nt/functional/tensor_files/colim_transform.cpp:565-588).  Pure data movement, HBM bound:
// one lane per output element, the fast index runs along Wo so stores are coalesced and,
// for stride 1, so are the loads.
#include "ntg_common.h"

namespace ntg {

struct UnfoldParams {
    int64_t batch, channels, height, width;
    int64_t k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c;
    int64_t Ho, Wo, ccol, total;
};

template <class T>
__global__ void __launch_bounds__(256) unfold2d_kernel(const T* __restrict__ im, T* __restrict__ col, const UnfoldParams u) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < u.total; idx += stride) {
        const int64_t w = idx % u.Wo;
        int64_t t = idx / u.Wo;
        const int64_t h = t % u.Ho;
        t /= u.Ho;
        const int64_t c = t % u.ccol;
        const int64_t b = t / u.ccol;
        const int64_t j = c % u.k_c;
        const int64_t i = (c / u.k_c) % u.k_r;
        const int64_t c_im = c / (u.k_r * u.k_c);
        const int64_t hp = h * u.s_r - u.p_r + i * u.d_r;
        const int64_t wp = w * u.s_c - u.p_c + j * u.d_c;
        T v = 0;
        if (hp >= 0 && hp < u.height && wp >= 0 && wp < u.width)
            v = im[((b * u.channels + c_im) * u.height + hp) * u.width + wp];
        col[idx] = v;
    }
}

// The same matrix, 16 bytes of consecutive outputs per lane (V = 16 / sizeof(T) elements of one row of col) and 32-bit
// index arithmetic with multiply-shift divisions: for L = Ho*Wo a multiple of V every vector lies inside one row
// (b, kk) of col and is 16-byte aligned.  One workgroup covers 256 vectors of one row, so b and the tap (c, i, j) are
// uniform; a lane splits its first l into (h, w) once and walks on element by element (the vector may cross the end
// of an output row).
struct UnfoldVecParams {
    int channels, height, width, k_c, s_r, s_c, p_r, p_c, d_r, d_c, Wo, ccol, vec_per_row, blocks_per_row;
    FastDiv div_bpr, div_ccol, div_krc, div_kc, div_wo;
    int k_rc;
    int64_t L;
};

template <class T>
__global__ void __launch_bounds__(256) unfold2d_vec_kernel(const T* __restrict__ im, T* __restrict__ col, const UnfoldVecParams u) {
    constexpr int V = 16 / (int)sizeof(T);
    const uint32_t row = fast_div(blockIdx.x, u.div_bpr);
    const uint32_t lv = (blockIdx.x - row * (uint32_t)u.blocks_per_row) * 256u + threadIdx.x;
    if (lv >= (uint32_t)u.vec_per_row) return;
    const uint32_t b = fast_div(row, u.div_ccol), kk = row - b * (uint32_t)u.ccol;
    const uint32_t c = fast_div(kk, u.div_krc), rem = kk - c * (uint32_t)u.k_rc;
    const uint32_t i = fast_div(rem, u.div_kc), j = rem - i * (uint32_t)u.k_c;
    const T* plane = im + ((int64_t)b * u.channels + c) * ((int64_t)u.height * u.width);
    const uint32_t l0 = lv * V;
    uint32_t h = fast_div(l0, u.div_wo), w = l0 - h * (uint32_t)u.Wo;
    const int dh = (int)i * u.d_r - u.p_r, dw = (int)j * u.d_c - u.p_c;
    T v[V];
#pragma unroll
    for (int e = 0; e < V; ++e) {
        const int hp = (int)h * u.s_r + dh, wp = (int)w * u.s_c + dw;
        const bool ok = (unsigned)hp < (unsigned)u.height && (unsigned)wp < (unsigned)u.width;
        v[e] = ok ? plane[(int64_t)hp * u.width + wp] : (T)0;
        if (++w == (uint32_t)u.Wo) { w = 0; ++h; }
    }
    typedef uint32_t u32x4v __attribute__((ext_vector_type(4)));
    u32x4v o;
    __builtin_memcpy(&o, v, 16);
    *reinterpret_cast<u32x4v*>(col + (int64_t)row * u.L + l0) = o;
}

// col2im, the adjoint of the above (im2col_backward_cpu, nt/functional/cpu/unfold2d_backward.cpp:9-56):
//   im[b, c, y, x] (+)= sum over taps (i, j) of col[b, c*kh*kw + i*kw + j, h*Wo + w]
//   with  y = h*s_r - p_r + i*d_r,  x = w*s_c - p_c + j*d_c.
// Written as a gather -- one lane per image element, taps visited in ascending (i, j), which
// is the order in which the reference's scatter loop reaches that element -- so there are no
// atomics and the floating-point sum is reproducible.
template <class T, class Acc>
__global__ void __launch_bounds__(256) col2im_kernel(const T* __restrict__ col, T* __restrict__ im, const UnfoldParams u, const int accumulate) {
    const int64_t total = u.batch * u.channels * u.height * u.width;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
        const int64_t x = idx % u.width;
        int64_t t = idx / u.width;
        const int64_t y = t % u.height;
        t /= u.height;
        const int64_t c = t % u.channels;
        const int64_t b = t / u.channels;
        Acc acc = accumulate ? (Acc)im[idx] : (Acc)0;
        for (int64_t i = 0; i < u.k_r; ++i) {
            const int64_t hn = y + u.p_r - i * u.d_r;
            if (hn < 0 || hn % u.s_r != 0) continue;
            const int64_t h = hn / u.s_r;
            if (h >= u.Ho) continue;
            for (int64_t j = 0; j < u.k_c; ++j) {
                const int64_t wn = x + u.p_c - j * u.d_c;
                if (wn < 0 || wn % u.s_c != 0) continue;
                const int64_t w = wn / u.s_c;
                if (w >= u.Wo) continue;
                const int64_t cc = (c * u.k_r + i) * u.k_c + j;
                acc += (Acc)col[((b * u.ccol + cc) * u.Ho + h) * u.Wo + w];
            }
        }
        im[idx] = (T)acc;
    }
}

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

static unsigned grid_for(int64_t total) {
    int64_t blocks = (total + 255) / 256;
    if (blocks > 256 * 64) blocks = 256 * 64;
    return (unsigned)(blocks < 1 ? 1 : blocks);
}

// Split-K epilogue: C (+)= sum over the k ranges of part[s][m][n], s ascending, starting from C0 (the incoming C, the
// broadcast bias, or zero).  One rounding to T at the end.
template <class T, class P, class Acc>
__global__ void __launch_bounds__(256) splitk_reduce_kernel(const P* __restrict__ part, const int splits, const GemmParams p) {
    const int64_t total = (int64_t)p.M * p.N;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    T* C = static_cast<T*>(p.C);
    const T* bias = static_cast<const T*>(p.bias);
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
        const int64_t m = idx / p.N, n = idx - m * p.N;
        T* cp = C + m * p.ldc + n;
        Acc acc = (Acc)0;
        if (p.cmode == C_ACCUMULATE) acc = (Acc)*cp;
        else if (p.cmode == C_BIAS) acc = (Acc)bias[m * p.bias_rs + n * p.bias_cs];
        for (int s = 0; s < splits; ++s) acc += (Acc)part[(int64_t)s * total + idx];
        *cp = (T)acc;
    }
}

// The same sum, four consecutive columns per thread with 16-byte accesses to the partial sums (rows of C and of the
// partial matrices must start on a multiple of four elements); the partial loads of four k ranges are in flight together.
template <class T, class P, class Acc>
__global__ void __launch_bounds__(256) splitk_reduce_vec_kernel(const P* __restrict__ part, const int splits, const GemmParams p) {
    typedef T TV __attribute__((ext_vector_type(4)));
    typedef P PV __attribute__((ext_vector_type(4)));
    const int64_t nq = p.N / 4, total = (int64_t)p.M * p.N, quads = (int64_t)p.M * nq;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    T* C = static_cast<T*>(p.C);
    const T* bias = static_cast<const T*>(p.bias);
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
            for (int u = 0; u < 4; ++u) v[u] = *reinterpret_cast<const PV*>(pp + (int64_t)(s + u) * total);
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[e] += (Acc)v[u][e];
        }
        for (; s < splits; ++s) {
            const PV v = *reinterpret_cast<const PV*>(pp + (int64_t)s * total);
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[e] += (Acc)v[e];
        }
        TV o;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = (T)acc[e];
        *cp = o;
    }
}

template <class T, class P, class Acc>
static void launch_splitk_reduce_t(const void* part, int splits, const GemmParams& p, hipStream_t s) {
    const int64_t total = (int64_t)p.M * p.N;
    const bool vec = p.N % 4 == 0 && p.ldc % 4 == 0 && (reinterpret_cast<uintptr_t>(p.C) % (4 * sizeof(T))) == 0 &&
                     (reinterpret_cast<uintptr_t>(part) % (4 * sizeof(P))) == 0;
    if (vec) hipLaunchKernelGGL((splitk_reduce_vec_kernel<T, P, Acc>), dim3(grid_for(total / 4)), dim3(256), 0, s, (const P*)part, splits, p);
    else hipLaunchKernelGGL((splitk_reduce_kernel<T, P, Acc>), dim3(grid_for(total)), dim3(256), 0, s, (const P*)part, splits, p);
}

hipError_t launch_splitk_reduce(int dtype, const void* part, int splits, const GemmParams& p, hipStream_t s) {
    const int64_t total = (int64_t)p.M * p.N;
    if (total == 0) return hipSuccess;
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
    case DT_F32: hipLaunchKernelGGL((reduce_batch_kernel<float, float>), g, b, 0, s, (const float*)part, (float*)out, batch, n, accumulate); break;
    case DT_F64: hipLaunchKernelGGL((reduce_batch_kernel<double, double>), g, b, 0, s, (const double*)part, (double*)out, batch, n, accumulate); break;
    case DT_F16: hipLaunchKernelGGL((reduce_batch_kernel<_Float16, float>), g, b, 0, s, (const _Float16*)part, (_Float16*)out, batch, n, accumulate); break;
    case DT_BF16: hipLaunchKernelGGL((reduce_batch_kernel<__bf16, float>), g, b, 0, s, (const __bf16*)part, (__bf16*)out, batch, n, accumulate); break;
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

// ---- the same two transforms over up to NTG_MAX_SPATIAL axes (unfold3d / unfoldnd and their adjoints:
// nt/functional/cpu/unfold3d.cpp:9-80, unfoldnd.cpp, unfold3d_backward.cpp, unfoldnd_backward.cpp).
// Row index of col: ((c*k0 + t0)*k1 + t1)*... ; column index: (o0*out1 + o1)*... ; last axis fastest.
template <class T>
__global__ void __launch_bounds__(256) unfoldnd_kernel(const T* __restrict__ im, T* __restrict__ col, const UnfoldNdParams u) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < u.total; idx += stride) {
        int64_t l = idx % u.L;
        int64_t t = idx / u.L;
        const int64_t c = t % u.ccol;
        const int64_t b = t / u.ccol;
        int64_t tap = c % u.taps;
        const int64_t c_im = c / u.taps;
        int64_t off = 0, mult = 1;
        bool ok = true;
        for (int a = u.nd - 1; a >= 0; --a) {
            const int64_t o = l % u.out[a];
            l /= u.out[a];
            const int64_t kk = tap % u.k[a];
            tap /= u.k[a];
            const int64_t pos = o * u.s[a] - u.p[a] + kk * u.d[a];
            ok = ok && pos >= 0 && pos < u.size[a];
            off += pos * mult;
            mult *= u.size[a];
        }
        T v = 0;
        if (ok) v = im[(b * u.channels + c_im) * u.vol + off];
        col[idx] = v;
    }
}

// gather form of the adjoint: taps visited in ascending order, as the reference's scatter loop reaches an element
template <class T, class Acc>
__global__ void __launch_bounds__(256) col2imnd_kernel(const T* __restrict__ col, T* __restrict__ im, const UnfoldNdParams u, const int accumulate) {
    const int64_t total = u.batch * u.channels * u.vol;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
        int64_t pos[NTG_MAX_SPATIAL];
        int64_t r = idx;
        for (int a = u.nd - 1; a >= 0; --a) {
            pos[a] = r % u.size[a];
            r /= u.size[a];
        }
        const int64_t c = r % u.channels;
        const int64_t b = r / u.channels;
        Acc acc = accumulate ? (Acc)im[idx] : (Acc)0;
        for (int64_t tap = 0; tap < u.taps; ++tap) {
            int64_t tt = tap, l = 0, mult = 1;
            bool ok = true;
            for (int a = u.nd - 1; a >= 0 && ok; --a) {
                const int64_t kk = tt % u.k[a];
                tt /= u.k[a];
                const int64_t on = pos[a] + u.p[a] - kk * u.d[a];
                if (on < 0 || on % u.s[a] != 0 || on / u.s[a] >= u.out[a]) { ok = false; break; }
                l += (on / u.s[a]) * mult;
                mult *= u.out[a];
            }
            if (ok) acc += (Acc)col[((b * u.ccol + c * u.taps + tap) * u.L) + l];
        }
        im[idx] = (T)acc;
    }
}

hipError_t launch_unfoldnd(int64_t es, const void* im, void* col, const UnfoldNdParams& u, hipStream_t s) {
    if (u.total == 0) return hipSuccess;
    const dim3 g(grid_for(u.total)), b(256);
    switch (es) {
    case 1: hipLaunchKernelGGL(unfoldnd_kernel<uint8_t>, g, b, 0, s, (const uint8_t*)im, (uint8_t*)col, u); break;
    case 2: hipLaunchKernelGGL(unfoldnd_kernel<uint16_t>, g, b, 0, s, (const uint16_t*)im, (uint16_t*)col, u); break;
    case 4: hipLaunchKernelGGL(unfoldnd_kernel<uint32_t>, g, b, 0, s, (const uint32_t*)im, (uint32_t*)col, u); break;
    case 8: hipLaunchKernelGGL(unfoldnd_kernel<uint64_t>, g, b, 0, s, (const uint64_t*)im, (uint64_t*)col, u); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_col2imnd(int dtype, const void* col, void* im, const UnfoldNdParams& u, int accumulate, hipStream_t s) {
    const int64_t total = u.batch * u.channels * u.vol;
    if (total == 0) return hipSuccess;
    const dim3 g(grid_for(total)), b(256);
    switch (dtype) {
    case DT_F32: hipLaunchKernelGGL((col2imnd_kernel<float, float>), g, b, 0, s, (const float*)col, (float*)im, u, accumulate); break;
    case DT_F64: hipLaunchKernelGGL((col2imnd_kernel<double, double>), g, b, 0, s, (const double*)col, (double*)im, u, accumulate); break;
    case DT_F16: hipLaunchKernelGGL((col2imnd_kernel<_Float16, float>), g, b, 0, s, (const _Float16*)col, (_Float16*)im, u, accumulate); break;
    case DT_BF16: hipLaunchKernelGGL((col2imnd_kernel<__bf16, float>), g, b, 0, s, (const __bf16*)col, (__bf16*)im, u, accumulate); break;
    case DT_I8: case DT_U8: hipLaunchKernelGGL((col2imnd_kernel<uint8_t, uint8_t>), g, b, 0, s, (const uint8_t*)col, (uint8_t*)im, u, accumulate); break;
    case DT_I16: case DT_U16: hipLaunchKernelGGL((col2imnd_kernel<uint16_t, uint16_t>), g, b, 0, s, (const uint16_t*)col, (uint16_t*)im, u, accumulate); break;
    case DT_I32: case DT_U32: hipLaunchKernelGGL((col2imnd_kernel<uint32_t, uint32_t>), g, b, 0, s, (const uint32_t*)col, (uint32_t*)im, u, accumulate); break;
    case DT_I64: case DT_U64: hipLaunchKernelGGL((col2imnd_kernel<uint64_t, uint64_t>), g, b, 0, s, (const uint64_t*)col, (uint64_t*)im, u, accumulate); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

static hipError_t fill_params(UnfoldParams& u, int64_t batch, int64_t channels, int64_t height, int64_t width,
                              int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c, int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c) {
    u.batch = batch; u.channels = channels; u.height = height; u.width = width;
    u.k_r = k_r; u.k_c = k_c; u.s_r = s_r; u.s_c = s_c; u.p_r = p_r; u.p_c = p_c; u.d_r = d_r; u.d_c = d_c;
    u.Ho = (height + 2 * p_r - d_r * (k_r - 1) - 1) / s_r + 1;
    u.Wo = (width + 2 * p_c - d_c * (k_c - 1) - 1) / s_c + 1;
    if (u.Ho <= 0 || u.Wo <= 0) return hipErrorInvalidValue;
    u.ccol = channels * k_r * k_c;
    u.total = batch * u.ccol * u.Ho * u.Wo;
    return hipSuccess;
}

hipError_t launch_col2im(int dtype, const void* col, void* im,
                         int64_t batch, int64_t channels, int64_t height, int64_t width,
                         int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c,
                         int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c, int accumulate, hipStream_t s) {
    UnfoldParams u;
    hipError_t e = fill_params(u, batch, channels, height, width, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c);
    if (e != hipSuccess) return e;
    const int64_t total = batch * channels * height * width;
    if (total == 0) return hipSuccess;
    int64_t blocks = (total + 255) / 256;
    if (blocks > 256 * 64) blocks = 256 * 64;
    const dim3 g((unsigned)blocks), b(256);
    switch (dtype) {
    case DT_F32: hipLaunchKernelGGL((col2im_kernel<float, float>), g, b, 0, s, (const float*)col, (float*)im, u, accumulate); break;
    case DT_F64: hipLaunchKernelGGL((col2im_kernel<double, double>), g, b, 0, s, (const double*)col, (double*)im, u, accumulate); break;
    case DT_F16: hipLaunchKernelGGL((col2im_kernel<_Float16, float>), g, b, 0, s, (const _Float16*)col, (_Float16*)im, u, accumulate); break;
    case DT_BF16: hipLaunchKernelGGL((col2im_kernel<__bf16, float>), g, b, 0, s, (const __bf16*)col, (__bf16*)im, u, accumulate); break;
    case DT_I8: case DT_U8: hipLaunchKernelGGL((col2im_kernel<uint8_t, uint8_t>), g, b, 0, s, (const uint8_t*)col, (uint8_t*)im, u, accumulate); break;
    case DT_I16: case DT_U16: hipLaunchKernelGGL((col2im_kernel<uint16_t, uint16_t>), g, b, 0, s, (const uint16_t*)col, (uint16_t*)im, u, accumulate); break;
    case DT_I32: case DT_U32: hipLaunchKernelGGL((col2im_kernel<uint32_t, uint32_t>), g, b, 0, s, (const uint32_t*)col, (uint32_t*)im, u, accumulate); break;
    case DT_I64: case DT_U64: hipLaunchKernelGGL((col2im_kernel<uint64_t, uint64_t>), g, b, 0, s, (const uint64_t*)col, (uint64_t*)im, u, accumulate); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_unfold2d(int64_t es, const void* im, void* col,
                           int64_t batch, int64_t channels, int64_t height, int64_t width,
                           int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c,
                           int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c, hipStream_t s) {
    UnfoldParams u;
    u.batch = batch; u.channels = channels; u.height = height; u.width = width;
    u.k_r = k_r; u.k_c = k_c; u.s_r = s_r; u.s_c = s_c; u.p_r = p_r; u.p_c = p_c; u.d_r = d_r; u.d_c = d_c;
    u.Ho = (height + 2 * p_r - d_r * (k_r - 1) - 1) / s_r + 1;
    u.Wo = (width + 2 * p_c - d_c * (k_c - 1) - 1) / s_c + 1;
    if (u.Ho <= 0 || u.Wo <= 0) return hipErrorInvalidValue;
    u.ccol = channels * k_r * k_c;
    u.total = batch * u.ccol * u.Ho * u.Wo;
    if (u.total == 0) return hipSuccess;
    {
        // 16-byte stores when every row of col is a whole number of vectors and all sizes fit 32-bit arithmetic
        const int64_t L = u.Ho * u.Wo, V = 16 / es, rows = batch * u.ccol;
        const int64_t lim = 1 << 24;
        if (L % V == 0 && (reinterpret_cast<uintptr_t>(col) & 15) == 0 && L < 0x7fffffffLL && rows < 0x7fffffffLL &&
            height < lim && width < lim && k_r * d_r < lim && k_c * d_c < lim && u.Ho * s_r < lim && u.Wo * s_c < lim && p_r < lim && p_c < lim &&
            p_r > -lim && p_c > -lim && u.ccol < 0x7fffffffLL) {
            UnfoldVecParams q;
            q.channels = (int)channels; q.height = (int)height; q.width = (int)width; q.k_c = (int)k_c;
            q.s_r = (int)s_r; q.s_c = (int)s_c; q.p_r = (int)p_r; q.p_c = (int)p_c; q.d_r = (int)d_r; q.d_c = (int)d_c;
            q.Wo = (int)u.Wo; q.ccol = (int)u.ccol; q.k_rc = (int)(k_r * k_c); q.L = L;
            q.vec_per_row = (int)(L / V);
            q.blocks_per_row = (q.vec_per_row + 255) / 256;
            const int64_t nblocks = rows * q.blocks_per_row;
            if (nblocks <= 0x7fffffffLL) {
                q.div_bpr = make_fastdiv((uint32_t)q.blocks_per_row); q.div_ccol = make_fastdiv((uint32_t)q.ccol);
                q.div_krc = make_fastdiv((uint32_t)q.k_rc); q.div_kc = make_fastdiv((uint32_t)q.k_c); q.div_wo = make_fastdiv((uint32_t)q.Wo);
                const dim3 g((unsigned)nblocks), t(256);
                switch (es) {
                case 1: hipLaunchKernelGGL(unfold2d_vec_kernel<uint8_t>, g, t, 0, s, (const uint8_t*)im, (uint8_t*)col, q); break;
                case 2: hipLaunchKernelGGL(unfold2d_vec_kernel<uint16_t>, g, t, 0, s, (const uint16_t*)im, (uint16_t*)col, q); break;
                case 4: hipLaunchKernelGGL(unfold2d_vec_kernel<uint32_t>, g, t, 0, s, (const uint32_t*)im, (uint32_t*)col, q); break;
                case 8: hipLaunchKernelGGL(unfold2d_vec_kernel<uint64_t>, g, t, 0, s, (const uint64_t*)im, (uint64_t*)col, q); break;
                default: return hipErrorInvalidValue;
                }
                return hipGetLastError();
            }
        }
    }
    int64_t blocks = (u.total + 255) / 256;
    if (blocks > 256 * 64) blocks = 256 * 64;   // grid-stride beyond 64 workgroups per CU
    switch (es) {
    case 1: hipLaunchKernelGGL(unfold2d_kernel<uint8_t>, dim3((unsigned)blocks), dim3(256), 0, s, (const uint8_t*)im, (uint8_t*)col, u); break;
    case 2: hipLaunchKernelGGL(unfold2d_kernel<uint16_t>, dim3((unsigned)blocks), dim3(256), 0, s, (const uint16_t*)im, (uint16_t*)col, u); break;
    case 4: hipLaunchKernelGGL(unfold2d_kernel<uint32_t>, dim3((unsigned)blocks), dim3(256), 0, s, (const uint32_t*)im, (uint32_t*)col, u); break;
    case 8: hipLaunchKernelGGL(unfold2d_kernel<uint64_t>, dim3((unsigned)blocks), dim3(256), 0, s, (const uint64_t*)im, (uint64_t*)col, u); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace ntg
