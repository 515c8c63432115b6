// im2col on the GPU: col[b, c*kh*kw + i*kw + j, h*Wo + w] = im[b, c, h*s_r - p_r + i*d_r, w*s_c - p_c + j*d_c]
// (zero where the tap falls in the padding).  Same layout as the reference's im2col_cpu
// (nt/functional/cpu/unfold2d.cpp:12-112) behind functional::unfold2d(..., transpose_out=true)
// (nt/functional/tensor_files/colim_transform.cpp:565-588).  Pure data movement, HBM bound:
// one lane per output element, the fast index runs along Wo so stores are coalesced and,
// for stride 1, so are the loads.
#include "ntg_common.h"

namespace ntg {

// a 16-byte element that is only moved (Complex128)
struct alignas(16) Bytes16 {
    uint64_t lo, hi;
    __host__ __device__ Bytes16() = default;
    __host__ __device__ Bytes16(int) : lo(0), hi(0) {}
};

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

// The same gather in 32-bit arithmetic (every size and the number of image elements below 2^31): the element index is
// split with multiply-shift divisions, a tap row or column is skipped as soon as it falls before the image (the
// position only decreases with the tap index), and "divisible by the stride" is one more multiply-shift.  Taps are
// still visited in ascending (i, j), so the sum has the same order.
struct Col2imFastParams {
    int channels, height, width, k_r, k_c, s_r, s_c, p_r, p_c, d_r, d_c, Ho, Wo;
    uint32_t total;
    int64_t L, ccol;
    FastDiv div_w, div_h, div_c, div_sr, div_sc;
};

template <class T, class Acc>
__global__ void __launch_bounds__(256) col2im_fast_kernel(const T* __restrict__ col, T* __restrict__ im, const Col2imFastParams u, const int accumulate) {
    const uint32_t idx = blockIdx.x * 256u + threadIdx.x;
    if (idx >= u.total) return;
    uint32_t t = fast_div(idx, u.div_w);
    const int x = (int)(idx - t * (uint32_t)u.width);
    uint32_t t2 = fast_div(t, u.div_h);
    const int y = (int)(t - t2 * (uint32_t)u.height);
    const uint32_t b = fast_div(t2, u.div_c), c = t2 - b * (uint32_t)u.channels;
    Acc acc = accumulate ? (Acc)im[idx] : (Acc)0;
    const T* colc = col + ((int64_t)b * u.ccol + (int64_t)c * u.k_r * u.k_c) * u.L;      // row (c, 0, 0) of this image's col
    int hn = y + u.p_r;
    for (int i = 0; i < u.k_r && hn >= 0; ++i, hn -= u.d_r) {
        const uint32_t h = fast_div((uint32_t)hn, u.div_sr);
        if ((int)h * u.s_r != hn || (int)h >= u.Ho) continue;
        const T* rowp = colc + (int64_t)i * u.k_c * u.L + (int64_t)h * u.Wo;
        int wn = x + u.p_c;
        for (int j = 0; j < u.k_c && wn >= 0; ++j, wn -= u.d_c) {
            const uint32_t w = fast_div((uint32_t)wn, u.div_sc);
            if ((int)w * u.s_c != wn || (int)w >= u.Wo) continue;
            acc += (Acc)rowp[(int64_t)j * u.L + w];
        }
    }
    im[idx] = (T)acc;
}

template <class T, class Acc>
static void launch_col2im_fast(const void* col, void* im, const Col2imFastParams& q, int accumulate, hipStream_t s) {
    hipLaunchKernelGGL((col2im_fast_kernel<T, Acc>), dim3((q.total + 255u) / 256u), dim3(256), 0, s, (const T*)col, (T*)im, q, accumulate);
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
    case 16: hipLaunchKernelGGL(unfoldnd_kernel<Bytes16>, g, b, 0, s, (const Bytes16*)im, (Bytes16*)col, u); break;
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
    // complex: the two lanes of an element are added separately in the lane's type, taps in the same ascending order
    case DT_C32: hipLaunchKernelGGL((col2imnd_kernel<LanePair<_Float16>, LanePair<_Float16>>), g, b, 0, s, (const LanePair<_Float16>*)col, (LanePair<_Float16>*)im, u, accumulate); break;
    case DT_C64: hipLaunchKernelGGL((col2imnd_kernel<LanePair<float>, LanePair<float>>), g, b, 0, s, (const LanePair<float>*)col, (LanePair<float>*)im, u, accumulate); break;
    case DT_C128: hipLaunchKernelGGL((col2imnd_kernel<LanePair<double>, LanePair<double>>), g, b, 0, s, (const LanePair<double>*)col, (LanePair<double>*)im, u, accumulate); break;
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
    const int64_t lim = 1LL << 30;
    if (total < 0x7fffffffLL && u.k_r * u.d_r < lim && u.k_c * u.d_c < lim && u.p_r < lim && u.p_c < lim && u.p_r > -lim && u.p_c > -lim &&
        u.Ho * u.s_r < lim && u.Wo * u.s_c < lim && height < lim && width < lim && u.k_r < lim && u.k_c < lim && u.p_r >= 0 && u.p_c >= 0) {
        Col2imFastParams q;
        q.channels = (int)channels; q.height = (int)height; q.width = (int)width; q.k_r = (int)u.k_r; q.k_c = (int)u.k_c;
        q.s_r = (int)u.s_r; q.s_c = (int)u.s_c; q.p_r = (int)u.p_r; q.p_c = (int)u.p_c; q.d_r = (int)u.d_r; q.d_c = (int)u.d_c;
        q.Ho = (int)u.Ho; q.Wo = (int)u.Wo; q.total = (uint32_t)total; q.L = u.Ho * u.Wo; q.ccol = u.ccol;
        q.div_w = make_fastdiv((uint32_t)width); q.div_h = make_fastdiv((uint32_t)height); q.div_c = make_fastdiv((uint32_t)channels);
        q.div_sr = make_fastdiv((uint32_t)u.s_r); q.div_sc = make_fastdiv((uint32_t)u.s_c);
        switch (dtype) {
        case DT_F32: launch_col2im_fast<float, float>(col, im, q, accumulate, s); break;
        case DT_F64: launch_col2im_fast<double, double>(col, im, q, accumulate, s); break;
        case DT_F16: launch_col2im_fast<_Float16, float>(col, im, q, accumulate, s); break;
        case DT_BF16: launch_col2im_fast<__bf16, float>(col, im, q, accumulate, s); break;
        case DT_I8: case DT_U8: launch_col2im_fast<uint8_t, uint8_t>(col, im, q, accumulate, s); break;
        case DT_I16: case DT_U16: launch_col2im_fast<uint16_t, uint16_t>(col, im, q, accumulate, s); break;
        case DT_I32: case DT_U32: launch_col2im_fast<uint32_t, uint32_t>(col, im, q, accumulate, s); break;
        case DT_I64: case DT_U64: launch_col2im_fast<uint64_t, uint64_t>(col, im, q, accumulate, s); break;
        case DT_C32: launch_col2im_fast<LanePair<_Float16>, LanePair<_Float16>>(col, im, q, accumulate, s); break;
        case DT_C64: launch_col2im_fast<LanePair<float>, LanePair<float>>(col, im, q, accumulate, s); break;
        case DT_C128: launch_col2im_fast<LanePair<double>, LanePair<double>>(col, im, q, accumulate, s); break;
        default: return hipErrorInvalidValue;
        }
        return hipGetLastError();
    }
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
    case DT_C32: hipLaunchKernelGGL((col2im_kernel<LanePair<_Float16>, LanePair<_Float16>>), g, b, 0, s, (const LanePair<_Float16>*)col, (LanePair<_Float16>*)im, u, accumulate); break;
    case DT_C64: hipLaunchKernelGGL((col2im_kernel<LanePair<float>, LanePair<float>>), g, b, 0, s, (const LanePair<float>*)col, (LanePair<float>*)im, u, accumulate); break;
    case DT_C128: hipLaunchKernelGGL((col2im_kernel<LanePair<double>, LanePair<double>>), g, b, 0, s, (const LanePair<double>*)col, (LanePair<double>*)im, u, accumulate); break;
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
        if (es < 16 && L % V == 0 && (reinterpret_cast<uintptr_t>(col) & 15) == 0 && L < 0x7fffffffLL && rows < 0x7fffffffLL &&
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
    case 16: hipLaunchKernelGGL(unfold2d_kernel<Bytes16>, dim3((unsigned)blocks), dim3(256), 0, s, (const Bytes16*)im, (Bytes16*)col, u); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace ntg
