// Copies that bring operands with rows that are not 16-byte multiples onto the DMA-fed kernels: the matrix is copied into
// a workspace with its rows padded to whole 16-byte chunks (zeros in the padding, which add nothing to any sum), the
// product runs on the copies, and a result whose own rows are not 16-byte multiples is copied back.  HBM bound; one lane
// per 16 bytes of the padded side.
#include "ntg_common.h"

namespace ntg {

typedef uint32_t padx4 __attribute__((ext_vector_type(4)));

// dst[b][r][0 .. ld_dst) = src[b][r][0 .. cols) followed by zeros, for r < rows; rows r in [rows, rows_dst) are zeros.
// dst rows are 16-byte aligned (ld_dst a multiple of V = 16 / sizeof(T) elements); src has any pitch and alignment.
template <class T>
__global__ void __launch_bounds__(256) pad_copy_kernel(const T* __restrict__ src, const int64_t ld_src, const int64_t s_src,
                                                       T* __restrict__ dst, const int64_t ld_dst, const int64_t s_dst,
                                                       const int64_t rows, const int64_t cols, const int64_t rows_dst, const int64_t batch) {
    constexpr int V = 16 / (int)sizeof(T);
    const int64_t vpr = ld_dst / V, total = batch * rows_dst * vpr;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int64_t v = i % vpr, r = (i / vpr) % rows_dst, b = i / (vpr * rows_dst);
        T tmp[V];
        const T* s = src + b * s_src + r * ld_src + v * V;
#pragma unroll
        for (int e = 0; e < V; ++e) tmp[e] = (r < rows && v * V + e < cols) ? s[e] : (T)0;
        padx4 w;
        __builtin_memcpy(&w, tmp, 16);
        *reinterpret_cast<padx4*>(dst + b * s_dst + r * ld_dst + v * V) = w;
    }
}

// dst[b][r][0 .. cols) = src[b][r][0 .. cols): src rows are 16-byte aligned with pitch ld_src, dst has any pitch and alignment
template <class T>
__global__ void __launch_bounds__(256) unpad_copy_kernel(const T* __restrict__ src, const int64_t ld_src, const int64_t s_src,
                                                         T* __restrict__ dst, const int64_t ld_dst, const int64_t s_dst,
                                                         const int64_t rows, const int64_t cols, const int64_t batch) {
    constexpr int V = 16 / (int)sizeof(T);
    const int64_t vpr = (cols + V - 1) / V, total = batch * rows * vpr;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int64_t v = i % vpr, r = (i / vpr) % rows, b = i / (vpr * rows);
        const padx4 w = *reinterpret_cast<const padx4*>(src + b * s_src + r * ld_src + v * V);
        T tmp[V];
        __builtin_memcpy(tmp, &w, 16);
        T* d = dst + b * s_dst + r * ld_dst + v * V;
#pragma unroll
        for (int e = 0; e < V; ++e)
            if (v * V + e < cols) d[e] = tmp[e];
    }
}

// dst[b][m][n] = bias[b * bs + m * rs + n * cs] for m < rows, n < cols, zeros in the padding (rows_dst x ld_dst per item):
// the initial accumulator of cpu::linear (matmult_cpu.cpp:1637-1647) laid out with padded rows
template <class T>
__global__ void __launch_bounds__(256) bias_fill_kernel(const T* __restrict__ bias, const int64_t bs, const int64_t rs, const int64_t cs,
                                                        T* __restrict__ dst, const int64_t ld_dst, const int64_t s_dst,
                                                        const int64_t rows, const int64_t cols, const int64_t rows_dst, const int64_t batch) {
    const int64_t total = batch * rows_dst * ld_dst;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int64_t n = i % ld_dst, m = (i / ld_dst) % rows_dst, b = i / (ld_dst * rows_dst);
        dst[b * s_dst + m * ld_dst + n] = (m < rows && n < cols) ? bias[b * bs + m * rs + n * cs] : (T)0;
    }
}

hipError_t launch_pad_copy(int64_t es, const void* src, int64_t ld_src, int64_t s_src, void* dst, int64_t ld_dst, int64_t s_dst,
                           int64_t rows, int64_t cols, int64_t rows_dst, int64_t batch, hipStream_t s) {
    const int64_t total = batch * rows_dst * (ld_dst * es / 16);
    if (total <= 0) return hipSuccess;
    const dim3 g(grid_for(total)), t(256);
    if (es == 1) hipLaunchKernelGGL(pad_copy_kernel<uint8_t>, g, t, 0, s, (const uint8_t*)src, ld_src, s_src, (uint8_t*)dst, ld_dst, s_dst, rows, cols, rows_dst, batch);
    else if (es == 2) hipLaunchKernelGGL(pad_copy_kernel<uint16_t>, g, t, 0, s, (const uint16_t*)src, ld_src, s_src, (uint16_t*)dst, ld_dst, s_dst, rows, cols, rows_dst, batch);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}

hipError_t launch_unpad_copy(int64_t es, const void* src, int64_t ld_src, int64_t s_src, void* dst, int64_t ld_dst, int64_t s_dst,
                             int64_t rows, int64_t cols, int64_t batch, hipStream_t s) {
    const int64_t total = batch * rows * ((cols * es + 15) / 16);
    if (total <= 0) return hipSuccess;
    const dim3 g(grid_for(total)), t(256);
    if (es == 1) hipLaunchKernelGGL(unpad_copy_kernel<uint8_t>, g, t, 0, s, (const uint8_t*)src, ld_src, s_src, (uint8_t*)dst, ld_dst, s_dst, rows, cols, batch);
    else if (es == 2) hipLaunchKernelGGL(unpad_copy_kernel<uint16_t>, g, t, 0, s, (const uint16_t*)src, ld_src, s_src, (uint16_t*)dst, ld_dst, s_dst, rows, cols, batch);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}

hipError_t launch_bias_fill(int64_t es, const void* bias, int64_t bs, int64_t rs, int64_t cs, void* dst, int64_t ld_dst, int64_t s_dst,
                            int64_t rows, int64_t cols, int64_t rows_dst, int64_t batch, hipStream_t s) {
    const int64_t total = batch * rows_dst * ld_dst;
    if (total <= 0) return hipSuccess;
    const dim3 g(grid_for(total)), t(256);
    if (es == 1) hipLaunchKernelGGL(bias_fill_kernel<uint8_t>, g, t, 0, s, (const uint8_t*)bias, bs, rs, cs, (uint8_t*)dst, ld_dst, s_dst, rows, cols, rows_dst, batch);
    else if (es == 2) hipLaunchKernelGGL(bias_fill_kernel<uint16_t>, g, t, 0, s, (const uint16_t*)bias, bs, rs, cs, (uint16_t*)dst, ld_dst, s_dst, rows, cols, rows_dst, batch);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}

}  // namespace ntg
