// Copies that bring operands (1, 2, 4 or 8 bytes per element) with rows that are not 16-byte multiples onto the DMA-fed kernels: the matrix is copied into
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
                                                       const int64_t rows, const int64_t cols, const int64_t rows_dst, const int64_t batch, const int sh) {
    constexpr int V = 16 / (int)sizeof(T);
    // a block covers 256 >> sh consecutive rows (of all items, counted through) x 1 << sh chunks of 16 bytes; blockIdx.y
    // counts the pieces of rows longer than 256 chunks (sh = 8)
    const int64_t vpr = ld_dst / V, v = (int64_t)blockIdx.y * 256 + (threadIdx.x & ((1u << sh) - 1u));
    const int64_t gr = (int64_t)blockIdx.x * (256 >> sh) + (threadIdx.x >> sh);
    if (v >= vpr || gr >= batch * rows_dst) return;
    const int64_t b = batch == 1 ? 0 : gr / rows_dst, r = gr - b * rows_dst;
    const T* s = src + b * s_src + r * ld_src + v * V;
    padx4 w;
    if (r < rows && v * V + V <= cols) {
        // 16 bytes inside the row: one load, whatever the address (global memory takes unaligned vector accesses)
        __builtin_memcpy(&w, s, 16);
    } else {
        T tmp[V];
#pragma unroll
        for (int e = 0; e < V; ++e) tmp[e] = (r < rows && v * V + e < cols) ? s[e] : (T)0;
        __builtin_memcpy(&w, tmp, 16);
    }
    *reinterpret_cast<padx4*>(dst + b * s_dst + r * ld_dst + v * V) = w;
}

// dst[b][r][0 .. cols) = src[b][r][0 .. cols): src rows are 16-byte aligned with pitch ld_src, dst has any pitch and alignment
template <class T>
__global__ void __launch_bounds__(256) unpad_copy_kernel(const T* __restrict__ src, const int64_t ld_src, const int64_t s_src,
                                                         T* __restrict__ dst, const int64_t ld_dst, const int64_t s_dst,
                                                         const int64_t rows, const int64_t cols, const int64_t batch, const int sh) {
    constexpr int V = 16 / (int)sizeof(T);
    const int64_t vpr = (cols + V - 1) / V, v = (int64_t)blockIdx.y * 256 + (threadIdx.x & ((1u << sh) - 1u));
    const int64_t gr = (int64_t)blockIdx.x * (256 >> sh) + (threadIdx.x >> sh);
    if (v >= vpr || gr >= batch * rows) return;
    const int64_t b = batch == 1 ? 0 : gr / rows, r = gr - b * rows;
    const padx4 w = *reinterpret_cast<const padx4*>(src + b * s_src + r * ld_src + v * V);
    T* d = dst + b * s_dst + r * ld_dst + v * V;
    if (v * V + V <= cols) {
        __builtin_memcpy(d, &w, 16);                 // (one store, aligned or not)
    } else {
        T tmp[V];
        __builtin_memcpy(tmp, &w, 16);
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

// log2 of the lanes a block gives to one row: rows of up to 256 chunks share a block with their neighbours
static int row_shift(int64_t vpr) {
    int sh = 0;
    while (sh < 8 && (1 << sh) < vpr) ++sh;
    return sh;
}

hipError_t launch_pad_copy(int64_t es, const void* src, int64_t ld_src, int64_t s_src, void* dst, int64_t ld_dst, int64_t s_dst,
                           int64_t rows, int64_t cols, int64_t rows_dst, int64_t batch, hipStream_t s) {
    const int64_t vpr = ld_dst * es / 16;
    const int sh = row_shift(vpr);
    const int64_t gx = (batch * rows_dst + (256 >> sh) - 1) / (256 >> sh), gy = (vpr + 255) / 256;
    if (gx <= 0 || gy <= 0) return hipSuccess;
    if (gx > 0x7fffffffLL || gy > 65535) return hipErrorInvalidValue;
    const dim3 g((unsigned)gx, (unsigned)gy), t(256);
    if (es == 1) hipLaunchKernelGGL(pad_copy_kernel<uint8_t>, g, t, 0, s, (const uint8_t*)src, ld_src, s_src, (uint8_t*)dst, ld_dst, s_dst, rows, cols, rows_dst, batch, sh);
    else if (es == 2) hipLaunchKernelGGL(pad_copy_kernel<uint16_t>, g, t, 0, s, (const uint16_t*)src, ld_src, s_src, (uint16_t*)dst, ld_dst, s_dst, rows, cols, rows_dst, batch, sh);
    else if (es == 4) hipLaunchKernelGGL(pad_copy_kernel<uint32_t>, g, t, 0, s, (const uint32_t*)src, ld_src, s_src, (uint32_t*)dst, ld_dst, s_dst, rows, cols, rows_dst, batch, sh);
    else if (es == 8) hipLaunchKernelGGL(pad_copy_kernel<uint64_t>, g, t, 0, s, (const uint64_t*)src, ld_src, s_src, (uint64_t*)dst, ld_dst, s_dst, rows, cols, rows_dst, batch, sh);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}

hipError_t launch_unpad_copy(int64_t es, const void* src, int64_t ld_src, int64_t s_src, void* dst, int64_t ld_dst, int64_t s_dst,
                             int64_t rows, int64_t cols, int64_t batch, hipStream_t s) {
    const int64_t vpr = (cols * es + 15) / 16;
    const int sh = row_shift(vpr);
    const int64_t gx = (batch * rows + (256 >> sh) - 1) / (256 >> sh), gy = (vpr + 255) / 256;
    if (gx <= 0 || gy <= 0) return hipSuccess;
    if (gx > 0x7fffffffLL || gy > 65535) return hipErrorInvalidValue;
    const dim3 g((unsigned)gx, (unsigned)gy), t(256);
    if (es == 1) hipLaunchKernelGGL(unpad_copy_kernel<uint8_t>, g, t, 0, s, (const uint8_t*)src, ld_src, s_src, (uint8_t*)dst, ld_dst, s_dst, rows, cols, batch, sh);
    else if (es == 2) hipLaunchKernelGGL(unpad_copy_kernel<uint16_t>, g, t, 0, s, (const uint16_t*)src, ld_src, s_src, (uint16_t*)dst, ld_dst, s_dst, rows, cols, batch, sh);
    else if (es == 4) hipLaunchKernelGGL(unpad_copy_kernel<uint32_t>, g, t, 0, s, (const uint32_t*)src, ld_src, s_src, (uint32_t*)dst, ld_dst, s_dst, rows, cols, batch, sh);
    else if (es == 8) hipLaunchKernelGGL(unpad_copy_kernel<uint64_t>, g, t, 0, s, (const uint64_t*)src, ld_src, s_src, (uint64_t*)dst, ld_dst, s_dst, rows, cols, batch, sh);
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
    else if (es == 4) hipLaunchKernelGGL(bias_fill_kernel<uint32_t>, g, t, 0, s, (const uint32_t*)bias, bs, rs, cs, (uint32_t*)dst, ld_dst, s_dst, rows, cols, rows_dst, batch);
    else if (es == 8) hipLaunchKernelGGL(bias_fill_kernel<uint64_t>, g, t, 0, s, (const uint64_t*)bias, bs, rs, cs, (uint64_t*)dst, ld_dst, s_dst, rows, cols, rows_dst, batch);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}

}  // namespace ntg
