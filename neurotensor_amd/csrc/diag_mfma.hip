// Measurement aid (no counterpart in the reference): the matrix instruction of the 16-bit product kernels on operands that
// stay in registers.  What it measures is the rate the matrix pipes sustain on given operand VALUES before any data
// movement: the power manager lowers the clock as operand bits toggle, so random operands and all-zero operands give
// different rates for the same instruction stream.  The figure bounds what a product kernel can reach on such data.
//
// One workgroup = 4 wavefronts (one per SIMD), each with the 4 x 4 accumulator blocks of the 256 x 256 tile kernel
// (256 accumulator registers).  Four fragment sets (4 A + 4 B fragments of 16 bytes each) are loaded once from
// `operands`; a pass multiplies the 16 block pairs of every set in the product kernel's serpentine order, so
// consecutive instructions see different operand registers, as they do there.
#include "../../include/ntgemm.h"
#include "gemm_mfma_impl.h"

namespace ntg {
namespace {

constexpr int DIAG_SETS = 4;

template <int DT>
__global__ void __launch_bounds__(256) diag_mfma_kernel(const u32x4* __restrict__ operands, const int64_t iters, float* __restrict__ sink) {
    using E = Elem<DT>;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    u32x4 af[DIAG_SETS][4], bf[DIAG_SETS][4];
#pragma unroll
    for (int s = 0; s < DIAG_SETS; ++s)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            af[s][i] = operands[((wave * DIAG_SETS + s) * 8 + i) * 64 + lane];
            bf[s][i] = operands[((wave * DIAG_SETS + s) * 8 + 4 + i) * 64 + lane];
        }
    typename E::AccV acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
    for (int64_t it = 0; it < iters; ++it) {
#pragma unroll
        for (int s = 0; s < DIAG_SETS; ++s)
#pragma unroll
            for (int q = 0; q < 16; ++q) {
                const int i = q / 4, j = (i & 1) ? 3 - (q % 4) : (q % 4);
                E::mma(acc[i][j], bf[s][j], af[s][i]);
            }
    }
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) sum += acc[i][j][r];
    sink[(int64_t)blockIdx.x * 256 + threadIdx.x] = sum;
}

}  // namespace
}  // namespace ntg

extern "C" int ntg_diag_mfma_rate_dev(int dtype, const void* operands, int64_t iters, int64_t workgroups, float* sink, void* stream) {
    if (!operands || !sink || iters < 0 || workgroups < 1 || workgroups > (1 << 20)) return NTG_ERR_INVALID_ARGUMENT;
    if ((reinterpret_cast<uintptr_t>(operands) & 15) != 0) return NTG_ERR_INVALID_ARGUMENT;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 g((unsigned)workgroups), t(256);
    if (dtype == ntg::DT_BF16)
        hipLaunchKernelGGL(ntg::diag_mfma_kernel<ntg::DT_BF16>, g, t, 0, s, static_cast<const ntg::u32x4*>(operands), iters, sink);
    else if (dtype == ntg::DT_F16)
        hipLaunchKernelGGL(ntg::diag_mfma_kernel<ntg::DT_F16>, g, t, 0, s, static_cast<const ntg::u32x4*>(operands), iters, sink);
    else
        return NTG_ERR_UNSUPPORTED_DTYPE;
    return hipGetLastError() == hipSuccess ? NTG_OK : NTG_ERR_DEVICE;
}
