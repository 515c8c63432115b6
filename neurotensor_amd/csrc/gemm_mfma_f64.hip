// Float64 instantiations of the MFMA GEMMs (v_mfma_f64_16x16x4_f64): the DMA-fed LDS ring for 16-byte aligned rows,
// the register-staged kernel for everything else and for the gathering convolutions.
#include "gemm_ring64_impl.h"
namespace ntg {
// Tile edge of the DMA-fed kernel (64 or 128): the kernel is bound by the matrix pipe at either size, so the tile only
// decides how evenly the work spreads over 256 CUs; 64 x 64 tiles balance four times finer and lose a few percent.
static int ring64_tile_edge(const GemmParams& p) {
    const int64_t t128 = (int64_t)((p.M + 127) / 128) * ((p.N + 127) / 128) * p.batch;
    const int64_t t64 = (int64_t)((p.M + 63) / 64) * ((p.N + 63) / 64) * p.batch;
    const double cost128 = (double)((t128 + 255) / 256), cost64 = 1.07 * 0.25 * (double)((t64 + 255) / 256);
    return cost64 < cost128 ? 64 : 128;
}
hipError_t launch_gemm_mfma_f64(bool ta, bool tb, const GemmParams& p, hipStream_t s) {
    if ((p.tailA || p.tailB) && !ring64_eligible(p, ta)) return hipErrorInvalidValue;       // (only the DMA-fed kernel reads copied tail rows)
    if (ring64_eligible(p, ta))
        return ring64_tile_edge(p) == 64 ? launch_ring64_wb<1>(ta, tb, p, s) : launch_ring64_wb<2>(ta, tb, p, s);
    // rows that are not 16-byte aligned (or pointer tables): register-staged kernel
    const int64_t big_tiles = (int64_t)((p.M + 127) / 128) * ((p.N + 127) / 128) * p.batch;
    if (big_tiles >= 192 && p.M > 64 && p.N > 64) return launch_trans<DT_F64, 4, 4, 16>(ta, tb, p, s);   // a 128-wide tile would be half empty   // 128 x 128 x 16 tile
    return launch_trans<DT_F64, 2, 2, 16>(ta, tb, p, s);                          // 64 x 64 x 16 tile
}
// the DMA-fed kernel or nothing (the gated pair of an unvouched pointer-table batch)
hipError_t launch_gemm_ring_only_f64(bool ta, bool tb, const GemmParams& p, hipStream_t s, bool* taken) {
    *taken = ring64_eligible(p, ta) && p.act == ACT_NONE;        // (this kernel's epilogue has no clamp)
    if (!*taken) return hipSuccess;
    return ring64_tile_edge(p) == 64 ? launch_ring64_wb<1>(ta, tb, p, s) : launch_ring64_wb<2>(ta, tb, p, s);
}
// convolution / conv_dkernel with op(B) gathered from the image (tb: col^T), nd = 2 or 3 spatial axes
template <int ND>
static hipError_t launch_conv_nd_f64(bool tb, const GemmParams& p, hipStream_t s) {
    const int64_t big_tiles = (int64_t)((p.M + 127) / 128) * ((p.N + 127) / 128) * p.batch;
    if (big_tiles >= 192 && p.M > 64 && p.N > 64)
        return tb ? launch_conv_cfg<DT_F64, true, ND, 4, 4, 16>(p, s) : launch_conv_cfg<DT_F64, false, ND, 4, 4, 16>(p, s);
    return tb ? launch_conv_cfg<DT_F64, true, ND, 2, 2, 16>(p, s) : launch_conv_cfg<DT_F64, false, ND, 2, 2, 16>(p, s);
}
hipError_t launch_conv_mfma_f64(bool tb, int nd, const GemmParams& p, hipStream_t s) {
    return nd == 3 ? launch_conv_nd_f64<3>(tb, p, s) : launch_conv_nd_f64<2>(tb, p, s);
}
}  // namespace ntg
