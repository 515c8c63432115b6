// Float32 instantiations of the MFMA GEMMs (v_mfma_f32_32x32x2_f32): the DMA-fed LDS ring for 16-byte aligned rows,
// the register-staged kernel for everything else and for the gathering convolutions.
#include "gemm_ring_impl.h"
namespace ntg {
// Tile edge of the DMA-fed kernel for Float32 (64 or 128).  The 32x32x2 MFMA is slow enough that LDS traffic never
// binds, so the tile only decides how evenly the work spreads: a CU's time is the number of tiles it is handed
// times the tile's MFMA time; 64 x 64 tiles balance four times finer and lose about 7 % to their single
// accumulator block per wavefront.
static int ring_f32_tile_edge(const GemmParams& p) {
    const int64_t t128 = (int64_t)((p.M + 127) / 128) * ((p.N + 127) / 128) * p.batch;
    const int64_t t64 = (int64_t)((p.M + 63) / 64) * ((p.N + 63) / 64) * p.batch;
    const double cost128 = (double)((t128 + 255) / 256), cost64 = 1.07 * 0.25 * (double)((t64 + 255) / 256);
    return cost64 < cost128 ? 64 : 128;
}

hipError_t launch_gemm_mfma_f32(bool ta, bool tb, const GemmParams& p, hipStream_t s) {
    if (ring_eligible(p, ta, 4))
        return ring_f32_tile_edge(p) == 64 ? launch_ring_wb<DT_F32, 1>(ta, tb, p, s) : launch_ring_wb<DT_F32, 2>(ta, tb, p, s);
    // rows that are not 16-byte aligned (or pointer tables): register-staged kernel, 128 x 128 x 32 tiles unless that
    // leaves most of the 256 CUs idle; then 64 x 64 x 32
    const int64_t big_tiles = (int64_t)((p.M + 127) / 128) * ((p.N + 127) / 128) * p.batch;
    if (big_tiles >= 192 && p.M > 64 && p.N > 64) return launch_trans<DT_F32, 2, 2, 32>(ta, tb, p, s);   // a 128-wide tile would be half empty
    return launch_trans<DT_F32, 1, 1, 32>(ta, tb, p, s);
}
hipError_t launch_gemm_ring_only_f32(bool ta, bool tb, const GemmParams& p, hipStream_t s, bool* taken) {
    *taken = ring_eligible(p, ta, 4);
    if (!*taken) return hipSuccess;
    return ring_f32_tile_edge(p) == 64 ? launch_ring_wb<DT_F32, 1>(ta, tb, p, s) : launch_ring_wb<DT_F32, 2>(ta, tb, p, s);
}
// convolution / conv_dkernel with op(B) gathered from the image (tb: col^T), nd = 2 or 3 spatial axes
template <int ND>
static hipError_t launch_conv_nd_f32(bool tb, const GemmParams& p, hipStream_t s) {
    const int64_t big_tiles = (int64_t)((p.M + 127) / 128) * ((p.N + 127) / 128) * p.batch;
    if (big_tiles >= 192 && p.M > 64 && p.N > 64)
        return tb ? launch_conv_cfg<DT_F32, true, ND, 2, 2, 32>(p, s) : launch_conv_cfg<DT_F32, false, ND, 2, 2, 32>(p, s);
    return tb ? launch_conv_cfg<DT_F32, true, ND, 1, 1, 32>(p, s) : launch_conv_cfg<DT_F32, false, ND, 1, 1, 32>(p, s);
}
// the DMA-fed kernel gathers the operand itself when A (weights or output gradient) and C have 16-byte rows
static bool ring_conv_eligible(const GemmParams& p) {
    return p.K % 4 == 0 && p.N % 4 == 0 && p.ldc % 4 == 0 && p.sC % 4 == 0 && p.vecA_ok && p.lda % 4 == 0 && p.sA % 4 == 0 &&
           p.lda < (1 << 21) && !p.Aptr && !p.Bptr && !p.Cptr &&
           ((reinterpret_cast<uintptr_t>(p.A) & 15) == 0) && ((reinterpret_cast<uintptr_t>(p.C) & 15) == 0) &&
           ((reinterpret_cast<uintptr_t>(p.B) & 3) == 0);
}
hipError_t launch_conv_mfma_f32(bool tb, int nd, const GemmParams& p, hipStream_t s) {
    // tile edge by the same evenness rule as the plain product (padding of M = O/g and N = Ho*Wo to the tile counts as work)
    if (nd == 2 && ring_conv_eligible(p)) return ring_f32_tile_edge(p) == 128 ? launch_ring_conv_cfg<2>(tb, p, s) : launch_ring_conv_cfg<1>(tb, p, s);
    return nd == 3 ? launch_conv_nd_f32<3>(tb, p, s) : launch_conv_nd_f32<2>(tb, p, s);
}
hipError_t launch_conv_nhwc_f32(const GemmParams& p, hipStream_t s) {
    return ring_f32_tile_edge(p) == 128 ? launch_ring_nhwc_cfg<DT_F32, 2>(p, s) : launch_ring_nhwc_cfg<DT_F32, 1>(p, s);
}
hipError_t launch_conv_nhwc_dw_f32(bool ta, const GemmParams& p, hipStream_t s) {
    const bool big = ring_f32_tile_edge(p) == 128;
    if (ta) return big ? launch_ring_nhwc_dw_cfg<DT_F32, 2, true>(p, s) : launch_ring_nhwc_dw_cfg<DT_F32, 1, true>(p, s);
    return big ? launch_ring_nhwc_dw_cfg<DT_F32, 2>(p, s) : launch_ring_nhwc_dw_cfg<DT_F32, 1>(p, s);
}
}  // namespace ntg
