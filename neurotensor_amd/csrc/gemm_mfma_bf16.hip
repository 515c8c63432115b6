// BFloat16 instantiations of the MFMA GEMM (v_mfma_f32_32x32x16_bf16, fp32 accumulate).
#include "gemm_ring_impl.h"
namespace ntg {
hipError_t launch_gemm_mfma_bf16(bool ta, bool tb, const GemmParams& p, hipStream_t s) {
    if ((p.tailA || p.tailB) && !ring_eligible(p, ta)) return hipErrorInvalidValue;       // (only the DMA-fed kernel reads copied tail rows)
    if (ring_eligible(p, ta)) return launch_ring16<DT_BF16>(ta, tb, p, s);   // DMA-fed LDS ring; the tile (256 x 256 .. 64 x 64, 192 x 256, 128 x 256) follows ring16_tile_edge
    const int64_t big_tiles = (int64_t)((p.M + 255) / 256) * ((p.N + 255) / 256) * p.batch;
    if (big_tiles >= 256) return launch_trans<DT_BF16, 4, 4, 64>(ta, tb, p, s);   // 256 x 256 x 64
    return launch_trans<DT_BF16, 2, 2, 64>(ta, tb, p, s);                          // 128 x 128 x 64
}
hipError_t launch_gemm_ring_only_bf16(bool ta, bool tb, const GemmParams& p, hipStream_t s, bool* taken) {
    *taken = ring_eligible(p, ta);
    return *taken ? launch_ring16<DT_BF16>(ta, tb, p, s) : hipSuccess;
}
// convolution / conv_dkernel with op(B) gathered from the image (tb: col^T), nd = 2 or 3 spatial axes.  128 x 128 x 64 tiles,
// two workgroups per CU: the gather's registers do not fit beside a 256 x 256 accumulator.
hipError_t launch_conv_mfma_bf16(bool tb, int nd, const GemmParams& p, hipStream_t s) {
    if (nd == 3) return tb ? launch_conv_cfg<DT_BF16, true, 3, 2, 2, 64>(p, s) : launch_conv_cfg<DT_BF16, false, 3, 2, 2, 64>(p, s);
    return tb ? launch_conv_cfg<DT_BF16, true, 2, 2, 2, 64>(p, s) : launch_conv_cfg<DT_BF16, false, 2, 2, 2, 64>(p, s);
}
hipError_t launch_conv_nhwc_bf16(const GemmParams& p, hipStream_t s) {
    return launch_conv_nhwc16_planned(p, s, [&](int te, const GemmParams& q) {
        if (te == 256) return launch_ring_nhwc_cfg<DT_BF16, 4>(q, s);
        if (te == 64) return launch_ring_nhwc_cfg<DT_BF16, 1>(q, s);
        return launch_ring_nhwc_cfg<DT_BF16, 2>(q, s);
    });
}
hipError_t launch_conv_nhwc_dw_bf16(bool ta, const GemmParams& p, hipStream_t s) {
    return launch_conv_nhwc16_planned(p, s, [&](int te, const GemmParams& q) {
        if (ta) {
            if (te == 256) return launch_ring_nhwc_dw_cfg<DT_BF16, 4, true>(q, s);
            if (te == 64) return launch_ring_nhwc_dw_cfg<DT_BF16, 1, true>(q, s);
            return launch_ring_nhwc_dw_cfg<DT_BF16, 2, true>(q, s);
        }
        if (te == 256) return launch_ring_nhwc_dw_cfg<DT_BF16, 4>(q, s);
        if (te == 64) return launch_ring_nhwc_dw_cfg<DT_BF16, 1>(q, s);
        return launch_ring_nhwc_dw_cfg<DT_BF16, 2>(q, s);
    });
}
}  // namespace ntg
