// Float64 instantiations of the MFMA GEMM (v_mfma_f64_16x16x4_f64).
#include "gemm_mfma_impl.h"
namespace ntg {
hipError_t launch_gemm_mfma_f64(bool ta, bool tb, const GemmParams& p, hipStream_t s) {
    const int64_t big_tiles = (int64_t)((p.M + 127) / 128) * ((p.N + 127) / 128) * p.batch;
    if (big_tiles >= 192 && p.M > 64 && p.N > 64) return launch_trans<DT_F64, 4, 4, 16>(ta, tb, p, s);   // a 128-wide tile would be half empty   // 128 x 128 x 16 tile
    return launch_trans<DT_F64, 2, 2, 16>(ta, tb, p, s);                          // 64 x 64 x 16 tile
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
