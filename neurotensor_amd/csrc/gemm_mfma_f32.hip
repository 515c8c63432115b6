// Float32 instantiations of the MFMA GEMM (v_mfma_f32_32x32x2_f32).
#include "gemm_mfma_impl.h"
namespace ntg {
hipError_t launch_gemm_mfma_f32(bool ta, bool tb, const GemmParams& p, hipStream_t s) {
    // 128 x 128 x 32 tiles unless that leaves most of the 256 CUs idle; then 64 x 64 x 32
    const int64_t big_tiles = (int64_t)((p.M + 127) / 128) * ((p.N + 127) / 128) * p.batch;
    if (big_tiles >= 192 && p.M > 64 && p.N > 64) return launch_trans<DT_F32, 2, 2, 32>(ta, tb, p, s);   // a 128-wide tile would be half empty
    return launch_trans<DT_F32, 1, 1, 32>(ta, tb, p, s);
}
// convolution / conv_dkernel with op(B) gathered from the image (tb: col^T), nd = 2 or 3 spatial axes
template <int ND>
static hipError_t launch_conv_nd_f32(bool tb, const GemmParams& p, hipStream_t s) {
    const int64_t big_tiles = (int64_t)((p.M + 127) / 128) * ((p.N + 127) / 128) * p.batch;
    if (big_tiles >= 192 && p.M > 64 && p.N > 64)
        return tb ? launch_conv_cfg<DT_F32, true, ND, 2, 2, 32>(p, s) : launch_conv_cfg<DT_F32, false, ND, 2, 2, 32>(p, s);
    return tb ? launch_conv_cfg<DT_F32, true, ND, 1, 1, 32>(p, s) : launch_conv_cfg<DT_F32, false, ND, 1, 1, 32>(p, s);
}
hipError_t launch_conv_mfma_f32(bool tb, int nd, const GemmParams& p, hipStream_t s) {
    return nd == 3 ? launch_conv_nd_f32<3>(tb, p, s) : launch_conv_nd_f32<2>(tb, p, s);
}
}  // namespace ntg
