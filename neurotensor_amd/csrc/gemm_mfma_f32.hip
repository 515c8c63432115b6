// Float32 instantiations of the MFMA GEMM (v_mfma_f32_32x32x2_f32).
#include "gemm_mfma_impl.h"
namespace ntg {
hipError_t launch_gemm_mfma_f32(bool ta, bool tb, const GemmParams& p, hipStream_t s) {
    // 128 x 128 x 32 tiles unless that leaves most of the 256 CUs idle; then 64 x 64 x 32
    const int64_t big_tiles = (int64_t)((p.M + 127) / 128) * ((p.N + 127) / 128) * p.batch;
    if (big_tiles >= 192) return launch_trans<DT_F32, 2, 2, 32>(ta, tb, p, s);
    return launch_trans<DT_F32, 1, 1, 32>(ta, tb, p, s);
}
}  // namespace ntg
