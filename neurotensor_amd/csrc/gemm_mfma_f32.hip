// Float32 instantiations of the MFMA GEMM (v_mfma_f32_32x32x2_f32).
#include "gemm_mfma_impl.h"
namespace ntg {
hipError_t launch_gemm_mfma_f32(bool ta, bool tb, const GemmParams& p, hipStream_t s) {
    return launch_trans<DT_F32, 2, 2, 32>(ta, tb, p, s);   // 128 x 128 x 32 tile
}
}  // namespace ntg
