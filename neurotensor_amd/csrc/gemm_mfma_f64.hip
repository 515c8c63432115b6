// Float64 instantiations of the MFMA GEMM (v_mfma_f64_16x16x4_f64).
#include "gemm_mfma_impl.h"
namespace ntg {
hipError_t launch_gemm_mfma_f64(bool ta, bool tb, const GemmParams& p, hipStream_t s) {
    return launch_trans<DT_F64, 4, 4, 16>(ta, tb, p, s);   // 128 x 128 x 16 tile
}
}  // namespace ntg
