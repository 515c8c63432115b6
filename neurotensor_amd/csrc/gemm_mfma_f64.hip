// Float64 instantiations of the MFMA GEMM (v_mfma_f64_16x16x4_f64).
#include "gemm_mfma_impl.h"
namespace ntg {
hipError_t launch_gemm_mfma_f64(bool ta, bool tb, const GemmParams& p, hipStream_t s) {
    const int64_t big_tiles = (int64_t)((p.M + 127) / 128) * ((p.N + 127) / 128) * p.batch;
    if (big_tiles >= 192) return launch_trans<DT_F64, 4, 4, 16>(ta, tb, p, s);   // 128 x 128 x 16 tile
    return launch_trans<DT_F64, 2, 2, 16>(ta, tb, p, s);                          // 64 x 64 x 16 tile
}
}  // namespace ntg
