// Int8 / UInt8 on the matrix pipe: v_mfma_i32_32x32x32_i8 in the DMA-fed LDS ring kernel.  The reference multiplies and
// adds 8-bit integers with wrap-around in the element type (nt/mp/simde_traits/simde_traits_avx2.h:668-670); the low 8 bits
// of the exact products' 32-bit sum are that result for either signedness, so the outputs are bit-identical.  Rows that are
// not 16-byte multiples, and pointer-table batches, stay on the vector-ALU kernel.
#include "gemm_ring_impl.h"
namespace ntg {
hipError_t launch_gemm_mfma_i8(int dtype, bool ta, bool tb, const GemmParams& p, hipStream_t s) {
    if (!ring_eligible(p, ta, 1)) return launch_gemm_valu(dtype, ta, tb, p, s);
    const int te = ring16_tile_edge(p.M, p.N, p.K, p.batch);
    if (te == 256) return launch_ring_wb<DT_I8, 4>(ta, tb, p, s);
    if (te == 64) return launch_ring_wb<DT_I8, 1>(ta, tb, p, s);
    return launch_ring_wb<DT_I8, 2>(ta, tb, p, s);
}
}  // namespace ntg
