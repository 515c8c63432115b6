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

// Products with so few output elements that 64 x 64 tiles reach fewer than half of the CUs (config 1, 512^3: 64 tiles, each a
// chain of k / 2 MFMAs of 64 cycles on one wavefront per block): one workgroup per 32 x 32 tile of C, four wavefronts with one
// 16 x 16 block each on v_mfma_f32_16x16x4, whose four lane groups are multiplied in a row -- per output element four fused
// multiply-adds in ascending k, the same chain c = C0; c = fma(a_k, b_k, c) that the 32x32x2 kernels compute (both checked
// against fmaf chains on the host), so the results are bit-identical to theirs and the choice between the kernels is free.
// The chain of a block is k / 4 instructions of 32 cycles: four times shorter, on four times as many workgroups.
// Operands go through LDS in stages of 128 k (four 16-byte loads of A and four of B per thread and stage, the loads of the
// next four stages in flight behind the multiplies): a K-contiguous operand is stored [row][132 floats], an M/N-contiguous
// one [k][48 floats], both free of bank conflicts for the one-dword-per-lane reads of the MFMA operands.
// Needs what the DMA-fed kernel needs (16-byte rows and pointers); C0 / bias start the chain, relu clamps in the epilogue.
template <bool TA, bool TB, bool SHORTK>
__global__ void __launch_bounds__(256) gemm_small16_f32_kernel(const GemmParams p) {
    constexpr int KB = 128, LDK = KB + 4, LDM = 48, NP = KB / 32;       // NP 16-byte pieces of each operand per thread and stage
    constexpr int A_STAGE = TA ? KB * LDM : 32 * LDK, B_STAGE = TB ? 32 * LDK : KB * LDM;
    __shared__ __attribute__((aligned(16))) float sA[2][A_STAGE];
    __shared__ __attribute__((aligned(16))) float sB[2][B_STAGE];
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    if (p.gate && *p.gate != p.gate_want) return;       // (uniform: the other kernel of a gated pair does this product)
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int bi = wave >> 1, bj = wave & 1, li = lane & 15, lg = lane >> 4;
    const int tiles = p.tiles_m * p.tiles_n;
    const int b = (int)blockIdx.x / tiles, t = (int)blockIdx.x - b * tiles;
    const int m0 = (t / p.tiles_n) * 32, n0 = (t % p.tiles_n) * 32;
    // (pointers into global memory, said so: loads through a generic pointer count as LDS operations as well, and every wait
    //  for an operand read from LDS would then wait for the stages in flight too)
    typedef __attribute__((address_space(1))) const float* gcfp;
    typedef __attribute__((address_space(1))) float* gfp;
    const gcfp A = (gcfp)(p.Aptr ? static_cast<const float*>(p.Aptr[b]) : static_cast<const float*>(p.A) + operand_offset(p, b, p.sA, p.sAk));
    const gcfp B = (gcfp)(p.Bptr ? static_cast<const float*>(p.Bptr[b]) : static_cast<const float*>(p.B) + operand_offset(p, b, p.sB, p.sBk));
    const gfp C = (gfp)(p.Cptr ? static_cast<float*>(p.Cptr[b]) : static_cast<float*>(p.C) + (int64_t)b * p.sC);

    // this lane's four results: row m, columns n .. n + 3 (the operands are handed to the MFMA the other way round, so that
    // a lane's four accumulator registers are consecutive columns of one row)
    const int m = m0 + bi * 16 + li, n = n0 + bj * 16 + 4 * lg;
    const bool c_ok = m < p.M && n < p.N;                        // (N is a multiple of 4: the four columns exist together)
    f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
    if (c_ok) {
        if (p.cmode == C_ACCUMULATE) acc = *(__attribute__((address_space(1))) const f32x4*)(C + (int64_t)m * p.ldc + n);
        else if (p.cmode == C_BIAS) {
            const gcfp bias = (gcfp)(static_cast<const float*>(p.bias) + (int64_t)b * p.bias_bs + (int64_t)m * p.bias_rs + (int64_t)n * p.bias_cs);
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[e] = bias[(int64_t)e * p.bias_cs];
        }
    }

    // Piece u of this thread: a K-contiguous operand has 32 pieces (128 k) per row, rows tid / 32 + 8 u; an M/N-contiguous one
    // 8 pieces (32 rows or columns of C) per k-row, k-rows tid / 8 + 32 u.  The sizes along the contiguous axis are multiples
    // of 4, so a piece lies inside the matrix or outside as a whole.  A piece outside is fetched from the last piece inside
    // instead (no branch, so the loads of several stages stay in flight and are waited for one stage at a time): rows of A
    // and columns of B past the edge only reach elements of C that are not stored, and k past the end is never multiplied.
    const int k_last = p.K - 4, m_last = TA ? p.M - 4 : p.M - 1, n_last = TB ? p.N - 1 : p.N - 4;
    auto load_a_piece = [&](int k0, int u, f32x4 (&v)[NP]) __attribute__((always_inline)) {
        if constexpr (TA) {
            int k = k0 + (tid >> 3) + 32 * u, mm = m0 + (tid & 7) * 4;
            k = k < p.K ? k : p.K - 1;
            mm = mm < m_last ? mm : m_last;
            v[u] = *(__attribute__((address_space(1))) const f32x4*)(A + (int64_t)k * p.lda + mm);
        } else {
            int mm = m0 + (tid >> 5) + 8 * u, k = k0 + (tid & 31) * 4;
            mm = mm < m_last ? mm : m_last;
            k = k < k_last ? k : k_last;
            v[u] = *(__attribute__((address_space(1))) const f32x4*)(A + (int64_t)mm * p.lda + k);
        }
    };
    auto load_b_piece = [&](int k0, int u, f32x4 (&v)[NP]) __attribute__((always_inline)) {
        if constexpr (TB) {
            int nn = n0 + (tid >> 5) + 8 * u, k = k0 + (tid & 31) * 4;
            nn = nn < n_last ? nn : n_last;
            k = k < k_last ? k : k_last;
            v[u] = *(__attribute__((address_space(1))) const f32x4*)(B + (int64_t)nn * p.ldb + k);
        } else {
            int k = k0 + (tid >> 3) + 32 * u, nn = n0 + (tid & 7) * 4;
            k = k < p.K ? k : p.K - 1;
            nn = nn < n_last ? nn : n_last;
            v[u] = *(__attribute__((address_space(1))) const f32x4*)(B + (int64_t)k * p.ldb + nn);
        }
    };
    auto load_a = [&](int k0, f32x4 (&v)[NP]) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < NP; ++u) load_a_piece(k0, u, v);
    };
    auto load_b = [&](int k0, f32x4 (&v)[NP]) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < NP; ++u) load_b_piece(k0, u, v);
    };
    // piece u of both operands of one stage, from registers to LDS buffer `buf`
    auto store_piece = [&](int buf, int u, const f32x4 (&va)[NP], const f32x4 (&vb)[NP]) __attribute__((always_inline)) {
        if constexpr (TA) *reinterpret_cast<f32x4*>(&sA[buf][((tid >> 3) + 32 * u) * LDM + (tid & 7) * 4]) = va[u];
        else *reinterpret_cast<f32x4*>(&sA[buf][((tid >> 5) + 8 * u) * LDK + (tid & 31) * 4]) = va[u];
        if constexpr (TB) *reinterpret_cast<f32x4*>(&sB[buf][((tid >> 5) + 8 * u) * LDK + (tid & 31) * 4]) = vb[u];
        else *reinterpret_cast<f32x4*>(&sB[buf][((tid >> 3) + 32 * u) * LDM + (tid & 7) * 4]) = vb[u];
    };
    // DEPTH stages of loads in flight (stage kt + DEPTH is requested before stage kt is multiplied): every workgroup walks
    // through k in step with all the others, so each stage is the first touch of its cache lines and comes at the latency of
    // memory, not of the L2 cache -- with four stages of 128 k a product of k <= 512 asks for everything at once.
    // Control flow is laid out so that the number of loads in flight is the same on every path to each wait (the compiler
    // counts them; where paths with different counts meet it waits for everything): no branch inside a stage, a main loop
    // of whole rounds of DEPTH stages that always request (past the end: the last pieces again), and the last one to DEPTH
    // stages as straight-line code without requests.
    constexpr int DEPTH = 4;
    static_assert(KB / 32 == NP, "one piece of each operand goes to LDS per group of eight instructions");
    const int KT = (p.K + KB - 1) / KB;
    f32x4 va[DEPTH][NP], vb[DEPTH][NP];
    load_a(0, va[0]); load_b(0, vb[0]);
#pragma unroll
    for (int sg = 1; sg < DEPTH; ++sg) {
        // SHORTK (fewer than DEPTH stages): a short k asks for nothing it does not use, at the price of inexact waits
        if (!SHORTK || sg < KT) { load_a(sg * KB, va[sg]); load_b(sg * KB, vb[sg]); }
        else {                          // (never multiplied, but handed to LDS like any stage: defined values)
#pragma unroll
            for (int u = 0; u < NP; ++u) va[sg][u] = vb[sg][u] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        }
    }
#pragma unroll
    for (int u = 0; u < NP; ++u) store_piece(0, u, va[0], vb[0]);
    __syncthreads();
    // Stage kt (in LDS buffer SLOT % 2, its registers free again): request stage kt + DEPTH (REQUEST), multiply, and hand
    // stage kt + 1 (which arrived long ago) to the other LDS buffer a piece at a time between the groups of instructions, so
    // that only the barrier and the first operand reads of the next stage are left outside the chain's shadow.
    auto stage = [&](int kt, auto slot_tag, auto request_tag) __attribute__((always_inline)) {
        constexpr int SLOT = decltype(slot_tag)::value, NEXT = (SLOT + 1) % DEPTH, buf = SLOT & 1;
        constexpr bool REQUEST = decltype(request_tag)::value;
        const float* a_s = sA[buf];
        const float* b_s = sB[buf];
        const int steps = p.K - kt * KB < KB ? (p.K - kt * KB) / 4 : KB / 4;      // (K is a multiple of 4: whole instructions)
        // (groups of eight instructions; the sixteen operand reads of the next group are issued before the instructions of this
        //  one, so that the chain never waits for LDS)
        auto read_group = [&](int q0, float (&av)[8], float (&bv)[8]) __attribute__((always_inline)) {
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int k = 4 * (q0 + u) + lg;
                av[u] = TA ? a_s[k * LDM + bi * 16 + li] : a_s[(bi * 16 + li) * LDK + k];
                bv[u] = TB ? b_s[(bj * 16 + li) * LDK + k] : b_s[k * LDM + bj * 16 + li];
            }
        };
        if (steps == KB / 4) {
            float av[2][8], bv[2][8];
            read_group(0, av[0], bv[0]);
#pragma unroll
            for (int g = 0; g < KB / 32; ++g) {
                // One group: its eight instructions (a dependent chain: 40 cycles each, the issue slots between them free), and
                // in their shadow the operand reads of the next group, one piece of stage kt + 1 on its way to LDS and one piece
                // of each operand of stage kt + DEPTH requested.  Left alone the scheduler puts all of that between two groups
                // (the chain idle meanwhile) and sinks every read to just before its instruction; the recipe below deals the
                // other instructions out behind the MFMAs, and nothing crosses the end of the group.
                if (g + 1 < KB / 32) read_group(8 * (g + 1), av[(g + 1) & 1], bv[(g + 1) & 1]);
                store_piece(buf ^ 1, g, va[NEXT], vb[NEXT]);
                if constexpr (REQUEST) {
                    load_a_piece((kt + DEPTH) * KB, g, va[SLOT]);
                    load_b_piece((kt + DEPTH) * KB, g, vb[SLOT]);
                }
#pragma unroll
                for (int u = 0; u < 8; ++u) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(bv[g & 1][u], av[g & 1][u], acc, 0, 0, 0);
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                // one MFMA
                    __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);                // LDS reads of the next group
                    if (u == 2 || u == 5) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);     // LDS writes of the hand-over
                    __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);                // address arithmetic
                    if (REQUEST && (u == 3 || u == 6)) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);   // the requests
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        } else {
            // (the last stage of a k that is not a multiple of 128: never a stage that requests, kt + DEPTH < KT there)
            for (int q = 0; q < steps; ++q) {
                const int k = 4 * q + lg;
                const float av = TA ? a_s[k * LDM + bi * 16 + li] : a_s[(bi * 16 + li) * LDK + k];
                const float bv = TB ? b_s[(bj * 16 + li) * LDK + k] : b_s[k * LDM + bj * 16 + li];
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(bv, av, acc, 0, 0, 0);
            }
#pragma unroll
            for (int u = 0; u < NP; ++u) store_piece(buf ^ 1, u, va[NEXT], vb[NEXT]);
        }
        __syncthreads();
    };
    using S0 = std::integral_constant<int, 0>; using S1 = std::integral_constant<int, 1>;
    using S2 = std::integral_constant<int, 2>; using S3 = std::integral_constant<int, 3>;
    int kt = 0;
    for (; kt + DEPTH < KT; kt += DEPTH) {
        stage(kt, S0{}, std::true_type{});
        stage(kt + 1, S1{}, std::true_type{});
        stage(kt + 2, S2{}, std::true_type{});
        stage(kt + 3, S3{}, std::true_type{});
    }
    stage(kt, S0{}, std::false_type{});                  // (K >= 64: at least one stage)
    if (kt + 1 < KT) {
        stage(kt + 1, S1{}, std::false_type{});
        if (kt + 2 < KT) {
            stage(kt + 2, S2{}, std::false_type{});
            if (kt + 3 < KT) stage(kt + 3, S3{}, std::false_type{});
        }
    }
    if (c_ok) {
        if (p.act == ACT_RELU) {
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[e] = acc[e] > 0.0f ? acc[e] : 0.0f;
        }
        *(__attribute__((address_space(1))) f32x4*)(C + (int64_t)m * p.ldc + n) = acc;
    }
}

// where the kernel above is ahead of the 64 x 64 tiles: those would reach fewer than half of the CUs, and k is deep enough for
// the shorter chain to matter.  The results do not depend on the choice.
static bool small16_f32_wins(const GemmParams& p) {
    const int64_t t64 = (int64_t)((p.M + 63) / 64) * ((p.N + 63) / 64) * p.batch;
    return t64 <= 128 && p.K >= 64 && p.M > 32 && p.cmode != C_PARTIAL && p.krange_items == 0 && !p.tailA && !p.tailB;
}
static hipError_t launch_small16_f32(bool ta, bool tb, const GemmParams& pin, hipStream_t s) {
    GemmParams p = pin;
    p.tiles_m = (p.M + 31) / 32;
    p.tiles_n = (p.N + 31) / 32;
    const int64_t blocks = (int64_t)p.tiles_m * p.tiles_n * p.batch;
    if (blocks <= 0) return hipSuccess;
    const dim3 g((unsigned)blocks), t(256);
    const bool short_k = p.K <= 3 * 128;                 // fewer stages than the kernel keeps in flight
#define NTG_SMALL16(TA_, TB_) \
    do { if (short_k) hipLaunchKernelGGL((gemm_small16_f32_kernel<TA_, TB_, true>), g, t, 0, s, p); \
         else hipLaunchKernelGGL((gemm_small16_f32_kernel<TA_, TB_, false>), g, t, 0, s, p); } while (0)
    if (ta) { if (tb) NTG_SMALL16(true, true); else NTG_SMALL16(true, false); }
    else { if (tb) NTG_SMALL16(false, true); else NTG_SMALL16(false, false); }
#undef NTG_SMALL16
    return hipGetLastError();
}

hipError_t launch_gemm_mfma_f32(bool ta, bool tb, const GemmParams& p, hipStream_t s) {
    if ((p.tailA || p.tailB) && !ring_eligible(p, ta, 4)) return hipErrorInvalidValue;       // (only the DMA-fed kernel reads copied tail rows)
    if (ring_eligible(p, ta, 4) && small16_f32_wins(p)) return launch_small16_f32(ta, tb, p, s);
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
    if (small16_f32_wins(p)) return launch_small16_f32(ta, tb, p, s);
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
