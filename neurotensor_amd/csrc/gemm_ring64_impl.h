// DMA-fed MFMA GEMM for gfx950, Float64:  C[M,N] (+)= op(A) . op(B)  with 16-byte aligned rows
// (leading dimensions and contiguous extents multiples of 2 elements).  The Float64 sibling of
// gemm_ring_impl.h: same 4-stage LDS ring filled by global_load_lds_dwordx4, same K-major tile
// layout, but built on v_mfma_f64_16x16x4_f64, whose blocks are 16 x 16 and whose four lane
// groups (lane / 16) each hold one k of a block -- so one 16-byte fragment read covers a whole
// K-step (64 bytes = 8 k per row: lane group g reads k = 2 g, 2 g + 1, element e of every lane
// feeding the e-th of two MFMAs) and a K-step is not split into halves.
//
//   * WB = 2: 128 x 128 tile, 4 wavefronts (2 x 2) of 64 x 64 = 4 x 4 blocks (128 accumulator registers);
//     WB = 1: 64 x 64 tile, 2 x 2 blocks per wavefront.  4 x 16 (8) KiB of LDS: two (four) workgroups per CU.
//   * One barrier per K-step, at its start: it publishes tile kt+1 (whose fragments are prefetched
//     while tile kt is multiplied) and frees the stage of tile kt for the DMA of tile kt+4.
//   * K-major operands: [row][64 B], 16-byte slot kv at kv ^ ((row >> 1) & 3), one ds_read_b128 per
//     block.  MN-major operands: [k][tile edge doubles], one ds_read_b64 per block and k parity; the
//     16 lanes of a group read 128 consecutive bytes.
//   * The MFMA is issued in natural order: a lane holds C[16 i + 4 r + lane/16][16 j + lane%16], so the
//     16 lanes of a group store 128 consecutive bytes of one row; no LDS staging in the epilogue.
#pragma once
#include "gemm_ring_impl.h"

namespace ntg {

typedef double doublex2 __attribute__((ext_vector_type(2)));

template <bool TA, bool TB, bool RAGGED, int WB>
__global__ void __launch_bounds__(256) gemm_ring64_kernel(const GemmParams p) {
    using G = RingGeom<WB, 8>;
    constexpr bool A_KC = !TA, B_KC = TB;
    constexpr int BK = G::BK;                 // 8
    constexpr int NBL = 2 * WB;               // 16 x 16 blocks per wavefront along m and n
    constexpr int WT = 32 * WB;               // wavefront's share of the tile edge
    constexpr int NT = 2 * WB;                // DMA instructions per wavefront and K-step (A + B)

    __shared__ __attribute__((aligned(1024))) char st0[G::STAGE_BYTES];
    __shared__ __attribute__((aligned(1024))) char st1[G::STAGE_BYTES];
    __shared__ __attribute__((aligned(1024))) char st2[G::STAGE_BYTES];
    __shared__ __attribute__((aligned(1024))) char st3[G::STAGE_BYTES];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int lr = lane & 15, lg = lane >> 4;

    if (p.gate && *p.gate != p.gate_want) return;       // (uniform: the other kernel of a gated pair does this product)
    const int lid = xcd_contiguous_id(blockIdx.x, gridDim.x);
    const int tiles = p.tiles_m * p.tiles_n;
    const int b = lid / tiles;
    int tm, tn;
    tile_coords(lid - b * tiles, p.tiles_m, p.tiles_n, 8, tm, tn);
    const int m0 = tm * G::BM, n0 = tn * G::BN;

    const double* A = p.Aptr ? static_cast<const double*>(p.Aptr[b]) : static_cast<const double*>(p.A) + operand_offset(p, b, p.sA, p.sAk);
    const double* B = p.Bptr ? static_cast<const double*>(p.Bptr[b]) : static_cast<const double*>(p.B) + operand_offset(p, b, p.sB, p.sBk);
    NTG_GLOBAL double* C = (NTG_GLOBAL double*)(p.Cptr ? static_cast<double*>(p.Cptr[b]) : static_cast<double*>(p.C) + (int64_t)b * p.sC);   // (global memory: no FLAT instructions)

    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const int KT = (p.K + BK - 1) / BK;
    const int last = KT - 1;
    const int kr = p.K - last * BK;           // k that exist in the last K-step (2, 4, 6 or 8)
    const int mvalid = p.M - m0 < G::BM ? p.M - m0 : G::BM;
    const int nvalid = p.N - n0 < G::BN ? p.N - n0 : G::BN;
    uint32_t offA[WB], offB[WB], offAt[WB], offBt[WB];
    dma_offsets<A_KC, RAGGED, WB, 8>(offA, p.lda, wave, lane, mvalid, BK);
    dma_offsets<B_KC, RAGGED, WB, 8>(offB, p.ldb, wave, lane, nvalid, BK);
    dma_offsets<A_KC, RAGGED, WB, 8>(offAt, p.lda, wave, lane, mvalid, kr);
    dma_offsets<B_KC, RAGGED, WB, 8>(offBt, p.ldb, wave, lane, nvalid, kr);
    const char* baseA = reinterpret_cast<const char*>(A) + (A_KC ? (int64_t)m0 * p.lda : (int64_t)m0) * 8;
    const char* baseB = reinterpret_cast<const char*>(B) + (B_KC ? (int64_t)n0 * p.ldb : (int64_t)n0) * 8;
    const int64_t advA = (A_KC ? (int64_t)BK : (int64_t)BK * p.lda) * 8;
    const int64_t advB = (B_KC ? (int64_t)BK : (int64_t)BK * p.ldb) * 8;
    auto tile_src = [&](const char* base) __attribute__((always_inline)) -> const void* {
        const uint64_t bu = reinterpret_cast<uint64_t>(base);
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)bu);
        const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(bu >> 32));
        return reinterpret_cast<const void*>(((uint64_t)hi << 32) | lo);
    };
    // K-steps past the end re-fetch the last one (into stages nobody reads any more): the loop body stays branch free
    // (guarded instantiation: the last k-rows of an M/N-contiguous operand that is read in place may come from a zero-padded copy)
    auto srcA = [&](int kt) __attribute__((always_inline)) {
        const int kc = kt < last ? kt : last;
        if constexpr (RAGGED && !A_KC) {
            if (p.tailA && kc * BK >= p.tail_k0)                   // (uniform)
                return tile_src(static_cast<const char*>(p.tailA) + ((int64_t)b * p.s_tailA + (int64_t)(kc * BK - p.tail_k0) * p.lda + m0) * 8);
        }
        return tile_src(baseA + (int64_t)kc * advA);
    };
    auto srcB = [&](int kt) __attribute__((always_inline)) {
        const int kc = kt < last ? kt : last;
        if constexpr (RAGGED && !B_KC) {
            if (p.tailB && kc * BK >= p.tail_k0)                   // (uniform)
                return tile_src(static_cast<const char*>(p.tailB) + ((int64_t)b * p.s_tailB + (int64_t)(kc * BK - p.tail_k0) * p.ldb + n0) * 8);
        }
        return tile_src(baseB + (int64_t)kc * advB);
    };

    // fragment read r of an operand: K-major r = block; MN-major r = 2 * block + k parity
    constexpr int NRA = A_KC ? NBL : 2 * NBL, NRB = B_KC ? NBL : 2 * NBL, NR = NRA + NRB;
    auto read_op = [&](doublex2 (&frag)[NBL], const char* tile, bool kc, int wbase, int r) __attribute__((always_inline)) {
        if (kc) {
            const int row = wbase + 16 * r + lr;
            const int slot = lg ^ ((lr >> 1) & 3);               // (row >> 1) & 3: wbase and 16 r are multiples of 8
            frag[r] = *reinterpret_cast<const doublex2*>(tile + row * 64 + slot * 16);
        } else {
            const int blk = r >> 1, e = r & 1;
            const int krow = 2 * lg + e, mnl = wbase + 16 * blk + lr;
            const double v = *reinterpret_cast<const double*>(tile + krow * G::MN_ROW_BYTES + mnl * 8);
            if (e == 0) frag[blk].x = v; else frag[blk].y = v;
        }
    };

    doublex4 acc[NBL][NBL];
#pragma unroll
    for (int i = 0; i < NBL; ++i)
#pragma unroll
        for (int j = 0; j < NBL; ++j) acc[i][j] = doublex4{0.0, 0.0, 0.0, 0.0};

    // prologue: tiles 0..3 in flight (4 NT instructions)
    dma_tile<WB>(srcA(0), 0 >= last ? offAt : offA, lds_addr_of(st0), wave_u);
    dma_tile<WB>(srcB(0), 0 >= last ? offBt : offB, lds_addr_of(st0) + G::TILE_BYTES, wave_u);
    dma_tile<WB>(srcA(1), 1 >= last ? offAt : offA, lds_addr_of(st1), wave_u);
    dma_tile<WB>(srcB(1), 1 >= last ? offBt : offB, lds_addr_of(st1) + G::TILE_BYTES, wave_u);
    dma_tile<WB>(srcA(2), 2 >= last ? offAt : offA, lds_addr_of(st2), wave_u);
    dma_tile<WB>(srcB(2), 2 >= last ? offBt : offB, lds_addr_of(st2) + G::TILE_BYTES, wave_u);
    dma_tile<WB>(srcA(3), 3 >= last ? offAt : offA, lds_addr_of(st3), wave_u);
    dma_tile<WB>(srcB(3), 3 >= last ? offBt : offB, lds_addr_of(st3) + G::TILE_BYTES, wave_u);

    doublex2 af[2][NBL], bf[2][NBL];          // fragment double buffer: [K-step parity][block]

    NTG_WAIT_VMCNT(3 * NT);                   // tile 0 has landed
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int r = 0; r < NRA; ++r) read_op(af[0], st0, A_KC, wm * WT, r);
#pragma unroll
    for (int r = 0; r < NRB; ++r) read_op(bf[0], st0 + G::TILE_BYTES, B_KC, wn * WT, r);

    // RAGGED: a lane's fragment holds k = 2 lg, 2 lg + 1 of the K-step; K is even, so it is entirely real or entirely past the end
    auto mask_tail = [&](int buf) {
        const bool ok = 2 * lg < kr;
#pragma unroll
        for (int i = 0; i < NBL; ++i) {
            af[buf][i].x = ok ? af[buf][i].x : 0.0; af[buf][i].y = ok ? af[buf][i].y : 0.0;
            bf[buf][i].x = ok ? bf[buf][i].x : 0.0; bf[buf][i].y = ok ? bf[buf][i].y : 0.0;
        }
    };

    constexpr int NMMA = NBL * NBL * 2;       // MFMAs per K-step
    // One K-step.  `cur` holds tile kt (its fragments are in registers, buffer `buf`), `nxt` tile kt+1.
    auto iteration = [&](int kt, int buf, char* cur, const char* nxt) __attribute__((always_inline)) {
        // issued after tile kt+1: tiles kt+2, kt+3
        NTG_WAIT_VMCNT(2 * NT);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // my reads of `cur` (issued during the previous K-step) are complete
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (RAGGED && kt == last && kr < BK) mask_tail(buf);
        const void* sa = srcA(kt + 4);
        const void* sb = srcB(kt + 4);
        const bool tail = kt + 4 >= last;
        const uint32_t lds_a = lds_addr_of(cur), lds_b = lds_a + G::TILE_BYTES;
#pragma unroll
        for (int q = 0; q < NMMA; ++q) {
            const int e = q / (NBL * NBL), pr = q % (NBL * NBL);
            const int i = pr / NBL, j = (i & 1) ? NBL - 1 - (pr % NBL) : (pr % NBL);
            const double av = e == 0 ? af[buf][i].x : af[buf][i].y, bv = e == 0 ? bf[buf][j].x : bf[buf][j].y;
            acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(av, bv, acc[i][j], 0, 0, 0);
            if (q < NRA) read_op(af[buf ^ 1], nxt, A_KC, wm * WT, q);
            else if (q < NR) read_op(bf[buf ^ 1], nxt + G::TILE_BYTES, B_KC, wn * WT, q - NRA);
            constexpr int DGAP = NMMA / NT;
            if (q % DGAP == DGAP - 1) {
                const int x = q / DGAP;
                if (x < WB) dma_1k(sa, (RAGGED && tail) ? offAt[x] : offA[x], lds_a + (uint32_t)(wave_u * WB + x) * 1024u);
                else dma_1k(sb, (RAGGED && tail) ? offBt[x - WB] : offB[x - WB], lds_b + (uint32_t)(wave_u * WB + x - WB) * 1024u);
            }
        }
#pragma unroll
        for (int q = 0; q < NMMA; ++q) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);               // one MFMA
            if (q < NR) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // one LDS read
        }
    };

    for (int kt = 0; kt < KT; kt += 4) {
        iteration(kt, 0, st0, st1);
        if (kt + 1 < KT) iteration(kt + 1, 1, st1, st2);
        if (kt + 2 < KT) iteration(kt + 2, 0, st2, st3);
        if (kt + 3 < KT) iteration(kt + 3, 1, st3, st0);
    }
    NTG_WAIT_VMCNT(0);                        // the clamped tail DMAs have landed before the workgroup's LDS is released

    // ---- epilogue: straight from the accumulators; the 16 lanes of a group cover 128 consecutive bytes of a row ----
    const NTG_GLOBAL double* bias = (const NTG_GLOBAL double*)static_cast<const double*>(p.bias);
    const int cmode = p.cmode;
#pragma unroll
    for (int i = 0; i < NBL; ++i)
#pragma unroll
        for (int j = 0; j < NBL; ++j) {
            const int n = n0 + wn * WT + 16 * j + lr;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = m0 + wm * WT + 16 * i + 4 * r + lg;
                if (RAGGED && (m >= p.M || n >= p.N)) continue;
                NTG_GLOBAL double* cp = C + (int64_t)m * p.ldc + n;
                double v = acc[i][j][r];
                if (cmode == C_ACCUMULATE) v += *cp;
                else if (cmode == C_BIAS) v += bias[(int64_t)b * p.bias_bs + (int64_t)m * p.bias_rs + (int64_t)n * p.bias_cs];
                *cp = v;
            }
        }
}

// 16-byte aligned rows everywhere; per-lane DMA offsets are 32-bit (128 rows of lda doubles below 4 GiB)
static inline bool ring64_eligible(const GemmParams& p, bool ta) {
    return p.K >= 2 && p.K % 2 == 0 && p.N % 2 == 0 && (!ta || p.M % 2 == 0) &&
           ((!p.Aptr && !p.Bptr && !p.Cptr) || (p.ptrs_aligned && p.Aptr && p.Bptr && p.Cptr)) && p.vecA_ok && p.vecB_ok && p.lda < (1 << 21) && p.ldb < (1 << 21) &&
           ((reinterpret_cast<uintptr_t>(p.A) & 15) == 0) && ((reinterpret_cast<uintptr_t>(p.B) & 15) == 0) &&
           ((reinterpret_cast<uintptr_t>(p.C) & 7) == 0);
}

template <bool TA, bool TB, int WB>
static hipError_t launch_ring64_cfg(const GemmParams& pin, hipStream_t s) {
    constexpr int TE = RingGeom<WB, 8>::BM;
    GemmParams p = pin;
    p.tiles_m = (p.M + TE - 1) / TE;
    p.tiles_n = (p.N + TE - 1) / TE;
    const int64_t blocks = (int64_t)p.tiles_m * p.tiles_n * p.batch;
    if (blocks <= 0) return hipSuccess;
    if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
    if (p.M % TE == 0 && p.N % TE == 0 && p.K % 8 == 0 && !p.tailA && !p.tailB)      // (copied tail rows: the guarded instantiation reads them)
        hipLaunchKernelGGL((gemm_ring64_kernel<TA, TB, false, WB>), dim3((unsigned)blocks), dim3(256), 0, s, p);
    else
        hipLaunchKernelGGL((gemm_ring64_kernel<TA, TB, true, WB>), dim3((unsigned)blocks), dim3(256), 0, s, p);
    return hipGetLastError();
}

template <int WB>
static hipError_t launch_ring64_wb(bool ta, bool tb, const GemmParams& p, hipStream_t s) {
    if (ta) return tb ? launch_ring64_cfg<true, true, WB>(p, s) : launch_ring64_cfg<true, false, WB>(p, s);
    return tb ? launch_ring64_cfg<false, true, WB>(p, s) : launch_ring64_cfg<false, false, WB>(p, s);
}

}  // namespace ntg
