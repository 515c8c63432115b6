// 16-bit (Float16 / BFloat16) MFMA GEMM for gfx950, fast path:
//   C[M,N] (+)= op(A) . op(B),  16-byte aligned rows (leading dimensions and contiguous extents
//   multiples of 8 elements); M, N, K need not be multiples of the tile (the
//   RAGGED instantiation clamps DMA source addresses, zeroes the k tail in registers and
//   guards the stores).  Everything else goes through the general kernel in gemm_mfma_impl.h.
//
// Shape of the kernel
//   * 256 x 256 tile of C per workgroup, 4 wavefronts (2 x 2), each owning 128 x 128 =
//     4 x 4 blocks of v_mfma_f32_32x32x16_{f16,bf16}; 256 accumulator registers per lane.
//     A second instantiation (WB = 2) has 128 x 128 tiles, 64 x 64 per wavefront, half the
//     LDS and two workgroups per CU: problems of up to 128 large tiles run on it, so that
//     mid-sized products still put a workgroup on every CU.  The numbers below are the large
//     tile's; the small one halves the per-operand tile, DMA and read counts.
//   * K advances in steps of 32 through a 4-deep ring of LDS stages (4 x 32 KiB).  Global
//     memory is copied straight into LDS (global_load_lds_dwordx4): no staging registers,
//     three to four K-steps of loads in flight while one is being multiplied.  One barrier
//     per K-step, placed between its two k16 halves; the DMA instructions and the LDS
//     fragment reads are slotted between the MFMAs one at a time, so neither the CU's single
//     address unit nor LDS latency ever holds up the matrix pipe.
//   * LDS layouts are conflict free for the reads the MFMA operands need:
//       operand stored K-contiguous  -> [row][32 k] (64 B rows), 16-byte slot kv stored at
//                                        kv ^ ((row >> 1) & 3); one ds_read_b128 per block;
//       operand stored MN-contiguous -> [k][256 mn] (512 B rows), 16-byte chunk c stored at
//                                        c ^ (2 * (k & 3)); ds_read_b64_tr_b16 turns four k-rows
//                                        into "4 consecutive k per lane", i.e. the transpose
//                                        is done by the LDS read, never in memory.
//     Because the DMA writes 64 consecutive 16-byte slots per instruction, the swizzle is
//     applied by choosing which global chunk each lane fetches.
//   * The MFMA is issued with the operands swapped (B fragment first), so a lane holds four
//     consecutive columns of one row of C; the epilogue stages 32-row slabs through LDS in
//     fp32 and touches C with 16-byte accesses only (C0 is added in fp32 before the single
//     rounding to the 16-bit type).
#pragma once
#include "gemm_mfma_impl.h"

#include <type_traits>

namespace ntg {

typedef short shortx4 __attribute__((ext_vector_type(4)));
typedef float floatx4v __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void* lds_ptr_t;

#define NTG_WAIT_VMCNT(N) __builtin_amdgcn_s_waitcnt(((N) & 0xF) | (7 << 4) | (15 << 8) | (((N) >> 4) << 14))

template <int DT>
struct Cvt16;
template <> struct Cvt16<DT_F16> {
    static __device__ __forceinline__ float up(uint16_t v) { return (float)__builtin_bit_cast(_Float16, v); }
    static __device__ __forceinline__ uint16_t down(float v) { return __builtin_bit_cast(uint16_t, (_Float16)v); }
};
template <> struct Cvt16<DT_BF16> {
    static __device__ __forceinline__ float up(uint16_t v) { return __builtin_bit_cast(float, (uint32_t)v << 16); }
    static __device__ __forceinline__ uint16_t down(float v) { return __builtin_bit_cast(uint16_t, (__bf16)v); }
};

// WB = 32 x 32 blocks per wavefront along each of m and n: 4 -> 256 x 256 tile, 2 -> 128 x 128 tile
template <int WB>
struct G16 {
    static constexpr int BM = 64 * WB, BN = 64 * WB, BK = 32, NST = 4;
    static constexpr int WT = 32 * WB;                   // edge of a wavefront's share of the tile
    static constexpr int TILE_BYTES = BM * BK * 2;       // one operand tile, 16 / 8 KiB
    static constexpr int STAGE_BYTES = 2 * TILE_BYTES;   // 32 / 16 KiB
    static constexpr int MN_ROW_BYTES = BM * 2;          // one k-row of an MN-contiguous operand tile
    static constexpr int CHUNKS = BM / 8;                // 16-byte chunks in such a row
};

// Per-lane BYTE offsets (relative to the tile's first element at K-step 0) of this wavefront's
// WB DMA instructions into one operand tile.  Instruction j = WB*wave + jj fills LDS bytes
// [1024 j, 1024 j + 1024) of the tile:
//   K-contiguous operand: rows 16 j + lane/4, 16-byte slot lane%4 holds kv = slot ^ ((row>>1)&3)
//   MN-contiguous operand (CH = 8 WB chunks per k-row): k-rows (64/CH) j + lane/CH, slot lane%CH
//                          holds chunk = slot ^ (2*(krow&3))
// With RAGGED, mn_valid (1..BM rows/columns of the tile that exist) and k_valid (8..32 k of
// the K-step that exist, a multiple of 8) clamp the SOURCE address into the matrix: lanes
// whose data does not exist fetch a neighbouring chunk instead.  Rows/columns past the edge
// only ever reach accumulators that the epilogue does not store; k past the end is zeroed
// in the fragment registers before it is multiplied.
template <bool KC, bool RAGGED, int WB>
__device__ __forceinline__ void dma_offsets(uint32_t (&off)[WB], int64_t ld, int wave, int lane, int mn_valid, int k_valid) {
    constexpr int CH = G16<WB>::CHUNKS;
#pragma unroll
    for (int jj = 0; jj < WB; ++jj) {
        const int j = wave * WB + jj;
        if constexpr (KC) {
            int row = 16 * j + (lane >> 2);
            int kv = (lane & 3) ^ ((row >> 1) & 3);
            if constexpr (RAGGED) {
                row = row < mn_valid ? row : mn_valid - 1;
                kv = kv < (k_valid >> 3) ? kv : (k_valid >> 3) - 1;
            }
            off[jj] = (uint32_t)(((int64_t)row * ld + kv * 8) * 2);
        } else {
            int krow = (64 / CH) * j + lane / CH;
            int chunk = (lane % CH) ^ (2 * (krow & 3));
            if constexpr (RAGGED) {
                krow = krow < k_valid ? krow : k_valid - 1;
                chunk = chunk < (mn_valid >> 3) ? chunk : (mn_valid >> 3) - 1;
            }
            off[jj] = (uint32_t)(((int64_t)krow * ld + chunk * 8) * 2);
        }
    }
}

// One DMA instruction: 64 lanes x 16 bytes from  base + off  (uniform base, per-lane offset)
// to LDS bytes [lds_addr, lds_addr + 1024).  Written as inline assembly so that the only
// waits on these loads are the explicit s_waitcnt vmcnt(N) of the pipeline: the compiler's
// own tracking of LDS-DMA writes made every read of one of the four stages wait for all
// outstanding loads.  The memory clobber keeps LDS reads from being moved across it.
__device__ __forceinline__ void dma_1k(const void* base, uint32_t off, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :: "s"(lds_addr), "v"(off), "s"(base) : "memory");
}

template <int WB>
__device__ __forceinline__ void dma_tile(const void* sbase, const uint32_t (&off)[WB], uint32_t lds_tile, int wave_u) {
#pragma unroll
    for (int jj = 0; jj < WB; ++jj) dma_1k(sbase, off[jj], lds_tile + (uint32_t)(wave_u * WB + jj) * 1024u);
}

__device__ __forceinline__ uint32_t lds_addr_of(const char* p) {
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)p;
}

template <int DT, bool TA, bool TB, bool RAGGED, int WB>
__global__ void __launch_bounds__(256) gemm16_kernel(const GemmParams p) {
    using E = Elem<DT>;
    using T = typename E::T;
    using G = G16<WB>;
    constexpr bool A_KC = !TA, B_KC = TB;
    constexpr int BK = G::BK;
    constexpr int WT = G::WT;

    __shared__ __attribute__((aligned(1024))) char st0[G::STAGE_BYTES];
    __shared__ __attribute__((aligned(1024))) char st1[G::STAGE_BYTES];
    __shared__ __attribute__((aligned(1024))) char st2[G::STAGE_BYTES];
    __shared__ __attribute__((aligned(1024))) char st3[G::STAGE_BYTES];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    const int lid = xcd_contiguous_id(blockIdx.x, gridDim.x);
    const int tiles = p.tiles_m * p.tiles_n;
    const int b = lid / tiles;
    int tm, tn;
    tile_coords(lid - b * tiles, p.tiles_m, p.tiles_n, 4, tm, tn);
    const int m0 = tm * G::BM, n0 = tn * G::BN;

    const T* A = static_cast<const T*>(p.A) + (int64_t)b * p.sA;
    const T* B = static_cast<const T*>(p.B) + (int64_t)b * p.sB;
    T* C = static_cast<T*>(p.C) + (int64_t)b * p.sC;

    // ---- DMA sources: uniform tile base (advances by adv bytes per K-step) + per-lane offsets ----
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const int KT = (p.K + BK - 1) / BK;
    const int last = KT - 1;
    const int kr = p.K - last * BK;                                  // k that exist in the last K-step (8..32)
    const int mvalid = p.M - m0 < G::BM ? p.M - m0 : G::BM;
    const int nvalid = p.N - n0 < G::BN ? p.N - n0 : G::BN;
    uint32_t offA[WB], offB[WB];      // K-steps before the last
    uint32_t offAt[WB], offBt[WB];    // the last K-step (RAGGED: k clamped to what exists)
    dma_offsets<A_KC, RAGGED, WB>(offA, p.lda, wave, lane, mvalid, BK);
    dma_offsets<B_KC, RAGGED, WB>(offB, p.ldb, wave, lane, nvalid, BK);
    dma_offsets<A_KC, RAGGED, WB>(offAt, p.lda, wave, lane, mvalid, kr);
    dma_offsets<B_KC, RAGGED, WB>(offBt, p.ldb, wave, lane, nvalid, kr);
    const char* baseA = reinterpret_cast<const char*>(A) + (A_KC ? (int64_t)m0 * p.lda : (int64_t)m0) * 2;
    const char* baseB = reinterpret_cast<const char*>(B) + (B_KC ? (int64_t)n0 * p.ldb : (int64_t)n0) * 2;
    const int64_t advA = (A_KC ? (int64_t)BK : (int64_t)BK * p.lda) * 2;
    const int64_t advB = (B_KC ? (int64_t)BK : (int64_t)BK * p.ldb) * 2;
    // uniform (scalar) source pointer of one operand tile
    auto tile_src = [&](const char* base) -> const void* {
        const uint64_t bu = reinterpret_cast<uint64_t>(base);
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)bu);
        const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(bu >> 32));
        return reinterpret_cast<const void*>(((uint64_t)hi << 32) | lo);
    };

    // ---- per-lane LDS read offsets (bytes inside an operand tile), for k16-step ks ----
    // K-major: block b of the wavefront, row = wbase + 32 b + lane%32, slot (2 ks + lane/32) ^ ((row>>1)&3)
    // MN-major: two transposing reads per block; see the header comment
    auto frag_off_km = [&](int wbase, int blk, int ks) -> int {
        const int row = wbase + blk * 32 + (lane & 31);
        const int slot = (2 * ks + (lane >> 5)) ^ ((lane >> 1) & 3);
        return row * 64 + slot * 16;
    };
    auto frag_off_mm = [&](int wbase, int blk, int ks, int half) -> int {
        const int bl = lane >> 4, s = lane & 15, e = s >> 2, q = s & 3;
        const int krow = 16 * ks + 8 * (bl >> 1) + 4 * half + e;
        const int mnl = wbase + blk * 32 + 16 * (bl & 1) + 4 * q;
        const int chunk = (mnl >> 3) ^ (2 * e);
        return krow * G::MN_ROW_BYTES + chunk * 16 + (mnl & 7) * 2;
    };

    // One LDS read instruction of an operand's fragment set for k16-step ks.  A K-major
    // operand takes WB reads (one ds_read_b128 per block), an MN-major one 2 WB (two transposing
    // 8-byte reads per block); read r lands in frag[r / per_block] (half r % per_block).
    auto read_op = [&](u32x4 (&frag)[WB], const char* tile, bool kc, int wbase, int ks, int r) {
        if (kc) {
            frag[r] = *reinterpret_cast<const u32x4*>(tile + frag_off_km(wbase, r, ks));
        } else {
            const int blk = r >> 1, half = r & 1;
            const shortx4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (__attribute__((address_space(3))) shortx4*)(tile + frag_off_mm(wbase, blk, ks, half)));
            typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
            const u32x2 w = __builtin_bit_cast(u32x2, v);
            frag[blk][2 * half] = w[0];
            frag[blk][2 * half + 1] = w[1];
        }
    };
    constexpr int NRA = A_KC ? WB : 2 * WB, NRB = B_KC ? WB : 2 * WB, NR = NRA + NRB;
    constexpr int NMMA = WB * WB;                        // MFMAs per k16-step
    constexpr int RPM = (NR + NMMA - 1) / NMMA;          // LDS reads slotted behind each MFMA

    floatx16 acc[WB][WB];
#pragma unroll
    for (int i = 0; i < WB; ++i)
#pragma unroll
        for (int j = 0; j < WB; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    // K-steps past the end are clamped to the last one: the tail iterations then issue the
    // same DMA traffic as the steady state (into stages nobody reads any more), which keeps
    // the loop body free of branches and the vmcnt bookkeeping uniform.
    auto srcA = [&](int kt) { return tile_src(baseA + (int64_t)(kt < last ? kt : last) * advA); };
    auto srcB = [&](int kt) { return tile_src(baseB + (int64_t)(kt < last ? kt : last) * advB); };

    // prologue: tiles 0..2 and the A half of tile 3 in flight (7 WB instructions)
    dma_tile<WB>(srcA(0), 0 >= last ? offAt : offA, lds_addr_of(st0), wave_u);
    dma_tile<WB>(srcB(0), 0 >= last ? offBt : offB, lds_addr_of(st0) + G::TILE_BYTES, wave_u);
    dma_tile<WB>(srcA(1), 1 >= last ? offAt : offA, lds_addr_of(st1), wave_u);
    dma_tile<WB>(srcB(1), 1 >= last ? offBt : offB, lds_addr_of(st1) + G::TILE_BYTES, wave_u);
    dma_tile<WB>(srcA(2), 2 >= last ? offAt : offA, lds_addr_of(st2), wave_u);
    dma_tile<WB>(srcB(2), 2 >= last ? offBt : offB, lds_addr_of(st2) + G::TILE_BYTES, wave_u);
    dma_tile<WB>(srcA(3), 3 >= last ? offAt : offA, lds_addr_of(st3), wave_u);

    u32x4 af[2][WB], bf[2][WB];   // fragment double buffer: [k16-step parity][block]

    // all reads of one fragment set, back to back (prologue only)
    auto load_frags = [&](const char* stage, int ks, int buf) {
#pragma unroll
        for (int r = 0; r < NRA; ++r) read_op(af[buf], stage, A_KC, wm * WT, ks, r);
#pragma unroll
        for (int r = 0; r < NRB; ++r) read_op(bf[buf], stage + G::TILE_BYTES, B_KC, wn * WT, ks, r);
    };
    // WB^2 MFMAs on fragment set `cur_buf`, with the NR reads of the next set (stage/ks ->
    // `nxt_buf`) slotted RPM (one; up to two for the 128 x 128 tile) per MFMA, so LDS latency is
    // always covered by matrix work and never more than NR (<= 16) reads are outstanding.  WB DMA
    // instructions (one operand tile's share of this wavefront) are spread over the step as
    // well -- issued in a burst right after the barrier, the four wavefronts would queue up
    // behind the CU's one address unit and stall their MFMA streams.
    auto mma_step_prefetch = [&](int cur_buf, const char* stage, int ks, int nxt_buf,
                                 const void* src, const uint32_t (&off_main)[WB], const uint32_t (&off_tail)[WB], bool tail_tile,
                                 uint32_t lds_tile) {
        uint32_t off[WB];
#pragma unroll
        for (int x = 0; x < WB; ++x) off[x] = (RAGGED && tail_tile) ? off_tail[x] : off_main[x];
#pragma unroll
        for (int q = 0; q < NMMA; ++q) {
            // serpentine order: consecutive MFMAs always share one operand fragment
            const int i = q / WB, j = (i & 1) ? WB - 1 - (q % WB) : (q % WB);
            E::mma(acc[i][j], bf[cur_buf][j], af[cur_buf][i]);   // D rows <-> n, cols <-> m
#pragma unroll
            for (int r = q * RPM; r < (q + 1) * RPM; ++r) {
                if (r < NRA) read_op(af[nxt_buf], stage, A_KC, wm * WT, ks, r);
                else if (r < NR) read_op(bf[nxt_buf], stage + G::TILE_BYTES, B_KC, wn * WT, ks, r - NRA);
            }
            if (q % WB == WB - 1) dma_1k(src, off[q / WB], lds_tile + (uint32_t)(wave_u * WB + q / WB) * 1024u);
        }
#pragma unroll
        for (int q = 0; q < NMMA; ++q) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);               // one MFMA
            const int nrd = NR - q * RPM < RPM ? NR - q * RPM : RPM;
            if (nrd == 2) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0); // its LDS reads
            else if (nrd == 1) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
    };

    // tile 0 must have landed before its first fragments are read
    NTG_WAIT_VMCNT(5 * WB);
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    load_frags(st0, 0, 0);

    // One K-step.  `cur` holds tile kt (its k16-step 0 fragments are already in registers),
    // `nxt` holds tile kt+1, `prv` held tile kt-1.  The single barrier sits between the two
    // k16-steps: by then every wavefront has issued and received its last reads of `cur`, so
    // the stage goes back to the DMA at once: the A half of tile kt+4 is fetched during the
    // second k16-step, its B half during the first k16-step of the next K-step.  Tile kt+1,
    // first touched in the second half, has had three K-steps to arrive.
    // RAGGED: zero the k >= K part of a fragment set of the last K-step.  Every lane's fragment
    // covers 8 consecutive k starting at 16 ks + 8 (lane / 32) in both LDS layouts, and K is a
    // multiple of 8, so a lane's fragment is either entirely real or entirely past the end.
    auto mask_tail = [&](int buf, int ks) {
        const bool ok = 16 * ks + 8 * (lane >> 5) < kr;
#pragma unroll
        for (int i = 0; i < WB; ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                af[buf][i][e] = ok ? af[buf][i][e] : 0u;
                bf[buf][i][e] = ok ? bf[buf][i][e] : 0u;
            }
    };

    auto iteration = [&](int kt, char* cur, const char* nxt, char* prv) {
        if (RAGGED && kt == last && kr < BK) mask_tail(0, 0);
        mma_step_prefetch(0, cur, 1, 1, srcB(kt + 3), offB, offBt, kt + 3 >= last, lds_addr_of(prv) + G::TILE_BYTES);
        // outstanding now: tiles kt+1, kt+2, kt+3 (2 WB instructions each): wait for the oldest
        NTG_WAIT_VMCNT(4 * WB);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // my reads of `cur` are complete
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (RAGGED && kt == last && kr < BK) mask_tail(1, 1);
        // (the last K-step prefetches fragments from a stage holding a clamped tile; unused)
        mma_step_prefetch(1, nxt, 0, 0, srcA(kt + 4), offA, offAt, kt + 4 >= last, lds_addr_of(cur));
    };

    for (int kt = 0; kt < KT; kt += 4) {
        iteration(kt, st0, st1, st3);
        if (kt + 1 < KT) iteration(kt + 1, st1, st2, st0);
        if (kt + 2 < KT) iteration(kt + 2, st2, st3, st1);
        if (kt + 3 < KT) iteration(kt + 3, st3, st0, st2);
    }
    NTG_WAIT_VMCNT(0);              // clamped tail DMAs have landed
    __builtin_amdgcn_s_barrier();   // all fragment reads done: LDS is free for the epilogue
    asm volatile("" ::: "memory");

    // ---- epilogue: per wavefront, WB 32-row slabs through a private fp32 LDS region ----
    // 32 rows x SROW bytes (the wavefront's WT columns in fp32) per wavefront; 16-byte slot s of
    // row r lives at s ^ (r & 7).  LPR lanes cover a row (8 columns each), so one step of the
    // read-back moves RPS rows.
    constexpr int SROW = WT * 4, LPR = WT / 8, RPS = 64 / LPR, NSTEP = 32 / RPS;
    char* slab = ((wave & 2) ? st1 : st0) + (wave & 1) * (32 * SROW);
    uint16_t* Cu = reinterpret_cast<uint16_t*>(C);
    const int col = 8 * (lane % LPR);              // this lane's 8 consecutive columns in the slab
    const int n = n0 + wn * WT + col;
    auto epilogue = [&](auto cmode_tag) {
        constexpr int CM = decltype(cmode_tag)::value;
        const uint16_t* bias = static_cast<const uint16_t*>(p.bias);
#pragma unroll
        for (int i = 0; i < WB; ++i) {
            // C0 of the whole slab is requested before the LDS round trip
            u32x4 c0[NSTEP];
            if constexpr (CM == C_ACCUMULATE) {
#pragma unroll
                for (int t = 0; t < NSTEP; ++t) {
                    const int m = m0 + wm * WT + 32 * i + RPS * t + lane / LPR;
                    if (!RAGGED || (m < p.M && n < p.N)) c0[t] = *reinterpret_cast<const u32x4*>(Cu + (int64_t)m * p.ldc + n);
                    else c0[t] = u32x4{0u, 0u, 0u, 0u};
                }
            }
            // lane holds rows m = 32 i + lane%32, cols 32 j + 8 rq + 4 (lane/32) + (0..3)
#pragma unroll
            for (int j = 0; j < WB; ++j)
#pragma unroll
                for (int rq = 0; rq < 4; ++rq) {
                    floatx4v v = {acc[i][j][4 * rq], acc[i][j][4 * rq + 1], acc[i][j][4 * rq + 2], acc[i][j][4 * rq + 3]};
                    const int slot = 8 * j + 2 * rq + (lane >> 5);
                    *reinterpret_cast<floatx4v*>(slab + (lane & 31) * SROW + ((slot ^ (lane & 7)) * 16)) = v;
                }
            // 32 rows x WT cols: NSTEP steps of RPS rows; a lane owns 8 consecutive columns
#pragma unroll
            for (int t = 0; t < NSTEP; ++t) {
                const int row = RPS * t + lane / LPR;
                const int sl = 2 * (lane % LPR);
                const floatx4v lo = *reinterpret_cast<const floatx4v*>(slab + row * SROW + ((sl ^ (row & 7)) * 16));
                const floatx4v hi = *reinterpret_cast<const floatx4v*>(slab + row * SROW + (((sl + 1) ^ (row & 7)) * 16));
                float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                const int m = m0 + wm * WT + 32 * i + row;
                if (RAGGED && (m >= p.M || n >= p.N)) continue;     // N % 8 == 0: a lane's 8 columns exist or not together
                if constexpr (CM == C_PARTIAL) {
                    // split-K: the fp32 sums of this k range go to a float matrix; rounding happens after the reduction
                    float* wp = static_cast<float*>(p.C) + (int64_t)b * p.sC + (int64_t)m * p.ldc + n;
                    *reinterpret_cast<floatx4v*>(wp) = lo;
                    *reinterpret_cast<floatx4v*>(wp + 4) = hi;
                    continue;
                }
                if constexpr (CM == C_ACCUMULATE) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) v[e] += Cvt16<DT>::up((uint16_t)(c0[t][e >> 1] >> (16 * (e & 1))));
                } else if constexpr (CM == C_BIAS) {
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        v[e] += Cvt16<DT>::up(bias[(int64_t)b * p.bias_bs + (int64_t)m * p.bias_rs + (int64_t)(n + e) * p.bias_cs]);
                }
                u32x4 o;
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    o[e] = (uint32_t)Cvt16<DT>::down(v[2 * e]) | ((uint32_t)Cvt16<DT>::down(v[2 * e + 1]) << 16);
                *reinterpret_cast<u32x4*>(Cu + (int64_t)m * p.ldc + n) = o;
            }
        }
    };
    if (p.cmode == C_ACCUMULATE) epilogue(std::integral_constant<int, C_ACCUMULATE>{});
    else if (p.cmode == C_PARTIAL) epilogue(std::integral_constant<int, C_PARTIAL>{});
    else if (p.cmode == C_BIAS) epilogue(std::integral_constant<int, C_BIAS>{});
    else epilogue(std::integral_constant<int, C_OVERWRITE>{});
}

// true when the fast kernel can serve the problem: 16-byte aligned rows everywhere (leading
// dimensions, batch strides, base pointers) and every contiguous extent a multiple of 8
// elements.  M, N and K themselves may be ragged with respect to the tile.
static inline bool gemm16_eligible(const GemmParams& p, bool ta) {
    return p.K >= 8 && p.K % 8 == 0 && p.N % 8 == 0 && (!ta || p.M % 8 == 0) &&
           !p.Aptr && !p.Bptr && !p.Cptr && p.vecA_ok && p.vecB_ok &&
           p.ldc % 8 == 0 && p.sC % 8 == 0 && p.lda < (1 << 22) && p.ldb < (1 << 22) &&
           ((reinterpret_cast<uintptr_t>(p.A) & 15) == 0) && ((reinterpret_cast<uintptr_t>(p.B) & 15) == 0) &&
           ((reinterpret_cast<uintptr_t>(p.C) & 15) == 0);
}

template <int DT, bool TA, bool TB, int WB>
static hipError_t launch_gemm16_cfg(const GemmParams& pin, hipStream_t s) {
    constexpr int TE = G16<WB>::BM;
    GemmParams p = pin;
    p.tiles_m = (p.M + TE - 1) / TE;
    p.tiles_n = (p.N + TE - 1) / TE;
    const int64_t blocks = (int64_t)p.tiles_m * p.tiles_n * p.batch;
    if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
    if (p.M % TE == 0 && p.N % TE == 0 && p.K % 32 == 0)
        hipLaunchKernelGGL((gemm16_kernel<DT, TA, TB, false, WB>), dim3((unsigned)blocks), dim3(256), 0, s, p);
    else
        hipLaunchKernelGGL((gemm16_kernel<DT, TA, TB, true, WB>), dim3((unsigned)blocks), dim3(256), 0, s, p);
    return hipGetLastError();
}

template <int DT, int WB>
static hipError_t launch_gemm16_wb(bool ta, bool tb, const GemmParams& p, hipStream_t s) {
    if (ta) return tb ? launch_gemm16_cfg<DT, true, true, WB>(p, s) : launch_gemm16_cfg<DT, true, false, WB>(p, s);
    return tb ? launch_gemm16_cfg<DT, false, true, WB>(p, s) : launch_gemm16_cfg<DT, false, false, WB>(p, s);
}

template <int DT>
static hipError_t launch_gemm16(bool ta, bool tb, const GemmParams& p, hipStream_t s) {
    if (gemm16_tile_edge(p.M, p.N, p.batch) == 256) return launch_gemm16_wb<DT, 4>(ta, tb, p, s);
    return launch_gemm16_wb<DT, 2>(ta, tb, p, s);
}

}  // namespace ntg
