// DMA-fed MFMA GEMM for gfx950 (Float16, BFloat16, Float32), the fast path:
//   C[M,N] (+)= op(A) . op(B),  16-byte aligned rows (leading dimensions and contiguous extents
//   multiples of one 16-byte chunk: 8 or 4 elements); M, N, K need not be multiples of the tile
//   (the RAGGED instantiation clamps DMA source addresses, zeroes the k tail in registers and
//   guards the stores).  Everything else goes through the general kernel in gemm_mfma_impl.h.
//
// Shape of the kernel
//   * One workgroup = 4 wavefronts (2 x 2), each owning WB x WB blocks of 32 x 32:
//       WB = 4: 256 x 256 tile, 256 accumulator registers per lane, one workgroup per CU (16-bit, large products);
//       WB = 2: 128 x 128 tile, half the LDS, two workgroups per CU (16-bit up to 128 large tiles, so that
//               mid-sized products still put a workgroup on every CU; Float32);
//       WB = 1: 64 x 64 tile (Float32 when that spreads the work more evenly over the 256 CUs).
//     The numbers below are the large tile's; the smaller ones scale the per-operand tile, DMA and read counts.
//   * 16-bit: v_mfma_f32_32x32x16_{f16,bf16} on 16-byte fragments (8 k per lane).  Float32: the same 16-byte
//     fragment holds 4 k, element e feeding the e-th of four v_mfma_f32_32x32x2_f32 -- all byte geometry (tiles,
//     stages, DMA instructions, K-major reads) is shared; a K-step is 64 bytes of k per row (32 or 16 elements).
//   * K advances through a 4-deep ring of LDS stages (4 x 32 KiB).  Global
//     memory is copied straight into LDS (global_load_lds_dwordx4): no staging registers,
//     three to four K-steps of loads in flight while one is being multiplied.  One barrier
//     per K-step, placed between its two halves; the DMA instructions and the LDS
//     fragment reads are slotted between the MFMAs one at a time, so neither the CU's single
//     address unit nor LDS latency ever holds up the matrix pipe.
//   * 16- and 8-bit plain products on 128 x 128 and 128 x 256 tiles take K-steps of 128 bytes of k per row instead (KD = 2
//     of the kernel template: whole cache lines of a K-contiguous operand, one barrier per sixteen MFMAs, fragments read
//     two quarter-steps ahead; four stages of 32 KiB or three of 48 KiB, one workgroup per CU).  Same order of summation.
//   * LDS layouts are conflict free for the reads the MFMA operands need:
//       operand stored K-contiguous  -> [row][64 B of k], 16-byte slot kv stored at
//                                        kv ^ ((row >> 1) & 3); one ds_read_b128 per block;
//       operand stored MN-contiguous -> [k][tile edge], 16-bit: 16-byte chunk c stored at
//                                        c ^ (2 * (k & 3)); ds_read_b64_tr_b16 turns four k-rows
//                                        into "4 consecutive k per lane", i.e. the transpose
//                                        is done by the LDS read, never in memory;
//                                        Float32: chunk c at c ^ (8 * ((k >> 2) & 1)), one
//                                        ds_read_b32 per block and k (32 consecutive floats per
//                                        half-wavefront, the halves in different bank halves).
//     Because the DMA writes 64 consecutive 16-byte slots per instruction, the swizzle is
//     applied by choosing which global chunk each lane fetches.
//   * The MFMA is issued with the operands swapped (B fragment first), so a lane holds four
//     consecutive columns of one row of C; the epilogue stages 32-row slabs through LDS in
//     fp32 and touches C with 16-byte accesses only (C0 is added in fp32 before the single
//     rounding to a 16-bit type).
#pragma once
#include "gemm_mfma_impl.h"

#include <type_traits>
#include <cstdlib>

namespace ntg {

typedef short shortx4 __attribute__((ext_vector_type(4)));
typedef float floatx4v __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void* lds_ptr_t;

#define NTG_WAIT_VMCNT(N) __builtin_amdgcn_s_waitcnt(((N) & 0xF) | (7 << 4) | (15 << 8) | (((N) >> 4) << 14))

// Int8 / UInt8 (one kernel: products and sums are taken modulo 2^32 in the accumulators and the low 8 bits of
// the result are the same for both signednesses, which is the reference's wrapping arithmetic in the element type)
typedef int intx16 __attribute__((ext_vector_type(16)));
typedef int intx4 __attribute__((ext_vector_type(4)));
typedef int intx2v __attribute__((ext_vector_type(2)));
template <> struct Elem<DT_I8> {
    using T = uint8_t; using AccS = int; using AccV = intx16;
    static __device__ __forceinline__ void mma(AccV& c, u32x4 a, u32x4 b) {
        c = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(intx4, a), __builtin_bit_cast(intx4, b), c, 0, 0, 0);
    }
};

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
// ES = bytes per element (2: Float16 / BFloat16, 4: Float32).  A K-step is 64 bytes of k for every row (32 or 16
// elements), so the byte geometry of tiles, stages and DMA instructions is the same for both element sizes.
// KD = 64-byte runs of k per row and K-step: 1, or 2 for the deep K-step of the small 16-bit tiles (see gemm_ring_kernel)
template <int WB, int ES, int KD = 1>
struct RingGeom {
    static constexpr int KB = 64 * KD;                   // bytes of k per row and K-step
    static constexpr int BM = 64 * WB, BN = 64 * WB, BK = KB / ES, NST = 4;
    static constexpr int VEL = 16 / ES;                  // elements per 16-byte chunk
    static constexpr int WT = 32 * WB;                   // edge of a wavefront's share of the tile
    static constexpr int TILE_BYTES = BM * KB;           // one operand tile, 16 / 8 KiB (twice that with KD = 2)
    static constexpr int NI = WB * KD;                   // DMA instructions per wavefront and operand tile
    static constexpr int STAGE_BYTES = 2 * TILE_BYTES;   // 32 / 16 KiB
    static constexpr int MN_ROW_BYTES = BM * ES;         // one k-row of an MN-contiguous operand tile
    static constexpr int CHUNKS = MN_ROW_BYTES / 16;     // 16-byte chunks in such a row (16 .. 64)
    static constexpr int ROWS_PER_DMA = 64 / CHUNKS;     // k-rows of such a tile that one DMA instruction fills (1 .. 4)
};

// Per-lane BYTE offsets (relative to the tile's first element at K-step 0) of this wavefront's
// WB DMA instructions into one operand tile.  Instruction j = WB*wave + jj fills LDS bytes
// [1024 j, 1024 j + 1024) of the tile:
//   K-contiguous operand: rows 16 j + lane/4, 16-byte slot lane%4 holds kv = slot ^ km_swz(row)
//   MN-contiguous operand (CH chunks per k-row): piece 64 j + lane of the tile = k-row (64 j + lane) / CH, slot (64 j + lane) % CH, holds
//                          chunk = slot ^ (2*(krow&3)) for 16-bit elements (what the transposing
//                          reads need), slot ^ mn8_swizzle(krow) for 8-bit elements,
//                          slot ^ (8*(krow&1)) for Float32 (the two consecutive k-rows that one
//                          ds_read_b32 touches land in different halves of the 64 banks)
// With RAGGED, mn_valid (1..BM rows/columns of the tile that exist) and k_valid (k of the
// K-step that exist, a multiple of one chunk) clamp the SOURCE address into the matrix: lanes
// whose data does not exist fetch a neighbouring chunk instead.  Rows/columns past the edge
// only ever reach accumulators that the epilogue does not store; k past the end is zeroed
// in the fragment registers before it is multiplied.
// 8-bit MN-contiguous tiles: chunk c of k-row krow is stored at c ^ mn8_swizzle(krow), which puts the eight k-rows that
// one transposing read touches into different 16-byte bank groups (CH = chunks per k-row)
template <int CH>
__device__ __forceinline__ int mn8_swizzle(int krow) { return CH >= 8 ? (krow & 7) : ((krow & 7) >> 1); }

// 128-byte rows (KD = 2): 16-byte slot kv of row r is stored at kv ^ swz8(r).  Eight consecutive rows get eight different
// values, and so do the eight rows of either parity among sixteen consecutive ones: whichever way the banks repeat
// (every 128 or every 256 bytes), the lanes that one pass of a ds_read_b128 serves hit different banks.
__device__ __forceinline__ int swz8(int row) { return (row & 7) ^ ((row >> 3) & 1); }

// 64-byte rows (K-major tiles, KD = 1): 16-byte slot kv of row r is stored at kv ^ km_swz(r): read 16 bytes per lane, eight
// lanes to a pass, rows r .. r + 7 hit eight different 16-byte bank groups.  (Float32 plain products read such rows one dword
// per lane; taking bits 2 and 3 of the row for them instead was measured and changed nothing.)
template <int ES>
__device__ __forceinline__ int km_swz(int row) { return (row >> 1) & 3; }

template <bool KC, bool RAGGED, int WB, int ES, int KD = 1>
__device__ __forceinline__ void dma_offsets(uint32_t (&off)[WB * KD], int64_t ld, int wave, int lane, int mn_valid, int k_valid) {
    constexpr int CH = RingGeom<WB, ES>::CHUNKS, VEL = RingGeom<WB, ES>::VEL;
#pragma unroll
    for (int jj = 0; jj < WB * KD; ++jj) {
        const int j = wave * WB * KD + jj;
        if constexpr (KC) {
            // (KD = 2: an instruction covers 8 rows of 128 bytes, whole cache lines)
            int row = KD == 2 ? 8 * j + (lane >> 3) : 16 * j + (lane >> 2);
            int kv = KD == 2 ? (lane & 7) ^ swz8(row) : (lane & 3) ^ km_swz<ES>(row);
            if constexpr (RAGGED) {
                row = row < mn_valid ? row : mn_valid - 1;
                kv = kv < k_valid / VEL ? kv : k_valid / VEL - 1;
            }
            off[jj] = (uint32_t)(((int64_t)row * ld + kv * VEL) * ES);
        } else {
            // (CH = 24, the 192-row tile: three instructions fill eight k-rows, a k-row may begin inside an instruction)
            int krow = (64 * j + lane) / CH;
            int chunk = ((64 * j + lane) % CH) ^ (ES == 2 ? 2 * (krow & 3) : ES == 4 ? 8 * (krow & 1) : ES == 1 ? mn8_swizzle<CH>(krow) : 0);   // Float64: stored as is
            if constexpr (RAGGED) {
                krow = krow < k_valid ? krow : k_valid - 1;
                chunk = chunk < mn_valid / VEL ? chunk : mn_valid / VEL - 1;
            }
            off[jj] = (uint32_t)(((int64_t)krow * ld + chunk * VEL) * ES);
        }
    }
}

// One DMA instruction: 64 lanes x 16 bytes from  base + off  (uniform base, per-lane offset)
// to LDS bytes [lds_addr, lds_addr + 1024).  Written as inline assembly so that the only
// waits on these loads are the explicit s_waitcnt vmcnt(N) of the pipeline: the compiler's
// own tracking of LDS-DMA writes made every read of one of the four stages wait for all
// outstanding loads.  The memory clobber keeps LDS reads from being moved across it.  m0 is not
// in the clobber list: it is a reserved register to the compiler, which never keeps a value in it
// across statements (it loads m0 right before each of its own uses) and rejects it in a clobber
// list with a "reserved register" diagnostic.
__device__ __forceinline__ void dma_1k(const void* base, uint32_t off, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :: "s"(lds_addr), "v"(off), "s"(base) : "memory");
}

// One gathering DMA instruction: 64 lanes x 4 bytes, every lane from its own address, to LDS bytes
// [lds_addr, lds_addr + 256).
__device__ __forceinline__ void dma_dword(const void* addr, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off"
                 :: "s"(lds_addr), "v"(addr) : "memory");
}
// what the padding taps of a gathered convolution operand read
static __device__ __attribute__((aligned(16))) const uint32_t ring_zero_word[4] = {0u, 0u, 0u, 0u};

template <int WB>   // (WB = instructions per wavefront)
__device__ __forceinline__ void dma_tile(const void* sbase, const uint32_t (&off)[WB], uint32_t lds_tile, int wave_u) {
#pragma unroll
    for (int jj = 0; jj < WB; ++jj) dma_1k(sbase, off[jj], lds_tile + (uint32_t)(wave_u * WB + jj) * 1024u);
}

__device__ __forceinline__ uint32_t lds_addr_of(const char* p) {
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)p;
}

// CONV = 0: plain product.  CONV = 1 / 2 (Float32, two spatial axes): op(B) is the never-stored im2col matrix col[kk][l]
// of the image at p.B (1: convolution, C[o][l]; 2: its transpose col^T[l][kk], the weight gradient C[o][kk]), described by
// p.conv.  Its LDS tile is [k-row][BN floats]; one DMA instruction gathers 64 consecutive columns of one k-row, the
// address being a wave-uniform term of the k-row plus a per-lane term of the column that is fixed for the whole K loop
// (convolution: the tap (c, r, q) is uniform, the pixel per lane; weight gradient: the other way round).  Padding taps
// and columns / k-rows past the edge read a zero word instead, so the tile in LDS is exact and the multiply loop is the
// plain one.  Wavefront w gathers k-rows 4 w .. 4 w + 3 of every K-step.
// WBN_ != 0: a rectangular tile, 64 WB_ rows x 64 WBN_ columns (plain products only).
// KD_ = 2 (16-bit plain products on 128 x 128 tiles): a K-step is 128 bytes of k per row, so a K-contiguous operand is
// fetched in whole 128-byte cache lines (half the requests to L2 of the 64-byte K-step) and the one barrier of a K-step
// comes every sixteen MFMAs instead of every eight; the four stages are 32 KiB each (one workgroup per CU).  Fragments
// are read two quarter-steps ahead (four sets in registers), the whole of tile kt + 3 is fetched during K-step kt.
// With WBN_ = 4 (128 x 256 tiles) the stages are 48 KiB and there are three of them: tile kt + 2 is fetched from the
// barrier of K-step kt - 1 (which frees its stage) to the barrier of K-step kt.
// entries of the weight gradient's LDS table of window origins (16 + 128 KiB beside the 256 x 256 tile's ring; 14 + 64 KiB
// on the smaller tiles, so that two workgroups still share a CU)
constexpr int dw_table_entries(int wb) { return wb == 4 ? 6144 : 3584; }

template <int DT, bool TA, bool TB, bool RAGGED, int WB_, int CONV = 0, int WBN_ = 0, int KD_ = 1>
__global__ void __launch_bounds__(256) gemm_ring_kernel(const GemmParams p) {
    using E = Elem<DT>;
    using T = typename E::T;
    constexpr int ES = sizeof(T);
    constexpr int WBM = WB_, WBN = WBN_ ? WBN_ : WB_;    // 32 x 32 blocks per wavefront along m / along n
    constexpr int WB = WBN;                              // (the gathered operand is B; gathering kernels have square tiles)
    static_assert(CONV == 0 || WBM == WBN, "gathering kernels have square tiles");
    constexpr int KD = KD_;
    static_assert(KD == 1 || (KD == 2 && CONV == 0 && (ES == 2 || ES == 1) && WB_ == 2 && (WBN_ == 0 || WBN_ == 4)), "deep K-steps: 16- and 8-bit plain products on 128 x 128 and 128 x 256 tiles");
    constexpr bool RING3 = KD == 2 && WBN_ == 4;         // three stages of 48 KiB
    using GA = RingGeom<WBM, ES, KD>;                    // geometry of the A tile
    using G = RingGeom<WBN, ES, KD>;                     // geometry of the B tile
    constexpr int A_TILE_BYTES = GA::TILE_BYTES, STAGE_BYTES = GA::TILE_BYTES + G::TILE_BYTES;
    constexpr int WTM = GA::WT, WTN = G::WT;             // a wavefront's share of the tile: WTM rows x WTN columns
    constexpr bool GATHER4 = CONV == 1 || CONV == 2;     // op(B) gathered element by element from an NCHW image
    constexpr bool GATHER16 = CONV == 3 || CONV == 5;    // op(B) = col^T gathered in 16-byte pieces from a channels-last image
    constexpr bool HALO = CONV == 5;                     // ... whose copy carries the padding as pixels of zeros: every tap of every window exists
    constexpr bool GATHERW = CONV == 4;                  // op(B) = col^T of a channels-last image, 16-byte pieces along the channels (weight gradient)
    constexpr bool A_KC = !TA, B_KC = GATHER4 ? false : GATHER16 ? true : GATHERW ? false : TB;
    constexpr int BK = G::BK;
    static_assert(!GATHER4 || (ES == 4 && !TA && RAGGED), "gathered operands: Float32, A stored [m][k], guarded edges");
    static_assert(!GATHER16 || ((ES == 4 || ES == 2) && !TA && RAGGED), "channels-last gather: 16/32-bit floats, A stored [m][k], guarded edges");
    static_assert(!GATHERW || ((ES == 4 || ES == 2) && !TB && RAGGED), "channels-last weight gradient: 16/32-bit floats, guarded edges");
    constexpr int NA = WBM * KD, NB = GATHER4 ? 4 * WB : WBN * KD;   // DMA instructions per wavefront and K-step for the A / B tile
    // B instructions issued in the first / second half-step (the second also carries the A tile's).  Splitting a gathered
    // tile between the two was measured slower than issuing all of it in the first.
    constexpr int NB1 = NB, NB2 = NB - NB1;

    __shared__ __attribute__((aligned(1024))) char st0[STAGE_BYTES];
    __shared__ __attribute__((aligned(1024))) char st1[STAGE_BYTES];
    __shared__ __attribute__((aligned(1024))) char st2[STAGE_BYTES];
    __shared__ __attribute__((aligned(1024))) char st3[RING3 ? 1024 : STAGE_BYTES];
    // channels-last weight gradient: byte offset of every output pixel's window origin inside one (bordered) image
    constexpr int DW_TABLE = CONV == 4 ? dw_table_entries(WB) : 1;
    __shared__ int dw_tab[DW_TABLE];

    if (p.gate && *p.gate != p.gate_want) return;       // (uniform: the other kernel of a gated pair does this product)
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    const int lid = p.group_m < 0 ? (int)blockIdx.x : xcd_contiguous_id(blockIdx.x, gridDim.x);      // (group_m != 0: measurement only, see ring_tile_order_override)
    const int tiles = p.tiles_m * p.tiles_n;
    const int b = lid / tiles;
    int tm, tn;
    tile_coords(lid - b * tiles, p.tiles_m, p.tiles_n, p.group_m > 0 ? p.group_m : p.group_m < 0 ? -p.group_m : 4, tm, tn);
    const int m0 = tm * GA::BM, n0 = tn * G::BN;

    // (pointer tables: one uniform load per operand; everything below is base + offset either way)
    const T* A = p.Aptr ? static_cast<const T*>(p.Aptr[b]) : static_cast<const T*>(p.A) + operand_offset(p, b, p.sA, p.sAk);
    const T* B = p.Bptr ? static_cast<const T*>(p.Bptr[b]) : static_cast<const T*>(p.B) + operand_offset(p, b, p.sB, p.sBk);
    T* C = p.Cptr ? static_cast<T*>(p.Cptr[b]) : static_cast<T*>(p.C) + (int64_t)b * p.sC;

    using AccV = typename E::AccV;
    using AccS = typename E::AccS;
    AccV acc[WBM][WBN];
#pragma unroll
    for (int i = 0; i < WBM; ++i)
#pragma unroll
        for (int j = 0; j < WBN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = (AccS)0;
    // Float32: the accumulators start from C0 (C itself, or the bias), so that every output element is the reference's chain
    // c = C0; c = fma(a_k, b_k, c) for ascending k, bit for bit, and the epilogue only stores.  A lane holds rows
    // 32 i + lane % 32 and columns 32 j + 8 rq + 4 (lane / 32) + (0..3) of its wavefront's part of the tile.
    if constexpr (ES == 4 && std::is_same<AccS, float>::value) {
        if (p.cmode == C_ACCUMULATE || p.cmode == C_BIAS) {            // (uniform)
            const bool from_c = p.cmode == C_ACCUMULATE;
            const NTG_GLOBAL float* bias = (const NTG_GLOBAL float*)static_cast<const float*>(p.bias);
            const bool vec_ok = from_c ? (p.ldc % 4 == 0 && (reinterpret_cast<uintptr_t>(C) & 15) == 0)
                                       : (p.bias_cs == 1 && p.bias_rs % 4 == 0 && p.bias_bs % 4 == 0 && (reinterpret_cast<uintptr_t>(p.bias) & 15) == 0);
            const int64_t cstep = from_c ? 1 : p.bias_cs;
            typedef float f32x4 __attribute__((ext_vector_type(4)));
#pragma unroll
            for (int i = 0; i < WBM; ++i) {
                const int m = m0 + wm * WTM + 32 * i + (lane & 31);
#pragma unroll
                for (int j = 0; j < WBN; ++j)
#pragma unroll
                    for (int rq = 0; rq < 4; ++rq) {
                        const int nn = n0 + wn * WTN + 32 * j + 8 * rq + 4 * (lane >> 5);
                        f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f};
                        if (m < p.M && nn < p.N) {
                            const NTG_GLOBAL float* src = from_c ? (const NTG_GLOBAL float*)reinterpret_cast<const float*>(C) + (int64_t)m * p.ldc + nn
                                                      : bias + (int64_t)b * p.bias_bs + (int64_t)m * p.bias_rs + (int64_t)nn * p.bias_cs;
                            if (vec_ok && nn + 4 <= p.N) v = *(const NTG_GLOBAL f32x4*)src;
                            else {
#pragma unroll
                                for (int e = 0; e < 4; ++e)
                                    if (nn + e < p.N) v[e] = src[(int64_t)e * cstep];
                            }
                        }
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[i][j][4 * rq + e] = v[e];
                    }
            }
        }
    }


    // ---- DMA sources: uniform tile base (advances by adv bytes per K-step) + per-lane offsets ----
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const int KT = (p.K + BK - 1) / BK;
    const int last = KT - 1;
    const int kr = p.K - last * BK;                                  // k that exist in the last K-step (a multiple of one chunk)
    const int mvalid = p.M - m0 < GA::BM ? p.M - m0 : GA::BM;
    const int nvalid = p.N - n0 < G::BN ? p.N - n0 : G::BN;
    uint32_t offA[WBM * KD], offB[WBN * KD];      // K-steps before the last
    uint32_t offAt[WBM * KD], offBt[WBN * KD];    // the last K-step (RAGGED: k clamped to what exists)
    dma_offsets<A_KC, RAGGED, WBM, ES, KD>(offA, p.lda, wave, lane, mvalid, BK);
    dma_offsets<B_KC, RAGGED, WBN, ES, KD>(offB, p.ldb, wave, lane, nvalid, BK);
    dma_offsets<A_KC, RAGGED, WBM, ES, KD>(offAt, p.lda, wave, lane, mvalid, kr);
    dma_offsets<B_KC, RAGGED, WBN, ES, KD>(offBt, p.ldb, wave, lane, nvalid, kr);
    const char* baseA = reinterpret_cast<const char*>(A) + (A_KC ? (int64_t)m0 * p.lda : (int64_t)m0) * ES;
    const char* baseB = reinterpret_cast<const char*>(B) + (B_KC ? (int64_t)n0 * p.ldb : (int64_t)n0) * ES;
    const int64_t advA = (A_KC ? (int64_t)BK : (int64_t)BK * p.lda) * ES;
    const int64_t advB = (B_KC ? (int64_t)BK : (int64_t)BK * p.ldb) * ES;
    // ---- gathered operand: per-lane constants of this lane's WB columns (64 h + lane) of the tile ----
    //   convolution:      lanepart = byte offset of the output pixel's window origin without padding, cmask = one bit per
    //                     tap row (bits 0..7) and tap column (bits 8..15) that falls inside the image; 0 past the edge
    //   weight gradient:  lanepart = byte offset of the tap inside the image slice, cmask = r*d_r | q*d_c << 16,
    //                     0x80008000 (never inside) past the edge
    uint32_t lanepart[WB], cmask[WB];
    if constexpr (GATHER4) {
        const ConvGeom& g = p.conv;
#pragma unroll
        for (int h = 0; h < WB; ++h) {
            const int n = n0 + 64 * h + lane;
            if constexpr (CONV == 1) {
                const uint32_t l = n < p.N ? (uint32_t)n : 0u;
                const uint32_t oh = fast_div(l, g.div_wo), ow = l - oh * (uint32_t)g.Wo;
                const int ih0 = (int)oh * g.s_r - g.p_r, iw0 = (int)ow * g.s_c - g.p_c;
                uint32_t m = 0;
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    if (t < g.k_r && (unsigned)(ih0 + t * g.d_r) < (unsigned)g.H) m |= 1u << t;
                    if (t < g.k_c && (unsigned)(iw0 + t * g.d_c) < (unsigned)g.W) m |= 256u << t;
                }
                cmask[h] = n < p.N ? m : 0u;
                lanepart[h] = (oh * (uint32_t)g.s_r * (uint32_t)g.W + ow * (uint32_t)g.s_c) * 4u;
            } else {
                const uint32_t kk = n < p.N ? (uint32_t)n : 0u;
                const uint32_t c = fast_div(kk, g.div_krc), rem = kk - c * (uint32_t)g.k_rc;
                const uint32_t r = fast_div(rem, g.div_kc), q = rem - r * (uint32_t)g.k_c;
                cmask[h] = n < p.N ? (r * (uint32_t)g.d_r) | ((q * (uint32_t)g.d_c) << 16) : 0x80008000u;
                lanepart[h] = (c * (uint32_t)g.chan + r * (uint32_t)g.d_r * (uint32_t)g.W + q * (uint32_t)g.d_c) * 4u;
            }
        }
    }
    // Wave-uniform state of the four k-rows (4 wave + i) this wavefront gathers, kept in scalar registers and advanced
    // by one K-step (16 k) after each use, so the loop body holds no division: a k-row index is the mixed-radix number
    // (hi, mid, lo) = (c, r, q) with radices (k_r, k_c) for the convolution, (-, oh, ow) with radix Wo for the weight
    // gradient; adding 16 = (d_hi, d_mid, d_lo) needs one carry per digit.  st_up is the byte offset that the digits
    // contribute (padding included, so it may be negative).
    int st_lo[4], st_mid[4], st_up[4], st_k[4];
    int cv_r0 = 1, cv_r1 = 1, cv_dlo = 0, cv_dmid = 0, cv_dup = 0, cv_carry_lo = 0, cv_carry_mid = 0;
    if constexpr (GATHER4) {
        const ConvGeom& g = p.conv;
        const int s_lo = (CONV == 1 ? g.d_c : g.s_c) * 4, s_mid = (CONV == 1 ? g.d_r : g.s_r) * g.W * 4, s_hi = g.chan * 4;
        cv_r0 = CONV == 1 ? g.k_c : g.Wo;
        cv_r1 = CONV == 1 ? g.k_r : 0x7fffffff;
        const FastDiv& dv0 = CONV == 1 ? g.div_kc : g.div_wo;
        const uint32_t t16 = fast_div((uint32_t)BK, dv0);
        cv_dlo = BK - (int)t16 * cv_r0;
        const uint32_t h16 = CONV == 1 ? t16 / (uint32_t)cv_r1 : 0u;
        cv_dmid = (int)t16 - (int)h16 * (CONV == 1 ? cv_r1 : 0);
        cv_dup = (int)h16 * s_hi + cv_dmid * s_mid + cv_dlo * s_lo;
        cv_carry_lo = s_mid - cv_r0 * s_lo;
        cv_carry_mid = CONV == 1 ? s_hi - cv_r1 * s_mid : 0;
        const int base0 = -(g.p_r * g.W + g.p_c) * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t idx = (uint32_t)(4 * wave_u + i);
            const uint32_t t = fast_div(idx, dv0);
            st_lo[i] = (int)(idx - t * (uint32_t)cv_r0);
            const uint32_t hi = CONV == 1 ? t / (uint32_t)cv_r1 : 0u;
            st_mid[i] = (int)t - (int)hi * (CONV == 1 ? cv_r1 : 0);
            st_up[i] = base0 + (int)hi * s_hi + st_mid[i] * s_mid + st_lo[i] * s_lo;
            st_k[i] = (int)idx;
        }
    }
    // Instruction x (0 .. 4 WB - 1) of this wavefront's share of the NEXT gathered tile (tiles are gathered in K order):
    // k-row 4 wave + x / WB, columns 64 (x % WB) .. + 63; the k-row's state moves on after its last instruction.
    auto conv_dma = [&](int x, uint32_t lds_tile) __attribute__((always_inline)) {
        if constexpr (GATHER4) {
            const ConvGeom& g = p.conv;
            const int i = x / WB, h = x % WB;
            const int krow = 4 * wave_u + i;
            const char* img = reinterpret_cast<const char*>(B);
            const bool krow_ok = st_k[i] < p.K;                    // uniform
            bool ok;
            if constexpr (CONV == 1) {
                const uint32_t sr = krow_ok ? (uint32_t)st_mid[i] : 31u, sq = 8u + (uint32_t)st_lo[i];
                ok = ((cmask[h] >> sr) & (cmask[h] >> sq) & 1u) != 0u;
            } else {
                const int ih0 = krow_ok ? st_mid[i] * g.s_r - g.p_r : -(1 << 20), iw0 = st_lo[i] * g.s_c - g.p_c;
                ok = ((uint32_t)(ih0 + (int)(cmask[h] & 0xffffu)) < (uint32_t)g.H) & ((uint32_t)(iw0 + (int)(cmask[h] >> 16)) < (uint32_t)g.W);
            }
            const char* src = ok ? img + (int64_t)st_up[i] + lanepart[h] : reinterpret_cast<const char*>(ring_zero_word);
            dma_dword(src, lds_tile + (uint32_t)(krow * G::MN_ROW_BYTES + h * 256));
            if (h == WB - 1) {
                int lo = st_lo[i] + cv_dlo, mid = st_mid[i] + cv_dmid, up = st_up[i] + cv_dup;
                const bool c0 = lo >= cv_r0;
                lo = c0 ? lo - cv_r0 : lo;
                mid = c0 ? mid + 1 : mid;
                up = c0 ? up + cv_carry_lo : up;
                const bool c1 = mid >= cv_r1;
                mid = c1 ? mid - cv_r1 : mid;
                up = c1 ? up + cv_carry_mid : up;
                st_lo[i] = lo; st_mid[i] = mid; st_up[i] = up; st_k[i] += BK;
            }
        }
    };
    auto conv_tile = [&](uint32_t lds_tile) __attribute__((always_inline)) {
#pragma unroll
        for (int x = 0; x < 4 * WB; ++x) conv_dma(x, lds_tile);
    };

    // ---- channels-last gather (CONV = 3): the image at p.B is stored [pixel][channel] (p.conv.chan = channels per pixel),
    // the weights at A [m][(r, q, c)], so a K-step is 64 bytes of consecutive channels of ONE tap for every output pixel:
    // the B tile [pixel row][64 B] is filled by the same WB 16-byte DMA instructions per wavefront as a stored K-major
    // operand, each lane's address being a wave-uniform term of the K-step (tap and first channel, advanced by counters
    // in scalar registers) plus a per-lane term of its output pixel and 16-byte slot; padding taps read zeros.
    // Few channels (p.conv.tap_step = T = 2 or 4): a pixel holds 64 / T bytes of channels and a K-step covers T consecutive
    // taps of one tap row (the row padded to p.conv.kq_pad taps with zero weights): a lane's 16-byte slot then belongs to
    // tap q + tq3 of the step, which shifts its address and its validity bit.
    uint32_t lanepart3[WB], cmask3[WB], tq3[WB];
    int k3_c0 = 0, k3_q = 0, k3_r = 0, k3_up = 0, k3_k = 0, k3_cg = 1;
    if constexpr (GATHER16) {
        const ConvGeom& g = p.conv;
        k3_cg = p.K / g.k_rc;
        k3_up = -(g.p_r * g.W + g.p_c) * g.chan * ES;
#pragma unroll
        for (int x = 0; x < WB; ++x) {
            const int row = 16 * (wave * WB + x) + (lane >> 2);
            const int n = n0 + row;
            const uint32_t l = (n < p.N ? (uint32_t)n : 0u) + (uint32_t)g.n_base;
            const uint32_t oh = fast_div(l, g.div_wo), ow = l - oh * (uint32_t)g.Wo;
            const int ih0 = (int)oh * g.s_r - g.p_r, iw0 = (int)ow * g.s_c - g.p_c;
            uint32_t m = 0;
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                if (t < g.k_r && (unsigned)(ih0 + t * g.d_r) < (unsigned)g.H) m |= 1u << t;
                if (t < g.k_c && (unsigned)(iw0 + t * g.d_c) < (unsigned)g.W) m |= 256u << t;
            }
            cmask3[x] = n < p.N ? m : 0u;
            const uint32_t kv = (uint32_t)((lane & 3) ^ km_swz<ES>(row));
            uint32_t tq = 0u, cho = kv * 16u;
            if (g.tap_step > 1) {
                const uint32_t cb = 64u / (uint32_t)g.tap_step;        // bytes of channels per pixel: 16 or 32
                tq = cho / cb;
                cho -= tq * cb;
            }
            tq3[x] = tq;
            lanepart3[x] = (oh * (uint32_t)g.s_r * (uint32_t)g.W + ow * (uint32_t)g.s_c + tq * (uint32_t)g.d_c) * (uint32_t)g.chan * (uint32_t)ES + cho;
        }
    }
    // instruction x (0 .. WB - 1) of this wavefront's share of the NEXT gathered tile; the K-step's counters move on after the last
    auto conv3_dma = [&](int x, uint32_t lds_tile) __attribute__((always_inline)) {
        if constexpr (GATHER16) {
            const ConvGeom& g = p.conv;
            const char* img = reinterpret_cast<const char*>(B);
            if constexpr (HALO) {
                // the image carries its padding (p.conv describes the padded image, padding 0): no tap is ever outside, the
                // address is a uniform base plus the lane's constant offset, exactly the DMA of a stored operand
                // (K-steps past the end re-read tap 0: their stage is never multiplied)
                const int64_t up = k3_k < p.K ? (int64_t)k3_up : 0;
                dma_1k(img + up, lanepart3[x], lds_tile + (uint32_t)(wave_u * WB + x) * 1024u);
            } else {
            const uint32_t sr = k3_k < p.K ? (uint32_t)k3_r : 31u, sq = 8u + (uint32_t)k3_q + tq3[x];
            const bool ok = ((cmask3[x] >> sr) & (cmask3[x] >> sq) & 1u) != 0u;
            const char* src = ok ? img + (int64_t)k3_up + lanepart3[x] : reinterpret_cast<const char*>(ring_zero_word);
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                         :: "s"(lds_tile + (uint32_t)(wave_u * WB + x) * 1024u), "v"(src) : "memory");
            }
            if (HALO && g.tap_inner && x == WB - 1) {
                // one K-step on, taps inside a run of 64 bytes of channels: the next tap of this run, else the next run.  The
                // taps of one run reach the same few pixels of the copy again and again while they are still in the XCD's L2;
                // with the taps outermost every tap streamed the whole panel of the image through it again.
                int q = k3_q + 1, r = k3_r, c0 = k3_c0, up = k3_up + g.d_c * g.chan * ES;
                const bool w0 = q >= g.k_c;
                q = w0 ? 0 : q;
                r = w0 ? r + 1 : r;
                up = w0 ? up - g.k_c * g.d_c * g.chan * ES + g.d_r * g.W * g.chan * ES : up;
                const bool w1 = r >= g.k_r;
                r = w1 ? 0 : r;
                c0 = w1 ? c0 + BK : c0;
                up = w1 ? up - g.k_r * g.d_r * g.W * g.chan * ES + BK * ES : up;
                k3_c0 = c0; k3_up = up; k3_q = q; k3_r = r; k3_k += BK;
            }
            if (!(HALO && g.tap_inner) && x == WB - 1) {
                // one K-step on: the next 64 bytes of channels of this tap, else the next tap (or the next tap_step taps)
                const bool merged = g.tap_step > 1;
                const int qstep = merged ? g.tap_step : 1, qend = merged ? g.kq_pad : g.k_c;
                int c0 = k3_c0 + BK, up = k3_up + BK * ES, q = k3_q, r = k3_r;
                const bool w0 = merged || c0 >= k3_cg;
                up = merged ? k3_up + qstep * g.d_c * g.chan * ES : w0 ? up - k3_cg * ES + g.d_c * g.chan * ES : up;
                c0 = w0 ? c0 - k3_cg : c0;
                q = w0 ? q + qstep : q;
                const bool w1 = q >= qend;
                q = w1 ? 0 : q;
                up = w1 ? up - qend * g.d_c * g.chan * ES + g.d_r * g.W * g.chan * ES : up;
                r = w1 ? r + 1 : r;
                k3_c0 = merged ? 0 : c0; k3_up = up; k3_q = q; k3_r = r; k3_k += BK;
            }
        }
    };

    // ---- channels-last weight gradient (CONV = 4): C[o][(r, q, c)] = sum over output pixels l of A[o][l] * x[pixel(l, r, q)][c].
    // The B tile is the MN-major one of a stored [k][n] operand (k = output pixel, n = (tap, channel)), filled by the same
    // WB 16-byte DMA instructions per wavefront; a lane's 16 bytes are channels c .. of ONE tap for the whole K loop
    // (tap reach and byte offset kept per lane), and its k-row moves on by BK output pixels per K-step: the pixel is
    // split into (row, column) with one multiply-shift division per instruction.  Padding and k >= K read zeros.
    // Several images may share one K loop (p.conv.fold_L = output pixels per image, 0: one image): k then counts the
    // output pixels of consecutive images, and one more division gives the image, p.conv.fold_stride elements apart.
    int krow4[WB], noff4[WB];
    uint32_t tap4[WB];
    int k4_k = 0, k4_base = 0;
    if constexpr (GATHERW) {
        const ConvGeom& g = p.conv;
        constexpr int CH = G::CHUNKS;
        if (g.k_ranges) k4_base = b * p.K;                         // this item's first output pixel, counted through the images
        const uint32_t cgc = (uint32_t)(g.n_total ? g.n_total : p.N) / (uint32_t)g.k_rc;   // channels of the slice: N = taps * channels
#pragma unroll
        for (int x = 0; x < WB; ++x) {
            const int j = wave * WB + x;
            const int krow = (64 / CH) * j + lane / CH;
            const int chunk = (lane % CH) ^ (ES == 2 ? 2 * (krow & 3) : 8 * (krow & 1));
            const int n = n0 + chunk * G::VEL;
            const uint32_t nn = (n < p.N ? (uint32_t)n : 0u) + (uint32_t)g.n_base;
            const uint32_t t = nn / cgc, c = nn - t * cgc;
            const uint32_t r = fast_div(t, g.div_kc), q = t - r * (uint32_t)g.k_c;
            krow4[x] = n < p.N ? krow : 0x40000000;                       // columns past the edge: never inside
            tap4[x] = (r * (uint32_t)g.d_r) | ((q * (uint32_t)g.d_c) << 16);
            noff4[x] = (((int)(r * (uint32_t)g.d_r) - g.p_r) * g.W + ((int)(q * (uint32_t)g.d_c) - g.p_c)) * g.chan * ES + (int)c * ES;
        }
    }
    // Table form (p.conv.pix_table = output pixels per image, at most DW_TABLE - BK; the copy of the image carries its padding
    // as pixels of zeros, so every tap of every window exists): the window origin's byte offset of each output pixel is
    // computed once per workgroup into LDS, BK entries of zeros behind them.  A K-step then lies inside ONE image (per-image
    // items, or k ranges whose images are whole K-steps): image and first pixel are wave-uniform counters, a lane reads its
    // pixel's entry one K-step ahead, and the per-instruction work is two additions instead of two divisions and the tests.
    int pre4[WB];
    int t4_pix = 0, t4_pixn = 0;
    int64_t t4_img = 0, t4_imgn = 0;
    if constexpr (GATHERW) {
        const ConvGeom& g = p.conv;
        if (g.pix_table) {                                        // (uniform)
            const int Lp = g.pix_table;
            for (int i = tid; i < Lp + BK; i += 256) {
                const uint32_t oh = fast_div((uint32_t)i, g.div_wo), ow = (uint32_t)i - oh * (uint32_t)g.Wo;
                dw_tab[i] = i < Lp ? (int)((oh * (uint32_t)g.s_r * (uint32_t)g.W + ow * (uint32_t)g.s_c) * (uint32_t)g.chan * (uint32_t)ES) : 0;
            }
            __syncthreads();
            if (g.k_ranges) {
                const uint32_t im0 = fast_div((uint32_t)k4_base, g.div_fold);
                t4_pix = k4_base - (int)im0 * Lp;
                t4_img = (int64_t)im0 * g.fold_stride * ES;
            }
            t4_pixn = t4_pix + BK;
            t4_imgn = t4_img;
            if (g.k_ranges && t4_pixn >= Lp) { t4_pixn -= Lp; t4_imgn += g.fold_stride * ES; }
#pragma unroll
            for (int x = 0; x < WB; ++x) pre4[x] = dw_tab[t4_pix + (krow4[x] & 63)];
        }
    }
    auto conv4_dma = [&](int x, uint32_t lds_tile) __attribute__((always_inline)) {
        if constexpr (GATHERW) {
            const ConvGeom& g = p.conv;
            const char* img = reinterpret_cast<const char*>(B);
            if (g.pix_table) {                                     // (uniform)
                const uint32_t lk = (uint32_t)(k4_k + krow4[x]);
                const char* src = lk < (uint32_t)p.K ? img + (t4_img + (int64_t)(pre4[x] + noff4[x])) : reinterpret_cast<const char*>(ring_zero_word);
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                             :: "s"(lds_tile + (uint32_t)(wave_u * WB + x) * 1024u), "v"(src) : "memory");
                const int pn = t4_pixn < g.pix_table ? t4_pixn : g.pix_table;      // (K-steps past the end: the zeros behind the table)
                pre4[x] = dw_tab[pn + (krow4[x] & 63)];
                if (x == WB - 1) {
                    k4_k += BK;
                    t4_pix = t4_pixn; t4_img = t4_imgn;
                    t4_pixn += BK;
                    if (g.k_ranges && t4_pixn >= g.pix_table) { t4_pixn -= g.pix_table; t4_imgn += g.fold_stride * ES; }
                }
                return;
            }
            const uint32_t lk = (uint32_t)(k4_k + krow4[x]), l = lk + (uint32_t)k4_base;
            uint32_t li = l, im = 0u;
            if (g.fold_L) {                                        // (uniform)
                im = fast_div(l, g.div_fold);
                li = l - im * (uint32_t)g.fold_L;
            }
            const uint32_t oh = fast_div(li, g.div_wo), ow = li - oh * (uint32_t)g.Wo;
            const int ih0 = (int)oh * g.s_r - g.p_r, iw0 = (int)ow * g.s_c - g.p_c;
            const bool ok = (lk < (uint32_t)p.K) & ((uint32_t)(ih0 + (int)(tap4[x] & 0xffffu)) < (uint32_t)g.H) &
                            ((uint32_t)(iw0 + (int)(tap4[x] >> 16)) < (uint32_t)g.W);
            const int off = (int)((oh * (uint32_t)g.s_r * (uint32_t)g.W + ow * (uint32_t)g.s_c) * (uint32_t)g.chan * (uint32_t)ES) + noff4[x];
            const char* src = ok ? img + ((int64_t)im * g.fold_stride * ES + (int64_t)off) : reinterpret_cast<const char*>(ring_zero_word);
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                         :: "s"(lds_tile + (uint32_t)(wave_u * WB + x) * 1024u), "v"(src) : "memory");
            if (x == WB - 1) k4_k += BK;
        }
    };

    // uniform (scalar) source pointer of one operand tile
    auto tile_src = [&](const char* base) __attribute__((always_inline)) -> const void* {
        const uint64_t bu = reinterpret_cast<uint64_t>(base);
        const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)bu);
        const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(bu >> 32));
        return reinterpret_cast<const void*>(((uint64_t)hi << 32) | lo);
    };

    // ---- per-lane LDS read offsets (bytes inside an operand tile), for half-step ks (0, 1) of a K-step ----
    // A lane's fragment of one block is 16 bytes of k: lanes 0..31 hold the first 16 bytes of the half-step of
    // their row, lanes 32..63 the second (8 + 8 consecutive k of 16-bit elements for one 32x32x16 MFMA).
    // Float32: a v_mfma_f32_32x32x2 is, per output element, two fused multiply-adds in a row -- first the k of lanes 0..31,
    // then the k of lanes 32..63 (checked against fmaf chains on the host, bit for bit) -- so the four MFMAs of a half-step
    // multiply k = (0, 1), (2, 3), (4, 5), (6, 7) in that order and every output element is the reference's own chain
    // c = fma(a_k, b_k, c) in ascending k.  Both layouts are therefore read one dword per element, element e = k 2 e + lane / 32
    // (a 16-byte read of a K-major row would hand a lane four consecutive k, and rearranging them with cross-lane moves in the
    // MFMA stream was measured 4 % slower per K-major operand).  The channels-last convolution (CONV = 3 / 5: both operands
    // K-major), whose k runs taps-outermost and so cannot be the reference's order anyway, keeps the 16-byte reads: element e
    // of both operands is k = e (lanes 0..31) | 4 + e (lanes 32..63), the same pairs on both sides.
    // K-major: block b of the wavefront, row = wbase + 32 b + lane%32, slot (2 ks + lane/32) ^ ((row>>1)&3)
    // MN-major, 16-bit: two transposing reads per block; see the header comment
    // MN-major, Float32: four ds_read_b32 per block, element e from k-row 8 ks + 2 e + lane/32
    auto frag_off_km = [&](int wbase, int blk, int ks) -> int {
        const int row = wbase + blk * 32 + (lane & 31);
        if constexpr (KD == 2) return row * 128 + (((2 * ks + (lane >> 5)) ^ swz8(lane & 31)) * 16);   // (wbase + 32 blk is a multiple of 16)
        const int slot = (2 * ks + (lane >> 5)) ^ ((lane >> 1) & 3);
        return row * 64 + slot * 16;
    };
    // (mnrow = bytes of one k-row of the operand's MN-major tile, chunks = 16-byte chunks in it)
    auto frag_off_mm = [&](int mnrow, int wbase, int blk, int ks, int half) -> int {
        const int bl = lane >> 4, s = lane & 15, e = s >> 2, q = s & 3;
        const int krow = 16 * ks + 8 * (bl >> 1) + 4 * half + e;
        const int mnl = wbase + blk * 32 + 16 * (bl & 1) + 4 * q;
        const int chunk = (mnl >> 3) ^ (2 * e);
        return krow * mnrow + chunk * 16 + (mnl & 7) * 2;
    };
    // 8-bit: ds_read_b64_tr_b8 works on groups of 16 lanes; lane i of a group reads the 8 bytes (mn) 8 (i & 1) .. + 7 of
    // k-row i >> 1 and receives, as lane s, the 8 consecutive k of mn s.  Read t (0, 1) of a block covers
    // k = 32 ks + 16 (lane / 32) + 8 t .. + 7 for mn = 32 blk + lane % 32.
    auto frag_off_mm8 = [&](int mnrow, int wbase, int blk, int ks, int t) -> int {
        const int grp = lane >> 4, i = lane & 15;
        const int krow = 32 * ks + 16 * (grp >> 1) + 8 * t + (i >> 1);
        const int mnl = wbase + blk * 32 + 16 * (grp & 1) + 8 * (i & 1);
        const int chunk = (mnl >> 4) ^ (mnrow / 16 >= 8 ? (krow & 7) : ((krow & 7) >> 1));      // mn8_swizzle of the operand
        return krow * mnrow + chunk * 16 + (mnl & 15);
    };
    auto frag_off_mm32 = [&](int mnrow, int wbase, int blk, int ks, int e) -> int {
        const int krow = 8 * ks + 2 * e + (lane >> 5);                    // MFMA e of the half-step multiplies k = 2 e (lanes 0..31) and 2 e + 1
        const int mnl = wbase + blk * 32 + (lane & 31);
        if constexpr (GATHER4) return krow * mnrow + mnl * 4;            // gathered tiles are stored unswizzled
        return krow * mnrow + ((mnl * 4) ^ (128 * (lane >> 5)));      // krow & 1 == lane / 32
    };

    // One LDS read instruction of an operand's fragment set for half-step ks.  A K-major
    // operand takes WB reads (one ds_read_b128 per block), an MN-major one 2 WB (two transposing
    // 8-byte reads per block; Float32: 4 WB four-byte reads); read r lands in frag[r / per_block].
    auto read_op = [&](auto& frag, int mnrow, const char* tile, bool kc, int wbase, int ks, int r) {
        if (kc) {
            if constexpr (ES == 4 && !GATHER16) {
                // Float32 (read r = block r / 4, element e = r % 4): element e is k = 2 e + lane / 32 of the half-step (see above),
                // dword (2 e + lane / 32) % 4 of the 16-byte slot 2 ks + e / 2 of the row
                const int blk = r >> 2, e = r & 3;
                const int row = wbase + blk * 32 + (lane & 31), sw = km_swz<4>(lane & 31);
                frag[blk][e] = *reinterpret_cast<const uint32_t*>(tile + row * 64 + (((2 * ks + (e >> 1)) ^ sw) * 16) + 8 * (e & 1) + 4 * (lane >> 5));
            } else
            frag[r] = *reinterpret_cast<const u32x4*>(tile + frag_off_km(wbase, r, ks));
        } else if constexpr (ES == 4) {
            frag[r >> 2][r & 3] = *reinterpret_cast<const uint32_t*>(tile + frag_off_mm32(mnrow, wbase, r >> 2, ks, r & 3));
        } else if constexpr (ES == 1) {
            const int blk = r >> 1, t = r & 1;
            const intx2v v = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
                (__attribute__((address_space(3))) intx2v*)(tile + frag_off_mm8(mnrow, wbase, blk, ks, t)));
            frag[blk][2 * t] = (uint32_t)v[0];
            frag[blk][2 * t + 1] = (uint32_t)v[1];
        } else {
            const int blk = r >> 1, half = r & 1;
            const shortx4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (__attribute__((address_space(3))) shortx4*)(tile + frag_off_mm(mnrow, wbase, blk, ks, half)));
            typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
            const u32x2 w = __builtin_bit_cast(u32x2, v);
            frag[blk][2 * half] = w[0];
            frag[blk][2 * half + 1] = w[1];
        }
    };
    constexpr int MNRB = ES == 4 ? 4 : 2;                // reads of one block of an MN-major operand per half-step
    constexpr bool KM128 = ES != 4 || GATHER16;          // K-major fragments come in one 16-byte read
    constexpr int NRA = A_KC && KM128 ? WBM : MNRB * WBM, NRB = B_KC && KM128 ? WBN : MNRB * WBN, NR = NRA + NRB;
    constexpr int MPP = ES == 4 ? 4 : 1;                 // MFMAs per pair of fragments
    constexpr int NMMA = WBM * WBN * MPP;                // MFMAs per half-step
    constexpr int RPM = (NR + NMMA - 1) / NMMA;          // LDS reads slotted behind each MFMA

    // K-steps past the end are clamped to the last one: the tail iterations then issue the
    // same DMA traffic as the steady state (into stages nobody reads any more), which keeps
    // the loop body free of branches and the vmcnt bookkeeping uniform.
    // (guarded instantiation: the last k-rows of an M/N-contiguous operand that is read in place may come from a zero-padded copy)
    constexpr bool TAIL_ROWS = RAGGED && CONV == 0;
    auto srcA = [&](int kt) __attribute__((always_inline)) {
        const int kc = kt < last ? kt : last;
        if constexpr (TAIL_ROWS && !A_KC) {
            if (p.tailA && kc * BK >= p.tail_k0)                   // (uniform)
                return tile_src(static_cast<const char*>(p.tailA) + ((int64_t)b * p.s_tailA + (int64_t)(kc * BK - p.tail_k0) * p.lda + m0) * ES);
        }
        if constexpr (GATHERW && A_KC) {
            if (p.conv.a_steps) {                                  // (uniform) K-step counted through the images -> image, step inside it
                const uint32_t gs = (uint32_t)(b * KT + kc), im = fast_div(gs, p.conv.div_a_steps);
                return tile_src(baseA + ((int64_t)im * p.conv.a_image_stride * ES + (int64_t)(gs - im * (uint32_t)p.conv.a_steps) * advA));
            }
        }
        return tile_src(baseA + (int64_t)kc * advA);
    };
    auto srcB = [&](int kt) __attribute__((always_inline)) {
        const int kc = kt < last ? kt : last;
        if constexpr (TAIL_ROWS && !B_KC) {
            if (p.tailB && kc * BK >= p.tail_k0)                   // (uniform)
                return tile_src(static_cast<const char*>(p.tailB) + ((int64_t)b * p.s_tailB + (int64_t)(kc * BK - p.tail_k0) * p.ldb + n0) * ES);
        }
        return tile_src(baseB + (int64_t)kc * advB);
    };

    // prologue: tiles 0..2 and the A half of tile 3 in flight (3 (NA + NB) + NA instructions)
    auto b_tile = [&](int kt, uint32_t lds_tile) __attribute__((always_inline)) {
        if constexpr (GATHER4) conv_tile(lds_tile);        // (tiles past the last one are all zeros; nobody reads them)
        else if constexpr (GATHER16) {
#pragma unroll
            for (int x = 0; x < WB; ++x) conv3_dma(x, lds_tile);
        } else if constexpr (GATHERW) {
#pragma unroll
            for (int x = 0; x < WB; ++x) conv4_dma(x, lds_tile);
        }
        else dma_tile<WBN * KD>(srcB(kt), kt >= last ? offBt : offB, lds_tile, wave_u);
    };
    if constexpr (ES == 4 && std::is_same<AccS, float>::value) {
        if (p.cmode == C_ACCUMULATE || p.cmode == C_BIAS) {
            // The starting values (requested first thing, their latency behind the set-up above) are taken here, before the first
            // DMA instruction is issued: the compiler counts only its own loads, so its wait for them would otherwise stand in
            // front of the first MFMA and cover every DMA load issued since -- the whole fill of the ring instead of the first tile.
#pragma unroll
            for (int i = 0; i < WBM; ++i)
#pragma unroll
                for (int j = 0; j < WBN; ++j) asm volatile("" : "+v"(acc[i][j]));
        }
    }
    dma_tile<NA>(srcA(0), 0 >= last ? offAt : offA, lds_addr_of(st0), wave_u);
    b_tile(0, lds_addr_of(st0) + A_TILE_BYTES);
    dma_tile<NA>(srcA(1), 1 >= last ? offAt : offA, lds_addr_of(st1), wave_u);
    b_tile(1, lds_addr_of(st1) + A_TILE_BYTES);
    // instruction y (A's first, then B's) of this wavefront's share of tile kt, into the stage at lds_stage
    auto tile_dma = [&](int y, int kt, uint32_t lds_stage) __attribute__((always_inline)) {
        const bool tail = RAGGED && kt >= last;
        if (y < NA) dma_1k(srcA(kt), tail ? offAt[y] : offA[y], lds_stage + (uint32_t)(wave_u * NA + y) * 1024u);
        else dma_1k(srcB(kt), tail ? offBt[y - NA] : offB[y - NA], lds_stage + A_TILE_BYTES + (uint32_t)(wave_u * NB + y - NA) * 1024u);
    };
    if constexpr (RING3) {
#pragma unroll
        for (int y = 0; y < (NA + NB) / 2; ++y) tile_dma(y, 2, lds_addr_of(st2));     // first half of tile 2
    } else {
        dma_tile<NA>(srcA(2), 2 >= last ? offAt : offA, lds_addr_of(st2), wave_u);
        b_tile(2, lds_addr_of(st2) + A_TILE_BYTES);
        if constexpr (KD == 1) dma_tile<NA>(srcA(3), 3 >= last ? offAt : offA, lds_addr_of(st3), wave_u);
    }

    constexpr int NBUF = 2 * KD;
    u32x4 af[NBUF][WBM], bf[NBUF][WBN];   // fragment sets: [half-step parity][block]; deep K-steps: [quarter-step][block]

    // all reads of one fragment set, back to back (prologue only)
    auto load_frags = [&](const char* stage, int ks, int buf) {
#pragma unroll
        for (int r = 0; r < NRA; ++r) read_op(af[buf], GA::MN_ROW_BYTES, stage, A_KC, wm * WTM, ks, r);
#pragma unroll
        for (int r = 0; r < NRB; ++r) read_op(bf[buf], G::MN_ROW_BYTES, stage + A_TILE_BYTES, B_KC, wn * WTN, ks, r);
    };
    // The NMMA MFMAs of one half-step on fragment set `cur_buf`, with the NR reads of the next set (stage/ks ->
    // `nxt_buf`) slotted RPM (one; two for the small 16-bit tiles) per MFMA, so LDS latency is
    // always covered by matrix work and only a few reads are outstanding at a time.  The step's DMA
    // instructions (one operand tile's share of this wavefront) are spread over the step as
    // well -- issued in a burst right after the barrier, the four wavefronts would queue up
    // behind the CU's one address unit and stall their MFMA streams.
    // `issue(x)` emits DMA instruction x of the NDMA that this step carries.
    auto mma_step_prefetch = [&](int cur_buf, const char* stage, int ks, int nxt_buf, auto ndma_tag, auto ngather_tag, auto&& issue) __attribute__((always_inline)) {
        constexpr int NDMA = decltype(ndma_tag)::value, NGATHER = decltype(ngather_tag)::value;
#pragma unroll
        for (int q = 0; q < NMMA; ++q) {
            // serpentine order: consecutive MFMAs always share one operand fragment
            const int e = q / (WBM * WBN), pr = q % (WBM * WBN);
            const int i = pr / WBN, j = (i & 1) ? WBN - 1 - (pr % WBN) : (pr % WBN);
            if constexpr (ES != 4) {
                E::mma(acc[i][j], bf[cur_buf][j], af[cur_buf][i]);   // D rows <-> n, cols <-> m
            } else {
                // (copies first: __builtin_bit_cast applied to a vector-element lvalue reads element 0)
                const uint32_t bu = bf[cur_buf][j][e], au = af[cur_buf][i][e];
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(__builtin_bit_cast(float, bu), __builtin_bit_cast(float, au), acc[i][j], 0, 0, 0);
            }
#pragma unroll
            for (int r = q * RPM; r < (q + 1) * RPM; ++r) {
                if (r < NRA) read_op(af[nxt_buf], GA::MN_ROW_BYTES, stage, A_KC, wm * WTM, ks, r);
                else if (r < NR) read_op(bf[nxt_buf], G::MN_ROW_BYTES, stage + A_TILE_BYTES, B_KC, wn * WTN, ks, r - NRA);
            }
            constexpr int DGAP = NMMA >= NDMA ? NMMA / NDMA : 1, DPER = NMMA >= NDMA ? 1 : NDMA / NMMA;   // MFMAs between two DMA instructions / DMA instructions per MFMA
            if (q % DGAP == DGAP - 1) {
#pragma unroll
                for (int x = 0; x < DPER; ++x)
                    if ((q / DGAP) * DPER + x < NDMA) issue((q / DGAP) * DPER + x);
            }
        }
#pragma unroll
        for (int q = 0; q < NMMA; ++q) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);               // one MFMA
            const int nrd = NR - q * RPM < RPM ? NR - q * RPM : RPM;
            if (nrd == 4) __builtin_amdgcn_sched_group_barrier(0x100, 4, 0); // its LDS reads
            else if (nrd == 3) __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);
            else if (nrd == 2) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
            else if (nrd == 1) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            if constexpr (NGATHER > 0) {
                // the gather's address arithmetic, dealt out evenly: what does not fit under one MFMA delays the next
                constexpr int VPG = GATHERW ? 20 : 8;          // vector instructions per gathering DMA, roughly
                __builtin_amdgcn_sched_group_barrier(0x002, (VPG * NGATHER + NMMA - 1) / NMMA + 1, 0);   // VALU
                __builtin_amdgcn_sched_group_barrier(0x004, (10 * NGATHER + NMMA - 1) / NMMA, 0);      // SALU
            }
        }
    };

    // tile 0 must have landed before its first fragments are read
    NTG_WAIT_VMCNT(RING3 ? (NA + NB) + (NA + NB) / 2 : 2 * (NA + NB) + (KD == 1 ? NA : 0));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    load_frags(st0, 0, 0);
    if constexpr (KD == 2) load_frags(st0, 1, 1);

    // One K-step.  `cur` holds tile kt (its half-step 0 fragments are already in registers),
    // `nxt` holds tile kt+1, `prv` held tile kt-1.  The single barrier sits between the two
    // half-steps: by then every wavefront has issued and received its last reads of `cur`, so
    // the stage goes back to the DMA at once: the A half of tile kt+4 is fetched during the
    // second half-step, its B half during the first half-step of the next K-step.  Tile kt+1,
    // first touched in the second half, has had three K-steps to arrive.
    // RAGGED: zero the k >= K part of a fragment set of the last K-step.  Every lane's fragment
    // covers one chunk of consecutive k (8 or 4) starting at (32 bytes) ks + (16 bytes) (lane / 32) in both
    // LDS layouts, and K is a multiple of the chunk, so a lane's fragment is either entirely real or
    // entirely past the end.
    // (Float32: element e of a fragment is k = 2 e + lane / 32 of the half-step in both layouts; the channels-last convolution keeps
    //  the 16-byte fragments: k 0..3 | k 4..7)
    auto mask_tail = [&](int buf, int ks) {
        const bool ok = (32 / ES) * ks + (16 / ES) * (lane >> 5) < kr;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const bool oke = 8 * ks + 2 * e + (lane >> 5) < kr;
            const bool oka = ES == 4 && !GATHER16 ? oke : ok, okb = ES == 4 && !GATHER16 ? oke : ok;
#pragma unroll
            for (int i = 0; i < WBM; ++i) af[buf][i][e] = oka ? af[buf][i][e] : 0u;
#pragma unroll
            for (int j = 0; j < WBN; ++j) bf[buf][j][e] = okb ? bf[buf][j][e] : 0u;
        }
    };

    // (inlined by force: as a call, the stage pointers would arrive in vector registers and could not feed M0)
    auto iteration = [&](int kt, char* cur, const char* nxt, char* prv) __attribute__((always_inline)) {
        if (RAGGED && kt == last && kr < BK) mask_tail(0, 0);
        {
            const void* src = nullptr;
            if constexpr (CONV == 0) src = srcB(kt + 3);
            const bool tail = kt + 3 >= last;
            const uint32_t lds_tile = lds_addr_of(prv) + A_TILE_BYTES;
            mma_step_prefetch(0, cur, 1, 1, std::integral_constant<int, NB1>{}, std::integral_constant<int, (CONV ? NB1 : 0)>{},
                              [&](int x) __attribute__((always_inline)) {
                if constexpr (GATHER4) conv_dma(x, lds_tile);
                else if constexpr (GATHER16) conv3_dma(x, lds_tile);
                else if constexpr (GATHERW) conv4_dma(x, lds_tile);
                else dma_1k(src, (RAGGED && tail) ? offBt[x] : offB[x], lds_tile + (uint32_t)(wave_u * WB + x) * 1024u);
            });
        }
        // issued since the last instruction of tile kt+1: A(kt+2), B(kt+2), A(kt+3) and the first NB1 of B(kt+3)
        NTG_WAIT_VMCNT(2 * (NA + NB) - NB2);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // my reads of `cur` are complete
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (RAGGED && kt == last && kr < BK) mask_tail(1, 1);
        // (the last K-step prefetches fragments from a stage holding a clamped tile; unused)
        {
            const void* src = srcA(kt + 4);
            const bool tail = kt + 4 >= last;
            const uint32_t lds_tile = lds_addr_of(cur), lds_gather = lds_addr_of(prv) + A_TILE_BYTES;
            mma_step_prefetch(1, nxt, 0, 0, std::integral_constant<int, NB2 + NA>{}, std::integral_constant<int, NB2>{},
                              [&](int x) __attribute__((always_inline)) {
                if (x < NB2) conv_dma(NB1 + x, lds_gather);       // rest of B(kt+3)
                else dma_1k(src, (RAGGED && tail) ? offAt[x - NB2] : offA[x - NB2], lds_tile + (uint32_t)(wave_u * WBM + x - NB2) * 1024u);
            });
        }
    };

    // One deep K-step (KD = 2): four quarter-steps, fragment set q holding quarter-step q.  Sets 0 and 1 of tile kt are in
    // registers on entry; quarter-steps 0 and 1 read sets 2 and 3 from `cur`, then the barrier (every wavefront is done
    // with `cur`, which the next K-step refills, and tile kt + 1 has landed), and quarter-steps 2 and 3 read sets 0 and 1 of
    // `nxt`.  `prv` went back to the DMA at the previous K-step's barrier: the whole of tile kt + 3 is fetched into it, a
    // quarter of the instructions per quarter-step.
    auto iteration_deep = [&](int kt, char* cur, const char* nxt, char* prv) __attribute__((always_inline)) {
      if constexpr (KD == 2) {
        static_assert((NA + NB) % 4 == 0, "a quarter of the tile's DMA instructions per quarter-step");
        constexpr int PER = (NA + NB) / 4;
        const bool lastk = RAGGED && kt == last && kr < BK;
        const void* sa = srcA(kt + 3);
        const void* sb = srcB(kt + 3);
        const bool tail = kt + 3 >= last;
        const uint32_t lds_a = lds_addr_of(prv), lds_b = lds_addr_of(prv) + A_TILE_BYTES;
        auto issue_at = [&](int y) __attribute__((always_inline)) {
            if (y < NA) dma_1k(sa, (RAGGED && tail) ? offAt[y] : offA[y], lds_a + (uint32_t)(wave_u * NA + y) * 1024u);
            else dma_1k(sb, (RAGGED && tail) ? offBt[y - NA] : offB[y - NA], lds_b + (uint32_t)(wave_u * NB + y - NA) * 1024u);
        };
        using NP = std::integral_constant<int, PER>;
        using N0 = std::integral_constant<int, 0>;
        if (lastk) mask_tail(0, 0);
        mma_step_prefetch(0, cur, 2, 2, NP{}, N0{}, [&](int x) __attribute__((always_inline)) { issue_at(x); });
        if (lastk) mask_tail(1, 1);
        mma_step_prefetch(1, cur, 3, 3, NP{}, N0{}, [&](int x) __attribute__((always_inline)) { issue_at(PER + x); });
        // issued since the last instruction of tile kt+1: tile kt+2 and half of tile kt+3
        NTG_WAIT_VMCNT((NA + NB) + 2 * PER);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // my reads of `cur` are complete
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (lastk) mask_tail(2, 2);
        mma_step_prefetch(2, nxt, 0, 0, NP{}, N0{}, [&](int x) __attribute__((always_inline)) { issue_at(2 * PER + x); });
        if (lastk) mask_tail(3, 3);
        mma_step_prefetch(3, nxt, 1, 1, NP{}, N0{}, [&](int x) __attribute__((always_inline)) { issue_at(3 * PER + x); });
      }
    };

    // ... with three stages: `prv` (tile kt - 1's) takes the second half of tile kt + 2 during quarter-steps 0 and 1, `cur` the
    // first half of tile kt + 3 after the barrier.  Tile kt + 1 has landed at the barrier when at most the instructions of
    // tile kt + 2 are outstanding.
    auto iteration_deep3 = [&](int kt, char* cur, const char* nxt, char* prv) __attribute__((always_inline)) {
      if constexpr (RING3) {
        static_assert((NA + NB) % 4 == 0, "a quarter of the tile's DMA instructions per quarter-step");
        constexpr int PER = (NA + NB) / 4;
        const bool lastk = RAGGED && kt == last && kr < BK;
        const uint32_t lds_prv = lds_addr_of(prv), lds_cur = lds_addr_of(cur);
        using NP = std::integral_constant<int, PER>;
        using N0 = std::integral_constant<int, 0>;
        if (lastk) mask_tail(0, 0);
        mma_step_prefetch(0, cur, 2, 2, NP{}, N0{}, [&](int x) __attribute__((always_inline)) { tile_dma(2 * PER + x, kt + 2, lds_prv); });
        if (lastk) mask_tail(1, 1);
        mma_step_prefetch(1, cur, 3, 3, NP{}, N0{}, [&](int x) __attribute__((always_inline)) { tile_dma(3 * PER + x, kt + 2, lds_prv); });
        NTG_WAIT_VMCNT(NA + NB);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // my reads of `cur` are complete
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (lastk) mask_tail(2, 2);
        mma_step_prefetch(2, nxt, 0, 0, NP{}, N0{}, [&](int x) __attribute__((always_inline)) { tile_dma(x, kt + 3, lds_cur); });
        if (lastk) mask_tail(3, 3);
        mma_step_prefetch(3, nxt, 1, 1, NP{}, N0{}, [&](int x) __attribute__((always_inline)) { tile_dma(PER + x, kt + 3, lds_cur); });
      }
    };

    if constexpr (RING3) {
        for (int kt = 0; kt < KT; kt += 3) {
            iteration_deep3(kt, st0, st1, st2);
            if (kt + 1 < KT) iteration_deep3(kt + 1, st1, st2, st0);
            if (kt + 2 < KT) iteration_deep3(kt + 2, st2, st0, st1);
        }
    } else
    for (int kt = 0; kt < KT; kt += 4) {
        if constexpr (KD == 2) {
            iteration_deep(kt, st0, st1, st3);
            if (kt + 1 < KT) iteration_deep(kt + 1, st1, st2, st0);
            if (kt + 2 < KT) iteration_deep(kt + 2, st2, st3, st1);
            if (kt + 3 < KT) iteration_deep(kt + 3, st3, st0, st2);
        } else {
            iteration(kt, st0, st1, st3);
            if (kt + 1 < KT) iteration(kt + 1, st1, st2, st0);
            if (kt + 2 < KT) iteration(kt + 2, st2, st3, st1);
            if (kt + 3 < KT) iteration(kt + 3, st3, st0, st2);
        }
    }
    NTG_WAIT_VMCNT(0);              // clamped tail DMAs have landed
    __builtin_amdgcn_s_barrier();   // all fragment reads done: LDS is free for the epilogue
    asm volatile("" ::: "memory");

    // ---- epilogue: per wavefront, WB 32-row slabs through a private fp32 LDS region ----
    // 32 rows x SROW bytes (the wavefront's WTN columns in fp32) per wavefront; 16-byte slot s of
    // row r lives at s ^ (r & 7).  LPR lanes cover a row (8 columns each), so one step of the
    // read-back moves RPS rows.
    constexpr int SROW = WTN * 4, LPR = WTN / 8, RPS = 64 / LPR, NSTEP = 32 / RPS;
    // (two slabs fit into one stage unless the tile is wider than tall: then every wavefront takes a stage of its own)
    // (three stages of 48 KiB: three 16-KiB slabs in the first, the fourth in the second)
    char* slab = RING3 ? (wave == 3 ? st1 : st0 + wave * (32 * SROW))
               : WBN > WBM ? (wave == 0 ? st0 : wave == 1 ? st1 : wave == 2 ? st2 : st3)
                           : ((wave & 2) ? st1 : st0) + (wave & 1) * (32 * SROW);
    // (C and the bias through pointers into global memory: as FLAT instructions their loads and stores would count as LDS
    //  operations too, and every wait for a slab read would wait for the stores of the slab before it)
    NTG_GLOBAL char* Cb = (NTG_GLOBAL char*)reinterpret_cast<char*>(C);
    const int col = 8 * (lane % LPR);              // this lane's 8 consecutive columns in the slab
    const int n = n0 + wn * WTN + col;
    constexpr int NV = ES == 4 ? 2 : 1;            // 16-byte vectors of C per lane and row: 8 columns of 1 (half a vector), 2 or 4 bytes
    // (only the channels-last convolution meets rows of C that are not 16-byte multiples; uniform)
    const bool c_rows_16 = !GATHER16 || (p.ldc % G::VEL == 0 && p.sC % G::VEL == 0 && (reinterpret_cast<uintptr_t>(p.C) & 15) == 0);
    typedef AccS accx4 __attribute__((ext_vector_type(4)));
    typedef uint32_t u32x2v __attribute__((ext_vector_type(2)));
    // (uniform) the bias is contiguous along the columns and every lane's 8 values start on a 16-byte boundary
    const bool bias_rows_16 = ES != 1 && p.bias && p.bias_cs == 1 && p.bias_rs % G::VEL == 0 && p.bias_bs % G::VEL == 0 &&
                              (reinterpret_cast<uintptr_t>(p.bias) & 15) == 0;
    auto epilogue = [&](auto cmode_tag) {
        constexpr int CM = decltype(cmode_tag)::value;
        const NTG_GLOBAL T* bias = (const NTG_GLOBAL T*)static_cast<const T*>(p.bias);
        // one bias row for every row of C (cpu::linear's [n] vector): the lane's 8 columns never change, one load for the whole tile
        AccS bias_row[8] = {};
        const bool bias_row_const = CM == C_BIAS && bias_rows_16 && p.bias_rs == 0 && (!RAGGED || n + 8 <= p.N);
        if constexpr (CM == C_BIAS && ES != 1) {
            if (bias_row_const) {
                const NTG_GLOBAL T* bp = bias + (int64_t)b * p.bias_bs + (int64_t)n;
                if constexpr (ES == 2) {
                    const u32x4 bv = *(const NTG_GLOBAL u32x4*)bp;
#pragma unroll
                    for (int e = 0; e < 8; ++e) bias_row[e] = Cvt16<DT>::up((uint16_t)(bv[e >> 1] >> (16 * (e & 1))));
                } else {
                    const accx4 b0 = *(const NTG_GLOBAL accx4*)bp, b1 = *(const NTG_GLOBAL accx4*)(bp + 4);
#pragma unroll
                    for (int e = 0; e < 4; ++e) { bias_row[e] = b0[e]; bias_row[4 + e] = b1[e]; }
                }
            }
        }
        // C0 of a whole slab is requested one slab ahead: the loads of slab i + 1 are in flight while slab i goes through LDS
        // and out to memory (the rows of two slabs are different rows of C, but the compiler cannot know that and would
        // keep every load behind the stores before it).
        u32x4 c0s[2][NSTEP][NV];
        auto load_c0 = [&](int i, u32x4 (&c0)[NSTEP][NV]) __attribute__((always_inline)) {
            if constexpr (CM == C_ACCUMULATE) {
#pragma unroll
                for (int t = 0; t < NSTEP && c_rows_16; ++t) {
                    const int m = m0 + wm * WTM + 32 * i + RPS * t + lane / LPR;
#pragma unroll
                    for (int v = 0; v < NV; ++v) {
                        if (!RAGGED || (m < p.M && n + 4 * v < p.N)) {
                            if constexpr (ES == 1) {
                                const u32x2v c8 = *(const NTG_GLOBAL u32x2v*)(Cb + (int64_t)m * p.ldc + n);
                                c0[t][v] = u32x4{c8[0], c8[1], 0u, 0u};
                            } else {
                                c0[t][v] = *(const NTG_GLOBAL u32x4*)(Cb + ((int64_t)m * p.ldc + n) * ES + 16 * v);
                            }
                        } else c0[t][v] = u32x4{0u, 0u, 0u, 0u};
                    }
                }
            }
        };
        load_c0(0, c0s[0]);
#pragma unroll
        for (int i = 0; i < WBM; ++i) {
            u32x4 (&c0)[NSTEP][NV] = c0s[i & 1];
            if (i + 1 < WBM) load_c0(i + 1, c0s[(i + 1) & 1]);
            // lane holds rows m = 32 i + lane%32, cols 32 j + 8 rq + 4 (lane/32) + (0..3)
#pragma unroll
            for (int j = 0; j < WBN; ++j)
#pragma unroll
                for (int rq = 0; rq < 4; ++rq) {
                    accx4 v = {acc[i][j][4 * rq], acc[i][j][4 * rq + 1], acc[i][j][4 * rq + 2], acc[i][j][4 * rq + 3]};
                    const int slot = 8 * j + 2 * rq + (lane >> 5);
                    *reinterpret_cast<accx4*>(slab + (lane & 31) * SROW + ((slot ^ (lane & 7)) * 16)) = v;
                }
            // 32 rows x WTN cols: NSTEP steps of RPS rows; a lane owns 8 consecutive columns
#pragma unroll
            for (int t = 0; t < NSTEP; ++t) {
                const int row = RPS * t + lane / LPR;
                const int sl = 2 * (lane % LPR);
                const accx4 lo = *reinterpret_cast<const accx4*>(slab + row * SROW + ((sl ^ (row & 7)) * 16));
                const accx4 hi = *reinterpret_cast<const accx4*>(slab + row * SROW + (((sl + 1) ^ (row & 7)) * 16));
                AccS v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
                const int m = m0 + wm * WTM + 32 * i + row;
                // 16-bit: N % 8 == 0, a lane's 8 columns exist or not together; Float32: N % 4 == 0, the halves separately
                if (RAGGED && (m >= p.M || n >= p.N)) continue;
                if constexpr (GATHER16) {
                    // output planes whose rows are not 16-byte multiples (Ho*Wo = 49, 900, ...): element-wise stores
                    if (!c_rows_16) {
                        NTG_GLOBAL T* ce = (NTG_GLOBAL T*)Cb + (int64_t)m * p.ldc + n;
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            if (n + e >= p.N) break;
                            AccS val = v[e];
                            if constexpr (CM == C_ACCUMULATE) val += (AccS)ce[e];
                            else if constexpr (CM == C_BIAS) val += (AccS)bias[(int64_t)b * p.bias_bs + (int64_t)m * p.bias_rs + (int64_t)(n + e) * p.bias_cs];
                            ce[e] = (T)val;
                        }
                        continue;
                    }
                }
                const bool hi_ok = !RAGGED || ES != 4 || n + 4 < p.N;
                if constexpr (CM == C_PARTIAL) {
                    // split-K: the fp32 sums of this k range go to a float matrix; rounding happens after the reduction
                    // (8-bit operands: the 32-bit integer sums, for the byte-plane form of the wider integer products)
                    NTG_GLOBAL float* wp = (NTG_GLOBAL float*)static_cast<float*>(p.C) + (int64_t)b * p.sC + (int64_t)m * p.ldc + n;
                    *(NTG_GLOBAL accx4*)wp = lo;
                    if (hi_ok) *(NTG_GLOBAL accx4*)(wp + 4) = hi;
                    continue;
                }
                if constexpr (CM == C_ACCUMULATE) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        if constexpr (ES == 2) v[e] += Cvt16<DT>::up((uint16_t)(c0[t][0][e >> 1] >> (16 * (e & 1))));
                        else if constexpr (ES == 1) v[e] += (int)((c0[t][0][e >> 2] >> (8 * (e & 3))) & 0xffu);
                        else { const uint32_t cu = c0[t][e >> 2][e & 3]; v[e] += __builtin_bit_cast(float, cu); }
                    }
                } else if constexpr (CM == C_BIAS) {
                    const NTG_GLOBAL T* bp = bias + (int64_t)b * p.bias_bs + (int64_t)m * p.bias_rs + (int64_t)n * p.bias_cs;
                    if (bias_row_const) {
#pragma unroll
                        for (int e = 0; e < 8; ++e) v[e] += bias_row[e];
                    } else if (bias_rows_16 && (ES != 4 || hi_ok)) {
                        // a bias that runs along the columns (cpu::linear's [n] vector): the lane's 8 values in 16-byte loads
                        if constexpr (ES == 2) {
                            const u32x4 bv = *(const NTG_GLOBAL u32x4*)bp;
#pragma unroll
                            for (int e = 0; e < 8; ++e) v[e] += Cvt16<DT>::up((uint16_t)(bv[e >> 1] >> (16 * (e & 1))));
                        } else if constexpr (ES == 4) {
                            const accx4 b0 = *(const NTG_GLOBAL accx4*)bp, b1 = *(const NTG_GLOBAL accx4*)(bp + 4);
#pragma unroll
                            for (int e = 0; e < 4; ++e) { v[e] += b0[e]; v[4 + e] += b1[e]; }
                        }
                    } else {
#pragma unroll
                        for (int e = 0; e < 8; ++e)
                            if (ES != 4 || e < 4 || hi_ok) v[e] += (AccS)bp[(int64_t)e * p.bias_cs];
                    }
                }
                if constexpr (ES != 1) {
                    if (p.act == ACT_RELU) {                   // (uniform) relu_ on the result before its one rounding: the same bits
#pragma unroll
                        for (int e = 0; e < 8; ++e) v[e] = v[e] > (AccS)0 ? v[e] : (AccS)0;
                    }
                }
                NTG_GLOBAL char* cp = Cb + ((int64_t)m * p.ldc + n) * ES;
                if constexpr (ES == 2) {
                    u32x4 o;
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        o[e] = (uint32_t)Cvt16<DT>::down(v[2 * e]) | ((uint32_t)Cvt16<DT>::down(v[2 * e + 1]) << 16);
                    *(NTG_GLOBAL u32x4*)cp = o;
                } else if constexpr (ES == 1) {
                    u32x2v o;                       // the low 8 bits of each sum: wrapping arithmetic in the element type
#pragma unroll
                    for (int h = 0; h < 2; ++h)
                        o[h] = ((uint32_t)v[4 * h] & 0xffu) | (((uint32_t)v[4 * h + 1] & 0xffu) << 8) |
                               (((uint32_t)v[4 * h + 2] & 0xffu) << 16) | ((uint32_t)v[4 * h + 3] << 24);
                    *(NTG_GLOBAL u32x2v*)cp = o;
                } else {
                    *(NTG_GLOBAL accx4*)cp = accx4{v[0], v[1], v[2], v[3]};
                    if (hi_ok) *(NTG_GLOBAL accx4*)(cp + 16) = accx4{v[4], v[5], v[6], v[7]};
                }
            }
        }
    };
    if constexpr (ES == 4 && std::is_same<AccS, float>::value) {
        // (C0 or the bias went into the accumulators before the K loop)
        if (p.cmode == C_PARTIAL) epilogue(std::integral_constant<int, C_PARTIAL>{});
        else epilogue(std::integral_constant<int, C_OVERWRITE>{});
    } else {
        if (p.cmode == C_ACCUMULATE) epilogue(std::integral_constant<int, C_ACCUMULATE>{});
        else if (p.cmode == C_PARTIAL) epilogue(std::integral_constant<int, C_PARTIAL>{});
        else if (p.cmode == C_BIAS) epilogue(std::integral_constant<int, C_BIAS>{});
        else epilogue(std::integral_constant<int, C_OVERWRITE>{});
    }
}

// true when the fast kernel can serve the problem: 16-byte aligned rows everywhere (leading
// dimensions, batch strides, base pointers) and every contiguous extent a multiple of one 16-byte
// chunk (es = element size: 8 or 4 elements).  M, N and K themselves may be ragged with respect
// to the tile.  Per-lane DMA offsets are 32-bit: 256 rows of lda elements must stay below 4 GiB.
// Pointer tables qualify when the caller vouches for the entries' alignment (p.ptrs_aligned).
static inline bool ring_eligible(const GemmParams& p, bool ta, int es = 2) {
    const int vel = 16 / es;
    const int64_t ldmax = (int64_t)(1 << 23) / es;
    return p.K >= vel && p.K % vel == 0 && p.N % vel == 0 && (!ta || p.M % vel == 0) &&
           ((!p.Aptr && !p.Bptr && !p.Cptr) || (p.ptrs_aligned && p.Aptr && p.Bptr && p.Cptr && p.cmode != C_PARTIAL)) && p.vecA_ok && p.vecB_ok &&
           p.ldc % vel == 0 && (p.Cptr || p.sC % vel == 0) && p.lda < ldmax && p.ldb < ldmax &&
           ((reinterpret_cast<uintptr_t>(p.A) & 15) == 0) && ((reinterpret_cast<uintptr_t>(p.B) & 15) == 0) &&
           ((reinterpret_cast<uintptr_t>(p.C) & 15) == 0);
}

// Measurement knob (read once): NTG_TILE_GROUP_M = g makes groups of g tile rows instead of 4 in the tile order of the plain
// products (with 32 CUs per XCD: 4 -> every XCD works on 4 x 8 tiles at a time, 2 -> 2 x 16, 8 -> 8 x 4 ...); a negative
// value also deals the workgroups to the XCDs round-robin as the hardware numbers them.  Results do not depend on it.
static inline int ring_tile_order_override() {
    static const int v = [] { const char* e = getenv("NTG_TILE_GROUP_M"); return e ? atoi(e) : 0; }();
    return v;
}

// WBN != 0: rectangular tiles of 64 WB rows x 64 WBN columns
template <int DT, bool TA, bool TB, int WB, int WBN = 0, int KD = 1>
static hipError_t launch_ring_cfg(const GemmParams& pin, hipStream_t s) {
    constexpr int ES = (int)sizeof(typename Elem<DT>::T);
    constexpr int TEM = RingGeom<WB, ES>::BM, TEN = RingGeom<(WBN ? WBN : WB), ES>::BM, BK = RingGeom<WB, ES, KD>::BK;
    GemmParams p = pin;
    p.tiles_m = (p.M + TEM - 1) / TEM;
    p.tiles_n = (p.N + TEN - 1) / TEN;
    p.group_m = ring_tile_order_override();
    const int64_t blocks = (int64_t)p.tiles_m * p.tiles_n * p.batch;
    if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
    if (p.M % TEM == 0 && p.N % TEN == 0 && p.K % BK == 0 && !p.tailA && !p.tailB)      // (copied tail rows: the guarded instantiation reads them)
        hipLaunchKernelGGL((gemm_ring_kernel<DT, TA, TB, false, WB, 0, WBN, KD>), dim3((unsigned)blocks), dim3(256), 0, s, p);
    else
        hipLaunchKernelGGL((gemm_ring_kernel<DT, TA, TB, true, WB, 0, WBN, KD>), dim3((unsigned)blocks), dim3(256), 0, s, p);
    return hipGetLastError();
}

// convolution (tb = false) or weight gradient (tb = true) with op(B) gathered from the image; Float32, two spatial axes
template <int WB>
static hipError_t launch_ring_conv_cfg(bool tb, const GemmParams& pin, hipStream_t s) {
    constexpr int TE = RingGeom<WB, 4>::BM;
    GemmParams p = pin;
    p.tiles_m = (p.M + TE - 1) / TE;
    p.tiles_n = (p.N + TE - 1) / TE;
    const int64_t blocks = (int64_t)p.tiles_m * p.tiles_n * p.batch;
    if (blocks <= 0) return hipSuccess;
    if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
    if (tb) hipLaunchKernelGGL((gemm_ring_kernel<DT_F32, false, false, true, WB, 2>), dim3((unsigned)blocks), dim3(256), 0, s, p);
    else hipLaunchKernelGGL((gemm_ring_kernel<DT_F32, false, false, true, WB, 1>), dim3((unsigned)blocks), dim3(256), 0, s, p);
    return hipGetLastError();
}

// ... from a channels-last image that carries its padding as zero pixels (CONV = 5)
template <int DT, int WB>
static hipError_t launch_ring_nhwc_halo_cfg(const GemmParams& pin, hipStream_t s) {
    constexpr int TE = RingGeom<WB, (int)sizeof(typename Elem<DT>::T)>::BM;
    GemmParams p = pin;
    p.tiles_m = (p.M + TE - 1) / TE;
    p.tiles_n = (p.N + TE - 1) / TE;
    const int64_t blocks = (int64_t)p.tiles_m * p.tiles_n * p.batch;
    if (blocks <= 0) return hipSuccess;
    if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
    hipLaunchKernelGGL((gemm_ring_kernel<DT, false, true, true, WB, 5>), dim3((unsigned)blocks), dim3(256), 0, s, p);
    return hipGetLastError();
}

// convolution with op(B) gathered in 16-byte pieces from a channels-last image (see CONV = 3)
template <int DT, int WB>
static hipError_t launch_ring_nhwc_cfg(const GemmParams& pin, hipStream_t s) {
    if (pin.conv.halo) return launch_ring_nhwc_halo_cfg<DT, WB>(pin, s);
    constexpr int TE = RingGeom<WB, (int)sizeof(typename Elem<DT>::T)>::BM;
    GemmParams p = pin;
    p.tiles_m = (p.M + TE - 1) / TE;
    p.tiles_n = (p.N + TE - 1) / TE;
    const int64_t blocks = (int64_t)p.tiles_m * p.tiles_n * p.batch;
    if (blocks <= 0) return hipSuccess;
    if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
    hipLaunchKernelGGL((gemm_ring_kernel<DT, false, true, true, WB, 3>), dim3((unsigned)blocks), dim3(256), 0, s, p);
    return hipGetLastError();
}

// weight gradient of a convolution with op(B) gathered from a channels-last image (see CONV = 4)
template <int DT, int WB, bool TA = false>
static hipError_t launch_ring_nhwc_dw_cfg(const GemmParams& pin, hipStream_t s) {
    constexpr int TE = RingGeom<WB, (int)sizeof(typename Elem<DT>::T)>::BM;
    GemmParams p = pin;
    p.tiles_m = (p.M + TE - 1) / TE;
    p.tiles_n = (p.N + TE - 1) / TE;
    const int64_t blocks = (int64_t)p.tiles_m * p.tiles_n * p.batch;
    if (blocks <= 0) return hipSuccess;
    if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
    // (more output pixels per image than the table holds: the divisions per instruction, which serve a bordered copy as well)
    if (p.conv.pix_table + 64 > dw_table_entries(WB)) p.conv.pix_table = 0;
    hipLaunchKernelGGL((gemm_ring_kernel<DT, TA, false, true, WB, 4>), dim3((unsigned)blocks), dim3(256), 0, s, p);
    return hipGetLastError();
}

template <int DT, int WB, int WBN = 0, int KD = 1>
static hipError_t launch_ring_wb(bool ta, bool tb, const GemmParams& p, hipStream_t s) {
    if (ta) return tb ? launch_ring_cfg<DT, true, true, WB, WBN, KD>(p, s) : launch_ring_cfg<DT, true, false, WB, WBN, KD>(p, s);
    return tb ? launch_ring_cfg<DT, false, true, WB, WBN, KD>(p, s) : launch_ring_cfg<DT, false, false, WB, WBN, KD>(p, s);
}

// items [b0, b0 + nb) of a strided batch as a product of their own
static inline GemmParams ring_batch_range(const GemmParams& p, int64_t es, int b0, int nb) {
    GemmParams q = p;
    q.A = static_cast<const char*>(p.A) + (int64_t)b0 * p.sA * es;
    q.B = static_cast<const char*>(p.B) + (int64_t)b0 * p.sB * es;
    q.C = static_cast<char*>(p.C) + (int64_t)b0 * p.sC * es;
    if (p.bias) q.bias = static_cast<const char*>(p.bias) + (int64_t)b0 * p.bias_bs * es;
    if (p.tailA) q.tailA = static_cast<const char*>(p.tailA) + (int64_t)b0 * p.s_tailA * es;
    if (p.tailB) q.tailB = static_cast<const char*>(p.tailB) + (int64_t)b0 * p.s_tailB * es;
    q.batch = nb;
    return q;
}

// 16-bit products: tile edge from the cost estimate; a batch that leaves a small rest of tiles after whole rounds
// over the CUs goes out as two launches (see ring16_plan).  launch(edge, params) starts one of them.
template <class Launch>
static hipError_t launch_ring16_planned(const GemmParams& p, hipStream_t s, Launch&& launch, int rect = RECT_NONE) {
    Ring16Plan pl = ring16_plan(p.M, p.N, p.K, p.batch, rect);
    if (p.cmode == C_PARTIAL || p.Aptr || p.Bptr || p.Cptr) pl.head = p.batch;
    if (pl.head >= p.batch) return launch(pl.edge, p);
    const hipError_t e = launch(pl.edge, ring_batch_range(p, 2, 0, pl.head));
    if (e != hipSuccess) return e;
    return launch(pl.tail_edge, ring_batch_range(p, 2, pl.head, p.batch - pl.head));
}

// channels-last convolution and weight gradient, 16-bit: the leading columns of every item, then the remaining ones on a tile
// of their own (see ring16_column_split); each part planned over the batch like any other
template <class Launch>
static hipError_t launch_conv_nhwc16_planned(const GemmParams& p, hipStream_t s, Launch&& launch) {
    if (p.conv.k_ranges) return launch(ring16_tile_edge(p.M, p.N, p.K, p.batch), p);     // items are k ranges: one launch, planned by the caller
    const int64_t head_cols = p.cmode == C_PARTIAL ? 0 : ring16_column_split(p.M, p.N, p.K, p.batch);
    if (head_cols == 0) return launch_ring16_planned(p, s, launch);
    GemmParams head = p, tail = p;
    head.N = (int)head_cols;
    tail.N = p.N - (int)head_cols;
    tail.conv.n_base = p.conv.n_base + (int)head_cols;
    head.conv.n_total = tail.conv.n_total = p.conv.n_total ? p.conv.n_total : p.N;
    tail.C = static_cast<char*>(p.C) + head_cols * 2;
    if (p.bias) tail.bias = static_cast<const char*>(p.bias) + head_cols * p.bias_cs * 2;
    const hipError_t e = launch_ring16_planned(head, s, launch);
    if (e != hipSuccess) return e;
    return launch_ring16_planned(tail, s, launch);
}

// the two sub-products of a split single product (see ring16_split): leading columns / rows, then the remaining strip
static inline void ring_split_params(const GemmParams& p, bool ta, bool tb, int64_t es, const Ring16Split& sp, GemmParams& head, GemmParams& tail) {
    head = p;
    tail = p;
    const char* A = static_cast<const char*>(p.A);
    const char* B = static_cast<const char*>(p.B);
    char* C = static_cast<char*>(p.C);
    const char* bias = static_cast<const char*>(p.bias);
    if (sp.axis == 1) {                          // columns [0, head) | [head, N)
        head.N = (int)sp.head;
        tail.N = p.N - (int)sp.head;
        tail.B = B + (tb ? sp.head * p.ldb : sp.head) * es;
        if (p.tailB) tail.tailB = static_cast<const char*>(p.tailB) + sp.head * es;       // (copied k-rows exist for B stored [k][n] only)
        tail.C = C + sp.head * es;
        if (bias) tail.bias = bias + sp.head * p.bias_cs * es;
    } else {                                     // rows [0, head) | [head, M)
        head.M = (int)sp.head;
        tail.M = p.M - (int)sp.head;
        tail.A = A + (ta ? sp.head : sp.head * p.lda) * es;
        if (p.tailA) tail.tailA = static_cast<const char*>(p.tailA) + sp.head * es;       // (... for A stored [k][m] only)
        tail.C = C + sp.head * p.ldc * es;
        if (bias) tail.bias = bias + sp.head * p.bias_rs * es;
    }
}

template <int DT>
static hipError_t launch_ring16(bool ta, bool tb, const GemmParams& p, hipStream_t s) {
    auto launch = [&](int te, const GemmParams& q) {
        if (te == 256) return launch_ring_wb<DT, 4>(ta, tb, q, s);
        if (te == 224) return launch_ring_wb<DT, 3, 4>(ta, tb, q, s);      // 192 rows x 256 columns
        if (te == 192) return launch_ring_wb<DT, 2, 4, 2>(ta, tb, q, s);   // 128 rows x 256 columns, deep K-steps
        if (te == 64) return launch_ring_wb<DT, 1>(ta, tb, q, s);
        // 128 x 128: the deep K-step unless many tiles with a short k queue up on every CU (see ring16_deep128)
        if (ring16_deep128(ring16_tiles(128, q.M, q.N, q.batch), q.K)) return launch_ring_wb<DT, 2, 0, 2>(ta, tb, q, s);
        return launch_ring_wb<DT, 2>(ta, tb, q, s);
    };
    const int rect = RECT_128 | RECT_192 | (!ta && tb ? RECT_BOTH_K : 0);
    if (p.batch == 1 && p.cmode != C_PARTIAL && !p.Aptr && !p.Bptr && !p.Cptr) {
        const Ring16Split sp = ring16_split(p.M, p.N, p.K, rect);
        if (sp.axis) {
            GemmParams head, tail;
            ring_split_params(p, ta, tb, 2, sp, head, tail);
            const hipError_t e = launch(sp.head_edge, head);
            if (e != hipSuccess) return e;
            return launch(sp.tail_edge, tail);
        }
    }
    if (p.batch > 1 && p.cmode != C_PARTIAL && !p.Aptr && !p.Bptr && !p.Cptr) {
        // a batch whose tiles are whole rounds over the CUs plus a fraction: leading columns of every item, then the rest
        // (see ring16_column_split; the same products, tiled differently)
        const int64_t head_cols = ring16_column_split(p.M, p.N, p.K, p.batch, rect);
        if (head_cols) {
            GemmParams head = p, tail = p;
            head.N = (int)head_cols;
            tail.N = p.N - (int)head_cols;
            tail.B = static_cast<const char*>(p.B) + head_cols * (tb ? p.ldb : 1) * 2;
            if (p.tailB) tail.tailB = static_cast<const char*>(p.tailB) + head_cols * 2;
            tail.C = static_cast<char*>(p.C) + head_cols * 2;
            if (p.bias) tail.bias = static_cast<const char*>(p.bias) + head_cols * p.bias_cs * 2;
            const hipError_t e = launch_ring16_planned(head, s, launch, rect);
            if (e != hipSuccess) return e;
            return launch_ring16_planned(tail, s, launch, rect);
        }
    }
    return launch_ring16_planned(p, s, launch, rect);
}

}  // namespace ntg
