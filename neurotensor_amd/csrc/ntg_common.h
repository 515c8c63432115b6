// Shared declarations of the gfx950 matmult backend (device + host side).
#pragma once
#include <hip/hip_runtime.h>
#include <cstdlib>
#include <stdint.h>

// A pointer known to point into global memory.  The pointers of GemmParams are generic; a load through a generic pointer is a
// FLAT instruction, which counts as an LDS operation as well and may return out of order with the global ones, so the
// compiler can only wait for ALL outstanding loads at once: kernels that keep several steps of loads in flight cast their
// operand pointers with this first.
#define NTG_GLOBAL __attribute__((address_space(1)))

namespace ntg {

// numeric values follow nt::DType (nt/dtype/DType_enum.h:14-20); BF16/U64 are extensions
enum DType : int {
    DT_F16 = 0, DT_F32 = 1, DT_F64 = 2,
    DT_C32 = 4, DT_C64 = 5, DT_C128 = 6,      // interleaved (re, im) pairs of half / float / double
    DT_I8 = 7, DT_I16 = 8, DT_I32 = 9, DT_I64 = 10,
    DT_U8 = 12, DT_U16 = 13, DT_U32 = 14,
    DT_BF16 = 100, DT_U64 = 101
};

// how the kernel treats the incoming C
enum CMode : int {
    C_OVERWRITE = 0,   // C  = op(A).op(B)          (caller knows C would be zeros)
    C_ACCUMULATE = 1,  // C += op(A).op(B)          (contract of nt_matmult, nt_matmult.hpp:370-378)
    C_BIAS = 2,        // C  = bias (+) op(A).op(B) (cpu::linear, matmult_cpu.cpp:1637-1647)
    C_PARTIAL = 3      // internal: write the 32-bit accumulators (fp32 sums of a split-K range; integer sums of 8-bit operands) to a 4-byte matrix at C; DMA kernel only
};

// Unsigned division by a divisor fixed at launch (round-up multiplier form): exact for every
// 32-bit n.  q = (t + ((n - t) >> s1)) >> s2  with  t = mulhi(m, n).
struct FastDiv { uint32_t m, s1, s2; };
static inline FastDiv make_fastdiv(uint32_t d) {
    uint32_t l = 0;
    while ((1ull << l) < d) ++l;
    FastDiv f;
    f.m = (uint32_t)(((1ull << 32) * ((1ull << l) - d)) / d + 1);
    f.s1 = l < 1 ? l : 1;
    f.s2 = l > 0 ? l - 1 : 0;
    return f;
}

// Geometry of an operand that is the im2col matrix of an image and is never stored:
//   col(kk, l) = im[c, od*s_d - p_d + t*d_d, oh*s_r - p_r + r*d_r, ow*s_c - p_c + q*d_c]   (0 in the padding)
//   kk = ((c*k_d + t)*k_r + r)*k_c + q,   l = (od*Ho + oh)*Wo + ow
// (the matrix nt::functional::unfold2d / unfold3d(..., transpose_out = true) would produce,
// nt/functional/cpu/unfold2d.cpp:12-112, unfold3d.cpp:9-80).  Two spatial axes: D = k_d = s_d = d_d = 1, p_d = 0.
struct ConvGeom {
    int D, H, W, chan;       // chan = D*H*W, the channel stride
    int s_d, s_r, s_c, p_d, p_r, p_c, d_d, d_r, d_c;
    int k_d, k_r, k_c, k_rc, k_drc, Wo, HoWo;
    int last;                // index of the last element of the image slice at p.B (loads are clamped to it)
    FastDiv div_kdrc, div_krc, div_kc, div_wo, div_howo;
    // channels-last weight gradient with several images per K loop: output pixels per image (0: one image per item),
    // its divider, and the elements from one image to the next
    int fold_L;
    FastDiv div_fold;
    int64_t fold_stride;
    // channels-last convolution of few channels: taps of one tap row per K-step (0 / 1: one tap) and the padded row length
    int tap_step, kq_pad;
    // channels-last convolution: the copy of the image carries the padding as pixels of zeros (H, W, chan describe the padded
    // image, p_r = p_c = 0), so the gather needs no validity test
    int halo;
    // ... and k runs (64-byte run of channels, tap, channel inside the run) instead of (tap, channel): the taps of a run reach
    // the same pixels while they are in L2 (unit strides; the weights are permuted to match)
    int tap_inner;
    // channels-last convolution and weight gradient: column n of this launch is column n + n_base of the whole product
    // (a launch on the trailing columns); n_total = columns of the whole product (0: this launch has them all)
    int n_base, n_total;
    // channels-last weight gradient, items = k ranges: the k axis is the output pixels of ALL images counted through, item b
    // covers pixels [b K, (b + 1) K) of it (K a whole number of K-steps, and so is an image: a K-step never straddles two).
    // The gathered operand finds image and pixel by division (fold_L, fold_stride as above); dY, read where it lies as
    // [image][out channel][pixel], jumps a_image_stride elements after every a_steps K-steps.  0: off.
    int k_ranges, a_steps;
    FastDiv div_a_steps;
    int64_t a_image_stride;
    // channels-last weight gradient on a copy that carries the padding as pixels of zeros (H, W describe the padded image,
    // p_r = p_c = 0): output pixels per image when the kernel keeps their window origins in an LDS table, 0: off
    int pix_table;
};

struct GemmParams {
    const void* A;
    const void* B;
    void* C;
    // pointer tables in device memory (nt_matmult_batch's A[]/B[]/C[]); null => strided addressing
    const void* const* Aptr;
    const void* const* Bptr;
    void* const* Cptr;
    // C_BIAS: C0(b,i,j) = bias[b*bias_bs + i*bias_rs + j*bias_cs]
    const void* bias;
    int64_t bias_bs, bias_rs, bias_cs;
    int64_t lda, ldb, ldc;   // row length of the stored matrices, in elements
    int64_t sA, sB, sC;      // batch strides in elements, 0 = the same matrix for every item
    // A batch whose items are each split into k ranges (split-K of a batch): launch index b = range * krange_items + item,
    // A and B of it lie at item * sA + range * sAk (sB, sBk); C (the partial sums) at b * sC.  0: a plain batch.
    int krange_items;
    int64_t sAk, sBk;
    int M, N, K, batch;      // logical sizes (after the transpose flags)
    int cmode;
    int tiles_m, tiles_n;
    int vecA_ok, vecB_ok;    // 16-byte vector loads are legal for every row of A / B
    // Padded-copy form (DMA-fed kernels): an operand stored [k][m] / [k][n] whose rows keep the 16-byte rule is read where it lies, and only
    // its k-rows from tail_k0 (a multiple of the K-step) on come from a small copy that continues with rows of zeros up to the padded K
    // (same row pitch as the operand; s_tail = elements between the items' copies, 0 = one for all).  Null: none.
    const void* tailA;
    const void* tailB;
    int64_t s_tailA, s_tailB;
    int tail_k0;
    int keep_k_order;        // never split along k (the caller wants the one chain per element in ascending k)
    // Pointer tables whose entries' alignment the library found out on the device (see gemm_ptrs): the product is launched on
    // the DMA-fed kernel AND on the register-staged one; a kernel whose gate_want differs from *gate returns at once.
    const int* gate;
    int gate_want;
    int ptrs_aligned;        // pointer tables only: the caller vouches that every entry is a multiple of 16 bytes (the tables
                             // live in device memory, the host cannot look); lets table batches onto the DMA-fed kernels
    int group_m;             // DMA-fed kernels: tile rows per group of the tile order (0: the default, 4; see tile_coords)
    int act;                 // ACT_RELU: the stored result is max(result, 0) (relu_ of the reference = clamp_(x, 0): NaN and -0 become +0);
                             // honoured by the DMA-fed Float16 / BFloat16 / Float32 kernels and the split-K reduction only
    ConvGeom conv;           // used by the implicit-im2col kernels only: B = image, op(B) = col or col^T
};
enum { ACT_NONE = 0, ACT_RELU = 1 };

// Tile the DMA-fed 16-bit kernel uses for M x N x K x batch: square with edge 256, 128 or 64, or (plain products only)
// 128 rows x 256 columns (code 192) or 192 rows x 256 columns (code 224).  Larger tiles need less LDS traffic per flop (a CU sustains
// about 0.5 of its MFMA peak on the 256-column tiles, 0.4 / 0.25 on 128-wide / 64-wide ones at full load; 0.64 on
// 256-wide and 0.55 on the rectangular tiles while most CUs are idle and the clock is high), smaller ones spread the
// work over the 256 CUs more evenly, waste less on the padding of M and N, and hide a tile's prologue and epilogue
// (about 3 / 4 / 5 / 1.5 / 0.6 us of exposed latency per tile of 256 x 256 / 192 x 256 / 128 x 256 / 128 x 128 /
// 64 x 64; the 256-column tiles have their CU to themselves, the 128-wide ones share a CU in pairs) behind their
// neighbours on the CU.  Estimated time = tiles per CU x (tile time + exposed latency).
static inline int ring16_tile_rows(int t) { return t == 224 ? 192 : t == 192 ? 128 : t; }
static inline int ring16_tile_cols(int t) { return t == 224 || t == 192 ? 256 : t; }
// 128 x 128 tiles come in two forms: the deep K-step (128 bytes of k per row: whole cache lines of a K-contiguous operand,
// half as many barriers; 128 KiB of LDS, one workgroup per CU) and the 64-byte K-step with two workgroups per CU, which
// is ahead only where many tiles with a short k queue up on every CU (the second workgroup hides the first one's prologue
// and epilogue): 1024 tiles at k = 1024 took 40.6 us against 44.6, 1024 tiles at k = 4096 145 against 134.
static inline bool ring16_deep128(int64_t nt, int64_t K) { return nt <= 256 || K >= 2048; }
static inline double ring16_cost_us(int t, int64_t nt, int64_t K) {
    const double cu_flops_per_us = 9.77e6;                      // 2500 TFLOP/s over 256 CUs
    // (measured per-tile figures: fraction of the CU's MFMA peak in the K loop, and microseconds of prologue + epilogue;
    //  the 64-byte K-step on 128 x 128 tiles is bound by the LDS of its CU whether one or two workgroups share it; 64 x 64
    //  tiles with a deep k on many CUs run at 0.15 - 0.19: 256 tiles at k = 4096 took 21 us)
    const bool deep = t == 128 && ring16_deep128(nt, K);
    const double f = t == 256 ? (nt >= 192 ? 0.5 : 0.64) : t == 224 || t == 192 ? (nt >= 192 ? 0.5 : 0.55)
                   : t == 128 ? (deep ? (nt > 256 ? 0.45 : nt >= 192 ? 0.5 : 0.565) : 0.3) : (nt >= 96 && K >= 1536 ? 0.18 : 0.25);
    const double latency = t == 256 ? 3.0 : t == 224 ? 4.0 : t == 192 ? 5.0 : t == 128 ? (deep ? (nt >= 192 ? 7.0 : 4.0) : 1.5) : 0.6;
    const double area = (double)ring16_tile_rows(t) * ring16_tile_cols(t);
    return (double)((nt + 255) / 256) * (2.0 * area * (double)K / (cu_flops_per_us * f) + latency);
}
static inline int64_t ring16_tiles(int t, int64_t M, int64_t N, int64_t batch) {
    const int r = ring16_tile_rows(t), c = ring16_tile_cols(t);
    return ((M + r - 1) / r) * ((N + c - 1) / c) * batch;
}
// rect: which rectangular tiles are candidates (RECT_128 | RECT_192).  They win where they fill whole rounds over the
// CUs better than the square tiles (3072 x 3072 outputs: 192 tiles of 192 x 256 against 144 of 256 x 256; 2048 x 4096:
// 256 tiles of 128 x 256 against 128 or 512) and K is long enough to carry their latency.  Over many rounds the
// 128 x 256 tile was measured slower than the estimate says (2 x 4736 x 5888, K = 8192: 891 us against 816 us on
// 256-wide tiles), so it has to be 10 % ahead of the larger tiles, and the 192 x 256 tile 5 % ahead of the 256-wide one
// where that one has more than two rounds (12 x 968 x 4136, K = 2048: 244 us against 216 us at estimates of 226 and
// 232); the smaller tiles then have to beat the chosen estimate as it stands.
// RECT_BOTH_K: both operands are K-contiguous (A . B^T, the Linear forward).  The tiles with 64-byte K-steps then fetch every
// cache line of both operands in two halves, one K-step apart, and run about 6 % slower than on A . B (4096^3: 117.8 us
// against 111.8); the 128 x 256 tile with its 128-byte K-steps does not, and up to k = 4096 it is as fast as its estimate
// (beyond, over many rounds, it falls 2 - 10 % behind the 256 x 256 tile whatever the storage form).
enum { RECT_NONE = 0, RECT_128 = 1, RECT_192 = 2, RECT_BOTH_K = 4 };
static inline int ring16_tile_edge(int64_t M, int64_t N, int64_t K, int64_t batch, int rect = RECT_NONE) {
    // (measurement knob, read once: NTG_TILE_EDGE = 256 / 224 / 192 / 128 / 64 forces the tile; results do not depend on it)
    static const int forced = [] { const char* e = getenv("NTG_TILE_EDGE"); return e ? atoi(e) : 0; }();
    if (forced == 256 || forced == 128 || forced == 64 || (forced == 224 && (rect & RECT_192)) || (forced == 192 && (rect & RECT_128))) return forced;
    int best = 256;
    double best_us = 0.0;
    for (int t : {256, 224, 192, 128, 64}) {
        if ((t == 224 && !(rect & RECT_192)) || (t == 192 && !(rect & RECT_128))) continue;
        // (a longer k: the 128 x 256 tile's own deficit outweighs the halves; a shorter one: its prologue and epilogue do)
        const bool both_k = (rect & RECT_BOTH_K) != 0 && K > 2048 && K <= 4096;
        const int64_t nt = ring16_tiles(t, M, N, batch);
        const bool lines = t == 192 || (t == 128 && ring16_deep128(nt, K));       // 128-byte K-steps: whole cache lines
        const double us = ring16_cost_us(t, nt, K) * (both_k && !lines ? 1.0 / 0.94 : 1.0);
        const double margin = t == 192 ? (both_k ? 1.0 : 0.9) : t == 224 && ring16_tiles(256, M, N, batch) > 512 ? 0.95 : 1.0;
        if (t == 256 || us < margin * best_us) { best = t; best_us = us; }
    }
    return best;
}

// A batched product whose tiles fill the 256 CUs a whole number of times plus a small rest would spend a full tile time
// on that rest.  The plan then gives the first `head` items the chosen tile (as many as fit in whole rounds) and the
// remaining ones a tile chosen for them alone (usually the next smaller one, spread over all CUs), as two launches; the
// estimate has to improve by 7 % (the second launch costs a few microseconds).  head == batch: one launch.
struct Ring16Plan { int edge, head, tail_edge; };
static inline Ring16Plan ring16_plan(int64_t M, int64_t N, int64_t K, int64_t batch, int rect = RECT_NONE) {
    Ring16Plan pl;
    pl.edge = pl.tail_edge = ring16_tile_edge(M, N, K, batch, rect);
    pl.head = (int)batch;
    if (batch < 2 || pl.edge == 64) return pl;
    const int64_t per_item = ring16_tiles(pl.edge, M, N, 1), total = per_item * batch;
    const int64_t full = total / 256;
    if (full < 1 || total % 256 == 0) return pl;
    const int64_t head = full * 256 / per_item;
    if (head < 1 || head >= batch) return pl;
    const int tail_edge = ring16_tile_edge(M, N, K, batch - head, rect);
    const double split_us = ring16_cost_us(pl.edge, per_item * head, K) +
                            ring16_cost_us(tail_edge, ring16_tiles(tail_edge, M, N, batch - head), K) + 2.0;
    if (split_us < 0.93 * ring16_cost_us(pl.edge, total, K)) { pl.head = (int)head; pl.tail_edge = tail_edge; }
    return pl;
}

static inline double ring16_plan_cost_us(const Ring16Plan& pl, int64_t M, int64_t N, int64_t K, int64_t batch) {
    if (pl.head >= batch) return ring16_cost_us(pl.edge, ring16_tiles(pl.edge, M, N, batch), K);
    return ring16_cost_us(pl.edge, ring16_tiles(pl.edge, M, N, pl.head), K) +
           ring16_cost_us(pl.tail_edge, ring16_tiles(pl.tail_edge, M, N, batch - pl.head), K) + 2.0;
}
// A batch of products can leave the CUs badly filled in two ways that a split along the columns mends: columns that are
// whole tiles plus a narrow rest (a convolution of 56 x 56 images: 3136 output pixels = 12 tiles of 256 and 64 more spend a
// whole tile on that rest in every item), and tile counts that are whole rounds over the CUs plus a fraction (the weight
// gradient of the same layer: 9 tiles of 256 x 256 per image, 576 = 2.25 rounds; columns 0 .. 2047 of every image are 512
// tiles = two rounds, the last 256 columns go to 128 x 128 tiles).  The split gives the leading head_cols columns of every
// item to one (planned) launch and the remaining columns to another, each on the tile chosen for it alone.
// head_cols = columns of the first launch, a multiple of 128; 0: no split.  It has to be 5 % ahead of the batch plan.
static inline int64_t ring16_column_split(int64_t M, int64_t N, int64_t K, int64_t batch, int rect = RECT_NONE) {
    if (N < 256) return 0;
    // candidates (a handful, so that planning stays a few microseconds on the launch path): for 256- and 128-wide tile
    // columns, the whole tile columns before a narrow rest, and the largest count of tile columns whose tiles over the whole
    // batch are whole rounds of the 256 CUs -- as head and, mirrored, as tail
    int64_t cand[8];
    int nc = 0;
    auto add = [&](int64_t c) {
        if (c <= 0 || c >= N || c % 128 != 0) return;
        for (int i = 0; i < nc; ++i)
            if (cand[i] == c) return;
        cand[nc++] = c;
    };
    for (int64_t tc : {(int64_t)256, (int64_t)128}) {
        add(N / tc * tc);
        const int64_t per_col = ((M + tc - 1) / tc) * batch;             // tiles of one tile column over the batch (square tiles)
        int64_t g = per_col, h = 256;
        while (h) { const int64_t r = g % h; g = h; h = r; }              // gcd(per_col, 256)
        const int64_t q0 = 256 / g, q = (N / tc) / q0 * q0;
        add(q * tc);
        add(N - q * tc);
    }
    double best = 0.95 * ring16_plan_cost_us(ring16_plan(M, N, K, batch, rect), M, N, K, batch);
    int64_t best_cols = 0;
    for (int i = 0; i < nc; ++i) {
        const int64_t c = cand[i];
        const double us = ring16_plan_cost_us(ring16_plan(M, c, K, batch, rect), M, c, K, batch) +
                          ring16_plan_cost_us(ring16_plan(M, N - c, K, batch, rect), M, N - c, K, batch) + 2.0;
        if (us < best) { best = us; best_cols = c; }
    }
    return best_cols;
}

// A single large product whose tiles fill the 256 CUs a whole number of times plus a rest spends a full tile time on that
// rest (8192 x 11008 on 256 x 256 tiles: 1376 tiles = 5.4 rounds, the sixth round a third full).  The split gives the
// leading tile columns (axis 1) or tile rows (axis 2) to the chosen tile -- as many as make whole rounds, or nearly -- and
// the remaining strip to a tile chosen for it alone (usually 128 x 256: twice the tiles, each half as long), as two
// launches on sub-matrices of the same operands.  `head` = elements of the split axis in the first launch; axis 0: no split.
// The estimate has to improve by 5 % (the second launch costs a few microseconds).
struct Ring16Split { int axis; int64_t head; int head_edge, tail_edge; };
static inline Ring16Split ring16_split(int64_t M, int64_t N, int64_t K, int rect = RECT_NONE) {
    Ring16Split sp = {0, 0, 0, 0};
    const int edge = ring16_tile_edge(M, N, K, 1, rect);
    if (edge == 64) return sp;
    const int64_t tr = ring16_tile_rows(edge), tc = ring16_tile_cols(edge);
    const int64_t tm = (M + tr - 1) / tr, tn = (N + tc - 1) / tc, T = tm * tn;
    if (T <= 256 || T % 256 == 0) return sp;
    double best = 0.95 * ring16_cost_us(edge, T, K);
    for (int axis = 1; axis <= 2; ++axis) {
        const int64_t count = axis == 1 ? tn : tm, other = axis == 1 ? tm : tn, step = axis == 1 ? tc : tr;
        // candidates: the counts of leading tile columns / rows that make whole rounds over the CUs (the largest two), and all
        // but the last one or two -- a handful, so that planning stays on the order of a microsecond
        int64_t g = other, h = 256;
        while (h) { const int64_t r = g % h; g = h; h = r; }              // gcd(other, 256)
        const int64_t q0 = 256 / g, qmax = (count - 1) / q0 * q0;
        const int64_t cands[4] = {qmax, qmax - q0, count - 1, count - 2};
        for (int ci = 0; ci < 4; ++ci) {
            const int64_t c = cands[ci];
            if (c < 1 || c >= count) continue;
            const int64_t rest = (axis == 1 ? N : M) - c * step;
            const int64_t Mt = axis == 1 ? M : rest, Nt = axis == 1 ? rest : N;
            const int te = ring16_tile_edge(Mt, Nt, K, 1, rect);
            const double us = ring16_cost_us(edge, other * c, K) + ring16_cost_us(te, ring16_tiles(te, Mt, Nt, 1), K) + 2.0;
            if (us < best) { best = us; sp.axis = axis; sp.head = c * step; sp.head_edge = edge; sp.tail_edge = te; }
        }
    }
    return sp;
}

static inline int64_t elem_size(int dt) {
    switch (dt) {
    case DT_I8: case DT_U8: return 1;
    case DT_F16: case DT_BF16: case DT_I16: case DT_U16: return 2;
    case DT_F32: case DT_I32: case DT_U32: return 4;
    case DT_F64: case DT_I64: case DT_U64: return 8;
    case DT_C32: return 4;
    case DT_C64: return 8;
    case DT_C128: return 16;
    default: return 0;
    }
}

// launchers implemented in the .hip files; all return a hipError_t
hipError_t launch_gemm_mfma(int dtype, bool ta, bool tb, const GemmParams& p, hipStream_t s);
// Float16 / BFloat16 / Float32 on the DMA-fed kernel or not at all (*taken = false, nothing launched): the kernel whose
// epilogue applies GemmParams::act
hipError_t launch_gemm_ring_only(int dtype, bool ta, bool tb, const GemmParams& p, hipStream_t s, bool* taken);
// C[b][m][n] = max(C[b][m][n], 0) in place (floating dtypes)
hipError_t launch_relu_inplace(int dtype, void* C, int64_t ldc, int64_t sC, int64_t M, int64_t N, int64_t batch, hipStream_t s);
hipError_t launch_gemm_valu(int dtype, bool ta, bool tb, const GemmParams& p, hipStream_t s);
hipError_t launch_gemm_mfma_i8(int dtype, bool ta, bool tb, const GemmParams& p, hipStream_t s);   // Int8 / UInt8: MFMA where rows are 16-byte multiples
hipError_t launch_gemm_complex(int dtype, bool ta, bool tb, const GemmParams& p, hipStream_t s);   // Complex32 / 64 / 128: lane-wise products on (re, im) pairs
hipError_t launch_gemm_skinny(int dtype, bool ta, bool tb, const GemmParams& p, hipStream_t s, bool* handled);
// op(B) is the im2col matrix of the image at p.B (tb: its transpose); floating dtypes only
hipError_t launch_conv_mfma(int dtype, bool tb, const GemmParams& p, hipStream_t s);
hipError_t launch_unfold2d(int64_t elem_size, const void* im, void* col,
                           int64_t batch, int64_t channels, int64_t height, int64_t width,
                           int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c,
                           int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c, hipStream_t s);

hipError_t launch_col2im(int dtype, const void* col, void* im,
                         int64_t batch, int64_t channels, int64_t height, int64_t width,
                         int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c,
                         int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c, int accumulate, hipStream_t s);

// unfold / col2im over 1..NTG_MAX_SPATIAL axes (slowest first); filled by the C API
#define NTG_MAX_SPATIAL 4
struct UnfoldNdParams {
    int nd;
    int64_t batch, channels;
    int64_t size[NTG_MAX_SPATIAL], k[NTG_MAX_SPATIAL], s[NTG_MAX_SPATIAL], p[NTG_MAX_SPATIAL], d[NTG_MAX_SPATIAL], out[NTG_MAX_SPATIAL];
    int64_t taps, L, vol, ccol, total;   // prod k, prod out, prod size, channels*taps, batch*ccol*L
};
hipError_t launch_unfoldnd(int64_t elem_size, const void* im, void* col, const UnfoldNdParams& u, hipStream_t s);
hipError_t launch_col2imnd(int dtype, const void* col, void* im, const UnfoldNdParams& u, int accumulate, hipStream_t s);

// split-K: out (+)= sum over s of part[s] (s ascending), fp32 accumulation for the 16-bit dtypes whose partials are float
hipError_t launch_splitk_reduce(int dtype, const void* part, int splits, const GemmParams& p, hipStream_t s);

// conv2d backward helpers (unfold2d.hip): ordered sum of per-image weight gradients; weights of
// the gradient-to-image convolution
hipError_t launch_reduce_batch(int dtype, const void* part, void* out, int64_t batch, int64_t n, int accumulate, hipStream_t s);
// Where the pixels of a channels-last copy go when the copy carries a border of zero pixels: pixel (h, w) of a W-wide image is
// pixel (h + top) * Wp + (w + left) of a padded image of Hp x Wp pixels.  nullptr / Wp == 0: no border.
struct HaloMap { int64_t W, H, Wp, Hp, top, left; };
// A weight permutation that the launch of a channels-last copy can take along (its blocks share the elements after
// their tiles): kind 1 = launch_weights_channels_last(w, wp, rows = a, cg, cgp, taps, chunk), kind 2 =
// launch_flip_weights_channels_last(w, wp, groups = a, og, ogp, cg, taps, chunk).
struct WeightsJob { int kind; const void* w; void* wp; int64_t a, og, ogp, cg, cgp, taps, chunk; };
// With `halo`, pixels go to their places inside the bordered copy.  When the 16-byte kernel serves the copy it also zeroes
// the border and runs `job` in the same launch and sets *took_along; otherwise the caller launches those two itself.
hipError_t launch_nchw_to_nhwc(int64_t elem_size, const void* in, void* out, int64_t batch, int64_t C, int64_t P, hipStream_t s, const HaloMap* halo = nullptr,
                               const WeightsJob* job = nullptr, bool* took_along = nullptr);
hipError_t launch_halo_zero(int64_t elem_size, void* out, int64_t batch, int64_t C, const HaloMap& halo, hipStream_t s);   // zeros the border pixels
hipError_t launch_weights_channels_last(int64_t es, const void* w, void* wp, int64_t rows, int64_t cg, int64_t cgp, int64_t taps, hipStream_t s, int64_t chunk = 0);
hipError_t launch_weights_channels_last_rows(int64_t es, const void* w, void* wp, int64_t rows, int64_t cg, int64_t cgp, int64_t k_r, int64_t k_c,
                                             int64_t kq_pad, hipStream_t s);   // tap rows padded from k_c to kq_pad taps
hipError_t launch_nchw_to_nhwc_padded(int64_t es, const void* in, void* out, int64_t batch, int64_t groups, int64_t cg, int64_t cgp, int64_t P, hipStream_t s,
                                      const HaloMap* halo = nullptr);
hipError_t launch_flip_weights_channels_last(int64_t es, const void* w, void* wt, int64_t groups, int64_t og, int64_t ogp, int64_t cg, int64_t taps, hipStream_t s, int64_t chunk = 0);
// channels-last convolution (image [B][pixel][C], weights [O][(r, q, c)]); F16 / BF16 / F32, two spatial axes
hipError_t launch_conv_nhwc(int dtype, const GemmParams& p, hipStream_t s);
// Image gradient of a strided convolution as one stride-1 convolution per phase of the image (see conv_dimage_phases):
// where the phase planes lie in the temporary buffer (element offsets; -1: the phase has no taps) and how image
// coordinates map to them.  Strides up to 4.
struct PhaseLayout {
    int H, W, p_r, p_c, s_r, s_c;
    uint32_t total;              // batch * channels * H * W
    int a0r[4], a0c[4], hp[4], wp[4];
    int64_t off[16];
    FastDiv div_w, div_h, div_sr, div_sc;
};
hipError_t launch_phase_weights(int64_t es, const void* w, void* wt, int64_t groups, int64_t og, int64_t ogp, int64_t cg, int64_t k_r, int64_t k_c,
                                int64_t er, int64_t ec, int64_t s_r, int64_t s_c, int64_t Mr, int64_t Mc, hipStream_t s);
hipError_t launch_phase_interleave(int dtype, const void* tmp, void* im, const PhaseLayout& q, int accumulate, hipStream_t s);
// 16-, 32- and 64-bit integer products on the 8-bit matrix pipe as byte planes (see gemm_mfma_i8.hip); planes = bytes per element
struct IntPlanesParams { int M, N, K, Kp, Np, batch; int64_t lda, ldb, sA, sB; int ta, tb; };
hipError_t launch_int_split_planes(int planes, const void* A, const void* B, void* a_planes, void* b_planes, const IntPlanesParams& q, hipStream_t s);
hipError_t launch_int_combine(int planes, const void* parts, const GemmParams& p, int Np, hipStream_t s);
hipError_t launch_conv_nhwc_dw(int dtype, bool ta, const GemmParams& p, hipStream_t s);   // ta: A (the output gradient) stored [k][m]
hipError_t launch_reduce_batch_taps_last(int dtype, const void* part, void* out, int64_t batch, int64_t rows, int64_t cg, int64_t cgp,
                                         int64_t taps, int accumulate, hipStream_t s);   // part rows hold cgp >= cg channels per tap
hipError_t launch_flip_weights(int64_t elem_size, const void* w, void* wt, int64_t groups, int64_t og, int64_t cg, int64_t taps, hipStream_t s);

// padded copies of operands whose rows are not 16-byte multiples (pad_copy.hip); es = 1, 2, 4 or 8 bytes per element, sizes in elements
hipError_t launch_pad_copy(int64_t es, const void* src, int64_t ld_src, int64_t s_src, void* dst, int64_t ld_dst, int64_t s_dst,
                           int64_t rows, int64_t cols, int64_t rows_dst, int64_t batch, hipStream_t s);
hipError_t launch_unpad_copy(int64_t es, const void* src, int64_t ld_src, int64_t s_src, void* dst, int64_t ld_dst, int64_t s_dst,
                             int64_t rows, int64_t cols, int64_t batch, hipStream_t s);
hipError_t launch_bias_fill(int64_t es, const void* bias, int64_t bs, int64_t rs, int64_t cs, void* dst, int64_t ld_dst, int64_t s_dst,
                            int64_t rows, int64_t cols, int64_t rows_dst, int64_t batch, hipStream_t s);

// grid of a grid-stride element-wise kernel (256 lanes per workgroup, at most 64 workgroups per CU)
static inline unsigned grid_for(int64_t total) {
    int64_t blocks = (total + 255) / 256;
    if (blocks > 256 * 64) blocks = 256 * 64;
    return (unsigned)(blocks < 1 ? 1 : blocks);
}

#ifdef __HIPCC__
// One element of the complex dtypes as the reference's element-wise code treats it: two lanes (re, im) of the real type,
// added lane by lane in that type (my_complex<T>::operator+=; complex_32 adds in half, rounding every sum).
template <class R>
struct LanePair {
    R re, im;
    LanePair() = default;
    __device__ __forceinline__ LanePair(int z) : re((R)z), im((R)z) {}      // (Acc)0
    __device__ __forceinline__ LanePair& operator+=(const LanePair& o) {
        re = re + o.re;
        im = im + o.im;
        return *this;
    }
};

// element offset of launch index b's A (stride = p.sA, kstride = p.sAk) or B operand
__device__ __forceinline__ int64_t operand_offset(const GemmParams& p, int b, int64_t stride, int64_t kstride) {
    if (p.krange_items == 0) return (int64_t)b * stride;
    const int range = b / p.krange_items, item = b - range * p.krange_items;
    return (int64_t)item * stride + (int64_t)range * kstride;
}

__device__ __forceinline__ uint32_t fast_div(uint32_t n, const FastDiv& f) {
    const uint32_t t = __umulhi(f.m, n);
    return (t + ((n - t) >> f.s1)) >> f.s2;
}

// Workgroup ids are dealt round-robin to the 8 XCDs; make the ids that land on one
// XCD (its own L2) a contiguous range of logical tile ids.
__device__ __forceinline__ int xcd_contiguous_id(int bid, int nb) {
    const int NX = 8;
    const int base = nb / NX, rem = nb % NX;
    const int x = bid % NX, q = bid / NX;
    return x * base + (x < rem ? x : rem) + q;
}

// logical id -> (tile_m, tile_n): column-major inside groups of GROUP_M tile rows,
// so a contiguous id range covers a compact rectangle of C.
__device__ __forceinline__ void tile_coords(int t, int tiles_m, int tiles_n, int GROUP_M, int& tm, int& tn) {
    const int group_size = GROUP_M * tiles_n;
    const int g = t / group_size;
    const int first_m = g * GROUP_M;
    const int gm = (tiles_m - first_m < GROUP_M) ? tiles_m - first_m : GROUP_M;
    const int r = t - g * group_size;
    tm = first_m + r % gm;
    tn = r / gm;
}
#endif

}  // namespace ntg
