// LDS-tiled MFMA GEMM for gfx950:  C (+)= op(A) . op(B)   (row-major, dense)
//
// Replaces the packed SIMD path of the reference, pack_multiply_directly_var_threaded
// (nt/functional/cpu/matmult/nt_matmult.hpp:124-225) and its micro kernel
// (nt_matmult_simde.hpp:301-350), for Float32, Float64, Float16 and BFloat16.
//
// One workgroup = 4 wavefronts in a 2x2 grid; each wavefront owns WBM x WBN MFMA blocks
// (32x32 for fp32/fp16/bf16, 16x16 for fp64) of a BM x BN tile of C and walks K in steps
// of BK through double-buffered LDS.  transpose_a / transpose_b, leading dimensions,
// batch strides (0 = broadcast) and pointer-table batches are absorbed by the loaders:
// nothing is copied or re-laid-out in global memory.
//
// LDS layouts ("vec" = 16 bytes):
//   K-major  [tile row][BK/VE vecs + 1 pad vec]   for operands stored K-contiguous; a lane
//            reads one vec = VE consecutive k of its row.  The odd row stride makes the
//            16 rows read together fall into 16 different 16-byte bank groups.
//   MN-major [k row][tile rows]                    fp32/fp64 operands stored MN-contiguous;
//            a lane reads WB consecutive rows at one k, so MFMA block b of the wavefront
//            covers tile rows  lane_row*WB + b  (interleaved) and no transposition exists.
//   16-bit operands stored MN-contiguous are transposed in registers (8x8 sub-blocks,
//   v_perm_b32) on their way into the K-major layout, because an MFMA lane needs 8
//   consecutive k packed in 4 registers.
#pragma once
#include "ntg_common.h"

namespace ntg {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef double doublex4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <int DT> struct Elem;

template <> struct Elem<DT_F32> {
    using T = float; using AccS = float; using AccV = floatx16;
    static constexpr int R = 32, G = 2, VE = 4, ACCN = 16;
    static __device__ __forceinline__ void mma(AccV& c, float a, float b) { c = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0); }
};
template <> struct Elem<DT_F64> {
    using T = double; using AccS = double; using AccV = doublex4;
    static constexpr int R = 16, G = 4, VE = 2, ACCN = 4;
    static __device__ __forceinline__ void mma(AccV& c, double a, double b) { c = __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0); }
};
template <> struct Elem<DT_F16> {
    using T = _Float16; using AccS = float; using AccV = floatx16;
    static constexpr int R = 32, G = 2, VE = 8, ACCN = 16;
    static __device__ __forceinline__ void mma(AccV& c, u32x4 a, u32x4 b) {
        c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(halfx8, a), __builtin_bit_cast(halfx8, b), c, 0, 0, 0);
    }
};
template <> struct Elem<DT_BF16> {
    using T = __bf16; using AccS = float; using AccV = floatx16;
    static constexpr int R = 32, G = 2, VE = 8, ACCN = 16;
    static __device__ __forceinline__ void mma(AccV& c, u32x4 a, u32x4 b) {
        c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
};

// row of the R x R result block held in accumulator register r of `lane`
template <int R> __device__ __forceinline__ int acc_row(int r, int lane);
template <> __device__ __forceinline__ int acc_row<32>(int r, int lane) { return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3); }
template <> __device__ __forceinline__ int acc_row<16>(int r, int lane) { return 4 * r + (lane >> 4); }

// Pointers into the operands carry the global address space, so that their loads and stores
// are global_* instructions (vmcnt only) and never share the LDS counter with the ds_reads.
#define NTG_GLOBAL __attribute__((address_space(1)))
template <class T> using gptr = const NTG_GLOBAL T*;
template <class T> using gptr_mut = NTG_GLOBAL T*;

template <class T, int VE, bool ALIGNED>
__device__ __forceinline__ u32x4 ldvec(gptr<T> src, bool outer_ok, int c0, int cmax, bool vec_ok) {
    if constexpr (ALIGNED) {
        return *reinterpret_cast<gptr<u32x4>>(src);
    } else {
        u32x4 r = {0u, 0u, 0u, 0u};
        if (outer_ok) {
            if (vec_ok && c0 + VE <= cmax) {
                r = *reinterpret_cast<gptr<u32x4>>(src);
            } else {
                T tmp[VE];
#pragma unroll
                for (int e = 0; e < VE; ++e) tmp[e] = (c0 + e < cmax) ? src[e] : (T)0.0f;
                __builtin_memcpy(&r, tmp, 16);
            }
        }
        return r;
    }
}

// Implicit im2col.  Element (kk, l) of the never-stored matrix described by ConvGeom is
//   im[c, oh*s_r - p_r + r*d_r, ow*s_c - p_c + q*d_c]     kk = (c, r, q),  l = (oh, ow)
// Its byte offset is the sum of a term in kk (ConvRow::roff) and a term in l (ConvCol::off0);
// whichever of the two is fixed for a thread over the whole k loop is computed once.
// Every load is unconditional: the offset is clamped into the image (a padding tap reads some
// neighbouring element), nothing consumes the value, so all of a tile's loads stay in flight; one
// bit per element says whether it is real, and conv_mask() zeroes the rest when the tile is
// written to LDS.  The bit of element e sits at bit 8*(e%4) of mask word e/4.
// ND = 2 or 3 spatial axes (compile time: the two-axis kernels carry no depth arithmetic)
struct ConvRow { uint32_t roff, t, r, q; int dd, dh, dw; bool valid; };
struct ConvCol { uint32_t off0; int id0, ih0, iw0; };

template <class T, int ND>
__device__ __forceinline__ ConvRow conv_row(const ConvGeom& g, int kk, bool valid) {
    ConvRow o;
    uint32_t c, rem;
    if constexpr (ND == 3) {
        c = fast_div((uint32_t)kk, g.div_kdrc);
        const uint32_t rem3 = (uint32_t)kk - __umul24(c, (uint32_t)g.k_drc);
        o.t = fast_div(rem3, g.div_krc);
        rem = rem3 - __umul24(o.t, (uint32_t)g.k_rc);
        o.dd = (int)__umul24(o.t, (uint32_t)g.d_d) - g.p_d;
    } else {
        c = fast_div((uint32_t)kk, g.div_krc);
        rem = (uint32_t)kk - __umul24(c, (uint32_t)g.k_rc);
        o.t = 0;
        o.dd = 0;
    }
    o.r = fast_div(rem, g.div_kc);
    o.q = rem - __umul24(o.r, (uint32_t)g.k_c);
    o.valid = valid;
    o.dh = valid ? (int)__umul24(o.r, (uint32_t)g.d_r) - g.p_r : -(1 << 29);   // far outside: every tap is padding
    o.dw = (int)__umul24(o.q, (uint32_t)g.d_c) - g.p_c;
    o.roff = (c * (uint32_t)g.chan + ((uint32_t)o.dd * (uint32_t)g.H + (uint32_t)o.dh) * (uint32_t)g.W + (uint32_t)o.dw) * (uint32_t)sizeof(T);
    return o;
}

template <class T, int ND>
__device__ __forceinline__ ConvCol conv_col(const ConvGeom& g, int l, bool valid) {
    ConvCol o;
    uint32_t rem = (uint32_t)l;
    o.id0 = 0;
    if constexpr (ND == 3) {
        const uint32_t od = fast_div((uint32_t)l, g.div_howo);
        rem = (uint32_t)l - od * (uint32_t)g.HoWo;
        o.id0 = (int)__umul24(od, (uint32_t)g.s_d);
    }
    const uint32_t oh = fast_div(rem, g.div_wo);
    const uint32_t ow = rem - oh * (uint32_t)g.Wo;
    o.ih0 = valid ? (int)__umul24(oh, (uint32_t)g.s_r) : -(1 << 29);
    o.iw0 = (int)__umul24(ow, (uint32_t)g.s_c);
    o.off0 = (((uint32_t)o.id0 * (uint32_t)g.H + (uint32_t)o.ih0) * (uint32_t)g.W + (uint32_t)o.iw0) * (uint32_t)sizeof(T);
    return o;
}

// For a fixed column: bit t of `dm` / bit r of `hm` / bit q of `wm` say whether that tap plane / row / column falls
// inside the image (kernels up to 8 taps per axis; larger ones use the stored im2col matrix).
template <int ND>
__device__ __forceinline__ void conv_tap_masks(const ConvGeom& g, const ConvCol& col, uint32_t& dm, uint32_t& hm, uint32_t& wm) {
    dm = 0xffu;
    hm = 0;
    wm = 0;
    if constexpr (ND == 3) dm = 0;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        if constexpr (ND == 3) dm |= ((t < g.k_d) & ((unsigned)(col.id0 + t * g.d_d - g.p_d) < (unsigned)g.D)) ? (1u << t) : 0u;
        hm |= ((t < g.k_r) & ((unsigned)(col.ih0 + t * g.d_r - g.p_r) < (unsigned)g.H)) ? (1u << t) : 0u;
        wm |= ((t < g.k_c) & ((unsigned)(col.iw0 + t * g.d_c - g.p_c) < (unsigned)g.W)) ? (1u << t) : 0u;
    }
}

template <class T>
__device__ __forceinline__ T conv_load(gptr<T> im, const ConvGeom& g, uint32_t off) {
    const int lim = g.last * (int)sizeof(T);
    int boff = (int)off;
    boff = boff < 0 ? 0 : boff;
    boff = boff > lim ? lim : boff;
    return *reinterpret_cast<gptr<T>>(reinterpret_cast<gptr<char>>(im) + (uint32_t)boff);
}

template <class T, int VE>
__device__ __forceinline__ u32x4 conv_mask(u32x4 v, const uint32_t* okm) {
    auto bit = [&](int e) { return (uint32_t)(((int32_t)(okm[e >> 2] << (31 - 8 * (e & 3)))) >> 31); };   // all ones / all zeros
    if constexpr (sizeof(T) == 4) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] &= bit(e);
    } else if constexpr (sizeof(T) == 8) {
#pragma unroll
        for (int e = 0; e < 2; ++e) { v[2 * e] &= bit(e); v[2 * e + 1] &= bit(e); }
    } else {
#pragma unroll
        for (int d = 0; d < 4; ++d) v[d] &= __builtin_amdgcn_perm(bit(2 * d + 1), bit(2 * d), 0x07060100u);
    }
    return v;
}

// One operand's BMN x BK tile: global -> registers -> LDS.
//   KC: stored K-contiguous in global memory (A without transpose_a, B with transpose_b)
//   KM: K-major LDS layout
template <int DT, bool KC, bool KM, int TMN, int BK, bool ALIGNED>
struct TileLoader {
    using T = typename Elem<DT>::T;
    static constexpr int VE = Elem<DT>::VE;
    static constexpr int KV = BK / VE;
    static constexpr int S = KV + 1;
    static constexpr int MV = TMN / VE;
    static constexpr int LDS_BYTES = KM ? TMN * S * 16 : BK * MV * 16;
    static constexpr bool TRANSPOSE = (!KC && KM);
    static constexpr int KG = BK / 8;
    static constexpr int NSB = KG * (TMN / 8);
    static constexpr int NQ = (NSB + 255) / 256;
    static constexpr int NV = TRANSPOSE ? 8 * NQ : (TMN * BK / VE) / 256;
    static_assert(TRANSPOSE ? (VE == 8) : ((TMN * BK / VE) % 256 == 0), "tile does not split over 256 threads");
    static_assert(KM || !KC, "K-contiguous operands always use the K-major layout");

    u32x4 v[NV];

    __device__ __forceinline__ void load(gptr<T> base, int64_t ld, int mn0, int k0, int MN, int K, bool vec_ok, int tid) {
        if constexpr (!TRANSPOSE && KC) {
#pragma unroll
            for (int p = 0; p < NV; ++p) {
                const int vi = tid + p * 256;
                const int row = vi / KV, kv = vi % KV;
                const int mn = mn0 + row, k = k0 + kv * VE;
                v[p] = ldvec<T, VE, ALIGNED>(base + (int64_t)mn * ld + k, mn < MN, k, K, vec_ok);
            }
        } else if constexpr (!TRANSPOSE) {
#pragma unroll
            for (int p = 0; p < NV; ++p) {
                const int vi = tid + p * 256;
                const int kr = vi / MV, mv = vi % MV;
                const int k = k0 + kr, mn = mn0 + mv * VE;
                v[p] = ldvec<T, VE, ALIGNED>(base + (int64_t)k * ld + mn, k < K, mn, MN, vec_ok);
            }
        } else {
#pragma unroll
            for (int q = 0; q < NQ; ++q) {
                const int sb = tid + q * 256;
                if (NSB % 256 == 0 || sb < NSB) {
                    const int kg = sb % KG, mv = sb / KG;
                    const int mn = mn0 + mv * 8;
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        const int k = k0 + kg * 8 + i;
                        v[q * 8 + i] = ldvec<T, VE, ALIGNED>(base + (int64_t)k * ld + mn, k < K, mn, MN, vec_ok);
                    }
                }
            }
        }
    }

    // Same tile, but the operand is the never-stored im2col matrix of `im`: the vectors run
    // along output pixels l, the other index is kk = (channel, tap).
    //   !KC: tile = col[k0.., mn0..]   (k = kk, mn = l)      KC: tile = col^T  (mn = kk, k = l)
    // conv_setup() computes what stays fixed for the thread, load_conv() gathers one tile and
    // conv_finish() zeroes the padding before store().
    static constexpr int NFIX = !KC ? (TRANSPOSE ? NQ * 8 : VE) : NV;
    static constexpr int NE = NV * VE;              // elements a thread gathers per tile
    static constexpr int NW = (VE + 3) / 4;         // mask words per vector
    uint32_t coff[!KC ? NFIX : 1];                  // !KC: byte offsets of the thread's fixed columns ...
    uint32_t hpk[!KC ? (NFIX + 3) / 4 : 1];         //      ... and their tap masks, 8 bits per column
    uint32_t wpk[!KC ? (NFIX + 3) / 4 : 1];
    uint32_t dpk[!KC ? (NFIX + 3) / 4 : 1];         //      (depth taps; three spatial axes only)
    ConvCol ccol[KC ? VE : 1];                      //  KC: this tile's columns
    ConvRow crow[KC ? NFIX : 1];                    //  KC: fixed rows;    !KC: the row being gathered
    uint32_t okm[NV][NW];
    uint32_t raw16[sizeof(T) == 2 ? NV * VE : 1];

    template <int ND>
    __device__ __forceinline__ void conv_setup(const ConvGeom& g, int mn0, int MN, int tid) {
        if constexpr (!TRANSPOSE && KC) {
            static_assert(256 % KV == 0, "a thread keeps the same k offsets for every vector it loads");
#pragma unroll
            for (int p = 0; p < NV; ++p) {
                const int row = (tid + p * 256) / KV;
                crow[p] = conv_row<T, ND>(g, mn0 + row, mn0 + row < MN);
            }
        } else {
            static_assert(TRANSPOSE || 256 % MV == 0, "a thread keeps the same columns for every vector it loads");
#pragma unroll
            for (int i = 0; i < (NFIX + 3) / 4; ++i) hpk[i] = wpk[i] = dpk[i] = 0;
#pragma unroll
            for (int i = 0; i < NFIX; ++i) {
                // threads past NSB sub-blocks compute columns they never use
                const int l = TRANSPOSE ? mn0 + ((tid + (i / 8) * 256) / KG) * 8 + (i % 8) : mn0 + (tid % MV) * VE + i;
                const ConvCol c = conv_col<T, ND>(g, l, l < MN);
                uint32_t dm, hm, wm;
                conv_tap_masks<ND>(g, c, dm, hm, wm);
                coff[i] = c.off0;
                hpk[i / 4] |= hm << (8 * (i % 4));
                wpk[i / 4] |= wm << (8 * (i % 4));
                dpk[i / 4] |= dm << (8 * (i % 4));
            }
        }
    }

    // element idx (0 .. NE-1, a compile-time constant after unrolling) of the tile at k0
    template <int ND>
    __device__ __forceinline__ void conv_elem(int idx, gptr<T> im, const ConvGeom& g, int k0, int K, int tid) {
        const int pv = idx / VE, e = idx % VE;
        if constexpr (TRANSPOSE && NSB % 256 != 0) {
            if (tid + (pv / 8) * 256 >= NSB) return;      // whole wavefronts: this thread owns no sub-block here
        }
        T x;
        if constexpr (!TRANSPOSE && KC) {
            if (idx == 0) {
                const int kv = tid % KV;
#pragma unroll
                for (int c = 0; c < VE; ++c) ccol[c] = conv_col<T, ND>(g, k0 + kv * VE + c, k0 + kv * VE + c < K);
            }
            const int ih = ccol[e].ih0 + crow[pv].dh;
            const int iw = ccol[e].iw0 + crow[pv].dw;
            bool ok = ((unsigned)ih < (unsigned)g.H) & ((unsigned)iw < (unsigned)g.W);   // no short circuit: branch-free
            if constexpr (ND == 3) ok = ok & ((unsigned)(ccol[e].id0 + crow[pv].dd) < (unsigned)g.D);
            if (e % 4 == 0) okm[pv][e / 4] = 0;
            okm[pv][e / 4] |= ok ? (1u << (8 * (e % 4))) : 0u;
            x = conv_load<T>(im, g, ccol[e].off0 + crow[pv].roff);
        } else {
            const int cb = TRANSPOSE ? (pv / 8) * 8 : 0;      // first fixed column of this vector
            if (e == 0) {
                const int kk = TRANSPOSE ? k0 + ((tid + (pv / 8) * 256) % KG) * 8 + (pv % 8) : k0 + (tid + pv * 256) / MV;
                crow[0] = conv_row<T, ND>(g, kk, kk < K);
            }
            if (e % 4 == 0) {
                uint32_t m = (hpk[(cb + e) / 4] >> crow[0].r) & (wpk[(cb + e) / 4] >> crow[0].q) & 0x01010101u;
                if constexpr (ND == 3) m &= dpk[(cb + e) / 4] >> crow[0].t;
                okm[pv][e / 4] = crow[0].valid ? m : 0u;
            }
            x = conv_load<T>(im, g, coff[cb + e] + crow[0].roff);
        }
        if constexpr (sizeof(T) == 4) {
            v[pv][e] = __builtin_bit_cast(uint32_t, x);
        } else if constexpr (sizeof(T) == 8) {
            const uint64_t bits = __builtin_bit_cast(uint64_t, x);
            v[pv][2 * e] = (uint32_t)bits;
            v[pv][2 * e + 1] = (uint32_t)(bits >> 32);
        } else {
            raw16[idx] = __builtin_bit_cast(uint16_t, x);   // packed in conv_finish(): packing here would wait for the load
        }
    }

    // slice s of ns of a tile's gather: the kernel spreads the slices between its MFMAs
    template <int ND>
    __device__ __forceinline__ void conv_slice(int s, int ns, gptr<T> im, const ConvGeom& g, int k0, int K, int tid) {
#pragma unroll
        for (int idx = 0; idx < NE; ++idx)
            if (idx >= s * NE / ns && idx < (s + 1) * NE / ns) conv_elem<ND>(idx, im, g, k0, K, tid);
    }

    template <int ND>
    __device__ __forceinline__ void load_conv(gptr<T> im, const ConvGeom& g, int k0, int K, int tid) {
        conv_slice<ND>(0, 1, im, g, k0, K, tid);
    }

    __device__ __forceinline__ void conv_finish() {
        if constexpr (sizeof(T) == 2) {
#pragma unroll
            for (int p = 0; p < NV; ++p)
#pragma unroll
                for (int d = 0; d < 4; ++d) v[p][d] = raw16[p * 8 + 2 * d] | (raw16[p * 8 + 2 * d + 1] << 16);
        }
#pragma unroll
        for (int p = 0; p < NV; ++p) v[p] = conv_mask<T, VE>(v[p], okm[p]);
    }

    __device__ __forceinline__ void store(char* lds, int tid) const {
        if constexpr (!TRANSPOSE && KC) {
#pragma unroll
            for (int p = 0; p < NV; ++p) {
                const int vi = tid + p * 256;
                const int row = vi / KV, kv = vi % KV;
                *reinterpret_cast<u32x4*>(lds + (row * S + kv) * 16) = v[p];
            }
        } else if constexpr (!TRANSPOSE) {
#pragma unroll
            for (int p = 0; p < NV; ++p) {
                const int vi = tid + p * 256;
                *reinterpret_cast<u32x4*>(lds + vi * 16) = v[p];
            }
        } else {
#pragma unroll
            for (int q = 0; q < NQ; ++q) {
                const int sb = tid + q * 256;
                if (NSB % 256 == 0 || sb < NSB) {
                    const int kg = sb % KG, mv = sb / KG;
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        // output vec j = tile row mv*8+j, k = kg*8 .. kg*8+7:
                        // dword d packs element j of source vecs 2d and 2d+1
                        u32x4 o;
#pragma unroll
                        for (int d = 0; d < 4; ++d) {
                            const uint32_t lo = v[q * 8 + 2 * d][j >> 1];
                            const uint32_t hi = v[q * 8 + 2 * d + 1][j >> 1];
                            o[d] = (j & 1) ? __builtin_amdgcn_perm(hi, lo, 0x07060302u)
                                           : __builtin_amdgcn_perm(hi, lo, 0x05040100u);
                        }
                        *reinterpret_cast<u32x4*>(lds + ((mv * 8 + j) * S + kg) * 16) = o;
                    }
                }
            }
        }
    }
};

template <int DT, bool TA, bool TB, int WBM, int WBN, int BK>
struct GemmShape {
    using E = Elem<DT>;
    using T = typename E::T;
    static constexpr bool IS16 = sizeof(T) == 2;
    static constexpr bool A_KC = !TA, B_KC = TB;
    static constexpr bool A_KM = IS16 || A_KC, B_KM = IS16 || B_KC;
    static constexpr int BM = 2 * WBM * E::R, BN = 2 * WBN * E::R;
    static constexpr int LDS_A = TileLoader<DT, A_KC, A_KM, BM, BK, true>::LDS_BYTES;
    static constexpr int LDS_B = TileLoader<DT, B_KC, B_KM, BN, BK, true>::LDS_BYTES;
    static constexpr int STAGE = LDS_A + LDS_B;
    static constexpr int LDS_TOTAL = 2 * STAGE;
    static constexpr int GROUP_M = (1024 / BM) > 0 ? (1024 / BM) : 1;
};

// CONV = 2 / 3: op(B) is the implicit im2col matrix (two / three spatial axes) of the image at p.B (p.conv), see load_conv.
template <int DT, bool TA, bool TB, int WBM, int WBN, int BK, bool ALIGNED, int CONV = 0>
__global__ void __launch_bounds__(256) gemm_mfma_kernel(const GemmParams p) {
    using SH = GemmShape<DT, TA, TB, WBM, WBN, BK>;
    using E = Elem<DT>;
    using T = typename E::T;
    using AccS = typename E::AccS;
    using AccV = typename E::AccV;
    constexpr int R = E::R, G = E::G, VE = E::VE;
    constexpr bool IS16 = SH::IS16;
    constexpr bool A_KM = SH::A_KM, B_KM = SH::B_KM;
    constexpr int BM = SH::BM, BN = SH::BN;
    using LA = TileLoader<DT, SH::A_KC, A_KM, BM, BK, ALIGNED>;
    using LB = TileLoader<DT, SH::B_KC, B_KM, BN, BK, ALIGNED>;
    constexpr int SA = LA::S, SB = LB::S;

    extern __shared__ __attribute__((aligned(16))) char smem[];

    if (p.gate && *p.gate != p.gate_want) return;       // (uniform: the other kernel of a gated pair does this product)
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int lr = lane % R, lg = lane / R;

    const int lid = xcd_contiguous_id(blockIdx.x, gridDim.x);
    const int tiles = p.tiles_m * p.tiles_n;
    const int b = lid / tiles;
    int tm, tn;
    tile_coords(lid - b * tiles, p.tiles_m, p.tiles_n, SH::GROUP_M, tm, tn);
    const int m0 = tm * BM, n0 = tn * BN;

    const gptr<T> A = (gptr<T>)(p.Aptr ? static_cast<const T*>(((gptr<const void*>)p.Aptr)[b]) : static_cast<const T*>(p.A) + operand_offset(p, b, p.sA, p.sAk));
    const gptr<T> B = (gptr<T>)(p.Bptr ? static_cast<const T*>(((gptr<const void*>)p.Bptr)[b]) : static_cast<const T*>(p.B) + operand_offset(p, b, p.sB, p.sBk));
    const gptr_mut<T> C = (gptr_mut<T>)(p.Cptr ? static_cast<T*>(((gptr<void*>)p.Cptr)[b]) : static_cast<T*>(p.C) + (int64_t)b * p.sC);
    const bool vecA = p.vecA_ok && ((reinterpret_cast<uintptr_t>(A) & 15) == 0);
    const bool vecB = p.vecB_ok && ((reinterpret_cast<uintptr_t>(B) & 15) == 0);

    AccV acc[WBM][WBN];
#pragma unroll
    for (int i = 0; i < WBM; ++i)
#pragma unroll
        for (int j = 0; j < WBN; ++j)
#pragma unroll
            for (int r = 0; r < E::ACCN; ++r) acc[i][j][r] = (AccS)0;
    // Float32: the accumulators start from C0 (C itself, or the bias): every output element is then the reference's chain
    // c = C0; c = fma(a_k, b_k, c) in ascending k, bit for bit, as in the DMA-fed kernel; the epilogue only stores.
    constexpr bool CHAIN_FROM_C0 = std::is_same<T, float>::value;
    if constexpr (CHAIN_FROM_C0) {
        if (p.cmode == C_ACCUMULATE || p.cmode == C_BIAS) {            // (uniform)
            const gptr<T> bias0 = (gptr<T>)static_cast<const T*>(p.bias);
#pragma unroll
            for (int i = 0; i < WBM; ++i)
#pragma unroll
                for (int j = 0; j < WBN; ++j) {
                    const int n = n0 + (B_KM ? (wn * WBN + j) * R + lr : (wn * R + lr) * WBN + j);
#pragma unroll
                    for (int r = 0; r < E::ACCN; ++r) {
                        const int lrow = acc_row<R>(r, lane);
                        const int m = m0 + (A_KM ? (wm * WBM + i) * R + lrow : (wm * R + lrow) * WBM + i);
                        if (m < p.M && n < p.N)
                            acc[i][j][r] = p.cmode == C_ACCUMULATE ? (AccS)C[(int64_t)m * p.ldc + n]
                                                                   : (AccS)bias0[(int64_t)b * p.bias_bs + (int64_t)m * p.bias_rs + (int64_t)n * p.bias_cs];
                    }
                }
        }
    }

    LA la;
    LB lb;
    const int KT = (p.K + BK - 1) / BK;

    auto load_b = [&](int k0) {
        if constexpr (CONV != 0) lb.template load_conv<CONV>(B, p.conv, k0, p.K, tid);
        else lb.load(B, p.ldb, n0, k0, p.N, p.K, vecB, tid);
    };
    if constexpr (CONV != 0) lb.template conv_setup<CONV>(p.conv, n0, p.N, tid);

    la.load(A, p.lda, m0, 0, p.M, p.K, vecA, tid);
    load_b(0);
    if constexpr (CONV != 0) lb.conv_finish();
    la.store(smem, tid);
    lb.store(smem + SH::LDS_A, tid);
    __syncthreads();

    for (int kt = 0; kt < KT; ++kt) {
        const char* sA = smem + (kt & 1) * SH::STAGE;
        const char* sB = sA + SH::LDS_A;
        // The gathering kernels load unconditionally (the last pass re-reads the last tile into the
        // idle stage), so that the loop body is one scheduling region and the address arithmetic
        // of the gather can sit in the shadow of the MFMAs.
        const bool more = CONV != 0 || (kt + 1 < KT);
        const int k_next = (CONV != 0 && kt + 1 >= KT ? kt : kt + 1) * BK;
        if (more) {
            la.load(A, p.lda, m0, k_next, p.M, p.K, vecA, tid);
            if constexpr (CONV == 0) load_b(k_next);
        }
        // CONV: slice `step` of NSTEP of the next tile's gather follows each group of MFMAs; only LDS
        // reads and scalar work may move across the fence, so the slice stays with its group.
        constexpr int NSTEP = IS16 ? BK / 16 : BK / G;
        auto gather_slice = [&](int step) {
            if constexpr (CONV != 0) {
                lb.template conv_slice<CONV>(step, NSTEP, B, p.conv, k_next, p.K, tid);
                __builtin_amdgcn_sched_barrier(0x104);
            }
        };

        if constexpr (IS16) {
            constexpr int KQ = BK / 16;
#pragma unroll
            for (int kq = 0; kq < KQ; ++kq) {
                u32x4 af[WBM], bf[WBN];
#pragma unroll
                for (int i = 0; i < WBM; ++i)
                    af[i] = *reinterpret_cast<const u32x4*>(sA + (((wm * WBM + i) * R + lr) * SA + kq * G + lg) * 16);
#pragma unroll
                for (int j = 0; j < WBN; ++j)
                    bf[j] = *reinterpret_cast<const u32x4*>(sB + (((wn * WBN + j) * R + lr) * SB + kq * G + lg) * 16);
#pragma unroll
                for (int i = 0; i < WBM; ++i)
#pragma unroll
                    for (int j = 0; j < WBN; ++j) E::mma(acc[i][j], af[i], bf[j]);
                gather_slice(kq);
            }
        } else {
            constexpr int KQ = BK / (G * VE);
            typedef T TVA __attribute__((ext_vector_type(WBM)));
            typedef T TVB __attribute__((ext_vector_type(WBN)));
            typedef T TVE __attribute__((ext_vector_type(VE)));
#pragma unroll
            for (int kq = 0; kq < KQ; ++kq) {
                T af[WBM][VE], bf[WBN][VE];
                // Float32: MFMA e of the group multiplies k = 2 e (lanes 0..31) and 2 e + 1 (lanes 32..63), two fused
                // multiply-adds in that order per output element, so that every element is the chain c = fma(a_k, b_k, c) in
                // ascending k -- the order of the DMA-fed kernel and of the reference.  A K-major fragment arrives as
                // k 0..3 | k 4..7 and is rearranged with two v_permlane32_swap; an MN-major one is read that way.
                constexpr bool ASC = sizeof(T) == 4;
                auto ascend = [](T (&f)[VE]) {
                    if constexpr (ASC) {
                        typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
                        const u32x2 a = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(uint32_t, f[0]), __builtin_bit_cast(uint32_t, f[1]), false, false);
                        const u32x2 c = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(uint32_t, f[2]), __builtin_bit_cast(uint32_t, f[3]), false, false);
                        const uint32_t a0 = a[0], a1 = a[1], c0 = c[0], c1 = c[1];
                        f[0] = __builtin_bit_cast(T, a0); f[1] = __builtin_bit_cast(T, c0); f[2] = __builtin_bit_cast(T, a1); f[3] = __builtin_bit_cast(T, c1);
                    }
                };
                if constexpr (A_KM) {
#pragma unroll
                    for (int i = 0; i < WBM; ++i) {
                        const TVE t = *reinterpret_cast<const TVE*>(sA + (((wm * WBM + i) * R + lr) * SA + kq * G + lg) * 16);
#pragma unroll
                        for (int e = 0; e < VE; ++e) af[i][e] = t[e];
                        ascend(af[i]);
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < VE; ++e) {
                        const int krow = ASC ? kq * G * VE + e * G + lg : (kq * G + lg) * VE + e;
                        const TVA t = *reinterpret_cast<const TVA*>(sA + ((int)sizeof(T)) * (krow * BM + (wm * R + lr) * WBM));
#pragma unroll
                        for (int i = 0; i < WBM; ++i) af[i][e] = t[i];
                    }
                }
                if constexpr (B_KM) {
#pragma unroll
                    for (int j = 0; j < WBN; ++j) {
                        const TVE t = *reinterpret_cast<const TVE*>(sB + (((wn * WBN + j) * R + lr) * SB + kq * G + lg) * 16);
#pragma unroll
                        for (int e = 0; e < VE; ++e) bf[j][e] = t[e];
                        ascend(bf[j]);
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < VE; ++e) {
                        const int krow = ASC ? kq * G * VE + e * G + lg : (kq * G + lg) * VE + e;
                        const TVB t = *reinterpret_cast<const TVB*>(sB + ((int)sizeof(T)) * (krow * BN + (wn * R + lr) * WBN));
#pragma unroll
                        for (int j = 0; j < WBN; ++j) bf[j][e] = t[j];
                    }
                }
#pragma unroll
                for (int e = 0; e < VE; ++e) {
#pragma unroll
                    for (int i = 0; i < WBM; ++i)
#pragma unroll
                        for (int j = 0; j < WBN; ++j) E::mma(acc[i][j], af[i][e], bf[j][e]);
                    gather_slice(kq * VE + e);
                }
            }
        }
        if (more) {
            char* dA = smem + ((kt + 1) & 1) * SH::STAGE;
            if constexpr (CONV != 0) {
                // the gathered values are first touched here, after the MFMAs of this tile
                __builtin_amdgcn_sched_barrier(0);
                lb.conv_finish();
            }
            la.store(dA, tid);
            lb.store(dA + SH::LDS_A, tid);
        }
        __syncthreads();
    }

    // epilogue: every lane owns ACCN elements per block; C0 comes from C (accumulate),
    // from the broadcast bias (linear) or is zero (overwrite)
    const int cmode = p.cmode;
    const gptr<T> bias = (gptr<T>)static_cast<const T*>(p.bias);
#pragma unroll
    for (int i = 0; i < WBM; ++i) {
#pragma unroll
        for (int j = 0; j < WBN; ++j) {
            const int n = n0 + (B_KM ? (wn * WBN + j) * R + lr : (wn * R + lr) * WBN + j);
#pragma unroll
            for (int r = 0; r < E::ACCN; ++r) {
                const int lrow = acc_row<R>(r, lane);
                const int m = m0 + (A_KM ? (wm * WBM + i) * R + lrow : (wm * R + lrow) * WBM + i);
                if ((ALIGNED && CONV == 0) || (m < p.M && n < p.N)) {
                    const gptr_mut<T> cp = C + (int64_t)m * p.ldc + n;
                    AccS val = acc[i][j][r];
                    if constexpr (!CHAIN_FROM_C0) {
                        if (cmode == C_ACCUMULATE) val += (AccS)(*cp);
                        else if (cmode == C_BIAS) val += (AccS)bias[(int64_t)b * p.bias_bs + (int64_t)m * p.bias_rs + (int64_t)n * p.bias_cs];
                    }
                    *cp = (T)val;
                }
            }
        }
    }
}

template <int DT, bool TA, bool TB, int WBM, int WBN, int BK>
static hipError_t launch_cfg(const GemmParams& pin, hipStream_t s) {
    using SH = GemmShape<DT, TA, TB, WBM, WBN, BK>;
    GemmParams p = pin;
    p.tiles_m = (p.M + SH::BM - 1) / SH::BM;
    p.tiles_n = (p.N + SH::BN - 1) / SH::BN;
    const int64_t blocks = (int64_t)p.tiles_m * p.tiles_n * p.batch;
    if (blocks <= 0) return hipSuccess;
    if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
    constexpr int VE = Elem<DT>::VE;
    const bool aligned = (p.M % SH::BM == 0) && (p.N % SH::BN == 0) && (p.K % BK == 0) &&
                         p.vecA_ok && p.vecB_ok && !p.Aptr && !p.Bptr &&
                         ((reinterpret_cast<uintptr_t>(p.A) & 15) == 0) && ((reinterpret_cast<uintptr_t>(p.B) & 15) == 0) &&
                         (p.sA % VE == 0) && (p.sB % VE == 0);
    // tiles above 64 KiB of LDS need the opt-in once per kernel
    if (aligned) {
        auto k = gemm_mfma_kernel<DT, TA, TB, WBM, WBN, BK, true>;
        static hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize, SH::LDS_TOTAL);
        if (attr != hipSuccess) return attr;
        hipLaunchKernelGGL(k, dim3((unsigned)blocks), dim3(256), SH::LDS_TOTAL, s, p);
    } else {
        auto k = gemm_mfma_kernel<DT, TA, TB, WBM, WBN, BK, false>;
        static hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize, SH::LDS_TOTAL);
        if (attr != hipSuccess) return attr;
        hipLaunchKernelGGL(k, dim3((unsigned)blocks), dim3(256), SH::LDS_TOTAL, s, p);
    }
    return hipGetLastError();
}

// op(B) = implicit im2col matrix (TB: transposed).  ALIGNED here speaks of A only (whole tiles,
// 16-byte rows); the gathered operand and the stores are always guarded.
template <int DT, bool TB, int ND, int WBM, int WBN, int BK>
static hipError_t launch_conv_cfg(const GemmParams& pin, hipStream_t s) {
    using SH = GemmShape<DT, false, TB, WBM, WBN, BK>;
    GemmParams p = pin;
    p.tiles_m = (p.M + SH::BM - 1) / SH::BM;
    p.tiles_n = (p.N + SH::BN - 1) / SH::BN;
    const int64_t blocks = (int64_t)p.tiles_m * p.tiles_n * p.batch;
    if (blocks <= 0) return hipSuccess;
    if (blocks > 0x7fffffffLL) return hipErrorInvalidValue;
    constexpr int VE = Elem<DT>::VE;
    const bool a_aligned = (p.M % SH::BM == 0) && (p.K % BK == 0) && p.vecA_ok && !p.Aptr &&
                           ((reinterpret_cast<uintptr_t>(p.A) & 15) == 0) && (p.sA % VE == 0);
    if (a_aligned) {
        auto k = gemm_mfma_kernel<DT, false, TB, WBM, WBN, BK, true, ND>;
        static hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize, SH::LDS_TOTAL);
        if (attr != hipSuccess) return attr;
        hipLaunchKernelGGL(k, dim3((unsigned)blocks), dim3(256), SH::LDS_TOTAL, s, p);
    } else {
        auto k = gemm_mfma_kernel<DT, false, TB, WBM, WBN, BK, false, ND>;
        static hipError_t attr = hipFuncSetAttribute(reinterpret_cast<const void*>(k), hipFuncAttributeMaxDynamicSharedMemorySize, SH::LDS_TOTAL);
        if (attr != hipSuccess) return attr;
        hipLaunchKernelGGL(k, dim3((unsigned)blocks), dim3(256), SH::LDS_TOTAL, s, p);
    }
    return hipGetLastError();
}

template <int DT, int WBM, int WBN, int BK>
static hipError_t launch_trans(bool ta, bool tb, const GemmParams& p, hipStream_t s) {
    if (ta) return tb ? launch_cfg<DT, true, true, WBM, WBN, BK>(p, s) : launch_cfg<DT, true, false, WBM, WBN, BK>(p, s);
    return tb ? launch_cfg<DT, false, true, WBM, WBN, BK>(p, s) : launch_cfg<DT, false, false, WBM, WBN, BK>(p, s);
}

}  // namespace ntg
