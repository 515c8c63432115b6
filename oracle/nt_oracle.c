/*
 * nt_oracle.c -- CPU restatement of NeuroTensor's dense matmult path.
 * TEST INFRASTRUCTURE ONLY (see nt_oracle.h): the checker, never the product.
 *
 * Build: see oracle/Makefile (gcc -O2 -mavx2 -mfma -mf16c -ffp-contract=off -fopenmp).
 * -ffp-contract=off keeps every rounding where the source puts it; the only
 * fused operations are the explicit fmaf()/fma()/_mm256_fmadd_* calls, which
 * is what the reference's SimdTraits<T>::fmadd lowers to on an AVX2+FMA host
 * (nt/mp/simde_traits/simde_traits_avx2.h:250-256 fp32, :366-372 fp64,
 * :1230-1236 fp16-as-fp32, :444-446 int32, :523-540 int64).
 */
#include "nt_oracle.h"

#include <immintrin.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------------- */
/* 16-bit float conversions (software, round-to-nearest-even)                */
/* ------------------------------------------------------------------------- */

static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* IEEE binary16 <- binary32, RNE; same result as vcvtps2ph imm=0, the store
 * the reference uses for Float16 tiles (simde_traits_avx2.h:1160-1165). */
uint16_t oracle_f32_to_f16(float f) {
    uint32_t x = f32_bits(f);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t ax = x & 0x7fffffffu;
    if (ax >= 0x7f800000u) {                       /* inf / nan */
        if (ax > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((ax >> 13) & 0x3ffu));
        return (uint16_t)(sign | 0x7c00u);
    }
    if (ax >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);  /* rounds to >= 65520 -> inf */
    if (ax < 0x33000001u) return (uint16_t)sign;   /* <= 2^-25 rounds to 0 (ties-to-even) */
    int32_t e = (int32_t)(ax >> 23) - 127;
    uint32_t man = (ax & 0x7fffffu) | 0x800000u;   /* 24-bit significand */
    uint32_t shift;
    uint32_t half_exp;
    if (e < -14) { shift = (uint32_t)(13 + (-14 - e)); half_exp = 0; }
    else { shift = 13; half_exp = (uint32_t)(e + 15); }
    uint32_t q = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1u))) q++;
    uint32_t h;
    if (half_exp == 0) h = q;                       /* subnormal; q may carry into exp=1 */
    else h = ((half_exp - 1) << 10) + q;            /* q carries the implicit bit (0x400) */
    return (uint16_t)(sign | h);
}

/* binary32 <- binary16, exact (vcvtph2ps, simde_traits_avx2.h:1133-1138) */
float oracle_f16_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1fu;
    uint32_t m = h & 0x3ffu;
    uint32_t out;
    if (e == 0) {
        if (m == 0) out = sign;
        else {
            int sh = 0;
            while (!(m & 0x400u)) { m <<= 1; sh++; }
            m &= 0x3ffu;
            out = sign | ((uint32_t)(127 - 15 - sh + 1) << 23) | (m << 13);
        }
    } else if (e == 31) out = sign | 0x7f800000u | (m << 13);
    else out = sign | ((e + 112u) << 23) | (m << 13);
    return bits_f32(out);
}

/* bfloat16 <- binary32, RNE.  The reference's bfloat16_t struct truncates
 * (nt/types/bfloat16.h:20-24) but it is not a DType and has no matmult; this
 * build's BFloat16 extension rounds to nearest even like the GPU's convert. */
uint16_t oracle_f32_to_bf16(float f) {
    uint32_t x = f32_bits(f);
    if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u);
    uint32_t lsb = (x >> 16) & 1u;
    x += 0x7fffu + lsb;
    return (uint16_t)(x >> 16);
}
float oracle_bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

int64_t oracle_elem_size(int dt) {
    switch (dt) {
    case OR_I8: case OR_U8: return 1;
    case OR_F16: case OR_F16_LANE8: case OR_BF16: case OR_I16: case OR_U16: return 2;
    case OR_F32: case OR_I32: case OR_U32: return 4;
    case OR_F64: case OR_I64: case OR_U64: return 8;
    case OR_C32: return 4;
    case OR_C64: return 8;
    case OR_C128: return 16;
    default: return 0;
    }
}

/* ------------------------------------------------------------------------- */
/* Closed form.  Element access is the four index forms of matmult_naive      */
/* (nt_matmult.hpp:249,261,274,286):                                          */
/*   A(i,kk) = ta ? A[kk*m + i] : A[i*k + kk]                                 */
/*   B(kk,j) = tb ? B[j*k + kk] : B[kk*n + j]                                 */
/*   C(i,j)  = C[i*n + j], accumulated in place                               */
/* Per element: c = C0; for kk = 0..k-1 ascending: c = fma(A(i,kk),B(kk,j),c) */
/* which is what the packed path computes, because k tiles are visited in     */
/* ascending order (nt_matmult.hpp:196) and inside a tile kk ascends          */
/* (nt_matmult_simde.hpp:338-340, second_loop_direct_2 :272-277), and the     */
/* zero padded tail steps are fma(0,0,c) == c.                                */
/* ------------------------------------------------------------------------- */

/* B(kk, :) as a contiguous row: copies the stored-transposed operand once.
 * A pure relayout, no arithmetic. */
static void* rowmajor_kn(const void* B, int64_t k, int64_t n, int tb, int64_t es) {
    if (!tb) return (void*)B;
    char* out = (char*)malloc((size_t)(k * n * es));
    const char* src = (const char*)B;
    for (int64_t j = 0; j < n; ++j)
        for (int64_t kk = 0; kk < k; ++kk)
            memcpy(out + (kk * n + j) * es, src + (j * k + kk) * es, (size_t)es);
    return out;
}

#define A_IDX(i, kk) (ta ? ((kk) * m + (i)) : ((i) * k + (kk)))

static void closed_f32(const float* A, const float* Bkn, float* C, int64_t m, int64_t k, int64_t n, int ta) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < m; ++i) {
        float* c = C + i * n;
        for (int64_t kk = 0; kk < k; ++kk) {
            const float a = A[A_IDX(i, kk)];
            const float* b = Bkn + kk * n;
            for (int64_t j = 0; j < n; ++j) c[j] = fmaf(a, b[j], c[j]);
        }
    }
}

static void closed_f64(const double* A, const double* Bkn, double* C, int64_t m, int64_t k, int64_t n, int ta) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < m; ++i) {
        double* c = C + i * n;
        for (int64_t kk = 0; kk < k; ++kk) {
            const double a = A[A_IDX(i, kk)];
            const double* b = Bkn + kk * n;
            for (int64_t j = 0; j < n; ++j) c[j] = fma(a, b[j], c[j]);
        }
    }
}

/* Float16: lanes are fp32 inside a 16-wide k tile; C is widened on load and
 * narrowed (RNE) on store once per k tile (nt_matmult_simde.hpp:316-349 with
 * tile_size 16 = 2*pack 8, simde_traits_avx2.h:1130-1132). */
static void closed_f16_tile(const uint16_t* A, const uint16_t* Bkn, uint16_t* C, int64_t m, int64_t k, int64_t n, int ta, int64_t tile) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < m; ++i) {
        float* acc = (float*)malloc((size_t)n * sizeof(float));
        uint16_t* c = C + i * n;
        for (int64_t k0 = 0; k0 < k; k0 += tile) {
            const int64_t k1 = (k0 + tile < k) ? k0 + tile : k;
            for (int64_t j = 0; j < n; ++j) acc[j] = oracle_f16_to_f32(c[j]);
            for (int64_t kk = k0; kk < k1; ++kk) {
                const float a = oracle_f16_to_f32(A[A_IDX(i, kk)]);
                const uint16_t* b = Bkn + kk * n;
                for (int64_t j = 0; j < n; ++j) acc[j] = fmaf(a, oracle_f16_to_f32(b[j]), acc[j]);
            }
            for (int64_t j = 0; j < n; ++j) c[j] = oracle_f32_to_f16(acc[j]);
        }
        free(acc);
    }
}

static void closed_f16(const uint16_t* A, const uint16_t* Bkn, uint16_t* C, int64_t m, int64_t k, int64_t n, int ta) {
    closed_f16_tile(A, Bkn, C, m, k, n, ta, 16);
}
/* One lane (the real parts, or the imaginary parts) of a complex_32 product on its own: the same half values and float
 * chains as closed_c32 below, k tiles of 8 (OR_F16_LANE8; used to restate the complex convolutions plane by plane). */
static void closed_f16_lane8(const uint16_t* A, const uint16_t* Bkn, uint16_t* C, int64_t m, int64_t k, int64_t n, int ta) {
    closed_f16_tile(A, Bkn, C, m, k, n, ta, 8);
}

/* BFloat16 (this build's extension, no reference function): fp32 chain over
 * all of K starting from the widened C, one RNE narrowing at the end. */
static void closed_bf16(const uint16_t* A, const uint16_t* Bkn, uint16_t* C, int64_t m, int64_t k, int64_t n, int ta) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < m; ++i) {
        float* acc = (float*)malloc((size_t)n * sizeof(float));
        uint16_t* c = C + i * n;
        for (int64_t j = 0; j < n; ++j) acc[j] = oracle_bf16_to_f32(c[j]);
        for (int64_t kk = 0; kk < k; ++kk) {
            const float a = oracle_bf16_to_f32(A[A_IDX(i, kk)]);
            const uint16_t* b = Bkn + kk * n;
            for (int64_t j = 0; j < n; ++j) acc[j] = fmaf(a, oracle_bf16_to_f32(b[j]), acc[j]);
        }
        for (int64_t j = 0; j < n; ++j) c[j] = oracle_f32_to_bf16(acc[j]);
        free(acc);
    }
}

/* Integers: multiply and add wrap in the element width (mullo/add lanes,
 * simde_traits_avx2.h:444-446, 523-540, 590-592, 668-670, 810-812); computed
 * here in the unsigned type of the same width, which is the same residue. */
#define CLOSED_INT(NAME, UT)                                                                   \
    static void NAME(const UT* A, const UT* Bkn, UT* C, int64_t m, int64_t k, int64_t n, int ta) { \
        _Pragma("omp parallel for schedule(static)")                                           \
        for (int64_t i = 0; i < m; ++i) {                                                      \
            UT* c = C + i * n;                                                                 \
            for (int64_t kk = 0; kk < k; ++kk) {                                               \
                const UT a = A[A_IDX(i, kk)];                                                  \
                const UT* b = Bkn + kk * n;                                                    \
                for (int64_t j = 0; j < n; ++j) c[j] = (UT)(c[j] + (UT)(a * b[j]));            \
            }                                                                                  \
        }                                                                                      \
    }
CLOSED_INT(closed_u8, uint8_t)
CLOSED_INT(closed_u16, uint16_t)
CLOSED_INT(closed_u32, uint32_t)
CLOSED_INT(closed_u64, uint64_t)

/* Complex types.  The reference runs them through the SAME generic micro kernel
 * (nt_matmult_simde.hpp:301-350): a C tile row is two vectors of interleaved
 * (re, im) lanes; broadcast(A + kk) = set1(a) fills a vector with (a.re, a.im,
 * a.re, a.im, ...) (simde_traits_avx2.h:928-937 complex_64, :1037-1044
 * complex_128, :1285-1294 and :1365 complex_32 -- set_ps lists lanes from the
 * highest down, so lane 2t holds re and lane 2t+1 im, the memory order of
 * my_complex {re, im}, nt/types/complex.h:109); fmadd is the plain lane-wise
 * _mm256_fmadd_ps / _pd (:996-1002, :1106-1112, :1367-1373).  Hence per element
 *     c.re = fma(a.re, b.re, c.re);   c.im = fma(a.im, b.im, c.im)
 * for kk ascending: two independent real products, one on the real parts and
 * one on the imaginary parts -- NOT the complex product.  complex_32 keeps
 * float lanes inside a k tile of 2 * pack_size = 8 (pack_size 4, :1275) and
 * converts half <-> float at the tile's load / store (:1276-1303), so it rounds
 * to half every 8 k.  No test of the reference pins a complex matmult value:
 * parity unpinned by any reference fixture; the restatement follows the code. */
static void closed_c64(const float* A, const float* Bkn, float* C, int64_t m, int64_t k, int64_t n, int ta) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < m; ++i) {
        float* c = C + 2 * i * n;
        for (int64_t kk = 0; kk < k; ++kk) {
            const float* a = A + 2 * A_IDX(i, kk);
            const float* b = Bkn + 2 * kk * n;
            for (int64_t j = 0; j < 2 * n; ++j) c[j] = fmaf(a[j & 1], b[j], c[j]);
        }
    }
}
static void closed_c128(const double* A, const double* Bkn, double* C, int64_t m, int64_t k, int64_t n, int ta) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < m; ++i) {
        double* c = C + 2 * i * n;
        for (int64_t kk = 0; kk < k; ++kk) {
            const double* a = A + 2 * A_IDX(i, kk);
            const double* b = Bkn + 2 * kk * n;
            for (int64_t j = 0; j < 2 * n; ++j) c[j] = fma(a[j & 1], b[j], c[j]);
        }
    }
}
static void closed_c32(const uint16_t* A, const uint16_t* Bkn, uint16_t* C, int64_t m, int64_t k, int64_t n, int ta) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < m; ++i) {
        float* acc = (float*)malloc((size_t)(2 * n) * sizeof(float));
        uint16_t* c = C + 2 * i * n;
        for (int64_t k0 = 0; k0 < k; k0 += 8) {
            const int64_t k1 = (k0 + 8 < k) ? k0 + 8 : k;
            for (int64_t j = 0; j < 2 * n; ++j) acc[j] = oracle_f16_to_f32(c[j]);
            for (int64_t kk = k0; kk < k1; ++kk) {
                const uint16_t* a = A + 2 * A_IDX(i, kk);
                const float av[2] = {oracle_f16_to_f32(a[0]), oracle_f16_to_f32(a[1])};
                const uint16_t* b = Bkn + 2 * kk * n;
                for (int64_t j = 0; j < 2 * n; ++j) acc[j] = fmaf(av[j & 1], oracle_f16_to_f32(b[j]), acc[j]);
            }
            for (int64_t j = 0; j < 2 * n; ++j) c[j] = oracle_f32_to_f16(acc[j]);
        }
        free(acc);
    }
}

int oracle_matmult(int dt, const void* A, const void* B, void* C,
                   int64_t m, int64_t k, int64_t n, int ta, int tb) {
    const int64_t es = oracle_elem_size(dt);
    if (es == 0 || m < 0 || k < 0 || n < 0) return -1;
    if (m == 0 || n == 0 || k == 0) return 0;
    void* Bkn = rowmajor_kn(B, k, n, tb, es);
    switch (dt) {
    case OR_F32: closed_f32((const float*)A, (const float*)Bkn, (float*)C, m, k, n, ta); break;
    case OR_F64: closed_f64((const double*)A, (const double*)Bkn, (double*)C, m, k, n, ta); break;
    case OR_F16: closed_f16((const uint16_t*)A, (const uint16_t*)Bkn, (uint16_t*)C, m, k, n, ta); break;
    case OR_F16_LANE8: closed_f16_lane8((const uint16_t*)A, (const uint16_t*)Bkn, (uint16_t*)C, m, k, n, ta); break;
    case OR_BF16: closed_bf16((const uint16_t*)A, (const uint16_t*)Bkn, (uint16_t*)C, m, k, n, ta); break;
    case OR_I8: case OR_U8: closed_u8((const uint8_t*)A, (const uint8_t*)Bkn, (uint8_t*)C, m, k, n, ta); break;
    case OR_I16: case OR_U16: closed_u16((const uint16_t*)A, (const uint16_t*)Bkn, (uint16_t*)C, m, k, n, ta); break;
    case OR_I32: case OR_U32: closed_u32((const uint32_t*)A, (const uint32_t*)Bkn, (uint32_t*)C, m, k, n, ta); break;
    case OR_I64: case OR_U64: closed_u64((const uint64_t*)A, (const uint64_t*)Bkn, (uint64_t*)C, m, k, n, ta); break;
    case OR_C64: closed_c64((const float*)A, (const float*)Bkn, (float*)C, m, k, n, ta); break;
    case OR_C128: closed_c128((const double*)A, (const double*)Bkn, (double*)C, m, k, n, ta); break;
    case OR_C32: closed_c32((const uint16_t*)A, (const uint16_t*)Bkn, (uint16_t*)C, m, k, n, ta); break;
    default: if (tb) free(Bkn); return -1;
    }
    if (tb) free(Bkn);
    return 0;
}

int oracle_matmult_batch(int dt, const void* const* A, const void* const* B, void* const* C,
                         int64_t batches, int64_t m, int64_t k, int64_t n, int ta, int tb) {
    /* serial over items, pointers may repeat (nt_matmult.hpp:228-235) */
    for (int64_t b = 0; b < batches; ++b) {
        int rc = oracle_matmult(dt, A[b], B[b], C[b], m, k, n, ta, tb);
        if (rc) return rc;
    }
    return 0;
}

/* Literal triple loop with the reference's four index expressions
 * (nt_matmult.hpp:244-292); `C[..] += A[..] * B[..]` is evaluated with the
 * same fused step as the packed path so the two agree bit for bit. */
#define NAIVE_LOOP(T, STEP)                                                        \
    do {                                                                           \
        const T* a_ = (const T*)A; const T* b_ = (const T*)B; T* c_ = (T*)C;       \
        for (int64_t i = 0; i < m; ++i)                                            \
            for (int64_t j = 0; j < n; ++j)                                        \
                for (int64_t kk = 0; kk < k; ++kk) {                               \
                    const T av = ta ? a_[kk * m + i] : a_[i * k + kk];             \
                    const T bv = tb ? b_[j * k + kk] : b_[kk * n + j];             \
                    T* cp = &c_[i * n + j];                                        \
                    STEP;                                                          \
                }                                                                  \
    } while (0)

int oracle_matmult_naive(int dt, const void* A, const void* B, void* C,
                         int64_t m, int64_t k, int64_t n, int ta, int tb) {
    switch (dt) {
    case OR_F32: NAIVE_LOOP(float, *cp = fmaf(av, bv, *cp)); return 0;
    case OR_F64: NAIVE_LOOP(double, *cp = fma(av, bv, *cp)); return 0;
    case OR_I8: case OR_U8: NAIVE_LOOP(uint8_t, *cp = (uint8_t)(*cp + (uint8_t)(av * bv))); return 0;
    case OR_I16: case OR_U16: NAIVE_LOOP(uint16_t, *cp = (uint16_t)(*cp + (uint16_t)(av * bv))); return 0;
    case OR_I32: case OR_U32: NAIVE_LOOP(uint32_t, *cp = *cp + av * bv); return 0;
    case OR_I64: case OR_U64: NAIVE_LOOP(uint64_t, *cp = *cp + av * bv); return 0;
    case OR_F16: {
        /* per element: widen C, up to 16 fused steps in fp32, narrow; repeat */
        const uint16_t* a_ = (const uint16_t*)A; const uint16_t* b_ = (const uint16_t*)B; uint16_t* c_ = (uint16_t*)C;
        for (int64_t i = 0; i < m; ++i)
            for (int64_t j = 0; j < n; ++j)
                for (int64_t k0 = 0; k0 < k; k0 += 16) {
                    float acc = oracle_f16_to_f32(c_[i * n + j]);
                    for (int64_t kk = k0; kk < k0 + 16 && kk < k; ++kk) {
                        const uint16_t av = ta ? a_[kk * m + i] : a_[i * k + kk];
                        const uint16_t bv = tb ? b_[j * k + kk] : b_[kk * n + j];
                        acc = fmaf(oracle_f16_to_f32(av), oracle_f16_to_f32(bv), acc);
                    }
                    c_[i * n + j] = oracle_f32_to_f16(acc);
                }
        return 0;
    }
    case OR_BF16: {
        const uint16_t* a_ = (const uint16_t*)A; const uint16_t* b_ = (const uint16_t*)B; uint16_t* c_ = (uint16_t*)C;
        for (int64_t i = 0; i < m; ++i)
            for (int64_t j = 0; j < n; ++j) {
                float acc = oracle_bf16_to_f32(c_[i * n + j]);
                for (int64_t kk = 0; kk < k; ++kk) {
                    const uint16_t av = ta ? a_[kk * m + i] : a_[i * k + kk];
                    const uint16_t bv = tb ? b_[j * k + kk] : b_[kk * n + j];
                    acc = fmaf(oracle_bf16_to_f32(av), oracle_bf16_to_f32(bv), acc);
                }
                c_[i * n + j] = oracle_f32_to_bf16(acc);
            }
        return 0;
    }
    case OR_C64: case OR_C128: case OR_C32: {
        /* the literal loop on (re, im) pairs; complex_32 in k tiles of 8 */
        for (int64_t i = 0; i < m; ++i)
            for (int64_t j = 0; j < n; ++j)
                for (int c = 0; c < 2; ++c) {
                    const int64_t ci = 2 * (i * n + j) + c;
                    if (dt == OR_C64) {
                        float acc = ((float*)C)[ci];
                        for (int64_t kk = 0; kk < k; ++kk)
                            acc = fmaf(((const float*)A)[2 * (ta ? kk * m + i : i * k + kk) + c], ((const float*)B)[2 * (tb ? j * k + kk : kk * n + j) + c], acc);
                        ((float*)C)[ci] = acc;
                    } else if (dt == OR_C128) {
                        double acc = ((double*)C)[ci];
                        for (int64_t kk = 0; kk < k; ++kk)
                            acc = fma(((const double*)A)[2 * (ta ? kk * m + i : i * k + kk) + c], ((const double*)B)[2 * (tb ? j * k + kk : kk * n + j) + c], acc);
                        ((double*)C)[ci] = acc;
                    } else {
                        uint16_t* c_ = (uint16_t*)C;
                        for (int64_t k0 = 0; k0 < k; k0 += 8) {
                            float acc = oracle_f16_to_f32(c_[ci]);
                            for (int64_t kk = k0; kk < k0 + 8 && kk < k; ++kk)
                                acc = fmaf(oracle_f16_to_f32(((const uint16_t*)A)[2 * (ta ? kk * m + i : i * k + kk) + c]),
                                           oracle_f16_to_f32(((const uint16_t*)B)[2 * (tb ? j * k + kk : kk * n + j) + c]), acc);
                            c_[ci] = oracle_f32_to_f16(acc);
                        }
                    }
                }
        return 0;
    }
    default: return -1;
    }
}

/* ------------------------------------------------------------------------- */
/* Tiled restatement of pack_multiply_directly_var_threaded                   */
/* (nt_matmult.hpp:124-225): TILE = 2*pack (nt_matmult_simde.hpp:34-35),      */
/* pack block PB = TILE*21*21 rows/cols (:138-142), k tile OUTERMOST (:196),  */
/* A block repacked per (k,i) (:201), B block per (k,i,j) (:205), a parallel  */
/* 2-D sweep over TILE x TILE tiles of C (:206-217), each tile loading C,     */
/* doing TILE fused steps per row and storing C (nt_matmult_simde.hpp:316-349)*/
/* Threads are capped at 21 (nt_matmult_macros.h:42, nt_matmult.hpp:129).     */
/* ------------------------------------------------------------------------- */

#define NT_THREAD_CAP 21

int oracle_tiled_threads(int threads) {
    int hw = 1;
#ifdef _OPENMP
    hw = omp_get_num_procs();
#endif
    if (threads <= 0) threads = hw;
    if (threads > NT_THREAD_CAP) threads = NT_THREAD_CAP;
    if (threads < 1) threads = 1;
    return threads;
}

/* pack_threaded (nt_matmult.hpp:84-96): ROWS x COLS block of a row-major
 * source starting at (start_row,start_col), zero padded on both edges. */
#define DEFINE_PACKERS(SFX, T)                                                                            \
    static void pack_##SFX(const T* src, T* block, int64_t ROWS, int64_t COLS, int64_t start_row,         \
                           int64_t start_col, int64_t src_rows, int64_t src_cols, int nt) {               \
        int64_t maxr = src_rows - start_row; if (maxr > ROWS) maxr = ROWS;                                \
        int64_t ncol = src_cols - start_col; if (ncol > COLS) ncol = COLS;                                \
        const T* s = src + start_row * src_cols + start_col;                                              \
        _Pragma("omp parallel for schedule(static) num_threads(nt)")                                      \
        for (int64_t i = 0; i < maxr; ++i) {                                                              \
            T* d = block + i * COLS;                                                                      \
            memcpy(d, s + i * src_cols, (size_t)ncol * sizeof(T));                                        \
            for (int64_t c = ncol; c < COLS; ++c) d[c] = (T)0;                                            \
        }                                                                                                 \
        memset(block + maxr * COLS, 0, (size_t)((ROWS - maxr) * COLS) * sizeof(T));                       \
    }                                                                                                     \
    /* pack_transpose_threaded (nt_matmult.hpp:109-122): the source is stored transposed               */ \
    /* ([block cols, block rows]); the whole block is zeroed first, then filled column by column.      */ \
    static void packT_##SFX(const T* src, T* block, int64_t ROWS, int64_t COLS, int64_t start_col,        \
                            int64_t start_row, int64_t src_cols, int64_t src_rows, int nt) {              \
        int64_t maxr = src_rows - start_row; if (maxr > COLS) maxr = COLS;                                \
        int64_t ncol = src_cols - start_col; if (ncol > ROWS) ncol = ROWS;                                \
        const T* s = src + start_row * src_cols + start_col;                                              \
        memset(block, 0, (size_t)(ROWS * COLS) * sizeof(T));                                              \
        _Pragma("omp parallel for schedule(static) num_threads(nt)")                                      \
        for (int64_t r = 0; r < maxr; ++r) {                                                              \
            const T* sr = s + r * src_cols;                                                               \
            for (int64_t c = 0; c < ncol; ++c) block[c * COLS + r] = sr[c];                               \
        }                                                                                                 \
    }
DEFINE_PACKERS(b16, uint16_t)
DEFINE_PACKERS(b32, uint32_t)
DEFINE_PACKERS(b64, uint64_t)

/* Micro kernels: C tile (rows x cols, ragged edges handled through a dense
 * TILE x TILE staging copy, which is what the masked loads/stores amount to)
 * += Apack[rows x TILE] . Bpack[TILE x TILE], B row stride = PB. */

static void micro_f32(const float* Ap, const float* Bp, int64_t PB, float* C, int64_t ldc, int64_t cols, int64_t rows) {
    enum { TILE = 16 };
    __m256 b0[TILE], b1[TILE];
    for (int kk = 0; kk < TILE; ++kk) { b0[kk] = _mm256_loadu_ps(Bp + kk * PB); b1[kk] = _mm256_loadu_ps(Bp + kk * PB + 8); }
    float tmp[TILE];
    for (int64_t i = 0; i < rows; ++i) {
        float* crow = C + i * ldc;
        __m256 c0, c1;
        if (cols == TILE) { c0 = _mm256_loadu_ps(crow); c1 = _mm256_loadu_ps(crow + 8); }
        else { memset(tmp, 0, sizeof tmp); memcpy(tmp, crow, (size_t)cols * 4); c0 = _mm256_loadu_ps(tmp); c1 = _mm256_loadu_ps(tmp + 8); }
        const float* a = Ap + i * TILE;
        for (int kk = 0; kk < TILE; ++kk) {
            const __m256 av = _mm256_broadcast_ss(a + kk);
            c0 = _mm256_fmadd_ps(av, b0[kk], c0);
            c1 = _mm256_fmadd_ps(av, b1[kk], c1);
        }
        if (cols == TILE) { _mm256_storeu_ps(crow, c0); _mm256_storeu_ps(crow + 8, c1); }
        else { _mm256_storeu_ps(tmp, c0); _mm256_storeu_ps(tmp + 8, c1); memcpy(crow, tmp, (size_t)cols * 4); }
    }
}

static void micro_f64(const double* Ap, const double* Bp, int64_t PB, double* C, int64_t ldc, int64_t cols, int64_t rows) {
    enum { TILE = 8 };
    __m256d b0[TILE], b1[TILE];
    for (int kk = 0; kk < TILE; ++kk) { b0[kk] = _mm256_loadu_pd(Bp + kk * PB); b1[kk] = _mm256_loadu_pd(Bp + kk * PB + 4); }
    double tmp[TILE];
    for (int64_t i = 0; i < rows; ++i) {
        double* crow = C + i * ldc;
        __m256d c0, c1;
        if (cols == TILE) { c0 = _mm256_loadu_pd(crow); c1 = _mm256_loadu_pd(crow + 4); }
        else { memset(tmp, 0, sizeof tmp); memcpy(tmp, crow, (size_t)cols * 8); c0 = _mm256_loadu_pd(tmp); c1 = _mm256_loadu_pd(tmp + 4); }
        const double* a = Ap + i * TILE;
        for (int kk = 0; kk < TILE; ++kk) {
            const __m256d av = _mm256_broadcast_sd(a + kk);
            c0 = _mm256_fmadd_pd(av, b0[kk], c0);
            c1 = _mm256_fmadd_pd(av, b1[kk], c1);
        }
        if (cols == TILE) { _mm256_storeu_pd(crow, c0); _mm256_storeu_pd(crow + 4, c1); }
        else { _mm256_storeu_pd(tmp, c0); _mm256_storeu_pd(tmp + 4, c1); memcpy(crow, tmp, (size_t)cols * 8); }
    }
}

static void micro_f16(const uint16_t* Ap, const uint16_t* Bp, int64_t PB, uint16_t* C, int64_t ldc, int64_t cols, int64_t rows) {
    enum { TILE = 16 };
    __m256 b0[TILE], b1[TILE];
    for (int kk = 0; kk < TILE; ++kk) {
        b0[kk] = _mm256_cvtph_ps(_mm_loadu_si128((const __m128i*)(Bp + kk * PB)));
        b1[kk] = _mm256_cvtph_ps(_mm_loadu_si128((const __m128i*)(Bp + kk * PB + 8)));
    }
    uint16_t tmp[TILE];
    for (int64_t i = 0; i < rows; ++i) {
        uint16_t* crow = C + i * ldc;
        const uint16_t* cs = crow;
        if (cols != TILE) { memset(tmp, 0, sizeof tmp); memcpy(tmp, crow, (size_t)cols * 2); cs = tmp; }
        __m256 c0 = _mm256_cvtph_ps(_mm_loadu_si128((const __m128i*)cs));
        __m256 c1 = _mm256_cvtph_ps(_mm_loadu_si128((const __m128i*)(cs + 8)));
        const uint16_t* a = Ap + i * TILE;
        for (int kk = 0; kk < TILE; ++kk) {
            const __m256 av = _mm256_set1_ps(oracle_f16_to_f32(a[kk]));
            c0 = _mm256_fmadd_ps(av, b0[kk], c0);
            c1 = _mm256_fmadd_ps(av, b1[kk], c1);
        }
        uint16_t* cd = (cols == TILE) ? crow : tmp;
        _mm_storeu_si128((__m128i*)cd, _mm256_cvtps_ph(c0, 0));
        _mm_storeu_si128((__m128i*)(cd + 8), _mm256_cvtps_ph(c1, 0));
        if (cols != TILE) memcpy(crow, tmp, (size_t)cols * 2);
    }
}

static void micro_i32(const uint32_t* Ap, const uint32_t* Bp, int64_t PB, uint32_t* C, int64_t ldc, int64_t cols, int64_t rows) {
    enum { TILE = 16 };
    __m256i b0[TILE], b1[TILE];
    for (int kk = 0; kk < TILE; ++kk) {
        b0[kk] = _mm256_loadu_si256((const __m256i*)(Bp + kk * PB));
        b1[kk] = _mm256_loadu_si256((const __m256i*)(Bp + kk * PB + 8));
    }
    uint32_t tmp[TILE];
    for (int64_t i = 0; i < rows; ++i) {
        uint32_t* crow = C + i * ldc;
        const uint32_t* cs = crow;
        if (cols != TILE) { memset(tmp, 0, sizeof tmp); memcpy(tmp, crow, (size_t)cols * 4); cs = tmp; }
        __m256i c0 = _mm256_loadu_si256((const __m256i*)cs);
        __m256i c1 = _mm256_loadu_si256((const __m256i*)(cs + 8));
        const uint32_t* a = Ap + i * TILE;
        for (int kk = 0; kk < TILE; ++kk) {
            const __m256i av = _mm256_set1_epi32((int)a[kk]);
            c0 = _mm256_add_epi32(_mm256_mullo_epi32(av, b0[kk]), c0);
            c1 = _mm256_add_epi32(_mm256_mullo_epi32(av, b1[kk]), c1);
        }
        uint32_t* cd = (cols == TILE) ? crow : tmp;
        _mm256_storeu_si256((__m256i*)cd, c0);
        _mm256_storeu_si256((__m256i*)(cd + 8), c1);
        if (cols != TILE) memcpy(crow, tmp, (size_t)cols * 4);
    }
}

/* int64: the reference multiplies lane by lane in scalar code and adds with
 * add_epi64 (simde_traits_avx2.h:523-540): plain wrapping 64-bit arithmetic. */
static void micro_i64(const uint64_t* Ap, const uint64_t* Bp, int64_t PB, uint64_t* C, int64_t ldc, int64_t cols, int64_t rows) {
    enum { TILE = 8 };
    for (int64_t i = 0; i < rows; ++i) {
        uint64_t acc[TILE];
        uint64_t* crow = C + i * ldc;
        for (int j = 0; j < TILE; ++j) acc[j] = (j < cols) ? crow[j] : 0;
        const uint64_t* a = Ap + i * TILE;
        for (int kk = 0; kk < TILE; ++kk) {
            const uint64_t av = a[kk];
            const uint64_t* b = Bp + kk * PB;
            for (int j = 0; j < TILE; ++j) acc[j] += av * b[j];
        }
        for (int j = 0; j < cols; ++j) crow[j] = acc[j];
    }
}

#define DEFINE_TILED(SFX, T, PK, TILE_, MICRO)                                                                 \
    static int tiled_##SFX(const T* A, const T* B, T* C, int64_t m, int64_t k, int64_t n, int ta, int tb, int nt) { \
        const int64_t TILE = TILE_;                                                                            \
        const int64_t PB = TILE * NT_THREAD_CAP * NT_THREAD_CAP;                                               \
        T* Apack = (T*)aligned_alloc(64, (size_t)(PB * TILE) * sizeof(T));                                     \
        T* Bpack = (T*)aligned_alloc(64, (size_t)(PB * TILE) * sizeof(T));                                     \
        if (!Apack || !Bpack) { free(Apack); free(Bpack); return -2; }                                         \
        for (int64_t k0 = 0; k0 < k; k0 += TILE) {                                                             \
            for (int64_t i0 = 0; i0 < m; i0 += PB) {                                                           \
                const int64_t irMax = (m - i0 < PB) ? m - i0 : PB;                                             \
                if (ta) packT_##PK((const void*)A, (void*)Apack, PB, TILE, i0, k0, m, k, nt);                  \
                else pack_##PK((const void*)A, (void*)Apack, PB, TILE, i0, k0, m, k, nt);                      \
                for (int64_t j0 = 0; j0 < n; j0 += PB) {                                                       \
                    const int64_t jrMax = (n - j0 < PB) ? n - j0 : PB;                                         \
                    if (tb) packT_##PK((const void*)B, (void*)Bpack, TILE, PB, k0, j0, k, n, nt);              \
                    else pack_##PK((const void*)B, (void*)Bpack, TILE, PB, k0, j0, k, n, nt);                  \
                    const int64_t irT = (irMax + TILE - 1) / TILE, jrT = (jrMax + TILE - 1) / TILE;            \
                    _Pragma("omp parallel for collapse(2) schedule(dynamic, 8) num_threads(nt)")               \
                    for (int64_t ir = 0; ir < irT; ++ir)                                                       \
                        for (int64_t jr = 0; jr < jrT; ++jr) {                                                 \
                            const int64_t rows = (irMax - ir * TILE < TILE) ? irMax - ir * TILE : TILE;        \
                            const int64_t cols = (jrMax - jr * TILE < TILE) ? jrMax - jr * TILE : TILE;        \
                            MICRO(Apack + ir * TILE * TILE, Bpack + jr * TILE, PB,                             \
                                  C + (i0 + ir * TILE) * n + j0 + jr * TILE, n, cols, rows);                   \
                        }                                                                                      \
                }                                                                                              \
            }                                                                                                  \
        }                                                                                                      \
        free(Apack); free(Bpack);                                                                              \
        return 0;                                                                                              \
    }

/* the packers are typed by element width only */
static void pack_b16v(const void* s, void* b, int64_t R, int64_t Cc, int64_t sr, int64_t sc, int64_t nr, int64_t nc, int nt) { pack_b16((const uint16_t*)s, (uint16_t*)b, R, Cc, sr, sc, nr, nc, nt); }
static void packT_b16v(const void* s, void* b, int64_t R, int64_t Cc, int64_t sc, int64_t sr, int64_t ncol, int64_t nrow, int nt) { packT_b16((const uint16_t*)s, (uint16_t*)b, R, Cc, sc, sr, ncol, nrow, nt); }
static void pack_b32v(const void* s, void* b, int64_t R, int64_t Cc, int64_t sr, int64_t sc, int64_t nr, int64_t nc, int nt) { pack_b32((const uint32_t*)s, (uint32_t*)b, R, Cc, sr, sc, nr, nc, nt); }
static void packT_b32v(const void* s, void* b, int64_t R, int64_t Cc, int64_t sc, int64_t sr, int64_t ncol, int64_t nrow, int nt) { packT_b32((const uint32_t*)s, (uint32_t*)b, R, Cc, sc, sr, ncol, nrow, nt); }
static void pack_b64v(const void* s, void* b, int64_t R, int64_t Cc, int64_t sr, int64_t sc, int64_t nr, int64_t nc, int nt) { pack_b64((const uint64_t*)s, (uint64_t*)b, R, Cc, sr, sc, nr, nc, nt); }
static void packT_b64v(const void* s, void* b, int64_t R, int64_t Cc, int64_t sc, int64_t sr, int64_t ncol, int64_t nrow, int nt) { packT_b64((const uint64_t*)s, (uint64_t*)b, R, Cc, sc, sr, ncol, nrow, nt); }

DEFINE_TILED(f32, float, b32v, 16, micro_f32)
DEFINE_TILED(f64, double, b64v, 8, micro_f64)
DEFINE_TILED(f16, uint16_t, b16v, 16, micro_f16)
DEFINE_TILED(i32, uint32_t, b32v, 16, micro_i32)
DEFINE_TILED(i64, uint64_t, b64v, 8, micro_i64)

int oracle_tiled_matmult(int dt, const void* A, const void* B, void* C,
                         int64_t m, int64_t k, int64_t n, int ta, int tb, int threads) {
    const int nt = oracle_tiled_threads(threads);
    if (m <= 0 || n <= 0 || k <= 0) return (m < 0 || n < 0 || k < 0) ? -1 : 0;
    switch (dt) {
    case OR_F32: return tiled_f32((const float*)A, (const float*)B, (float*)C, m, k, n, ta, tb, nt);
    case OR_F64: return tiled_f64((const double*)A, (const double*)B, (double*)C, m, k, n, ta, tb, nt);
    case OR_F16: return tiled_f16((const uint16_t*)A, (const uint16_t*)B, (uint16_t*)C, m, k, n, ta, tb, nt);
    case OR_I32: case OR_U32: return tiled_i32((const uint32_t*)A, (const uint32_t*)B, (uint32_t*)C, m, k, n, ta, tb, nt);
    case OR_I64: case OR_U64: return tiled_i64((const uint64_t*)A, (const uint64_t*)B, (uint64_t*)C, m, k, n, ta, tb, nt);
    default: return -1;
    }
}

int oracle_tiled_matmult_batch(int dt, const void* const* A, const void* const* B, void* const* C,
                               int64_t batches, int64_t m, int64_t k, int64_t n, int ta, int tb, int threads) {
    for (int64_t b = 0; b < batches; ++b) {   /* serial over items: nt_matmult.hpp:228-235 */
        int rc = oracle_tiled_matmult(dt, A[b], B[b], C[b], m, k, n, ta, tb, threads);
        if (rc) return rc;
    }
    return 0;
}

/* ------------------------------------------------------------------------- */
/* im2col / col2im                                                            */
/* ------------------------------------------------------------------------- */

/* im2col_cpu, cpu/unfold2d.cpp:12-112.  col[b, c, h*Wo + w] with
 * c = c_im*kr*kc + i*kc + j  <-  im[b, c_im, h*s_r - p_r + i*d_r, w*s_c - p_c + j*d_c];
 * positions that fall in the padding are not written (col arrives zeroed,
 * colim_transform.cpp:581). */
int oracle_unfold2d(int64_t es, const void* im_, void* col_,
                    int64_t batch, int64_t channels, int64_t height, int64_t width,
                    int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c,
                    int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c) {
    const int64_t Ho = (height + 2 * p_r - d_r * (k_r - 1) - 1) / s_r + 1;
    const int64_t Wo = (width + 2 * p_c - d_c * (k_c - 1) - 1) / s_c + 1;
    if (Ho <= 0 || Wo <= 0) return -1;
    const int64_t ccol = channels * k_r * k_c;
    const char* im = (const char*)im_;
    char* col = (char*)col_;
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t b = 0; b < batch; ++b)
        for (int64_t c = 0; c < ccol; ++c) {
            const int64_t wo = c % k_c, ho = (c / k_c) % k_r, c_im = c / k_r / k_c;
            for (int64_t h = 0; h < Ho; ++h) {
                const int64_t hp = h * s_r - p_r + ho * d_r;
                if (hp < 0 || hp >= height) continue;
                for (int64_t w = 0; w < Wo; ++w) {
                    const int64_t wp = w * s_c - p_c + wo * d_c;
                    if (wp < 0 || wp >= width) continue;
                    memcpy(col + (((b * ccol + c) * Ho + h) * Wo + w) * es,
                           im + (((b * channels + c_im) * height + hp) * width + wp) * es, (size_t)es);
                }
            }
        }
    return 0;
}

/* im2col_backward_cpu, cpu/unfold2d_backward.cpp:9-56: scatter-add in the
 * order batch, c, h, w (that order fixes the floating point sum). */
int oracle_unfold2d_backward(int dt, const void* col_, void* im_,
                    int64_t batch, int64_t channels, int64_t height, int64_t width,
                    int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c,
                    int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c) {
    const int64_t Ho = (height + 2 * p_r - d_r * (k_r - 1) - 1) / s_r + 1;
    const int64_t Wo = (width + 2 * p_c - d_c * (k_c - 1) - 1) / s_c + 1;
    if (Ho <= 0 || Wo <= 0) return -1;
    if (dt != OR_F32 && dt != OR_F64) return -1;
    const int64_t ccol = channels * k_r * k_c;
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < batch; ++b)
        for (int64_t c = 0; c < ccol; ++c) {
            const int64_t wo = c % k_c, ho = (c / k_c) % k_r, c_im = c / k_r / k_c;
            for (int64_t h = 0; h < Ho; ++h)
                for (int64_t w = 0; w < Wo; ++w) {
                    const int64_t hp = h * s_r - p_r + ho * d_r;
                    const int64_t wp = w * s_c - p_c + wo * d_c;
                    if (hp < 0 || hp >= height || wp < 0 || wp >= width) continue;
                    const int64_t ci = ((b * ccol + c) * Ho + h) * Wo + w;
                    const int64_t ii = ((b * channels + c_im) * height + hp) * width + wp;
                    if (dt == OR_F32) ((float*)im_)[ii] += ((const float*)col_)[ci];
                    else ((double*)im_)[ii] += ((const double*)col_)[ci];
                }
        }
    return 0;
}
