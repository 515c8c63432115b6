/*
 * nt_oracle.h -- CPU restatement of NeuroTensor's dense matmult path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or
 * calls this code: it is the checker for the parity tests, the smoke test and
 * the "cpu_baseline" leg of the benchmark, never the product path.
 *
 * Every function names the reference file:line it restates.  Two families:
 *
 *   oracle_matmult*        closed form: per output element a sequential-k
 *                          chain  c <- op(c, A(i,k), B(k,j))  in the element
 *                          type, starting from the incoming C (accumulate
 *                          contract of nt_matmult, nt_matmult.hpp:370-378).
 *   oracle_tiled_matmult*  the reference's loop nest restated (k-tile
 *                          outermost, packed blocks, tile x tile micro kernel,
 *                          thread cap 21): nt_matmult.hpp:124-225 and
 *                          nt_matmult_simde.hpp:301-350.  Bitwise equal to the
 *                          closed form; it exists to be *timed* as the host
 *                          baseline and to check the closed form's claim.
 *
 * Pinning (see tests/test_oracle_*.py):
 *   fp32 linear grads / conv2d output+grads / unfold  <- the reference's own
 *       committed PyTorch fixtures (the .npy files under tests/golden).
 *   fp32/fp64 GEMM  <- numpy float64 GEMM, identity/permutation operands,
 *       explicit-transpose equivalence (bitwise), batch == per item (bitwise),
 *       tiled == closed form (bitwise), naive triple loop on tiny inputs.
 *   integer GEMM    <- exact modular arithmetic vs numpy/python big ints.
 *   fp16 GEMM       <- numpy float16 rounding of an independently computed
 *       chunked sum (16-wide k tiles), software half conversion checked
 *       against numpy for all 65536 bit patterns.
 *   complex GEMM    <- parity unpinned by any reference fixture (none holds a complex
 *       matmult value).  The reference's generic micro kernel multiplies the
 *       interleaved (re, im) lanes element-wise (simde_traits_avx2.h:928-937,
 *       :996-1002): the result is one real product of the real parts and one
 *       of the imaginary parts, not the complex product.  Pinned by that
 *       reduction (bitwise equal to the real oracle on the two planes), by a
 *       literal vector-lane walk of the micro kernel on tiny inputs, and, for
 *       complex_32, by an independent numpy restatement of the 8-wide k tiles.
 *   bf16 GEMM       <- parity unpinned: the reference has no BFloat16 DType
 *       (nt/types/bfloat16.h:4-5); this build defines it (fp32 accumulate over
 *       all K, one round-to-nearest-even at the end).
 */
#ifndef NT_ORACLE_H
#define NT_ORACLE_H
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* numeric values follow nt::DType (nt/dtype/DType_enum.h:14-20 expanded from
 * nt/dtype/compatible/DTypeDeclareMacros.h:5-33); BF16/U64 are extensions. */
enum oracle_dtype {
    OR_F16 = 0, OR_F32 = 1, OR_F64 = 2,
    OR_C32 = 4, OR_C64 = 5, OR_C128 = 6,      /* interleaved (re, im) pairs of half / float / double */
    OR_I8 = 7, OR_I16 = 8, OR_I32 = 9, OR_I64 = 10,
    OR_U8 = 12, OR_U16 = 13, OR_U32 = 14,
    OR_BF16 = 100, OR_U64 = 101,
    OR_F16_LANE8 = 200                        /* oracle_matmult only: half values, float chains rounded to half every 8 k (one lane of complex_32) */
};

int64_t oracle_elem_size(int dtype);

/* C[m,n] += op(A) . op(B); ta => A stored [k,m]; tb => B stored [n,k]. */
int oracle_matmult(int dtype, const void* A, const void* B, void* C,
                   int64_t m, int64_t k, int64_t n, int ta, int tb);
/* same arithmetic, literal i/j/k triple loop (nt_matmult.hpp:238-292 index forms) */
int oracle_matmult_naive(int dtype, const void* A, const void* B, void* C,
                         int64_t m, int64_t k, int64_t n, int ta, int tb);
int oracle_matmult_batch(int dtype, const void* const* A, const void* const* B, void* const* C,
                         int64_t batches, int64_t m, int64_t k, int64_t n, int ta, int tb);

/* the reference's blocked/packed/threaded loop nest; threads<=0 -> min(21, cores) */
int oracle_tiled_matmult(int dtype, const void* A, const void* B, void* C,
                         int64_t m, int64_t k, int64_t n, int ta, int tb, int threads);
int oracle_tiled_matmult_batch(int dtype, const void* const* A, const void* const* B, void* const* C,
                               int64_t batches, int64_t m, int64_t k, int64_t n, int ta, int tb, int threads);
int oracle_tiled_threads(int threads);

/* im2col, col[B, C*kh*kw, Ho*Wo] (cpu/unfold2d.cpp:12-112); col must be zeroed by the caller */
int oracle_unfold2d(int64_t elem_size, const void* im, void* col,
                    int64_t batch, int64_t channels, int64_t height, int64_t width,
                    int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c,
                    int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c);
/* col2im scatter-add into a zeroed/accumulating image (fp32 / fp64) */
int oracle_unfold2d_backward(int dtype, const void* col, void* im,
                    int64_t batch, int64_t channels, int64_t height, int64_t width,
                    int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c,
                    int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c);

/* half <-> float helpers exposed so the tests can pin them against numpy */
uint16_t oracle_f32_to_f16(float f);
float    oracle_f16_to_f32(uint16_t h);
uint16_t oracle_f32_to_bf16(float f);
float    oracle_bf16_to_f32(uint16_t h);

#ifdef __cplusplus
}
#endif
#endif
