/*
 * ntgemm.h -- C ABI of the MI355X (gfx950) backend for NeuroTensor's dense matmult path.
 *
 * The library behind this header replaces the reference's static library `nt_matmult`
 * (CMakeLists.txt:88-90, cmake/matmult_sources.cmake:3-21), whose only exports are the
 * per-dtype instantiations of
 *
 *   nt::functional::cpu::nt_matmult<T>        nt/functional/cpu/matmult/nt_matmult.h:6-7
 *   nt::functional::cpu::nt_matmult_batch<T>  nt/functional/cpu/matmult/nt_matmult.h:9-10
 *
 * and offers, for callers that keep their tensors in device memory, the fused forms the
 * layers above need (bias-initialised GEMM for cpu::linear, im2col + GEMM for conv2d).
 *
 * Conventions (identical to the reference, nt_matmult.hpp:238-292, 370-394):
 *   - all matrices are dense row-major; sizes are LOGICAL (after the transpose flags):
 *     a_rows = m, a_cols = b_rows = k, b_cols = n;
 *   - transpose_a != 0 means A is STORED [k, m]; transpose_b != 0 means B is STORED [n, k];
 *   - the GEMM ACCUMULATES: C[m, n] += op(A) . op(B); the caller initialises C;
 *   - A and B are read-only and may alias each other; C must not alias an input.
 *
 * Results against the reference's: the integer and complex types are bit-identical.  Float32 products are bit-identical too --
 * every element is the reference's chain c = C0; c = fma(a[i,k], b[k,j], c) in ascending k (nt_matmult.hpp:196: k tiles
 * outermost and ascending) -- through the host-pointer entry points always, through the device entry points unless a
 * workspace lets the product be split along k or it has at most 32 rows (NTG_GEMM_KEEP_K_ORDER switches both off), and so is
 * the Float32 convolution on the gathering kernels (no workspace: unfold + matmult, conv.cpp:86-95).  Float64, Float16 and
 * BFloat16 results agree to the bounds stated with the tests (their matrix instructions do not sum k in a chain).
 *
 * Every entry point returns 0 (NTG_OK) or a non-zero ntg_status and never throws;
 * ntg_last_error() returns a thread-local description of the last failure.
 * Host-pointer entry points are synchronous (results are in C on return) and thread-safe
 * (concurrent callers take turns on the library's staging buffers).
 * Device-pointer entry points (suffix _dev) enqueue on the given HIP stream and return.
 */
#ifndef NTGEMM_H
#define NTGEMM_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Values equal nt::DType (nt/dtype/DType_enum.h:14-20, expanded from
 * nt/dtype/compatible/DTypeDeclareMacros.h:5-33) so a caller can pass
 * static_cast<int>(tensor.dtype()).  BFLOAT16 and UINT64 are extensions: the reference
 * has no BFloat16 DType (nt/types/bfloat16.h:4-5) and instantiates uint64_t only at the
 * kernel level (nt_matmult_uint64.cpp).  The complex types hold interleaved (re, im) pairs of half / float / double; their
 * matmult is the reference's: its generic micro kernel multiplies the interleaved lanes element-wise
 * (nt/mp/simde_traits/simde_traits_avx2.h:928-937, :996-1002), so the result is one real product of the real parts and one
 * of the imaginary parts (Complex32 rounded to half every 8 k), NOT the complex product.  Every entry point serves them:
 * the convolutions over one to four axes, their gradients and the transposed convolutions unfold into the workspace and
 * run that product like the reference (nt/functional/tensor_files/conv.cpp:69-175, :318-535, :538-745; the unfold adjoint
 * adds taps lane by lane in the lane's type, the weight gradient adds the per-image products in batch order in that type).
 * The 128-bit types (Float128 = 3, int128 = 11, uint128 = 15) stay on the reference's matmult_naive. */
typedef enum ntg_dtype {
    NTG_FLOAT16 = 0,
    NTG_FLOAT32 = 1,
    NTG_FLOAT64 = 2,
    NTG_COMPLEX32 = 4,
    NTG_COMPLEX64 = 5,
    NTG_COMPLEX128 = 6,
    NTG_INT8 = 7,
    NTG_INT16 = 8,
    NTG_INT32 = 9,
    NTG_INT64 = 10,
    NTG_UINT8 = 12,
    NTG_UINT16 = 13,
    NTG_UINT32 = 14,
    NTG_BFLOAT16 = 100,
    NTG_UINT64 = 101
} ntg_dtype;

typedef enum ntg_status {
    NTG_OK = 0,
    NTG_ERR_INVALID_ARGUMENT = 1,
    NTG_ERR_UNSUPPORTED_DTYPE = 2,
    NTG_ERR_DEVICE = 3,          /* a HIP call failed; see ntg_last_error() */
    NTG_ERR_OUT_OF_MEMORY = 4,
    NTG_ERR_NO_DEVICE = 5
} ntg_status;

/* what the GEMM does with the incoming C */
typedef enum ntg_c_mode {
    NTG_C_OVERWRITE = 0,   /* C  = op(A).op(B); legal replacement of "zeros then accumulate"
                              (matmult_cpu.cpp:110, :707) */
    NTG_C_ACCUMULATE = 1,  /* C += op(A).op(B); the nt_matmult contract */
    NTG_C_BIAS = 2         /* C  = bias (+) op(A).op(B); cpu::linear's "clone the expanded
                              bias, then accumulate" (matmult_cpu.cpp:1637-1647) in one pass */
} ntg_c_mode;

const char* ntg_last_error(void);
int ntg_version(void);
int64_t ntg_dtype_size(int dtype);          /* bytes per element, 0 if unsupported */
int ntg_device_count(void);                 /* gfx950 devices visible to HIP */

/* ------------------------------------------------------------------------------------ */
/* Host-pointer entry points: the drop-in seam.                                           */
/* ------------------------------------------------------------------------------------ */

/* Replaces nt::functional::cpu::nt_matmult<T> (nt_matmult.h:6-7; nt_matmult.hpp:370-378).
 * Same argument list with the dtype made explicit; a_cols must equal b_rows. */
int ntg_matmult(int dtype, const void* A, const void* B, void* C,
                int64_t a_rows, int64_t a_cols, int64_t b_rows, int64_t b_cols,
                int transpose_a, int transpose_b);

/* Replaces nt::functional::cpu::nt_matmult_batch<T> (nt_matmult.h:9-10;
 * nt_matmult.hpp:386-394, 228-235).  A/B/C are arrays of `batches` host pointers; all
 * items share one shape and one flag pair; A/B entries may repeat (that is how the
 * dispatcher broadcasts, matmult_cpu.cpp:883) and each distinct matrix is uploaded once. */
int ntg_matmult_batch(int dtype, const void* const* A, const void* const* B, void* const* C,
                      int64_t batches, int64_t a_rows, int64_t a_cols, int64_t b_rows, int64_t b_cols,
                      int transpose_a, int transpose_b);

/* Replaces the 2-D body of nt::functional::cpu::linear (matmult_cpu.cpp:1624-1647):
 * Y[m, n] = broadcast(bias) + op(X) . op(W).  bias is [bias_rows, bias_cols] with
 * bias_rows in {1, m} and bias_cols in {1, n}. */
int ntg_linear(int dtype, const void* X, const void* W, const void* bias, void* Y,
               int64_t m, int64_t k, int64_t n, int transpose_x, int transpose_w,
               int64_t bias_rows, int64_t bias_cols);

/* Replaces nt::functional::cpu::unfold2d_ with transpose_out = true
 * (nt/functional/cpu/unfold2d.cpp:219-235, im2col_cpu :12-112):
 * col[batch, channels*k_r*k_c, Ho*Wo] is fully written (zeros in the padding). */
int ntg_unfold2d(int dtype, const void* image, void* col,
                 int64_t batch, int64_t channels, int64_t height, int64_t width,
                 int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c,
                 int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c);

/* Replaces the groups == 1 and groups > 1 bodies of nt::functional::conv2d
 * (nt/functional/tensor_files/conv.cpp:69-119): out[batch, out_channels, Ho, Wo].
 * kernel is [out_channels, channels/groups, k_r, k_c]. */
int ntg_conv2d(int dtype, const void* image, const void* kernel, void* out,
               int64_t batch, int64_t channels, int64_t height, int64_t width,
               int64_t out_channels, int64_t k_r, int64_t k_c,
               int64_t s_r, int64_t s_c, int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c,
               int64_t groups);

/* Replaces nt::functional::cpu::unfold2d_backward_ with transpose_out = true (col2im,
 * nt/functional/cpu/unfold2d_backward.cpp:9-56, :158): image[batch, channels, height, width]
 * receives the scatter-add of col[batch, channels*k_r*k_c, Ho*Wo]; accumulate != 0 adds to
 * the incoming image like the reference does, 0 overwrites it. */
int ntg_unfold2d_backward(int dtype, const void* col, void* image,
                          int64_t batch, int64_t channels, int64_t height, int64_t width,
                          int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c,
                          int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c, int accumulate);

/* Replaces the dim == 2 bodies of nt::functional::conv_dimage (conv.cpp:318-346) and
 * conv_dkernel (conv.cpp:444-471):
 *   d_image  (+)= col2im( W2d^T . dY_b )                 [batch, channels, height, width]
 *   d_kernel (+)= sum_b dY_b . col_b^T                   [out_channels, channels/groups, k_r, k_c]
 * grad_out is dY [batch, out_channels, Ho, Wo].  Either output may be NULL to skip it.
 * accumulate != 0 adds into the outputs (the reference's += on the gradient tensors). */
int ntg_conv2d_backward(int dtype, const void* image, const void* kernel, const void* grad_out,
                        void* d_image, void* d_kernel,
                        int64_t batch, int64_t channels, int64_t height, int64_t width,
                        int64_t out_channels, int64_t k_r, int64_t k_c,
                        int64_t s_r, int64_t s_c, int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c,
                        int64_t groups, int accumulate);

/* The host-pointer entry points stage their operands through buffers the library keeps between calls: a device arena
 * that only grows, 32 MiB of pinned host memory and a private stream per GPU (so a sequence of calls pays no
 * hipMalloc / hipFree, and copies run chunk by chunk with the CPU side of one chunk overlapping the DMA of the
 * previous one).  This call gives all of it back; the next host-pointer call allocates afresh.  No counterpart in the
 * reference (its pack buffers are static, nt/functional/cpu/matmult/nt_matmult_blocks.h:12-16). */
int ntg_release_host_buffers(void);

/* ------------------------------------------------------------------------------------ */
/* Device-pointer entry points (buffers already in HBM; asynchronous on `stream`).        */
/* `stream` is a hipStream_t passed as void*; NULL is the default stream.                 */
/* ------------------------------------------------------------------------------------ */

typedef struct ntg_gemm_desc {
    int32_t dtype;              /* ntg_dtype */
    int32_t transpose_a;
    int32_t transpose_b;
    int32_t c_mode;             /* ntg_c_mode */
    int64_t m, k, n;            /* logical sizes */
    int64_t lda, ldb, ldc;      /* row length of the STORED matrices in elements; 0 = dense */
    int64_t batches;            /* >= 1 */
    int64_t stride_a, stride_b, stride_c;   /* elements between items; 0 on A/B = broadcast */
    const void* bias;           /* device pointer, NTG_C_BIAS only */
    int64_t bias_batch_stride, bias_row_stride, bias_col_stride;   /* elements; 0 = broadcast */
    void* workspace;            /* optional device scratch, 256-byte aligned, ntg_gemm_workspace_bytes(desc) bytes: lets a   */
    int64_t workspace_bytes;    /* single product with few output tiles and a deep k be split along k (deterministic), and  */
                                /* a large 16/32/64-bit integer product run as byte planes on the 8-bit matrix pipe (bit-exact) */
    int64_t flags;              /* NTG_GEMM_* bits below; 0 for none */
} ntg_gemm_desc;

/* ntg_gemm_ptrs_dev only: the caller vouches that EVERY entry of the three pointer tables is a multiple of 16 bytes.  The
 * tables live in device memory, so the host side of the library cannot look; with the vouch (and rows that are 16-byte
 * multiples) a table batch runs on the DMA-fed kernels like its strided twin.  An entry that breaks the promise makes the
 * kernel read from a misaligned address (wrong results, not a fault).  Without the vouch, floating-point and 8-bit
 * batches of some size (from 8 GFLOP; Float32 and Float64 from 32, 8-bit integers from 1) have their entries looked at on the device: one small kernel sets a
 * flag, then the product is launched on both kernel families and the one the flag does not name returns at once -- two
 * extra launches (about 4 us), the same bits; smaller batches run on the register-staged kernels.  The flags live in a static
 * array of the library's device code: make the first such call on a device outside a stream capture. */
#define NTG_GEMM_PTRS_ALIGNED16 1
/* Keep the reference's order of summation: never split this product along k (workspace or not), and run products of up to 32
 * rows on the tile kernels instead of the streaming ones (which share k out between wavefronts).  A Float32 product is then
 * the reference's own sum bit for bit -- every element is c = C0; c = fma(a[i,k], b[k,j], c) for ascending k, what the
 * k-outer loop nest of nt_matmult.hpp:196 computes.  Without the flag that also holds for every Float32 product of more than
 * 32 rows that is given no workspace.  The host-pointer entry points set it for Float32 themselves (the transfers hide what
 * the faster forms would gain); ntg_gemm_workspace_bytes honours it. */
#define NTG_GEMM_KEEP_K_ORDER 2

/* Bytes of workspace with which ntg_gemm_dev runs its faster form (0: there is none for this product): a split along k
 * for shapes such as [256, 8192] x [8192, 8192] (planned from one item's sizes, so a batch is offered its item's split with
 * the partial sums of every item); zero-padded copies of large 8-bit, 16-bit, Float32 and Float64 operands whose rows, pitches
 * or base pointers are not 16-byte multiples, so that they run on the DMA-fed kernels (same results: zeros add nothing);
 * or, for large Int16 / Int32 / Int64 products and their unsigned forms, the
 * 3 / 10 / 36 products of balanced byte planes on v_mfma_i32_32x32x32_i8, whose sum modulo 2^W is the reference's wrapping
 * result (nt/mp/simde_traits/simde_traits_avx2.h:810-812, :444-446, :523-540: multiply and add in the element type).  Without a workspace the same result is computed by the
 * plain kernels.  The reference has no counterpart: its k loop is always serial (nt_matmult.hpp:196). */
int64_t ntg_gemm_workspace_bytes(const ntg_gemm_desc* desc);

/* nt_matmult<T> on device buffers: C += op(A).op(B), dense leading dimensions. */
int ntg_matmult_dev(int dtype, const void* dA, const void* dB, void* dC,
                    int64_t m, int64_t k, int64_t n, int transpose_a, int transpose_b, void* stream);

/* General strided/broadcast batch; what functional::matmult's N-D x K-D paths
 * (matmult_cpu.cpp:863-1005) lower to when the views are affine. */
int ntg_gemm_dev(const ntg_gemm_desc* desc, const void* dA, const void* dB, void* dC, void* stream);

/* ntg_gemm_dev followed by relu_ on the result, in one pass: C = max(result, 0), where result is what ntg_gemm_dev would
 * have stored (so Linear -> ReLU, nt::functional::relu_(linear(x, w, b)), is one launch with c_mode = NTG_C_BIAS).  relu_ is
 * clamp_(x, 0) (nt/functional/tensor_files/activation_functions.cpp:141-143), i.e. max(x, 0) with 0 returned for NaN and
 * for -0 (nt/functional/cpu/min_max.cpp:45-63, :115-121); rounding is monotonic and keeps the sign, so clamping the sum
 * before its one rounding gives the bits of clamping the stored value.  Float16, BFloat16, Float32, Float64.  The DMA-fed
 * kernels and the split-K reduction clamp in their epilogue; where another kernel serves the product a second small
 * kernel clamps C in place.  With k = 0 and NTG_C_ACCUMULATE the call is relu_ itself on the matrix at dC (dA, dB may be
 * null).  The reference's other activations (sigmoid, silu, gelu: SVML exp / tanh / pow) are not offered
 * as epilogues: their bits are those of its vector maths library, which this library cannot reproduce. */
int ntg_gemm_relu_dev(const ntg_gemm_desc* desc, const void* dA, const void* dB, void* dC, void* stream);

/* ntg_gemm_dev for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc): it has NO counterpart in the reference.  Same arguments, results bit-identical to
 * ntg_gemm_dev called with a workspace of ntg_gemm_workspace_bytes(desc) bytes; desc->workspace and desc->workspace_bytes
 * are ignored.  The split along k, the byte-plane products of the wide integers and the padded copies of unaligned 8- and
 * 16-bit operands keep their intermediate data in a fixed array of NTG_NOALLOC_SCRATCH_BYTES bytes that is part of the
 * library's device code (every GPU the library runs on holds its copy until the process ends); the call itself allocates and
 * frees no memory.  A product whose workspace form needs more than that is rejected with NTG_ERR_INVALID_ARGUMENT: use
 * ntg_gemm_dev with your own workspace, or -- it allocates nothing either -- ntg_gemm_dev with workspace = NULL, which runs
 * the plain kernels (same integer results; a floating product that would have been split along k is then summed in one
 * range, so its last bits may differ).  All calls on one GPU share the array.  Calls on one stream are ordered by the
 * stream.  Calls on different streams or from different threads are ordered by the library: a call is enqueued as a whole
 * (a mutex per GPU) and makes its stream wait for an event recorded behind the previous user's last kernel.  A stream under
 * capture takes no part in that ordering (an event recorded inside a capture cannot be waited for from outside): graphs
 * that contain such calls must not run while other users of the array are in flight.  The first call on a device looks the
 * array's address up (hipGetSymbolAddress) and creates the event: make that call before a stream capture begins. */
#define NTG_NOALLOC_SCRATCH_BYTES (64ll << 20)
int ntg_gemm_noalloc_dev(const ntg_gemm_desc* desc, const void* dA, const void* dB, void* dC, void* stream);

/* Measurement aid with NO counterpart in the reference (bench.py reports it beside the headline): `iters` passes of the
 * 16-bit product kernels' matrix instruction (v_mfma_f32_32x32x16, Float16 or BFloat16) on operand fragments that stay in
 * registers -- no LDS and no global memory in the loop -- on `workgroups` workgroups of four wavefronts with the 4 x 4
 * accumulator blocks of the 256 x 256 tile.  `operands`: NTG_DIAG_MFMA_OPERAND_BYTES bytes of 16-bit values in device memory
 * (16-byte aligned), loaded once; `sink`: 256 floats per workgroup.  One pass of one workgroup is
 * NTG_DIAG_MFMA_FLOPS_PER_PASS floating-point operations.  The rate depends on the operand VALUES (the clock falls as
 * operand bits toggle): random against all-zero operands is what the figure is for. */
#define NTG_DIAG_MFMA_OPERAND_BYTES (128 << 10)
#define NTG_DIAG_MFMA_FLOPS_PER_PASS 8388608ll
int ntg_diag_mfma_rate_dev(int dtype, const void* operands, int64_t iters, int64_t workgroups, float* sink, void* stream);

/* nt_matmult_batch<T> with the pointer tables themselves in device memory.  desc->workspace is not used: a table batch is
 * never split along k, so an item whose single-product form ntg_gemm_workspace_bytes offers a split (the order of summation
 * over k then differs) is, for bit-identical results alone and in a batch, better sent through ntg_gemm_dev item by item --
 * what ntg_matmult_batch and the C++ facade do with such lists. */
int ntg_gemm_ptrs_dev(const ntg_gemm_desc* desc, const void* const* dA, const void* const* dB,
                      void* const* dC, void* stream);

int ntg_unfold2d_dev(int dtype, const void* image, void* col,
                     int64_t batch, int64_t channels, int64_t height, int64_t width,
                     int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c,
                     int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c, void* stream);

/* Bytes of device workspace ntg_conv2d_dev needs.  0 for the floating dtypes: their GEMM gathers
 * the im2col operand (nt/functional/cpu/unfold2d.cpp:12-112) from the image tile by tile and the
 * unfolded matrix of conv.cpp:87-94 is never stored; the integer dtypes unfold into the workspace. */
int64_t ntg_conv2d_forward_workspace_bytes(int dtype, int64_t batch, int64_t channels, int64_t height, int64_t width,
                                           int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c,
                                           int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c);

/* Bytes of device workspace with which ntg_conv2d_dev runs its fastest form.  For Float32 whose channels per group are a
 * multiple of 16, Float16 / BFloat16 with at least 8 channels per group (padded with zeros to a multiple of 32 in the
 * copy), and groups of up to 32 bytes of channels in all three (RGB input layers: pixels of 16 or 32 bytes, several taps
 * per K-step), that is a channels-last copy of the image (with the padding as a border of zero pixels where the channels
 * of a group fill whole 64-byte runs) plus the weights with the channel index fastest; the convolution (conv.cpp:86-118)
 * then gathers its operand in 16-byte pieces.  Otherwise the figure of
 * ntg_conv2d_forward_workspace_bytes.  ntg_conv2d_dev accepts any smaller workspace and falls back to its other forms. */
int64_t ntg_conv2d_fast_workspace_bytes(int dtype, int64_t batch, int64_t channels, int64_t height, int64_t width,
                                        int64_t out_channels, int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c,
                                        int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c, int64_t groups);

/* bytes of the full im2col buffer (what ntg_unfold2d_dev writes and ntg_conv2d_backward_dev needs). */
int64_t ntg_conv2d_workspace_bytes(int dtype, int64_t batch, int64_t channels, int64_t height, int64_t width,
                                   int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c,
                                   int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c);

int ntg_conv2d_dev(int dtype, const void* image, const void* kernel, void* out,
                   void* workspace, int64_t workspace_bytes,
                   int64_t batch, int64_t channels, int64_t height, int64_t width,
                   int64_t out_channels, int64_t k_r, int64_t k_c,
                   int64_t s_r, int64_t s_c, int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c,
                   int64_t groups, void* stream);

int ntg_unfold2d_backward_dev(int dtype, const void* col, void* image,
                              int64_t batch, int64_t channels, int64_t height, int64_t width,
                              int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c,
                              int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c, int accumulate, void* stream);

/* Bytes of device workspace ntg_conv2d_backward_dev needs when both gradients are requested.  Floating dtypes with
 * kernels up to 8x8 compute conv_dkernel (conv.cpp:444-471) without the stored im2col matrix (workspace = the per-image
 * weight gradients, batch * out_channels * channels/groups * k_r * k_c elements) and, at stride 1, conv_dimage
 * (conv.cpp:318-346) as well; every other case needs the im2col-sized buffer (ntg_conv2d_workspace_bytes).  Where
 * conv_dimage can run in its channels-last form (Float32 / Float16 / BFloat16, two axes, stride 1, the out channels of a
 * group filling whole 64-byte runs) the figure also covers a channels-last copy of grad_out plus the flipped weights; the
 * call still accepts the smaller amount and then gathers from grad_out as it lies. */
int64_t ntg_conv2d_backward_workspace_bytes(int dtype, int64_t batch, int64_t channels, int64_t height, int64_t width,
                                            int64_t out_channels, int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c,
                                            int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c, int64_t groups);

/* workspace: at least ntg_conv2d_backward_workspace_bytes */
int ntg_conv2d_backward_dev(int dtype, const void* image, const void* kernel, const void* grad_out,
                            void* d_image, void* d_kernel, void* workspace, int64_t workspace_bytes,
                            int64_t batch, int64_t channels, int64_t height, int64_t width,
                            int64_t out_channels, int64_t k_r, int64_t k_c,
                            int64_t s_r, int64_t s_c, int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c,
                            int64_t groups, int accumulate, void* stream);

/* functional::conv_transpose2d (nt/functional/tensor_files/conv.cpp:614-676; conv_transpose1d :538-612 is the same call
 * with in_h == 1 and k_r == 1).  input [batch, in_channels, in_h, in_w], kernel [in_channels, out_channels/groups, k_r, k_c],
 * out [batch, out_channels, (in_h-1)*s_r - 2*p_r + d_r*(k_r-1) + 1 + op_r, likewise for columns].  The reference dilates the
 * input by the stride, pads it by output_padding, unfolds it and multiplies by the channel-swapped, tap-reversed kernel;
 * this backend computes the same sums as the image gradient of the matching convolution.  output_padding must be smaller
 * than stride. */
int64_t ntg_conv_transpose2d_workspace_bytes(int dtype, int64_t batch, int64_t in_channels, int64_t in_h, int64_t in_w,
                                             int64_t out_channels, int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c,
                                             int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c, int64_t op_r, int64_t op_c, int64_t groups);
int ntg_conv_transpose2d_dev(int dtype, const void* input, const void* kernel, void* out, void* workspace, int64_t workspace_bytes,
                             int64_t batch, int64_t in_channels, int64_t in_h, int64_t in_w, int64_t out_channels,
                             int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c, int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c,
                             int64_t op_r, int64_t op_c, int64_t groups, void* stream);
/* host pointers, synchronous */
int ntg_conv_transpose2d(int dtype, const void* input, const void* kernel, void* out,
                         int64_t batch, int64_t in_channels, int64_t in_h, int64_t in_w, int64_t out_channels,
                         int64_t k_r, int64_t k_c, int64_t s_r, int64_t s_c, int64_t p_r, int64_t p_c, int64_t d_r, int64_t d_c,
                         int64_t op_r, int64_t op_c, int64_t groups);

/* ---- convolutions over 1..4 spatial axes -----------------------------------------------------------------------
 * functional::conv3d (nt/functional/tensor_files/conv.cpp:122-175), convnd (:177-316), conv_dimage / conv_dkernel for
 * dim == 3 and the dynamic case (:347, :472), conv_transpose3d (:678-745), conv_transposend (:747-905); unfold3d / unfoldnd
 * and their adjoints (nt/functional/cpu/unfold3d.cpp:9-80, unfoldnd.cpp, unfold3d_backward.cpp, unfoldnd_backward.cpp).
 * size / kernel_size / stride / padding / dilation / output_padding point to `ndim` values, slowest axis first
 * (depth, rows, columns).  image [batch, channels, size...], kernel [out_channels, channels/groups, kernel_size...]
 * (transposed: [in_channels, out_channels/groups, kernel_size...]).  ndim 1 and 2 run on the conv2d entry points above;
 * ndim 3 gathers the unfolded operand inside the GEMM for the floating dtypes (workspace as for conv2d); ndim 4, the
 * integer dtypes and kernels wider than 8 taps unfold into the workspace like the reference.  `backward` selects the
 * workspace of the gradient call. */
int ntg_unfoldnd_dev(int dtype, const void* image, void* col, int64_t batch, int64_t channels, int ndim, const int64_t* size,
                     const int64_t* kernel_size, const int64_t* stride, const int64_t* padding, const int64_t* dilation, void* stream);
int ntg_unfoldnd_backward_dev(int dtype, const void* col, void* image, int64_t batch, int64_t channels, int ndim, const int64_t* size,
                              const int64_t* kernel_size, const int64_t* stride, const int64_t* padding, const int64_t* dilation,
                              int accumulate, void* stream);
int64_t ntg_convnd_workspace_bytes(int dtype, int64_t batch, int64_t channels, int64_t out_channels, int ndim, const int64_t* size,
                                   const int64_t* kernel_size, const int64_t* stride, const int64_t* padding, const int64_t* dilation,
                                   int64_t groups, int backward);
int ntg_convnd_dev(int dtype, const void* image, const void* kernel, void* out, void* workspace, int64_t workspace_bytes,
                   int64_t batch, int64_t channels, int64_t out_channels, int ndim, const int64_t* size, const int64_t* kernel_size,
                   const int64_t* stride, const int64_t* padding, const int64_t* dilation, int64_t groups, void* stream);
int ntg_convnd_backward_dev(int dtype, const void* image, const void* kernel, const void* grad_out, void* d_image, void* d_kernel,
                            void* workspace, int64_t workspace_bytes, int64_t batch, int64_t channels, int64_t out_channels, int ndim,
                            const int64_t* size, const int64_t* kernel_size, const int64_t* stride, const int64_t* padding,
                            const int64_t* dilation, int64_t groups, int accumulate, void* stream);
int64_t ntg_conv_transposend_workspace_bytes(int dtype, int64_t batch, int64_t in_channels, int64_t out_channels, int ndim,
                                             const int64_t* in_size, const int64_t* kernel_size, const int64_t* stride,
                                             const int64_t* padding, const int64_t* dilation, const int64_t* output_padding, int64_t groups);
int ntg_conv_transposend_dev(int dtype, const void* input, const void* kernel, void* out, void* workspace, int64_t workspace_bytes,
                             int64_t batch, int64_t in_channels, int64_t out_channels, int ndim, const int64_t* in_size,
                             const int64_t* kernel_size, const int64_t* stride, const int64_t* padding, const int64_t* dilation,
                             const int64_t* output_padding, int64_t groups, void* stream);
/* host pointers, synchronous */
int ntg_convnd(int dtype, const void* image, const void* kernel, void* out, int64_t batch, int64_t channels, int64_t out_channels, int ndim,
               const int64_t* size, const int64_t* kernel_size, const int64_t* stride, const int64_t* padding, const int64_t* dilation,
               int64_t groups);
int ntg_convnd_backward(int dtype, const void* image, const void* kernel, const void* grad_out, void* d_image, void* d_kernel,
                        int64_t batch, int64_t channels, int64_t out_channels, int ndim, const int64_t* size, const int64_t* kernel_size,
                        const int64_t* stride, const int64_t* padding, const int64_t* dilation, int64_t groups, int accumulate);
int ntg_conv_transposend(int dtype, const void* input, const void* kernel, void* out, int64_t batch, int64_t in_channels,
                         int64_t out_channels, int ndim, const int64_t* in_size, const int64_t* kernel_size, const int64_t* stride,
                         const int64_t* padding, const int64_t* dilation, const int64_t* output_padding, int64_t groups);

#ifdef __cplusplus
}
#endif
#endif /* NTGEMM_H */
