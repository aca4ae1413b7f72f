/*
 * C ABI of the gfx950 TCEC library (libwmmae_tcec.so).
 *
 * The reference (wmmae/wmma_extension) is a header-only device library; the
 * only host-callable GEMM it contains is the launcher of its batched test
 * kernel.  This header is the host boundary of the rebuilt hot path: a
 * BLAS-style driver for the error-corrected SGEMM, the two stages it is made
 * of, and entry points that run the reference's one-warp test kernels on the
 * header-only device API (include/wmma_extension/...) so that host programs
 * and ctypes/cgo/JNI bindings can exercise that API without a device compiler.
 *
 * Conventions
 *   - every pointer named A, B, C, X, tiles, ... is a DEVICE pointer unless the
 *     comment says host; alpha/beta are HOST pointers
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *     all work is asynchronous on that stream, nothing synchronises
 *   - return value: WMMAE_STATUS_SUCCESS (0) or a negative wmmae_status
 *   - no state a caller could observe (the library remembers, per device, the
 *     compute-unit count and which kernels it has raised the LDS limit for);
 *     calls may come from any thread
 *   - matrices follow the column-major BLAS convention; the reference's layout
 *     (A row-major m x k, B column-major k x n, C column-major m x n,
 *     test/tcec/batch_gemm.cu:259-260, 542-543) is transa='T', transb='N',
 *     exactly as in its cublasSgemmBatched comparator (batch_gemm.cu:619-621)
 */
#ifndef WMMAE_TCEC_H
#define WMMAE_TCEC_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  WMMAE_STATUS_SUCCESS = 0,
  WMMAE_STATUS_INVALID_VALUE = -1,  /* bad size, flag or enum value */
  WMMAE_STATUS_NULL_POINTER = -2,   /* a required pointer is NULL */
  WMMAE_STATUS_BAD_LEADING_DIM = -3,/* lda/ldb/ldc smaller than the matrix */
  WMMAE_STATUS_NOT_SUPPORTED = -4,  /* valid request this build cannot run */
  WMMAE_STATUS_WORKSPACE_TOO_SMALL = -5,
  WMMAE_STATUS_RUNTIME_ERROR = -6,  /* a HIP call failed */
  WMMAE_STATUS_MISALIGNED = -7      /* packed buffer not 16-byte aligned */
} wmmae_status;

/*
 * Arithmetic policies.  They mirror the reference's
 * Policy<Op, ErrorCorrection, ...> / default_policy<T, EC> choices
 * (tcec/detail/policy.hpp:50-99):
 *   F16_EC     T = half,  with_ec     v ~ hi + lo/2048, 3 MFMAs per product
 *   F16_NOEC   T = half,  without_ec  1 MFMA
 *   BF16X3_EC  T = tf32,  with_ec     gfx950 has no tf32 matrix op; the policy
 *              is carried by a three-term bf16 split (6 MFMAs), fp32 range
 *   BF16X2_EC  T = bfloat16, with_ec  two-term bf16 split (3 MFMAs, ~16 bits)
 *   BF16_NOEC  T = bfloat16, without_ec
 */
typedef enum {
  WMMAE_POLICY_F16_EC = 0,
  WMMAE_POLICY_F16_NOEC = 1,
  WMMAE_POLICY_BF16X3_EC = 2,
  WMMAE_POLICY_BF16X2_EC = 3,
  WMMAE_POLICY_BF16_NOEC = 4
} wmmae_policy;

/* flags for the GEMM entry points */
#define WMMAE_FLAG_RN_MAIN 1 /* accumulate the leading product with fp32 adds
                                outside the matrix core (the reference's
                                mma_rn_sync, tcec/tcec.hpp:640-706) */
/* wmmae_tcec_sgemm*: take this path instead of the one the time estimates
 * choose (at most one of the three; WMMAE_STATUS_NOT_SUPPORTED when the
 * arguments do not allow it).  No counterpart in the reference, whose harness
 * fixes one kernel configuration at compile time. */
#define WMMAE_FLAG_PATH_PACKED 2 /* split pass + GEMM on packed operands */
#define WMMAE_FLAG_PATH_FUSED 4  /* the single kernel for small products */
#define WMMAE_FLAG_PATH_DIRECT 8 /* the packed path's GEMM kernel splitting the
                                    fp32 operands itself: needs op(A) and op(B)
                                    with k contiguous ('T','N'), k >= 4, a
                                    policy of one or two terms, no RN_MAIN */

/* Text for a wmmae_status value.  (No counterpart in the reference: its
 * harness aborts through WMMAE_CUDA_CHECK_ERROR, test/tcec/utils.hpp:11-20.) */
const char *wmmae_status_string(int status);

/* what: 0 = library version (major*10000 + minor*100 + patch),
 *       1 = compute units of the current device,
 *       2 = max engine clock in kHz,
 *       3 = number of policies
 * (No counterpart in the reference, which is header-only.) */
int wmmae_query(int what, long long *out);

/* ------------------------------------------------------------------ GEMM
 * C = alpha * op(A) * op(B) + beta * C with TCEC arithmetic.
 * Replaces: launch_bgemm + bgemm_kernel of the reference's GEMM harness
 * (test/tcec/batch_gemm.cu:261-386, 433-443) and stands where that harness
 * calls cublasSgemmBatched (batch_gemm.cu:619-621).
 *
 * workspace holds the split operands (and K slices for K-heavy shapes); size
 * from wmmae_tcec_sgemm_workspace_bytes.  workspace == NULL lets the library
 * take it from the stream-ordered allocator (hipMallocAsync / hipFreeAsync on
 * `stream`; measured at 3 to 9 us a call on MI355X, which a product of 20 us
 * feels - keep a workspace across calls where calls are small).  Products
 * whose operand elements are used by few tiles (small m and n, or a short k;
 * an estimate of both paths' times decides; no K slices; operands readable
 * 16 bytes at a time) are split inside the GEMM
 * kernel (as the reference's bgemm_kernel splits at fragment load,
 * batch_gemm.cu:196-386): they use no workspace, allocate nothing and ignore
 * the workspace arguments.  Batches of medium-sized matrices and K-heavy
 * products with k contiguous in both operands run the packed path's GEMM
 * kernel on the fp32 operands directly (it splits them on their way into LDS):
 * no packed copy; the workspace then only holds K slices.  All paths give the
 * same bits as long as no K slices are made (those add the partial sums'
 * rounding).
 *
 * wmmae_tcec_sgemm_workspace_bytes is an upper bound over the paths: packed
 * A + packed B + K slices, whichever path the call then takes.  A product the
 * library runs on the fp32 operands directly (wmmae_tcec_sgemm_path 3 or 4)
 * touches only the K slices, wmmae_tcec_gemm_packed_workspace_bytes of it, and
 * path 0 nothing; a caller that knows its products take those paths may pass
 * that much.  A workspace that is not 16-byte aligned is WMMAE_STATUS_MISALIGNED
 * on the packed path, which cannot do without it; the other two paths then run
 * without K slices. */
int wmmae_tcec_sgemm_workspace_bytes(int m, int n, int k, int batch, int policy,
                                     size_t *bytes);

/* Which of these the GEMM entry points take for a shape (no counterpart in the
 * reference, whose harness fixes one kernel configuration at compile time,
 * batch_gemm.cu:408-431, 659): *path = 0 the single kernel that splits the
 * operands on the fly (no workspace), 1 packed operands in the workspace,
 * 2 packed operands and K slices (when the workspace has room for them),
 * 3 the packed path's GEMM kernel loading and splitting the fp32 operands
 * itself (no packed operands), 4 the same with K slices.  3 and 4 assume
 * k contiguous in both operands ('T','N') and need k >= 4; other layouts
 * take 1 and 2.
 * The answer is for op(A) = 'T', op(B) = 'N' with tight leading dimensions
 * (lda = ldb = k) and 16-byte aligned bases: with k a multiple of 4 the
 * single kernel reads such operands 16 bytes at a time, which is what the
 * time estimates behind the choice assume; other leading dimensions or bases
 * can move a product from path 0 to another one. */
int wmmae_tcec_sgemm_path(int m, int n, int k, int batch, int policy, int flags,
                          int *path);

int wmmae_tcec_sgemm(char transa, char transb, int m, int n, int k,
                     const float *alpha, const float *A, int lda,
                     const float *B, int ldb, const float *beta, float *C,
                     int ldc, int policy, int flags, void *workspace,
                     size_t workspace_bytes, void *stream);

int wmmae_tcec_sgemm_strided_batched(char transa, char transb, int m, int n,
                                     int k, const float *alpha, const float *A,
                                     int lda, long long stride_a,
                                     const float *B, int ldb,
                                     long long stride_b, const float *beta,
                                     float *C, int ldc, long long stride_c,
                                     int batch, int policy, int flags,
                                     void *workspace, size_t workspace_bytes,
                                     void *stream);

/* wmmae_tcec_sgemm for callers that cannot allocate device memory (tight
 * serving loops, harnesses that forbid hipMalloc, code that will be captured
 * into a HIP graph).  No counterpart in the reference.  Same arguments and
 * results as wmmae_tcec_sgemm; the workspace is a fixed device array of
 * WMMAE_STATIC_SCRATCH_BYTES inside the library image (every GPU the library
 * runs on holds it until the process ends), so the call makes no hipMalloc /
 * hipFree of any kind.  On the packed path (wmmae_tcec_sgemm_path 1, 2) the
 * array holds the split operands, and products whose split operands need more
 * (wmmae_tcec_pack_bytes of A and of B; fp16 hi+lo: 4*(m+n)*k bytes rounded up
 * to 16 rows and 32 of k) return WMMAE_STATUS_WORKSPACE_TOO_SMALL; K slices
 * are made only when they fit behind the operands.  On the path that reads the
 * fp32 operands directly (3, 4) the array holds K slices only, from its start,
 * and a product of any size succeeds (without K slices when they do not fit);
 * path 0 does not touch the array.  All calls on one GPU share the one array:
 * calls that overlap in time on the same GPU (two streams, two threads) race
 * and must be serialised by the caller.  Nothing in the array has to survive
 * between calls and nothing is assumed zero.
 * The first call on a device looks the array's address up
 * (hipGetSymbolAddress) and the first launch of each kernel sets its LDS
 * limit (hipFuncSetAttribute): make one call per shape class outside stream
 * capture before capturing. */
#define WMMAE_STATIC_SCRATCH_BYTES (64u << 20)
int wmmae_tcec_sgemm_static(char transa, char transb, int m, int n, int k,
                            const float *alpha, const float *A, int lda,
                            const float *B, int ldb, const float *beta,
                            float *C, int ldc, int policy, int flags,
                            void *stream);

/* Batched product on device arrays of matrix pointers, the calling convention
 * of the reference's launch_bgemm(conf, m, n, k, alpha, a_ptr_array, lda,
 * b_ptr_array, ldb, beta, c_ptr_array, ldc, batch) (batch_gemm.cu:433-443) and
 * of cublasSgemmBatched.  A_array, B_array, C_array are DEVICE arrays of
 * `batch` device pointers. */
int wmmae_tcec_sgemm_batched(char transa, char transb, int m, int n, int k,
                             const float *alpha, const float *const *A_array,
                             int lda, const float *const *B_array, int ldb,
                             const float *beta, float *const *C_array, int ldc,
                             int batch, int policy, int flags, void *workspace,
                             size_t workspace_bytes, void *stream);

/* The two stages, for callers that keep an operand split across many
 * products.  A packed operand is `rows` x k (rows = m for op(A), n for op(B))
 * with element (r, l) read from X[r*row_stride + l*k_stride]; the packed form
 * is opaque, 16-byte aligned, and only meaningful with the same policy.
 * Replaces: the per-warp split inside tcec::load_matrix_sync
 * (tcec/tcec.hpp:194-236), done once per element instead. */
int wmmae_tcec_pack_bytes(int rows, int k, int batch, int policy,
                          size_t *bytes);
int wmmae_tcec_pack(int policy, int rows, int k, const float *X,
                    long long row_stride, long long k_stride,
                    long long batch_stride, int batch, void *packed,
                    size_t packed_bytes, void *stream);
/* workspace (optional, may be NULL): room for K slices, used when the output
 * has too few tiles to fill the chip (K-heavy shapes: every tile is cut), or
 * when its tiles leave the last round over the compute units mostly empty
 * (single large products: only that round's tiles are cut); size from
 * wmmae_tcec_gemm_packed_workspace_bytes (0 when no cut would be made).
 * Without it the product runs uncut.
 * Replaces: launch_bgemm on operands that are already split,
 * test/tcec/batch_gemm.cu:433-443 (the reference's kernel has no K slices: its
 * grid is one block per output tile and batch entry, :396-399, :418). */
int wmmae_tcec_gemm_packed_workspace_bytes(int policy, int m, int n, int k,
                                           int batch, size_t *bytes);
int wmmae_tcec_gemm_packed(int policy, int m, int n, int k, const float *alpha,
                           const void *packed_a, const void *packed_b,
                           const float *beta, float *C, int ldc,
                           long long stride_c, int batch, int flags,
                           void *workspace, size_t workspace_bytes,
                           void *stream);

/* ------------------------------------------- device-API harness kernels
 * Each runs one of the reference's test kernels, rebuilt on the gfx950
 * headers, on caller-provided device buffers. */

/* Fragment primitives over num_tiles 16x16 fp32 tiles (256 floats each).
 * Outputs per tile: a_row, a_col, b_row, b_col: 64 lanes x 4 fp16 registers of
 * a 16x16x16 fragment filled through foreach_ij; acc_out: 256 floats (tile
 * read row-major through foreach, stored column-major); vec_out: 32 floats
 * (load_vector/store_vector round trip of tile[0..15] and tile[16..31]).
 * Replaces: test/primitive/foreach_ij.cu:20-92, wmma.load_vector.cu:44-72,
 * wmma.store_vector.cu:36-42. */
int wmmae_primitive_tiles(const float *tiles, long long num_tiles, void *a_row,
                          void *a_col, void *b_row, void *b_col,
                          float *acc_out, float *vec_out, void *stream);

/* Integer layout tables of fragment<use, m, n, k> (use: 0 matrix_a, 1
 * matrix_b, 2 accumulator; elem: 0 half, 1 bfloat16, 2 float accumulator is
 * implied by use == 2).  col != 0 selects col_major / mem_col_major.
 *   ij[(lane*R + reg)*2 + {0,1}], mem_index[lane*R + reg], v_index[lane*R + reg]
 *   (-1 = not visited by foreach_v), map_tid/map_fid[i*cols + j]
 * Replaces: test/primitive/map.cu:11-58 and research/fragment_analysis. */
int wmmae_layout_dump(int use, int m, int n, int k, int col, int *ij,
                      int *mem_index, int *v_index, int *map_tid, int *map_fid,
                      void *stream);

/* One-wave TCEC product D = A*B (+C), every operand in one tcec::fragment.
 * shape: 0 -> m=n=k=32, 1 -> (m,n,k) = (16,48,64) [(32,64,32) for inst 2];
 * type: 0 half, 1 bfloat16, 2 tf32, 3 float (the fp32 policy
 * default_policy<float, without_ec, op_simt>, reference docs/mma_f32.md:139-152:
 * ec must be 0, inst is ignored, the shape is 16x16x16; with ec != 0 the
 * entry points return WMMAE_STATUS_NOT_SUPPORTED); ec: 1 with_ec, 0 without_ec;
 * inst: 0 -> 16x16x32, 1 -> 16x16x16, 2 -> 32x32x16; *_col: memory layouts
 * (1 = column major, dense leading dimension); c may be NULL;
 * rounding: 0 mma_sync, 1 mma_rn_sync, 2 mma_rz_sync.
 * Replaces: mma_kernel_abcd / mma_kernel_abd, test/tcec/mma.cu:23-100. */
int wmmae_tcec_mma_tile(int shape, int type, int ec, int inst, float *d,
                        const float *a, const float *b, const float *c,
                        int a_col, int b_col, int c_col, int d_col,
                        int rounding, void *stream);

/* Same with m=n=k=32, 16x16x32, operands loaded through the load_matrix_sync
 * overload that takes the memory layout from the fragment's Layout argument
 * (tcec/tcec.hpp:281-291). */
int wmmae_tcec_mma_tile_native(int type, int ec, int a_frag_col,
                               int b_frag_col, float *d, const float *a,
                               const float *b, int d_col, void *stream);

/* y = A*x (left_vector == 0) or y^T = x^T*A (left_vector != 0), N = 32, through
 * tcec::load_vector / store_vector.  Replaces: test/tcec/matvec.cu:21-50. */
int wmmae_tcec_matvec(int type, int ec, float *y, const float *a,
                      const float *x, int a_col, int left_vector,
                      void *stream);

/* 16-bit split terms held by a 32x32x32 operand fragment (use 0/1) after
 * load_matrix_sync (from_vector == 0) or load_vector (from_vector != 0):
 * terms[(term*E + e)*64 + lane], E = fragment num_elements, e = index of x(e).
 * type 0..2 only (fp32 fragments hold no 16-bit terms).  mem_col 0 / 1: src
 * is row- / column-major; 2: src (rows of 32 k for use 0, columns of 32 k for
 * use 1, 16-byte aligned) is first staged into an LDS tile in the swizzled
 * layout (tcec::row_major_swizzled / col_major_swizzled) with utils::cp_async
 * and loaded from there - the same terms as mem_col = use.
 * Replaces: test/tcec/vector.cu:15-61 and test/tcec/elementwise.cu:7-26. */
int wmmae_tcec_frag_dump(int use, int type, int ec, int frag_col,
                         unsigned short *terms, const float *src,
                         int from_vector, int mem_col, void *stream);

/* Element access on a 32x32 TCEC accumulator: fill_fragment(base), x(i) +=
 * lane*100 + i, dx(i) = i (with_ec), optional neg(), optional integrate(),
 * store column-major into out[0..1024); out[1024 + lane] = x(0) + x(last) read
 * through the const accessors.  inst as in wmmae_tcec_mma_tile.
 * Replaces: test/tcec/elementwise.cu:7-26 (and the fill part of
 * test/primitive/fill.cu). */
int wmmae_tcec_elementwise(int type, int ec, int inst, float *out, float base,
                           int do_neg, int do_integrate, void *stream);

/* C = alpha*A*B + beta*C by a tiled kernel written only against the public
 * tcec:: device API: fp32 tiles staged in LDS by utils::cp_async (two stages),
 * split at fragment load in every wave (tcec::load_matrix_sync), tcec::mma_sync.
 * A row-major m x k (lda), B column-major k x n (ldb), C column-major (ldc);
 * m, n multiples of 128, k of 32, lda/ldb multiples of 4, 16-byte aligned.
 * type/ec as in wmmae_tcec_mma_tile.
 * Replaces: bgemm_kernel + mma_core + dmem2smem, test/tcec/batch_gemm.cu:74-116,
 * 196-386: what a user of the headers gets, beside wmmae_tcec_sgemm. */
int wmmae_tcec_api_gemm(int type, int ec, int m, int n, int k,
                        const float *alpha, const float *A, int lda,
                        const float *B, int ldb, const float *beta, float *C,
                        int ldc, void *stream);
/* The same kernel with the product of every k step issued by tcec::mma_sync
 * (rounding 0, as above), mma_rn_sync (1) or mma_rz_sync (2)
 * (tcec/tcec.hpp:640-706, 773-831, 896-927).  On gfx950 the matrix core
 * accumulates with round-to-nearest-even, so the chained variant is as accurate
 * as the reference's default and faster. */
int wmmae_tcec_api_gemm_rounding(int type, int ec, int rounding, int m, int n,
                                 int k, const float *alpha, const float *A,
                                 int lda, const float *B, int ldb,
                                 const float *beta, float *C, int ldc,
                                 void *stream);
/* The same kernel on device arrays of `batch` matrix pointers (each 16-byte
 * aligned), the calling convention of the reference's launch_bgemm
 * (test/tcec/batch_gemm.cu:433-443). */
int wmmae_tcec_api_gemm_batched(int type, int ec, int m, int n, int k,
                                const float *alpha,
                                const float *const *A_array, int lda,
                                const float *const *B_array, int ldb,
                                const float *beta, float *const *C_array,
                                int ldc, int batch, void *stream);

/* One-wave complex TCEC product D = A*B (+C), m = n = k = 32, operands in
 * tcec::fragment_complex (16x16x32 policy; 16x16x16 for type 3).  a, b, c, d:
 * 32 x 32 interleaved (re, im) fp32 pairs, dense; *_col: memory layouts;
 * c may be NULL; rounding as in wmmae_tcec_mma_tile.  mul != 1 (a power of
 * two) routes A through load_matrix_sync_with_mul and D through the scaled
 * store with 1/mul.
 * Replaces: mma_kernel_abcd / mma_kernel_abd, test/tcec/mma_complex.cu:22-101. */
int wmmae_tcec_mma_complex(int type, int ec, float *d, const float *a,
                           const float *b, const float *c, int a_col, int b_col,
                           int c_col, int d_col, int rounding, float mul,
                           void *stream);

/* One MMA D = A*B (+C) through mtk::wmma::mma::load_matrix_sync / mma_sync /
 * store_matrix_sync.  elem: 0 half, 1 bfloat16, 2 float; shape: 0 16x16x16,
 * 1 16x16x32, 2 32x32x8, 3 32x32x16 (float: shapes 0 and 2); a (M x K),
 * b (K x N), c, d (M x N): fp32 images, dense, *_col = 1 for column major;
 * c may be NULL.  shape + 8: the same MMA through the policy-dispatched
 * function objects of tcec::detail (reference:
 * include/wmma_extension/tcec/detail/functions.hpp:10-348, compute_mem_offset
 * of tcec/detail/common.hpp:32-63).  Replaces: test/primitive/mma.cu:11-45. */
int wmmae_primitive_mma(int elem, int shape, float *d, const float *a,
                        const float *b, const float *c, int a_col, int b_col,
                        int c_col, int d_col, void *stream);

/* Error-corrected 16x16x16 half product built with foreach only (A, dA, B, dB
 * fragments filled from the callback's mem_index, three MMAs).  a: 16x16
 * column-major, b: 16x16 row-major, d: column-major.
 * Replaces: test/primitive/foreach.cu:24-80. */
int wmmae_foreach_ec(float *d, const float *a, const float *b, void *stream);

/* y^T = x^T * E, 16 elements, E 16x16 column-major: load_vector into a
 * row_major matrix_a fragment, one MMA, store_vector of the first row.
 * Replaces: test/primitive/gevm.cu:22-43. */
int wmmae_gevm(float *y, const float *x, const float *e, void *stream);

/* Elementwise operators on 16x16x16 fragments: a, b are 16x16 row-major fp32
 * tiles cast to the element type on the way in, out is the result fragment
 * cast back.  op: 0 a+b, 1 a-b, 2 a*alpha, 3 a/alpha, 4 fma(alpha,a,b) =
 * alpha*a + b, 5 fma(a,alpha,b) = a + alpha*b; use: 0 matrix_a, 1 matrix_b, 2 accumulator (elem 2 only);
 * elem: 0 half, 1 bfloat16, 2 float.
 * Replaces: test/primitive/operators.cu:14-57. */
int wmmae_fragment_ops(int op, int use, int elem, float alpha, const float *a,
                       const float *b, float *out, void *stream);

/* An fp32 accumulator (shape 0: 16x16x16, 1: 32x32x8) filled with 1 plus
 * add_eye(alpha) (identity == 0) or make_identity_matrix (identity != 0),
 * stored column-major into out.
 * Replaces: make_eye_kernel, test/primitive/add_eye.cu:24-30. */
int wmmae_fragment_eye(int shape, int identity, float alpha, float *out,
                       void *stream);

/* h (16x16 column-major) = u v^T by one MMA on make_direct_product_fragment
 * (terms 2) / _c3 (terms 3) operands; elem 0 half, 1 bfloat16; from_float != 0
 * uses the fp32-vector overloads, else the (x, dx) ones.
 * Replaces: direct_product_kernel, test/primitive/direct_product.cu:44-99. */
int wmmae_direct_product(int elem, int terms, int from_float, const float *u,
                         const float *v, float *h, void *stream);

/* utils::cp_async<size> (size 4, 8 or 16 bytes per lane): 128 threads move 256
 * elements from src to dst through LDS.  mode 0: lane-linear destinations
 * (the reference's test), 1: scattered destinations, 2: every third thread
 * inactive (its element comes back as zero), 3: two copies in flight released
 * one after the other, 4 and 5: modes 0 and 2 through
 * utils::cp_async::cp_async_lane_linear (size 4 or 16; size 8 returns
 * WMMAE_STATUS_NOT_SUPPORTED).  src must be `size`-aligned.
 * Replaces: cp_async_test_kernel, test/utils/cp_async.cu:15-25. */
int wmmae_utils_cp_async(int size, int mode, void *dst, const void *src,
                         void *stream);

/* utils::cp_async as a three-stage pipeline written with the reference's
 * group calls (cp_async<size>, commit, wait_group<2>): one wave moves `groups`
 * (1..8) groups of `copies` (1..4) copies of 64 x size bytes from src to dst
 * through a ring of three LDS buffers; dst is written after the pipeline has
 * drained, so the copies are the wave's only vector-memory instructions while
 * it runs.  pending (device, groups + 2 ints): the wave's outstanding
 * vector-memory instructions, read from the hardware, [0] with the first three
 * groups out, [1 + g] right after the wait_group<2> that releases group g (at
 * most 2 * copies; above zero while the younger groups are still in flight),
 * [1 + groups] after wait_all (zero).
 * Replaces: the commit / wait_group use of utils.hpp:29-64 (the reference has
 * no test of it). */
int wmmae_utils_cp_async_pipeline(int size, int copies, int groups, void *dst,
                                  const void *src, int *pending, void *stream);

/* One wave prints (device printf, the process's stdout) a 16x16x16 half
 * matrix_a fragment loaded from src (16x16 row-major fp32) with
 * mtk::wmma::print_fragment, then a 32x32 TCEC accumulator filled with `base`
 * (error part 2048*lane) with tcec::print_fragment: a title line and one line
 * per lane each.  type 0..2, ec as in wmmae_tcec_mma_tile.
 * Replaces: test/primitive/print_fragment.cu (detail/print.hpp,
 * tcec/detail/print.hpp:11-55). */
int wmmae_print_fragment(int type, int ec, const float *src, float base,
                         void *stream);

/* out[i] = utils::cast<DST>(in[i]); dst_type 0 half, 1 bfloat16 (out: 16-bit
 * patterns), 2 tf32, 3 float (out: fp32).
 * Replaces: test/utils/cast.cu:1-6 (utils::cast, utils.hpp:21-26). */
int wmmae_utils_cast(int dst_type, const float *in, void *out, long long n,
                     void *stream);

#ifdef __cplusplus
}
#endif
#endif /* WMMAE_TCEC_H */
