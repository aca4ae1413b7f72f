/*
 * Measurement aids of libwmmae_tcec.so that are no part of the product ABI
 * (include/wmmae_tcec.h): they exist for the test suite and for bench.py.
 * Same conventions: device pointers, `stream` a hipStream_t as void*, return 0
 * or a negative wmmae_status.
 */
#ifndef WMMAE_TCEC_AUX_H
#define WMMAE_TCEC_AUX_H

#ifdef __cplusplus
extern "C" {
#endif

/* Measurement aid (no counterpart in the reference): one wave writes nsamples
 * pairs out[2i] = constant-rate counter (100 MHz), out[2i+1] = shader cycle
 * counter, one pair every period_ticks of the constant counter, then ends
 * (nsamples * period_ticks <= 1e9, i.e. 10 s).  Launched on a second stream it
 * records the shader clock while other kernels run. */
int wmmae_clock_samples(unsigned long long *out, int nsamples,
                        long long period_ticks, void *stream);

/* One raw MFMA D = A*B + C on 16-bit patterns (type 0 half, 1 bfloat16);
 * (m,n,k) one of (16,16,16), (16,16,32), (32,32,8), (32,32,16); a: m x k,
 * b: k x n, c/d: m x n, all row-major.
 * The instruction under the reference's test/primitive/mma.cu:11-45
 * (mma::mma_sync on one tile), bare: the probe the oracle's model of the matrix
 * core's accumulate arithmetic is measured and checked with. */
int wmmae_mfma_probe(int type, int m, int n, int k, float *d,
                     const unsigned short *a, const unsigned short *b,
                     const float *c, void *stream);

/* Probe of the pipeline hazard that wmma_extension_amd/isa_check.py looks for
 * in the generated code (no counterpart in the reference): one wave multiplies
 * a 16x32 tile of ones by a 32x16 tile of ones (bf16, 16x16x32 MFMA placed by
 * inline asm) right after a vector-ALU instruction has overwritten two of each
 * lane's eight k of the A operand with twos.  d: 256 floats (the wave's
 * accumulator registers), each 40 if the matrix core read the new register
 * contents and 32 if it read the old ones.  producer 0: v_mov_b32, 1:
 * v_accvgpr_read_b32; gap 0: the write directly in front of the MFMA, 1:
 * s_nop 0 between them, 2: s_nop 1, 3: one unrelated vector instruction. */
int wmmae_mfma_source_hazard_probe(int producer, int gap, float *d,
                                   void *stream);

/* Host only, no device access (no counterpart in the reference): where the
 * GEMM kernel that reads the fp32 operands itself begins a lane's 16-byte read
 * of k stage `stage` (32 floats a stage) of a row of k contiguous floats, in
 * floats from the row's start, computed by the address arithmetic the kernel
 * is compiled from.  tail != 0: the kernel variant for k % 32 != 0.  lane
 * 0..63, k >= 4, 0 <= stage < ceil(k / 32).  For a test that every read lies
 * inside its row: 0 <= *first and *first + 4 <= k. */
int wmmae_direct_read_first(int tail, int k, int stage, int lane,
                            long long *first);

/* Host only (no counterpart in the reference): the number of K slices
 * wmmae_tcec_sgemm* cuts a product into on the path it takes for these
 * arguments (flags as there, path flags included; a workspace of
 * wmmae_tcec_sgemm_workspace_bytes assumed).  1: K is not cut, or the single
 * kernel runs.  The two GEMM kernels plan their slices for their own tiles, so
 * the counts of the forced packed and the forced direct path may differ - and
 * with them the last bits of C, since the slices' partial sums are rounded. */
int wmmae_tcec_sgemm_k_slices(int m, int n, int k, int batch, int policy,
                              int flags, int *slices);

/* Host only (no counterpart in the reference): the time estimates the driver
 * chooses its path with, in seconds, for op(A) = 'T', op(B) = 'N' with tight
 * leading dimensions and aligned bases: seconds[0] the single kernel,
 * seconds[1] split passes + GEMM on packed operands, seconds[2] the GEMM kernel
 * that splits the fp32 operands itself; infinity for a path the product cannot
 * take.  The smallest is the path wmmae_tcec_sgemm* takes.  For checking the
 * estimates against measured times. */
int wmmae_tcec_path_estimates(int m, int n, int k, int batch, int policy,
                              double *seconds);

/* Measurement hook (no counterpart in the reference): the calling thread's
 * next wmmae_tcec_sgemm* / wmmae_tcec_gemm_packed calls record `begin_event`
 * on their stream right before the MFMA GEMM kernel of the packed or the direct
 * path and `end_event` right after it (after the fold of its K slices, where
 * there is one), so that a caller can time that kernel inside a whole call
 * (hipEventElapsedTime after the events have completed).  Both hipEvent_t, or
 * both NULL to switch the hook off.  The single-kernel ("fused") path records
 * nothing.  The events stay the caller's. */
int wmmae_tcec_time_gemm_kernel(void *begin_event, void *end_event);

/* Test hook (no counterpart in the reference): the calling thread's next
 * wmmae_tcec_sgemm* / wmmae_tcec_gemm_packed calls and workspace queries cut K
 * into `slices` slices (at most 32, at least six k stages of 32 each: smaller
 * products get fewer) instead of what the time estimates choose; 0 restores
 * the estimates.  For running two paths on the same cut of K, where they give
 * the same bits. */
int wmmae_tcec_force_k_slices(int slices);

#ifdef __cplusplus
}
#endif
#endif /* WMMAE_TCEC_AUX_H */
