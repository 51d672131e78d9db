/*
 * sbvr_hip.h -- C ABI of libsbvr_hip.so, the MI355X (gfx950) implementation of
 * the SBVR compressed-domain linear layer.
 *
 * Every entry point takes plain device pointers and sizes, launches on the HIP
 * stream it is given (a hipStream_t passed as void*; NULL is the default
 * stream), never synchronises, never allocates and never throws: the return
 * value is 0 on success or one of the negative SBVR_HIP_E* codes, and
 * sbvr_hip_last_error() returns a text for the last failure on the calling
 * thread.  Tensors are dense, row-major, in the layouts that sbvr/core.py of the
 * reference produces (cited per function).
 *
 * The names below replace, one for one, the launchers that the reference's
 * pybind wrappers call (sbvr/kernels/sbvr_ops.cpp); the file and lines of each
 * are given with the declaration.
 */
#ifndef SBVR_HIP_H
#define SBVR_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SBVR_HIP_OK 0
#define SBVR_HIP_EINVAL (-1)      /* null pointer, non-positive or misaligned size */
#define SBVR_HIP_EUNSUPPORTED (-2) /* a shape or format no kernel here covers */
#define SBVR_HIP_ELAUNCH (-3)     /* HIP reported an error at launch */
#define SBVR_HIP_EWORKSPACE (-4)  /* workspace missing or too small */

/* ABI version of this header (major*100 + minor); 101 added the one-row linears with a fused prologue,
 * 102 sbvr_hip_linear_f16_noalloc and sbvr_hip_linear_f16_stream_floor, 103 sbvr_hip_read_floor. */
int sbvr_hip_version(void);

/* Text of the last error raised on this thread ("" if none). */
const char *sbvr_hip_last_error(void);

/* Which kernel the last successful sbvr_hip_linear_f16* call on this thread launched (0 before the first):
 * the routing depends on the shape and on the device (see sbvr_hip_linear_f16), and the kernels differ in
 * how they round, so a caller or a test that cares can ask. */
#define SBVR_HIP_KERNEL_PORTABLE 1       /* one thread per output */
#define SBVR_HIP_KERNEL_DECODE 2         /* up to 16 rows (8 by default), plane sums on the matrix cores, exact activations */
#define SBVR_HIP_KERNEL_ROWS32 3         /* up to 32 rows (9..32 by default), weights decoded to fp16 in registers */
#define SBVR_HIP_KERNEL_PREFILL 4        /* weights decoded to fp16 tiles in LDS */
#define SBVR_HIP_KERNEL_PREFILL_SPLIT 5  /* the same with K split across workgroups (workspace given) */
int sbvr_hip_last_kernel(void);

/* How that launch treated the weights (0 before the first):
 *   EXACT      coefficients applied to plane sums in fp32, no per-weight rounding (decode and portable kernels);
 *   DECODE     every weight rounded to fp16 once, as decode() of sbvr/core.py:927-949 produces it (bin_combs @
 *              coeff, :345-366): the kernels that decode by table look-up;
 *   PLANEWISE  every weight an fp16 sum built plane by plane, S - 1 roundings (the kernels that decode
 *              arithmetically: 6 and 8 planes, groups of 32 or 64 elements). */
#define SBVR_HIP_ROUNDING_EXACT 1
#define SBVR_HIP_ROUNDING_DECODE 2
#define SBVR_HIP_ROUNDING_PLANEWISE 3
int sbvr_hip_last_rounding(void);

/* Checks that `device` is a gfx950 part and caches its properties.
 * Replaces sbvr_cuda_init, sbvr/kernels/sbvr_ops.cpp:122-150. */
int sbvr_hip_init(int device);

/* Bytes of device workspace sbvr_hip_linear_f16 wants for this shape (0 if
 * none).  The workspace must be zero-filled once after allocation; every call
 * leaves it zero-filled.  Calls that share a workspace must not overlap in
 * time.  Where the decode kernel splits K across workgroups the workspace is
 * required; for the 32-row kernel with few columns and the prefill kernel with
 * few output tiles it is optional: without it that launch is not split along K,
 * which is slower but gives the same result up to the order of the fp32
 * additions. */
size_t sbvr_hip_linear_f16_workspace(int M, int N, int K, int S, int G);

/*
 * out[m,n] = f16( sum_g sum_j coeff_cache[coeff_idx[g,n], j]
 *                   * sum_{k in group g, bit_j(n,k)=1} x[m,k] )  (+ bias[n])
 *
 * i.e. x @ decode(W)^T for a weight W (N,K) held in the reference's default
 * layout (sbvr/core.py:724-731, 782-805):
 *   x           (M, K)      fp16
 *   bvr         (K/32, N, S) uint32, bit k%32 of bvr[k/32, n, j] = plane j of W[n,k]
 *   coeff_idx   (K/G, N)    uint8 (idx_bytes 1) or uint16 (idx_bytes 2)
 *   coeff_cache (L, S)      fp16
 *   bias        (N) fp16 or NULL; added after the sum is rounded to fp16, as
 *               sbvr/kernels/sbvr_kernel.cu:555-559 does
 *   out         (M, N)      fp16
 * fp32 accumulation, one rounding to fp16.  K must be a multiple of G and G of
 * 32.  Which kernel runs (sbvr_hip_last_kernel() tells) depends on the shape:
 *   decode kernel   M <= 16, N >= 16, K and G multiples of 128 with G/128 a power
 *                   of two, S in {2,3,4,6,8}: plane sums on the matrix cores over
 *                   the raw bit planes, the fp16 activations represented exactly;
 *                   within 2 fp16 ulps of the exact sum.  Taken for up to 8 rows
 *                   of such a shape, and for 9..16 rows where the 32-row kernel's
 *                   table look-up form has no instance (6 or 8 planes) or flags
 *                   bit 1 is set (5..16 rows in a variant whose waves share the
 *                   activation operands, where N >= 32 for up to 8 rows, 64 beyond);
 *   32-row kernel   up to 32 rows.  Its table look-up form (2, 3 or 4 planes, K and
 *                   G multiples of 64: a weight is looked up among the subset sums
 *                   of its group's coefficient line; with a workspace and few
 *                   columns K is split across workgroups through the decode
 *                   kernel's accumulators) is taken for 9..32 rows: from 9 rows on
 *                   it is the faster one (4096 -> 14336, 4 planes, 16 rows: 15.4 us
 *                   against 20 us).  Its arithmetic form (K and G multiples of 32,
 *                   S in {2,3,4,6,8}; same results) takes 17..32 rows otherwise, and
 *                   5..16 rows of shapes the decode kernel does not cover (N < 16,
 *                   K or G not a multiple of 128);
 *   prefill kernel  M > 32 (or 17..32 with flags bit 1), K and G multiples of 64,
 *                   same S; with a workspace and few output tiles, K is split
 *                   across workgroups.  With 2, 3 or 4 planes and K and G multiples
 *                   of 128 it is the kernel that decodes by table look-up in
 *                   registers (256 x 256 output tiles, the weights never in LDS),
 *                   otherwise the one that decodes weight tiles into LDS; same
 *                   results up to the order of the fp32 additions;
 *   portable kernel everything else (one thread per output), and with flags bit 0.
 * The 32-row and prefill kernels decode the weights to fp16 first.  Their table
 * look-up forms (2..4 planes) round the sum of a weight's coefficients once,
 * which is how decode() of sbvr/core.py:927-949 produces a weight (bin_combs @
 * coeff, :345-366): against x @ decode(W)^T they are as close as the decode
 * kernel is to the unrounded weights (2 fp16 ulps).  Their arithmetic forms (6
 * and 8 planes, groups of 32 or 64) add the coefficients up in fp16 plane by
 * plane.  Either way the error against unrounded weights is a few 1e-3 of the
 * RMS output, within the 1e-2 relative bound for outputs that are not small
 * against it.  sbvr_hip_last_rounding() tells which of the three a call took.
 * The reference has no kernel of exactly this form (its fp16-activation
 * kernels, sbvr_kernel.cu:121-359 behind sbvr_ops.cpp:79-120, want the
 * trans=True layout); this is the operator its models/sbvr_llama.py:86-87
 * SBVRLinear.forward stands for.
 * flags: bit 0 forces the portable kernel; bit 1 keeps the 32-row kernel out
 * (5..16 rows then take the decode kernel, exact in weights and activations,
 * 17..32 the prefill kernel).
 * Range: where the decode kernel splits K across workgroups, a workgroup's
 * partial sum is clamped to +-130000 before it is added up in fixed point;
 * partial sums beyond twice the fp16 range that would cancel to a finite total
 * come out as a wrong finite value instead.
 */
int sbvr_hip_linear_f16(const void *x, const uint32_t *bvr, const void *coeff_idx,
                        int idx_bytes, const void *coeff_cache, const void *bias,
                        void *out, int M, int N, int K, int S, int G, int L,
                        void *workspace, size_t workspace_bytes, int flags,
                        void *stream);

/*
 * sbvr_hip_linear_f16 for callers that cannot allocate device memory or bring
 * a workspace (code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc).  It has no counterpart in the reference.  Same
 * arguments and results as sbvr_hip_linear_f16 without the workspace pair: the
 * split-K accumulators of the decode and 32-row kernels live in a 4 MiB array
 * inside the library (one copy per GPU, held until the process ends), which
 * holds M * N <= 524288 of them.  The one limit, up to 32 rows: a launch that
 * splits K across workgroups and has more outputs than that runs unsplit where
 * its kernel can (the table look-up kernel of 9 to 32 rows) and is refused
 * with SBVR_HIP_EWORKSPACE where it cannot (the decode kernels, up to 8 rows);
 * launches that do not split K never touch the array and have no limit.  With
 * more than 32 rows the prefill kernel runs without its optional workspace,
 * i.e. not split along K.
 * The call allocates and frees nothing.  Calls that overlap in time on one GPU
 * share the array and race: serialise them (one stream, or events).
 */
int sbvr_hip_linear_f16_noalloc(const void *x, const uint32_t *bvr, const void *coeff_idx,
                                int idx_bytes, const void *coeff_cache, const void *bias,
                                void *out, int M, int N, int K, int S, int G, int L,
                                int flags, void *stream);

/*
 * The same operator for one row (M = 1) with the elementwise step that feeds
 * it folded into its activation load, which saves a kernel launch per use in a
 * batch-1 decode step.  Same arguments as sbvr_hip_linear_f16 unless listed;
 * only shapes the decode kernel covers (N >= 16, K and G multiples of 128 with
 * G/128 a power of two, S in {2,3,4,6,8}); SBVR_HIP_EUNSUPPORTED otherwise (the
 * caller then runs the two steps separately).
 *
 * _swiglu: gate_up is (1, 2K) fp16 = gate | up; the row multiplied with the
 * weight is fp16(fp16(silu(gate)) * up), the argument of down_proj in
 * models/sbvr_llama.py:238-239 (LlamaMLP.forward).
 *
 * _add_rmsnorm: r = fp16(x + delta) is written to x_out, and the row
 * multiplied with the weight is norm_weight * fp16(r * rsqrt(mean(r^2) + eps)):
 * the residual add of models/sbvr_llama.py:396-400 (LlamaDecoderLayer.forward)
 * followed by LlamaRMSNorm.forward, :118-124.  x, delta, x_out: (K) fp16,
 * 16-byte aligned; x_out must not be x or delta.  K <= 16384.
 */
int sbvr_hip_linear_f16_swiglu(const void *gate_up, const uint32_t *bvr, const void *coeff_idx,
                               int idx_bytes, const void *coeff_cache, const void *bias,
                               void *out, int M, int N, int K, int S, int G, int L,
                               void *workspace, size_t workspace_bytes, void *stream);

int sbvr_hip_linear_f16_add_rmsnorm(const void *x, const void *delta, const void *norm_weight, float eps,
                                    void *x_out, const uint32_t *bvr, const void *coeff_idx,
                                    int idx_bytes, const void *coeff_cache, const void *bias,
                                    void *out, int N, int K, int S, int G, int L,
                                    void *workspace, size_t workspace_bytes, void *stream);

/*
 * Measurement aid, no counterpart in the reference: the launch that
 * sbvr_hip_linear_f16 would make for one row of this shape (same grid, same
 * workgroups, the same plane-word and line-index requests in the same order)
 * with everything else left out: no activations, no arithmetic, nothing
 * written to out.  Its duration is what the memory system alone needs for the
 * weight stream of that launch; bench.py --stream-floor times it beside the
 * real kernel.  Same shape limits as the fused one-row linears above.
 */
int sbvr_hip_linear_f16_stream_floor(const uint32_t *bvr, const void *coeff_idx, int idx_bytes,
                                     const void *coeff_cache, void *out, int N, int K, int S, int G, int L,
                                     void *workspace, size_t workspace_bytes, void *stream);

/*
 * Measurement aid, no counterpart in the reference: a launch that only reads
 * `bytes` of buf (a buffer of buf_bytes), whatever grid the linear would use:
 * `workgroups` x `waves` waves (waves <= 16) each request bytes / 1024 /
 * (workgroups * waves) units of 1 KiB, one 16-byte load per lane (the decode
 * kernel's request), `ahead` of them in flight (1, 2, 3, 4, 7, 8, 14 or 16; a
 * divisor of the units per wave), and do nothing else.  pattern 0: at any time
 * the grid reads one contiguous band (unit i of wave w is KiB i * waves_total
 * + w); 1: every wave walks its own contiguous piece; 2: the decode kernel's
 * own pattern over rows of row_bytes (one 32-bit word of K for all columns)
 * with win_bytes of every row per workgroup and 256 bytes of four consecutive
 * rows per unit.  sink: 256 bytes of device memory, never written.  bench.py
 * --read-floor times it over weight copies that rotate through more than the
 * 256 MB memory-side cache.
 */
int sbvr_hip_read_floor(const void *buf, size_t buf_bytes, size_t bytes, int workgroups, int waves, int ahead,
                        int pattern, int row_bytes, int win_bytes, void *sink, void *stream);

/*
 * Query, no counterpart in the reference and no device needed: the launch shape
 * the decode kernels would get for M <= 16 rows of this shape on a device of
 * `cus` compute units.  plan[0..7] = {kind, column tiles per wave, sub-groups
 * of 128 per wave, row tiles, waves per workgroup, column windows, parts of K
 * across workgroups, the most waves the kernel instance may be launched with};
 * kind 1: sbvr_gemv_mfma_kernel, 2: sbvr_gemv_batch_kernel, 0 (all zero): the
 * decode kernels do not cover the shape.
 */
int sbvr_hip_decode_plan(int M, int N, int K, int S, int G, int cus, int *plan);

/*
 * fp16 activations against a weight encoded with trans=True (groups along N):
 *   r_bvr (N/32, K, S) uint32, r_coeff_idx (N/G, K), r_coeff_cache (L, S) fp16
 *   out[m,n] = f16( bias[n] + sum_k x[m,k] * sum_j c[idx[n/G,k], j] * bit_j )
 * Replaces launch_cuda_sbvr_row_deq_mm_T, sbvr/kernels/sbvr_kernel.cu:876-912,
 * called from sbvr_row_deq_mm_T, sbvr/kernels/sbvr_ops.cpp:79-120.
 */
int sbvr_hip_row_deq_mm_T(const void *x, const uint32_t *r_bvr, const void *r_coeff_idx,
                          int idx_bytes, const void *r_coeff_cache, const void *bias,
                          void *out, int M, int N, int K, int S, int G, int L,
                          void *stream);

/*
 * The same product with room for a split of K across workgroups: a workspace of
 * sbvr_hip_row_deq_mm_T_workspace(M, N) bytes (M*N 64-bit accumulators, zero-filled once, 8-byte
 * aligned, left zero by every call; it may be the workspace of sbvr_hip_linear_f16, not used by
 * two calls at once; 0 bytes for a call whose column workgroups already fill the device: it is
 * never split, e.g. any prefill-sized M).  With 4 planes, K a multiple of 128 and groups of 64 columns and more the
 * plane sums run on the matrix cores, and where the columns alone would leave CUs idle (N = 4096
 * on an MI355X) the parts of K are summed through the accumulators, in fixed point, so the result
 * does not depend on their order.  workspace NULL: as sbvr_hip_row_deq_mm_T.  The reference's
 * operator has no such argument (sbvr_ops.cpp:79-120); its bindings here bring their own.
 */
int sbvr_hip_row_deq_mm_T_ws(const void *x, const uint32_t *r_bvr, const void *r_coeff_idx,
                             int idx_bytes, const void *r_coeff_cache, const void *bias,
                             void *out, int M, int N, int K, int S, int G, int L,
                             void *workspace, size_t workspace_bytes, void *stream);
size_t sbvr_hip_row_deq_mm_T_workspace(int M, int N);

/*
 * Both operands SBVR-encoded (default uint32 layout on both sides):
 *   out[m,n] = f16( sum_g sum_l sum_r popcount_g(L_l & R_r) * a_l * b_r ) (+ bias[n])
 * Replaces launch_cuda_sbvr_mm_T, sbvr/kernels/sbvr_kernel.cu:914-1022, called
 * from sbvr_mm_T, sbvr/kernels/sbvr_ops.cpp:35-76.
 */
int sbvr_hip_mm_T(const uint32_t *l_bvr, const void *l_coeff_idx, int l_idx_bytes,
                  const void *l_coeff_cache, const uint32_t *r_bvr,
                  const void *r_coeff_idx, int r_idx_bytes, const void *r_coeff_cache,
                  const void *bias, void *out, int M, int N, int K, int Sl, int Sr,
                  int G, int Ll, int Lr, void *stream);

/*
 * The same product with room for a split of K across workgroups: a workspace of
 * sbvr_hip_mm_T_workspace(M, N) bytes (M*N 64-bit accumulators, zero-filled once, 8-byte aligned,
 * left zero by every call; it may be the workspace of sbvr_hip_linear_f16, not used by two calls
 * at once).  One left row of up to 4 planes (the case the reference's kernels are written for,
 * sbvr_kernel.cu:464-562) at the decode kernel's shapes (N >= 16, K and G multiples of 128, G / 128
 * a power of two, 2, 3, 4, 6 or 8 right planes) runs on that kernel: the left operand's planes,
 * each times its coefficient, are its batch rows, the popcounts come out of the matrix cores and the
 * rows are added up in fp32 before the one rounding.  Where that launch splits K across workgroups
 * (N = 4096 at K = 14336 on an MI355X) it needs the workspace; without one, and for every other
 * shape, the popcount kernels of sbvr_hip_mm_T run.  The reference's operator has no such argument
 * (sbvr_ops.cpp:35-76); its bindings here bring their own.
 */
int sbvr_hip_mm_T_ws(const uint32_t *l_bvr, const void *l_coeff_idx, int l_idx_bytes,
                     const void *l_coeff_cache, const uint32_t *r_bvr,
                     const void *r_coeff_idx, int r_idx_bytes, const void *r_coeff_cache,
                     const void *bias, void *out, int M, int N, int K, int Sl, int Sr,
                     int G, int Ll, int Lr, void *workspace, size_t workspace_bytes, void *stream);
size_t sbvr_hip_mm_T_workspace(int M, int N);

#ifdef __cplusplus
}
#endif
#endif /* SBVR_HIP_H */
