/* meshslice_hip.h — C ABI of libmeshslice_hip.so
 *
 * MI355X (gfx950) kernels for the per-device local contraction of MeshSlice's sliced 2-D GEMM.
 * One call = the whole local work of ONE mesh device for ONE sharded matmul: all S slices that
 * the device receives from its all-gathers (output-stationary), or all S partial-output chunks
 * that it hands to its reduce-scatters (LHS- / RHS-stationary).
 *
 * The reference has no FFI seam; each entry point replaces the einsum / matmul calls of one
 * per-device body of the reference's TensorParallel.py (cited per function).
 *
 * Conventions
 *   - every pointer is a DEVICE pointer owned by the caller, 16-byte aligned; the slice / chunk
 *     pointer arrays themselves are HOST arrays of S device pointers, read during the call;
 *   - matrices are row-major with a leading dimension in ELEMENTS;
 *   - in_dtype / out_dtype: MS_DTYPE_F32 or MS_DTYPE_BF16; products accumulate in fp32 across the
 *     full contraction (all slices) and are rounded once (round-to-nearest-even) on output;
 *   - contiguous extents and leading dimensions must be multiples of 8 (bf16) or 4 (fp32)
 *     elements — implied by the reference's block size of 8; other extents are free;
 *   - calls are asynchronous on `stream` (a hipStream_t; NULL = the default stream);
 *   - return 0 on success, MS_ERR_* (< 0) otherwise; ms_last_error() then describes the failure;
 *   - the library allocates no device memory.  State it keeps: per host thread, the last error text, the forced tile
 *     variant (ms_set_variant), the reserved compute units (ms_set_reserved_cus) and what ms_query reports of the
 *     thread's last call; per process, a table of device facts and, for ms_gemm_os_noalloc alone, one fixed scratch
 *     array per device in the code object with the stream that used it last;
 *   - calls from several host threads, and calls on several streams, are safe together; the one shared resource is a
 *     split-contraction workspace (ms_gemm_os_ws: the caller's; ms_gemm_os_noalloc: the built-in array), whose rules
 *     stand at those entry points.
 */
#ifndef MESHSLICE_HIP_H
#define MESHSLICE_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MS_DTYPE_F32 0
#define MS_DTYPE_BF16 1

#define MS_OK 0
#define MS_ERR_ARG (-1)         /* bad argument: null pointer, size <= 0, alignment / divisibility */
#define MS_ERR_UNSUPPORTED (-2) /* dtype combination or device architecture not supported */
#define MS_ERR_HIP (-3)         /* a HIP runtime call failed */

#define MS_MAX_SLICES 64        /* largest S accepted by one call */

/* ms_query() selectors */
#define MS_QUERY_CU_COUNT 0     /* compute units of the current device */
#define MS_QUERY_CLOCK_KHZ 1    /* peak engine clock */
#define MS_QUERY_IS_GFX950 2    /* 1 if the current device is gfx950 */
#define MS_QUERY_LDS_BYTES 3    /* LDS bytes per workgroup */
#define MS_QUERY_MAX_SLICES 4   /* MS_MAX_SLICES */
#define MS_QUERY_LAST_LAUNCHES 5 /* kernels launched by the calling thread's last ms_gemm_* call (a product whose tiles
                                   would leave much of the last round of compute units idle is done in two launches) */
#define MS_QUERY_LAST_SPLITS 7   /* ways in which that launch split the contraction (1: not split) */
#define MS_QUERY_LAST_VARIANT 6  /* kernel variant (tile shape, see ms_set_variant) of the first of those launches: 1..14 for
                                   the bf16 kernels, 21..25 for the fp32 kernel.  Lets a measurement name the kernel it timed. */
#define MS_QUERY_LAST_GRID 8     /* workgroups of the first of those launches: the compute units it ran on (at most the
                                   device's, less the reserved ones; fewer when that fills every round of the launch) */

/* Library version, major*10000 + minor*100 + patch. */
int ms_version(void);

/* Text of the last error raised on the calling thread ("" if none). */
const char *ms_last_error(void);

/* Device / library facts; returns -1 for an unknown selector or on a HIP error. */
long ms_query(int what);

/* Output-stationary: C[m,n] = sum_{s<S} A_s[m,k_slice] @ B_s[k_slice,n].
 * Replaces the contractions of MeshFlow_OS (reference TensorParallel.py:162,167,172); with S == 1
 * it is Collective_OS (TensorParallel.py:22).  A_s is the s-th all-gathered column slice of the
 * activations (lda), B_s the s-th all-gathered row slice of the weights (ldb).  C is written in
 * out_dtype (ldc).  A call is one kernel launch on `stream`, or two (disjoint column ranges of C) when one
 * tile shape alone would leave much of its last round of compute units idle. */
int ms_gemm_os(const void *const *A_slices, const void *const *B_slices, int S,
               int m, int n, int k_slice, int lda, int ldb,
               void *C, int ldc, int in_dtype, int out_dtype, void *stream);

/* Output-stationary with a fused epilogue (bf16 operands only):
 *     Y = act(sum_s A_s @ B_s) + residual          (fp32, then one rounding to out_dtype into C)
 *     row_sum[i]   += sum_j Y[i,j]                 (optional, fp32 atomics)
 *     row_sumsq[i] += sum_j Y[i,j]^2               (optional, fp32 atomics)
 * Folds into the local product the element-wise work the reference's transformer block does right
 * after an output-stationary layer: the GELU after ff1 (reference ShardedLayers.py:181-182), the
 * residual add before a layer norm (:178,:184) and that norm's local row moments, which the mesh
 * then sums over its columns (mn_l / sqmn_l, :125-126: divide by n for the means).
 * activation: MS_ACT_NONE or MS_ACT_GELU (tanh form, the default of jax.nn.gelu).  residual: [m,n] in
 * out_dtype with leading dimension ldr, or NULL; it may be C itself (every element is read before it is
 * written), which turns one call per slice into the reference's running sum C += A_s @ B_s
 * (TensorParallel.py:167) for callers that issue each slice's product as its all-gather completes.
 * row_sum / row_sumsq: [m] fp32 vectors the caller has zeroed, or NULL; the order of the atomic additions is not fixed, so their last bits can differ from
 * run to run. */
#define MS_ACT_NONE 0
#define MS_ACT_GELU 1
int ms_gemm_os_fused(const void *const *A_slices, const void *const *B_slices, int S,
                     int m, int n, int k_slice, int lda, int ldb,
                     void *C, int ldc, int in_dtype, int out_dtype,
                     int activation, const void *residual, int ldr,
                     float *row_sum, float *row_sumsq, void *stream);

/* Output-stationary with a workspace: ms_gemm_os_fused (activation MS_ACT_NONE, residual / row_sum / row_sumsq NULL: the
 * plain product of ms_gemm_os) that may split the contraction.  A product with a small output and a long contraction
 * (the backward-data GEMM of an LHS-stationary layer on a large mesh: 2048 x 1536 x 12288 is 64 tiles for 256 compute
 * units) leaves most of the device idle if every output tile is one work item.  With a workspace the call may cut the
 * K range of every tile into 2..8 parts that run on different compute units; each part leaves its fp32 partial tile in
 * the workspace, and the part that finishes last adds them up in a fixed order (so the result does not depend on
 * timing: the same call gives the same bits every time) and writes its part of C.  Only the plain product is split: with
 * an activation, a residual or row moments the call runs as ms_gemm_os_fused does.  bf16 and fp32 products split alike.
 * No counterpart in the reference, where XLA picks the contraction's schedule.
 * workspace: device memory, 256-byte aligned, prepared once with ms_workspace_init and then reusable by any number of
 * calls, one at a time (calls that share a workspace must not overlap: same stream, or ordered by events);
 * ms_workspace_bytes() is the size with which no product is refused a split for lack of room, a smaller one only
 * narrows the choice.  workspace == NULL behaves like ms_gemm_os_fused. */
int ms_gemm_os_ws(const void *const *A_slices, const void *const *B_slices, int S,
                  int m, int n, int k_slice, int lda, int ldb,
                  void *C, int ldc, int in_dtype, int out_dtype,
                  int activation, const void *residual, int ldr,
                  float *row_sum, float *row_sumsq,
                  void *workspace, size_t workspace_bytes, void *stream);

/* ms_gemm_os_ws (plain product) for callers that cannot allocate device memory or be handed a workspace: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference.  The
 * split-contraction workspace is a fixed array inside the library's code object (4096 + 48 MiB per device, held until the
 * process ends); the call allocates and frees nothing.  A product whose exchange of partial tiles would not fit that
 * array is refused with MS_ERR_UNSUPPORTED (the message names the sizes) — use ms_gemm_os_ws there.  Only products that
 * split their contraction touch the array (few output tiles, a long contraction); all such calls on one device share it.
 * Calls on one stream are ordered by the stream.  A call that arrives on another stream than the array's previous user
 * first waits for the device to go idle (hipDeviceSynchronize, under a per-device lock held until the call's kernels
 * are queued), so eager calls from several streams or host threads never meet in the array — at the price of that wait
 * whenever the stream changes.  What is NOT ordered: a call made while `stream` is being captured launches nothing
 * now, so replays of such a graph must be kept from overlapping other users of the array by the caller (replay on one
 * stream, or order with events); and the first call on a device that needs the array looks its address up
 * (hipGetSymbolAddress), which should happen outside a capture. */
int ms_gemm_os_noalloc(const void *const *A_slices, const void *const *B_slices, int S,
                       int m, int n, int k_slice, int lda, int ldb,
                       void *C, int ldc, int in_dtype, int out_dtype, void *stream);

/* Bytes of workspace that let every product split its contraction on the current device (0 on a HIP error). */
size_t ms_workspace_bytes(void);

/* Prepares a workspace for ms_gemm_os_ws: clears its arrival counters (the first 4096 bytes) on `stream`.  Needed once
 * after allocation; every call leaves the counters cleared again. */
int ms_workspace_init(void *workspace, size_t bytes, void *stream);

/* LHS-stationary: for s < S, Y_s[m,n_slice] = A[m,k] @ W_s[n_slice,k]^T  (fp32 out).
 * Replaces the contractions of MeshFlow_LS (TensorParallel.py:181,187); S == 1 is Collective_LS
 * (TensorParallel.py:26).  A is the device's own shard; W_s the s-th all-gathered row slice of the
 * [out,in] weights; Y_s is the partial-output chunk the mesh reduce-scatters over its columns.
 * The tile list is chunk-major and the workgroups take tiles in list order, so the chunks tend to complete in slice
 * order, but a plain call promises nothing before it has ended on its stream; a consumer that wants Y_s earlier uses
 * ms_gemm_ls_signal. */
int ms_gemm_ls(const void *A, int lda, const void *const *W_slices, int ldw, int S,
               int m, int n_slice, int k,
               float *const *Y_chunks, int ldy, int in_dtype, void *stream);

/* RHS-stationary: for s < S, Y_s[m_slice,n] = X_s[k,m_slice]^T @ W[k,n]  (fp32 out).
 * Replaces the contractions of MeshFlow_RS (TensorParallel.py:203,209); S == 1 is Collective_RS
 * (TensorParallel.py:31).  X_s is the s-th all-gathered column slice of the [in,tokens] operand,
 * stored [k,m_slice] and used transposed; W is the device's own shard. */
int ms_gemm_rs(const void *const *X_slices, int ldx, const void *W, int ldw, int S,
               int m_slice, int n, int k,
               float *const *Y_chunks, int ldy, int in_dtype, void *stream);

/* ms_gemm_ls / ms_gemm_rs with the chunks written in out_dtype (MS_DTYPE_F32 or MS_DTYPE_BF16; Y_chunks then
 * points to buffers of that type, ldy in elements).  bf16 chunks are what the reference itself hands to its
 * reduce-scatter for bf16 operands (the einsum result takes the operand dtype, TensorParallel.py:181-189,
 * :203-212): half the bytes to write and to reduce, one rounding of the fp32 accumulator per chunk element.
 * The fp32 entry points above keep the partial sums exact until after the reduction. */
int ms_gemm_ls_ex(const void *A, int lda, const void *const *W_slices, int ldw, int S,
                  int m, int n_slice, int k,
                  void *const *Y_chunks, int ldy, int in_dtype, int out_dtype, void *stream);
int ms_gemm_rs_ex(const void *const *X_slices, int ldx, const void *W, int ldw, int S,
                  int m_slice, int n, int k,
                  void *const *Y_chunks, int ldy, int in_dtype, int out_dtype, void *stream);

/* ms_gemm_ls_ex / ms_gemm_rs_ex with completion counters, so that the reduce-scatter of chunk s (the psum_scatter that
 * follows each einsum in MeshFlow_LS / MeshFlow_RS, TensorParallel.py:182-189, :204-212) can start while the later
 * chunks are still being computed.  chunk_done points to S unsigned counters in device memory, zero before the call;
 * the kernel adds 1 to chunk_done[s] after each output tile of Y_s is in memory (system-scope release: whoever reads
 * the count, from another stream or, through a copy, from the host, then reads the counted tiles).  Y_s is complete
 * when chunk_done[s] == *tiles_per_chunk, which the call writes (host memory) before it returns.  The counters are
 * only added to: clear them before the next call. */
int ms_gemm_ls_signal(const void *A, int lda, const void *const *W_slices, int ldw, int S,
                      int m, int n_slice, int k,
                      void *const *Y_chunks, int ldy, int in_dtype, int out_dtype,
                      unsigned *chunk_done, int *tiles_per_chunk, void *stream);
int ms_gemm_rs_signal(const void *const *X_slices, int ldx, const void *W, int ldw, int S,
                      int m_slice, int n, int k,
                      void *const *Y_chunks, int ldy, int in_dtype, int out_dtype,
                      unsigned *chunk_done, int *tiles_per_chunk, void *stream);

/* ms_gemm_os_ws (without the fused epilogue) whose kernel reads slice s of A and of B only after slice_ready[s] has
 * become non-zero: the output-stationary body of the reference gathers slice k + 1 while slice k is being multiplied
 * (MeshFlow_OS, TensorParallel.py:163-171, where XLA overlaps the all-gathers with the einsum of the slice before);
 * here the product is ONE launch that may be enqueued before any slice has arrived, and whoever fills slice s (a
 * gather on another stream) sets slice_ready[s] afterwards, with ms_signal_set on that stream or with any store that
 * is a release at system scope.  slice_ready points to S + 1 words of device memory: words 0 .. S-1 are the flags,
 * zero until their slice is complete (flags of slices that are already there are set before the call); word S must be
 * zero before the call and is set to 1 by the kernel when a wait for a slice lasted longer than timeout_ms (1..60000):
 * the kernel then goes on and ends, and the contents of C are void.  The caller reads that word after the stream has
 * been synchronised.
 * The kernels are persistent and hold every register of the compute units they run on (see ms_set_reserved_cus): a
 * producer that needs compute units of this device (a copy or collective kernel) only runs beside a waiting product if
 * units have been reserved for it; without them both stand still until the timeout. */
int ms_gemm_os_gated(const void *const *A_slices, const void *const *B_slices, int S,
                     int m, int n, int k_slice, int lda, int ldb,
                     void *C, int ldc, int in_dtype, int out_dtype,
                     void *workspace, size_t workspace_bytes,
                     unsigned *slice_ready, unsigned timeout_ms, void *stream);

/* ms_gemm_ls_signal / ms_gemm_rs_signal behind the same gate: the kernel reads the gathered operand slice of chunk s
 * (W_s, X_s) only after slice_ready[s] has become non-zero, as MeshFlow_LS / MeshFlow_RS gather slice k + 1 while chunk k
 * is being multiplied (TensorParallel.py:176-189, :198-212); the stationary operand (A, W) is read from the start.
 * slice_ready and timeout_ms as in ms_gemm_os_gated (S flags and the status word).  chunk_done and tiles_per_chunk may
 * both be NULL (no completion counters); with them one launch has both ends open: slices arrive while it runs, and chunks
 * are handed on as they complete.  The tile list is chunk-major, so a launch of more workgroups than one chunk has
 * tiles starts on several chunks at once and each workgroup waits for its own chunk's slice. */
int ms_gemm_ls_gated(const void *A, int lda, const void *const *W_slices, int ldw, int S,
                     int m, int n_slice, int k,
                     void *const *Y_chunks, int ldy, int in_dtype, int out_dtype,
                     unsigned *chunk_done, int *tiles_per_chunk,
                     unsigned *slice_ready, unsigned timeout_ms, void *stream);
int ms_gemm_rs_gated(const void *const *X_slices, int ldx, const void *W, int ldw, int S,
                     int m_slice, int n, int k,
                     void *const *Y_chunks, int ldy, int in_dtype, int out_dtype,
                     unsigned *chunk_done, int *tiles_per_chunk,
                     unsigned *slice_ready, unsigned timeout_ms, void *stream);

/* Sets *flag = value (device memory) once everything enqueued on `stream` before the call has completed, as a release
 * at system scope: the producer's half of the gated calls (and a way to clear or preset flags in stream order).  No
 * counterpart in the reference, where XLA orders the gathers and the einsums. */
int ms_signal_set(unsigned *flag, unsigned value, void *stream);

/* Timing helpers (replace the wall-clock loop of CostModel.estimateMatmul, reference
 * CostModel.py:74-98): run the same call `warmup` times untimed, then `reps` times, each launch
 * bracketed by HIP events on `stream`; ms_out[r] receives the r-th launch's milliseconds.
 * Synchronise the stream before returning. */
int ms_time_os(const void *const *A_slices, const void *const *B_slices, int S,
               int m, int n, int k_slice, int lda, int ldb,
               void *C, int ldc, int in_dtype, int out_dtype, void *stream,
               int warmup, int reps, float *ms_out);
int ms_time_ls(const void *A, int lda, const void *const *W_slices, int ldw, int S,
               int m, int n_slice, int k,
               float *const *Y_chunks, int ldy, int in_dtype, void *stream,
               int warmup, int reps, float *ms_out);
int ms_time_rs(const void *const *X_slices, int ldx, const void *W, int ldw, int S,
               int m_slice, int n, int k,
               float *const *Y_chunks, int ldy, int in_dtype, void *stream,
               int warmup, int reps, float *ms_out);
/* The same for ms_gemm_os_ws (plain product) and for ms_gemm_ls_ex / ms_gemm_rs_ex (chunks in out_dtype). */
int ms_time_os_ws(const void *const *A_slices, const void *const *B_slices, int S,
                  int m, int n, int k_slice, int lda, int ldb,
                  void *C, int ldc, int in_dtype, int out_dtype,
                  void *workspace, size_t workspace_bytes, void *stream,
                  int warmup, int reps, float *ms_out);
int ms_time_ls_ex(const void *A, int lda, const void *const *W_slices, int ldw, int S,
                  int m, int n_slice, int k,
                  void *const *Y_chunks, int ldy, int in_dtype, int out_dtype, void *stream,
                  int warmup, int reps, float *ms_out);
int ms_time_rs_ex(const void *const *X_slices, int ldx, const void *W, int ldw, int S,
                  int m_slice, int n, int k,
                  void *const *Y_chunks, int ldy, int in_dtype, int out_dtype, void *stream,
                  int warmup, int reps, float *ms_out);

/* Block-cyclic slices of a shard, all S of them in one pass over it:
 *     axis 1:  dst_slices[s][r, (b / S) * B + e] = src[r, b * B + e]   for column blocks b with b % S == s
 *     axis 0:  dst_slices[s][(b / S) * B + e, c] = src[b * B + e, c]   for row blocks b with b % S == s
 * Replaces the reshape to (.., L/(S*B), S, B) and the dynamic_slice_in_dim along the S axis with which a
 * mesh device cuts slice s out of its shard before the all-gather (TensorParallel.py:155-158, :177-178,
 * :198-199).  src is [rows, cols] (ld_src); slice s is [rows, cols / S] (axis 1) or [rows / S, cols]
 * (axis 0) with leading dimension ld_dst, so a slice can be written straight into its place in a larger
 * gathered buffer.  The sliced extent must be a multiple of S * B.  dtype only sets the element size.
 * Pointers need the alignment of one element; 16-byte aligned pointers, row lengths and leading
 * dimensions (and B elements a multiple of 16 bytes for axis 1) select the 16-byte kernels. */
int ms_pack_slices(const void *src, int ld_src, int rows, int cols, int axis, int S, int B,
                   void *const *dst_slices, int ld_dst, int dtype, void *stream);

/* The inverse placement, for a device's output shard, with the sum a reduce-scatter takes on the way:
 *     axis 1:  out[r, (h * S + s) * B + e] = sum_{p<P} chunks[p * S + s][row_off + r, col_off + h * B + e]
 *     axis 0:  out[(h * S + s) * B + e, c] = sum_{p<P} chunks[p * S + s][row_off + h * B + e, col_off + c]
 * Replaces psum_scatter of partial chunk s (the sum over the P peers and the choice of this device's
 * window, TensorParallel.py:182,188,204,210), the dynamic_update_slice_in_dim that puts the result at
 * slice position s of the (.., S, B) view of the output shard (:184,190,206,211) and the final reshape
 * (:193,:214).  out is [rows, cols] (ld_out) in out_dtype; each chunk has leading dimension ld_chunk and
 * element type in_dtype, and (row_off, col_off) is the corner of the window of every chunk that this
 * device keeps, [rows, cols / S] (axis 1) or [rows / S, cols] (axis 0).  With P == 1 (chunks already
 * reduced, as after a real reduce-scatter) it is a pure placement.  The sum runs in fp32 in peer order
 * and is rounded once (round-to-nearest-even) to out_dtype.  P * S <= 64. */
int ms_unpack_chunks(const void *const *chunks, int P, int S, int ld_chunk, int row_off, int col_off,
                     int rows, int cols, int axis, int B, void *out, int ld_out,
                     int in_dtype, int out_dtype, void *stream);

/* Measurement aid (no counterpart in the reference): the rate at which the current device sustains a bare
 * stream of one bf16 MFMA instruction — operands and accumulators resident in registers, no memory traffic.
 * Under its package power limit the device clocks such a stream below the data-sheet frequency, by an amount
 * that depends on the instruction, on the waves per SIMD that issue it and on the operand data, so this is
 * the practical ceiling against which a kernel's achieved rate can be read.
 * shape: MS_MFMA_32X32X16 (v_mfma_f32_32x32x16_bf16, 8 passes) or MS_MFMA_16X16X32 (v_mfma_f32_16x16x32_bf16,
 * 4 passes); waves_per_simd: 1 or 2 (workgroups of 4 or 8 waves, one per compute unit).
 * operands: 16 fragments x 64 lanes x 8 bf16 (16 KB, 16-byte aligned), typically drawn like the GEMM's inputs;
 * sink: one float per launched thread (256 x waves_per_simd x CU count floats) that receives the sums;
 * iters: loop trips of 64 MFMAs per wave.  Launches warmup + reps kernels on `stream`, waits, and returns the
 * mean milliseconds per launch in *ms_out and the FLOPs of one launch in *flops_per_launch. */
#define MS_MFMA_32X32X16 0
#define MS_MFMA_16X16X32 1
int ms_probe_mfma_stream_ex(const void *operands, float *sink, int shape, int waves_per_simd, int iters,
                            int warmup, int reps, float *ms_out, double *flops_per_launch, void *stream);

/* ms_probe_mfma_stream_ex for MS_MFMA_32X32X16 at one wave per SIMD, the instruction and occupancy of the
 * big-tile bf16 kernels; reads the first 8 fragments (8 KB) of operands. */
int ms_probe_mfma_stream(const void *operands, float *sink, int iters, int warmup, int reps,
                         float *ms_out, double *flops_per_launch, void *stream);

/* Measurement aid (no counterpart in the reference): the output-stationary 256x384x64 kernel on the 16x16x32 MFMA
 * (bf16 in, bf16 out; what ms_gemm_os runs on BASELINE's configuration 2) with parts of its K loop left out, timed on
 * the caller's operands: what a part costs is the difference to skip = 0 on the same data, tile loop and clock.
 * skip (one of the built combinations 0, 1, 2, 3, 4, 8, 16, 24) is a sum of
 *   1  no global -> LDS loads inside the K loop (the stage buffers keep the tile's first two stages),
 *   2  no fragment reads inside the K loop (the registers keep the tile's first fragments),
 *   4  no MFMAs (nor, with nothing left to consume them, fragment reads): the operand stream alone,
 *   8  no wait for the loads before a K step's barrier,   16  no barrier inside the K loop.
 * With skip != 0 the contents of C are WRONG (and with 8 or 16 the kernel races on its own LDS buffers): C is scratch
 * here.  Arguments as ms_gemm_os with in_dtype = out_dtype = MS_DTYPE_BF16; launches warmup + reps kernels on `stream`,
 * waits, and returns the mean milliseconds per launch in *ms_out. */
int ms_probe_os_parts(int skip, const void *const *A_slices, const void *const *B_slices, int S,
                      int m, int n, int k_slice, int lda, int ldb, void *C, int ldc,
                      int warmup, int reps, float *ms_out, void *stream);

/* Measurement aid (no counterpart in the reference): the rate of a bare L2 -> LDS stream.  One workgroup of four
 * waves per compute unit issues nothing but 128-bit direct-to-LDS buffer loads, 80 KB per workgroup and step (the
 * stage size of the 256x384x64 kernels); the workgroups that share an XCD walk the same region of region_steps x 80 KB
 * of `buffer` round and round (8 regions, one per XCD: buffer_bytes >= 8 x region_steps x 81920), so with
 * region_steps <= 48 every load after the first round hits in that XCD's 4 MB L2.  A wave has at most
 * in_flight_steps (1..3) steps' loads outstanding.  sink: one float the kernel may write (it never does for finite
 * data).  Returns the mean milliseconds per launch in *ms_out and the bytes one launch moves in *bytes_per_launch. */
int ms_probe_l2_lds_stream(const void *buffer, size_t buffer_bytes, int region_steps, int in_flight_steps, int steps,
                           int warmup, int reps, float *sink, float *ms_out, double *bytes_per_launch, void *stream);

/* Hook for tests and measurements (thread-local): later bf16 calls on this thread use tile variant `variant % 100`
 * (1..14, 0 = the library's choice) and split the contraction `variant / 100` ways (2..8, 0 = the library's choice;
 * a forced split needs a workspace and an output-stationary product).  21..25 name the fp32 kernel's tiles instead
 * (256x128, 128x192, 128x128, 64x64, 192x192; split counts as above): fp32 calls then use that tile and bf16 calls the library's choice,
 * as fp32 calls do under 1..14.  Unknown ids are rejected with MS_ERR_ARG. */
int ms_set_variant(int variant);

/* Compute units that the GEMM launches of the calling thread leave free (default 0; returns MS_ERR_ARG outside
 * [0, 1024]).  The kernels are persistent, at most one workgroup per compute unit (fewer when that fills all rounds of
 * the launch evenly; two of the 128x128 kernel while nothing is reserved), holding all of the unit's registers: nothing
 * else runs on a unit until its workgroup has ended.  A caller that overlaps the chunks' reduce-scatter with
 * the product (the point of the sliced dataflows, TensorParallel.py:182-189, :204-212) reserves the units that the
 * collective's kernels need; multiples of 8 keep the workgroup-to-XCD mapping of the tile walk.  No counterpart in
 * the reference, where XLA schedules both. */
int ms_set_reserved_cus(int n);

#ifdef __cplusplus
}
#endif
#endif /* MESHSLICE_HIP_H */
