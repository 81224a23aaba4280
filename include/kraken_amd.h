/*
 * kraken_amd.h — C ABI of libkraken_amd.so
 *
 * The local (one-rank) arithmetic of Kraken's fused communication+compute
 * kernels, written for AMD MI355X (gfx950).  The W peer symmetric-memory
 * buffers of the reference are W buffers on this GPU, given in one of two
 * forms: as the W slices of one device tensor ("stack": slice r starts at
 * stack + r * slice_stride  elements), or, in the kr_*_ptrs_bf16 entry
 * points, as a table of W device pointers to separate allocations.
 *
 * Conventions for every entry point
 *   - all data pointers are DEVICE pointers; bf16 = 2-byte bfloat16;
 *   - `stream` is a hipStream_t (NULL = the default stream); a call enqueues
 *     its kernel(s) on that stream and returns without synchronising;
 *   - the library keeps no state between calls and is re-entrant (two exceptions, both named
 *     where they apply: the tuning switches of the environment are read once per process, and
 *     kr_gemm_reduce_noalloc_bf16 uses a device array of the library's own);
 *   - return value: 0 on success; a negative KR_ERR_* code when the arguments
 *     are rejected on the host BEFORE anything is launched (so argument
 *     validation can be exercised on a machine without a GPU); a positive
 *     value is a hipError_t reported by the launch.
 *   - accumulation is fp32 in ascending slice order r = 0..W-1, and results
 *     are rounded to bf16 once (round-to-nearest-even) at the store.
 *
 * The reference has no FFI layer: each function below names the Triton kernel
 * and host wrapper of the reference whose arithmetic it replaces.
 */
#ifndef KRAKEN_AMD_H
#define KRAKEN_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* argument errors (returned before any launch) */
#define KR_OK                 0
#define KR_ERR_NULL_POINTER  -1  /* a required pointer is NULL                      */
#define KR_ERR_ALIGNMENT     -2  /* pointer or stride not 16-byte aligned           */
#define KR_ERR_NUMEL_MOD8    -3  /* element count not a multiple of 8 (128 bit)     */
#define KR_ERR_BAD_DIM       -4  /* negative/zero/inconsistent dimension            */
#define KR_ERR_WORLD_SIZE    -5  /* W outside 1..KR_MAX_WORLD                       */
#define KR_ERR_BIAS_SHAPE    -6  /* bias_numel is neither numel nor D               */
#define KR_ERR_ROW_TOO_LONG  -7  /* D above KR_MAX_ROW for the row-resident kernels */
#define KR_ERR_BAND          -8  /* row band outside [0, M) or M % W != 0           */
#define KR_ERR_LAYOUT        -9  /* operand strides not supported                   */
#define KR_ERR_STRIPE       -10  /* stripe block not a multiple of 8 / bad rank     */
#define KR_ERR_SCRATCH      -11  /* shape needs more than KR_STATIC_SCRATCH_BYTES   */

#define KR_MAX_WORLD 16
#define KR_MAX_ROW   65536

/* Library/ABI version: major*10000 + minor*100 + patch. */
int kr_version(void);

/* Human-readable text for a return code of this library (never NULL). */
const char* kr_strerror(int code);

/* The KRAKEN_AMD_* environment switches (testing and tuning) are read once per process, on the
 * first call that consults them; this reads them again. */
void kr_reload_env(void);

/*
 * W-way elementwise reduce with optional bias.
 *   out[i] = bf16( [bias] + sum_{r=0..W-1} fp32(stack[r*slice_stride + i]) ),  0 <= i < numel
 * bias == NULL: plain sum.  Otherwise bias_numel is either numel (bias has
 * the shape of the input, as the reference passes it) or D (a vector
 * broadcast over rows of length D, numel % D == 0).
 * bias_first != 0: acc starts at bias, slices added after (one-shot order);
 * bias_first == 0: slices summed from 0.0f, bias added last (two-shot order).
 * Requirements: numel % 8 == 0, D % 8 == 0, slice_stride % 8 == 0, all
 * pointers 16-byte aligned, 1 <= W <= KR_MAX_WORLD.  numel == 0 is a no-op.
 *
 * Replaces the reduce loops of
 *   kraken/comm/one_shot_all_reduce.py:36-48          (one_shot_all_reduce_kernel)
 *   kraken/comm/two_shot_all_reduce.py:51-62          (own share of two_shot_all_reduce_kernel)
 *   kraken/fused/one_shot_all_reduce_bias.py:76-94    (one_shot_all_reduce_bias_kernel)
 *   kraken/fused/two_shot_all_reduce_bias.py:66-83    (two_shot_all_reduce_bias_kernel)
 * A two-shot share is this call with `stack`, `bias` and `numel` restricted
 * to the rank's contiguous chunk.
 */
int kr_reduce_bf16(const void* stack, int W, int64_t slice_stride, int64_t numel,
                   const void* bias, int64_t bias_numel, int64_t D, int bias_first,
                   void* out, void* stream);

/*
 * Two-shot share with the reference's interleaved ownership: the flat input is
 * cut into stripes of stripe_block*W elements and rank `rank` owns elements
 * [rank*stripe_block, (rank+1)*stripe_block) of every stripe
 * (kraken/comm/two_shot_all_reduce.py:51-54, kraken/fused/two_shot_all_reduce_bias.py:66-69).
 * The owned elements (those below numel) are reduced (bias, if given, has
 * numel elements and is added last) and written COMPACTLY to out in ascending
 * order; *the caller sizes out* with kr_striped_share_numel().
 * Requirements as kr_reduce_bf16 plus stripe_block % 8 == 0, 0 <= rank < W.
 */
int kr_reduce_striped_bf16(const void* stack, int W, int64_t slice_stride, int64_t numel,
                           const void* bias, int64_t stripe_block, int rank,
                           void* out, void* stream);

/* Number of elements rank `rank` owns under the striped ownership above
 * (negative KR_ERR_* on bad arguments). */
int64_t kr_striped_share_numel(int64_t numel, int W, int64_t stripe_block, int rank);

/*
 * W-way reduce + bias + RMSNorm, one pass over the input.  For each of `rows`
 * rows of length D:
 *   s[c] = [bias] + sum_{r=0..W-1} fp32(stack[r*slice_stride + row*D + c])     (fp32, bias first)
 *   y[row*D + c] = bf16( s[c] * rsqrt(mean_c(s^2) + eps) * fp32(w[c]) )
 * bias: NULL, or [rows*D] (bias_is_vector == 0), or [D] (bias_is_vector != 0).
 * w: [D] bf16.  Requirements: D % 8 == 0, D <= KR_MAX_ROW, slice_stride % 8 == 0.
 *
 * Replaces kraken/fused/one_shot_all_reduce_bias_rms_norm.py:73-91
 * and      kraken/fused/two_shot_all_reduce_bias_rms_norm.py:87-94,110-121
 * (the row is kept in fp32 registers between the reduce and the norm; the
 * reference's two-shot variant rounds it to bf16 in between).
 */
int kr_reduce_rmsnorm_bf16(const void* stack, int W, int64_t slice_stride, int64_t rows, int64_t D,
                           const void* bias, int bias_is_vector, const void* w, float eps,
                           void* y, void* stream);

/*
 * kr_reduce_rmsnorm_bf16 / kr_reduce_rmsnorm_ptrs_bf16 with a workspace, for a few long rows
 * (decode shapes: up to 64 rows whose W * D * 2 input bytes make one compute unit's intake the
 * kernel's time).  A row is then spread over many compute units, one wavefront per 512 elements,
 * and the wavefronts of a row exchange their partial sums of squares through the workspace and add
 * them in a fixed order (results are reproducible run to run and equal the one-workgroup form up
 * to the fp32 rounding of that order).
 * `workspace`: device memory, 16-byte aligned, of at least kr_rmsnorm_workspace_bytes(W, rows, D)
 * bytes (0: this shape is not split; the value does not depend on the shape otherwise, so one
 * buffer serves every call).  It must be ZERO before its first use and is afterwards kept
 * consistent by the kernels themselves (no clearing between calls, also not between replays of a
 * captured graph; clearing it again between calls is harmless).  Calls that use one workspace
 * must not overlap (same stream, or otherwise ordered).  workspace == NULL, a workspace that is
 * too small, or a shape that does not profit: exactly the entry point without workspace.
 * The exchange is a bounded wait (seconds; the wavefronts of a row run at the same time, so it
 * normally lasts a microsecond): a row whose wavefronts did not meet within the bound, which only
 * a workspace shared by overlapping calls or a GPU that other work keeps full for that long can
 * cause, is written as NaN, and 1 + the row's index is stored to *status (device int32, 4-byte
 * aligned, may be NULL; zeroed by the caller; never written otherwise).  After such a time-out the
 * workspace must be zeroed again before its next use (a late wavefront of the failed call may
 * have left a slot that the next call would take for a fresh one).  The wavefronts of a row can
 * only meet if all of them are resident together: the launch is at most 1024 one-wave workgroups,
 * which an otherwise idle GPU starts at once, but a kernel on another stream that keeps every
 * compute unit full (a GEMM, say) can delay some of them by its own run time.
 * No counterpart in the reference (one 1024-thread CTA per row whatever the shape,
 * kraken/fused/one_shot_all_reduce_bias_rms_norm.py:144-145).
 */
int64_t kr_rmsnorm_workspace_bytes(int W, int64_t rows, int64_t D);
int kr_reduce_rmsnorm_ws_bf16(const void* stack, int W, int64_t slice_stride, int64_t rows, int64_t D,
                              const void* bias, int bias_is_vector, const void* w, float eps,
                              void* y, void* workspace, int64_t workspace_bytes, int32_t* status,
                              void* stream);
int kr_reduce_rmsnorm_ptrs_ws_bf16(const void* const* bufs, int W, int64_t rows, int64_t D,
                                   const void* bias, int bias_is_vector, const void* w, float eps,
                                   void* y, void* workspace, int64_t workspace_bytes, int32_t* status,
                                   void* stream);

/*
 * Stand-alone RMSNorm: y = bf16( x * rsqrt(mean(x^2) + eps) * w ), row-wise.
 * Replaces kraken/fused/rms_norm.py:34-43 (_rms_norm_kernel).
 */
int kr_rmsnorm_bf16(const void* x, const void* w, float eps, int64_t rows, int64_t D,
                    void* y, void* stream);

/*
 * bf16 GEMM (fp32 accumulate on the matrix cores) with a fused reduce(+bias)
 * epilogue:
 *   C = A[M,K] @ B[K,N]
 *   for rows m in [band_row0, band_row0 + band_rows):
 *       out[m - band_row0, n] = cast( C[m,n] + sum_{j<n_peers} fp32(peers[j][m - band_row0, n]) + [bias[n]] )
 *   for rows m outside the band, if c_full != NULL:   c_full[m, n] = bf16(C[m,n])
 * A: element (m,k) at A[m*lda_m + k*lda_k]; lda_k must be 1.
 * B: element (k,n) at B[k*ldb_k + n*ldb_n]; either ldb_n == 1 (row-major B)
 *    or ldb_k == 1 (B transposed-contiguous, "NT").
 * peers: n_peers contiguous [band_rows, N] bf16 matrices, peers_stride elements apart
 *        (NULL with n_peers == 0 for a plain GEMM).  bias: [N] bf16 or NULL.
 * out: [band_rows, N], row stride N; bf16, or fp32 when out_is_fp32 != 0.
 * c_full: [M, N] bf16, row stride N, or NULL.
 * tile_pivot: row offset (in rows) by which the order of M tiles is rotated;
 *        changes scheduling only, never the result.
 * Requirements: K % 8 == 0, N % 8 == 0, leading strides % 8 == 0, pointers
 * 16-byte aligned, 0 <= band_row0, band_row0 + band_rows <= M; row strides up to
 * about 8 M elements (128 rows of an operand must lie within 2 GiB, else
 * KR_ERR_LAYOUT).
 * Rounding: the sum is formed in fp32 and rounded once at the store; with a
 * bf16 result, tiles whose peers are added in the epilogue round the product
 * to bf16 before the sum, as gemm_reduce_scatter_fused.py:72 does.
 * Non-finite input: for shapes the 256x256 kernel takes (more than 128 tiles
 * of 256x256, K % 64 == 0), the peers of tiles lying wholly in the band are added
 * on the matrix cores, where an Inf/NaN in a peer also turns the rest of the
 * aligned 16-column block of its row into NaN (32 columns with
 * KRAKEN_AMD_GEMM_MFMA=32).  This default DEVIATES from the reference, whose
 * epilogue adds the peers element by element
 * (gemm_one_shot_all_reduce_fused.py:85-92) and so keeps a non-finite value in its
 * own element; finite inputs give the same results either way.
 * KRAKEN_AMD_GEMM_PEERS=epilogue in the environment selects the reference's
 * behaviour.
 *
 * Replaces
 *   kraken/fused/gemm_one_shot_all_reduce_fused.py:56-99   (band = all rows)
 *   kraken/fused/gemm_reduce_scatter_fused.py:63-72,102-145 (band = this rank's M/W rows)
 *   kraken/fused/all_gather_matmul.py:87-123               (n_peers = 0, tile_pivot = rank*m)
 */
int kr_gemm_reduce_bf16(const void* A, int64_t lda_m, int64_t lda_k,
                        const void* B, int64_t ldb_k, int64_t ldb_n,
                        int64_t M, int64_t N, int64_t K,
                        const void* peers, int n_peers, int64_t peers_stride,
                        const void* bias,
                        int64_t band_row0, int64_t band_rows,
                        void* c_full, void* out, int out_is_fp32,
                        int64_t tile_pivot, void* stream);

/*
 * Pointer-table forms.  `bufs` (`peers` for the GEMM) is a HOST array of W
 * (n_peers) device pointers, one buffer per rank, each 16-byte aligned and at
 * least as long as the stacked form's slice would be; it is copied into the
 * launch, so the array may be reused as soon as the call returns.  Everything
 * else -- arithmetic, order of the adds, requirements, error codes -- is that
 * of the stacked entry point of the same name, whose kernels these share
 * (results are bit-identical for equal inputs).
 *
 * They replace the same reference kernels as their stacked forms, at the
 * interface those kernels actually have -- one buffer per rank, handed over
 * either as a tuple of W tensors from `symm_mem_hdl.get_buffer(i, ...)`
 *   kraken/comm/one_shot_all_reduce.py:93-97,103        (read at :44)
 *   kraken/fused/gemm_one_shot_all_reduce_fused.py:141-146,157 (read at :86-91)
 *   kraken/fused/gemm_reduce_scatter_fused.py:196-201,212      (read at :120)
 * or as the device table `symm_mem_hdl.buffer_ptrs_dev`, read by
 * `tl.load(buffer_ptrs + i)`
 *   kraken/comm/two_shot_all_reduce.py:141              (read at :59)
 *   kraken/fused/one_shot_all_reduce_bias.py:158        (read at :88)
 *   kraken/fused/two_shot_all_reduce_bias.py:175        (read at :74)
 *   kraken/fused/one_shot_all_reduce_bias_rms_norm.py:150     (read at :78)
 *   kraken/fused/two_shot_all_reduce_bias_rms_norm.py:202     (read at :89).
 * A binding that holds the rendezvous handle passes the data pointers of its
 * W buffers; the local rank's buffer is one of the W entries for the reduces
 * and is left out (n_peers = W - 1, each entry moved on to the band's first
 * row) for the GEMM.
 */
int kr_reduce_ptrs_bf16(const void* const* bufs, int W, int64_t numel,
                        const void* bias, int64_t bias_numel, int64_t D, int bias_first,
                        void* out, void* stream);
int kr_reduce_striped_ptrs_bf16(const void* const* bufs, int W, int64_t numel,
                                const void* bias, int64_t stripe_block, int rank,
                                void* out, void* stream);
int kr_reduce_rmsnorm_ptrs_bf16(const void* const* bufs, int W, int64_t rows, int64_t D,
                                const void* bias, int bias_is_vector, const void* w, float eps,
                                void* y, void* stream);
int kr_gemm_reduce_ptrs_bf16(const void* A, int64_t lda_m, int64_t lda_k,
                             const void* B, int64_t ldb_k, int64_t ldb_n,
                             int64_t M, int64_t N, int64_t K,
                             const void* const* peers, int n_peers,
                             const void* bias,
                             int64_t band_row0, int64_t band_rows,
                             void* c_full, void* out, int out_is_fp32,
                             int64_t tile_pivot, void* stream);

/*
 * kr_gemm_reduce_bf16 / kr_gemm_reduce_ptrs_bf16 with a workspace, for shapes whose output tiles
 * do not fill the CUs: few tiles in all (few rows: M of a few hundred), or a last partial round
 * of 256x256 tiles that is mostly empty (tile count = 256 r + tail, tail <= 96, K >= 4096; with
 * r = 0 and a long K loop all tiles are such a tail).
 * The K loop of those tiles is split over S workgroups per tile.  Two launches (three for the
 * tail form: the full rounds run as usual first): the S partial products go to the workspace in fp32; a
 * second kernel sums them in the order 0..S-1 and applies the epilogue (peers, bias, band, c_full)
 * with the adds in the same order and the same rounding as the one-pass kernel.  Results are
 * reproducible run to run and differ from the unsplit result only by the fp32 rounding of the
 * order in which the k-steps are summed.  `workspace`: device memory, 16-byte aligned, of at
 * least kr_gemm_workspace_bytes(M, N, K) bytes (0: this shape is not split); its contents
 * before the call do not matter and are undefined after it.  Calls that use one workspace must
 * not overlap (same stream, or otherwise ordered).  workspace == NULL, a workspace that is too
 * small, or a shape that does not profit: exactly the entry point without workspace.
 * No counterpart in the reference (its GEMM kernels launch one program per output tile,
 * kraken/fused/gemm_reduce_scatter_fused.py:202-204, gemm_one_shot_all_reduce_fused.py:149-153).
 */
int64_t kr_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K);
int kr_gemm_reduce_ws_bf16(const void* A, int64_t lda_m, int64_t lda_k,
                           const void* B, int64_t ldb_k, int64_t ldb_n,
                           int64_t M, int64_t N, int64_t K,
                           const void* peers, int n_peers, int64_t peers_stride,
                           const void* bias,
                           int64_t band_row0, int64_t band_rows,
                           void* c_full, void* out, int out_is_fp32,
                           int64_t tile_pivot,
                           void* workspace, int64_t workspace_bytes, void* stream);
int kr_gemm_reduce_ptrs_ws_bf16(const void* A, int64_t lda_m, int64_t lda_k,
                                const void* B, int64_t ldb_k, int64_t ldb_n,
                                int64_t M, int64_t N, int64_t K,
                                const void* const* peers, int n_peers,
                                const void* bias,
                                int64_t band_row0, int64_t band_rows,
                                void* c_full, void* out, int out_is_fp32,
                                int64_t tile_pivot,
                                void* workspace, int64_t workspace_bytes, void* stream);

/*
 * kr_gemm_reduce_ws_bf16 for callers that can neither allocate a workspace nor let the library
 * allocate: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * It has no counterpart in the reference.  Arguments, arithmetic, tile choice and results are
 * those of kr_gemm_reduce_ws_bf16 called with a workspace of KR_STATIC_SCRATCH_BYTES bytes
 * (bit-identical output); the workspace is a device array inside the library (64 MiB of device
 * memory on every GPU the library is used on, held until the process ends), looked up once per
 * device, and the call performs no allocation of any kind.  A shape whose split would need more
 * (kr_gemm_workspace_bytes(M, N, K) > KR_STATIC_SCRATCH_BYTES) is refused with KR_ERR_SCRATCH
 * before anything is launched; shapes that are not split use no scratch at all.  Every call on
 * one GPU shares that GPU's array: calls that may overlap (different streams without an
 * ordering between them, or several host threads) race on it and must be serialised by the
 * caller.  Nothing in the array has to start at zero (the first launch overwrites every word
 * the second reads), so a call leaves nothing behind that a later call depends on.
 * The first use on a device looks the array up (hipGetSymbolAddress), which can make the HIP
 * runtime load the library's code for that device and with it allocate the array: call kr_init()
 * once per device, with that device current and outside any graph capture, before the first call
 * that must not allocate.  The array used is the one of the device that is current at the call,
 * which must be the device `stream` belongs to (as for any launch).
 */
#define KR_STATIC_SCRATCH_BYTES (64ll << 20)
/* Loads the library's device code for the current device and resolves its scratch array, so that
 * no later call has to (0, or the hipError_t of the lookup).  Idempotent and thread-safe; it has no
 * counterpart in the reference and is needed only by callers of kr_gemm_reduce_noalloc_bf16. */
int kr_init(void);
int kr_gemm_reduce_noalloc_bf16(const void* A, int64_t lda_m, int64_t lda_k,
                                const void* B, int64_t ldb_k, int64_t ldb_n,
                                int64_t M, int64_t N, int64_t K,
                                const void* peers, int n_peers, int64_t peers_stride,
                                const void* bias,
                                int64_t band_row0, int64_t band_rows,
                                void* c_full, void* out, int out_is_fp32,
                                int64_t tile_pivot, void* stream);

/*
 * All-gather matmul that consumes A while it is still arriving:  C[M,N] = A[M,K] @ B[K,N]  (bf16, fp32
 * accumulate, bf16 result), where A is the gathered matrix of W shards of M/W rows, filled by
 * copies that run on another stream while this kernel runs.  The rows arrive in W*splits_per_rank
 * blocks of comm_rows = M / (W*splits_per_rank) rows; progress[b] is 0 until block b (rows
 * [b*comm_rows, (b+1)*comm_rows)) is complete and is then set to 1 by kr_stream_write_value32
 * behind the block's copy.  An output tile whose rows lie in the local shard (rows
 * [rank*M/W, (rank+1)*M/W)) reads them from A_local [M/W, K] (row stride lda_local) and never
 * waits; any other tile first waits until the flags of the blocks it covers are 1, then reads A.
 * The order of the M tiles is rotated so that the local shard's tiles come first, the other
 * shards following in the order rank+1, rank+2, ... in which the copies are issued.
 *   A_local == NULL: local tiles wait for their flags and read A like the others.
 *   progress == NULL: nothing waits (A is complete); A_local is then not used.
 *   wait_limit_us: bound of one tile's wait in microseconds (<= 0: 5 s).  A tile whose flag does
 *     not come in time stores 1 + block index to *status (if status != NULL; the caller zeroes
 *     it beforehand), computes on whatever A holds and exits; tiles that start after that do
 *     not wait.  The kernel therefore always ends; *status != 0 afterwards means C is invalid.
 * A: k-contiguous, row stride lda_m; B as for kr_gemm_reduce_bf16; progress and status are
 * device pointers, 4-byte aligned.  Requirements: M % (W*splits_per_rank) == 0, 0 <= rank < W,
 * K % 8 == 0, N % 8 == 0.  The caller must have the copies (and their flag writes) enqueued
 * on another stream before or right after this call, or the tiles wait until the limit.
 *
 * Replaces kraken/fused/all_gather_matmul.py:25-123 (_matmul_kernel_tma_persistent_w_progress;
 * flag wait :95-110 = wait_gmem_barrier, kraken/_ptx_utils/gmem_barrier_arrive_wait.py:26-68)
 * as launched by _matmul_w_progress (:147-219).
 */
int kr_all_gather_matmul_bf16(const void* A, int64_t lda_m, const void* A_local, int64_t lda_local,
                              const void* B, int64_t ldb_k, int64_t ldb_n,
                              int64_t M, int64_t N, int64_t K,
                              int W, int rank, int splits_per_rank,
                              const uint32_t* progress, int64_t wait_limit_us, int32_t* status,
                              void* C, void* stream);

/*
 * Stream-ordered flag write: *addr = value once everything enqueued on `stream` before this call
 * has completed, with its results visible to kernels that read the flag (release at system scope).
 * Replaces symm_mem_hdl.stream_write_value32 as used behind every chunk copy of the
 * copy-engine all-gather (kraken/comm/copy_engine_all_gather.py:47-53).
 */
int kr_stream_write_value32(uint32_t* addr, uint32_t value, void* stream);

/*
 * Producer GEMM of the copy-engine reduce-scatter:  C[M,N] = A[M,K] @ B[K,N]  (bf16, fp32
 * accumulate, bf16 result, every row written to C), announcing its progress per destination rank
 * while it runs.  Rank r's band is rows [r*M/W, (r+1)*M/W) of C.  The order of the M tiles is
 * rotated so that the band of rank+1 is finished first, then rank+2, ..., the own band last.
 * A workgroup that has stored a tile adds 1 to progress[r] for every band r the tile's rows
 * touch; the workgroup whose add completes band r (all column tiles of all row tiles that
 * overlap the band) stores 1 to signal_pad[r].  When signal_pad[r] is 1, band r of C is complete
 * and visible to a copy that is ordered behind the flag (kr_stream_wait_value32).
 * progress and signal_pad: uint32[W] in device memory, 4-byte aligned, zeroed by the caller
 * before the call.  The count a band reaches depends on the kernel's tile size (128 or 256
 * rows); only signal_pad is meant to be waited on.  M % W == 0, 0 <= rank < W, K % 8 == 0,
 * N % 8 == 0; M == 0 or N == 0: nothing is launched and no flag is set.
 * A, B as for kr_gemm_reduce_bf16.
 *
 * Replaces kraken/fused/gemm_reduce_scatter_ce_persistent.py:46-134
 * (_gemm_producer_persistent_kernel: tile order :88,102, progress counters and signals :117-132)
 * as launched by gemm_producer_w_progress (:178-242).
 */
int kr_gemm_producer_bf16(const void* A, int64_t lda_m, int64_t lda_k,
                          const void* B, int64_t ldb_k, int64_t ldb_n,
                          int64_t M, int64_t N, int64_t K,
                          void* C, int W, int rank,
                          uint32_t* progress, uint32_t* signal_pad, void* stream);

/*
 * Stream-ordered wait: what is enqueued on `stream` behind this call starts once *addr == value
 * (a one-wave kernel that polls the word at system scope).  The wait is bounded: after
 * wait_limit_us microseconds (0: 5 s) the kernel stores 1 to *status (device int32, may be NULL)
 * and ends all the same, so the stream always drains; the caller checks status afterwards.
 * The writer must already be enqueued on another stream, or the wait runs to its limit.
 * Replaces driver.cuStreamWaitValue32(stream, addr, 1, CU_STREAM_WAIT_VALUE_EQ) in front of
 * every band copy of copy_engine_scatter
 * (kraken/fused/gemm_reduce_scatter_ce_persistent.py:153-163).
 */
int kr_stream_wait_value32(const uint32_t* addr, uint32_t value, int64_t wait_limit_us,
                           int32_t* status, void* stream);

/*
 * The two flag primitives of the kernels above in one launch, for testing them on their own:
 * `producers` workgroups each set flags[block] to 1 (release exchange), `consumers` further
 * workgroups each wait until the flag of producer (block - producers) / (consumers / producers)
 * reads 1 (acquire loads in a loop).  flags: uint32[producers] in device memory, zeroed by the
 * caller.  A consumer whose flag does not come within wait_limit_us microseconds (0: 5 s)
 * stores 1 + flag index to *status (device int32, may be NULL) and ends, so the launch always
 * drains.  consumers % producers == 0.
 * Replaces arrive_gmem_barrier / wait_gmem_barrier
 * (kraken/_ptx_utils/gmem_barrier_arrive_wait.py:7-23, 26-68) as exercised by
 * test/test_ptx_utils.py:80-116.
 */
int kr_flag_arrive_wait(uint32_t* flags, int producers, int consumers, int64_t wait_limit_us,
                        int32_t* status, void* stream);

/*
 * Stream-ordered device-to-device copy of `bytes` bytes that runs on the GPU's copy engines
 * (SDMA) and not as a copy kernel, so it takes no compute units from a GEMM running beside it.
 * Source and destination must not overlap.  bytes == 0: nothing is done.
 * Replaces the `.copy_()` calls that the reference issues on its backend stream for the copy
 * engines: the chunk copies of the all-gather (kraken/comm/copy_engine_all_gather.py:44-46) and
 * the band copies of copy_engine_scatter
 * (kraken/fused/gemm_reduce_scatter_ce_persistent.py:165-169).
 */
int kr_copy_engine_memcpy(void* dst, const void* src, int64_t bytes, void* stream);

/*
 * Tile reduce of the copy-engine reduce-scatter variant: `in` is [W*rows, N]
 * bf16 (band r holds what rank r pushed), and
 *   out[m, n] = sum_{i=0..W-1} in[((i + rank + 1) % W) * rows + m, n]
 * accumulated in rotated order starting at rank+1.  acc_bf16 != 0 rounds the
 * running sum to bf16 after every add (what the reference does); 0 keeps fp32.
 * Replaces kraken/fused/gemm_reduce_scatter_ce_persistent.py:245-281.
 */
int kr_reduce_rotated_bf16(const void* in, int W, int64_t rows, int64_t N, int rank,
                           int acc_bf16, void* out, void* stream);

/*
 * fp32 operands for the bf16 GEMM entry points: x = hi + lo with hi = bf16(x), lo = bf16(x - hi),
 * written in one pass as the three bf16 blocks of a product that is three times as long:
 *   [a_hi | a_hi | a_lo] @ [b_hi ; b_lo ; b_hi] = a_hi b_hi + a_hi b_lo + a_lo b_hi
 * (a @ b without the a_lo b_lo term: about 16 mantissa bits, fp32 accumulate).  The reference
 * passes fp32 operands to tl.dot, which multiplies them in TF32
 * (kraken/fused/gemm_one_shot_all_reduce_fused.py:56-64, test/test_gemm_allreduce.py:57-58).
 *   x: [rows, cols] fp32, row stride ld_x (elements), columns contiguous; cols % 8 == 0
 *   side_by_side != 0: out is [rows, 3*cols] bf16, block b of a row at columns [b*cols, (b+1)*cols)
 *                      (row stride ld_out >= 3*cols) -- an operand whose reduction dimension is contiguous
 *   side_by_side == 0: out is [3*rows, cols] bf16, block b at rows [b*rows, (b+1)*rows)
 *                      (row stride ld_out >= cols) -- a row-major right operand [K, N]
 *   pattern 0: blocks hi, hi, lo (left operand); 1: hi, lo, hi (right operand)
 */
int kr_split_fp32(const void* x, int64_t rows, int64_t cols, int64_t ld_x, int side_by_side, int pattern,
                  void* out, int64_t ld_out, void* stream);

/*
 * fp8 operands (e4m3fn: bias 7, no infinities, largest finite 448) for the bf16 GEMM entry points,
 * and fp32 results back to fp8, for the fp8 branch of the all-gather matmul
 * (kraken/fused/all_gather_matmul.py:53,121,213: fp8 operands, fp32 accumulate, fp8 result).  Every
 * e4m3 value is a bf16 value, so the bf16 product of converted operands, accumulated in fp32, is
 * what an fp8 matrix-core instruction with fp32 accumulation computes; the fp32 result is rounded
 * to fp8 once.
 *   kr_cast_fp8_to_bf16: dst[i] = bf16(src[i]), exact; src n bytes, dst n bf16.
 *   kr_cast_f32_to_fp8:  dst[i] = e4m3(src[i]), round to nearest even; finite values of magnitude
 *     448 and more (infinities included) give +-448 (the saturating conversion the reference's
 *     generated code uses); NaN stays NaN.
 * n % 16 == 0; pointers 16-byte aligned; n == 0: nothing is launched.
 */
int kr_cast_fp8_to_bf16(const void* src, int64_t n, void* dst, void* stream);
int kr_cast_f32_to_fp8(const void* src, int64_t n, void* dst, void* stream);

/*
 * out[M, N] = A[M, K] @ Bt[N, K]^T on fp8 (e4m3fn) operands with fp32 accumulation, on the fp8
 * matrix-core instruction (v_mfma_f32_16x16x128_f8f6f4): the product of the fp8 branch of
 * kraken/fused/all_gather_matmul.py:53,121,213 (tl.dot of float8e4nv tiles, fp32 accumulator,
 * result cast to the operands' type) at twice the bf16 rate, without widening the operands.
 *   A: row-major, lda bytes between rows; Bt: the right operand transposed (k contiguous), ldb
 *   bytes between its rows -- the layout the reference's benchmark passes (`b.T` of an [N, K] tensor).
 *   out_kind: 0 = bf16, 1 = fp32, 2 = fp8 (e4m3fn; fp32 sums rounded once, nearest even, magnitudes
 *   from 448 on give +-448, NaN stays NaN -- the conversion of kr_cast_f32_to_fp8); out is [M, N]
 *   contiguous.
 * M % 256 == 0, N % 256 == 0, K % 128 == 0 (other shapes: convert with kr_cast_fp8_to_bf16 and use the
 * bf16 entry points); lda, ldb >= K and multiples of 16; pointers 16-byte aligned.
 */
int kr_gemm_fp8(const void* A, int64_t lda, const void* Bt, int64_t ldb, int64_t M, int64_t N, int64_t K,
                void* out, int out_kind, void* stream);

/*
 * kr_gemm_fp8 for an A whose rows arrive while the kernel runs -- the fp8 form of kr_all_gather_matmul_bf16
 * (same flags, local shard, tile order, wait limit and status word; see there), which is what the reference's
 * one kernel is when its shards are fp8 (kraken/fused/all_gather_matmul.py:25-123 with
 * dtype = tl.float8e4nv, :53, :121, launched by _matmul_w_progress :147-219).
 *   A, A_local: fp8, row strides lda, lda_local in bytes (multiples of 16); Bt, out, out_kind as for kr_gemm_fp8.
 * M % 256 == 0, N % 256 == 0, K % 128 == 0, M % (W * splits_per_rank) == 0, 0 <= rank < W.
 */
int kr_all_gather_matmul_fp8(const void* A, int64_t lda, const void* A_local, int64_t lda_local, const void* Bt,
                             int64_t ldb, int64_t M, int64_t N, int64_t K, int W, int rank, int splits_per_rank,
                             const uint32_t* progress, int64_t wait_limit_us, int32_t* status, void* out, int out_kind,
                             void* stream);

/*
 * Which kernel kr_gemm_reduce_*_bf16 would run for a shape (contiguous operands), decided by the
 * same code that launches it; for benchmarks and logs that want to name the kernel they timed.
 * No counterpart in the reference (its tile sizes are keyword arguments of the wrappers,
 * kraken/fused/gemm_one_shot_all_reduce_fused.py:128-133).  Nothing is launched.
 *   b_transposed: B is given transposed-contiguous ([N, K] memory); 0: row-major [K, N]
 *   workspace_bytes: size of the workspace the call would be given (0: none)
 *   plan[0] workgroup tile: 256 (256x256 tile, global->LDS loads without registers) or 128
 *   plan[1] matrix-core block of the k loop: 16 (v_mfma_f32_16x16x32_bf16) or 32 (32x32x16)
 *   plan[2] 128 tile: workgroups per tile that share its K loop (1: one pass)
 *   plan[3] 256 tile: tiles of the last partial round that are split, plan[4] parts of each
 *   plan[5] column panels per scheduling group
 *   plan[6] 1: tiles that lie wholly in the reduce band add the peers on the matrix cores
 *   plan[7] bit 0: M or N is not a multiple of the tile (bounds-checked edge tiles); bit 1: the
 *           tile is 256 x 224 (a plain product with transposed-contiguous B that fills whole rounds
 *           of the compute units with 224-column tiles and not with 256-column ones)
 */
int kr_gemm_plan(int64_t M, int64_t N, int64_t K, int b_transposed, int n_peers, int64_t band_rows,
                 int has_bias, int has_c_full, int64_t workspace_bytes, int32_t plan[8]);

/*
 * Measurement aids, without a counterpart in the reference: the plainest kernels that move a
 * given number of bytes, so that a benchmark can state what a launch of that size costs on this
 * machine before any arithmetic is added.
 *   kr_probe_read: every byte of [src, src + bytes) is loaded once (128-bit non-temporal loads,
 *     one per thread up to 16 MiB, 256-thread workgroups); nothing is written.  `sink` may be
 *     NULL (it only keeps the loads alive for the compiler).
 *   kr_probe_copy: the same loads, each followed by a 128-bit non-temporal store to dst.
 * bytes % 16 == 0; src, dst 16-byte aligned; bytes == 0: nothing is launched.
 */
int kr_probe_read(const void* src, int64_t bytes, void* sink, void* stream);
int kr_probe_copy(const void* src, void* dst, int64_t bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* KRAKEN_AMD_H */
