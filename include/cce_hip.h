/*
 * C ABI of libcce_hip.so: Cut Cross-Entropy kernels for AMD gfx950 (MI355X).
 *
 * Every entry point is stream-ordered (work is enqueued on `stream`, a
 * hipStream_t passed as void*), takes plain device pointers and sizes, never
 * allocates device memory, never synchronises, and returns 0 on success or a
 * non-zero status (a hipError_t value, or one of the CCE_ERR_* codes below).
 * All scratch memory comes in through the `workspace` argument, sized by the
 * matching *_workspace_bytes() query, so that a caller's allocator sees every
 * byte the loss path uses.
 *
 * Each function names the reference interface it replaces
 * (paths relative to the apple/ml-cross-entropy checkout).
 *
 * Common conventions
 *   e        [n_rows, d]  row-major, row stride `stride_e` elements, unit column stride
 *   c        [v, d]       row stride `stride_cv`, column stride `stride_cd` (elements)
 *   valids   [b] int32    rows of `e` that take part (NULL: rows 0..b-1, b == n_rows)
 *   targets  [n_rows] int64, read at (row + shift); a target t enters as
 *            t - target_offset and matches no column when outside [0, v)
 *   dtype    element type of e, c, bias: CCE_DTYPE_BF16 or CCE_DTYPE_F16
 *   softcap  <= 0 (or NaN) switches soft-capping off
 */
#ifndef CCE_HIP_H
#define CCE_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CCE_OK 0
#define CCE_ERR_INVALID_ARGUMENT 10001
#define CCE_ERR_UNSUPPORTED_DTYPE 10002
#define CCE_ERR_WORKSPACE_TOO_SMALL 10003
#define CCE_ERR_MISALIGNED 10004
#define CCE_ERR_STATIC_SCRATCH_LIMIT 10005

#define CCE_DTYPE_BF16 0
#define CCE_DTYPE_F16 1

/* Granularity of the forward tile statistic (rows x vocabulary entries per cell). */
#define CCE_STAT_ROWS 32
#define CCE_STAT_COLS 32

/* Number of uint64 slots in the backward counter block, counted in sub-tiles of 32 rows x 32
 * classes (the granularity of the gradient filter):
 * [0] sub-tiles in the plane, [1] sub-tiles whose logits the dE pass recomputed,
 * [2] sub-tiles that entered the dE product, [3] sub-tiles that entered the dC product. */
#define CCE_NUM_COUNTERS 4

/* Library ABI version (bumped when a signature below changes). */
int cce_version(void);

/* First 16 hex digits of the SHA-256 over the library's sources as they were when it was built (the order of
 * csrc/Makefile: SRCS, then HDRS); lets a binding refuse a library that is older than the sources beside it. */
const char* cce_source_hash(void);

/* Human-readable text for a status returned by any function below. */
const char* cce_error_string(int status);

/* Number of floats in the forward tile statistic for b valid rows and v classes:
 * ceil(b / CCE_STAT_ROWS) * ceil(v / CCE_STAT_COLS). */
int64_t cce_tile_stat_elems(int64_t b, int64_t v);

/* Scratch bytes cce_lse_forward needs (split-vocabulary partial max / sum-exp). */
int64_t cce_lse_forward_workspace_bytes(int64_t b, int64_t v, int64_t d);

/*
 * lse[i] = log sum_v exp(softcap(e[valids[i]] . c[v] + bias[v])),  i in [0, b).
 * Replaces cce_lse_forward_kernel (cut_cross_entropy/cce_lse_forward.py:170-237)
 * and its Triton body (:12-117).
 *   lse        [b] float, written (not accumulated)
 *   logit_avg  NULL, or [v] float: receives (1/b) sum_i logit[i, v]  (reference :95-97)
 *   tile_max   NULL, or [cce_tile_stat_elems(b, v)] float: max soft-capped logit of
 *              every CCE_STAT_ROWS x CCE_STAT_COLS cell (row-major over cells); lets
 *              cce_backward prove a tile filtered without recomputing it
 */
int cce_lse_forward(const void* e, const void* c, const void* bias, const int32_t* valids,
                    float* lse, float* logit_avg, float* tile_max,
                    void* workspace, int64_t workspace_bytes,
                    int64_t n_rows, int64_t b, int64_t v, int64_t d,
                    int64_t stride_e, int64_t stride_cv, int64_t stride_cd,
                    float softcap, int dtype, void* stream);

/* Size of the per-GPU static scratch array behind cce_lse_forward_static. */
#define CCE_STATIC_SCRATCH_BYTES (8 * 1024 * 1024)

/*
 * cce_lse_forward without a workspace argument, for callers that cannot allocate device memory (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference, whose launcher allocates its outputs and locks with torch on every
 * call (cut_cross_entropy/cce_lse_forward.py:193-204).  Same arguments, results and kernels as
 * cce_lse_forward; the split-vocabulary partials go to a static device array of
 * CCE_STATIC_SCRATCH_BYTES that each GPU the library runs on holds until the process ends.  The call
 * allocates and frees nothing.  Shapes whose cce_lse_forward_workspace_bytes() exceeds the array
 * return CCE_ERR_STATIC_SCRATCH_LIMIT (c2 needs 0.5 MB, E [65536, 3584] x C [152064, 3584] 2 MB).
 * All calls on one GPU share the array: calls that overlap in time on one GPU race; calls on one
 * stream, or otherwise ordered, are safe (a launch writes every partial before reading it, so nothing
 * carries over from the previous call).  With logit_avg the call also launches a small fill kernel for it and the
 * forward adds to it with float atomics, as cce_lse_forward does.
 */
int cce_lse_forward_static(const void* e, const void* c, const void* bias, const int32_t* valids,
                           float* lse, float* logit_avg, float* tile_max,
                           int64_t n_rows, int64_t b, int64_t v, int64_t d,
                           int64_t stride_e, int64_t stride_cv, int64_t stride_cd,
                           float softcap, int dtype, void* stream);

/*
 * Set-up of cce_lse_forward_static for the CURRENT device: looks up the address of that device's copy of the
 * static array (hipGetSymbolAddress, which may load the code object) and keeps it.  cce_lse_forward_static does
 * the same by itself on its first call on a device; a caller whose first call would fall inside a HIP graph
 * capture, where nothing may be loaded, calls this once per device beforehand.  Both look the array up for the
 * device that is current in the calling thread: the caller makes the device of `stream` current first.
 * No counterpart in the reference (see cce_lse_forward_static).
 */
int cce_lse_forward_static_init(void);

/*
 * out[i] = softcap(-(e[valids[i]] . c[t_i]) - bias[t_i]),  t_i = targets[valids[i] + shift] - target_offset;
 * out[i] = 0 when t_i is outside [0, v).
 * Replaces indexed_neg_dot_forward_kernel (cut_cross_entropy/indexed_dot.py:101-158,
 * Triton body :11-85) including the soft-capping the reference applies on the host (:150-151).
 */
int cce_indexed_neg_dot(const void* e, const void* c, const int64_t* targets, const void* bias,
                        const int32_t* valids, float* out,
                        int64_t n_rows, int64_t b, int64_t v, int64_t d,
                        int64_t stride_e, int64_t stride_cv, int64_t stride_cd,
                        int64_t shift, int64_t target_offset,
                        float softcap, int dtype, void* stream);

/* Scratch bytes cce_backward needs: one survivor bit per 32 x 32 sub-tile, each 32-row group's bits
 * padded to whole 32-bit words, then a count and one int32 per 32-class group (the class groups its second,
 * full dC pass takes over from the light one). */
int64_t cce_backward_workspace_bytes(int64_t b, int64_t v, int64_t d);

/*
 * Gradients of  sum_i d_out_i * nll_i + d_lse_i * lse_i  w.r.t. e, c and bias.
 * Replaces cce_backward_kernel (cut_cross_entropy/cce_backward.py:346-521, Triton
 * body :20-310).  Per valid row i and class v, with z the raw logit, s = softcap(z),
 * p = exp(s - lse_i), y = [v == t_i], g = grad_scale * d_out_i, h = d_lse_i:
 *     dz = (p (g + h) - y g) (1 - (s / softcap)^2)
 *     d_e[row_i] += sum_v dz c[v];  d_c[v] += sum_i dz e[row_i];  d_bias[v] += sum_i dz.
 * A tile of the (row, class) plane whose every |p - y| is below filter_eps is dropped
 * from d_e when filter_e, and from d_c and d_bias when filter_c (gradient filtering,
 * reference :211-216; the reference drops a tile from d_bias only when both flags are set, the
 * difference lies within what filtering is allowed to drop).  filter_eps < 0 switches filtering off.
 *
 *   lse        [b] float      (the global LSE when c is a vocabulary shard)
 *   d_out      [n_rows] float read at (row + shift), or one float when d_out_is_scalar
 *   d_lse      NULL or [n_rows] float read at (row + shift)
 *   vocab_order NULL or [v] int32 permutation of the classes; tiles are formed over the
 *              permuted order (reference :153-155).  Disables the tile_max shortcut.
 *   tile_max   NULL or the statistic written by cce_lse_forward for the same inputs
 *   d_e        NULL or [n_rows, d] accumulated into (caller zero-fills); float when
 *              d_e_is_fp32 else `dtype`; same strides as e
 *   d_c        NULL or [v, d], written: every element when b > 0 (zeros where no tile survived), nothing
 *              when b == 0; need not be initialised; float when d_c_is_fp32 else `dtype`; same strides as c
 *   d_bias     NULL or [v] float, accumulated into
 *   counters   NULL or CCE_NUM_COUNTERS uint64, accumulated into
 */
int cce_backward(const void* e, const void* c, const void* bias,
                 const float* lse, const float* d_out, int d_out_is_scalar, const float* d_lse,
                 const int32_t* valids, const int32_t* vocab_order, const int64_t* targets,
                 const float* tile_max,
                 void* d_e, void* d_c, float* d_bias,
                 void* workspace, int64_t workspace_bytes, uint64_t* counters,
                 int64_t n_rows, int64_t b, int64_t v, int64_t d,
                 int64_t stride_e, int64_t stride_cv, int64_t stride_cd,
                 float grad_scale, float filter_eps, int filter_e, int filter_c,
                 int d_e_is_fp32, int d_c_is_fp32,
                 int64_t shift, int64_t target_offset,
                 float softcap, int dtype, void* stream);

/*
 * count += number of cells of the forward statistic (CCE_STAT_ROWS x CCE_STAT_COLS) whose bound
 * exp(tile_max - min lse of the cell's rows) reaches filter_eps, i.e. the cells cce_backward has to recompute.
 * The fraction count / cce_tile_stat_elems(b, v) tells a caller whether filtering can pay at all (near-uniform
 * soft-max distributions flag almost every cell; the unfiltered cce_backward_dense is then faster and exact).
 * The reference has no counterpart: its kernel meets every tile anyway (cut_cross_entropy/cce_backward.py:170-216).
 *   tile_max, lse  as written by cce_lse_forward for the same b, v;   count  one uint64, accumulated into
 */
int cce_count_flagged_cells(const float* tile_max, const float* lse, int64_t b, int64_t v, float filter_eps,
                            uint64_t* count, void* stream);

/* The logit gradient of one vocabulary chunk, written out, for the unfiltered backward.
 *
 * Restates the first half of the Triton backward body (cut_cross_entropy/cce_backward.py:
 * logit recompute :170-188, softmax minus one-hot :196-207, d_out / d_lse scaling :238-248,
 * soft-cap gradient :251, rounding to the input type :256) with the gradient filter off.  What the
 * reference does next inside the same kernel -- the two products d_e += dz . c (:262-275) and
 * d_c += dz^T . e (:289-302), through atomics -- is not done here: with every dz in play they are dense
 * matrix products (d_e[rows] += dz . c, d_c = dz^T . e[rows], d_bias = column sums of dz) on the [b, v] matrix
 * this function fills, chunk of the vocabulary by chunk.  cce_backward_dense runs dz and products in one call,
 * cce_backward_products the products alone.
 *
 *   c, bias    the chunk's rows: v classes starting at the caller's offset
 *   lse        [b] float, the LSE over the WHOLE vocabulary
 *   dz         [b, ldz] in `dtype`, or float when dz_is_fp32 (for callers that pass fp32 matrices split
 *              into 16-bit parts along d and want the gradient at that accuracy); row i = valid row i
 *              (rows compacted through valids), ldz >= v
 *   target_offset  first class of the chunk (plus the shard start, if any)
 * Needs 16-byte aligned e, c, dz, unit stride_cd, row strides that are multiples of 8, ldz a multiple of 8
 * (4 when dz_is_fp32) and d a
 * multiple of 64; anything else returns CCE_ERR_MISALIGNED and the caller uses cce_backward.
 */
int cce_backward_dz(const void* e, const void* c, const void* bias,
                    const float* lse, const float* d_out, int d_out_is_scalar, const float* d_lse,
                    const int32_t* valids, const int64_t* targets,
                    void* dz, int64_t ldz, int dz_is_fp32,
                    int64_t n_rows, int64_t b, int64_t v, int64_t d,
                    int64_t stride_e, int64_t stride_cv, int64_t stride_cd,
                    float grad_scale, int64_t shift, int64_t target_offset,
                    float softcap, int dtype, void* stream);

/* Workspace bytes of cce_backward_dense for a dz buffer of at most `max_dz_bytes` (the function rounds it down to
 * whole 256-class tiles of b rows, at most 16384 classes -- or, where it walks by rows, to whole 256-row blocks of all
 * classes -- and never goes below one tile), plus the 16-bit compensation term of the gradient it carries from
 * launch to launch when `d_e_in_workspace` (d_e wanted in the 16-bit input type): [b, d] for dE, or [v, d] for dC
 * where b >= 2 v and the walk goes by blocks of rows (see cce_backward_dense).
 * cce_backward_dense_fixed_bytes is the second part alone; cce_backward_dense_dz_bytes the size of a dz buffer of
 * `units` classes per chunk (rows per block where the walk goes by rows), for a caller that sizes the workspace
 * against a limit of its own. */
int64_t cce_backward_dense_workspace_bytes(int64_t b, int64_t v, int64_t d, int d_e_in_workspace,
                                           int64_t max_dz_bytes);
int64_t cce_backward_dense_fixed_bytes(int64_t b, int64_t v, int64_t d, int d_e_in_workspace);
int64_t cce_backward_dense_dz_bytes(int64_t b, int64_t v, int64_t d, int d_e_in_workspace, int64_t units);

/*
 * The whole unfiltered backward in one call: d_e, d_c, d_bias of cce_backward with the gradient filter
 * off (filter_eps = None in cut_cross_entropy/cce_backward.py:346-521, i.e. the cce_exact / cce_kahan_full*
 * presets).  Replaces the same Triton body (:20-310), both halves: the logit recompute and dz (:170-256) and
 * the two products d_e += dz . c (:262-275), d_c += dz^T . e (:289-302), which the reference accumulates with
 * atomics.  Here the vocabulary is walked in chunks; per chunk the dz of the chunk is written to the
 * workspace in the input type, d_c[chunk] = dz^T . e and d_bias[chunk] = column sums of dz are complete and
 * written once, and d_e accumulates over the chunks: in fp32 when d_e is float, else as a pair of 16-bit
 * numbers, d_e itself and a compensation term in the workspace (the "Kahan" buffers of the reference's
 * cce_kahan* presets, :374-385: 16 bits of mantissa carried from chunk to chunk, d_e final after the last).
 *
 *   d_e      NULL or [n_rows, d]: float when d_e_is_fp32 (accumulated into: the caller zero-fills), else `dtype`
 *            (the rows of valid tokens are written, whatever they held); rows that are not valid tokens are
 *            not touched in either case
 *   d_c      NULL or [v, d] with the strides of c; float when d_c_is_fp32 else `dtype`; written, not accumulated
 *   d_bias   NULL or [v] float, accumulated into.  The column sums run over dz as rounded to `dtype` (what the
 *            products multiply); cce_backward and the reference (:253-256) sum dz before that rounding, so the
 *            two differ by the rounding of each term (2^-9 relative for bf16, unbiased)
 *   workspace  256-byte aligned; at least cce_backward_dense_workspace_bytes(b, v, d, d_e in `dtype`, 0) bytes.
 *            Anything beyond that enlarges the chunks (fewer, better filled launches) up to 16384 classes.
 * With a 16-bit d_e and b >= 2 v (rounded up to 256: a vocabulary shard) the walk goes over blocks of ROWS with the
 * whole vocabulary each instead: d_e of a block is complete after its launch and written once, and it is d_c that
 * is carried from block to block (a 16-bit d_c as a pair with a [v, d] compensation term in the workspace, an fp32
 * d_c in place).  The same number of launches for the same dz buffer, with the smaller matrix as the one that is
 * read and written once per launch.
 * Layout requirements as for cce_backward_dz (16-byte aligned e, c and d_e, unit stride_cd, row strides that
 * are multiples of 8, d a multiple of 64), else CCE_ERR_MISALIGNED and the caller uses cce_backward.
 */
int cce_backward_dense(const void* e, const void* c, const void* bias,
                       const float* lse, const float* d_out, int d_out_is_scalar, const float* d_lse,
                       const int32_t* valids, const int64_t* targets,
                       void* d_e, void* d_c, float* d_bias,
                       void* workspace, int64_t workspace_bytes,
                       int64_t n_rows, int64_t b, int64_t v, int64_t d,
                       int64_t stride_e, int64_t stride_cv, int64_t stride_cd,
                       float grad_scale, int d_e_is_fp32, int d_c_is_fp32,
                       int64_t shift, int64_t target_offset,
                       float softcap, int dtype, void* stream);

/*
 * The two matrix products of one vocabulary chunk on their own, for a caller that forms dz itself and wants
 * fp32 results: the fp32 path of the Python host splits dz, c and e into 16-bit parts and sums the cross terms
 * with one call per term.  The products of the reference's kernel (cut_cross_entropy/cce_backward.py:262-275
 * and :289-302) as 16-bit-in, fp32-accumulate matrix products on the tiles cce_backward_dense runs, both in one
 * launch:
 *     d_e[i, :] += sum_v dz[i, v] c[v, :]                    i < b   (d_e: a [b, d] float accumulator, row stride ld_de)
 *     d_c[v, :] (+)= sum_i dz[i, v] e[valids[i], :]          v < n_cls  (float, row stride ld_dc; added to when
 *                                                            d_c_accumulate, else written)
 *   dz   [b, ldz] in `dtype`; ldz >= n_cls rounded up to 64, and the columns up to there must hold finite values
 *   c    [n_cls, d] row stride stride_cv (NULL when d_e is NULL);  e  [*, d] row stride stride_e (NULL when d_c is NULL)
 * Pointers 16-byte aligned, ldz / stride_cv / stride_e multiples of 8, d a multiple of 8, ld_de / ld_dc multiples
 * of 4; else CCE_ERR_MISALIGNED.
 */
int cce_backward_products(const void* dz, int64_t ldz, const void* c, int64_t stride_cv,
                          const void* e, int64_t stride_e, const int32_t* valids,
                          float* d_e, int64_t ld_de, float* d_c, int64_t ld_dc, int d_c_accumulate,
                          int64_t b, int64_t n_cls, int64_t d, int dtype, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* CCE_HIP_H */
