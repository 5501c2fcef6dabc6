/*
 * nengo_hip.h -- C ABI of the MI355X (gfx950) timestep kernels.
 *
 * One simulator timestep of a Nengo model is a fixed sequence of "plans"
 * (ragged gather-GEMV, neuron update, synapse filter, copies, probes ...).
 * In the reference every plan is an OpenCL kernel generated from a Mako
 * template and bound with `kernel.set_args(...)` inside a `plan_*` function;
 * the entry points below are what those `plan_*` functions bind instead.
 *
 * Conventions (all entry points):
 *   - `stream` is a `hipStream_t` passed as `void*` (NULL = default stream).
 *   - every `*_data` / `X` / `Y` pointer is a DEVICE pointer to a flat float32
 *     (or int32 where stated) buffer; all offsets inside the int32 work lists
 *     are ELEMENT offsets into those buffers, exactly like the `*_starts`
 *     arrays the reference kernels receive (nengo_ocl/raggedarray.py:31-236,
 *     nengo_ocl/clraggedarray.py:65-184).
 *   - work lists (`items`, `dots`, `tasks`, `blocks`, `desc`) are DEVICE int32
 *     tables built once at plan time and owned by the caller; the library
 *     only reads them during the launch.  Float scalars ride in them as raw
 *     IEEE-754 bits.
 *   - nothing here allocates, frees or synchronises (except where stated):
 *     kernels are enqueued on `stream` and the call returns.
 *   - return value: 0 on success, otherwise a `hipError_t` (or a negative
 *     NHIP_E_* code for argument errors); `nhip_error_string` describes both.
 *     No entry point throws or aborts.
 *   - one stream per simulator; entry points are re-entrant but the caller
 *     serialises work that touches the same buffers.
 */
#ifndef NENGO_HIP_H
#define NENGO_HIP_H

#ifdef __cplusplus
extern "C" {
#endif

#define NHIP_ABI_VERSION 1

#define NHIP_E_BADARG (-1)   /* null pointer / negative count / unknown mode   */
#define NHIP_E_BADCLASS (-2) /* GEMV class (lanes-per-row, vector width) unknown */
#define NHIP_E_RTC (-3)      /* run-time compilation failed (see the log)          */
#define NHIP_E_TOOBIG (-4)   /* the request does not fit the workspace it was given */

/* ---- library ---------------------------------------------------------- */
int nhip_abi_version(void);
const char *nhip_error_string(int err);
/* device facts of the current device: compute units, wavefront size, LDS bytes
 * per work-group, gcn arch name (copied, NUL-terminated, into `name`). */
int nhip_device_info(int *n_cu, int *wave_size, int *lds_bytes, char *name, int name_len);

/* ---- ragged gather-GEMV ------------------------------------------------
 * For every output item b:
 *     Y[b] = beta_b * Yin[b] + gamma_b + alpha_b * sum_d  A[b,d] @ X[b,d]
 * replaces: clra_gemv.py `plan_block_gemv` / `block_impl` (:861-1175, kernels
 * `fn` :1010-1060 and `reduce` :1122-1155), and the `ref_impl` /
 * `reduce_impl` / `many_dots_impl` family (:264-858).  One launch computes
 * the final Y directly (no partial-sum buffer, no second kernel).
 *
 *   items : int32[n_items][8]  {y_start, y_stride0, yin_start, yin_stride0,
 *                               dot_begin, n_dots, M, 0}
 *   coefs : float[n_items][4]  {alpha, beta, gamma, 0}
 *   dots  : int32[n_dots][8]   {a_start, a_stride0, N, x_start, x_stride0,
 *                               tile_rows, log2_N, stage}
 *                               (A rows are contiguous: a_stride1 == 1; the last
 *                               three are read by nhip_gemv_tile only (stage: with
 *                               pow2_cols >= 2, see there): tile_rows =
 *                               nhip_gemv_tile_rows(N, blk_words), log2_N = the
 *                               exponent when N is a power of two, else -1)
 *   tasks : int32[n_tasks][4]  {item, row0, n_rows, 0}
 *
 * `flavor` 0 = one work-group (256 threads) per task, X staged in LDS and
 * shared by the group's four waves; rows per task <= nhip_gemv_rows_per_task.
 * `flavor` 1 = one wave per task (four tasks per group), X read through L1;
 * for many tiny items.  `flavor` 2 = the summation order of the reference's block
 * kernel (four strided partial sums per 128-column tile, tiles added in order) for
 * small items: every task is ONE row (n_rows == 1), a wave takes 64 / lpr consecutive
 * tasks of whatever items; lpr 4 (any widths) or 1 (every dot product of the launch
 * has at most 4 columns), vec 1: bit-identical to a float32
 * restatement of that kernel.  With lpr 64 (and 16-word task records) the launch is the
 * lpr 1 one with tasks of up to 64 consecutive rows of one item (n_rows <= 64) that a wave
 * takes whole, lane l the row row0 + l: the records are then read once per wave instead
 * of once per row, and the parts of an input sum are fetched by the lanes side by side.  `lpr` = lanes cooperating on one row (1,2,...,64, or
 * 256 for flavor 0); `vec` = 4 (16-byte loads; needs a_start % 4 == 0 and
 * a_stride0 % 4 == 0 for every dot of the launch) or 1.  `passes` (flavor 0) =
 * rows each lane accumulates at once, i.e. independent loads in flight: 2, 4, 8,
 * or 0 for the class default; (flavor 2) = 16 when the task records are the 16-word
 * ones described with nhip_gemv_rows_lif, else 0.  The host validates these
 * preconditions; the kernel trusts them. */
int nhip_gemv(void *stream, int flavor, int lpr, int vec, int passes, const int *items,
              const float *coefs, const int *dots, const int *tasks, int n_tasks,
              const float *A, const float *X, const float *Yin, float *Y);
/* rows one task of the given class covers at most (0 if the class is unknown) */
int nhip_gemv_rows_per_task(int flavor, int lpr, int vec, int passes);

/* The same operation in the reference's summation order for coefficients that the
 * reference writes into its kernel text as double-precision literals (alpha, beta or
 * gamma the same for every item: clra_gemv.py:20-34, used at :1058, :1148, :1153):
 * alpha * (tile sum), beta * y_in and sum + gamma are formed in double and rounded to
 * float32 once each.  Identical to nhip_gemv (flavor 2) whenever float32 holds the
 * coefficients exactly; the host takes this entry point when it does not.
 *   dcoefs : double[n_items][4] {alpha, beta, gamma, 0}
 *   tasks  : int32[n_tasks][4] {item, row, 1, 0} -- one output row per task
 * `items` and `dots` as for nhip_gemv. */
int nhip_gemv_rows_literal(void *stream, const int *items, const double *dcoefs, const int *dots,
                           const int *tasks, int n_tasks, const float *A, const float *X,
                           const float *Yin, float *Y);

/* The same operation and the same four tables, summed in the ORDER of the
 * reference's block kernel (clra_gemv.py:1043-1058, :1148-1153: four strided
 * partial sums per 128-column tile, one fused multiply-add per element,
 * (s0+s2)+(s1+s3), tiles added in order), for large items: a wave owns the rows
 * of one task (four tasks per 256-thread group, at most 256 rows per task) and
 * streams the matrix through a wave-private LDS block of `blk_words` float32 (a
 * multiple of 4, >= 528; 2176 = 8.5 KiB by default), so the result is
 * bit-identical to a float32 restatement of that kernel while HBM is still read in
 * whole lines.  nhip_gemv_tile_rows(N, blk_words) = rows of a dot product with N
 * columns that fit one LDS block (a power of two; goes into the dots table).
 * The task table of these entry points is wider than nhip_gemv's, so that a wave
 * starts streaming after one read:
 *   tasks : int32[n_tasks][24] {item, row0, n_rows, 0,  the item's row of `items` (8),
 *                               alpha, beta, gamma (float bits), 0,
 *                               the item's first row of `dots` (8; zeros without dots)}
 * `vec` as for nhip_gemv.  `pow2_cols` selects the kernel: 0 = any shape; 1 = every
 * dot product of the launch has a power-of-two column count >= 4 (log2_N set),
 * vec == 4 and a_stride0 < 2^22; 2 = every dot product has 5 columns or more (a
 * row whose length is no multiple of 4 followed by readable memory up to the next
 * one), vec == 4, a_stride0 < 2^22 and blk_words == 2176: the kernel whose
 * stage shapes are compile-time constants (fewest instructions per byte); the last
 * word of a dots row then says which: 3 (N <= 8: stages of 8 columns, blocks of 128
 * rows), 4 (N <= 16: 16 columns, 64 rows), 5 (N <= 32: 32 columns, 32 rows), 6 (N <=
 * 64: 64 columns, 32 rows), 7 (N < 512: 128 columns, 16 rows) or
 * 9 (512 columns, 4 rows); tasks should be whole blocks.  The kernel comes in five
 * instances, by the stages the launch may hold (each stage a launch does not need
 * costs the others registers): 3 = stages 5 and 6 only, and no task of more than 128
 * rows (a smaller LDS footprint and fewer registers: four waves per SIMD); 5 = the
 * same with stages 3 and 4 too; 2 = stages 5, 6, 9; 4 = stages 5, 6, 7, 9; 6 = any;
 * 7 = stages 3 to 6 for matrices whose rows lie back to back (a_stride0 == N <= 64, any
 * value: rows need not be 16-byte aligned) from a_start % 4 == 0, with every task
 * starting at a row that is a multiple of 4 and 12 readable bytes behind each matrix: a
 * row block is then one aligned run of memory and is read in 16-byte quads. */
int nhip_gemv_tile(void *stream, int vec, int pow2_cols, int blk_words, const int *items,
                   const float *coefs, const int *dots, const int *tasks, int n_tasks,
                   const float *A, const float *X, const float *Yin, float *Y);
int nhip_gemv_tile_rows(int n_cols, int blk_words);
/* nhip_gemv_tile followed by nhip_lif on its outputs, in one launch: replaces
 * `plan_block_gemv` (clra_gemv.py:1193-1195) + `plan_lif`
 * (clra_nonlinearities.py:1028-1146) when the GEMV output is the neurons' input
 * current.  Row r of item b is the current of neuron r of population b:
 *   pops : int32[n_items][8] {v_start, w_start, s_start, decay, tau, ref, amp, pflags}
 * (tau / ref / amp: float bits, or with bit 0/1/2 of pflags set the element offset
 * of a per-neuron vector in TAU / REF / AMP; bit 8 of pflags: the item has a
 * population -- items without it only get Y; bit 9: `decay` holds the float bits of
 * -expm1(-dt / tau) formed as the kernel would (float quotient, expm1 in double,
 * rounded once to float), allowed when tau is a scalar and upsample == 1: the
 * launch then evaluates transcendental functions only for the few neurons that
 * leave their refractory period or spike in this step; bit 11, with bit 9, scalar amp,
 * s_start even and every task of the item starting at a multiple of 32 rows: the launch
 * leaves the spikes as one BIT per neuron -- bit r % 64 of the 64-bit word r / 64 at
 * S + s_start, set where neuron r spiked -- and writes no float of S for the item; for
 * spikes that only nhip_gemv_events reads, see its `x_bits`).
 * Y is still written.  V, W, S must not overlap anything the launch reads through
 * A, X or Yin; dt, upsample as for nhip_lif.  Results are bit-identical to the two
 * separate calls. */
int nhip_gemv_tile_lif(void *stream, int vec, int pow2_cols, int blk_words, const int *items,
                       const float *coefs, const int *dots, const int *tasks, int n_tasks,
                       const float *A, const float *X, const float *Yin, float *Y,
                       const int *pops, double dt, int upsample, float *V, float *W, float *S,
                       const float *TAU, const float *REF, const float *AMP);
/* The same launch when the vector operand of an item's first dot product is itself a sum
 * of vectors that a small-item GEMV launch would form just before (the decoded inputs of
 * an ensemble added up: `_plan_MultiDotInc` on the `in` signal, simulator.py:746-816,
 * followed by the encoders' GEMV and `plan_lif`): the launch forms the sum itself,
 *   x[c] = (...(0 + v_0[c] * s_0) + v_1[c] * s_1) + ...,   every product rounded on its own,
 * which is what that GEMV gives for Y = 0 * Y + sum_k v_k * s_k (one-column dot products,
 * alpha = 1, beta = 0, gamma = 0) as long as the old Y is finite, and stores it where that
 * launch would have: at the operand's own place (x_start of the dot product, stride 1).
 *   parts : int32[n][2] {start of vector v_k, start of scalar s_k}, offsets into X
 * An item with such an operand names its parts in the spare words of its task records:
 * task.pad = first part, item.pad = number of parts (0: the operand is read as usual);
 * its first dot product must have at most 64 columns.  X and Y must be the same buffer,
 * the launch one of the compile-time-shape kernel (pow2_cols >= 2), and no part may
 * overlap an operand that the launch writes.  Results are bit-identical to the separate
 * launches. */
int nhip_gemv_tile_lif_sums(void *stream, int vec, int pow2_cols, int blk_words,
                            const int *items, const float *coefs, const int *dots,
                            const int *tasks, int n_tasks, const float *A, const float *X,
                            const float *Yin, float *Y, const int *pops, double dt,
                            int upsample, float *V, float *W, float *S, const float *TAU,
                            const float *REF, const float *AMP, const int *parts);

/* nhip_gemv_tile followed by the step of first-order filters on its outputs, in one
 * launch: replaces `plan_block_gemv` (clra_gemv.py:1193-1195) + the simple case of
 * `plan_linearfilter` (clra_nonlinearities.py:577-803, one numerator and at most one
 * denominator coefficient: a decoded value and the synapses of the connections
 * that carry it).  Row r of item b is the new input of element r of each of the
 * item's filters:
 *   item_targets : int32[n_items][2] {first target, number of targets}
 *   targets      : int32[n][4] {y_start, a0 bits, b0 bits, na}
 *   F[y_start + r] = b0 * y - a0 * F[y_start + r]   (na == 1)   or   b0 * y   (na == 0)
 * Y is still written.  The filter outputs must not overlap anything the launch reads
 * through A, X or Yin.  Results are bit-identical to the two separate calls.
 * The kernels of this entry point read an item's range of targets from its task
 * records, so that a wave needs no further read before it can start: tasks[t][3] =
 * first target and tasks[t][11] = number of targets of the task's item, i.e. the
 * item's row of `item_targets` (which nhip_gemv_rows_filter reads). */
int nhip_gemv_tile_filter(void *stream, int vec, int pow2_cols, int blk_words, const int *items,
                          const float *coefs, const int *dots, const int *tasks, int n_tasks,
                          const float *A, const float *X, const float *Yin, float *Y,
                          const int *item_targets, const int *targets, float *F);

/* A learning rule's outer-product update done by the launch that streams the learned
 * matrices anyway (reference: `_plan_SimPES`, simulator.py:1334-1345, an outer-product
 * `plan_elementwise_inc` of its own, clra_nonlinearities.py:414-574, and a `plan_copy` that
 * adds the result to the weights).  nhip_gemv_tile_filter with one more table:
 *   learn : int32[n_tasks][4] {e_start, f_start, alpha (float bits), flags}, one row per
 *           TASK.  flags bit 0: the task's matrix (its item's only dot product, rows on
 *           16-byte boundaries, a multiple of 4 columns, at most 64 rows in the task) is
 *           learned: after a block of it has gone into the sums as it was read, element
 *           (i, j) is written back as A[i][j] + (alpha * X[e_start + i]) * X[f_start + j],
 *           every product and the sum rounded on their own -- the bits of the separate
 *           launches.  Nothing in the launch may write X[e_start ..] or X[f_start ..];
 *           f_start must be a multiple of 4.
 * Only for pow2_cols = 2 (else NHIP_E_BADCLASS).  A is written: it is not const here. */
int nhip_gemv_tile_filter_learn(void *stream, int vec, int pow2_cols, int blk_words,
                                const int *items, const float *coefs, const int *dots,
                                const int *tasks, int n_tasks, float *A, const float *X,
                                const float *Yin, float *Y, const int *item_targets,
                                const int *targets, float *F, const int *learn);

/* nhip_gemv_tile_lif / nhip_gemv_tile_lif_sums (`parts` may be NULL: no input sums) that
 * also steps first-order filters of the populations' spikes -- the pre-synaptic activities
 * a learning rule reads (reference: the `plan_linearfilter` of the rule's pre-synaptic
 * synapse, clra_nonlinearities.py:577-803, a launch at the end of the step).  The step is
 * DEFERRED: the task that is about to replace the spikes of neurons [row0, row0 + n) with
 * this step's first computes, from the spikes of the previous step,
 *     Fdef[f_start + i] = b0 * S_old[i] - a0 * Fdef[f_start + i]     (or b0 * S_old[i])
 * so that between two steps Fdef holds the filter output as it was BEFORE the previous
 * step's update; whoever reads it from the host applies the pending step (the same two
 * rounded operations).  With zero initial spikes and outputs the first such step changes
 * nothing, as it must.
 *   deferred : int32[n_items][4] {f_start, a0 (float bits), b0 (float bits), flags}; flags
 *              bit 0: the item's population has such a filter, bit 1: it has a0.
 * Only for pow2_cols = 3 (else NHIP_E_BADCLASS). */
int nhip_gemv_tile_lif_deferred(void *stream, int vec, int pow2_cols, int blk_words,
                                const int *items, const float *coefs, const int *dots,
                                const int *tasks, int n_tasks, const float *A, const float *X,
                                const float *Yin, float *Y, const int *pops, double dt,
                                int upsample, float *V, float *W, float *S, const float *TAU,
                                const float *REF, const float *AMP, const int *parts,
                                const int *deferred, float *Fdef);

/* The same two epilogues for launches of small items (nhip_gemv with flavor 2, whose
 * `items`, `coefs`, `dots` and `tasks` tables these take; `lpr` 4, 1 or 64): the
 * neuron update / filter step of a row runs in the lane that holds the row's sum.
 * `pops`, `item_targets`, `targets` and the other arguments as above.
 * `task_words` = 4: tasks as for nhip_gemv.  = 16: every task record also holds its
 * item and coefficients (a launch of a few thousand rows is a chain of dependent
 * reads, and this takes one out of it; nhip_gemv takes such tables for flavor 2
 * with `passes` = 16):
 *   tasks : int32[n_tasks][16] {item, row0, 1 (lpr 64: n_rows), e0,  the item's row of `items` with its
 *                               last word = e1,  alpha, beta, gamma (float bits), e2}
 * e0, e1, e2 let the epilogue start its own reads at once: nhip_gemv_rows_lif
 * v_start, w_start, pflags of the item's row of `pops`; nhip_gemv_rows_filter first
 * target, number of targets, 0; nhip_gemv 0, 0, 0. */
int nhip_gemv_rows_lif(void *stream, int lpr, int task_words, const int *items, const float *coefs,
                       const int *dots, const int *tasks, int n_tasks, const float *A,
                       const float *X, const float *Yin, float *Y, const int *pops, double dt,
                       int upsample, float *V, float *W, float *S, const float *TAU,
                       const float *REF, const float *AMP);
/* nhip_gemv_rows_lif that forms input sums itself, as nhip_gemv_tile_lif_sums does for
 * large items (replaces the same three reference steps): the vector operand of an item's
 * first dot product -- every dot product of such an item has at most 4 columns -- or the
 * rows of an item without dot products, is x[c] = (...(0 + v_0[c] s_0) + v_1[c] s_1) + ...
 *   sum_ranges : int32[n_items][2] {first part, number of parts} (0 parts: none)
 *   parts      : int32[n][2] {start of vector v_k, start of scalar s_k}, offsets into X
 * The first row of an item stores the sum at the operand's place (x_start of the dot
 * product, stride 1); X and Y must be the same buffer; no part may overlap anything the
 * launch writes.  Bit-identical to the separate launches while the old sums are finite. */
int nhip_gemv_rows_lif_sums(void *stream, int lpr, int task_words, const int *items,
                            const float *coefs, const int *dots, const int *tasks, int n_tasks,
                            const float *A, const float *X, const float *Yin, float *Y,
                            const int *pops, double dt, int upsample, float *V, float *W,
                            float *S, const float *TAU, const float *REF, const float *AMP,
                            const int *sum_ranges, const int *parts);
int nhip_gemv_rows_filter(void *stream, int lpr, int task_words, const int *items,
                          const float *coefs, const int *dots, const int *tasks, int n_tasks,
                          const float *A,
                          const float *X, const float *Yin, float *Y, const int *item_targets,
                          const int *targets, float *F);

/* ---- sparse matrix-vector products -----------------------------------------
 * Y[b] (=|+=) A[b] @ X[b] for many sparse matrices in one launch.
 * replaces: `plan_sparse_dot_inc` / `spmv_csr_impl` / `spmv_ellpack_impl`
 * (clra_gemv.py:1494-1646, :1649-1755, :1919-1948), which run one launch per
 * matrix.  Layout: sliced ELLPACK with slices of 64 rows, four elements of a row per
 * 16 bytes: element k of row r of a slice is at data_start + 256 (k / 4) + 4 r + k % 4
 * in `cols` (column index) and `vals`; rows are padded to `width`, the slice's longest
 * row rounded up to a multiple of 4; row r of a slice has row_len[len_start + r]
 * elements.  `cols` and `vals` are 16-byte aligned and every data_start is a multiple
 * of 4 (NHIP_E_BADARG otherwise; the table is not read on the host, so a data_start
 * or width that is no multiple of 4 is the caller's error).
 *   slices : int32[n_slices][8] {data_start, width, len_start, n_rows (<= 64),
 *                                x_start, y_start (of the slice's first row), inc, window}
 * window >= 0 (a multiple of 4, with x_start a multiple of 4 and X 16-byte aligned): the
 * 1024 elements of the item's X from `window` on are copied to LDS first and read from
 * there (they must lie inside X); window < 0: none.  Results do not depend on it.
 * X and Y items are contiguous vectors.  Each row is summed in column order with one
 * fused multiply-add per element (starting from the old y when inc), like the
 * reference's CSR kernel. */
int nhip_spmv_sell(void *stream, const int *slices, int n_slices, const int *row_len,
                   const int *cols, const float *vals, const float *X, float *Y);

/* Y[b] = beta[b] Y_in[b] + alpha[b] A[b] X[b] + gamma[b] for items with one dot product,
 * whose X is mostly zero (decoders and weights applied to the spikes of a population): `plan_block_gemv` (clra_gemv.py:861-1175) restricted to such
 * items, visiting only the columns whose x is not zero -- in the reference's order, with its
 * operations, so the result is that of nhip_gemv_tile (a running sum that underflows to -0
 * aside) -- and reading only those columns of A.  For that the matrices are handed over
 * transposed, in a buffer of their own:
 *   items : int32[n_items][16] {at_start, mp, M, N, x_start, y_start, y_stride0, yin_start,
 *           yin_stride0, bits of alpha, beta, gamma, first_target, n_targets, row0, x_bits}
 *           a record stands for rows row0 .. row0 + M - 1 (M <= 64) of a matrix whose
 *           column c is AT[at_start + c * mp + row]; y_start / yin_start are those of the
 *           matrix's row 0; a matrix of more than 64 rows is several records; x_bits != 0:
 *           X + x_start (x_start even) holds one bit per column in 64-bit words, as
 *           nhip_gemv_tile_lif leaves them with bit 11 of pflags, and x_bits is the float
 *           bits of the value a set bit stands for (a clear bit: zero)
 *   AT    : the transposed matrices; X, Yin, Y: the buffers the offsets refer to
 *   targets, F : first-order filters stepped on the fresh y, as for nhip_gemv_tile_filter
 *           (both NULL: none); an item's range of targets is in its record
 * max_cols: the largest N of the items (when it says 4096 or less, only the first 4096
 * columns of every item are visited).  One work-group per record.  A sequence armed with nhip_gemv_tile_carry rides in
 * the launch. */
int nhip_gemv_events(void *stream, const int *items, int n_items, const float *AT,
                     const float *X, const float *Yin, float *Y, const int *targets, float *F,
                     int max_cols);

/* The same product for an X that is mostly zero (the spikes of a population; no
 * counterpart in the reference, whose kernels multiply every stored element).  All slices
 * read one X of `n_cols` elements at X + x_start (n_cols <= 1,179,648).  `mask` is a
 * workspace of (n_cols + 127) / 128 * 4 words, 16-byte aligned, that the call fills with one
 * bit per element of X ("is not +0.0") in a first launch; the second launch keeps it in LDS
 * and takes the constant +0.0 instead of reading X where the bit is clear.  Bit-identical to
 * nhip_spmv_sell whatever X and the matrices hold.  NHIP_E_TOOBIG when X is longer than the
 * limit.  Events armed with nhip_time_next_launch time the first, short launch. */
int nhip_spmv_sell_skip(void *stream, const int *slices, int n_slices, const int *row_len,
                        const int *cols, const float *vals, const float *X, float *Y,
                        int x_start, int n_cols, unsigned *mask);

/* Either product followed, row by row, by the first-order filters that read its output
 * (`plan_sparse_dot_inc` followed by `plan_linearfilter`, clra_nonlinearities.py:577-803,
 * simple case y = b0 x - a0 y or y = b0 x of :630-650): saves the filter launch and a pass
 * over the product.
 *   slice_epi : int32[n_slices][4] {first target, number of targets, first row of the slice
 *               in its matrix, 0}
 *   targets   : int32[][4] {y_start of the filter output, bits of a0, bits of b0, number of
 *               denominator coefficients (0 or 1)}, as for nhip_gemv_tile_filter
 *   F         : buffer of the filter outputs
 * mask == NULL: the ordinary product (x_start, n_cols unused); else as nhip_spmv_sell_skip. */
int nhip_spmv_sell_filter(void *stream, const int *slices, int n_slices, const int *row_len,
                          const int *cols, const float *vals, const float *X, float *Y,
                          const int *slice_epi, const int *targets, float *F, int x_start,
                          int n_cols, unsigned *mask);

/* ---- neurons -----------------------------------------------------------
 * LIF with refractory state and spike-time interpolation.
 * replaces: clra_nonlinearities.py `plan_lif` (:1028-1146, non-adaptive,
 * fastlif=False) through `_plan_template` (:1286-1483).
 *   desc : int32[n_blocks][12] {j_start, v_start, w_start, s_start, count,
 *                               tau, ref, amp, pflags, 0, 0, 0}
 * `tau/ref/amp` are float bits, or (if bit 0/1/2 of pflags is set) element
 * offsets into `TAU/REF/AMP` for per-neuron parameter vectors. */
int nhip_lif(void *stream, const int *desc, int n_blocks, double dt, int upsample,
             const float *J, float *V, float *W, float *S, const float *TAU,
             const float *REF, const float *AMP);
/* LIF rate curve.  replaces: `plan_lif_rate` (:1149-1197).
 *   desc : int32[n_blocks][8] {j_start, r_start, count, tau, ref, amp, pflags, 0} */
int nhip_lif_rate(void *stream, const int *desc, int n_blocks, const float *J, float *R,
                  const float *TAU, const float *REF, const float *AMP);
/* The other neuron types share one work-list row per block of one population:
 *   desc : int32[n_blocks][16] {j_start, out_start, v_start, w_start, n_start, count,
 *                               pflags, 0, p0, p1, p2, p3, p4, 0, 0, 0}
 * p0.. are the type's parameters in the order of its pointer arguments, as float
 * bits or (bit k of pflags set) element offsets of per-neuron vectors; offsets of
 * arrays a type does not use are ignored.
 * Adaptive LIF: the LIF update on J - N, then N += (dt / tau_n) (inc_n S - N);
 * parameters tau, ref, amp, tau_n, inc_n.  replaces: `plan_lif` with N, tau_n, inc_n
 * (:1028-1146). */
int nhip_alif(void *stream, const int *desc, int n_blocks, double dt, int upsample,
              const float *J, float *V, float *W, float *S, float *N, const float *TAU,
              const float *REF, const float *AMP, const float *TAU_N, const float *INC_N);
/* Adaptive LIF rate.  replaces: `plan_lif_rate` with N, tau_n, inc_n (:1149-1197). */
int nhip_alif_rate(void *stream, const int *desc, int n_blocks, double dt, const float *J,
                   float *R, float *N, const float *TAU, const float *REF, const float *AMP,
                   const float *TAU_N, const float *INC_N);
/* R = amp max(J, 0).  replaces: `plan_rectified_linear` (:1238-1258). */
int nhip_relu(void *stream, const int *desc, int n_blocks, const float *J, float *R,
              const float *AMP);
/* V += dt max(J, 0); spikes = floor(V); V -= spikes; S = amp spikes / dt.
 * replaces: `plan_spiking_rectified_linear` (:1200-1235). */
int nhip_spiking_relu(void *stream, const int *desc, int n_blocks, double dt, const float *J,
                      float *V, float *S, const float *AMP);
/* R = 1 / (ref (1 + exp(-J))), 0 below J = -88, 1 / ref above J = 15.
 * replaces: `plan_sigmoid` (:1261-1283). */
int nhip_sigmoid(void *stream, const int *desc, int n_blocks, const float *J, float *R,
                 const float *REF);

/* ---- synapses ----------------------------------------------------------
 * Direct-form linear filter step  y <- sum_p b[p] x[n-p] - sum_p a[p] y[n-1-p]
 * with ring buffers for orders > 1; fast paths for (na,nb) = (0,1) and (1,1).
 * replaces: `plan_linearfilter` (:577-803) -- both its `linearfilter` kernel
 * and the `linearfilter_inc` position kernel (positions advance in the same
 * launch, after a block-wide barrier).
 *   desc : int32[n_blocks][16] {x_start, x_stride0, x_stride1, y_start,
 *          y_stride0, y_stride1, shape1, offset, count, na, nb, a_start,
 *          b_start, xbuf_start, ybuf_start, size}
 *   pos  : int32[n_blocks][2]  {xbuf_pos, ybuf_pos}   (read and advanced) */
int nhip_linearfilter(void *stream, const int *desc, int *pos, int n_blocks, int lanes,
                      const float *X, float *Y, const float *A, const float *B, float *Xbuf,
                      float *Ybuf);

/* ---- element-wise ------------------------------------------------------
 * `lanes` (here and for the synapse filter above, the inputs and the probes below) =
 * threads that work on one row of the work list: 256 (one group per row, for long
 * rows) or a power of two from 1 to 64 (a group then takes 256 / lanes rows side by
 * side, for models with very many very short signals).  The host picks it per launch from the
 * row lengths; results do not depend on it. */
/* Y (=|+=) alpha * A * X with scalar/row/column broadcasting, or outer product.
 * replaces: `plan_elementwise_inc` (:414-574).
 *   desc : int32[n_blocks][16] {a_start, a_shape0, a_shape1, a_stride0, x_start,
 *          x_shape0, x_shape1, x_stride0, y_start, y_shape1, y_stride0, offset,
 *          count, alpha_bits, flags(bit0 outer, bit1 inc), 0} */
int nhip_elementwise_inc(void *stream, const int *desc, int n_blocks, int lanes, const float *A,
                         const float *X, float *Y);
/* Outer-product increment Y (=|+=) (alpha a) (x) x and, in the same launch, the step of
 * the first-order filters that produce its column operands: a record's work-group owns
 * all rows of up to 128 columns of one matrix, so it is the only reader of those elements
 * of the filter output and steps them once its part of the matrix is written.
 * replaces: `plan_elementwise_inc` with outer=True (:414-574) followed by
 * `plan_linearfilter` (:577-803, its cases (na,nb) = (0,1) and (1,1)) on the vector the
 * outer product has just read -- the end of a PES step.  Element by element the same
 * rounded operations as the two kernels.
 *   desc : int32[n_records][16] {a_start, a_stride0 (0: one value for all rows),
 *          x_start, x_stride0 (0: one value for all columns), y_start, y_stride0,
 *          rows (<= 256), col0, ncols (<= 128), alpha_bits,
 *          flags (bit0 inc, bit1 filter present, bit2 filter has a0, bit3 no outer
 *          product: the record only steps a filter), s_start, f_start (filter input /
 *          output; column c of the record at *_start + c), a0_bits, b0_bits, 0};
 *          y_start, y_stride0, col0 and ncols are multiples of 4 (16-byte accesses)
 *   A, X, Y : buffers of the outer product;  S, F : of the filters (F may be X). */
int nhip_outer_filter(void *stream, const int *desc, int n_records, const float *A,
                      const float *X, float *Y, const float *S, float *F);
/* Weight-update rules that write a delta matrix per connection (row i = post
 * neuron, column j = pre element; delta rows are contiguous):
 *   BCM  delta[i,j] = alpha * post[i] * (post[i] - theta[i]) * pre[j]
 *   OJA  delta[i,j] = alpha * post[i] * (pre[j] - beta * weights[i,j] * post[i])
 *   VOJA delta[i,j] = alpha * learn * post[i] * (scale[i] * pre[j] - enc[i,j])
 * each product and difference rounded separately, left to right.
 * replaces: `plan_bcm` (:2082-2169), `plan_oja` (:2172-2277), `plan_voja`
 * (:2280-2405).  AUX is theta (vector), weights or encoders (matrix, rows
 * contiguous); LEARN and SCALE are read by VOJA only.  With `inc` the change is added
 * to DELTA instead of stored (DELTA may then be the weight / encoder matrix itself,
 * also when it is AUX: the learning step and the `Copy(delta -> weights, inc)` that
 * follows it in the reference's graph in one pass).
 *   desc : int32[n_blocks][16] {pre_start, pre_stride0, post_start, post_stride0,
 *          aux_start, aux_stride0, delta_start, delta_stride0, shape1, offset,
 *          count, alpha_bits, beta_bits, learn_start, scale_start, scale_stride0} */
#define NHIP_RULE_BCM 1
#define NHIP_RULE_OJA 2
#define NHIP_RULE_VOJA 3
int nhip_learning_rule(void *stream, int rule, int inc, const int *desc, int n_blocks,
                       const float *PRE, const float *POST, const float *AUX, float *DELTA,
                       const float *LEARN, const float *SCALE);
/* ---- convolution, pooling -------------------------------------------------
 * Y = conv2d(X, F) over one image signal (Y is set, not incremented, like the
 * reference's kernel), or local filtering (one filter bank per output pixel).
 * replaces: `plan_conv2d` (:1762-1969; biases unsupported there too).
 *   geom : HOST int32[21] {nxi, nxj, nc, nyi, nyj, nf, si, sj, sti, stj, pi, pj,
 *          x_start, y_start, f_start, channels_last, local, tile_i, tile_j,
 *          tile_f, c_chunk}
 * X is (nxi, nxj, nc) with channels last, else (nc, nxi, nxj); Y likewise with nf;
 * F is (si, sj, nc, nf), or for local filtering (nf, nc, si, sj, nyi, nyj).  A group
 * computes tile_i x tile_j output pixels x tile_f filters (product <= 256) and
 * stages c_chunk channels of the input patch and of its filters' taps in LDS at a
 * time (<= 64 KiB).  Each
 * output is accumulated over channel, kernel row, kernel column in that order with
 * one fused multiply-add per term. */
int nhip_conv2d(void *stream, const int *geom, const float *X, const float *F, float *Y);
/* Average pooling, channels first; window elements outside the image (bottom /
 * right edge) and NaN inputs are left out of the mean.
 * replaces: `plan_pool2d` (:1972-2079).
 *   geom : HOST int32[11] {nc, nyi, nyj, nxi, nxj, si, sj, sti, stj, x_start, y_start} */
int nhip_pool2d(void *stream, const int *geom, const float *X, float *Y);

/* ---- white noise -----------------------------------------------------------
 * Y[item] (=|+=) a fresh sample per element, from Uniform(p0, p1) or
 * Gaussian(mean p0, std p1), times sqrt_dt_inv where flagged.
 * replaces: `plan_whitenoise`, `init_rngs`, `create_rngs` (:1486-1675).  The
 * reference draws from RANLUX states in device memory; this library uses the
 * counter-based Philox4x32-10 generator: the block of four 32-bit words for
 * elements 4q..4q+3 of call n is philox(counter {q, n, 0, 0}, key {seed, 0}), so
 * the sample streams are not the reference's (whose streams are not nengo's
 * either), and the only state is the call count.  An item is cut into blocks of
 * elements [offset, offset + count), offset a multiple of 4; every block carries its
 * own copy of the call count.
 *   desc     : int32[n_blocks][8] {y_start (of the item), count, dist, p0_bits,
 *                                  p1_bits, flags(bit0 scale, bit1 inc), seed, offset}
 *   counters : int32[n_blocks], read and advanced by one per call (zero them to
 *              restart the streams) */
#define NHIP_DIST_UNIFORM 0
#define NHIP_DIST_GAUSSIAN 1
int nhip_whitenoise(void *stream, const int *desc, int n_blocks, int *counters,
                    double sqrt_dt_inv, float *Y);
/* out[t] = philox4x32_10(counter = in[t][0..3], key = in[t][4..5]) for n blocks
 * (known-answer testing of the generator). */
int nhip_philox4x32(void *stream, const unsigned *counters_keys, unsigned *out, int n);

/* 2-D strided Y (=|+=) X.  replaces: `plan_copy` (:217-304).
 *   desc : int32[n_blocks][8] {x_start, y_start, shape1, x_stride0, y_stride0,
 *                              offset, count, inc} */
int nhip_copy(void *stream, const int *desc, int n_blocks, int lanes, const float *X, float *Y);
/* gather/scatter  Y[yi[k]*ys] (=|+=) X[xi[k]*xs].  replaces: `plan_slicedcopy` (:307-411).
 *   desc : int32[n_blocks][8] {x_start, x_stride0, y_start, y_stride0, xi_start,
 *                              yi_start, count, inc} */
int nhip_slicedcopy(void *stream, const int *desc, int n_blocks, int lanes, const float *X,
                    float *Y, const int *XI, const int *YI);
/* constant fill.  replaces: `plan_reset` (:147-214).
 *   blocks : int32[n_blocks][4] {start, count, value_bits, 0} */
int nhip_reset(void *stream, const int *blocks, int n_blocks, int lanes, float *Y);
/* step += 1; time = dt * step (dt in double, rounded once).
 * replaces: `plan_timeupdate` (:113-144). */
int nhip_timeupdate(void *stream, float *step_data, int step_start, float *time_data,
                    int time_start, double dt);

/* ---- inputs and outputs ------------------------------------------------ */
/* table playback  y = S[row(step) , :].  replaces: `plan_presentinput` (:1678-1759).
 *   desc : int32[n][8] {y_start, m, t_start, s_start, nt, pt_bits, has_pt, 0} */
int nhip_presentinput(void *stream, const int *desc, int n, int lanes, float dt, float *Y,
                      const float *T, const float *S);
/* y[k] = f(x[k]) for a fixed table of unary functions (opcode: 0 identity, 1 sin,
 * 2 cos, 3 tanh, 4 exp, 5 square).  replaces the generated `direct` kernel of
 * `plan_direct` (:954-1025) for the expressions the function translator
 * reduces to one of these.
 *   desc : int32[n][4] {x_start, y_start, count, 0} */
int nhip_direct_unary(void *stream, int opcode, const int *desc, int n, int lanes, const float *X,
                      float *Y);
/* probe gather with per-probe float countdown.  replaces: `plan_probes` (:806-951).
 *   desc : int32[n][8] {x_start, shape0, shape1, stride0, stride1, y_start, capacity, 0}
 * `capacity` = rows of Y[i]; a sample that would land beyond it is dropped (the
 * position still advances), so an undrained buffer can never be overrun. */
int nhip_probes(void *stream, const int *desc, int n, int lanes, float *countdowns,
                int *bufpositions, const float *periods, const float *X, float *Y);
/* End-of-batch drain of the probe buffers in one device-to-host transfer.
 * replaces: the host loop of `Simulator._probe` (simulator.py:499-520: one transfer
 * of `bufpositions`, one whole-buffer transfer per probe, a fill, two `finish()`),
 * and the reads of the step counter and clock behind `sim.n_steps` / `sim.time`.
 * A kernel packs into `staging` (device workspace of `staging_words` floats), in words:
 *   [0] signals[step_start], [1] signals[time_start], [2 .. 2+n) bufpositions (int bits),
 *   zero padding up to NHIP_DRAIN_HEADER(n); then for probe i its first
 *   min(bufpositions[i], capacity_i, rows_bound) rows at
 *   NHIP_DRAIN_HEADER(n) + rows_bound * wprefix_i (row-major, width_i words per row),
 *   the rest of its rows_bound rows zero (every transferred word is defined by the call);
 * then bufpositions is zeroed, the first NHIP_DRAIN_HEADER(n) + rows_bound * total_width
 * words are copied to `host_out` (HOST memory of at least that size; pinned memory makes
 * the copy a single DMA) and the stream is synchronised: on return `host_out` is valid.
 *   desc : int32[n][4] {y_start, width, wprefix, capacity}, wprefix_i = sum of width_j, j < i
 *   total_width = sum of widths, max_width = the largest; rows_bound = the caller's upper
 *   bound on rows buffered since the last drain (rows beyond it are not transferred; the
 *   reported counts still tell).  NHIP_E_TOOBIG if the block does not fit `staging`. */
#define NHIP_DRAIN_HEADER(n) ((((n) + 2) + 63) / 64 * 64)
int nhip_probes_drain(void *stream, const int *desc, int n_probes, int total_width,
                      int max_width, int rows_bound, int *bufpositions, const float *Y,
                      const float *signals, int step_start, int time_start, float *staging,
                      long long staging_words, float *host_out);
/* The same drain for callers that cannot allocate device memory or bring a workspace
 * (code under graph capture rules, tight serving loops, harnesses that forbid
 * hipMalloc): no counterpart in the reference.  The staging block is a file-scope
 * device array of NHIP_DRAIN_STATIC_WORDS floats (4 MiB) that every GPU the library runs
 * on holds until the process ends; its address on the current device is looked up once
 * per device, on the first call there.  Allocates nothing, provided `host_out` is
 * pinned host memory (a pageable target makes the runtime stage the copy itself).
 * NHIP_E_TOOBIG when NHIP_DRAIN_HEADER(n) + rows_bound * total_width exceeds
 * NHIP_DRAIN_STATIC_WORDS.  All calls on one GPU share the array: calls that overlap
 * on one GPU (different streams or host threads) race; the array keeps the last
 * call's block, and every word a call transfers is written by that call first. */
#define NHIP_DRAIN_STATIC_WORDS (1 << 20)
int nhip_probes_drain_static(void *stream, const int *desc, int n_probes, int total_width,
                             int max_width, int rows_bound, int *bufpositions, const float *Y,
                             const float *signals, int step_start, int time_start,
                             float *host_out);
/* fill an int32 device array (used to zero probe buffer positions without a
 * memset node, so that it may also be recorded into a graph) */
int nhip_fill_i32(void *stream, int *dst, int n, int value);

/* ---- several small operations in one launch ------------------------------
 * One 256-thread group runs the given operations one after the other (a group
 * barrier in between), each exactly as its own entry point would: for the short
 * operations of a step (clock, inputs, small copies and filters, probes), whose
 * cost is the launch, not the work.  The reference launches each of them
 * separately (plan.py:137-149).  `ops` is a DEVICE array of NhipSeqOp; the pointer
 * slots hold the device-pointer arguments of the matching nhip_* call in order:
 *   RESET {blocks, Y}   COPY {desc, X, Y}   SLICEDCOPY {desc, X, Y, XI, YI}
 *   ELEMENTWISE_INC {desc, A, X, Y}   LINEARFILTER {desc, pos, X, Y, A, B, Xbuf, Ybuf}
 *   TIMEUPDATE {step_data + step_start, time_data + time_start} (d0 = dt)
 *   PRESENTINPUT {desc, Y, T, S} (d0 = dt)   DIRECT_UNARY {desc, X, Y} (i0 = opcode)
 *   PROBES {desc, countdowns, bufpositions, periods, X, Y} */
enum {
    NHIP_SEQ_RESET = 1,
    NHIP_SEQ_COPY = 2,
    NHIP_SEQ_SLICEDCOPY = 3,
    NHIP_SEQ_ELEMENTWISE_INC = 4,
    NHIP_SEQ_LINEARFILTER = 5,
    NHIP_SEQ_TIMEUPDATE = 6,
    NHIP_SEQ_PRESENTINPUT = 7,
    NHIP_SEQ_DIRECT_UNARY = 8,
    NHIP_SEQ_PROBES = 9
};
typedef struct NhipSeqOp {
    int kind;                /* NHIP_SEQ_* */
    int n_blocks;            /* rows of the operation's work list (1 for TIMEUPDATE) */
    int i0;                  /* DIRECT_UNARY: opcode */
    int lanes;               /* threads per work-list row, as for the matching entry point */
    double d0;               /* TIMEUPDATE, PRESENTINPUT: dt */
    unsigned long long p[8]; /* device pointers, see above */
} NhipSeqOp;                 /* 88 bytes */
/* at most 16 operations; `lanes` of every record as for the matching entry point
 * (256 for TIMEUPDATE).  n_staged = the sum of n_blocks over the operations with
 * lanes == 256, at most 128: their rows are staged in LDS (the library cannot read
 * the device table to check it). */
int nhip_sequence(void *stream, const void *ops, int n_ops, int n_staged);
/* The same with up to NHIP_SEQ_MAX_CHAINS chains side by side, a work-group each:
 * `ops` holds the chains one after the other, chain c has chain_ops[c] operations
 * (1 ... 16) and chain_staged[c] staged rows (HOST arrays).  Operations of different
 * chains must not touch the same memory unless both only read it; inside a chain the
 * order of `ops` holds.  No counterpart in the reference, which runs every plan as a
 * launch of its own (plan.py:128-135). */
#define NHIP_SEQ_MAX_CHAINS 4
int nhip_sequence_chains(void *stream, const void *ops, const int *chain_ops,
                         const int *chain_staged, int n_chains);
/* The same chains without a launch of their own: they ride in the calling thread's NEXT
 * large-item GEMV launch (nhip_gemv_tile_lif, nhip_gemv_tile_lif_sums or
 * nhip_gemv_tile_filter with pow2_cols >= 2), one extra work-group per chain that runs
 * beside the groups of the GEMV.  For chains that touch nothing that launch reads or
 * writes (unless both only read it).  This call only records its arguments (`ops` must stay
 * valid until that launch has run; the host arrays are copied); the launch consumes them,
 * and fails with NHIP_E_BADARG if it cannot carry them (another kernel class, no epilogue,
 * an empty task list).  n_chains = 0 disarms.  `needs` names the operations of the chains
 * that not every carrying kernel holds (the library cannot read the device table): the
 * launch that visits active columns only (nhip_gemv_events) runs on half the registers of
 * the others and refuses chains that need any of them.  No counterpart in the reference
 * (plan.py:128-149 runs every plan as a launch of its own). */
#define NHIP_SEQ_NEEDS_UNARY 1         /* an NHIP_SEQ_DIRECT_UNARY operation */
#define NHIP_SEQ_NEEDS_HIGHER_ORDER 2  /* a linear filter with more than one coefficient on a side */
int nhip_gemv_tile_carry(const void *ops, const int *chain_ops, const int *chain_staged,
                         int n_chains, int needs);

/* ---- function nodes compiled at run time ----------------------------------
 * replaces: `plan_direct` (:954-1025), which builds an OpenCL program from the
 * translated body of a Python function.  `source` is HIP source text holding
 *     extern "C" __global__ void <kernel_name>(int n, const int *t_starts,
 *         const float *T, const int *x_starts, const float *X,
 *         const int *y_starts, float *Y)
 * in which thread k < n computes instance k: it reads its time at T + t_starts[k]
 * and its input vector at X + x_starts[k] (either may be unused and NULL) and
 * writes its output vector at Y + y_starts[k].
 * nhip_rtc_compile compiles for `arch` (NULL: gfx950) and needs no device; the
 * compiler's messages are copied into `log`.  nhip_rtc_load loads the code on the
 * current device (once per program) and looks the kernel up; nhip_rtc_destroy
 * unloads and frees (no launch of the program may be pending or recorded). */
int nhip_rtc_compile(const char *source, const char *arch, void **program_out, char *log,
                     int log_len);
int nhip_rtc_load(void *program, const char *kernel_name, void **function_out);
int nhip_rtc_destroy(void *program);
int nhip_rtc_launch_direct(void *stream, void *function, int n, const int *t_starts,
                           const float *T, const int *x_starts, const float *X,
                           const int *y_starts, float *Y);

/* ---- executor ----------------------------------------------------------
 * replaces the Python launch loop of `Plans.enqueue_n_times` (plan.py:137-149):
 * the plan sequence of one (or several) timesteps is recorded once from the
 * stream into a graph and replayed. */
int nhip_capture_begin(void *stream);
int nhip_capture_end(void *stream, void **graph_exec_out);
/* Hands an instantiated graph to the device ahead of its first launch (nothing is
 * executed), so that the first launch costs what every later one costs. */
int nhip_graph_upload(void *graph_exec, void *stream);
int nhip_graph_launch(void *graph_exec, void *stream, int n_times);
int nhip_graph_destroy(void *graph_exec);
int nhip_stream_sync(void *stream);
/* The next kernel launched by the calling thread through this library carries
 * `start` and `stop` itself: their difference is the kernel's own duration, without
 * the dispatch latency and end-of-kernel cache maintenance that events recorded
 * around a launch include (the figure a kernel trace shows).  Both NULL cancels.
 * Not for launches that are being recorded into a graph, and not for
 * nhip_rtc_launch_direct (which launches through the module API). */
int nhip_time_next_launch(void *start, void *stop);
/* 1 while events armed by nhip_time_next_launch wait for a launch (an entry point
 * that returned without launching, e.g. on an empty work list, leaves them so), else 0. */
int nhip_launch_events_pending(void);

/* events on `stream` (for per-plan and whole-run timing) */
int nhip_event_create(void **event_out);
int nhip_event_record(void *event, void *stream);
int nhip_event_elapsed_ms(void *start, void *stop, float *ms_out); /* syncs on `stop` */
int nhip_event_destroy(void *event);

/* Calibration (no counterpart in the reference): what the device does with the traffic
 * of a GEMV launch with a neuron epilogue when nothing else is asked of the kernel.  Every
 * wave streams 128 rows x `cols` floats of the row-major `A` (n_rows x cols, 16-byte aligned,
 * n_rows a multiple of 128, cols a multiple of 8), then reads `n_reads` and writes `n_writes`
 * vectors of 128 floats at its rows (`R`: n_reads x n_rows, `W`: n_writes x n_rows floats,
 * at least one float each); `nontemporal` != 0 writes with non-temporal stores.  Its
 * duration is the floor against which bench.py reports the duration of the dominant launch. */
int nhip_calib_stream_mix(void *stream, const float *A, long long n_rows, int cols,
                          const float *R, int n_reads, float *W, int n_writes, int nontemporal);

#ifdef __cplusplus
}
#endif
#endif /* NENGO_HIP_H */
