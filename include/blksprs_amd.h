/*
 * C ABI of the MI355X (gfx950) block-sparse compute library, libblksprs_amd.so.
 *
 * Every entry point takes plain device pointers, sizes and a HIP stream and
 * returns 0 on success or a negative BSA_E* code; bsa_last_error() then holds a
 * message for the calling thread.  Nothing here allocates device memory: the
 * caller owns every buffer, including the workspace of the LUT builder.  All
 * kernels are enqueued on `stream` (a hipStream_t passed as void*); only
 * bsa_lut_packed / bsa_lut_contraction_offsets with a non-NULL `stats_host`
 * wait for the stream, because the caller needs the counts to size its outputs.
 *
 * A block-sparse tensor is the triple (blocks, layout, sbs): `layout` is a
 * contiguous (B, R, C) array of 0/1 bytes, `blocks` is (nnz, sbs, sbs) holding
 * the active blocks in row-major order of the layout.
 *
 * Each declaration names the reference interface it stands in for
 * (paths relative to the FelixSchoen/blksprs checkout).
 */
#ifndef BLKSPRS_AMD_H
#define BLKSPRS_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BSA_ABI_VERSION 3

/* error codes */
#define BSA_OK 0
#define BSA_EINVAL (-1)  /* bad argument (shape, dtype, alignment, NULL pointer) */
#define BSA_ELAUNCH (-2) /* the HIP runtime refused a launch or copy */
#define BSA_ELIMIT (-3)  /* a size exceeds what the kernels index */

/* element types of matmul / attention operands */
#define BSA_F32 0
#define BSA_F16 1
#define BSA_BF16 2

typedef void *bsa_stream_t; /* hipStream_t */

int bsa_abi_version(void);
const char *bsa_last_error(void);
/* One line naming the compiler the library was built with ("hipcc: <version line of hipcc --version>; flags: ...").
 * Some kernels place their own waits for memory around loads the compiler does not see; a red bit-identity test
 * after a toolchain change is read next to this line.  No counterpart in the reference. */
const char *bsa_build_info(void);

/* ------------------------------------------------------------------ LUTs */

/* Bytes of scratch bsa_lut_packed / bsa_lut_contraction_offsets need for n entries. */
size_t bsa_lut_workspace_bytes(int64_t n);

/*
 * Reverse index of a layout: packed[i] = (number of ones before i) if
 * layout[i] else -1, int64, over the flattened layout.
 * Replaces build_packed_indices (blksprs/utils/tools.py:38-57) and the
 * `layout.sum().item()` block counts (blksprs/ops/matmul.py:270-273,
 * blksprs/ops/conversion.py:286-288).
 *
 * row_len > 0 additionally writes the CSR row offsets row_offsets[n/row_len+1]
 * (int32; the cumsum of per-row counts with a leading 0 of
 * _build_segmented_indices, blksprs/ops/flash_attention.py:1923-1949) and the
 * largest row count.  stats_dev[0] = count, stats_dev[1] = max row count
 * (0 when row_len == 0).  If stats_host != NULL the two values are copied to it
 * and the stream is synchronised.
 */
int bsa_lut_packed(const uint8_t *layout, int64_t n, int64_t row_len, int64_t *packed,
                   int32_t *row_offsets, int64_t *stats_dev, int64_t *stats_host,
                   void *workspace, size_t workspace_bytes, bsa_stream_t stream);

/*
 * bsa_lut_packed for callers that cannot allocate device memory (code under HIP graph capture, serving loops,
 * harnesses that forbid hipMalloc): the same launches and the same results, but the scan's scratch (one int32
 * count and one int64 offset per tile of 2048 layout entries) lives in a file-scope device array of 96 KiB that
 * every device the library runs on holds until the process ends, so no workspace is passed and nothing is
 * allocated or freed.  n may be at most bsa_lut_packed_static_max_entries() (2^24 layout entries); a larger n
 * returns BSA_ELIMIT.  The counts stay on the device (stats_dev as in bsa_lut_packed; no host copy, no wait for
 * the stream).  The first call on a device looks up the array's device address (hipGetSymbolAddress); make that
 * call outside a capture.  All calls on one device share the array: the call overwrites every entry it reads,
 * so nothing needs clearing between calls, but two calls that overlap on one device (different streams or
 * threads) race.  This entry point has no counterpart in the reference.
 */
int64_t bsa_lut_packed_static_max_entries(void);
int bsa_lut_packed_static(const uint8_t *layout, int64_t n, int64_t row_len, int64_t *packed,
                          int32_t *row_offsets, int64_t *stats_dev, bsa_stream_t stream);

/*
 * Coordinates of the active blocks, int64 [count, 3] = (b, r, c) in row-major
 * order: torch.nonzero(layout) of build_layout_indices
 * (blksprs/utils/tools.py:33-35), derived from the reverse index.
 */
int bsa_lut_nonzero(const int64_t *packed, int64_t B, int64_t R, int64_t C, int64_t *coords,
                    bsa_stream_t stream);

/*
 * CSR column ids (int32 [count], ascending inside a row): the `indices` of
 * _build_segmented_indices (blksprs/ops/flash_attention.py:1945-1947).
 */
int bsa_lut_csr_indices(const int64_t *packed, int64_t n, int64_t C, int32_t *indices,
                        bsa_stream_t stream);

/*
 * Per-row descending sort of the reverse index (active blocks first, then -1):
 * packed_indices_sorted of softmax_fused_build_layout_cache
 * (blksprs/ops/softmax.py:652-657), int64 [n_rows * C].
 */
int bsa_lut_sorted_rows(const int32_t *row_offsets, int64_t n_rows, int64_t C, int64_t *sorted,
                        bsa_stream_t stream);

/*
 * Lists over pairs of neighbouring rows of a layout (0/1 bytes [B, R, C]): the groups of two query blocks the
 * attention forward kernel gives to one workgroup (bsa_attn_fwd_records takes their entries).
 * bsa_lut_pair_union writes the union of rows 2 g and 2 g + 1 as bytes [B, ceil(R / 2), C]; scanned with
 * bsa_lut_packed (row_len = C) it yields the groups' offsets and the reverse index union_packed, from which
 * bsa_lut_pair_entries writes, for the p-th active position of the union, entries[p] = column |
 * first row active << 28 | second row active << 29 (C < 2^28).  No counterpart in the reference.
 */
int bsa_lut_pair_union(const uint8_t *layout, int64_t B, int64_t R, int64_t C, uint8_t *uni, bsa_stream_t stream);
int bsa_lut_pair_entries(const uint8_t *layout, const int64_t *union_packed, int64_t B, int64_t R, int64_t C,
                         int32_t *entries, bsa_stream_t stream);

/*
 * Boolean block product lo[b,i,j] = OR_k lx[b,i,k] & ly[b,k,j]:
 * build_sparsity_layout_matmul (blksprs/layouting/sparsity_layout.py:244-258).
 */
int bsa_layout_matmul(const uint8_t *lx, const uint8_t *ly, int64_t B, int64_t R, int64_t K,
                      int64_t C, uint8_t *lo, bsa_stream_t stream);

/*
 * Contraction lists of a block-sparse product, phase 1.  For every position
 * (b,i,j) of the output layout that is active (pidx_o >= 0) counts the k with
 * x(b,i,k) and y(b,k,j) both active and writes the exclusive prefix of those
 * counts over positions to pos_offsets (int32 [B*R*C + 1]); stats_dev[0] = total
 * number of (x block, y block) pairs.  The reference has no such list: its
 * kernel scans every k of every output block (blksprs/ops/matmul.py:191-226).
 * mask_x: uint64 [B*R*W], mask_y: uint64 [B*C*W], W = ceil(K/64) (scratch the
 * caller provides; they are inputs of phase 2).
 */
int bsa_lut_contraction_offsets(const int64_t *pidx_x, const int64_t *pidx_y,
                                const int64_t *pidx_o, int64_t B, int64_t R, int64_t K, int64_t C,
                                uint64_t *mask_x, uint64_t *mask_y, int32_t *pos_offsets,
                                int64_t *stats_dev, int64_t *stats_host, void *workspace,
                                size_t workspace_bytes, bsa_stream_t stream);

/*
 * Phase 2: pair_offsets int32 [nnz_o + 1] and pairs int32 [total, 2] =
 * (index of the x block, index of the y block), ascending k inside an output
 * block (the accumulation order of blksprs/ops/matmul.py:191-242).
 */
int bsa_lut_contraction_pairs(const int64_t *pidx_x, const int64_t *pidx_y, const int64_t *pidx_o,
                              int64_t B, int64_t R, int64_t K, int64_t C, const uint64_t *mask_x,
                              const uint64_t *mask_y, const int32_t *pos_offsets, int64_t nnz_o,
                              int32_t *pair_offsets, int32_t *pairs, bsa_stream_t stream);

/* ------------------------------------------------------------ conversion */

/*
 * Gather the active sbs x sbs tiles of a dense (B, rows, cols) array into
 * (nnz, sbs, sbs).  Bit-exact copy for any element size in {1,2,4,8}.
 * Replaces to_sparse_forward / to_sparse_kernel (blksprs/ops/conversion.py:191-276).
 */
int bsa_to_sparse(const void *dense, const int64_t *coords, void *blocks, int64_t nnz, int64_t rows,
                  int64_t cols, int sbs, int elem_size, bsa_stream_t stream);

/*
 * Scatter compressed blocks into a dense (B, R*sbs, C*sbs) array; inactive
 * tiles receive the element whose bit pattern is the low elem_size bytes of
 * fill_bits.  One pass over the output (the reference fills and then
 * overwrites).  Replaces to_dense_forward / to_dense_kernel
 * (blksprs/ops/conversion.py:463-557).
 */
int bsa_to_dense(const void *blocks, const int64_t *packed, void *dense, int64_t B, int64_t R,
                 int64_t C, int64_t nnz, int sbs, int elem_size, uint64_t fill_bits,
                 bsa_stream_t stream);

/* ------------------------------------------------------------- row-wise */

/*
 * Row-wise sum (op 0) or maximum (op 1) over the active blocks of each block
 * row; fp32 accumulation, rounded once to `dtype`.  row_offsets: int32
 * [n_rows + 1] CSR offsets of the layout flattened to (B*R, C); packed_out:
 * int64 [n_rows] reverse index of the (B, R, 1) output layout (-1 for block
 * rows without blocks).  out is [n_out, sbs, sbs] (column 0 holds the result,
 * the other columns 0 for the sum and -inf for the maximum) or, with
 * slice_only, [n_out, sbs, 1].  A maximum over a row that holds a NaN is NaN.
 * Replaces row_wise_sum_forward / row_wise_sum_kernel and row_wise_max_forward
 * / row_wise_max_kernel (blksprs/ops/misc/row_wise.py:103-205, :283-419), which
 * accumulate with atomics into an fp32 buffer and convert afterwards.
 */
int bsa_row_reduce(const void *x, const int32_t *row_offsets, const int64_t *packed_out, void *out,
                   int64_t n_rows, int64_t n_out, int64_t nnz, int sbs, int dtype, int op, int slice_only,
                   bsa_stream_t stream);

/*
 * out[n][e][:] = x[n][e][:] + y[packed_rows[b * R + r]][e][0] for block
 * n = coords[n] = (b, r, c); y is [n_y, sbs, y_cols] with y_cols 1 or sbs.
 * Blocks whose row has no entry in y are written as zeros.  Replaces
 * row_wise_add_forward / row_wise_add_kernel
 * (blksprs/ops/misc/row_wise.py:488-603).
 */
int bsa_row_add(const void *x, const int64_t *coords, const int64_t *packed_rows, const void *y, void *out,
                int64_t nnz, int64_t n_y, int64_t B, int64_t R, int y_cols, int sbs, int dtype,
                bsa_stream_t stream);

/* --------------------------------------------------------------- softmax */

/*
 * Row-wise softmax over the active blocks of each block row, fp32.
 * row_offsets: int32 [n_rows + 1] CSR offsets of the layout flattened to
 * (B*R, C).  Replaces softmax_fused_forward / softmax_fused_kernel and the
 * five-kernel softmax_forward (blksprs/ops/softmax.py:93-144, :437-570).
 */
int bsa_softmax_fwd(const float *x, float *out, const int32_t *row_offsets, int64_t n_rows,
                    int64_t nnz, int sbs, bsa_stream_t stream);

/*
 * dx = y * (g - sum_row(y * g)).  Replaces softmax_fused_backward /
 * softmax_backward (blksprs/ops/softmax.py:156-207, :478-513, :574-638).
 */
int bsa_softmax_bwd(const float *grad_out, const float *y, float *grad_in,
                    const int32_t *row_offsets, int64_t n_rows, int64_t nnz, int sbs,
                    bsa_stream_t stream);

/* ---------------------------------------------------------------- matmul */

/*
 * out[n] = sum over the pairs of output block n of x[px] @ y[py], fp32
 * accumulation, result rounded once to `dtype`; an output block with no pair is
 * written as zeros.  Replaces matmul_forward / matmul_kernel
 * (blksprs/ops/matmul.py:70-253).  trans_x / trans_y read the x / y blocks
 * transposed (block[c][r] instead of block[r][c]); the reference materialises
 * such operands with transpose() first (blksprs/ops/matmul.py:135-143).
 * block_order (int32 [nnz_o], a permutation, or NULL for identity) is the order in
 * which output blocks are worked on; it only affects cache behaviour, never results.
 */
int bsa_matmul(const void *x, const void *y, void *out, const int32_t *pair_offsets,
               const int32_t *pairs, const int32_t *block_order, int64_t nnz_o, int64_t nnz_x, int64_t nnz_y, int sbs, int dtype,
               int trans_x, int trans_y, bsa_stream_t stream);

/*
 * Work orders of the matmul kernels, built on the device without a read by the host (integer only; a stable sort by a
 * key computed from tables already on the device).  workspace: bsa_lut_order_workspace_bytes(n) bytes, 256-byte
 * aligned, n = the number of items sorted (blocks, or n_rows << parts_log2).  No counterpart in the reference, whose
 * kernels take output blocks in launch order (blksprs/ops/matmul.py:88-128); an order changes which blocks are in
 * flight together, never a result.
 *
 * bsa_lut_block_order: order (int32 [n], a permutation) lists the n active blocks of a layout, given by their
 * coordinates layout_indices (int64 [n, 3]: batch, row, column, as bsa_lut_nonzero writes them), by super-tiles of
 * tile x tile blocks of the n_rows x n_cols block grid: the super-tiles of a batch entry row by row, the blocks of
 * a super-tile row by row.  It is the block_order argument of bsa_matmul.
 *
 * bsa_lut_row_work_table: the work_table argument of bsa_matmul_rows_records (see there for the entries' format
 * and for why the order is what it is): table_len = 8 * ceil(n_rows / 8) << parts_log2 entries; every XCD's
 * contiguous eighth of the rows batch entry by batch entry (rows_per_batch rows each), part by part, the rows
 * with the most (x, y) pairs first (pair_offsets, row_offsets_o as for bsa_matmul_rows_records; max_work: a bound
 * on the pairs of one row, e.g. inner blocks times output columns).  pair_up != 0: within such a group longest,
 * shortest, second longest, ...; sweep > 0: every second run of `sweep` entries of a group carries
 * BSA_ROWS_DOWNWARD.
 */
size_t bsa_lut_order_workspace_bytes(int64_t n);
int bsa_lut_block_order(const int64_t *layout_indices, int64_t n, int64_t n_rows, int64_t n_cols, int tile,
                        int32_t *order, void *workspace, size_t workspace_bytes, bsa_stream_t stream);
int bsa_lut_row_work_table(const int32_t *pair_offsets, const int32_t *row_offsets_o, int64_t n_rows,
                           int64_t rows_per_batch, int parts_log2, int pair_up, int64_t max_work, int sweep,
                           int32_t *table, int64_t table_len, void *workspace, size_t workspace_bytes,
                           bsa_stream_t stream);

#define BSA_ROWS_RECORD_INTS 128
#define BSA_ROWS_DOWNWARD (1 << 30)

/*
 * Layout-to-LUT step of bsa_matmul_rows (integer only): one record of BSA_ROWS_RECORD_INTS int32 per work
 * table entry.  x_row_offsets and o_row_offsets are the int32 CSR row offsets (n_rows + 1 entries,
 * rows = B * R) of the x layout and of the output layout as bsa_lut_packed(row_len = ...) writes them; n_cols
 * is the number of block columns of the output layout.  A workgroup of bsa_matmul_rows computes one part of a
 * row: the row's output blocks are cut into 2^parts_log2 runs of equal length (parts_log2 0..3; more parts keep
 * fewer y blocks in flight at the price of loading the x row once per part); a part holds at most 64 blocks, so
 * n_cols <= 64 << parts_log2 (BSA_EINVAL otherwise).  work_table (n_items int32) is the order in which parts
 * are handed to workgroups: entry row << parts_log2 | part, or -1 for nothing; every (row, part) once; with
 * BSA_ROWS_DOWNWARD or'ed in, the part's blocks are computed from the highest column down (same results: the
 * order of the products inside a block does not change), so that a part that starts when its neighbours on the
 * XCD end finds the y blocks of the high columns still in the L2.  NULL
 * (with parts_log2 == 0 and n_items == n_rows): rows 0, 1, 2, ...  Workgroup g runs on XCD g % 8, so a table
 * that gives position 8 k + c to the k-th item of a contiguous eighth c of the rows, heaviest rows first, keeps
 * the y blocks in flight on one L2 few and the tail of the launch short.  A record holds the row (-1: nothing),
 * the row's first x block and their number, the part's first output block and their number, the mask of the
 * part's blocks without pairs, the pair range of every block of the part, and for each of the kernel's eight
 * waves the mask of the blocks it computes: the blocks in ascending order, each given to the wave with the
 * fewest pairs so far.  No counterpart in the
 * reference, whose kernel (blksprs/ops/matmul.py:147-253) takes one output block per program.
 */
int bsa_matmul_rows_records(const int32_t *work_table, int64_t n_items, int parts_log2,
                            const int32_t *pair_offsets, const int32_t *x_row_offsets,
                            const int32_t *o_row_offsets, int64_t n_rows, int64_t n_cols, int64_t nnz_x,
                            int32_t *records, bsa_stream_t stream);

/*
 * The same product as bsa_matmul for fp16 / bf16 operands with sbs == 64, organised by output block row: the
 * x blocks of a row are kept in LDS while the row's output blocks are computed.  records (n_items records
 * from bsa_matmul_rows_records, built for the same pair_offsets) says what the workgroups compute: workgroup g
 * takes items_per_workgroup records one after the other, the records 8 (items_per_workgroup (g / 8) + r) + g % 8
 * (consecutive entries of the work table's list for XCD g % 8; a table that pairs a long row with a short one
 * gives every workgroup the same amount of work).  Bit-identical results to bsa_matmul (same accumulation
 * order).  Same reference counterpart as bsa_matmul.
 */
int bsa_matmul_rows(const void *x, const void *y, void *out, const int32_t *pair_offsets,
                    const int32_t *pairs, const int32_t *records, int64_t n_items, int items_per_workgroup,
                    int64_t nnz_o, int64_t nnz_x, int64_t nnz_y, int sbs, int dtype, bsa_stream_t stream);

/*
 * The two backward products of bsa_matmul for 16-bit operands and 64 x 64 blocks, dX = dO Y^T and dY = X^T dO
 * (blksprs/ops/matmul.py:130-145), by LINES: a line is a block row of dX resp. a block column of dY.  All output
 * blocks of a line need the same line of dO (the streamed operand: row i resp. column j of dO) and each pairs it
 * with its own blocks of the other operand (the private operand: Y(k, j) resp. X(i, k)).  One workgroup takes up
 * to 16 output blocks of a line, keeps their accumulators in registers for the whole line and streams the line
 * of dO through LDS once, so dO is read once per launch.  No lists are needed: the kernel finds its blocks in the
 * reverse indices (-1: inactive) of the three layouts, addressed through strides so that one kernel serves rows
 * and columns:
 *   streamed block t of line (b, l):  pidx_streamed[b * streamed_strides[0] + l * streamed_strides[1] + t * streamed_strides[2]]
 *   output block u of line (b, l):    pidx_out[b * out_strides[0] + l * out_strides[1] + u * out_strides[2]]
 *   private block of (u, t):          pidx_private[b * private_strides[0] + u * private_strides[1] + t * private_strides[2]]
 * with t < n_streamed, u < n_outputs (at most 512 each).  dX: lines are the rows of x's layout (B, R, K), streamed =
 * dO with the output layout (B, R, C): strides (R C, C, 1); out = dX: (R K, K, 1); private = y (B, K, C):
 * (K C, C, 1); contract_rows = 0 (the columns of both blocks are contracted).  dY: lines are the columns of y's
 * layout, streamed = dO: (R C, 1, C); out = dY: (K C, 1, C); private = x: (R K, 1, K); contract_rows = 1.
 * Every active output block is written (zeros without a pair); the products of a block are added in ascending
 * order of t, in fp32, and rounded once.
 * part_table (int32 [1 + nnz_out / 16 + n_batches * lines_per_batch]) is written by bsa_matmul_lines_parts from
 * the same argument block (it reads pidx_out and the sizes only; scratch: 4 * lines + 2 int32): [0] = the
 * number of parts (a part = up to 16 output blocks of a line: ceil(blocks / 16) parts per line), then one entry
 * line << 6 | part per part in the order in which workgroups take them: batch entry by batch entry, inside a
 * batch entry first the parts of more than 8 blocks, then the others, each group in the order of the lines
 * (workgroups that run side by side then do about the same work and walk the streamed operand in step).  It
 * depends on the output's layout only.
 * error: NULL, or 32 int32 on the device, zero before the launch: [0] becomes 1 if one of the kernel's bounded
 * waits between the waves of a workgroup ran out (the results are then wrong; it never does unless the device
 * loses a wave), and the other entries then hold what the first such wave saw (its wave number, which wait, the
 * streamed block it waited for, its copying duty, the line's length, the workgroup, the eight waves' positions
 * and the first ten slots' announcements, the line and part, its output blocks): for the library's own tests.
 */
typedef struct bsa_lines_args {
  const void *streamed, *priv; /* blocks of the streamed and of the private operand */
  void *out;
  const int64_t *pidx_streamed, *pidx_private, *pidx_out;
  const int32_t *part_table;
  int64_t n_batches, lines_per_batch, n_streamed, n_outputs;
  int64_t streamed_strides[3], out_strides[3], private_strides[3];
  int64_t nnz_streamed, nnz_private, nnz_out;
  int32_t *error;
} bsa_lines_args;

int bsa_matmul_lines_parts(const bsa_lines_args *args, int32_t *scratch, int32_t *part_table, bsa_stream_t stream);
int bsa_matmul_lines(const bsa_lines_args *args, int contract_rows, int sbs, int dtype, bsa_stream_t stream);

/*
 * Block gather with element transposition: out[o] = transpose(blocks[packed[(b * R + r) * C + c]]) with
 * (b, r, c) = coords[o] (int64 [nnz_out, 3], the non-zero coordinates of the OUTPUT layout, shape (B, R, C));
 * `packed` is an int64 table over the output layout that names the source block of every position (-1 or
 * out of [0, nnz_in): the output block becomes zeros).  With the packed indices of a layout arranged in
 * transposed order this is the reference's transpose: x.transpose(-1, -2) followed by flow_pull_kernel,
 * blksprs/ops/transpose.py:44-52, blksprs/ops/flow.py:11-111.  elem_size in {1, 2, 4, 8}.
 */
int bsa_transpose_blocks(const void *blocks, const int64_t *coords, const int64_t *packed, void *out,
                         int64_t nnz_out, int64_t nnz_in, int64_t B, int64_t R, int64_t C, int sbs, int elem_size,
                         bsa_stream_t stream);

/*
 * Sparsity layout of a dense (B, R * sbs, C * sbs) array: layout[b][r][c] = 1 where the block holds an
 * element != 0 (NaN counts, -0.0 does not).  `layout` (B * R * C bytes) must be zero on entry: the kernel
 * only stores ones.  elem_size in {1, 2, 4, 8}; is_float says whether the elements are IEEE floating
 * point (fp16 / bf16 / fp32 / fp64), whose sign bit does not make a value non-zero.
 * Replaces build_sparsity_layout_kernel, blksprs/layouting/sparsity_layout.py:41-109.
 */
int bsa_layout_from_dense(const void *dense, uint8_t *layout, int64_t B, int64_t R, int64_t C, int sbs,
                          int elem_size, int is_float, bsa_stream_t stream);

/* ------------------------------------------------------------- attention */

/*
 * Arguments of the block-sparse flash-attention kernels.  Layout shapes:
 * q/o (B, nq, nh) resp. (B, nq, nhv); k (B, nk, nh); v (B, nk, nhv); the
 * attention layout, mask and bias layouts (B, nq, nk).  pidx_* are int64
 * reverse indices of those layouts (-1 = inactive); NULL mask/bias = absent;
 * NULL causal_lengths = no native causal predicate.  lse and delta are fp32
 * (B, nq, sbs); lse is in the log2 domain.
 */
typedef struct bsa_attn_args {
  const void *q, *k, *v;
  void *o;            /* forward: output blocks (dtype); backward: the saved output */
  const void *d_o;    /* backward: gradient of o */
  void *dq, *dk, *dv; /* backward outputs (dtype) */
  float *lse;         /* forward output / backward input */
  float *delta;       /* backward scratch: rowsum(o * d_o) */
  const void *mask;   /* compressed mask blocks, one byte per element: 1 = masked, 0 = kept */
  const void *bias;   /* compressed bias blocks (dtype) */
  float *dbias;       /* backward: fp32 (n_bias_blocks, sbs, sbs) or NULL */
  const int64_t *pidx_q, *pidx_k, *pidx_v, *pidx_o, *pidx_mask, *pidx_bias;
  const int32_t *key_offsets, *key_indices;     /* CSR of the attention layout rows */
  const int32_t *query_offsets, *query_indices; /* CSR of its transpose */
  const int64_t *causal_lengths;                /* int64 [B] or NULL */
  int64_t B, nq, nk, nh, nhv;
  int64_t n_q_blocks, n_k_blocks, n_v_blocks, n_o_blocks, n_mask_blocks, n_bias_blocks;
  int32_t sbs;
  int32_t dtype;     /* BSA_F32 / BSA_F16 / BSA_BF16 */
  int32_t mask_kind; /* 0 = none, 1 = one byte per element (0 or 1) */
  float scale;
  /* Optional, forward only (group_size 0: not used, the generic kernels run): the attention layout as lists
   * over groups of group_size (1 or 2) neighbouring query blocks.  group_offsets has
   * B * ceil(nq / group_size) + 1 entries; group_records holds BSA_ATTN_RECORD_INTS int32 per list entry, filled
   * by bsa_attn_fwd_records.  With group_size 2 one workgroup fetches a K / V block once for both query blocks
   * of a pair.  No counterpart in the reference. */
  const int32_t *group_offsets, *group_records;
  int32_t group_size;
  /* Backward only.  Scratch of bsa_attn_bwd_scratch_bytes(...) bytes in which bsa_attn_bwd first writes, per query
   * block and per key block, one record for every pair that some score survives (a pair whose mask block masks
   * everything, or that the causal predicate rules out as a whole, adds nothing to any gradient and is then
   * neither fetched nor computed); the matrix-core kernels walk those records.  NULL: the generic kernels run.
   * n_layout_blocks = number of active blocks of the attention layout (= key_offsets[B * nq]).
   * No counterpart in the reference, which visits every pair (blksprs/ops/flash_attention.py:1322-1330). */
  void *bwd_scratch;
  int64_t n_layout_blocks;
  /* Non-zero: bwd_scratch still holds what an earlier bsa_attn_bwd call wrote for the same layouts, packed
   * indices, head counts, mask values and causal lengths (the records depend on nothing else), and the call
   * reads it without writing it again.  Either way every call writes 64 bytes of the scratch (the tickets by
   * which its dK / dV kernel hands key rows to the workgroups that stay for the launch), so two calls that
   * overlap in time (different streams) need a scratch each. */
  int64_t bwd_scratch_ready;
  /* Size of bwd_scratch in bytes (checked against bsa_attn_bwd_scratch_bytes(...)), or 0 for "large enough". */
  int64_t bwd_scratch_bytes;
  /* Optional room for dS, bsa_attn_bwd_ds_bytes(...) bytes (16-byte aligned), used by the 16-bit kernels for 64 x 64
   * blocks only: the dK / dV kernel then leaves dS of every visited pair there (one 64 x 64 block of the operand
   * type per active block of the attention layout) and dQ = dS K is a product of its own.  NULL or fewer bytes: the
   * dQ kernel forms the scores and dS of its pairs a second time, as the reference does
   * (blksprs/ops/flash_attention.py:1228-1480); keeping dS trades memory for a third of the backward's matrix-core
   * work.  Nothing in it is read after the call returns its work to the stream: it carries nothing from one call
   * to the next and may be handed to other work that follows on the same stream. */
  void *bwd_ds;
  int64_t bwd_ds_bytes;
} bsa_attn_args;

#define BSA_ATTN_RECORD_INTS 16

/*
 * Expands grouped list entries into the records bsa_attn_fwd walks (layout-to-LUT step, integer only).  Reads
 * from args: B, nq, nk, nh (<= 2), nhv (<= 2), pidx_k, pidx_v, pidx_mask / pidx_bias (NULL: none),
 * group_offsets, group_size.  group_entries[e] = key_block | active_for_first << 28 | active_for_second << 29,
 * key blocks ascending within a group (the union of the key lists of the group's query blocks, in the order
 * of _build_segmented_indices, blksprs/ops/flash_attention.py:1923-1950).  records receives
 * BSA_ATTN_RECORD_INTS int32 per entry.  No counterpart in the reference: it resolves the packed indices
 * there inside the kernel loop (blksprs/ops/flash_attention.py:1058-1175).
 */
int bsa_attn_fwd_records(const bsa_attn_args *args, const int32_t *group_entries, int32_t *records,
                         bsa_stream_t stream);

/*
 * o = softmax(scale * q k^T + bias, masked) v over the active key blocks of
 * each query block, plus lse.  Replaces _FlashAttentionAutograd.forward /
 * flash_attention_kernel (blksprs/ops/flash_attention.py:312-503, :994-1224).
 * Every block of `o` that is active in the output layout is written.
 */
int bsa_attn_fwd(const bsa_attn_args *args, bsa_stream_t stream);

/*
 * dead[m] = 1 where block m of a compressed mask (one byte per element, 0 or 1; 64 x 64 blocks only) masks every
 * position, else 0.  A pair whose mask block is dead adds nothing to the output or to any gradient, so a caller
 * may drop it from the lists it hands to bsa_attn_fwd.  No counterpart in the reference, which visits every pair
 * (blksprs/ops/flash_attention.py:1058-1175).
 */
int bsa_attn_mask_dead(const void *mask, int64_t n_mask_blocks, int32_t sbs, uint8_t *dead, bsa_stream_t stream);

/* Size in bytes of bsa_attn_args.bwd_scratch for these sizes (16-byte aligned buffer). */
size_t bsa_attn_bwd_scratch_bytes(int64_t B, int64_t nq, int64_t nk, int64_t n_layout_blocks, int64_t n_mask_blocks);
/* Size in bytes of bsa_attn_args.bwd_ds for an attention layout of n_layout_blocks active blocks:
 * n_layout_blocks * 8192 for sbs 64, 0 for the block sizes whose kernels do not keep dS. */
size_t bsa_attn_bwd_ds_bytes(int64_t n_layout_blocks, int32_t sbs);

/*
 * dq, dk, dv (and dbias) from the saved lse.  Replaces
 * _FlashAttentionAutograd.backward and its three kernels
 * (blksprs/ops/flash_attention.py:505-787, :1228-1735).  Every block of dq, dk,
 * dv (and dbias) is written, zeros where nothing contributes.
 */
int bsa_attn_bwd(const bsa_attn_args *args, bsa_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* BLKSPRS_AMD_H */
