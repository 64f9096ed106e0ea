/*
 * plexus_hip.h -- C ABI of libplexus_hip.so: the GCN-layer hot path of Plexus as gfx950 kernels.
 *
 * The reference (hpcgroup/plexus) is pure Python and has no FFI: its hot path is a handful of
 * stock PyTorch operator calls inside two autograd functions.  Each entry point below replaces one
 * of those operator calls; the citation names the call it replaces.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless its name ends in `_host`;
 *   - matrices are row-major with an explicit leading dimension in ELEMENTS (ld >= row width);
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream); calls are
 *     stream-ordered and asynchronous, they never synchronise the device unless stated;
 *   - the return value is 0 on success or a negative plx_status; nothing throws;
 *     plx_last_error() gives a thread-local message for the last failure;
 *   - two calls allocate device memory (hipMalloc, outside any caller's allocator), both of them plan construction and
 *     both released by plx_spmm_plan_destroy: plx_spmm_plan_create (the tables of the split rows, a few counters during
 *     the call, and -- where it builds them by itself -- the tables of the hub pass) and plx_spmm_plan_build_hub (the
 *     tables of the hub pass: 5 bytes per entry of a hub row, reported by plx_spmm_plan_info(plan, 8)).  No other call
 *     allocates: scratch comes from the caller, sized by the matching *_workspace_bytes query;
 *   - results are deterministic: no atomics, fixed summation order for given inputs and plan.
 */
#ifndef PLEXUS_HIP_H
#define PLEXUS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum plx_status {
    PLX_OK = 0,
    PLX_ERR_INVALID = -1,     /* bad argument (null pointer, negative size, ld < width, ...) */
    PLX_ERR_HIP = -2,         /* a HIP runtime call failed; see plx_last_error() */
    PLX_ERR_WORKSPACE = -3,   /* workspace missing or too small */
    PLX_ERR_UNSUPPORTED = -4, /* shape outside what the kernels cover */
    PLX_ERR_NOMEM = -5        /* host or device allocation failed */
} plx_status;

/* epilogue / prologue flags of the GEMM entry points */
#define PLX_GEMM_RELU 1u    /* C = max(C, 0) (examples/train.py:77-78 fused into the producer) */
#define PLX_GEMM_DROPOUT 2u /* after the ReLU: zero with probability p, scale the rest by 1 / (1 - p).  Understood by the
                             * entry points that take (p, seed, offset): plx_gemm_nt_bf16, plx_gemm_nn_f32_split_dropout;
                             * the others refuse it (PLX_ERR_UNSUPPORTED / PLX_ERR_INVALID) rather than ignore it */

int plx_version(void);
const char *plx_error_string(int status);
const char *plx_last_error(void);

/* ------------------------------------------------------------------------------------------
 * CSR preparation.  torch CSR tensors carry int64 crow/col indices (plexus/utils/dataloader.py:367-371
 * moves them to the device as they are); the kernels read int32.
 * ---------------------------------------------------------------------------------------- */

/* rowptr32[i] = rowptr64[i] (M+1 entries), col32[j] = col64[j] (nnz entries).  The caller has
 * checked nnz < 2^31 and K < 2^31. */
int plx_csr_narrow_i64(int64_t M, int64_t nnz, const int64_t *rowptr64, const int64_t *col64, int32_t *rowptr32,
                       int32_t *col32, void *stream);

/* CSR of the transpose, built on the device: rowptr_t[K+1], col_t[nnz], val_t[nnz]; rows in order, columns
 * ascending within a row -- entry for entry what adj_local.transpose(0, 1).to_sparse_csr() gives on the host
 * (plexus/utils/dataloader.py:368).  Stable radix sort by column plus streaming kernels; `workspace` must be
 * 256-byte aligned. */
size_t plx_csr_transpose_workspace_bytes(int64_t M, int64_t K, int64_t nnz);
int plx_csr_transpose_f32(int64_t M, int64_t K, int64_t nnz, const int32_t *rowptr, const int32_t *col, const float *val,
                          int32_t *rowptr_t, int32_t *col_t, float *val_t, void *workspace, size_t workspace_bytes, void *stream);

/* A rank's CSR block from an edge list, on the device: keep the edges with r0 <= row < r1 and c0 <= col < c1,
 * re-base them to the block, sort by (row, col) and add the weights of duplicate edges -- the sequence
 * mask / re-base / sparse_coo_tensor / to_sparse_csr of plexus/utils/dataloader.py:343-367 (and
 * benchmarking/spmm.py:67-84).  rowptr has r1 - r0 + 1 entries; col_out / val_out need room for n_edges entries;
 * the number of stored entries is returned in *nnz_host (the call synchronises `stream` twice to learn it).
 * Duplicates of an edge are added one after the other in their input order. */
size_t plx_coo_block_to_csr_workspace_bytes(int64_t n_edges, int64_t block_rows, int64_t block_cols);
int plx_coo_block_to_csr_f32(int64_t n_edges, const int64_t *row, const int64_t *col, const float *weight, int64_t r0, int64_t r1,
                             int64_t c0, int64_t c1, int32_t *rowptr, int32_t *col_out, float *val_out, int64_t *nnz_host,
                             void *workspace, size_t workspace_bytes, void *stream);

/* Graph preprocessing on the device (plexus/utils/dataset.py:128-243).  The reference permutes the adjacency
 * matrix with sparse products P.A.P2^T, P[i, perm[i]] = 1 (:137-190), i.e. new[i, j] = old[perm[i], perm2[j]]:
 * an edge (r, c) moves to (inv_perm[r], inv_perm2[c]).
 *   plx_invert_permutation_i64: inv[perm[i]] = i.
 *   plx_relabel_edges_i64: (row_out[e], col_out[e]) = (map_row[row[e]], map_col[col[e]]); an id outside
 *     [0, n_rows) / [0, n_cols) gives -1, which plx_coo_block_to_csr_f32 then drops.  Outputs may alias inputs.
 *   plx_csr_to_coo_i64: the edge list (row, col) of a CSR matrix in storage order, int64 as torch edge lists
 *     are -- the to_edge_index step of :195-199. */
int plx_invert_permutation_i64(int64_t n, const int64_t *perm, int64_t *inv, void *stream);
int plx_relabel_edges_i64(int64_t n_edges, const int64_t *row, const int64_t *col, const int64_t *map_row, int64_t n_rows,
                          const int64_t *map_col, int64_t n_cols, int64_t *row_out, int64_t *col_out, void *stream);
int plx_csr_to_coo_i64(int64_t M, int64_t nnz, const int32_t *rowptr, const int32_t *col, int64_t *row_out, int64_t *col_out,
                       void *stream);

/* The permuted adjacency from the CSR of the transpose, in one sort: with `in` an M x K matrix,
 *   out[new_col[c], i] = in[perm_rows[i], c]   for every stored entry,
 * a K x M CSR matrix, rows in order and columns ascending within a row.  Called on A^T with perm_rows = perm2 and
 * new_col = the inverse of perm it yields P.A.P2^T of plexus/utils/dataset.py:137-190 (entry (i, j) of which is
 * A[perm[i], perm2[j]]).  Whole rows of the source are walked in their new order and their column ids renumbered;
 * one stable radix sort by the renumbered id then leaves every row of the result ascending, because the walk
 * already was -- half the sorting passes of building the matrix from its relabelled edge list.  perm_rows must be
 * a permutation of [0, M) and new_col of [0, K): ids out of range, or rows that do not select exactly nnz entries,
 * give PLX_ERR_INVALID.  rowptr_out has K + 1 entries, col_out / val_out nnz; the call synchronises `stream` once. */
size_t plx_csr_permute_transposed_workspace_bytes(int64_t M, int64_t K, int64_t nnz);
int plx_csr_permute_transposed_f32(int64_t M, int64_t K, int64_t nnz, const int32_t *rowptr, const int32_t *col, const float *val,
                                   const int64_t *perm_rows, const int64_t *new_col, int32_t *rowptr_out, int32_t *col_out,
                                   float *val_out, void *workspace, size_t workspace_bytes, void *stream);

/* D^-1/2 (A + I) D^-1/2 as a CSR matrix straight from an edge list -- T.GCNNorm followed by the CSR conversion,
 * plexus/utils/dataset.py:101 and :158-160.  A vertex without a self loop gets one of weight 1, d is the weighted
 * in-degree (the sum over the edges that point at a vertex, loops included), duplicate edges are summed, and
 * edges that name a vertex outside [0, N) are dropped.  `weight` may be NULL (unit weights).  With `transposed`
 * the result is the transpose, which the reference aggregates with for directed graphs (dataset.py:166-168).
 * One stable radix sort by column and one by row order the entries; the degrees are read off between the two, so
 * neither a transpose nor a second pass over the edge list is needed.  rowptr has N + 1 entries; col_out / val_out
 * need room for n_edges + N entries; *nnz_host receives the number stored (the call synchronises `stream` once). */
size_t plx_gcn_norm_edges_workspace_bytes(int64_t n_edges, int64_t N);
int plx_gcn_norm_edges_f32(int64_t n_edges, const int64_t *row, const int64_t *col, const float *weight, int64_t N, int transposed,
                           int32_t *rowptr, int32_t *col_out, float *val_out, int64_t *nnz_host, void *workspace,
                           size_t workspace_bytes, void *stream);

/* Host-only row analysis behind plx_spmm_plan_create, exported so it can be tested without a GPU.
 * Rows longer than seg_len are split into ceil(len/seg_len) near-equal segments.  Writes at most
 * `cap_long` row ids to long_rows_host, cap_long+1 entries to seg_first_host and `cap_seg` entries to
 * seg_begin_host / seg_end_host (any of them may be NULL to only count).  n_long / n_seg receive
 * the totals. */
int plx_spmm_segments_host(int64_t M, const int32_t *rowptr_host, int32_t seg_len, int64_t *n_long, int64_t *n_seg,
                           int32_t *long_rows_host, int32_t *seg_first_host, int64_t cap_long, int32_t *seg_begin_host,
                           int32_t *seg_end_host, int64_t cap_seg);

/* ------------------------------------------------------------------------------------------
 * CSR SpMM  Y[M x D] = A[M x K] . H[K x D]
 *   replaces torch.sparse.mm(edge_index, H)      plexus/gcn_conv.py:98, :188   (AGG = A.H)
 *        and torch.sparse.mm(adj_t, grad_agg)    plexus/gcn_conv.py:265       (GRAD_H = A^T.GRAD_AGG,
 *                                                 A^T being its own CSR, dataloader.py:368)
 * ---------------------------------------------------------------------------------------- */
typedef struct plx_spmm_plan plx_spmm_plan;

/* Reads rowptr and col on the device (synchronises `stream`; two counters and the two short tables that row-range
 * products need cross to the host, nothing else), finds the rows to split and keeps their segment tables on the
 * device.  Checks once that rowptr runs from 0 to nnz without decreasing and that
 * every column index lies in [0, K) (PLX_ERR_INVALID otherwise): the SpMM itself trusts them.
 * rowptr/col are BORROWED: they must outlive the plan and keep their contents.
 * seg_len <= 0 selects the default (1024, or 4096 when rows hold 128 entries or more on average). */
int plx_spmm_plan_create(plx_spmm_plan **plan, int64_t M, int64_t K, int64_t nnz, const int32_t *rowptr,
                         const int32_t *col, int32_t seg_len, void *stream);
int plx_spmm_plan_destroy(plx_spmm_plan *plan);
/* what == 0: rows, 1: cols, 2: nnz, 3: long rows, 4: segments, 5: seg_len, 6: hub rows, 7: entries in hub rows,
 * 8: bytes of the hub pass's tables (both layouts), 9 / 10: hub rows / entries in hub rows of the wide layout */
int64_t plx_spmm_plan_info(const plx_spmm_plan *plan, int what);
/* Copies the plan's tables to host arrays (any of them may be NULL): long rows [long rows], seg_first [long rows + 1],
 * seg_begin / seg_end [segments] -- the layout of plx_spmm_segments_host.  For inspection and tests; synchronous. */
int plx_spmm_plan_tables_host(const plx_spmm_plan *plan, int32_t *long_rows_host, int32_t *seg_first_host, int32_t *seg_begin_host,
                              int32_t *seg_end_host);
/* Column slicing of H.  When the rows of H taken whole overflow the last-level cache while a 256-byte slice of every row
 * stays in it, and every row is gathered often, whole-matrix products run as passes over 256-byte column slices
 * (233 K rows, 492 entries per row, 602 fp32 columns: 31.0 -> 18.4 ms).  The choice depends on the plan, the width and
 * the element size only, and every product of a sliced shape -- whole matrix or row range, sliced in place, from a
 * line-aligned copy, or in one pass when neither is possible -- sums each element in the same order, so they agree bit
 * for bit.  mode 0: decide by that rule (the default); 1: slice whenever a row exceeds 256 bytes; -1: never. */
int plx_spmm_plan_set_slicing(plx_spmm_plan *plan, int mode);
/* The hub pass.  On a power-law graph a third of the entries sit in a few thousand rows; gathered row by row they miss
 * the cache like every other row.  A plan may carry tables that let those rows ("hub rows": the longest of the split
 * rows, cut into at most 9,216 parts of at most 16 * seg_len entries) walk the columns together, window after window of
 * 4,096 columns, one eighth of the columns per XCD, so that a row of H fetched for one of them is found in that XCD's
 * L2 by the others (2.45 M nodes, 126 M entries, 128 fp32 columns: 7.3 -> 5.7 ms).  The tables cost 5 bytes per entry
 * of a hub row.  plx_spmm_plan_create builds them by itself where it expects a gain: short rows on average (fewer
 * than 128 entries, the shapes that do not take column slices), 512-byte rows of H beyond 128 MB in total, an eighth
 * of the entries in hub rows.  plx_spmm_plan_build_hub builds them for any plan with split rows (synchronises
 * `stream`).  A product uses the pass when the tables exist, the mode allows it, the shape is not a sliced one, a row
 * of H holds at least 512 bytes in 128 columns (256 where a hub row has four or more entries per window on average), H
 * as passed spans less than 4 GiB and its base, row pitch and width are multiples of 4 elements; a row range runs the
 * whole pass if it holds a hub row.  The order of every sum is fixed by the plan: the same operands give the same bits
 * on every call and in every row range, but not the bits of a product without the pass (the two agree to fp32
 * rounding).  plx_spmm_csr_f32_static never uses it.
 * The tables are cut out of the rows by bisection, so the columns of every split row must ascend (what to_sparse_csr()
 * gives, plexus/utils/dataloader.py:367; the other products take the columns of a row in any order): on a matrix where
 * they do not, plx_spmm_plan_build_hub returns PLX_ERR_UNSUPPORTED and plx_spmm_plan_create leaves the tables out.
 * mode 0: use the pass where possible (the default), -1: never. */
int plx_spmm_plan_build_hub(plx_spmm_plan *plan, void *stream);
int plx_spmm_plan_set_hub(plx_spmm_plan *plan, int mode);
/* A second set of tables for bf16 products whose rows of H hold 512 bytes or more (256 columns: the bf16 counterpart of
 * 128 fp32 columns).  The regular tables give every wavefront 36 sums of 128 columns, so such a product runs them once
 * per 128-column tile, reading every stream, column index and value again and loading 8 bytes per lane; in this layout
 * a wavefront owns 18 sums of 256 columns (the same LDS), a hub row is cut into parts of 32 * seg_len entries, and half a
 * wavefront reads a whole 512-byte row with 16 bytes per lane (2.45 M nodes, 126 M entries, 256 bf16 columns).  Never built by
 * plx_spmm_plan_create, which does not know the storage type; costs another 5 bytes per entry of a hub row; same
 * requirements and return values as plx_spmm_plan_build_hub; used when it exists, the mode allows the pass, the width is a
 * multiple of 8 and H is 16-byte aligned with a pitch that is a multiple of 8 (other operands take the regular tables
 * by the rule above). */
int plx_spmm_plan_build_hub_wide(plx_spmm_plan *plan, void *stream);
/* The tables of the hub pass (wide == 0: the regular layout, else the wide one), for inspection and tests; synchronous.
 * plx_spmm_plan_hub_info, what == 0: hub rows, 1: slots in use, 2: entries in hub rows, 3: stored stream entries (every
 * stream padded to a multiple of 64), 4: columns per window, 5: windows, 6: windows per column range (8 ranges), 7: sums
 * per wavefront, 8: slots of the layout (256 wavefronts x sums per wavefront), 9: streams (2,048: one per wavefront and
 * range; 0 without tables).  plx_spmm_plan_hub_tables_host copies to host arrays (any of them may be NULL):
 *   hub_row [slots of the layout]: row of a slot, -1 for an unused slot; wavefront w of a range owns slots
 *     w * sums_per_wavefront ...;  rows [hub rows]; row_slot_first [hub rows + 1] and row_slots [slots in use]: the slots
 *     of a hub row, one per part, in part order;
 *   stream s = range * 256 + wavefront: stream_first [streams] its first stored entry, stream_total [streams] its
 *     entries; stream_pos / stream_run [stored]: position of an entry in the CSR arrays and its slot among the
 *     wavefront's own (padding: position 0, slot 255); stream_mark [streams x windows per range]: number of the 64-entry
 *     batch in which a window of the range begins. */
int64_t plx_spmm_plan_hub_info(const plx_spmm_plan *plan, int wide, int what);
int plx_spmm_plan_hub_tables_host(const plx_spmm_plan *plan, int wide, int32_t *hub_row_host, int32_t *rows_host, int32_t *row_slot_first_host,
                                  int32_t *row_slots_host, int64_t *stream_first_host, int32_t *stream_total_host, int32_t *stream_pos_host,
                                  uint8_t *stream_run_host, int32_t *stream_mark_host);
/* bytes of scratch an fp32 SpMM of width D needs (plx_spmm_workspace_bytes_bf16: a bf16 one -- the hub pass, the column
 * slices and the copy below go by the bytes of a row, so the two types differ, and a product given less than its own
 * query asks for returns PLX_ERR_WORKSPACE): fp32 partial sums of the split rows, the partial sums
 * of the hub pass where the plan has one and the width takes it, plus -- when rows of D fp32
 * elements laid end to end straddle more 128-byte lines than they have to and every row of H is gathered often
 * enough to repay a copy -- room for a copy of H in rows that start on lines, which whole-matrix products then
 * gather from (0.2 ms of copying against 3 ms saved at K = 232,965, D = 602, 492 gathers per row).  0 if neither
 * applies; for a sliced shape (above) whose contiguous rows do not start on 128-byte lines, room for that copy as well.
 * The result does not depend on whether the copy is used. */
size_t plx_spmm_workspace_bytes(const plx_spmm_plan *plan, int64_t D);
size_t plx_spmm_workspace_bytes_bf16(const plx_spmm_plan *plan, int64_t D);

/* fp32 values, fp32 H and Y. */
int plx_spmm_csr_f32(const plx_spmm_plan *plan, const float *val, const float *H, int64_t ldh, int64_t D, float *Y,
                     int64_t ldy, void *workspace, size_t workspace_bytes, void *stream);
/* Rows [row_begin, row_end) of the same product: only those rows of Y (the base of the full M x D output) are
 * written.  The row-chunked aggregation of plexus/gcn_conv.py:67-128 (extract_csr_submatrix + SpMM per chunk +
 * torch.cat) without building sub-matrices; a caller can hand each finished chunk on (e.g. to a collective on
 * another stream) while the next one runs.  Chunks of one plan may run concurrently: their scratch rows in
 * `workspace` are disjoint. */
int plx_spmm_csr_rows_f32(const plx_spmm_plan *plan, int64_t row_begin, int64_t row_end, const float *val, const float *H,
                          int64_t ldh, int64_t D, float *Y, int64_t ldy, void *workspace, size_t workspace_bytes,
                          void *stream);
/* A product computed chunk by chunk in stream order, as the blocked aggregation of plexus/gcn_conv.py:67-128 does: the calls
 * share plan, val, H, D and workspace and differ in their row range; `first_chunk` != 0 on the first of them.  Same rows,
 * same bits as plx_spmm_csr_rows_f32, but what the chunks have in common is computed once: where the plan has a hub
 * pass, the first chunk runs it for every hub row and leaves its partial sums in the workspace, and the later chunks
 * only add up the hub rows of their range (plx_spmm_csr_rows_f32 runs the whole pass in every range that holds a hub
 * row: three times on a 2.45 M-row matrix in chunks of a million rows).  A later chunk must therefore follow the first
 * in stream order and find the workspace as the first left it; chunks after the first may still overlap each other. */
int plx_spmm_csr_chunk_f32(const plx_spmm_plan *plan, int64_t row_begin, int64_t row_end, int first_chunk, const float *val, const float *H,
                           int64_t ldh, int64_t D, float *Y, int64_t ldy, void *workspace, size_t workspace_bytes, void *stream);
/* The whole-matrix fp32 product for callers that CANNOT ALLOCATE device memory or bring a workspace (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * The row kernel of plx_spmm_csr_f32 with the same bits, but the partial sums of the split rows live in a static device
 * array of PLX_SPMM_STATIC_SCRATCH_BYTES (32 MiB, held by every GPU the library runs on until the process ends),
 * H is never copied into line-aligned rows and the hub pass is never taken (its partial sums would not fit): on a plan
 * with hub tables the result is that of plx_spmm_csr_f32 with the pass switched off, bit for bit.  The call allocates nothing; the array's device address is looked up on
 * the first call on each device (make that call outside a capture).  A plan whose split rows need more than the
 * array holds -- segments x ceil(D / 4) x 16 bytes -- is refused with PLX_ERR_WORKSPACE.  All calls on one GPU share
 * the array: calls that may overlap there (different streams or host threads) race, so order them. */
#define PLX_SPMM_STATIC_SCRATCH_BYTES (32u << 20)
size_t plx_spmm_static_scratch_bytes(void);
int plx_spmm_csr_f32_static(const plx_spmm_plan *plan, const float *val, const float *H, int64_t ldh, int64_t D, float *Y,
                            int64_t ldy, void *stream);
/* fp32 values, bf16 H and Y (raw uint16 bit patterns), fp32 accumulation, round-to-nearest-even store. */
int plx_spmm_csr_bf16(const plx_spmm_plan *plan, const float *val, const uint16_t *H, int64_t ldh, int64_t D,
                      uint16_t *Y, int64_t ldy, void *workspace, size_t workspace_bytes, void *stream);
/* rows [row_begin, row_end) of the bf16 product, as plx_spmm_csr_rows_f32 (plexus/gcn_conv.py:67-128) */
int plx_spmm_csr_rows_bf16(const plx_spmm_plan *plan, int64_t row_begin, int64_t row_end, const float *val, const uint16_t *H,
                           int64_t ldh, int64_t D, uint16_t *Y, int64_t ldy, void *workspace, size_t workspace_bytes,
                           void *stream);
/* chunk of a bf16 product computed chunk by chunk, as plx_spmm_csr_chunk_f32 */
int plx_spmm_csr_chunk_bf16(const plx_spmm_plan *plan, int64_t row_begin, int64_t row_end, int first_chunk, const float *val,
                            const uint16_t *H, int64_t ldh, int64_t D, uint16_t *Y, int64_t ldy, void *workspace, size_t workspace_bytes,
                            void *stream);

/* ------------------------------------------------------------------------------------------
 * Dense products of the layer (all replace tuned_matmul -> torch.mm, plexus/utils/matmul_tuning.py:94-95)
 * ---------------------------------------------------------------------------------------- */

/* C[M x N] = A[M x K] . B[K x N]               OUT = AGG . W         plexus/gcn_conv.py:211 */
int plx_gemm_nn_f32(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B, int64_t ldb,
                    float *C, int64_t ldc, unsigned flags, void *stream);

/* C[M x N] = (A ⊙ [mask > 0])[M x K] . B[N x K]^T   GRAD_AGG = GRAD_OUT . W^T   plexus/gcn_conv.py:256-258
 * mask (same shape and ld as A) may be NULL; when given, A is multiplied elementwise by (mask > 0)
 * on the way in -- the ReLU backward of examples/train.py:77-78 fused into the consumer. */
int plx_gemm_nt_f32(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B, int64_t ldb,
                    float *C, int64_t ldc, const float *mask, int64_t ldmask, void *stream);

/* The same two products on the bf16 matrix cores with fp32-level accuracy: every fp32 operand is split exactly
 * into three bf16 pieces and six piece products are accumulated in fp32 (the terms left out are below the
 * rounding of an fp32 product), which costs 2.7 times less matrix-core time than the fp32 MFMA and leaves the
 * products bound by HBM.  Same arguments and meaning as plx_gemm_nn_f32 / plx_gemm_nt_f32 (same reference call
 * sites) plus a workspace of plx_gemm_f32_split_workspace_bytes(N, K) bytes (16-byte aligned) for the pieces of
 * B.  Requires K > 0; for N or K above 128 also an even K and A (and mask) 8-byte aligned with even leading
 * dimensions -- 128-bit loads when all of these are multiples of 4 elements / 16 bytes, pairs of 64-bit loads
 * otherwise (PLX_ERR_INVALID for odd shapes -- the caller then uses the entry points above).
 * Inf, NaN and finite values of 3.3895e38 or more (whose bf16 rounding overflows) behave as in the fp32 kernels
 * above: an operand that holds one raises a flag on the device and the product is redone by the fp32 MFMA kernel (a
 * launch that is always enqueued and returns at once otherwise). */
size_t plx_gemm_f32_split_workspace_bytes(int64_t N, int64_t K);
int plx_gemm_nn_f32_split(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B, int64_t ldb, float *C,
                          int64_t ldc, unsigned flags, void *workspace, size_t workspace_bytes, void *stream);
int plx_gemm_nt_f32_split(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B, int64_t ldb, float *C,
                          int64_t ldc, const float *mask, int64_t ldmask, void *workspace, size_t workspace_bytes, void *stream);

/* The ReLU mask as one bit per element.  plx_gemm_nn_f32_split_bits is plx_gemm_nn_f32_split that also writes the sign
 * bits of C: bit c % 32 of word sign_bits[row * ldw + c / 32] is set when C[row][c] > 0 (ldw >= ceil(N / 32) words; bits
 * of columns past N are 0).  plx_gemm_nt_f32_split_bits is plx_gemm_nt_f32_split that reads the mask of A in that form
 * (`mask_bits`, ldw >= ceil(K / 32)) where its kernel can -- weights of at most 128 x 128, A read with 128-bit loads --
 * and the fp32 `mask`, which must say the same, elsewhere and in the guarded fp32 launch: GRAD_AGG = (GRAD_OUT ⊙ mask) . W^T
 * of a hidden layer then reads 1/32 of the mask's bytes (2,449,029 x 128: 0.76 -> 0.55 ms).  Same results bit for bit.
 * plx_sign_bits_f32 writes the bits of any matrix.   examples/train.py:77-78 (F.relu between the layers) */
int plx_gemm_nn_f32_split_bits(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B, int64_t ldb, float *C,
                               int64_t ldc, unsigned flags, uint32_t *sign_bits, int64_t ldw, void *workspace, size_t workspace_bytes,
                               void *stream);
int plx_gemm_nt_f32_split_bits(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B, int64_t ldb, float *C,
                               int64_t ldc, const float *mask, int64_t ldmask, const uint32_t *mask_bits, int64_t ldw, void *workspace,
                               size_t workspace_bytes, void *stream);
int plx_sign_bits_f32(int64_t M, int64_t N, const float *X, int64_t ldx, uint32_t *sign_bits, int64_t ldw, void *stream);

/* Dropout for fp32 storage, fused after the ReLU of the forward product (examples/train.py:77-78 is where a model puts it;
 * the reference's Net has none, this follows plx_gemm_nt_bf16).  The mask is the one defined there: element e (row-major
 * linear index row * N + col) is kept iff 16-bit lane e % 8 of Philox-4x32-10(counter = (e / 8, offset), key = seed) is
 * >= round(p * 65536), and a kept element is scaled by 1 / (1 - p) -- a host regenerates it from (seed, offset, p).
 *   plx_gemm_nn_f32_split_dropout: plx_gemm_nn_f32_split_bits with PLX_GEMM_DROPOUT honoured: C = dropout(relu(A . B))
 *     and, if sign_bits is not NULL, the bits of that C (zero where the ReLU or the dropout zeroed it: the mask the
 *     backward products need).  For weights of at most 128 x 128 and N a multiple of 8 the product's kernel applies the
 *     mask to its accumulators (one call of the generator per 8 elements); other shapes take a pass over C.
 *   plx_gemm_nt_f32_split_scaled: plx_gemm_nt_f32_split_bits (mask_bits may be NULL) times alpha, the 1 / (1 - p) of the
 *     backward pass: GRAD_AGG = alpha * (GRAD_OUT (.) mask) . W^T; alpha multiplies the weight before it is split, so
 *     alpha = 1 gives the bits of the unscaled entry point and a power of two scales them exactly.
 *   plx_dropout_f32: the same mask applied in place to any fp32 matrix (after plx_gemm_nn_f32 for operands the split
 *     products do not take). */
int plx_gemm_nn_f32_split_dropout(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B, int64_t ldb, float *C,
                                  int64_t ldc, unsigned flags, float dropout_p, uint64_t seed, uint64_t offset, uint32_t *sign_bits,
                                  int64_t ldw, void *workspace, size_t workspace_bytes, void *stream);
int plx_gemm_nt_f32_split_scaled(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B, int64_t ldb, float *C,
                                 int64_t ldc, const float *mask, int64_t ldmask, const uint32_t *mask_bits, int64_t ldw, float alpha,
                                 void *workspace, size_t workspace_bytes, void *stream);
int plx_dropout_f32(int64_t M, int64_t N, float *X, int64_t ldx, float dropout_p, uint64_t seed, uint64_t offset, void *stream);

/* C[K x N] = A[M x K]^T . (B ⊙ [mask > 0])[M x N]   GRAD_W = AGG^T . GRAD_OUT   plexus/gcn_conv.py:237-239
 * The reduction over M is split over workgroups; partial tiles go to `workspace` and are summed
 * in a fixed order. */
size_t plx_gemm_tn_workspace_bytes(int64_t M, int64_t N, int64_t K);
int plx_gemm_tn_f32(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B, int64_t ldb,
                    float *C, int64_t ldc, const float *mask, int64_t ldmask, void *workspace,
                    size_t workspace_bytes, void *stream);

/* GRAD_W on the bf16 matrix cores with fp32-level accuracy, as the two split products above: both operands are split
 * into three exact bf16 pieces on their way into LDS (transposed there, since the contraction runs over their rows), six
 * piece products per block are accumulated in fp32, the rows are cut into one stretch per compute unit whose partial
 * tiles are added in a fixed order in fp64, and the result is multiplied by alpha (1 / (1 - p) after a dropout layer).
 * `mask_bits` (may be NULL; ldw >= ceil(N / 32)) is the mask of B as one bit per element, as plx_gemm_nn_f32_split_bits
 * writes it; the fp32 `mask`, which must say the same, is read where no bits are given and by the fp32 MFMA launch
 * that redoes the product when an operand holds Inf, NaN or a value next to FLT_MAX (always enqueued, returns at once
 * otherwise).  Any alignment: the split kernel takes operands that are 16-byte aligned with leading dimensions, K and N
 * multiples of 4, and also an unmasked B of at most 64 columns in rows of any alignment beside such an A (the 47-wide gradient
 * of a last layer, read element by element); every other shape goes to the fp32 MFMA kernel of plx_gemm_tn_f32.  Same
 * reference call site: plexus/gcn_conv.py:237-239. */
size_t plx_gemm_tn_f32_split_workspace_bytes(int64_t M, int64_t N, int64_t K);
int plx_gemm_tn_f32_split(int64_t M, int64_t N, int64_t K, const float *A, int64_t lda, const float *B, int64_t ldb, float *C, int64_t ldc,
                          const float *mask, int64_t ldmask, const uint32_t *mask_bits, int64_t ldw, float alpha, void *workspace,
                          size_t workspace_bytes, void *stream);

/* ---- bf16 storage, fp32 accumulation (raw uint16 bit patterns; the reference has no reduced-precision
 *      path, these follow the same call sites as the fp32 entry points above) ----
 *
 * C[M x N] = epilogue(alpha * (A ⊙ [mask > 0])[M x K] . B[N x K]^T), C bf16.
 *   forward  OUT = AGG . W: pass B = W^T stored [N_out x K_in] (plx_cast_f32_bf16 with transpose = 1 makes it
 *   from the fp32 weight), flags PLX_GEMM_RELU and/or PLX_GEMM_DROPOUT;
 *   backward GRAD_AGG = GRAD_OUT . W^T: pass B = W stored [K_in x N_out], mask = the layer's output,
 *   alpha = 1 / (1 - p) when the forward applied dropout.
 * Dropout is counter-based so that a host can regenerate the mask: element e (row-major linear index
 * r * N + c) is kept iff 16-bit lane (e % 8) of Philox-4x32-10(counter = (e / 8, offset), key = seed) is
 * >= round(p * 65536); lane i is the low (i even) or high (i odd) half of output word i / 2. */
int plx_gemm_nt_bf16(int64_t M, int64_t N, int64_t K, const uint16_t *A, int64_t lda, const uint16_t *B, int64_t ldb,
                     uint16_t *C, int64_t ldc, const uint16_t *mask, int64_t ldmask, float alpha, unsigned flags,
                     float dropout_p, uint64_t seed, uint64_t offset, void *stream);

/* C[K x N] (fp32) = alpha * A[M x K]^T . (B ⊙ [mask > 0])[M x N]      GRAD_W = AGG^T . GRAD_OUT
 * For K and N up to 256 with more than one 128 x 128 tile, and for an unmasked B of at most 64 columns in rows that take no
 * 16-byte loads, one workgroup per stretch of rows holds the whole tile of C and every operand is read once. */
size_t plx_gemm_tn_bf16_workspace_bytes(int64_t M, int64_t N, int64_t K);
int plx_gemm_tn_bf16(int64_t M, int64_t N, int64_t K, const uint16_t *A, int64_t lda, const uint16_t *B, int64_t ldb,
                     float *C, int64_t ldc, const uint16_t *mask, int64_t ldmask, float alpha, void *workspace,
                     size_t workspace_bytes, void *stream);

/* The mask of a bf16 hidden layer as one bit per element, as for fp32 storage above (bit c % 32 of word
 * [row * ldw + c / 32] says that element (row, c) is positive; examples/train.py:77-78 is the ReLU it stands for).
 *   plx_gemm_nt_bf16_bits: plx_gemm_nt_bf16 that also writes the bits of its result C (after ReLU and dropout) to
 *     `relu_bits` (may be NULL; ldw_out >= ceil(N / 32)) -- for N, K <= 256 with N a multiple of 8 and 16-byte rows of C,
 *     PLX_ERR_UNSUPPORTED otherwise -- and reads the mask of A from `mask_bits` (may be NULL; ldw >= ceil(K / 32)) where
 *     it can: N, K <= 256, A in 16-byte rows with K a multiple of 8, rows of bits 16-byte aligned with ldw a multiple
 *     of 4 and at least 4 (K <= 128) or 8 words.  The bf16 `mask`, which must say the same, is read elsewhere.
 *   plx_gemm_tn_bf16_bits: plx_gemm_tn_bf16 reading the mask of B from `mask_bits` (ldw >= ceil(N / 32)) in the kernel
 *     that holds a whole tile of up to 256 x 256 (16-byte rows, K and N multiples of 8, more than one 128 x 128 tile),
 *     from `mask` elsewhere.
 * A hidden layer of 2,449,029 x 256 then reads 78 MB of mask in each backward product in place of 1.25 GB.  Same
 * results bit for bit as with the bf16 mask.   Reference call sites as plx_gemm_nt_bf16 / plx_gemm_tn_bf16. */
int plx_gemm_nt_bf16_bits(int64_t M, int64_t N, int64_t K, const uint16_t *A, int64_t lda, const uint16_t *B, int64_t ldb,
                          uint16_t *C, int64_t ldc, const uint16_t *mask, int64_t ldmask, const uint32_t *mask_bits, int64_t ldw,
                          uint32_t *relu_bits, int64_t ldw_out, float alpha, unsigned flags, float dropout_p, uint64_t seed,
                          uint64_t offset, void *stream);
int plx_gemm_tn_bf16_bits(int64_t M, int64_t N, int64_t K, const uint16_t *A, int64_t lda, const uint16_t *B, int64_t ldb,
                          float *C, int64_t ldc, const uint16_t *mask, int64_t ldmask, const uint32_t *mask_bits, int64_t ldw,
                          float alpha, void *workspace, size_t workspace_bytes, void *stream);

/* Y = bf16(X) (transpose = 0, Y is [M x N]) or bf16(X^T) (transpose = 1, Y is [N x M]); X is [M x N] fp32. */
int plx_cast_f32_bf16(int64_t M, int64_t N, const float *X, int64_t ldx, uint16_t *Y, int64_t ldy, int transpose,
                      void *stream);

/* Copies M rows of row_bytes bytes from one row pitch to another (fp32 or bf16 matrices whose rows are padded
 * differently; everything a multiple of 2 bytes).  Used where a narrow matrix is padded to 16-byte rows for the SpMM
 * of a layer that transforms before it aggregates; it has no counterpart in the reference. */
int plx_copy_rows(int64_t M, int64_t row_bytes, const void *src, int64_t src_pitch_bytes, void *dst, int64_t dst_pitch_bytes,
                  void *stream);

/* Y = max(X, 0) and dX = dY ⊙ [Y > 0] for callers that keep F.relu outside the layer
 * (examples/train.py:77-78).  Outputs may alias inputs. */
int plx_relu_f32(int64_t M, int64_t N, const float *X, int64_t ldx, float *Y, int64_t ldy, void *stream);
int plx_relu_bwd_f32(int64_t M, int64_t N, const float *dY, int64_t lddy, const float *Y, int64_t ldy, float *dX,
                     int64_t lddx, void *stream);

/* ------------------------------------------------------------------------------------------
 * Row-softmax cross-entropy, forward and gradient in one pass
 *   replaces the operator chain of TensorParallelCrossEntropy.forward/backward,
 *   plexus/cross_entropy.py:35-101 and :111-114, at one rank.
 *
 *   classes c >= num_classes have probability 0; rows with (row_offset + i) >= num_nodes or
 *   label < 0 have a zero softmax row; labels outside [0, C) give a zero one-hot row;
 *   loss = sum_i -log(max(p[i, label_i], 1e-9)) / num_nodes;
 *   dlogits = (softmax - onehot) / num_nodes * gscale.
 * Inputs are NOT modified (the reference overwrites padded logits and labels in place).
 * loss receives one float.  dlogits may alias logits.
 * ---------------------------------------------------------------------------------------- */
size_t plx_softmax_xent_workspace_bytes(int64_t M, int64_t C);
int plx_softmax_xent_f32(int64_t M, int64_t C, const float *logits, int64_t ld, const int64_t *labels,
                         int64_t num_nodes, int64_t num_classes, int64_t row_offset, float gscale, float *loss,
                         float *dlogits, int64_t ldd, void *workspace, size_t workspace_bytes, void *stream);
/* y[i] = x[i] * (*scale) over a contiguous tensor, `scale` being one float ON THE DEVICE: the multiplication by the
 * upstream gradient in TensorParallelCrossEntropy.backward (plexus/cross_entropy.py:114), whose scalar autograd
 * delivers as a device tensor -- reading it in the kernel keeps the host from waiting.  y may alias x.
 * The bf16 variant takes raw bit patterns and rounds to nearest even. */
int plx_scale_by_device_scalar_f32(int64_t n, const float *x, const float *scale, float *y, void *stream);
int plx_scale_by_device_scalar_bf16(int64_t n, const uint16_t *x, const float *scale, uint16_t *y, void *stream);
/* bf16 logits and gradient, fp32 math and fp32 loss */
int plx_softmax_xent_bf16(int64_t M, int64_t C, const uint16_t *logits, int64_t ld, const int64_t *labels,
                          int64_t num_nodes, int64_t num_classes, int64_t row_offset, float gscale, float *loss,
                          uint16_t *dlogits, int64_t ldd, void *workspace, size_t workspace_bytes, void *stream);

/* ------------------------------------------------------------------------------------------
 * Symmetric GCN normalisation of a CSR matrix that already holds its self loops
 *   val_out[j] = val_in[j] / sqrt(d[row(j)] d[col[j]]),  d[i] = sum of row i of val_in
 *   (the device-side counterpart of T.GCNNorm, plexus/utils/dataset.py:101).
 * dinv is scratch of M floats.  Requires a square matrix.  val_out may alias val_in.
 * ---------------------------------------------------------------------------------------- */
int plx_gcn_norm_csr_f32(int64_t M, const int32_t *rowptr, const int32_t *col, const float *val_in, float *val_out,
                         float *dinv, void *stream);

/* ------------------------------------------------------------------------------------------
 * AdamW step over one flat fp32 tensor, in one pass
 *   replaces optimizer.step() of torch.optim.AdamW(lr, weight_decay) over the weights and the input
 *   features, examples/train.py:155-159 and :110 (decoupled weight decay, bias-corrected moments,
 *   no amsgrad):
 *     p *= 1 - lr * weight_decay;  m += (g - m) (1 - beta1);  v = beta2 v + (1 - beta2) g^2;
 *     p -= lr / (1 - beta1^step) * m / (sqrt(v) / sqrt(1 - beta2^step) + eps)
 *   `step` is the 1-based count of this update.  The hyperparameters are doubles, as the Python optimizer holds
 *   them; each is rounded to fp32 where torch rounds it (1 - beta is formed in double first), so the moments and
 *   the parameters follow torch.optim.AdamW to within a few roundings of fp32.
 * ---------------------------------------------------------------------------------------- */
int plx_adamw_f32(int64_t n, float *param, const float *grad, float *exp_avg, float *exp_avg_sq, double lr, double beta1,
                  double beta2, double eps, double weight_decay, int64_t step, void *stream);
/* same update with a bf16 gradient (fp32 parameter and moments); optionally also writes bf16(param) to
 * param_bf16 (may be NULL) so that the next forward needs no separate cast pass */
int plx_adamw_f32_grad_bf16(int64_t n, float *param, const uint16_t *grad, float *exp_avg, float *exp_avg_sq, double lr,
                            double beta1, double beta2, double eps, double weight_decay, int64_t step, uint16_t *param_bf16,
                            void *stream);

#ifdef __cplusplus
}
#endif
#endif /* PLEXUS_HIP_H */
