/*
 * C ABI of the MI355X (gfx950) compressed-binary-matrix (CBM) multiply.
 *
 * Two shared libraries implement it:
 *   libcbm_host.so  -- host-only (g++/OpenMP): format construction.           [cbm_build_host ...]
 *   libcbm_hip.so   -- HIP kernels for gfx950 and their launchers.            [cbm_spmm_f32 ...]
 *
 * Conventions
 *   * plain pointers and sizes only; every `const T* dev` / `T* dev` argument of the device
 *     library is a DEVICE pointer owned by the caller; the library never allocates, frees or
 *     retains caller memory and never synchronises: work is enqueued on `stream`
 *     (a hipStream_t passed as void*, NULL = the default stream) and the call returns.
 *   * every function returns CBM_OK (0) or a CBM_ERR_* code; nothing calls exit() (the
 *     reference's helpers.hpp:58-84 does on MKL failure).
 *   * matrices X, Y, Z are row-major fp32 with a row stride `ld*` given in ELEMENTS (>= d).
 *   * index arrays are int32, as in the reference (it is built LP64: cbm/setup.py:14-16).
 *
 * Each entry point names the function of /root/reference/cbm/cbm_extensions.cpp it replaces.
 */
#ifndef CBM_HIP_H
#define CBM_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
    CBM_OK = 0,
    CBM_ERR_NULL = 1,        /* a required pointer is NULL                         */
    CBM_ERR_ALLOC = 2,       /* host allocation failed (builder only)              */
    CBM_ERR_SHAPE = 3,       /* size / stride / index out of the supported range   */
    CBM_ERR_LAUNCH = 4,      /* the HIP runtime rejected a launch                  */
    CBM_ERR_INTERNAL = 5,    /* an internal invariant failed                       */
    CBM_ERR_UNSUPPORTED = 6, /* valid request this build does not implement        */
    CBM_ERR_SCRATCH = 7      /* the shape needs more scratch than the static array of
                                cbm_spmm_update_static_f32 holds                     */
};

/* Floats of the per-device static scratch array of cbm_spmm_update_static_f32 (128 MiB).  The array is part
 * of the library's device image: every device a process uses the library on gives up this much memory from
 * the moment the library's code is loaded there, whether or not that entry point is ever called.  A build
 * that wants less (or more) defines the macro on the compiler's command line, for the library and its users
 * alike. */
#ifndef CBM_STATIC_SCRATCH_FLOATS
#define CBM_STATIC_SCRATCH_FLOATS (32 * 1024 * 1024)
#endif

/* flags of cbm_spmm_f32 / csr_spmm_f32 */
enum {
    CBM_SPMM_WORKSPACE_READY = 1, /* workspace already holds cbm_relayout_slabs_f32(X): do not copy again */
    CBM_SPMM_RELU = 2,            /* store max(z, 0) instead of z (after the left scale of root children) */
    CBM_SPMM_WORKSPACE_PRESCALED = 4, /* with WORKSPACE_READY, cbm_spmm_f32 with m only: the copy was made by
                                     cbm_relayout_slabs_scaled_f32(X, m) (or the masked variant with m) */
    CBM_SPMM_SCHED_BATCHED = 8    /* row_sched comes from cbm_schedule_rows_batched (n + 1 descriptors) */
};

/* flags of cbm_propagate_f32 */
enum {
    CBM_PROP_SCALE_ROOTS = 1  /* normalised only: first do Y[r,:] *= m[r] for children of the root */
};

/* flags of cbm_spmm_update_f32 / cbm_spmm_update_static_f32 (CBM_PROP_SCALE_ROOTS is accepted and
 * has no effect there: the SpMM epilogue scales the children of the root) */
enum {
    CBM_UPDATE_RELU = 2,            /* Y = max(A_hat X, 0): the activation of a GCN layer
                                       (benchmark/parallel/benchmark_gcn_cpu.py:84-88 applies it as a
                                       separate pass); in the SpMM epilogue when the tree is flat,
                                       one extra pass over Y otherwise */
    CBM_UPDATE_WORKSPACE_READY = 4, /* as CBM_SPMM_WORKSPACE_READY */
    CBM_UPDATE_WORKSPACE_PRESCALED = 8, /* as CBM_SPMM_WORKSPACE_PRESCALED */
    CBM_UPDATE_SCHED_BATCHED = 16   /* as CBM_SPMM_SCHED_BATCHED */
};

/* The CBM format as built on the host.  All arrays are malloc'd by cbm_build_host and are
 * released together by cbm_format_free.
 *   rowptr/idx   delta matrix in CSR form; idx = column | (negative entry ? 1u<<31 : 0),
 *                columns ascending within a row (what the reference stores as a torch sparse
 *                CSR with values +-1, cbm/cbm.py:56-58)
 *   parent       parent row in the arborescence, -1 for children of the virtual root
 *   order        rows sorted by (level, id); level 0 = children of the virtual root
 *   level_off    n_levels + 1 offsets into order[]
 *   mst_row/col  the reference's tree CSR (cbm_extensions.cpp:274-286): N+2 offsets, row N is
 *                the virtual root; N children, ascending id within a parent */
typedef struct cbm_format {
    int32_t n;
    int32_t n_levels;
    int32_t is_symmetric;   /* 1 if the input pattern equals its transpose (A_hat^T = A_hat) */
    int32_t reserved;
    int64_t nnz;            /* delta non-zeros = weight of the arborescence */
    int64_t nnz_a;          /* non-zeros of the input matrix after de-duplication */
    int64_t n_candidates;   /* edges of the distance graph, root edges included */
    int64_t msa_weight;
    int32_t* rowptr;        /* [n + 1]        */
    uint32_t* idx;          /* [nnz]          */
    int32_t* parent;        /* [n]            */
    int32_t* order;         /* [n]            */
    int32_t* level_off;     /* [n_levels + 1] */
    int32_t* mst_row;       /* [n + 2]        */
    int32_t* mst_col;       /* [n]            */
} cbm_format;

/* ------------------------------------------------------------------ libcbm_host.so ---------- */

const char* cbm_host_version(void);

/* Build the format from a COO list (row[k], col[k]) of a 0/1 N x N matrix; duplicates are merged,
 * any order.  alpha is the reference's pruning parameter: row u may serve as parent of row v only
 * if hamming(u, v) < nnz(v) - alpha.  threads <= 0 means all OpenMP threads.  HOST pointers.
 * Replaces cbm_init_v1_ (cbm_extensions.cpp:8-326) and cbm_init_v2_ (:328-644); the
 * normalisation vector of v2 is not an input: the kernels apply it. */
int cbm_build_host(const int32_t* row, const int32_t* col, int64_t n_edges, int32_t n, int32_t alpha,
                   int32_t threads, cbm_format* out);

/* The same build in stages, so that the row intersections -- the dominant cost for large graphs
 * -- can be computed elsewhere (cbm_row_intersections on the GPU) and handed back:
 *   cbm_builder_create   CSR of the input with sorted unique columns, and its transpose
 *   cbm_builder_arrays   HOST views of those arrays (valid until cbm_builder_free):
 *                          rowptr[n+1], col[nnz]           rows of A
 *                          colptr_t[n+1], row_t[nnz]       columns of A (row ids ascending)
 *                          after[nnz]                      per entry (r, c) of A: first position in
 *                                                          row_t of a row id > r inside column c
 *                          row_nnz[n]                      entries per row
 *   cbm_builder_finish   candidate edges, arborescence, deltas.  pairs = (i, j, s) with i < j and
 *                        s = |row_i ^ row_j| in any order, holding at least every pair with
 *                        2 s > min(nnz_i, nnz_j) + alpha; n_pairs < 0 computes them on the host.
 *   cbm_builder_set_max_levels   optional, before finish: no tree level beyond max_levels (0 = no
 *                        limit, the default and what the reference does).  A row that would land
 *                        deeper is re-attached to the virtual root together with its subtree:
 *                        fewer dependent launches per multiply for a few more delta entries (nnz
 *                        then exceeds msa_weight).  No reference counterpart; alpha is the
 *                        reference's only knob for the same trade (cbm_extensions.cpp:75-103).
 * cbm_build_host is create + finish(n_pairs = -1) + free.  Replaces the mkl_sparse_syrk step of
 * cbm_init_v1_/_v2_ (cbm_extensions.cpp:46-65) as a separable stage. */
typedef struct cbm_builder cbm_builder;
struct cbm_pair { int32_t i, j, s; };
int cbm_builder_create(const int32_t* row, const int32_t* col, int64_t n_edges, int32_t n, int32_t threads,
                       cbm_builder** out);
int cbm_builder_arrays(const cbm_builder* b, const int64_t** rowptr, const int32_t** col, const int64_t** colptr_t,
                       const int32_t** row_t, const int64_t** after, const int32_t** row_nnz, int64_t* nnz);
int cbm_builder_finish(cbm_builder* b, int32_t alpha, const struct cbm_pair* pairs, int64_t n_pairs,
                       struct cbm_format* out);
int cbm_builder_set_max_levels(cbm_builder* b, int32_t max_levels);
void cbm_builder_free(cbm_builder* b);

void cbm_format_free(cbm_format* f);

/* Seconds the calling thread's last cbm_build_host spent in its four phases: CSR + transpose,
 * candidate edges, arborescence, tree arrays + deltas.  (The reference times construction as a
 * whole, benchmark/parallel/cbm_creation.py:42-51.) */
void cbm_build_host_timings(double* out4);

/* Row schedule for the SpMM kernels: rows sorted by descending number of 64-entry gather rounds
 * (stable, so rows of similar length keep their natural order), one descriptor of 4 int32 per
 * row: { rowptr[r], rowptr[r + 1], r, bit pattern of the left scale }.  The left scale is m[r]
 * for children of the root (parent[r] < 0) when m is given, 1.0f otherwise.  Long rows start
 * first and a cyclic deal of the schedule gives every wavefront the same mix of row lengths.
 * HOST pointers; sched_out holds 4 * n int32.  parent and m may be NULL (scale 1.0f).
 * No reference counterpart: MKL keeps its own scheduling inside mkl_sparse_s_mm. */
int cbm_schedule_rows(const int32_t* rowptr, const int32_t* parent, const float* m, int32_t n,
                      int32_t* sched_out);

/* cbm_schedule_rows for matrices with many SHORT rows -- the delta rows of a matrix that compresses well
 * hold a handful of entries each.  Rows of more than batch_max_entries entries (at most 64) come first, in
 * the order of cbm_schedule_rows; the others follow, sorted by descending number of 8-entry chunks (stable),
 * and the slab kernel takes them a BATCH at a time: every lane group of a wavefront (8 rows per wavefront on
 * 128-byte slabs) sums a row of its own, entries strictly in order, so that one index load and one round of
 * gathers serve 8 rows instead of one and no sum is reduced across lanes.  sched_out holds 4 * (n + 1)
 * int32: the n descriptors and a trailer { rows before the batched part, batch_max_entries,
 * CBM_SCHED_BATCH_MAGIC, 0 }; pass it with CBM_SPMM_SCHED_BATCHED (CBM_UPDATE_SCHED_BATCHED).  The fp32
 * order of a batched row is the in-order sum (as if cbm_spmm_summation_groups were 1 for that row) wherever
 * the slab kernel runs; other kernels walk the same descriptors and ignore the trailer.  HOST pointers.
 * No reference counterpart (MKL schedules rows internally). */
#define CBM_SCHED_BATCH_MAGIC 0x62617463
int cbm_schedule_rows_batched(const int32_t* rowptr, const int32_t* parent, const float* m, int32_t n,
                              int32_t batch_max_entries, int32_t* sched_out);

/* cbm_schedule_rows for matrices with very long rows (hubs of a power-law graph): a row with more
 * than `chunk` entries (chunk >= 64) is cut into pieces of `chunk` entries, each with a descriptor
 * of its own { start, end, slot | CBM_SCHED_PIECE, bits(1.0f) }, so that different wavefronts
 * gather different pieces; a piece's sum goes to slot `slot` of a scratch area instead of Z, and
 * the pieces of a row are added in order afterwards (no atomics: the result does not depend on
 * which wavefront ran which piece).  long_rows_out gets 4 int32 per cut row: { row, first slot,
 * number of pieces, bit pattern of the left scale }.  cbm_schedule_split_count returns the number
 * of descriptors (and the number of cut rows), -1 on bad input.  Used through cbm_spmm_tiled_f32.
 * HOST pointers.  No reference counterpart (MKL schedules rows internally). */
#define CBM_SCHED_PIECE 0x40000000
int64_t cbm_schedule_split_count(const int32_t* rowptr, int32_t n, int32_t chunk, int32_t* n_long_out);
int cbm_schedule_rows_split(const int32_t* rowptr, const int32_t* parent, const float* m, int32_t n, int32_t chunk,
                            int32_t* sched_out, int32_t* long_rows_out);

/* cbm_schedule_rows_split that ALSO cuts every row where its (ascending) columns pass from one
 * block of ceil(n / col_blocks) consecutive columns to the next (col_blocks >= 2; idx as in
 * cbm_format), and orders the descriptors by column block first (then longest first): all
 * wavefronts gather from the same col_blocks-th of X at about the same time, which keeps that part
 * of the slab-major copy in the XCDs' L2s -- for matrices whose rows are long (hundreds of entries)
 * and scattered over more of X than the L2s hold.  Runs longer than `chunk` are cut further
 * (chunk = 0: never; else >= 64).  A row that ends up as one piece keeps an ordinary descriptor.
 * col_blocks <= 1 is cbm_schedule_rows_split.  Same output formats; cbm_schedule_blocks_count
 * returns the number of descriptors (and of cut rows), -1 on bad input.  HOST pointers.  No
 * reference counterpart (MKL schedules rows internally). */
int64_t cbm_schedule_blocks_count(const int32_t* rowptr, const uint32_t* idx, int32_t n, int32_t chunk, int32_t col_blocks,
                                  int32_t* n_long_out);
int cbm_schedule_rows_blocks(const int32_t* rowptr, const uint32_t* idx, const int32_t* parent, const float* m, int32_t n,
                             int32_t chunk, int32_t col_blocks, int32_t* sched_out, int32_t* long_rows_out);

/* Split of a packed delta matrix (rowptr, idx as in cbm_format) into entries that cluster and the
 * rest, for cbm_spmm_tiled_f32.  Rows are cut into panels of CBM_TILING_PANEL_ROWS, columns into
 * tiles of tile_rows (1024); a (panel, tile) block that holds at least min_block_entries entries
 * becomes a "local" block, whose tile of X the kernel stages in LDS; every other entry is "remote"
 * and stays in an ordinary packed CSR.
 *   panel_ptr[n_panels + 1]   blocks of each panel (ascending tile)
 *   blk_tile[n_blocks]        tile index of each block (first row of X it covers = tile * tile_rows)
 *   seg[n_blocks][panel_rows + 1]  per block and panel row: start of the row's segment in lidx, in
 *                             units of 8 entries; a segment holds the row's entries inside the
 *                             block, padded to a multiple of 8, ordered by the class
 *                             q = (column - row) mod 4 in the order q = 0, 2, 1, 3, ascending inside a
 *                             class: the two 128-byte rows (four 64-byte rows of the half slab) the
 *                             kernel serves in one LDS cycle then read different bank halves (quarters)
 *   lidx[nnz_local_padded]    (row of X - first row of the tile) * 8 | (negative ? 1 << 15 : 0);
 *                             padding = tile_rows * 8, the all-zero row behind the tile
 *   rowptr_r / idx_r          the remote entries, packed like idx, columns ascending
 * The columns of every row must ascend strictly and lie below n (the fill takes a block's entries of
 * a row as one run): anything else is CBM_ERR_SHAPE, running out of memory CBM_ERR_ALLOC.
 * threads <= 0 means all OpenMP threads.  HOST pointers; release with cbm_tiling_free.  No reference
 * counterpart: the reference hands its delta matrix to mkl_sparse_s_mm as it is
 * (cbm_extensions.cpp:1133-1159). */
#define CBM_TILING_PANEL_ROWS 256
typedef struct cbm_tiling {
    int32_t n, tile_rows, panel_rows, n_panels, n_blocks, has_negative;
    int64_t nnz_local, nnz_local_padded, nnz_remote;
    int32_t* panel_ptr;
    int32_t* blk_tile;
    int32_t* seg;
    uint16_t* lidx;
    int32_t* rowptr_r;
    uint32_t* idx_r;
} cbm_tiling;
int cbm_tile_rows(const int32_t* rowptr, const uint32_t* idx, int32_t n, int32_t tile_rows, int64_t min_block_entries,
                  int32_t threads, cbm_tiling* out);
void cbm_tiling_free(cbm_tiling* t);

/* Plan of the tree walk by SUBTREES (cbm_propagate_subtrees_f32): the rows below level `cut` of the
 * arborescence, as one sequence per subtree in depth-first pre-order, so that ONE launch walks all of
 * them -- a wavefront per (bin of subtrees, 64 feature columns) carries a row's value down to its
 * children in registers and LDS and touches global memory only to read the row's own SpMM result and to
 * write its final value (two row accesses per tree edge instead of three, none of them dependent on the
 * previous one).  The reference's walk has the same shape -- parallel over the children of the root,
 * depth-first with a stack inside a subtree (cbm_extensions.cpp:1166-1218) -- on CPU threads.
 *   cut        rows of levels 0 .. cut are final before the launch (level 0 after the SpMM, levels 1 .. cut
 *              by the level-by-level launches); every row of level `cut` that has children heads a task
 *   entries    [n_entries][2] int32 { row, ctl }: ctl & 63 = where the parent's value is: 0 = the row just
 *              before this one, 1 .. CBM_WALK_MAX_SLOTS = that LDS slot, CBM_WALK_LOAD_ONLY = this row is a
 *              task's head: final already, only loaded; (ctl >> 8) & 63 = slot to keep this row's value in
 *              (0 = none; rows with two or more children).  Children are visited lightest subtree first,
 *              so at most log2(subtree size) + 1 slots are live at once
 *   bin_off    [n_bins + 1] offsets into entries: a bin is what one wavefront walks (whole tasks, longest
 *              first, small ones packed together up to about n_entries / target_bins entries)
 *   n_slots    most slots any task uses;  longest_bin  entries of the longest bin (the critical path)
 * HOST pointers; release with cbm_walk_plan_free.  CBM_ERR_UNSUPPORTED if a task needs more than
 * CBM_WALK_MAX_SLOTS slots (a tree of more than 2^31 rows would). */
#define CBM_WALK_LOAD_ONLY 63
#define CBM_WALK_MAX_SLOTS 31
#define CBM_WALK_MIN_BIN 32
typedef struct cbm_walk_plan {
    int32_t n, cut, n_entries, n_bins, n_slots, reserved;
    int64_t longest_bin;
    int32_t* entries;
    int32_t* bin_off;
} cbm_walk_plan;
int cbm_walk_plan_build(const int32_t* parent, const int32_t* order, const int32_t* level_off, int32_t n,
                        int32_t n_levels, int32_t cut, int32_t target_bins, cbm_walk_plan* out);
void cbm_walk_plan_free(cbm_walk_plan* p);

/* Plan of the ONE-LAUNCH multiply by subtrees (cbm_spmm_update_subtrees_f32), for deep trees whose delta rows
 * are short: the walk plan at cut 0 extended to every child of the root (also those without children), with
 * the delta entries of the rows laid end to end in walk order, so that a wavefront streams them, sums a row
 * on the spot and takes its walk step without the SpMM result ever going through memory.
 *   gidx       [n_elems] uint32: the delta entries (col | sign << 31, as idx) of a bin's rows in walk order;
 *              CBM_STREAM_LAST marks a row's last entry; an empty row has one stand-in entry with
 *              CBM_STREAM_DUMMY (| LAST) whose column is the row itself and which adds nothing; every bin is
 *              padded to a multiple of 64 entries with unmarked copies of its last entry's column (summed
 *              into an accumulator that is never stored)
 *   ginfo      [n_elems][2] int32 { row, ctl } (ctl as in cbm_walk_plan.entries; CBM_WALK_LOAD_ONLY = a child of
 *              the root: its sum, times m[row] when normalised, is its value): for every stretch of 64 stream
 *              entries of a bin, the rows that END inside that stretch, in order, starting at the stretch's
 *              first position; positions no row landed in hold { first row of the bin, 0 }
 *   bin_goff   [n_bins + 1] offsets into gidx / ginfo, multiples of 64: a bin is what one wavefront streams
 *              (whole subtrees, heaviest first, small ones packed together up to about 1 / target_bins of
 *              the total weight)
 *   n_slots    most LDS slots any subtree uses;  heaviest_bin  weight of the heaviest bin, a row weighing its
 *              stream entries + CBM_STREAM_ROW_COST (what the time of the wavefront that walks it follows; bins
 *              are packed by this weight)
 * n must be below 2^29 (the column shares its word with the sign and the two marks).  HOST pointers; release
 * with cbm_walk_stream_free.  CBM_ERR_UNSUPPORTED as for cbm_walk_plan_build.  No reference counterpart: the
 * reference keeps the SpMM (MKL) and the walk apart (cbm_extensions.cpp:1133-1218). */
#define CBM_STREAM_LAST 0x40000000u
#define CBM_STREAM_DUMMY 0x20000000u
#define CBM_STREAM_COL_MASK 0x1fffffffu
#define CBM_STREAM_MIN_BIN 64
#define CBM_STREAM_ROW_COST 5
typedef struct cbm_walk_stream {
    int32_t n, n_bins, n_slots, n_elems;
    int64_t heaviest_bin;
    uint32_t* gidx;
    int32_t* ginfo;
    int32_t* bin_goff;
} cbm_walk_stream;
int cbm_walk_stream_build(const int32_t* rowptr, const uint32_t* idx, const int32_t* parent, const int32_t* order,
                          const int32_t* level_off, int32_t n, int32_t n_levels, int32_t target_bins,
                          cbm_walk_stream* out);
void cbm_walk_stream_free(cbm_walk_stream* p);

/* ------------------------------------------------------------------ libcbm_hip.so ----------- */

const char* cbm_version(void);
const char* cbm_status_string(int status);

/* Choice of the SpMM kernel for later calls of this process: 0 = automatic (default), 1 = always
 * one wavefront per row, 2 = reserved (same as 0).  A tuning and test hook; no reference
 * counterpart. */
int cbm_set_spmm_kernel(int kind);

/* Resident wavefronts per SIMD of the slab SpMM kernel for later calls of this process: 0 =
 * automatic (default: 4 when rows average 128 entries or more and a 128-byte slab of X exceeds an
 * XCD's L2, 6 when it does not or rows average 32 or more, else all the registers allow), 1..8 =
 * fixed.  A tuning hook; no reference counterpart. */
int cbm_set_spmm_occupancy(int waves_per_simd);

/* Tiled multiply (cbm_spmm_tiled_f32) for later calls of this process: 1 (default) = when the plan
 * cuts no rows, the kernel of the local blocks also gathers the remote entries, straight from the
 * slab-major copy and strictly in entry order (one launch instead of two, no pass over Z in
 * between); 0 = the remote entries always go through the slab kernel first (8 or 16 partial sums).
 * A tuning hook; no reference counterpart. */
int cbm_set_tiled_fused(int on);

/* How many interleaved partial sums the SpMM keeps per output element for this shape (1 = the
 * entries of a row are accumulated strictly in order; g > 1 = entry k goes to partial sum
 * k mod g and the g sums are added as a balanced tree).  Lets a checker reproduce the fp32
 * summation order bit for bit.  No reference counterpart (MKL does not document its order). */
int cbm_spmm_summation_groups(int32_t d, int64_t ldx, int64_t ldz, const void* X_dev, const void* Z_dev,
                              int32_t have_workspace);

/* Trailing columns of this shape that the SpMM sums in 16 interleaved partial sums instead of the
 * number cbm_spmm_summation_groups reports: with a workspace, when the last d mod 32 columns are
 * at most 16 (and the full 128-byte slabs split evenly over the XCDs: 0, 1, 2, 4 or a multiple of
 * 8 of them), those columns are kept as a 64-byte half slab in the slab-major copy and gathered
 * with 4 lanes per entry -- a width of 41 then moves 48 floats per delta entry instead of 64.
 * 0 = no such columns.  No reference counterpart. */
int cbm_spmm_tail_columns(int32_t d, int64_t ldx, int64_t ldz, const void* X_dev, const void* Z_dev, int32_t have_workspace);

/* Floats of workspace that cbm_spmm_f32 / cbm_spmm_update_f32 / csr_spmm_f32 use for this shape when
 * given one: the size of the slab-major copy of X (n rows x 128-byte slabs, the slab count
 * rounded up for odd widths, or a 64-byte half slab for the last columns, see
 * cbm_spmm_tail_columns), or 0 where the copy would buy nothing: d = 32, 64, 128 or 256 with
 * 128-byte-aligned rows whose stride ldx is an ODD number of 128-byte lines (e.g. ldx = d + 32),
 * which spreads the lines of a slab over all L2 channels by itself.  The workspace stays
 * optional: without it, widths that are a multiple of 32 gather from the row-major X and all
 * others take one wavefront per row. */
int64_t cbm_spmm_workspace_floats(int32_t n, int32_t d, int64_t ldx, int64_t ldz, const void* X_dev, const void* Z_dev);

/* coef[k] = +-m[column of entry k] for the packed entries idx[0 .. nnz): the delta VALUES of the
 * reference's normalised builder (cbm_extensions.cpp:504-585), expanded on the device once so
 * that cbm_spmm_f32 can stream them instead of gathering m[col] per entry.  Optional. */
int cbm_expand_coef_f32(const uint32_t* idx_dev, const float* m_dev, float* coef_dev, int64_t nnz, void* stream);

/* Z = D * diag(m) * X for the packed delta matrix D (m == NULL: Z = D * X).  coef, if not NULL,
 * must be the output of cbm_expand_coef_f32 for (idx, m); the result is the same, the kernel
 * streams coef instead of gathering m.  If `parent` and `m` are both given, rows with
 * parent[r] < 0 are additionally scaled by m[r] (the first step of the normalised tree walk,
 * cbm_extensions.cpp:910-940, folded into the producer).  row_sched, if not NULL, is the row
 * schedule written by cbm_schedule_rows (4 int32 per row, 16-byte aligned): rows are then
 * processed in that order, rowptr is not read (may be NULL) and the left scale comes from it.
 * workspace, if not NULL, is caller-owned device memory of cbm_spmm_workspace_floats() floats
 * (16-byte aligned, disjoint from X and Z): X is first copied there slab-major (zero-padded to
 * whole 128-byte slabs), so that the gathered lines of a slab are consecutive in memory instead of
 * a row apart and odd widths (d = 41, 602, unaligned rows) run on the slab kernel too.  The fp32
 * summation order with and without it can differ (cbm_spmm_summation_groups reports both), and
 * with m the copy is pre-scaled (see cbm_relayout_slabs_scaled_f32): coef is then not read.  The
 * copy pays off when rows have more than a few entries.
 * nnz is the number of entries (rowptr[n]); it only sizes the launch (long rows run with fewer
 * resident wavefronts, see cbm_set_spmm_occupancy) and may be 0 if unknown.
 * Replaces the mkl_sparse_s_create_csr + mkl_sparse_s_mm pair of every *_spmm_update function
 * (cbm_extensions.cpp:678-704, :875-900, :1133-1159, :1251-1277); overwrites Z (beta = 0). */
int cbm_spmm_f32(const int32_t* rowptr_dev, const uint32_t* idx_dev, int64_t nnz, const float* m_dev,
                 const float* coef_dev, const int32_t* parent_dev, const int32_t* row_sched_dev, const float* X_dev, float* Z_dev,
                 float* workspace_dev, int32_t flags, int32_t n, int32_t d, int64_t ldx, int64_t ldz,
                 void* stream);

/* The slab-major copy of X that cbm_spmm_f32 / csr_spmm_f32 make into their workspace, as a call
 * of its own: several multiplies by different matrices with the SAME X can then share one copy
 * (pass the workspace with CBM_SPMM_WORKSPACE_READY; the multiply then reads only the copy).
 * Any width; workspace holds cbm_relayout_floats(n, d) floats. */
int cbm_relayout_slabs_f32(const float* X_dev, float* workspace_dev, int32_t n, int32_t d, int64_t ldx, void* stream);
int64_t cbm_relayout_floats(int32_t n, int32_t d);

/* The same copy with a ReLU gradient folded in: the copy holds X[r][c] where mask[r][c] > 0 and 0
 * elsewhere (mask: n x d, row stride ldm; typically the output of the forward multiply made with
 * CBM_UPDATE_RELU, X the gradient arriving at it).  The backward multiply then runs from the copy
 * with WORKSPACE_READY and never reads X.  No reference counterpart: the reference's layers have
 * no backward pass (gnns/message_passing/cbm_message_passing.py:16-60 mutate a cached output). */
int cbm_relayout_slabs_masked_f32(const float* X_dev, const float* mask_dev, const float* scale_dev /* nullable */,
                                  float* workspace_dev, int32_t n, int32_t d, int64_t ldx, int64_t ldm, void* stream);

/* The copy with row r multiplied by scale[r] (one rounded fp32 product per element).  With
 * scale = m this is what a normalised cbm_spmm_f32 makes by itself when it copies X: the right-hand
 * diagonal of diag(m) A diag(m) is applied once per row of X, and the delta entries then carry
 * only their sign (no coefficient array is streamed, coef may be NULL).  The reference applies the
 * same diagonal per delta entry as the value +-m[col] (cbm_extensions.cpp:504-585); the two
 * differ in fp32 rounding only: fma(+-m[c], x, acc) there, acc +- fl(m[c] * x) here.  A copy made
 * by this call is announced to the multiply with WORKSPACE_READY | WORKSPACE_PRESCALED.
 * cbm_relayout_slabs_masked_f32 takes the same vector (NULL = no scaling). */
int cbm_relayout_slabs_scaled_f32(const float* X_dev, const float* scale_dev, float* workspace_dev, int32_t n, int32_t d,
                                  int64_t ldx, void* stream);

/* In-place tree propagation over Y (which holds Z on entry), level by level.
 *   m == NULL : Y[v,:] += Y[parent[v],:]
 *               replaces seq_/omp_s_update_csr_int32_ and omp_s_update_avx_int32_
 *               (cbm_extensions.cpp:742-786, :1485-1610, :1612-1705) and the walk inside
 *               seq_/omp_s_spmm_update_csr_int32_ (:713-738, :1166-1218)
 *   m != NULL : Y[v,:] = fma(Y[u,:], 1/m[u], Y[v,:]) * m[v], u = parent[v]; the last d mod 8
 *               columns use (Y[v] + Y[u]/m[u]) * m[v] exactly as the reference's scalar tail;
 *               with CBM_PROP_SCALE_ROOTS, children of the root are first scaled by m[r].
 *               replaces seq_/omp_s_fused_update_csr_int32_ (:998-1105, :1376-1483) and the walk
 *               inside seq_/omp_s_fused_spmm_update_csr_int32_ (:908-995, :1285-1373)
 * level_off_host is a HOST array (launch shapes are derived from it); level_off_dev is the same
 * array in device memory (read by kernels that walk several levels in one launch). */
int cbm_propagate_f32(const int32_t* parent_dev, const int32_t* order_dev, const int32_t* level_off_dev,
                      const int32_t* level_off_host, int32_t n_levels, const float* m_dev, float* Y_dev,
                      int32_t n, int32_t d, int64_t ldy, int32_t flags, void* stream);

/* A walk plan (cbm_walk_plan_build) in DEVICE memory.  The struct itself lives in HOST memory. */
typedef struct cbm_walk_dev {
    int32_t cut, n_entries, n_bins, n_slots;
    const int32_t* entries;     /* [n_entries][2], 8-byte aligned */
    const int32_t* bin_off;     /* [n_bins + 1] */
} cbm_walk_dev;

/* cbm_propagate_f32 with the rows below level walk->cut walked by subtrees in one launch: levels
 * 1 .. cut run level by level as in cbm_propagate_f32, then one wavefront per (bin of the plan, 64 feature
 * columns) walks its subtrees depth-first.  Per row the arithmetic is that of cbm_propagate_f32, so Y is
 * bit-identical to it; what changes is the number of dependent launches (cut + 1 instead of one per tree
 * level) and the traffic (a row's parent value comes from a register or LDS, not from Y).  The plan must
 * have been built from the same parent / order / level_off.  flags: CBM_PROP_SCALE_ROOTS as in
 * cbm_propagate_f32; CBM_UPDATE_RELU = one pass Y = max(Y, 0) after the walk.
 * Replaces the same walks as cbm_propagate_f32 (cbm_extensions.cpp:1166-1218, :1285-1373), whose
 * parallelisation -- threads over the children of the root, a stack inside each subtree -- it mirrors. */
int cbm_propagate_subtrees_f32(const cbm_walk_dev* walk, const int32_t* parent_dev, const int32_t* order_dev,
                               const int32_t* level_off_dev, const int32_t* level_off_host, int32_t n_levels,
                               const float* m_dev, float* Y_dev, int32_t n, int32_t d, int64_t ldy, int32_t flags,
                               void* stream);

/* A multiply stream (cbm_walk_stream_build) in DEVICE memory.  The struct itself lives in HOST memory. */
typedef struct cbm_walk_stream_dev {
    int32_t n, n_bins, n_slots, n_elems;
    const uint32_t* gidx;       /* [n_elems] */
    const int32_t* ginfo;       /* [n_elems][2], 8-byte aligned */
    const int32_t* bin_goff;    /* [n_bins + 1] */
} cbm_walk_stream_dev;

/* Y = A_hat * X in ONE launch for a deep tree with short delta rows: one wavefront per (bin of the stream,
 * 64 feature columns) walks its subtrees depth-first and sums every row's delta entries on the spot, so the
 * SpMM result never goes to memory and back.  A row's sum runs strictly in entry order (fma(+-1 or +-m[col],
 * x, acc) from zero, the reference's per-entry arithmetic, cbm_extensions.cpp:504-585); the walk step per
 * row is that of cbm_propagate_f32.  flags: CBM_UPDATE_RELU (in the store; children still read the raw
 * value).  X must not alias Y.
 * m == NULL replaces seq_/omp_s_spmm_update_csr_int32_ (cbm_extensions.cpp:650-740, :1108-1219);
 * m != NULL replaces seq_/omp_s_fused_spmm_update_csr_int32_ (:845-996, :1224-1374). */
int cbm_spmm_update_subtrees_f32(const cbm_walk_stream_dev* stream_plan, const float* m_dev, const float* X_dev,
                                 float* Y_dev, int32_t n, int32_t d, int64_t ldx, int64_t ldy, int32_t flags,
                                 void* stream);

/* Y = A_hat * X in one call: cbm_spmm_f32 followed by cbm_propagate_f32 on the same stream.
 * m == NULL replaces seq_/omp_s_spmm_update_csr_int32_ (cbm_extensions.cpp:650-740, :1108-1219);
 * m != NULL replaces seq_/omp_s_fused_spmm_update_csr_int32_ (:845-996, :1224-1374). */
int cbm_spmm_update_f32(const int32_t* rowptr_dev, const uint32_t* idx_dev, int64_t nnz, const float* m_dev,
                        const float* coef_dev, const int32_t* parent_dev, const int32_t* row_sched_dev,
                        const int32_t* order_dev,
                        const int32_t* level_off_dev, const int32_t* level_off_host, int32_t n_levels,
                        const float* X_dev, float* Y_dev, float* workspace_dev, int32_t n, int32_t d,
                        int64_t ldx, int64_t ldy, int32_t flags, void* stream);

/* Deepest tree (levels, children of the root = level 0) that cbm_spmm_update_paths_f32 walks in one launch. */
#define CBM_PATH_MAX_LEVELS 16

/* cbm_spmm_update_f32 for SHALLOW trees, where a launch per level costs more than the level's work
 * (replaces the same reference functions).  With 2 <= n_levels <= CBM_PATH_MAX_LEVELS the SpMM writes
 * Z into z_scratch (n rows of stride (d + 3) & ~3 floats, 16-byte aligned, cbm_spmm_update_paths_scratch_floats)
 * and ONE more launch finishes the product: the wavefront of row v follows parent[] up to the child of
 * the root above it and adds the rows of Z down that path, with the arithmetic of cbm_propagate_f32
 * step by step, so Y is bit for bit what cbm_spmm_update_f32 returns; CBM_UPDATE_RELU goes into that
 * launch's store.  Rows recompute their ancestors' values (sum of depths row reads instead of n), which
 * pays while the rows stay in cache and the levels are few: the caller decides.  Any other depth (flat,
 * or deeper than the limit) is handed to cbm_spmm_update_f32 unchanged and z_scratch is not touched.
 * z_scratch must not overlap X, Y or the workspace. */
int cbm_spmm_update_paths_f32(const int32_t* rowptr_dev, const uint32_t* idx_dev, int64_t nnz, const float* m_dev,
                              const float* coef_dev, const int32_t* parent_dev, const int32_t* row_sched_dev,
                              const int32_t* order_dev, const int32_t* level_off_dev,
                              const int32_t* level_off_host, int32_t n_levels, const float* X_dev, float* Y_dev,
                              float* workspace_dev, float* z_scratch_dev, int32_t n, int32_t d, int64_t ldx,
                              int64_t ldy, int32_t flags, void* stream);

/* Y = A_hat * X in ONE launch, for small matrices whose tree is shallow (n_levels <= CBM_PATH_MAX_LEVELS)
 * and sparse (replaces the same reference functions as cbm_spmm_update_f32): the wavefront of row v
 * computes the delta-row sums of v and of all its ancestors and combines them top-down.  Entries are
 * accumulated strictly in order (as one wavefront per row does, cbm_spmm_summation_groups = 1) with
 * the coefficient +-1 (m == NULL), +-m[col] gathered, or coef[k] streamed; the tree steps use the
 * arithmetic of cbm_propagate_f32: Y is bit for bit what cbm_set_spmm_kernel(1) + cbm_spmm_update_f32
 * return.  Work grows to the sum over rows of the delta entries on their ancestor paths, so this pays
 * only where a launch costs more than those gathers (a few thousand rows, few rows with parents); the
 * caller decides.  No workspace, no scratch.  flags: CBM_UPDATE_RELU. */
int cbm_spmm_update_single_f32(const int32_t* rowptr_dev, const uint32_t* idx_dev, const float* m_dev, const float* coef_dev,
                               const int32_t* parent_dev, int32_t n_levels, const float* X_dev, float* Y_dev, int32_t n,
                               int32_t d, int64_t ldx, int64_t ldy, int32_t flags, void* stream);

/* Floats of z_scratch that cbm_spmm_update_paths_f32 uses: n * ((d + 3) & ~3) for 2 <= n_levels <=
 * CBM_PATH_MAX_LEVELS, else 0 (the call then falls back to cbm_spmm_update_f32). */
int64_t cbm_spmm_update_paths_scratch_floats(int32_t n, int32_t d, int32_t n_levels);

/* cbm_spmm_update_f32 for callers that cannot allocate device memory -- code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc -- and therefore cannot bring the
 * workspace of the slab-major copy of X either.  No counterpart in the reference.  Same arguments
 * minus the workspace, same result bit for bit as cbm_spmm_update_f32 with a workspace of
 * cbm_spmm_workspace_floats() floats: the copy goes to a static device array of
 * CBM_STATIC_SCRATCH_FLOATS floats (128 MiB) that every device the library runs on holds until the
 * process ends.  A shape whose copy needs more (cbm_relayout_floats(n, d) floats) is rejected with
 * CBM_ERR_SCRATCH and nothing is enqueued.  The call
 * allocates and frees nothing, on host or device.  All calls on one device share that device's
 * array: calls that may overlap in time on one device (different streams, different threads)
 * race on it; serialise them.  The array keeps the previous call's contents; every float the
 * gather reads is rewritten by the copy first.  "Bit for bit" holds while the process-wide hooks
 * (cbm_set_spmm_kernel) are not changed by another thread during the call: the size of the copy and the
 * launch plan are both derived from them. */
int cbm_spmm_update_static_f32(const int32_t* rowptr_dev, const uint32_t* idx_dev, int64_t nnz, const float* m_dev,
                               const float* coef_dev, const int32_t* parent_dev, const int32_t* row_sched_dev,
                               const int32_t* order_dev, const int32_t* level_off_dev,
                               const int32_t* level_off_host, int32_t n_levels, const float* X_dev, float* Y_dev,
                               int32_t n, int32_t d, int64_t ldx, int64_t ldy, int32_t flags, void* stream);

/* A tiling (cbm_tile_rows) in DEVICE memory, plus what the kernels of the tiled multiply need:
 *   sched_r    row schedule of the remote part, or NULL (natural order).  With local blocks
 *              (n_blocks > 0) its left scales must all be 1 (cbm_schedule_rows(rowptr_r, NULL, NULL)
 *              or cbm_schedule_rows_split with parent = m = NULL): the kernel of the local part
 *              applies row_scale.  Without local blocks (n_blocks = 0, e.g. cbm_tile_rows with a
 *              min_block_entries no block reaches: the struct then only carries a split schedule)
 *              the schedule carries the left scales and row_scale is not read.
 *   n_sched_r  descriptors in sched_r; 0 means n (one per row, no row is cut)
 *   n_long / long_rows   rows cut by cbm_schedule_rows_split, 4 int32 each; their piece sums use
 *              (number of pieces) x 32 x ceil(d / 32) floats of the workspace behind the copy of X
 *   row_scale  [n] left scale per row: m[r] for children of the root, 1 elsewhere; NULL = no scale
 * The struct itself lives in HOST memory. */
typedef struct cbm_tiling_dev {
    int32_t n_panels, n_blocks, tile_rows, has_negative;
    int64_t nnz_remote;
    const int32_t* panel_ptr;
    const int32_t* blk_tile;
    const int32_t* seg;
    const uint16_t* lidx;
    const int32_t* rowptr_r;
    const uint32_t* idx_r;
    const int32_t* sched_r;
    const float* row_scale;
    int32_t n_sched_r, n_long, n_pieces, reserved;
    const int32_t* long_rows;
} cbm_tiling_dev;

/* Floats of workspace cbm_spmm_tiled_f32 needs: the slab-major copy of X plus the piece sums of
 * cut rows. */
int64_t cbm_spmm_tiled_workspace_floats(const cbm_tiling_dev* t, int32_t n, int32_t d);

/* cbm_spmm_f32 for a matrix whose entries cluster (community structure): Z = D diag(m) X with the
 * remote entries gathered by the slab kernel and the local blocks gathered from tiles of X staged
 * in LDS (1024 rows x 128 bytes per workgroup), which spares them the trip through L1 and L2.
 * workspace is REQUIRED (cbm_spmm_tiled_workspace_floats(t, n, d) floats): both kernels read the slab-major
 * copy, scaled by m when m is given (so no entry carries a coefficient).  flags: CBM_SPMM_RELU;
 * CBM_SPMM_WORKSPACE_READY (with m: together with CBM_SPMM_WORKSPACE_PRESCALED).  Per output
 * element the fp32 sum is (remote entries, summed as cbm_spmm_f32 sums a row) + (local entries,
 * one after the other in storage order -- blocks by ascending tile, by class (column - row) mod 4 inside a block,
 * see cbm_tile_rows -- starting from zero), then the left scale, then the ReLU.  Worth it when most entries are local: 232 965 rows x 491 entries, 89 % of them in
 * blocks of a 50-community graph, d = 128: 1.99 ms against 2.78 ms for cbm_spmm_f32.
 * Replaces the same mkl_sparse_s_mm call as cbm_spmm_f32 (cbm_extensions.cpp:1133-1159). */
int cbm_spmm_tiled_f32(const cbm_tiling_dev* t, const float* m_dev, const float* X_dev, float* Z_dev, float* workspace_dev,
                       int32_t flags, int32_t n, int32_t d, int64_t ldx, int64_t ldz, void* stream);

/* cbm_spmm_update_f32 on a tiling: cbm_spmm_tiled_f32 followed by cbm_propagate_f32. */
int cbm_spmm_update_tiled_f32(const cbm_tiling_dev* t, const float* m_dev, const int32_t* parent_dev,
                              const int32_t* order_dev, const int32_t* level_off_dev, const int32_t* level_off_host,
                              int32_t n_levels, const float* X_dev, float* Y_dev, float* workspace_dev, int32_t n,
                              int32_t d, int64_t ldx, int64_t ldy, int32_t flags, void* stream);

/* Row intersections for the builder on the GPU: appends to pairs[] every (i, j > i, s) with
 * s = |row_i ^ row_j| and 2 s > min(nnz_i, nnz_j) + alpha, in no particular order, and adds their
 * number to *n_pairs (which may exceed capacity: then only the first `capacity` were stored and the
 * call must be repeated with a larger buffer).  The six input arrays are device copies of
 * cbm_builder_arrays(); ticket = 1 uint32 and n_pairs = 1 uint64, both zero on entry; groups =
 * number of workgroups, e.g. cbm_row_intersections_groups() (one per CU).  No scratch memory:
 * the counters live in LDS.  Feed the result to cbm_builder_finish.
 * Replaces mkl_sparse_syrk + the admission scan of cbm_init_v1_/_v2_ (cbm_extensions.cpp:46-103). */
int cbm_row_intersections_groups(void);
int cbm_row_intersections(const int64_t* rowptr_dev, const int32_t* col_dev, const int64_t* colptr_t_dev,
                          const int32_t* row_t_dev, const int64_t* after_dev, const int32_t* row_nnz_dev, int32_t n,
                          int32_t alpha, int32_t groups, uint32_t* ticket_dev, struct cbm_pair* pairs_dev,
                          int64_t capacity, unsigned long long* n_pairs_dev, void* stream);

/* Plain CSR SpMM  Y = A * X  (val == NULL means all ones): the hand-written GPU baseline.
 * Replaces seq_/omp_s_spmm_csr_int32_ (cbm_extensions.cpp:790-843, :1707-1755). */
int csr_spmm_f32(const int32_t* rowptr_dev, const int32_t* col_dev, int64_t nnz, const float* val_dev,
                 const int32_t* row_sched_dev, const float* X_dev, float* Y_dev, float* workspace_dev,
                 int32_t flags, int32_t n, int32_t d, int64_t ldx, int64_t ldy, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* CBM_HIP_H */
