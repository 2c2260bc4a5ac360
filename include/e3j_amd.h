/* C ABI of the MI355X (gfx950) fused message-passing convolution library.
 *
 * Every entry point takes plain device pointers, sizes and a HIP stream and
 * returns a status code; nothing here names a tensor framework.  The operand
 * lists are those of the reference's two XLA-FFI targets for this path,
 * "convolution" and "convolution_bwd" (lib/e3j_ops/ffi/e3j_ops.h:379-472 and
 * :478-594), minus `coef_ranges` (a CUDA launch-balancing artefact) and plus
 * the memory layout, an optional edge permutation on the forward and the id of
 * a compile-time-unrolled kernel.
 *
 * Conventions
 *  - Values are float32 (or float64 / float16 on the table-driven kernels; float16 computes in
 *    half precision with fused multiply-adds, lib/e3j_ops/cuda/utils.cuh:108-112); indices int32.
 *  - TRAILING layout: x (N, X, K), s (E, S, K), out/dm (N, Z, K).
 *    LEADING  layout: x (N, K, X), s (E, K, S), out/dm (N, K, Z).  y is (E, Y).
 *  - A CSR adjacency groups edge positions by one endpoint: `row_ptr` (N+1)
 *    and, per position, the other endpoint `other` (E).  A position whose
 *    `other` lies outside [0, N), or that lies at or past row_ptr[N], is a
 *    padding edge: it contributes nothing and gets dy = ds = 0
 *    (lib/e3j_ops/cuda/convolution/fwd.cuh:368, bwd.cuh:225-226,308-319).
 *  - `edge_perm` (E) maps a CSR position to the row of y / s / dy / ds it
 *    refers to; NULL means identity (lib/e3j_ops/ffi/e3j_ops.h:543-548).
 *  - `coef` is the packed table {val; i; j; k; l} of lib/e3j_ops/cuda/convolution.cuh:31-44,
 *    resident in device memory; `coef_idx_bytes` is 1 (uint8) or 4 (int32).
 *  - Launches are asynchronous on `stream`; with debug > 0 the stream is
 *    synchronised before returning so device faults surface at the call
 *    (lib/e3j_ops/cuda/convolution/launch_fwd.cuh:255-263).
 *  - Rows of nodes without live edges are written as exact zeros.
 *  - Alignment: any element-aligned pointer is accepted by the forward and the two grouped
 *    backwards; the compile-time-unrolled kernels are used when x, s, out / dm, dx and ds are
 *    16-byte aligned (true of whole allocations), otherwise the table-driven kernels run (which
 *    then need `coef`).  The ordered and tiled backwards and e3j_amd_radial_linear_* require
 *    16-byte aligned operands and return E3J_AMD_INVALID_ARGUMENT otherwise.
 */
#ifndef E3J_AMD_H_
#define E3J_AMD_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Status codes; names follow the reference's error classes (lib/e3j_ops/ffi/error.h:22-105). */
enum {
    E3J_AMD_OK = 0,
    E3J_AMD_INVALID_ARGUMENT = 1,
    E3J_AMD_UNIMPLEMENTED = 2,
    E3J_AMD_INTERNAL = 3
};

enum { E3J_AMD_LAYOUT_LEADING = 0, E3J_AMD_LAYOUT_TRAILING = 1 }; /* src/e3j/utils/options.py:144-145 */
enum { E3J_AMD_F32 = 0, E3J_AMD_F64 = 1, E3J_AMD_F16 = 2 };

/* Problem sizes, the counterpart of convolution::Params (lib/e3j_ops/cuda/convolution.cuh:46-60). */
typedef struct e3j_amd_conv_params {
    int32_t num_nodes;
    int64_t num_edges;
    int32_t num_coef;
    int32_t num_x;
    int32_t num_y;
    int32_t num_out;
    int32_t num_scalars;
    int32_t channels;
    int32_t layout;         /* E3J_AMD_LAYOUT_* */
    int32_t val_dtype;      /* E3J_AMD_F32 / E3J_AMD_F64 / E3J_AMD_F16 */
    int32_t coef_idx_bytes; /* 1 or 4 */
    int32_t signature;      /* id from e3j_amd_find_signature, or -1: table-driven kernel */
    float   coef_scale;     /* unrolled kernels: table = coef_scale * built-in table (1 by default) */
    int32_t debug;
    /* Unrolled kernels: bit k set = the kernel reads -y[:, k] and returns -dy[:, k].  With the
     * parity signs of y this runs a symmetric graph's edges in the reversed direction (the
     * SENDER ordering, src/e3j/ops/convolution.py:166-176) on the unsigned built-in table.
     * Must be 0 for the table-driven kernels, which take the signs in the table. */
    uint32_t y_flip;
    /* Optional processing order of the CSR rows (device, num_nodes entries, a permutation of
     * 0..num_nodes-1), e.g. from e3j_amd_locality_order; NULL = natural order.  It only
     * changes which rows run together (cache reuse of gathered rows), never the results. */
    const int32_t *row_order;
    /* Long rows of the forward pass (unrolled kernels, trailing layout; anything else answers
     * E3J_AMD_UNIMPLEMENTED when one of these is set).  One wave sums a row edge by edge, so a
     * receiver with very many edges would hold one wave for the whole launch.  With row_cap > 0
     * the wave of a row longer than row_cap sums only its first row_piece edges (row_piece <=
     * row_cap; 0 means row_cap).  The rest of every such row is listed in `segments`, in
     * pieces of row_piece edges (e3j_amd_row_segments_build), and summed by a second call of
     * e3j_amd_convolution_fwd with `segments` set, which ADDS to `out` with float atomics (so it
     * runs after the first call, on the same stream, and the sum of a split row depends on the
     * order of the additions).  segments: device, int32: [0] = number of pieces n (at most
     * max_segments are run), [4 + 3 i ...] = (row, first position, end position) of piece i.
     * partials (optional, with `segments`): device scratch of e3j_amd_row_partials_bytes bytes,
     * 16-byte aligned.  The second call then sums every piece into a scratch row of its own and
     * adds the rows of a receiver's pieces to its output row one after another, in the order of
     * their positions: the result is the same bits in every run (the list must keep the pieces of
     * one row adjacent and in position order, as e3j_amd_row_segments_build writes it). */
    int32_t row_cap;
    int32_t row_piece;
    int32_t max_segments;
    const int32_t *segments;
    float *partials;
    /* Table-driven kernels: optional device memory of e3j_amd_table_plan_bytes bytes for the plan
     * of the table (see e3j_amd_set_table_plans), 4-byte aligned.  The call writes the plan there
     * and reads it back on the same stream (calls that share the memory must not overlap).  With
     * it the call allocates nothing and the planned kernels also run on a stream that is being
     * captured into a graph; NULL: memory from the stream's pool, and none under capture. */
    int32_t *table_plan;
    /* E3J_AMD_PLAN_BUILD (0): the call builds the plan of its table (into table_plan, or into pool
     * memory) and launches both forms of the table-driven kernels, of which the one the plan's flag
     * names runs.  E3J_AMD_PLAN_READY: table_plan holds the plan of this very table (same `coef`
     * contents and column order, same sizes), built by e3j_amd_table_plan_status with table_plan set,
     * which reported that the planned kernels take the table: nothing is built and only the planned
     * kernel is launched; the plan is only read, so calls on any stream may share it.
     * E3J_AMD_PLAN_NONE: the call does not plan (a table the status call reported as not taken). */
    int32_t table_plan_state;
    /* float64 operands on the unrolled kernels (signature >= 0, val_dtype = E3J_AMD_F64; trailing
     * layout, receiver-grouped calls): HOST pointer to the E3J_AMD_F64_CLASSES doubles that
     * e3j_amd_find_signature_f64 returned for the table.  The float64 kernels do not carry the
     * table's values as literals with one scale factor (exact to float32 rounding only): they read
     * one value per class of entries of equal magnitude from this array, which is copied into the
     * launch, so a table of the signature's structure is served to float64 accuracy whatever its
     * values.  coef_scale is not used then. */
    const double *coef_classes;
} e3j_amd_conv_params;
enum { E3J_AMD_PLAN_BUILD = 0, E3J_AMD_PLAN_READY = 1, E3J_AMD_PLAN_NONE = 2 };
enum { E3J_AMD_F64_CLASSES = 64 };

/* Message of the last failure on the calling thread ("" if none). */
const char *e3j_amd_last_error(void);

/* Library version string. */
const char *e3j_amd_version(void);

/* Forward: replaces the "convolution" target (lib/e3j_ops/ffi/e3j_ops.h:379-472;
 * kernel lib/e3j_ops/cuda/convolution/fwd.cuh:289-403).
 * CSR grouped by receiver: other = sender per position, row_ptr = receiver_ptr. */
int e3j_amd_convolution_fwd(const e3j_amd_conv_params *p, const void *coef,
                            const void *x, const void *y, const void *s,
                            const int32_t *sender, const int32_t *receiver_ptr,
                            const int32_t *edge_perm, void *out, void *stream);

/* Backward, operands of the reference: replaces the "convolution_bwd" target
 * (lib/e3j_ops/ffi/e3j_ops.h:478-594; kernel lib/e3j_ops/cuda/convolution/bwd.cuh:116-321).
 * CSR grouped by SENDER (the transposed adjacency): receiver_t = receiver per
 * position, sender_ptr = row pointer by sender, edge_perm = position -> original
 * edge (NULL under SENDER ordering).  `coef` is the FORWARD table (i, j, k, l);
 * the reference's three transposed copies are not needed.  dx is accumulated
 * row-locally without atomics: results are bit-reproducible run to run.
 * With p->signature >= 0 (trailing layout, float32, 16-byte aligned operands) the
 * compile-time-unrolled kernels serve this grouping too: a wave per (sender, 64 channels)
 * keeps the sender's x row and its dx sums in registers and gathers the dm rows of the
 * receivers; `coef` is then not read.  dy of an edge is added by channels / 64 waves: the
 * same bits in every run up to 128 channels (two addends), equal up to the order of four
 * additions at 256.  Other operands run the table-driven kernel, which owns dx and dy. */
int e3j_amd_convolution_bwd_sender(const e3j_amd_conv_params *p, const void *coef,
                                   const void *x, const void *y, const void *s, const void *dm,
                                   const int32_t *receiver_t, const int32_t *sender_ptr,
                                   const int32_t *edge_perm,
                                   void *dx, void *dy, void *ds, void *stream);

/* Backward on the forward's own receiver-grouped CSR (no transpose, no sort):
 * same results as e3j_amd_convolution_bwd_sender up to the summation order of dx,
 * which is accumulated with float atomics.  This is the grouping the reference
 * recommends for its Mosaic-GPU backend (src/e3j/core/convolution.py:77-82). */
int e3j_amd_convolution_bwd_receiver(const e3j_amd_conv_params *p, const void *coef,
                                     const void *x, const void *y, const void *s, const void *dm,
                                     const int32_t *sender, const int32_t *receiver_ptr,
                                     const int32_t *edge_perm,
                                     void *dx, void *dy, void *ds, void *stream);

/* The same backward on the forward's receiver CSR without any atomic: every wave stores the dx
 * contribution of its CSR positions into a buffer, which is then summed per sender in ascending
 * position order, and dy sums of waves that share an edge are combined in a fixed order.
 * Bit-reproducible from run to run like the reference's backward
 * (tests/test_ops/test_convolution_op.py:329-342), at the price of one more pass over
 * E * num_x * channels floats.  Needs a compile-time-unrolled kernel (p->signature >= 0),
 * else E3J_AMD_UNIMPLEMENTED.  workspace: device memory, at least
 * e3j_amd_convolution_bwd_ordered_workspace_bytes(p) bytes (about E * (num_x * channels +
 * channels / 16 * num_y) floats); contents on entry and exit are irrelevant. */
size_t e3j_amd_convolution_bwd_ordered_workspace_bytes(const e3j_amd_conv_params *p);
int e3j_amd_convolution_bwd_ordered(const e3j_amd_conv_params *p, const void *coef, const void *x,
                                    const void *y, const void *s, const void *dm,
                                    const int32_t *sender, const int32_t *receiver_ptr,
                                    const int32_t *edge_perm, void *dx, void *dy, void *ds,
                                    void *workspace, void *stream);

/* The receiver-grouped backward over tiles of receivers.  Neighbouring receivers share most of
 * their senders; a workgroup takes `tile_rows` receivers that are consecutive in the row order,
 * keeps their dm rows in LDS and walks the tile's edges sorted by sender, so that the dx
 * contributions of one sender are summed on chip and leave as one set of float atomics per
 * (tile, sender) instead of one per edge.  Same results as e3j_amd_convolution_bwd_receiver up
 * to the summation order of dx.  Needs a compile-time-unrolled kernel of the trailing layout with
 * at least 64 channels (else E3J_AMD_UNIMPLEMENTED) and a schedule built for the same adjacency,
 * edge_perm and p->row_order.  No counterpart in the reference; prior art for grouping the
 * backward by receivers with dx added into a zero-filled buffer:
 * src/e3j/pallas_ops/convolution/mosaic_gpu/bwd.py:336-457.
 *
 * Schedule: the edge positions of every tile sorted by sender (padding edges last; a tile of
 * more than 512 positions lists its live positions in row order, unsorted, then its padding
 * positions: the kernel only needs equal senders side by side to sum them), as three
 * parallel arrays, and work descriptors (tile, begin, end, 0) that cut the tiles' lists into
 * pieces of at most `max_work_edges` positions (long rows are thereby shared by several
 * workgroups).  All pointers are device memory owned by the caller. */
typedef struct e3j_amd_tile_schedule {
    int32_t tile_rows;     /* receivers per tile */
    int32_t num_work;      /* entries of `work` (an upper bound of the entries in use) */
    const int32_t *work;   /* (num_work, 4): (tile, begin, end, 0), the entries in use first (a tile
                              without positions takes one with begin == end); the fourth field of
                              entry 0 holds their number, the entries behind them are not read */
    const int32_t *sender; /* (E) sender of the position, -1 for a padding edge */
    const int32_t *edge;   /* (E) row of y / s / dy / ds */
    const int32_t *local;  /* (E) index of the position's receiver within its tile */
} e3j_amd_tile_schedule;
/* The list of pieces for e3j_amd_conv_params.segments: every row of the CSR longer than row_cap
 * is cut into pieces of at most row_piece positions (1 <= row_piece <= row_cap), and all but the
 * first are listed (the forward pass with p->row_cap / row_piece set sums the first).
 * `segments` holds 4 + 3 * max_segments int32; e3j_amd_row_segments_max bounds the number of
 * pieces for any graph with that many edges.  One small kernel after a 16-byte fill; no workspace.  No counterpart in the
 * reference, whose forward kernel also walks the edges of a receiver one after another in one
 * block (lib/e3j_ops/cuda/convolution/fwd.cuh:346-363). */
int64_t e3j_amd_row_segments_max(int64_t num_edges, int32_t row_piece);
/* Bytes of e3j_amd_conv_params.partials for a list of up to max_segments pieces: a row of
 * num_out * channels floats per piece and a numbered copy of the list. */
size_t e3j_amd_row_partials_bytes(int64_t max_segments, int32_t num_out, int32_t channels);
int e3j_amd_row_segments_build(const int32_t *receiver_ptr, int32_t num_nodes, int32_t row_cap,
                               int32_t row_piece, int32_t max_segments, int32_t *segments,
                               void *stream);
/* Largest `tile_rows` the tiled backward of a signature takes (its LDS holds the dm rows of a
 * tile), 0 if the signature has no tiled backward. */
int32_t e3j_amd_tile_rows(int32_t signature);
/* The `tile_rows` the tiled backward of a signature is tuned for (leaves room in the LDS for the
 * number of workgroups per CU its launch shape wants), 0 if the signature has no tiled backward. */
int32_t e3j_amd_tile_rows_default(int32_t signature);
/* Number of work descriptors to provide for a graph (upper bound used by the builder). */
int64_t e3j_amd_tile_schedule_num_work(int32_t num_nodes, int64_t num_edges, int32_t tile_rows,
                                       int32_t max_work_edges);
size_t e3j_amd_tile_schedule_workspace_bytes(int32_t num_nodes, int64_t num_edges, int32_t tile_rows);
/* Builds the schedule of a receiver-grouped CSR (sender per position, receiver_ptr), optional
 * edge_perm and optional row order, into work (num_work, 4), t_sender, t_edge, t_local (E each). */
int e3j_amd_tile_schedule_build(const int32_t *sender, const int32_t *receiver_ptr,
                                const int32_t *edge_perm, const int32_t *row_order,
                                int32_t num_nodes, int64_t num_edges, int32_t tile_rows,
                                int32_t max_work_edges, int32_t *work, int32_t *t_sender,
                                int32_t *t_edge, int32_t *t_local, void *workspace, void *stream);
int e3j_amd_convolution_bwd_tiled(const e3j_amd_conv_params *p, const void *x, const void *y,
                                  const void *s, const void *dm, const int32_t *sender,
                                  const int32_t *receiver_ptr, const int32_t *edge_perm,
                                  const e3j_amd_tile_schedule *schedule, void *dx, void *dy, void *ds,
                                  void *stream);

/* Match a HOST copy of a packed forward table against the tables of the
 * compile-time-unrolled kernels built into the library, up to one uniform
 * positive factor (the 1/avg_num_neighbors the reference folds into the values,
 * src/e3j/core/convolution.py:135-140), which is returned in *coef_scale, and, when
 * y_flip is not NULL, up to one sign per y component (the parity signs the reference folds
 * into the table for the SENDER ordering, src/e3j/ops/convolution.py:166-176), returned as
 * a bit mask for e3j_amd_conv_params.y_flip (tables with more than 32 y components match
 * only without signs).  Returns the signature id (>= 0) or -1.  Takes the place of the reference's
 * trace-time launch planning (src/e3j/ops/convolution.py:178-208).
 * val_dtype: E3J_AMD_F32, or E3J_AMD_F16 for a table of half values (float16 operands on the float16
 * unrolled kernels: trailing layout, forward and receiver-grouped backward, operands 4-byte aligned);
 * entries then agree within half rounding.  float64 tables: e3j_amd_find_signature_f64. */
int e3j_amd_find_signature(const void *coef_host, int32_t coef_idx_bytes, int32_t val_dtype,
                           int32_t num_coef, int32_t num_x, int32_t num_y, int32_t num_out,
                           int32_t num_scalars, int32_t channels, int32_t layout,
                           float *coef_scale,
                           uint32_t *y_flip);

/* The same look-up for a float64 table (host memory, packed with double values), for float64
 * operands on the unrolled kernels.  The table must have the entries of a built-in (or registered)
 * table whose float64 kernels are built: the same coordinates, the same signs up to one sign per y
 * component (*y_flip), and equal magnitudes (to 1e-13) wherever the built-in table has equal
 * magnitudes.  The magnitudes themselves are free: coef_classes (E3J_AMD_F64_CLASSES doubles, host)
 * receives one per class, for e3j_amd_conv_params.coef_classes.  Returns the id or -1.  No
 * counterpart in the reference, whose kernel reads the table at run time for every dtype
 * (tests/test_ops/test_dtype.py:56-71). */
int e3j_amd_find_signature_f64(const void *coef_host, int32_t coef_idx_bytes, int32_t num_coef,
                               int32_t num_x, int32_t num_y, int32_t num_out, int32_t num_scalars,
                               int32_t channels, int32_t layout, double *coef_classes, uint32_t *y_flip);

/* The table-driven kernels (calls with signature < 0, and calls whose operands an unrolled kernel
 * cannot take) come in two forms.  For a float32 or float16 table (float16: values held as half,
 * arithmetic in float; the sender-grouped backward only) in which every output coordinate uses one
 * scalar, with at most 128 output coordinates, 16 x coordinates, 64 y components, 64 scalars and
 * 2048 entries, the call first turns the table into a plan on the device (one small kernel; the
 * plan lives in memory of the stream's pool, hipMallocAsync, for the length of the call) and runs
 * kernels that keep x and the accumulators in registers; any other table and float64 run the
 * kernels that index LDS columns by the table's coordinates (float16 there: arithmetic in half).  Whether a table fits is
 * decided on the device, without a read-back.  on = 0 switches the planned form off for later
 * calls (process-wide, atomic; initial value from E3J_AMD_TABLE_PLANS, default 1).  The plan (a few
 * KB) lives in e3j_amd_conv_params.table_plan when the caller brings that memory, else in memory of
 * the stream's pool for the length of the call; without the caller's memory a call on a stream that
 * is being captured into a graph allocates nothing and runs the LDS-column kernels.  Results
 * agree to rounding (the planned form sums per output coordinate in a different order).
 * No counterpart in the reference, which has one table-driven kernel
 * (lib/e3j_ops/cuda/convolution/fwd.cuh:88-153). */
void e3j_amd_set_table_plans(int32_t on);
/* Whether the planned form takes a table, and what its plan looks like: builds the plan of the
 * device-resident table `coef` (the operand of the convolution calls; coef_cols_ji as for the
 * backward entry points), waits for it and writes status[0] = 1 if the planned kernels take the
 * table (0: sizes beyond the limits, or an output coordinate with two scalars), status[1] = its
 * non-empty (output coordinate, x coordinate) cells, status[2] = the (16 output coordinates x 4 x
 * coordinates) blocks the loops visit, status[3] = scalars no entry uses.  With p->table_plan set the
 * plan is built in that memory and stays there: later calls with table_plan_state =
 * E3J_AMD_PLAN_READY (if status[0] is 1) use it without building it again.  Synchronises (and
 * allocates when p->table_plan is NULL): for tests and set-up code, not for the hot path. */
int e3j_amd_table_plan_status(const e3j_amd_conv_params *p, const void *coef, int32_t coef_cols_ji,
                              int32_t *status, void *stream);
/* Bytes of e3j_amd_conv_params.table_plan for the sizes in `p` (num_coef, num_scalars and the
 * dimensions); 0 when the planned form does not take these sizes or this value type (nothing to
 * bring then). */
size_t e3j_amd_table_plan_bytes(const e3j_amd_conv_params *p);

/* Adds a signature compiled at run time (e3j_amd/jit.py generates the kernels of a table
 * the library was not built for, compiles them against this library and hands over the entry
 * its plugin exports).  Returns the new signature id, which e3j_amd_find_signature reports
 * from then on, or -1.  The entry must stay loaded for the life of the process.  Counterpart
 * of the trace-time unrolling of the reference's Pallas kernels
 * (src/e3j/pallas_ops/convolution/mosaic_gpu/fwd.py:162-177). */
int e3j_amd_register_signature(const void *entry);

/* Number of signatures (built-in and registered) and a printable description of one. */
int e3j_amd_num_signatures(void);
const char *e3j_amd_signature_name(int signature);

/* Graph preparation on the device, replacing the per-call XLA ops of
 * GraphCSR (src/e3j/data/graph.py:49-73).
 * e3j_amd_csr_row_ptr: row_ptr = [0] + cumsum(bincount(key, length = num_nodes)),
 *   keys outside [0, num_nodes) dropped.  workspace: >= e3j_amd_csr_workspace_bytes(). */
size_t e3j_amd_csr_workspace_bytes(int32_t num_nodes, int64_t num_edges);
int e3j_amd_csr_row_ptr(const int32_t *key, int64_t num_edges, int32_t num_nodes,
                        int32_t *row_ptr, void *workspace, void *stream);
/* e3j_amd_csr_row_ptr_static: the same row pointers for callers that cannot allocate or bring a
 *   workspace (code under HIP graph capture, serving loops, harnesses that forbid hipMalloc).  The
 *   scan's temporary storage lives in a 256 KiB device array inside the library (one copy per GPU,
 *   held until the process ends); the call allocates nothing.  num_nodes above
 *   e3j_amd_csr_row_ptr_static_max_nodes() is refused with E3J_AMD_INVALID_ARGUMENT.  Every call
 *   on a GPU uses that GPU's one array: calls that overlap on one GPU (different streams or
 *   threads) race; calls on one stream are ordered.  No counterpart in the reference. */
int32_t e3j_amd_csr_row_ptr_static_max_nodes(void);
int e3j_amd_csr_row_ptr_static(const int32_t *key, int64_t num_edges, int32_t num_nodes,
                               int32_t *row_ptr, void *stream);
/* e3j_amd_sort_edges: stable counting sort of edge positions by key (out-of-range
 *   keys last): perm (E), other_sorted = other[perm] (E), row_ptr (N+1). */
int e3j_amd_sort_edges(const int32_t *key, const int32_t *other, int64_t num_edges,
                       int32_t num_nodes, int32_t *perm, int32_t *other_sorted,
                       int32_t *row_ptr, void *workspace, void *stream);

/* e3j_amd_wrap_index: global node ids of a sharded graph to shard-local ids,
 *   out[i] = index[i] mod num_nodes, the sentinel INT32_MAX kept
 *   (replaces wrap_global_index, src/e3j/ops/convolution.py:39-51). */
int e3j_amd_wrap_index(const int32_t *index, int64_t n, int32_t num_nodes, int32_t *out,
                       void *stream);

/* e3j_amd_locality_order: a processing order of the nodes in which nodes that are close in
 *   the graph are close in the order, from `rounds` sweeps of minimum-label propagation over
 *   a CSR adjacency (other, row_ptr): clusters of nodes within `rounds` hops of a local
 *   minimum id, ordered hierarchically.  order (N): a permutation.
 *   workspace: >= e3j_amd_order_workspace_bytes().
 *   No counterpart in the reference, whose kernels walk the rows in index order
 *   (lib/e3j_ops/cuda/convolution/fwd.cuh:346). */
size_t e3j_amd_order_workspace_bytes(int32_t num_nodes);
int e3j_amd_locality_order(const int32_t *other, const int32_t *row_ptr, int32_t num_nodes,
                           int32_t rounds, int32_t *order, void *workspace, void *stream);

/* e3j_amd_pair_rows: reorders a processing order for the backward over tiles of two receivers.
 *   Rows that share most of their senders are put side by side (greedy matching over a few
 *   rounds: rows that pick each other as the row with the most senders in common are paired),
 *   pairs first, each on an even and the next odd position, in the order their earlier member
 *   had in order_in (NULL: index order); unpaired rows (also those without edges or with more
 *   than 128) follow in their old order.  order_out (N): a permutation; must not alias order_in.
 *   Results of the convolution do not depend on it; the tiled backward issues one set of dx
 *   atomics per sender a pair shares.  workspace: >= e3j_amd_pair_rows_workspace_bytes().
 *   No counterpart in the reference. */
size_t e3j_amd_pair_rows_workspace_bytes(int32_t num_nodes, int64_t num_edges);
int e3j_amd_pair_rows(const int32_t *other, const int32_t *row_ptr, int32_t num_nodes, int64_t num_edges,
                      const int32_t *order_in, int32_t *order_out, void *workspace, void *stream);

/* Edge featurisation next to the convolution: real spherical harmonics of `num` vectors
 * (num, 3) for the degrees 0..l_max (l_max <= 6), out (num, (l_max + 1)^2), and the
 * vector-Jacobian product dvec (num, 3) for a cotangent dout of that shape.  Order, harmonic
 * frame and normalisations of the reference's Harmonics module
 * (src/e3j/core/harmonics.py:25-42,92-101; src/e3j/utils/spherical_harmonics.py:33-38,66-75):
 * normalization 0 "integral", 1 "component", 2 "norm"; normalize != 0 projects the vectors
 * on the unit sphere first (zero vectors are left as they are).  val_dtype: E3J_AMD_F32/F64. */
int e3j_amd_harmonics(const void *vec, int64_t num, int32_t l_max, int32_t normalize,
                      int32_t normalization, int32_t val_dtype, void *out, void *stream);
int e3j_amd_harmonics_bwd(const void *vec, const void *dout, int64_t num, int32_t l_max,
                          int32_t normalize, int32_t normalization, int32_t val_dtype, void *dvec,
                          void *stream);

/* Edge featurisation from atom positions in one launch (the producer of the convolution's operands
 * y and, through e3j_amd_radial_linear_fwd, s): per edge e the vector
 * positions[sender[e]] - positions[receiver[e]] (+ shift[e], the lattice translation of a periodic
 * cell; NULL: none), then
 *   y (num_edges, (l_max + 1)^2)          harmonics of its direction, as e3j_amd_harmonics with normalize = 1
 *   basis (num_edges, num_basis)          sqrt(2 / cutoff) sin(n pi r / cutoff) / r, n = 1..num_basis, times the
 *                                         envelope 1 - 10 t^3 + 15 t^4 - 6 t^5, t = min(r / cutoff, 1)   (NULL: not written)
 *   h (layers, num_edges, hidden)         silu(basis w1[layer]), w1 (layers, num_basis, hidden): the hidden layer
 *                                         of the radial network of each convolution layer (NULL or hidden = 0: none)
 * An edge with an endpoint outside [0, num_nodes) or of zero length gets zeros.  The backward entry
 * point recomputes the chain from the positions and writes dpositions (num_nodes, 3) (zero-filled by
 * the call, contributions added with float atomics) for the cotangents dy, dbasis, dh (each may be NULL).
 * No counterpart in the reference, whose callers build these arrays with separate XLA ops
 * (Harmonics: src/e3j/core/harmonics.py:45-101; edge_scalars of src/e3j/core/convolution.py:342-350
 * arrive ready-made). */
typedef struct e3j_amd_edge_features_params {
    int64_t num_edges;
    int32_t num_nodes;
    int32_t l_max;          /* <= 6 */
    int32_t normalization;  /* 0 integral, 1 component, 2 norm */
    int32_t num_basis;      /* 1..16 */
    int32_t hidden;         /* width of the hidden layer, 0: none */
    int32_t layers;         /* hidden layers evaluated side by side */
    float   cutoff;
    int32_t val_dtype;      /* E3J_AMD_F32 / E3J_AMD_F64 */
} e3j_amd_edge_features_params;
int e3j_amd_edge_features_fwd(const e3j_amd_edge_features_params *p, const void *positions,
                              const int32_t *sender, const int32_t *receiver, const void *shift,
                              const void *w1, void *y, void *basis, void *h, void *stream);
int e3j_amd_edge_features_bwd(const e3j_amd_edge_features_params *p, const void *positions,
                              const int32_t *sender, const int32_t *receiver, const void *shift,
                              const void *w1, const void *dy, const void *dbasis, const void *dh,
                              void *dpositions, void *stream);

/* Regroups node rows around the per-degree channel mixing that follows a convolution: element
 * (n, i, k) of a plain array (num_nodes, rows, channels) sits at row_base[i] + n * row_stride[i] + k of
 * the regrouped array (row_base, row_stride: device, `rows` int64 each, multiples of 4 floats / 2
 * doubles).  to_plain = 0 copies plain -> regrouped, 1 regrouped -> plain; every row moves in
 * 16-byte pieces, one launch.  With row_base / row_stride describing A_l[(n, m), (u, k)] per output
 * degree, the mixing x'[n, m, :] = sum_u out[n, base_l + u dim_l + m, :] W_l[u] becomes one matrix
 * product per degree, and its backward writes every cotangent row once.  No counterpart in the
 * reference (an einsum per degree under XLA, src/e3j/core/linear.py). */
int e3j_amd_rows_regroup(const void *src, void *dst, int64_t num_nodes, int32_t rows, int32_t channels,
                         const int64_t *row_base, const int64_t *row_stride, int32_t to_plain,
                         int32_t val_dtype, void *stream);
/* The same mixing in one launch on the matrix cores (float32, 64 or 128 channels, 16-byte aligned
 * operands): no regrouped copies, no library products.  The convolution's output has, for each of
 * num_degrees output degrees in row order, mul[l] copies of dim[l] = 2l + 1 rows (mul, dim: HOST
 * arrays, num_degrees <= 8).  transpose = 0: src (num_nodes, sum mul dim, channels), weights the
 * concatenation of W_l[u][k][c] (mul[l] x channels x channels each), dst (num_nodes, sum dim,
 * channels) with dst[n, m_l, c] = sum_{u, k} src[n, base_l + u dim_l + m, k] W_l[u][k][c].
 * transpose = 1 (the backward pass): src (num_nodes, sum dim, channels), weights the
 * concatenation of the transposed W_l[u][c][k], dst (num_nodes, sum mul dim, channels) with
 * dst[n, base_l + u dim_l + m, k] = sum_c src[n, m_l, c] W_l[u][k][c].  Every row of dst is
 * written once.  No counterpart in the reference (src/e3j/core/linear.py:125-243 under XLA). */
int e3j_amd_channel_mix(const void *src, void *dst, const void *weights, int64_t num_nodes, int32_t channels,
                        int32_t num_degrees, const int32_t *mul, const int32_t *dim, int32_t transpose,
                        void *stream);

/* Last layer of the radial network that produces the convolution's per-edge, per-path weights:
 * s (num_edges, n) = h (num_edges, inner) w (inner, n), n = paths * channels, float32, row-major,
 * on the matrix cores.  inner: 8, 16, 32, 64 or 128; n: a multiple of 32.  No counterpart in the
 * reference, which leaves the radial network to the caller (edge_scalars of
 * src/e3j/core/convolution.py:342-350 arrive ready-made); it is the dense contraction next to the
 * convolution, and the operand the convolution reads most. */
int e3j_amd_radial_linear_fwd(const float *h, const float *w, float *s, int64_t num_edges,
                              int32_t inner, int32_t n, void *stream);
/* Its backward with respect to h for inner sizes of 64 and 128: dh (num_edges, inner) = ds w^T, with
 * the weights passed transposed, wt (n, inner) row-major; ds is read once.  Smaller inner sizes
 * return E3J_AMD_UNIMPLEMENTED: the library product already reads ds near the rate of the memory. */
int e3j_amd_radial_linear_bwd_input(const float *ds, const float *wt, float *dh, int64_t num_edges,
                                    int32_t inner, int32_t n, void *stream);
/* Its backward with respect to the weights: dw (inner, n) = h^T ds, ds (num_edges, n) read once,
 * summed over the edges in a fixed order (bit-reproducible).  workspace: device memory of
 * e3j_amd_radial_linear_bwd_weight_workspace_bytes(num_edges, inner, n) bytes. */
size_t e3j_amd_radial_linear_bwd_weight_workspace_bytes(int64_t num_edges, int32_t inner, int32_t n);
int e3j_amd_radial_linear_bwd_weight(const float *h, const float *ds, float *dw, void *workspace,
                                     int64_t num_edges, int32_t inner, int32_t n, void *stream);

/* Row-wise sparse tensor product, the edge-wise sibling of the convolution (no gather, no
 * scatter): z[r] = sum_n val_n x[r, j_n] (*) y[r, k_n] -> z[r, i_n].  Operands and sizes of the
 * reference's "tensor_product" / "tensor_product_bwd" targets (lib/e3j_ops/ffi/e3j_ops.h:124-253,
 * :258-372; Params of lib/e3j_ops/cuda/tensor_product.cuh:58-95) minus `coef_ranges`.
 * Channel modes (src/e3j/utils/options.py:154-168):
 *   OUTER z[r, i, cx, cy] = x[r, j, cx] y[r, k, cy]; an operand without channel axis has channels 1
 *   INNER z[r, i]         = sum_c x[r, j, c] y[r, k, c]
 *   MAP   z[r, i, c]      = x[r, j, c] y[r, k, c]
 * TRAILING layout: x (R, X, Cx), y (R, Y, Cy), z (R, Z, Cx, Cy) / (R, Z) / (R, Z, C);
 * LEADING layout: x (R, Cx, X), y (R, Cy, Y), z (R, Cx, Cy, Z) / (R, Z) / (R, C, Z).
 * `coef` is the packed table {val; i; j; k} of lib/e3j_ops/cuda/tensor_product.cuh:98-111 in
 * device memory (8, 16, 16, 32, 8, 16 bytes per entry for uint8/float32, int32/float32,
 * uint8/float64, int32/float64, uint8/float16, int32/float16).  Any channel count is accepted (the reference requires powers
 * of two in the trailing layout, e3j_ops.h:168-185). */
enum { E3J_AMD_MODE_OUTER = 0, E3J_AMD_MODE_INNER = 1, E3J_AMD_MODE_MAP = 2 };
typedef struct e3j_amd_tp_params {
    int64_t num_rows;
    int32_t num_coef;
    int32_t num_x;
    int32_t num_y;
    int32_t num_out;
    int32_t channels_x;
    int32_t channels_y;
    int32_t mode;           /* E3J_AMD_MODE_* of the forward pass */
    int32_t layout;         /* E3J_AMD_LAYOUT_* */
    int32_t val_dtype;      /* E3J_AMD_F32 / E3J_AMD_F64 / E3J_AMD_F16 */
    int32_t coef_idx_bytes; /* 1 or 4 */
    /* != 0: entries with equal output index are contiguous and the output indices ascend (the
     * order sparse_coo and Coef.transpose produce, src/e3j/utils/sparse.py:76-126,
     * src/e3j/ops/coef.py:174-184); every output coordinate is then written once.  0: any
     * order; the result is zero-filled first and runs are added. */
    int32_t coef_sorted;
    int32_t debug;
    int32_t signature;      /* id from e3j_amd_tp_find_signature, or -1: table-driven kernel */
    float   coef_scale;     /* unrolled kernels: table = coef_scale * built-in table */
    /* float64 with a signature: the E3J_AMD_F64_CLASSES coefficient classes that
     * e3j_amd_tp_find_signature_f64 returned for the table, in HOST memory (read during the call). */
    const double *coef_classes;
} e3j_amd_tp_params;
int e3j_amd_tensor_product_fwd(const e3j_amd_tp_params *p, const void *coef, const void *x, const void *y,
                               void *z, void *stream);
/* Cotangents dx (shape of x) and dy (shape of y) for the output cotangent dz.  `coef_bwd` holds
 * two tables of num_coef entries each, the forward table with its index columns permuted to
 * (j, i, k) and to (k, i, j) and sorted by the new first column
 * (src/e3j/ops/tensor_product.py:331-338); `p` describes the forward pass.  Coordinates of x or y
 * that no coefficient touches get zeros.  OUTER mode needs channels_x == 1 or channels_y == 1
 * (as the reference, src/e3j/ops/tensor_product.py:322-326); both layouts are served. */
int e3j_amd_tensor_product_bwd(const e3j_amd_tp_params *p, const void *coef_bwd, const void *x, const void *y,
                               const void *dz, void *dx, void *dy, void *stream);

/* Compile-time-unrolled kernels of the tensor product exist for built-in Clebsch-Gordan tables
 * and three channel modes, `kind` 0 MAP, 1 OUTER with channels_y == 1, 2 INNER: in the
 * trailing layout for the channel counts they were built for (32, 64, 128; float16 and float64
 * operands: 64, 128), in the leading layout (float32) for any multiple of 4 channels (kinds 1 and
 * 2, which sum over the channels: 64, 128 or 256), operands 16-byte aligned and num_rows *
 * channels >= 64.  The lookup compares a packed forward table in HOST memory (val_dtype
 * E3J_AMD_F32 or E3J_AMD_F16) with the built-in ones (same entries in the same order, up to one
 * positive factor returned in *coef_scale; half values within their rounding) and returns an id
 * for e3j_amd_tp_params.signature, or -1.  With a signature the `coef` / `coef_bwd` operands of
 * the two entry points above are not read and may be NULL.  No counterpart in the reference,
 * whose kernels are table-driven only. */
int e3j_amd_tp_find_signature(const void *coef_host, int32_t coef_idx_bytes, int32_t val_dtype,
                              int32_t num_coef, int32_t num_x, int32_t num_y, int32_t num_out,
                              int32_t channels, int32_t kind, int32_t layout, float *coef_scale);
/* The same for a table of float64 values.  The float64 kernels carry no coefficient values: they
 * read one value per class of entries that have one magnitude in the built-in table, so the
 * caller's table may hold any values of that structure (float32-rounded ones, exact ones, a
 * normalisation folded in), provided the entries of a class agree to float64 rounding and every
 * sign is the built-in one.  coef_classes: E3J_AMD_F64_CLASSES doubles, filled on a match; pass
 * them in e3j_amd_tp_params.coef_classes. */
int e3j_amd_tp_find_signature_f64(const void *coef_host, int32_t coef_idx_bytes, int32_t num_coef,
                                  int32_t num_x, int32_t num_y, int32_t num_out, int32_t channels,
                                  int32_t kind, int32_t layout, double *coef_classes);
int e3j_amd_tp_num_signatures(void);
const char *e3j_amd_tp_signature_name(int id);
/* Adds the kernels of one table compiled at run time (an entry produced by the generator of this
 * library, `e3j_amd/codegen/gen_tp.py`, living in a shared library that stays loaded); returns
 * its id or -1.  The counterpart of e3j_amd_register_signature for the tensor product. */
int e3j_amd_tp_register_signature(const void *entry);

/* XLA-FFI handlers (C ABI of xla/ffi/api/c_api.h): `XLA_FFI_Error* handler(XLA_FFI_CallFrame*)`.
 * Operand order of "convolution"/"convolution_bwd" as in lib/e3j_ops/ffi/e3j_ops.h:457-472,575-594;
 * attrs: num_nodes, debug (reference) + layout, signature (optional). */
void *e3j_amd_xla_convolution(void *call_frame);
void *e3j_amd_xla_convolution_bwd(void *call_frame);
void *e3j_amd_xla_convolution_bwd_receiver(void *call_frame);
void *e3j_amd_xla_convolution_bwd_ordered(void *call_frame);
/* "tensor_product" / "tensor_product_bwd" (lib/e3j_ops/ffi/e3j_ops.h:238-253,358-372): operands coef,
 * x, y [, coef_ranges] -> z and coef (two stacked tables), x, y, dz [, coef_ranges] -> dx, dy; attrs
 * num_out (forward), mode, layout, debug (reference) + signature, coef_scale, coef_sorted (optional). */
void *e3j_amd_xla_tensor_product(void *call_frame);
void *e3j_amd_xla_tensor_product_bwd(void *call_frame);

#ifdef __cplusplus
}
#endif
#endif /* E3J_AMD_H_ */
