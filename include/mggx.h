/*
 * mggx.h -- C ABI of libmggx.so: MGG's neighbor-partitioned GNN aggregation
 * path (NP-split SpMM + dense node update + row softmax) for AMD MI355X
 * (gfx950).  Plain pointers and sizes only; no HIP, torch or C++ types.
 *
 * MGG itself has no FFI: its path is a set of C++ free functions and param
 * classes in headers (include/neighbor_utils.cuh, layer_new.cuh,
 * gnn_layer.cuh of MGG_OSDI23).  The header-only C++ layer under
 * include/mgg/ re-creates those signatures and forwards to the entry points
 * below; each entry point names the reference function it stands in for.
 *
 * Conventions
 *   - every function returns 0 on success, a negative MGGX_E* code otherwise;
 *     mggx_last_error() gives the message of the calling thread's last error
 *     (the reference prints and exit()s: the C++ layer does that translation).
 *   - "d_" pointers are device (HBM) addresses, everything else is host memory.
 *   - node ids are int32 (`nidType = int`, neighbor_utils.cuh:15); element
 *     offsets are computed in 64 bits inside the kernels.
 *   - feature tables are row-major [rows x ld] with ld >= dim (the reference
 *     always has ld == dim).
 *   - all device work is issued on the stream set by mggx_set_stream()
 *     (default: the null stream) and is asynchronous unless stated; the dense-core path of the aggregation also uses a
 *     second stream of the library's own, forked from and joined to that stream by events inside the call, so every
 *     call is still ordered on the caller's stream as a whole.
 *   - after a first call of the same shape (which builds the cached plan and grows the library's scratch), the
 *     compute entry points only launch kernels -- no allocation, memset or synchronisation -- and may be captured
 *     into a HIP graph.  What a capture uses (plans, scratch blocks) is never freed or evicted before
 *     mggx_release_cached(); a call that would have to build a plan or grow the scratch while the stream is capturing
 *     returns MGGX_EINVAL instead (run it once outside the capture first).  mggx_sag_np_div_tune, the *_device
 *     preparation calls and first calls synchronise.
 *   - one host thread per device at a time; the library keeps per-process
 *     state (stream, workspace, plan cache) without locks, as MGG runs one
 *     host thread per GPU.
 */
#ifndef MGGX_H
#define MGGX_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MGGX_OK 0
#define MGGX_EINVAL (-1)   /* bad argument (shape, knob, NULL pointer) */
#define MGGX_EHIP (-2)     /* a HIP runtime call failed */
#define MGGX_ENOMEM (-3)   /* allocation failed */
#define MGGX_EIO (-4)      /* file could not be opened / short read */
#define MGGX_EFORMAT (-5)  /* file contents inconsistent */
#define MGGX_ELIMIT (-6)   /* size beyond what this entry point supports */

/* aggregation flags */
#define MGGX_AGG_ACCUMULATE 1u /* out += result (mgg_SAG_np_div never zeroes out, neighbor_utils.cuh:1458) */
#define MGGX_AGG_GIN 2u        /* out = (1+eps)*x_self + sum (mgg_GIN_np_div_cuda, neighbor_utils.cuh:1660-1665) */
#define MGGX_AGG_RELU 4u       /* max(0, .) applied after the sum (not in the reference; off by default) */
#define MGGX_AGG_SOFTMAX 8u    /* row softmax over the dim columns applied last, inside the kernels that finish a row: the
                                * aggregation and the softmax_forward that follows it in the reference's last layer
                                * (src/mgg_np_div_mem.cu:221-225, include/gnn_layer.cuh:36-40) as one call */

/* feature element types */
#define MGGX_F32 0
#define MGGX_BF16 1

const char *mggx_last_error(void);
const char *mggx_version(void);

/* ---- runtime (replaces the cudaSetDevice/cudaMalloc/cudaMemcpy/cudaFree calls
 *      of the reference mains, e.g. src/mgg_np_div_kernel.cu:86,116-153,223-228) ---- */
int mggx_init(int device);
int mggx_device_name(char *buf, size_t len);
int mggx_set_stream(void *hip_stream);
int mggx_sync(void);
int mggx_malloc(void **d_ptr, size_t bytes);
int mggx_free(void *d_ptr);
/* The two feature tables of an aggregation call (this rank's rows; the rows the reference reaches with remote GETs) out
 * of ONE allocation, the remote table right behind the local one (256-byte aligned).  Where the two tables of a call lie
 * is what decides how mggx_sag_np_div forms gather addresses: inside one window of under 2 GiB it uses 32-bit buffer
 * offsets, otherwise 64-bit addresses -- same sums, but two kernel variants.  With tables from this call the variant
 * is a function of their sizes, not of where an allocator happened to put two separate blocks.  Free with
 * mggx_free(*d_local); *d_remote is an interior pointer and must not be freed on its own. */
int mggx_malloc_tables(void **d_local, size_t local_bytes, void **d_remote, size_t remote_bytes);
int mggx_memset(void *d_ptr, int value, size_t bytes);
int mggx_memcpy_h2d(void *d_dst, const void *src, size_t bytes);
int mggx_memcpy_d2h(void *dst, const void *d_src, size_t bytes);
int mggx_memcpy_d2d(void *d_dst, const void *d_src, size_t bytes);
/* HIP-event stopwatch on the library's stream (replaces the commented cudaEvent
 * blocks, neighbor_utils.cuh:812-833). */
int mggx_timer_create(void **timer);
int mggx_timer_start(void *timer);
int mggx_timer_stop(void *timer);
int mggx_timer_elapsed_ms(void *timer, float *ms); /* synchronises on the stop event */
int mggx_timer_destroy(void *timer);
/* Frees the workspace and every cached plan (also what captured graphs may still point at: destroy those first). */
int mggx_release_cached(void);
/* Drops what the library remembers about the CSR array at this device address (cached partition plans, search
 * results): call it before freeing or rewriting an index array that aggregation calls have seen, when the memory is
 * not released through mggx_free (which does this itself) -- an allocator may hand the same address out again.
 * A caller that forgets to is still covered: cached records are found by address, but every kernel of a call first
 * compares the live edge counts of the arrays (ptr_l[rows], ptr_r[rows]) with the counts its records were built for
 * (level 1, the default: two scalar loads per kernel), and at level 2 a one-workgroup kernel on the call's stream also
 * compares a fingerprint of the arrays (their last entries and up to 512 entries of each at a fixed stride) with the
 * one taken when the record was made (about 8 microseconds per call).  On a mismatch every kernel of that call returns
 * at once (the output is left as it was, nothing is read through stale indices), and the next library call on this
 * thread, mggx_sync() included, drops the records and returns MGGX_EINVAL; calling again then works on the arrays as
 * they are.  Neither check sees an edit that keeps the edge counts and misses every sampled entry -- mggx_forget()
 * stays the rule for in-place edits.  mggx_set_plan_check(level): 0 = off, 1 = edge counts, 2 = edge counts and
 * fingerprint. */
int mggx_forget(const void *d_ptr);
int mggx_set_plan_check(int level);

/* What the library holds and what its set-up has cost so far (host clock, milliseconds, since the process started). */
typedef struct mggx_cache_stats_t {
    int64_t plans, plan_bytes;             /* cached partition plans (descriptors, row offsets) and their device bytes */
    int64_t core_plans, core_plan_bytes;   /* dense-core plans (ranking, index lists, remaining CSR) */
    int64_t workspace_bytes;               /* carry buffer and per-block partial rows */
    int64_t core_scratch_bytes;            /* staged core table and the partial rows of the core kernel's workgroups */
    int64_t retired_bytes;                 /* outgrown blocks kept because a captured graph may point at them */
    double plan_build_ms, core_plan_build_ms, search_ms;  /* search_ms excludes the plan builds inside the search */
} mggx_cache_stats_t;
int mggx_cache_stats(mggx_cache_stats_t *out);

/* ---- host-side graph preparation (CPU; replaces the host code of the path) ---- */

/* nodesPerPE = ceil(V/nGPU), lb = nodesPerPE*pe, ub = min(lb+nodesPerPE, V)
 * (src/mgg_np_div_kernel.cu:90-95). */
int mggx_range_partition(int num_nodes, int num_gpus, int pe, int *nodes_per_pe, int *lb, int *ub);

/* split_CSR<int> (include/neighbor_utils.cuh:381-405).  Call once with the four
 * output arrays NULL to get n_local/n_remote, then again with
 * local_ptr/remote_ptr sized (ub-lb)+1 and the column arrays sized as returned. */
int mggx_split_csr(const int *ptr, const int *col, int lb, int ub,
                   int *local_ptr, int *remote_ptr, int *local_col, int *remote_col,
                   int64_t *n_local, int64_t *n_remote);

/* Compact staging of the remote rows of a share (no counterpart in the reference, which issues one nvshmem GET per
 * remote neighbor, include/neighbor_utils.cuh:1432-1452; this is the list a pre-exchange of remote rows would fetch).
 * fetch_ids = the distinct ids of remote_col, most referenced first, ties by ascending id; remote_col_compact[e] =
 * position of remote_col[e] in fetch_ids.  Staging row i of the remote table = feature row fetch_ids[i]
 * (mggx_gather_rows) and passing remote_col_compact as d_col_r gives the same sums, from a table with one row per
 * distinct id and the hot rows packed together.  Call with both outputs NULL to get *n_unique first. */
int mggx_compact_remote(const int *remote_col, int64_t n_remote, int *remote_col_compact, int *fetch_ids,
                        int64_t *n_unique);

/* Layout of the dense-core path (no counterpart in the reference), exposed for inspection and tests: ranks the rows of
 * a local CSR by degree (ties by id), takes the first core_rows (rounded down to a multiple of 512) as the core, and
 * splits the CSR into the core x core block -- as index lists per 64-row slice and tile of tile_cols core columns
 * (256 in the library), lists of a slice padded to the longest, in chunks of 4:
 * idx[((blk_off[g * ntiles + t] + k / 4) * 64 + lane) * 4 + k % 4] = tile offset of a core neighbor of the row of rank
 * 64 g + lane inside tile t, or tile_cols + r (r < 16) for a padding slot: one of 16 zero columns the kernel keeps
 * behind a tile.  A block is in bank order: entries and padding slots of the 16 lanes of a group are placed so that, as
 * far as the lists allow, the 16 columns read at one position differ mod 16 (blocks of up to 256 positions) --
 * and the remaining CSR (rem_ptr, rem_col: row and edge order kept, ids unchanged).
 * build returns sizes[5] = {core rows, entries of blk_off, entries of idx, entries of rem_col, edges in the core block};
 * fetch copies the arrays out (any may be NULL) and releases the handle: order[core], rank[rows] (-1 outside the core),
 * blk_off, idx, rem_ptr[rows + 1], rem_col. */
int mggx_core_layout_build(const int *ptr, const int *col, int rows, int lb, int core_rows, int tile_cols, void **handle,
                           int64_t *sizes);
int mggx_core_layout_fetch(void *handle, int *order, int *rank, unsigned *blk_off, unsigned short *idx, int *rem_ptr,
                           int *rem_col);

/* The same layout as the aggregation itself builds it: on the GPU, from the device copy of the CSR (a stable radix sort
 * by degree, a counting pass, two prefix sums, a fill pass; only scalars travel to the host), bit-identical to
 * mggx_core_layout_build.  Builds (or finds) the cached dense-core plan of (d_ptr, d_col, rows, lb, core_rows), returns
 * sizes[5] as above and copies the arrays that are not NULL to host memory: call once with NULL arrays for the sizes.
 * Synchronises. */
int mggx_core_layout_device(const int *d_ptr, const int *d_col, int rows, int lb, int core_rows, int64_t *sizes, int *order,
                            int *rank, unsigned *blk_off, unsigned short *idx, int *rem_ptr, int *rem_col);

/* build_part<int> (include/neighbor_utils.cuh:411-460).  part_ptr has
 * num_parts+1 entries, part2node num_parts, node2part num_nodes+2 (the
 * reference's layout).  compat != 0 reproduces the reference's terminal entry
 * (left 0 when the last node has no neighbors); compat == 0 always writes
 * indptr[num_nodes] there.  NULL arrays: only *num_parts is produced. */
int mggx_build_part(const int *indptr, int num_nodes, int part_size, int compat,
                    int *part_ptr, int *part2node, int *node2part, int *num_parts);

/* Binary CSR triple of include/graph.hpp:9-130 as instantiated
 * graph<long,long,int,int,int,int>: <beg> int64[V+1], <csr> int64[E], <weight> int32[E].
 * Read: first call with NULL arrays returns the counts. */
int mggx_graph_read(const char *beg_file, const char *csr_file, const char *weight_file,
                    int *vert_count, int *edge_count, int *beg_pos, int *csr, int *weight);
int mggx_graph_write(const char *beg_file, const char *csr_file, const char *weight_file,
                     int vert_count, const int *beg_pos, const int *csr, const int *weight /* NULL: all 1 */);

/* MatrixMarket-style text loader, assemble_csr_matrix_new (include/csr_formatter.h:112-144).
 * First call with NULL arrays returns M (rows) and L (entries). */
int mggx_mtx_read(const char *path, int *num_rows, int *num_entries, int *row_ptr, int *col_ind);

/* Text edge list -> the binary CSR triple (<prefix>_beg_pos.bin, _csr.bin, _weight.bin).  Stands in for the
 * reference's dataset/0_to_base_zero.py + dataset/1_txt2bin.py, whose text_to_bin tool is not part of the reference
 * tree.  is_mtx != 0: MatrixMarket-style input (1-based, size line); else a 0-based "src dst" list.  Edges are grouped
 * by source, file order kept inside a row; weights are 1. */
int mggx_edgelist_to_bin(const char *path, int is_mtx, const char *out_prefix, int *num_nodes, int64_t *num_edges);

/* Deterministic synthetic graphs (no counterpart in the reference, which only
 * loads files).  Both produce a sorted, duplicate-free CSR of the symmetrised
 * graph with one self loop per node.  Two-call protocol: gen -> sizes, then
 * fetch copies the arrays out and releases the generator's storage.
 *   rmat: 2^scale id space trimmed to num_nodes by rejection; quadrant
 *         probabilities a,b,c (d = 1-a-b-c); num_draws undirected edges are
 *         drawn (duplicates and loops are dropped afterwards, so the distinct
 *         count is lower and is reported through nnz);
 *         scramble != 0 relabels ids with a seeded bijection.
 *         row_lo/row_hi: only rows in [row_lo,row_hi) are kept (a rank's share);
 *         pass 0,num_nodes for the whole graph.
 *   er:   G(n, p = avg_degree/(n-1)) over unordered pairs. */
int mggx_gen_rmat(int scale, int num_nodes, int64_t num_draws, double a, double b, double c,
                  uint64_t seed, int scramble, int row_lo, int row_hi, int threads,
                  void **handle, int64_t *nnz);
int mggx_gen_er(int num_nodes, double avg_degree, uint64_t seed, void **handle, int64_t *nnz);
int mggx_gen_fetch(void *handle, int *row_ptr /* rows+1 */, int *col /* nnz */);
/* N(0,1) / U[-1,1) / Glorot-uniform fills from the same counter-based generator. */
int mggx_fill_normal(float *dst, int64_t n, uint64_t seed);
int mggx_fill_uniform(float *dst, int64_t n, float lo, float hi, uint64_t seed);

/* ---- device-side neighbor partitioning ---- */

/* build_part on the GPU: d_indptr[num_nodes+1] -> the three arrays of
 * mggx_build_part, bit-identical (same compat switch).  Call with NULL output
 * arrays to get *num_parts (synchronises), then with arrays of the right size. */
int mggx_build_part_device(const int *d_indptr, int num_nodes, int part_size, int compat,
                           int *d_part_ptr, int *d_part2node, int *d_node2part, int *num_parts);

/* split_CSR on the GPU (include/neighbor_utils.cuh:381-405), bit-identical to mggx_split_csr: d_ptr/d_col are the
 * whole graph's CSR on the device.  Call once with the two column arrays NULL: fills d_local_ptr/d_remote_ptr
 * ((ub-lb)+1 entries each) and returns the totals (synchronises); then again with column arrays of those sizes. */
int mggx_split_csr_device(const int *d_ptr, const int *d_col, int lb, int ub, int *d_local_ptr, int *d_remote_ptr,
                          int *d_local_col, int *d_remote_col, int64_t *n_local, int64_t *n_remote);

/* mggx_compact_remote on the GPU (sort, run-length encode, sort by count, remap): d_remote_col is the device copy of
 * the remote column array; same two-call protocol, bit-identical outputs (device arrays).  Synchronises. */
int mggx_compact_remote_device(const int *d_remote_col, int64_t n_remote, int *d_remote_col_compact, int *d_fetch_ids,
                               int64_t *n_unique);

/* ---- aggregation ---- */

typedef struct mggx_agg_opts {
    uint32_t flags;              /* MGGX_AGG_* */
    float eps;                   /* GIN epsilon */
    int64_t ld_in;               /* row stride of in_local/in_remote in elements; 0 = dim */
    int64_t ld_out;              /* row stride of out in elements; 0 = dim */
    const float *d_row_scale_out;/* [ub-lb] multiplies each finished sum (NULL = 1) */
    int in_dtype;                /* MGGX_F32 or MGGX_BF16 (out is always fp32) */
    int col_block_rows;          /* column-blocked order: 0 = library decides, -1 = off, > 0 = neighbor ids per block */
    int core_rows;               /* dense core served from LDS: 0 = library decides, -1 = off, > 0 = rows in the core */
} mggx_agg_opts;

typedef struct mggx_agg_knobs {
    int ps, wpb, dist;           /* partSize / warpPerBlock / interleaved_dist */
    int col_block_rows;          /* > 0: column-blocked with that many ids per block; -1: plain order */
    int core_rows;               /* > 0: dense core of that many rows; -1: none */
} mggx_agg_knobs;

/* mgg_SAG_np_div / mgg_GIN_np_div (include/neighbor_utils.cuh:787-841, 902-958;
 * kernels :1351-1460, :1554-1667):
 *   out[v,:] (=|+=) sum_{u in N_local(v)} in_local[u - lb,:] + sum_{u in N_remote(v)} in_remote[u,:]
 * for v in [0, ub-lb).  d_in_remote is the table the reference reaches with
 * nvshmem GETs: row u = row (u % nodes_per_pe) of PE (u / nodes_per_pe), i.e.
 * the concatenation of all PEs' tables indexed by GLOBAL id; it may alias
 * d_in_local (single GPU) or be NULL when d_ptr_r is NULL / has no edges.
 * ps/wpb/dist are MGG's partSize / warpPerBlock / interleaved_dist: partitions
 * of <= ps neighbors of one row, wpb 64-lane wavefronts per workgroup, dist
 * consecutive partition rounds per wavefront.  They change speed, never the
 * mathematical result.  ps = 0, wpb = 0 and/or dist = 0 let the library choose (by rule, or
 * what mggx_sag_np_div_tune measured on the same arrays).  opts may be NULL (fp32, overwrite, ld == dim).
 * Column-blocked order (opts->col_block_rows): for a local-only CSR whose rows are sorted by neighbor id and long
 * (>= 20 neighbors per block and row), the partitions are walked block by block of neighbor ids, so the part of the
 * feature table in use at any time is small enough to stay in cache; each block leaves a partial row in library
 * scratch and a second kernel sums them in block order and applies the epilogue.  Same result up to summation order.
 * Dense core (opts->core_rows; fp32, local-only CSR, dim <= 64): the core_rows highest-degree rows (rounded down to a
 * multiple of 512) are ranked by degree; the edges among them leave the CSR and are summed from LDS -- the feature rows
 * of 256 core columns at a time staged with whole-line reads, one lane per core row walking an index list -- and the
 * rest of the CSR runs as usual on top.  Pays on graphs whose high-degree rows hold most edges among themselves; its
 * plan is built on the GPU on first use (milliseconds).  The core block runs on a second stream of the library's, forked from and joined to the
 * caller's stream by events inside the call (LDS-bound work beside cache-bound work).  Same result up to summation order.
 * With core_rows = 0 the library picks the size itself (possibly none) from the degree histogram: it grows the core
 * while the predicted padding of the added rows' index lists costs less than the gathers they remove.
 * MGGX_AGG_SOFTMAX (fp32 tables): the finished rows leave as their row softmax, on every path above.
 * The partition plan of (d_ptr_l, d_ptr_r, d_col_r, rows, ps) -- and d_col_l for the column-blocked order -- is built on
 * first use and cached by pointer identity.  The arrays stay the caller's: what happens when they are rewritten in
 * place or their address is reused is described at mggx_set_plan_check (mggx_forget() drops what hangs on one array,
 * mggx_release_cached() everything). */
int mggx_sag_np_div(float *d_out, const void *d_in_local, const void *d_in_remote,
                    const int *d_ptr_l, const int *d_col_l, const int *d_ptr_r, const int *d_col_r,
                    int lb, int ub, int dim, int nodes_per_pe,
                    int ps, int wpb, int dist, const mggx_agg_opts *opts);

/* The design-space search of bench_MGG_DSE_dist_ps.py:12-42 / bench_MGG_DSE_dist_wpb.py (one process launch per
 * setting there) as one call: runs the aggregation of mggx_sag_np_div over ps (as given, or {16, 32} when 0) x plain /
 * column-blocked order (where the rows are long enough, unless opts fixes it) x without a dense core / with one of
 * 32, 40, 48, 64 or 80 Ki rows (where eligible, unless opts fixes it) x wpb in {4, 8, 16} x dist in
 * {1, 2, 4, 8, 16} -- one untimed and two timed calls back to back per setting; the four fastest settings and the setting
 * the library's own rules and cost model would pick then meet again, twice over eight calls each, the faster of the two
 * counting (a plan built a moment ago runs slower for its first calls) -- returns the fastest setting and its time (ms
 * per call in that last round), and
 * remembers it, so later mggx_sag_np_div calls on the same CSR arrays with the same dim and in_dtype that leave
 * wpb = dist = col_block_rows = core_rows = 0 (and ps = 0 or the winning ps) use it.  d_out holds a valid result afterwards.
 * Synchronises; not for stream capture.  MGGX_AGG_ACCUMULATE is rejected (the repeated runs would add up).
 * Either out-pointer may be NULL. */
int mggx_sag_np_div_tune(float *d_out, const void *d_in_local, const void *d_in_remote,
                         const int *d_ptr_l, const int *d_col_l, const int *d_ptr_r, const int *d_col_r,
                         int lb, int ub, int dim, int nodes_per_pe, int ps, const mggx_agg_opts *opts,
                         mggx_agg_knobs *best, float *ms_best);

/* SAG_host / SAG_cuda_kernel (include/neighbor_utils.cuh:463-506, 2373-2447) and
 * the local half of SAG_host_fused_interleaved (:593-676, 2598-2688): explicit
 * partition arrays from build_part; out[part2node[p],:] += sum over the
 * partition of in[col - lowbound,:].  Accumulates, as the reference does.
 * Partition lengths are taken from d_row_ptr (so the reference's missing
 * terminal part_ptr entry cannot drop the last partition). */
int mggx_sag_parts(float *d_out, const float *d_in, const int *d_row_ptr, const int *d_col,
                   const int *d_part_ptr, const int *d_part2node,
                   int lowbound, int num_nodes, int num_parts, int ps, int dim, int wpb, int dist);

/* mggx_sag_parts for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments, same result bit for bit, but the
 * call allocates nothing and caches nothing: the partition descriptors, the per-row offsets and the carry buffer of the
 * call live in a fixed array of MGGX_STATIC_SCRATCH_BYTES that is part of the library's device code (every GPU the
 * library runs on holds its own copy until the process ends; its address is looked up once per device, in mggx_init or
 * on the first call there).  A call whose 16 bytes per partition + 4 bytes per row + carry buffer (two partial rows per
 * workgroup) do not fit returns MGGX_ELIMIT.  The call only launches kernels on the library's stream -- no allocation,
 * no memset, no copy to the host, no synchronisation.  Every call on a GPU uses that GPU's one array: calls that may
 * overlap on one GPU (two streams, two host threads) race; issue them on one stream.
 * Cost: the array is part of the library's code object, so every process that loads the library holds it on every GPU it
 * touches (64 MiB per process and GPU by default), whether or not this entry point is ever called; a build for many
 * processes per GPU can shrink it with -DMGGX_STATIC_SCRATCH_BYTES=<bytes> (the limit a call meets is the built library's).
 * If the array's address cannot be looked up, mggx_init still succeeds and only this entry point returns the error. */
#ifndef MGGX_STATIC_SCRATCH_BYTES
#define MGGX_STATIC_SCRATCH_BYTES (64u << 20)
#endif
int mggx_sag_parts_static(float *d_out, const float *d_in, const int *d_row_ptr, const int *d_col,
                          const int *d_part_ptr, const int *d_part2node,
                          int lowbound, int num_nodes, int num_parts, int ps, int dim, int wpb, int dist);

/* SpMM_cuda_kernel via sparse_beg_forward / sparse_hidden_forward
 * (include/gnn_kernel.cuh:9-71, gnn_layer.cuh:86-161): whole graph on one GPU,
 * out[v,:] += sum_{u in N(v)} in[u,:].  ps = 0 / wpb = 0 let the library choose; the rounds per wavefront and the
 * partition order follow the same rules as mggx_sag_np_div. */
int mggx_spmm(float *d_out, const float *d_in, const int *d_row_ptr, const int *d_col,
              int num_nodes, int dim, int ps, int wpb);

/* ---- dense node update and softmax ---- */

typedef struct mggx_dense_opts {
    int64_t ld_x;                /* 0 = d1 */
    int64_t ld_out;              /* 0 = d2 */
    const float *d_row_scale;    /* [n] multiplies each output row (NULL = 1) */
    uint32_t relu;               /* max(0,.) epilogue (not in the reference) */
} mggx_dense_opts;

/* dense_beg_forward / dense_hidden_forward / *_new_forward
 * (include/gnn_layer.cuh:22-52; geometry layer_new.cuh:222-229): the column-major
 * cublasSgemm(N,N,m=d2,n=rows,k=d1) == row-major Out[n x d2] = X[n x d1] . W[d1 x d2],
 * alpha 1, beta 0, fp32, on MFMA. */
int mggx_dense_xw(float *d_out, const float *d_x, const float *d_w, int64_t n, int d1, int d2,
                  const mggx_dense_opts *opts);

typedef struct mggx_mlp2_opts {
    int64_t ld_x;                /* 0 = d1 */
    int64_t ld_out;              /* 0 = d3 */
    const float *d_row_scale;    /* [n] multiplies each output row (NULL = 1) */
    uint32_t relu_mid;           /* max(0,.) between the two products */
    uint32_t relu_out;           /* what follows the second product and the row scale: 0 nothing, 1 max(0,.),
                                  * 2 the row softmax over the d3 columns (softmax_new_forward, include/gnn_layer.cuh:36-40,
                                  * as the last call of a forward: the logits never make a round trip through memory) */
} mggx_mlp2_opts;

/* Two consecutive updates in one pass, Out[n x d3] = act(X[n x d1] . Wa[d1 x h]) . Wb[h x d3], fp32 on MFMA: what two
 * dense_hidden_forward calls (include/gnn_layer.cuh:28-33) compute, without writing and re-reading the n x h
 * intermediate (a GIN layer's 2-layer MLP).  h <= 64, d3 <= 64 and both matrices must fit in LDS; otherwise
 * MGGX_ELIMIT is returned and the caller issues two mggx_dense_xw calls. */
int mggx_mlp2_xw(float *d_out, const float *d_x, const float *d_wa, const float *d_wb, int64_t n, int d1, int h, int d3,
                 const mggx_mlp2_opts *opts);

/* The same update on the bf16 matrix cores (no counterpart in the reference, which is fp32 only): W is bf16
 * [d1 x d2]; X is fp32 (rounded to bf16, nearest even, inside the kernel) or bf16 (x_dtype); products are
 * accumulated in fp32; Out is fp32 or bf16 (out_dtype).  Strides are in elements of the respective type. */
int mggx_dense_xw_bf16(void *d_out, const void *d_x, const void *d_w_bf16, int64_t n, int d1, int d2,
                       int x_dtype, int out_dtype, const mggx_dense_opts *opts);

/* softmax_forward / softmax_new_forward (include/gnn_layer.cuh:15-20,36-40):
 * cudnnSoftmaxForward(ACCURATE, MODE_CHANNEL) on (n, c, 1, 1) == stable row
 * softmax.  In place (d_out == d_in) is allowed. */
int mggx_softmax_rows(float *d_out, const float *d_in, int64_t n, int c, int64_t ld_in, int64_t ld_out);

/* d_dst row i = d_table row d_ids[i], i < n; rows of row_bytes bytes (a multiple of 16, both tables 16-byte aligned):
 * stages a compact remote table from a table indexed by global id. */
int mggx_gather_rows(void *d_dst, const void *d_table, const int *d_ids, int64_t n, size_t row_bytes);

/* fp32 -> bf16 (round to nearest even) for staging bf16 feature tables. */
int mggx_cast_f32_to_bf16(void *d_dst, const float *d_src, int64_t n);

/* Plain device copy kernel of n bytes (n % 16 == 0): the known-size yardstick the
 * profiler's HBM byte counters are scaled against. */
int mggx_copy_bytes(void *d_dst, const void *d_src, size_t n);
/* The same copy as one workgroup per 16 KiB with non-temporal loads and stores, four loads in flight per thread: a
 * second copy kernel, so the copy ceiling quoted beside the bandwidth-bound kernels does not rest on one variant. */
int mggx_copy_bytes_nt(void *d_dst, const void *d_src, size_t n);

/* Yardstick for a 2 : 1 read / write stream (no counterpart in the reference): n fp32 values (n % 8 == 0, both arrays on
 * 16-byte boundaries) to bf16 by truncation, 32 bytes in and 16 bytes out per lane with the streaming hint, in pieces of
 * 2048 values.  persistent_workgroups = 0: workgroups in launch order, each converting pieces_per_workgroup consecutive
 * pieces one after the other; > 0: that many workgroups striding over all pieces.  What the dense update's access
 * pattern is measured against: the order in which the chip walks through memory decides 6.2 against 5.1 TB/s. */
int mggx_convert_probe(void *d_dst, const float *d_src, int64_t n, int pieces_per_workgroup, int persistent_workgroups);

/* Yardstick for row gathers (no counterpart in the reference): at least n_gathers loads of row_bytes bytes (16..256, in
 * 16-byte pieces) from rows at pseudo-random indices of a table of `rows` rows with a stride of ld_bytes, eight loads in
 * flight per lane group, no index array and no reduction; *n_done (optional) receives the exact number issued.  d_sink
 * must hold 262144 floats (one sum per thread, so the loads are not optimised away).  What this sustains on a table of
 * a given size is the ceiling the aggregation kernels are measured against where their table is cache resident. */
int mggx_gather_probe(float *d_sink, const void *d_table, int64_t rows, size_t ld_bytes, size_t row_bytes,
                      int64_t n_gathers, unsigned seed, int64_t *n_done);

/* Yardstick for the dense-core kernel (no counterpart in the reference): at least n_reads row reads of row_bytes bytes
 * (16..256, in 16-byte pieces) from an LDS tile of 256 columns laid out like that kernel's, at pseudo-random columns,
 * one row per lane and step, summed in registers; no memory traffic inside the loop.  d_sink as for mggx_gather_probe.
 * What this sustains is the ceiling of the core x core block's sums. */
int mggx_lds_probe(float *d_sink, size_t row_bytes, int64_t n_reads, unsigned seed, int64_t *n_done);

/* How the aggregation kernels address feature rows: 0 (default) picks per call -- 32-bit buffer offsets when both
 * tables lie inside one window of < 2 GiB and < 2^24 rows, 64-bit addresses otherwise; 1 always uses 64-bit
 * addresses.  Results are identical; the switch exists for tests and measurements. */
int mggx_set_gather_addressing(int mode);

/* Name and launch count of the aggregation kernel the last mggx_sag_np_div /
 * mggx_sag_parts / mggx_spmm call dispatched (for matching profiler rows). */
int mggx_last_agg_kernel(char *buf, size_t len);

#ifdef __cplusplus
}
#endif
#endif /* MGGX_H */
