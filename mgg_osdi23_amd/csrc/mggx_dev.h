// Device-side internals of libmggx.so (HIP translation units only).
#ifndef MGGX_DEV_H
#define MGGX_DEV_H

#include <hip/hip_runtime.h>

#include <list>
#include <vector>

#include "mggx_internal.h"

#define MGGX_HIP(call)                                                                               \
    do {                                                                                             \
        hipError_t e_ = (call);                                                                      \
        if (e_ != hipSuccess)                                                                        \
            return mggx::fail(MGGX_EHIP, "%s failed: %s (%s:%d)", #call, hipGetErrorString(e_),      \
                              __FILE__, __LINE__);                                                   \
    } while (0)

#define MGGX_LAUNCH_CHECK(name)                                                                      \
    do {                                                                                             \
        hipError_t e_ = hipGetLastError();                                                           \
        if (e_ != hipSuccess)                                                                        \
            return mggx::fail(MGGX_EHIP, "launch of %s failed: %s", name, hipGetErrorString(e_));    \
    } while (0)

namespace mggx {

// Partition descriptor consumed by the aggregation kernels, one per neighbor
// partition, in row-major order with a row's local partitions before its
// remote ones.
//   x: first edge index inside col_l / col_r; bit 31 set = remote side
//   y: destination row (0-based inside the share)
//   z: number of neighbors (1..ps) | FIRST<<30 | LAST<<31
//   w: unused (0)
static constexpr unsigned DESC_REMOTE = 0x80000000u;
static constexpr unsigned DESC_FIRST = 0x40000000u;  // first partition of its row
static constexpr unsigned DESC_LAST = 0x80000000u;   // last partition of its row
static constexpr unsigned DESC_LEN_MASK = 0x3FFFFFFFu;

// Content checks of the caller's CSR arrays behind a cached record.  The records are found by device address, and an
// address says nothing about what is stored there now (arrays rewritten in place, memory freed through another allocator
// and handed out again).  Two checks, both on the device, so that a call stays asynchronous:
//   edge counts (level 1, default)  every kernel of a call first compares the arrays' live edge counts -- ptr_l[rows],
//                                   ptr_r[rows], two scalar loads -- with the counts its records were built for;
//   fingerprint (level 2)           before the call's kernels, a one-workgroup kernel takes a fingerprint of the arrays
//                                   (their last entries and up to 512 entries of each at a fixed stride), compares it
//                                   with the one stored when the record was made and writes the verdict to a word
//                                   every kernel of the call reads first (about 8 us per call).
// A kernel that finds its gate closed returns at once: a stale plan never produces sums or reads through stale indices.
// The mismatch also goes to a host-visible word; the next library call reports it as MGGX_EINVAL after dropping the
// records of those arrays.
struct Gate {
    const int *ok = nullptr;     // level 2: verdict word of the fingerprint kernel (0 = stale)
    const int *cnt_l = nullptr;  // level 1: &ptr_l[rows] of the caller's CSR ...
    const int *cnt_r = nullptr;  //          ... and &ptr_r[rows] (NULL: no remote side)
    int want_l = 0, want_r = 0;  //          the edge counts the records were built for
    volatile int *flag = nullptr;
    int tag = 0;
};

__device__ __forceinline__ bool gate_closed(const Gate &g)
{
    if (g.ok && *g.ok == 0) return true;
    if (g.cnt_l) {
        const bool bad = *g.cnt_l != g.want_l || (g.cnt_r && *g.cnt_r != g.want_r);
        if (bad) {
            *g.flag = g.tag;
            return true;
        }
    }
    return false;
}

struct Guard {
    const int *arr[4] = {nullptr, nullptr, nullptr, nullptr};  // fingerprinted arrays ...
    long long len[4] = {0, 0, 0, 0};                           // ... and their lengths
    const int *cnt_l = nullptr, *cnt_r = nullptr;              // where the live edge counts are
    int want_l = 0, want_r = 0;
    unsigned long long *d_fp = nullptr;  // device: [0] fingerprint, [1] verdict word (as int) -- one 16-byte allocation
    int id = 0;                          // reported through the host flag on a mismatch
    bool armed = false;
    const int *ok() const { return reinterpret_cast<const int *>(d_fp + 1); }
};

struct Plan {
    // cache key
    const int *d_ptr_l = nullptr;
    const int *d_ptr_r = nullptr;
    const int *d_part_ptr = nullptr;   // explicit-partition plans only
    const int *d_part2node = nullptr;  // explicit-partition plans only
    int rows = 0;
    int ps = 0;                  // the caller's partition size (MGG's partSize)
    int caller_parts = 0;        // explicit-partition plans: the caller's partition count (part of the cache key)
    // What a slot of the kernel sums at a time: for ps >= 16 one partition; for smaller ps the largest whole number of
    // consecutive partitions of one row and side with at most 16 neighbors between them (unit = ps * floor(16 / ps)
    // neighbors).  Consecutive partitions of a row are consecutive edges, so such a group is one edge range: one
    // descriptor and one slot instead of up to 16, each one sixteenth full.  The reference's kernel only ever sees
    // dist * ps neighbors per warp (neighbor_utils.cuh:1395-1398); the summation order stays a function of the knobs.
    int unit = 0;
    // contents (device)
    int4 *d_desc = nullptr;      // [num_parts] one per unit
    int *d_off = nullptr;        // [rows+1] first descriptor of each row
    int *d_empty_rows = nullptr; // rows without any partition
    int num_parts = 0;
    int num_empty = 0;
    int64_t nnz_l = 0, nnz_r = 0;
    int max_col_r = -1;        // largest remote neighbor id (bounds the remote table)
    // Column-blocked plans: the neighbor ids [lb, lb + real_rows) are cut into `blocks` ranges of `block_rows` ids and
    // `rows` = blocks * real_rows virtual rows; virtual row c * real_rows + v holds row v's neighbors inside block c,
    // so the descriptor order walks the feature table block by block.  Plain plans: blocks == 1, rows == real_rows.
    const int *d_col_l = nullptr;  // cache key of blocked plans (they depend on the column values)
    const int *d_col_r = nullptr;  // cache key of plans with remote edges (max_col_r depends on the values)
    int real_rows = 0;
    int block_rows = 0;
    int block_lb = 0;          // id of the first row of block 0 (part of the cache key)
    int blocks = 1;
    bool unsuitable = false;   // blocked plan asked for, but the rows are not sorted by neighbor id
    bool pinned = false;       // used inside a stream capture: a captured graph holds its device addresses, so its device
                               // blocks are never freed before mggx_release_cached (dropped from the cache, they are retired)
    int graph_serial = 0;      // the graph record (GraphInfo::serial) this plan was built under; a call under another record
                               // of the same addresses -- the arrays may hold another graph now -- rebuilds it
    size_t bytes = 0;          // device memory held
    Guard guard;               // explicit-partition plans only (the others are guarded through their GraphInfo)
};

// Scratch layout of the dense core.  Staged table: slice s of the rank-i node's row at tab[s * tab_stride(core) + i]; the
// stride carries a few rows more than the core size: with a power-of-two core the slices of a tile would otherwise all
// start in the same memory channel.  Partial rows: one per workgroup of the LDS kernel and row of its row group, at
// partial[(slot * group_rows + rank % group_rows) * n4 + piece]; the slots of row group g are
// wg_base[g] .. wg_base[g + 1] - 1.
__host__ __device__ inline size_t tab_stride(int core) { return (size_t)core + 16; }
constexpr int CORE_GROUP_ROWS = 256;  // core rows per workgroup of the LDS kernel (4 wavefronts, one row per lane) ...
constexpr int CORE_GROUP_ROWS_WIDE = 512;  // ... and where rows are summed in two halves (CorePlan::group_rows)
static_assert(CORE_GROUP_ROWS == 1 << 8 && CORE_GROUP_ROWS_WIDE == 1 << 9, "the kernels that finish rows shift by 8 or 9");
// Wide groups where rows are summed in halves and the staged table is well beyond an L2 (12 MB = three of them): every
// row group re-reads that table once per call.  Held against graphs of width 64 that the setting was not read off: cores
// of 16.8-21 MB gain 3-7 %, one of 10.5 MB lost 7 % with wide groups (profiles/rules_on_held_out_graphs.md).
inline int core_group_rows(int n4, int core_rows)
{
    return n4 > 12 && (size_t)core_rows * (size_t)n4 * 16 > ((size_t)12 << 20) ? CORE_GROUP_ROWS_WIDE : CORE_GROUP_ROWS;
}

// Dense-core plan of a local-only CSR (layout: CoreLayout in mggx_internal.h), built on the GPU and kept there.
struct CorePlan {
    // cache key
    const int *d_ptr_l = nullptr;
    const int *d_col_l = nullptr;
    int rows = 0, lb = 0, asked = 0;
    int group_rows = CORE_GROUP_ROWS;  // core rows per workgroup of the LDS kernel: 256 or 512
    // contents
    int core = 0, ntiles = 0;
    int64_t core_nnz = 0, rem_nnz = 0;
    int *d_order = nullptr, *d_rank = nullptr;
    unsigned *d_blk_off = nullptr;
    unsigned short *d_idx = nullptr;
    int *d_rem_ptr = nullptr, *d_rem_col = nullptr;
    // Workgroups of the LDS kernel: every row group's tiles cut into runs of about equal work.  How many runs pays depends
    // on the row width (narrow rows: many short ones; wide rows: fewer, their partial rows are dearer), so a plan holds
    // one table per number asked for, made from `work` when first needed.
    struct Cut {
        int target = 0;            // workgroups asked for
        int nwg = 0;               // workgroups made
        int4 *d_wgs = nullptr;     // [nwg] {row group, first tile, end tile, slot of the partial rows}, in launch order
        int *d_wg_base = nullptr;  // [core / CORE_GROUP_ROWS + 1] first slot of every row group
    };
    std::vector<Cut> cuts;
    std::vector<int> work;    // [core / CORE_GROUP_ROWS][ntiles] list chunks of a row group in a tile (host copy)
    long long total_chunks = 0;
    bool unsuitable = false;  // no core of whole units fits, or the ids do not allow it
    bool pinned = false;      // used inside a stream capture: its device blocks outlive the cache entry (retired, not freed)
    int graph_serial = 0;     // as Plan::graph_serial
    size_t bytes = 0;         // device memory held
};

// What is known about a CSR the aggregation has been called with (keyed by pointer identity).
struct GraphInfo {
    const int *d_ptr_l = nullptr;
    const int *d_ptr_r = nullptr;
    const int *d_col_l = nullptr;
    const int *d_col_r = nullptr;
    int rows = 0;
    // degree profile for the dense-core cost model: sum of the degrees of ranks [64 s, 64 s + 64) for the 2048 highest-degree
    // slices (rows ranked by falling degree), fetched once per record
    std::vector<float> slice_deg;
    bool have_profile = false;
    struct Predicted { int dim; int block_rows; unsigned long long table_bytes; int core_rows; };
    std::vector<Predicted> predicted;  // what the cost model said for a row width (evaluated once, a millisecond of host time)
    bool internal = false;  // arrays owned by the library (the remainder CSR of a dense-core plan): no content check
    bool pinned = false;    // used inside a stream capture: never evicted
    int serial = 0;         // unique per record: plans remember the record they were built under
    Guard guard;
    int64_t nnz_l = 0, nnz_r = 0;
    // knobs measured best by mggx_sag_np_div_tune for a row width and element type; used where a call passes 0
    struct Tuned { int dim, dtype, ps, wpb, dist, block_rows, core_rows; };
    std::vector<Tuned> tuned;
};

struct State {
    int device = -1;
    hipStream_t stream = nullptr;
    void *ws = nullptr;
    size_t ws_bytes = 0;
    std::vector<Plan *> plans;
    std::list<GraphInfo> graphs;  // least recently used first; a list, so records stay where they are while others come and go
    std::vector<CorePlan *> cores;
    void *core_ws = nullptr;      // staged core table and partial rows of the dense-core path (grow-only)
    hipStream_t side_stream = nullptr;  // the core block runs here, beside the rest of the CSR on `stream`
    hipEvent_t side_fork = nullptr, side_join = nullptr;
    size_t core_ws_bytes = 0;
    char last_kernel[224] = "";
    int gather_addressing = 0;  // 0 = choose per call, 1 = always 64-bit addresses
    // content checks of cached records (Guard)
    int plan_check = 1;            // 0: checks off (the caller vouches for its arrays), 1: live edge counts, 2: + fingerprint kernel
    volatile int *h_stale = nullptr;  // pinned host word the check kernel writes a record id to on a mismatch
    int next_guard_id = 1;
    int next_graph_serial = 1;
    // blocks a captured graph may still point at: kept until mggx_release_cached instead of being freed on growth
    bool ws_captured = false, core_ws_captured = false;
    std::vector<void *> retired;
    size_t retired_bytes = 0;
    // host-clock time spent on set-up so far (mggx_cache_stats)
    double plan_build_ms = 0.0, core_plan_build_ms = 0.0, search_ms = 0.0;
};

State &state();
int ensure_init();
// Grow-only scratch owned by the library; valid until the next call that grows it.
int workspace(size_t bytes, void **p);

// d_out[0..n] = exclusive prefix sum of d_in[0..n) (d_out has n+1 entries); the
// total is also copied to *total_host when non-NULL (synchronises).
int exclusive_scan_i32(const int *d_in, int *d_out, int n, long long *total_host);

// True while the library's stream is being captured into a HIP graph.
bool capturing();
// Content checks (see Gate).  guard_arm stores the fingerprint of a new record; guard_check builds the gate of a call from
// the record (and, at level 2, takes the fingerprint again on the stream); stale_poll reports a mismatch an earlier call
// found (MGGX_EINVAL, after dropping the records) -- called on entry of every compute call and by mggx_sync.
int guard_arm(Guard &g);
int guard_check(Guard &g, Gate *gate);
// `retire`: a captured graph may still launch the check kernel that writes this record's verdict word -- the word is kept
// until mggx_release_cached instead of being freed.
void guard_free(Guard &g, bool retire = false);
// Hands a device block a captured graph may still point at to the list mggx_release_cached frees.
void retire_block(void *p, size_t bytes);
int stale_poll();
// graph_serial: GraphInfo::serial of the call's graph record; a cached plan built under another record is rebuilt.
int plan_get(const int *d_ptr_l, const int *d_ptr_r, const int *d_col_r, int rows, int ps, int graph_serial, Plan **out);
// Column-blocked plan of a local-only CSR; (*out)->unsuitable is set when the rows are not sorted by neighbor id.
int plan_get_blocked(const int *d_ptr_l, const int *d_col_l, int rows, int lb, int ps, int block_rows, int graph_serial, Plan **out);
int graph_info(const int *d_ptr_l, const int *d_ptr_r, const int *d_col_l, const int *d_col_r, int rows, bool internal, GraphInfo **out);
int plan_get_explicit(const int *d_row_ptr, const int *d_part_ptr, const int *d_part2node, int rows,
                      int num_parts, int ps, Plan **out);
// Neighbors per kernel slot for a partition size (see Plan::unit).
inline int unit_of(int ps) { return ps >= 16 ? ps : ps * (16 / ps); }
// Explicit partition arrays -> unit descriptors and the first unit of each row, into caller-provided device arrays, with
// kernels on the library's stream only.  Partitions per unit g = unit_of(ps) / ps.  g == 1: one descriptor per partition,
// d_tmp unused.  g > 1: d_tmp holds explicit_tmp_ints(rows) ints of scratch; the number of units stays on the device
// (d_off[rows]) and *units_bound receives a host-side upper bound for it.
size_t explicit_tmp_ints(int rows);
int explicit_desc_fill(const int *d_row_ptr, const int *d_part_ptr, const int *d_part2node, int rows, int num_parts, int ps,
                       int4 *d_desc, int *d_off, int *d_tmp, long long *units_bound);
// d_out[0..n] = exclusive prefix sum of d_in[0..n) with caller-provided scratch of scan_tmp_bytes(n) bytes: three kernels on
// the library's stream, no allocation, no copy, no synchronisation (the total is d_out[n])
size_t scan_tmp_bytes(int n);
int exclusive_scan_i32_device(const int *d_in, int *d_out, int n, void *d_tmp);
// Device address of the static scratch array of mggx_sag_parts_static on the current device.
int static_scratch_ptr(unsigned char **out);
void plan_free(Plan *p);
int forget_pointer(const void *d_ptr);
int core_plan_get(const int *d_ptr_l, const int *d_col_l, int rows, int lb, int core, int group_rows, int graph_serial, CorePlan **out);
// Cost model of the dense core (degree histogram x row width): the core size that is predicted to pay for this CSR, a
// multiple of 4096, or -1 for none.  table_bytes = rows x row pitch of the feature table.  Fetches the record's degree
// profile on first use (one sort of the degrees on the device, 4 KiB to the host; synchronises).
// block_rows: the column-block size the call would use for this CSR (> 0), or <= 0 where it is not eligible for the
// column-blocked order; min_per_row_block: neighbors per row and block a CSR needs for that order (what the core leaves is
// held to the same bar).
int predict_core_rows(GraphInfo &g, int dim, unsigned long long table_bytes, int block_rows, int min_per_row_block, int *core_rows);
void core_plan_free(CorePlan *p);
int run_core_stage(CorePlan *p, const float *d_in, int dim, long long ld_in, const Gate &gate, hipStream_t stream);
int run_core_sums(CorePlan *p, int dim, const Gate &gate, hipStream_t stream);
int run_core_finish(CorePlan *p, float *d_out, int dim, long long ld_out, const float *d_row_scale, int relu, int softmax, const Gate &gate,
                    hipStream_t stream);
// Where run_core_sums leaves the core block's sums: [slot][row in its group][ceil(dim/4)] float4, and the first slot of
// every row group (CorePlan::Cut::d_wg_base of the cut used for this width).
int core_row_sums(CorePlan *p, int dim, const float4 **sums);
// Second stream of the dense-core path (created on first use, default priority) and the two events that fork and join it.
int core_side_stream(hipStream_t *stream, hipEvent_t *fork, hipEvent_t *join);

}  // namespace mggx
#endif
