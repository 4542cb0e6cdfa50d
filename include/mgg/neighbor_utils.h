// Host API of MGG's neighbor-partitioned aggregation, source-compatible with
// MGG_OSDI23 include/neighbor_utils.cuh: split_CSR (:381-405), build_part
// (:411-460), mgg_SAG_np_div (:787-841), mgg_GIN_np_div (:902-958), SAG_host
// (:463-506), SAG_host_fused_interleaved (:593-676).  Plain C++ over the libmggx
// C ABI: no device header is included here.
//
// One GPU runs one rank's share.  The rows other ranks own, which the reference
// pulls with NVSHMEM GETs from the same symmetric address on the owning PE, are
// read from a table staged in this GPU's memory: mgg_stage_remote(d_table)
// registers it (row u of the table = global node u, i.e. the ranks' buffers
// back to back).  Without a staged table the input buffer itself is used, which
// is exact for a single-rank run.
#ifndef MGG_NEIGHBOR_UTILS_H
#define MGG_NEIGHBOR_UTILS_H

#include <cstdio>
#include <cstdlib>
#include <string>
#include <type_traits>
#include <vector>

#include "mgg/utils.h"
#include "mggx.h"

#define WARP_SIZE 64  // lanes of a gfx950 wavefront (the reference's 32-lane warp, neighbor_utils.cuh:13)
using nidType = int;

struct mgg_runtime_options {
    const void *remote_table = nullptr;  // global-id-indexed feature table; nullptr = the input buffer
    bool accumulate = true;              // mgg_SAG_np_div adds into `output` as the reference does (:1458)
    bool synchronize = true;             // the reference waits for the device after every call (:835)
    int col_block_rows = 0;              // column-blocked partition order: 0 = library decides, -1 = off, N = ids per block
    int core_rows = 0;                   // dense core served from LDS: 0 = library decides, -1 = off, N = rows in the core
    bool softmax = false;                // mgg_SAG_np_div ends in the row softmax of the last layer (softmax_forward folded in)
};
inline mgg_runtime_options &mgg_options()
{
    static mgg_runtime_options o;
    return o;
}
inline void mgg_stage_remote(const void *d_table) { mgg_options().remote_table = d_table; }

// Rows [lb,ub) of a CSR split into the neighbors inside the range and those
// outside it; returns {local_ptr, remote_ptr, local_col_idx, remote_col_idx}.
template <typename T>
std::vector<std::vector<T>> split_CSR(std::vector<T> &origin_ptr, std::vector<T> &origin_col_idx, T lb, T ub)
{
    const size_t rows = (size_t)(ub - lb);
    std::vector<T> local_ptr(rows + 1, 0), remote_ptr(rows + 1, 0), local_col, remote_col;
    if constexpr (std::is_same<T, int>::value) {
        int64_t nl = 0, nr = 0;
        int dummy = 0;  // non-null arrays even when a side, or the whole graph, has no edge
        const int *col = origin_col_idx.empty() ? &dummy : origin_col_idx.data();
        MGG_CHECK(mggx_split_csr(origin_ptr.data(), col, lb, ub, nullptr, nullptr, nullptr, nullptr, &nl, &nr));
        local_col.resize((size_t)nl);
        remote_col.resize((size_t)nr);
        MGG_CHECK(mggx_split_csr(origin_ptr.data(), col, lb, ub, local_ptr.data(), remote_ptr.data(),
                                 nl ? local_col.data() : &dummy, nr ? remote_col.data() : &dummy, &nl, &nr));
    } else {
        for (T i = lb; i < ub; ++i) {
            for (T e = origin_ptr[i]; e < origin_ptr[i + 1]; ++e) {
                const T u = origin_col_idx[e];
                (lb <= u && u < ub ? local_col : remote_col).push_back(u);
            }
            local_ptr[(size_t)(i - lb) + 1] = (T)local_col.size();
            remote_ptr[(size_t)(i - lb) + 1] = (T)remote_col.size();
        }
    }
    return {local_ptr, remote_ptr, local_col, remote_col};
}

// Neighbor partitions of at most partSize edges that never cross a row; returns
// {partPtr, part2Node, node2Part} laid out exactly as the reference does,
// including its unwritten terminal partPtr entry when the last node is isolated.
template <typename T>
std::vector<std::vector<T>> build_part(std::string name, std::vector<T> &indptr, T num_nodes, T partSize)
{
    std::vector<T> partPtr, part2Node, node2Part;
    if constexpr (std::is_same<T, int>::value) {
        int n = 0;
        MGG_CHECK(mggx_build_part(indptr.data(), num_nodes, partSize, 1, nullptr, nullptr, nullptr, &n));
        partPtr.assign((size_t)n + 1, 0);
        part2Node.assign((size_t)n, 0);
        node2Part.assign((size_t)num_nodes + 2, 0);
        int dummy = 0;
        MGG_CHECK(mggx_build_part(indptr.data(), num_nodes, partSize, 1, partPtr.data(), n ? part2Node.data() : &dummy,
                                  node2Part.data(), &n));
    } else {
        T total = 0;
        node2Part.push_back(0);
        for (T i = 0; i < num_nodes; ++i) {
            total += (indptr[i + 1] - indptr[i] + partSize - 1) / partSize;
            node2Part.push_back(total);
        }
        node2Part.push_back(total);
        partPtr.assign((size_t)total + 1, 0);
        part2Node.assign((size_t)total, 0);
        size_t p = 0;
        for (T i = 0; i < num_nodes; ++i)
            for (T b = indptr[i]; b < indptr[i + 1]; b += partSize) {
                partPtr[p] = b;
                part2Node[p++] = i;
            }
        if (num_nodes > 0 && indptr[num_nodes] > indptr[num_nodes - 1]) partPtr[p] = indptr[num_nodes];
    }
    printf("%s, num_nodes: %d, part_size, %d, num_parts, %d\n", name.c_str(), (int)num_nodes, (int)partSize,
           (int)part2Node.size());
    return {partPtr, part2Node, node2Part};
}

inline void mgg_finish_call(int rc, const char *what)
{
    if (rc == MGGX_OK && mgg_options().synchronize) rc = mggx_sync();
    if (rc != MGGX_OK) {
        printf("CUDA error @%s: %s\n", what, mggx_last_error());  // the reference's message shape (:838)
        exit(-1);
    }
}

// output[v] += sum of the local and remote neighbor rows of v, v in [0, ub-lb).
inline void mgg_SAG_np_div(float *output, const float *input, const nidType *row_pointers_l, const nidType *column_index_l,
                           const nidType *row_pointers_r, const nidType *column_index_r, const nidType lb, const nidType ub,
                           const int dim, const int nodePerPE, const int peid, const int np_size, const int warpPerBlock,
                           const int interleaved_dist)
{
    (void)peid;
    mggx_agg_opts o{};
    o.flags = (mgg_options().accumulate ? MGGX_AGG_ACCUMULATE : 0) | (mgg_options().softmax ? MGGX_AGG_SOFTMAX : 0);
    o.col_block_rows = mgg_options().col_block_rows;
    o.core_rows = mgg_options().core_rows;
    const void *remote = mgg_options().remote_table ? mgg_options().remote_table : input;
    mgg_finish_call(mggx_sag_np_div(output, input, remote, row_pointers_l, column_index_l, row_pointers_r, column_index_r, lb,
                                    ub, dim, nodePerPE, np_size, warpPerBlock, interleaved_dist, &o),
                    "mgg_SAG_np_div_cuda");
}

// output[v] = (1 + eps) * input[v] + sum of the neighbor rows of v.
inline void mgg_GIN_np_div(float *output, const float *input, const nidType *row_pointers_l, const nidType *column_index_l,
                           const nidType *row_pointers_r, const nidType *column_index_r, const nidType lb, const nidType ub,
                           const int dim, const int nodePerPE, const int peid, const int np_size, const int warpPerBlock,
                           const int interleaved_dist, float eps)
{
    (void)peid;
    mggx_agg_opts o{};
    o.flags = MGGX_AGG_GIN;
    o.eps = eps;
    o.col_block_rows = mgg_options().col_block_rows;
    o.core_rows = mgg_options().core_rows;
    const void *remote = mgg_options().remote_table ? mgg_options().remote_table : input;
    mgg_finish_call(mggx_sag_np_div(output, input, remote, row_pointers_l, column_index_l, row_pointers_r, column_index_r, lb,
                                    ub, dim, nodePerPE, np_size, warpPerBlock, interleaved_dist, &o),
                    "mgg_GIN_np_div_cuda");
}

// The reference finds (partSize, warpPerBlock, interleaved_dist) per dataset by launching one run per setting
// (bench_MGG_DSE_dist_ps.py, bench_MGG_DSE_dist_wpb.py); this does the search on the caller's own buffers in one
// call.  Later mgg_SAG_np_div calls on the same CSR arrays with warpPerBlock = interleaved_dist = 0 (and np_size 0
// or the returned one) run with the returned setting.  `output` is overwritten.
inline mggx_agg_knobs mgg_tune_np_div(float *output, const float *input, const nidType *row_pointers_l,
                                      const nidType *column_index_l, const nidType *row_pointers_r,
                                      const nidType *column_index_r, const nidType lb, const nidType ub, const int dim,
                                      const int nodePerPE, const int np_size, float *best_ms = nullptr)
{
    mggx_agg_opts o{};
    o.col_block_rows = mgg_options().col_block_rows;
    o.core_rows = mgg_options().core_rows;
    mggx_agg_knobs k{};
    const void *remote = mgg_options().remote_table ? mgg_options().remote_table : input;
    mgg_finish_call(mggx_sag_np_div_tune(output, input, remote, row_pointers_l, column_index_l, row_pointers_r, column_index_r,
                                         lb, ub, dim, nodePerPE, np_size, &o, &k, best_ms),
                    "mgg_tune_np_div");
    return k;
}

// Explicit partition arrays (from build_part), local rows only:
// output[part2Node[p]] += sum over partition p of input[col - lowbound].
template <typename IDType, typename dataType, typename paraType>
void SAG_host(dataType *output, const dataType *input, const IDType *row_pointers, const IDType *column_index,
              const IDType *part_pointers, const IDType *part2Node, const IDType lowbound, const IDType num_nodes,
              const IDType num_parts, const paraType partSize, const paraType dim, const paraType dimWorker,
              const paraType warpPerBlock)
{
    static_assert(std::is_same<IDType, int>::value && std::is_same<dataType, float>::value, "int ids and float features");
    (void)dimWorker;
    mgg_finish_call(mggx_sag_parts(output, input, row_pointers, column_index, part_pointers, part2Node, lowbound, num_nodes,
                                   num_parts, (int)partSize, (int)dim, (int)warpPerBlock, 1),
                    "SAG_cuda_kernel");
}

// The reference's kernel runs the local partitions only (its remote half is
// commented out, neighbor_utils.cuh:2693-2759); so does this wrapper.
// `num_nodes` is the row count the reference passes as local_ptr.size().
template <typename IDType, typename dataType, typename paraType>
void SAG_host_fused_interleaved(dataType *output, const dataType *input, const IDType *local_row_pointers,
                                const IDType *local_column_index, const IDType *local_part_pointers,
                                const IDType *local_part2Node, const IDType local_num_parts,
                                const IDType *remote_row_pointers, const IDType *remote_column_index,
                                const IDType *remote_part_pointers, const IDType *remote_part2Node,
                                const IDType remote_num_parts, const IDType num_nodes, const IDType lowbound,
                                const paraType partSize, const paraType dim, const paraType dimWorker, paraType warpPerBlock,
                                paraType interleaved_dist = 1)
{
    static_assert(std::is_same<IDType, int>::value && std::is_same<dataType, float>::value, "int ids and float features");
    (void)remote_row_pointers; (void)remote_column_index; (void)remote_part_pointers; (void)remote_part2Node;
    (void)remote_num_parts; (void)dimWorker;
    const IDType rows = num_nodes > 0 ? num_nodes - 1 : 0;  // local_ptr.size() = rows + 1
    mgg_finish_call(mggx_sag_parts(output, input, local_row_pointers, local_column_index, local_part_pointers, local_part2Node,
                                   lowbound, rows, local_num_parts, (int)partSize, (int)dim, (int)warpPerBlock,
                                   (int)interleaved_dist),
                    "SAG_cuda_kernel_fused_interleaved");
}

#endif
