// Shared set-up of the harness programs: command line, graph load, one rank's
// share of the range partition, device upload.  The programs keep the command
// line and the log lines of the reference's mains (src/mgg_np_div_kernel.cu:47-57,
// 103,192,195) so the reference's bench/analysis scripts can drive and parse them:
//   <prog> beg.bin csr.bin weight.bin nGPU partSize warpPerBlock dist dim hidden out [--pe K] [--iters N] [--validate] [--tune]
//          [--compact-remote] [--fuse-softmax]
// nGPU is the number of ranks the graph is partitioned for; the one real GPU
// runs rank --pe (default 0) with the other ranks' rows staged in its memory.
#ifndef MGG_HARNESS_COMMON_H
#define MGG_HARNESS_COMMON_H

#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <ctime>
#include <iostream>
#include <vector>

#include "mgg/csr_formatter.h"
#include "mgg/gnn_layer.h"
#include "mgg/graph.h"
#include "mgg/layer_new.h"
#include "mgg/neighbor_utils.h"
#include "mgg/utils.h"

struct HarnessArgs {
    const char *beg_file, *csr_file, *weight_file;
    int num_GPUs, partSize, warpPerBlock, interleaved_dist, dim, hiddenSize, outdim;
    int pe = 0, iters = 100;
    bool validate = false;
    bool tune = false;  // search warpPerBlock / interleaved_dist / partition order on this input first (mgg_tune_np_div)
    bool compact_remote = false;  // stage the remote rows compactly: one row per distinct remote id, most referenced first
    bool fuse_softmax = false;    // mgg_np_div_mem: the last aggregation ends in the softmax instead of a softmax_forward call
};

inline bool parse_args(int argc, char *argv[], HarnessArgs &a)
{
    if (argc < 11) {
        printf("Usage: %s beg.bin csr.bin weight.bin num_GPUs partSize warpPerblock interleaved_dist dim hidden out "
               "[--pe K] [--iters N] [--validate] [--tune] [--compact-remote] [--fuse-softmax]\n", argv[0]);
        return false;
    }
    a.beg_file = argv[1];
    a.csr_file = argv[2];
    a.weight_file = argv[3];
    a.num_GPUs = atoi(argv[4]);
    a.partSize = atoi(argv[5]);
    a.warpPerBlock = atoi(argv[6]);
    a.interleaved_dist = atoi(argv[7]);
    a.dim = atoi(argv[8]);
    a.hiddenSize = atoi(argv[9]);
    a.outdim = atoi(argv[10]);
    for (int i = 11; i < argc; ++i) {
        if (!strcmp(argv[i], "--pe") && i + 1 < argc) a.pe = atoi(argv[++i]);
        else if (!strcmp(argv[i], "--iters") && i + 1 < argc) a.iters = atoi(argv[++i]);
        else if (!strcmp(argv[i], "--validate")) a.validate = true;
        else if (!strcmp(argv[i], "--tune")) a.tune = true;
        else if (!strcmp(argv[i], "--compact-remote")) a.compact_remote = true;
        else if (!strcmp(argv[i], "--fuse-softmax")) a.fuse_softmax = true;
    }
    if (a.num_GPUs < 1 || a.pe < 0 || a.pe >= a.num_GPUs || a.iters < 1) {
        printf("bad --pe/--iters/num_GPUs\n");
        return false;
    }
    return true;
}

// One rank's share: the split CSR on the host and on the device.
struct Share {
    nidType numNodes = 0, numEdges = 0, nodesPerPE = 0, lb = 0, ub = 0;
    std::vector<nidType> global_row_ptr, global_col_ind;
    std::vector<nidType> local_ptr, remote_ptr, local_col, remote_col;
    nidType *d_row_ptr_l = nullptr, *d_col_ind_l = nullptr, *d_row_ptr_r = nullptr, *d_col_ind_r = nullptr;
};

template <typename T>
inline T *to_device(const std::vector<T> &v)
{
    void *p = nullptr;
    MGG_CHECK(mggx_malloc(&p, (v.size() ? v.size() : 1) * sizeof(T)));
    if (!v.empty()) MGG_CHECK(mggx_memcpy_h2d(p, v.data(), v.size() * sizeof(T)));
    return static_cast<T *>(p);
}

inline float *device_filled(size_t count, float value)
{
    std::vector<float> h(count, value);
    return to_device(h);
}

inline void load_share(const HarnessArgs &a, Share &s)
{
    std::cout << "Graph File: " << a.beg_file << '\n';
    auto *g = new graph<long, long, nidType, nidType, nidType, nidType>(a.beg_file, a.csr_file, a.weight_file);
    s.global_row_ptr.assign(g->beg_pos, g->beg_pos + g->vert_count + 1);
    s.global_col_ind.assign(g->csr, g->csr + g->edge_count);
    std::cout << "Complete loading graphs !!" << std::endl;
    s.numNodes = (nidType)s.global_row_ptr.size() - 1;
    s.numEdges = (nidType)s.global_col_ind.size();
    MGG_CHECK(mggx_range_partition(s.numNodes, a.num_GPUs, a.pe, &s.nodesPerPE, &s.lb, &s.ub));
    if (s.ub < s.lb) s.ub = s.lb;

    std::clock_t c0 = std::clock();
    auto split = split_CSR<nidType>(s.global_row_ptr, s.global_col_ind, s.lb, s.ub);
    std::clock_t c1 = std::clock();
    printf("Preproc (ms): %.3f\n", 1000.0 * (c1 - c0) / CLOCKS_PER_SEC);
    s.local_ptr = split[0];
    s.remote_ptr = split[1];
    s.local_col = split[2];
    s.remote_col = split[3];
    s.d_row_ptr_l = to_device(s.local_ptr);
    s.d_col_ind_l = to_device(s.local_col);
    s.d_row_ptr_r = to_device(s.remote_ptr);
    s.d_col_ind_r = to_device(s.remote_col);
}

// Compact staging of a share's remote rows (what a pre-exchange of remote rows between the ranks would deliver): the
// distinct remote ids, most referenced first, found on the device; `table` (indexed by global id, row_floats wide) gathered
// into a table with one row per distinct id; the remote column array rewritten to positions in it.  Returns the compact
// table and replaces s.d_col_ind_r.  The gather is what a layer pays per call; the compaction once per graph.
struct CompactRemote {
    nidType *d_fetch_ids = nullptr;
    int64_t n_unique = 0;
};

inline double now_ms();

inline CompactRemote compact_remote_columns(Share &s)
{
    CompactRemote c;
    const int64_t n = (int64_t)s.remote_col.size();
    const double t0 = now_ms();
    MGG_CHECK(mggx_compact_remote_device(s.d_col_ind_r, n, nullptr, nullptr, &c.n_unique));
    void *d_compact = nullptr, *d_ids = nullptr;
    MGG_CHECK(mggx_malloc(&d_compact, (size_t)(n ? n : 1) * sizeof(nidType)));
    MGG_CHECK(mggx_malloc(&d_ids, (size_t)(c.n_unique ? c.n_unique : 1) * sizeof(nidType)));
    MGG_CHECK(mggx_compact_remote_device(s.d_col_ind_r, n, (nidType *)d_compact, (nidType *)d_ids, &c.n_unique));
    MGG_CHECK(mggx_sync());
    printf("Compact staging: %lld distinct remote rows of %lld remote neighbors, found in %.3f ms\n", (long long)c.n_unique, (long long)n,
           now_ms() - t0);
    MGG_CHECK(mggx_free(s.d_col_ind_r));
    s.d_col_ind_r = (nidType *)d_compact;
    c.d_fetch_ids = (nidType *)d_ids;
    return c;
}

// One staged table for `dim` floats per row from the table indexed by global id.
inline float *stage_compact(const CompactRemote &c, const float *d_global_table, int dim)
{
    void *d = nullptr;
    MGG_CHECK(mggx_malloc(&d, (size_t)(c.n_unique ? c.n_unique : 1) * dim * sizeof(float)));
    if (dim % 4) {
        printf("compact staging needs rows of whole 16-byte pieces (dim %% 4 == 0)\n");
        exit(-1);
    }
    MGG_CHECK(mggx_gather_rows(d, d_global_table, c.d_fetch_ids, c.n_unique, (size_t)dim * sizeof(float)));
    return (float *)d;
}

inline double now_ms()
{
    using namespace std::chrono;
    return duration<double, std::milli>(steady_clock::now().time_since_epoch()).count();
}

#endif
