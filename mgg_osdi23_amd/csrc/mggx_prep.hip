// Device-side preparation of a share's remote side: the compact staging order of mggx_compact_remote, computed on
// the GPU with rocPRIM's sort and run-length primitives (bit-identical to the host version).
#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/device/device_run_length_encode.hpp>

#include "mggx_dev.h"

namespace mggx {
namespace {

__global__ void __launch_bounds__(256) k_iota(int *__restrict__ v, int n)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) v[i] = i;
}

// order[pos] = index (into the ascending id list) of the id staged at position pos
__global__ void __launch_bounds__(256) k_rank_and_fetch(const int *__restrict__ order, const int *__restrict__ ids, int u,
                                                        int *__restrict__ rank, int *__restrict__ fetch_ids)
{
    const int pos = blockIdx.x * 256 + threadIdx.x;
    if (pos >= u) return;
    const int i = order[pos];
    rank[i] = pos;
    fetch_ids[pos] = ids[i];
}

__global__ void __launch_bounds__(256) k_remap(const int *__restrict__ col, long long n, const int *__restrict__ ids, int u,
                                              const int *__restrict__ rank, int *__restrict__ out)
{
    for (long long e = (long long)blockIdx.x * 256 + threadIdx.x; e < n; e += (long long)gridDim.x * 256) {
        const int key = col[e];
        int lo = 0, hi = u;  // first index with ids[idx] >= key; key is present
        while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            if (ids[mid] < key) lo = mid + 1;
            else hi = mid;
        }
        out[e] = rank[lo];
    }
}

__global__ void k_min_i32(const int *__restrict__ sorted, int *__restrict__ out) { *out = sorted[0]; }

struct DeviceBuffers {
    std::vector<void *> ptrs;
    ~DeviceBuffers()
    {
        for (void *p : ptrs) (void)hipFree(p);
    }
    template <typename T>
    int get(T **p, size_t count)
    {
        void *q = nullptr;
        if (hipMalloc(&q, std::max<size_t>(count, 1) * sizeof(T)) != hipSuccess)
            return fail(MGGX_ENOMEM, "compact_remote_device: %zu bytes of scratch", count * sizeof(T));
        ptrs.push_back(q);
        *p = static_cast<T *>(q);
        return MGGX_OK;
    }
};

}  // namespace
}  // namespace mggx

using mggx::fail;

MGGX_EXPORT int mggx_compact_remote_device(const int *d_remote_col, int64_t n_remote, int *d_remote_col_compact, int *d_fetch_ids,
                                           int64_t *n_unique)
{
    int rc = mggx::ensure_init();
    if (rc) return rc;
    if (n_remote < 0 || (n_remote && !d_remote_col)) return fail(MGGX_EINVAL, "compact_remote_device: bad remote_col");
    if (n_remote > 0x7fffffffLL) return fail(MGGX_ELIMIT, "compact_remote_device: more than 2^31-1 edges");
    if ((d_remote_col_compact == nullptr) != (d_fetch_ids == nullptr))
        return fail(MGGX_EINVAL, "compact_remote_device: pass both output arrays or neither");
    if (n_remote == 0) {
        if (n_unique) *n_unique = 0;
        return MGGX_OK;
    }
    hipStream_t stream = mggx::state().stream;
    const size_t n = (size_t)n_remote;
    mggx::DeviceBuffers buf;
    int *sorted = nullptr, *ids = nullptr, *cnt = nullptr, *runs = nullptr, *first = nullptr;
    if ((rc = buf.get(&sorted, n)) || (rc = buf.get(&ids, n)) || (rc = buf.get(&cnt, n)) || (rc = buf.get(&runs, 1)) ||
        (rc = buf.get(&first, 1)))
        return rc;

    // 1. ascending ids, 2. distinct ids and how often each occurs
    size_t tmp_bytes = 0, need = 0;
    MGGX_HIP(rocprim::radix_sort_keys(nullptr, need, d_remote_col, sorted, n, 0, 32, stream));
    tmp_bytes = need;
    MGGX_HIP(rocprim::run_length_encode(nullptr, need, sorted, (unsigned)n, ids, cnt, runs, stream));
    tmp_bytes = std::max(tmp_bytes, need);
    char *tmp = nullptr;
    if ((rc = buf.get(&tmp, tmp_bytes))) return rc;
    need = tmp_bytes;
    MGGX_HIP(rocprim::radix_sort_keys(tmp, need, d_remote_col, sorted, n, 0, 32, stream));
    need = tmp_bytes;
    MGGX_HIP(rocprim::run_length_encode(tmp, need, sorted, (unsigned)n, ids, cnt, runs, stream));
    mggx::k_min_i32<<<1, 1, 0, stream>>>(sorted, first);
    int host_vals[2] = {0, 0};
    MGGX_HIP(hipMemcpyAsync(&host_vals[0], runs, sizeof(int), hipMemcpyDeviceToHost, stream));
    MGGX_HIP(hipMemcpyAsync(&host_vals[1], first, sizeof(int), hipMemcpyDeviceToHost, stream));
    MGGX_HIP(hipStreamSynchronize(stream));
    const int u = host_vals[0];
    if (host_vals[1] < 0) return fail(MGGX_EFORMAT, "compact_remote_device: negative neighbor id %d", host_vals[1]);
    if (n_unique) *n_unique = u;
    if (!d_fetch_ids) return MGGX_OK;

    // 3. staging order: most referenced first; the sort is stable, so equal counts keep ascending id
    int *iota = nullptr, *order = nullptr, *cnt_sorted = nullptr, *rank = nullptr;
    if ((rc = buf.get(&iota, (size_t)u)) || (rc = buf.get(&order, (size_t)u)) || (rc = buf.get(&cnt_sorted, (size_t)u)) ||
        (rc = buf.get(&rank, (size_t)u)))
        return rc;
    mggx::k_iota<<<(u + 255) / 256, 256, 0, stream>>>(iota, u);
    need = 0;
    MGGX_HIP(rocprim::radix_sort_pairs_desc(nullptr, need, cnt, cnt_sorted, iota, order, (size_t)u, 0, 32, stream));
    char *tmp2 = tmp;
    if (need > tmp_bytes && (rc = buf.get(&tmp2, need))) return rc;
    MGGX_HIP(rocprim::radix_sort_pairs_desc(tmp2, need, cnt, cnt_sorted, iota, order, (size_t)u, 0, 32, stream));
    // 4. position of every id in that order, the list itself, and the rewritten column array
    mggx::k_rank_and_fetch<<<(u + 255) / 256, 256, 0, stream>>>(order, ids, u, rank, d_fetch_ids);
    long long blocks = ((long long)n + 255) / 256;
    if (blocks > 256 * 64) blocks = 256 * 64;
    mggx::k_remap<<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(d_remote_col, (long long)n, ids, u, rank, d_remote_col_compact);
    MGGX_LAUNCH_CHECK("compact_remote_device kernels");
    MGGX_HIP(hipStreamSynchronize(stream));  // the scratch buffers are freed on return
    return MGGX_OK;
}
