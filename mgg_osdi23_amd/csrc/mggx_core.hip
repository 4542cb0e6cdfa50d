// Dense core of a power-law graph served from LDS.
//
// Where a few thousand high-degree rows hold most of the edges among themselves, the aggregation of that core x core
// block does not need one gather per edge from the caches: the feature rows of 256 core columns at a time are staged
// in LDS with whole-line reads, and every lane owns one core row and adds the LDS rows its index list names
// (sliced-ELL lists over degree-ranked rows, so the 64 lanes of a wavefront have lists of similar length).  The
// block's sums go to partial rows per column segment.  This kernel is bound by the LDS, the ordinary aggregation of
// the rest of the CSR by the caches, so the caller runs the two side by side on two streams; k_core_finish then adds
// the partial rows to the output the aggregation wrote.
#include <algorithm>
#include <chrono>
#include <new>

#include "mggx_dev.h"

namespace mggx {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef unsigned short us4 __attribute__((ext_vector_type(4)));

constexpr int CORE_TC = 256;    // core columns per LDS tile
constexpr int CORE_WAVES = 4;   // slices (of 64 rows) per workgroup: as small as the aggregation's own workgroups, so the two
                                // kernels of a call, running side by side, find room on a CU equally easily

// tab[s * core + i] = elements 4 s .. 4 s + 3 of the feature row of the rank-i node (zero past dim)
__global__ void __launch_bounds__(256) k_core_stage(v4f *__restrict__ tab, const float *__restrict__ in, const int *__restrict__ order,
                                                    int core, int n4, int dim, long long ld_in, const Gate gate)
{
    if (gate_closed(gate)) return;
    const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (long long)core * n4) return;
    const int s = (int)(idx / core), i = (int)(idx % core);
    const float *row = in + (long long)order[i] * ld_in + 4 * s;
    v4f v;
    v.x = 4 * s < dim ? row[0] : 0.f;
    v.y = 4 * s + 1 < dim ? row[1] : 0.f;
    v.z = 4 * s + 2 < dim ? row[2] : 0.f;
    v.w = 4 * s + 3 < dim ? row[3] : 0.f;
    tab[idx] = v;
}

// One workgroup = CORE_WAVES slices x one segment of `tiles_per_seg` column tiles; lane = core row.
// partial[(seg * core + rank) * N4 + s]
template <int N4>
__global__ void __launch_bounds__(CORE_WAVES * 64) k_core_sell(const unsigned *__restrict__ blk_off, const unsigned short *__restrict__ idx,
                                                               const v4f *__restrict__ tab, v4f *__restrict__ partial, int core, int ntiles,
                                                               int tiles_per_seg, const Gate gate)
{
    constexpr int TC = CORE_TC, TP = TC + 1;  // column TC of every slice row is zero: what padding entries read
    extern __shared__ v4f tile[];             // [N4][TP]
    if (gate_closed(gate)) return;
    const int lane = (int)(threadIdx.x & 63u), wave = (int)(threadIdx.x >> 6);
    const int g = (int)blockIdx.x * CORE_WAVES + wave;
    const int seg = (int)blockIdx.y;
    v4f acc[N4];
#pragma unroll
    for (int s = 0; s < N4; ++s) acc[s] = (v4f){0.f, 0.f, 0.f, 0.f};
    if ((int)threadIdx.x < N4) tile[(int)threadIdx.x * TP + TC] = (v4f){0.f, 0.f, 0.f, 0.f};
    const int t0 = seg * tiles_per_seg;
    const us4 *p = reinterpret_cast<const us4 *>(idx) + lane;
    unsigned pos = blk_off[(size_t)g * ntiles + t0];
    const unsigned end_seg = blk_off[(size_t)g * ntiles + t0 + tiles_per_seg];
    const us4 pad = (us4){0xFFFF, 0xFFFF, 0xFFFF, 0xFFFF};
    us4 cur = pos < end_seg ? p[(size_t)pos * 64] : pad;  // the lists of a slice's tiles follow one another: read one chunk ahead
    for (int tt = 0; tt < tiles_per_seg; ++tt) {
        const int t = t0 + tt;
        __syncthreads();
        for (int i = (int)threadIdx.x; i < N4 * TC; i += CORE_WAVES * 64) {
            const int s = i / TC, c = i % TC;
            tile[s * TP + c] = tab[(size_t)s * core + (size_t)t * TC + c];
        }
        const unsigned b1 = blk_off[(size_t)g * ntiles + t + 1];
        __syncthreads();
        while (pos < b1) {
            const us4 nxt = pos + 1 < end_seg ? p[(size_t)(pos + 1) * 64] : pad;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int c = cur[j];
                const v4f *q = tile + (c < TC ? c : TC);
                // at most eight LDS reads in flight per entry: wide rows otherwise cost a wavefront a hundred registers, and
                // this kernel shares each SIMD's register file with the aggregation running beside it
                constexpr int H = N4 > 8 ? (N4 + 1) / 2 : N4;
#pragma unroll
                for (int s = 0; s < H; ++s) acc[s] += q[s * TP];
                if constexpr (H < N4) {
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int s = H; s < N4; ++s) acc[s] += q[s * TP];
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            cur = nxt;
            ++pos;
        }
    }
    const int r = g * 64 + lane;
#pragma unroll
    for (int s = 0; s < N4; ++s) partial[((size_t)seg * core + r) * N4 + s] = acc[s];
}

// Adds the core block's sums to output rows that already hold the rest of the aggregation:
// out[v][d] = act(out[v][d] + scale[v] * sum over segments of the partial rows of v).  all_rows = 0: one thread per
// element of the core rows only (idx -> rank -> row); all_rows = 1: every row (needed when act is the ReLU).
__global__ void __launch_bounds__(256) k_core_finish(float *__restrict__ out, const float *__restrict__ partial, const int *__restrict__ rank,
                                                     const int *__restrict__ order, const float *__restrict__ rs, int rows, int dim,
                                                     long long ld_out, int core, int n4, int nseg, int relu, int all_rows, const Gate gate)
{
    if (gate_closed(gate)) return;
    const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (long long)(all_rows ? rows : core) * dim) return;
    const int i = (int)(idx / dim), d = (int)(idx % dim);
    const int v = all_rows ? i : order[i];
    const int r = all_rows ? rank[i] : i;
    float sum = 0.f;
    if (r >= 0) {
        for (int seg = 0; seg < nseg; ++seg) sum += partial[(((size_t)seg * core + r) * n4 + (d >> 2)) * 4 + (d & 3)];
        if (rs) sum *= rs[v];
    }
    float *o = out + (long long)v * ld_out + d;
    float t = *o + sum;
    if (relu) t = fmaxf(t, 0.f);
    *o = t;
}

// The same, four columns per thread, where the output rows take 16-byte accesses.
__global__ void __launch_bounds__(256) k_core_finish4(float *__restrict__ out, const v4f *__restrict__ partial, const int *__restrict__ rank,
                                                      const int *__restrict__ order, const float *__restrict__ rs, int rows, int n4,
                                                      long long ld_out, int core, int nseg, int relu, int all_rows, const Gate gate)
{
    if (gate_closed(gate)) return;
    const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (long long)(all_rows ? rows : core) * n4) return;
    const int i = (int)(idx / n4), q = (int)(idx % n4);
    const int v = all_rows ? i : order[i];
    const int r = all_rows ? rank[i] : i;
    v4f sum = {0.f, 0.f, 0.f, 0.f};
    if (r >= 0) {
        for (int seg = 0; seg < nseg; ++seg) sum += partial[((size_t)seg * core + r) * n4 + q];
        if (rs) sum *= rs[v];
    }
    v4f *o = reinterpret_cast<v4f *>(out + (long long)v * ld_out + 4 * q);
    v4f t = *o + sum;
    if (relu) { t.x = fmaxf(t.x, 0.f); t.y = fmaxf(t.y, 0.f); t.z = fmaxf(t.z, 0.f); t.w = fmaxf(t.w, 0.f); }
    *o = t;
}

template <int N4>
int launch_sell(const CorePlan *p, const v4f *tab, v4f *partial, const Gate &gate, hipStream_t stream)
{
    const size_t lds = (size_t)N4 * (CORE_TC + 1) * sizeof(v4f);
    static bool raised = false;  // per instantiation
    if (lds > 48 * 1024 && !raised) {
        MGGX_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(k_core_sell<N4>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        raised = true;
    }
    // row groups vary fastest in the grid: workgroups that run side by side then read the same tiles, and a CU holds dense
    // and sparse row groups at once (the reverse order measured 25 % slower)
    const dim3 grid((unsigned)(p->core / (CORE_WAVES * 64)), (unsigned)p->nseg);
    k_core_sell<N4><<<grid, dim3(CORE_WAVES * 64), lds, stream>>>(p->d_blk_off, p->d_idx, tab, partial, p->core, p->ntiles, p->ntiles / p->nseg, gate);
    MGGX_LAUNCH_CHECK("k_core_sell");
    return MGGX_OK;
}

void core_plan_free_arrays(CorePlan *p)
{
    if (p->d_order) (void)hipFree(p->d_order);
    if (p->d_rank) (void)hipFree(p->d_rank);
    if (p->d_blk_off) (void)hipFree(p->d_blk_off);
    if (p->d_idx) (void)hipFree(p->d_idx);
    if (p->d_rem_ptr) (void)hipFree(p->d_rem_ptr);
    if (p->d_rem_col) (void)hipFree(p->d_rem_col);
}

template <typename T>
int upload(T **d, const std::vector<T> &h, size_t min_elems = 1)
{
    const size_t n = std::max(h.size(), min_elems);
    if (hipMalloc((void **)d, n * sizeof(T)) != hipSuccess) return fail(MGGX_ENOMEM, "core plan: %zu bytes of device memory", n * sizeof(T));
    if (!h.empty() && hipMemcpy(*d, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice) != hipSuccess)
        return fail(MGGX_EHIP, "core plan: upload failed");
    return MGGX_OK;
}

}  // namespace

void core_plan_free(CorePlan *p)
{
    if (!p) return;
    forget_pointer(p->d_rem_ptr);  // plans and records of the remainder CSR hang on these addresses
    forget_pointer(p->d_rem_col);
    core_plan_free_arrays(p);
    delete p;
}

int core_side_stream(hipStream_t *stream, hipEvent_t *fork, hipEvent_t *join)
{
    State &s = state();
    if (!s.side_stream) {
        MGGX_HIP(hipStreamCreateWithFlags(&s.side_stream, hipStreamNonBlocking));
        MGGX_HIP(hipEventCreateWithFlags(&s.side_fork, hipEventDisableTiming));
        MGGX_HIP(hipEventCreateWithFlags(&s.side_join, hipEventDisableTiming));
    }
    *stream = s.side_stream;
    *fork = s.side_fork;
    *join = s.side_join;
    return MGGX_OK;
}

int core_plan_get(const int *d_ptr_l, const int *d_col_l, int rows, int lb, int core, CorePlan **out)
{
    State &s = state();
    for (size_t i = 0; i < s.cores.size(); ++i) {
        CorePlan *p = s.cores[i];
        if (p->d_ptr_l == d_ptr_l && p->d_col_l == d_col_l && p->rows == rows && p->lb == lb && p->asked == core) {
            if (i + 1 != s.cores.size()) {  // most recently used last
                s.cores.erase(s.cores.begin() + (long)i);
                s.cores.push_back(p);
            }
            if (!p->pinned && capturing()) p->pinned = true;
            *out = p;
            return MGGX_OK;
        }
    }
    if (rows < 1 || !d_ptr_l || !d_col_l) return fail(MGGX_EINVAL, "core plan: empty or NULL CSR");
    if (capturing()) return fail(MGGX_EINVAL, "core plan: first use of this CSR and core size inside a stream capture; call once outside the capture first");
    const auto t0 = std::chrono::steady_clock::now();
    MGGX_HIP(hipStreamSynchronize(s.stream));
    CorePlan *p = new (std::nothrow) CorePlan;
    if (!p) return fail(MGGX_ENOMEM, "core plan");
    p->d_ptr_l = d_ptr_l;
    p->d_col_l = d_col_l;
    p->rows = rows;
    p->lb = lb;
    p->asked = core;
    int rc = MGGX_OK;
    try {
        std::vector<int> ptr((size_t)rows + 1);
        if (hipMemcpy(ptr.data(), d_ptr_l, ptr.size() * sizeof(int), hipMemcpyDeviceToHost) != hipSuccess) rc = fail(MGGX_EHIP, "core plan: reading the CSR");
        std::vector<int> col(rc ? 0 : (size_t)std::max(ptr[rows], 0));
        if (!rc && !col.empty() && hipMemcpy(col.data(), d_col_l, col.size() * sizeof(int), hipMemcpyDeviceToHost) != hipSuccess)
            rc = fail(MGGX_EHIP, "core plan: reading the CSR");
        CoreLayout L;
        if (!rc) {
            const int lrc = core_layout_build(ptr.data(), col.data(), rows, lb, core, CORE_TC, &L);
            if (lrc == MGGX_EINVAL) p->unsuitable = true;  // remembered: the caller falls back to the ordinary path
            else rc = lrc;
        }
        if (!rc && !p->unsuitable) {
            p->core = L.core;
            p->ntiles = L.ntiles;
            p->core_nnz = L.core_nnz;
            p->rem_nnz = (int64_t)L.rem_col.size();
            // segments: enough workgroups to fill the chip a few times over, whole tiles each
            int nseg = 1;
            while (nseg * 2 <= p->ntiles && (p->ntiles % (nseg * 2)) == 0 && (long long)(p->core / (CORE_WAVES * 64)) * nseg < 2048) nseg *= 2;
            p->nseg = nseg;
            rc = upload(&p->d_order, L.order);
            if (!rc) rc = upload(&p->d_rank, L.rank);
            if (!rc) rc = upload(&p->d_blk_off, L.blk_off);
            if (!rc) rc = upload(&p->d_idx, L.idx, 256);
            if (!rc) rc = upload(&p->d_rem_ptr, L.rem_ptr);
            if (!rc) rc = upload(&p->d_rem_col, L.rem_col);
            p->bytes = (L.order.size() + L.rank.size() + L.rem_ptr.size() + L.rem_col.size()) * sizeof(int) + L.blk_off.size() * sizeof(unsigned) +
                       std::max<size_t>(L.idx.size(), 256) * sizeof(unsigned short);
        }
    } catch (const std::bad_alloc &) {
        rc = fail(MGGX_ENOMEM, "core plan: out of host memory");
    }
    if (rc) {
        core_plan_free_arrays(p);
        delete p;
        return rc;
    }
    if (s.cores.size() >= 4)  // these plans are large (about 3 bytes per edge): keep the four most recently used, and any a captured graph holds
        for (size_t i = 0; i < s.cores.size(); ++i)
            if (!s.cores[i]->pinned) {
                CorePlan *old = s.cores[i];
                s.cores.erase(s.cores.begin() + (long)i);
                core_plan_free(old);
                break;
            }
    s.cores.push_back(p);
    s.core_plan_build_ms += std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
    *out = p;
    return MGGX_OK;
}

// Scratch of the dense-core path: the staged core table, then one partial row per core row and segment.
static int core_scratch(const CorePlan *p, int n4, v4f **tab, v4f **partial)
{
    State &s = state();
    const size_t tab_bytes = ((size_t)p->core * n4 * sizeof(v4f) + 255) & ~(size_t)255;
    const size_t part_bytes = (size_t)p->nseg * p->core * n4 * sizeof(v4f);
    if (tab_bytes + part_bytes > s.core_ws_bytes) {
        if (capturing()) return fail(MGGX_EINVAL, "core: the scratch block would have to grow inside a stream capture; run the largest call once outside it first");
        MGGX_HIP(hipDeviceSynchronize());  // both streams may still use the old block
        if (s.core_ws) {
            if (s.core_ws_captured) {  // a captured graph may still point at it: kept until mggx_release_cached
                s.retired.push_back(s.core_ws);
                s.retired_bytes += s.core_ws_bytes;
                s.core_ws_captured = false;
            } else {
                (void)hipFree(s.core_ws);
            }
        }
        s.core_ws = nullptr;
        s.core_ws_bytes = 0;
        if (hipMalloc(&s.core_ws, tab_bytes + part_bytes) != hipSuccess) return fail(MGGX_ENOMEM, "core: %zu bytes of scratch", tab_bytes + part_bytes);
        s.core_ws_bytes = tab_bytes + part_bytes;
    }
    if (!s.core_ws_captured && capturing()) s.core_ws_captured = true;
    *tab = static_cast<v4f *>(s.core_ws);
    *partial = reinterpret_cast<v4f *>(static_cast<char *>(s.core_ws) + tab_bytes);
    return MGGX_OK;
}

// The core's feature rows into the slice-major table, on `stream` (a few microseconds on an idle chip, ten times that
// beside the aggregation: the caller runs it before the two big kernels start).
int run_core_stage(CorePlan *p, const float *d_in, int dim, long long ld_in, const Gate &gate, hipStream_t stream)
{
    const int n4 = (dim + 3) / 4;
    if (n4 < 1 || n4 > 16) return fail(MGGX_ELIMIT, "core: dim %d outside 1..64", dim);
    v4f *tab = nullptr, *partial = nullptr;
    int rc = core_scratch(p, n4, &tab, &partial);
    if (rc) return rc;
    const long long n = (long long)p->core * n4;
    k_core_stage<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream>>>(tab, d_in, p->d_order, p->core, n4, dim, ld_in, gate);
    MGGX_LAUNCH_CHECK("k_core_stage");
    return MGGX_OK;
}

// The core block's sums from the staged table into the library's partial rows, on `stream`.
int run_core_sums(CorePlan *p, int dim, const Gate &gate, hipStream_t stream)
{
    const int n4 = (dim + 3) / 4;
    if (n4 < 1 || n4 > 16) return fail(MGGX_ELIMIT, "core: dim %d outside 1..64", dim);
    v4f *tab = nullptr, *partial = nullptr;
    int rc = core_scratch(p, n4, &tab, &partial);
    if (rc) return rc;
    switch (n4) {
#define MGGX_CASE(N) case N: rc = launch_sell<N>(p, tab, partial, gate, stream); break;
        MGGX_CASE(1) MGGX_CASE(2) MGGX_CASE(3) MGGX_CASE(4) MGGX_CASE(5) MGGX_CASE(6) MGGX_CASE(7) MGGX_CASE(8)
        MGGX_CASE(9) MGGX_CASE(10) MGGX_CASE(11) MGGX_CASE(12) MGGX_CASE(13) MGGX_CASE(14) MGGX_CASE(15) MGGX_CASE(16)
#undef MGGX_CASE
        default: rc = fail(MGGX_ELIMIT, "core: dim %d", dim);
    }
    return rc;
}

// out += scale * (partial rows of the core), then the ReLU if asked for, on `stream`.
int run_core_finish(CorePlan *p, float *d_out, int dim, long long ld_out, const float *d_row_scale, int relu, const Gate &gate, hipStream_t stream)
{
    const int n4 = (dim + 3) / 4;
    v4f *tab = nullptr, *partial = nullptr;
    int rc = core_scratch(p, n4, &tab, &partial);  // sized by run_core_sums already: only hands the pointers out
    if (rc) return rc;
    const int all_rows = relu ? 1 : 0;
    const long long nrows = all_rows ? p->rows : p->core;
    if (dim % 4 == 0 && ld_out % 4 == 0 && (reinterpret_cast<uintptr_t>(d_out) & 15u) == 0) {
        const long long n = nrows * n4;
        k_core_finish4<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream>>>(d_out, partial, p->d_rank, p->d_order, d_row_scale, p->rows, n4,
                                                                                     ld_out, p->core, p->nseg, relu, all_rows, gate);
    } else {
        const long long n = nrows * dim;
        k_core_finish<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream>>>(d_out, reinterpret_cast<const float *>(partial), p->d_rank,
                                                                                    p->d_order, d_row_scale, p->rows, dim, ld_out, p->core, n4,
                                                                                    p->nseg, relu, all_rows, gate);
    }
    MGGX_LAUNCH_CHECK("k_core_finish");
    return MGGX_OK;
}

}  // namespace mggx
