// Runtime half of libmggx.so: device selection, stream, memory, timers, the
// library-owned workspace and small utility kernels.
#include <algorithm>
#include <cstdio>
#include <cstring>

#include "mggx_dev.h"

namespace mggx {

State &state()
{
    static State s;
    return s;
}

int ensure_init()
{
    State &s = state();
    if (s.device >= 0) return MGGX_OK;
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0)
        return fail(MGGX_EHIP, "no HIP device available (%s)", e == hipSuccess ? "device count is 0" : hipGetErrorString(e));
    int cur = 0;
    MGGX_HIP(hipGetDevice(&cur));
    s.device = cur;
    return MGGX_OK;
}

int workspace(size_t bytes, void **p)
{
    State &s = state();
    if (bytes > s.ws_bytes) {
        if (capturing()) return fail(MGGX_EINVAL, "the workspace would have to grow inside a stream capture; run the largest call once outside it first");
        if (s.ws) {
            MGGX_HIP(hipStreamSynchronize(s.stream));
            if (s.ws_captured) {  // a captured graph may still point at it: kept until mggx_release_cached
                s.retired.push_back(s.ws);
                s.retired_bytes += s.ws_bytes;
                s.ws_captured = false;
            } else {
                MGGX_HIP(hipFree(s.ws));
            }
            s.ws = nullptr;
            s.ws_bytes = 0;
        }
        size_t want = bytes + bytes / 4 + 4096;
        hipError_t e = hipMalloc(&s.ws, want);
        if (e != hipSuccess) {
            s.ws = nullptr;
            return fail(MGGX_ENOMEM, "workspace of %zu bytes: %s", want, hipGetErrorString(e));
        }
        s.ws_bytes = want;
    }
    if (!s.ws_captured && capturing()) s.ws_captured = true;
    *p = s.ws;
    return MGGX_OK;
}

}  // namespace mggx

using mggx::fail;
using mggx::state;

MGGX_EXPORT int mggx_init(int device)
{
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0)
        return fail(MGGX_EHIP, "no HIP device available (%s)", e == hipSuccess ? "device count is 0" : hipGetErrorString(e));
    if (device < 0 || device >= count) return fail(MGGX_EINVAL, "init: device %d of %d", device, count);
    MGGX_HIP(hipSetDevice(device));
    hipDeviceProp_t prop;
    MGGX_HIP(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(MGGX_EHIP, "init: device %d is %s; this library carries gfx950 code only", device, prop.gcnArchName);
    state().device = device;
    // Set-up of the allocation-free entry point: its array's address on this device is looked up now.  Should the lookup
    // fail, only that entry point is unavailable (mggx_sag_parts_static asks again and reports the error itself).
    unsigned char *scratch_addr = nullptr;
    (void)mggx::static_scratch_ptr(&scratch_addr);
    return MGGX_OK;
}

MGGX_EXPORT int mggx_device_name(char *buf, size_t len)
{
    if (!buf || !len) return fail(MGGX_EINVAL, "device_name: NULL buffer");
    int rc = mggx::ensure_init();
    if (rc) return rc;
    hipDeviceProp_t prop;
    MGGX_HIP(hipGetDeviceProperties(&prop, state().device));
    snprintf(buf, len, "%s (%s, %d CUs)", prop.name, prop.gcnArchName, prop.multiProcessorCount);
    return MGGX_OK;
}

MGGX_EXPORT int mggx_set_stream(void *hip_stream)
{
    state().stream = static_cast<hipStream_t>(hip_stream);
    return MGGX_OK;
}

MGGX_EXPORT int mggx_sync(void)
{
    MGGX_HIP(hipStreamSynchronize(state().stream));
    return mggx::stale_poll();  // a content check that ran on the stream may have found changed CSR arrays
}

MGGX_EXPORT int mggx_malloc(void **d_ptr, size_t bytes)
{
    if (!d_ptr) return fail(MGGX_EINVAL, "malloc: NULL result pointer");
    int rc = mggx::ensure_init();
    if (rc) return rc;
    *d_ptr = nullptr;
    hipError_t e = hipMalloc(d_ptr, bytes ? bytes : 1);
    if (e != hipSuccess) return fail(MGGX_ENOMEM, "malloc of %zu bytes: %s", bytes, hipGetErrorString(e));
    return MGGX_OK;
}

MGGX_EXPORT int mggx_malloc_tables(void **d_local, size_t local_bytes, void **d_remote, size_t remote_bytes)
{
    if (!d_local || !d_remote) return fail(MGGX_EINVAL, "malloc_tables: NULL result pointer");
    int rc = mggx::ensure_init();
    if (rc) return rc;
    *d_local = *d_remote = nullptr;
    const size_t first = (std::max<size_t>(local_bytes, 1) + 255) & ~(size_t)255;
    void *p = nullptr;
    hipError_t e = hipMalloc(&p, first + std::max<size_t>(remote_bytes, 1));
    if (e != hipSuccess) return fail(MGGX_ENOMEM, "malloc_tables of %zu + %zu bytes: %s", local_bytes, remote_bytes, hipGetErrorString(e));
    *d_local = p;
    *d_remote = static_cast<char *>(p) + first;
    return MGGX_OK;
}

MGGX_EXPORT int mggx_free(void *d_ptr)
{
    if (!d_ptr) return MGGX_OK;
    int rc = mggx::forget_pointer(d_ptr);  // a later allocation may get the same address
    if (rc) return rc;
    MGGX_HIP(hipFree(d_ptr));
    return MGGX_OK;
}

MGGX_EXPORT int mggx_memset(void *d_ptr, int value, size_t bytes)
{
    if (!bytes) return MGGX_OK;
    if (!d_ptr) return fail(MGGX_EINVAL, "memset: NULL pointer");
    MGGX_HIP(hipMemsetAsync(d_ptr, value, bytes, state().stream));
    return MGGX_OK;
}

MGGX_EXPORT int mggx_memcpy_h2d(void *d_dst, const void *src, size_t bytes)
{
    if (!bytes) return MGGX_OK;
    if (!d_dst || !src) return fail(MGGX_EINVAL, "memcpy_h2d: NULL pointer");
    MGGX_HIP(hipMemcpyAsync(d_dst, src, bytes, hipMemcpyHostToDevice, state().stream));
    MGGX_HIP(hipStreamSynchronize(state().stream));
    return MGGX_OK;
}

MGGX_EXPORT int mggx_memcpy_d2h(void *dst, const void *d_src, size_t bytes)
{
    if (!bytes) return MGGX_OK;
    if (!dst || !d_src) return fail(MGGX_EINVAL, "memcpy_d2h: NULL pointer");
    MGGX_HIP(hipMemcpyAsync(dst, d_src, bytes, hipMemcpyDeviceToHost, state().stream));
    MGGX_HIP(hipStreamSynchronize(state().stream));
    return MGGX_OK;
}

MGGX_EXPORT int mggx_memcpy_d2d(void *d_dst, const void *d_src, size_t bytes)
{
    if (!bytes) return MGGX_OK;
    if (!d_dst || !d_src) return fail(MGGX_EINVAL, "memcpy_d2d: NULL pointer");
    MGGX_HIP(hipMemcpyAsync(d_dst, d_src, bytes, hipMemcpyDeviceToDevice, state().stream));
    return MGGX_OK;
}

namespace {
struct Timer {
    hipEvent_t start, stop;
};
}  // namespace

MGGX_EXPORT int mggx_timer_create(void **timer)
{
    if (!timer) return fail(MGGX_EINVAL, "timer_create: NULL");
    int rc = mggx::ensure_init();
    if (rc) return rc;
    Timer *t = new Timer;
    if (hipEventCreate(&t->start) != hipSuccess || hipEventCreate(&t->stop) != hipSuccess) {
        delete t;
        return fail(MGGX_EHIP, "timer_create: hipEventCreate failed");
    }
    *timer = t;
    return MGGX_OK;
}

MGGX_EXPORT int mggx_timer_start(void *timer)
{
    if (!timer) return fail(MGGX_EINVAL, "timer_start: NULL");
    MGGX_HIP(hipEventRecord(static_cast<Timer *>(timer)->start, state().stream));
    return MGGX_OK;
}

MGGX_EXPORT int mggx_timer_stop(void *timer)
{
    if (!timer) return fail(MGGX_EINVAL, "timer_stop: NULL");
    MGGX_HIP(hipEventRecord(static_cast<Timer *>(timer)->stop, state().stream));
    return MGGX_OK;
}

MGGX_EXPORT int mggx_timer_elapsed_ms(void *timer, float *ms)
{
    if (!timer || !ms) return fail(MGGX_EINVAL, "timer_elapsed_ms: NULL");
    Timer *t = static_cast<Timer *>(timer);
    MGGX_HIP(hipEventSynchronize(t->stop));
    MGGX_HIP(hipEventElapsedTime(ms, t->start, t->stop));
    return MGGX_OK;
}

MGGX_EXPORT int mggx_timer_destroy(void *timer)
{
    if (!timer) return MGGX_OK;
    Timer *t = static_cast<Timer *>(timer);
    (void)hipEventDestroy(t->start);
    (void)hipEventDestroy(t->stop);
    delete t;
    return MGGX_OK;
}

MGGX_EXPORT int mggx_release_cached(void)
{
    mggx::State &s = state();
    if (s.device >= 0) MGGX_HIP(hipStreamSynchronize(s.stream));
    {   // dense-core plans first: freeing one also forgets the plans of its remainder CSR
        std::vector<mggx::CorePlan *> cores;
        cores.swap(s.cores);
        for (mggx::CorePlan *c : cores) mggx::core_plan_free(c);
    }
    if (s.core_ws) {
        MGGX_HIP(hipFree(s.core_ws));
        s.core_ws = nullptr;
        s.core_ws_bytes = 0;
    }
    for (mggx::Plan *p : s.plans) mggx::plan_free(p);
    s.plans.clear();
    for (mggx::GraphInfo &g : s.graphs) mggx::guard_free(g.guard);
    s.graphs.clear();
    if (s.ws) {
        MGGX_HIP(hipFree(s.ws));
        s.ws = nullptr;
        s.ws_bytes = 0;
    }
    for (void *p : s.retired) (void)hipFree(p);
    s.retired.clear();
    s.retired_bytes = 0;
    s.ws_captured = s.core_ws_captured = false;
    if (s.h_stale) *s.h_stale = 0;
    return MGGX_OK;
}

MGGX_EXPORT int mggx_set_plan_check(int on)
{
    if (on < 0 || on > 2) return fail(MGGX_EINVAL, "set_plan_check: level %d (0, 1 or 2)", on);
    state().plan_check = on;
    return MGGX_OK;
}

MGGX_EXPORT int mggx_cache_stats(mggx_cache_stats_t *out)
{
    if (!out) return fail(MGGX_EINVAL, "cache_stats: NULL");
    mggx::State &s = state();
    *out = mggx_cache_stats_t{};
    for (const mggx::Plan *p : s.plans) {
        out->plans += 1;
        out->plan_bytes += (int64_t)p->bytes;
    }
    for (const mggx::CorePlan *c : s.cores) {
        out->core_plans += 1;
        out->core_plan_bytes += (int64_t)c->bytes;
    }
    out->workspace_bytes = (int64_t)s.ws_bytes;
    out->core_scratch_bytes = (int64_t)s.core_ws_bytes;
    out->retired_bytes = (int64_t)s.retired_bytes;
    out->plan_build_ms = s.plan_build_ms;
    out->core_plan_build_ms = s.core_plan_build_ms;
    out->search_ms = s.search_ms;
    return MGGX_OK;
}

// ---------------------------------------------------------------------------
// Utility kernels.
namespace {

__global__ void __launch_bounds__(256) k_copy16(int4 *__restrict__ dst, const int4 *__restrict__ src, size_t n16)
{
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * 256;
    for (; i < n16; i += stride) dst[i] = src[i];
}

// The same copy with streaming hints: four 16-byte non-temporal loads in flight per thread before the first store, one
// workgroup per 16 KiB, no grid-stride loop.  Second opinion on the copy ceiling.
__global__ void __launch_bounds__(256) k_copy16_nt(int4 *__restrict__ dst, const int4 *__restrict__ src, size_t n16)
{
    typedef int v4i __attribute__((ext_vector_type(4)));
    const size_t base = (size_t)blockIdx.x * 1024 + threadIdx.x;
    v4i v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const size_t i = base + 256 * (size_t)j;
        if (i < n16) v[j] = __builtin_nontemporal_load(reinterpret_cast<const v4i *>(src) + i);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const size_t i = base + 256 * (size_t)j;
        if (i < n16) __builtin_nontemporal_store(v[j], reinterpret_cast<v4i *>(dst) + i);
    }
}

__global__ void __launch_bounds__(256) k_cast_bf16(unsigned short *__restrict__ dst, const float *__restrict__ src, long long n)
{
    long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    const long long stride = (long long)gridDim.x * 256;
    for (; i < n; i += stride) {
        unsigned u = __float_as_uint(src[i]);
        unsigned r;
        if ((u & 0x7F800000u) == 0x7F800000u && (u & 0x007FFFFFu)) r = (u >> 16) | 0x40u;  // quiet NaN
        else r = (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;                                    // round to nearest even
        dst[i] = (unsigned short)r;
    }
}

// Yardstick: fp32 -> bf16 (truncated) of n8 groups of 8 values, 32 bytes in and 16 out per lane with the streaming hint.
// Pieces of 2048 values (8 KB in, 4 KB out) per round of a workgroup; workgroup b takes pieces [b * per_wg, (b + 1) * per_wg)
// one after the other, or, with stride_pieces > 0, pieces b, b + stride_pieces, ... (a persistent grid).
__global__ void __launch_bounds__(256) k_convert_probe(unsigned *__restrict__ dst, const float *__restrict__ src, long long n8, long long pieces,
                                                       int per_wg, long long stride_pieces)
{
    typedef float v4f_p __attribute__((ext_vector_type(4)));
    typedef unsigned v4u_p __attribute__((ext_vector_type(4)));
    const auto pack = [](float a, float b) { return (__float_as_uint(a) >> 16) | (__float_as_uint(b) & 0xFFFF0000u); };
    long long piece = stride_pieces > 0 ? (long long)blockIdx.x : (long long)blockIdx.x * per_wg;
    const long long end = stride_pieces > 0 ? pieces : min(pieces, piece + per_wg), step = stride_pieces > 0 ? stride_pieces : 1;
    for (; piece < end; piece += step) {
        const long long i = piece * 256 + threadIdx.x;
        if (i >= n8) continue;
        const v4f_p a = __builtin_nontemporal_load(reinterpret_cast<const v4f_p *>(src) + 2 * i);
        const v4f_p b = __builtin_nontemporal_load(reinterpret_cast<const v4f_p *>(src) + 2 * i + 1);
        const v4u_p o = {pack(a.x, a.y), pack(a.z, a.w), pack(b.x, b.y), pack(b.z, b.w)};
        __builtin_nontemporal_store(o, reinterpret_cast<v4u_p *>(dst) + i);
    }
}

// dst row i = table row ids[i]; rows of v16 16-byte pieces
__global__ void __launch_bounds__(256) k_gather_rows(int4 *__restrict__ dst, const int4 *__restrict__ table, const int *__restrict__ ids,
                                                     long long n, int v16)
{
    const long long total = n * v16;
    for (long long idx = (long long)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (long long)gridDim.x * 256) {
        const long long i = idx / v16;
        const int p = (int)(idx % v16);
        dst[idx] = table[(long long)ids[i] * v16 + p];
    }
}

// Yardstick for gathers: every slot of LPR lanes loads rows at pseudo-random indices of the table, eight loads in
// flight, with no index array to read and no reduction structure; each lane sums what it loads and stores the sum.
typedef unsigned probe_v4u __attribute__((ext_vector_type(4)));

template <int LPR>
__global__ void __launch_bounds__(256) k_gather_probe(float *__restrict__ sink, const char *__restrict__ table, unsigned rows,
                                                      unsigned ld_bytes, int lanes_on, int iters, unsigned seed)
{
    constexpr int S = 64 / LPR;
    const int lane = (int)(threadIdx.x & 63u), wave = (int)(threadIdx.x >> 6);
    const int slot = lane / LPR, l = lane % LPR;
    unsigned x = ((((unsigned)blockIdx.x * 4u + (unsigned)wave) * S + (unsigned)slot) + 1u) * 2654435761u ^ seed;
    x ^= x >> 15; x *= 2246822519u; x ^= x >> 13;
    const bool on = l < lanes_on;
    const unsigned cofs = 16u * (unsigned)(on ? l : 0);
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; ++it) {
        unsigned r[8];
        probe_v4u v[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            x = x * 1664525u + 1013904223u;
            r[t] = __umulhi(x ^ (x >> 16), rows);
            v[t] = (probe_v4u){0u, 0u, 0u, 0u};
        }
        if (on) {
#pragma unroll
            for (int t = 0; t < 8; ++t) v[t] = *reinterpret_cast<const probe_v4u *>(table + (size_t)r[t] * ld_bytes + cofs);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < 8; ++t) {
            acc[0] += __uint_as_float(v[t].x); acc[1] += __uint_as_float(v[t].y);
            acc[2] += __uint_as_float(v[t].z); acc[3] += __uint_as_float(v[t].w);
        }
    }
    sink[(size_t)blockIdx.x * 256 + threadIdx.x] = acc[0] + acc[1] + acc[2] + acc[3];
}

constexpr int PROBE_BLOCKS = 1024;

// Yardstick for the dense-core kernel's LDS reads: every lane adds N4 16-byte pieces of an LDS tile row at a
// pseudo-random column per step (tile [N4][257] like the core kernel's, 4 wavefronts per workgroup), four steps per
// index draw; no global memory traffic inside the loop.
typedef float probe_v4f __attribute__((ext_vector_type(4)));

template <int N4>
__global__ void __launch_bounds__(256) k_lds_probe(float *__restrict__ sink, int iters, unsigned seed)
{
    constexpr int TC = 256, TP = TC + 1;
    extern __shared__ probe_v4f probe_tile[];
    for (int i = (int)threadIdx.x; i < N4 * TP; i += 256) probe_tile[i] = (probe_v4f){1.f, 0.f, 0.f, 0.f};
    __syncthreads();
    unsigned x = ((unsigned)blockIdx.x * 256u + threadIdx.x + 1u) * 2654435761u ^ seed;
    probe_v4f acc[N4];
#pragma unroll
    for (int s = 0; s < N4; ++s) acc[s] = (probe_v4f){0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; ++it) {
        x = x * 1664525u + 1013904223u;
        const unsigned r = x ^ (x >> 13);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const probe_v4f *q = probe_tile + ((r >> (8 * j)) & 255u);
#pragma unroll
            for (int s = 0; s < N4; ++s) acc[s] += q[s * TP];
        }
    }
    probe_v4f t = acc[0];
#pragma unroll
    for (int s = 1; s < N4; ++s) t += acc[s];
    sink[(size_t)blockIdx.x * 256 + threadIdx.x] = t.x + t.y + t.z + t.w;
}

template <int N4>
int launch_lds_probe(float *sink, int blocks, int iters, unsigned seed, hipStream_t stream)
{
    const size_t lds = (size_t)N4 * 257 * sizeof(probe_v4f);
    static bool raised = false;
    if (lds > 48 * 1024 && !raised) {
        MGGX_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(k_lds_probe<N4>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        raised = true;
    }
    k_lds_probe<N4><<<dim3((unsigned)blocks), dim3(256), lds, stream>>>(sink, iters, seed);
    MGGX_LAUNCH_CHECK("k_lds_probe");
    return MGGX_OK;
}

// Workgroups of the LDS yardstick: as many as are resident at once (160 KB of LDS and 8 workgroups of 4 wavefronts per
// CU), so the launch is one full wave of workgroups and no second, partly filled one dilutes the rate.
int lds_probe_blocks(size_t lds_bytes)
{
    static int cus = 0;
    if (!cus) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return PROBE_BLOCKS;
        cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    }
    const long long fit = std::min<long long>(8, (160 * 1024) / (long long)lds_bytes);
    return (int)std::min<long long>(PROBE_BLOCKS, std::max<long long>(1, fit) * cus);
}

}  // namespace

MGGX_EXPORT int mggx_lds_probe(float *d_sink, size_t row_bytes, int64_t n_reads, unsigned seed, int64_t *n_done)
{
    if (!d_sink || row_bytes < 16 || row_bytes > 256 || (row_bytes % 16) || n_reads < 1)
        return fail(MGGX_EINVAL, "lds_probe: NULL sink, or rows not 16..256 bytes in 16-byte pieces");
    const int blocks = lds_probe_blocks(row_bytes / 16 * 257 * sizeof(probe_v4f));
    const long long per_iter = (long long)blocks * 256 * 4;
    const long long iters = (n_reads + per_iter - 1) / per_iter;
    if (iters > 0x7fffffffLL) return fail(MGGX_ELIMIT, "lds_probe: too many reads");
    int rc;
    switch ((int)(row_bytes / 16)) {
#define MGGX_CASE(N) case N: rc = launch_lds_probe<N>(d_sink, blocks, (int)iters, seed, state().stream); break;
        MGGX_CASE(1) MGGX_CASE(2) MGGX_CASE(3) MGGX_CASE(4) MGGX_CASE(5) MGGX_CASE(6) MGGX_CASE(7) MGGX_CASE(8)
        MGGX_CASE(9) MGGX_CASE(10) MGGX_CASE(11) MGGX_CASE(12) MGGX_CASE(13) MGGX_CASE(14) MGGX_CASE(15) MGGX_CASE(16)
#undef MGGX_CASE
        default: rc = fail(MGGX_EINVAL, "lds_probe: row of %zu bytes", row_bytes);
    }
    if (rc) return rc;
    if (n_done) *n_done = iters * per_iter;
    return MGGX_OK;
}

MGGX_EXPORT int mggx_gather_probe(float *d_sink, const void *d_table, int64_t rows, size_t ld_bytes, size_t row_bytes,
                                  int64_t n_gathers, unsigned seed, int64_t *n_done)
{
    if (!d_sink || !d_table || rows < 1 || rows > 0x7fffffffLL || row_bytes < 16 || row_bytes > 256 || (row_bytes % 16) ||
        ld_bytes < row_bytes || (ld_bytes % 16) || ld_bytes > 0xffffffffull || n_gathers < 1 ||
        (reinterpret_cast<uintptr_t>(d_table) & 15u))
        return fail(MGGX_EINVAL, "gather_probe: NULL pointer, rows of 16..256 bytes in 16-byte pieces, or misaligned table");
    const int lanes_on = (int)(row_bytes / 16);
    const int lpr = lanes_on <= 4 ? 4 : 16;
    const long long per_iter = (long long)PROBE_BLOCKS * 4 * (64 / lpr) * 8;
    long long iters = (n_gathers + per_iter - 1) / per_iter;
    if (iters > 0x7fffffffLL) return fail(MGGX_ELIMIT, "gather_probe: too many gathers");
    if (lpr == 4)
        k_gather_probe<4><<<dim3(PROBE_BLOCKS), dim3(256), 0, state().stream>>>(d_sink, (const char *)d_table, (unsigned)rows,
                                                                                 (unsigned)ld_bytes, lanes_on, (int)iters, seed);
    else
        k_gather_probe<16><<<dim3(PROBE_BLOCKS), dim3(256), 0, state().stream>>>(d_sink, (const char *)d_table, (unsigned)rows,
                                                                                  (unsigned)ld_bytes, lanes_on, (int)iters, seed);
    MGGX_LAUNCH_CHECK("k_gather_probe");
    if (n_done) *n_done = iters * per_iter;
    return MGGX_OK;
}

MGGX_EXPORT int mggx_copy_bytes(void *d_dst, const void *d_src, size_t n)
{
    if (!d_dst || !d_src || (n % 16)) return fail(MGGX_EINVAL, "copy_bytes: NULL pointer or size not a multiple of 16");
    if (!n) return MGGX_OK;
    const size_t n16 = n / 16;
    size_t blocks = (n16 + 255) / 256;
    if (blocks > 256 * 64) blocks = 256 * 64;
    k_copy16<<<dim3((unsigned)blocks), dim3(256), 0, state().stream>>>((int4 *)d_dst, (const int4 *)d_src, n16);
    MGGX_LAUNCH_CHECK("k_copy16");
    return MGGX_OK;
}

MGGX_EXPORT int mggx_copy_bytes_nt(void *d_dst, const void *d_src, size_t n)
{
    if (!d_dst || !d_src || (n % 16)) return fail(MGGX_EINVAL, "copy_bytes_nt: NULL pointer or size not a multiple of 16");
    if (!n) return MGGX_OK;
    const size_t n16 = n / 16;
    const size_t blocks = (n16 + 1023) / 1024;
    if (blocks > 0x7fffffffull) return fail(MGGX_ELIMIT, "copy_bytes_nt: %zu bytes", n);
    k_copy16_nt<<<dim3((unsigned)blocks), dim3(256), 0, state().stream>>>((int4 *)d_dst, (const int4 *)d_src, n16);
    MGGX_LAUNCH_CHECK("k_copy16_nt");
    return MGGX_OK;
}

MGGX_EXPORT int mggx_gather_rows(void *d_dst, const void *d_table, const int *d_ids, int64_t n, size_t row_bytes)
{
    if (n < 0 || (n && (!d_dst || !d_table || !d_ids)) || row_bytes == 0 || (row_bytes % 16) ||
        ((reinterpret_cast<uintptr_t>(d_dst) | reinterpret_cast<uintptr_t>(d_table)) & 15u))
        return fail(MGGX_EINVAL, "gather_rows: NULL pointer, or rows not 16-byte multiples / aligned");
    if (!n) return MGGX_OK;
    const long long total = (long long)n * (long long)(row_bytes / 16);
    long long blocks = (total + 255) / 256;
    if (blocks > 256 * 64) blocks = 256 * 64;
    k_gather_rows<<<dim3((unsigned)blocks), dim3(256), 0, state().stream>>>((int4 *)d_dst, (const int4 *)d_table, d_ids, (long long)n,
                                                                             (int)(row_bytes / 16));
    MGGX_LAUNCH_CHECK("k_gather_rows");
    return MGGX_OK;
}

MGGX_EXPORT int mggx_cast_f32_to_bf16(void *d_dst, const float *d_src, int64_t n)
{
    if (n < 0 || (n && (!d_dst || !d_src))) return fail(MGGX_EINVAL, "cast_f32_to_bf16: bad argument");
    if (!n) return MGGX_OK;
    long long blocks = (n + 255) / 256;
    if (blocks > 256 * 64) blocks = 256 * 64;
    k_cast_bf16<<<dim3((unsigned)blocks), dim3(256), 0, state().stream>>>((unsigned short *)d_dst, d_src, (long long)n);
    MGGX_LAUNCH_CHECK("k_cast_bf16");
    return MGGX_OK;
}

MGGX_EXPORT int mggx_convert_probe(void *d_dst, const float *d_src, int64_t n, int pieces_per_workgroup, int persistent_workgroups)
{
    if (n < 0 || n % 8 || pieces_per_workgroup < 1 || persistent_workgroups < 0 || (n && (!d_dst || !d_src)) ||
        (reinterpret_cast<uintptr_t>(d_dst) & 15u) || (reinterpret_cast<uintptr_t>(d_src) & 15u))
        return fail(MGGX_EINVAL, "convert_probe: bad argument");
    if (!n) return MGGX_OK;
    const long long n8 = n / 8, pieces = (n8 + 255) / 256;
    const long long wgs = persistent_workgroups ? std::min<long long>(persistent_workgroups, pieces) : (pieces + pieces_per_workgroup - 1) / pieces_per_workgroup;
    if (wgs > 0x7fffffffLL) return fail(MGGX_ELIMIT, "convert_probe: too many workgroups");
    k_convert_probe<<<dim3((unsigned)wgs), dim3(256), 0, state().stream>>>((unsigned *)d_dst, d_src, n8, pieces, pieces_per_workgroup,
                                                                          persistent_workgroups ? wgs : 0);
    MGGX_LAUNCH_CHECK("k_convert_probe");
    return MGGX_OK;
}

MGGX_EXPORT int mggx_set_gather_addressing(int mode)
{
    if (mode != 0 && mode != 1) return fail(MGGX_EINVAL, "set_gather_addressing: mode %d", mode);
    state().gather_addressing = mode;
    return MGGX_OK;
}

MGGX_EXPORT int mggx_last_agg_kernel(char *buf, size_t len)
{
    if (!buf || !len) return fail(MGGX_EINVAL, "last_agg_kernel: NULL buffer");
    snprintf(buf, len, "%s", state().last_kernel);
    return MGGX_OK;
}
