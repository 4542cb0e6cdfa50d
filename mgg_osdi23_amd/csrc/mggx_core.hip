// Dense core of a power-law graph served from LDS.
//
// Where a few thousand high-degree rows hold most of the edges among themselves, the aggregation of that core x core
// block does not need one gather per edge from the caches: the feature rows of 256 core columns at a time are staged
// in LDS with whole-line reads, and every lane owns one core row and adds the LDS rows its index list names
// (sliced-ELL lists over degree-ranked rows, so the 64 lanes of a wavefront have lists of similar length).  The
// block's sums go to partial rows, one per row and run of column tiles a workgroup takes.  This kernel is bound by the
// LDS, the ordinary aggregation of the rest of the CSR by the caches, so the caller runs the two side by side on two
// streams; k_core_finish then adds the partial rows to the output the aggregation wrote.
#include <algorithm>
#include <chrono>
#include <cmath>
#include <functional>
#include <new>
#include <type_traits>

#include <rocprim/device/device_radix_sort.hpp>

#include "mggx_dev.h"

namespace mggx {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef unsigned short us4 __attribute__((ext_vector_type(4)));

#ifndef MGGX_CORE_WAVES_PER_EU
#define MGGX_CORE_WAVES_PER_EU 0
#endif
#if MGGX_CORE_WAVES_PER_EU > 0
#define MGGX_CORE_OCCUPANCY __attribute__((amdgpu_waves_per_eu(MGGX_CORE_WAVES_PER_EU)))
#elif defined(MGGX_CORE_NUM_VGPR)
#define MGGX_CORE_OCCUPANCY __attribute__((amdgpu_num_vgpr(MGGX_CORE_NUM_VGPR)))
#else
#define MGGX_CORE_OCCUPANCY
#endif
#ifndef MGGX_CORE_READS
#define MGGX_CORE_READS 8  // LDS reads of one list entry issued back to back (see core_sell_body)
#endif

template <int I, int N, typename F>
__device__ __forceinline__ void static_for_core(F &&f)
{
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for_core<I + 1, N>(f);
    }
}

constexpr int CORE_TC = 256;    // core columns per LDS tile
constexpr int CORE_ZERO_COLS = 16;  // zero columns behind them: what the lists' padding entries point at (k_core_bank_order)
// Slices (of 64 rows) per workgroup, WAVES below: 4 -- as small as the aggregation's own workgroups, so the two kernels
// of a call, running side by side, find room on a CU equally easily -- or 8 where rows are summed in two halves: every
// workgroup stages every tile of its run, so the tiles staged per call are (row groups) x (tiles); with 98,304 core rows
// of 256 bytes that is 9.7 GB of L2 reads per call at 4 slices and half of it at 8 (2.45 M-node graph, width 64: 2.93 ->
// 2.68 ms per aggregation with two 8-wavefront workgroups per CU; one 16-wavefront workgroup: 2.66; at widths 16 and 44 on
// the 233 K-node graph, whose 15 / 45 MB tables sit in the L2, 8 slices cost 15 and 33 %).

// tab[s * tab_stride(core) + i] = elements 4 s .. 4 s + 3 of the feature row of the rank-i node (zero past dim)
__global__ void __launch_bounds__(256) k_core_stage(v4f *__restrict__ tab, const float *__restrict__ in, const int *__restrict__ order,
                                                    int core, int n4, int dim, long long ld_in, int vec_in, const Gate gate)
{
    if (gate_closed(gate)) return;
    const int i = (int)(blockIdx.x * 256 + threadIdx.x), s = (int)blockIdx.y;  // (no division by a run-time value: one slice per grid row)
    if (i >= core) return;
    const float *row = in + (long long)order[i] * ld_in + 4 * s;
    v4f v;
    if (vec_in && 4 * s + 3 < dim) {
        v = *reinterpret_cast<const v4f *>(row);
    } else {
        v.x = 4 * s < dim ? row[0] : 0.f;
        v.y = 4 * s + 1 < dim ? row[1] : 0.f;
        v.z = 4 * s + 2 < dim ? row[2] : 0.f;
        v.w = 4 * s + 3 < dim ? row[3] : 0.f;
    }
    tab[(size_t)s * tab_stride(core) + i] = v;
}

// The body for the 16-byte pieces [S0, S0 + NS) of rows of N4 pieces.
template <int N4, int S0, int NS, int WAVES>
__device__ __forceinline__ void core_sell_body(const unsigned *__restrict__ blk_off, const unsigned short *__restrict__ idx,
                                               const v4f *__restrict__ tab, v4f *__restrict__ partial, const int4 wg, int core, int ntiles,
                                               v4f *tile)
{
    constexpr int TC = CORE_TC, TP = TC + CORE_ZERO_COLS;  // columns TC .. TP - 1 of every slice row are zero: what padding entries read; tile[NS][TP]
    const int lane = (int)(threadIdx.x & 63u), wave = (int)(threadIdx.x >> 6);
    const int g = wg.x * WAVES + wave;
    const int t0 = wg.y, t1 = wg.z;
    v4f acc[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s) acc[s] = (v4f){0.f, 0.f, 0.f, 0.f};
    if ((int)threadIdx.x < NS * CORE_ZERO_COLS)
        tile[((int)threadIdx.x / CORE_ZERO_COLS) * TP + TC + (int)threadIdx.x % CORE_ZERO_COLS] = (v4f){0.f, 0.f, 0.f, 0.f};
    const us4 *p = reinterpret_cast<const us4 *>(idx) + lane;
    unsigned pos = blk_off[(size_t)g * ntiles + t0];
    const unsigned end_run = blk_off[(size_t)g * ntiles + t1];
    const us4 pad = (us4){TC, TC, TC, TC};
    us4 cur = pos < end_run ? p[(size_t)pos * 64] : pad;  // the lists of a slice's tiles follow one another: read one chunk ahead
    for (int t = t0; t < t1; ++t) {
        __syncthreads();
        for (int i = (int)threadIdx.x; i < NS * TC; i += WAVES * 64) {
            const int s = i / TC, c = i % TC;
            tile[s * TP + c] = tab[(size_t)(S0 + s) * tab_stride(core) + (size_t)t * TC + c];
        }
        const unsigned b1 = blk_off[(size_t)g * ntiles + t + 1];
        __syncthreads();
        while (pos < b1) {
            const us4 nxt = pos + 1 < end_run ? p[(size_t)(pos + 1) * 64] : pad;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int c = cur[j];
                const v4f *q = tile + c;  // a column of the tile or, for a padding entry, one of the zero columns behind it
                // at most MGGX_CORE_READS LDS reads in flight per entry: wide rows otherwise cost a wavefront a hundred
                // registers, and this kernel shares each SIMD's register file with the aggregation running beside it
                constexpr int GROUPS = (NS + MGGX_CORE_READS - 1) / MGGX_CORE_READS, H = (NS + GROUPS - 1) / GROUPS;
                static_for_core<0, GROUPS>([&](auto gg) {
                    constexpr int s0 = decltype(gg)::value * H, s1 = s0 + H < NS ? s0 + H : NS;
#pragma unroll
                    for (int s = s0; s < s1; ++s) acc[s] += q[s * TP];
                    if constexpr (GROUPS > 1) __builtin_amdgcn_sched_barrier(0);
                });
            }
            cur = nxt;
            ++pos;
        }
    }
    const size_t r = (size_t)wg.w * (WAVES * 64) + (size_t)(wave * 64 + lane);
#pragma unroll
    for (int s = 0; s < NS; ++s) partial[r * N4 + S0 + s] = acc[s];
}

// One workgroup = WAVES slices (a row group) x a run of column tiles [x all pieces of the rows, or one half of
// them when SPLIT: blockIdx.y]; lane = core row.  Row groups and tiles are both sorted by degree, so the work of a
// (row group, tile) cell spans two orders of magnitude: the plan cuts every row group's tiles into runs of about equal
// list length (wgs[i] = {row group, first tile, end tile, slot}), so all workgroups take about the same time and the
// launch has no tail of a few heavy ones.
// partial[(slot * WAVES * 64 + row in the group) * N4 + s]
template <int N4, bool SPLIT, int WAVES>
__global__ void __launch_bounds__(WAVES * 64) MGGX_CORE_OCCUPANCY k_core_sell(const unsigned *__restrict__ blk_off, const unsigned short *__restrict__ idx,
                                                               const v4f *__restrict__ tab, v4f *__restrict__ partial,
                                                               const int4 *__restrict__ wgs, int core, int ntiles, const Gate gate)
{
    extern __shared__ v4f tile[];
    if (gate_closed(gate)) return;
    const int4 wg = wgs[blockIdx.x];
    if constexpr (!SPLIT) {
        core_sell_body<N4, 0, N4, WAVES>(blk_off, idx, tab, partial, wg, core, ntiles, tile);
    } else {
        constexpr int A = (N4 + 1) / 2;
        if (blockIdx.y == 0) core_sell_body<N4, 0, A, WAVES>(blk_off, idx, tab, partial, wg, core, ntiles, tile);
        else core_sell_body<N4, A, N4 - A, WAVES>(blk_off, idx, tab, partial, wg, core, ntiles, tile);
    }
}

// The partial rows of a row group (one per workgroup that worked on it) summed, in slot order, into one row per core row:
// sums[r * n4 + q], r = rank.  It follows the LDS kernel on its stream, which as a rule is done before the gather kernel
// beside it, so the kernel that finishes the rows after the join reads one partial row per core row at an address the
// rank alone gives (one dependent load instead of the row group's slot range and a walk over up to a dozen slots;
// 36,864 core rows of the 233 K-node graph at width 41: 113 -> 62 us of finishing kernel went into that walk).  `sums` is
// the staged table's memory, which nobody reads once the LDS kernel has finished.
__global__ void __launch_bounds__(256) k_core_reduce(v4f *__restrict__ sums, const v4f *__restrict__ partial, const int *__restrict__ wg_base, int core,
                                                     int n4, int group_shift, int g_shift, const Gate gate)
{
    if (gate_closed(gate)) return;
    const int G = 1 << g_shift, group_rows = 1 << group_shift;
    const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
    const long long r_ll = idx >> g_shift;
    const int q = (int)(idx & (G - 1));
    if (r_ll >= core || q >= n4) return;
    const int r = (int)r_ll, grp = r >> group_shift, in_grp = r & (group_rows - 1);
    const int s1 = wg_base[grp + 1];
    int slot = wg_base[grp];
    const size_t stride = (size_t)group_rows * n4;
    const v4f *src = partial + (size_t)in_grp * n4 + q;
    v4f sum = {0.f, 0.f, 0.f, 0.f};
    for (; slot + 4 <= s1; slot += 4) {  // four partial rows in flight, summed in order
        const v4f p0 = src[(size_t)slot * stride], p1 = src[(size_t)(slot + 1) * stride];
        const v4f p2 = src[(size_t)(slot + 2) * stride], p3 = src[(size_t)(slot + 3) * stride];
        sum += p0;
        sum += p1;
        sum += p2;
        sum += p3;
    }
    for (; slot < s1; ++slot) sum += src[(size_t)slot * stride];
    sums[(size_t)r * n4 + q] = sum;
}

// Adds the core block's sums to output rows that already hold the rest of the aggregation:
// out[v] = post(out[v] + scale[v] * sums[rank of v]), post = ReLU and / or row softmax.
// G lanes per row (a power of two >= ceil(dim/4)), lane q holds columns 4 q .. 4 q + 3.  all_rows = 0: the core rows only
// (index -> rank -> row); all_rows = 1: every row (needed when there is a post-operation).
__global__ void __launch_bounds__(256) k_core_finish(float *__restrict__ out, const v4f *__restrict__ sums, const int *__restrict__ rank,
                                                     const int *__restrict__ order, const float *__restrict__ rs, int rows, int dim,
                                                     long long ld_out, int core, int g_shift, int relu, int softmax, int all_rows, int vec_out,
                                                     const Gate gate)
{
    if (gate_closed(gate)) return;
    const int G = 1 << g_shift;  // lanes per row, a power of two: shifts, not divisions by a run-time value
    const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
    const long long i_ll = idx >> g_shift;
    const int q = (int)(idx & (G - 1)), n4 = (dim + 3) >> 2;
    if (i_ll >= (all_rows ? rows : core)) return;  // G divides 64: the lanes of a row leave together
    const int i = (int)i_ll;
    const int v = all_rows ? i : order[i];
    const int r = all_rows ? rank[i] : i;
    const bool lane_on = q < n4;
    float val[4] = {0.f, 0.f, 0.f, 0.f};
    bool on[4];
    float *o = out + (long long)v * ld_out + 4 * q;
    const bool whole = vec_out && 4 * q + 3 < dim;  // this lane's four elements as one 16-byte access
    if (lane_on) {
        v4f sum = {0.f, 0.f, 0.f, 0.f};
        v4f cur = {0.f, 0.f, 0.f, 0.f};
        if (whole) {
            cur = *reinterpret_cast<const v4f *>(o);
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (4 * q + j < dim) cur[j] = o[j];
        }
        if (r >= 0) {
            sum = sums[(size_t)r * n4 + q];
            if (rs) sum *= rs[v];
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            on[j] = 4 * q + j < dim;
            val[j] = on[j] ? cur[j] + sum[j] : 0.f;
            if (relu) val[j] = fmaxf(val[j], 0.f);
        }
    } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) on[j] = false;
    }
    if (softmax) {
        const int lane = (int)(threadIdx.x & 63u);
        float m = -3.0e38f;
#pragma unroll
        for (int j = 0; j < 4; ++j) m = on[j] ? fmaxf(m, val[j]) : m;
        for (int s = 1; s < G; s <<= 1) m = fmaxf(m, __shfl(m, lane ^ s, 64));
        float tot = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            val[j] = on[j] ? __expf(val[j] - m) : 0.f;
            tot += val[j];
        }
        for (int s = 1; s < G; s <<= 1) tot += __shfl(tot, lane ^ s, 64);
        const float inv = 1.0f / tot;
#pragma unroll
        for (int j = 0; j < 4; ++j) val[j] *= inv;
    }
    if (lane_on) {
        if (whole) {
            *reinterpret_cast<v4f *>(o) = (v4f){val[0], val[1], val[2], val[3]};
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (on[j]) o[j] = val[j];
        }
    }
}

// ---- the plan, built on the GPU (same arrays, bit for bit, as core_layout_build makes on the host) ----

__global__ void __launch_bounds__(256) k_core_deg(const int *__restrict__ ptr, int rows, int *__restrict__ deg, int *__restrict__ ids)
{
    const int v = blockIdx.x * 256 + threadIdx.x;
    if (v >= rows) return;
    deg[v] = ptr[v + 1] - ptr[v];
    ids[v] = v;
}

// sorted = row ids by falling degree, ties by rising id: the first `core` are the core, in rank order
__global__ void __launch_bounds__(256) k_core_rank(const int *__restrict__ sorted, int rows, int core, int *__restrict__ order, int *__restrict__ rank)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= rows) return;
    const int v = sorted[i];
    if (i < core) {
        order[i] = v;
        rank[v] = i;
    } else {
        rank[v] = -1;
    }
}

// Bank order of the lists.  The LDS has 64 banks of 4 bytes: a 16-byte read of a wavefront is served 16 lanes at a time
// (lanes 16 k .. 16 k + 15 together), in one cycle when the 16 pieces lie in 16 different groups of four banks -- tile
// columns that differ mod 16 -- and otherwise in as many cycles as the fullest group has distinct addresses (measured
// with SQ_LDS_BANK_CONFLICT on access patterns made for it: 4 cycles per read at best, 12.2 with random columns; the
// lists in edge order took 8.3, about a third of the kernel's time).  Which entry of its list a lane reads at which
// position is free -- the sum does not care -- and so is where in the list its padding goes, so the entries of a
// (slice, tile) block are placed for the 16 lanes of a group together: position by position, first the lanes that
// have no padding left to spend, then the others, each in lane order, a lane takes the first of its remaining entries
// (looking from residue (lane + p) mod 16 upwards, edge order inside a residue) whose residue no lane of the group has
// taken at this position; a lane that finds none spends a padding slot if it has one, else takes a residue twice.
// Padding slots point at one of CORE_ZERO_COLS zero columns behind the tile, tc + r, with r the residues still free
// at that position in turn.  On the 233 K-node benchmark graph that leaves 4.01 cycles per read.  One wavefront per
// block, lane = list; a block of more than BANK_MAX_POS positions (only a CSR with repeated edges has one) keeps its
// edge order.  The host-side builder does the same (core_bank_order).
constexpr int BANK_MAX_POS = 256;
static_assert(CORE_TC <= 256, "k_core_bank_order keeps tile offsets in bytes");

// the lowest set bit of the 16-bit mask m when looking from bit k upwards, cyclically; -1 if m is empty
__device__ __forceinline__ int first_from(unsigned m, int k)
{
    const unsigned mr = ((m >> k) | (m << (16 - k))) & 0xFFFFu;
    return mr ? ((__ffs((int)mr) - 1 + k) & 15) : -1;
}

__global__ void __launch_bounds__(64) k_core_bank_order(const int *__restrict__ blk_off, unsigned short *__restrict__ idx, int tc)  // tc <= 256
{
    __shared__ unsigned char srt[BANK_MAX_POS][64];    // [position][lane]: a lane's entries (tile offsets below 256) by residue, edge order inside one
    const int lane = (int)threadIdx.x, i = lane & 15;
    const unsigned b0 = (unsigned)blk_off[blockIdx.x], b1 = (unsigned)blk_off[blockIdx.x + 1];
    const int P = 4 * (int)(b1 - b0);
    if (P == 0) return;
    us4 *lists = reinterpret_cast<us4 *>(idx);
    if (P > BANK_MAX_POS) {  // more entries than columns (a CSR with repeated edges): edge order, padding on the first zero column
        for (unsigned c = b0; c < b1; ++c) {
            us4 e = lists[(size_t)c * 64 + lane];
#pragma unroll
            for (int j = 0; j < 4; ++j) e[j] = e[j] == 0xFFFF ? (unsigned short)tc : e[j];
            lists[(size_t)c * 64 + lane] = e;
        }
        return;
    }
    int cnt[16], head[16], tail[16];
#pragma unroll
    for (int g = 0; g < 16; ++g) cnt[g] = 0;
    int left = 0;
    for (unsigned c = b0; c < b1; ++c) {
        const us4 e = lists[(size_t)c * 64 + lane];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const unsigned short v = e[j];
            if (v != 0xFFFF) {
                ++left;
#pragma unroll
                for (int g = 0; g < 16; ++g) cnt[g] += (v & 15) == g;
            }
        }
    }
    unsigned have = 0;
    {
        int at = 0;
#pragma unroll
        for (int g = 0; g < 16; ++g) {
            head[g] = tail[g] = at;
            at += cnt[g];
            have |= cnt[g] ? 1u << g : 0u;
        }
    }
    for (unsigned c = b0; c < b1; ++c) {
        const us4 e = lists[(size_t)c * 64 + lane];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const unsigned short v = e[j];
            if (v != 0xFFFF) {
#pragma unroll
                for (int g = 0; g < 16; ++g)
                    if ((v & 15) == g) srt[tail[g]++][lane] = (unsigned char)v;
            }
        }
    }
    for (int p0 = 0; p0 < P; p0 += 4) {
        us4 e;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int p = p0 + j;
            const int slack = P - p - left;  // padding slots this lane has yet to place
            const int k0 = (i + p) & 15;
            unsigned used = 0;               // residues taken at this position, the same in all lanes of a group
            int r = -1;
            for (int pass = 0; pass < 2; ++pass) {
                const bool mine = left > 0 && (slack == 0) == (pass == 0);
                for (int t = 0; t < 16; ++t) {
                    int rr = -1;
                    if (mine && i == t) {
                        rr = first_from(have & ~used, k0);
                        if (rr < 0 && slack == 0) rr = first_from(have, k0);
                        r = rr;
                    }
                    used |= (unsigned)__shfl(rr >= 0 ? 1 << rr : 0, (lane & 48) | t);
                }
            }
            unsigned short v;
            const unsigned long long pads = __ballot(r < 0);
            if (r >= 0) {
                int h = 0;
#pragma unroll
                for (int g = 0; g < 16; ++g) {
                    h = r == g ? head[g] : h;
                    head[g] += r == g;
                    if (r == g && head[g] == tail[g]) have &= ~(1u << g);
                }
                v = srt[h][lane];
                --left;
            } else {
                const int k = __popc((unsigned)(pads >> (lane & 48)) & ((1u << i) - 1u));  // padding lanes of the group before this one
                unsigned f = ~used & 0xFFFFu;
                for (int t = 0; t < k && f; ++t) f &= f - 1;
                v = (unsigned short)(tc + (f ? __ffs((int)f) - 1 : (k & 15)));
            }
            e[j] = v;
        }
        lists[(size_t)(b0 + p0 / 4) * 64 + lane] = e;
    }
}

constexpr int BUILD_WAVES = 4;  // rows per workgroup of the two passes below (one wavefront each)

// Pass 1, one wavefront per row: how many neighbors of a core row fall into each tile of core columns (cnt, one
// 16-bit count per core row and tile), and how many neighbors every row keeps in the remaining CSR.  flag |= 1 on a
// neighbor id outside [lb, lb + rows) or a list longer than 65534.
__global__ void __launch_bounds__(BUILD_WAVES * 64) k_core_count(const int *__restrict__ ptr, const int *__restrict__ col,
                                                                 const int *__restrict__ rank, const int *__restrict__ sorted, int rows, int lb,
                                                                 int ntiles, int tc, unsigned short *__restrict__ cnt, int *__restrict__ keep,
                                                                 int *__restrict__ flag)
{
    extern __shared__ int hist_all[];  // [BUILD_WAVES][ntiles]
    const int lane = (int)(threadIdx.x & 63u), wave = (int)(threadIdx.x >> 6);
    int *hist = hist_all + (size_t)wave * ntiles;
    for (long long at = (long long)blockIdx.x * BUILD_WAVES + wave; at < rows; at += (long long)gridDim.x * BUILD_WAVES) {
        const int v = sorted[at];  // rows in rank order: the longest first
        const int i = rank[v];
        const int beg = ptr[v], end = ptr[v + 1];
        if (i >= 0)
            for (int t = lane; t < ntiles; t += 64) hist[t] = 0;
        int kept = 0, bad = 0;
        for (int e = beg + lane; e < end; e += 64) {
            const int u = col[e] - lb;
            if (u < 0 || u >= rows) {
                bad = 1;
                ++kept;
                continue;
            }
            const int j = rank[u];
            if (i >= 0 && j >= 0) atomicAdd(&hist[j / tc], 1);
            else ++kept;
        }
        for (int o = 32; o > 0; o >>= 1) kept += __shfl_xor(kept, o, 64);
        if (i >= 0) {
            for (int t = lane; t < ntiles; t += 64) {
                const int c = hist[t];
                if (c > 0xFFFE) bad = 1;
                cnt[(size_t)i * ntiles + t] = (unsigned short)(c > 0xFFFE ? 0xFFFE : c);
            }
        }
        if (lane == 0) keep[v] = kept;
        if (bad) *flag = 1;
    }
}

// chunks[g * ntiles + t] = list positions of block (slice g, tile t) in units of 4: the longest of the slice's 64 lists, rounded up
__global__ void __launch_bounds__(256) k_core_widths(const unsigned short *__restrict__ cnt, int nslices, int ntiles, int *__restrict__ chunks)
{
    const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (long long)nslices * ntiles) return;
    const int g = (int)(idx / ntiles), t = (int)(idx % ntiles);
    int w = 0;
    for (int l = 0; l < 64; ++l) w = max(w, (int)cnt[(size_t)(g * 64 + l) * ntiles + t]);
    chunks[idx] = (w + 3) / 4;
}

// work[g * ntiles + t] = list chunks of the `waves` slices of row group g in tile t
__global__ void __launch_bounds__(256) k_core_group_work(const int *__restrict__ chunks, int groups, int ntiles, int waves, int *__restrict__ work)
{
    const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (long long)groups * ntiles) return;
    const int g = (int)(idx / ntiles), t = (int)(idx % ntiles);
    int w = 0;
    for (int k = 0; k < waves; ++k) w += chunks[(size_t)(g * waves + k) * ntiles + t];
    work[idx] = w;
}

// Pass 2, one wavefront per row, 64 neighbors at a time in edge order: neighbors that stay go to the remaining CSR (order
// kept); a core row's core neighbors go to the list of their tile, the k-th of a tile (in edge order) to list position k.
// Inside a group of 64 every lane finds the lanes with the same tile by one ballot per bit of the tile number; the counts
// so far per tile and the row's block offsets sit in LDS, and the next group's ids and ranks are fetched ahead.
__global__ void __launch_bounds__(BUILD_WAVES * 64) k_core_fill(const int *__restrict__ ptr, const int *__restrict__ col,
                                                                const int *__restrict__ rank, const int *__restrict__ sorted, int rows, int lb,
                                                                int ntiles, int tc, const int *__restrict__ blk_off,
                                                                const int *__restrict__ rem_ptr, unsigned short *__restrict__ idx,
                                                                int *__restrict__ rem_col)
{
    extern __shared__ int fill_lds[];  // [BUILD_WAVES][2][ntiles]: entries already in each tile's list; the row's block offsets
    const int lane = (int)(threadIdx.x & 63u), wave = (int)(threadIdx.x >> 6);
    volatile int *cur = fill_lds + (size_t)wave * 2 * ntiles;
    volatile int *blk = cur + ntiles;
    const unsigned long long below = lane == 0 ? 0ull : (~0ull >> (64 - lane));
    int tile_bits = 0;
    while ((1 << tile_bits) < ntiles) ++tile_bits;
    // Rows in rank order: the 64 rows of a slice are then filled by neighbouring wavefronts at about the same time, and
    // their 8-byte pieces of the same 512-byte list chunks meet in the L2 instead of each going to memory as a partial
    // line; the longest rows also start first.
    for (long long at = (long long)blockIdx.x * BUILD_WAVES + wave; at < rows; at += (long long)gridDim.x * BUILD_WAVES) {
        const int v = sorted[at];
        const int i = rank[v];
        const int beg = ptr[v], end = ptr[v + 1];
        int w = rem_ptr[v];
        if (i < 0) {  // every neighbor stays
            for (int e = beg + lane; e < end; e += 64) rem_col[w + (e - beg)] = col[e];
            continue;
        }
        const size_t row_blocks = (size_t)(i / 64) * ntiles;
        for (int t = lane; t < ntiles; t += 64) {
            cur[t] = 0;
            blk[t] = blk_off[row_blocks + t];
        }
        const size_t lane_base = (size_t)(i % 64) * 4;
        // the next group's neighbor ids and their ranks are fetched while the current group is placed: a long row is one
        // wavefront's work from end to end, and without this every group would wait for two trips to memory
        int c_next = beg + lane < end ? col[beg + lane] : 0;
        int j_next = beg + lane < end ? rank[c_next - lb] : -1;
        for (int e0 = beg; e0 < end; e0 += 64) {
            const int e = e0 + lane;
            const bool valid = e < end;
            const int c = c_next, j = j_next;
            if (e0 + 64 < end) {
                const int en = e + 64;
                c_next = en < end ? col[en] : 0;
                j_next = en < end ? rank[c_next - lb] : -1;
            }
            const bool in_core = valid && j >= 0;
            const unsigned long long stay = __ballot(valid && !in_core);
            if (valid && !in_core) rem_col[w + __popcll(stay & below)] = c;
            w += __popcll(stay);
            if (!__any(in_core)) continue;
            // the lanes of this group with the same tile as this lane: one ballot per bit of the tile number
            const int t = in_core ? j / tc : 0;
            unsigned long long same = __ballot(in_core);
            for (int b = 0; b < tile_bits; ++b) {
                const bool bit = (t >> b) & 1;
                const unsigned long long m = __ballot(bit);
                same &= bit ? m : ~m;
            }
            if (in_core) {
                const int k = cur[t] + __popcll(same & below);
                const size_t chunk = (size_t)blk[t] + (size_t)(k / 4);
                idx[chunk * 256 + lane_base + (size_t)(k % 4)] = (unsigned short)(j % tc);
                if ((same & ~below & ~(1ull << lane)) == 0) cur[t] = k + 1;  // the last lane of its tile in this group
            }
        }
    }
}

// Rows of more than 192 bytes are summed in two halves by two workgroups (blockIdx.y): half the accumulators per lane
// (81 instead of 119 registers at 256 bytes), at the price of walking the index lists twice.  Their workgroups have 8
// wavefronts (see WAVES above) and ask for a third of the LDS, which holds a CU to two of them -- 16 wavefronts of this
// kernel -- and leaves the aggregation beside them the room it had (2.45 M-node graph, width 64, per aggregation:
// whole rows 3.01 ms; halves, 4 wavefronts, three workgroups per CU 2.92; halves, 8 wavefronts, two per CU 2.68, one per
// CU 3.05; at width 44 halves gain nothing: 1.42 against 1.40 ms).
template <int N4, int WAVES>
int launch_sell_as(const CorePlan *p, const CorePlan::Cut &cut, const v4f *tab, v4f *partial, const Gate &gate, hipStream_t stream)
{
    constexpr bool SPLIT = N4 > 12;
    constexpr int NS = SPLIT ? (N4 + 1) / 2 : N4;
    size_t lds = (size_t)NS * (CORE_TC + CORE_ZERO_COLS) * sizeof(v4f);
    if (SPLIT) lds = std::max<size_t>(lds, (160u << 10) / (WAVES == 8 ? 3 : 4) + 256);
    static bool raised = false;  // per instantiation
    if (lds > 48 * 1024 && !raised) {
        MGGX_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(k_core_sell<N4, SPLIT, WAVES>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        raised = true;
    }
    k_core_sell<N4, SPLIT, WAVES><<<dim3((unsigned)cut.nwg, SPLIT ? 2u : 1u), dim3(WAVES * 64), lds, stream>>>(p->d_blk_off, p->d_idx, tab, partial, cut.d_wgs,
                                                                                                            p->core, p->ntiles, gate);
    MGGX_LAUNCH_CHECK("k_core_sell");
    return MGGX_OK;
}
template <int N4>
int launch_sell(const CorePlan *p, const CorePlan::Cut &cut, const v4f *tab, v4f *partial, const Gate &gate, hipStream_t stream)
{
    if (p->group_rows == CORE_GROUP_ROWS) return launch_sell_as<N4, CORE_GROUP_ROWS / 64>(p, cut, tab, partial, gate, stream);
    if constexpr (N4 > 12)
        if (p->group_rows == CORE_GROUP_ROWS_WIDE) return launch_sell_as<N4, CORE_GROUP_ROWS_WIDE / 64>(p, cut, tab, partial, gate, stream);
    return fail(MGGX_EINVAL, "core: a plan with row groups of %d rows for rows of %d pieces", p->group_rows, N4);
}

// A plan that was used inside a stream capture: a captured graph still holds the addresses of its arrays, so they are
// retired (freed by mggx_release_cached) instead of freed.
void core_plan_free_arrays(CorePlan *p)
{
    const bool keep = p->pinned;
    size_t left = keep ? p->bytes : 0;  // the plan's bytes, accounted to the first retired block
    const auto drop = [&](void *q) {
        if (!q) return;
        if (keep) {
            retire_block(q, left);
            left = 0;
        } else {
            (void)hipFree(q);
        }
    };
    drop(p->d_order);
    drop(p->d_rank);
    drop(p->d_blk_off);
    drop(p->d_idx);
    drop(p->d_rem_ptr);
    drop(p->d_rem_col);
    for (CorePlan::Cut &c : p->cuts) {
        drop(c.d_wgs);
        drop(c.d_wg_base);
    }
    p->d_order = p->d_rank = p->d_rem_ptr = p->d_rem_col = nullptr;
    p->d_blk_off = nullptr;
    p->d_idx = nullptr;
    p->cuts.clear();
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

namespace {

struct Scratch {  // device temporaries of one plan build, freed on the way out
    std::vector<void *> ptrs;
    ~Scratch()
    {
        for (void *q : ptrs) (void)hipFree(q);
    }
    template <typename T>
    int get(T **q, size_t count)
    {
        void *r = nullptr;
        if (hipMalloc(&r, std::max<size_t>(count, 1) * sizeof(T)) != hipSuccess) return fail(MGGX_ENOMEM, "core plan: %zu bytes of scratch", count * sizeof(T));
        ptrs.push_back(r);
        *q = static_cast<T *>(r);
        return MGGX_OK;
    }
};

template <typename T>
int device_array(T **q, size_t count)
{
    if (hipMalloc((void **)q, std::max<size_t>(count, 1) * sizeof(T)) != hipSuccess) return fail(MGGX_ENOMEM, "core plan: %zu bytes of device memory", count * sizeof(T));
    return MGGX_OK;
}

}  // namespace

// The arrays of core_layout_build (mggx_internal.h), made on the GPU from the caller's device CSR: a stable radix sort
// by falling degree gives the ranking, one pass counts list lengths per (core row, tile), two prefix sums place the
// blocks and the remaining rows, a second pass fills lists and remaining CSR in edge order.  Only scalars come back to
// the host.  p->unsuitable is set where the host version refuses (no whole unit of rows, ids out of range).
static int core_plan_build_device(CorePlan *p, int tc)
{
    State &s = state();
    const int rows = p->rows, lb = p->lb;
    int core = std::min(p->asked, rows);
    const int unit = tc > 512 ? tc : 512;
    core = core / unit * unit;
    if (core < unit) {
        p->unsuitable = true;
        return MGGX_OK;
    }
    const int ntiles = core / tc, nslices = core / 64;
    if (ntiles > 2048) return fail(MGGX_ELIMIT, "core plan: %d core rows", core);
    Scratch tmp;
    int *deg = nullptr, *deg_sorted = nullptr, *ids = nullptr, *sorted = nullptr, *keep = nullptr, *chunks = nullptr, *flag = nullptr, *blk = nullptr, *work = nullptr;
    unsigned short *cnt = nullptr;
    int rc;
    if ((rc = tmp.get(&deg, (size_t)rows)) || (rc = tmp.get(&deg_sorted, (size_t)rows)) || (rc = tmp.get(&ids, (size_t)rows)) ||
        (rc = tmp.get(&sorted, (size_t)rows)) || (rc = tmp.get(&keep, (size_t)rows)) || (rc = tmp.get(&chunks, (size_t)nslices * ntiles)) ||
        (rc = tmp.get(&flag, 1)) || (rc = tmp.get(&cnt, (size_t)core * ntiles)) || (rc = tmp.get(&blk, (size_t)nslices * ntiles + 1)) ||
        (rc = tmp.get(&work, (size_t)(nslices / (p->group_rows / 64)) * ntiles)))
        return rc;
    if ((rc = device_array(&p->d_order, (size_t)core)) || (rc = device_array(&p->d_rank, (size_t)rows)) ||
        (rc = device_array(&p->d_blk_off, (size_t)nslices * ntiles + 1)) || (rc = device_array(&p->d_rem_ptr, (size_t)rows + 1)))
        return rc;
    MGGX_HIP(hipMemsetAsync(flag, 0, sizeof(int), s.stream));
    const unsigned row_blocks = (unsigned)((rows + 255) / 256);
    k_core_deg<<<row_blocks, 256, 0, s.stream>>>(p->d_ptr_l, rows, deg, ids);
    size_t need = 0;
    MGGX_HIP(rocprim::radix_sort_pairs_desc(nullptr, need, deg, deg_sorted, ids, sorted, (size_t)rows, 0, 32, s.stream));
    char *sort_tmp = nullptr;
    if ((rc = tmp.get(&sort_tmp, need))) return rc;
    MGGX_HIP(rocprim::radix_sort_pairs_desc(sort_tmp, need, deg, deg_sorted, ids, sorted, (size_t)rows, 0, 32, s.stream));
    k_core_rank<<<row_blocks, 256, 0, s.stream>>>(sorted, rows, core, p->d_order, p->d_rank);
    const unsigned wave_blocks = (unsigned)std::min<long long>(((long long)rows + BUILD_WAVES - 1) / BUILD_WAVES, 256 * 64);
    const size_t lds = (size_t)BUILD_WAVES * ntiles * sizeof(int);
    k_core_count<<<wave_blocks, BUILD_WAVES * 64, lds, s.stream>>>(p->d_ptr_l, p->d_col_l, p->d_rank, sorted, rows, lb, ntiles, tc, cnt, keep, flag);
    MGGX_LAUNCH_CHECK("k_core_count");
    long long rem_nnz = 0, total_chunks = 0;
    rc = exclusive_scan_i32(keep, p->d_rem_ptr, rows, &rem_nnz);
    if (rc) return rc;
    const long long nblk = (long long)nslices * ntiles;
    k_core_widths<<<(unsigned)((nblk + 255) / 256), 256, 0, s.stream>>>(cnt, nslices, ntiles, chunks);
    rc = exclusive_scan_i32(chunks, blk, (int)nblk, &total_chunks);
    if (rc) return rc;
    int bad = 0, nnz = 0;
    MGGX_HIP(hipMemcpyAsync(&bad, flag, sizeof(int), hipMemcpyDeviceToHost, s.stream));
    MGGX_HIP(hipMemcpyAsync(&nnz, p->d_ptr_l + rows, sizeof(int), hipMemcpyDeviceToHost, s.stream));
    MGGX_HIP(hipMemcpyAsync(p->d_blk_off, blk, sizeof(int) * ((size_t)nblk + 1), hipMemcpyDeviceToDevice, s.stream));
    MGGX_HIP(hipStreamSynchronize(s.stream));
    if (bad) {  // a neighbor id outside [lb, lb + rows), or more than 65534 parallel edges into one tile: not this path's input
        p->unsuitable = true;
        return MGGX_OK;
    }
    if (total_chunks > (long long)(0xFFFFFFFFull / 64)) return fail(MGGX_ELIMIT, "core plan: %lld list chunks", total_chunks);
    const size_t idx_elems = std::max<size_t>((size_t)total_chunks * 256, 256);
    if ((rc = device_array(&p->d_idx, idx_elems)) || (rc = device_array(&p->d_rem_col, (size_t)rem_nnz))) return rc;
    MGGX_HIP(hipMemsetAsync(p->d_idx, 0xFF, idx_elems * sizeof(unsigned short), s.stream));
    k_core_fill<<<wave_blocks, BUILD_WAVES * 64, 2 * lds, s.stream>>>(p->d_ptr_l, p->d_col_l, p->d_rank, sorted, rows, lb, ntiles, tc, blk, p->d_rem_ptr, p->d_idx,
                                                                  p->d_rem_col);
    MGGX_LAUNCH_CHECK("k_core_fill");
    {
        const long long cells = (long long)(core / 64) * ntiles;
        k_core_bank_order<<<(unsigned)cells, 64, 0, s.stream>>>(blk, p->d_idx, tc);
        MGGX_LAUNCH_CHECK("k_core_bank_order");
    }
    MGGX_HIP(hipStreamSynchronize(s.stream));
    p->core = core;
    p->ntiles = ntiles;
    p->rem_nnz = rem_nnz;
    p->core_nnz = (int64_t)nnz - rem_nnz;
    // What cutting the LDS kernel's work into workgroups needs later: one number per (row group, tile), reduced on the GPU
    // (64 KB for a core of 32,768 rows)
    const int groups = core / p->group_rows;
    k_core_group_work<<<(unsigned)(((long long)groups * ntiles + 255) / 256), 256, 0, s.stream>>>(chunks, groups, ntiles, p->group_rows / 64, work);
    MGGX_LAUNCH_CHECK("k_core_group_work");
    p->work.resize((size_t)groups * ntiles);
    MGGX_HIP(hipMemcpyAsync(p->work.data(), work, p->work.size() * sizeof(int), hipMemcpyDeviceToHost, s.stream));
    MGGX_HIP(hipStreamSynchronize(s.stream));
    p->total_chunks = total_chunks;
    p->bytes = ((size_t)core + 2 * (size_t)rows + 1 + (size_t)rem_nnz + (size_t)nblk + 1) * sizeof(int) + idx_elems * sizeof(unsigned short);
    return MGGX_OK;
}

int core_plan_get(const int *d_ptr_l, const int *d_col_l, int rows, int lb, int core, int group_rows, int graph_serial, CorePlan **out)
{
    State &s = state();
    for (size_t i = 0; i < s.cores.size(); ++i) {
        CorePlan *p = s.cores[i];
        // a plan belongs to the graph record it was built under (see drop_plans_of_record): it carries its own copy of that
        // graph's remaining CSR and index lists, and a later record of the same addresses may stand for another graph
        if (p->d_ptr_l == d_ptr_l && p->d_col_l == d_col_l && p->rows == rows && p->lb == lb && p->asked == core && p->group_rows == group_rows && p->graph_serial == graph_serial) {
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
    p->group_rows = group_rows;
    p->graph_serial = graph_serial;
    int rc = core_plan_build_device(p, CORE_TC);
    if (rc) {
        core_plan_free_arrays(p);
        delete p;
        return rc;
    }
    if (s.cores.size() >= 8)  // these plans are large (about 3 bytes per edge): keep the eight most recently used (the search compares
                              // up to six core sizes and must not rebuild one between its rounds), and any a captured graph holds
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

// The workgroups of the LDS kernel for rows of n4 16-byte pieces: every row group's tiles cut into runs of about
// total / target list chunks (a run ends where half of the next tile would overshoot that), so no workgroup runs much
// longer than the others -- row groups and tiles are both sorted by degree, and equal numbers of tiles would differ in
// work a hundredfold.  Narrow rows: about 3072 workgroups (short ones; the kernel's own tail matters most); wide rows:
// about 1280 (every workgroup costs 256 partial rows that the finishing kernel reads back).  Measured on the 233 K-node
// graph at widths 16 / 44 and the 2.45 M-node graph at width 64: 1024 / 1536 / 2048 / 3072 workgroups give
// 0.72 / 0.62 / 0.59 / 0.57, 1.41 / 1.42 / 1.43 / 1.53 and 3.02 / 2.98 / 3.01 / 3.03 ms per aggregation.
// Launch order: the first run of every row group, then the second of those that have one, ... -- neighbors in the
// launch, which share a CU, then read different rows' lists and mostly the same tiles.
static int core_cut(CorePlan *p, int n4, const CorePlan::Cut **out)
{
    const int want = n4 <= 6 ? 3072 : 1280;
    for (const CorePlan::Cut &c : p->cuts)
        if (c.target == want) {
            *out = &c;
            return MGGX_OK;
        }
    if (capturing()) return fail(MGGX_EINVAL, "core: first use of this core with rows of this width inside a stream capture; call once outside the capture first");
    const int groups = p->core / p->group_rows, ntiles = p->ntiles;
    const long long target = std::max<long long>((p->total_chunks + want - 1) / want, 1);
    std::vector<int4> runs;  // row-group-major: slot order
    std::vector<int> wg_base((size_t)groups + 1, 0);
    int longest = 0;
    for (int g = 0; g < groups; ++g) {
        long long acc = 0;
        int first = 0;
        for (int t = 0; t < ntiles; ++t) {
            const int w = p->work[(size_t)g * ntiles + t];
            if (t > first && acc + w / 2 > target) {
                runs.push_back(make_int4(g, first, t, (int)runs.size()));
                first = t;
                acc = 0;
            }
            acc += w;
        }
        runs.push_back(make_int4(g, first, ntiles, (int)runs.size()));
        wg_base[(size_t)g + 1] = (int)runs.size();
        longest = std::max(longest, wg_base[(size_t)g + 1] - wg_base[(size_t)g]);
    }
    std::vector<int4> launch;
    launch.reserve(runs.size());
    for (int k = 0; k < longest; ++k)
        for (int g = 0; g < groups; ++g)
            if (wg_base[(size_t)g] + k < wg_base[(size_t)g + 1]) launch.push_back(runs[(size_t)wg_base[(size_t)g] + k]);
    CorePlan::Cut c;
    c.target = want;
    c.nwg = (int)launch.size();
    int rc;
    if ((rc = device_array(&c.d_wgs, launch.size()))) return rc;
    if ((rc = device_array(&c.d_wg_base, wg_base.size()))) {
        (void)hipFree(c.d_wgs);
        return rc;
    }
    hipError_t e = hipMemcpy(c.d_wgs, launch.data(), launch.size() * sizeof(int4), hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMemcpy(c.d_wg_base, wg_base.data(), wg_base.size() * sizeof(int), hipMemcpyHostToDevice);
    if (e != hipSuccess) {  // a cut that is kept must be complete: later calls find it by its target alone
        (void)hipFree(c.d_wgs);
        (void)hipFree(c.d_wg_base);
        return fail(MGGX_EHIP, "core: uploading the workgroup table: %s", hipGetErrorString(e));
    }
    p->cuts.reserve(4);  // pointers into the vector are handed out: two targets exist
    p->cuts.push_back(c);
    p->bytes += launch.size() * sizeof(int4) + wg_base.size() * sizeof(int);
    *out = &p->cuts.back();
    return MGGX_OK;
}

// Scratch of the dense-core path: the staged core table, then one partial row per workgroup of the LDS kernel and row of its group.
static int core_scratch(CorePlan *p, int n4, v4f **tab, v4f **partial, const CorePlan::Cut **cut_out = nullptr)
{
    State &s = state();
    const CorePlan::Cut *cut = nullptr;
    const int rc_cut = core_cut(p, n4, &cut);
    if (rc_cut) return rc_cut;
    if (cut_out) *cut_out = cut;
    const size_t tab_bytes = (tab_stride(p->core) * n4 * sizeof(v4f) + 255) & ~(size_t)255;
    const size_t part_bytes = (size_t)cut->nwg * p->group_rows * n4 * sizeof(v4f);
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
    const int vec_in = ld_in % 4 == 0 && (reinterpret_cast<uintptr_t>(d_in) & 15u) == 0;
    k_core_stage<<<dim3((unsigned)((p->core + 255) / 256), (unsigned)n4), dim3(256), 0, stream>>>(tab, d_in, p->d_order, p->core, n4, dim, ld_in, vec_in, gate);
    MGGX_LAUNCH_CHECK("k_core_stage");
    return MGGX_OK;
}

// The core block's sums from the staged table into the library's partial rows, on `stream`.
int run_core_sums(CorePlan *p, int dim, const Gate &gate, hipStream_t stream)
{
    const int n4 = (dim + 3) / 4;
    if (n4 < 1 || n4 > 16) return fail(MGGX_ELIMIT, "core: dim %d outside 1..64", dim);
    v4f *tab = nullptr, *partial = nullptr;
    const CorePlan::Cut *cut = nullptr;
    int rc = core_scratch(p, n4, &tab, &partial, &cut);
    if (rc) return rc;
    switch (n4) {
#define MGGX_CASE(N) case N: rc = launch_sell<N>(p, *cut, tab, partial, gate, stream); break;
        MGGX_CASE(1) MGGX_CASE(2) MGGX_CASE(3) MGGX_CASE(4) MGGX_CASE(5) MGGX_CASE(6) MGGX_CASE(7) MGGX_CASE(8)
        MGGX_CASE(9) MGGX_CASE(10) MGGX_CASE(11) MGGX_CASE(12) MGGX_CASE(13) MGGX_CASE(14) MGGX_CASE(15) MGGX_CASE(16)
#undef MGGX_CASE
        default: rc = fail(MGGX_ELIMIT, "core: dim %d", dim);
    }
    if (rc) return rc;
    int g_shift = 0;
    while ((1 << g_shift) < n4) ++g_shift;
    const long long n = (long long)p->core << g_shift;
    k_core_reduce<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream>>>(tab, partial, cut->d_wg_base, p->core, n4,
                                                                                p->group_rows == CORE_GROUP_ROWS_WIDE ? 9 : 8, g_shift, gate);
    MGGX_LAUNCH_CHECK("k_core_reduce");
    return MGGX_OK;
}

// out += scale * (the core block's sum of the row, as k_core_reduce left it), then the ReLU and / or the row softmax if asked for, on `stream`.
int run_core_finish(CorePlan *p, float *d_out, int dim, long long ld_out, const float *d_row_scale, int relu, int softmax, const Gate &gate,
                    hipStream_t stream)
{
    const int n4 = (dim + 3) / 4;
    v4f *tab = nullptr, *partial = nullptr;
    const CorePlan::Cut *cut = nullptr;
    int rc = core_scratch(p, n4, &tab, &partial, &cut);  // sized by run_core_sums already: only hands the pointers out
    if (rc) return rc;
    const int all_rows = (relu || softmax) ? 1 : 0;
    int g_shift = 0;
    while ((1 << g_shift) < n4) ++g_shift;
    const long long n = (long long)(all_rows ? p->rows : p->core) << g_shift;
    const int vec_out = ld_out % 4 == 0 && (reinterpret_cast<uintptr_t>(d_out) & 15u) == 0;
    k_core_finish<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream>>>(d_out, tab, p->d_rank, p->d_order, d_row_scale, p->rows, dim, ld_out,
                                                                                p->core, g_shift, relu, softmax, all_rows, vec_out, gate);
    MGGX_LAUNCH_CHECK("k_core_finish");
    return MGGX_OK;
}

// Where k_core_reduce leaves the core's sums of the call in flight: [core][n4] pieces of 16 bytes, indexed by rank.
int core_row_sums(CorePlan *p, int dim, const float4 **sums)
{
    const int n4 = (dim + 3) / 4;
    v4f *tab = nullptr, *partial = nullptr;
    const int rc = core_scratch(p, n4, &tab, &partial);
    if (rc) return rc;
    *sums = reinterpret_cast<const float4 *>(tab);
    return MGGX_OK;
}

}  // namespace mggx

// ---------------------------------------------------------------------------
// Cost model: which core size pays.
//
// Rows are ranked by degree.  Under the configuration model an edge joins ranks i and j with probability
// d_i d_j / nnz, so the list of a row of rank i for the tile of columns [256 t, 256 t + 256) holds lambda = d_i D_t / nnz
// entries on average (D_t = degree sum of the tile's columns, at most 256), and the 64 lists of a slice are padded to
// the longest of them, rounded up to 4: E[4 ceil(max of 64 Poisson(lambda) / 4)], tabulated once.  That gives the
// useful and the padded entries of any core size from the degree histogram alone (within 3 % of the built plans on the
// benchmark graphs).  Growing the core by a band of 4096 rows pays while what the band takes off the gather kernel
// costs more there than it costs the LDS kernel:
//     useful entries x BETA x (1 + 64-byte sectors of a row) x F  >=  padded entries x ALPHA x ceil(dim/4) [x HALVES]
// (a gathered row: a fixed part plus one part per sector; a padded list entry: ceil(dim/4) 16-byte LDS reads; rows of more
// than 12 pieces are summed in two halves by two workgroups, which leaves the gather kernel beside them more room:
// HALVES).  F says where the gathers of what the core leaves are served from:
//     1                            that rest is still gathered in column-blocked order (it has the neighbors per row and
//                                  block that order asks for): the XCDs' L2s
//     h + (1 - h) x F_CACHE        row-major order, table within the 256 MB last-level cache; h = the share of the rest's
//     h + (1 - h) x F_MEMORY       gathers that go to its hottest 4 MB of rows (one XCD's L2) -- again from the degree
//                                  histogram: a column of rank j < K keeps d_j (1 - S_K) of its edges outside the core
//                                  (S_K = the core rows' share of all degrees), a column beyond the core all d_j
// Provenance of the constants: BETA 9 ps is the scale; ALPHA 1.40, HALVES 0.7, F_CACHE 3.0, F_MEMORY 4.0 put the rule
// into the flat bottom (within 2 %) of TWELVE measured core-size sweeps at once: the 233 K-node graph at widths 16 and
// 44 and the 2.45 M-node graph at width 64 (the benchmark graphs; the first version of this model -- one threshold, a
// factor of 3.2 beyond 256 MB -- was fitted on those three alone) and nine graphs from other RMAT settings (a from 0.45 to
// 0.65), sizes (0.3 - 2 M nodes), mean degrees (70 - 620) and widths (16 - 64), on which the first version and two
// intermediate ones were up to 29 % off; graphs and sweeps: dse.py --mode heldout.  The 4 MB are the size of an L2.
// HALVES_WIDE 0.62: rows in halves in row groups of 512 rows (core_group_rows) re-read the staged table half as often;
// 0.55 put the core of a 700 K-node graph of width 64 at 86,016 rows, 4 % slower than 81,920; with 0.62 the four graphs
// of that width are within 1.3 % of their sweeps' best.
// The model stops at 98,304 rows.
namespace mggx {
namespace {

constexpr int PROFILE_SLICES = 2048;  // 131072 ranks
constexpr double ALPHA_PS = 1.40, BETA_PS = 9.0, HALVES = 0.7, HALVES_WIDE = 0.62, F_CACHE = 3.0, F_MEMORY = 4.0;
constexpr unsigned long long L2_BYTES = 4ull << 20, LAST_LEVEL_CACHE_BYTES = 256ull << 20;
constexpr int MODEL_STEP = 4096, MODEL_MAX_CORE = 98304;

__global__ void __launch_bounds__(256) k_degrees(const int *__restrict__ ptr, int rows, int *__restrict__ deg)
{
    const int v = blockIdx.x * 256 + threadIdx.x;
    if (v < rows) deg[v] = ptr[v + 1] - ptr[v];
}

// slice_sum[s] = sum of sorted[64 s .. 64 s + 63] (sorted: falling degrees), one wavefront per slice
__global__ void __launch_bounds__(256) k_slice_sums(const int *__restrict__ sorted, int rows, int slices, float *__restrict__ slice_sum)
{
    const int s = blockIdx.x * 4 + (int)(threadIdx.x >> 6), lane = (int)(threadIdx.x & 63u);
    if (s >= slices) return;
    const int i = s * 64 + lane;
    float d = i < rows ? (float)sorted[i] : 0.f;
    for (int o = 32; o > 0; o >>= 1) d += __shfl_xor(d, o, 64);
    if (lane == 0) slice_sum[s] = d;
}

// E[4 ceil(max of 64 independent Poisson(lambda) / 4)] on a logarithmic grid of lambda
struct PaddingTable {
    static constexpr int N = 96;
    double lo = 1e-3, hi = 300.0, v[N];
    PaddingTable()
    {
        for (int i = 0; i < N; ++i) {
            const double lam = lo * std::pow(hi / lo, (double)i / (N - 1));
            // P(X <= m) by the recurrence of the Poisson terms; E = sum_j 4 (1 - F(4 j)^64)
            double term = std::exp(-lam), cdf = term, e = 0.0;
            int m = 0;
            for (int j = 0; j < 400; ++j) {
                while (m < 4 * j) {
                    ++m;
                    term *= lam / m;
                    cdf += term;
                }
                const double miss = 1.0 - std::pow(std::min(cdf, 1.0), 64.0);
                e += 4.0 * miss;
                if (miss < 1e-12 && 4 * j > lam) break;
            }
            v[i] = e;
        }
    }
    double operator()(double lam) const
    {
        if (lam <= lo) return 256.0 * lam;  // 4 P(some lane has an entry) ~ 4 x 64 lambda
        if (lam >= hi) return lam + 4.0 * std::sqrt(lam);
        const double x = std::log(lam / lo) / std::log(hi / lo) * (N - 1);
        const int i = std::min((int)x, N - 2);
        return v[i] + (v[i + 1] - v[i]) * (x - i);
    }
};

int fetch_degree_profile(GraphInfo &g)
{
    State &s = state();
    if (g.have_profile) return MGGX_OK;
    if (capturing()) return fail(MGGX_EINVAL, "cost model: first use of these CSR arrays inside a stream capture; call once outside the capture first");
    const int rows = g.rows;
    const int slices = std::min(PROFILE_SLICES, (rows + 63) / 64);
    Scratch tmp;
    int *deg = nullptr, *sorted = nullptr;
    float *d_sum = nullptr;
    char *sort_tmp = nullptr;
    int rc;
    if ((rc = tmp.get(&deg, (size_t)rows)) || (rc = tmp.get(&sorted, (size_t)rows)) || (rc = tmp.get(&d_sum, (size_t)slices))) return rc;
    k_degrees<<<(unsigned)((rows + 255) / 256), 256, 0, s.stream>>>(g.d_ptr_l, rows, deg);
    size_t need = 0;
    MGGX_HIP(rocprim::radix_sort_keys_desc(nullptr, need, deg, sorted, (size_t)rows, 0, 32, s.stream));
    if ((rc = tmp.get(&sort_tmp, need))) return rc;
    MGGX_HIP(rocprim::radix_sort_keys_desc(sort_tmp, need, deg, sorted, (size_t)rows, 0, 32, s.stream));
    k_slice_sums<<<(unsigned)((slices + 3) / 4), 256, 0, s.stream>>>(sorted, rows, slices, d_sum);
    MGGX_LAUNCH_CHECK("k_slice_sums");
    g.slice_deg.assign((size_t)slices, 0.f);
    MGGX_HIP(hipMemcpyAsync(g.slice_deg.data(), d_sum, sizeof(float) * (size_t)slices, hipMemcpyDeviceToHost, s.stream));
    MGGX_HIP(hipStreamSynchronize(s.stream));
    g.have_profile = true;
    return MGGX_OK;
}

}  // namespace

int predict_core_rows(GraphInfo &g, int dim, unsigned long long table_bytes, int block_rows, int min_per_row_block, int *core_rows)
{
    static const PaddingTable padded;
    *core_rows = -1;
    if (g.rows < 2 * MODEL_STEP || g.nnz_l <= 0) return MGGX_OK;
    for (const GraphInfo::Predicted &p : g.predicted)
        if (p.dim == dim && p.block_rows == block_rows && p.table_bytes == table_bytes) {
            *core_rows = p.core_rows;
            return MGGX_OK;
        }
    int rc = fetch_degree_profile(g);
    if (rc) return rc;
    const int n4 = (dim + 3) / 4;
    const int sectors = (dim * 4 + 63) / 64;
    // per padded list entry; rows in halves are cheaper beside the gather kernel, and cheaper again in wide row groups
    const auto entry_at = [&](int k) {
        return ALPHA_PS * n4 * (n4 > 12 ? (core_group_rows(n4, k) == CORE_GROUP_ROWS_WIDE ? HALVES_WIDE : HALVES) : 1.0);
    };
    const double nnz = (double)g.nnz_l;
    const int max_core = std::min({MODEL_MAX_CORE, g.rows / 2 / MODEL_STEP * MODEL_STEP, (int)g.slice_deg.size() * 64 / MODEL_STEP * MODEL_STEP});
    // useful and padded entries of the block (slices [s0, s1) x tiles [t0, t1))
    const auto block = [&](int s0, int s1, int t0, int t1, double *useful, double *pad) {
        for (int sl = s0; sl < s1; ++sl) {
            const double d = g.slice_deg[(size_t)sl] / 64.0;
            for (int t = t0; t < t1; ++t) {
                const double dt = (double)g.slice_deg[4 * (size_t)t] + g.slice_deg[4 * (size_t)t + 1] + g.slice_deg[4 * (size_t)t + 2] + g.slice_deg[4 * (size_t)t + 3];
                const double lam = std::min(d * dt / nnz, 256.0);
                *useful += 64.0 * lam;
                *pad += 64.0 * padded(lam);
            }
        }
    };
    // h: of the gathers a core of k rows leaves, the share that goes to the hottest L2_BYTES of table rows
    const double row_bytes = (double)table_bytes / (double)g.rows;
    const size_t hot_slices = (size_t)std::max(1.0, (double)L2_BYTES / row_bytes / 64.0);
    std::vector<double> w(g.slice_deg.size());
    const auto hot_share = [&](int k) {
        double core_deg = 0.0;
        for (int sl = 0; sl < k / 64; ++sl) core_deg += g.slice_deg[(size_t)sl];
        const double outside = 1.0 - core_deg / nnz;  // of a core column's edges, the share whose row is not in the core
        for (size_t sl = 0; sl < w.size(); ++sl) w[sl] = g.slice_deg[sl] * (sl < (size_t)(k / 64) ? outside : 1.0);
        const size_t take = std::min(hot_slices, w.size());
        std::partial_sort(w.begin(), w.begin() + (long)take, w.end(), std::greater<double>());
        double hot = 0.0;
        for (size_t i = 0; i < take; ++i) hot += w[i];
        const double left = nnz - core_deg * (core_deg / nnz);  // all edges but the core x core block
        return left > 0.0 ? std::min(1.0, hot / left) : 1.0;
    };
    const double far = table_bytes <= LAST_LEVEL_CACHE_BYTES ? F_CACHE : F_MEMORY;
    const double blocks = block_rows > 0 ? std::ceil((double)g.rows / block_rows) : 0.0;
    int best = 0;
    double taken = 0.0;
    for (int k = MODEL_STEP; k <= max_core; k += MODEL_STEP) {
        // the band the core grows by: new rows x all tiles, old rows x new tiles
        double useful = 0.0, pad = 0.0;
        block((k - MODEL_STEP) / 64, k / 64, 0, k / 256, &useful, &pad);
        block(0, (k - MODEL_STEP) / 64, (k - MODEL_STEP) / 256, k / 256, &useful, &pad);
        double f = 1.0;
        const bool rest_blocked = block_rows > 0 && nnz - taken - useful >= (double)min_per_row_block * blocks * (double)g.rows;
        if (!rest_blocked) {
            const double h = hot_share(k);
            f = h + (1.0 - h) * far;
        }
        if (pad <= 0.0 || useful * BETA_PS * (1 + sectors) * f < pad * entry_at(k)) break;
        best = k;
        taken += useful;
    }
    if (best >= 2 * MODEL_STEP) *core_rows = best;
    g.predicted.push_back({dim, block_rows, table_bytes, *core_rows});
    return MGGX_OK;
}

}  // namespace mggx

using mggx::fail;

MGGX_EXPORT int mggx_core_layout_device(const int *d_ptr, const int *d_col, int rows, int lb, int core_rows, int64_t *sizes, int *order,
                                        int *rank, unsigned *blk_off, unsigned short *idx, int *rem_ptr, int *rem_col)
{
    int rc = mggx::ensure_init();
    if (rc) return rc;
    if (!sizes) return fail(MGGX_EINVAL, "core_layout_device: NULL sizes");
    mggx::GraphInfo *g = nullptr;
    rc = mggx::graph_info(d_ptr, nullptr, d_col, nullptr, rows, false, &g);
    if (rc) return rc;
    mggx::CorePlan *p = nullptr;
    rc = mggx::core_plan_get(d_ptr, d_col, rows, lb, core_rows, mggx::CORE_GROUP_ROWS, g->serial, &p);
    if (rc) return rc;
    if (p->unsuitable) return fail(MGGX_EINVAL, "core layout: no core of whole 512-row units in %d rows, or a neighbor id outside [lb, lb + rows)", rows);
    const int64_t nblk = (int64_t)(p->core / 64) * p->ntiles + 1;
    unsigned chunks = 0;
    MGGX_HIP(hipMemcpy(&chunks, p->d_blk_off + (nblk - 1), sizeof(unsigned), hipMemcpyDeviceToHost));
    sizes[0] = p->core;
    sizes[1] = nblk;
    sizes[2] = (int64_t)chunks * 256;
    sizes[3] = p->rem_nnz;
    sizes[4] = p->core_nnz;
    if (order) MGGX_HIP(hipMemcpy(order, p->d_order, sizeof(int) * (size_t)p->core, hipMemcpyDeviceToHost));
    if (rank) MGGX_HIP(hipMemcpy(rank, p->d_rank, sizeof(int) * (size_t)rows, hipMemcpyDeviceToHost));
    if (blk_off) MGGX_HIP(hipMemcpy(blk_off, p->d_blk_off, sizeof(unsigned) * (size_t)nblk, hipMemcpyDeviceToHost));
    if (idx && chunks) MGGX_HIP(hipMemcpy(idx, p->d_idx, sizeof(unsigned short) * (size_t)chunks * 256, hipMemcpyDeviceToHost));
    if (rem_ptr) MGGX_HIP(hipMemcpy(rem_ptr, p->d_rem_ptr, sizeof(int) * ((size_t)rows + 1), hipMemcpyDeviceToHost));
    if (rem_col && p->rem_nnz) MGGX_HIP(hipMemcpy(rem_col, p->d_rem_col, sizeof(int) * (size_t)p->rem_nnz, hipMemcpyDeviceToHost));
    return MGGX_OK;
}
