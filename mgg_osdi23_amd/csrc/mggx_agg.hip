// Neighbor-partitioned aggregation (SpMM) for gfx950, wave64.
//
// Work decomposition
//   partition  <= ps neighbors of one destination row (MGG's neighbor partition)
//   slot       LPR adjacent lanes of a wavefront that together hold one feature
//              row (16 bytes per lane on the vector paths); a slot sums one
//              partition per round, so a wavefront sums S = 64/LPR partitions
//              at once and every gather instruction touches S feature rows
//   round      the S partitions a wavefront works on together; a wavefront
//              runs `dist` consecutive rounds (MGG's interleaved_dist)
//   workgroup  wpb wavefronts = wpb*S*dist consecutive partitions
// Partitions are laid out row-major (a row's local partitions, then its remote
// ones), so the partitions of one row are adjacent and every level combines
// neighbors only:
//   slots      segmented scan over the slots of a round (cross-lane moves)
//   rounds     a wavefront carries its open row from round to round in registers
//   wavefronts a row that crosses wavefronts is finished through LDS
//   workgroups a row that crosses workgroups leaves two partial rows in a
//              carry buffer; a small second kernel sums them in a fixed order
// No atomics anywhere; the summation order depends only on (ps, wpb, dist, dim).
// Index stream: a wavefront fetches the descriptors and the first ids of its next few rounds together into its own
// piece of LDS (two HBM latencies per four rounds instead of per round, with no feature row in flight meanwhile) and
// the rounds read them from there; the 16 lanes or so of a slot read the same words.
#include <algorithm>
#include <chrono>
#include <cstring>
#include <type_traits>

#include "mggx_dev.h"

// Device memory of mggx_sag_parts_static, the entry point that allocates nothing: the partition descriptors, the first
// descriptor of each row and the carry buffer of one call.  Every GPU the library runs on holds its own copy, at its
// own address, until the process ends; every call on a GPU shares that GPU's copy.  In host code this name is only a
// handle for hipGetSymbolAddress: static_scratch_ptr() below asks the runtime for the array's device address once per
// device, and that address is what kernels and host calls get.
static __device__ __align__(256) unsigned char scratch[MGGX_STATIC_SCRATCH_BYTES];

namespace mggx {
namespace {

#ifndef MGGX_BATCH
#define MGGX_BATCH 8
#endif
// Build-time experiment switches (both 0 in the library): a floor on the wavefronts per SIMD the compiler must leave room
// for in k_agg's register budget, and extra dynamic LDS per workgroup (limits how many workgroups a CU holds).
#ifndef MGGX_AGG_WAVES_PER_EU
#define MGGX_AGG_WAVES_PER_EU 0
#endif
#ifndef MGGX_AGG_LDS_PAD
#define MGGX_AGG_LDS_PAD 0
#endif
#if MGGX_AGG_WAVES_PER_EU > 0
#define MGGX_AGG_OCCUPANCY __attribute__((amdgpu_waves_per_eu(MGGX_AGG_WAVES_PER_EU)))
#elif defined(MGGX_AGG_NUM_VGPR)
#define MGGX_AGG_OCCUPANCY __attribute__((amdgpu_num_vgpr(MGGX_AGG_NUM_VGPR)))
#else
#define MGGX_AGG_OCCUPANCY
#endif

constexpr int HDR_VALID = 1;   // entry holds a partial row
constexpr int HDR_ENDS = 2;    // head entry: the row ends inside this unit
constexpr int HDR_STARTS = 4;  // tail entry: the row started inside this unit

constexpr int MODE_F32_VEC4 = 0;     // fp32 rows, one 16-byte load per lane
constexpr int MODE_F32_STRIDED = 1;  // fp32 rows of any width/alignment, dword loads, lane-strided
constexpr int MODE_BF16_VEC8 = 2;    // bf16 rows, one 16-byte load (8 values) per lane, fp32 accumulation

struct AggArgs {
    float *out;
    const void *in_l;
    const void *in_r;
    const int *col_l;
    const int *col_r;
    const int4 *desc;
    const int *off;
    const float *rs_out;
    Gate gate;      // closed = the plan is stale (the caller's CSR arrays changed): every kernel returns at once
    int2 *c_hdr;   // [2 * workgroups]: head, tail
    float *c_val;  // [2 * workgroups][cpad]
    long long ld_in, ld_out;
    int num_parts;
    const int *num_parts_dev; // when set: the descriptor count is read from here (it was made on the device and never copied back;
                              // num_parts is then a host-side upper bound that sizes the grid)
    int nnz_l, nnz_r;
    const int *nnz_l_dev;     // when set: the local edge count is read from here (a caller that may not copy it to the host)
    int lb, dim, ps, dist, cpad;
    int parts_per_wg;
    int ppw_shift;            // log2(parts_per_wg) where that is a power of two (every setting of the rules), else -1
    int stage_off;            // dynamic LDS, in floats: where the wavefronts' staged descriptors and ids start
    int stage_rounds;         // rounds staged at a time (1 .. the kernel's STAGE)
    unsigned flags;
    float eps;
    int in_is_bf16;
    // gather addressing
    unsigned ld_bytes;        // row stride of the feature tables in bytes
    const void *win_base;     // buffer-load path: one window over both tables ...
    unsigned win_bytes;       // ... of this many bytes,
    unsigned delta_l, delta_r;// ... the tables starting at these byte offsets;
    int sentinel;             // ... and a row index whose offset falls outside the window (reads as zero)
};

// Which workgroup descriptor q belongs to.  (An integer division by a run-time value costs some forty instructions; the
// kernels that finish rows ask this several times per row.)
__device__ __forceinline__ int wg_of_part(const AggArgs &a, int q) { return a.ppw_shift >= 0 ? q >> a.ppw_shift : q / a.parts_per_wg; }

// What padding neighbors read on the 64-bit address path: 4 KiB of zeros.
static __device__ __align__(256) float g_zero_row[1024];

template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F &&f)
{
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

__device__ __forceinline__ int lane_id() { return (int)(threadIdx.x & 63u); }

// value of lane `src` (any lane of the wavefront)
__device__ __forceinline__ int lane_read(int v, int src) { return __builtin_amdgcn_ds_bpermute(src << 2, v); }
__device__ __forceinline__ float lane_read(float v, int src)
{
    return __int_as_float(__builtin_amdgcn_ds_bpermute(src << 2, __float_as_int(v)));
}

// Rows of 16 lanes swapped between two registers without a trip through the LDS crossbar (gfx950):
// rows_from_even(v) = {v.row0, v.row0, v.row2, v.row2}, rows_from_odd(v) = {v.row1, v.row1, v.row3, v.row3},
// low_half(v) = {v.row0, v.row1, v.row0, v.row1}, high_half(v) = {v.row2, v.row3, v.row2, v.row3}.
__device__ __forceinline__ int rows_from_even(int v) { return (int)__builtin_amdgcn_permlane16_swap((unsigned)v, (unsigned)v, false, false)[0]; }
__device__ __forceinline__ int rows_from_odd(int v) { return (int)__builtin_amdgcn_permlane16_swap((unsigned)v, (unsigned)v, false, false)[1]; }
__device__ __forceinline__ int low_half(int v) { return (int)__builtin_amdgcn_permlane32_swap((unsigned)v, (unsigned)v, false, false)[0]; }
__device__ __forceinline__ int high_half(int v) { return (int)__builtin_amdgcn_permlane32_swap((unsigned)v, (unsigned)v, false, false)[1]; }
__device__ __forceinline__ float rows_from_even(float v) { return __int_as_float(rows_from_even(__float_as_int(v))); }
__device__ __forceinline__ float rows_from_odd(float v) { return __int_as_float(rows_from_odd(__float_as_int(v))); }
__device__ __forceinline__ float low_half(float v) { return __int_as_float(low_half(__float_as_int(v))); }
__device__ __forceinline__ float high_half(float v) { return __int_as_float(high_half(__float_as_int(v))); }

// Moves inside a row of 16 lanes with DPP (no LDS crossbar): CTRL = 0x110 + n: lane i takes lane i - n of its row (row_shr:n),
// 0x120 + n: lane (i - n) mod 16 (row_ror:n); BANKS: which groups of four lanes of every row take the value (the others,
// and lanes whose source falls outside the row, keep `keep`).
template <int CTRL, int BANKS>
__device__ __forceinline__ int row_move(int keep, int v) { return __builtin_amdgcn_update_dpp(keep, v, CTRL, 0xF, BANKS, false); }
// every lane gets the value of the same lane position in the LAST 4-lane slot of its 16-lane row
__device__ __forceinline__ int last_quad_of_row(int v)
{
    int b = row_move<0x124, 0x1>(v, v);  // lanes 0-3 <- 12-15
    b = row_move<0x128, 0x2>(b, v);      // lanes 4-7 <- 12-15
    return row_move<0x12C, 0x4>(b, v);   // lanes 8-11 <- 12-15
}
// The value of the slot a lane's 4-lane slot combines with at level J of the slot scan below (valid where the slot takes
// one): the last slot of the lower half of its group of 2^(J+1) slots.
template <int LPR, int J>
__device__ __forceinline__ int scan_source(int v)
{
    static_assert(LPR == 4, "slots of 4 lanes");
    if constexpr (J == 0) return row_move<0x114, 0xF>(v, v);                                 // slots 1, 3 <- slots 0, 2
    else if constexpr (J == 1) return row_move<0x118, 0x8>(row_move<0x114, 0x4>(v, v), v);   // slots 2, 3 <- slot 1
    else if constexpr (J == 2) return rows_from_even(last_quad_of_row(v));                   // rows 1, 3 <- the last slot of rows 0, 2
    else return low_half(rows_from_odd(last_quad_of_row(v)));                                // rows 2, 3 <- the last slot of row 1
}
template <int LPR, int J>
__device__ __forceinline__ float scan_source(float v) { return __int_as_float(scan_source<LPR, J>(__float_as_int(v))); }
// every lane gets the value of the same lane position in the last slot of the wavefront (slots of 4, 16 or 32 lanes)
template <int LPR>
__device__ __forceinline__ int last_slot(int v)
{
    if constexpr (LPR == 32) return high_half(v);
    else if constexpr (LPR == 16) return high_half(rows_from_odd(v));
    else return high_half(rows_from_odd(last_quad_of_row(v)));
}
template <int LPR>
__device__ __forceinline__ float last_slot(float v) { return __int_as_float(last_slot<LPR>(__float_as_int(v))); }

template <int MODE>
struct ModeTraits {
    static constexpr int NV = MODE == MODE_BF16_VEC8 ? 8 : 4;
};

// feature index of value i held by lane l of a slot
template <int LPR, int MODE>
__device__ __forceinline__ int elem_of(int l, int i)
{
    if constexpr (MODE == MODE_F32_STRIDED) return l + i * LPR;
    else return ModeTraits<MODE>::NV * l + i;
}

typedef unsigned v4u __attribute__((ext_vector_type(4)));

template <int MODE>
__device__ __forceinline__ void unpack16(float (&v)[ModeTraits<MODE>::NV], const v4u t)
{
    if constexpr (MODE == MODE_BF16_VEC8) {
        v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xFFFF0000u);
        v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xFFFF0000u);
        v[4] = __uint_as_float(t.z << 16); v[5] = __uint_as_float(t.z & 0xFFFF0000u);
        v[6] = __uint_as_float(t.w << 16); v[7] = __uint_as_float(t.w & 0xFFFF0000u);
    } else {
        v[0] = __uint_as_float(t.x); v[1] = __uint_as_float(t.y); v[2] = __uint_as_float(t.z); v[3] = __uint_as_float(t.w);
    }
}

// Per-slot addressing state of one round.  `cofs` is this lane's byte offset inside a row (lanes past the row width
// use lane 0's offset: they load valid memory and their values are dropped).
//   buffer path: offset = (row & 0xFFFFFF) * ld_bytes + cbase inside one window holding both tables; a padding
//                neighbor carries the sentinel row, whose offset lies past the window, and reads as zero
//   64-bit path: address = base + row * ld_bytes; a padding neighbor (row < 0) reads the zero row
template <int LPR, int MODE, bool BUF>
struct Gather {
    static constexpr int NV = ModeTraits<MODE>::NV;
    __amdgpu_buffer_rsrc_t rsrc;
    unsigned ld24;
    unsigned cbase;        // buffer path: table offset in the window + cofs
    const char *base;      // 64-bit path: table + cofs
    const char *zero;      // 64-bit path: zero row + cofs
    unsigned ld_bytes;
    unsigned sofs[4];      // strided mode: byte offsets of this lane's 4 elements inside a row

    // The 16 bytes this lane holds of one row, as loaded (unpacked only when summed, so a batch in flight costs four
    // registers per row whatever the element type).
    __device__ __forceinline__ v4u load(int row) const
    {
        if constexpr (BUF) {
            const unsigned off = ((unsigned)row & 0xFFFFFFu) * ld24 + cbase;
            if constexpr (MODE == MODE_F32_STRIDED) {
                v4u t;
                t.x = __builtin_amdgcn_raw_buffer_load_b32(rsrc, off + sofs[0], 0, 0);
                t.y = __builtin_amdgcn_raw_buffer_load_b32(rsrc, off + sofs[1], 0, 0);
                t.z = __builtin_amdgcn_raw_buffer_load_b32(rsrc, off + sofs[2], 0, 0);
                t.w = __builtin_amdgcn_raw_buffer_load_b32(rsrc, off + sofs[3], 0, 0);
                return t;
            } else {
                return __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, 0, 0);
            }
        } else {
            const char *p = row >= 0 ? base + (unsigned long long)(unsigned)row * ld_bytes : zero;
            if constexpr (MODE == MODE_F32_STRIDED) {
                v4u t;
                t.x = *reinterpret_cast<const unsigned *>(p + sofs[0]);
                t.y = *reinterpret_cast<const unsigned *>(p + sofs[1]);
                t.z = *reinterpret_cast<const unsigned *>(p + sofs[2]);
                t.w = *reinterpret_cast<const unsigned *>(p + sofs[3]);
                return t;
            } else {
                return *reinterpret_cast<const v4u *>(p);
            }
        }
    }
};

__device__ __forceinline__ float load_self(const AggArgs &a, int row, int d)
{
    if (a.in_is_bf16) {
        const unsigned short h = static_cast<const unsigned short *>(a.in_l)[(long long)row * a.ld_in + d];
        return __uint_as_float((unsigned)h << 16);
    }
    return static_cast<const float *>(a.in_l)[(long long)row * a.ld_in + d];
}

// One finished output element before the store: scale, GIN self term, accumulate, ReLU.
__device__ __forceinline__ float epilogue_value(const AggArgs &a, int row, int d, float sum)
{
    float v = a.rs_out ? sum * a.rs_out[row] : sum;
    if (a.flags & MGGX_AGG_GIN) v += (1.0f + a.eps) * load_self(a, row, d);
    if (a.flags & MGGX_AGG_ACCUMULATE) v += a.out[(long long)row * a.ld_out + d];
    if (a.flags & MGGX_AGG_RELU) v = fmaxf(v, 0.0f);
    return v;
}

__device__ __forceinline__ void finish_elem(const AggArgs &a, int row, int d, float sum)
{
    a.out[(long long)row * a.ld_out + d] = epilogue_value(a, row, d, sum);
}

// Row softmax over values spread across a group of G adjacent lanes (G a power of two, the group aligned to G), NPL values
// per lane, `on[i]` false for slots past the row width: v[i] <- exp(v[i] - max) / sum.  Every lane of the group must be
// active.  The epilogue of the last layer (MGGX_AGG_SOFTMAX), so that the logits never make a round trip through memory.
template <int NPL>
__device__ __forceinline__ void group_softmax(float (&v)[NPL], const bool (&on)[NPL], int G)
{
    const int lane = lane_id();
    float m = -3.0e38f;
#pragma unroll
    for (int i = 0; i < NPL; ++i) m = on[i] ? fmaxf(m, v[i]) : m;
    for (int o = 1; o < G; o <<= 1) m = fmaxf(m, lane_read(m, lane ^ o));
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < NPL; ++i) {
        v[i] = on[i] ? __expf(v[i] - m) : 0.f;
        sum += v[i];
    }
    for (int o = 1; o < G; o <<= 1) sum += lane_read(sum, lane ^ o);
    const float inv = 1.0f / sum;
#pragma unroll
    for (int i = 0; i < NPL; ++i) v[i] *= inv;
}

// Output rows are written once and not read again by the aggregation: stored with the streaming hint.
__device__ __forceinline__ void store_row16(float *p, float x, float y, float z, float w)
{
    typedef float v4f_s __attribute__((ext_vector_type(4)));
    __builtin_nontemporal_store((v4f_s){x, y, z, w}, reinterpret_cast<v4f_s *>(p));
}

// Finishes this lane's NV elements of a complete row held in registers.  SMX: the kernel variant that serves calls with
// the softmax epilogue (a variant of its own: inlined into every kernel, the few registers of this branch cost the wide-row
// kernels a wavefront of occupancy per SIMD on every call).
template <int LPR, int MODE, bool SMX>
__device__ __forceinline__ void finish_row(const AggArgs &a, int row, int l, const float (&acc)[ModeTraits<MODE>::NV])
{
    constexpr int NV = ModeTraits<MODE>::NV;
    if constexpr (SMX) {  // the slot's LPR lanes hold the whole row: softmax across them, then the store
        float v[NV];
        bool on[NV];
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int d = elem_of<LPR, MODE>(l, i);
            on[i] = d < a.dim;
            v[i] = on[i] ? epilogue_value(a, row, d, acc[i]) : 0.f;
        }
        group_softmax<NV>(v, on, LPR);
#pragma unroll
        for (int i = 0; i < NV; ++i)
            if (on[i]) a.out[(long long)row * a.ld_out + elem_of<LPR, MODE>(l, i)] = v[i];
        return;
    }
    if constexpr (MODE == MODE_F32_VEC4) {
        if (a.flags == 0 && a.rs_out == nullptr) {
            if (NV * l + 3 < a.dim) {
                store_row16(a.out + (long long)row * a.ld_out + 4 * l, acc[0], acc[1], acc[2], acc[3]);
            } else if (NV * l < a.dim) {  // the last, partial piece of a row whose width is not a multiple of 4
                float *o = a.out + (long long)row * a.ld_out + 4 * l;
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (4 * l + i < a.dim) o[i] = acc[i];
            }
            return;
        }
    }
    if constexpr (MODE == MODE_BF16_VEC8) {
        if (a.flags == 0 && a.rs_out == nullptr) {
            if (NV * l < a.dim) {
                float *o = a.out + (long long)row * a.ld_out + 8 * l;
                store_row16(o, acc[0], acc[1], acc[2], acc[3]);
                store_row16(o + 4, acc[4], acc[5], acc[6], acc[7]);
            }
            return;
        }
    }
    if constexpr (MODE == MODE_F32_VEC4) {
        // the same epilogue as finish_elem on this lane's four contiguous elements, with vector loads and one store
        if (NV * l < a.dim) {
            const float sc = a.rs_out ? a.rs_out[row] : 1.0f;
            float4 v = make_float4(acc[0] * sc, acc[1] * sc, acc[2] * sc, acc[3] * sc);
            if (a.flags & MGGX_AGG_GIN) {
                const float4 s = *reinterpret_cast<const float4 *>(static_cast<const float *>(a.in_l) + (long long)row * a.ld_in + 4 * l);
                const float k = 1.0f + a.eps;
                v.x += k * s.x; v.y += k * s.y; v.z += k * s.z; v.w += k * s.w;
            }
            float4 *o = reinterpret_cast<float4 *>(a.out + (long long)row * a.ld_out + 4 * l);
            if (a.flags & MGGX_AGG_ACCUMULATE) {
                const float4 p = *o;
                v.x += p.x; v.y += p.y; v.z += p.z; v.w += p.w;
            }
            if (a.flags & MGGX_AGG_RELU) {
                v.x = fmaxf(v.x, 0.f); v.y = fmaxf(v.y, 0.f); v.z = fmaxf(v.z, 0.f); v.w = fmaxf(v.w, 0.f);
            }
            if (NV * l + 3 < a.dim) {
                store_row16(reinterpret_cast<float *>(o), v.x, v.y, v.z, v.w);
            } else {
                const float t[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (4 * l + i < a.dim) reinterpret_cast<float *>(o)[i] = t[i];
            }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int d = elem_of<LPR, MODE>(l, i);
        if (d < a.dim) finish_elem(a, row, d, acc[i]);
    }
}

// One wavefront-wide aggregation kernel; see the file header for the scheme.
// Dynamic LDS: int2 hdr[2*wpb] (head, tail per wavefront), then float vals[2*wpb][cpad].
template <int LPR, int MODE, bool BUF, bool SMX>
__global__ void __launch_bounds__(1024) MGGX_AGG_OCCUPANCY k_agg(const AggArgs a)
{
    constexpr int NV = ModeTraits<MODE>::NV;
    constexpr int S = 64 / LPR;
    constexpr int CH = LPR > 16 ? LPR : 16;  // neighbor ids fetched per slot per chunk
    constexpr int IPL = CH / LPR;            // ids fetched per lane
    constexpr int CHP = CH + 4;              // words between the staged ids of neighbouring slots: 16 slots' 16-byte reads of
                                             // the same position then fall into 16 different bank groups
    constexpr int BATCH = MGGX_BATCH;        // gathers issued back to back
    static_assert(CH % BATCH == 0, "the gathers of a chunk of ids are issued in whole batches");
    // With 16 slots a wavefront reads its ids 1 KiB at a time and its descriptors 256 B at a time -- whole cache lines
    // that nobody reads again: those loads carry the streaming hint, which leaves the caches to the feature rows
    // (-5 % at width 16).  With fewer slots adjacent wavefronts share those lines and the hint costs 1-3 %.
    constexpr bool STREAM = S >= 16;
    // rounds whose descriptors and first ids a wavefront fetches at once (1.3 - 5 KiB of LDS per wavefront; measured on
    // the benchmark graphs: 4 rounds are as good as 8, 1 round is 5 - 10 % slower where the feature table is cache resident)
    constexpr int STAGE = LPR >= 4 ? 4 : LPR == 2 ? 2 : 1;
    // Slots of 4, 16 and 32 lanes combine and carry their sums with DPP row moves and the row- / half-swap instructions
    // instead of ds_bpermute.  Slots of 8 lanes keep ds_bpermute: their DPP form (written and measured) is 2 % faster to
    // 11 % slower beside the LDS kernel (233 K-node graph at width 24 / 32: 0.80 -> 0.78 / 0.91 -> 0.97 ms, 2.45 M-node graph
    // at width 32: 1.59 -> 1.77 ms) and the same without it.
    constexpr bool OFF_CROSSBAR = LPR == 4 || LPR == 16 || LPR == 32;
    extern __shared__ __align__(16) float lds[];
    if (gate_closed(a.gate)) return;
    const int num_parts = a.num_parts_dev ? *a.num_parts_dev : a.num_parts;

    const int lane = lane_id();
    const int wave = (int)(threadIdx.x >> 6);
    const int wpb = (int)(blockDim.x >> 6);
    const int slot = lane / LPR;
    const int l = lane % LPR;
    const int slot_base = slot * LPR;

    int2 *hdr = reinterpret_cast<int2 *>(lds);
    float *vals = lds + 4 * wpb;
    if (lane == 0) {
        hdr[2 * wave] = make_int2(-1, 0);
        hdr[2 * wave + 1] = make_int2(-1, 0);
    }

    const long long q_wave = ((long long)blockIdx.x * wpb + wave) * ((long long)S * a.dist);

    // this lane's place inside a feature row
    Gather<LPR, MODE, BUF> g;
    g.ld_bytes = a.ld_bytes;
    g.ld24 = a.ld_bytes & 0xFFFFFFu;
    unsigned cofs;
    if constexpr (MODE == MODE_F32_STRIDED) {
        cofs = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int dd = l + i * LPR;
            g.sofs[i] = 4u * (unsigned)(dd < a.dim ? dd : 0);
        }
    } else {
        cofs = 16u * (unsigned)(NV * l < a.dim ? l : 0);
    }
    if constexpr (BUF) g.rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(a.win_base), 0, a.win_bytes, 0x00020000);
    g.zero = reinterpret_cast<const char *>(g_zero_row) + cofs;
    const int pad_id = BUF ? a.sentinel : -1;  // what a slot holds past the end of its partition
    const bool lane_on = MODE == MODE_F32_STRIDED ? l < a.dim : NV * l < a.dim;

    float acc[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) acc[i] = 0.0f;
    int has_first = 0;    // the open run includes its row's first partition
    bool c_open = false;  // wavefront-uniform: slot S-1 holds a row that continues in the next round

    // A slot's descriptor, or an empty one (no row, no neighbors) past the end of the plan or of this wavefront's rounds.
    auto load_desc = [&](long long q, bool in_range) -> int4 {
        int4 d = make_int4(0, -1, 0, 0);
        if (in_range && q < num_parts) {
            if constexpr (STREAM) {
                typedef int v4i_a __attribute__((ext_vector_type(4)));
                const v4i_a dv = __builtin_nontemporal_load(reinterpret_cast<const v4i_a *>(a.desc + q));
                d = make_int4(dv.x, dv.y, dv.z, dv.w);
            } else {
                d = a.desc[q];
            }
        }
        return d;
    };
    // This lane's IPL neighbor ids of the chunk starting at neighbor k0 of the partition d describes, in two steps so that
    // the loads of several partitions can be in flight together: issue_ids only loads (no branch around a load: a lane
    // with nothing to fetch reads a word of the descriptor array instead, so no wait lands between two loads), and
    // finish_ids turns what arrived into row indices of the partition's table (pad_id past the end of the partition).
    const int *const dummy = reinterpret_cast<const int *>(a.desc);
    auto issue_ids = [&](const int4 &d, int k0, int (&raw)[IPL]) {
        const int len = (int)((unsigned)d.z & DESC_LEN_MASK);
        const bool remote = d.x < 0;
        const long long start = (long long)((unsigned)d.x & 0x7FFFFFFFu);
        const int *col = remote ? a.col_r : a.col_l;
        const int kk = k0 + l * IPL;
        const long long e0 = start + kk;
        if constexpr (IPL == 4) {
            const int nnz_side = remote ? a.nnz_r : (a.nnz_l_dev ? *a.nnz_l_dev : a.nnz_l);
            const bool whole = kk < len && e0 + 4 <= nnz_side;  // the 16 bytes lie inside the array
            typedef int v4i_u __attribute__((ext_vector_type(4), aligned(4)));
            const v4i_u tv = __builtin_nontemporal_load(reinterpret_cast<const v4i_u *>(whole ? col + e0 : dummy));
            raw[0] = tv.x; raw[1] = tv.y; raw[2] = tv.z; raw[3] = tv.w;
            if (__any(kk < len && !whole)) {  // the last few ids of the array: one by one
#pragma unroll
                for (int t = 0; t < IPL; ++t)
                    if (kk < len && !whole && kk + t < len) raw[t] = col[e0 + t];
            }
        } else {
#pragma unroll
            for (int t = 0; t < IPL; ++t) raw[t] = *(kk + t < len ? col + e0 + t : dummy);
        }
    };
    auto finish_ids = [&](const int4 &d, int k0, const int (&raw)[IPL], int (&ids)[IPL]) {
        const int len = (int)((unsigned)d.z & DESC_LEN_MASK);
        const int idbase = d.x < 0 ? 0 : a.lb;
        const int kk = k0 + l * IPL;
#pragma unroll
        for (int t = 0; t < IPL; ++t) ids[t] = (kk + t < len) ? raw[t] - idbase : pad_id;
    };
    // One window of gathers of a chunk of CH neighbors: get_rid4(q) gives neighbors 4 q .. 4 q + 3's rows in the slot's table.
    static_assert(BATCH % 4 == 0, "ids are read four at a time");
    auto gather_chunk = [&](int len, int k0, auto get_rid4) {
        static_for<0, CH / BATCH>([&](auto bb) {
            constexpr int b = decltype(bb)::value;
            if (__any(len > k0 + b * BATCH)) {
                int rid[BATCH];
                static_for<0, BATCH / 4>([&](auto qq) {  // four ids per 16-byte read
                    constexpr int q4 = decltype(qq)::value;
                    const int4 r4 = get_rid4(std::integral_constant<int, b * BATCH / 4 + q4>{});
                    rid[4 * q4] = r4.x; rid[4 * q4 + 1] = r4.y; rid[4 * q4 + 2] = r4.z; rid[4 * q4 + 3] = r4.w;
                });
                // lanes past the row width neither load nor sum (their sums stay zero and are never stored): a quad
                // of idle lanes costs the address unit nothing, and no register of the batch needs clearing
                if (lane_on) {
                    v4u raw[BATCH];
                    static_for<0, BATCH>([&](auto tt) {
                        constexpr int t = decltype(tt)::value;
                        raw[t] = g.load(rid[t]);
                    });
                    // keep every load of the batch in flight before the first sum waits on one
                    __builtin_amdgcn_sched_barrier(0);
                    static_for<0, BATCH>([&](auto tt) {
                        constexpr int t = decltype(tt)::value;
                        float v[NV];
                        unpack16<MODE>(v, raw[t]);
#pragma unroll
                        for (int i = 0; i < NV; ++i) acc[i] += v[i];
                    });
                }
            }
        });
    };

    // The index stream comes from HBM, the feature rows (where the kernel is at its fastest) from the caches.  A
    // wavefront that fetched descriptor, then ids, then rows in every round would wait out two HBM latencies per
    // round with no row in flight.  Instead it fetches the descriptors and the first CH ids of each partition for
    // STAGE rounds at a time -- all descriptor loads in flight together, then all id loads -- into its own piece of
    // LDS, and the rounds read them from there (every lane of a slot reads the same words).
    const int nst = a.stage_rounds < STAGE ? a.stage_rounds : STAGE;
    float *const stage = static_cast<float *>(__builtin_assume_aligned(lds + a.stage_off, 16));  // stage_off is a multiple of 4
    int4 *st_desc = reinterpret_cast<int4 *>(stage) + (size_t)wave * (nst * S);
    int *st_ids = reinterpret_cast<int *>(stage) + (size_t)wpb * (nst * S * 4) + (size_t)wave * (nst * S * CHP);

    for (int j0 = 0; j0 < a.dist; j0 += nst) {
        if (q_wave + (long long)j0 * S >= num_parts) break;
        {
            int4 dd[STAGE];
            int idv[STAGE][IPL];
#pragma unroll
            for (int u = 0; u < STAGE; ++u) dd[u] = load_desc(q_wave + (long long)(j0 + u) * S + slot, u < nst && j0 + u < a.dist);
#pragma unroll
            for (int u = 0; u < STAGE; ++u) {
                issue_ids(dd[u], 0, idv[u]);
                if (u < nst && l == 0) st_desc[u * S + slot] = dd[u];
            }
#pragma unroll
            for (int u = 0; u < STAGE; ++u) {
                int ids[IPL];
                finish_ids(dd[u], 0, idv[u], ids);
                if (u < nst) {
                    int *dst = st_ids + (u * S + slot) * CHP + l * IPL;
#pragma unroll
                    for (int t = 0; t < IPL; ++t) dst[t] = ids[t];
                }
            }
        }
        // the lanes of this wavefront read what other lanes of it wrote
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    for (int u = 0; u < nst; ++u) {
        const int j = j0 + u;
        if (j >= a.dist) break;
        const long long q0 = q_wave + (long long)j * S;
        if (q0 >= num_parts) break;
        const long long q = q0 + slot;
        const bool pv = q < num_parts;
        const int4 d = st_desc[u * S + slot];

        // carried partial row of the previous round: slot S-1 -> slot 0
        float cv[NV];
        int c_first = 0;
        if (c_open) {
            if constexpr (OFF_CROSSBAR) {
#pragma unroll
                for (int i = 0; i < NV; ++i) cv[i] = last_slot<LPR>(acc[i]);
                c_first = last_slot<LPR>(has_first);
            } else {
                const int src = (lane + 64 - LPR) & 63;
#pragma unroll
                for (int i = 0; i < NV; ++i) cv[i] = lane_read(acc[i], src);
                c_first = lane_read(has_first, src);
            }
        }
#pragma unroll
        for (int i = 0; i < NV; ++i) acc[i] = 0.0f;

        const int row = d.y;
        const int len = (int)((unsigned)d.z & DESC_LEN_MASK);
        const bool remote = d.x < 0;
        if constexpr (BUF) g.cbase = (remote ? a.delta_r : a.delta_l) + cofs;
        else g.base = static_cast<const char *>(remote ? a.in_r : a.in_l) + cofs;

        // neighbors [0, CH) of the partition were staged; a longer partition (ps > CH) fetches each further chunk of ids
        // into the same words when it gets there
        int *pid = st_ids + (u * S + slot) * CHP;
        for (int k0 = 0; k0 < a.ps; k0 += CH) {
            if (!__any(len > k0)) break;
            if (k0 > 0) {
                int raw_ids[IPL], ids[IPL];
                issue_ids(d, k0, raw_ids);
                finish_ids(d, k0, raw_ids, ids);
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
#pragma unroll
                for (int t = 0; t < IPL; ++t) pid[l * IPL + t] = ids[t];
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            }
            gather_chunk(len, k0, [&](auto q4) { return *reinterpret_cast<const int4 *>(static_cast<const int *>(__builtin_assume_aligned(pid, 16)) + 4 * decltype(q4)::value); });
        }

        // ---- combine the slots of this round ----
        has_first = ((unsigned)d.z & DESC_FIRST) ? 1 : 0;
        if (c_open && slot == 0) {
#pragma unroll
            for (int i = 0; i < NV; ++i) acc[i] += cv[i];
            has_first |= c_first;
        }
        // segmented inclusive scan over slots, keyed by row (equal rows are adjacent)
        if constexpr (OFF_CROSSBAR) {
            // No lane of this scan goes through the LDS crossbar.  At level j the slots whose bit j is set take the last
            // slot of the lower half of their group of 2^(j+1) slots (which by then holds the sum of its run so far): S - 1
            // additions in log2 S levels.  Slots that are whole rows of 16 lanes or halves of the wavefront move with the
            // row- and half-swap instructions; slots of 4 lanes move inside their row with DPP (row_shr, row_ror with bank
            // masks) and from row to row with a broadcast of the row's last slot followed by the same swaps.
            const auto step = [&](auto from, bool lower) {
                const int prow = from(row);
                const bool take = lower && prow == row && row >= 0;
                if (__any(take)) {
                    const int pf = from(has_first);
                    has_first |= take ? pf : 0;
#pragma unroll
                    for (int i = 0; i < NV; ++i) {
                        const float pvv = from(acc[i]);
                        acc[i] += take ? pvv : 0.0f;
                    }
                }
            };
            if constexpr (LPR == 16) {
                step([](auto v) { return rows_from_even(v); }, (slot & 1) != 0);
                step([](auto v) { return low_half(rows_from_odd(v)); }, slot >= 2);
            } else if constexpr (LPR == 32) {
                step([](auto v) { return low_half(v); }, slot == 1);
            } else {
                static_for<0, 4>([&](auto jj) {
                    constexpr int J = decltype(jj)::value;
                    if constexpr ((1 << J) < S) step([](auto v) { return scan_source<LPR, J>(v); }, ((slot >> J) & 1) != 0);
                });
            }
        } else {
        static_for<0, 6>([&](auto oo) {
            constexpr int o = 1 << decltype(oo)::value;
            if constexpr (o < S) {
                constexpr int SH = o * LPR;
                const int src = lane >= SH ? lane - SH : lane;
                const int prow = lane_read(row, src);
                const bool take = lane >= SH && prow == row && row >= 0;
                if (__any(take)) {
                    const int pf = lane_read(has_first, src);
                    has_first |= take ? pf : 0;
#pragma unroll
                    for (int i = 0; i < NV; ++i) {
                        const float pvv = lane_read(acc[i], src);
                        acc[i] += take ? pvv : 0.0f;
                    }
                }
            }
        });
        }
        // The last slot of each run now holds the run's sum.  A run ends where its row ends (the descriptor of a row's last
        // partition says so: the next descriptor, if any, belongs to another row) and at the last slot of the round.
        const bool row_done = ((unsigned)d.z & DESC_LAST) != 0;
        const bool run_last = pv && (row_done || slot == S - 1);
        const bool last_round = (j == a.dist - 1) || (q0 + S >= num_parts);
        bool keep_open = false;
        if (run_last) {
            if (row_done && has_first) {
                finish_row<LPR, MODE, SMX>(a, row, l, acc);
            } else if (!row_done && !last_round) {
                keep_open = true;  // slot S-1 only: continues in the next round
            } else {
                // partial row leaving this wavefront: head (started earlier) or tail (continues later)
                const int e = has_first ? 2 * wave + 1 : 2 * wave;
                const int f = HDR_VALID | (has_first ? HDR_STARTS : 0) | (row_done ? HDR_ENDS : 0);
                if (l == 0) hdr[e] = make_int2(row, f);
                float *dst = vals + (size_t)e * a.cpad;
#pragma unroll
                for (int i = 0; i < NV; ++i) {
                    const int dd = elem_of<LPR, MODE>(l, i);
                    if (dd < a.dim) dst[dd] = acc[i];
                }
            }
        }
        c_open = __any(keep_open);
    }
    }

    __syncthreads();
    if (wave != 0) return;

    // ---- combine the wavefronts of this workgroup (wavefront 0; lane = feature index mod 64) ----
    const int wg = (int)blockIdx.x;
    if (lane == 0) {
        a.c_hdr[2 * wg] = make_int2(-1, 0);
        a.c_hdr[2 * wg + 1] = make_int2(-1, 0);
    }
    float s[4] = {0.f, 0.f, 0.f, 0.f};
    bool open = false, started = false;
    int orow = -1;
    auto emit = [&](bool ends) {
        if (started && ends) {
            if (SMX) {
                float v[4];
                bool on[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    on[i] = lane + 64 * i < a.dim;
                    v[i] = on[i] ? epilogue_value(a, orow, lane + 64 * i, s[i]) : 0.f;
                }
                group_softmax<4>(v, on, 64);
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (on[i]) a.out[(long long)orow * a.ld_out + lane + 64 * i] = v[i];
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int dd = lane + 64 * i;
                    if (dd < a.dim) finish_elem(a, orow, dd, s[i]);
                }
            }
        } else {
            const int e = started ? 2 * wg + 1 : 2 * wg;
            if (lane == 0) a.c_hdr[e] = make_int2(orow, HDR_VALID | (started ? HDR_STARTS : 0) | (ends ? HDR_ENDS : 0));
            float *dst = a.c_val + (size_t)e * a.cpad;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int dd = lane + 64 * i;
                if (dd < a.dim) dst[dd] = s[i];
            }
        }
    };
    for (int w = 0; w < wpb; ++w) {
        const int2 h = hdr[2 * w];
        if (h.y & HDR_VALID) {
            if (!open) {
                open = true;
                started = false;
                orow = h.x;
#pragma unroll
                for (int i = 0; i < 4; ++i) s[i] = 0.f;
            }
            const float *src = vals + (size_t)(2 * w) * a.cpad;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int dd = lane + 64 * i;
                if (dd < a.dim) s[i] += src[dd];
            }
            if (h.y & HDR_ENDS) {
                emit(true);
                open = false;
            }
        }
        const int2 t = hdr[2 * w + 1];
        if (t.y & HDR_VALID) {
            open = true;
            started = true;
            orow = t.x;
            const float *src = vals + (size_t)(2 * w + 1) * a.cpad;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int dd = lane + 64 * i;
                s[i] = dd < a.dim ? src[dd] : 0.f;
            }
        }
    }
    if (open) emit(false);
}

// What the main kernel leaves open, in one launch.  Workgroups [0, fix_blocks): rows that cross workgroups -- the
// workgroup where such a row starts left a tail entry, every later workgroup up to the one where it ends a head entry.
// A wavefront finishes 64/comp_lanes consecutive workgroup slots at once: lane = (walker, component) with `comp_lanes` a
// power of two >= dim (<= 64; wider rows use one walker per wavefront and up to four components per lane); a walker whose
// slot holds a tail sums that row's chain of head entries in order, four loads in flight.  Workgroups from fix_blocks
// on: rows with no neighbor at all (their sum is zero), one group of comp_lanes lanes per row.
__global__ void __launch_bounds__(256) k_agg_tail(const AggArgs a, int num_wg, int comp_lanes, int fix_blocks, const int *__restrict__ empty_rows,
                                                  int n_empty)
{
    if (gate_closed(a.gate)) return;
    const int lane = lane_id();
    const int group = 64 / comp_lanes;
    const int c0 = lane % comp_lanes;
    float total[4] = {0.f, 0.f, 0.f, 0.f};
    int row;
    if ((int)blockIdx.x < fix_blocks) {
        const long long b = ((long long)blockIdx.x * 4 + (threadIdx.x >> 6)) * group + lane / comp_lanes;
        if (b >= num_wg - 1) return;
        const int2 t = a.c_hdr[2 * b + 1];
        if (!(t.y & HDR_VALID)) return;
        row = t.x;
        const int n = wg_of_part(a, a.off[row + 1] - 1) - (int)b;  // head entries of workgroups b+1 .. b+n
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = c0 + i * comp_lanes;
            if (c >= a.dim) break;
            float tot = a.c_val[(size_t)(2 * b + 1) * a.cpad + c];
            int k = 0;
            for (; k + 4 <= n; k += 4) {
                const float v0 = a.c_val[(size_t)(2 * (b + 1 + k)) * a.cpad + c];
                const float v1 = a.c_val[(size_t)(2 * (b + 2 + k)) * a.cpad + c];
                const float v2 = a.c_val[(size_t)(2 * (b + 3 + k)) * a.cpad + c];
                const float v3 = a.c_val[(size_t)(2 * (b + 4 + k)) * a.cpad + c];
                tot += v0;
                tot += v1;
                tot += v2;
                tot += v3;
            }
            for (; k < n; ++k) tot += a.c_val[(size_t)(2 * (b + 1 + k)) * a.cpad + c];
            total[i] = tot;
        }
    } else {
        const long long e = ((long long)((int)blockIdx.x - fix_blocks) * 4 + (threadIdx.x >> 6)) * group + lane / comp_lanes;
        if (e >= n_empty) return;
        row = empty_rows[e];
    }
    float v[4];
    bool on[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int c = c0 + i * comp_lanes;
        on[i] = c < a.dim;
        v[i] = on[i] ? epilogue_value(a, row, c, total[i]) : 0.f;
    }
    if (a.flags & MGGX_AGG_SOFTMAX) group_softmax<4>(v, on, comp_lanes);
#pragma unroll
    for (int i = 0; i < 4; ++i)
        if (on[i]) a.out[(long long)row * a.ld_out + c0 + i * comp_lanes] = v[i];
}

// What a column-blocked plan leaves open, in one launch: out[v] = epilogue(sum over blocks c of the partial row of
// virtual row c * rows + v, blocks in order [+ the dense core's partial rows of v]).  A virtual row that the main kernel
// finished lies in `part`; one that crossed workgroups is the sum of its chain in the carry buffer (the tail entry of the
// workgroup it starts in, then the head entries of the following ones); one without neighbors is zero -- all told by the
// plan's row offsets, so no fix-up pass, no zero fill and no separate reduction run.  G lanes per row (a power of two
// >= dim/4), lane q holds columns 4 q .. 4 q + 3; the epilogue is the caller's (row scale, accumulate, ReLU, softmax).
struct CoreMergeArgs {
    const float4 *sums;  // [core][n4]: the dense core's sum per core row, indexed by rank (k_core_reduce), or NULL
    const int *rank;     // [rows]: rank in the core or -1
};

template <int B>  // blocks per batch: 4, or all of them where a plan has 5 to 8 (one round of dependent loads instead of two)
__global__ void __launch_bounds__(256) k_agg_finish_blocked(const AggArgs a, const float *__restrict__ part, int rows, int blocks, int ldp, int g_shift,
                                                            const CoreMergeArgs cm)
{
    if (gate_closed(a.gate)) return;
    const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
    const int G = 1 << g_shift;  // lanes per row, a power of two
    const long long v_ll = idx >> g_shift;
    const int q = (int)(idx & (G - 1));
    const int n4 = (a.dim + 3) >> 2;
    if (v_ll >= rows) return;  // G divides 64: the lanes of a row leave together
    const int v = (int)v_ll;
    float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
    const bool lane_on = q < n4;
    if (lane_on) {
        int r = -1;  // rank in the dense core: asked for before anything else, its row of sums is read last
        if (cm.sums) {
            r = cm.rank[v];
        }
        // B blocks at a time: their row offsets first, then their partial rows, all in flight before the first sum
        for (int c0 = 0; c0 < blocks; c0 += B) {
            int o0[B], o1[B];
#pragma unroll
            for (int j = 0; j < B; ++j) {
                const long long vr = (long long)min(c0 + j, blocks - 1) * rows + v;
                o0[j] = a.off[vr];
                o1[j] = a.off[vr + 1];
            }
            float4 p[B];
            bool chain[B];
#pragma unroll
            for (int j = 0; j < B; ++j) {
                const bool there = c0 + j < blocks && o1[j] > o0[j];
                chain[j] = there && wg_of_part(a, o0[j]) != wg_of_part(a, o1[j] - 1);
                p[j] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (there && !chain[j]) p[j] = *reinterpret_cast<const float4 *>(part + ((long long)(c0 + j) * rows + v) * ldp + 4 * q);
            }
#pragma unroll
            for (int j = 0; j < B; ++j) {
                if (chain[j]) {  // the row crossed workgroups in this block: tail entry of the first, head entries of the others
                    const int w0 = wg_of_part(a, o0[j]), w1 = wg_of_part(a, o1[j] - 1);
                    p[j] = *reinterpret_cast<const float4 *>(a.c_val + (size_t)(2 * w0 + 1) * a.cpad + 4 * q);
                    for (int w = w0 + 1; w <= w1; ++w) {
                        const float4 h = *reinterpret_cast<const float4 *>(a.c_val + (size_t)(2 * w) * a.cpad + 4 * q);
                        p[j].x += h.x; p[j].y += h.y; p[j].z += h.z; p[j].w += h.w;
                    }
                }
                t.x += p[j].x; t.y += p[j].y; t.z += p[j].z; t.w += p[j].w;
            }
        }
        if (cm.sums) {
            if (r >= 0) {
                const float4 p = cm.sums[(size_t)r * n4 + q];
                t.x += p.x; t.y += p.y; t.z += p.z; t.w += p.w;
            }
        }
    }
    float val[4] = {t.x, t.y, t.z, t.w};
    bool on[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        on[i] = lane_on && 4 * q + i < a.dim;
        val[i] = on[i] ? epilogue_value(a, v, 4 * q + i, val[i]) : 0.f;
    }
    if (a.flags & MGGX_AGG_SOFTMAX) group_softmax<4>(val, on, G);
    float *o = a.out + (long long)v * a.ld_out + 4 * q;
    if (lane_on) {
        if (4 * q + 3 < a.dim && (a.ld_out & 3) == 0 && (reinterpret_cast<uintptr_t>(a.out) & 15u) == 0) {
            *reinterpret_cast<float4 *>(o) = make_float4(val[0], val[1], val[2], val[3]);
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (on[i]) o[i] = val[i];
        }
    }
}

int pow2_ceil(int x)
{
    int p = 1;
    while (p < x) p <<= 1;
    return p;
}

template <int MODE, bool BUF, bool SMX>
int launch_agg(int lpr, dim3 grid, dim3 block, size_t lds_bytes, hipStream_t stream, const AggArgs &a)
{
    switch (lpr) {
#define MGGX_CASE(L)                                                      \
    case L:                                                               \
        if (lds_bytes > (48u << 10))                                      \
            (void)hipFuncSetAttribute(reinterpret_cast<const void *>(&k_agg<L, MODE, BUF, SMX>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes); \
        k_agg<L, MODE, BUF, SMX><<<grid, block, lds_bytes, stream>>>(a);  \
        break;
        MGGX_CASE(1)
        MGGX_CASE(2)
        MGGX_CASE(4)
        MGGX_CASE(8)
        MGGX_CASE(16)
        MGGX_CASE(32)
        MGGX_CASE(64)
#undef MGGX_CASE
        default:
            return fail(MGGX_EINVAL, "aggregation: no kernel for %d lanes per row", lpr);
    }
    return MGGX_OK;
}

// `fixed` != NULL: the carry buffer comes from that block (the static scratch) instead of the library's grow-only
// workspace, and a call that does not fit is refused; nothing is allocated on that path.
struct FixedScratch {
    unsigned char *ptr;
    size_t bytes;
    const int *nnz_l_dev;
    const int *num_parts_dev;  // NULL: the plan's own count is exact
};

// The dense core's side of a call, handed to the aggregation of the remaining CSR: where a column-blocked plan ends in
// its finish kernel anyway, that kernel also waits for the core block (event `join`), adds its partial rows and applies
// the caller's whole epilogue (`merged` is set); otherwise the post-operations (ReLU, softmax) are left out here and the
// caller adds the core afterwards.
struct CoreMerge {
    const float4 *sums;
    const int *rank;
    int group_rows;  // of the core beside this call (the rules look at it)
    hipEvent_t join;
    bool merged;
};

int run_agg(Plan *plan, float *d_out, const void *d_in_l, const void *d_in_r, const int *d_col_l, const int *d_col_r,
            int lb, int dim, int wpb, int dist, const mggx_agg_opts &o_in, const Gate &gate, const FixedScratch *fixed = nullptr, CoreMerge *cm = nullptr)
{
    mggx_agg_opts o = o_in;
    State &st = state();
    if (dim < 1 || dim > 256) return fail(MGGX_ELIMIT, "aggregation: dim %d outside 1..256", dim);
    if (wpb < 0 || wpb > 16) return fail(MGGX_EINVAL, "aggregation: wpb %d outside 0..16 (0 = choose)", wpb);
    if (dist < 0) return fail(MGGX_EINVAL, "aggregation: dist %d must not be negative (0 = choose)", dist);
    const long long ld_in = o.ld_in ? o.ld_in : dim, ld_out = o.ld_out ? o.ld_out : dim;
    if (ld_in < dim || ld_out < dim) return fail(MGGX_EINVAL, "aggregation: row stride smaller than dim");
    if (plan->rows == 0) return MGGX_OK;
    if (!d_out || !d_in_l) return fail(MGGX_EINVAL, "aggregation: NULL feature pointer");
    const bool blocked = plan->blocks > 1 && plan->num_parts > 0;
    if (cm && !blocked) o.flags &= ~(MGGX_AGG_RELU | MGGX_AGG_SOFTMAX);  // the caller applies them after adding the core
    if (plan->nnz_r > 0 && (!d_in_r || !d_col_r)) return fail(MGGX_EINVAL, "aggregation: remote edges but no remote table");
    if (plan->nnz_l > 0 && !d_col_l) return fail(MGGX_EINVAL, "aggregation: local edges but no column array");

    int mode, lpr;
    const auto aligned16 = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; };
    if (o.in_dtype == MGGX_BF16) {
        if (dim % 8 || ld_in % 8 || ld_out % 4 || !aligned16(d_in_l) || (d_in_r && !aligned16(d_in_r)) || !aligned16(d_out))
            return fail(MGGX_EINVAL, "aggregation: bf16 tables need dim %% 8 == 0, ld_in %% 8 == 0 and 16-byte alignment");
        if (o.flags & MGGX_AGG_SOFTMAX) return fail(MGGX_EINVAL, "aggregation: the softmax epilogue takes fp32 tables (the last layer's logits)");
        mode = MODE_BF16_VEC8;
        lpr = pow2_ceil(dim / 8);
    } else if (o.in_dtype == MGGX_F32) {
        // 16-byte accesses per lane wherever the tables allow them: rows that start on 16-byte boundaries and are at least
        // ceil(dim/4) pieces long (a width that is not a multiple of 4 reads up to three padding columns of its own row
        // pitch and never stores them)
        const long long dim4 = (dim + 3) & ~3;
        const bool out_ok = blocked || (ld_out % 4 == 0 && ld_out >= dim4 && aligned16(d_out));  // blocked plans write their own partial rows
        const bool vec = ld_in % 4 == 0 && ld_in >= dim4 && out_ok && aligned16(d_in_l) && (!d_in_r || aligned16(d_in_r));
        mode = vec ? MODE_F32_VEC4 : MODE_F32_STRIDED;
        lpr = pow2_ceil((dim + 3) / 4);
    } else {
        return fail(MGGX_EINVAL, "aggregation: unknown input dtype %d", o.in_dtype);
    }
    const int slots = 64 / lpr;
    // 0 = let the library choose.  Few slots per wavefront (wide rows): 8 wavefronts and 16 rounds, so a workgroup still
    // covers a few thousand neighbors; column-blocked plans: 4 wavefronts (they share the chip with the dense core's
    // 4-wavefront workgroups); in row-major order beside a dense core: 8 wavefronts and 4 rounds, 8 rounds where the core
    // works in wide row groups (width 52 to 64, staged table beyond 12 MB: seven graphs of 0.7 to 3 M nodes at width 64 are
    // 1.4 - 3.7 % faster with 8 than with 4, one of them by 0.1 %; at width 48, narrow groups, 8 rounds cost 1.1 %); short
    // rows (under 3 partitions per row): 4 wavefronts.  Many slots (narrow rows): 4 wavefronts, 4 rounds; 8 rounds where a column-blocked
    // plan is left with short rows (under 8 partitions per row and block); 2 rounds for rows of 84 to 128 bytes (8 slots)
    // in row-major order beside a dense core -- there a wavefront's share is 16 partitions, as with 4 slots and 4 rounds.
    // Provenance: wpb x dist sweeps on the three benchmark graphs and the bf16 share (each choice within 1 % of the best
    // cell there), re-checked on graphs of other generators, sizes, degrees and widths: within 4 % of the best cell on
    // every one of twenty-four, after two changes they forced -- beside a core in row-major order the first version took
    // 4 wavefronts, which two 1 M-node graphs at widths 41 and 64 answered with 10 - 17 % over 8 wavefronts; and it took 4
    // rounds at 8 slots, 4 - 7 % over 2 rounds on two graphs of widths 24 and 32 (then, on three graphs made for the
    // purpose: widths 24 / 28 / 28 -0.1 / -3.6 / -1.8 % with 2 rounds; two graphs of width 20 were 1.4 and 2.7 % slower with 2,
    // three of widths 12 to 16 within 0.6 % except one 2.5 % faster: both stay at 4).
    const double per_row = (double)plan->num_parts / (double)(plan->rows > 0 ? plan->rows : 1);
    const bool beside_core = cm != nullptr;
    if (wpb == 0) wpb = (beside_core && !blocked && slots <= 4) ? 8 : (blocked || slots > 4 || per_row < 3.0) ? 4 : 8;
    if (dist == 0) {
        if (slots <= 4) dist = (beside_core && !blocked) ? (cm->group_rows == CORE_GROUP_ROWS_WIDE ? 8 : 4) : 16;
        else if (blocked && per_row < 8.0) dist = 8;
        else if (beside_core && !blocked && slots == 8 && dim > 20) dist = 2;
        else dist = 4;
    }
    const long long parts_per_wg = (long long)wpb * slots * dist;
    if (parts_per_wg > 0x3fffffffLL) return fail(MGGX_ELIMIT, "aggregation: wpb*dist too large");
    const long long num_wg = (plan->num_parts + parts_per_wg - 1) / parts_per_wg;
    if (num_wg > 0x7fffffffLL) return fail(MGGX_ELIMIT, "aggregation: too many workgroups");
    const int cpad = (dim + 3) & ~3;

    AggArgs a{};
    const int ldp = (dim + 3) & ~3;  // row stride of the per-block partial sums of a column-blocked plan
    a.out = d_out;
    a.in_l = d_in_l;
    a.in_r = d_in_r ? d_in_r : d_in_l;
    a.col_l = d_col_l;
    a.col_r = d_col_r;
    a.desc = plan->d_desc;
    a.off = plan->d_off;
    a.rs_out = blocked ? nullptr : o.d_row_scale_out;
    a.gate = gate;
    a.ld_in = ld_in;
    a.ld_out = blocked ? ldp : ld_out;
    a.num_parts = plan->num_parts;
    a.num_parts_dev = fixed ? fixed->num_parts_dev : nullptr;
    a.nnz_l = (int)plan->nnz_l;
    a.nnz_r = (int)plan->nnz_r;
    a.nnz_l_dev = fixed ? fixed->nnz_l_dev : nullptr;
    a.lb = lb;
    a.dim = dim;
    a.ps = plan->unit;  // what a slot sums at a time: whole partitions of one row, at most max(ps, 16) neighbors
    a.dist = dist;
    a.cpad = cpad;
    a.parts_per_wg = (int)parts_per_wg;
    a.ppw_shift = -1;
    if ((parts_per_wg & (parts_per_wg - 1)) == 0)
        for (a.ppw_shift = 0; (1LL << a.ppw_shift) < parts_per_wg;) ++a.ppw_shift;
    a.flags = blocked ? 0u : o.flags;
    a.eps = o.eps;
    a.in_is_bf16 = o.in_dtype == MGGX_BF16;

    // Gather addressing.  Extent of each table: the local one holds the share's rows, the remote one at least the
    // largest remote id.  When both fit one window of < 2 GiB and < 2^24 rows, offsets are 32-bit buffer offsets.
    const unsigned long long esize = a.in_is_bf16 ? 2 : 4;
    const unsigned long long ld_bytes = (unsigned long long)ld_in * esize;
    if (ld_bytes > 0xFFFFFFFFull) return fail(MGGX_ELIMIT, "aggregation: row stride of %llu bytes", ld_bytes);
    a.ld_bytes = (unsigned)ld_bytes;
    bool buf = false;
    {
        const unsigned long long pl = reinterpret_cast<uintptr_t>(a.in_l), pr = reinterpret_cast<uintptr_t>(a.in_r);
        const unsigned long long el = pl + (unsigned long long)plan->real_rows * ld_bytes;
        const bool has_r = plan->nnz_r > 0;
        const unsigned long long er = has_r ? pr + ((unsigned long long)plan->max_col_r + 1) * ld_bytes : el;
        const unsigned long long lo = has_r ? (pl < pr ? pl : pr) : pl;
        const unsigned long long hi = el > er ? el : er;
        const unsigned long long win = hi - lo;
        const unsigned long long sentinel = (win + ld_bytes - 1) / ld_bytes;
        if (win < 0x7FF00000ull && ld_bytes < (1ull << 24) && sentinel < (1ull << 24) - 1 && plan->real_rows < (1 << 24) &&
            (!has_r || plan->max_col_r < (1 << 24) - 1) && st.gather_addressing == 0) {
            buf = true;
            a.win_base = reinterpret_cast<const void *>(static_cast<uintptr_t>(lo));
            a.win_bytes = (unsigned)win;
            a.delta_l = (unsigned)(pl - lo);
            a.delta_r = has_r ? (unsigned)(pr - lo) : 0;
            a.sentinel = (int)sentinel;
        }
    }

    if (num_wg > 0) {
        const size_t hdr_bytes = (size_t)num_wg * 2 * sizeof(int2);
        const size_t hdr_pad = (hdr_bytes + 255) & ~(size_t)255;
        void *ws = nullptr;
        const size_t carry_bytes = (hdr_pad + (size_t)num_wg * 2 * cpad * sizeof(float) + 255) & ~(size_t)255;
        const size_t part_bytes = blocked ? (size_t)plan->rows * ldp * sizeof(float) : 0;
        int rc = MGGX_OK;
        if (fixed) {
            if (blocked || carry_bytes > fixed->bytes)
                return fail(MGGX_ELIMIT, "aggregation: %zu bytes of carry buffer for %lld workgroups exceed the static scratch (%zu left)",
                            carry_bytes, num_wg, fixed->bytes);
            ws = fixed->ptr;
        } else {
            rc = workspace(carry_bytes + part_bytes, &ws);
        }
        if (rc) return rc;
        a.c_hdr = static_cast<int2 *>(ws);
        a.c_val = reinterpret_cast<float *>(static_cast<char *>(ws) + hdr_pad);
        if (blocked) {
            a.out = reinterpret_cast<float *>(static_cast<char *>(ws) + carry_bytes);
        }
        // dynamic LDS: head/tail entries of the wavefronts, then their staged descriptors and ids (see k_agg); fewer
        // rounds are staged at a time when many wavefronts per workgroup would take more than 40 KiB
        const int stage_max = lpr >= 4 ? 4 : lpr == 2 ? 2 : 1;
        const int ch = lpr > 16 ? lpr : 16;
        const size_t round_bytes = (size_t)slots * ((size_t)(ch + 4) * 4 + 16);  // per slot: the staged ids (CHP words) and the descriptor
        int stage = stage_max < dist ? stage_max : dist;
        while (stage > 1 && (size_t)wpb * stage * round_bytes > (40u << 10)) stage /= 2;
        const size_t carry_lds = ((size_t)wpb * 2 * sizeof(int2) + (size_t)wpb * 2 * cpad * sizeof(float) + 15) & ~(size_t)15;
        a.stage_off = (int)(carry_lds / sizeof(float));
        a.stage_rounds = stage;
        const size_t lds_bytes = carry_lds + (size_t)wpb * stage * round_bytes + (size_t)MGGX_AGG_LDS_PAD;
        if (lds_bytes > (160u << 10)) return fail(MGGX_ELIMIT, "aggregation: %zu bytes of LDS per workgroup (wpb %d, dim %d)", lds_bytes, wpb, dim);
        const dim3 grid((unsigned)num_wg), block((unsigned)(64 * wpb));
        const bool smx = (a.flags & MGGX_AGG_SOFTMAX) != 0;  // fp32 tables only (checked above)
        if (buf) {
            if (mode == MODE_F32_VEC4) rc = smx ? launch_agg<MODE_F32_VEC4, true, true>(lpr, grid, block, lds_bytes, st.stream, a)
                                                : launch_agg<MODE_F32_VEC4, true, false>(lpr, grid, block, lds_bytes, st.stream, a);
            else if (mode == MODE_F32_STRIDED) rc = smx ? launch_agg<MODE_F32_STRIDED, true, true>(lpr, grid, block, lds_bytes, st.stream, a)
                                                        : launch_agg<MODE_F32_STRIDED, true, false>(lpr, grid, block, lds_bytes, st.stream, a);
            else rc = launch_agg<MODE_BF16_VEC8, true, false>(lpr, grid, block, lds_bytes, st.stream, a);
        } else {
            if (mode == MODE_F32_VEC4) rc = smx ? launch_agg<MODE_F32_VEC4, false, true>(lpr, grid, block, lds_bytes, st.stream, a)
                                                : launch_agg<MODE_F32_VEC4, false, false>(lpr, grid, block, lds_bytes, st.stream, a);
            else if (mode == MODE_F32_STRIDED) rc = smx ? launch_agg<MODE_F32_STRIDED, false, true>(lpr, grid, block, lds_bytes, st.stream, a)
                                                        : launch_agg<MODE_F32_STRIDED, false, false>(lpr, grid, block, lds_bytes, st.stream, a);
            else rc = launch_agg<MODE_BF16_VEC8, false, false>(lpr, grid, block, lds_bytes, st.stream, a);
        }
        if (rc) return rc;
        MGGX_LAUNCH_CHECK("k_agg");
    }
    if (blocked) {
        // one kernel finishes a column-blocked call: per-block partial rows and carry chains summed per row, the dense
        // core's partial rows on top where there are any, then the caller's epilogue
        AggArgs r = a;
        const float *part = a.out;
        r.out = d_out;
        r.ld_out = ld_out;
        r.rs_out = o.d_row_scale_out;
        r.flags = o.flags;
        CoreMergeArgs cma{nullptr, nullptr};
        if (cm) {
            MGGX_HIP(hipStreamWaitEvent(st.stream, cm->join, 0));
            cma = CoreMergeArgs{cm->sums, cm->rank};
            cm->merged = true;
        }
        const int G = pow2_ceil((dim + 3) / 4);
        int g_shift = 0;
        while ((1 << g_shift) < G) ++g_shift;
        const long long n = (long long)plan->real_rows * G;
        const dim3 fgrid((unsigned)((n + 255) / 256));
        switch (plan->blocks) {
#define MGGX_CASE(NB) case NB: k_agg_finish_blocked<NB><<<fgrid, dim3(256), 0, st.stream>>>(r, part, plan->real_rows, plan->blocks, ldp, g_shift, cma); break;
            MGGX_CASE(5) MGGX_CASE(6) MGGX_CASE(7) MGGX_CASE(8)
#undef MGGX_CASE
            default: k_agg_finish_blocked<4><<<fgrid, dim3(256), 0, st.stream>>>(r, part, plan->real_rows, plan->blocks, ldp, g_shift, cma);
        }
        MGGX_LAUNCH_CHECK("k_agg_finish_blocked");
    } else {
        // rows that cross workgroups and rows without neighbors, in one launch
        const bool touch_empty = !(o.flags & MGGX_AGG_ACCUMULATE) || (o.flags & (MGGX_AGG_GIN | MGGX_AGG_RELU | MGGX_AGG_SOFTMAX));
        const int n_empty = touch_empty ? plan->num_empty : 0;
        const int comp_lanes = dim >= 64 ? 64 : pow2_ceil(dim);
        const long long per_block = 4 * (64 / comp_lanes);
        const long long fix_blocks = num_wg > 1 ? (num_wg - 1 + per_block - 1) / per_block : 0;
        const long long empty_blocks = (n_empty + per_block - 1) / per_block;
        if (fix_blocks + empty_blocks > 0) {
            k_agg_tail<<<dim3((unsigned)(fix_blocks + empty_blocks)), dim3(256), 0, st.stream>>>(a, (int)num_wg, comp_lanes, (int)fix_blocks,
                                                                                               plan->d_empty_rows, n_empty);
            MGGX_LAUNCH_CHECK("k_agg_tail");
        }
    }
    snprintf(st.last_kernel, sizeof(st.last_kernel), "k_agg<%d,%d,%d> grid=%lld block=%d parts=%d blocks=%d ps=%d wpb=%d dist=%d addr=%s", lpr, mode, (int)buf,
             num_wg, 64 * wpb, plan->num_parts, plan->blocks, plan->ps, wpb, dist, buf ? "buffer32" : "flat64");
    return MGGX_OK;
}

}  // namespace
}  // namespace mggx

using mggx::fail;

namespace mggx {
namespace {

constexpr int DEFAULT_BLOCK_ROWS = 48 * 1024;  // neighbor ids per column block (sweeps on the 233 K-node benchmark graph)

// A column-blocked plan re-reads and re-writes a partial output row per block: it pays off when rows are long.
constexpr int MIN_NEIGHBORS_PER_ROW_AND_BLOCK = 20;
bool blocking_eligible(const GraphInfo &g, int block_rows)
{
    if (g.nnz_r > 0 || g.rows < 2 * (long long)block_rows) return false;
    const long long blocks = ((long long)g.rows + block_rows - 1) / block_rows;
    return g.nnz_l >= MIN_NEIGHBORS_PER_ROW_AND_BLOCK * blocks * (long long)g.rows;
}

struct Knobs {
    int ps, wpb, dist, block_rows;  // block_rows: > 0 column-blocked, -1 plain
    int core_rows;                  // > 0: that many highest-degree rows form a dense core served from LDS, -1: none
};

// The dense-core path pays for a plan and partial rows: worth considering on a local-only fp32 CSR with many rows
// beyond the core and a mean degree of 16 or more (on a power-law graph of mean degree 50 the 32 Ki highest-degree rows
// already hold enough edges among themselves for a quarter less time).
bool core_eligible(const GraphInfo &g, int dim, int dtype, int core_rows)
{
    return g.nnz_r == 0 && dtype == MGGX_F32 && dim <= 64 && g.rows >= 2 * (long long)core_rows && g.nnz_l >= 16 * (long long)g.rows;
}

// Fills in the knobs the caller left at 0: from the search's result for this CSR, width and element type where there is
// one, else by rule -- ps 16; the column-blocked order for long sorted rows; the dense core where the cost model over the
// degree histogram predicts a gain (its size too).  wpb and dist left at 0 are settled per plan in run_agg.
int resolve_knobs(GraphInfo &g, int dim, int dtype, int ps, int wpb, int dist, int block_rows, int core_rows, unsigned long long table_bytes,
                  Knobs *out)
{
    const GraphInfo::Tuned *t = nullptr;
    for (const GraphInfo::Tuned &e : g.tuned)
        if (e.dim == dim && e.dtype == dtype) t = &e;
    Knobs k{ps, wpb, dist, block_rows, core_rows};
    if (t && (ps == 0 || ps == t->ps) && wpb == 0 && dist == 0 && block_rows == 0 && core_rows == 0) {
        *out = Knobs{t->ps, t->wpb, t->dist, t->block_rows, t->core_rows};
        return MGGX_OK;
    }
    if (k.ps == 0) k.ps = 16;
    if (k.block_rows == 0) k.block_rows = blocking_eligible(g, DEFAULT_BLOCK_ROWS) ? DEFAULT_BLOCK_ROWS : -1;
    if (k.core_rows == 0) {
        k.core_rows = -1;
        if (core_eligible(g, dim, dtype, 8192)) {
            const int rc = predict_core_rows(g, dim, table_bytes, k.block_rows, MIN_NEIGHBORS_PER_ROW_AND_BLOCK, &k.core_rows);
            if (rc) return rc;
        }
    }
    *out = k;
    return MGGX_OK;
}

// `gate`: the call's content check of the caller's CSR arrays; every kernel launched below looks at it first.
int run_knobs(const GraphInfo &g, const Knobs &k, float *d_out, const void *d_in_local, const void *d_in_remote, const int *d_ptr_l,
              const int *d_col_l, const int *d_ptr_r, const int *d_col_r, int lb, int ub, int dim, const mggx_agg_opts &o, const Gate &gate, CoreMerge *cm = nullptr)
{
    Plan *plan = nullptr;
    int rc;
    if (k.core_rows > 0 && ub - lb >= 1024 && g.nnz_r == 0 && g.nnz_l > 0 && d_col_l && o.in_dtype == MGGX_F32 && dim >= 1 && dim <= 64 && d_out &&
        d_in_local) {
        CorePlan *cp = nullptr;
        rc = core_plan_get(d_ptr_l, d_col_l, ub - lb, lb, k.core_rows, core_group_rows((dim + 3) / 4, std::min(k.core_rows, ub - lb)), g.serial, &cp);
        if (rc) return rc;
        if (!cp->unsuitable) {
            // The core block is bound by the LDS, the rest of the CSR by the caches: they run side by side.  The core's sums
            // go to partial rows on a second stream while the rest of the CSR runs here.  Where that rest ends in the finish
            // kernel of a column-blocked plan, the same kernel joins the side stream, adds the core's partial rows and
            // applies the caller's epilogue; otherwise the rest runs with the epilogue except its post-operations (ReLU,
            // softmax), and k_core_finish adds the partial rows (times the row scale) and applies those last.
            const long long ld_in = o.ld_in ? o.ld_in : dim, ld_out = o.ld_out ? o.ld_out : dim;
            if (ld_in < dim || ld_out < dim) return fail(MGGX_EINVAL, "aggregation: row stride smaller than dim");
            State &st0 = state();
            hipStream_t side;
            hipEvent_t fork, join;
            rc = core_side_stream(&side, &fork, &join);
            if (rc) return rc;
            rc = run_core_stage(cp, static_cast<const float *>(d_in_local), dim, ld_in, gate, st0.stream);
            if (rc) return rc;
            MGGX_HIP(hipEventRecord(fork, st0.stream));
            MGGX_HIP(hipStreamWaitEvent(side, fork, 0));
            rc = run_core_sums(cp, dim, gate, side);
            const hipError_t er = hipEventRecord(join, side);
            int rc2 = MGGX_OK;
            GraphInfo *gr = nullptr;
            CoreMerge cm{nullptr, cp->d_rank, cp->group_rows, join, false};
            if (!rc) rc2 = core_row_sums(cp, dim, &cm.sums);
            if (!rc && !rc2) rc2 = graph_info(cp->d_rem_ptr, nullptr, cp->d_rem_col, nullptr, ub - lb, true, &gr);
            if (!rc && !rc2 && er == hipSuccess) {
                Knobs k2 = k;
                k2.core_rows = -1;
                if (k2.block_rows > 0 && !blocking_eligible(*gr, k2.block_rows)) k2.block_rows = -1;
                rc2 = run_knobs(*gr, k2, d_out, d_in_local, nullptr, cp->d_rem_ptr, cp->d_rem_col, nullptr, nullptr, lb, ub, dim, o, gate, &cm);
            }
            // the caller's stream takes the side stream back in whatever happened, so no work of this call outlives it unordered
            const hipError_t ew = er == hipSuccess ? (cm.merged ? hipSuccess : hipStreamWaitEvent(st0.stream, join, 0)) : er;
            if (rc) return rc;
            if (rc2) return rc2;
            if (ew != hipSuccess) return fail(MGGX_EHIP, "aggregation: joining the side stream: %s", hipGetErrorString(ew));
            if (!cm.merged) {
                rc = run_core_finish(cp, d_out, dim, ld_out, o.d_row_scale_out, (o.flags & MGGX_AGG_RELU) ? 1 : 0, (o.flags & MGGX_AGG_SOFTMAX) ? 1 : 0, gate,
                                     st0.stream);
                if (rc) return rc;
            }
            State &st = state();
            const size_t n = strlen(st.last_kernel);
            snprintf(st.last_kernel + n, sizeof(st.last_kernel) - n, " core=%d core_nnz=%lld rem_nnz=%lld%s", cp->core, (long long)cp->core_nnz,
                     (long long)cp->rem_nnz, cm.merged ? " merged_finish" : "");
            return MGGX_OK;
        }
    }
    if (k.block_rows > 0 && g.nnz_r == 0 && d_col_l && ub - lb >= 2 * (long long)k.block_rows) {
        rc = plan_get_blocked(d_ptr_l, d_col_l, ub - lb, lb, k.ps, k.block_rows, g.serial, &plan);
        if (rc) return rc;
        if (plan->unsuitable) plan = nullptr;
    }
    if (!plan) {
        rc = plan_get(d_ptr_l, d_ptr_r, d_col_r, ub - lb, k.ps, g.serial, &plan);
        if (rc) return rc;
    }
    return run_agg(plan, d_out, d_in_local, d_in_remote, d_col_l, d_col_r, lb, dim, k.wpb, k.dist, o, gate, nullptr, cm);
}

int check_np_div_args(const char *who, const int *d_ptr_l, int lb, int ub, int nodes_per_pe, int &ps, int block_rows, int core_rows)
{
    if (core_rows < -1) return fail(MGGX_EINVAL, "%s: core_rows %d (0 = choose, -1 = off)", who, core_rows);
    if (ub < lb || !d_ptr_l) return fail(MGGX_EINVAL, "%s: bad row range [%d,%d) or NULL row pointers", who, lb, ub);
    if (ps < 0) return fail(MGGX_EINVAL, "%s: ps %d must not be negative (0 = choose)", who, ps);
    if (nodes_per_pe < ub - lb) return fail(MGGX_EINVAL, "%s: nodes_per_pe %d smaller than the row range", who, nodes_per_pe);
    if (block_rows < -1) return fail(MGGX_EINVAL, "%s: col_block_rows %d (0 = choose, -1 = off)", who, block_rows);
    if (ps > (int)DESC_LEN_MASK) ps = (int)DESC_LEN_MASK;  // longer than any row: same partitions
    return MGGX_OK;
}

}  // namespace
}  // namespace mggx

MGGX_EXPORT int mggx_sag_np_div(float *d_out, const void *d_in_local, const void *d_in_remote, const int *d_ptr_l,
                                const int *d_col_l, const int *d_ptr_r, const int *d_col_r, int lb, int ub, int dim,
                                int nodes_per_pe, int ps, int wpb, int dist, const mggx_agg_opts *opts)
{
    int rc = mggx::ensure_init();
    if (rc) return rc;
    mggx_agg_opts o{};
    if (opts) o = *opts;
    rc = mggx::check_np_div_args("sag_np_div", d_ptr_l, lb, ub, nodes_per_pe, ps, o.col_block_rows, o.core_rows);
    if (rc) return rc;
    rc = mggx::stale_poll();
    if (rc) return rc;
    mggx::GraphInfo *g = nullptr;
    rc = mggx::graph_info(d_ptr_l, d_ptr_r, d_col_l, d_col_r, ub - lb, false, &g);
    if (rc) return rc;
    mggx::Gate gate;
    rc = mggx::guard_check(g->guard, &gate);
    if (rc) return rc;
    mggx::Knobs k;
    rc = mggx::resolve_knobs(*g, dim, o.in_dtype, ps, wpb, dist, o.col_block_rows, o.core_rows,
                             (unsigned long long)(ub - lb) * (unsigned long long)(o.ld_in ? o.ld_in : dim) * (o.in_dtype == MGGX_BF16 ? 2 : 4), &k);
    if (rc) return rc;
    return mggx::run_knobs(*g, k, d_out, d_in_local, d_in_remote, d_ptr_l, d_col_l, d_ptr_r, d_col_r, lb, ub, dim, o, gate);
}

MGGX_EXPORT int mggx_sag_np_div_tune(float *d_out, const void *d_in_local, const void *d_in_remote, const int *d_ptr_l,
                                     const int *d_col_l, const int *d_ptr_r, const int *d_col_r, int lb, int ub, int dim,
                                     int nodes_per_pe, int ps, const mggx_agg_opts *opts, mggx_agg_knobs *best_out, float *ms_best)
{
    int rc = mggx::ensure_init();
    if (rc) return rc;
    mggx_agg_opts o{};
    if (opts) o = *opts;
    rc = mggx::check_np_div_args("sag_np_div_tune", d_ptr_l, lb, ub, nodes_per_pe, ps, o.col_block_rows, o.core_rows);
    if (rc) return rc;
    if (o.flags & MGGX_AGG_ACCUMULATE) return fail(MGGX_EINVAL, "sag_np_div_tune: repeated runs would accumulate; clear MGGX_AGG_ACCUMULATE");
    rc = mggx::stale_poll();
    if (rc) return rc;
    if (mggx::capturing()) return fail(MGGX_EINVAL, "sag_np_div_tune: not inside a stream capture");
    mggx::GraphInfo *g = nullptr;
    rc = mggx::graph_info(d_ptr_l, d_ptr_r, d_col_l, d_col_r, ub - lb, false, &g);
    if (rc) return rc;
    mggx::Gate gate;
    rc = mggx::guard_check(g->guard, &gate);  // one fingerprint check for the whole search
    if (rc) return rc;
    mggx::State &st = mggx::state();
    const auto search_t0 = std::chrono::steady_clock::now();
    const double build_ms0 = st.plan_build_ms + st.core_plan_build_ms;
    hipEvent_t e0, e1;
    MGGX_HIP(hipEventCreate(&e0));
    MGGX_HIP(hipEventCreate(&e1));
    // the grid: ps as given, or {16, 32}; plain and, where rows are long enough, column-blocked; wpb x dist
    int pss[2] = {ps, 0}, n_ps = 1;
    if (ps == 0) { pss[0] = 16; pss[1] = 32; n_ps = 2; }
    int blks[2] = {-1, 0}, n_blk = 1;
    if (o.col_block_rows > 0) blks[0] = o.col_block_rows;
    else if (o.col_block_rows == 0 && mggx::blocking_eligible(*g, mggx::DEFAULT_BLOCK_ROWS)) { blks[1] = mggx::DEFAULT_BLOCK_ROWS; n_blk = 2; }
    int cores[6] = {-1, 0, 0, 0, 0, 0}, n_core = 1;  // without a dense core and, where it may pay, with one of five sizes
    if (o.core_rows > 0) {
        cores[0] = o.core_rows;
    } else if (o.core_rows == 0) {
        static const int sizes[] = {32 * 1024, 40 * 1024, 48 * 1024, 64 * 1024, 80 * 1024};
        for (int c : sizes)
            if (mggx::core_eligible(*g, dim, o.in_dtype, c)) cores[n_core++] = c;
    }
    static const int wpbs[] = {8, 4, 16}, dists[] = {1, 2, 4, 8, 16};
    // `timed` back-to-back calls of one setting between two events (after `untimed` ones): ms per call
    auto measure = [&](const mggx::Knobs &k, int untimed, int timed, float *ms_out) -> int {
        int r = MGGX_OK;
        for (int i = 0; i < untimed && !r; ++i)
            r = mggx::run_knobs(*g, k, d_out, d_in_local, d_in_remote, d_ptr_l, d_col_l, d_ptr_r, d_col_r, lb, ub, dim, o, gate);
        if (r) return r;
        hipError_t e = hipEventRecord(e0, st.stream);
        for (int i = 0; i < timed && !r; ++i)
            r = mggx::run_knobs(*g, k, d_out, d_in_local, d_in_remote, d_ptr_l, d_col_l, d_ptr_r, d_col_r, lb, ub, dim, o, gate);
        if (e == hipSuccess) e = hipEventRecord(e1, st.stream);
        if (e == hipSuccess) e = hipEventSynchronize(e1);
        float ms = 0.f;
        if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
        if (e != hipSuccess && !r) r = fail(MGGX_EHIP, "sag_np_div_tune: timing failed: %s", hipGetErrorString(e));
        *ms_out = ms / (float)timed;
        return r;
    };
    // The grid is measured coarsely (one untimed call, two timed ones back to back); the four fastest settings and the
    // one the library's rules and cost model pick then meet again, twice over eight calls each, so that a setting cannot
    // win on one lucky measurement, and the result is never slower than leaving the knobs at 0 by more than the noise.
    constexpr int FINALISTS = 4;
    mggx::Knobs top[FINALISTS + 1];
    float top_ms[FINALISTS + 1];
    int n_top = 0;
    mggx::Knobs bk{pss[0], 8, 1, blks[0], cores[0]};
    {
        float warm = 0.f;  // plans built, clocks up
        rc = measure(bk, 1, 4, &warm);
    }
    for (int ci = 0; ci < n_core && !rc; ++ci)
    for (int pi = 0; pi < n_ps && !rc; ++pi)
        for (int bi = 0; bi < n_blk && !rc; ++bi)
            for (int wi = 0; wi < 3 && !rc; ++wi)
                for (int di = 0; di < 5 && !rc; ++di) {
                    const mggx::Knobs k{pss[pi], wpbs[wi], dists[di], blks[bi], cores[ci]};
                    float ms = 0.f;
                    rc = measure(k, 1, 2, &ms);
                    if (rc) break;
                    int at = n_top;
                    while (at > 0 && top_ms[at - 1] > ms) --at;
                    if (at < FINALISTS) {
                        const int last = n_top < FINALISTS ? n_top : FINALISTS - 1;
                        for (int i = last; i > at; --i) { top[i] = top[i - 1]; top_ms[i] = top_ms[i - 1]; }
                        top[at] = k;
                        top_ms[at] = ms;
                        if (n_top < FINALISTS) ++n_top;
                    }
                }
    if (!rc && n_top > 0) {
        // the setting the knobs left at 0 would get without a search (what this search must not lose to)
        mggx::Knobs by_rule{};
        std::vector<mggx::GraphInfo::Tuned> keep;
        keep.swap(g->tuned);  // an earlier search's result is not "by rule"
        const unsigned long long table_bytes = (unsigned long long)(ub - lb) * (unsigned long long)(o.ld_in ? o.ld_in : dim) *
                                               (o.in_dtype == MGGX_BF16 ? 2ull : 4ull);
        rc = mggx::resolve_knobs(*g, dim, o.in_dtype, ps, 0, 0, o.col_block_rows, o.core_rows, table_bytes, &by_rule);
        keep.swap(g->tuned);
        if (!rc) {
            top[n_top] = by_rule;
            top_ms[n_top] = 0.f;
            ++n_top;
        }
    }
    // Two passes, the faster one counts: a plan built a moment ago (the rule's core size, if the grid did not hold it) runs
    // 5 - 10 % slower for its first dozen calls, which the first pass absorbs.
    float best = -1.f;
    float final_ms[FINALISTS + 1];
    for (int pass = 0; pass < 2 && !rc; ++pass)
        for (int i = 0; i < n_top && !rc; ++i) {
            float ms = 0.f;
            rc = measure(top[i], 2, 8, &ms);
            if (!rc && (pass == 0 || ms < final_ms[i])) final_ms[i] = ms;
        }
    for (int i = 0; i < n_top && !rc; ++i)
        if (best < 0.f || final_ms[i] < best) { best = final_ms[i]; bk = top[i]; }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (rc) return rc;
    // leave the winner's result in d_out and remember it
    rc = mggx::run_knobs(*g, bk, d_out, d_in_local, d_in_remote, d_ptr_l, d_col_l, d_ptr_r, d_col_r, lb, ub, dim, o, gate);
    if (rc) return rc;
    MGGX_HIP(hipStreamSynchronize(st.stream));
    if (bk.wpb == 0 || bk.dist == 0) {  // the rule's setting won: report what the rule made of it for this plan
        const char *w = strstr(st.last_kernel, " wpb=");
        int rw = 0, rd = 0;
        if (w && sscanf(w, " wpb=%d dist=%d", &rw, &rd) == 2) { bk.wpb = rw; bk.dist = rd; }
    }
    // the search's own time: what the plan builds inside it took is accounted for separately
    st.search_ms += std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - search_t0).count() -
                    (st.plan_build_ms + st.core_plan_build_ms - build_ms0);
    bool found = false;
    for (mggx::GraphInfo::Tuned &t : g->tuned)
        if (t.dim == dim && t.dtype == o.in_dtype) { t.ps = bk.ps; t.wpb = bk.wpb; t.dist = bk.dist; t.block_rows = bk.block_rows; t.core_rows = bk.core_rows; found = true; }
    if (!found) g->tuned.push_back({dim, o.in_dtype, bk.ps, bk.wpb, bk.dist, bk.block_rows, bk.core_rows});
    if (best_out) { best_out->ps = bk.ps; best_out->wpb = bk.wpb; best_out->dist = bk.dist; best_out->col_block_rows = bk.block_rows; best_out->core_rows = bk.core_rows; }
    if (ms_best) *ms_best = best;
    return MGGX_OK;
}

MGGX_EXPORT int mggx_sag_parts(float *d_out, const float *d_in, const int *d_row_ptr, const int *d_col,
                               const int *d_part_ptr, const int *d_part2node, int lowbound, int num_nodes,
                               int num_parts, int ps, int dim, int wpb, int dist)
{
    int rc = mggx::ensure_init();
    if (rc) return rc;
    if (!d_row_ptr || !d_part_ptr || !d_part2node || num_nodes < 0 || num_parts < 0 || ps < 1)
        return fail(MGGX_EINVAL, "sag_parts: bad argument");
    mggx::Plan *plan = nullptr;
    rc = mggx::stale_poll();
    if (rc) return rc;
    rc = mggx::plan_get_explicit(d_row_ptr, d_part_ptr, d_part2node, num_nodes, num_parts, ps, &plan);
    if (rc) return rc;
    mggx::Gate gate;
    rc = mggx::guard_check(plan->guard, &gate);
    if (rc) return rc;
    mggx_agg_opts o{};
    o.flags = MGGX_AGG_ACCUMULATE;
    return mggx::run_agg(plan, d_out, d_in, nullptr, d_col, nullptr, lowbound, dim, wpb, dist, o, gate);
}

namespace mggx {

namespace {
constexpr int MAX_DEVICES = 64;
unsigned char *g_scratch_ptr[MAX_DEVICES];  // device address of `scratch` on each device, once asked for
}  // namespace

// Address of this device's copy of the static scratch array (asked for once per device, with that device current).
int static_scratch_ptr(unsigned char **out)
{
    int dev = -1;
    MGGX_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= MAX_DEVICES) return fail(MGGX_ELIMIT, "static scratch: device index %d", dev);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) return fail(MGGX_EHIP, "static scratch: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
        g_scratch_ptr[dev] = static_cast<unsigned char *>(p);
    }
    *out = g_scratch_ptr[dev];
    return MGGX_OK;
}

}  // namespace mggx

MGGX_EXPORT int mggx_sag_parts_static(float *d_out, const float *d_in, const int *d_row_ptr, const int *d_col,
                                      const int *d_part_ptr, const int *d_part2node, int lowbound, int num_nodes,
                                      int num_parts, int ps, int dim, int wpb, int dist)
{
    int rc = mggx::ensure_init();
    if (rc) return rc;
    if (!d_row_ptr || !d_part_ptr || !d_part2node || num_nodes < 0 || num_parts < 0 || ps < 1)
        return fail(MGGX_EINVAL, "sag_parts_static: bad argument");
    if (num_nodes == 0 || num_parts == 0) return MGGX_OK;  // out += nothing
    unsigned char *base = nullptr;
    rc = mggx::static_scratch_ptr(&base);
    if (rc) return rc;
    // layout of the scratch: descriptors | first descriptor of each row | [scratch of the unit builder, ps < 16] | carry
    // buffer (sized by run_agg)
    const auto pad = [](size_t b) { return (b + 255) & ~(size_t)255; };
    const bool grouped = mggx::unit_of(ps) != ps;
    const size_t desc_bytes = pad(sizeof(int4) * (size_t)num_parts), off_bytes = pad(sizeof(int) * ((size_t)num_nodes + 1));
    const size_t tmp_bytes = grouped ? pad(sizeof(int) * mggx::explicit_tmp_ints(num_nodes)) : 0;
    if (desc_bytes + off_bytes + tmp_bytes >= (size_t)MGGX_STATIC_SCRATCH_BYTES)
        return fail(MGGX_ELIMIT, "sag_parts_static: %d partitions over %d rows need %zu bytes of descriptors; the static scratch holds %zu",
                    num_parts, num_nodes, desc_bytes + off_bytes + tmp_bytes, (size_t)MGGX_STATIC_SCRATCH_BYTES);
    mggx::Plan plan;  // lives for this call only; its arrays are views into the scratch
    plan.d_ptr_l = d_row_ptr;
    plan.d_part_ptr = d_part_ptr;
    plan.d_part2node = d_part2node;
    plan.rows = plan.real_rows = num_nodes;
    plan.ps = ps;
    plan.unit = mggx::unit_of(ps);
    plan.caller_parts = num_parts;
    plan.d_desc = reinterpret_cast<int4 *>(base);
    plan.d_off = reinterpret_cast<int *>(base + desc_bytes);
    plan.nnz_l = 1;  // "has local edges"; the kernels read the count itself from d_row_ptr[num_nodes]
    long long bound = num_parts;
    rc = mggx::explicit_desc_fill(d_row_ptr, d_part_ptr, d_part2node, num_nodes, num_parts, ps, plan.d_desc, plan.d_off,
                                  reinterpret_cast<int *>(base + desc_bytes + off_bytes), &bound);
    if (rc) return rc;
    // ps < 16: several partitions per descriptor; their number stays on the device (d_off[rows]) and the grid is sized by a bound
    plan.num_parts = (int)bound;
    const size_t used = desc_bytes + off_bytes + tmp_bytes;
    const mggx::FixedScratch fx{base + used, (size_t)MGGX_STATIC_SCRATCH_BYTES - used, d_row_ptr + num_nodes, grouped ? plan.d_off + num_nodes : nullptr};
    mggx_agg_opts o{};
    o.flags = MGGX_AGG_ACCUMULATE;
    return mggx::run_agg(&plan, d_out, d_in, nullptr, d_col, nullptr, lowbound, dim, wpb, dist, o, mggx::Gate{}, &fx);
}

MGGX_EXPORT int mggx_spmm(float *d_out, const float *d_in, const int *d_row_ptr, const int *d_col, int num_nodes,
                          int dim, int ps, int wpb)
{
    int rc = mggx::ensure_init();
    if (rc) return rc;
    if (!d_row_ptr || num_nodes < 0 || ps < 0) return fail(MGGX_EINVAL, "spmm: bad argument");
    mggx_agg_opts o{};
    o.flags = MGGX_AGG_ACCUMULATE;
    rc = mggx::stale_poll();
    if (rc) return rc;
    mggx::GraphInfo *g = nullptr;
    rc = mggx::graph_info(d_row_ptr, nullptr, d_col, nullptr, num_nodes, false, &g);
    if (rc) return rc;
    mggx::Gate gate;
    rc = mggx::guard_check(g->guard, &gate);
    if (rc) return rc;
    // the whole graph on one GPU: the same knob rules (and column-blocked order for long rows) as mggx_sag_np_div
    mggx::Knobs k;
    rc = mggx::resolve_knobs(*g, dim, MGGX_F32, ps, wpb, 0, 0, 0, (unsigned long long)num_nodes * dim * 4, &k);
    if (rc) return rc;
    return mggx::run_knobs(*g, k, d_out, d_in, nullptr, d_row_ptr, d_col, nullptr, nullptr, 0, num_nodes, dim, o, gate);
}
