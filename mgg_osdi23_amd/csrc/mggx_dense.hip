// Dense node update Out = X . W on the matrix cores (fp32 and bf16 MFMA), and the row softmax.
#include <algorithm>

#include "mggx_dev.h"

// Where k_wt_image leaves the bf16 update's weight matrix for the workgroups of k_dense_xw_bf16_lines (one per GPU the
// library runs on; calls on the library's stream follow one another).  In host code the name is only a handle for
// hipGetSymbolAddress.
static __device__ __align__(256) unsigned short wt_image[128 * (128 + 8)];

namespace mggx {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));

constexpr int GEMM_KC = 64;       // K extent of the W tile staged in LDS by the chunked kernel
constexpr int GEMM_ROWS_WG = 64;  // 4 wavefronts x 16 rows
constexpr size_t LDS_RESIDENT_LIMIT = 72 * 1024;  // keep W resident in LDS up to this size (two workgroups per CU)

struct DenseArgs {
    void *out;
    const void *x;
    const void *w;
    const float *rs;
    long long n;
    long long ld_x, ld_out;
    int d1, d2;
    int relu;
    int vec_out;  // bit 0: rows of out may be written 4 elements at a time (alignment and stride allow it);
                  // bit 1: and they are whole 128-byte lines written once: streaming stores;
                  // bit 2: bf16 rows may be written 8 elements (16 bytes) at a time
    int stream_x; // rows of X are whole 128-byte lines per K group (d1 % 64 == 0, aligned base and pitch)
    int tiles_per_wave;  // k_dense_xw_bf16_lines: rounds of consecutive tiles per workgroup
};

// v_mfma_f32_16x16x4_f32 operand layout (wave64):
//   A (16 x 4): lane L holds A[L % 16][L / 16]
//   B (4 x 16): lane L holds B[L / 16][L % 16]
//   D (16 x 16): lane L holds D[4 * (L / 16) + r][L % 16], r = 0..3
// Each lane loads 4 consecutive K values of one X row; MFMA step t then multiplies the K indices {4*(L/16) + t},
// and B is read from LDS with the same index, so the sum over K is complete after 4 steps per 16 K values.
__device__ __forceinline__ void load_x4(float (&xv)[4], const float *xrow, int kb, int d1, bool row_ok)
{
    xv[0] = xv[1] = xv[2] = xv[3] = 0.f;
    if (!row_ok) return;
    if (kb + 3 < d1) {
        float4 t4;
        __builtin_memcpy(&t4, xrow + kb, 16);
        xv[0] = t4.x; xv[1] = t4.y; xv[2] = t4.z; xv[3] = t4.w;
    } else {
#pragma unroll
        for (int t = 0; t < 4; ++t)
            if (kb + t < d1) xv[t] = xrow[kb + t];
    }
}

// Branch-free form for the resident kernels.  `xrow` is a valid row (callers clamp the row index; results of rows
// past the end are never stored).  `mode` is the same for the whole wavefront:
//   0  the 64-wide K group lies inside the row: plain 16-byte loads
//   1  d1 % 4 == 0: a lane's 4 values are all inside or all outside; load from a clamped offset, zero if outside
//   2  any d1: four dword loads from clamped offsets, zeroed one by one
__device__ __forceinline__ void load_x4u(float (&xv)[4], const float *xrow, int kb, int d1, int mode)
{
    if (mode == 3) {  // as mode 0, and every 64-wide K group of a row is two whole cache lines read once: streaming hint
        typedef float v4f_u __attribute__((ext_vector_type(4), aligned(16)));
        const v4f_u t4 = __builtin_nontemporal_load(reinterpret_cast<const v4f_u *>(xrow + kb));
        xv[0] = t4.x; xv[1] = t4.y; xv[2] = t4.z; xv[3] = t4.w;
    } else if (mode == 0) {
        float4 t4;
        __builtin_memcpy(&t4, xrow + kb, 16);
        xv[0] = t4.x; xv[1] = t4.y; xv[2] = t4.z; xv[3] = t4.w;
    } else if (mode == 1) {
        float4 t4;
        __builtin_memcpy(&t4, xrow + min(kb, d1 - 4), 16);
        const bool in = kb < d1;
        xv[0] = in ? t4.x : 0.f; xv[1] = in ? t4.y : 0.f; xv[2] = in ? t4.z : 0.f; xv[3] = in ? t4.w : 0.f;
    } else {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const float v = xrow[min(kb + t, d1 - 1)];
            xv[t] = kb + t < d1 ? v : 0.f;
        }
    }
}
__device__ __forceinline__ int x_group_mode(int k_first, int width, int d1, int chunk)
{
    return k_first + width <= d1 ? 0 : (d1 % chunk == 0 ? 1 : 2);
}

template <int NB>
__device__ __forceinline__ void store_tile_f32(const DenseArgs &a, const v4f (&acc)[NB], long long row_base, int c0, int i)
{
    float *out = static_cast<float *>(a.out);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const long long orow = row_base + r;
        if (orow >= a.n) continue;
        const float scale = a.rs ? a.rs[orow] : 1.0f;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const int c = c0 + nb * 16 + i;
            if (c < a.d2) {
                float v = acc[nb][r] * scale;
                if (a.relu) v = fmaxf(v, 0.f);
                out[orow * a.ld_out + c] = v;
            }
        }
    }
}

// The resident kernels form every product transposed -- W as the A operand, X as the B operand (both operand layouts
// give lane L the element (L % 16, L / 16), so the loads are the same) -- which leaves lane L with
// D[row L % 16][16 nb + 4 (L / 16) + r], r = 0..3: four consecutive columns of one output row, one 16-byte store.
// bf16 output with the columns of W staged pairwise interleaved (paired_column below): lane (row, kq) holds the eight
// consecutive columns 32 p + 8 kq .. + 7 in acc[2 p] and acc[2 p + 1] -- one 16-byte store, 64 contiguous bytes per row and
// instruction (unpaired: 8-byte stores, 32 bytes per row and instruction, and the write path, not the reads, set the pace).
template <int NB>
__device__ __forceinline__ void store_rows_bf16_paired(void *out, long long ld_out, float scale, int relu, const v4f (&acc)[NB],
                                                       long long row, bool row_ok, int c0, int kq)
{
    static_assert(NB % 2 == 0, "pairs of 16-column blocks");
    if (!row_ok) return;
    typedef unsigned v4u_s __attribute__((ext_vector_type(4)));
#pragma unroll
    for (int p = 0; p < NB / 2; ++p) {
        unsigned pk[4];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            float v[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                v[r] = acc[2 * p + h][r] * scale;
                if (relu) v[r] = fmaxf(v[r], 0.f);
            }
            const v2bf q0 = __builtin_convertvector((v2f){v[0], v[1]}, v2bf), q1 = __builtin_convertvector((v2f){v[2], v[3]}, v2bf);
            __builtin_memcpy(&pk[2 * h], &q0, 4);
            __builtin_memcpy(&pk[2 * h + 1], &q1, 4);
        }
        __bf16 *o = static_cast<__bf16 *>(out) + row * ld_out + c0 + 32 * p + 8 * kq;
        __builtin_nontemporal_store((v4u_s){pk[0], pk[1], pk[2], pk[3]}, reinterpret_cast<v4u_s *>(o));
    }
}
// Which column of W the LDS column slot j (16-column block j / 16, position j % 16) holds when blocks are paired.
__device__ __forceinline__ int paired_column(int j)
{
    const int nb = j >> 4, m = j & 15;
    return 32 * (nb >> 1) + 8 * (m >> 2) + 4 * (nb & 1) + (m & 3);
}

template <int NB, bool OUT_BF16>
__device__ __forceinline__ void store_rows(void *out, long long ld_out, int d2, float scale, int relu, int vec_out,
                                           const v4f (&acc)[NB], long long row, bool row_ok, int c0, int kq)
{
    if (!row_ok) return;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        const int c = c0 + nb * 16 + 4 * kq;
        if (c >= d2) continue;
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            v[r] = acc[nb][r] * scale;
            if (relu) v[r] = fmaxf(v[r], 0.f);
        }
        if constexpr (OUT_BF16) {
            __bf16 *o = static_cast<__bf16 *>(out) + row * ld_out + c;
            const v2bf p0 = __builtin_convertvector((v2f){v[0], v[1]}, v2bf);
            const v2bf p1 = __builtin_convertvector((v2f){v[2], v[3]}, v2bf);
            if (vec_out && c + 3 < d2) {
                const __bf16 q[4] = {p0[0], p0[1], p1[0], p1[1]};
                __builtin_memcpy(__builtin_assume_aligned(o, 8), q, 8);
            } else {
                o[0] = p0[0];
                if (c + 1 < d2) o[1] = p0[1];
                if (c + 2 < d2) o[2] = p1[0];
                if (c + 3 < d2) o[3] = p1[1];
            }
        } else {
            float *o = static_cast<float *>(out) + row * ld_out + c;
            if (vec_out && c + 3 < d2) {
                if (vec_out & 2) __builtin_nontemporal_store((v4f){v[0], v[1], v[2], v[3]}, reinterpret_cast<v4f *>(o));
                else *reinterpret_cast<float4 *>(o) = make_float4(v[0], v[1], v[2], v[3]);
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (c + r < d2) o[r] = v[r];
            }
        }
    }
}

// Row softmax of a finished 16-row tile in the transposed-product layout, before it is stored: lane (row i, kq) holds the
// columns 16 nb + 4 kq + r of its row, so a row's values sit in the four lanes i, i + 16, i + 32, i + 48.  acc <- exp(scale
// acc - max) / sum over the d2 columns that exist (the rest become 0 and are not stored).  All 64 lanes take part.
template <int NB>
__device__ __forceinline__ void tile_row_softmax(v4f (&acc)[NB], float scale, int d2, int kq)
{
    float m = -3.0e38f;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            acc[nb][r] *= scale;
            if (16 * nb + 4 * kq + r < d2) m = fmaxf(m, acc[nb][r]);
        }
    m = fmaxf(m, __shfl_xor(m, 16));
    m = fmaxf(m, __shfl_xor(m, 32));
    float sum = 0.f;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float e = 16 * nb + 4 * kq + r < d2 ? __expf(acc[nb][r] - m) : 0.f;
            acc[nb][r] = e;
            sum += e;
        }
    sum += __shfl_xor(sum, 16);
    sum += __shfl_xor(sum, 32);
    const float inv = 1.0f / sum;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[nb][r] *= inv;
}

// A finished 16-row tile whose rows are packed (ld_out = d2) but no multiple of 16 bytes (47 floats): stored from the
// operand layout it would leave as 4-byte pieces, four lanes to a row.  The tile itself is one contiguous run of 16 d2
// floats that starts on a 16-byte boundary, so it goes through the wavefront's piece of LDS, laid out as in memory, and
// leaves in 16-byte stores of whole consecutive lines.  `v` already carries scale and activation.
template <int NB>
__device__ __forceinline__ void store_tile_flat(float *out, float *piece, int d2, long long n, const v4f (&v)[NB], long long tile, int i,
                                                int kq, int lane)
{
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int c = 16 * nb + 4 * kq + r;
            if (c < d2) piece[i * d2 + c] = v[nb][r];
        }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int span = (int)min(16LL, n - tile * 16) * d2;  // floats of the tile that exist
    float *dst = out + tile * 16 * d2;
    for (int f = 4 * lane; f < span; f += 256) {
        if (f + 3 < span) {
            __builtin_nontemporal_store(*reinterpret_cast<const v4f *>(piece + f), reinterpret_cast<v4f *>(dst + f));
        } else {
            for (int t = 0; f + t < span; ++t) dst[f + t] = piece[f + t];
        }
    }
    __builtin_amdgcn_wave_barrier();  // the piece is free for the next tile once every lane has read its part
}

// W kept whole in LDS; the 8 wavefronts of a workgroup walk over 16-row tiles of X.  K is cut into groups of 64.
// FULL (d1 >= 64): every group is a whole 64 wide -- the last one is shifted back to [d1 - 64, d1) and the W rows
// it shares with the group before are zero in LDS, so every X load is a plain in-row 16-byte load with no tail
// handling.  !FULL (d1 < 64): one group, loads clamped and masked.  X is read one group ahead of the matrix cores;
// the group after the last one of a tile is the first one of the wavefront's next tile.
constexpr int RES_THREADS = 512;

// K index held by LDS row r (-1: a zero row)
template <bool FULL>
__device__ __forceinline__ int lds_row_k(int r, int ngroups, int d1)
{
    if constexpr (FULL) {
        const int g = r >> 6;
        if (g < ngroups - 1) return r;
        const int k = d1 - 64 + (r & 63);
        return k >= 64 * g ? k : -1;
    } else {
        return r < d1 ? r : -1;
    }
}

// KMODE: 0 = d1 < 64, 1 = d1 >= 64, 2 = d1 >= 64 and every K group of a row is whole cache lines (streamed)
template <int KMODE>
__device__ __forceinline__ void load_group(float (&x)[4][4], const float *xrow, int g, int ngroups, int d1, int kq)
{
    if constexpr (KMODE >= 1) {
        const int ks = (g == ngroups - 1 ? d1 - 64 : 64 * g) + 4 * kq;
        constexpr int mode = KMODE == 2 ? 3 : 0;
#pragma unroll
        for (int gg = 0; gg < 4; ++gg) load_x4u(x[gg], xrow, ks + 16 * gg, d1, mode);
    } else {
        const int mode = d1 % 4 == 0 ? 1 : 2;
        const int ngg = (d1 + 15) >> 4;  // 16-wide K steps that hold anything
#pragma unroll
        for (int gg = 0; gg < 4; ++gg) {
            if (gg < ngg) {
                load_x4u(x[gg], xrow, 16 * gg + 4 * kq, d1, mode);
            } else {
                x[gg][0] = x[gg][1] = x[gg][2] = x[gg][3] = 0.f;
            }
        }
    }
}

// The wait for loaded values happens where this is called.  The counter such a wait uses counts loads and stores alike, in
// order: where the compiler places the wait for a prefetched operand after the stores of a finished tile (the end of a
// loop body), the wavefront sits there until those stores are acknowledged; called before the stores, the wait only
// covers the loads, which were issued long before, and the stores have the whole next tile to complete.
__device__ __forceinline__ void arrived(float (&x)[4][4], float &s)
{
    asm volatile("" : "+v"(x[0][0]), "+v"(x[0][1]), "+v"(x[0][2]), "+v"(x[0][3]), "+v"(x[1][0]), "+v"(x[1][1]), "+v"(x[1][2]),
                 "+v"(x[1][3]), "+v"(x[2][0]), "+v"(x[2][1]), "+v"(x[2][2]), "+v"(x[2][3]), "+v"(x[3][0]), "+v"(x[3][1]),
                 "+v"(x[3][2]), "+v"(x[3][3]), "+v"(s));
}

// acc[nb] += Wt-block^T . X-group, transposed product (see store_rows)
template <int NB, int RS>
__device__ __forceinline__ void mfma_group(v4f (&acc)[NB], const float *wt_group, const float (&x)[4][4], int i, int kq, int ngg)
{
#pragma unroll
    for (int gg = 0; gg < 4; ++gg) {
        if (gg >= ngg) break;  // d1 < 64: the remaining 16-wide K steps are all zero
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const float *wrow = wt_group + (16 * gg + 4 * kq + t) * RS + i;
#pragma unroll
            for (int nb = 0; nb < NB; ++nb)
                acc[nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(wrow[nb * 16], x[gg][t], acc[nb], 0, 0, 0);
        }
    }
}

template <int NB, int KMODE>
__global__ void __launch_bounds__(RES_THREADS, 4) k_dense_xw_resident(const DenseArgs a)
{
    constexpr bool FULL = KMODE >= 1;
    constexpr int RS = NB * 16 + 4;  // LDS row stride in floats; the +4 keeps the four K groups on distinct banks
    constexpr int WAVES = RES_THREADS / 64;
    extern __shared__ float wt[];
    const int lane = (int)(threadIdx.x & 63u);
    const int wave = (int)(threadIdx.x >> 6);
    const int i = lane & 15, kq = lane >> 4;
    const int c0 = (int)blockIdx.y * (NB * 16);
    const int ngroups = (a.d1 + 63) >> 6;
    const int ngg = FULL ? 4 : (a.d1 + 15) >> 4;
    const float *w = static_cast<const float *>(a.w);
    for (int idx = (int)threadIdx.x; idx < ngroups * 64 * NB * 16; idx += RES_THREADS) {
        const int r = idx / (NB * 16), j = idx % (NB * 16);
        const int k = lds_row_k<FULL>(r, ngroups, a.d1);
        wt[r * RS + j] = (k >= 0 && c0 + j < a.d2) ? w[(long long)k * a.d2 + c0 + j] : 0.f;
    }
    __syncthreads();

    // One flat loop over (tile, K group): the loads of the next item are issued first and may not sink below the
    // scheduling barrier, so they fly while the matrix cores work on the current item.
    const long long tiles = (a.n + 15) / 16;
    const long long stride = (long long)gridDim.x * WAVES;
    long long tile = (long long)blockIdx.x * WAVES + wave;
    if (tile >= tiles) return;
    const float *x = static_cast<const float *>(a.x);
    float xv[4][4], xn[4][4];
    float scale = 1.0f, scale_next = 1.0f;
    {
        const long long row = min(tile * 16 + i, a.n - 1);
        load_group<KMODE>(xv, x + row * a.ld_x, 0, ngroups, a.d1, kq);
        if (a.rs) scale = a.rs[row];
        arrived(xv, scale);
    }
    v4f acc[NB];
    int g = 0;
    for (;;) {
        const bool last_g = g + 1 == ngroups;
        const long long ntile = last_g ? tile + stride : tile;
        const int ng = last_g ? 0 : g + 1;
        {
            const long long nrow = min(ntile * 16 + i, a.n - 1);
            load_group<KMODE>(xn, x + nrow * a.ld_x, ng, ngroups, a.d1, kq);
            scale_next = scale;
            if (last_g && a.rs) scale_next = a.rs[nrow];
        }
        __builtin_amdgcn_sched_barrier(0);
        if (g == 0) {
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) acc[nb] = (v4f){0.f, 0.f, 0.f, 0.f};
        }
        mfma_group<NB, RS>(acc, wt + g * 64 * RS, xv, i, kq, ngg);
        __builtin_amdgcn_sched_barrier(0);  // (not hoisted into the matrix-core work above)
        arrived(xn, scale_next);    // before the stores
        if (last_g) {
            const long long row = tile * 16 + i;
            store_rows<NB, false>(a.out, a.ld_out, a.d2, scale, a.relu, a.vec_out, acc, row, row < a.n, c0, kq);
        }
#pragma unroll
        for (int gg = 0; gg < 4; ++gg)
#pragma unroll
            for (int t = 0; t < 4; ++t) xv[gg][t] = xn[gg][t];
        scale = scale_next;
        tile = ntile;
        g = ng;
        if (tile >= tiles) break;
    }
}

// Narrow updates (d2 <= 16) of densely packed rows that are not whole cache lines (602 floats = 2,408 bytes): read row by
// row, every 64-float piece of a row straddles three lines and the lines are fetched more than once.  Here a tile of 16
// rows is read as what it is in memory, one contiguous run of 16 d1 floats starting on a 64-byte boundary: the 512
// threads of the workgroup load it 8 KB per instruction with the streaming hint and lay it down flat in LDS.  K is cut
// into 8 slices, one per wavefront, so a wavefront keeps its slice of W in SW registers for the whole launch (lane
// (column i, kq) holds W[KW w + 4 s + kq][i], s < SW) and reads its slice of the tile with 4-byte LDS reads in which
// the four kq of a row are neighbors (two lanes per bank for every d1 that is not a multiple of 8); the 8 partial
// tiles (16 x 16) meet in LDS and wavefront 0 stores the tile.  The loads of the next tile are in flight in registers
// while this one is multiplied, so one LDS buffer is enough: 49 KB per workgroup at d1 = 602, three workgroups per CU
// (80 registers).  A workgroup takes FLAT_TILES consecutive tiles and ends: short-lived workgroups in launch order keep
// the chip inside a narrow moving window of the array (233,000 x 602 -> 16, ms: 2 tiles 0.120, 3 0.108, 4 0.106, 6 0.110,
// 8 0.112, 16 0.116; as many long-lived workgroups as fit, equal contiguous shares: 0.109; W costs every workgroup
// 38 KB of L2 reads).
constexpr int FLAT_WAVES = 8;
constexpr int FLAT_THREADS = FLAT_WAVES * 64;
constexpr int FLAT_TILES = 4;  // consecutive tiles per workgroup
// LDS floats of the tile: the 16 rows and what the last wavefront's K slice reads past them (masked), and never less than
// the whole rounds of 16-byte pieces the workgroup lays down
inline __host__ __device__ int flat_tile_floats(int d1, int sw)
{
    const int need = (16 * d1 + FLAT_WAVES * 4 * sw + 3) & ~3, laid = 4 * FLAT_WAVES * 64 * (sw / 4);
    return need > laid ? need : laid;
}

template <int SW>
__global__ void __launch_bounds__(FLAT_THREADS, SW <= 20 ? 6 : 4) k_dense_xw_flat(const DenseArgs a)
{
    constexpr int NL = SW / 4;   // 16-byte loads per thread and tile: 16 d1 floats <= 512 SW floats = NL x 512 x 4
    constexpr int KW = 4 * SW;   // K values per wavefront
    static_assert(SW % 4 == 0, "whole rounds of loads");
    extern __shared__ __align__(16) float lds_flat[];
    const int tid = (int)threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int i = lane & 15, kq = lane >> 4;
    const int d1 = a.d1;
    float *xt = lds_flat;
    float *red = lds_flat + flat_tile_floats(d1, SW);
    const float *x = static_cast<const float *>(a.x);
    const float *w = static_cast<const float *>(a.w);
    const long long tiles = (a.n + 15) / 16;
    const long long tile0 = (long long)blockIdx.x * a.tiles_per_wave;
    const long long tile_end = min(tiles, tile0 + a.tiles_per_wave);
    if (tile0 >= tiles) return;
    // First row of a tile.  The last tile of an array whose rows are no multiple of 16 is the last 16 rows: it overlaps the
    // tile before it (those rows are computed and stored twice, the same values) and may start off a 16-byte boundary.
    const auto first_row = [&](long long tile) { return min(tile * 16, a.n - 16); };

    typedef float v4f_any __attribute__((ext_vector_type(4), aligned(4)));
    v4f xr[NL];
    const auto issue = [&](long long tile) {
        const char *src = reinterpret_cast<const char *>(x + first_row(tile) * d1);
#pragma unroll
        for (int j = 0; j < NL; ++j) {  // uniform base + unsigned 32-bit lane offset: one register per load for the address
            const unsigned f = 4u * (unsigned)(j * FLAT_THREADS + tid);
            xr[j] = __builtin_nontemporal_load(reinterpret_cast<const v4f_any *>(src + 4u * min(f, (unsigned)(16 * d1 - 4))));
        }
    };
    const auto lay_down = [&]() {
#pragma unroll
        for (int j = 0; j < NL; ++j)
            *reinterpret_cast<v4f *>(xt + 4 * (j * FLAT_THREADS + tid)) = xr[j];  // past the tile: copies nobody reads
    };

    // The first tile and this wavefront's slice of W, all loads in flight together; every one of them has arrived before
    // the loop below starts (a wait for W inside the loop would also wait for the next tile's loads, issued just before).
    issue(tile0);
    float wreg[SW];
    const int kbase = KW * wave + kq;
#pragma unroll
    for (int s = 0; s < SW; ++s) wreg[s] = w[min(kbase + 4 * s, d1 - 1) * a.d2 + min(i, a.d2 - 1)];
#pragma unroll
    for (int s = 0; s < SW; ++s) {
        // (the empty statement keeps the compiler from moving each load under the condition below, a branch and a wait per
        // load)
        asm volatile("" : "+v"(wreg[s]));
        wreg[s] = (kbase + 4 * s < d1 && i < a.d2) ? wreg[s] : 0.f;
    }
    lay_down();
    __syncthreads();

    const float *xrow = xt + i * d1 + kbase;
    // MORE: another tile follows; its loads are issued first.  (Two instantiations instead of a branch, so that every wait
    // inside counts exactly the loads that were issued before it.)
    const auto one_tile = [&](long long tile, auto more_c) {
        constexpr bool MORE = decltype(more_c)::value;
        const long long row = first_row(tile) + i;
        float scale = 1.0f;  // asked for before the next tile: waiting for it later does not wait for the tile
        if (wave == 0 && a.rs) scale = a.rs[row];
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (MORE) issue(tile + 1);
        __builtin_amdgcn_sched_barrier(0);
        v4f acc = (v4f){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < SW; ++s) {
            const float xv = xrow[4 * s];
            acc = __builtin_amdgcn_mfma_f32_16x16x4f32(wreg[s], kbase + 4 * s < d1 ? xv : 0.f, acc, 0, 0, 0);
            if (s % 4 == 3) __builtin_amdgcn_sched_barrier(0);  // at most four LDS values waiting
        }
        *reinterpret_cast<v4f *>(red + (wave * 64 + lane) * 4) = acc;
        __syncthreads();
        if (wave == 0) {
            v4f sum[1];
            sum[0] = *reinterpret_cast<const v4f *>(red + lane * 4);
#pragma unroll
            for (int ww = 1; ww < FLAT_WAVES; ++ww) sum[0] += *reinterpret_cast<const v4f *>(red + (ww * 64 + lane) * 4);
            store_rows<1, false>(a.out, a.ld_out, a.d2, scale, a.relu, a.vec_out, sum, row, true, 0, kq);
        }
        if constexpr (MORE) lay_down();
        __syncthreads();
    };
    for (long long tile = tile0; tile + 1 < tile_end; ++tile) one_tile(tile, std::true_type{});
    one_tile(tile_end - 1, std::false_type{});
}

// Two updates in one pass, Out = act(X . Wa) . Wb, both weight matrices resident in LDS (h <= 64, d3 <= 64).
// The transposed first product leaves lane L with T[row L % 16][16 nb + 4 (L / 16) + r], r = 0..3: four consecutive
// K values of one row of the intermediate, which is exactly the operand the second product wants.  The
// intermediate never leaves the registers.
struct MlpArgs {
    float *out;
    const float *x, *wa, *wb, *rs;
    long long n, ld_x, ld_out;
    int d1, h, d3;
    int relu_mid, relu_out, vec_out, stream_x;  // relu_out: 0 none, 1 ReLU, 2 row softmax
    int flat_out;  // k_mlp2_split: packed rows that are no multiple of 16 bytes leave as whole tiles (store_tile_flat)
};

template <int NB1, int NB2, int KMODE>
__global__ void __launch_bounds__(RES_THREADS, 4) k_mlp2_resident(const MlpArgs a)
{
    constexpr bool FULL = KMODE >= 1;
    constexpr int RS1 = NB1 * 16 + 4, RS2 = NB2 * 16 + 4;
    constexpr int WAVES = RES_THREADS / 64;
    extern __shared__ float wt[];
    const int lane = (int)(threadIdx.x & 63u);
    const int wave = (int)(threadIdx.x >> 6);
    const int i = lane & 15, kq = lane >> 4;
    const int ngroups = (a.d1 + 63) >> 6;
    const int ngg = FULL ? 4 : (a.d1 + 15) >> 4;
    float *wta = wt, *wtb = wt + ngroups * 64 * RS1;
    for (int idx = (int)threadIdx.x; idx < ngroups * 64 * NB1 * 16; idx += RES_THREADS) {
        const int r = idx / (NB1 * 16), j = idx % (NB1 * 16);
        const int k = lds_row_k<FULL>(r, ngroups, a.d1);
        wta[r * RS1 + j] = (k >= 0 && j < a.h) ? a.wa[(long long)k * a.h + j] : 0.f;
    }
    for (int idx = (int)threadIdx.x; idx < NB1 * 16 * NB2 * 16; idx += RES_THREADS) {
        const int k = idx / (NB2 * 16), j = idx % (NB2 * 16);
        wtb[k * RS2 + j] = (k < a.h && j < a.d3) ? a.wb[(long long)k * a.d3 + j] : 0.f;
    }
    __syncthreads();

    const long long tiles = (a.n + 15) / 16;
    const long long stride = (long long)gridDim.x * WAVES;
    long long tile = (long long)blockIdx.x * WAVES + wave;
    if (tile >= tiles) return;
    float xv[4][4], xn[4][4];
    float scale = 1.0f, scale_next = 1.0f;
    {
        const long long row = min(tile * 16 + i, a.n - 1);
        load_group<KMODE>(xv, a.x + row * a.ld_x, 0, ngroups, a.d1, kq);
        if (a.rs) scale = a.rs[row];
        arrived(xv, scale);
    }
    v4f acc1[NB1];
    int g = 0;
    for (;;) {
        const bool last_g = g + 1 == ngroups;
        const long long ntile = last_g ? tile + stride : tile;
        const int ng = last_g ? 0 : g + 1;
        {
            const long long nrow = min(ntile * 16 + i, a.n - 1);
            load_group<KMODE>(xn, a.x + nrow * a.ld_x, ng, ngroups, a.d1, kq);
            scale_next = scale;
            if (last_g && a.rs) scale_next = a.rs[nrow];
        }
        __builtin_amdgcn_sched_barrier(0);
        if (g == 0) {
#pragma unroll
            for (int nb = 0; nb < NB1; ++nb) acc1[nb] = (v4f){0.f, 0.f, 0.f, 0.f};
        }
        mfma_group<NB1, RS1>(acc1, wta + g * 64 * RS1, xv, i, kq, ngg);
        __builtin_amdgcn_sched_barrier(0);  // (not hoisted into the matrix-core work above)
        arrived(xn, scale_next);    // before the stores
        if (last_g) {
            v4f acc2[NB2];
#pragma unroll
            for (int nb = 0; nb < NB2; ++nb) acc2[nb] = (v4f){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int nb = 0; nb < NB1; ++nb) {
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    float tv = acc1[nb][t];
                    if (a.relu_mid) tv = fmaxf(tv, 0.f);
                    const float *wrow = wtb + (16 * nb + 4 * kq + t) * RS2 + i;
#pragma unroll
                    for (int nb2 = 0; nb2 < NB2; ++nb2)
                        acc2[nb2] = __builtin_amdgcn_mfma_f32_16x16x4f32(wrow[nb2 * 16], tv, acc2[nb2], 0, 0, 0);
                }
            }
            const long long row = tile * 16 + i;
            if (a.relu_out == 2) {  // row softmax of the (scaled) result instead of ReLU
                tile_row_softmax<NB2>(acc2, scale, a.d3, kq);
                store_rows<NB2, false>(a.out, a.ld_out, a.d3, 1.0f, 0, a.vec_out, acc2, row, row < a.n, 0, kq);
            } else {
                store_rows<NB2, false>(a.out, a.ld_out, a.d3, scale, a.relu_out, a.vec_out, acc2, row, row < a.n, 0, kq);
            }
        }
#pragma unroll
        for (int gg = 0; gg < 4; ++gg)
#pragma unroll
            for (int t = 0; t < 4; ++t) xv[gg][t] = xn[gg][t];
        scale = scale_next;
        tile = ntile;
        g = ng;
        if (tile >= tiles) break;
    }
}

// The same two-layer update, 64 -> 64 -> d3 (33 ... 64), on the bf16 matrix cores with fp32 results: every fp32 operand is
// split exactly into three bf16 parts, x = x1 + x2 + x3 (x1 = bf16(x), x2 = bf16(x - x1), x3 = bf16(x - x1 - x2): 24
// mantissa bits, the subtractions are exact), and a product x w becomes the six bf16 products that matter,
// x1 w1 + (x1 w2 + x2 w1) + (x1 w3 + x2 w2 + x3 w1) -- each exact in the fp32 accumulator, what is dropped is below
// 2^-24 of |x w|.  Six v_mfma_f32_16x16x32_bf16 do the work of eight v_mfma_f32_16x16x4_f32 at a sixteenth of the
// cycles each, so the kernel that the fp32 matrix cores held at 68 % busy becomes bound by memory.
// Layout as in k_mlp2_resident (transposed products; lane (i, kb) = (L % 16, L / 16)): the first product leaves the lane
// with T[row i][16 nb + 4 kb + r], r = 0..3; the second wants eight K values per lane and step, and takes for step s the
// columns {16 (2 s) + 4 kb + r} and {16 (2 s + 1) + 4 kb + r} -- Wb is staged with its K order permuted to match
// (split_k_slot), so the intermediate never leaves the registers.
// LDS: the three parts of Wa^T and of Wb^T, [part][column][72] bf16 (rows of 144 bytes: 16-byte reads, staggered banks).
constexpr int SPLIT_KP = 64 + 8;

// The three bf16 parts of two floats, packed in pairs (low half = first value).
__device__ __forceinline__ void split_pair(float a, float b, unsigned &hi, unsigned &mid, unsigned &lo)
{
    const auto pack = [](float x, float y) {
        const v2bf q = __builtin_convertvector((v2f){x, y}, v2bf);
        unsigned u;
        __builtin_memcpy(&u, &q, 4);
        return u;
    };
    hi = pack(a, b);
    float ra = a - __uint_as_float(hi << 16), rb = b - __uint_as_float(hi & 0xFFFF0000u);
    mid = pack(ra, rb);
    ra -= __uint_as_float(mid << 16);
    rb -= __uint_as_float(mid & 0xFFFF0000u);
    lo = pack(ra, rb);
}
__device__ __forceinline__ void split8(const float (&x)[8], v8bf &hi, v8bf &mid, v8bf &lo)
{
    unsigned h[4], m[4], l[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) split_pair(x[2 * t], x[2 * t + 1], h[t], m[t], l[t]);
    __builtin_memcpy(&hi, h, 16);
    __builtin_memcpy(&mid, m, 16);
    __builtin_memcpy(&lo, l, 16);
}
// position in a staged row of Wb^T of the K index k (see above): step k / 32, lane group (k / 4) % 4, slot 4 ((k / 16) % 2) + k % 4
__device__ __forceinline__ int split_k_slot(int k) { return 32 * (k >> 5) + 8 * ((k >> 2) & 3) + 4 * ((k >> 4) & 1) + (k & 3); }

template <int NB2>
__global__ void __launch_bounds__(RES_THREADS, 4) k_mlp2_split(const MlpArgs a)
{
    constexpr int NB1 = 4, KP = SPLIT_KP, WAVES = RES_THREADS / 64;
    constexpr int PART_A = NB1 * 16 * KP, PART_B = NB2 * 16 * KP;  // bf16 elements per part
    extern __shared__ __align__(16) float lds_raw[];
    unsigned short *wa = reinterpret_cast<unsigned short *>(lds_raw), *wb = wa + 3 * PART_A;
    const int lane = (int)(threadIdx.x & 63u), wave = (int)(threadIdx.x >> 6);
    const int i = lane & 15, kb = lane >> 4;
    // The weights, split and transposed, once per (persistent) workgroup.  Short-lived workgroups in launch order with the
    // weights copied from a prepared image were measured too (as in k_dense_xw_bf16_lines): 0.32-0.34 ms against 0.31 --
    // this kernel reads X in the operand layout and stores 64-byte pieces, and without whole-line traffic the launch order
    // buys nothing.  Whole rows through LDS (16 wavefronts, one workgroup per CU) were measured as well: 0.304 against
    // 0.308 ms at 64 columns out, 0.394 against 0.374 at 47 -- memory is not what holds this kernel; per 16-row tile it
    // issues 96 matrix-core instructions, 48 16-byte LDS reads of weights and some 260 vector instructions of splitting.
    for (int idx = (int)threadIdx.x; idx < 64 * 64; idx += RES_THREADS) {
        const int k = idx >> 6, c = idx & 63;
        unsigned h, m, l;
        split_pair(a.wa[(long long)k * 64 + c], 0.f, h, m, l);
        wa[c * KP + k] = (unsigned short)h;
        wa[PART_A + c * KP + k] = (unsigned short)m;
        wa[2 * PART_A + c * KP + k] = (unsigned short)l;
    }
    for (int idx = (int)threadIdx.x; idx < 64 * NB2 * 16; idx += RES_THREADS) {
        const int k = idx / (NB2 * 16), c = idx % (NB2 * 16);
        unsigned h, m, l;
        split_pair(c < a.d3 ? a.wb[(long long)k * a.d3 + c] : 0.f, 0.f, h, m, l);
        const int at = c * KP + split_k_slot(k);
        wb[at] = (unsigned short)h;
        wb[PART_B + at] = (unsigned short)m;
        wb[2 * PART_B + at] = (unsigned short)l;
    }
    __syncthreads();
    const __bf16 *wab = reinterpret_cast<const __bf16 *>(wa), *wbb = reinterpret_cast<const __bf16 *>(wb);

    const long long tiles = (a.n + 15) / 16;
    const long long stride = (long long)gridDim.x * WAVES;
    long long tile = (long long)blockIdx.x * WAVES + wave;
    if (tile >= tiles) return;
    typedef float v4f_x __attribute__((ext_vector_type(4), aligned(16)));
    v4f_x xn[4];  // the lane's 8 floats of K step 0 and of K step 1
    const auto issue = [&](long long t) {
        const float *xrow = a.x + min(t * 16 + i, a.n - 1) * a.ld_x + 8 * kb;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            xn[2 * ks] = *reinterpret_cast<const v4f_x *>(xrow + 32 * ks);
            xn[2 * ks + 1] = *reinterpret_cast<const v4f_x *>(xrow + 32 * ks + 4);
        }
    };
    issue(tile);
    float scale = a.rs ? a.rs[min(tile * 16 + i, a.n - 1)] : 1.0f;
    asm volatile("" : "+v"(xn[0]), "+v"(xn[1]), "+v"(xn[2]), "+v"(xn[3]), "+v"(scale));  // waited for here, not at the head of the loop (see its end)
    const float floor_mid = a.relu_mid ? 0.f : -3.4e38f;  // ReLU between the layers as one max per value
    // acc += the six products of a split operand pair, smallest first
    const auto six = [](v4f acc, const v8bf (&w)[3], const v8bf (&x)[3]) {
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[2], x[0], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[1], x[1], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[0], x[2], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[1], x[0], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[0], x[1], acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[0], x[0], acc, 0, 0, 0);
        return acc;
    };
    for (;;) {
        v8bf xs[2][3];
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const float x8[8] = {xn[2 * ks][0], xn[2 * ks][1], xn[2 * ks][2], xn[2 * ks][3], xn[2 * ks + 1][0], xn[2 * ks + 1][1], xn[2 * ks + 1][2], xn[2 * ks + 1][3]};
            split8(x8, xs[ks][0], xs[ks][1], xs[ks][2]);
        }
        const long long ntile = tile + stride;
        const bool more = ntile < tiles;
        float scale_next = 1.0f;
        if (more) {  // wavefront-uniform
            issue(ntile);
            if (a.rs) scale_next = a.rs[min(ntile * 16 + i, a.n - 1)];
        }
        __builtin_amdgcn_sched_barrier(0);
        v4f acc1[NB1];
#pragma unroll
        for (int nb = 0; nb < NB1; ++nb) acc1[nb] = (v4f){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
            for (int nb = 0; nb < NB1; ++nb) {
                v8bf w3[3];
#pragma unroll
                for (int p = 0; p < 3; ++p) w3[p] = *reinterpret_cast<const v8bf *>(wab + p * PART_A + (16 * nb + i) * KP + 32 * ks + 8 * kb);
                acc1[nb] = six(acc1[nb], w3, xs[ks]);
            }
        }
        v4f acc2[NB2];
#pragma unroll
        for (int nb = 0; nb < NB2; ++nb) acc2[nb] = (v4f){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int st = 0; st < 2; ++st) {
            float t8[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                t8[e] = fmaxf(acc1[2 * st + (e >> 2)][e & 3], floor_mid);
            }
            v8bf ts[3];
            split8(t8, ts[0], ts[1], ts[2]);
#pragma unroll
            for (int nb = 0; nb < NB2; ++nb) {
                v8bf w3[3];
#pragma unroll
                for (int p = 0; p < 3; ++p) w3[p] = *reinterpret_cast<const v8bf *>(wbb + p * PART_B + (16 * nb + i) * KP + 32 * st + 8 * kb);
                acc2[nb] = six(acc2[nb], w3, ts);
            }
        }
        // The next tile's loads are waited for here, before this tile's stores are issued: the counter the wait uses
        // counts loads and stores alike, in order, so a wait placed after the stores would sit until they are acknowledged.
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("" : "+v"(xn[0]), "+v"(xn[1]), "+v"(xn[2]), "+v"(xn[3]), "+v"(scale_next));
        const long long row = tile * 16 + i;
        if (a.flat_out) {
            if (a.relu_out == 2) {
                tile_row_softmax<NB2>(acc2, scale, a.d3, kb);
            } else {
#pragma unroll
                for (int nb = 0; nb < NB2; ++nb)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        acc2[nb][r] *= scale;
                        if (a.relu_out) acc2[nb][r] = fmaxf(acc2[nb][r], 0.f);
                    }
            }
            store_tile_flat<NB2>(a.out, reinterpret_cast<float *>(wb + 3 * PART_B) + wave * (16 * NB2 * 16), a.d3, a.n, acc2, tile, i, kb, lane);
        } else if (a.relu_out == 2) {  // row softmax of the (scaled) result instead of ReLU
            tile_row_softmax<NB2>(acc2, scale, a.d3, kb);
            store_rows<NB2, false>(a.out, a.ld_out, a.d3, 1.0f, 0, a.vec_out, acc2, row, row < a.n, 0, kb);
        } else {
            store_rows<NB2, false>(a.out, a.ld_out, a.d3, scale, a.relu_out, a.vec_out, acc2, row, row < a.n, 0, kb);
        }
        if (!more) break;
        tile = ntile;
        scale = scale_next;
    }
}

// W staged in K chunks (any d1): fallback when W does not fit in LDS.
template <int NB>
__global__ void __launch_bounds__(256) k_dense_xw(const DenseArgs a)
{
    constexpr int RS = NB * 16 + 4;
    __shared__ float wt[GEMM_KC * RS];
    const int lane = (int)(threadIdx.x & 63u);
    const int wave = (int)(threadIdx.x >> 6);
    const int i = lane & 15, kq = lane >> 4;
    const long long row = (long long)blockIdx.x * GEMM_ROWS_WG + wave * 16 + i;
    const int c0 = (int)blockIdx.y * (NB * 16);
    const bool row_ok = row < a.n;
    const float *xrow = static_cast<const float *>(a.x) + (row_ok ? row : 0) * a.ld_x;
    const float *w = static_cast<const float *>(a.w);

    v4f acc[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[nb] = (v4f){0.f, 0.f, 0.f, 0.f};

    for (int k0 = 0; k0 < a.d1; k0 += GEMM_KC) {
        __syncthreads();
        for (int idx = (int)threadIdx.x; idx < GEMM_KC * NB * 16; idx += 256) {
            const int k = idx / (NB * 16), j = idx % (NB * 16);
            float v = 0.f;
            if (k0 + k < a.d1 && c0 + j < a.d2) v = w[(long long)(k0 + k) * a.d2 + c0 + j];
            wt[k * RS + j] = v;
        }
        __syncthreads();
#pragma unroll
        for (int ks = 0; ks < GEMM_KC / 16; ++ks) {
            float xv[4];
            load_x4(xv, xrow, k0 + ks * 16 + 4 * kq, a.d1, row_ok);
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const float *wrow = wt + (ks * 16 + 4 * kq + t) * RS + i;
#pragma unroll
                for (int nb = 0; nb < NB; ++nb)
                    acc[nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(xv[t], wrow[nb * 16], acc[nb], 0, 0, 0);
            }
        }
    }
    store_tile_f32<NB>(a, acc, (long long)blockIdx.x * GEMM_ROWS_WG + wave * 16 + 4 * kq, c0, i);
}

// bf16 matrix cores: v_mfma_f32_16x16x32_bf16 (wave64)
//   A (16 x 32): lane L holds A[L % 16][8 * (L / 16) .. + 8)
//   B (32 x 16): lane L holds B[8 * (L / 16) .. + 8)[L % 16]
//   D (16 x 16): lane L holds D[4 * (L / 16) + r][L % 16], r = 0..3
// W (bf16, [d1][d2]) is kept transposed in LDS, Wt[column][k], so a lane's 8 K values are one 16-byte read.
// X is fp32 (rounded to bf16, nearest even, on the fly) or bf16; the accumulator and the epilogue are fp32; the
// output is fp32 or bf16.
// 8 consecutive K values of one row as bf16, branch-free; `mode` as in load_x4u with chunks of 8 (wavefront-uniform).
template <bool X_F32>
__device__ __forceinline__ v8bf load_x8_bf16(const void *xbase, long long row, long long ld_x, int k, int d1, int mode)
{
    v8bf av;
    if constexpr (X_F32) {
        const float *xrow = static_cast<const float *>(xbase) + row * ld_x;
        float f[8];
        if (mode <= 1) {
            const int kc = mode == 0 ? k : min(k, d1 - 8);
            float4 t0, t1;
            __builtin_memcpy(&t0, xrow + kc, 16);
            __builtin_memcpy(&t1, xrow + kc + 4, 16);
            f[0] = t0.x; f[1] = t0.y; f[2] = t0.z; f[3] = t0.w;
            f[4] = t1.x; f[5] = t1.y; f[6] = t1.z; f[7] = t1.w;
            if (mode == 1) {
                const bool in = k < d1;
#pragma unroll
                for (int t = 0; t < 8; ++t) f[t] = in ? f[t] : 0.f;
            }
        } else {
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const float v = xrow[min(k + t, d1 - 1)];
                f[t] = k + t < d1 ? v : 0.f;
            }
        }
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const v2bf p = __builtin_convertvector((v2f){f[2 * t], f[2 * t + 1]}, v2bf);
            av[2 * t] = p[0];
            av[2 * t + 1] = p[1];
        }
    } else {
        const unsigned short *xrow = static_cast<const unsigned short *>(xbase) + row * ld_x;
        unsigned short h[8];
        if (mode <= 1) {
            __builtin_memcpy(h, xrow + (mode == 0 ? k : min(k, d1 - 8)), 16);
            if (mode == 1) {
                const bool in = k < d1;
#pragma unroll
                for (int t = 0; t < 8; ++t) h[t] = in ? h[t] : (unsigned short)0;
            }
        } else {
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                const unsigned short v = xrow[min(k + t, d1 - 1)];
                h[t] = k + t < d1 ? v : (unsigned short)0;
            }
        }
        __builtin_memcpy(&av, h, 16);
    }
    return av;
}

// Like the fp32 kernels the product is formed transposed (W as the A operand), so a lane ends up with four
// consecutive columns of one output row; X is read one K step (32 values per row) ahead, across tile boundaries.
template <int NB, bool X_F32, bool OUT_BF16>
__global__ void __launch_bounds__(256) k_dense_xw_bf16(const DenseArgs a)
{
    extern __shared__ __align__(16) float lds_raw[];
    __bf16 *wt = reinterpret_cast<__bf16 *>(lds_raw);
    const int lane = (int)(threadIdx.x & 63u);
    const int wave = (int)(threadIdx.x >> 6);
    const int i = lane & 15, kb = lane >> 4;
    const int c0 = (int)blockIdx.y * (NB * 16);
    const int d1p = (a.d1 + 31) & ~31;
    const int KP = d1p + 8;  // row stride of Wt in bf16: the +8 (16 bytes) staggers rows over the banks
    const unsigned short *w = static_cast<const unsigned short *>(a.w);
    unsigned short *wts = reinterpret_cast<unsigned short *>(wt);
    // bf16 output in whole 16-byte pieces (all NB blocks inside d2, rows of out on 16-byte boundaries): columns staged pairwise
    // interleaved, so a lane ends up with eight consecutive columns (store_rows_bf16_paired)
    const bool paired = OUT_BF16 && NB % 2 == 0 && (a.vec_out & 4) != 0 && c0 + NB * 16 <= a.d2;
    for (int idx = (int)threadIdx.x; idx < d1p * NB * 16; idx += 256) {
        const int k = idx / (NB * 16), j = idx % (NB * 16);
        const int col = c0 + (paired ? paired_column(j) : j);
        wts[j * KP + k] = (k < a.d1 && col < a.d2) ? w[(long long)k * a.d2 + col] : (unsigned short)0;
    }
    __syncthreads();

    const long long tiles = (a.n + 15) / 16;
    const long long stride = (long long)gridDim.x * 4;
    long long tile = (long long)blockIdx.x * 4 + wave;
    if (tile >= tiles) return;
    float scale = 1.0f, scale_next = 1.0f;
    v8bf av;
    {
        const long long row = min(tile * 16 + i, a.n - 1);
        av = load_x8_bf16<X_F32>(a.x, row, a.ld_x, 8 * kb, a.d1, x_group_mode(0, 32, a.d1, 8));
        if (a.rs) scale = a.rs[row];
        asm volatile("" : "+v"(av), "+v"(scale));  // as arrived()
    }
    v4f acc[NB];
    int k0 = 0;
    for (;;) {  // flat loop over (tile, K step of 32); the next step's X is in flight during the MFMAs
        const bool last_k = k0 + 32 >= d1p;
        const long long ntile = last_k ? tile + stride : tile;
        const int nk = last_k ? 0 : k0 + 32;
        const long long nrow = min(ntile * 16 + i, a.n - 1);
        v8bf an = load_x8_bf16<X_F32>(a.x, nrow, a.ld_x, nk + 8 * kb, a.d1, x_group_mode(nk, 32, a.d1, 8));
        scale_next = scale;
        if (last_k && a.rs) scale_next = a.rs[nrow];
        __builtin_amdgcn_sched_barrier(0);
        if (k0 == 0) {
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) acc[nb] = (v4f){0.f, 0.f, 0.f, 0.f};
        }
        const int k = k0 + 8 * kb;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            v8bf bv;
            bv = *reinterpret_cast<const v8bf *>(wt + (size_t)(nb * 16 + i) * KP + k);  // one 16-byte LDS read (rows of Wt are 16-byte multiples)
            acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bv, av, acc[nb], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("" : "+v"(an), "+v"(scale_next));  // as arrived(): before the stores
        if (last_k) {
            const long long row = tile * 16 + i;
            if constexpr (OUT_BF16 && NB % 2 == 0) {
                if (paired) store_rows_bf16_paired<NB>(a.out, a.ld_out, scale, a.relu, acc, row, row < a.n, c0, kb);
                else store_rows<NB, OUT_BF16>(a.out, a.ld_out, a.d2, scale, a.relu, a.vec_out, acc, row, row < a.n, c0, kb);
            } else {
                store_rows<NB, OUT_BF16>(a.out, a.ld_out, a.d2, scale, a.relu, a.vec_out, acc, row, row < a.n, c0, kb);
            }
        }
        av = an;
        scale = scale_next;
        tile = ntile;
        k0 = nk;
        if (tile >= tiles) break;
    }
}

// The same product for fp32 X and bf16 output with every access to memory in whole lines: a wavefront reads the 16 rows of
// its tile as they lie in memory (a row's bytes on neighbouring lanes, streaming hint), rounds them to bf16 into its own
// piece of LDS, and the matrix cores take their operand layout from there; the finished tile goes back through the same
// piece of LDS and leaves as whole rows too.  The operand layout read straight from memory touches a quarter of a line per
// lane and the memory system answers it at 5.4-5.9 TB/s where it answers whole lines at 6.8-7.0 (13.9 M rows of 128 -> 128:
// 2.03 ms with the operand layout and a persistent grid, 1.85 with this kernel).  The next tile's rows are in flight while the current one is
// converted, multiplied and stored.  D1 in {64, 128}, all NB * 16 columns of W, rows of X and of the output on 16-byte
// boundaries.
constexpr int LINES_WAVES = 8;
constexpr int WT_IMAGE_MAX = 128 * (128 + 8);  // bf16 elements

// image[j * (d1 + 8) + k] = W[k][paired_column(j)]: W transposed with its columns in the order the paired 16-byte stores
// want, as the workgroups of k_dense_xw_bf16_lines copy it into LDS
__global__ void __launch_bounds__(256) k_wt_image(unsigned short *__restrict__ image, const unsigned short *__restrict__ w, int d1, int d2)
{
    const int idx = (int)(blockIdx.x * 256 + threadIdx.x);
    if (idx >= d1 * d2) return;
    const int k = idx / d2, c = idx % d2;  // reads along rows of W
    // slot j with paired_column(j) == c
    const int p = c >> 5, q = c & 31, kq = q >> 3, h = (q >> 2) & 1, m = q & 3;
    const int j = 16 * (2 * p + h) + 4 * kq + m;
    image[j * (d1 + 8) + k] = w[idx];
}
template <int NB, int D1>
__global__ void __launch_bounds__(LINES_WAVES * 64) k_dense_xw_bf16_lines(const DenseArgs a)
{
    static_assert(NB % 2 == 0 && (D1 == 64 || D1 == 128), "shapes this variant is written for");
    extern __shared__ __align__(16) float lds_raw[];
    constexpr int D2 = NB * 16;
    constexpr int KP = D1 + 8;                       // row stride of Wt in bf16 (staggers rows over the banks)
    constexpr int XP = D1 * 2 + 16, OP = D2 * 2 + 16;  // bytes per row of a wavefront's X tile / output tile in LDS
    constexpr int TILE_BYTES = 16 * (XP > OP ? XP : OP);
    constexpr int LR = D1 / 4, RPI = 64 / LR, NLD = 16 / RPI;    // lanes per X row, rows per load instruction, loads per tile
    constexpr int LRO = D2 / 8, RPO = 64 / LRO, NST = 16 / RPO;  // the same for the output rows (8 bf16 per lane)
    typedef unsigned v4u_s __attribute__((ext_vector_type(4)));
    typedef unsigned v2u_s __attribute__((ext_vector_type(2)));
    const int lane = (int)(threadIdx.x & 63u), wave = (int)(threadIdx.x >> 6);
    const int i = lane & 15, kb = lane >> 4;
    unsigned short *wts = reinterpret_cast<unsigned short *>(lds_raw);
    const __bf16 *wt = reinterpret_cast<const __bf16 *>(lds_raw);
    char *mine = reinterpret_cast<char *>(lds_raw) + (size_t)D2 * KP * 2 + (size_t)wave * TILE_BYTES;
    // Workgroups are short-lived and take their tiles in launch order -- a.tiles_per_wave rounds of LINES_WAVES
    // consecutive tiles -- so what the whole chip has in flight at any moment is one narrow window of X and of the output
    // moving through memory.  A 2:1 read/write stream converted by one-shot workgroups in launch order runs at
    // 6.1-6.2 TB/s; by workgroups that each walk through 16 / 64 pieces, or stride over the whole array: 5.4 / 5.2.
    // Against that stands what a workgroup pays before its first tile (the copy of W), so: 8 rounds (13.9 M rows of
    // 128 -> 128: 1 / 2 / 4 / 8 / 16 rounds 2.12 / 1.93 / 1.88 / 1.85 / 1.92 ms; a persistent grid striding over all
    // tiles 2.02).
    const long long tiles = (a.n + 15) / 16;
    const long long stride = LINES_WAVES;
    const long long first = (long long)blockIdx.x * LINES_WAVES * a.tiles_per_wave;
    const long long tiles_end = min(tiles, first + (long long)LINES_WAVES * a.tiles_per_wave);
    long long tile = first + wave;
    const bool any_tile = tile < tiles_end;
    if (!any_tile) tile = tiles - 1;  // stays for the barrier below; stores nothing
    const float *x = static_cast<const float *>(a.x);
    const int xr = lane / LR, xc = lane % LR;
    v4f xin[NLD];
    const auto issue = [&](long long t) {
#pragma unroll
        for (int j = 0; j < NLD; ++j) {
            const long long row = min(t * 16 + j * RPI + xr, a.n - 1);
            xin[j] = __builtin_nontemporal_load(reinterpret_cast<const v4f *>(x + row * a.ld_x + 4 * xc));
        }
    };
    issue(tile);  // the first tile's rows are on their way while W is copied
    float scale = a.rs ? a.rs[min(tile * 16 + i, a.n - 1)] : 1.0f;
    {  // a.w: the image k_wt_image made of W (Wt[column slot][k], rows of KP bf16), copied as it lies
        typedef unsigned v4u_c __attribute__((ext_vector_type(4)));
        const v4u_c *src = static_cast<const v4u_c *>(a.w);
        v4u_c *dst = reinterpret_cast<v4u_c *>(lds_raw);
        for (int idx = (int)threadIdx.x; idx < D2 * KP * 2 / 16; idx += LINES_WAVES * 64) dst[idx] = src[idx];
    }
    __syncthreads();

    if (!any_tile) return;
    for (;;) {
#pragma unroll
        for (int j = 0; j < NLD; ++j) {
            const v2bf p0 = __builtin_convertvector((v2f){xin[j][0], xin[j][1]}, v2bf), p1 = __builtin_convertvector((v2f){xin[j][2], xin[j][3]}, v2bf);
            unsigned pk[2];
            __builtin_memcpy(&pk[0], &p0, 4);
            __builtin_memcpy(&pk[1], &p1, 4);
            *reinterpret_cast<v2u_s *>(mine + (j * RPI + xr) * XP + xc * 8) = (v2u_s){pk[0], pk[1]};
        }
        const long long ntile = tile + stride;
        const bool more = ntile < tiles_end;
        float scale_next = 1.0f;
        if (more) {  // wavefront-uniform
            issue(ntile);
            if (a.rs) scale_next = a.rs[min(ntile * 16 + i, a.n - 1)];
        }
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        v4f acc[NB];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) acc[nb] = (v4f){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < D1 / 32; ++ks) {
            v8bf av;
            av = *reinterpret_cast<const v8bf *>(mine + i * XP + (32 * ks + 8 * kb) * 2);
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                v8bf bv;
                bv = *reinterpret_cast<const v8bf *>(wt + (size_t)(nb * 16 + i) * KP + 32 * ks + 8 * kb);
                acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bv, av, acc[nb], 0, 0, 0);
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int p = 0; p < NB / 2; ++p) {
            unsigned pk[4];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                float v[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    v[r] = acc[2 * p + h][r] * scale;
                    if (a.relu) v[r] = fmaxf(v[r], 0.f);
                }
                const v2bf q0 = __builtin_convertvector((v2f){v[0], v[1]}, v2bf), q1 = __builtin_convertvector((v2f){v[2], v[3]}, v2bf);
                __builtin_memcpy(&pk[2 * h], &q0, 4);
                __builtin_memcpy(&pk[2 * h + 1], &q1, 4);
            }
            *reinterpret_cast<v4u_s *>(mine + i * OP + (32 * p + 8 * kb) * 2) = (v4u_s){pk[0], pk[1], pk[2], pk[3]};
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        {
            const int orow = lane / LRO, oc = lane % LRO;
            char *out = static_cast<char *>(a.out);
#pragma unroll
            for (int j = 0; j < NST; ++j) {
                const int r = j * RPO + orow;
                const v4u_s v = *reinterpret_cast<const v4u_s *>(mine + r * OP + oc * 16);
                const long long row = tile * 16 + r;
                if (row < a.n)
                    __builtin_nontemporal_store(v, reinterpret_cast<v4u_s *>(out + (row * a.ld_out) * 2 + oc * 16));
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        if (!more) break;
        tile = ntile;
        scale = scale_next;
    }
}

// Row softmax: G lanes per row (G = power of two <= 64), exp(x - max) / sum.
__global__ void __launch_bounds__(256) k_softmax_rows(float *__restrict__ out, const float *__restrict__ in, long long n, int c,
                                                      long long ld_in, long long ld_out, int G)
{
    const int lane = (int)(threadIdx.x & 63u);
    const int g = lane / G, l = lane % G;
    const int rows_per_wave = 64 / G;
    const long long wave_id = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    const long long row = wave_id * rows_per_wave + g;
    const bool ok = row < n;
    const float *x = in + (ok ? row : 0) * ld_in;
    if (c <= 4 * G) {
        // the whole row lives in registers: one read, one write
        float v[4];
        float m = -INFINITY;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int j = l + t * G;
            v[t] = j < c ? x[j] : -INFINITY;
            m = fmaxf(m, v[t]);
        }
        for (int o = G >> 1; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
        float s = 0.f;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            v[t] = __expf(v[t] - m);  // exp(-inf) = 0 for the padding
            s += v[t];
        }
        for (int o = G >> 1; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
        const float inv = 1.0f / s;
        if (ok) {
            float *o_ = out + row * ld_out;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const int j = l + t * G;
                if (j < c) o_[j] = v[t] * inv;
            }
        }
        return;
    }
    float m = -INFINITY;
    for (int j = l; j < c; j += G) m = fmaxf(m, x[j]);
    for (int o = G >> 1; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
    float s = 0.f;
    for (int j = l; j < c; j += G) s += __expf(x[j] - m);
    for (int o = G >> 1; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
    const float inv = 1.0f / s;
    if (ok) {
        float *o_ = out + row * ld_out;
        for (int j = l; j < c; j += G) o_[j] = __expf(x[j] - m) * inv;
    }
}

// columns are covered in chunks of NB*16; pick the widest chunk that wastes no block
int pick_nb(int d2)
{
    const int blocks16 = (d2 + 15) / 16;
    int nb = blocks16 >= 8 ? 8 : blocks16;
    if (nb == 5) nb = 6;
    if (nb == 7) nb = 8;
    return nb;
}

template <template <int> class Launcher>
int dispatch_nb(int nb, dim3 grid, size_t lds, hipStream_t stream, const DenseArgs &a)
{
    switch (nb) {
        case 1: Launcher<1>::run(grid, lds, stream, a); break;
        case 2: Launcher<2>::run(grid, lds, stream, a); break;
        case 3: Launcher<3>::run(grid, lds, stream, a); break;
        case 4: Launcher<4>::run(grid, lds, stream, a); break;
        case 6: Launcher<6>::run(grid, lds, stream, a); break;
        default: Launcher<8>::run(grid, lds, stream, a); break;
    }
    return MGGX_OK;
}

template <typename K>
void allow_lds(K kernel, size_t lds)
{
    if (lds > 48 * 1024) (void)hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
}

template <int NB>
struct LaunchResident {
    static void run(dim3 grid, size_t lds, hipStream_t s, const DenseArgs &a)
    {
        if (a.d1 >= 64 && a.stream_x) {
            allow_lds(k_dense_xw_resident<NB, 2>, lds);
            k_dense_xw_resident<NB, 2><<<grid, dim3(RES_THREADS), lds, s>>>(a);
        } else if (a.d1 >= 64) {
            allow_lds(k_dense_xw_resident<NB, 1>, lds);
            k_dense_xw_resident<NB, 1><<<grid, dim3(RES_THREADS), lds, s>>>(a);
        } else {
            allow_lds(k_dense_xw_resident<NB, 0>, lds);
            k_dense_xw_resident<NB, 0><<<grid, dim3(RES_THREADS), lds, s>>>(a);
        }
    }
};
template <int NB>
struct LaunchChunked {
    static void run(dim3 grid, size_t, hipStream_t s, const DenseArgs &a) { k_dense_xw<NB><<<grid, dim3(256), 0, s>>>(a); }
};
template <bool X_F32, bool OUT_BF16>
struct LaunchBf16 {
    template <int NB>
    struct L {
        static void run(dim3 grid, size_t lds, hipStream_t s, const DenseArgs &a)
        {
            allow_lds(k_dense_xw_bf16<NB, X_F32, OUT_BF16>, lds);
            k_dense_xw_bf16<NB, X_F32, OUT_BF16><<<grid, dim3(256), lds, s>>>(a);
        }
    };
};

void launch_flat(int sw, dim3 grid, size_t lds, hipStream_t s, const DenseArgs &a)
{
    const auto go = [&](auto kernel) {
        allow_lds(kernel, lds);
        kernel<<<grid, dim3(FLAT_THREADS), lds, s>>>(a);
    };
    switch (sw) {
        case 4: go(k_dense_xw_flat<4>); break;
        case 8: go(k_dense_xw_flat<8>); break;
        case 12: go(k_dense_xw_flat<12>); break;
        case 16: go(k_dense_xw_flat<16>); break;
        case 20: go(k_dense_xw_flat<20>); break;
        default: go(k_dense_xw_flat<24>); break;
    }
}

// persistent grid: enough workgroups to fill the device a few times over, never more than there are 64-row groups
unsigned persistent_blocks(long long n)
{
    const long long groups = (n + 127) / 128;
    const long long want = 256 * 4;
    return (unsigned)(groups < want ? (groups > 0 ? groups : 1) : want);
}

}  // namespace
}  // namespace mggx

using mggx::fail;

MGGX_EXPORT int mggx_dense_xw(float *d_out, const float *d_x, const float *d_w, int64_t n, int d1, int d2,
                              const mggx_dense_opts *opts)
{
    int rc = mggx::ensure_init();
    if (rc) return rc;
    if (n < 0 || d1 < 1 || d2 < 1) return fail(MGGX_EINVAL, "dense_xw: n=%lld d1=%d d2=%d", (long long)n, d1, d2);
    if (n == 0) return MGGX_OK;
    if (!d_out || !d_x || !d_w) return fail(MGGX_EINVAL, "dense_xw: NULL pointer");
    if (d_out == d_x) return fail(MGGX_EINVAL, "dense_xw: in-place update is not supported");
    mggx_dense_opts o{};
    if (opts) o = *opts;
    mggx::DenseArgs a{};
    a.out = d_out;
    a.x = d_x;
    a.w = d_w;
    a.rs = o.d_row_scale;
    a.n = n;
    a.ld_x = o.ld_x ? o.ld_x : d1;
    a.ld_out = o.ld_out ? o.ld_out : d2;
    a.d1 = d1;
    a.d2 = d2;
    a.relu = o.relu != 0;
    a.vec_out = a.ld_out % 4 == 0 && (reinterpret_cast<uintptr_t>(d_out) & 15u) == 0;
    if (d2 % 32 == 0 && a.ld_out % 32 == 0 && (reinterpret_cast<uintptr_t>(d_out) & 127u) == 0) a.vec_out |= 2;
    a.stream_x = d1 % 64 == 0 && a.ld_x % 32 == 0 && (reinterpret_cast<uintptr_t>(d_x) & 127u) == 0;
    if (a.ld_x < d1 || a.ld_out < d2) return fail(MGGX_EINVAL, "dense_xw: row stride smaller than width");
    hipStream_t stream = mggx::state().stream;
    if (d2 <= 16 && a.ld_x == d1 && d1 >= 128 && d1 <= 768 && d1 % 8 != 0 && n >= 4096 &&
        (reinterpret_cast<uintptr_t>(d_x) & 15u) == 0) {
        const int sw = ((d1 + 31) / 32 + 3) & ~3;  // K steps per wavefront, in whole rounds of loads
        const size_t lds_flat = ((size_t)mggx::flat_tile_floats(d1, sw) + mggx::FLAT_WAVES * 256) * sizeof(float);
        a.tiles_per_wave = mggx::FLAT_TILES;
        const long long tiles = (n + 15) / 16;
        const dim3 grid((unsigned)((tiles + a.tiles_per_wave - 1) / a.tiles_per_wave));
        mggx::launch_flat(sw, grid, lds_flat, stream, a);
        MGGX_LAUNCH_CHECK("k_dense_xw_flat");
        return MGGX_OK;
    }
    const int nb = mggx::pick_nb(d2);
    const int gy = ((d2 + 15) / 16 + nb - 1) / nb;
    const size_t lds = (size_t)((d1 + 63) & ~63) * (nb * 16 + 4) * sizeof(float);
    if (lds <= mggx::LDS_RESIDENT_LIMIT) {
        const dim3 grid(mggx::persistent_blocks(n), (unsigned)gy);
        mggx::dispatch_nb<mggx::LaunchResident>(nb, grid, lds, stream, a);
        MGGX_LAUNCH_CHECK("k_dense_xw_resident");
    } else {
        const long long gx = (n + mggx::GEMM_ROWS_WG - 1) / mggx::GEMM_ROWS_WG;
        if (gx > 0x7fffffffLL) return fail(MGGX_ELIMIT, "dense_xw: too many rows");
        mggx::dispatch_nb<mggx::LaunchChunked>(nb, dim3((unsigned)gx, (unsigned)gy), 0, stream, a);
        MGGX_LAUNCH_CHECK("k_dense_xw");
    }
    return MGGX_OK;
}

namespace mggx {
namespace {
template <int NB1, int NB2>
void launch_mlp2(dim3 grid, size_t lds, hipStream_t s, const MlpArgs &a)
{
    if (a.d1 >= 64 && a.stream_x) {
        allow_lds(k_mlp2_resident<NB1, NB2, 2>, lds);
        k_mlp2_resident<NB1, NB2, 2><<<grid, dim3(RES_THREADS), lds, s>>>(a);
    } else if (a.d1 >= 64) {
        allow_lds(k_mlp2_resident<NB1, NB2, 1>, lds);
        k_mlp2_resident<NB1, NB2, 1><<<grid, dim3(RES_THREADS), lds, s>>>(a);
    } else {
        allow_lds(k_mlp2_resident<NB1, NB2, 0>, lds);
        k_mlp2_resident<NB1, NB2, 0><<<grid, dim3(RES_THREADS), lds, s>>>(a);
    }
}
template <int NB1>
void launch_mlp2_nb2(int nb2, dim3 grid, size_t lds, hipStream_t s, const MlpArgs &a)
{
    switch (nb2) {
        case 1: launch_mlp2<NB1, 1>(grid, lds, s, a); break;
        case 2: launch_mlp2<NB1, 2>(grid, lds, s, a); break;
        case 3: launch_mlp2<NB1, 3>(grid, lds, s, a); break;
        default: launch_mlp2<NB1, 4>(grid, lds, s, a); break;
    }
}
}  // namespace
}  // namespace mggx

MGGX_EXPORT int mggx_mlp2_xw(float *d_out, const float *d_x, const float *d_wa, const float *d_wb, int64_t n, int d1,
                             int h, int d3, const mggx_mlp2_opts *opts)
{
    int rc = mggx::ensure_init();
    if (rc) return rc;
    if (n < 0 || d1 < 1 || h < 1 || d3 < 1) return fail(MGGX_EINVAL, "mlp2_xw: n=%lld d1=%d h=%d d3=%d", (long long)n, d1, h, d3);
    if (h > 64 || d3 > 64) return fail(MGGX_ELIMIT, "mlp2_xw: h=%d and d3=%d must be <= 64 (use two mggx_dense_xw calls)", h, d3);
    if (n == 0) return MGGX_OK;
    if (!d_out || !d_x || !d_wa || !d_wb) return fail(MGGX_EINVAL, "mlp2_xw: NULL pointer");
    if (d_out == d_x) return fail(MGGX_EINVAL, "mlp2_xw: in-place update is not supported");
    mggx_mlp2_opts o{};
    if (opts) o = *opts;
    mggx::MlpArgs a{};
    a.out = d_out;
    a.x = d_x;
    a.wa = d_wa;
    a.wb = d_wb;
    a.rs = o.d_row_scale;
    a.n = n;
    a.ld_x = o.ld_x ? o.ld_x : d1;
    a.ld_out = o.ld_out ? o.ld_out : d3;
    a.d1 = d1;
    a.h = h;
    a.d3 = d3;
    a.relu_mid = o.relu_mid != 0;
    if (o.relu_out > 2) return fail(MGGX_EINVAL, "mlp2_xw: relu_out=%u (0 none, 1 ReLU, 2 row softmax)", o.relu_out);
    a.relu_out = (int)o.relu_out;
    a.vec_out = a.ld_out % 4 == 0 && (reinterpret_cast<uintptr_t>(d_out) & 15u) == 0;
    if (d3 % 32 == 0 && a.ld_out % 32 == 0 && (reinterpret_cast<uintptr_t>(d_out) & 127u) == 0) a.vec_out |= 2;
    a.stream_x = d1 % 64 == 0 && a.ld_x % 32 == 0 && (reinterpret_cast<uintptr_t>(d_x) & 127u) == 0;
    if (a.ld_x < d1 || a.ld_out < d3) return fail(MGGX_EINVAL, "mlp2_xw: row stride smaller than width");
    const int nb1 = (h + 15) / 16, nb2 = (d3 + 15) / 16;
    if (d1 == 64 && h == 64 && d3 > 32 && n >= 4096 && a.ld_x % 4 == 0 && (reinterpret_cast<uintptr_t>(d_x) & 15u) == 0) {
        // the shape of a GIN layer's MLP: the split-operand kernel on the bf16 matrix cores (fp32 results)
        size_t lds_split = (size_t)3 * (64 + nb2 * 16) * mggx::SPLIT_KP * sizeof(unsigned short);
        a.flat_out = a.ld_out == d3 && d3 % 4 != 0 && (reinterpret_cast<uintptr_t>(d_out) & 15u) == 0;  // (64 packed columns: 0.271 -> 0.352 ms, 16 rows to a bank)
        if (a.flat_out) lds_split += (size_t)(mggx::RES_THREADS / 64) * 16 * nb2 * 16 * sizeof(float);  // a tile per wavefront
        hipStream_t stream = mggx::state().stream;
        const dim3 grid(mggx::persistent_blocks(n));
        if (nb2 == 3) {
            mggx::allow_lds(mggx::k_mlp2_split<3>, lds_split);
            mggx::k_mlp2_split<3><<<grid, dim3(mggx::RES_THREADS), lds_split, stream>>>(a);
        } else {
            mggx::allow_lds(mggx::k_mlp2_split<4>, lds_split);
            mggx::k_mlp2_split<4><<<grid, dim3(mggx::RES_THREADS), lds_split, stream>>>(a);
        }
        MGGX_LAUNCH_CHECK("k_mlp2_split");
        return MGGX_OK;
    }
    const size_t lds = ((size_t)((d1 + 63) & ~63) * (nb1 * 16 + 4) + (size_t)nb1 * 16 * (nb2 * 16 + 4)) * sizeof(float);
    if (lds > mggx::LDS_RESIDENT_LIMIT) return fail(MGGX_ELIMIT, "mlp2_xw: weights of %zu bytes do not fit in LDS (d1 <= ~%d at h = %d)", lds,
                                                    (int)(mggx::LDS_RESIDENT_LIMIT / 4 / (nb1 * 16 + 4)) - 64, h);
    const dim3 grid(mggx::persistent_blocks(n));
    hipStream_t stream = mggx::state().stream;
    switch (nb1) {
        case 1: mggx::launch_mlp2_nb2<1>(nb2, grid, lds, stream, a); break;
        case 2: mggx::launch_mlp2_nb2<2>(nb2, grid, lds, stream, a); break;
        case 3: mggx::launch_mlp2_nb2<3>(nb2, grid, lds, stream, a); break;
        default: mggx::launch_mlp2_nb2<4>(nb2, grid, lds, stream, a); break;
    }
    MGGX_LAUNCH_CHECK("k_mlp2_resident");
    return MGGX_OK;
}

MGGX_EXPORT int mggx_dense_xw_bf16(void *d_out, const void *d_x, const void *d_w_bf16, int64_t n, int d1, int d2,
                                   int x_dtype, int out_dtype, const mggx_dense_opts *opts)
{
    int rc = mggx::ensure_init();
    if (rc) return rc;
    if (n < 0 || d1 < 1 || d2 < 1) return fail(MGGX_EINVAL, "dense_xw_bf16: n=%lld d1=%d d2=%d", (long long)n, d1, d2);
    if ((x_dtype != MGGX_F32 && x_dtype != MGGX_BF16) || (out_dtype != MGGX_F32 && out_dtype != MGGX_BF16))
        return fail(MGGX_EINVAL, "dense_xw_bf16: unknown dtype");
    if (n == 0) return MGGX_OK;
    if (!d_out || !d_x || !d_w_bf16) return fail(MGGX_EINVAL, "dense_xw_bf16: NULL pointer");
    if (d_out == d_x) return fail(MGGX_EINVAL, "dense_xw_bf16: in-place update is not supported");
    mggx_dense_opts o{};
    if (opts) o = *opts;
    mggx::DenseArgs a{};
    a.out = d_out;
    a.x = d_x;
    a.w = d_w_bf16;
    a.rs = o.d_row_scale;
    a.n = n;
    a.ld_x = o.ld_x ? o.ld_x : d1;
    a.ld_out = o.ld_out ? o.ld_out : d2;
    a.d1 = d1;
    a.d2 = d2;
    a.relu = o.relu != 0;
    a.vec_out = a.ld_out % 4 == 0 && (reinterpret_cast<uintptr_t>(d_out) & (out_dtype == MGGX_BF16 ? 7u : 15u)) == 0;
    if (out_dtype == MGGX_BF16 && a.ld_out % 8 == 0 && (reinterpret_cast<uintptr_t>(d_out) & 15u) == 0) a.vec_out |= 4;  // 16-byte pieces of 8 bf16
    if (a.ld_x < d1 || a.ld_out < d2) return fail(MGGX_EINVAL, "dense_xw_bf16: row stride smaller than width");
    const int nb = mggx::pick_nb(d2);
    const int gy = ((d2 + 15) / 16 + nb - 1) / nb;
    const size_t lds = (size_t)(nb * 16) * (((d1 + 31) & ~31) + 8) * 2;
    if (lds > 150 * 1024) return fail(MGGX_ELIMIT, "dense_xw_bf16: W tile of %zu bytes does not fit in LDS (d1 <= ~580 at 128 columns)", lds);
    hipStream_t stream = mggx::state().stream;
    if (x_dtype == MGGX_F32 && out_dtype == MGGX_BF16 && (d1 == 64 || d1 == 128) && (d2 == 64 || d2 == 128) && n >= 4096 && (a.vec_out & 4) != 0 &&
        a.ld_x % 4 == 0 && (reinterpret_cast<uintptr_t>(d_x) & 15u) == 0) {
        static unsigned short *image_of[16] = {};
        int dev = -1;
        MGGX_HIP(hipGetDevice(&dev));
        if (dev < 0 || dev >= 16) return fail(MGGX_ELIMIT, "dense_xw_bf16: device index %d", dev);
        if (!image_of[dev]) {
            void *q = nullptr;
            const hipError_t e = hipGetSymbolAddress(&q, HIP_SYMBOL(wt_image));
            if (e != hipSuccess || !q) return fail(MGGX_EHIP, "dense_xw_bf16: hipGetSymbolAddress: %s", hipGetErrorString(e));
            image_of[dev] = static_cast<unsigned short *>(q);
        }
        mggx::k_wt_image<<<dim3((unsigned)((d1 * d2 + 255) / 256)), dim3(256), 0, stream>>>(image_of[dev], static_cast<const unsigned short *>(d_w_bf16), d1, d2);
        MGGX_LAUNCH_CHECK("k_wt_image");
        a.w = image_of[dev];
        a.tiles_per_wave = 8;
        const long long tiles = (n + 15) / 16, per_wg = (long long)mggx::LINES_WAVES * a.tiles_per_wave;
        const unsigned wgs = (unsigned)((tiles + per_wg - 1) / per_wg);
        const auto launch = [&](auto kernel, int nb_, int d1_) {
            const size_t tile_bytes = 16 * (size_t)std::max(d1_ * 2 + 16, nb_ * 32 + 16);
            const size_t lds_lines = (size_t)(nb_ * 16) * (d1_ + 8) * 2 + mggx::LINES_WAVES * tile_bytes;
            mggx::allow_lds(kernel, lds_lines);
            kernel<<<dim3(wgs), dim3(mggx::LINES_WAVES * 64), lds_lines, stream>>>(a);
        };
        if (d1 == 128 && d2 == 128) launch(mggx::k_dense_xw_bf16_lines<8, 128>, 8, 128);
        else if (d1 == 128) launch(mggx::k_dense_xw_bf16_lines<4, 128>, 4, 128);
        else if (d2 == 128) launch(mggx::k_dense_xw_bf16_lines<8, 64>, 8, 64);
        else launch(mggx::k_dense_xw_bf16_lines<4, 64>, 4, 64);
        MGGX_LAUNCH_CHECK("k_dense_xw_bf16_lines");
        return MGGX_OK;
    }
    const dim3 grid(mggx::persistent_blocks(n), (unsigned)gy);
    if (x_dtype == MGGX_F32 && out_dtype == MGGX_F32) mggx::dispatch_nb<mggx::LaunchBf16<true, false>::L>(nb, grid, lds, stream, a);
    else if (x_dtype == MGGX_F32) mggx::dispatch_nb<mggx::LaunchBf16<true, true>::L>(nb, grid, lds, stream, a);
    else if (out_dtype == MGGX_F32) mggx::dispatch_nb<mggx::LaunchBf16<false, false>::L>(nb, grid, lds, stream, a);
    else mggx::dispatch_nb<mggx::LaunchBf16<false, true>::L>(nb, grid, lds, stream, a);
    MGGX_LAUNCH_CHECK("k_dense_xw_bf16");
    return MGGX_OK;
}

MGGX_EXPORT int mggx_softmax_rows(float *d_out, const float *d_in, int64_t n, int c, int64_t ld_in, int64_t ld_out)
{
    int rc = mggx::ensure_init();
    if (rc) return rc;
    if (n < 0 || c < 1) return fail(MGGX_EINVAL, "softmax_rows: n=%lld c=%d", (long long)n, c);
    if (n == 0) return MGGX_OK;
    if (!d_out || !d_in) return fail(MGGX_EINVAL, "softmax_rows: NULL pointer");
    if (!ld_in) ld_in = c;
    if (!ld_out) ld_out = c;
    if (ld_in < c || ld_out < c) return fail(MGGX_EINVAL, "softmax_rows: row stride smaller than width");
    int G = 1;  // lanes per row: up to four values per lane stay in registers
    while (G * 4 < c && G < 64) G <<= 1;
    const long long rows_per_block = 4 * (64 / G);
    const long long blocks = (n + rows_per_block - 1) / rows_per_block;
    if (blocks > 0x7fffffffLL) return fail(MGGX_ELIMIT, "softmax_rows: too many rows");
    mggx::k_softmax_rows<<<dim3((unsigned)blocks), dim3(256), 0, mggx::state().stream>>>(d_out, d_in, (long long)n, c,
                                                                                       (long long)ld_in, (long long)ld_out, G);
    MGGX_LAUNCH_CHECK("k_softmax_rows");
    return MGGX_OK;
}
