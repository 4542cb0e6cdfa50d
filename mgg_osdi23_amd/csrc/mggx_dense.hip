// Dense node update Out = X . W on the fp32 matrix cores, and the row softmax.
#include "mggx_dev.h"

namespace mggx {
namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int GEMM_KC = 64;       // K extent of the W tile staged in LDS
constexpr int GEMM_ROWS_WG = 64;  // 4 wavefronts x 16 rows

struct DenseArgs {
    float *out;
    const float *x;
    const float *w;
    const float *rs;
    long long n;
    long long ld_x, ld_out;
    int d1, d2;
    int relu;
};

// v_mfma_f32_16x16x4_f32 operand layout (wave64):
//   A (16 x 4): lane L holds A[L % 16][L / 16]
//   B (4 x 16): lane L holds B[L / 16][L % 16]
//   D (16 x 16): lane L holds D[4 * (L / 16) + r][L % 16], r = 0..3
// Each lane loads 4 consecutive K values of one X row; MFMA step t then
// multiplies the K indices {4*(L/16) + t}, and B is read from LDS with the same
// index, so the sum over K is complete after 4 steps per 16 K values.
template <int NB>
__global__ void __launch_bounds__(256) k_dense_xw(const DenseArgs a)
{
    constexpr int RS = NB * 16 + 4;  // LDS row stride in floats; the +4 keeps the four K groups on distinct banks
    __shared__ float wt[GEMM_KC * RS];
    const int lane = (int)(threadIdx.x & 63u);
    const int wave = (int)(threadIdx.x >> 6);
    const int i = lane & 15, kq = lane >> 4;
    const long long row = (long long)blockIdx.x * GEMM_ROWS_WG + wave * 16 + i;
    const int c0 = (int)blockIdx.y * (NB * 16);
    const bool row_ok = row < a.n;
    const float *xrow = a.x + (row_ok ? row : 0) * a.ld_x;

    v4f acc[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[nb] = (v4f){0.f, 0.f, 0.f, 0.f};

    for (int k0 = 0; k0 < a.d1; k0 += GEMM_KC) {
        __syncthreads();
        for (int idx = (int)threadIdx.x; idx < GEMM_KC * NB * 16; idx += 256) {
            const int k = idx / (NB * 16), j = idx % (NB * 16);
            float v = 0.f;
            if (k0 + k < a.d1 && c0 + j < a.d2) v = a.w[(long long)(k0 + k) * a.d2 + c0 + j];
            wt[k * RS + j] = v;
        }
        __syncthreads();
#pragma unroll
        for (int ks = 0; ks < GEMM_KC / 16; ++ks) {
            const int kb = k0 + ks * 16 + 4 * kq;
            float xv[4] = {0.f, 0.f, 0.f, 0.f};
            if (row_ok) {
                if (kb + 3 < a.d1) {
                    float4 t4;
                    __builtin_memcpy(&t4, xrow + kb, 16);
                    xv[0] = t4.x; xv[1] = t4.y; xv[2] = t4.z; xv[3] = t4.w;
                } else {
#pragma unroll
                    for (int t = 0; t < 4; ++t)
                        if (kb + t < a.d1) xv[t] = xrow[kb + t];
                }
            }
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const float *wrow = wt + (ks * 16 + 4 * kq + t) * RS + i;
#pragma unroll
                for (int nb = 0; nb < NB; ++nb)
                    acc[nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(xv[t], wrow[nb * 16], acc[nb], 0, 0, 0);
            }
        }
    }

    const long long row_base = (long long)blockIdx.x * GEMM_ROWS_WG + wave * 16 + 4 * kq;
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
                a.out[orow * a.ld_out + c] = v;
            }
        }
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
    if (a.ld_x < d1 || a.ld_out < d2) return fail(MGGX_EINVAL, "dense_xw: row stride smaller than width");
    const long long gx = (n + mggx::GEMM_ROWS_WG - 1) / mggx::GEMM_ROWS_WG;
    if (gx > 0x7fffffffLL) return fail(MGGX_ELIMIT, "dense_xw: too many rows");
    hipStream_t stream = mggx::state().stream;
    const int blocks16 = (d2 + 15) / 16;
    // columns are covered in chunks of NB*16; pick the widest chunk that wastes no block
    int nb = blocks16 >= 8 ? 8 : blocks16;
    if (nb == 5) nb = 6;
    if (nb == 7) nb = 8;
    const int gy = (blocks16 + nb - 1) / nb;
    const dim3 grid((unsigned)gx, (unsigned)gy), block(256);
    switch (nb) {
        case 1: mggx::k_dense_xw<1><<<grid, block, 0, stream>>>(a); break;
        case 2: mggx::k_dense_xw<2><<<grid, block, 0, stream>>>(a); break;
        case 3: mggx::k_dense_xw<3><<<grid, block, 0, stream>>>(a); break;
        case 4: mggx::k_dense_xw<4><<<grid, block, 0, stream>>>(a); break;
        case 6: mggx::k_dense_xw<6><<<grid, block, 0, stream>>>(a); break;
        default: mggx::k_dense_xw<8><<<grid, block, 0, stream>>>(a); break;
    }
    MGGX_LAUNCH_CHECK("k_dense_xw");
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
    int G = 1;
    while (G < c && G < 64) G <<= 1;
    const long long rows_per_block = 4 * (64 / G);
    const long long blocks = (n + rows_per_block - 1) / rows_per_block;
    if (blocks > 0x7fffffffLL) return fail(MGGX_ELIMIT, "softmax_rows: too many rows");
    mggx::k_softmax_rows<<<dim3((unsigned)blocks), dim3(256), 0, mggx::state().stream>>>(d_out, d_in, (long long)n, c,
                                                                                       (long long)ld_in, (long long)ld_out, G);
    MGGX_LAUNCH_CHECK("k_softmax_rows");
    return MGGX_OK;
}
