// Internal declarations shared by the translation units of libmggx.so.
#ifndef MGGX_INTERNAL_H
#define MGGX_INTERNAL_H

#include <cstdarg>
#include <cstddef>
#include <cstdint>
#include <vector>

#include "mggx.h"

#define MGGX_EXPORT extern "C" __attribute__((visibility("default")))

namespace mggx {

// Records a printf-style message for mggx_last_error() and returns `code`.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

// splitmix64 finaliser: the counter-based generator behind every synthetic input.
static inline uint64_t mix64(uint64_t x)
{
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}
static inline uint64_t rnd64(uint64_t seed, uint64_t i, uint64_t j)
{
    return mix64(mix64(seed ^ (i * 0xD1342543DE82EF95ull)) + j);
}

// Dense-core layout of a local CSR (host arrays).  The `core` highest-degree rows, ranked by degree (ties by id), form
// a core x core block whose edges leave the CSR and are stored as sliced ELL lists: slice g = ranks [64 g, 64 g + 64),
// tile t = core columns (by rank) [tc t, tc t + tc); block (g, t) holds, per lane (= rank inside the slice), the tile
// offsets of that row's neighbors inside the tile and padding slots (tc + r, r < 16: zero columns behind the tile) up to
// the longest list of the slice rounded up to 4, in bank order (core_bank_order):
// idx[((blk_off[g * ntiles + t] + k / 4) * 64 + lane) * 4 + k % 4].  Every other edge stays in (rem_ptr, rem_col),
// row order and edge order kept, column ids unchanged.
struct CoreLayout {
    int rows = 0, core = 0, tc = 0, ntiles = 0;
    int64_t core_nnz = 0;
    std::vector<int> order;            // [core] row (0-based in the share) of rank i
    std::vector<int> rank;             // [rows] rank of the row, -1 outside the core
    std::vector<unsigned> blk_off;     // [core / 64 * ntiles + 1], in chunks of 4 list positions
    std::vector<unsigned short> idx;   // [blk_off.back() * 256]
    std::vector<int> rem_ptr, rem_col; // what is left of the CSR
};
// core is rounded down to a multiple of 512 (and of tc); returns MGGX_EINVAL when nothing is left of it.
int core_layout_build(const int *ptr, const int *col, int rows, int lb, int core, int tc, CoreLayout *out);

}  // namespace mggx
#endif
