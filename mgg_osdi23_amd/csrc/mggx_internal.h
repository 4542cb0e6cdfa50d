// Internal declarations shared by the translation units of libmggx.so.
#ifndef MGGX_INTERNAL_H
#define MGGX_INTERNAL_H

#include <cstdarg>
#include <cstddef>
#include <cstdint>

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

}  // namespace mggx
#endif
