// Error convention and small host helpers of the MGG host API.
// Counterpart of MGG_OSDI23 include/utils.cuh (gpuErrchk :18-26, SAG_ref :71-86,
// compare_array :120-128, check_equal :130-138) and include/cublas_utils.h
// (CUDA_CHECK :44-52), rebuilt over the libmggx C ABI.
#ifndef MGG_UTILS_H
#define MGG_UTILS_H

#include <cstdio>
#include <cstdlib>
#include <iostream>
#include <string>
#include <vector>

#include "mggx.h"

// The reference prints and exits on any device error (utils.cuh:18-26); every
// wrapper in this layer routes libmggx status codes through the same behaviour.
#define gpuErrchk(ans) { mggAssert((ans), __FILE__, __LINE__); }
#define MGG_CHECK(ans) { mggAssert((ans), __FILE__, __LINE__); }
inline void mggAssert(int code, const char *file, int line, bool abort = true)
{
    if (code != MGGX_OK) {
        fprintf(stderr, "GPUassert: %s %s %d\n", mggx_last_error(), file, line);
        if (abort) exit(code);
    }
}

// Serial CPU scatter-gather used by the reference for validation only
// (utils.cuh:71-86): update[nid] += input[col[e]] for every edge of nid.
inline void SAG_ref(float *update, float *input, int *node_ptr, int *column_index, int numNode, int numEdges, int ebdDim)
{
    (void)numEdges;
    for (int v = 0; v < numNode; ++v)
        for (int e = node_ptr[v]; e < node_ptr[v + 1]; ++e) {
            const float *src = input + (size_t)column_index[e] * ebdDim;
            float *dst = update + (size_t)v * ebdDim;
            for (int d = 0; d < ebdDim; ++d) dst[d] += src[d];
        }
}

inline void init_origin_node(float *origin_node, int ebdDim, int numNodes, float init_val)
{
    for (size_t i = 0; i < (size_t)numNodes * ebdDim; ++i) origin_node[i] = init_val;
}

template <typename T>
void print_array(std::string name, std::vector<T> &array, int len = 10)
{
    std::cout << name << ":\t";
    for (int i = 0; i < len && i < (int)array.size(); ++i) std::cout << array[i] << ' ';
    std::cout << std::endl;
}

// exact comparisons, as the reference validates with all-ones inputs (utils.cuh:120-138)
inline bool compare_array(float *ref, float *output, int len)
{
    for (int i = 0; i < len; ++i)
        if (ref[i] != output[i]) {
            printf("ref: %.3f -- out: %.3f\n", ref[i], output[i]);
            return false;
        }
    return true;
}

inline bool check_equal(float *ref, float *output, int len, int dim, int lb_ref = 0)
{
    for (int i = 0; i < len; ++i)
        if (ref[lb_ref + i] != output[i]) {
            printf("[%d] ref: %.3f -- out: %.3f\n", i / dim, ref[lb_ref + i], output[i]);
            return false;
        }
    return true;
}

#endif
