// Parameter objects of MGG's layers, source-compatible with MGG_OSDI23
// include/layer_new.cuh: softmax_param (:13-55), softmax_new_param (:59-103),
// sparse_param_beg (:107-157), sparse_param_hidden (:160-207), dense_param_beg
// (:210-269), dense_param_new_beg (:272-333), dense_param_new_hidden (:336-393),
// dense_param_hidden (:396-451).  Same constructors, same public fields for
// shapes, buffers and launch geometry; the cuBLAS/cuDNN handles have no
// counterpart (the dense update and the softmax are libmggx kernels).
// As in the reference, the objects own W and (for the non-"new" classes) their
// output buffer, W is all ones, and nothing is released on destruction.
#ifndef MGG_LAYER_NEW_H
#define MGG_LAYER_NEW_H

#include <algorithm>
#include <cstdlib>
#include <cstring>

#include "mgg/utils.h"
#include "mggx.h"

static int n_partition = 1;  // layer_new.cuh:11

namespace mgg_detail {
inline float *device_floats(size_t count, bool zero)
{
    void *p = nullptr;
    MGG_CHECK(mggx_malloc(&p, count * sizeof(float)));
    if (zero) MGG_CHECK(mggx_memset(p, 0, count * sizeof(float)));
    return static_cast<float *>(p);
}
inline void copy_name(char (&dst)[8], const char *src)
{
    strncpy(dst, src, 7);
    dst[7] = '\0';
}
}  // namespace mgg_detail

class softmax_param {
  public:
    softmax_param(const char *name_in, float *d_in_input, int numNodes_in, int dim_in)
    {
        mgg_detail::copy_name(name, name_in);
        numNodes = numNodes_in;
        dim = dim_in;
        d_in = d_in_input;
        alpha = 1.0f;
        beta = 0.0f;
        d_out = mgg_detail::device_floats((size_t)numNodes * dim, true);
    }
    int numNodes, dim;
    float *d_out, *d_in;
    float alpha, beta;
    char name[8];
};

class softmax_new_param {
  public:
    softmax_new_param(const char *name_in, float *d_in_input, float *d_out_ext, int numNodes_in, int dim_in)
    {
        mgg_detail::copy_name(name, name_in);
        numNodes = numNodes_in;
        dim = dim_in;
        d_in = d_in_input;
        d_out = d_out_ext;
        alpha = 1.0f;
        beta = 0.0f;
    }
    int numNodes, dim;
    float *d_out, *d_in;
    float alpha, beta;
    char name[8];
};

// Launch geometry fields keep their reference meaning: one workgroup per node,
// warpPerBlock wavefronts each (WARP_SIZE is 64 on gfx950).
class sparse_param_beg {
  public:
    sparse_param_beg(const char *name_in, int *d_row_ptr_in, int *d_col_ind_in, int numNodes_in, int dim_in,
                     int partSize_in, int warpPerBlock_in)
    {
        mgg_detail::copy_name(name, name_in);
        numNodes = numNodes_in;
        dim = dim_in;
        d_row_ptr = d_row_ptr_in;
        d_col_ind = d_col_ind_in;
        warpPerBlock = warpPerBlock_in;
        partSize = partSize_in;
        const size_t count = (size_t)numNodes * dim;
        h_in = static_cast<float *>(malloc(count * sizeof(float)));
        h_out = static_cast<float *>(malloc(count * sizeof(float)));
        std::fill_n(h_in, count, 1.0f);
        std::fill_n(h_out, count, 0.0f);
        d_in = mgg_detail::device_floats(count, false);
        d_out = mgg_detail::device_floats(count, true);
        MGG_CHECK(mggx_memcpy_h2d(d_in, h_in, count * sizeof(float)));
        kernel_param();
    }
    int numNodes, dim;
    float *h_in, *h_out, *d_in, *d_out;
    int *d_row_ptr, *d_col_ind;
    int warpPerBlock, partSize, WARP_SIZE_;
    int block, grid, shared_memory;
    char name[8];

  private:
    void kernel_param()
    {
        WARP_SIZE_ = 64;
        block = warpPerBlock * WARP_SIZE_;
        grid = numNodes / n_partition;
        shared_memory = warpPerBlock * dim * (int)sizeof(float) + warpPerBlock * partSize * (int)sizeof(int);
    }
};

class sparse_param_hidden {
  public:
    sparse_param_hidden(const char *name_in, float *d_in_input, int *d_row_ptr_in, int *d_col_ind_in, int numNodes_in,
                        int dim_in, int partSize_in, int warpPerBlock_in)
    {
        mgg_detail::copy_name(name, name_in);
        numNodes = numNodes_in;
        dim = dim_in;
        d_in = d_in_input;
        d_row_ptr = d_row_ptr_in;
        d_col_ind = d_col_ind_in;
        warpPerBlock = warpPerBlock_in;
        partSize = partSize_in;
        h_in = h_out = nullptr;
        d_out = mgg_detail::device_floats((size_t)numNodes * dim, true);
        WARP_SIZE_ = 64;
        block = warpPerBlock * WARP_SIZE_;
        grid = numNodes / n_partition;
        shared_memory = warpPerBlock * dim * (int)sizeof(float) + warpPerBlock * partSize * (int)sizeof(int);
    }
    int numNodes, dim;
    float *h_in, *h_out, *d_in, *d_out;
    int *d_row_ptr, *d_col_ind;
    int warpPerBlock, partSize, WARP_SIZE_;
    int block, grid, shared_memory;
    char name[8];
};

// Shared body of the four dense parameter classes: Out[numNodes x dim2] = X[numNodes x dim1] . W[dim1 x dim2].
// m, n, k, ldx, ldw, ldout keep the column-major GEMM view of the reference (layer_new.cuh:222-229).
class dense_param_base {
  public:
    int m, n, k, ldx, ldw, ldout;
    int numNodes, dim1, dim2;
    float *h_W, *d_W, *d_W_new, *d_out, *d_in, *h_in;
    float alpha, beta;
    char name[8];

  protected:
    void setup(const char *name_in, float *d_in_ext, float *d_out_ext, int numNodes_in, int dim1_in, int dim2_in)
    {
        mgg_detail::copy_name(name, name_in);
        numNodes = numNodes_in;
        dim1 = dim1_in;
        dim2 = dim2_in;
        m = dim2, n = numNodes, k = dim1;
        ldx = dim1, ldw = dim2, ldout = dim2;
        alpha = 1.0f;
        beta = 0.0f;
        d_in = d_in_ext;
        h_in = nullptr;
        d_W_new = nullptr;
        const size_t wcount = (size_t)dim1 * dim2;
        h_W = static_cast<float *>(malloc(wcount * sizeof(float)));
        std::fill_n(h_W, wcount, 1.0f);  // the reference initialises W to ones (layer_new.cuh:243)
        d_W = mgg_detail::device_floats(wcount, false);
        MGG_CHECK(mggx_memcpy_h2d(d_W, h_W, wcount * sizeof(float)));
        if (d_out_ext) {
            d_out = d_out_ext;
        } else {
            d_out = mgg_detail::device_floats((size_t)numNodes * dim2, true);
        }
    }
};

class dense_param_beg : public dense_param_base {
  public:
    dense_param_beg(const char *name_in, float *d_in_ext, int numNodes_in, int dim1_in, int dim2_in)
    {
        setup(name_in, d_in_ext, nullptr, numNodes_in, dim1_in, dim2_in);
    }
};

class dense_param_hidden : public dense_param_base {
  public:
    dense_param_hidden(const char *name_in, float *d_in_input, int numNodes_in, int dim1_in, int dim2_in)
    {
        setup(name_in, d_in_input, nullptr, numNodes_in, dim1_in, dim2_in);
    }
};

class dense_param_new_beg : public dense_param_base {
  public:
    dense_param_new_beg(const char *name_in, float *d_in_ext, float *d_out_ext, int numNodes_in, int dim1_in, int dim2_in)
    {
        setup(name_in, d_in_ext, d_out_ext, numNodes_in, dim1_in, dim2_in);
    }
};

class dense_param_new_hidden : public dense_param_base {
  public:
    dense_param_new_hidden(const char *name_in, float *d_in_input, float *d_out_ext, int numNodes_in, int dim1_in,
                           int dim2_in)
    {
        setup(name_in, d_in_input, d_out_ext, numNodes_in, dim1_in, dim2_in);
    }
};

#endif
