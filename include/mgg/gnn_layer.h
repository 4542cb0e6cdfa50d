// Layer calls of MGG, source-compatible with MGG_OSDI23 include/gnn_layer.cuh:
// softmax_forward (:15-20), dense_beg_forward / dense_hidden_forward (:22-32),
// softmax_new_forward (:36-40), dense_beg_new_forward / dense_hidden_new_forward
// (:42-52), sparse_beg_forward / sparse_hidden_forward (:86-161).
//
// Dense update: Out = X . W with X = dp->d_in.  (The reference's call sites pass
// dp->d_out as the GEMM's input operand as well, gnn_layer.cuh:24-25, so d_in is
// never read there; the intended operand is used here.)  X and Out must be
// different buffers.
#ifndef MGG_GNN_LAYER_H
#define MGG_GNN_LAYER_H

#include "mgg/layer_new.h"
#include "mgg/neighbor_utils.h"
#include "mggx.h"

inline void softmax_forward(softmax_param *smx)
{
    MGG_CHECK(mggx_softmax_rows(smx->d_out, smx->d_in, smx->numNodes, smx->dim, 0, 0));
    MGG_CHECK(mggx_sync());  // the reference synchronises here (gnn_layer.cuh:19)
}

inline void softmax_new_forward(softmax_new_param *smx)
{
    MGG_CHECK(mggx_softmax_rows(smx->d_out, smx->d_in, smx->numNodes, smx->dim, 0, 0));
}

inline void mgg_dense_forward(dense_param_base *dp)
{
    MGG_CHECK(mggx_dense_xw(dp->d_out, dp->d_in, dp->d_W, dp->numNodes, dp->dim1, dp->dim2, nullptr));
}
inline void dense_beg_forward(dense_param_beg *dp) { mgg_dense_forward(dp); }
inline void dense_hidden_forward(dense_param_hidden *dp) { mgg_dense_forward(dp); }
inline void dense_beg_new_forward(dense_param_new_beg *dp) { mgg_dense_forward(dp); }
inline void dense_hidden_new_forward(dense_param_new_hidden *dp) { mgg_dense_forward(dp); }

// Whole graph on one GPU: d_out[v] += sum of d_in[u] over the neighbors u of v.
inline void sparse_beg_forward(sparse_param_beg *sp)
{
    mgg_finish_call(mggx_spmm(sp->d_out, sp->d_in, sp->d_row_ptr, sp->d_col_ind, sp->numNodes, sp->dim, sp->partSize,
                              sp->warpPerBlock),
                    " sparse_beg_forward");
}

inline void sparse_hidden_forward(sparse_param_hidden *sp)
{
    mgg_finish_call(mggx_spmm(sp->d_out, sp->d_in, sp->d_row_ptr, sp->d_col_ind, sp->numNodes, sp->dim, sp->partSize,
                              sp->warpPerBlock),
                    " sparse_hidden_forward");
}

#endif
