/*
 * mgg_oracle.c -- CPU restatement of MGG's neighbor-partitioned aggregation path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker the GPU library is
 * compared against and the "port" CPU baseline that bench.py times.  Nothing
 * in the shipped library links, loads or calls it.
 *
 * Every function cites the reference file:line it restates (paths relative
 * to the MGG_OSDI23 source tree).  Integer routines reproduce the reference
 * bit for bit, including its quirks; floating-point routines come in two
 * flavours: `*_f32` follows the reference kernel's accumulation structure
 * (per-warp partial sums, committed warp by warp) and `*_f64` accumulates in
 * double as the tolerance anchor.
 *
 * How each function is pinned (tests/test_cpu_graph_prep.py, tests/test_cpu_oracle_numerics.py):
 *   orc_range_partition  closed form + brute force
 *   orc_split_csr        reference templates compiled into oracle/_ref, golden fixtures, invariants
 *   orc_build_part       same (incl. the missing-sentinel and node2Part+2 quirks)
 *   orc_graph_load       reference loader compiled into oracle/_ref reads files our writer made
 *   orc_mtx_load         reference loader compiled into oracle/_ref on hand-written .mtx
 *   orc_sag_ref          reference SAG_ref compiled into oracle/_ref
 *   orc_sag_np_div_*     x==1 -> degree, one-hot -> adjacency row, dense A.X brute force, knob independence
 *   orc_gin_np_div_*     same + (1+eps) self term closed form
 *   orc_sag_parts_*      equals orc_sag_ref on the same CSR; closed forms
 *   orc_spmm_*           equals orc_sag_ref
 *   orc_dense_*          numpy matmul, all-ones closed form, identity W
 *   orc_softmax_rows     scipy.special.softmax, rows sum to one, shift invariance
 *   orc_gcn2_forward     all-ones integer closed form of the layer wiring
 *   orc_gin_forward      all-ones integer closed form of the layer wiring
 *   parity unpinned: none of the arithmetic; only the (nondeterministic)
 *   commit order of the reference's float atomics, which no run could pin.
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/stat.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------- */
/* range partition -- src/mgg_np_div_kernel.cu:90-95                          */
/* nodesPerPE = ceil(V/nGPU); lb = nodesPerPE*pe; ub = min(lb+nodesPerPE, V)  */
ORC_API void orc_range_partition(int num_nodes, int num_gpus, int pe,
                                 int *nodes_per_pe, int *lb, int *ub)
{
    int npp = (num_nodes + num_gpus - 1) / num_gpus;
    int l = npp * pe;
    int u = (l + npp) < num_nodes ? (l + npp) : num_nodes;
    *nodes_per_pe = npp;
    *lb = l;
    *ub = u;
}

/* ------------------------------------------------------------------------- */
/* split_CSR -- include/neighbor_utils.cuh:381-405                            */
/* Rows lb..ub-1; each neighbor goes to the local list when lb <= nid < ub,   */
/* else to the remote list; global ids are kept; order inside a row is kept;  */
/* both pointer arrays start at 0 and have (ub-lb)+1 entries.                 */
/* Two-call protocol: pass NULL column arrays to get the sizes only.          */
ORC_API void orc_split_csr(const int *ptr, const int *col, int lb, int ub,
                           int *local_ptr, int *remote_ptr,
                           int *local_col, int *remote_col,
                           int64_t *n_local, int64_t *n_remote)
{
    int64_t nl = 0, nr = 0;
    if (local_ptr) local_ptr[0] = 0;
    if (remote_ptr) remote_ptr[0] = 0;
    for (int i = lb; i < ub; i++) {
        for (int j = ptr[i]; j < ptr[i + 1]; j++) {
            int nid = col[j];
            if (lb <= nid && nid < ub) {
                if (local_col) local_col[nl] = nid;
                nl++;
            } else {
                if (remote_col) remote_col[nr] = nid;
                nr++;
            }
        }
        if (local_ptr) local_ptr[i - lb + 1] = (int)nl;
        if (remote_ptr) remote_ptr[i - lb + 1] = (int)nr;
    }
    if (n_local) *n_local = nl;
    if (n_remote) *n_remote = nr;
}

/* ------------------------------------------------------------------------- */
/* build_part -- include/neighbor_utils.cuh:411-460                           */
/* Returns numParts.  node2Part has num_nodes+2 entries (the reference pushes */
/* the running total once more after the loop, :429).  partPtr has numParts+1 */
/* entries, zero-initialised (:434); its terminal entry is written only while */
/* visiting the LAST node and only when that part ends at the node's end      */
/* (:453-454) -- so it stays 0 when the last node has no neighbors.           */
/* Pass NULL arrays to get numParts only.                                     */
ORC_API int orc_build_part(const int *indptr, int num_nodes, int part_size,
                           int *part_ptr, int *part2node, int *node2part)
{
    int num_parts = 0;
    if (node2part) node2part[0] = 0;
    for (int i = 0; i < num_nodes; i++) {
        int degree = indptr[i + 1] - indptr[i];
        int this_parts = (degree + part_size - 1) / part_size;
        num_parts += this_parts;
        if (node2part) node2part[i + 1] = num_parts;
    }
    if (node2part) node2part[num_nodes + 1] = num_parts;
    if (!part_ptr || !part2node) return num_parts;

    for (int p = 0; p <= num_parts; p++) part_ptr[p] = 0;
    int counter = 0;
    for (int i = 0; i < num_nodes; i++) {
        int degree = indptr[i + 1] - indptr[i];
        int this_parts = (degree + part_size - 1) / part_size;
        for (int pid = 0; pid < this_parts; pid++) {
            int beg = indptr[i] + pid * part_size;
            int end = (beg + part_size < indptr[i + 1]) ? beg + part_size : indptr[i + 1];
            part_ptr[counter] = beg;
            part2node[counter++] = i;
            if (i == num_nodes - 1 && end == indptr[i + 1])
                part_ptr[counter] = end;
        }
    }
    return num_parts;
}

/* ------------------------------------------------------------------------- */
/* binary CSR loader -- include/graph.h:11-37, include/graph.hpp:9-130,       */
/* instantiated graph<long,long,int,int,int,int> (mgg_np_div_kernel.cu:59):   */
/* vert_count = fsize(beg)/8 - 1; beg_pos int64[V+1]; edge_count = beg[V];    */
/* csr int64[E]; weight int32[E]; all narrowed to int.                        */
/* Returns 0 on success, negative on a failed open / short read (the          */
/* reference prints and asserts instead).  Two-call protocol via NULLs.       */
static int64_t orc_fsize(const char *fn)
{
    struct stat st;
    if (stat(fn, &st) == 0) return (int64_t)st.st_size;
    return -1;
}

ORC_API int orc_graph_load(const char *beg_file, const char *csr_file, const char *weight_file,
                           int *vert_count, int *edge_count,
                           int *beg_pos, int *csr, int *weight)
{
    int64_t fs = orc_fsize(beg_file);
    if (fs < 0) return -1;
    int64_t V = fs / (int64_t)sizeof(int64_t) - 1;
    FILE *f = fopen(beg_file, "rb");
    if (!f) return -1;
    int64_t *tmp = (int64_t *)malloc(sizeof(int64_t) * (size_t)(V + 1));
    if (fread(tmp, sizeof(int64_t), (size_t)(V + 1), f) != (size_t)(V + 1)) { fclose(f); free(tmp); return -2; }
    fclose(f);
    int64_t E = tmp[V];
    *vert_count = (int)V;
    *edge_count = (int)E;
    if (beg_pos) for (int64_t i = 0; i <= V; i++) beg_pos[i] = (int)tmp[i];
    free(tmp);
    if (E <= 0) return -3; /* graph.hpp:32 asserts beg_pos[V] > 0 */
    if (csr) {
        f = fopen(csr_file, "rb");
        if (!f) return -4;
        int64_t *t2 = (int64_t *)malloc(sizeof(int64_t) * (size_t)E);
        size_t got = fread(t2, sizeof(int64_t), (size_t)E, f);
        fclose(f);
        if (got != (size_t)E) { free(t2); return -5; }
        for (int64_t i = 0; i < E; i++) csr[i] = (int)t2[i];
        free(t2);
    }
    if (weight) {
        f = fopen(weight_file, "rb");
        if (!f) return -6;
        size_t got = fread(weight, sizeof(int32_t), (size_t)E, f);
        fclose(f);
        if (got != (size_t)E) return -7;
    }
    return 0;
}

/* ------------------------------------------------------------------------- */
/* MatrixMarket-style text loader -- include/csr_formatter.h:112-144          */
/* '%' comment lines, header "M N L", then L lines "row col val" (1-based).   */
/* col_ind is the file order of (col-1); row_ptr is the prefix sum of per-row */
/* counts -- so the file must be sorted by row for the pair to be a CSR.      */
/* Two-call protocol: NULL arrays -> sizes only.                              */
ORC_API int orc_mtx_load(const char *path, int *M_out, int *L_out, int *row_ptr, int *col_ind)
{
    FILE *f = fopen(path, "r");
    if (!f) return -1;
    int c;
    while ((c = fgetc(f)) == '%') {
        while ((c = fgetc(f)) != '\n' && c != EOF) {}
    }
    if (c != EOF) ungetc(c, f);
    int M, N, L;
    if (fscanf(f, "%d %d %d", &M, &N, &L) != 3) { fclose(f); return -2; }
    *M_out = M;
    *L_out = L;
    int *cnt = (int *)calloc((size_t)M + 1, sizeof(int));
    for (int l = 0; l < L; l++) {
        int r, cc;
        double v;
        if (fscanf(f, "%d %d %lf", &r, &cc, &v) != 3) { fclose(f); free(cnt); return -3; }
        cnt[r - 1]++;
        if (col_ind) col_ind[l] = cc - 1;
    }
    fclose(f);
    if (row_ptr) {
        row_ptr[0] = 0;
        for (int i = 0; i < M; i++) row_ptr[i + 1] = row_ptr[i] + cnt[i];
    }
    free(cnt);
    return 0;
}

/* ------------------------------------------------------------------------- */
/* SAG_ref -- include/utils.cuh:71-86: update[nid] += input[col[e]] (serial)  */
ORC_API void orc_sag_ref(float *update, const float *input, const int *node_ptr,
                         const int *column_index, int num_node, int dim)
{
    for (int nid = 0; nid < num_node; nid++) {
        for (int e = node_ptr[nid]; e < node_ptr[nid + 1]; e++) {
            int eid = column_index[e];
            for (int d = 0; d < dim; d++)
                update[(size_t)nid * dim + d] += input[(size_t)eid * dim + d];
        }
    }
}

/* ------------------------------------------------------------------------- */
/* Aggregation semantics of mgg_SAG_np_div_cuda -- neighbor_utils.cuh:1351-1460
 * and mgg_GIN_np_div_cuda -- :1554-1667.
 *
 * For destination row v (0 <= v < ub-lb), block of `wpb` warps:
 *   local loop  (:1395-1414): b = ptr_l[v] .. step dist*wpb*ps; warp w takes
 *       [b + w*dist*ps, +dist*ps) cut at the row end; tmp[w] += in[(nid % npp)]
 *   remote loop (:1432-1452): same tiling over ptr_r/col_r; the row fetched is
 *       row (nid % npp) of PE (nid / npp), i.e. row `nid` of the concatenated
 *       per-PE tables -- `in_remote` here is that concatenation, indexed by
 *       global id.
 *   commit (:1456-1458): out[v] += tmp[w] for every warp (float atomics; the
 *       order between warps is not defined by the reference -- warp order
 *       0..wpb-1 is used here).
 *   GIN (:1660-1665): out[v] = (1+eps)*in[v] first, then the commits.  The
 *       reference lets every warp execute that store (a race with the other
 *       warps' atomics); the intended value, (1+eps)*x_v + sum, is computed.
 *
 * flags: bit0 accumulate into `out` (the reference's SAG behaviour: out is
 *        never zeroed, :1458); otherwise out is overwritten.
 *        bit1 GIN self term with `eps`.
 * row_scale_in (may be NULL): every gathered row u is multiplied by
 *        row_scale_in[global id u]; row_scale_out (may be NULL): the finished
 *        sum of row v is multiplied by row_scale_out[v] (before the GIN self
 *        term and before accumulation).  Both NULL = the reference.  These two
 *        give D^-1/2 (A) D^-1/2 X without materialising edge weights.
 * ld_in / ld_out: row strides in elements (>= dim); the reference has ld==dim.
 */
#define ORC_ACCUMULATE 1
#define ORC_GIN 2

static void orc_row_np_div(double *acc64, float *acc32, int use64,
                           const float *in_local, const float *in_remote,
                           const int *ptr_l, const int *col_l, const int *ptr_r, const int *col_r,
                           int v, int dim, int64_t ld_in, int npp, int ps, int wpb, int dist,
                           const float *rs_in, float *tmp /* wpb*dim */)
{
    /* per-warp partial sums, as the kernel's shared-memory tmp[] */
    if (!use64) memset(tmp, 0, sizeof(float) * (size_t)wpb * dim);
    for (int side = 0; side < 2; side++) {
        const int *ptr = side ? ptr_r : ptr_l;
        const int *col = side ? col_r : col_l;
        if (!ptr) continue;
        int es = ptr[v], ee = ptr[v + 1];
        int64_t step = (int64_t)dist * wpb * ps;
        for (int64_t b = es; b < ee; b += step) {
            for (int w = 0; w < wpb; w++) {
                int64_t wb = b + (int64_t)w * dist * ps;
                int64_t we = wb + (int64_t)dist * ps;
                if (we > ee) we = ee;
                for (int64_t e = wb; e < we; e++) {
                    int nid = col[e];
                    const float *src = side ? in_remote + (int64_t)nid * ld_in
                                            : in_local + (int64_t)(nid % npp) * ld_in;
                    float s = rs_in ? rs_in[nid] : 1.0f;
                    if (use64) {
                        if (rs_in) for (int d = 0; d < dim; d++) acc64[d] += (double)s * (double)src[d];
                        else       for (int d = 0; d < dim; d++) acc64[d] += (double)src[d];
                    } else {
                        float *t = tmp + (size_t)w * dim;
                        if (rs_in) for (int d = 0; d < dim; d++) t[d] += s * src[d];
                        else       for (int d = 0; d < dim; d++) t[d] += src[d];
                    }
                }
            }
        }
    }
    if (!use64) {
        for (int d = 0; d < dim; d++) acc32[d] = 0.0f;
        for (int w = 0; w < wpb; w++)
            for (int d = 0; d < dim; d++) acc32[d] += tmp[(size_t)w * dim + d];
    }
}

static void orc_np_div_impl(float *out, const float *in_local, const float *in_remote,
                            const int *ptr_l, const int *col_l, const int *ptr_r, const int *col_r,
                            int lb, int ub, int dim, int64_t ld_in, int64_t ld_out, int npp,
                            int ps, int wpb, int dist, int flags, float eps,
                            const float *rs_in, const float *rs_out,
                            int use64, const int *rows, int n_rows, int nthreads)
{
    int R = ub - lb;
    int count = rows ? n_rows : R;
    (void)nthreads;
#ifdef _OPENMP
#pragma omp parallel num_threads(nthreads > 0 ? nthreads : 1)
#endif
    {
        double *acc64 = (double *)malloc(sizeof(double) * (size_t)dim);
        float *acc32 = (float *)malloc(sizeof(float) * (size_t)dim);
        float *tmp = (float *)malloc(sizeof(float) * (size_t)wpb * dim);
#ifdef _OPENMP
#pragma omp for schedule(dynamic, 64)
#endif
        for (int i = 0; i < count; i++) {
            int v = rows ? rows[i] : i;
            /* with a row list, results are written densely: out row i */
            float *o = out + (int64_t)(rows ? i : v) * ld_out;
            if (use64) for (int d = 0; d < dim; d++) acc64[d] = 0.0;
            orc_row_np_div(acc64, acc32, use64, in_local, in_remote, ptr_l, col_l, ptr_r, col_r,
                           v, dim, ld_in, npp, ps, wpb, dist, rs_in, tmp);
            for (int d = 0; d < dim; d++) {
                double s = use64 ? acc64[d] : (double)acc32[d];
                float so = rs_out ? rs_out[v] : 1.0f;
                double r;
                if (use64) {
                    r = rs_out ? s * (double)so : s;
                    if (flags & ORC_GIN) r += (1.0 + (double)eps) * (double)in_local[(int64_t)v * ld_in + d];
                    if (flags & ORC_ACCUMULATE) r += (double)o[d];
                    o[d] = (float)r;
                } else {
                    float rf = rs_out ? (float)s * so : (float)s;
                    if (flags & ORC_GIN) {
                        /* :1661 computes (1.0 + eps) in double, the product in double, stores float */
                        float self = (float)((1.0 + eps) * in_local[(int64_t)v * ld_in + d]);
                        rf = self + rf;
                    }
                    if (flags & ORC_ACCUMULATE) rf = o[d] + rf;
                    o[d] = rf;
                }
            }
        }
        free(acc64);
        free(acc32);
        free(tmp);
    }
}

ORC_API void orc_sag_np_div_f32(float *out, const float *in_local, const float *in_remote,
                                const int *ptr_l, const int *col_l, const int *ptr_r, const int *col_r,
                                int lb, int ub, int dim, int64_t ld_in, int64_t ld_out, int npp,
                                int ps, int wpb, int dist, int flags, float eps,
                                const float *rs_in, const float *rs_out, int nthreads)
{
    orc_np_div_impl(out, in_local, in_remote, ptr_l, col_l, ptr_r, col_r, lb, ub, dim, ld_in, ld_out,
                    npp, ps, wpb, dist, flags, eps, rs_in, rs_out, 0, NULL, 0, nthreads);
}

ORC_API void orc_sag_np_div_f64(float *out, const float *in_local, const float *in_remote,
                                const int *ptr_l, const int *col_l, const int *ptr_r, const int *col_r,
                                int lb, int ub, int dim, int64_t ld_in, int64_t ld_out, int npp,
                                int flags, float eps,
                                const float *rs_in, const float *rs_out, int nthreads)
{
    orc_np_div_impl(out, in_local, in_remote, ptr_l, col_l, ptr_r, col_r, lb, ub, dim, ld_in, ld_out,
                    npp, 1 << 30, 1, 1, flags, eps, rs_in, rs_out, 1, NULL, 0, nthreads);
}

/* Selected rows only (double accumulation); out is [n_rows x ld_out], row i  */
/* holding the result for rows[i].  ORC_ACCUMULATE is not meaningful here.    */
ORC_API void orc_sag_np_div_rows_f64(float *out, const int *rows, int n_rows,
                                     const float *in_local, const float *in_remote,
                                     const int *ptr_l, const int *col_l, const int *ptr_r, const int *col_r,
                                     int lb, int ub, int dim, int64_t ld_in, int64_t ld_out, int npp,
                                     int flags, float eps,
                                     const float *rs_in, const float *rs_out, int nthreads)
{
    orc_np_div_impl(out, in_local, in_remote, ptr_l, col_l, ptr_r, col_r, lb, ub, dim, ld_in, ld_out,
                    npp, 1 << 30, 1, 1, flags & ~ORC_ACCUMULATE, eps, rs_in, rs_out, 1, rows, n_rows, nthreads);
}

/* Sum over a row of |scale * x| -- the magnitude the fp32 tolerance is       */
/* expressed against: |gpu - oracle| <= tol * abs_sum.  Same addressing as    */
/* orc_sag_np_div_*.  `rows` may be NULL (all rows).                          */
ORC_API void orc_sag_np_div_abs_sum(float *out, const int *rows, int n_rows,
                                    const float *in_local, const float *in_remote,
                                    const int *ptr_l, const int *col_l, const int *ptr_r, const int *col_r,
                                    int lb, int ub, int dim, int64_t ld_in, int64_t ld_out, int npp,
                                    int flags, float eps,
                                    const float *rs_in, const float *rs_out, int nthreads)
{
    int R = ub - lb;
    int count = rows ? n_rows : R;
    (void)nthreads;
#ifdef _OPENMP
#pragma omp parallel for schedule(dynamic, 64) num_threads(nthreads > 0 ? nthreads : 1)
#endif
    for (int i = 0; i < count; i++) {
        int v = rows ? rows[i] : i;
        float *o = out + (int64_t)i * ld_out;
        for (int d = 0; d < dim; d++) {
            double a = 0.0;
            for (int side = 0; side < 2; side++) {
                const int *ptr = side ? ptr_r : ptr_l;
                const int *col = side ? col_r : col_l;
                if (!ptr) continue;
                for (int e = ptr[v]; e < ptr[v + 1]; e++) {
                    int nid = col[e];
                    const float *src = side ? in_remote + (int64_t)nid * ld_in
                                            : in_local + (int64_t)(nid % npp) * ld_in;
                    double s = rs_in ? (double)rs_in[nid] : 1.0;
                    a += fabs(s * (double)src[d]);
                }
            }
            if (rs_out) a *= fabs((double)rs_out[v]);
            if (flags & ORC_GIN) a += fabs((1.0 + (double)eps) * (double)in_local[(int64_t)v * ld_in + d]);
            o[d] = (float)a;
        }
    }
}

/* ------------------------------------------------------------------------- */
/* Explicit-partition aggregation -- SAG_host :463-506 / SAG_cuda_kernel      */
/* :2373-2447: one warp per partition p: srcId = part2Node[p]; neighbors      */
/* column_index[partPtr[p] .. partPtr[p+1]); gathered row = input[nid -       */
/* lowbound]; partial summed in fp32 from 0, then output[srcId] += partial.   */
/* A non-positive (partPtr[p+1]-partPtr[p]) contributes nothing, as the       */
/* kernel's loops simply do not run.                                          */
ORC_API void orc_sag_parts_f32(float *out, const float *in, const int *col,
                               const int *part_ptr, const int *part2node,
                               int lowbound, int num_parts, int dim)
{
    float *part = (float *)malloc(sizeof(float) * (size_t)dim);
    for (int p = 0; p < num_parts; p++) {
        int src = part2node[p];
        int beg = part_ptr[p], end = part_ptr[p + 1];
        for (int d = 0; d < dim; d++) part[d] = 0.0f;
        for (int e = beg; e < end; e++) {
            int nid = col[e] - lowbound;
            for (int d = 0; d < dim; d++) part[d] += in[(size_t)nid * dim + d];
        }
        if (end > beg)
            for (int d = 0; d < dim; d++) out[(size_t)src * dim + d] += part[d];
    }
    free(part);
}

/* ------------------------------------------------------------------------- */
/* Single-GPU whole-graph SpMM -- include/gnn_kernel.cuh:9-71:                */
/* block per node, warp w takes neighbors [b + ps*w, +ps) for b stepping by   */
/* ps*wpb; per-warp fp32 partial; out[v] += partial for every warp.           */
ORC_API void orc_spmm_f32(float *out, const float *in, const int *row_ptr, const int *col,
                          int num_nodes, int dim, int ps, int wpb)
{
    orc_np_div_impl(out, in, in, row_ptr, col, NULL, NULL, 0, num_nodes, dim, dim, dim,
                    0x7fffffff, ps, wpb, 1, ORC_ACCUMULATE, 0.0f, NULL, NULL, 0, NULL, 0, 1);
}

/* ------------------------------------------------------------------------- */
/* Dense node update -- include/layer_new.cuh:222-229 + gnn_layer.cuh:22-52:  */
/* column-major SGEMM(N,N, m=dim2, n=numNodes, k=dim1, A=W ld=dim2, B=X       */
/* ld=dim1, C=Out ld=dim2), alpha=1, beta=0  ==  row-major Out = X . W.       */
/* (The reference call sites pass d_out as B as well; the intended operand,   */
/* d_in, is used.)  f32: k-sequential fp32 FMA-free accumulation; f64: double.*/
ORC_API void orc_dense_f32(float *out, const float *X, const float *W, int64_t n, int d1, int d2,
                           int64_t ld_x, int64_t ld_out, int use64, int nthreads)
{
    (void)nthreads;
#ifdef _OPENMP
#pragma omp parallel for schedule(static) num_threads(nthreads > 0 ? nthreads : 1)
#endif
    for (int64_t i = 0; i < n; i++) {
        const float *x = X + i * ld_x;
        float *o = out + i * ld_out;
        if (use64) {
            double acc[512];
            for (int j0 = 0; j0 < d2; j0 += 512) {
                int jb = d2 - j0 < 512 ? d2 - j0 : 512;
                for (int j = 0; j < jb; j++) acc[j] = 0.0;
                for (int k = 0; k < d1; k++) {
                    double xv = (double)x[k];
                    const float *w = W + (size_t)k * d2 + j0;
                    for (int j = 0; j < jb; j++) acc[j] += xv * (double)w[j];
                }
                for (int j = 0; j < jb; j++) o[j0 + j] = (float)acc[j];
            }
        } else {
            float acc[512];
            for (int j0 = 0; j0 < d2; j0 += 512) {
                int jb = d2 - j0 < 512 ? d2 - j0 : 512;
                for (int j = 0; j < jb; j++) acc[j] = 0.0f;
                for (int k = 0; k < d1; k++) {
                    float xv = x[k];
                    const float *w = W + (size_t)k * d2 + j0;
                    for (int j = 0; j < jb; j++) acc[j] += xv * w[j];
                }
                for (int j = 0; j < jb; j++) o[j0 + j] = acc[j];
            }
        }
    }
}

/* ------------------------------------------------------------------------- */
/* Row softmax -- include/gnn_layer.cuh:15-20 + layer_new.cuh:32-37:          */
/* cudnnSoftmaxForward(ACCURATE, MODE_CHANNEL) on an (N, C, 1, 1) tensor ==   */
/* per row: exp(x - max) / sum exp(x - max), alpha=1, beta=0.                 */
ORC_API void orc_softmax_rows(float *out, const float *in, int64_t n, int c,
                              int64_t ld_in, int64_t ld_out, int nthreads)
{
    (void)nthreads;
#ifdef _OPENMP
#pragma omp parallel for schedule(static) num_threads(nthreads > 0 ? nthreads : 1)
#endif
    for (int64_t i = 0; i < n; i++) {
        const float *x = in + i * ld_in;
        float *o = out + i * ld_out;
        double m = -INFINITY;
        for (int j = 0; j < c; j++) if ((double)x[j] > m) m = (double)x[j];
        double s = 0.0;
        for (int j = 0; j < c; j++) s += exp((double)x[j] - m);
        for (int j = 0; j < c; j++) o[j] = (float)(exp((double)x[j] - m) / s);
    }
}

/* ------------------------------------------------------------------------- */
/* 2-layer GCN forward, layer order of src/mgg_np_div_mem.cu:211-227:         */
/*   Y1 = X.W1 ; H1 = Agg(Y1) ; Y2 = H1.W2 ; H2 = Agg(Y2) ; P = softmax(H2)   */
/* No bias, no activation.  The reference runs its second aggregation at      */
/* width `hidden` (:221-222); the real width, out_dim, is used here.          */
/* rs (may be NULL) = D^-1/2 per global node: Agg(Y) = diag(rs) A diag(rs) Y. */
/* Whole share in one call: X is [npp x in_dim] for the local rows; the       */
/* remote table of each aggregation is `Y` itself when remote_is_local != 0   */
/* (single-GPU whole graph, lb == 0), which is the only mode offered.         */
ORC_API void orc_gcn2_forward(float *P, float *H2_opt, float *H1_opt,
                              const float *X, const float *W1, const float *W2,
                              const int *ptr_l, const int *col_l, const int *ptr_r, const int *col_r,
                              int lb, int ub, int npp, int in_dim, int hidden, int out_dim,
                              const float *rs, int use64, int nthreads)
{
    int64_t R = ub - lb;
    float *Y1 = (float *)malloc(sizeof(float) * (size_t)R * hidden);
    float *H1 = (float *)malloc(sizeof(float) * (size_t)R * hidden);
    float *Y2 = (float *)malloc(sizeof(float) * (size_t)R * out_dim);
    float *H2 = (float *)malloc(sizeof(float) * (size_t)R * out_dim);
    const float *rs_out = rs ? rs + lb : NULL;
    orc_dense_f32(Y1, X, W1, R, in_dim, hidden, in_dim, hidden, use64, nthreads);
    if (use64)
        orc_sag_np_div_f64(H1, Y1, Y1, ptr_l, col_l, ptr_r, col_r, lb, ub, hidden, hidden, hidden, npp, 0, 0.f, rs, rs_out, nthreads);
    else
        orc_sag_np_div_f32(H1, Y1, Y1, ptr_l, col_l, ptr_r, col_r, lb, ub, hidden, hidden, hidden, npp, 16, 8, 1, 0, 0.f, rs, rs_out, nthreads);
    orc_dense_f32(Y2, H1, W2, R, hidden, out_dim, hidden, out_dim, use64, nthreads);
    if (use64)
        orc_sag_np_div_f64(H2, Y2, Y2, ptr_l, col_l, ptr_r, col_r, lb, ub, out_dim, out_dim, out_dim, npp, 0, 0.f, rs, rs_out, nthreads);
    else
        orc_sag_np_div_f32(H2, Y2, Y2, ptr_l, col_l, ptr_r, col_r, lb, ub, out_dim, out_dim, out_dim, npp, 16, 8, 1, 0, 0.f, rs, rs_out, nthreads);
    orc_softmax_rows(P, H2, R, out_dim, out_dim, out_dim, nthreads);
    if (H1_opt) memcpy(H1_opt, H1, sizeof(float) * (size_t)R * hidden);
    if (H2_opt) memcpy(H2_opt, H2, sizeof(float) * (size_t)R * out_dim);
    free(Y1); free(H1); free(Y2); free(H2);
}

/* ------------------------------------------------------------------------- */
/* GIN forward, layer order of src/mgg_np_div_gin_mem.cu:195-222:             */
/*   Y = X.W[0] ; for l in 1..L: H = GINAgg(Y, eps) ; Y = H.W[l] ; softmax(Y) */
/* W[0] is in_dim x hidden, W[1..L-1] hidden x hidden, W[L] hidden x out_dim  */
/* (the reference has L = 5).  Single-GPU whole graph (remote table = Y).     */
ORC_API void orc_gin_forward(float *P, float *logits_opt, const float *X, const float *const *W, int n_layers,
                             const int *ptr_l, const int *col_l, const int *ptr_r, const int *col_r,
                             int lb, int ub, int npp, int in_dim, int hidden, int out_dim,
                             float eps, int use64, int nthreads)
{
    int64_t R = ub - lb;
    int maxd = hidden > out_dim ? hidden : out_dim;
    float *Y = (float *)malloc(sizeof(float) * (size_t)R * maxd);
    float *H = (float *)malloc(sizeof(float) * (size_t)R * hidden);
    orc_dense_f32(Y, X, W[0], R, in_dim, hidden, in_dim, hidden, use64, nthreads);
    for (int l = 1; l <= n_layers; l++) {
        if (use64)
            orc_sag_np_div_f64(H, Y, Y, ptr_l, col_l, ptr_r, col_r, lb, ub, hidden, hidden, hidden, npp, ORC_GIN, eps, NULL, NULL, nthreads);
        else
            orc_sag_np_div_f32(H, Y, Y, ptr_l, col_l, ptr_r, col_r, lb, ub, hidden, hidden, hidden, npp, 16, 8, 1, ORC_GIN, eps, NULL, NULL, nthreads);
        int d2 = (l == n_layers) ? out_dim : hidden;
        orc_dense_f32(Y, H, W[l], R, hidden, d2, hidden, d2, use64, nthreads);
    }
    orc_softmax_rows(P, Y, R, out_dim, out_dim, out_dim, nthreads);
    if (logits_opt) memcpy(logits_opt, Y, sizeof(float) * (size_t)R * out_dim);
    free(Y); free(H);
}

ORC_API int orc_max_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
