// Exercises every entry of the drop-in C++ layer (include/mgg/*.h) on the GPU the way the reference validates itself:
// all-ones inputs, exact comparison against closed forms and against SAG_ref (include/utils.cuh:71-86, 130-138).
//   mgg_api_check <scratch dir>
// Prints one "[ok] ..." or "[FAIL] ..." line per check; the exit code is the number of failures.
#include <algorithm>
#include <string>

#include "harness_common.h"

static int g_fail = 0;

static void report(bool ok, const char *what)
{
    printf("[%s] %s\n", ok ? "ok" : "FAIL", what);
    if (!ok) ++g_fail;
}

static std::vector<float> from_device(const float *d, size_t count)
{
    std::vector<float> h(count);
    MGG_CHECK(mggx_sync());
    MGG_CHECK(mggx_memcpy_d2h(h.data(), d, count * sizeof(float)));
    return h;
}

static bool all_equal(const std::vector<float> &got, const std::vector<float> &row_value, int dim)
{
    for (size_t i = 0; i < got.size(); ++i)
        if (got[i] != row_value[i / dim]) {
            printf("  row %zu col %zu: got %.3f want %.3f\n", i / dim, i % dim, got[i], row_value[i / dim]);
            return false;
        }
    return true;
}

int main(int argc, char *argv[])
{
    if (argc < 2) {
        printf("Usage: %s <scratch dir>\n", argv[0]);
        return 64;
    }
    const std::string dir = argv[1];
    MGG_CHECK(mggx_init(0));

    // A small deterministic graph: node v points to itself, its two successors and three scattered nodes.
    const int V = 3000, dim = 16, ps = 4, wpb = 4;
    std::vector<int> ptr(1, 0), col;
    for (int v = 0; v < V; ++v) {
        std::vector<int> nb = {v, (v + 1) % V, (v + 2) % V, (int)((7LL * v + 3) % V), (int)((v * (long long)v) % V), (v / 2)};
        if (v % 5 == 0) nb.clear();  // isolated rows
        std::sort(nb.begin(), nb.end());
        nb.erase(std::unique(nb.begin(), nb.end()), nb.end());
        col.insert(col.end(), nb.begin(), nb.end());
        ptr.push_back((int)col.size());
    }
    const int E = (int)col.size();

    // ---- loaders: binary triple and text ----
    const std::string beg = dir + "/g_beg_pos.bin", csr = dir + "/g_csr.bin", wgt = dir + "/g_weight.bin";
    MGG_CHECK(mggx_graph_write(beg.c_str(), csr.c_str(), wgt.c_str(), V, ptr.data(), col.data(), nullptr));
    graph<long, long, nidType, nidType, nidType, nidType> g(beg.c_str(), csr.c_str(), wgt.c_str());
    bool ok = g.vert_count == V && g.edge_count == E;
    for (int i = 0; ok && i <= V; ++i) ok = g.beg_pos[i] == ptr[i];
    for (int e = 0; ok && e < E; ++e) ok = g.csr[e] == col[e] && g.weight[e] == 1;
    report(ok, "graph<long,long,int,int,int,int> reads back the binary triple");
    {
        const std::string mtx = dir + "/g.mtx";
        FILE *f = fopen(mtx.c_str(), "w");
        fprintf(f, "%%%%MatrixMarket matrix coordinate real general\n%d %d %d\n", V, V, E);
        for (int v = 0; v < V; ++v)
            for (int e = ptr[v]; e < ptr[v + 1]; ++e) fprintf(f, "%d %d 1.0\n", v + 1, col[e] + 1);
        fclose(f);
        CSR m = assemble_csr_matrix_new(mtx);
        report(m.row_ptr == ptr && m.col_ind == col, "assemble_csr_matrix_new reads the text form");
    }

    // ---- one rank's share ----
    const int nGPU = 4, pe = 1;
    int npp = 0, lb = 0, ub = 0;
    MGG_CHECK(mggx_range_partition(V, nGPU, pe, &npp, &lb, &ub));
    auto split = split_CSR<nidType>(ptr, col, lb, ub);
    const int R = ub - lb;
    auto lparts = build_part<nidType>("local", split[0], R, ps);
    auto rparts = build_part<nidType>("remote", split[1], R, ps);
    std::vector<float> deg(R), deg_l(R);
    for (int r = 0; r < R; ++r) {
        deg_l[r] = (float)(split[0][r + 1] - split[0][r]);
        deg[r] = deg_l[r] + (float)(split[1][r + 1] - split[1][r]);
    }
    report((int)lparts[1].size() + (int)rparts[1].size() >= (E / nGPU) / ps, "split_CSR / build_part produce partitions");
    int *d_pl = to_device(split[0]), *d_pr = to_device(split[1]), *d_cl = to_device(split[2]), *d_cr = to_device(split[3]);
    float *d_ones_all = device_filled((size_t)nGPU * npp * dim, 1.0f);  // every rank's rows, indexed by global id
    float *d_ones_loc = device_filled((size_t)npp * dim, 1.0f);
    mgg_stage_remote(d_ones_all);

    float *d_out = device_filled((size_t)R * dim, 0.0f);
    mgg_SAG_np_div(d_out, d_ones_loc, d_pl, d_cl, d_pr, d_cr, lb, ub, dim, npp, pe, ps, wpb, 2);
    report(all_equal(from_device(d_out, (size_t)R * dim), deg, dim), "mgg_SAG_np_div: ones -> degree");
    mgg_SAG_np_div(d_out, d_ones_loc, d_pl, d_cl, d_pr, d_cr, lb, ub, dim, npp, pe, ps, wpb, 2);
    {
        std::vector<float> twice(R);
        for (int r = 0; r < R; ++r) twice[r] = 2 * deg[r];
        report(all_equal(from_device(d_out, (size_t)R * dim), twice, dim), "mgg_SAG_np_div adds into its output, as the reference does");
    }
    mgg_GIN_np_div(d_out, d_ones_loc, d_pl, d_cl, d_pr, d_cr, lb, ub, dim, npp, pe, ps, wpb, 2, 0.5f);
    {
        std::vector<float> want(R);
        for (int r = 0; r < R; ++r) want[r] = deg[r] + 1.5f;
        report(all_equal(from_device(d_out, (size_t)R * dim), want, dim), "mgg_GIN_np_div: ones -> degree + 1 + eps, overwriting");
    }
    {
        float ms = 0.f;
        mggx_agg_knobs k = mgg_tune_np_div(d_out, d_ones_loc, d_pl, d_cl, d_pr, d_cr, lb, ub, dim, npp, 0, &ms);
        bool good = all_equal(from_device(d_out, (size_t)R * dim), deg, dim) && k.wpb > 0 && k.dist > 0 && ms > 0.f;
        mgg_options().accumulate = false;
        mgg_SAG_np_div(d_out, d_ones_loc, d_pl, d_cl, d_pr, d_cr, lb, ub, dim, npp, pe, 0, 0, 0);  // uses what the search found
        good = good && all_equal(from_device(d_out, (size_t)R * dim), deg, dim);
        mgg_options().accumulate = true;
        report(good, "mgg_tune_np_div, then a call that leaves the knobs to the library");
    }

    // ---- explicit partition arrays ----
    {
        int *d_pp = to_device(lparts[0]), *d_p2n = to_device(lparts[1]);
        MGG_CHECK(mggx_memset(d_out, 0, (size_t)R * dim * sizeof(float)));
        SAG_host<int, float, int>(d_out, d_ones_loc, d_pl, d_cl, d_pp, d_p2n, lb, R, (int)lparts[1].size(), ps, dim, 32, wpb);
        report(all_equal(from_device(d_out, (size_t)R * dim), deg_l, dim), "SAG_host: ones -> local degree");
        MGG_CHECK(mggx_memset(d_out, 0, (size_t)R * dim * sizeof(float)));
        int *d_rpp = to_device(rparts[0]), *d_rp2n = to_device(rparts[1]);
        SAG_host_fused_interleaved<int, float, int>(d_out, d_ones_loc, d_pl, d_cl, d_pp, d_p2n, (int)lparts[1].size(), d_pr, d_cr,
                                                    d_rpp, d_rp2n, (int)rparts[1].size(), R + 1, lb, ps, dim, 32, wpb, 2);
        report(all_equal(from_device(d_out, (size_t)R * dim), deg_l, dim), "SAG_host_fused_interleaved: ones -> local degree");
    }

    // ---- whole-graph layer objects ----
    {
        int *d_ptr = to_device(ptr), *d_col = to_device(col);
        std::vector<float> degw(V), ref((size_t)V * dim, 0.0f), ones((size_t)V * dim, 1.0f);
        for (int v = 0; v < V; ++v) degw[v] = (float)(ptr[v + 1] - ptr[v]);
        SAG_ref(ref.data(), ones.data(), ptr.data(), col.data(), V, E, dim);
        sparse_param_beg sp1("s-1", d_ptr, d_col, V, dim, ps, wpb);
        sparse_beg_forward(&sp1);
        std::vector<float> got = from_device(sp1.d_out, (size_t)V * dim);
        report(check_equal(ref.data(), got.data(), V * dim, dim), "sparse_beg_forward equals SAG_ref");
        dense_param_hidden dp("d-1", sp1.d_out, V, dim, 24);
        dense_hidden_forward(&dp);
        {
            std::vector<float> want(V);
            for (int v = 0; v < V; ++v) want[v] = degw[v] * dim;  // W is all ones
            report(all_equal(from_device(dp.d_out, (size_t)V * 24), want, 24), "dense_hidden_forward: X . ones");
        }
        sparse_param_hidden sp2("s-2", dp.d_out, d_ptr, d_col, V, 24, ps, wpb);
        sparse_hidden_forward(&sp2);
        {
            std::vector<float> want(V, 0.0f);
            for (int v = 0; v < V; ++v)
                for (int e = ptr[v]; e < ptr[v + 1]; ++e) want[v] += degw[col[e]] * dim;
            report(all_equal(from_device(sp2.d_out, (size_t)V * 24), want, 24), "sparse_hidden_forward on the update's output");
        }
        float *d_x = device_filled((size_t)V * 10, 1.0f), *d_y = device_filled((size_t)V * 8, 0.0f);
        dense_param_beg db("d-0", d_x, V, 10, 8);
        dense_beg_forward(&db);
        dense_param_new_beg dnb("d-n", d_x, d_y, V, 10, 8);
        dense_beg_new_forward(&dnb);
        dense_param_new_hidden dnh("d-h", d_y, device_filled((size_t)V * 4, 0.0f), V, 8, 4);
        dense_hidden_new_forward(&dnh);
        {
            std::vector<float> ten(V, 10.0f), eighty(V, 80.0f);
            report(all_equal(from_device(db.d_out, (size_t)V * 8), ten, 8) && all_equal(from_device(d_y, (size_t)V * 8), ten, 8) &&
                       all_equal(from_device(dnh.d_out, (size_t)V * 4), eighty, 4),
                   "dense_beg_forward / dense_beg_new_forward / dense_hidden_new_forward");
        }
        softmax_param sm("smx", dnh.d_out, V, 4);
        softmax_forward(&sm);
        float *d_p = device_filled((size_t)V * 4, 0.0f);
        softmax_new_param smn("smn", dnh.d_out, d_p, V, 4);
        softmax_new_forward(&smn);
        {
            std::vector<float> quarter(V, 0.25f);
            report(all_equal(from_device(sm.d_out, (size_t)V * 4), quarter, 4) && all_equal(from_device(d_p, (size_t)V * 4), quarter, 4),
                   "softmax_forward / softmax_new_forward: equal logits -> 1/4");
        }
    }
    printf("%d check(s) failed\n", g_fail);
    return g_fail;
}
