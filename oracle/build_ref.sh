#!/usr/bin/env bash
# Builds oracle/_ref/libmgg_ref.so from the reference's OWN host sources, read
# where they lie under $MGG_REFERENCE (default /root/reference).  TEST
# INFRASTRUCTURE ONLY: used to pin oracle/mgg_oracle.c and to generate the
# fixtures under tests/golden/.
#
# What is compiled (nothing else of the reference builds without nvcc, MPI,
# NVSHMEM, cuBLAS and cuDNN, none of which this image has):
#   include/graph.h + graph.hpp + wtime.h      unmodified, via #include
#   include/csr_formatter.h                     unmodified, via #include (needs <limits> first)
#   include/neighbor_utils.cuh lines 381-460    split_CSR<T>, build_part<T>: pure-STL templates that
#                                               sit in a header which also includes <nvshmem.h>, so the
#                                               two templates are streamed by line range into the
#                                               compiler's stdin (no copy is written anywhere)
#   include/utils.cuh lines 71-86               SAG_ref, same treatment (the header includes <cuda.h>)
# The line ranges are verified against the function names before compiling.
set -euo pipefail
REF="${MGG_REFERENCE:-/root/reference}"
HERE="$(cd "$(dirname "${BASH_SOURCE[0]}")" && pwd)"
OUT="$HERE/_ref"
if [ ! -d "$REF/include" ]; then
    echo "build_ref: $REF not present, skipping (prebuilt $OUT/libmgg_ref.so is used when it exists)"
    exit 0
fi
mkdir -p "$OUT"
NU="$REF/include/neighbor_utils.cuh"
UT="$REF/include/utils.cuh"
sed -n '382p' "$NU" | grep -q 'split_CSR'  || { echo "build_ref: split_CSR not at neighbor_utils.cuh:382"; exit 1; }
sed -n '412p' "$NU" | grep -q 'build_part' || { echo "build_ref: build_part not at neighbor_utils.cuh:412"; exit 1; }
sed -n '71p'  "$UT" | grep -q 'SAG_ref'    || { echo "build_ref: SAG_ref not at utils.cuh:71"; exit 1; }
{
    cat <<'EOF'
#include <limits>
#include <sstream>
#include <vector>
#include <string>
#include <cstdio>
#include <cstring>
#include <cstdint>
#include "graph.h"
#include "csr_formatter.h"
EOF
    sed -n '381,460p' "$NU"
    sed -n '71,86p' "$UT"
    cat <<'EOF'
typedef graph<long, long, int, int, int, int> ref_graph_t;
extern "C" {
// split_CSR<int>: returns sizes through n[4] = {|local_ptr|, |remote_ptr|, |local_col|, |remote_col|};
// arrays are copied out when non-NULL.
void ref_split_csr(const int* ptr, int64_t n_ptr, const int* col, int64_t n_col, int lb, int ub,
                   int* lp, int* rp, int* lc, int* rc, int64_t* n) {
    std::vector<int> p(ptr, ptr + n_ptr), c(col, col + n_col);
    auto r = split_CSR<int>(p, c, lb, ub);
    for (int i = 0; i < 4; i++) n[i] = (int64_t)r[i].size();
    if (lp) memcpy(lp, r[0].data(), r[0].size() * sizeof(int));
    if (rp) memcpy(rp, r[1].data(), r[1].size() * sizeof(int));
    if (lc) memcpy(lc, r[2].data(), r[2].size() * sizeof(int));
    if (rc) memcpy(rc, r[3].data(), r[3].size() * sizeof(int));
}
// build_part<int>: n[3] = {|partPtr|, |part2Node|, |node2Part|}
void ref_build_part(const int* indptr, int64_t n_ptr, int num_nodes, int part_size,
                    int* part_ptr, int* part2node, int* node2part, int64_t* n) {
    std::vector<int> p(indptr, indptr + n_ptr);
    auto r = build_part<int>(std::string("ref"), p, num_nodes, part_size);
    for (int i = 0; i < 3; i++) n[i] = (int64_t)r[i].size();
    if (part_ptr) memcpy(part_ptr, r[0].data(), r[0].size() * sizeof(int));
    if (part2node) memcpy(part2node, r[1].data(), r[1].size() * sizeof(int));
    if (node2part) memcpy(node2part, r[2].data(), r[2].size() * sizeof(int));
}
void ref_sag_ref(float* update, float* input, int* node_ptr, int* column_index,
                 int num_node, int num_edges, int dim) {
    SAG_ref(update, input, node_ptr, column_index, num_node, num_edges, dim);
}
// graph<long,long,int,int,int,int>: first call with NULL arrays gives the counts.
void ref_graph_load(const char* beg, const char* csr, const char* weight,
                    int* vert_count, int* edge_count, int* beg_pos, int* csr_out, int* weight_out) {
    ref_graph_t g(beg, csr, weight);
    *vert_count = g.vert_count;
    *edge_count = g.edge_count;
    if (beg_pos) memcpy(beg_pos, g.beg_pos, sizeof(int) * ((size_t)g.vert_count + 1));
    if (csr_out) memcpy(csr_out, g.csr, sizeof(int) * (size_t)g.edge_count);
    if (weight_out) memcpy(weight_out, g.weight, sizeof(int) * (size_t)g.edge_count);
}
// split_CSR<long> / build_part<long>: the same templates for 64-bit ids, sizes as above
void ref_split_csr_long(const long* ptr, int64_t n_ptr, const long* col, int64_t n_col, long lb, long ub,
                        long* lp, long* rp, long* lc, long* rc, int64_t* n) {
    std::vector<long> p(ptr, ptr + n_ptr), c(col, col + n_col);
    auto r = split_CSR<long>(p, c, lb, ub);
    for (int i = 0; i < 4; i++) n[i] = (int64_t)r[i].size();
    if (lp) memcpy(lp, r[0].data(), r[0].size() * sizeof(long));
    if (rp) memcpy(rp, r[1].data(), r[1].size() * sizeof(long));
    if (lc) memcpy(lc, r[2].data(), r[2].size() * sizeof(long));
    if (rc) memcpy(rc, r[3].data(), r[3].size() * sizeof(long));
}
void ref_build_part_long(const long* indptr, int64_t n_ptr, long num_nodes, long part_size,
                         long* part_ptr, long* part2node, long* node2part, int64_t* n) {
    std::vector<long> p(indptr, indptr + n_ptr);
    auto r = build_part<long>(std::string("ref"), p, num_nodes, part_size);
    for (int i = 0; i < 3; i++) n[i] = (int64_t)r[i].size();
    if (part_ptr) memcpy(part_ptr, r[0].data(), r[0].size() * sizeof(long));
    if (part2node) memcpy(part2node, r[1].data(), r[1].size() * sizeof(long));
    if (node2part) memcpy(node2part, r[2].data(), r[2].size() * sizeof(long));
}
// assemble_csr_matrix (which = 0) / assemble_simetric_csr_matrix (which = 1): n[3] = {|row_ptr|, |col_ind|, |val|};
// getBandwidth of the result in *bandwidth; printMatrix's output for the result with row_ptr[0] set to 1 into text (at most
// text_cap - 1 characters) when non-NULL
void ref_mtx_load_other(int which, const char* path, int* row_ptr, int* col_ind, double* val, int64_t* n, int* bandwidth,
                        char* text, int64_t text_cap) {
    CSR m = which ? assemble_simetric_csr_matrix(std::string(path)) : assemble_csr_matrix(std::string(path));
    n[0] = (int64_t)m.row_ptr.size();
    n[1] = (int64_t)m.col_ind.size();
    n[2] = (int64_t)m.val.size();
    if (row_ptr) memcpy(row_ptr, m.row_ptr.data(), m.row_ptr.size() * sizeof(int));
    if (col_ind) memcpy(col_ind, m.col_ind.data(), m.col_ind.size() * sizeof(int));
    if (val) memcpy(val, m.val.data(), m.val.size() * sizeof(double));
    if (bandwidth) *bandwidth = getBandwidth(m);
    if (text && text_cap > 0) {
        std::ostringstream os;
        std::streambuf* old = std::cout.rdbuf(os.rdbuf());
        CSR one_based = m;  // printMatrix reads col_ind[row_ptr[i-1] - 1 ...): with row_ptr[0] = 0 it would start before the array
        one_based.row_ptr[0] = 1;
        printMatrix(one_based);
        std::cout.rdbuf(old);
        const std::string t = os.str();
        const size_t k = std::min<size_t>(t.size(), (size_t)text_cap - 1);
        memcpy(text, t.data(), k);
        text[k] = 0;
    }
}
// assemble_csr_matrix_new: n[2] = {|row_ptr|, |col_ind|}
void ref_mtx_load(const char* path, int* row_ptr, int* col_ind, int64_t* n) {
    CSR m = assemble_csr_matrix_new(std::string(path));
    n[0] = (int64_t)m.row_ptr.size();
    n[1] = (int64_t)m.col_ind.size();
    if (row_ptr) memcpy(row_ptr, m.row_ptr.data(), m.row_ptr.size() * sizeof(int));
    if (col_ind) memcpy(col_ind, m.col_ind.data(), m.col_ind.size() * sizeof(int));
}
}
EOF
} | g++ -std=c++14 -O2 -w -fPIC -shared -I"$REF/include" -x c++ - -o "$OUT/libmgg_ref.so"
echo "build_ref: built $OUT/libmgg_ref.so"
