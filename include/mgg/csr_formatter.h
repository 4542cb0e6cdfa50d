// Text (MatrixMarket-style) graph loader with the interface of MGG_OSDI23
// include/csr_formatter.h: struct CSR (:13-17) and assemble_csr_matrix_new
// (:112-144), the loader the reference's mains use.  Leading '%' lines are
// comments, then "M N L", then L entries "row col value" (1-based).  col_ind
// keeps the file order, row_ptr is the prefix sum of per-row counts, val stays
// empty -- so the entries have to be sorted by row, as in the reference.
#ifndef MGG_CSR_FORMATTER_H
#define MGG_CSR_FORMATTER_H

#include <iostream>
#include <string>
#include <vector>

#include "mgg/utils.h"
#include "mggx.h"

struct CSR {
    std::vector<double> val;
    std::vector<int> col_ind;
    std::vector<int> row_ptr;
};

inline CSR assemble_csr_matrix_new(std::string filePath)
{
    CSR m;
    int rows = 0, entries = 0;
    MGG_CHECK(mggx_mtx_read(filePath.c_str(), &rows, &entries, nullptr, nullptr));
    m.row_ptr.resize((size_t)rows + 1);
    m.col_ind.resize((size_t)entries);
    MGG_CHECK(mggx_mtx_read(filePath.c_str(), &rows, &entries, m.row_ptr.data(), m.col_ind.data()));
    return m;
}

inline int getDegree(const std::vector<int> &row_ptr, int vertex) { return row_ptr[vertex] - row_ptr[vertex - 1]; }

inline std::vector<int> getAdjVertices(const std::vector<int> &col_ind, const std::vector<int> &row_ptr, int vertex)
{
    return std::vector<int>(col_ind.begin() + row_ptr[vertex - 1], col_ind.begin() + row_ptr[vertex]);
}

inline void printArray(const std::vector<int> &v)
{
    for (int x : v) std::cout << x << ' ';
    std::cout << '\n';
}

#endif
