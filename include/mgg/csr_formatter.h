// Text (MatrixMarket-style) graph loader with the interface of MGG_OSDI23
// include/csr_formatter.h: struct CSR (:13-17) and assemble_csr_matrix_new
// (:112-144), the loader the reference's mains use.  Leading '%' lines are
// comments, then "M N L", then L entries "row col value" (1-based).  col_ind
// keeps the file order, row_ptr is the prefix sum of per-row counts, val stays
// empty -- so the entries have to be sorted by row, as in the reference.
// The header's other entry points -- assemble_csr_matrix (:83-109), assemble_simetric_csr_matrix (:146-183), getBandwidth
// (:65-80), printMatrix (:31-53), which no main on the aggregation path calls -- are plain host code below.
#ifndef MGG_CSR_FORMATTER_H
#define MGG_CSR_FORMATTER_H

#include <algorithm>
#include <cstdlib>
#include <fstream>
#include <iostream>
#include <limits>
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

inline void printArray(const std::vector<double> &v)
{
    for (double x : v) std::cout << x << ' ';
    std::cout << '\n';
}

// The entries "row col value" of a MatrixMarket-style file after its '%' lines and its "M N L" line.
struct mgg_mtx_entries {
    int M = 0, N = 0, L = 0;
    std::vector<int> row, col;
    std::vector<double> val;
};
inline mgg_mtx_entries mgg_read_mtx_entries(const std::string &filePath)
{
    mgg_mtx_entries e;
    std::ifstream fin(filePath);
    while (fin.peek() == '%') fin.ignore(2048, '\n');
    fin >> e.M >> e.N >> e.L;
    e.row.assign((size_t)std::max(e.L, 0), 0);
    e.col.assign(e.row.size(), 0);
    e.val.assign(e.row.size(), 0.0);
    for (size_t k = 0; k < e.row.size(); ++k) fin >> e.row[k] >> e.col[k] >> e.val[k];
    return e;
}

// assemble_csr_matrix (csr_formatter.h:83-109), the older loader: ids stay 1-based, every entry's column and value are
// kept in file order, and row_ptr = {0, then for every entry whose row number exceeds every earlier one the number of
// entries read so far including it, then L + 1} -- rows without entries leave no mark, as in the reference.
inline CSR assemble_csr_matrix(std::string filePath)
{
    const mgg_mtx_entries e = mgg_read_mtx_entries(filePath);
    CSR m;
    m.col_ind = e.col;
    m.val = e.val;
    m.row_ptr.push_back(0);
    int highest = 1;
    for (size_t k = 0; k < e.row.size(); ++k)
        if (e.row[k] > highest) {
            highest = e.row[k];
            m.row_ptr.push_back((int)k + 1);
        }
    m.row_ptr.push_back((int)e.row.size() + 1);
    return m;
}

// assemble_simetric_csr_matrix (csr_formatter.h:146-183): every entry (r, c) is listed under row c (neighbor r) and, when
// r != c, under row r (neighbor c); rows 1..M in turn, each in file order; ids stay 1-based; row_ptr has M + 2 entries, the
// last one being the entry count + 1.  One pass over the entries per row in the reference; here one bucket per row.
inline CSR assemble_simetric_csr_matrix(std::string filePath)
{
    const mgg_mtx_entries e = mgg_read_mtx_entries(filePath);
    const int M = std::max(e.M, 0);
    std::vector<int> count((size_t)M + 2, 0);
    const auto inside = [&](int v) { return v >= 1 && v <= M; };
    for (size_t k = 0; k < e.row.size(); ++k) {
        if (inside(e.col[k])) ++count[(size_t)e.col[k]];
        if (e.row[k] != e.col[k] && inside(e.row[k])) ++count[(size_t)e.row[k]];
    }
    CSR m;
    m.row_ptr.assign((size_t)M + 1, 0);
    for (int l = 1; l <= M; ++l) m.row_ptr[(size_t)l] = m.row_ptr[(size_t)l - 1] + count[(size_t)l];
    const size_t total = (size_t)m.row_ptr[(size_t)M];
    m.col_ind.assign(total, 0);
    m.val.assign(total, 0.0);
    std::vector<int> at(m.row_ptr.begin(), m.row_ptr.end());
    for (size_t k = 0; k < e.row.size(); ++k) {
        if (inside(e.col[k])) {
            const size_t w = (size_t)at[(size_t)e.col[k] - 1]++;
            m.col_ind[w] = e.row[k];
            m.val[w] = e.val[k];
        }
        if (e.row[k] != e.col[k] && inside(e.row[k])) {
            const size_t w = (size_t)at[(size_t)e.row[k] - 1]++;
            m.col_ind[w] = e.col[k];
            m.val[w] = e.val[k];
        }
    }
    m.row_ptr.push_back((int)total + 1);
    return m;
}

// getBandwidth (csr_formatter.h:65-80): the largest |col_ind[j] - i| over the rows i = 1 .. row_ptr.size() - 2 that do
// not hold exactly one entry, row i spanning col_ind[row_ptr[i-1] .. row_ptr[i]); INT_MIN when no row qualifies.
inline int getBandwidth(const CSR &csr)
{
    int best = std::numeric_limits<int>::min();
    for (size_t i = 1; i + 1 < csr.row_ptr.size(); ++i) {
        const int b = csr.row_ptr[i - 1], e = csr.row_ptr[i];
        if (e - b == 1) continue;
        for (int j = b; j < e; ++j) best = std::max(best, std::abs(csr.col_ind[(size_t)j] - (int)i));
    }
    return best;
}

// printMatrix (csr_formatter.h:31-53): the matrix as dense text, for the 1-based layout of assemble_csr_matrix: row i holds
// col_ind[row_ptr[i-1] - 1 .. row_ptr[i] - 1); a column that occurs in the row prints the next unread value, the others 0.
inline void printMatrix(const CSR &csr)
{
    size_t next_val = 0;
    const size_t n = csr.row_ptr.size();
    for (size_t i = 1; i < n; ++i) {
        const auto first = csr.col_ind.begin() + (csr.row_ptr[i - 1] - 1), last = csr.col_ind.begin() + (csr.row_ptr[i] - 1);
        for (size_t j = 1; j < n; ++j) {
            if (std::find(first, last, (int)j) == last) std::cout << '0' << ' ';
            else std::cout << csr.val[next_val++] << ' ';
        }
        std::cout << std::endl;
    }
}

#endif
