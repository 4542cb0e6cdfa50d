// Exercises the host-only parts of include/mgg/*.h that no program under harness/ instantiates: split_CSR<T> and
// build_part<T> for a T other than int (their generic branches), and csr_formatter.h's older loaders with getBandwidth and
// printMatrix.  Reads "<what> ..." from the command line, prints arrays as "name: v v v" lines; the Python test compares
// them with the reference's own host code and with the committed fixtures.
//   host_layer_check split <file>   file: "n_ptr n_col lb ub ps", then the row pointers, then the column ids
//   host_layer_check mtx <file.mtx>
#include <cstdio>
#include <fstream>
#include <iostream>
#include <string>
#include <vector>

#include "mgg/csr_formatter.h"
#include "mgg/neighbor_utils.h"

template <typename T>
static void show(const char *name, const std::vector<T> &v)
{
    std::cout << name << ":";
    for (const T &x : v) std::cout << ' ' << x;
    std::cout << '\n';
}

template <typename T>
static void split_and_part(const char *tag, const std::vector<long> &ptr, const std::vector<long> &col, long lb, long ub, long ps)
{
    std::vector<T> p(ptr.begin(), ptr.end()), c(col.begin(), col.end());
    auto s = split_CSR<T>(p, c, (T)lb, (T)ub);
    const std::string t(tag);
    show((t + "_local_ptr").c_str(), s[0]);
    show((t + "_remote_ptr").c_str(), s[1]);
    show((t + "_local_col").c_str(), s[2]);
    show((t + "_remote_col").c_str(), s[3]);
    auto b = build_part<T>("parts", s[0], (T)(ub - lb), (T)ps);
    show((t + "_partPtr").c_str(), b[0]);
    show((t + "_part2Node").c_str(), b[1]);
    show((t + "_node2Part").c_str(), b[2]);
}

int main(int argc, char **argv)
{
    if (argc < 3) return 2;
    const std::string what = argv[1];
    if (what == "split") {
        std::ifstream f(argv[2]);
        long n_ptr = 0, n_col = 0, lb = 0, ub = 0, ps = 0;
        f >> n_ptr >> n_col >> lb >> ub >> ps;
        std::vector<long> ptr((size_t)n_ptr), col((size_t)n_col);
        for (long &x : ptr) f >> x;
        for (long &x : col) f >> x;
        split_and_part<long>("long", ptr, col, lb, ub, ps);
        split_and_part<int>("int", ptr, col, lb, ub, ps);
        split_and_part<long long>("longlong", ptr, col, lb, ub, ps);
        return 0;
    }
    if (what == "mtx") {
        for (int sym = 0; sym < 2; ++sym) {
            CSR m = sym ? assemble_simetric_csr_matrix(argv[2]) : assemble_csr_matrix(argv[2]);
            const std::string t = sym ? "sym" : "old";
            show((t + "_row_ptr").c_str(), m.row_ptr);
            show((t + "_col_ind").c_str(), m.col_ind);
            show((t + "_val").c_str(), m.val);
            std::cout << t << "_bandwidth: " << getBandwidth(m) << '\n';
            CSR one_based = m;  // printMatrix reads col_ind[row_ptr[i-1] - 1 ...)
            one_based.row_ptr[0] = 1;
            std::cout << t << "_text_begin\n";
            printMatrix(one_based);
            std::cout << t << "_text_end\n";
        }
        return 0;
    }
    return 2;
}
