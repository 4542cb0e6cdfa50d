// Host-side (CPU) half of libmggx.so: range partition, local/remote CSR split,
// neighbor-partition arrays, the binary and text graph formats, and the
// deterministic synthetic-graph and feature generators.  No GPU code here.
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <memory>
#include <new>
#include <string>
#include <vector>
#include <parallel/algorithm>
#include <omp.h>
#include <sys/stat.h>

#include "mggx_internal.h"

namespace mggx {

static thread_local char g_err[512] = "";

int fail(int code, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

}  // namespace mggx

using mggx::fail;

MGGX_EXPORT const char *mggx_last_error(void) { return mggx::g_err; }
MGGX_EXPORT const char *mggx_version(void) { return "mggx 0.1 (gfx950)"; }

// ---------------------------------------------------------------------------
// Range partition: contiguous node ranges of ceil(V/nGPU) rows per rank
// (reference: src/mgg_np_div_kernel.cu:90-95).
MGGX_EXPORT int mggx_range_partition(int num_nodes, int num_gpus, int pe, int *nodes_per_pe, int *lb, int *ub)
{
    if (num_nodes < 0 || num_gpus <= 0 || pe < 0 || pe >= num_gpus || !nodes_per_pe || !lb || !ub)
        return fail(MGGX_EINVAL, "range_partition: num_nodes=%d num_gpus=%d pe=%d", num_nodes, num_gpus, pe);
    const int64_t per = ((int64_t)num_nodes + num_gpus - 1) / num_gpus;
    const int64_t lo = per * pe;
    *nodes_per_pe = (int)per;
    *lb = (int)lo;
    *ub = (int)std::min<int64_t>(lo + per, num_nodes);  // may fall below lb for a trailing empty rank, as in the reference
    return MGGX_OK;
}

// ---------------------------------------------------------------------------
// Local/remote split of the rows [lb,ub) (reference: split_CSR,
// include/neighbor_utils.cuh:381-405).  Counting pass, then an order-preserving
// fill; both pointer arrays are 0-based over the share's rows.
MGGX_EXPORT int mggx_split_csr(const int *ptr, const int *col, int lb, int ub,
                               int *local_ptr, int *remote_ptr, int *local_col, int *remote_col,
                               int64_t *n_local, int64_t *n_remote)
{
    if (!ptr || !col || lb < 0 || ub < lb)
        return fail(MGGX_EINVAL, "split_csr: ptr/col NULL or bad range [%d,%d)", lb, ub);
    const int rows = ub - lb;
    int64_t total_local = 0, total_remote = 0;
    const bool fill = local_ptr && remote_ptr && local_col && remote_col;
    if (fill) { local_ptr[0] = 0; remote_ptr[0] = 0; }
    for (int r = 0; r < rows; ++r) {
        const int beg = ptr[lb + r], end = ptr[lb + r + 1];
        if (end < beg) return fail(MGGX_EFORMAT, "split_csr: row pointer decreases at row %d", lb + r);
        for (int e = beg; e < end; ++e) {
            const int u = col[e];
            const bool is_local = (u >= lb) & (u < ub);
            if (fill) {
                if (is_local) local_col[total_local] = u;
                else remote_col[total_remote] = u;
            }
            total_local += is_local;
            total_remote += !is_local;
        }
        if (total_local > std::numeric_limits<int>::max() || total_remote > std::numeric_limits<int>::max())
            return fail(MGGX_ELIMIT, "split_csr: more than 2^31-1 edges on one side");
        if (fill) { local_ptr[r + 1] = (int)total_local; remote_ptr[r + 1] = (int)total_remote; }
    }
    if (n_local) *n_local = total_local;
    if (n_remote) *n_remote = total_remote;
    return MGGX_OK;
}

// ---------------------------------------------------------------------------
// Compact staging of the remote rows.  The reference fetches every remote neighbor with its own GET
// (include/neighbor_utils.cuh:1432-1452); a share only ever touches the distinct ids in remote_col, so the staged
// table needs one row per distinct id.  They are ordered most-referenced first (ties by ascending id), which packs
// the hot rows into the same cache lines, and remote_col is rewritten to positions in that order.
MGGX_EXPORT int mggx_compact_remote(const int *remote_col, int64_t n_remote, int *remote_col_compact, int *fetch_ids,
                                    int64_t *n_unique)
{
    if (n_remote < 0 || (n_remote && !remote_col)) return fail(MGGX_EINVAL, "compact_remote: bad remote_col");
    if (n_remote > std::numeric_limits<int>::max()) return fail(MGGX_ELIMIT, "compact_remote: more than 2^31-1 edges");
    try {
        std::vector<int> sorted(remote_col, remote_col + n_remote);
        __gnu_parallel::sort(sorted.begin(), sorted.end());
        std::vector<int> ids, cnt;
        for (int64_t i = 0; i < n_remote;) {
            int64_t j = i;
            while (j < n_remote && sorted[j] == sorted[i]) ++j;
            if (sorted[i] < 0) return fail(MGGX_EFORMAT, "compact_remote: negative neighbor id %d", sorted[i]);
            ids.push_back(sorted[i]);
            cnt.push_back((int)(j - i));
            i = j;
        }
        const int64_t u = (int64_t)ids.size();
        if (n_unique) *n_unique = u;
        if (!remote_col_compact && !fetch_ids) return MGGX_OK;
        if (!remote_col_compact || !fetch_ids) return fail(MGGX_EINVAL, "compact_remote: pass both output arrays or neither");
        std::vector<int> order((size_t)u);
        for (int64_t i = 0; i < u; ++i) order[(size_t)i] = (int)i;
        __gnu_parallel::stable_sort(order.begin(), order.end(), [&](int x, int y) { return cnt[(size_t)x] > cnt[(size_t)y]; });
        std::vector<int> rank((size_t)u);  // position in staging order of the i-th smallest id
        for (int64_t pos = 0; pos < u; ++pos) {
            rank[(size_t)order[(size_t)pos]] = (int)pos;
            fetch_ids[pos] = ids[(size_t)order[(size_t)pos]];
        }
#pragma omp parallel for schedule(static)
        for (int64_t e = 0; e < n_remote; ++e) {
            const int64_t i = std::lower_bound(ids.begin(), ids.end(), remote_col[e]) - ids.begin();
            remote_col_compact[e] = rank[(size_t)i];
        }
    } catch (const std::bad_alloc &) {
        return fail(MGGX_ENOMEM, "compact_remote: out of host memory for %lld edges", (long long)n_remote);
    }
    return MGGX_OK;
}

// ---------------------------------------------------------------------------
// Neighbor-partition arrays (reference: build_part, include/neighbor_utils.cuh:411-460).
// Partition p of node i covers edges [indptr[i] + k*ps, min(.. + ps, indptr[i+1])).
// node2part is the exclusive prefix of partition counts with the total repeated
// once more at the end (num_nodes + 2 entries).
MGGX_EXPORT int mggx_build_part(const int *indptr, int num_nodes, int part_size, int compat,
                                int *part_ptr, int *part2node, int *node2part, int *num_parts)
{
    if (!indptr || num_nodes < 0 || part_size <= 0 || !num_parts)
        return fail(MGGX_EINVAL, "build_part: indptr NULL, num_nodes=%d, part_size=%d", num_nodes, part_size);
    int64_t total = 0;
    if (node2part) node2part[0] = 0;
    for (int i = 0; i < num_nodes; ++i) {
        const int64_t deg = (int64_t)indptr[i + 1] - indptr[i];
        if (deg < 0) return fail(MGGX_EFORMAT, "build_part: indptr decreases at node %d", i);
        total += (deg + part_size - 1) / part_size;
        if (total > std::numeric_limits<int>::max()) return fail(MGGX_ELIMIT, "build_part: too many partitions");
        if (node2part) node2part[i + 1] = (int)total;
    }
    if (node2part) node2part[num_nodes + 1] = (int)total;
    *num_parts = (int)total;
    if (!part_ptr || !part2node) return MGGX_OK;

    int p = 0;
    for (int i = 0; i < num_nodes; ++i) {
        for (int beg = indptr[i]; beg < indptr[i + 1]; beg += part_size) {
            part_ptr[p] = beg;
            part2node[p] = i;
            ++p;
        }
    }
    // Terminal entry.  The reference only writes it while visiting the last node,
    // so it stays at its zero initialisation when that node has no neighbors.
    const bool last_has_parts = num_nodes > 0 && indptr[num_nodes] > indptr[num_nodes - 1];
    part_ptr[p] = (compat && !last_has_parts) ? 0 : (num_nodes > 0 ? indptr[num_nodes] : 0);
    return MGGX_OK;
}

// ---------------------------------------------------------------------------
// Binary CSR files (reference: include/graph.hpp:9-130, graph<long,long,int,int,int,int>).
static int64_t file_size(const char *path)
{
    struct stat st;
    return stat(path, &st) == 0 ? (int64_t)st.st_size : -1;
}

template <typename FileT>
static int read_narrow(const char *path, int64_t count, int *dst, const char *what)
{
    FILE *f = fopen(path, "rb");
    if (!f) return fail(MGGX_EIO, "graph_read: %s file cannot open: %s", what, path);
    const size_t chunk = 1u << 20;
    std::vector<FileT> buf(std::min<int64_t>(count, (int64_t)chunk));
    int64_t done = 0;
    while (done < count) {
        const size_t want = (size_t)std::min<int64_t>(count - done, (int64_t)chunk);
        if (fread(buf.data(), sizeof(FileT), want, f) != want) {
            fclose(f);
            return fail(MGGX_EIO, "graph_read: short read in %s file %s", what, path);
        }
        for (size_t i = 0; i < want; ++i) dst[done + i] = (int)buf[i];
        done += (int64_t)want;
    }
    fclose(f);
    return MGGX_OK;
}

MGGX_EXPORT int mggx_graph_read(const char *beg_file, const char *csr_file, const char *weight_file,
                                int *vert_count, int *edge_count, int *beg_pos, int *csr, int *weight)
{
    if (!beg_file || !vert_count || !edge_count) return fail(MGGX_EINVAL, "graph_read: NULL argument");
    const int64_t bytes = file_size(beg_file);
    if (bytes < 0) return fail(MGGX_EIO, "graph_read: beg file cannot open: %s", beg_file);
    if (bytes < (int64_t)sizeof(int64_t) || bytes % (int64_t)sizeof(int64_t))
        return fail(MGGX_EFORMAT, "graph_read: %s is not a whole number of int64", beg_file);
    const int64_t verts = bytes / (int64_t)sizeof(int64_t) - 1;
    // edge count = last entry of the beg file
    int64_t last = 0;
    {
        FILE *f = fopen(beg_file, "rb");
        if (!f) return fail(MGGX_EIO, "graph_read: beg file cannot open: %s", beg_file);
        if (fseek(f, (long)(verts * (int64_t)sizeof(int64_t)), SEEK_SET) != 0 ||
            fread(&last, sizeof(int64_t), 1, f) != 1) {
            fclose(f);
            return fail(MGGX_EIO, "graph_read: short read in beg file %s", beg_file);
        }
        fclose(f);
    }
    if (last <= 0) return fail(MGGX_EFORMAT, "graph_read: edge count %lld must be positive", (long long)last);
    if (verts > std::numeric_limits<int>::max() || last > std::numeric_limits<int>::max())
        return fail(MGGX_ELIMIT, "graph_read: graph exceeds int32 indexing");
    *vert_count = (int)verts;
    *edge_count = (int)last;
    if (beg_pos) {
        int rc = read_narrow<int64_t>(beg_file, verts + 1, beg_pos, "beg");
        if (rc) return rc;
    }
    if (csr) {
        if (!csr_file) return fail(MGGX_EINVAL, "graph_read: csr file name NULL");
        if (file_size(csr_file) != last * (int64_t)sizeof(int64_t))
            return fail(MGGX_EFORMAT, "graph_read: %s does not hold %lld int64 entries", csr_file, (long long)last);
        int rc = read_narrow<int64_t>(csr_file, last, csr, "CSR");
        if (rc) return rc;
    }
    if (weight) {
        if (!weight_file) return fail(MGGX_EINVAL, "graph_read: weight file name NULL");
        if (file_size(weight_file) != last * (int64_t)sizeof(int32_t))
            return fail(MGGX_EFORMAT, "graph_read: %s does not hold %lld int32 entries", weight_file, (long long)last);
        int rc = read_narrow<int32_t>(weight_file, last, weight, "Weight");
        if (rc) return rc;
    }
    return MGGX_OK;
}

template <typename FileT>
static int write_widen(const char *path, int64_t count, const int *src, int fill_value)
{
    FILE *f = fopen(path, "wb");
    if (!f) return fail(MGGX_EIO, "graph_write: cannot create %s", path);
    const size_t chunk = 1u << 20;
    std::vector<FileT> buf(std::min<int64_t>(std::max<int64_t>(count, 1), (int64_t)chunk));
    int64_t done = 0;
    while (done < count) {
        const size_t n = (size_t)std::min<int64_t>(count - done, (int64_t)chunk);
        for (size_t i = 0; i < n; ++i) buf[i] = src ? (FileT)src[done + i] : (FileT)fill_value;
        if (fwrite(buf.data(), sizeof(FileT), n, f) != n) {
            fclose(f);
            return fail(MGGX_EIO, "graph_write: short write to %s", path);
        }
        done += (int64_t)n;
    }
    fclose(f);
    return MGGX_OK;
}

MGGX_EXPORT int mggx_graph_write(const char *beg_file, const char *csr_file, const char *weight_file,
                                 int vert_count, const int *beg_pos, const int *csr, const int *weight)
{
    if (!beg_file || !csr_file || !weight_file || !beg_pos || !csr || vert_count < 0)
        return fail(MGGX_EINVAL, "graph_write: NULL argument");
    const int64_t edges = beg_pos[vert_count];
    int rc = write_widen<int64_t>(beg_file, (int64_t)vert_count + 1, beg_pos, 0);
    if (!rc) rc = write_widen<int64_t>(csr_file, edges, csr, 0);
    if (!rc) rc = write_widen<int32_t>(weight_file, edges, weight, 1);
    return rc;
}

// ---------------------------------------------------------------------------
// Text loader (reference: assemble_csr_matrix_new, include/csr_formatter.h:112-144).
// Leading lines that start with '%' are comments; then "M N L"; then L entries
// "row col value", 1-based.  Columns keep file order; row pointers come from
// per-row counts, so the entries must be sorted by row.
MGGX_EXPORT int mggx_mtx_read(const char *path, int *num_rows, int *num_entries, int *row_ptr, int *col_ind)
{
    if (!path || !num_rows || !num_entries) return fail(MGGX_EINVAL, "mtx_read: NULL argument");
    FILE *f = fopen(path, "r");
    if (!f) return fail(MGGX_EIO, "mtx_read: cannot open %s", path);
    for (;;) {
        int ch = fgetc(f);
        if (ch != '%') {
            if (ch != EOF) ungetc(ch, f);
            break;
        }
        while ((ch = fgetc(f)) != '\n' && ch != EOF) {}
    }
    int rows = 0, cols = 0, entries = 0;
    if (fscanf(f, "%d %d %d", &rows, &cols, &entries) != 3 || rows < 0 || entries < 0) {
        fclose(f);
        return fail(MGGX_EFORMAT, "mtx_read: bad size line in %s", path);
    }
    *num_rows = rows;
    *num_entries = entries;
    if (!row_ptr && !col_ind) {
        fclose(f);
        return MGGX_OK;
    }
    std::vector<int> per_row((size_t)rows, 0);
    for (int i = 0; i < entries; ++i) {
        int r = 0, c = 0;
        double v = 0.0;
        if (fscanf(f, "%d %d %lf", &r, &c, &v) != 3) {
            fclose(f);
            return fail(MGGX_EFORMAT, "mtx_read: entry %d of %s is malformed", i, path);
        }
        if (r < 1 || r > rows) {
            fclose(f);
            return fail(MGGX_EFORMAT, "mtx_read: row index %d out of range in %s", r, path);
        }
        per_row[(size_t)r - 1]++;
        if (col_ind) col_ind[i] = c - 1;
    }
    fclose(f);
    if (row_ptr) {
        row_ptr[0] = 0;
        for (int i = 0; i < rows; ++i) row_ptr[i + 1] = row_ptr[i] + per_row[(size_t)i];
    }
    return MGGX_OK;
}

// ---------------------------------------------------------------------------
// Text edge list -> binary CSR triple.  Stands in for the reference's dataset pipeline (dataset/0_to_base_zero.py
// rewrites a .mtx to a 0-based "src dst" list, dataset/1_txt2bin.py hands it to an external text_to_bin tool that is
// not part of the reference tree).  Input: a MatrixMarket-style file (is_mtx != 0: '%' comments, a size line, then
// 1-based "row col [value]" lines) or a 0-based "src dst" list.  Output: <prefix>_beg_pos.bin / _csr.bin /
// _weight.bin in the layout mggx_graph_read expects; edges are grouped by source with a stable counting sort (file
// order is kept inside a row), weights are 1.
static int edgelist_to_bin_impl(const char *path, int is_mtx, const char *out_prefix, int *num_nodes, int64_t *num_edges)
{
    if (!path || !out_prefix) return fail(MGGX_EINVAL, "edgelist_to_bin: NULL argument");
    FILE *f = fopen(path, "r");
    if (!f) return fail(MGGX_EIO, "edgelist_to_bin: cannot open %s", path);
    struct Closer {  // closes the file on every way out, a thrown bad_alloc included
        FILE *f;
        ~Closer() { fclose(f); }
    } closer{f};
    std::vector<int> src, dst;
    long long declared_rows = 0;
    char line[512];
    bool size_line_pending = is_mtx != 0;
    while (fgets(line, sizeof(line), f)) {
        if (line[0] == '%' || line[0] == '#' || line[0] == '\n') continue;
        if (size_line_pending) {
            long long m = 0, n = 0, l = 0;
            if (sscanf(line, "%lld %lld %lld", &m, &n, &l) < 2) {
                return fail(MGGX_EFORMAT, "edgelist_to_bin: bad size line in %s", path);
            }
            declared_rows = std::max(m, n);
            if (declared_rows < 0 || declared_rows > std::numeric_limits<int>::max() - 1) {  // node ids are int32
                return fail(MGGX_ELIMIT, "edgelist_to_bin: %lld nodes declared in %s exceed int32 ids", declared_rows, path);
            }
            size_line_pending = false;
            continue;
        }
        long long a = 0, b = 0;
        if (sscanf(line, "%lld %lld", &a, &b) != 2) {
            return fail(MGGX_EFORMAT, "edgelist_to_bin: malformed line in %s: %.40s", path, line);
        }
        if (is_mtx) { --a; --b; }
        if (a < 0 || b < 0 || a > std::numeric_limits<int>::max() - 1 || b > std::numeric_limits<int>::max() - 1) {
            return fail(MGGX_EFORMAT, "edgelist_to_bin: node id out of range in %s", path);
        }
        src.push_back((int)a);
        dst.push_back((int)b);
    }
    if (src.empty()) return fail(MGGX_EFORMAT, "edgelist_to_bin: no edges in %s", path);
    if (src.size() > (size_t)std::numeric_limits<int>::max()) return fail(MGGX_ELIMIT, "edgelist_to_bin: too many edges");
    long long V = declared_rows;
    for (size_t i = 0; i < src.size(); ++i) V = std::max<long long>(V, std::max(src[i], dst[i]) + 1LL);
    if (V > std::numeric_limits<int>::max() - 1) return fail(MGGX_ELIMIT, "edgelist_to_bin: %lld nodes exceed int32 ids", V);
    std::vector<int> beg((size_t)V + 1, 0), csr(src.size());
    for (int s : src) beg[(size_t)s + 1]++;
    for (long long v = 0; v < V; ++v) beg[(size_t)v + 1] += beg[(size_t)v];
    std::vector<int> cursor(beg.begin(), beg.end() - 1);
    for (size_t i = 0; i < src.size(); ++i) csr[(size_t)cursor[(size_t)src[i]]++] = dst[i];
    const std::string p(out_prefix);
    int rc = mggx_graph_write((p + "_beg_pos.bin").c_str(), (p + "_csr.bin").c_str(), (p + "_weight.bin").c_str(), (int)V,
                              beg.data(), csr.data(), nullptr);
    if (rc) return rc;
    if (num_nodes) *num_nodes = (int)V;
    if (num_edges) *num_edges = (int64_t)src.size();
    return MGGX_OK;
}

// Allocation failures (a size line that declares billions of nodes, an edge list beyond host memory) come back as an
// error code: no exception crosses the C boundary.
MGGX_EXPORT int mggx_edgelist_to_bin(const char *path, int is_mtx, const char *out_prefix, int *num_nodes, int64_t *num_edges)
{
    try {
        return edgelist_to_bin_impl(path, is_mtx, out_prefix, num_nodes, num_edges);
    } catch (const std::bad_alloc &) {
        return fail(MGGX_ENOMEM, "edgelist_to_bin: out of host memory reading %s", path ? path : "(null)");
    }
}


// ---------------------------------------------------------------------------
// Synthetic graphs.
namespace {

struct GenResult {
    std::vector<int> row_ptr;
    std::vector<int> col;
};

// Seeded bijection on [0, 2^bits): odd multiply, xor-shift, odd multiply.
inline uint32_t scramble_id(uint32_t x, int bits, uint64_t seed)
{
    const uint32_t mask = bits >= 32 ? 0xFFFFFFFFu : ((1u << bits) - 1u);
    const uint32_t m1 = (uint32_t)(mggx::mix64(seed ^ 0x51ull) | 1ull);
    const uint32_t m2 = (uint32_t)(mggx::mix64(seed ^ 0xA7ull) | 1ull);
    const uint32_t add = (uint32_t)mggx::mix64(seed ^ 0x3Cull);
    const int sh = bits > 1 ? bits / 2 : 1;
    x = (x * m1 + add) & mask;
    x ^= x >> sh;
    x = (x * m2) & mask;
    x ^= x >> sh;
    return x & mask;
}

// Sorted, duplicate-free CSR over rows [row_lo,row_hi) from directed keys (row<<32 | col).
int keys_to_csr(std::vector<uint64_t> &keys, int row_lo, int row_hi, GenResult *out)
{
    __gnu_parallel::sort(keys.begin(), keys.end());
    keys.erase(std::unique(keys.begin(), keys.end()), keys.end());
    if (keys.size() > (size_t)std::numeric_limits<int>::max())
        return fail(MGGX_ELIMIT, "generator: %zu edges exceed int32 indexing", keys.size());
    const int rows = row_hi - row_lo;
    out->row_ptr.assign((size_t)rows + 1, 0);
    out->col.resize(keys.size());
    const int64_t n = (int64_t)keys.size();
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) out->col[(size_t)i] = (int)(uint32_t)keys[(size_t)i];
    // row pointers: first key index of each row (keys are sorted by row)
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) {
        const int r = (int)(keys[(size_t)i] >> 32) - row_lo;
        const int prev = i == 0 ? -1 : (int)(keys[(size_t)i - 1] >> 32) - row_lo;
        for (int q = prev + 1; q <= r; ++q) out->row_ptr[(size_t)q] = (int)i;
    }
    const int last = n == 0 ? -1 : (int)(keys[(size_t)n - 1] >> 32) - row_lo;
    for (int q = last + 1; q <= rows; ++q) out->row_ptr[(size_t)q] = (int)n;
    return MGGX_OK;
}

}  // namespace

MGGX_EXPORT int mggx_gen_rmat(int scale, int num_nodes, int64_t num_draws, double a, double b, double c,
                              uint64_t seed, int scramble, int row_lo, int row_hi, int threads,
                              void **handle, int64_t *nnz)
{
    if (scale < 1 || scale > 31 || num_nodes < 1 || (int64_t)num_nodes > ((int64_t)1 << scale) || num_draws < 0 ||
        a <= 0 || b < 0 || c < 0 || a + b + c >= 1.0 || row_lo < 0 || row_hi < row_lo || row_hi > num_nodes ||
        !handle || !nnz)
        return fail(MGGX_EINVAL, "gen_rmat: bad argument (scale=%d nodes=%d draws=%lld rows=[%d,%d))", scale,
                    num_nodes, (long long)num_draws, row_lo, row_hi);
    const uint32_t ta = (uint32_t)std::lround(a * 65536.0);
    const uint32_t tab = (uint32_t)std::lround((a + b) * 65536.0);
    const uint32_t tabc = (uint32_t)std::lround((a + b + c) * 65536.0);
    const int nthreads = threads > 0 ? threads : omp_get_max_threads();
    std::vector<std::vector<uint64_t>> local((size_t)nthreads);
#pragma omp parallel num_threads(nthreads)
    {
        std::vector<uint64_t> &mine = local[(size_t)omp_get_thread_num()];
        mine.reserve((size_t)(num_draws / nthreads / 2 + 1024));
#pragma omp for schedule(static)
        for (int64_t i = 0; i < num_draws; ++i) {
            for (uint64_t attempt = 0; attempt < 64; ++attempt) {
                uint32_t u = 0, v = 0;
                uint64_t bits = 0;
                for (int level = 0; level < scale; ++level) {
                    if ((level & 3) == 0) bits = mggx::rnd64(seed, (uint64_t)i, attempt * 16 + (uint64_t)(level >> 2));
                    const uint32_t r = (uint32_t)(bits & 0xFFFF);
                    bits >>= 16;
                    const uint32_t ubit = r >= tab;                       // quadrants c,d -> lower half rows
                    const uint32_t vbit = (r >= ta && r < tab) || r >= tabc;  // quadrants b,d -> right half cols
                    u = (u << 1) | ubit;
                    v = (v << 1) | vbit;
                }
                if (scramble) {
                    u = scramble_id(u, scale, seed);
                    v = scramble_id(v, scale, seed);
                }
                if (u >= (uint32_t)num_nodes || v >= (uint32_t)num_nodes || u == v) continue;
                if ((int)u >= row_lo && (int)u < row_hi) mine.push_back(((uint64_t)u << 32) | v);
                if ((int)v >= row_lo && (int)v < row_hi) mine.push_back(((uint64_t)v << 32) | u);
                break;
            }
        }
    }
    size_t total = (size_t)(row_hi - row_lo);
    for (auto &v : local) total += v.size();
    std::vector<uint64_t> keys;
    keys.reserve(total);
    for (auto &v : local) {
        keys.insert(keys.end(), v.begin(), v.end());
        std::vector<uint64_t>().swap(v);
    }
    for (int r = row_lo; r < row_hi; ++r) keys.push_back(((uint64_t)(uint32_t)r << 32) | (uint32_t)r);  // self loops
    std::unique_ptr<GenResult> res(new (std::nothrow) GenResult);
    if (!res) return fail(MGGX_ENOMEM, "gen_rmat: out of memory");
    int rc = keys_to_csr(keys, row_lo, row_hi, res.get());
    if (rc) return rc;
    *nnz = (int64_t)res->col.size();
    *handle = res.release();
    return MGGX_OK;
}

MGGX_EXPORT int mggx_gen_er(int num_nodes, double avg_degree, uint64_t seed, void **handle, int64_t *nnz)
{
    if (num_nodes < 2 || avg_degree < 0 || !handle || !nnz)
        return fail(MGGX_EINVAL, "gen_er: num_nodes=%d avg_degree=%g", num_nodes, avg_degree);
    const double p = std::min(1.0, avg_degree / (double)(num_nodes - 1));
    std::vector<uint64_t> keys;
    const int64_t pairs = (int64_t)num_nodes * (num_nodes - 1) / 2;
    keys.reserve((size_t)(p * (double)pairs * 2.2) + (size_t)num_nodes + 16);
    // Geometric skipping over the unordered pairs (u < v) in row-major order.
    if (p > 0) {
        const double log1mp = p < 1.0 ? std::log1p(-p) : 0.0;
        int64_t idx = -1;
        int u = 0;
        int64_t row_start = 0;  // index of pair (u, u+1)
        for (uint64_t k = 0;; ++k) {
            int64_t skip = 0;
            if (p < 1.0) {
                const double x = ((double)(mggx::rnd64(seed, k, 0) >> 11) + 0.5) * (1.0 / 9007199254740992.0);
                skip = (int64_t)std::floor(std::log(x) / log1mp);
            }
            idx += skip + 1;
            if (idx >= pairs || idx < 0) break;
            while (idx >= row_start + (num_nodes - 1 - u)) {
                row_start += num_nodes - 1 - u;
                ++u;
            }
            const int v = u + 1 + (int)(idx - row_start);
            keys.push_back(((uint64_t)(uint32_t)u << 32) | (uint32_t)v);
            keys.push_back(((uint64_t)(uint32_t)v << 32) | (uint32_t)u);
        }
    }
    for (int r = 0; r < num_nodes; ++r) keys.push_back(((uint64_t)(uint32_t)r << 32) | (uint32_t)r);
    std::unique_ptr<GenResult> res(new (std::nothrow) GenResult);
    if (!res) return fail(MGGX_ENOMEM, "gen_er: out of memory");
    int rc = keys_to_csr(keys, 0, num_nodes, res.get());
    if (rc) return rc;
    *nnz = (int64_t)res->col.size();
    *handle = res.release();
    return MGGX_OK;
}

MGGX_EXPORT int mggx_gen_fetch(void *handle, int *row_ptr, int *col)
{
    if (!handle) return fail(MGGX_EINVAL, "gen_fetch: NULL handle");
    std::unique_ptr<GenResult> res(static_cast<GenResult *>(handle));
    if (row_ptr) memcpy(row_ptr, res->row_ptr.data(), res->row_ptr.size() * sizeof(int));
    if (col) memcpy(col, res->col.data(), res->col.size() * sizeof(int));
    return MGGX_OK;
}

MGGX_EXPORT int mggx_fill_normal(float *dst, int64_t n, uint64_t seed)
{
    if (!dst || n < 0) return fail(MGGX_EINVAL, "fill_normal: NULL or negative size");
    const int64_t pairs = (n + 1) / 2;
#pragma omp parallel for schedule(static)
    for (int64_t k = 0; k < pairs; ++k) {
        const uint64_t r1 = mggx::rnd64(seed, (uint64_t)k, 1), r2 = mggx::rnd64(seed, (uint64_t)k, 2);
        const double u1 = ((double)(r1 >> 11) + 0.5) * (1.0 / 9007199254740992.0);
        const double u2 = ((double)(r2 >> 11) + 0.5) * (1.0 / 9007199254740992.0);
        const double rad = std::sqrt(-2.0 * std::log(u1));
        const double ang = 6.283185307179586476925 * u2;
        dst[2 * k] = (float)(rad * std::cos(ang));
        if (2 * k + 1 < n) dst[2 * k + 1] = (float)(rad * std::sin(ang));
    }
    return MGGX_OK;
}

MGGX_EXPORT int mggx_fill_uniform(float *dst, int64_t n, float lo, float hi, uint64_t seed)
{
    if (!dst || n < 0) return fail(MGGX_EINVAL, "fill_uniform: NULL or negative size");
#pragma omp parallel for schedule(static)
    for (int64_t k = 0; k < n; ++k) {
        const double u = (double)(mggx::rnd64(seed, (uint64_t)k, 3) >> 11) * (1.0 / 9007199254740992.0);
        dst[k] = (float)((double)lo + ((double)hi - (double)lo) * u);
    }
    return MGGX_OK;
}


// ---------------------------------------------------------------------------
// Dense-core layout (see mggx_internal.h).
namespace mggx {

// The lists of every (slice, tile) block in bank order, as k_core_bank_order leaves them on the GPU.  The 16 lanes of a
// group are placed together: position by position, first the lanes without padding left to spend, then the others, each
// in lane order, a lane takes the first of its remaining entries (looking from residue (lane + p) mod 16 upwards, edge
// order inside a residue) whose residue no lane of the group has taken at this position; a lane that finds none spends
// a padding slot if it has one, else takes a residue twice.  Padding slots become tc + r, r being the residues still
// free at that position in turn (the k-th padding lane of the group takes the k-th free one, or k mod 16).
static int first_from(unsigned m, int k)
{
    const unsigned mr = ((m >> k) | (m << (16 - k))) & 0xFFFFu;
    return mr ? ((__builtin_ctz(mr) + k) & 15) : -1;
}

void core_bank_order(unsigned short *idx, const unsigned *blk_off, size_t cells, int tc)
{
#pragma omp parallel for schedule(dynamic, 64)
    for (long long cell = 0; cell < (long long)cells; ++cell) {
        const unsigned b0 = blk_off[cell], b1 = blk_off[cell + 1];
        const int P = 4 * (int)(b1 - b0);
        if (P == 0) continue;
        auto at = [&](int p, int lane) -> unsigned short & { return idx[((size_t)(b0 + p / 4) * 64 + lane) * 4 + (p % 4)]; };
        if (P > 256) {  // as on the GPU: such a block keeps its edge order, its padding points at the first zero column
            for (int p = 0; p < P; ++p)
                for (int lane = 0; lane < 64; ++lane)
                    if (at(p, lane) == 0xFFFF) at(p, lane) = (unsigned short)tc;
            continue;
        }
        for (int grp = 0; grp < 4; ++grp) {
            std::vector<unsigned short> q[16][16];  // [lane of the group][residue]: entries in edge order
            size_t head[16][16] = {};
            int left[16];
            unsigned have[16];
            for (int i = 0; i < 16; ++i) {
                left[i] = 0;
                have[i] = 0;
                for (int p = 0; p < P; ++p) {
                    const unsigned short v = at(p, 16 * grp + i);
                    if (v != 0xFFFF) {
                        q[i][v & 15].push_back(v);
                        have[i] |= 1u << (v & 15);
                        ++left[i];
                    }
                }
            }
            for (int p = 0; p < P; ++p) {
                unsigned used = 0;
                int r[16];
                for (int i = 0; i < 16; ++i) r[i] = -1;
                for (int pass = 0; pass < 2; ++pass)
                    for (int i = 0; i < 16; ++i) {
                        const int slack = P - p - left[i];
                        if (left[i] == 0 || (slack == 0) != (pass == 0)) continue;
                        const int k0 = (i + p) & 15;
                        int rr = first_from(have[i] & ~used, k0);
                        if (rr < 0 && slack == 0) rr = first_from(have[i], k0);
                        r[i] = rr;
                        if (rr >= 0) used |= 1u << rr;
                    }
                int k = 0;
                for (int i = 0; i < 16; ++i) {
                    if (r[i] >= 0) {
                        at(p, 16 * grp + i) = q[i][r[i]][head[i][r[i]]++];
                        if (head[i][r[i]] == q[i][r[i]].size()) have[i] &= ~(1u << r[i]);
                        --left[i];
                    } else {
                        unsigned f = ~used & 0xFFFFu;
                        for (int t = 0; t < k && f; ++t) f &= f - 1;
                        at(p, 16 * grp + i) = (unsigned short)(tc + (f ? __builtin_ctz(f) : (k & 15)));
                        ++k;
                    }
                }
            }
        }
    }
}

int core_layout_build(const int *ptr, const int *col, int rows, int lb, int core, int tc, CoreLayout *out)
{
    if (!ptr || rows < 0 || tc < 64 || tc > 4096 || (tc % 64)) return fail(MGGX_EINVAL, "core layout: bad arguments");
    if (core > rows) core = rows;
    const int unit = tc > 512 ? tc : 512;  // whole workgroups of 8 slices and whole tiles
    core = core / unit * unit;
    if (core < unit || (unit % tc) || (unit % 512)) return fail(MGGX_EINVAL, "core layout: no core of whole %d-row units in %d rows", unit, rows);
    if (ptr[rows] > 0 && !col) return fail(MGGX_EINVAL, "core layout: NULL column array");
    CoreLayout &L = *out;
    L.rows = rows;
    L.core = core;
    L.tc = tc;
    L.ntiles = core / tc;
    const int ntiles = L.ntiles, nslices = core / 64;
    // rank by degree, ties by id
    std::vector<int> ids((size_t)rows);
    for (int v = 0; v < rows; ++v) ids[v] = v;
    __gnu_parallel::stable_sort(ids.begin(), ids.end(), [&](int a, int b) { return ptr[a + 1] - ptr[a] > ptr[b + 1] - ptr[b]; });
    L.order.assign(ids.begin(), ids.begin() + core);
    L.rank.assign((size_t)rows, -1);
    for (int i = 0; i < core; ++i) L.rank[L.order[i]] = i;
    // pass 1: list lengths per (core row, tile); what every row keeps
    std::vector<unsigned short> cnt((size_t)core * ntiles, 0);
    L.rem_ptr.assign((size_t)rows + 1, 0);
    int bad = 0;
#pragma omp parallel for schedule(dynamic, 256) reduction(| : bad)
    for (int v = 0; v < rows; ++v) {
        const int i = L.rank[v];
        int keep = 0;
        for (int e = ptr[v]; e < ptr[v + 1]; ++e) {
            const int u = col[e] - lb;
            if (u < 0 || u >= rows) { bad = 1; ++keep; continue; }
            const int j = L.rank[u];
            if (i >= 0 && j >= 0) {
                unsigned short &c = cnt[(size_t)i * ntiles + j / tc];
                if (c == 0xFFFE) { bad = 1; ++keep; continue; }  // a list that long cannot be a simple graph's
                ++c;
            } else {
                ++keep;
            }
        }
        L.rem_ptr[v + 1] = keep;
    }
    if (bad) return fail(MGGX_EINVAL, "core layout: a neighbor id outside [lb, lb + rows), or more than 65533 parallel edges");
    for (int v = 0; v < rows; ++v) L.rem_ptr[v + 1] += L.rem_ptr[v];
    // block offsets
    L.blk_off.assign((size_t)nslices * ntiles + 1, 0);
    uint64_t chunks = 0;
    for (int g = 0; g < nslices; ++g)
        for (int t = 0; t < ntiles; ++t) {
            int w = 0;
            for (int l = 0; l < 64; ++l) w = std::max<int>(w, cnt[(size_t)(g * 64 + l) * ntiles + t]);
            L.blk_off[(size_t)g * ntiles + t] = (unsigned)chunks;
            chunks += (uint64_t)(w + 3) / 4;
        }
    if (chunks > 0xFFFFFFFFull / 64) return fail(MGGX_ELIMIT, "core layout: %llu list chunks", (unsigned long long)chunks);
    L.blk_off[(size_t)nslices * ntiles] = (unsigned)chunks;
    L.idx.assign((size_t)chunks * 256, (unsigned short)0xFFFF);
    L.rem_col.assign((size_t)L.rem_ptr[rows], 0);
    // pass 2: fill
    int64_t core_nnz = 0;
#pragma omp parallel reduction(+ : core_nnz)
    {
        std::vector<int> cur((size_t)ntiles);
#pragma omp for schedule(dynamic, 256)
        for (int v = 0; v < rows; ++v) {
            const int i = L.rank[v];
            int w = L.rem_ptr[v];
            if (i >= 0) std::fill(cur.begin(), cur.end(), 0);
            for (int e = ptr[v]; e < ptr[v + 1]; ++e) {
                const int u = col[e] - lb;
                const int j = L.rank[u];
                if (i >= 0 && j >= 0) {
                    const int t = j / tc, k = cur[t]++;
                    const size_t chunk = (size_t)L.blk_off[(size_t)(i / 64) * ntiles + t] + (size_t)(k / 4);
                    L.idx[(chunk * 64 + (size_t)(i % 64)) * 4 + (size_t)(k % 4)] = (unsigned short)(j % tc);
                    ++core_nnz;
                } else {
                    L.rem_col[w++] = col[e];
                }
            }
        }
    }
    L.core_nnz = core_nnz;
    core_bank_order(L.idx.data(), L.blk_off.data(), (size_t)nslices * ntiles, tc);
    return MGGX_OK;
}

}  // namespace mggx

MGGX_EXPORT int mggx_core_layout_build(const int *ptr, const int *col, int rows, int lb, int core_rows, int tile_cols, void **handle,
                                       int64_t *sizes)
{
    if (!handle || !sizes) return fail(MGGX_EINVAL, "core_layout_build: NULL output");
    std::unique_ptr<mggx::CoreLayout> L(new (std::nothrow) mggx::CoreLayout);
    if (!L) return fail(MGGX_ENOMEM, "core_layout_build");
    int rc;
    try {
        rc = mggx::core_layout_build(ptr, col, rows, lb, core_rows, tile_cols, L.get());
    } catch (const std::bad_alloc &) {
        return fail(MGGX_ENOMEM, "core_layout_build: out of host memory");
    }
    if (rc) return rc;
    sizes[0] = L->core;
    sizes[1] = (int64_t)L->blk_off.size();
    sizes[2] = (int64_t)L->idx.size();
    sizes[3] = (int64_t)L->rem_col.size();
    sizes[4] = L->core_nnz;
    *handle = L.release();
    return MGGX_OK;
}

MGGX_EXPORT int mggx_core_layout_fetch(void *handle, int *order, int *rank, unsigned *blk_off, unsigned short *idx, int *rem_ptr, int *rem_col)
{
    if (!handle) return fail(MGGX_EINVAL, "core_layout_fetch: NULL handle");
    std::unique_ptr<mggx::CoreLayout> L(static_cast<mggx::CoreLayout *>(handle));
    if (order) memcpy(order, L->order.data(), L->order.size() * sizeof(int));
    if (rank) memcpy(rank, L->rank.data(), L->rank.size() * sizeof(int));
    if (blk_off) memcpy(blk_off, L->blk_off.data(), L->blk_off.size() * sizeof(unsigned));
    if (idx) memcpy(idx, L->idx.data(), L->idx.size() * sizeof(unsigned short));
    if (rem_ptr) memcpy(rem_ptr, L->rem_ptr.data(), L->rem_ptr.size() * sizeof(int));
    if (rem_col && !L->rem_col.empty()) memcpy(rem_col, L->rem_col.data(), L->rem_col.size() * sizeof(int));
    return MGGX_OK;
}
