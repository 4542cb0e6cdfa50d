// Binary CSR loader with the interface of MGG_OSDI23 include/graph.h:18-37
// (constructor graph.hpp:9-130): three files -- begin positions
// (file_index_t[V+1]), adjacency (file_vert_t[E]) and weights
// (file_weight_t[E]) -- read into beg_pos / csr / weight, converted element by
// element to the in-memory types.  Prints the reference's progress lines.
// Differences, on purpose: a file that cannot be opened or is short ends the
// program with a message (the reference prints and continues into undefined
// behaviour, graph.hpp:49,75,126), and the arrays are released with free().
#ifndef MGG_GRAPH_H
#define MGG_GRAPH_H

#include <cstdio>
#include <cstdlib>
#include <iostream>
#include <sys/stat.h>
#include <sys/time.h>

inline double wtime()
{
    struct timeval t;
    gettimeofday(&t, NULL);
    return (double)t.tv_sec + (double)t.tv_usec * 1.0e-6;
}

inline off_t fsize(const char *filename)
{
    struct stat st;
    if (stat(filename, &st) == 0) return st.st_size;
    return -1;
}

template <typename file_vert_t, typename file_index_t, typename file_weight_t,
          typename new_vert_t, typename new_index_t, typename new_weight_t>
class graph {
  public:
    new_index_t *beg_pos = nullptr;
    new_vert_t *csr = nullptr;
    new_vert_t *weight = nullptr;  // typed as the reference types it (graph.h:27)
    new_index_t vert_count = 0;
    new_index_t edge_count = 0;

    graph() {}
    ~graph() {}
    graph(const char *beg_file, const char *csr_file, const char *weight_file)
    {
        const double tm = wtime();
        const off_t beg_bytes = fsize(beg_file);
        if (beg_bytes < (off_t)sizeof(file_index_t)) die("beg file cannot open", beg_file);
        vert_count = (new_index_t)(beg_bytes / (off_t)sizeof(file_index_t) - 1);
        beg_pos = load<file_index_t, new_index_t>(beg_file, (size_t)vert_count + 1, "beg");
        edge_count = beg_pos[vert_count];
        std::cout << "Expected edge count: " << edge_count << "\n";
        if (!(edge_count > 0)) die("edge count must be positive in", beg_file);
        csr = load<file_vert_t, new_vert_t>(csr_file, (size_t)edge_count, "CSR");
        std::cout << edge_count << " " << edge_count << "\n";
        weight = load<file_weight_t, new_vert_t>(weight_file, (size_t)edge_count, "Weight");
        std::cout << "Graph load (success): " << vert_count << " verts, " << edge_count << " edges " << wtime() - tm
                  << " second(s)\n";
    }

  private:
    static void die(const char *what, const char *path)
    {
        std::cout << what << " " << path << "\n";
        exit(-1);
    }

    template <typename FileT, typename MemT>
    static MemT *load(const char *path, size_t count, const char *what)
    {
        FILE *f = fopen(path, "rb");
        if (!f) {
            std::cout << what << " file cannot open\n";
            exit(-1);
        }
        MemT *dst = static_cast<MemT *>(malloc(sizeof(MemT) * (count ? count : 1)));
        const size_t chunk = 1u << 20;
        FileT *buf = static_cast<FileT *>(malloc(sizeof(FileT) * chunk));
        size_t done = 0;
        while (done < count) {
            const size_t want = count - done < chunk ? count - done : chunk;
            if (fread(buf, sizeof(FileT), want, f) != want) {
                std::cout << what << " file is shorter than expected: " << path << "\n";
                exit(-1);
            }
            for (size_t i = 0; i < want; ++i) dst[done + i] = (MemT)buf[i];
            done += want;
        }
        free(buf);
        fclose(f);
        return dst;
    }
};

#endif
