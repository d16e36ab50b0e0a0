// Reader and writer of the graph file pair described in include/bel.h.
#include "bel.h"
#include <cerrno>
#include <cstdio>
#include <string>
#include <vector>

namespace {
struct File {
    FILE* f;
    File(const std::string& path, const char* mode) : f(fopen(path.c_str(), mode)) {}
    ~File() { if (f) fclose(f); }
    File(const File&) = delete;
    File& operator=(const File&) = delete;
};

int read_header(const std::string& path, uint64_t* first_word)
{
    File in(path, "rb");
    if (!in.f) return errno ? errno : ENOENT;
    uint64_t h[2];
    if (fread(h, sizeof(uint64_t), 2, in.f) != 2) return EIO;
    *first_word = h[0];
    return 0;
}

int read_words(const std::string& path, uint64_t first, uint64_t count, uint64_t* out)
{
    File in(path, "rb");
    if (!in.f) return errno ? errno : ENOENT;
    if (fseeko(in.f, (off_t)(BEL_HEADER_BYTES + first * sizeof(uint64_t)), SEEK_SET)) return errno;
    if (count && fread(out, sizeof(uint64_t), count, in.f) != count) return EIO;
    return 0;
}

int write_file(const std::string& path, const uint64_t* words, uint64_t n)
{
    File out(path, "wb");
    if (!out.f) return errno ? errno : EIO;
    const uint64_t h[2] = {n, 0};
    if (fwrite(h, sizeof(uint64_t), 2, out.f) != 2) return EIO;
    if (n && fwrite(words, sizeof(uint64_t), n, out.f) != n) return EIO;
    return fflush(out.f) ? EIO : 0;
}
} // namespace

extern "C" int bel_info(const char* prefix, uint64_t* n_offsets, uint64_t* n_edges)
{
    if (!prefix || !n_offsets || !n_edges) return EINVAL;
    if (int rc = read_header(std::string(prefix) + ".col", n_offsets)) return rc;
    return read_header(std::string(prefix) + ".dst", n_edges);
}

extern "C" int bel_read_offsets(const char* prefix, uint64_t* out, uint64_t n_offsets)
{
    if (!prefix || !out) return EINVAL;
    uint64_t n = 0, e = 0;
    if (int rc = bel_info(prefix, &n, &e)) return rc;
    if (n != n_offsets || n == 0) return EINVAL;
    if (int rc = read_words(std::string(prefix) + ".col", 0, n, out)) return rc;
    for (uint64_t i = 1; i < n; i++)
        if (out[i] < out[i - 1]) return EILSEQ;
    return out[0] == 0 && out[n - 1] == e ? 0 : EILSEQ;
}

extern "C" int bel_read_edges(const char* prefix, uint64_t first, uint64_t count, uint64_t* out)
{
    if (!prefix || (!out && count)) return EINVAL;
    uint64_t e = 0;
    if (int rc = read_header(std::string(prefix) + ".dst", &e)) return rc;
    if (first > e || count > e - first) return ERANGE;
    return read_words(std::string(prefix) + ".dst", first, count, out);
}

extern "C" int bel_write(const char* prefix, const uint64_t* offsets, uint64_t n_offsets, const uint64_t* edges, uint64_t n_edges)
{
    if (!prefix || !offsets || !n_offsets || (!edges && n_edges)) return EINVAL;
    if (offsets[0] != 0 || offsets[n_offsets - 1] != n_edges) return EINVAL;
    if (int rc = write_file(std::string(prefix) + ".col", offsets, n_offsets)) return rc;
    return write_file(std::string(prefix) + ".dst", edges, n_edges);
}
