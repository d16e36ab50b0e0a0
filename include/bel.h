/*
 * Graph files as the reference's graph benchmarks read them (benchmarks/bfs/main.cu:1238-1284; the same reader is in
 * benchmarks/cc, pagerank, sssp): for a graph stored under the name <f>,
 *
 *   <f>.col   u64 n (= V + 1), u64 ignored, then n offsets, u64 each
 *   <f>.dst   u64 E,            u64 ignored, then E neighbour ids, u64 each
 *
 * all little-endian.  On the backing store only the payload of <f>.dst lives (the 16-byte header is skipped when the
 * file is copied there), from a page-aligned byte offset on.
 */
#ifndef __BAM_BEL_H__
#define __BAM_BEL_H__
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

#define BEL_HEADER_BYTES 16

/* sizes from the two headers: n_offsets = V + 1, n_edges = E; 0 or errno */
int bel_info(const char* prefix, uint64_t* n_offsets, uint64_t* n_edges);
/* the n_offsets offsets of <prefix>.col into out; checks that they are non-decreasing and end at E */
int bel_read_offsets(const char* prefix, uint64_t* out, uint64_t n_offsets);
/* `count` neighbour ids from edge index `first` on */
int bel_read_edges(const char* prefix, uint64_t first, uint64_t count, uint64_t* out);
/* write both files */
int bel_write(const char* prefix, const uint64_t* offsets, uint64_t n_offsets, const uint64_t* edges, uint64_t n_edges);

#ifdef __cplusplus
}
#endif
#endif /* __BAM_BEL_H__ */
