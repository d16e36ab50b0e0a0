/*
 * CPU oracle for the GPU-side storage-access path.  TEST INFRASTRUCTURE ONLY:
 * nothing the library ships may include, link or call this file; only the
 * test-suite, the smoke check and the CPU-baseline leg of the benchmark do.
 *
 * Every function restates, in plain C, either the synthetic-input definition
 * the benchmarks use or the algorithm of the reference at the cited lines.
 *
 * Pinning status (what each function is checked against, see tests/test_oracle.py):
 *   bo_splitmix64            published SplitMix64 vectors (seed 1234567, seed 0)
 *   bo_store_sum             closed-form sums for the 2^24-element reduction
 *   bo_cmd_*                 NVMe 1.x SQE byte images
 *   bo_bfs_levels            reference sample graph (bfs/main.cu:1262-1263) + scipy BFS
 *   bo_cc_labels             reference sample graph + scipy connected_components
 *   bo_rmat_edges/bo_uniform_edges/bo_build_csr   independent numpy restatement
 *   bo_sssp_costs            hand-computed weighted graph + scipy dijkstra + the independent sweep bo_sssp_costs_sweep
 *   bo_sssp_costs_float      hand-computed graph whose sums round (2^24 + 1, 0.1f + 0.2f) + scipy dijkstra on weights that add exactly +
 *                            the independent sweep bo_sssp_costs_float_sweep + a numpy float32 relaxation
 *   bo_reduce_blocks/bo_scan numpy sums and cumsum, closed form n(n+1)/2 on 0..n-1, wrap-around mod 2^64
 *   bo_pagerank              hand-computed first sweeps on a 3-vertex path; sparse solve of (I - alpha P^T) x = (1 - alpha)
 *                            (scipy, double) with the bound 0 <= x - value <= x tolerance / (1 - alpha); bo_pagerank_limit
 *                            against the same solve
 *   cpu path (cpu_path.c)    closed-form sums + counter invariants of the
 *                            reference logs; simt::atomic semantics: parity unpinned
 */
#ifndef BAM_ORACLE_H
#define BAM_ORACLE_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

#define BO_INF32 0xFFFFFFFFu

uint64_t bo_splitmix64(uint64_t seed, uint64_t i);
void     bo_fill_store(uint64_t seed, uint64_t first, uint64_t n, uint64_t* out);
uint64_t bo_store_sum(uint64_t seed, uint64_t first, uint64_t stride, uint64_t count);
void     bo_gather_indices(uint64_t seed, uint64_t first_k, uint64_t n, uint64_t n_elems, uint64_t* out);
uint64_t bo_gather_sum(uint64_t store_seed, uint64_t idx_seed, uint64_t first_k, uint64_t n, uint64_t n_elems);
void     bo_block_lbas(uint64_t seed, uint64_t first_k, uint64_t n, uint64_t ns_bytes, uint32_t req_bytes, uint32_t lba_bytes, uint64_t* out);
uint64_t bo_block_checksum(uint64_t store_seed, uint64_t lba, uint32_t lba_bytes, uint32_t req_bytes);

void     bo_rmat_edges(uint64_t seed, uint32_t scale, uint64_t first_edge, uint64_t n, uint64_t* u, uint64_t* v);
void     bo_uniform_edges(uint64_t seed, uint64_t n_vertices, uint64_t first_pair, uint64_t n, uint64_t* u, uint64_t* v);
/* symmetrize, drop self loops, sort, dedup; offsets has n_vertices+1 entries, neigh must hold 2*n_pairs. returns E */
uint64_t bo_build_csr(uint64_t n_vertices, uint64_t n_pairs, const uint64_t* u, const uint64_t* v, uint64_t* offsets, uint64_t* neigh);
void     bo_bfs_sources(uint64_t seed, uint64_t n_vertices, const uint64_t* offsets, uint32_t n_src, uint64_t* out);

/* returns the number of kernel launches the reference host loop would make */
uint32_t bo_bfs_levels(uint64_t n_vertices, const uint64_t* offsets, const uint64_t* neigh, uint64_t src, uint32_t* levels);
uint32_t bo_bfs_levels_sweep(uint64_t n_vertices, const uint64_t* offsets, const uint64_t* neigh, uint64_t src, uint32_t* levels);
/* returns number of components */
uint64_t bo_cc_labels(uint64_t n_vertices, const uint64_t* offsets, const uint64_t* neigh, uint64_t* labels);
uint64_t bo_cc_labels_sweep(uint64_t n_vertices, const uint64_t* offsets, const uint64_t* neigh, uint64_t* labels, uint32_t* iters);
uint64_t bo_bfs_edges_scanned(uint64_t n_vertices, const uint64_t* offsets, const uint32_t* levels);

/* edge weights of the synthetic weighted graphs: weight of CSR entry e = 1 + splitmix64(seed ^ 0x3e16, e) mod 255 */
void     bo_edge_weights(uint64_t seed, uint64_t first, uint64_t n, uint32_t* out);
/* single-source shortest paths, 32-bit costs (benchmarks/sssp/main.cu:69, 174-201, 282-292: the fixed point of its
 * relax + update rounds); unreachable = BO_INF32.  Dijkstra with a binary heap; the sweep is plain Bellman-Ford rounds
 * and returns how many rounds changed something. */
void     bo_sssp_costs(uint64_t n_vertices, const uint64_t* offsets, const uint64_t* neigh, const uint32_t* weights, uint64_t src, uint32_t* costs);
uint32_t bo_sssp_costs_sweep(uint64_t n_vertices, const uint64_t* offsets, const uint64_t* neigh, const uint32_t* weights, uint64_t src, uint32_t* costs);
/* the same with single-precision weights and costs (benchmarks/sssp_float/main.cu:69, 194-217, 302-312, 529): weights >= 0,
 * unreached = BO_FAR_F32; bit-exact whatever the order of relaxation (see the .c file) */
#define BO_FAR_F32 1000000000.0f
void     bo_sssp_costs_float(uint64_t n_vertices, const uint64_t* offsets, const uint64_t* neigh, const float* weights, uint64_t src, float* costs);
uint32_t bo_sssp_costs_float_sweep(uint64_t n_vertices, const uint64_t* offsets, const uint64_t* neigh, const float* weights, uint64_t src, float* costs);

/* benchmarks/reduction/main.cu:166-195 and benchmarks/scan/main.cu:147-190, 89-100: per-block sums; running sums with a
 * leading zero (out holds n + 1 words) */
void     bo_reduce_blocks(const uint64_t* a, uint64_t n, uint32_t block, uint64_t* out);
void     bo_scan(const uint64_t* a, uint64_t n, uint64_t* out);
/* PageRank by residual pushes in single precision (benchmarks/pagerank/main.cu:107-115, 252-273, 412-421, 704-768);
 * returns the sweeps taken.  bo_pagerank_limit: the solution the pushes approach as the tolerance goes to 0. */
uint32_t bo_pagerank(uint64_t n_vertices, const uint64_t* offsets, const uint64_t* neigh, float alpha, float tolerance, uint32_t max_iterations,
                     float* value);
void     bo_pagerank_limit(uint64_t n_vertices, const uint64_t* offsets, const uint64_t* neigh, double alpha, uint32_t sweeps, double* x);

void     bo_cmd_rw(uint32_t dword[16], uint16_t cid, uint8_t opcode, uint32_t nsid, uint64_t prp1, uint64_t prp2, uint64_t slba, uint16_t n_blocks);

#ifdef __cplusplus
}
#endif
#endif
