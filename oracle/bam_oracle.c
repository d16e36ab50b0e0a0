/*
 * CPU oracle: synthetic inputs, closed forms and textbook graph algorithms.
 * TEST INFRASTRUCTURE ONLY -- see bam_oracle.h for the rules and pinning status.
 */
#include "bam_oracle.h"
#include <stdlib.h>
#include <string.h>

/* ---- SplitMix64 stream: i-th output for a given seed (Vigna's public-domain generator) ---- */
static inline uint64_t mix64(uint64_t z)
{
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

uint64_t bo_splitmix64(uint64_t seed, uint64_t i)
{
    return mix64(seed + (i + 1) * 0x9E3779B97F4A7C15ull);
}

void bo_fill_store(uint64_t seed, uint64_t first, uint64_t n, uint64_t* out)
{
    for (uint64_t k = 0; k < n; k++) out[k] = bo_splitmix64(seed, first + k);
}

/* sum of store[first + j*stride], j < count, mod 2^64: the checksum an array
 * reduction must produce whatever the cache or queue schedule was */
uint64_t bo_store_sum(uint64_t seed, uint64_t first, uint64_t stride, uint64_t count)
{
    uint64_t s = 0;
    for (uint64_t j = 0; j < count; j++) s += bo_splitmix64(seed, first + j * stride);
    return s;
}

/* random gather: idx_k = splitmix64(seed ^ 0x5eed, k) mod n_elems */
void bo_gather_indices(uint64_t seed, uint64_t first_k, uint64_t n, uint64_t n_elems, uint64_t* out)
{
    for (uint64_t k = 0; k < n; k++) out[k] = bo_splitmix64(seed ^ 0x5eedull, first_k + k) % n_elems;
}

uint64_t bo_gather_sum(uint64_t store_seed, uint64_t idx_seed, uint64_t first_k, uint64_t n, uint64_t n_elems)
{
    uint64_t s = 0;
    for (uint64_t k = 0; k < n; k++)
        s += bo_splitmix64(store_seed, bo_splitmix64(idx_seed ^ 0x5eedull, first_k + k) % n_elems);
    return s;
}

/* raw block bench: request k reads req_bytes at LBA (splitmix64(seed,k) mod (ns_bytes/req_bytes)) * (req_bytes/lba_bytes) */
void bo_block_lbas(uint64_t seed, uint64_t first_k, uint64_t n, uint64_t ns_bytes, uint32_t req_bytes, uint32_t lba_bytes, uint64_t* out)
{
    uint64_t n_units = ns_bytes / req_bytes;
    for (uint64_t k = 0; k < n; k++)
        out[k] = (bo_splitmix64(seed, first_k + k) % n_units) * (req_bytes / lba_bytes);
}

/* payload checksum of one request against the procedural namespace word[w] = splitmix64(store_seed, w) */
uint64_t bo_block_checksum(uint64_t store_seed, uint64_t lba, uint32_t lba_bytes, uint32_t req_bytes)
{
    uint64_t w0 = lba * (lba_bytes / 8), s = 0;
    for (uint32_t k = 0; k < req_bytes / 8; k++) s += bo_splitmix64(store_seed, w0 + k);
    return s;
}

/* ---- graph generators ---- */
/* RMAT a=.57 b=.19 c=.19 d=.05 as 32-bit integer thresholds: floor(p * 2^32) */
#define RMAT_T1 2448131358u               /* a          */
#define RMAT_T2 (RMAT_T1 + 816043786u)    /* a + b      */
#define RMAT_T3 (RMAT_T2 + 816043786u)    /* a + b + c  */

void bo_rmat_edges(uint64_t seed, uint32_t scale, uint64_t first_edge, uint64_t n, uint64_t* u, uint64_t* v)
{
    for (uint64_t k = 0; k < n; k++) {
        uint64_t e = first_edge + k, uu = 0, vv = 0;
        for (uint32_t l = 0; l < scale; l++) {
            uint32_t x = (uint32_t)(bo_splitmix64(seed, e * scale + l) >> 32);
            uint32_t q = x < RMAT_T1 ? 0 : x < RMAT_T2 ? 1 : x < RMAT_T3 ? 2 : 3;
            uu = (uu << 1) | (q >> 1);
            vv = (vv << 1) | (q & 1);
        }
        u[k] = uu; v[k] = vv;
    }
}

void bo_uniform_edges(uint64_t seed, uint64_t n_vertices, uint64_t first_pair, uint64_t n, uint64_t* u, uint64_t* v)
{
    for (uint64_t k = 0; k < n; k++) {
        uint64_t p = first_pair + k;
        u[k] = bo_splitmix64(seed, 2 * p) % n_vertices;
        v[k] = bo_splitmix64(seed, 2 * p + 1) % n_vertices;
    }
}

static void radix_sort_u64(uint64_t* a, uint64_t n, uint64_t max_key)
{
    uint64_t* b = (uint64_t*)malloc(n * sizeof(uint64_t));
    for (int shift = 0; shift < 64 && (max_key >> shift) != 0; shift += 8) {
        uint64_t cnt[257] = {0};
        for (uint64_t i = 0; i < n; i++) cnt[((a[i] >> shift) & 0xff) + 1]++;
        for (int d = 0; d < 256; d++) cnt[d + 1] += cnt[d];
        for (uint64_t i = 0; i < n; i++) b[cnt[(a[i] >> shift) & 0xff]++] = a[i];
        memcpy(a, b, n * sizeof(uint64_t));
    }
    free(b);
}

uint64_t bo_build_csr(uint64_t n_vertices, uint64_t n_pairs, const uint64_t* u, const uint64_t* v, uint64_t* offsets, uint64_t* neigh)
{
    uint64_t* keys = (uint64_t*)malloc(2 * n_pairs * sizeof(uint64_t) + 8);
    uint64_t m = 0;
    for (uint64_t k = 0; k < n_pairs; k++) {
        if (u[k] == v[k]) continue;
        keys[m++] = (u[k] << 32) | v[k];
        keys[m++] = (v[k] << 32) | u[k];
    }
    radix_sort_u64(keys, m, (n_vertices << 32) | 0xffffffffull);
    memset(offsets, 0, (n_vertices + 1) * sizeof(uint64_t));
    uint64_t e = 0;
    for (uint64_t k = 0; k < m; k++) {
        if (k && keys[k] == keys[k - 1]) continue;
        neigh[e++] = keys[k] & 0xffffffffull;
        offsets[(keys[k] >> 32) + 1]++;
    }
    for (uint64_t i = 0; i < n_vertices; i++) offsets[i + 1] += offsets[i];
    free(keys);
    return e;
}

/* first n_src vertices with degree > 0 among splitmix64(seed ^ 0xbf5, j) mod V, j = 0,1,... */
void bo_bfs_sources(uint64_t seed, uint64_t n_vertices, const uint64_t* offsets, uint32_t n_src, uint64_t* out)
{
    uint32_t got = 0;
    for (uint64_t j = 0; got < n_src && j < 64 * n_vertices + 1024; j++) {
        uint64_t s = bo_splitmix64(seed ^ 0xbf5ull, j) % n_vertices;
        if (offsets[s + 1] > offsets[s]) out[got++] = s;
    }
    while (got < n_src) out[got++] = 0;
}

/* ---- BFS ---- */
/* Textbook queue BFS.  Unreachable = 0xFFFFFFFF (bfs/main.cu:67,1559).  The
 * return value is the launch count of the reference host loop
 * (bfs/main.cu:1577-1736): one launch per level plus the final no-change one. */
uint32_t bo_bfs_levels(uint64_t n_vertices, const uint64_t* offsets, const uint64_t* neigh, uint64_t src, uint32_t* levels)
{
    uint64_t* q = (uint64_t*)malloc(n_vertices * sizeof(uint64_t));
    uint64_t head = 0, tail = 0;
    uint32_t maxl = 0;
    memset(levels, 0xFF, n_vertices * sizeof(uint32_t));
    levels[src] = 0; q[tail++] = src;
    while (head < tail) {
        uint64_t x = q[head++];
        for (uint64_t i = offsets[x]; i < offsets[x + 1]; i++) {
            uint64_t y = neigh[i];
            if (levels[y] == BO_INF32) {
                levels[y] = levels[x] + 1;
                if (levels[y] > maxl) maxl = levels[y];
                q[tail++] = y;
            }
        }
    }
    free(q);
    return maxl + 1;
}

/* Level-synchronous full sweep exactly as the reference kernel + host loop do
 * it (bfs/main.cu:658-689, 1557-1566, 1577-1736), executed serially. */
uint32_t bo_bfs_levels_sweep(uint64_t n_vertices, const uint64_t* offsets, const uint64_t* neigh, uint64_t src, uint32_t* levels)
{
    uint32_t level = 0, iter = 0;
    int changed;
    memset(levels, 0xFF, n_vertices * sizeof(uint32_t));
    levels[src] = 0;
    do {
        changed = 0;
        for (uint64_t x = 0; x < n_vertices; x++) {
            if (levels[x] != level) continue;
            for (uint64_t i = offsets[x]; i < offsets[x + 1]; i++)
                if (levels[neigh[i]] == BO_INF32) { levels[neigh[i]] = level + 1; changed = 1; }
        }
        iter++; level++;
    } while (changed);
    return iter;
}

uint64_t bo_bfs_edges_scanned(uint64_t n_vertices, const uint64_t* offsets, const uint32_t* levels)
{
    uint64_t s = 0;
    for (uint64_t x = 0; x < n_vertices; x++)
        if (levels[x] != BO_INF32) s += offsets[x + 1] - offsets[x];
    return s;
}

/* ---- CC ---- */
static uint64_t uf_find(uint64_t* p, uint64_t x)
{
    while (p[x] != x) { p[x] = p[p[x]]; x = p[x]; }
    return x;
}

/* Union-find keeping the smaller id as root: label[v] = smallest vertex id of
 * v's component, the unique fixed point of the reference's min-label
 * propagation (cc/main.cu:123-144) when every edge is treated as undirected. */
uint64_t bo_cc_labels(uint64_t n_vertices, const uint64_t* offsets, const uint64_t* neigh, uint64_t* labels)
{
    for (uint64_t x = 0; x < n_vertices; x++) labels[x] = x;
    for (uint64_t x = 0; x < n_vertices; x++)
        for (uint64_t i = offsets[x]; i < offsets[x + 1]; i++) {
            uint64_t a = uf_find(labels, x), b = uf_find(labels, neigh[i]);
            if (a < b) labels[b] = a; else if (b < a) labels[a] = b;
        }
    uint64_t comps = 0;
    for (uint64_t x = 0; x < n_vertices; x++) { labels[x] = uf_find(labels, x); comps += labels[x] == x; }
    return comps;
}

/* The reference iteration itself, serially: curr/next visit flags, cc_compute
 * on every edge of every visited vertex, swap, until nothing changed
 * (cc/main.cu:123-144, 595-617, 1410-1425, 1515-1521).  Component count as in
 * cc/main.cu:1629-1639 (number of distinct labels). */
uint64_t bo_cc_labels_sweep(uint64_t n_vertices, const uint64_t* offsets, const uint64_t* neigh, uint64_t* labels, uint32_t* iters)
{
    uint8_t* curr = (uint8_t*)malloc(n_vertices);
    uint8_t* next = (uint8_t*)calloc(n_vertices, 1);
    uint32_t it = 0;
    int changed;
    memset(curr, 1, n_vertices);
    for (uint64_t x = 0; x < n_vertices; x++) labels[x] = x;
    do {
        changed = 0;
        for (uint64_t x = 0; x < n_vertices; x++) {
            if (!curr[x]) continue;
            for (uint64_t i = offsets[x]; i < offsets[x + 1]; i++) {
                uint64_t y = neigh[i], cs = labels[x], cn = labels[y];
                if (cs == cn) continue;
                uint64_t tgt = cs < cn ? y : x, val = cs < cn ? cs : cn;
                if (val < labels[tgt]) labels[tgt] = val;
                next[tgt] = 1; changed = 1;
            }
        }
        memset(curr, 0, n_vertices);
        uint8_t* t = curr; curr = next; next = t;
        it++;
    } while (changed);
    if (iters) *iters = it;
    uint64_t comps = 0;
    memset(curr, 0, n_vertices);
    for (uint64_t x = 0; x < n_vertices; x++) if (!curr[labels[x]]) { curr[labels[x]] = 1; comps++; }
    free(curr); free(next);
    return comps;
}

/* ---- NVMe SQE image for READ/WRITE (NVMe 1.x, figure "Command Format"; nvm_cmd.h:54-88) ---- */
void bo_cmd_rw(uint32_t dword[16], uint16_t cid, uint8_t opcode, uint32_t nsid, uint64_t prp1, uint64_t prp2, uint64_t slba, uint16_t n_blocks)
{
    memset(dword, 0, 64);
    dword[0]  = ((uint32_t)cid << 16) | (opcode & 0x7f);
    dword[1]  = nsid;
    dword[6]  = (uint32_t)prp1;  dword[7]  = (uint32_t)(prp1 >> 32);
    dword[8]  = (uint32_t)prp2;  dword[9]  = (uint32_t)(prp2 >> 32);
    dword[10] = (uint32_t)slba;  dword[11] = (uint32_t)(slba >> 32);
    dword[12] = (uint32_t)((n_blocks - 1) & 0xffff);
}

/* ---- weighted graphs: single-source shortest paths ---- */
void bo_edge_weights(uint64_t seed, uint64_t first, uint64_t n, uint32_t* out)
{
    for (uint64_t k = 0; k < n; k++) out[k] = 1u + (uint32_t)(bo_splitmix64(seed ^ 0x3e16ull, first + k) % 255u);
}

typedef struct { uint64_t cost; uint64_t v; } heap_item;

static void heap_push(heap_item* h, uint64_t* n, heap_item x)
{
    uint64_t i = (*n)++;
    while (i) {
        uint64_t p = (i - 1) / 2;
        if (h[p].cost <= x.cost) break;
        h[i] = h[p];
        i = p;
    }
    h[i] = x;
}

static heap_item heap_pop(heap_item* h, uint64_t* n)
{
    heap_item top = h[0], last = h[--(*n)];
    uint64_t i = 0;
    for (;;) {
        uint64_t c = 2 * i + 1;
        if (c >= *n) break;
        if (c + 1 < *n && h[c + 1].cost < h[c].cost) c++;
        if (last.cost <= h[c].cost) break;
        h[i] = h[c];
        i = c;
    }
    h[i] = last;
    return top;
}

void bo_sssp_costs(uint64_t n_vertices, const uint64_t* offsets, const uint64_t* neigh, const uint32_t* weights, uint64_t src, uint32_t* costs)
{
    for (uint64_t v = 0; v < n_vertices; v++) costs[v] = BO_INF32;
    /* lazy deletion: at most one heap entry per relaxation */
    heap_item* heap = (heap_item*)malloc((offsets[n_vertices] + 1) * sizeof(heap_item));
    uint64_t n = 0;
    costs[src] = 0;
    heap_push(heap, &n, (heap_item){0, src});
    while (n) {
        heap_item it = heap_pop(heap, &n);
        if (it.cost != costs[it.v]) continue;
        for (uint64_t e = offsets[it.v]; e < offsets[it.v + 1]; e++) {
            uint64_t c = it.cost + weights[e];
            if (c < costs[neigh[e]]) {
                costs[neigh[e]] = (uint32_t)c;
                heap_push(heap, &n, (heap_item){c, neigh[e]});
            }
        }
    }
    free(heap);
}

/*
 * benchmarks/sssp_float/main.cu (WeightT = float :69, unreached = 1e9 :529, relax :194-217, update :302-312): the fixed point of
 * its rounds.  Every cost a vertex ever holds is the sum, added edge by edge in single precision from the source on, of
 * the weights along some path; adding a weight that is not negative never lowers a cost and keeps the order of two
 * costs, so the least such sum is what Dijkstra's order finds, whatever order the rounds relax in.  A cost that does
 * not come out below 1e9 is never adopted.  Costs that are not negative order as their bit patterns: the heap keys.
 */
static uint32_t float_bits(float f) { uint32_t u; memcpy(&u, &f, sizeof(u)); return u; }

void bo_sssp_costs_float(uint64_t n_vertices, const uint64_t* offsets, const uint64_t* neigh, const float* weights, uint64_t src, float* costs)
{
    for (uint64_t v = 0; v < n_vertices; v++) costs[v] = BO_FAR_F32;
    heap_item* heap = (heap_item*)malloc((offsets[n_vertices] + 1) * sizeof(heap_item));
    uint64_t n = 0;
    costs[src] = 0.0f;
    heap_push(heap, &n, (heap_item){0, src});
    while (n) {
        heap_item it = heap_pop(heap, &n);
        if (it.cost != float_bits(costs[it.v])) continue;
        for (uint64_t e = offsets[it.v]; e < offsets[it.v + 1]; e++) {
            const float c = costs[it.v] + weights[e];
            if (c < costs[neigh[e]]) {
                costs[neigh[e]] = c;
                heap_push(heap, &n, (heap_item){float_bits(c), neigh[e]});
            }
        }
    }
    free(heap);
}

uint32_t bo_sssp_costs_float_sweep(uint64_t n_vertices, const uint64_t* offsets, const uint64_t* neigh, const float* weights, uint64_t src, float* costs)
{
    for (uint64_t v = 0; v < n_vertices; v++) costs[v] = BO_FAR_F32;
    costs[src] = 0.0f;
    uint32_t rounds = 0;
    for (int changed = 1; changed;) {
        changed = 0;
        for (uint64_t v = n_vertices; v-- > 0;)                 /* highest vertex first: not the order of the heap */
            for (uint64_t e = offsets[v]; e < offsets[v + 1]; e++) {
                const float c = costs[v] + weights[e];
                if (c < costs[neigh[e]]) { costs[neigh[e]] = c; changed = 1; }
            }
        rounds += changed;
    }
    return rounds;
}

/* benchmarks/reduction/main.cu:166-195: block b of `block` threads sums elements [2 b block, 2 (b + 1) block) */
void bo_reduce_blocks(const uint64_t* a, uint64_t n, uint32_t block, uint64_t* out)
{
    const uint64_t per = 2ull * block, n_blocks = (n + per - 1) / per;
    for (uint64_t b = 0; b < n_blocks; b++) {
        uint64_t s = 0;
        for (uint64_t i = b * per; i < (b + 1) * per && i < n; i++) s += a[i];
        out[b] = s;
    }
}

/* benchmarks/scan/main.cu:370-373, 413-420: result[0] = 0, result[i + 1] = a[0] + ... + a[i] */
void bo_scan(const uint64_t* a, uint64_t n, uint64_t* out)
{
    out[0] = 0;
    for (uint64_t i = 0; i < n; i++) out[i + 1] = out[i] + a[i];
}

/*
 * benchmarks/pagerank/main.cu: initialize :107-115, push :252-273 (every neighbour of a flagged vertex receives the
 * vertex's delta), update :412-421, host loop :704-768.  Single precision as the reference (ValueT = float, :78);
 * the pushes of one sweep are added in vertex order here, in no fixed order on a GPU.
 */
uint32_t bo_pagerank(uint64_t n_vertices, const uint64_t* offsets, const uint64_t* neigh, float alpha, float tolerance, uint32_t max_iterations,
                     float* value)
{
    float* delta = (float*)malloc(n_vertices * sizeof(float));
    float* residual = (float*)malloc(n_vertices * sizeof(float));
    uint8_t* label = (uint8_t*)malloc(n_vertices);
    for (uint64_t v = 0; v < n_vertices; v++) {
        value[v] = 1.0f - alpha;
        delta[v] = (1.0f - alpha) * alpha / (offsets[v + 1] - offsets[v]);
        residual[v] = 0.0f;
        label[v] = 1;
    }
    uint32_t iter = 0;
    int changed;
    do {
        changed = 0;
        for (uint64_t v = 0; v < n_vertices; v++) {
            if (!label[v]) continue;
            for (uint64_t e = offsets[v]; e < offsets[v + 1]; e++) residual[neigh[e]] += delta[v];
            label[v] = 0;
        }
        iter++;
        for (uint64_t v = 0; v < n_vertices; v++) {
            if (residual[v] > tolerance) {
                value[v] += residual[v];
                delta[v] = residual[v] * alpha / (offsets[v + 1] - offsets[v]);
                residual[v] = 0.0f;
                label[v] = 1;
                changed = 1;
            }
        }
    } while (changed && iter < max_iterations);
    free(delta); free(residual); free(label);
    return iter;
}

/* what the pushes converge to as tolerance -> 0: x = (1 - alpha) + alpha * sum over in-neighbours u of x_u / degree(u),
 * by `sweeps` Jacobi steps in double precision (error <= alpha^sweeps * max x) */
void bo_pagerank_limit(uint64_t n_vertices, const uint64_t* offsets, const uint64_t* neigh, double alpha, uint32_t sweeps, double* x)
{
    double* y = (double*)malloc(n_vertices * sizeof(double));
    for (uint64_t v = 0; v < n_vertices; v++) x[v] = 1.0 - alpha;
    for (uint32_t k = 0; k < sweeps; k++) {
        for (uint64_t v = 0; v < n_vertices; v++) y[v] = 1.0 - alpha;
        for (uint64_t u = 0; u < n_vertices; u++) {
            const uint64_t deg = offsets[u + 1] - offsets[u];
            if (!deg) continue;
            const double share = alpha * x[u] / (double)deg;
            for (uint64_t e = offsets[u]; e < offsets[u + 1]; e++) y[neigh[e]] += share;
        }
        memcpy(x, y, n_vertices * sizeof(double));
    }
    free(y);
}

uint32_t bo_sssp_costs_sweep(uint64_t n_vertices, const uint64_t* offsets, const uint64_t* neigh, const uint32_t* weights, uint64_t src, uint32_t* costs)
{
    for (uint64_t v = 0; v < n_vertices; v++) costs[v] = BO_INF32;
    costs[src] = 0;
    uint32_t rounds = 0;
    for (int changed = 1; changed;) {
        changed = 0;
        for (uint64_t v = 0; v < n_vertices; v++) {
            if (costs[v] == BO_INF32) continue;
            for (uint64_t e = offsets[v]; e < offsets[v + 1]; e++) {
                uint64_t c = (uint64_t)costs[v] + weights[e];
                if (c < costs[neigh[e]]) { costs[neigh[e]] = (uint32_t)c; changed = 1; }
            }
        }
        rounds += changed;
    }
    return rounds;
}
