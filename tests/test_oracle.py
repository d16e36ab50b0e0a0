"""Pins the CPU oracle: golden vectors, library routines, an independent numpy restatement."""
import json
import os

import numpy as np
import pytest
import scipy.sparse as sp
import scipy.sparse.csgraph as csg

import oracle
from oracle import oracle_np as onp

G = os.path.join(os.path.dirname(__file__), "golden")


def _j(name):
    with open(os.path.join(G, name)) as f:
        return json.load(f)


def test_splitmix64_published_vectors():
    g = _j("splitmix64.json")
    L = oracle.lib()
    assert [L.bo_splitmix64(1234567, i) for i in range(5)] == [int(x) for x in g["seed_1234567"]]
    assert [L.bo_splitmix64(0, i) for i in range(3)] == [int(x, 16) for x in g["seed_0"]]
    # the sequential generator form: state += golden; out = mix(state)
    state, out = 1234567, []
    for _ in range(5):
        state = (state + 0x9E3779B97F4A7C15) & (2**64 - 1)
        z = state
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & (2**64 - 1)
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & (2**64 - 1)
        out.append(z ^ (z >> 31))
    assert out == [int(x) for x in g["seed_1234567"]]


def test_store_sums_closed_form():
    g = _j("splitmix64.json")
    L = oracle.lib()
    for seed in (0, 42):
        assert L.bo_store_sum(seed, 0, 1, 4096) == int(g["sum_first_4096"][str(seed)], 16)
        assert L.bo_store_sum(seed, 0, 8, 1 << 21) == int(g["cfg1_stride8_sum_2p21"][str(seed)], 16)
        ref = int(np.sum(onp.splitmix64(seed, np.arange(0, 1 << 24, 8, dtype=np.uint64)), dtype=np.uint64))
        assert ref == int(g["cfg1_stride8_sum_2p21"][str(seed)], 16)


def test_store_and_gather_match_numpy():
    s = oracle.store(42, 1000, 5000)
    assert np.array_equal(s, onp.splitmix64(42, np.arange(1000, 6000, dtype=np.uint64)))
    idx = oracle.gather_indices(42, 7, 4096, 1 << 20)
    ref = onp.splitmix64(42 ^ 0x5eed, np.arange(7, 7 + 4096, dtype=np.uint64)) % np.uint64(1 << 20)
    assert np.array_equal(idx, ref)
    tot = int(np.sum(onp.splitmix64(42, ref), dtype=np.uint64))
    assert oracle.lib().bo_gather_sum(42, 42, 7, 4096, 1 << 20) == tot


def test_block_lbas_and_checksum():
    lb = oracle.block_lbas(42, 0, 1000, 64 << 30, 4096, 512)
    ref = (onp.splitmix64(42, np.arange(1000, dtype=np.uint64)) % np.uint64((64 << 30) // 4096)) * np.uint64(8)
    assert np.array_equal(lb, ref)
    assert int(lb.max()) * 512 + 4096 <= 64 << 30
    for lba in (0, 8, int(lb[3])):
        w0 = lba * 64
        ref = int(np.sum(onp.splitmix64(7, np.arange(w0, w0 + 512, dtype=np.uint64)), dtype=np.uint64))
        assert oracle.lib().bo_block_checksum(7, lba, 512, 4096) == ref


def test_sqe_image_matches_nvme_spec_layout():
    d = np.zeros(16, dtype=np.uint32)
    oracle.lib().bo_cmd_rw(d, 0xBEEF, 0x02, 1, 0x1122334455667000, 0xAABBCCDD00112000, 0x0123456789ABCDEF, 8)
    b = d.tobytes()
    assert len(b) == 64
    assert b[0] == 0x02 and b[1] == 0x00          # opcode, FUSE/PSDT = 0
    assert b[2:4] == bytes([0xEF, 0xBE])          # CID, little endian
    assert b[4:8] == (1).to_bytes(4, "little")    # NSID
    assert b[8:24] == bytes(16)                   # CDW2-3, MPTR
    assert b[24:32] == (0x1122334455667000).to_bytes(8, "little")   # PRP1
    assert b[32:40] == (0xAABBCCDD00112000).to_bytes(8, "little")   # PRP2
    assert b[40:48] == (0x0123456789ABCDEF).to_bytes(8, "little")   # SLBA
    assert b[48:50] == (7).to_bytes(2, "little")  # NLB is zero based
    assert b[50:64] == bytes(14)


def test_reference_sample_graph():
    g = _j("sample_graph.json")
    off = np.array(g["offsets"], dtype=np.uint64)
    nb = np.array(g["edges"], dtype=np.uint64)
    for src, exp in g["bfs"].items():
        for sweep in (False, True):
            lv, it = oracle.bfs_levels(off, nb, int(src), sweep=sweep)
            assert lv.tolist() == exp["levels"], (src, sweep)
            assert it == exp["iterations"], (src, sweep)
    lb, comps = oracle.cc_labels(off, nb)
    assert lb.tolist() == g["cc"]["labels"] and comps == g["cc"]["components"]
    lb2, comps2, _ = oracle.cc_labels(off, nb, sweep=True)
    assert lb2.tolist() == g["cc"]["labels"] and comps2 == 2


@pytest.mark.parametrize("scale", [6, 10, 13])
def test_rmat_generator_and_csr_match_numpy(scale):
    n = 16 << scale
    u = np.empty(n, dtype=np.uint64)
    v = np.empty(n, dtype=np.uint64)
    oracle.lib().bo_rmat_edges(42, scale, 0, n, u, v)
    u2, v2 = onp.rmat_edges(42, scale, 0, n)
    assert np.array_equal(u, u2) and np.array_equal(v, v2)
    assert int(u.max()) < (1 << scale) and int(v.max()) < (1 << scale)
    # quadrant (0,0) must dominate: about a^scale-ish skew, at least more low ids than high
    assert (u < (1 << (scale - 1))).mean() > 0.7
    off, nb = oracle.rmat_csr(42, scale)
    off2, nb2 = onp.build_csr(1 << scale, u2, v2)
    assert np.array_equal(off, off2) and np.array_equal(nb, nb2)
    # symmetric, no self loops, sorted unique rows
    A = sp.csr_matrix((np.ones(len(nb), dtype=np.int8), nb.astype(np.int64), off.astype(np.int64)), shape=(1 << scale,) * 2)
    assert (A != A.T).nnz == 0 and A.diagonal().sum() == 0
    for r in range(0, 1 << scale, 97):
        row = nb[int(off[r]):int(off[r + 1])]
        assert np.all(row[1:] > row[:-1])


def _scipy_graph(off, nb):
    n = len(off) - 1
    return sp.csr_matrix((np.ones(len(nb), dtype=np.int8), nb.astype(np.int64), off.astype(np.int64)), shape=(n, n))


@pytest.mark.parametrize("seed,scale", [(42, 8), (0, 11), (7, 13)])
def test_bfs_against_scipy(seed, scale):
    off, nb = oracle.rmat_csr(seed, scale)
    A = _scipy_graph(off, nb)
    for src in oracle.bfs_sources(seed, off, 4):
        d = csg.shortest_path(A, method="D", unweighted=True, indices=int(src))
        exp = np.where(np.isinf(d), 0xFFFFFFFF, d).astype(np.uint32)
        lv, it = oracle.bfs_levels(off, nb, src)
        lv2, it2 = oracle.bfs_levels(off, nb, src, sweep=True)
        assert np.array_equal(lv, exp) and np.array_equal(lv2, exp)
        assert it == it2 == int(exp[exp != 0xFFFFFFFF].max()) + 1
        assert off[int(src) + 1] > off[int(src)]


@pytest.mark.parametrize("n_v,n_p", [(64, 40), (1000, 700), (5000, 9000)])
def test_cc_against_scipy(n_v, n_p):
    off, nb = oracle.uniform_csr(42, n_v, n_p)
    u, v = onp.uniform_edges(42, n_v, 0, n_p)
    off2, nb2 = onp.build_csr(n_v, u, v)
    assert np.array_equal(off, off2) and np.array_equal(nb, nb2)
    ncomp, lab = csg.connected_components(_scipy_graph(off, nb), directed=False)
    lb, comps = oracle.cc_labels(off, nb)
    lb2, comps2, iters = oracle.cc_labels(off, nb, sweep=True)
    assert comps == comps2 == ncomp and np.array_equal(lb, lb2) and iters >= 1
    # label = smallest vertex id of the component
    mins = np.full(ncomp, n_v, dtype=np.int64)
    np.minimum.at(mins, lab, np.arange(n_v))
    assert np.array_equal(lb.astype(np.int64), mins[lab])


# ---------------------------------------------------------------- weighted graphs (single-source shortest paths)

def test_edge_weights_definition():
    w = oracle.edge_weights(42, 1000, first=7)
    want = np.array([1 + onp.splitmix64(42 ^ 0x3e16, 7 + k) % 255 for k in range(1000)], dtype=np.uint32)
    assert np.array_equal(w, want) and w.min() >= 1 and w.max() <= 255


def test_sssp_hand_computed_graph():
    """a six-vertex graph worked out by hand: the cheap route 0-1-2-3 beats the direct edge 0-3; vertex 5 is unreachable;
    edge weights are per direction (2->1 costs more than 1->2)"""
    #        0:(1,w2)(3,w10)   1:(0,w2)(2,w3)   2:(1,w9)(3,w1)(4,w7)   3:(0,w10)(2,w1)   4:(2,w7)   5:-
    off = np.array([0, 2, 4, 7, 9, 10, 10], dtype=np.uint64)
    nb = np.array([1, 3, 0, 2, 1, 3, 4, 0, 2, 2], dtype=np.uint64)
    w = np.array([2, 10, 2, 3, 9, 1, 7, 10, 1, 7], dtype=np.uint32)
    inf = 0xFFFFFFFF
    assert oracle.sssp_costs(off, nb, w, 0).tolist() == [0, 2, 5, 6, 12, inf]
    assert oracle.sssp_costs(off, nb, w, 3).tolist() == [10, 10, 1, 0, 8, inf]
    assert oracle.sssp_costs(off, nb, w, 5).tolist() == [inf] * 5 + [0]
    costs, rounds = oracle.sssp_costs(off, nb, w, 0, sweep=True)
    assert costs.tolist() == [0, 2, 5, 6, 12, inf] and rounds >= 1


def test_sssp_float_hand_computed_graph_whose_sums_round():
    """0 -> 1 (2^24) -> 2 (1): 2^24 + 1 is not a float and rounds back to 2^24, which beats the direct edge of 2^24 + 2;
    0 -> 3 (0.1) -> 4 (0.2) -> 7 (0.4): the sum added edge by edge in single precision, one unit in the last place above
    the rounded exact sum; 5 cannot be reached; 6 only over a path whose cost does not stay below 1e9, which is never taken"""
    f = np.float32
    pairs = [(0, 1, f(16777216.0)), (1, 2, f(1.0)), (0, 2, f(16777218.0)), (0, 3, f(0.1)), (3, 4, f(0.2)), (4, 7, f(0.4)),
             (4, 6, f(1e9)), (5, 0, f(1.0))]
    n_v = 8
    off = np.zeros(n_v + 1, dtype=np.uint64)
    for u, _, _ in pairs:
        off[u + 1] += 1
    off = np.cumsum(off).astype(np.uint64)
    order = sorted(range(len(pairs)), key=lambda k: pairs[k][0])
    nb = np.array([pairs[k][1] for k in order], dtype=np.uint64)
    w = np.array([pairs[k][2] for k in order], dtype=np.float32)
    want = np.array([0.0, 16777216.0, 16777216.0, f(0.1), f(0.1) + f(0.2), 1e9, 1e9, 0.0], dtype=np.float32)
    want.view(np.uint32)[7] = 1060320052                                    # 0.70000005: (0.1f + 0.2f) + 0.4f
    assert np.float32(float(f(0.1)) + float(f(0.2)) + float(f(0.4))).view(np.uint32) == 1060320051      # the exact sum rounds elsewhere
    got = oracle.sssp_costs_float(off, nb, w, 0)
    assert got.view(np.uint32).tolist() == want.view(np.uint32).tolist()
    swept, rounds = oracle.sssp_costs_float(off, nb, w, 0, sweep=True)
    assert swept.view(np.uint32).tolist() == want.view(np.uint32).tolist() and rounds >= 1


@pytest.mark.parametrize("seed,scale", [(1, 8), (42, 11)])
def test_sssp_float_against_scipy_the_sweep_and_numpy(seed, scale):
    from scipy.sparse import csr_matrix
    from scipy.sparse.csgraph import dijkstra
    off, nb = oracle.rmat_csr(seed, scale)
    n_v = len(off) - 1
    wi = oracle.edge_weights(seed, len(nb))
    srcs = oracle.bfs_sources(seed, off, 2)
    # (a) weights that add exactly in single precision (small integers and quarters): the double-precision answer is the answer
    w_exact = (wi.astype(np.float32) * np.float32(0.25))
    g = csr_matrix((w_exact.astype(np.float64), nb.astype(np.int64), off.astype(np.int64)), shape=(n_v, n_v))
    for src in srcs:
        d = dijkstra(g, directed=True, indices=int(src))
        want = np.where(np.isinf(d), 1e9, d).astype(np.float32)
        assert np.array_equal(oracle.sssp_costs_float(off, nb, w_exact, int(src)), want)
    # (b) weights whose sums round: Dijkstra's order, the sweep from the highest vertex down and a numpy relaxation of
    # all edges at once must agree to the bit
    w = wi.astype(np.float32) * np.float32(0.37) + np.float32(1e-3)
    u = np.repeat(np.arange(n_v, dtype=np.int64), np.diff(off).astype(np.int64))
    v = nb.astype(np.int64)
    for src in srcs:
        got = oracle.sssp_costs_float(off, nb, w, int(src))
        swept, _ = oracle.sssp_costs_float(off, nb, w, int(src), sweep=True)
        assert np.array_equal(got.view(np.uint32), swept.view(np.uint32))
        c = np.full(n_v, 1e9, dtype=np.float32); c[int(src)] = 0
        while True:
            nxt = c.copy()
            np.minimum.at(nxt, v, c[u] + w)
            if np.array_equal(nxt, c):
                break
            c = nxt
        assert np.array_equal(got.view(np.uint32), c.view(np.uint32))
        assert len(np.unique(got)) > 100                                    # not a degenerate case


@pytest.mark.parametrize("seed,scale", [(42, 8), (0, 10), (7, 12)])
def test_sssp_against_scipy_and_the_sweep(seed, scale):
    off, nb = oracle.rmat_csr(seed, scale)
    w = oracle.edge_weights(seed, len(nb))
    n = len(off) - 1
    m = sp.csr_matrix((w.astype(np.float64), nb.astype(np.int64), off.astype(np.int64)), shape=(n, n))
    for src in oracle.bfs_sources(seed, off, 3):
        got = oracle.sssp_costs(off, nb, w, int(src))
        ref = csg.dijkstra(m, directed=True, indices=int(src))
        want = np.where(np.isinf(ref), 0xFFFFFFFF, ref).astype(np.uint64).astype(np.uint32)
        assert np.array_equal(got, want)
        swept, _ = oracle.sssp_costs(off, nb, w, int(src), sweep=True)
        assert np.array_equal(swept, got)
        # unreachable exactly where BFS does not reach
        assert np.array_equal(got == 0xFFFFFFFF, oracle.bfs_levels(off, nb, int(src))[0] == 0xFFFFFFFF)


# ---------------------------------------------------------------- reduction and scan

@pytest.mark.parametrize("n,block", [(0, 64), (1, 64), (127, 64), (128, 64), (129, 64), (5000, 256), (4096, 1024)])
def test_reduce_blocks_and_scan_against_numpy(n, block):
    a = oracle.store(42, 3, n) if n else np.zeros(0, dtype=np.uint64)
    per = 2 * block
    want = [int(a[b * per:(b + 1) * per].sum(dtype=np.uint64)) for b in range((n + per - 1) // per)]
    assert oracle.reduce_blocks(a, block).tolist() == want
    s = oracle.scan(a)
    assert len(s) == n + 1 and s[0] == 0
    assert np.array_equal(s[1:], np.cumsum(a, dtype=np.uint64))
    if n:
        assert int(s[-1]) == int(oracle.reduce_blocks(a, block).sum(dtype=np.uint64))


def test_scan_closed_form_and_wrap_around():
    n = 100000
    s = oracle.scan(np.arange(n, dtype=np.uint64))
    assert s.tolist() == [i * (i - 1) // 2 for i in range(n + 1)]
    big = np.full(5, 2**63, dtype=np.uint64)                       # sums leave 64 bits: kept mod 2^64
    assert oracle.scan(big).tolist() == [0, 2**63, 0, 2**63, 0, 2**63]
    assert oracle.reduce_blocks(big, 64).tolist() == [2**63]


# ---------------------------------------------------------------- PageRank

def _pagerank_solve(off, nb, alpha):
    """x = (1 - alpha) + alpha * P^T x, P = D^-1 A, solved directly in double precision"""
    import scipy.sparse.linalg as spl
    n = len(off) - 1
    deg = np.diff(off.astype(np.int64)).astype(np.float64)
    a = sp.csr_matrix((np.ones(len(nb)), nb.astype(np.int64), off.astype(np.int64)), shape=(n, n))
    inv = np.divide(1.0, deg, out=np.zeros(n), where=deg > 0)
    p_t = (sp.diags(inv) @ a).T.tocsc()
    return spl.spsolve(sp.identity(n, format="csc") - alpha * p_t, np.full(n, 1.0 - alpha))


def test_pagerank_first_sweeps_by_hand():
    """path 0 - 1 - 2, alpha 0.85: after one sweep every vertex has taken what its neighbours pushed from the initial
    deltas 0.1275, 0.06375, 0.1275; after two, the deltas made from those residuals"""
    off = np.array([0, 1, 3, 4], dtype=np.uint64)
    nb = np.array([1, 0, 2, 1], dtype=np.uint64)
    v, it = oracle.pagerank(off, nb, 0.85, 0.001, max_iterations=1)
    assert it == 1 and np.allclose(v, [0.21375, 0.405, 0.21375], rtol=1e-6)
    v, it = oracle.pagerank(off, nb, 0.85, 0.001, max_iterations=2)
    assert it == 2 and np.allclose(v, [0.322125, 0.513375, 0.322125], rtol=1e-6)
    # the limit, worked out from x0 = 0.15 + 0.425 x1, x1 = 0.15 + 1.7 x0
    x = oracle.pagerank_limit(off, nb, 0.85)
    assert np.allclose(x, [0.21375 / 0.2775, 0.15 + 1.7 * 0.21375 / 0.2775, 0.21375 / 0.2775], rtol=1e-12)
    v, it = oracle.pagerank(off, nb, 0.85, 1e-6, max_iterations=1000)
    assert it < 1000 and np.allclose(v, x, rtol=2e-5)


@pytest.mark.parametrize("seed,scale,tol", [(42, 8, 1e-3), (0, 10, 1e-3), (7, 12, 1e-4)])
def test_pagerank_against_a_direct_solve(seed, scale, tol):
    off, nb = oracle.rmat_csr(seed, scale)
    alpha = 0.85
    x = _pagerank_solve(off, nb, alpha)
    assert np.allclose(oracle.pagerank_limit(off, nb, alpha), x, rtol=1e-10)
    deg = np.diff(off.astype(np.int64))
    assert abs(x[deg > 0].sum() - (deg > 0).sum()) < 1e-6 * len(x)      # no dangling vertices among the connected: mass is kept
    assert np.allclose(x[deg == 0], 1 - alpha)
    v, it = oracle.pagerank(off, nb, alpha, tol, max_iterations=1000)
    assert it < 1000
    # whatever is left unpushed is at most `tol` per vertex: 0 <= x - value <= x * tol / (1 - alpha), up to float rounding
    slack = 1e-5 * x
    assert np.all(v <= x + slack) and np.all(v >= x * (1 - tol / (1 - alpha)) - slack)
