"""Pins the oracle's MVS and ClusterGCN restatements (edge lists per sample) against numpy
brute force and the rules of the reference's own validators
(src/tests/multiGPU/mvs.cu:12-101, src/tests/multiGPU/clustergcn.cu:10-93)."""
import numpy as np

from tests import graphs


def dense(g):
    A = np.zeros((g.n_vertices, g.n_vertices), dtype=bool)
    src = np.repeat(np.arange(g.n_vertices), np.diff(g.row_ptr))
    A[src, g.col] = True
    return A


def test_sample_counts_and_vertices_follow_the_reference_formulas(oracle):
    g = graphs.random_graph(n=300, mean_degree=4, seed=2)
    og = graphs.oracle_view(g)
    assert oracle.subgraph_num_samples(og, 32, 1500000) == (300 * 8 + 31) // 32 == 75
    assert oracle.subgraph_num_samples(og, 32, 50) == 50
    v = oracle.mvs_vertices(og, 75, 32)
    assert np.array_equal(v.ravel(), np.arange(75 * 32) % 300)
    c = oracle.clustergcn_vertices(og, 75, 16, 2)
    n_clusters = 300 // 16  # the last 12 vertices belong to no cluster
    want = [(((s * 2 + i) % n_clusters) * 16 + k) for s in range(75) for i in range(2) for k in range(16)]
    assert np.array_equal(c.ravel(), want)


def test_mvs_lists_hold_every_edge_leaving_the_batch(oracle):
    g = graphs.random_graph(n=200, mean_degree=7, seed=3, hub=4, isolated_every=6)
    og = graphs.oracle_view(g)
    verts = oracle.mvs_vertices(og, 50, 32)
    rows, cols, start = oracle.sample_mvs(og, verts)
    deg = np.diff(g.row_ptr)
    assert np.array_equal(np.diff(start.astype(np.int64)), deg[verts].sum(axis=1))
    for s in range(50):
        lo, hi = start[s], start[s + 1]
        want = sorted((v, c) for v in verts[s] for c in g.col[g.row_ptr[v]:g.row_ptr[v + 1]])
        assert sorted(zip(rows[lo:hi].tolist(), cols[lo:hi].tolist())) == want
    # order inside a list: slots l = j * 32 + nbr in groups of 64; slot (j, nbr) appends the
    # edges nbr, nbr + 32, ... of vertex j; inside a group first appends first
    s = 0  # holds the hub (vertex 4)
    want = []
    per_slot = [[(v, c) for c in g.col[g.row_ptr[v]:g.row_ptr[v + 1]][nbr::32]] for v in verts[s] for nbr in range(32)]
    for first in range(0, 1024, 64):
        group = per_slot[first:first + 64]
        for i in range(max(len(x) for x in group)):
            want += [x[i] for x in group if len(x) > i]
    lo, hi = start[s], start[s + 1]
    assert list(zip(rows[lo:hi].tolist(), cols[lo:hi].tolist())) == want
    assert max(len(x) for x in per_slot) > 1  # the hub makes some slots append several edges


def test_clustergcn_lists_are_the_induced_subgraph(oracle):
    g = graphs.random_graph(n=160, mean_degree=30, seed=4, isolated_every=5)
    og = graphs.oracle_view(g)
    A = dense(g)
    verts = oracle.clustergcn_vertices(og, 40, 16, 2)
    final, rows, cols, start = oracle.sample_clustergcn(og, verts)
    deg = np.diff(g.row_ptr)
    for s in range(40):
        mine = verts[s]
        want = [(v1, v2) for v1 in mine for v2 in mine if A[v1, v2]]  # (j, nbr) order
        lo, hi = start[s], start[s + 1]
        assert list(zip(rows[lo:hi].tolist(), cols[lo:hi].tolist())) == want
        # result row: the vertices that have edges, then INVALID
        assert np.array_equal(final[s, :32], np.where(deg[mine] > 0, mine, g.n_vertices))
        assert np.all(final[s, 32:] == g.n_vertices)
    assert start[-1] == len(rows) > 0
    # the reference validator's two rules
    for s in range(40):
        lo, hi = start[s], start[s + 1]
        listed = set(zip(rows[lo:hi].tolist(), cols[lo:hi].tolist()))
        assert all(A[r, c] for r, c in listed)
        assert all((v1, v2) in listed for v1 in verts[s] for v2 in verts[s] if v1 != v2 and A[v1, v2])
