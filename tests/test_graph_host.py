"""Host-side graph ingest of the library (no GPU involved): CSR layout, sort order,
max weight, the 12-byte binary edge list, seeded generators."""
import numpy as np
import pytest

import nextdoor_amd as nd


def test_csr_from_edges_sorts_by_destination_then_weight_and_keeps_duplicates():
    src = [2, 0, 0, 0, 2, 0]
    dst = [1, 3, 1, 3, 0, 2]
    w = [1.0, 5.0, 2.0, 4.0, 3.0, 2.5]
    g = nd.Graph.from_edges(src, dst, w)
    assert g.n_vertices == 4 and g.n_edges == 6
    assert list(g.row_ptr) == [0, 4, 4, 6, 6]
    assert list(g.col) == [1, 2, 3, 3, 0, 1]
    assert list(g.weight) == [2.0, 2.5, 4.0, 5.0, 3.0, 1.0]
    # max_weight = max(0, weights), 0 for a vertex without edges (graph.hpp:71-80)
    assert list(g.max_weight) == [5.0, 0.0, 3.0, 0.0]


def test_binary_edge_list_round_trip(tmp_path):
    rng = np.random.default_rng(0)
    n = 500
    src = rng.integers(0, 60, n).astype(np.int32)
    dst = rng.integers(0, 60, n).astype(np.int32)
    w = rng.random(n).astype(np.float32) * 4 + 1
    rec = np.zeros(n, dtype=[("s", "<i4"), ("d", "<i4"), ("w", "<f4")])
    rec["s"], rec["d"], rec["w"] = src, dst, w
    path = tmp_path / "g.data"
    rec.tofile(path)
    g = nd.Graph.load(path, "edge-list", "binary")
    ref = nd.Graph.from_edges(src, dst, w)
    assert np.array_equal(g.row_ptr, ref.row_ptr) and np.array_equal(g.col, ref.col)
    assert np.array_equal(g.weight, ref.weight)
    # numpy restatement of the layout
    order = np.lexsort((w, dst, src))
    assert np.array_equal(g.col, dst[order]) and np.array_equal(g.weight, w[order])
    V = max(src.max(), dst.max()) + 1
    assert g.n_vertices == V
    assert np.array_equal(g.row_ptr, np.concatenate([[0], np.cumsum(np.bincount(src, minlength=V))]))


def test_text_loaders(tmp_path):
    p = tmp_path / "e.txt"
    p.write_text("# comment\n0 1 2.5\n1 0 1.5\n1 2\n")
    g = nd.Graph.load(p, "edge-list", "text")
    assert list(g.row_ptr) == [0, 1, 3, 3] and list(g.col) == [1, 0, 2] and list(g.weight) == [2.5, 1.5, 1.0]
    a = tmp_path / "a.txt"
    a.write_text("10 20 1.0 30 2.0\n20 10 1.0\n30\n")
    g = nd.Graph.load(a, "adj-list", "text")
    assert g.n_vertices == 3 and list(g.col) == [1, 2, 0]


def test_loader_errors_are_reported():
    with pytest.raises(nd.NextDoorError):
        nd.Graph.load("/nonexistent/file", "edge-list", "binary")
    with pytest.raises(nd.NextDoorError):
        nd.Graph.load("/nonexistent/file", "bogus", "binary")
    with pytest.raises(nd.NextDoorError):
        nd.Graph.from_edges([0, -1], [1, 0])


def test_rmat_is_seeded_sorted_and_symmetric():
    a = nd.Graph.rmat(10, 8, seed=42, symmetrise=True)
    b = nd.Graph.rmat(10, 8, seed=42, symmetrise=True)
    c = nd.Graph.rmat(10, 8, seed=43, symmetrise=True)
    assert a.n_vertices == 1024 and a.n_edges == 2 * 8 * 1024
    assert np.array_equal(a.col, b.col) and np.array_equal(a.weight, b.weight)
    assert not np.array_equal(a.col, c.col)
    rp, col, w = a.row_ptr, a.col, a.weight
    assert w.min() >= 1.0 and w.max() < 5.0
    src = np.repeat(np.arange(1024), np.diff(rp))
    # sorted by (dst, weight) inside every adjacency
    same = src[1:] == src[:-1]
    assert np.all((col[1:] > col[:-1]) | ((col[1:] == col[:-1]) & (w[1:] >= w[:-1])) | ~same)
    # symmetric as a multiset of (u, v, w)
    fwd = np.lexsort((w, col, src))
    rev = np.lexsort((w, src, col))
    assert np.array_equal(src[fwd], col[rev]) and np.array_equal(col[fwd], src[rev]) and np.array_equal(w[fwd], w[rev])
    # skewed: the heaviest vertex has far more than the mean degree
    assert np.diff(rp).max() > 20 * np.diff(rp).mean()


def test_chung_lu_is_seeded_and_power_law():
    g = nd.Graph.chung_lu(5000, 80000, 2.1, seed=42)
    h = nd.Graph.chung_lu(5000, 80000, 2.1, seed=42)
    assert g.n_vertices == 5000 and g.n_edges == 80000
    assert np.array_equal(g.col, h.col)
    deg = np.diff(g.row_ptr)
    assert deg[:10].mean() > 30 * deg[2500:].mean()
