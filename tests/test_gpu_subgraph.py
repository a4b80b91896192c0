"""GPU parity of the edge-list apps (MVS, ClusterGCN) against the CPU oracle: the same lists,
byte for byte, in the same places."""
import numpy as np
import pytest

import nextdoor_amd as nd
from tests import graphs

pytestmark = pytest.mark.gpu

GRAPHS = {
    "sparse": dict(n=300, mean_degree=3, seed=1, isolated_every=7),
    "dense_hub": dict(n=1000, mean_degree=40, seed=2, hub=5),
}


@pytest.mark.parametrize("gname", list(GRAPHS))
@pytest.mark.parametrize("app,batch", [("MVS", 32), ("MVS5", 5)])
def test_mvs_matches_oracle(oracle, app, batch, gname):
    g = graphs.random_graph(**GRAPHS[gname])
    og = graphs.oracle_view(g)
    s = nd.Sampler(app, g, seed=42)
    try:
        n = oracle.subgraph_num_samples(og, batch, 1500000)
        assert (s.num_samples, s.steps, s.step_size(0), s.initial_sample_size) == (n, 1, batch, batch)
        assert s.final_sample_size == batch * batch
        verts = oracle.mvs_vertices(og, n, batch)
        assert np.array_equal(s.initial_contents, verts.ravel())
        want_rows, want_cols, want_start = oracle.sample_mvs(og, verts)
        for run in range(2):
            print("app", app, "graph", gname, "run", run, flush=True)
            s.do_transit_parallel(load_balancing=bool(run))
            rows, cols, start = s.adjacency()
            assert np.array_equal(start, want_start)
            assert np.array_equal(rows, want_rows) and np.array_equal(cols, want_cols)
            assert np.all(s.final_samples() == g.n_vertices)  # next() samples no vertex
        assert np.array_equal(s.sample_states().view(np.int32).reshape(n, batch), verts)
        assert s.counter(0) == len(want_rows)
        assert s.check_results() == (True, "")
        with pytest.raises(nd.NextDoorError):
            s.distinct()
    finally:
        s.close()


@pytest.mark.parametrize("gname", list(GRAPHS))
@pytest.mark.parametrize("app,cluster,per_sample", [("ClusterGCN", 16, 2), ("ClusterGCN3x2", 3, 2)])
def test_clustergcn_matches_oracle(oracle, app, cluster, per_sample, gname):
    g = graphs.random_graph(**GRAPHS[gname])
    og = graphs.oracle_view(g)
    s = nd.Sampler(app, g, seed=42)
    try:
        size = cluster * per_sample
        n = oracle.subgraph_num_samples(og, size, 2000000)
        assert (s.num_samples, s.steps, s.step_size(0), s.step_size(1)) == (n, 2, 1, size)
        assert s.final_sample_size == size + size * size
        verts = oracle.clustergcn_vertices(og, n, cluster, per_sample)
        assert np.array_equal(s.initial_contents, verts.ravel())
        want_final, want_rows, want_cols, want_start = oracle.sample_clustergcn(og, verts)
        for mode in ("transit", "sample"):
            print("app", app, "graph", gname, "mode", mode, flush=True)
            if mode == "transit":
                s.do_transit_parallel(load_balancing=True)
            else:
                s.do_sample_parallel()
            rows, cols, start = s.adjacency()
            assert np.array_equal(start, want_start)
            assert np.array_equal(rows, want_rows) and np.array_equal(cols, want_cols)
            assert np.array_equal(s.final_samples(), want_final)
        assert s.check_results() == (True, "")
    finally:
        s.close()


def test_power_law_graph_with_long_hub_lists(oracle):
    # R-MAT scale 14: the low vertex ids are hubs with thousands of edges, so single lanes of
    # MVS copy hundreds of edges and whole units interleave many rounds
    g = nd.Graph.rmat(14, 16, seed=7, symmetrise=True)
    og = graphs.oracle_view(g)
    assert np.diff(g.row_ptr).max() > 2000
    for app in ("MVS", "ClusterGCN"):
        s = nd.Sampler(app, g, seed=3)
        try:
            print("app", app, "rmat14", flush=True)
            s.do_transit_parallel()
            rows, cols, start = s.adjacency()
            if app == "MVS":
                want_rows, want_cols, want_start = oracle.sample_mvs(og, oracle.mvs_vertices(og, s.num_samples, 32))
            else:
                verts = oracle.clustergcn_vertices(og, s.num_samples, 16, 2)
                want_final, want_rows, want_cols, want_start = oracle.sample_clustergcn(og, verts)
                assert np.array_equal(s.final_samples(), want_final)
            assert np.array_equal(start, want_start)
            assert np.array_equal(rows, want_rows) and np.array_equal(cols, want_cols)
            assert s.check_results() == (True, "")
        finally:
            s.close()


def test_graph_without_edges_gives_empty_lists():
    g = nd.Graph.from_edges([], [], [], n_vertices=64)
    for app in ("MVS", "ClusterGCN"):
        s = nd.Sampler(app, g, seed=1)
        print("app", app, "no edges", flush=True)
        s.do_transit_parallel()
        rows, cols, start = s.adjacency()
        assert len(rows) == 0 and len(cols) == 0 and np.all(start == 0) and len(start) == s.num_samples + 1
        assert np.all(s.final_samples() == 64)
        s.close()


def test_other_apps_have_no_edge_lists():
    g = graphs.random_graph(n=100, mean_degree=4, seed=1)
    s = nd.Sampler("KHop3x2", g, seed=1)
    s.do_transit_parallel()
    with pytest.raises(nd.NextDoorError):
        s.adjacency()
    s.close()
