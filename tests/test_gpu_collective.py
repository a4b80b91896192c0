"""GPU parity of the layer-wise (CollectiveNeighborhood) engine against the CPU oracle:
collective-neighbourhood build, the reference's FastGCN/LADIES app (vertices, recorded
adjacency-matrix entries, the reference's validator) and the importance sampler."""
import numpy as np
import pytest

import nextdoor_amd as nd
from tests import graphs

pytestmark = pytest.mark.gpu

SEED = 42


def test_collective_neighborhood_matches_oracle(oracle):
    g = graphs.random_graph(n=400, mean_degree=5, seed=11, isolated_every=6, hub=9)
    og = graphs.oracle_view(g)
    rng = np.random.default_rng(0)
    S, B = 37, 300  # more transits than one scan chunk of 256
    transits = rng.integers(0, g.n_vertices + 1, (S, B)).astype(np.int32)  # includes INVALID (= n_vertices)
    transits[3] = g.n_vertices  # a sample with nothing but INVALID transits
    sizes, offsets, cols, weights, rows = nd.collective_neighborhood(g, transits, B, g.n_vertices, 1 << 22)
    assert offsets[0] == 0 and np.array_equal(np.cumsum(sizes), offsets[1:])
    for s in range(S):
        wc, ww, wr = oracle.collective_neighborhood(og, transits[s], g.n_vertices)
        assert sizes[s] == len(wc)
        assert np.array_equal(cols[offsets[s]:offsets[s + 1]], wc)
        assert np.array_equal(weights[offsets[s]:offsets[s + 1]], ww)
        assert np.array_equal(rows[s], wr)
    assert sizes[3] == 0


def layer_desc(oracle, s, kind):
    return oracle.app_desc(kind, s.steps, [s.step_size(k) for k in range(s.steps)],
                           initial_size=s.initial_sample_size)


@pytest.mark.parametrize("app,layers,batch", [("LayerLiteral2x8", 2, 8), ("LayerLiteral3x16", 3, 16)])
def test_layer_literal_matches_oracle(oracle, app, layers, batch):
    g = graphs.random_graph(n=300, mean_degree=8, seed=5, hub=2)
    og = graphs.oracle_view(g)
    s = nd.Sampler(app, g, seed=SEED)
    d = layer_desc(oracle, s, oracle.LAYER_LITERAL)
    roots = s.initial_contents
    assert np.array_equal(roots, np.arange(s.num_samples * batch) % g.n_vertices)  # fastgcnSampling.cu:75-85
    want, want_rows, want_cols = oracle.sample_layer_literal(og, d, SEED, roots)
    for lb in (False, True):
        print("app", app, "lb", lb, flush=True)
        s.do_transit_parallel(lb)
        got = s.final_samples()
        assert np.array_equal(got, want)
        # LayerSampleT: int len[L]; int row[L][B*B]; int col[L][B*B]; int val[L][B*B]
        st = s.sample_states().view(np.int32).reshape(s.num_samples, -1)
        bb = batch * batch
        assert st.shape[1] == layers + 3 * layers * bb
        got_rows = st[:, layers:layers + layers * bb].reshape(-1, layers, bb)
        got_cols = st[:, layers + layers * bb:layers + 2 * layers * bb].reshape(-1, layers, bb)
        assert np.array_equal(got_rows, want_rows) and np.array_equal(got_cols, want_cols)
        assert np.all(st[:, :layers] == 0)
    # the reference's own validator on the GPU result
    assert oracle.check_adjacency_matrix(og, d, roots, got, got_rows, got_cols, s.invalid_vertex)
    assert s.check_results() == (True, "")  # and the library's
    print("app", app, "sample parallel", flush=True)
    s.do_sample_parallel()
    assert np.array_equal(s.final_samples(), want)
    s.close()


@pytest.mark.parametrize("app", ["FastGCNImportance2x8", "FastGCNImportance3x16"])
@pytest.mark.parametrize("gname", ["sparse", "hub"])
def test_fastgcn_importance_matches_oracle(oracle, app, gname):
    g = (graphs.random_graph(n=300, mean_degree=3, seed=1, isolated_every=4) if gname == "sparse"
         else graphs.random_graph(n=2000, mean_degree=12, seed=2, hub=5))
    og = graphs.oracle_view(g)
    s = nd.Sampler(app, g, seed=SEED)
    d = layer_desc(oracle, s, oracle.FASTGCN_IMPORTANCE)
    roots = s.initial_contents
    assert roots.min() >= 0 and roots.max() < g.n_vertices
    want = oracle.sample_fastgcn_importance(og, d, SEED, roots)
    print("app", app, "graph", gname, flush=True)
    s.do_transit_parallel(True)
    got = s.final_samples()
    assert np.array_equal(got, want)
    # every drawn vertex is a neighbour of some vertex of the previous layer
    B = s.step_size(0)
    for row, init in list(zip(got, roots.reshape(-1, s.initial_sample_size)))[:40]:
        prev = init
        for k in range(s.steps):
            cur = row[k * B:(k + 1) * B]
            for v in cur[cur != s.invalid_vertex]:
                assert any(p != s.invalid_vertex and oracle.lib().ndo_has_edge(og.struct, int(p), int(v)) for p in prev)
            prev = cur
    s.do_transit_parallel(True)
    assert np.array_equal(s.final_samples(), want)
    assert s.check_results() == (True, "")
    s.close()


@pytest.mark.parametrize("app", ["FastGCNImportance2x8", "FastGCNImportance3x16", "LADIESImportance2x8",
                                 "LADIESImportance3x16"])
def test_importance_sampling_with_ready_made_hub_pieces(oracle, app, monkeypatch):
    """Vertices with many edges into one stretch of the vertex range contribute a piece built
    once per graph (a bitmap, or the importance sums) instead of their entries: same samples,
    with or without."""
    g = graphs.random_graph(n=2000, mean_degree=12, seed=2, hub=5)
    og = graphs.oracle_view(g)
    monkeypatch.setenv("ND_DENSE_PIECE_ENTRIES", "0")
    s = nd.Sampler(app, g, seed=SEED)
    assert s.counter(3) == 0
    ladies = app.startswith("LADIES")
    d = layer_desc(oracle, s, oracle.LADIES_IMPORTANCE if ladies else oracle.FASTGCN_IMPORTANCE)
    want = (oracle.sample_ladies_importance if ladies else oracle.sample_fastgcn_importance)(
        og, d, SEED, s.initial_contents)
    s.do_transit_parallel(True)
    assert np.array_equal(s.final_samples(), want)
    s.close()
    for entries in ("4", "16", "400"):
        monkeypatch.setenv("ND_DENSE_PIECE_ENTRIES", entries)
        s = nd.Sampler(app, g, seed=SEED)
        print("app", app, "pieces from", entries, "entries:", s.counter(3), flush=True)
        assert s.counter(3) > 0
        s.do_transit_parallel(True)
        assert np.array_equal(s.final_samples(), want)
        s.do_transit_parallel(True)
        assert np.array_equal(s.final_samples(), want)
        s.close()


@pytest.mark.parametrize("app", ["FastGCNImportance3x16", "LADIESImportance3x16"])
@pytest.mark.parametrize("pieces", ["default", "8", "0"])
def test_importance_sampling_over_several_stretches(oracle, app, pieces, monkeypatch):
    """130,000 vertices: two stretches of the FastGCN form, 19 of the LADIES form (two
    workgroups per sample), a hub with edges into all of them."""
    if pieces != "default":
        monkeypatch.setenv("ND_DENSE_PIECE_ENTRIES", pieces)
    g = graphs.random_graph(n=130000, mean_degree=3, seed=5, hub=8, isolated_every=6)
    og = graphs.oracle_view(g)
    s = nd.Sampler(app, g, seed=SEED)
    ladies = app.startswith("LADIES")
    d = layer_desc(oracle, s, oracle.LADIES_IMPORTANCE if ladies else oracle.FASTGCN_IMPORTANCE)
    want = (oracle.sample_ladies_importance if ladies else oracle.sample_fastgcn_importance)(
        og, d, SEED, s.initial_contents)
    print("app", app, "pieces", pieces, "built", s.counter(3), flush=True)
    # without pieces the hub's 260,000 edges go through the entry-by-entry path (and the
    # attempt to take a workgroup's stretches at once gives up on their number)
    assert (s.counter(3) > 0) == (pieces != "0")
    s.do_transit_parallel(True)
    assert np.array_equal(s.final_samples(), want)
    s.close()


def test_distinct_is_refused_for_layer_apps():
    g = graphs.random_graph(n=100, mean_degree=4, seed=1)
    s = nd.Sampler("LayerLiteral2x8", g, seed=SEED)
    s.do_transit_parallel(True)
    with pytest.raises(nd.NextDoorError):
        s.distinct()
    s.close()


@pytest.mark.parametrize("app", ["LADIESImportance2x8", "LADIESImportance3x16"])
@pytest.mark.parametrize("gname", ["sparse", "hub"])
def test_ladies_importance_matches_oracle(oracle, app, gname):
    g = (graphs.random_graph(n=300, mean_degree=3, seed=1, isolated_every=4) if gname == "sparse"
         else graphs.random_graph(n=2000, mean_degree=12, seed=2, hub=5))
    og = graphs.oracle_view(g)
    s = nd.Sampler(app, g, seed=SEED)
    d = layer_desc(oracle, s, oracle.LADIES_IMPORTANCE)
    roots = s.initial_contents
    want = oracle.sample_ladies_importance(og, d, SEED, roots)
    print("app", app, "graph", gname, flush=True)
    s.do_transit_parallel(True)
    got = s.final_samples()
    assert np.array_equal(got, want)
    # without replacement: no vertex twice inside a layer segment
    B = s.step_size(0)
    for row in got[:100]:
        for k in range(s.steps):
            seg = row[k * B:(k + 1) * B]
            seg = seg[seg != s.invalid_vertex]
            assert len(set(seg.tolist())) == len(seg)
    assert s.check_results() == (True, "")
    s.close()


@pytest.mark.parametrize("app,kind_name", [("FastGCNImportance3x16", "FASTGCN_IMPORTANCE"),
                                           ("LADIESImportance3x16", "LADIES_IMPORTANCE"),
                                           ("LayerLiteral3x16", "LAYER_LITERAL")])
def test_chunked_processing_gives_the_same_samples(oracle, app, kind_name, monkeypatch):
    g = graphs.random_graph(n=2000, mean_degree=12, seed=2, hub=5)
    s = nd.Sampler(app, g, seed=SEED)
    s.do_transit_parallel(True)
    whole = s.final_samples()
    assert s.counter(2) == s.steps  # one chunk per layer
    s.close()
    monkeypatch.setenv("ND_LAYER_CHUNK_ENTRIES", "3000")  # a few samples per chunk
    s = nd.Sampler(app, g, seed=SEED)
    s.do_transit_parallel(True)
    assert s.counter(2) > 3 * s.steps
    assert np.array_equal(s.final_samples(), whole)
    s.close()
