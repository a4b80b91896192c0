"""Committed fixtures under tests/golden/: the published Philox known-answer vectors, and the
samples of every short app on a small fixed graph (written by tests/golden/make_vectors.py
from this repository's oracle).  On the CPU the oracle must still reproduce them; on the GPU
the library must produce them through the C ABI - without the oracle in the loop."""
import json
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    with open(os.path.join(GOLDEN, name)) as f:
        return json.load(f)


def test_philox_known_answer_file(oracle):
    kat = load("philox4x32_10_kat.json")
    assert len(kat["vectors"]) == 3
    for v in kat["vectors"]:
        ctr = [int(x, 16) for x in v["counter"]]
        key = [int(x, 16) for x in v["key"]]
        assert [f"{x:08x}" for x in oracle.philox(ctr, key)] == v["expected"]


def test_oracle_still_produces_the_committed_vectors(oracle, tmp_path, monkeypatch):
    import importlib.util
    spec = importlib.util.spec_from_file_location("make_vectors", os.path.join(GOLDEN, "make_vectors.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    monkeypatch.setattr(mod, "HERE", str(tmp_path))
    mod.main()
    with open(tmp_path / "sampler_vectors.json") as f:
        fresh = json.load(f)
    assert fresh == load("sampler_vectors.json")


APPS = ["UniformRandomWalk8", "WeightedNode2Vec8", "WeightedNode2Vec8P4Q05", "WeightedNode2Vec8P05Q4", "DeepWalkPerVertex", "PPRPerVertex", "Node2VecPerVertex",
        "KHop3x2", "KHop4x3x2", "MultiRW4x6", "LayerLiteral2x8", "FastGCNImportance2x8", "LADIESImportance2x8",
        "MVS5", "ClusterGCN3x2"]


def test_fixture_covers_the_short_apps():
    assert sorted(load("sampler_vectors.json")["apps"]) == sorted(APPS)


@pytest.mark.gpu
@pytest.mark.parametrize("app", APPS)
def test_library_produces_the_committed_vectors(app):
    import nextdoor_amd as nd
    fx = load("sampler_vectors.json")
    gr, want = fx["graph"], fx["apps"][app]
    g = nd.Graph.from_csr(gr["row_ptr"], gr["col"], np.array(gr["weight"], np.float32))
    s = nd.Sampler(app, g, seed=fx["seed"])
    try:
        assert s.initial_contents.tolist() == want["initial"]
        for lb in (True, False):
            print("app", app, "lb", lb, flush=True)
            s.do_transit_parallel(lb)
            got = s.final_samples()
            if "final" in want:
                assert list(got.shape) == want["shape"]
                assert got.reshape(-1).tolist() == want["final"]
            if "list_start" in want:  # edge lists of MVS / ClusterGCN
                rows, cols, start = s.adjacency()
                assert start.tolist() == want["list_start"]
                assert rows.tolist() == want["rows"] and cols.tolist() == want["cols"]
        if "state_t" in want:  # Node2VecSample::t; -1 in the fixture = never set (the library keeps its initial value)
            st = s.sample_states().view(np.int32)
            t = np.array(want["state_t"])
            assert np.array_equal(st[t != -1], t[t != -1])
        if "walkers" in want:  # MultiRWSample: rootVertices[4], lastRootIdx
            st = s.sample_states().view(np.int32).reshape(s.num_samples, 5)
            assert st[:, :4].reshape(-1).tolist() == want["walkers"]
            assert st[:, 4].tolist() == want["last_root_idx"]
        if "rows" in want and "list_start" not in want:  # LayerSampleT<2, 8>: len[2], row[2][64], col[2][64], val[2][64]
            st = s.sample_states().view(np.int32).reshape(s.num_samples, -1)
            assert st[:, 2:2 + 128].reshape(-1).tolist() == want["rows"]
            assert st[:, 2 + 128:2 + 256].reshape(-1).tolist() == want["cols"]
    finally:
        s.close()


# ---- vectors decided by the reference's own functor sources --------------------------------
# tests/golden/reference_functor_vectors.json was written by make_reference_functor_vectors.py
# from the reference's khop.cu / randomWalks.cu compiled on the CPU (see that script); neither
# the reference tree nor that build is needed here.

REFERENCE_APPS = {"KHop": "KHOP", "DeepWalk": "DEEPWALK", "PPR": "PPR", "Node2Vec": "NODE2VEC", "Layer": "KHOP"}


@pytest.mark.parametrize("app", sorted(REFERENCE_APPS))
def test_oracle_produces_what_the_reference_functors_do(oracle, app):
    fx = load("reference_functor_vectors.json")
    gr, want = fx["graph"], fx["apps"][app]
    g = oracle.Graph(gr["row_ptr"], gr["col"], gr["weight"])
    d = oracle.app_desc(getattr(oracle, REFERENCE_APPS[app]), want["steps"], want["step_sizes"])
    final, state = oracle.sample_individual(g, d, fx["seed"], np.array(want["initial"], np.int32))
    assert list(final.shape) == want["shape"]
    assert final.reshape(-1).tolist() == want["final"]
    if "state_t" in want:
        moved = final[:, 0] != g.n_vertices
        assert np.array_equal(state[moved], np.array(want["state_t"], np.int32)[moved])


@pytest.mark.gpu
@pytest.mark.parametrize("app", sorted(REFERENCE_APPS))
def test_library_produces_what_the_reference_functors_do(app):
    """The registry apps under the reference's names and sizes: the first samples of a run are
    the fixture's (a sample's values depend on its index and root only)."""
    import nextdoor_amd as nd
    fx = load("reference_functor_vectors.json")
    gr, want = fx["graph"], fx["apps"][app]
    g = nd.Graph.from_csr(gr["row_ptr"], gr["col"], np.array(gr["weight"], np.float32))
    s = nd.Sampler(app, g, seed=fx["seed"])
    try:
        kept = want["shape"][0]
        assert s.num_samples == want["samples_of_the_app"]
        assert [s.step_size(k) for k in range(s.steps)] == want["step_sizes"]
        assert s.initial_contents[:kept].tolist() == want["initial"]
        for lb in (True, False):
            print("app", app, "lb", lb, flush=True)
            s.do_transit_parallel(load_balancing=lb)
            got = s.final_samples()[:kept]
            assert got.reshape(-1).tolist() == want["final"]
            if "state_t" in want:
                t = s.sample_states().view(np.int32)[:kept]
                moved = got[:, 0] != g.n_vertices
                assert np.array_equal(t[moved], np.array(want["state_t"], np.int32)[moved])
    finally:
        s.close()


def test_oracle_produces_what_the_reference_multirw_functor_does(oracle):
    fx = load("reference_functor_vectors.json")
    gr, want = fx["graph"], fx["apps"]["MultiRW"]
    g = oracle.Graph(gr["row_ptr"], gr["col"], gr["weight"])
    n, steps, n_roots = want["shape"][0], want["steps"], want["n_roots"]
    roots = np.array(want["roots"], np.int32).reshape(n, n_roots)
    assert np.array_equal(roots, oracle.multirw_roots(n, n_roots, g.n_vertices))
    final, walkers, last, _ = oracle.sample_multirw(g, fx["seed"], roots, steps)
    assert final.reshape(-1).tolist() == want["final"]
    assert walkers.reshape(-1).tolist() == want["walkers"] and last.tolist() == want["last_root_idx"]


@pytest.mark.gpu
def test_library_produces_what_the_reference_multirw_functor_does():
    import nextdoor_amd as nd
    fx = load("reference_functor_vectors.json")
    gr, want = fx["graph"], fx["apps"]["MultiRW"]
    g = nd.Graph.from_csr(gr["row_ptr"], gr["col"], np.array(gr["weight"], np.float32))
    s = nd.Sampler("MultiRW", g, seed=fx["seed"])
    try:
        n, n_roots = want["shape"][0], want["n_roots"]
        assert (s.num_samples, s.steps) == (n, want["steps"])
        for lb in (True, False):
            print("app MultiRW lb", lb, flush=True)
            s.do_transit_parallel(load_balancing=lb)
            assert s.final_samples().reshape(-1).tolist() == want["final"]
            state = s.sample_states().view(np.int32).reshape(n, n_roots + 1)
            assert state[:, :n_roots].reshape(-1).tolist() == want["walkers"]
            assert state[:, n_roots].tolist() == want["last_root_idx"]
    finally:
        s.close()
