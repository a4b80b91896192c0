"""The reference's own application sources on this engine.  oracle/_ref/libreference_apps_device.so
is src/apps/khop/khop.cu, src/apps/randomwalks/randomWalks.cu and src/apps/fastgcn/fastgcnSampling.cu
compiled by hipcc from the reference tree against the App contract header (oracle/Makefile),
instantiated on the engine and registered with the library under "Reference..." names - the
samplers dropped in unchanged.  What the GPU samples with them must be the oracle's bytes.
Skipped where that shared object has not been built (no reference tree at build time)."""
import ctypes as C
import os

import numpy as np
import pytest

import nextdoor_amd as nd
from tests import graphs, oracle_binding as ob

REF_LIB = os.path.join(ob.ORACLE_DIR, "_ref", "libreference_apps_device.so")
pytestmark = [pytest.mark.gpu,
              pytest.mark.skipif(not os.path.exists(REF_LIB), reason="oracle/_ref is built from the reference tree")]
SEED = 42


@pytest.fixture(scope="module")
def reference_apps():
    nd.app_names()  # the library first: the shared object registers its apps with it when loaded
    handle = C.CDLL(REF_LIB, mode=C.RTLD_GLOBAL)
    names = nd.app_names()
    for app in ("ReferenceKHop", "ReferenceDeepWalk", "ReferencePPR", "ReferenceNode2Vec", "ReferenceFastGCN"):
        assert app in names
    return handle


@pytest.mark.parametrize("gname", ["sparse", "hub"])
@pytest.mark.parametrize("app,kind,state", [("ReferenceKHop", "KHOP", False), ("ReferenceDeepWalk", "DEEPWALK", False),
                                            ("ReferencePPR", "PPR", False), ("ReferenceNode2Vec", "NODE2VEC", True)])
def test_reference_app_sources_on_the_engine_match_the_oracle(reference_apps, app, kind, state, gname):
    g = graphs.random_graph(**{"sparse": dict(n=300, mean_degree=3, seed=1, isolated_every=7),
                               "hub": dict(n=400, mean_degree=10, seed=2, hub=5)}[gname])
    og = graphs.oracle_view(g)
    s = nd.Sampler(app, g, seed=SEED)
    try:
        # the reference's own sizing: one k-hop sample per vertex, 100 walks per vertex
        assert s.num_samples == (g.n_vertices if kind == "KHOP" else 100 * g.n_vertices)
        d = ob.app_desc(getattr(ob, kind), s.steps, [s.step_size(k) for k in range(s.steps)])
        want, want_t = ob.sample_individual(og, d, SEED, s.initial_contents)
        for lb in (False, True):
            print("app", app, "graph", gname, "lb", lb, flush=True)
            s.do_transit_parallel(load_balancing=lb)
            assert np.array_equal(s.final_samples(), want)
            if state:
                t = s.sample_states().view(np.int32)
                moved = want[:, 0] != g.n_vertices
                assert np.array_equal(t[moved], want_t[moved])
        s.do_sample_parallel()
        assert np.array_equal(s.final_samples(), want)
    finally:
        s.close()


def test_reference_fastgcn_source_on_the_engine_matches_the_oracle(reference_apps):
    # 10,000 samples of 64 roots, 5 layers of 64 (fastgcnSampling.cu:1-4), the adjacency towards
    # the previous layer recorded in the sample state
    g = graphs.random_graph(n=500, mean_degree=30, seed=3, hub=9)
    og = graphs.oracle_view(g)
    s = nd.Sampler("ReferenceFastGCN", g, seed=SEED)
    try:
        B, layers = 64, 5
        assert (s.num_samples, s.steps, s.final_sample_size, s.initial_sample_size) == (10000, layers, layers * B, B)
        d = ob.app_desc(ob.LAYER_LITERAL, layers, [B] * layers, initial_size=B)
        check = 300  # samples compared with the oracle (every sample's state is 245 KB)
        roots = s.initial_contents.reshape(s.num_samples, B)
        want, want_rows, want_cols = ob.sample_layer_literal(og, d, SEED, roots[:check].reshape(-1))
        print("app ReferenceFastGCN", flush=True)
        s.do_transit_parallel(True)
        got = s.final_samples()
        assert np.array_equal(got[:check], want)
        state = s.sample_states().view(np.int32).reshape(s.num_samples, -1)[:check]
        cells = layers * B * B
        assert np.array_equal(state[:, layers:layers + cells].reshape(check, layers, B * B), want_rows)
        assert np.array_equal(state[:, layers + cells:layers + 2 * cells].reshape(check, layers, B * B), want_cols)
        assert s.check_results() == (True, "")
    finally:
        s.close()
