"""The reference's own application sources on this engine.  oracle/_ref/libreference_apps_device.so
is src/apps/khop/khop.cu, src/apps/randomwalks/randomWalks.cu, src/apps/fastgcn/fastgcnSampling.cu,
src/apps/ladies/ladiessampling.cu, src/apps/layer/layerSampling.cu and src/apps/multiRW/multiRW.cu
compiled by hipcc from the reference tree against the App contract header (oracle/Makefile),
instantiated on the engine and registered with the library under "Reference..." names - the
samplers dropped in unchanged.  What the GPU samples with them must be the oracle's bytes.
The shared object is built where the reference tree is (oracle/Makefile) and travels with the
tree; where the build was skipped because there was no reference tree, oracle/_ref does not
exist and there is nothing to test - but a build that was due and is missing is a failure."""
import ctypes as C
import os

import numpy as np
import pytest

import nextdoor_amd as nd
from tests import graphs, oracle_binding as ob

REF_DIR = os.path.join(ob.ORACLE_DIR, "_ref")
REF_LIB = os.path.join(REF_DIR, "libreference_apps_device.so")
# no oracle/_ref at all: the tree was built without the reference (nothing to run).  The
# directory or the reference tree without the library: the build that was due failed.
BUILD_WAS_DUE = os.path.isdir(REF_DIR) or os.path.exists("/root/reference/src/apps/khop/khop.cu")
pytestmark = [pytest.mark.gpu,
              pytest.mark.skipif(not os.path.exists(REF_LIB) and not BUILD_WAS_DUE,
                                 reason="built without the reference tree: no oracle/_ref")]
SEED = 42
ALL_REFERENCE_APPS = ("ReferenceKHop", "ReferenceDeepWalk", "ReferencePPR", "ReferenceNode2Vec", "ReferenceFastGCN",
                      "ReferenceLADIES", "ReferenceLayer", "ReferenceMultiRW")


@pytest.fixture(scope="module")
def reference_apps():
    assert os.path.exists(REF_LIB), "oracle/_ref/libreference_apps_device.so is missing although its build was due"
    nd.app_names()  # the library first: the shared object registers its apps with it when loaded
    handle = C.CDLL(REF_LIB, mode=C.RTLD_GLOBAL)
    names = nd.app_names()
    for app in ALL_REFERENCE_APPS:
        assert app in names
    return handle


@pytest.mark.parametrize("gname", ["sparse", "hub"])
@pytest.mark.parametrize("app,kind,state", [("ReferenceKHop", "KHOP", False), ("ReferenceDeepWalk", "DEEPWALK", False),
                                            ("ReferencePPR", "PPR", False), ("ReferenceNode2Vec", "NODE2VEC", True),
                                            ("ReferenceLayer", "KHOP", False)])
def test_reference_app_sources_on_the_engine_match_the_oracle(reference_apps, app, kind, state, gname):
    g = graphs.random_graph(**{"sparse": dict(n=300, mean_degree=3, seed=1, isolated_every=7),
                               "hub": dict(n=400, mean_degree=10, seed=2, hub=5)}[gname])
    og = graphs.oracle_view(g)
    s = nd.Sampler(app, g, seed=SEED)
    try:
        # the reference's own sizing: one k-hop sample per vertex, 100 walks per vertex
        assert s.num_samples == (g.n_vertices if kind == "KHOP" else 100 * g.n_vertices)
        if app == "ReferenceLayer":
            assert [s.step_size(k) for k in range(s.steps)] == [10, 25]
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


@pytest.mark.parametrize("app", ["ReferenceFastGCN", "ReferenceLADIES"])
def test_reference_fastgcn_source_on_the_engine_matches_the_oracle(reference_apps, app):
    # 10,000 samples of 64 roots, 5 layers of 64 (fastgcnSampling.cu:1-4, ladiessampling.cu:1-4),
    # the adjacency towards the previous layer recorded in the sample state
    g = graphs.random_graph(n=500, mean_degree=30, seed=3, hub=9)
    og = graphs.oracle_view(g)
    s = nd.Sampler(app, g, seed=SEED)
    try:
        B, layers = 64, 5
        assert (s.num_samples, s.steps, s.final_sample_size, s.initial_sample_size) == (10000, layers, layers * B, B)
        d = ob.app_desc(ob.LAYER_LITERAL, layers, [B] * layers, initial_size=B)
        check = 300  # samples compared with the oracle (every sample's state is 245 KB)
        roots = s.initial_contents.reshape(s.num_samples, B)
        want, want_rows, want_cols = ob.sample_layer_literal(og, d, SEED, roots[:check].reshape(-1))
        print("app", app, flush=True)
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


def test_reference_multirw_source_on_the_engine_matches_the_oracle(reference_apps):
    # src/apps/multiRW/multiRW.cu as it is: 100 walkers per sample whose start vertices its
    # initializeSample draws with rand(); they are read back from the sample states the
    # allocation left on the device and handed to the oracle
    g = graphs.random_graph(n=300, mean_degree=4, seed=13, hub=2, isolated_every=9)
    og = graphs.oracle_view(g)
    s = nd.Sampler("ReferenceMultiRW", g, seed=SEED)
    try:
        assert (s.steps, s.final_sample_size, s.num_samples) == (100, 100, g.n_vertices)
        roots = s.sample_states().view(np.int32).reshape(s.num_samples, 101)[:, :100].copy()
        assert roots.min() >= 0 and roots.max() < g.n_vertices and len(np.unique(roots)) > g.n_vertices // 2
        assert np.array_equal(s.initial_contents, roots[:, 0])  # multiRW.cu:68-73
        want, want_walkers, want_last, _ = ob.sample_multirw(og, SEED, roots, 100)
        for lb in (False, True, "sample_parallel"):
            print("app ReferenceMultiRW lb", lb, flush=True)
            if lb == "sample_parallel":
                s.do_sample_parallel()
            else:
                s.do_transit_parallel(load_balancing=lb)
            assert np.array_equal(s.final_samples(), want)
            state = s.sample_states().view(np.int32).reshape(s.num_samples, 101)
            assert np.array_equal(state[:, :100], want_walkers) and np.array_equal(state[:, 100], want_last)
    finally:
        s.close()
