"""Applications that are not compiled into the library.  tests/cpp/user_apps.hip holds two App
structs written on the contract the way a user of the reference writes them, built by hipcc
into a shared object of its own that registers them when it loads (ND_REGISTER_APP); what the
engine samples with them is the oracle's bytes.  Then the per-app Python module surface
(src/nextDoorPythonModule.cu:40-102) end to end on a binary edge-list file."""
import os

import numpy as np
import pytest

import nextdoor_amd as nd
from tests import graphs, oracle_binding as ob
from tests.cpp.build_cpp import USER_APPS_LIB

SEED = 42


@pytest.mark.gpu
@pytest.mark.parametrize("gname", ["sparse", "hub"])
@pytest.mark.parametrize("app,kind,sizes", [("UserThreeHop", "KHOP", [5, 3, 2]),
                                            ("UserShortDeepWalk", "DEEPWALK", [1] * 7)])
def test_apps_registered_from_their_own_shared_object_match_the_oracle(app, kind, sizes, gname):
    assert os.path.exists(USER_APPS_LIB), "tests/cpp/libuser_apps.so is built by __graft_entry__.build()"
    nd.load_app_library(USER_APPS_LIB)
    assert app in nd.app_names()
    g = graphs.random_graph(**{"sparse": dict(n=300, mean_degree=3, seed=1, isolated_every=7),
                               "hub": dict(n=400, mean_degree=10, seed=2, hub=5)}[gname])
    og = graphs.oracle_view(g)
    s = nd.Sampler(app, g, seed=SEED)
    try:
        assert [s.step_size(k) for k in range(s.steps)] == sizes
        assert s.num_samples == (g.n_vertices if kind == "KHOP" else 3 * g.n_vertices)
        if kind == "DEEPWALK":
            assert np.array_equal(s.initial_contents, np.arange(s.num_samples, dtype=np.int32) % g.n_vertices)
        d = ob.app_desc(getattr(ob, kind), s.steps, sizes)
        want, _ = ob.sample_individual(og, d, SEED, s.initial_contents)
        for lb in (False, True):
            print("app", app, "graph", gname, "lb", lb, flush=True)
            s.do_transit_parallel(load_balancing=lb)
            assert np.array_equal(s.final_samples(), want)
            assert s.check_results() == (True, "")
        s.do_sample_parallel()
        assert np.array_equal(s.final_samples(), want)
    finally:
        s.close()


@pytest.mark.gpu
@pytest.mark.parametrize("gname", ["sparse", "hub"])
def test_an_app_with_explicit_transits_and_several_transits_per_sample(gname):
    """stepTransits decides the next step's transits (src/nextdoor.cu:279-289) for an app that is
    not a walk: four transits per sample, step sizes 2, 3, 2; every schedule gives the oracle's bytes."""
    nd.load_app_library(USER_APPS_LIB)
    g = graphs.random_graph(**{"sparse": dict(n=300, mean_degree=3, seed=1, isolated_every=7),
                               "hub": dict(n=1200, mean_degree=10, seed=2, hub=5)}[gname])
    og = graphs.oracle_view(g)
    s = nd.Sampler("UserAnchorHop", g, seed=SEED)
    try:
        assert (s.steps, s.initial_sample_size, s.final_sample_size) == (3, 4, 8 + 24 + 48)
        anchors = s.initial_contents.reshape(-1, 4)
        assert np.array_equal(anchors, np.stack([(np.arange(g.n_vertices) * 7 + i * 13) % g.n_vertices
                                                 for i in range(4)], axis=1))
        want, _ = ob.sample_anchor_hop(og, SEED, anchors, [2, 3, 2])
        for mode in (False, True, "sample_parallel", True):
            print("UserAnchorHop", gname, mode, flush=True)
            if mode == "sample_parallel":
                s.do_sample_parallel()
            else:
                s.do_transit_parallel(load_balancing=mode)
            assert np.array_equal(s.final_samples(), want)
        with pytest.raises(nd.NextDoorError):  # explicit transits: the library has no validator
            s.check_results()
    finally:
        s.close()


def write_binary_edge_list(path, src, dst, weight):
    """The reference's binary edge list: 12-byte records (int32 src, int32 dst, float32 weight),
    src/graph.hpp:42-75."""
    rec = np.zeros(len(src), dtype=[("s", "<i4"), ("d", "<i4"), ("w", "<f4")])
    rec["s"], rec["d"], rec["w"] = src, dst, weight
    rec.tofile(path)


def edges_of(g):
    src = np.repeat(np.arange(g.n_vertices, dtype=np.int32), np.diff(g.row_ptr))
    return src, g.col.copy(), g.weight.copy()


@pytest.mark.gpu
def test_sampling_module_functions_end_to_end(tmp_path):
    """initSampling -> sample -> finalSampleLength -> finalSamplesArray -> freeDeviceMemory on a
    written file, a second initSampling on another graph and app, and the calls before
    initSampling (the sequence of src/apps/khop/KHopSamplingPy3 users, nextDoorPythonModule.cu)."""
    lib = nd._capi.lib()
    lib.nd_free_device_memory()
    module = nd.SamplingModule("KHop", seed=SEED)
    with pytest.raises(nd.NextDoorError, match="before initSampling"):
        module.sample()
    with pytest.raises(nd.NextDoorError, match="before initSampling"):
        module.finalSamplesArray()
    assert module.finalSampleLength() == 0
    with pytest.raises(nd.NextDoorError):
        module.initSampling(tmp_path / "missing.data")

    cases = [("KHop", ob.KHOP, graphs.random_graph(n=500, mean_degree=8, seed=11, hub=2)),
             ("DeepWalk", ob.DEEPWALK, graphs.random_graph(n=300, mean_degree=4, seed=12, isolated_every=5))]
    for i, (app, kind, g) in enumerate(cases):
        path = tmp_path / f"graph{i}.data"
        write_binary_edge_list(path, *edges_of(g))
        loaded = nd.Graph.load(str(path), "edge-list", "binary")
        assert np.array_equal(loaded.row_ptr, g.row_ptr) and np.array_equal(loaded.col, g.col)
        og = graphs.oracle_view(loaded)
        reference = nd.Sampler(app, loaded, seed=SEED)  # only for the shape and the roots
        steps, sizes, roots = reference.steps, [reference.step_size(k) for k in range(reference.steps)], reference.initial_contents.copy()
        final = reference.final_sample_size
        reference.close()
        want, _ = ob.sample_individual(og, ob.app_desc(kind, steps, sizes), SEED, roots)

        print("SamplingModule", app, flush=True)
        module = nd.SamplingModule(app, seed=SEED)
        module.initSampling(path)  # the second pass replaces the first module state
        for _ in range(2):  # sample() may be called again, as in the reference
            module.sample()
            assert module.finalSampleLength() == want.size
            got = module.finalSamplesArray()
            assert got.dtype == np.int32 and np.array_equal(got.reshape(-1, final), want)
        assert module.finalSamples()[:final] == want[0].tolist()
    # the same sampler from CSR arrays in memory
    app, kind, g = cases[0]
    module = nd.SamplingModule(app, seed=SEED)
    module.initSamplingFromCSR(g.row_ptr, g.col, g.weight)
    module.sample()
    reference = nd.Sampler(app, g, seed=SEED)
    want, _ = ob.sample_individual(graphs.oracle_view(g), ob.app_desc(kind, reference.steps, [reference.step_size(k) for k in range(reference.steps)]),
                                   SEED, reference.initial_contents.copy())
    reference.close()
    assert np.array_equal(module.finalSamplesArray().reshape(want.shape), want)
    module.freeDeviceMemory()
    assert module.finalSampleLength() == 0
    with pytest.raises(nd.NextDoorError, match="before initSampling"):
        module.sample()
    module.freeDeviceMemory()  # twice is harmless
