"""GPU parity of the transit-parallel engine against the CPU oracle: same graph, same
roots, same seed -> byte-identical final samples, with load balancing on and off,
for every IndividualNeighborhood app; plus the reference's check_results invariants."""
import numpy as np
import pytest

import nextdoor_amd as nd
from tests import graphs

pytestmark = pytest.mark.gpu

SEED = 42


# return and in-out parameters of the registered weighted node2vec instances (default 2, 0.5)
P_AND_Q = {"WeightedNode2Vec8P4Q05": (4.0, 0.5), "WeightedNode2Vec8P05Q4": (0.5, 4.0)}


def desc_for(oracle, sampler, kind, app=None):
    steps = sampler.steps
    p, q = P_AND_Q.get(app, (2.0, 0.5))
    return oracle.app_desc(kind, steps, [sampler.step_size(k) for k in range(steps)],
                           initial_size=sampler.initial_sample_size, p=p, q=q)


def run_and_compare(oracle, app, kind, g, check_state=False, modes=(False, True), inversion_period=1):
    og = graphs.oracle_view(g)
    s = nd.Sampler(app, g, seed=SEED)
    s.set_inversion_period(inversion_period)
    try:
        d = desc_for(oracle, s, kind, app)
        roots = s.initial_contents
        assert s.invalid_vertex == g.n_vertices
        want, want_state = oracle.sample_individual(og, d, SEED, roots)
        assert want.shape == (s.num_samples, s.final_sample_size)
        for lb in modes:
            print("app", app, "V", g.n_vertices, "E", g.n_edges, "lb", lb, flush=True)
            if lb == "sample_parallel":
                s.do_sample_parallel()
            else:
                s.do_transit_parallel(load_balancing=lb)
            got = s.final_samples()
            if not np.array_equal(got, want):
                bad = np.argwhere(got != want)
                raise AssertionError(f"{app} lb={lb}: {len(bad)} mismatches, first at {bad[0]}: "
                                     f"got {got[tuple(bad[0])]} want {want[tuple(bad[0])]}")
            if check_state:
                st = s.sample_states().view(np.int32)
                alive = want_state != -1
                assert np.array_equal(st[alive], want_state[alive])
        # the reference's own validator; its "nothing sampled only if the previous step had no
        # edges" clause does not hold for PPR, whose walks end at random (the reference runs
        # PPR unchecked: src/tests/singleGPU/ppr.cu:12-30)
        if kind != oracle.PPR:
            assert oracle.check_sampled_vertices(og, d, roots, got, s.invalid_vertex)
            assert s.check_results() == (True, "")  # the library's own validator
        assert oracle.check_exact_transits(og, d, roots, got, s.invalid_vertex)
        return got
    finally:
        s.close()


@pytest.mark.parametrize("period", [0, 3, 1000])
@pytest.mark.parametrize("app,kind_name,state", [
    ("UniformRandomWalk", "UNIFORM_WALK", False),
    ("PPRPerVertex", "PPR", False),
    ("Node2VecPerVertex", "NODE2VEC", True),
    ("WeightedNode2Vec", "WEIGHTED_NODE2VEC", True),
    ("KHop", "KHOP", False),
])
def test_samples_do_not_depend_on_the_inversion_period(oracle, app, kind_name, state, period):
    # walks that re-invert the sample -> transit map only now and then (or when the engine
    # sees fit) give the bytes of the oracle too; for other apps the setting changes nothing
    g = graphs.random_graph(n=1500, mean_degree=6, seed=9, hub=4, isolated_every=11)
    run_and_compare(oracle, app, getattr(oracle, kind_name), g, check_state=state, inversion_period=period)


@pytest.mark.parametrize("app,kind_name,state", [
    ("UniformRandomWalk", "UNIFORM_WALK", False),
    ("DeepWalkPerVertex", "DEEPWALK", False),
    ("WeightedNode2Vec", "WEIGHTED_NODE2VEC", True),
    ("KHop", "KHOP", False),
    ("KHop4x3x2", "KHOP", False),
])
def test_sample_parallel_mode_gives_the_same_samples(oracle, app, kind_name, state):
    # the reference's baseline schedule (no transit order, no load balancing), then the
    # transit-parallel one on the same sampler
    g = graphs.random_graph(n=1500, mean_degree=6, seed=9, hub=4, isolated_every=11)
    run_and_compare(oracle, app, getattr(oracle, kind_name), g, check_state=state,
                    modes=("sample_parallel", True, "sample_parallel"))


@pytest.mark.parametrize("app,kind_name,period", [
    ("UniformRandomWalk", "UNIFORM_WALK", 1),
    ("WeightedNode2Vec", "WEIGHTED_NODE2VEC", 1),
    ("WeightedNode2Vec", "WEIGHTED_NODE2VEC", 0),
    ("KHop", "KHOP", 1),
])
def test_recorded_passes_replay_to_the_same_samples(oracle, app, kind_name, period):
    # a pass recorded as a HIP graph, replayed several times with eager passes, fetches and
    # other modes in between: every replay must give the oracle's bytes
    g = graphs.random_graph(n=1500, mean_degree=6, seed=9, hub=4, isolated_every=11)
    og = graphs.oracle_view(g)
    s = nd.Sampler(app, g, seed=SEED)
    try:
        d = desc_for(oracle, s, getattr(oracle, kind_name))
        want, _ = oracle.sample_individual(og, d, SEED, s.initial_contents)
        s.set_inversion_period(period)
        s.set_launch_graph(1)
        for turn in range(7):
            lb = turn % 3 != 2
            eager = turn == 3
            print("app", app, "period", period, "turn", turn, "lb", lb, "eager", eager, flush=True)
            if eager:
                s.set_profiling(True)  # per-phase events: launches go out one by one
            s.do_transit_parallel(load_balancing=lb)
            if eager:
                s.set_profiling(False)
            assert np.array_equal(s.final_samples(), want), f"turn {turn}"
        s.set_launch_graph(0)
        s.do_transit_parallel(load_balancing=True)
        assert np.array_equal(s.final_samples(), want)
    finally:
        s.close()


def test_command_line_runs_checks_and_prints(oracle, tmp_path):
    import io
    from nextdoor_amd import __main__ as cli
    g = graphs.random_graph(n=120, mean_degree=4, seed=12)
    rec = np.zeros(g.n_edges, dtype=[("s", "<i4"), ("d", "<i4"), ("w", "<f4")])
    rec["s"] = np.repeat(np.arange(g.n_vertices), np.diff(g.row_ptr))
    rec["d"], rec["w"] = g.col, g.weight
    path = tmp_path / "g.data"
    rec.tofile(path)
    for kernel, extra in (("TransitParallel", ["-l"]), ("SampleParallel", [])):
        out = io.StringIO()
        print("cli KHop3x2", kernel, flush=True)
        rc = cli.run(["KHop3x2", "-g", str(path), "-t", "edge-list", "-f", "binary", "-n", "2", "-c", "-p",
                      "-k", kernel] + extra, out=out)
        text = out.getvalue()
        assert rc == 0, text
        assert "Graph has %d edges and %d vertices" % (g.n_edges, g.n_vertices) in text
        assert text.count("Contents of sample") == g.n_vertices and "Results Checked" in text
        d = oracle.app_desc(oracle.KHOP, 2, [3, 2])
        want, _ = oracle.sample_individual(graphs.oracle_view(g), d, 42, np.arange(g.n_vertices, dtype=np.int32))
        assert "totalSampledVertices %d" % np.count_nonzero(want != g.n_vertices) in text
        first = [l for l in text.splitlines() if l.startswith("Contents of sample 0 ")][0]
        assert first == "Contents of sample 0 [%s]" % "".join("%d, " % v for v in want[0])


GRAPHS = {
    "sparse": dict(n=300, mean_degree=3, seed=1, isolated_every=7),
    "dense_hub": dict(n=2000, mean_degree=12, seed=2, hub=5),
    # a tenth of all vertex pairs joined: a candidate is often a neighbour of the previous vertex
    "triangles": dict(n=160, mean_degree=16, seed=5, hub=7),
}


@pytest.mark.parametrize("gname", list(GRAPHS))
@pytest.mark.parametrize("app,kind_name,state", [
    ("UniformRandomWalk", "UNIFORM_WALK", False),
    ("DeepWalkPerVertex", "DEEPWALK", False),
    ("PPRPerVertex", "PPR", False),
    ("Node2VecPerVertex", "NODE2VEC", True),
    ("WeightedNode2Vec", "WEIGHTED_NODE2VEC", True),
    ("WeightedNode2Vec8P4Q05", "WEIGHTED_NODE2VEC", True),
    ("WeightedNode2Vec8P05Q4", "WEIGHTED_NODE2VEC", True),
    ("KHop", "KHOP", False),
    ("KHop4x3x2", "KHOP", False),
])
def test_app_matches_oracle(oracle, app, kind_name, state, gname):
    g = graphs.random_graph(**GRAPHS[gname])
    run_and_compare(oracle, app, getattr(oracle, kind_name), g, check_state=state)


@pytest.mark.parametrize("schedule", ["serial", "merged", "forked"])
@pytest.mark.parametrize("app,kind_name,state", [
    ("UniformRandomWalk", "UNIFORM_WALK", False),
    ("DeepWalkPerVertex", "DEEPWALK", False),
    ("WeightedNode2Vec", "WEIGHTED_NODE2VEC", True),
    ("KHop", "KHOP", False),
    ("KHop4x3x2", "KHOP", False),
])
def test_every_schedule_of_a_load_balanced_step_gives_the_oracle_bytes(oracle, app, kind_name, state, schedule,
                                                                        monkeypatch):
    """The two classes of a load-balanced step as one launch, side by side on two streams, or one
    after the other: the same bytes, on a graph whose hub gathers enough samples for work items and
    on a star, where one transit carries every sample every other step (the grid-wide case)."""
    monkeypatch.setenv("ND_STEP_SCHEDULE", schedule)
    g = graphs.random_graph(**GRAPHS["dense_hub"])
    run_and_compare(oracle, app, getattr(oracle, kind_name), g, check_state=state, modes=(True, True))
    n = 3000
    leaves = np.arange(1, n)
    star = nd.Graph.from_edges(np.concatenate([np.zeros(n - 1, int), leaves]),
                               np.concatenate([leaves, np.zeros(n - 1, int)]),
                               np.linspace(1, 4.9, 2 * (n - 1)).astype(np.float32))
    run_and_compare(oracle, app, getattr(oracle, kind_name), star, check_state=state, modes=(True, False, True))


def test_the_schedule_is_chosen_after_a_pass_that_found_work_items(oracle, monkeypatch):
    """Left to itself the engine runs the two classes one after the other until a classified pass
    has found work items, then as one launch (small steps) or on two streams (large ones); the
    counters say which, and every pass gives the oracle's bytes."""
    g = graphs.random_graph(**GRAPHS["dense_hub"])
    og = graphs.oracle_view(g)
    # the small walk with the two placing launches, which classify; left to itself a map this
    # small is placed by the kernel that emits it and every pair goes to the flat lanes
    monkeypatch.setenv("ND_SMALL_MAP", "1")
    for app, kind, small in (("UniformRandomWalk", oracle.UNIFORM_WALK, True), ("KHop40x30", oracle.KHOP, False)):
        s = nd.Sampler(app, g, seed=SEED)
        try:
            want, _ = oracle.sample_individual(og, desc_for(oracle, s, kind), SEED, s.initial_contents)
            for turn in range(3):
                print("app", app, "turn", turn, flush=True)
                s.do_transit_parallel(load_balancing=True)
                assert np.array_equal(s.final_samples(), want)
                passes, classified, merged, forked, serial = (s.counter(i) for i in range(5, 10))
                assert (passes, classified) == (turn + 1, turn + 1) and s.counter(4) > 0
                balanced_steps = s.steps - 1
                assert serial == balanced_steps  # the first pass only
                if small:
                    assert (merged, forked) == (turn * balanced_steps, 0)
                else:
                    assert merged + forked == turn * balanced_steps and forked >= turn
        finally:
            s.close()


def test_weighted_node2vec_instances_differ_where_the_biases_do(oracle):
    # p = 4, q = 0.5 against p = 0.5, q = 4 on a graph full of triangles: were the bias of a
    # candidate adjacent to the previous vertex mixed up with p or with 1, the two instances (or
    # one of them and the oracle) would agree where they must not
    g = graphs.random_graph(**GRAPHS["triangles"])
    a = run_and_compare(oracle, "WeightedNode2Vec8P4Q05", oracle.WEIGHTED_NODE2VEC, g, check_state=True)
    b = run_and_compare(oracle, "WeightedNode2Vec8P05Q4", oracle.WEIGHTED_NODE2VEC, g, check_state=True)
    c = run_and_compare(oracle, "WeightedNode2Vec8", oracle.WEIGHTED_NODE2VEC, g, check_state=True)
    assert (a != b).mean() > 0.2 and (a != c).mean() > 0.05 and (b != c).mean() > 0.05


def test_reference_sized_deepwalk_has_100_walks_per_vertex(oracle):
    # RandomWalkApp::numSamples (randomWalks.cu:23-26)
    g = graphs.random_graph(n=120, mean_degree=4, seed=3)
    s = nd.Sampler("DeepWalk", g, seed=SEED)
    assert s.num_samples == 100 * 120
    assert np.array_equal(s.initial_contents, np.arange(100 * 120) % 120)
    s.close()
    run_and_compare(oracle, "DeepWalk", oracle.DEEPWALK, g)


def test_walks_concentrated_on_one_transit(oracle):
    # star: every walk alternates hub <-> leaf, so every other step has ONE transit carrying
    # all samples (the grid-wide case) and the others have one sample per transit
    n = 3000
    leaves = np.arange(1, n)
    g = nd.Graph.from_edges(np.concatenate([np.zeros(n - 1, int), leaves]),
                            np.concatenate([leaves, np.zeros(n - 1, int)]),
                            np.linspace(1, 4.9, 2 * (n - 1)).astype(np.float32))
    for app, kind in [("UniformRandomWalk8", oracle.UNIFORM_WALK), ("WeightedNode2Vec8", oracle.WEIGHTED_NODE2VEC)]:
        run_and_compare(oracle, app, kind, g)


def test_graph_without_edges_gives_all_invalid(oracle):
    g = nd.Graph.from_csr(np.zeros(65, np.int32), np.zeros(0, np.int32))
    got = run_and_compare(oracle, "UniformRandomWalk8", oracle.UNIFORM_WALK, g)
    assert np.all(got == 64)


def test_single_vertex_self_loop(oracle):
    g = nd.Graph.from_edges([0], [0])
    got = run_and_compare(oracle, "KHop3x2", oracle.KHOP, g)
    assert np.all(got == 0)


def test_runs_are_reproducible_and_seed_matters(oracle):
    g = graphs.random_graph(n=500, mean_degree=6, seed=9)
    s = nd.Sampler("UniformRandomWalk8", g, seed=1)
    s.do_transit_parallel(True)
    a = s.final_samples()
    s.do_transit_parallel(True)
    b = s.final_samples()
    s.close()
    s2 = nd.Sampler("UniformRandomWalk8", g, seed=2)
    s2.do_transit_parallel(True)
    c = s2.final_samples()
    s2.close()
    assert np.array_equal(a, b) and not np.array_equal(a, c)


@pytest.mark.parametrize("app,gname", [("KHop", "dense_hub"), ("KHop", "sparse"), ("KHop4x3x2", "dense_hub"),
                                       ("KHop3x2", "sparse"), ("KHop40x30", "dense_hub"),
                                       ("KHop10x10", "dense_hub")])
def test_distinct_matches_oracle(oracle, app, gname):
    g = graphs.random_graph(**GRAPHS[gname])
    s = nd.Sampler(app, g, seed=SEED)
    d = desc_for(oracle, s, oracle.KHOP)
    s.do_transit_parallel(True)
    raw = s.final_samples()
    counts = s.distinct()
    got = s.final_samples()
    want, want_counts = oracle.distinct(d, raw, s.invalid_vertex)
    assert np.array_equal(got, want) and np.array_equal(counts, want_counts)
    # idempotent, and nothing but duplicates was dropped
    counts2 = s.distinct()
    assert np.array_equal(s.final_samples(), want) and np.array_equal(counts2, counts)
    for row_raw, row in zip(raw[:50], got[:50]):
        assert set(row_raw[row_raw != s.invalid_vertex]) == set(row[row != s.invalid_vertex])
    s.close()


@pytest.mark.parametrize("period", [1, 0, 3])
@pytest.mark.parametrize("app,n_roots,steps", [("MultiRW4x6", 4, 6), ("MultiRW", 100, 100)])
def test_multirw_matches_oracle(oracle, app, n_roots, steps, period):
    # the app with explicit transits (src/apps/multiRW/multiRW.cu): stepTransits picks the
    # walker of the next step; samples AND the walkers left in the sample state must agree
    g = graphs.random_graph(n=700, mean_degree=4, seed=13, hub=2, isolated_every=9)
    og = graphs.oracle_view(g)
    s = nd.Sampler(app, g, seed=SEED)
    try:
        s.set_inversion_period(period)
        assert (s.steps, s.final_sample_size, s.num_samples) == (steps, steps, g.n_vertices)
        roots = oracle.multirw_roots(s.num_samples, n_roots, g.n_vertices)
        assert np.array_equal(s.initial_contents, roots[:, 0])
        want, want_walkers, want_last, _ = oracle.sample_multirw(og, SEED, roots, steps)
        for lb in (False, True, "sample_parallel"):
            print("app", app, "period", period, "lb", lb, flush=True)
            if lb == "sample_parallel":
                s.do_sample_parallel()
            else:
                s.do_transit_parallel(load_balancing=lb)
            assert np.array_equal(s.final_samples(), want)
            state = s.sample_states().view(np.int32).reshape(s.num_samples, n_roots + 1)
            assert np.array_equal(state[:, :n_roots], want_walkers)
            assert np.array_equal(state[:, n_roots], want_last)
        with pytest.raises(nd.NextDoorError):  # explicit transits: the library has no validator
            s.check_results()
    finally:
        s.close()


def test_layer_sampling_app_is_khop_10_25(oracle):
    # src/apps/layer/layerSampling.cu: two hops with fan-outs 10 and 25
    g = graphs.random_graph(n=400, mean_degree=5, seed=21)
    got = run_and_compare(oracle, "Layer", oracle.KHOP, g)
    assert got.shape == (400, 10 + 250)


@pytest.mark.parametrize("app,kind_name,state", [
    ("UniformRandomWalk", "UNIFORM_WALK", False),
    ("PPRPerVertex", "PPR", False),
    ("WeightedNode2Vec", "WEIGHTED_NODE2VEC", True),
])
def test_two_sample_ranges_give_the_bytes_of_one(oracle, app, kind_name, state, monkeypatch):
    # large walks are sampled as two ranges of samples on two streams; forced here on a small
    # graph (odd sample count: ranges of different length)
    monkeypatch.setenv("ND_SAMPLE_RANGES", "2")
    g = graphs.random_graph(n=1501, mean_degree=6, seed=17, hub=4, isolated_every=11)
    run_and_compare(oracle, app, getattr(oracle, kind_name), g, check_state=state)
    run_and_compare(oracle, app, getattr(oracle, kind_name), g, check_state=state, inversion_period=0)


@pytest.mark.parametrize("app", ["KHop", "FastGCN", "MVS5"])
def test_a_new_graph_needs_a_new_alloc(oracle, app):
    """transferCSRToGPUs on a sampler that already ran: the buffers of the old graph are gone,
    sampling before the next allocNextDoorDataOnGPU is an error, and after it the samples are
    those of the new graph."""
    L = nd._capi.lib()
    small = graphs.random_graph(n=200, mean_degree=6, seed=21)
    large = graphs.random_graph(n=900, mean_degree=6, seed=22, hub=4)
    s = nd.Sampler(app, large, seed=SEED)
    try:
        s.do_transit_parallel(True)
        nd.check(L.nd_sampler_set_graph(s._h, small._h))
        s.graph = small
        with pytest.raises(nd.NextDoorError, match="alloc"):
            s.do_transit_parallel(True)
        nd.check(L.nd_sampler_alloc(s._h, SEED))
        s.do_transit_parallel(True)
        got = s.final_samples()
        fresh = nd.Sampler(app, small, seed=SEED)
        fresh.do_transit_parallel(True)
        want = fresh.final_samples()
        fresh.close()
        assert got.shape == want.shape and np.array_equal(got, want)
    finally:
        s.close()


@pytest.mark.parametrize("app,kind_name,state", [
    ("UniformRandomWalk", "UNIFORM_WALK", False),
    ("DeepWalk", "DEEPWALK", False),
    ("WeightedNode2Vec", "WEIGHTED_NODE2VEC", True),
])
def test_both_inversions_of_a_small_map_give_the_oracle_bytes(oracle, app, kind_name, state, monkeypatch):
    """Walks over a small map are inverted without a sort (counts per next transit, taken while
    the pairs are emitted): the emitting kernel places the pairs itself, or (ND_SMALL_MAP=1) two
    launches place them; ND_SMALL_MAP=0 sends the same map through the radix sort.  Also the
    largest map that still takes the first route, and a hub that gathers every walk."""
    g = graphs.random_graph(n=3000, mean_degree=8, seed=23, hub=7, isolated_every=13)
    run_and_compare(oracle, app, getattr(oracle, kind_name), g, check_state=state, modes=(False, True, True))
    for route in ("1", "0"):
        monkeypatch.setenv("ND_SMALL_MAP", route)
        run_and_compare(oracle, app, getattr(oracle, kind_name), g, check_state=state)
    monkeypatch.delenv("ND_SMALL_MAP")
    if app == "UniformRandomWalk":
        n = 1 << 17  # as many pairs as the small-map route takes; one more vertex takes the other route
        for vertices in (n, n + 1):
            src = np.arange(vertices)
            big = nd.Graph.from_edges(np.concatenate([src, src]), np.concatenate([(src * 7 + 1) % vertices, src % 5]),
                                      np.ones(2 * vertices, np.float32), n_vertices=vertices)
            run_and_compare(oracle, app, getattr(oracle, kind_name), big, check_state=state, modes=(True,))


@pytest.mark.parametrize("app,kind_name,state", [
    ("UniformRandomWalk", "UNIFORM_WALK", False),
    ("WeightedNode2Vec", "WEIGHTED_NODE2VEC", True),
])
def test_placed_pairs_that_find_no_place_spill(oracle, app, kind_name, state):
    """A small map whose pairs are placed by the kernel that emits them gives every vertex room for
    about twice the walks its share of the edge ends lets it expect.  Here that expectation is as
    wrong as it can be: every walk funnels through 16 vertices into ONE vertex that only 16 edges
    point to (room for a few dozen pairs), every third step, so nearly all pairs take the places
    past the counters' own."""
    n = 3000
    rest = np.arange(17, n)
    src = np.concatenate([rest, np.arange(1, 17), np.zeros(len(rest), np.int64)])
    dst = np.concatenate([1 + rest % 16, np.zeros(16, np.int64), rest])
    weights = (1.0 + (np.arange(len(src)) % 7)).astype(np.float32)
    g = nd.Graph.from_edges(src, dst, weights, n_vertices=n)
    run_and_compare(oracle, app, getattr(oracle, kind_name), g, check_state=state, modes=(True, False, True))


def test_small_map_inversion_classifies_every_run_by_the_rules(oracle, monkeypatch):
    """The placing launch of the small-map inversion (ND_SMALL_MAP=1) decides the load-balancing
    class of every run from the counts; what it reports (nd_sampler_counter) is what the rules
    give for the transits the oracle's walks are on, step by step."""
    monkeypatch.setenv("ND_SMALL_MAP", "1")
    work_from, item_outputs, cache_edges = nd.load_balancing_thresholds()
    # a hub that fits the LDS cache, one that does not, and a sparse rest
    n = 20000
    rng = np.random.default_rng(31)
    src = [rng.integers(0, n, 3 * n), np.full(4000, 7), rng.integers(0, n, 30000), np.full(9000, 11), rng.integers(0, n, 30000)]
    dst = [rng.integers(0, n, 3 * n), rng.integers(0, n, 4000), np.full(30000, 7), rng.integers(0, n, 9000), np.full(30000, 11)]
    g = nd.Graph.from_edges(np.concatenate(src), np.concatenate(dst), n_vertices=n)
    degree = np.diff(g.row_ptr)
    assert degree[7] < cache_edges < degree[11]
    s = nd.Sampler("UniformRandomWalk8", g, seed=SEED)
    try:
        s.do_transit_parallel(load_balancing=True)
        final = s.final_samples()
        want, _ = oracle.sample_individual(graphs.oracle_view(g), oracle.app_desc(oracle.UNIFORM_WALK, 8, [1] * 8), SEED,
                                           s.initial_contents)
        assert np.array_equal(final, want)
        looked = single = split = refused = items = 0
        for k in range(1, 8):
            transits = final[:, k - 1]
            transits = transits[transits != n]
            looked += len(transits)
            vertices, counts = np.unique(transits, return_counts=True)
            for v, c in zip(vertices.tolist(), counts.tolist()):
                if c < work_from or degree[v] == 0:
                    continue
                if degree[v] > cache_edges or min(degree[v], cache_edges) > 32 * c:
                    refused += c
                    continue
                n_items = -(-c // item_outputs)
                items += n_items
                if n_items > 1:
                    split += c
                else:
                    single += c
        assert single + split > 0 and refused > 0  # both hubs gather enough walks
        assert [s.counter(i) for i in range(5)] == [looked, single, split, refused, items]
    finally:
        s.close()
