"""The oracle's restatement of the reference's samplers against the reference's own functor
code: oracle/_ref/libreference_apps_host.so is the text of src/apps/khop/khop.cu,
src/apps/randomwalks/randomWalks.cu, src/apps/fastgcn/fastgcnSampling.cu,
src/apps/ladies/ladiessampling.cu, src/apps/layer/layerSampling.cu and src/apps/multiRW/multiRW.cu,
compiled from the reference tree as host C++ against the App contract header (oracle/Makefile) and run in a plain
CPU loop with the same slot layout and random streams.  Same graph, same roots, same seed ->
the same bytes.  Skipped where that library has not been built (no reference tree)."""
import ctypes as C
import os

import numpy as np
import pytest

from tests import oracle_binding as ob

REF_LIB = os.path.join(ob.ORACLE_DIR, "_ref", "libreference_apps_host.so")
pytestmark = pytest.mark.skipif(not os.path.exists(REF_LIB), reason="oracle/_ref is built from the reference tree")

KHOP, DEEPWALK, PPR, NODE2VEC, LAYER = range(5)
SEED = 42
i32p, f32p = C.POINTER(C.c_int32), C.POINTER(C.c_float)


@pytest.fixture(scope="module")
def ref():
    lib = C.CDLL(REF_LIB)
    lib.ref_app_shape.argtypes = [C.c_int, C.c_int32, i32p, i32p, C.POINTER(C.c_int64)]
    lib.ref_sample_individual.argtypes = [C.c_int, C.c_int32, C.c_int64, i32p, i32p, f32p, f32p, C.c_uint64, C.c_int64,
                                          i32p, i32p, i32p]
    lib.ref_sample_fastgcn.argtypes = [C.c_int32, C.c_int64, i32p, i32p, C.c_uint64, C.c_int64, i32p, i32p, i32p, i32p]
    lib.ref_sample_ladies.argtypes = lib.ref_sample_fastgcn.argtypes
    lib.ref_multirw_shape.argtypes = [i32p, i32p]
    lib.ref_sample_multirw.argtypes = [C.c_int32, C.c_int64, i32p, i32p, C.c_uint64, C.c_int64, i32p, i32p, i32p]
    return lib


def random_graph(n, mean_degree, seed, isolated_every=0, hub=None):
    """Directed multigraph, weights in [1, 5) that differ, adjacency sorted by (dst, weight)."""
    rng = np.random.default_rng(seed)
    m = n * mean_degree
    src, dst = rng.integers(0, n, m), rng.integers(0, n, m)
    if hub is not None:
        src = np.concatenate([src, np.full(2 * n, hub), rng.integers(0, n, 2 * n)])
        dst = np.concatenate([dst, rng.integers(0, n, 2 * n), np.full(2 * n, hub)])
    if isolated_every:
        keep = (src % isolated_every) != 1
        src, dst = src[keep], dst[keep]
    w = (rng.random(len(src)) * 4 + 1).astype(np.float32)
    adj = [[] for _ in range(n)]
    wts = [[] for _ in range(n)]
    for s, d, x in zip(src.tolist(), dst.tolist(), w.tolist()):
        adj[s].append(d)
        wts[s].append(x)
    return ob.Graph.from_adjacency(adj, wts)


def p(a, t):
    return a.ctypes.data_as(C.POINTER(t))


def reference_samples(ref, app, g, roots, state=False):
    steps, sizes, n = C.c_int32(), (C.c_int32 * 128)(), C.c_int64()
    assert ref.ref_app_shape(app, g.n_vertices, C.byref(steps), sizes, C.byref(n)) == 0
    F, per = 0, 1
    for k in range(steps.value):
        per *= sizes[k]
        F += per
    roots = np.ascontiguousarray(roots, np.int32)
    final = np.empty((len(roots), F), np.int32)
    t = np.empty(len(roots), np.int32)
    rc = ref.ref_sample_individual(app, g.n_vertices, len(g.col), p(g.row_ptr, C.c_int32), p(g.col, C.c_int32),
                                   p(g.weight, C.c_float), p(g.max_weight, C.c_float), SEED, len(roots),
                                   p(roots, C.c_int32), p(final, C.c_int32), p(t, C.c_int32) if state else None)
    assert rc == 0
    return steps.value, [sizes[k] for k in range(steps.value)], n.value, final, t


GRAPHS = {
    "sparse_with_dead_ends": dict(n=300, mean_degree=3, seed=1, isolated_every=7),
    "hub": dict(n=500, mean_degree=8, seed=2, hub=5),
    "dense_triangles": dict(n=90, mean_degree=14, seed=5),
}


@pytest.mark.parametrize("gname", list(GRAPHS))
@pytest.mark.parametrize("app,kind,state", [(KHOP, "KHOP", False), (DEEPWALK, "DEEPWALK", False), (PPR, "PPR", False),
                                            (NODE2VEC, "NODE2VEC", True), (LAYER, "KHOP", False)])
def test_oracle_gives_what_the_reference_functors_give(ref, app, kind, state, gname):
    g = random_graph(**GRAPHS[gname])
    n = g.n_vertices
    # the reference's own sizing: k-hop one sample per vertex; the walks 100 per vertex on graphs
    # under 256 K vertices, rooted at sample index mod |V| (randomWalks.cu:23-37); a tenth of those here
    steps, sizes, n_samples, _, _ = reference_samples(ref, app, g, np.zeros(0, np.int32))
    assert n_samples == (n if app in (KHOP, LAYER) else 100 * n)
    if app == LAYER:
        assert sizes == [10, 25]  # layerSampling.cu:5-8
    roots = np.arange(n if app in (KHOP, LAYER) else 10 * n, dtype=np.int32) % n
    _, _, _, want, want_t = reference_samples(ref, app, g, roots, state)
    d = ob.app_desc(getattr(ob, kind), steps, sizes)  # p = 2, q = 0.5 as the reference hard-codes them
    got, got_t = ob.sample_individual(g, d, SEED, roots)
    assert got.shape == want.shape
    assert np.array_equal(got, want)
    assert (want != n).any() and ((want == n).any() or gname != "sparse_with_dead_ends")
    if state:
        # Node2VecSample::t of walks that never took a step was never written by either side
        moved = want[:, 0] != n
        assert np.array_equal(got_t[moved], want_t[moved])


@pytest.mark.parametrize("app", ["fastgcn", "ladies"])
def test_oracle_gives_what_the_reference_fastgcn_app_gives(ref, app):
    # the layer-wise apps as the reference has them (fastgcnSampling.cu and ladiessampling.cu are
    # one text under two sets of names): 5 layers of 64 drawn uniformly from ALL vertices, the
    # adjacency towards the previous layer recorded in the sample state
    g = random_graph(n=400, mean_degree=30, seed=3, hub=9)
    n, B, layers, n_samples = g.n_vertices, 64, 5, 12
    roots = (np.arange(n_samples * B) * 7 % n).astype(np.int32)
    roots[B:2 * B] = n  # a sample whose roots are all "no vertex": nothing is sampled for it
    final = np.empty((n_samples, layers * B), np.int32)
    rows = np.empty((n_samples, layers, B * B), np.int32)
    cols = np.empty_like(rows)
    run = ref.ref_sample_fastgcn if app == "fastgcn" else ref.ref_sample_ladies
    rc = run(n, len(g.col), p(g.row_ptr, C.c_int32), p(g.col, C.c_int32), SEED, n_samples,
             p(roots, C.c_int32), p(final, C.c_int32), p(rows, C.c_int32), p(cols, C.c_int32))
    assert rc == 0
    d = ob.app_desc(ob.LAYER_LITERAL, layers, [B] * layers, initial_size=B)
    got, got_rows, got_cols = ob.sample_layer_literal(g, d, SEED, roots)
    assert np.array_equal(got, final)
    assert np.array_equal(got_rows, rows) and np.array_equal(got_cols, cols)
    assert (rows != -1).any() and np.all(final[1] == n)


def test_oracle_gives_what_the_reference_multirw_app_gives(ref):
    # src/apps/multiRW/multiRW.cu: 100 walkers per sample, 100 steps, stepTransits picks the
    # walker of the next step from the random state next() used; samples, walkers and lastRootIdx
    g = random_graph(n=200, mean_degree=4, seed=8, isolated_every=9, hub=3)
    n_roots, steps = C.c_int32(), C.c_int32()
    assert ref.ref_multirw_shape(C.byref(n_roots), C.byref(steps)) == 0
    assert (n_roots.value, steps.value) == (100, 100)
    n_samples = 40
    roots = ob.multirw_roots(n_samples, 100, g.n_vertices)
    walkers = roots.copy()
    last = np.empty(n_samples, np.int32)
    final = np.empty((n_samples, 100), np.int32)
    rc = ref.ref_sample_multirw(g.n_vertices, len(g.col), p(g.row_ptr, C.c_int32), p(g.col, C.c_int32), SEED, n_samples,
                                p(walkers, C.c_int32), p(last, C.c_int32), p(final, C.c_int32))
    assert rc == 0
    got, got_walkers, got_last, _ = ob.sample_multirw(g, SEED, roots, 100)
    assert np.array_equal(got, final)
    assert np.array_equal(got_walkers, walkers) and np.array_equal(got_last, last)
    assert (final == g.n_vertices).any() and (final != g.n_vertices).any()
