"""The library's host-side result validator (the reference's check_results.cu rules) and the
command line's argument handling.  No GPU involved: samples come from the CPU oracle."""
import io

import numpy as np
import pytest

import nextdoor_amd as nd
from nextdoor_amd import __main__ as cli
from tests import graphs

SEED = 7


def walk_samples(oracle, g, steps=6):
    og = graphs.oracle_view(g)
    d = oracle.app_desc(oracle.UNIFORM_WALK, steps, [1] * steps)
    roots = np.arange(g.n_vertices, dtype=np.int32)
    final, _ = oracle.sample_individual(og, d, SEED, roots)
    return og, d, roots, final


def test_oracle_walks_pass_and_a_foreign_vertex_is_named(oracle):
    g = graphs.random_graph(n=400, mean_degree=4, seed=3, isolated_every=9)
    og, d, roots, final = walk_samples(oracle, g)
    ok, why = nd.check_sampled_vertices(g, [1] * 6, roots, final)
    assert ok, why
    # put a vertex that is not adjacent to its predecessor into sample 17, step 3
    s, k = 17, 3
    while final[s, k - 1] == g.n_vertices:
        s += 1
    prev = final[s, k - 1]
    adj = set(g.col[g.row_ptr[prev]:g.row_ptr[prev + 1]])
    stranger = next(v for v in range(g.n_vertices) if v not in adj)
    bad = final.copy()
    bad[s, k] = stranger
    ok, why = nd.check_sampled_vertices(g, [1] * 6, roots, bad)
    assert not ok
    assert why == "Invalid '%d' in Sample '%d' at Step '%d'" % (stranger, s, k)
    assert not oracle.check_sampled_vertices(og, d, roots, bad, g.n_vertices)


def test_an_empty_step_is_only_accepted_when_the_previous_vertices_have_no_edges(oracle):
    g = graphs.random_graph(n=200, mean_degree=5, seed=4)
    og, d, roots, final = walk_samples(oracle, g, steps=3)
    s = next(i for i in range(g.n_vertices) if g.row_ptr[i + 1] > g.row_ptr[i])
    bad = final.copy()
    bad[s, :] = g.n_vertices  # nothing sampled although root s has edges
    ok, why = nd.check_sampled_vertices(g, [1, 1, 1], roots, bad)
    assert not ok and "no vertex sampled for sample '%d'" % s in why
    # a graph without edges: all INVALID is the only valid result
    lonely = nd.Graph.from_edges([], [], [], n_vertices=5)
    none = np.full((5, 3), 5, dtype=np.int32)
    assert nd.check_sampled_vertices(lonely, [1, 1, 1], np.arange(5), none)[0]


def test_khop_layout_agrees_with_the_oracle_validator_on_random_corruptions(oracle):
    g = graphs.random_graph(n=300, mean_degree=6, seed=5, hub=3)
    og = graphs.oracle_view(g)
    d = oracle.app_desc(oracle.KHOP, 2, [3, 2])
    roots = np.arange(g.n_vertices, dtype=np.int32)
    final, _ = oracle.sample_individual(og, d, SEED, roots)
    assert nd.check_sampled_vertices(g, [3, 2], roots, final)[0]
    rng = np.random.default_rng(0)
    disagreements = 0
    for trial in range(40):
        bad = final.copy()
        s, at = rng.integers(0, g.n_vertices), rng.integers(0, 9)
        bad[s, at] = rng.integers(0, g.n_vertices)
        mine = nd.check_sampled_vertices(g, [3, 2], roots, bad)[0]
        theirs = bool(oracle.check_sampled_vertices(og, d, roots, bad, g.n_vertices))
        # the library's rule is the reference's; both see the same corruptions
        disagreements += mine != theirs
    assert disagreements == 0


def test_collective_layout():
    # path 0 -> 1 -> 2 -> 3, two roots per sample, layers of 2
    g = nd.Graph.from_edges([0, 1, 2], [1, 2, 3], [1, 1, 1], n_vertices=4)
    roots = np.array([[0, 1]], dtype=np.int32)
    good = np.array([[1, 2, 2, 3]], dtype=np.int32)      # layer 0 from {0,1}, layer 1 from {1,2}
    assert nd.check_sampled_vertices(g, [2, 2], roots, good, collective=True)[0]
    bad = np.array([[1, 2, 2, 0]], dtype=np.int32)       # 0 is nobody's neighbour
    ok, why = nd.check_sampled_vertices(g, [2, 2], roots, bad, collective=True)
    assert not ok and why == "Invalid '0' in Sample '0' at Step '1'"


def test_command_line_usage_and_app_list():
    out = io.StringIO()
    assert cli.run(["--list-apps"], out=out) == 0
    names = out.getvalue().split()
    assert "KHop" in names and "DeepWalk" in names and "FastGCN" in names
    # as the reference's appMain: without the graph options only the usage is printed
    out = io.StringIO()
    assert cli.run(["KHop", "-n", "1"], out=out) == 0
    assert out.getvalue().startswith("usage:")
    assert cli.run(["KHop", "-g", "/nonexistent", "-t", "edge-list", "-f", "binary"], out=io.StringIO()) == 1
    assert cli.run(["KHop", "-g", "x", "-t", "edge-list", "-f", "binary", "-k", "Other"], out=io.StringIO()) == 2
