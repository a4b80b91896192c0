"""CPU oracle of the multi-dimensional random walk (src/apps/multiRW/multiRW.cu): a hand
evaluation of the app's rules from the pinned uniform draws, and the invariants that tie
every output to the walker that was moved."""
import numpy as np

SEED = 42


def adjacency(g, v):
    return g.col[g.row_ptr[v]:g.row_ptr[v + 1]]


def by_hand(oracle, g, seed, walkers, steps, sample):
    """The rules of multiRW.cu:27-49 and :84-92 and of the step kernel (nextdoor.cu:279-289),
    written out in Python on top of the pinned draws."""
    walkers = list(walkers)
    out, last, transit = [], 0, walkers[0]
    V = g.n_vertices
    for k in range(steps):
        draw = 0
        adj = adjacency(g, transit)
        if len(adj) == 0:
            out.append(V)
        else:
            if len(adj) == 1:
                v = int(adj[0])
            else:
                v = int(adj[oracle.rand_int(oracle.uniform(seed, sample, k, draw), len(adj))])
                draw += 1
            if k > 0:
                walkers[last] = v
            out.append(v)
        if k != steps - 1:
            last = oracle.rand_int(oracle.uniform(seed, sample, k, draw), len(walkers))
            transit = walkers[last]
    return out, walkers, last


def test_multirw_matches_a_hand_evaluation(oracle):
    # mixed degrees: 0 (vertex 5), 1 (vertices 3, 4) and more
    adj = [[1, 2, 3], [0, 2], [0, 1, 4, 6], [2], [2], [], [2, 0]]
    g = oracle.Graph.from_adjacency(adj)
    roots = np.array([[0, 3, 5], [5, 5, 1], [6, 2, 4], [4, 4, 4]], np.int32)
    steps = 9
    final, walkers, last, _ = oracle.sample_multirw(g, SEED, roots, steps, first_sample=7)
    for s in range(len(roots)):
        want_out, want_walkers, want_last = by_hand(oracle, g, SEED, roots[s], steps, 7 + s)
        assert final[s].tolist() == want_out
        assert walkers[s].tolist() == want_walkers
        assert last[s] == want_last


def test_every_output_is_a_neighbour_of_the_walker_that_moved(oracle):
    rng = np.random.default_rng(3)
    n = 60
    adj = [sorted(rng.choice(n, size=rng.integers(0, 6), replace=False).tolist()) for _ in range(n)]
    g = oracle.Graph.from_adjacency(adj)
    roots = oracle.multirw_roots(n, 4, n)
    assert roots.min() >= 0 and roots.max() < n
    final, walkers, last, transits = oracle.sample_multirw(g, SEED, roots, 12)
    assert np.array_equal(transits[:, 0], roots[:, 0])           # multiRW.cu:68-73
    for s in range(n):
        for k in range(12):
            t, v = transits[s, k], final[s, k]
            if len(adj[t]) == 0:
                assert v == n                                     # INVALID, the walker stays
            else:
                assert v in adj[t]
    # the walkers only ever hold start vertices or sampled vertices
    for s in range(n):
        allowed = set(roots[s].tolist()) | set(final[s].tolist())
        assert set(walkers[s].tolist()) <= allowed
    assert last.min() >= 0 and last.max() < 4


def test_walker_starts_are_a_fixed_uniform_stream(oracle):
    a = oracle.multirw_roots(2000, 3, 50)
    b = oracle.multirw_roots(2000, 3, 50)
    assert np.array_equal(a, b)
    counts = np.bincount(a.reshape(-1), minlength=50)
    expected = a.size / 50
    assert (((counts - expected) ** 2) / expected).sum() < 85.4   # chi-square, 49 dof, p = 0.001
    # defined as the pinned uniform draw of stream ("MRWR", sample, "ROOT", walker)
    assert a[5, 2] == oracle.rand_int(oracle.uniform(0x4D525752, 5, 0x524F4F54, 2), 50)
