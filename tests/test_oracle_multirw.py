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


# ---- explicit transits with several transits per sample ("anchor hop", the test application of
# ---- tests/cpp/user_apps.hip; the reference's contract: src/nextdoor.cu:279-289)

def anchor_hop_by_hand(oracle, g, seed, anchors, step_sizes, sample):
    """The app's rules written out on the pinned draws: next() is the k-hop rule, stepTransits
    follows it with the same random state and the index (thread number) % (transits per sample)."""
    V = g.n_vertices
    prev, out, T = [int(a) for a in anchors], [], len(anchors)
    for k, m in enumerate(step_sizes):
        nxt = []
        for j in range(T):
            for nbr in range(m):
                transit, draw = prev[j], 0
                slot = (sample * T + j) * m + nbr
                neighbor, chosen = V, V
                if transit != V:
                    adj = adjacency(g, transit)
                    if len(adj):
                        neighbor = int(adj[oracle.rand_int(oracle.uniform_grouped(seed, slot, k, draw), len(adj))])
                        draw += 1
                    if k != len(step_sizes) - 1:
                        x = oracle.rand_int(oracle.uniform_grouped(seed, slot, k, draw), len(anchors) + 1)
                        if x != len(anchors):
                            chosen = int(anchors[((j * m + nbr) % T + x) % len(anchors)])
                out.append(neighbor)
                nxt.append(chosen)
        prev, T = nxt, T * m
    return out


def test_anchor_hop_matches_a_hand_evaluation(oracle):
    adj = [[1, 2, 3], [0, 2], [0, 1, 4, 6], [2], [2], [], [2, 0], [5]]
    g = oracle.Graph.from_adjacency(adj)
    anchors = np.array([[0, 3, 5, 6], [5, 5, 1, 7], [6, 2, 4, 0]], np.int32)
    sizes = [2, 3, 2]
    final, _ = oracle.sample_anchor_hop(g, SEED, anchors, sizes, first_sample=11)
    assert final.shape == (3, 8 + 24 + 48)
    for s in range(len(anchors)):
        assert final[s].tolist() == anchor_hop_by_hand(oracle, g, SEED, anchors[s], sizes, 11 + s)


def test_anchor_hop_outputs_hang_on_anchors_and_dead_branches_stay_dead(oracle):
    rng = np.random.default_rng(5)
    n = 80
    adj = [sorted(rng.choice(n, size=rng.integers(0, 5), replace=False).tolist()) for _ in range(n)]
    g = oracle.Graph.from_adjacency(adj)
    anchors = np.stack([(np.arange(n) * 7 + i * 13) % n for i in range(4)], axis=1).astype(np.int32)
    sizes = [2, 3, 2]
    final, transits = oracle.sample_anchor_hop(g, SEED, anchors, sizes)
    base, T = 0, 4
    ended = 0
    for k, m in enumerate(sizes):
        for s in range(n):
            for j in range(T):
                t = transits[s, base + j * m]
                outs = final[s, base + j * m: base + (j + 1) * m]
                if k == 0:
                    assert t == anchors[s, j]
                if t == n:
                    ended += 1
                    assert np.all(outs == n)          # nothing is drawn from a branch that has ended
                    continue
                assert t in anchors[s]                 # every transit is one of the sample's anchors
                for v in outs:
                    assert (v == n and len(adj[t]) == 0) or v in adj[t]
        base += T * m
        T *= m
    assert ended > 50  # a fifth of the outputs choose no transit
