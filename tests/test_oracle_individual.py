"""Pins the oracle's IndividualNeighborhood samplers (walks, k-hop) with closed forms,
special cases that reduce to simpler samplers, hand-evaluated traces and distributions."""
import numpy as np
import pytest

SEED = 42


def path_graph(n):
    # 0 -> 1 -> ... -> n-1, last vertex has no edges
    return [[v + 1] if v + 1 < n else [] for v in range(n)]


def complete_graph(n):
    return [[u for u in range(n) if u != v] for v in range(n)]


def rint(u, n):
    return min(int(np.float32(u) * np.float32(n)), n - 1)


def test_uniform_walk_on_path_is_deterministic(oracle):
    n, steps = 12, 8
    g = oracle.Graph.from_adjacency(path_graph(n))
    d = oracle.app_desc(oracle.UNIFORM_WALK, steps, 1)
    final, _ = oracle.sample_individual(g, d, SEED, np.arange(n))
    for s in range(n):
        for k in range(steps):
            want = s + k + 1 if s + k + 1 < n else n  # INVALID = n once the walk falls off the end
            assert final[s, k] == want


def test_uniform_walk_closed_form_on_complete_graph(oracle):
    # final[s][k] = adj(prev)[min((int)(u * deg), deg - 1)], u = draw 0 of (slot = s, step = k)
    n, steps = 9, 20
    adj = complete_graph(n)
    g = oracle.Graph.from_adjacency(adj)
    d = oracle.app_desc(oracle.UNIFORM_WALK, steps, 1)
    final, _ = oracle.sample_individual(g, d, SEED, np.arange(n))
    for s in range(n):
        cur = s
        for k in range(steps):
            u = oracle.uniform(SEED, s, k, 0)
            cur = sorted(adj[cur])[rint(u, len(adj[cur]))]
            assert final[s, k] == cur


def test_first_sample_offsets_the_rng_slot(oracle):
    g = oracle.Graph.from_adjacency(complete_graph(7))
    d = oracle.app_desc(oracle.UNIFORM_WALK, 6, 1)
    roots = np.arange(7) % 7
    whole, _ = oracle.sample_individual(g, d, SEED, np.concatenate([roots, roots]))
    tail, _ = oracle.sample_individual(g, d, SEED, roots, first_sample=7)
    assert np.array_equal(whole[7:], tail)


def test_uniform_walk_is_uniform(oracle):
    n = 6
    g = oracle.Graph.from_adjacency(complete_graph(n))
    d = oracle.app_desc(oracle.UNIFORM_WALK, 1, 1)
    S = 30000
    final, _ = oracle.sample_individual(g, d, SEED, np.zeros(S, np.int32))
    counts = np.bincount(final[:, 0], minlength=n)[1:]
    expected = S / (n - 1)
    chi2 = ((counts - expected) ** 2 / expected).sum()
    assert chi2 < 20.5  # chi-square, 4 dof, p ~ 4e-4


def test_isolated_root_stays_invalid(oracle):
    g = oracle.Graph.from_adjacency([[], [0], [1]])
    for kind in (oracle.UNIFORM_WALK, oracle.DEEPWALK, oracle.PPR, oracle.NODE2VEC, oracle.WEIGHTED_NODE2VEC):
        d = oracle.app_desc(kind, 5, 1)
        final, _ = oracle.sample_individual(g, d, SEED, [0, 1, 2])
        assert np.all(final[0] == 3)
        assert final[1, 0] == 0 and np.all(final[1, 1:] == 3)
        assert list(final[2, :2]) == [1, 0] and np.all(final[2, 2:] == 3)


def test_khop_closed_form_and_layout(oracle):
    # canonical layout: [m0 step-0 draws][for each of them, m1 step-1 draws]
    n = 8
    adj = complete_graph(n)
    adj[3] = []  # a vertex without edges: its 2nd-hop slots stay INVALID
    adj = [[u for u in nb] for nb in adj]
    g = oracle.Graph.from_adjacency(adj)
    m0, m1 = 3, 2
    d = oracle.app_desc(oracle.KHOP, 2, [m0, m1])
    final, _ = oracle.sample_individual(g, d, SEED, np.arange(n))
    assert final.shape == (n, m0 + m0 * m1)
    for s in range(n):
        hop0 = []
        for nbr in range(m0):
            if not adj[s]:
                want = n
            else:
                u = oracle.uniform_grouped(SEED, s * m0 + nbr, 0, 0)  # step sizes > 1: the grouped stream
                want = sorted(adj[s])[rint(u, len(adj[s]))]
            hop0.append(want)
            assert final[s, nbr] == want
        for j, t in enumerate(hop0):
            for nbr in range(m1):
                if t == n or not adj[t]:
                    want = n
                else:
                    u = oracle.uniform_grouped(SEED, (s * m0 + j) * m1 + nbr, 1, 0)
                    want = sorted(adj[t])[rint(u, len(adj[t]))]
                assert final[s, m0 + j * m1 + nbr] == want


def test_deepwalk_with_equal_weights_reduces_to_uniform(oracle):
    # y = u * max_w <= w always, so the first candidate is accepted and draw 0 picks it
    n, steps = 10, 15
    g = oracle.Graph.from_adjacency(complete_graph(n), weights=[[2.5] * (n - 1)] * n)
    uni, _ = oracle.sample_individual(g, oracle.app_desc(oracle.UNIFORM_WALK, steps, 1), SEED, np.arange(n))
    dw, _, stats = oracle.sample_individual(g, oracle.app_desc(oracle.DEEPWALK, steps, 1), SEED, np.arange(n),
                                            want_stats=True)
    assert np.array_equal(uni, dw)
    assert stats["draws"] == 2 * n * steps  # one (index, height) pair per step


def test_deepwalk_follows_edge_weights(oracle):
    adj = [[1, 2, 3, 4], [0], [0], [0], [0]]
    w = [[1.0, 2.0, 3.0, 4.0], [1.0], [1.0], [1.0], [1.0]]
    g = oracle.Graph.from_adjacency(adj, w)
    S = 40000
    final, _ = oracle.sample_individual(g, oracle.app_desc(oracle.DEEPWALK, 1, 1), SEED, np.zeros(S, np.int32))
    counts = np.bincount(final[:, 0], minlength=5)[1:].astype(float)
    expected = S * np.array([1, 2, 3, 4]) / 10.0
    chi2 = ((counts - expected) ** 2 / expected).sum()
    assert chi2 < 17.7  # 3 dof, p ~ 5e-4


def test_deepwalk_rejection_trace(oracle):
    # evaluate the rejection loop by hand from the draw stream
    adj = [[1, 2, 3], [0], [0], [0]]
    w = [[1.0, 4.0, 2.0], [1.0], [1.0], [1.0]]
    g = oracle.Graph.from_adjacency(adj, w)
    S = 200
    final, _ = oracle.sample_individual(g, oracle.app_desc(oracle.DEEPWALK, 1, 1), SEED, np.zeros(S, np.int32))
    for s in range(S):
        draw = 0
        while True:
            x = rint(oracle.uniform(SEED, s, 0, draw), 3)
            y = np.float32(oracle.uniform(SEED, s, 0, draw + 1)) * np.float32(4.0)
            draw += 2
            if not y > np.float32(w[0][x]):
                break
        assert final[s, 0] == adj[0][x]


def test_ppr_stops_with_probability_one_percent(oracle):
    g = oracle.Graph.from_adjacency(complete_graph(5))
    S, steps = 20000, 3
    final, _ = oracle.sample_individual(g, oracle.app_desc(oracle.PPR, steps, 1), SEED, np.zeros(S, np.int32))
    stopped_first = (final[:, 0] == 5).mean()
    assert 0.006 < stopped_first < 0.014
    # exact: the walk ends at step k iff draw 0 of (s, k) < 0.01
    for s in range(300):
        alive = True
        for k in range(steps):
            if alive and oracle.uniform(SEED, s, k, 0) < np.float32(0.01):
                alive = False
            assert (final[s, k] == 5) == (not alive)


def node2vec_graph():
    #      0 - 1
    #      | X |      plus pendant 4 on 2, and 5 adjacent to 2 only
    #      2 - 3
    adj = [[1, 2, 3], [0, 2, 3], [0, 1, 3, 4, 5], [0, 1, 2], [2], [2]]
    return adj


def test_node2vec_literal_trace(oracle):
    adj = node2vec_graph()
    g = oracle.Graph.from_adjacency(adj)
    n, steps = len(adj), 6
    p, q = 2.0, 0.5
    final, state = oracle.sample_individual(g, oracle.app_desc(oracle.NODE2VEC, steps, 1, p=p, q=q), SEED,
                                            np.arange(n))
    for s in range(n):
        cur, t = s, None
        for k in range(steps):
            nb = sorted(adj[cur])
            if len(nb) == 1 or k == 0:
                nxt = nb[0]  # deterministic first edge (randomWalks.cu:144-147)
            else:
                draw = 0
                while True:
                    x = rint(oracle.uniform(SEED, s, k, draw), len(nb))
                    v = nb[x]
                    y = np.float32(oracle.uniform(SEED, s, k, draw + 1)) * np.float32(2.0)
                    draw += 2
                    if x == t:          # edge INDEX against vertex id, as the reference has it
                        h = p
                    elif v in adj[t]:
                        h = 1 / q
                    else:
                        h = 1.0
                    if y < h:
                        nxt = v
                        break
            t, cur = cur, nxt
            assert final[s, k] == cur
        assert state[s] == t


def test_node2vec_with_unit_parameters_accepts_first_candidate(oracle):
    # p = q = 1: h == 1 and y = u * 1 < 1 always, so steps >= 1 are uniform picks by draw 0
    adj = complete_graph(6)
    g = oracle.Graph.from_adjacency(adj)
    steps = 10
    final, _, stats = oracle.sample_individual(g, oracle.app_desc(oracle.NODE2VEC, steps, 1, p=1.0, q=1.0), SEED,
                                               np.arange(6), want_stats=True)
    for s in range(6):
        cur = s
        for k in range(steps):
            nb = sorted(adj[cur])
            cur = nb[0] if k == 0 else nb[rint(oracle.uniform(SEED, s, k, 0), len(nb))]
            assert final[s, k] == cur
    assert stats["draws"] == 2 * 6 * (steps - 1)


def test_weighted_node2vec_distribution(oracle):
    # walk 3 -> 2 (forced: 3's lightest... use a graph where step 0 is forced), then from 2
    # with t = 3: candidates 0,1 (adjacent to 3: h = 1/q = 2), 3 (== t: h = p = 2), 4, 5 (h = 1)
    adj = [[1, 2, 3], [0, 2, 3], [0, 1, 3, 4, 5], [2], [2], [2]]
    w = [[1, 1, 1], [1, 1, 1], [1.0, 2.0, 3.0, 4.0, 2.0], [1.0], [1.0], [1.0]]
    g = oracle.Graph.from_adjacency(adj, w)
    S = 60000
    final, state = oracle.sample_individual(g, oracle.app_desc(oracle.WEIGHTED_NODE2VEC, 2, 1), SEED,
                                            np.full(S, 3, np.int32))
    assert np.all(final[:, 0] == 2)  # single edge
    assert np.all(state == 2)
    h = np.array([1.0, 1.0, 2.0, 1.0, 1.0])  # 0,1 not adjacent to 3 here; 3 == t
    bias = h * np.array(w[2])
    counts = np.array([(final[:, 1] == v).sum() for v in (0, 1, 3, 4, 5)], dtype=float)
    expected = S * bias / bias.sum()
    chi2 = ((counts - expected) ** 2 / expected).sum()
    assert chi2 < 20.5


def weighted_node2vec_graph():
    # node2vec_graph() with weights that are exact in float32 and all different per vertex
    adj = node2vec_graph()
    w = [[1.0, 2.5, 4.0], [3.0, 1.5, 2.0], [1.0, 2.0, 3.0, 4.0, 2.5], [4.5, 1.0, 3.5], [2.0], [1.5]]
    return adj, w


@pytest.mark.parametrize("p,q", [(4.0, 0.5), (0.5, 4.0), (2.0, 0.5)])
def test_weighted_node2vec_trace(oracle, p, q):
    # Draw-by-draw evaluation of the definition: candidate i uses draw 2i for the edge index and
    # draw 2i + 1 for the height; h = p when the candidate IS the previous vertex, 1/q when it is
    # another neighbour of the previous vertex, 1 otherwise (and at step 0); accepted when
    # u * (max_weight * max(p, 1/q, 1)) < h * weight.  With p != 1/q != 1 the three branches give
    # different outcomes, so none of them can be swapped for another unnoticed.
    adj, w = weighted_node2vec_graph()
    g = oracle.Graph.from_adjacency(adj, w)
    n, steps = len(adj), 8
    f32 = np.float32
    inv_q = f32(1.0) / f32(q)
    h_max = max(f32(p), inv_q, f32(1.0))
    S = 40 * n  # 40 walks per root: enough draws to hit every branch many times
    roots = np.arange(S) % n
    final, state = oracle.sample_individual(g, oracle.app_desc(oracle.WEIGHTED_NODE2VEC, steps, 1, p=p, q=q), SEED,
                                            roots)
    seen = {"return": 0, "adjacent": 0, "far": 0, "rejected": 0}
    for s in range(S):
        cur, t = int(roots[s]), None
        for k in range(steps):
            nb = sorted(zip(adj[cur], w[cur]))
            if len(nb) == 1:
                nxt = nb[0][0]
            else:
                envelope = f32(max(x[1] for x in nb)) * h_max
                draw = 0
                while True:
                    x = rint(oracle.uniform(SEED, s, k, draw), len(nb))
                    y = f32(oracle.uniform(SEED, s, k, draw + 1)) * envelope
                    draw += 2
                    v, wx = nb[x][0], f32(nb[x][1])
                    if k == 0:
                        h, branch = f32(1.0), None
                    elif v == t:
                        h, branch = f32(p), "return"
                    elif v in adj[t]:
                        h, branch = inv_q, "adjacent"
                    else:
                        h, branch = f32(1.0), "far"
                    if y < h * wx:
                        nxt = v
                        if branch:
                            seen[branch] += 1
                        break
                    seen["rejected"] += 1
            t, cur = cur, nxt
            assert final[s, k] == cur, (s, k)
        assert state[s] == t
    assert min(seen.values()) > 50, seen


@pytest.mark.parametrize("p,q", [(4.0, 0.5), (0.5, 4.0)])
def test_weighted_node2vec_distribution_over_all_three_biases(oracle, p, q):
    # walks 0 -> 2 -> ?: the previous vertex is t = 0 and the candidates of 2 are 0 (== t: bias p),
    # 1 and 3 (neighbours of 0, not 0 itself: bias 1/q), 4 and 5 (bias 1); P(v) ~ bias * weight
    adj, w = weighted_node2vec_graph()
    g = oracle.Graph.from_adjacency(adj, w)
    S = 240000
    final, _ = oracle.sample_individual(g, oracle.app_desc(oracle.WEIGHTED_NODE2VEC, 2, 1, p=p, q=q), SEED,
                                        np.zeros(S, np.int32))
    second = final[final[:, 0] == 2, 1]  # the draws of step 1 are independent of those of step 0
    assert len(second) > S // 5
    bias = np.array([p, 1 / q, 1 / q, 1.0, 1.0]) * np.array(w[2])
    counts = np.array([(second == v).sum() for v in (0, 1, 3, 4, 5)], dtype=float)
    assert counts.sum() == len(second)
    expected = len(second) * bias / bias.sum()
    chi2 = ((counts - expected) ** 2 / expected).sum()
    assert chi2 < 20.5  # 4 dof, p ~ 4e-4
    # and the bias of the adjacent candidates is not the one of the other branches: with h = p
    # or h = 1 in their place the expected counts would be off by far more than the threshold
    for wrong in (p, 1.0):
        alt = np.array([p, wrong, wrong, 1.0, 1.0]) * np.array(w[2])
        alt = len(second) * alt / alt.sum()
        assert ((counts - alt) ** 2 / alt).sum() > 1000


def test_weighted_node2vec_step0_is_a_weighted_pick(oracle):
    adj = [[1, 2, 3, 4], [0], [0], [0], [0]]
    w = [[1.0, 2.0, 3.0, 4.0], [1.0], [1.0], [1.0], [1.0]]
    g = oracle.Graph.from_adjacency(adj, w)
    S = 40000
    final, _ = oracle.sample_individual(g, oracle.app_desc(oracle.WEIGHTED_NODE2VEC, 1, 1), SEED,
                                        np.zeros(S, np.int32))
    counts = np.bincount(final[:, 0], minlength=5)[1:].astype(float)
    expected = S * np.array([1, 2, 3, 4]) / 10.0
    assert (((counts - expected) ** 2) / expected).sum() < 17.7


def test_validators_accept_oracle_output_and_reject_corruption(oracle):
    rng = np.random.default_rng(1)
    n = 40
    adj = [sorted(set(rng.integers(0, n, rng.integers(0, 6)).tolist()) - {v}) for v in range(n)]
    g = oracle.Graph.from_adjacency(adj)
    for desc in (oracle.app_desc(oracle.UNIFORM_WALK, 6, 1), oracle.app_desc(oracle.KHOP, 2, [4, 3])):
        roots = np.arange(n)
        final, _ = oracle.sample_individual(g, desc, SEED, roots)
        assert oracle.check_sampled_vertices(g, desc, roots, final, n)
        assert oracle.check_exact_transits(g, desc, roots, final, n)
        bad = final.copy()
        # put a non-neighbour in the first slot of a sample whose root has edges
        s = next(v for v in range(n) if adj[v])
        bad[s, 0] = next(u for u in range(n) if u not in adj[s])
        assert not oracle.check_sampled_vertices(g, desc, roots, bad, n)
        assert not oracle.check_exact_transits(g, desc, roots, bad, n)
