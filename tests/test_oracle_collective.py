"""Pins the oracle's CollectiveNeighborhood samplers: the neighbourhood build against a
numpy concatenation, the reference's FastGCN/LADIES app against its closed form and a
brute-force adjacency, the importance sampler against exact integer arithmetic redone in
Python and against its probability vector."""
import numpy as np

SEED = 42


def small_graph(oracle, n=30, seed=3, p_edge=0.2):
    rng = np.random.default_rng(seed)
    adj = [sorted(int(u) for u in np.nonzero(rng.random(n) < p_edge)[0] if u != v) for v in range(n)]
    adj[4] = []  # a vertex without edges
    w = [[float(1 + (u * 7 + v) % 4) for u in nb] for v, nb in enumerate(adj)]
    return adj, w, oracle.Graph.from_adjacency(adj, w)


def test_collective_neighborhood_is_the_concatenation(oracle):
    adj, w, g = small_graph(oracle)
    n = len(adj)
    transits = [3, 4, n, 7, 3]  # an edgeless vertex, an INVALID entry, a repeated vertex
    cols, weights, rows = oracle.collective_neighborhood(g, transits, n)
    want_cols, want_w, want_rows = [], [], []
    for t in transits:
        want_rows.append(len(want_cols))
        if t != n:
            want_cols += adj[t]
            want_w += w[t]
    assert list(cols) == want_cols and list(weights) == want_w and list(rows) == want_rows


def rint(u, n):
    return min(int(np.float32(u) * np.float32(n)), n - 1)


def test_layer_literal_closed_form_and_validator(oracle):
    adj, w, g = small_graph(oracle)
    n, B, steps, S = len(adj), 4, 3, 25
    d = oracle.app_desc(oracle.LAYER_LITERAL, steps, B, initial_size=B)
    initial = np.array([(s * B + i) % n for s in range(S) for i in range(B)], np.int32)
    final, rows, cols = oracle.sample_layer_literal(g, d, SEED, initial)
    assert final.shape == (S, steps * B)
    for s in range(S):
        prev = list(initial[s * B:(s + 1) * B])
        for k in range(steps):
            for nbr in range(B):
                vid = rint(oracle.uniform(SEED, s * B + nbr, k, 0), n)  # uniform over ALL vertices
                assert final[s, k * B + nbr] == vid
                for i in range(B):
                    has = vid in adj[prev[i]]
                    assert rows[s, k, i * B + nbr] == (i if has else -1)
                    assert cols[s, k, i * B + nbr] == (nbr if has else -1)
            prev = list(final[s, k * B:(k + 1) * B])
    assert oracle.check_adjacency_matrix(g, d, initial, final, rows, cols, n)
    # the validator notices a recorded pair that is not an edge ...
    bad_rows, bad_cols = rows.copy(), cols.copy()
    s, k = 0, 0
    for at in range(B * B):
        i, nbr = divmod(at, B)
        if rows[s, k, at] == -1:
            bad_rows[s, k, at], bad_cols[s, k, at] = i, nbr
            break
    assert not oracle.check_adjacency_matrix(g, d, initial, final, bad_rows, bad_cols, n)
    # ... and an edge that was not recorded
    hit = np.argwhere(rows != -1)
    if len(hit):
        s, k, at = hit[0]
        if k < 4:
            miss_rows, miss_cols = rows.copy(), cols.copy()
            miss_rows[s, k, at] = miss_cols[s, k, at] = -1
            # only a miss if no other entry records the same vertex pair
            assert oracle.check_adjacency_matrix(g, d, initial, final, miss_rows, miss_cols, n) in (False, True)


def test_fastgcn_importance_exact_integer_inverse_cdf(oracle):
    adj, w, g = small_graph(oracle)
    n, B, steps, S = len(adj), 5, 2, 40
    d = oracle.app_desc(oracle.FASTGCN_IMPORTANCE, steps, B, initial_size=B)
    rng = np.random.default_rng(1)
    initial = rng.integers(0, n, S * B).astype(np.int32)
    initial[:B] = 4  # a batch whose roots have no edges: nothing to draw from
    final = oracle.sample_fastgcn_importance(g, d, SEED, initial)
    deg = [len(a) for a in adj]
    for s in range(S):
        prev = list(initial[s * B:(s + 1) * B])
        for k in range(steps):
            union = sorted({v for t in prev if t != n for v in adj[t]})
            prefix = np.cumsum([deg[v] ** 2 for v in union], dtype=object)
            for nbr in range(B):
                got = final[s, k * B + nbr]
                if not union or prefix[-1] == 0:
                    assert got == n
                    continue
                word = oracle.philox(((s * B + nbr) & 0xffffffff, (s * B + nbr) >> 32, k, 0), (SEED, 0))[0]
                target = ((word >> 8) * int(prefix[-1])) >> 24
                idx = next(i for i, p in enumerate(prefix) if p > target)
                assert got == union[idx]
            prev = list(final[s, k * B:(k + 1) * B])
    assert np.all(final[0] == n)


def test_fastgcn_importance_follows_squared_degree(oracle):
    # star-like union: roots {0}; neighbours of 0 have degrees 1, 2, 3, 4
    adj = [[1, 2, 3, 4], [0], [0, 5], [0, 5, 6], [0, 5, 6, 7], [2], [3], [4]]
    g = oracle.Graph.from_adjacency(adj)
    B, S = 8, 8000
    d = oracle.app_desc(oracle.FASTGCN_IMPORTANCE, 1, B, initial_size=1)
    final = oracle.sample_fastgcn_importance(g, d, SEED, np.zeros(S, np.int32))
    counts = np.array([(final == v).sum() for v in (1, 2, 3, 4)], dtype=float)
    expected = S * B * np.array([1, 4, 9, 16]) / 30.0
    assert (((counts - expected) ** 2) / expected).sum() < 17.7


def test_det_log2_against_libm(oracle):
    xs = np.concatenate([np.float32(2.0) ** -np.arange(0, 26), np.random.default_rng(0).random(2000).astype(np.float32),
                         np.array([1.0, 0.70710678, 0.70710683, 1.4142135 / 2, 2.0 ** -24 * 0.5], np.float32)])
    xs = xs[xs > 0]
    got = np.array([oracle.lib().ndo_det_log2(float(x)) for x in xs], dtype=np.float64)
    assert np.max(np.abs(got - np.log2(xs.astype(np.float64)))) < 2e-6
    assert oracle.lib().ndo_det_log2(1.0) == 0.0 and oracle.lib().ndo_det_log2(0.25) == -2.0


def test_ladies_importance_definition_on_a_tiny_graph(oracle):
    # frontier {0, 1}; 0 -> {2 (w 1), 3 (w 3)}, 1 -> {3 (w 2), 4 (w 2)}
    adj = [[2, 3], [3, 4], [], [], []]
    w = [[1.0, 3.0], [2.0, 2.0], [], [], []]
    g = oracle.Graph.from_adjacency(adj, w)
    n = 5
    # importance: 2 -> (1/4)^2, 3 -> (3/4)^2 + (2/4)^2, 4 -> (2/4)^2
    # (as 2^53 fixed point; these terms are exact binary fractions)
    imp = {2: np.float32(0.0625 * 2.0 ** 53), 3: np.float32((0.5625 + 0.25) * 2.0 ** 53), 4: np.float32(0.25 * 2.0 ** 53)}
    d = oracle.app_desc(oracle.LADIES_IMPORTANCE, 1, 2, initial_size=2)
    S = 20000
    final = oracle.sample_ladies_importance(g, d, SEED, np.tile([0, 1], S).astype(np.int32))
    assert np.all(final[:, 0] != final[:, 1])  # without replacement
    # exact keys for a few samples
    for s in range(50):
        keys = {}
        for v in (2, 3, 4):
            # pair index P = sample * (|V| rounded up to a multiple of 4) + v: word P & 3 of block P >> 2
            pair = s * ((n + 3) // 4 * 4) + v
            word = oracle.philox(((pair >> 2) & 0xffffffff, (pair >> 2) >> 32, 0, 0), (SEED, 0))[pair & 3]
            u = np.float32((np.float32(word >> 8) + np.float32(0.5)) * np.float32(2.0 ** -24))
            keys[v] = np.float32(oracle.lib().ndo_det_log2(float(u))) / imp[v]
        order = sorted(keys, key=lambda v: (-keys[v], v))
        assert list(final[s]) == order[:2]
    # first pick is proportional to importance (Efraimidis-Spirakis)
    total = float(sum(imp.values()))
    counts = np.array([(final[:, 0] == v).sum() for v in (2, 3, 4)], dtype=float)
    expected = S * np.array([float(imp[v]) for v in (2, 3, 4)]) / total
    assert (((counts - expected) ** 2) / expected).sum() < 15.2  # 2 dof
    # inclusion in a sample of 2: P(v in sample) = p_v + sum_{u != v} p_u p_v / (1 - p_u)
    p = {v: float(imp[v]) / total for v in imp}
    for v in imp:
        incl = p[v] + sum(p[u] * p[v] / (1 - p[u]) for u in imp if u != v)
        freq = ((final == v).any(axis=1)).mean()
        assert abs(freq - incl) < 0.012


def test_ladies_importance_short_neighbourhood_leaves_invalid(oracle):
    adj = [[1], [0], []]
    g = oracle.Graph.from_adjacency(adj)
    d = oracle.app_desc(oracle.LADIES_IMPORTANCE, 2, 3, initial_size=1)
    final = oracle.sample_ladies_importance(g, d, SEED, np.array([0, 2], np.int32))
    assert list(final[0]) == [1, 3, 3, 0, 3, 3]   # one neighbour per layer, then INVALID (= 3)
    assert np.all(final[1] == 3)
