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
