"""Small seeded graphs shared by the parity tests."""
import numpy as np

import nextdoor_amd as nd
from tests import oracle_binding as ob


def random_graph(n, mean_degree, seed, isolated_every=0, hub=None):
    """Directed multigraph with uniform weights in [1,5); optionally isolated vertices and a hub."""
    rng = np.random.default_rng(seed)
    m = n * mean_degree
    src = rng.integers(0, n, m)
    dst = rng.integers(0, n, m)
    if hub is not None:
        extra = n * 2
        src = np.concatenate([src, np.full(extra, hub), rng.integers(0, n, extra)])
        dst = np.concatenate([dst, rng.integers(0, n, extra), np.full(extra, hub)])
    if isolated_every:
        keep = (src % isolated_every) != 1
        src, dst = src[keep], dst[keep]
    w = (rng.random(len(src)) * 4 + 1).astype(np.float32)
    return nd.Graph.from_edges(src, dst, w, n_vertices=n)


def oracle_view(g):
    """The oracle's view of a library graph (same arrays, library's max_weight)."""
    return ob.Graph(g.row_ptr, g.col, g.weight, g.max_weight)
