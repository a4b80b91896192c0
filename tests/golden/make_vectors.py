"""Writes tests/golden/sampler_vectors.json: a small fixed graph and, for the apps compiled
into the library, the samples this repository's CPU oracle (oracle/nd_oracle.c) produces
on it with seed 42.  Nothing here comes from the reference tree; the reference holds no
golden vectors for this path, and its random numbers are not reproducible.  The fixture
lets the GPU tests check the library without running the oracle, and lets the CPU tests
notice an unintended change of the oracle.

    python tests/golden/make_vectors.py        # from the repository root

philox4x32_10_kat.json (the published Random123 known-answer vectors) is written by hand,
not by this script."""
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from tests import oracle_binding as ob  # noqa: E402

SEED = 42
HERE = os.path.dirname(os.path.abspath(__file__))


def make_graph():
    """24 vertices: a sparse random part, a hub (vertex 3), parallel edges, two vertices
    without out-edges (10, 17); weights are multiples of 0.5 in [1, 5) (exact in float32)."""
    rng = np.random.default_rng(2024)
    n = 24
    adj = [[] for _ in range(n)]
    wts = [[] for _ in range(n)]
    for v in range(n):
        if v in (10, 17):
            continue
        deg = int(rng.integers(1, 7)) if v != 3 else 18
        for _ in range(deg):
            adj[v].append(int(rng.integers(0, n)))
            wts[v].append(float(rng.integers(2, 10)) * 0.5)
    adj[5] += [3, 3, 3]          # parallel edges
    wts[5] += [1.5, 1.5, 4.0]
    row_ptr, col, w = [0], [], []
    for v in range(n):
        pairs = sorted(zip(adj[v], wts[v]))  # by (dst, weight), duplicates kept: src/graph.hpp:38,156
        col += [p[0] for p in pairs]
        w += [p[1] for p in pairs]
        row_ptr.append(len(col))
    return row_ptr, col, w


def desc(kind, steps, sizes, initial_size=1, p=2.0, q=0.5):
    return ob.app_desc(kind, steps, sizes, initial_size=initial_size, p=p, q=q)


def main():
    row_ptr, col, w = make_graph()
    g = ob.Graph(row_ptr, col, w)
    V = len(row_ptr) - 1
    ids = np.arange(V, dtype=np.int32)
    out = {"seed": SEED, "graph": {"row_ptr": row_ptr, "col": col, "weight": w}, "apps": {}}

    def individual(app, kind, steps, sizes, with_state=False, p=2.0, q=0.5):
        d = desc(kind, steps, sizes, p=p, q=q)
        final, state = ob.sample_individual(g, d, SEED, ids)
        entry = {"initial": ids.tolist(), "final": final.reshape(-1).tolist(), "shape": list(final.shape)}
        if with_state:
            entry["state_t"] = state.tolist()
        out["apps"][app] = entry

    individual("UniformRandomWalk8", ob.UNIFORM_WALK, 8, 1)
    individual("WeightedNode2Vec8", ob.WEIGHTED_NODE2VEC, 8, 1, with_state=True)
    individual("WeightedNode2Vec8P4Q05", ob.WEIGHTED_NODE2VEC, 8, 1, with_state=True, p=4.0, q=0.5)
    individual("WeightedNode2Vec8P05Q4", ob.WEIGHTED_NODE2VEC, 8, 1, with_state=True, p=0.5, q=4.0)
    individual("DeepWalkPerVertex", ob.DEEPWALK, 100, 1)
    individual("PPRPerVertex", ob.PPR, 100, 1)
    individual("Node2VecPerVertex", ob.NODE2VEC, 100, 1, with_state=True)
    individual("KHop3x2", ob.KHOP, 2, [3, 2])
    individual("KHop4x3x2", ob.KHOP, 3, [4, 3, 2])

    roots = ob.multirw_roots(V, 4, V)
    final, walkers, last, _ = ob.sample_multirw(g, SEED, roots, 6)
    out["apps"]["MultiRW4x6"] = {"initial": roots[:, 0].tolist(), "final": final.reshape(-1).tolist(),
                                 "shape": list(final.shape), "walkers": walkers.reshape(-1).tolist(),
                                 "last_root_idx": last.tolist()}

    # layer-wise apps: 2 layers of 8
    B = 8
    lit_roots = (np.arange(50 * B) % V).astype(np.int32)      # fastgcnSampling.cu:75-85
    d = desc(ob.LAYER_LITERAL, 2, [B, B], initial_size=B)
    final, rows, cols = ob.sample_layer_literal(g, d, SEED, lit_roots)
    out["apps"]["LayerLiteral2x8"] = {"initial": lit_roots.tolist(), "final": final.reshape(-1).tolist(),
                                      "shape": list(final.shape), "rows": rows.reshape(-1).tolist(),
                                      "cols": cols.reshape(-1).tolist()}
    imp_roots = np.array([ob.rand_int(ob.uniform(0x46475243, s * B + i, 0x524F4F54, 0), V)
                          for s in range(100) for i in range(B)], np.int32)
    for app, kind, fn in (("FastGCNImportance2x8", ob.FASTGCN_IMPORTANCE, ob.sample_fastgcn_importance),
                          ("LADIESImportance2x8", ob.LADIES_IMPORTANCE, ob.sample_ladies_importance)):
        d = desc(kind, 2, [B, B], initial_size=B)
        final = fn(g, d, SEED, imp_roots)
        out["apps"][app] = {"initial": imp_roots.tolist(), "final": final.reshape(-1).tolist(),
                            "shape": list(final.shape)}

    # edge-list apps: batches of 5 consecutive vertices; two clusters of 3
    n = ob.subgraph_num_samples(g, 5, 1500000)
    verts = ob.mvs_vertices(g, n, 5)
    rows, cols, start = ob.sample_mvs(g, verts)
    out["apps"]["MVS5"] = {"initial": verts.reshape(-1).tolist(), "rows": rows.tolist(), "cols": cols.tolist(),
                           "list_start": start.tolist()}
    n = ob.subgraph_num_samples(g, 6, 2000000)
    verts = ob.clustergcn_vertices(g, n, 3, 2)
    final, rows, cols, start = ob.sample_clustergcn(g, verts)
    out["apps"]["ClusterGCN3x2"] = {"initial": verts.reshape(-1).tolist(), "final": final.reshape(-1).tolist(),
                                    "shape": list(final.shape), "rows": rows.tolist(), "cols": cols.tolist(),
                                    "list_start": start.tolist()}

    with open(os.path.join(HERE, "sampler_vectors.json"), "w") as f:
        json.dump(out, f, separators=(",", ":"))
    print("wrote", os.path.join(HERE, "sampler_vectors.json"), os.path.getsize(os.path.join(HERE, "sampler_vectors.json")),
          "bytes")


if __name__ == "__main__":
    main()
