"""ctypes binding of the CPU oracle (oracle/libnd_oracle.so).  Test infrastructure only."""
import ctypes as C
import os
import subprocess

import numpy as np

ORACLE_DIR = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle")
LIB = os.path.join(ORACLE_DIR, "libnd_oracle.so")

MAX_STEPS = 128

UNIFORM_WALK, DEEPWALK, PPR, NODE2VEC, WEIGHTED_NODE2VEC, KHOP, LAYER_LITERAL, FASTGCN_IMPORTANCE, \
    LADIES_IMPORTANCE = range(9)

i32p = C.POINTER(C.c_int32)
f32p = C.POINTER(C.c_float)


class GraphStruct(C.Structure):
    _fields_ = [("n_vertices", C.c_int32), ("n_edges", C.c_int64), ("row_ptr", i32p), ("col", i32p),
                ("weight", f32p), ("max_weight", f32p)]


class AppDesc(C.Structure):
    _fields_ = [("kind", C.c_int), ("steps", C.c_int), ("step_size", C.c_int * MAX_STEPS),
                ("initial_size", C.c_int), ("p", C.c_float), ("q", C.c_float)]


class Stats(C.Structure):
    _fields_ = [("next_calls", C.c_int64), ("draws", C.c_int64), ("search_probes", C.c_int64),
                ("valid_outputs", C.c_int64), ("edge_reads", C.c_int64), ("weight_reads", C.c_int64),
                ("band_tests", C.c_int64)]

    def as_dict(self):
        return {k: getattr(self, k) for k, _ in self._fields_}


_lib = None


def build():
    subprocess.run(["make", "-C", ORACLE_DIR, "-s"], check=True)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            build()
        L = C.CDLL(LIB)
        L.ndo_philox4x32_10.argtypes = [C.POINTER(C.c_uint32), C.POINTER(C.c_uint32), C.POINTER(C.c_uint32)]
        L.ndo_uniform.restype = C.c_float
        L.ndo_uniform.argtypes = [C.c_uint64, C.c_uint64, C.c_uint32, C.c_uint32]
        L.ndo_uniform_grouped.restype = C.c_float
        L.ndo_uniform_grouped.argtypes = [C.c_uint64, C.c_uint64, C.c_uint32, C.c_uint32]
        L.ndo_rand_int.restype = C.c_int32
        L.ndo_rand_int.argtypes = [C.c_float, C.c_int32]
        for name in ("ndo_step_size_at_step", "ndo_number_of_transits", "ndo_sub_warp_size_at_step"):
            getattr(L, name).restype = C.c_int64
            getattr(L, name).argtypes = [C.POINTER(AppDesc), C.c_int]
        L.ndo_final_sample_size.restype = C.c_int64
        L.ndo_final_sample_size.argtypes = [C.POINTER(AppDesc)]
        L.ndo_max_bits.argtypes = [C.c_int32]
        L.ndo_sample_individual.argtypes = [C.POINTER(GraphStruct), C.POINTER(AppDesc), C.c_uint64, C.c_int64,
                                            C.c_int64, i32p, i32p, i32p, C.POINTER(Stats), C.c_int]
        L.ndo_sort_pairs.argtypes = [i32p, i32p, C.c_int64, i32p, i32p]
        L.ndo_unique_transits.restype = C.c_int64
        L.ndo_unique_transits.argtypes = [i32p, C.c_int64, C.c_int32, i32p, i32p, i32p, C.POINTER(C.c_int64)]
        L.ndo_kernel_class.argtypes = [C.c_int64, C.c_int64]
        L.ndo_distinct.argtypes = [C.POINTER(AppDesc), C.c_int64, C.c_int32, i32p, i32p]
        L.ndo_check_sampled_vertices.argtypes = [C.POINTER(GraphStruct), C.POINTER(AppDesc), C.c_int64, i32p, i32p,
                                                 C.c_int32, C.c_int]
        L.ndo_check_exact_transits.argtypes = [C.POINTER(GraphStruct), C.POINTER(AppDesc), C.c_int64, i32p, i32p,
                                               C.c_int32]
        L.ndo_has_edge.argtypes = [C.POINTER(GraphStruct), C.c_int32, C.c_int32]
        L.ndo_collective_neighborhood.restype = C.c_int64
        L.ndo_collective_neighborhood.argtypes = [C.POINTER(GraphStruct), i32p, C.c_int, C.c_int32, i32p, f32p, i32p]
        L.ndo_sample_layer_literal.argtypes = [C.POINTER(GraphStruct), C.POINTER(AppDesc), C.c_uint64, C.c_int64,
                                               C.c_int64, i32p, i32p, i32p, i32p, C.c_int]
        L.ndo_check_adjacency_matrix.argtypes = [C.POINTER(GraphStruct), C.POINTER(AppDesc), C.c_int64, i32p, i32p,
                                                 i32p, i32p, C.c_int32]
        u32p = C.POINTER(C.c_uint32)
        L.ndo_subgraph_num_samples.restype = C.c_int64
        L.ndo_subgraph_num_samples.argtypes = [C.POINTER(GraphStruct), C.c_int, C.c_int64]
        L.ndo_mvs_vertices.argtypes = [C.POINTER(GraphStruct), C.c_int64, C.c_int, i32p]
        L.ndo_clustergcn_vertices.argtypes = [C.POINTER(GraphStruct), C.c_int64, C.c_int, C.c_int, i32p]
        L.ndo_sample_mvs.restype = C.c_int64
        L.ndo_sample_mvs.argtypes = [C.POINTER(GraphStruct), C.c_int64, C.c_int, i32p, u32p, i32p, i32p]
        L.ndo_sample_clustergcn.restype = C.c_int64
        L.ndo_sample_clustergcn.argtypes = [C.POINTER(GraphStruct), C.c_int64, C.c_int, i32p, i32p, u32p, i32p, i32p]
        L.ndo_det_log2.restype = C.c_float
        L.ndo_det_log2.argtypes = [C.c_float]
        L.ndo_sample_ladies_importance.argtypes = [C.POINTER(GraphStruct), C.POINTER(AppDesc), C.c_uint64,
                                                   C.c_int64, C.c_int64, i32p, i32p, C.POINTER(Stats), C.c_int]
        L.ndo_sample_fastgcn_importance.argtypes = [C.POINTER(GraphStruct), C.POINTER(AppDesc), C.c_uint64,
                                                    C.c_int64, C.c_int64, i32p, i32p, C.POINTER(Stats), C.c_int]
        _lib = L
    return _lib


def _p(a, ct):
    return a.ctypes.data_as(C.POINTER(ct))


class Graph:
    """CSR arrays held as numpy, plus the struct the oracle takes."""

    def __init__(self, row_ptr, col, weight=None, max_weight=None):
        self.row_ptr = np.ascontiguousarray(row_ptr, dtype=np.int32)
        self.col = np.ascontiguousarray(col, dtype=np.int32)
        self.weight = (np.ones(len(self.col), np.float32) if weight is None
                       else np.ascontiguousarray(weight, dtype=np.float32))
        V = len(self.row_ptr) - 1
        if max_weight is None:
            mw = np.zeros(V, np.float32)
            for v in range(V):
                seg = self.weight[self.row_ptr[v]:self.row_ptr[v + 1]]
                if len(seg):
                    mw[v] = max(np.float32(0), seg.max())
            max_weight = mw
        self.max_weight = np.ascontiguousarray(max_weight, dtype=np.float32)
        self.n_vertices = V
        self.struct = GraphStruct(V, len(self.col), _p(self.row_ptr, C.c_int32), _p(self.col, C.c_int32),
                                  _p(self.weight, C.c_float), _p(self.max_weight, C.c_float))

    @classmethod
    def from_adjacency(cls, adj, weights=None):
        """adj: list of neighbour lists; sorted here by (dst, weight) like the reference loader."""
        row_ptr, col, w = [0], [], []
        for v, nb in enumerate(adj):
            ws = [1.0] * len(nb) if weights is None else list(weights[v])
            pairs = sorted(zip(nb, ws))
            col += [p[0] for p in pairs]
            w += [p[1] for p in pairs]
            row_ptr.append(len(col))
        return cls(row_ptr, col, w)


def app_desc(kind, steps, step_sizes, initial_size=1, p=2.0, q=0.5):
    d = AppDesc()
    d.kind, d.steps, d.initial_size, d.p, d.q = kind, steps, initial_size, p, q
    if isinstance(step_sizes, int):
        step_sizes = [step_sizes] * steps
    for i, s in enumerate(step_sizes):
        d.step_size[i] = s
    return d


def philox(ctr, key):
    c = (C.c_uint32 * 4)(*ctr)
    k = (C.c_uint32 * 2)(*key)
    o = (C.c_uint32 * 4)()
    lib().ndo_philox4x32_10(c, k, o)
    return list(o)


def uniform(seed, slot, step, draw):
    return lib().ndo_uniform(seed, slot, step, draw)


def uniform_grouped(seed, slot, step, draw):
    """The stream of steps with stepSize > 1 (first draw shared by four consecutive slots)."""
    return lib().ndo_uniform_grouped(seed, slot, step, draw)


def rand_int(u, n):
    return lib().ndo_rand_int(np.float32(u), n)


def final_sample_size(desc):
    return lib().ndo_final_sample_size(C.byref(desc))


def sample_individual(graph, desc, seed, initial, first_sample=0, n_threads=8, want_stats=False):
    initial = np.ascontiguousarray(initial, dtype=np.int32)
    n_samples = len(initial) // desc.initial_size
    F = final_sample_size(desc)
    final = np.empty(n_samples * F, dtype=np.int32)
    state = np.empty(n_samples, dtype=np.int32)
    stats = Stats()
    rc = lib().ndo_sample_individual(C.byref(graph.struct), C.byref(desc), seed, n_samples, first_sample,
                                     _p(initial, C.c_int32), _p(final, C.c_int32), _p(state, C.c_int32),
                                     C.byref(stats) if want_stats else None, n_threads)
    assert rc == 0, rc
    final = final.reshape(n_samples, F)
    return (final, state, stats.as_dict()) if want_stats else (final, state)


def sort_pairs(keys, vals):
    keys = np.ascontiguousarray(keys, dtype=np.int32)
    vals = np.ascontiguousarray(vals, dtype=np.int32)
    ko, vo = np.empty_like(keys), np.empty_like(vals)
    lib().ndo_sort_pairs(_p(keys, C.c_int32), _p(vals, C.c_int32), len(keys), _p(ko, C.c_int32), _p(vo, C.c_int32))
    return ko, vo


def unique_transits(sorted_keys, invalid):
    k = np.ascontiguousarray(sorted_keys, dtype=np.int32)
    n = len(k)
    u, c, o = (np.empty(max(n, 1), np.int32) for _ in range(3))
    nv = C.c_int64()
    r = lib().ndo_unique_transits(_p(k, C.c_int32), n, invalid, _p(u, C.c_int32), _p(c, C.c_int32),
                                  _p(o, C.c_int32), C.byref(nv))
    return u[:r], c[:r], o[:r], nv.value


def distinct(desc, final, invalid):
    final = np.ascontiguousarray(final, dtype=np.int32).copy()
    n_samples = final.shape[0]
    counts = np.empty(n_samples * desc.steps, np.int32)
    lib().ndo_distinct(C.byref(desc), n_samples, invalid, _p(final, C.c_int32), _p(counts, C.c_int32))
    return final, counts.reshape(n_samples, desc.steps)


def check_sampled_vertices(graph, desc, initial, final, invalid, n_threads=8):
    initial = np.ascontiguousarray(initial, dtype=np.int32)
    final = np.ascontiguousarray(final, dtype=np.int32)
    return bool(lib().ndo_check_sampled_vertices(C.byref(graph.struct), C.byref(desc), final.shape[0],
                                                 _p(initial, C.c_int32), _p(final, C.c_int32), invalid, n_threads))


def check_exact_transits(graph, desc, initial, final, invalid):
    initial = np.ascontiguousarray(initial, dtype=np.int32)
    final = np.ascontiguousarray(final, dtype=np.int32)
    return bool(lib().ndo_check_exact_transits(C.byref(graph.struct), C.byref(desc), final.shape[0],
                                               _p(initial, C.c_int32), _p(final, C.c_int32), invalid))


def collective_neighborhood(graph, transits, invalid):
    """(cols, weights, row_offsets) of one sample's collective neighbourhood."""
    t = np.ascontiguousarray(transits, dtype=np.int32)
    size = lib().ndo_collective_neighborhood(C.byref(graph.struct), _p(t, C.c_int32), len(t), invalid, None, None,
                                             None)
    cols, w, rows = np.empty(max(size, 1), np.int32), np.empty(max(size, 1), np.float32), np.empty(len(t), np.int32)
    lib().ndo_collective_neighborhood(C.byref(graph.struct), _p(t, C.c_int32), len(t), invalid, _p(cols, C.c_int32),
                                      _p(w, C.c_float), _p(rows, C.c_int32))
    return cols[:size], w[:size], rows


def sample_layer_literal(graph, desc, seed, initial, first_sample=0, n_threads=8):
    initial = np.ascontiguousarray(initial, dtype=np.int32)
    n = len(initial) // desc.initial_size
    F, B = final_sample_size(desc), desc.initial_size
    final = np.empty(n * F, np.int32)
    rows = np.full(n * desc.steps * B * B, -1, np.int32)
    cols = np.full(n * desc.steps * B * B, -1, np.int32)
    rc = lib().ndo_sample_layer_literal(C.byref(graph.struct), C.byref(desc), seed, n, first_sample,
                                        _p(initial, C.c_int32), _p(final, C.c_int32), _p(rows, C.c_int32),
                                        _p(cols, C.c_int32), n_threads)
    assert rc == 0
    return final.reshape(n, F), rows.reshape(n, desc.steps, B * B), cols.reshape(n, desc.steps, B * B)


def check_adjacency_matrix(graph, desc, initial, final, rows, cols, invalid):
    initial = np.ascontiguousarray(initial, dtype=np.int32)
    final = np.ascontiguousarray(final, dtype=np.int32)
    rows = np.ascontiguousarray(rows, dtype=np.int32)
    cols = np.ascontiguousarray(cols, dtype=np.int32)
    return bool(lib().ndo_check_adjacency_matrix(C.byref(graph.struct), C.byref(desc), final.shape[0],
                                                 _p(initial, C.c_int32), _p(final, C.c_int32), _p(rows, C.c_int32),
                                                 _p(cols, C.c_int32), invalid))


def sample_fastgcn_importance(graph, desc, seed, initial, first_sample=0, n_threads=8, want_stats=False):
    initial = np.ascontiguousarray(initial, dtype=np.int32)
    n = len(initial) // desc.initial_size
    F = final_sample_size(desc)
    final = np.empty(n * F, np.int32)
    stats = Stats()
    rc = lib().ndo_sample_fastgcn_importance(C.byref(graph.struct), C.byref(desc), seed, n, first_sample,
                                             _p(initial, C.c_int32), _p(final, C.c_int32), C.byref(stats), n_threads)
    assert rc == 0
    final = final.reshape(n, F)
    return (final, stats.as_dict()) if want_stats else final


def sample_ladies_importance(graph, desc, seed, initial, first_sample=0, n_threads=8, want_stats=False):
    initial = np.ascontiguousarray(initial, dtype=np.int32)
    n = len(initial) // desc.initial_size
    F = final_sample_size(desc)
    final = np.empty(n * F, np.int32)
    stats = Stats()
    rc = lib().ndo_sample_ladies_importance(C.byref(graph.struct), C.byref(desc), seed, n, first_sample,
                                            _p(initial, C.c_int32), _p(final, C.c_int32), C.byref(stats), n_threads)
    assert rc == 0
    final = final.reshape(n, F)
    return (final, stats.as_dict()) if want_stats else final


def multirw_roots(n_samples, n_roots, n_vertices, first_sample=0):
    """Start vertices of every sample's walkers (ndo_multirw_root)."""
    L = lib()
    L.ndo_multirw_root.restype = C.c_int32
    L.ndo_multirw_root.argtypes = [C.c_int64, C.c_int, C.c_int32]
    return np.array([[L.ndo_multirw_root(first_sample + s, i, n_vertices) for i in range(n_roots)]
                     for s in range(n_samples)], dtype=np.int32)


def sample_multirw(graph, seed, roots, steps, first_sample=0):
    """Returns (final [n, steps], walkers after the last step [n, n_roots], lastRootIdx [n],
    transit of every step [n, steps])."""
    L = lib()
    L.ndo_sample_multirw.restype = C.c_int
    L.ndo_sample_multirw.argtypes = [C.POINTER(GraphStruct), C.c_uint64, C.c_int64, C.c_int64, C.c_int, C.c_int,
                                     i32p, i32p, i32p, i32p]
    walkers = np.ascontiguousarray(roots, dtype=np.int32).copy()
    n, n_roots = walkers.shape
    final = np.empty((n, steps), np.int32)
    last = np.empty(n, np.int32)
    transits = np.empty((n, steps), np.int32)
    rc = L.ndo_sample_multirw(C.byref(graph.struct), seed, n, first_sample, n_roots, steps, _p(walkers, C.c_int32),
                              _p(last, C.c_int32), _p(final, C.c_int32), _p(transits, C.c_int32))
    assert rc == 0
    return final, walkers, last, transits


def sample_anchor_hop(graph, seed, anchors, step_sizes, first_sample=0):
    """Returns (final [n, F], transit of every transit's first output slot [n, F], -1 elsewhere)."""
    L = lib()
    L.ndo_sample_anchor_hop.restype = C.c_int
    L.ndo_sample_anchor_hop.argtypes = [C.POINTER(GraphStruct), C.c_uint64, C.c_int64, C.c_int64, C.c_int, i32p, C.c_int,
                                        C.POINTER(C.c_int), i32p, i32p]
    anchors = np.ascontiguousarray(anchors, dtype=np.int32)
    n, n_anchors = anchors.shape
    sizes = (C.c_int * len(step_sizes))(*step_sizes)
    F, per_step = 0, n_anchors
    for m in step_sizes:
        per_step *= m
        F += per_step
    final = np.empty((n, F), np.int32)
    transits = np.full((n, F), -1, np.int32)
    rc = L.ndo_sample_anchor_hop(C.byref(graph.struct), seed, n, first_sample, n_anchors, _p(anchors, C.c_int32),
                                 len(step_sizes), sizes, _p(final, C.c_int32), _p(transits, C.c_int32))
    assert rc == 0
    return final, transits


def subgraph_num_samples(graph, vertices_per_sample, cap):
    return lib().ndo_subgraph_num_samples(C.byref(graph.struct), vertices_per_sample, cap)


def mvs_vertices(graph, n_samples, batch):
    out = np.empty((n_samples, batch), dtype=np.int32)
    lib().ndo_mvs_vertices(C.byref(graph.struct), n_samples, batch, _p(out, C.c_int32))
    return out


def clustergcn_vertices(graph, n_samples, cluster_size, clusters_per_sample):
    out = np.empty((n_samples, cluster_size * clusters_per_sample), dtype=np.int32)
    lib().ndo_clustergcn_vertices(C.byref(graph.struct), n_samples, cluster_size, clusters_per_sample,
                                  _p(out, C.c_int32))
    return out


def sample_mvs(graph, vertices):
    """(rows, cols, list_start) of MVS over vertices[n_samples][batch]."""
    vertices = np.ascontiguousarray(vertices, dtype=np.int32)
    n, batch = vertices.shape
    start = np.zeros(n + 1, dtype=np.uint32)
    total = lib().ndo_sample_mvs(C.byref(graph.struct), n, batch, _p(vertices, C.c_int32), _p(start, C.c_uint32),
                                 None, None)
    rows, cols = np.empty(total, dtype=np.int32), np.empty(total, dtype=np.int32)
    lib().ndo_sample_mvs(C.byref(graph.struct), n, batch, _p(vertices, C.c_int32), _p(start, C.c_uint32),
                         _p(rows, C.c_int32), _p(cols, C.c_int32))
    return rows, cols, start


def sample_clustergcn(graph, vertices):
    """(final, rows, cols, list_start) of ClusterGCN over vertices[n_samples][n]."""
    vertices = np.ascontiguousarray(vertices, dtype=np.int32)
    n, per = vertices.shape
    start = np.zeros(n + 1, dtype=np.uint32)
    final = np.empty((n, per + per * per), dtype=np.int32)
    total = lib().ndo_sample_clustergcn(C.byref(graph.struct), n, per, _p(vertices, C.c_int32), _p(final, C.c_int32),
                                        _p(start, C.c_uint32), None, None)
    rows, cols = np.empty(total, dtype=np.int32), np.empty(total, dtype=np.int32)
    lib().ndo_sample_clustergcn(C.byref(graph.struct), n, per, _p(vertices, C.c_int32), _p(final, C.c_int32),
                                _p(start, C.c_uint32), _p(rows, C.c_int32), _p(cols, C.c_int32))
    return final, rows, cols, start
