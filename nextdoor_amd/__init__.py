"""Host-side mirror of the NextDoor sampling interface over libnextdoor_amd.so.

The compute path is the HIP library (csrc/, C ABI in include/nextdoor_amd.h).  This
package only loads it and mirrors, for Python callers, the two surfaces of the reference:

* the libNextDoor host API (src/libNextDoor.hpp:39-50): ``loadGraph`` ->
  :meth:`Graph.load`, ``transferCSRToGPUs`` + ``allocNextDoorDataOnGPU`` ->
  :meth:`Sampler.__init__`, ``doTransitParallelSampling`` ->
  :meth:`Sampler.do_transit_parallel`, ``getFinalSamples`` -> :meth:`Sampler.final_samples`,
  ``freeDeviceData`` -> :meth:`Sampler.free_device`;
* the per-app Python module functions (src/nextDoorPythonModule.cu:40-102):
  ``initSampling / sample / finalSamples / finalSampleLength / freeDeviceMemory /
  finalSamplesArray`` -> :class:`SamplingModule`.

There is no CPU fallback: without the built library and a GPU every sampling call raises.
"""
import ctypes as C

import numpy as np

from . import _capi
from ._capi import NextDoorError, check, lib

__all__ = ["Graph", "Sampler", "SamplingModule", "NextDoorError", "app_names", "load_app_library",
           "philox_fill_uniform", "sort_pairs", "sort_pairs_noalloc", "unique_transits", "classify_runs", "load_balancing_thresholds", "measure_gather_rate", "collective_neighborhood", "check_sampled_vertices"]


def app_names():
    L = lib()
    return [L.nd_app_name(i).decode() for i in range(L.nd_num_apps())]


_app_libraries = {}


def load_app_library(path):
    """Loads a shared object of applications that were compiled apart from the library (an App
    struct on the contract plus ``ND_REGISTER_APP(name, SampleType, App)``, built by hipcc and
    linked against libnextdoor_amd.so).  Its apps register themselves while it loads; returns
    the names that appeared.  The counterpart of compiling one's own app binary against the
    reference (src/apps/*/main.cu)."""
    import os
    L = lib()  # the library first: the registrations call into it
    before = set(app_names())
    real = os.path.realpath(path)
    if real not in _app_libraries:
        _app_libraries[real] = C.CDLL(real, mode=C.RTLD_GLOBAL)
    del L
    return sorted(set(app_names()) - before)


def check_sampled_vertices(graph, step_sizes, initial, final_samples, invalid=None, collective=False):
    """The reference's checkSampledVerticesResult rule (src/check_results.cu:162-299) on host
    arrays: ``initial`` is (num_samples, initial_size), ``final_samples`` (num_samples, F).
    Returns (True, "") or (False, first violation)."""
    initial = _as(initial, np.int32)
    final_samples = _as(final_samples, np.int32)
    n_samples = final_samples.shape[0]
    initial = initial.reshape(n_samples, -1) if n_samples else initial.reshape(0, 1)
    sizes = _as(step_sizes, np.int32)
    rc = lib().nd_check_sampled_vertices(graph._h, len(sizes), _ptr(sizes, C.c_int32), max(initial.shape[1], 1),
                                         int(collective), n_samples, _ptr(initial, C.c_int32),
                                         _ptr(final_samples, C.c_int32),
                                         graph.n_vertices if invalid is None else invalid)
    if rc < 0:
        raise NextDoorError(lib().nd_last_error().decode())
    return (True, "") if rc == 1 else (False, lib().nd_last_error().decode())


def _as(arr, dtype):
    return np.ascontiguousarray(arr, dtype=dtype)


def _ptr(arr, ctype):
    return arr.ctypes.data_as(C.POINTER(ctype))


class Graph:
    """Host CSR graph (the reference's ``CSR*``)."""

    def __init__(self, handle):
        self._h = handle

    @classmethod
    def load(cls, path, graph_type="edge-list", graph_format="binary"):
        h = C.c_void_p()
        check(lib().nd_graph_load(str(path).encode(), graph_type.encode(), graph_format.encode(), C.byref(h)))
        return cls(h)

    @classmethod
    def from_edges(cls, src, dst, weight=None, n_vertices=0):
        src, dst = _as(src, np.int32), _as(dst, np.int32)
        w = None if weight is None else _as(weight, np.float32)
        h = C.c_void_p()
        check(lib().nd_graph_from_edges(n_vertices, len(src), _ptr(src, C.c_int32), _ptr(dst, C.c_int32),
                                        None if w is None else _ptr(w, C.c_float), C.byref(h)))
        return cls(h)

    @classmethod
    def from_csr(cls, row_ptr, col, weight=None):
        row_ptr, col = _as(row_ptr, np.int32), _as(col, np.int32)
        w = None if weight is None else _as(weight, np.float32)
        h = C.c_void_p()
        check(lib().nd_graph_from_csr(len(row_ptr) - 1, len(col), _ptr(row_ptr, C.c_int32), _ptr(col, C.c_int32),
                                      None if w is None else _ptr(w, C.c_float), C.byref(h)))
        return cls(h)

    @classmethod
    def rmat(cls, scale, edge_factor, a=0.57, b=0.19, c=0.19, seed=42, symmetrise=False):
        h = C.c_void_p()
        check(lib().nd_graph_rmat(scale, edge_factor, a, b, c, seed, int(symmetrise), C.byref(h)))
        return cls(h)

    @classmethod
    def chung_lu(cls, n_vertices, n_edges, exponent, seed=42):
        h = C.c_void_p()
        check(lib().nd_graph_chung_lu(n_vertices, n_edges, exponent, seed, C.byref(h)))
        return cls(h)

    @property
    def n_vertices(self):
        return lib().nd_graph_num_vertices(self._h)

    @property
    def n_edges(self):
        return lib().nd_graph_num_edges(self._h)

    def _view(self, fn, n, dtype):
        if n == 0:
            return np.zeros(0, dtype=dtype)
        return np.ctypeslib.as_array(fn(self._h), shape=(n,))

    # zero-copy views into the library-owned arrays (valid while the Graph lives)
    @property
    def row_ptr(self):
        return self._view(lib().nd_graph_row_ptr, self.n_vertices + 1, np.int32)

    @property
    def col(self):
        return self._view(lib().nd_graph_col, self.n_edges, np.int32)

    @property
    def weight(self):
        return self._view(lib().nd_graph_weight, self.n_edges, np.float32)

    @property
    def max_weight(self):
        return self._view(lib().nd_graph_max_weight, self.n_vertices, np.float32)

    def close(self):
        if self._h:
            lib().nd_graph_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Sampler:
    """``NextDoorData<SampleType, App>`` plus the engine, for one app and one graph."""

    def __init__(self, app, graph, seed=42):
        self._h = C.c_void_p()
        self.graph = graph  # keeps the host CSR alive
        check(lib().nd_sampler_create(app.encode(), C.byref(self._h)))
        try:
            check(lib().nd_sampler_set_graph(self._h, graph._h))
            check(lib().nd_sampler_alloc(self._h, seed))
        except Exception:
            self.close()
            raise

    # shape algebra of the app
    @property
    def num_samples(self):
        return lib().nd_sampler_num_samples(self._h)

    @property
    def final_sample_size(self):
        return lib().nd_sampler_final_sample_size(self._h)

    @property
    def steps(self):
        return lib().nd_sampler_steps(self._h)

    def step_size(self, k):
        return lib().nd_sampler_step_size(self._h, k)

    @property
    def initial_sample_size(self):
        return lib().nd_sampler_initial_sample_size(self._h)

    @property
    def invalid_vertex(self):
        return lib().nd_sampler_invalid_vertex(self._h)

    @property
    def max_bits(self):
        return lib().nd_sampler_max_bits(self._h)

    @property
    def initial_contents(self):
        p, n = C.POINTER(C.c_int32)(), C.c_int64()
        check(lib().nd_sampler_initial_contents(self._h, C.byref(p), C.byref(n)))
        return np.ctypeslib.as_array(p, shape=(n.value,)).copy()

    def do_transit_parallel(self, load_balancing=True):
        check(lib().nd_sampler_do_transit_parallel(self._h, int(load_balancing)))

    def do_sample_parallel(self):
        """The reference's baseline mode: no transit order, no load balancing; same samples."""
        check(lib().nd_sampler_do_sample_parallel(self._h))

    def check_results(self):
        """The reference's result validators (src/check_results.cu) on the host.  Returns
        (True, "") or (False, first violation)."""
        ok = C.c_int()
        check(lib().nd_sampler_check_results(self._h, C.byref(ok)))
        return (True, "") if ok.value else (False, lib().nd_last_error().decode())

    def final_samples(self):
        """(num_samples, final_sample_size) int32 array; INVALID entries equal n_vertices."""
        p, n = C.POINTER(C.c_int32)(), C.c_int64()
        check(lib().nd_sampler_get_final_samples(self._h, C.byref(p), C.byref(n)))
        flat = np.ctypeslib.as_array(p, shape=(n.value,)).copy()
        return flat.reshape(self.num_samples, self.final_sample_size)

    def adjacency(self):
        """Edge lists of the apps with AdjacencyMatrix output on per-transit sampling (MVS,
        ClusterGCN): (rows, cols, list_start); sample i owns rows/cols[list_start[i]:list_start[i+1]]."""
        rows, cols = C.POINTER(C.c_int32)(), C.POINTER(C.c_int32)()
        start = C.POINTER(C.c_uint32)()
        n_edges, n_samples = C.c_int64(), C.c_int64()
        check(lib().nd_sampler_get_adjacency(self._h, C.byref(rows), C.byref(cols), C.byref(n_edges), C.byref(start),
                                             C.byref(n_samples)))
        take = lambda p, n, dt: (np.ctypeslib.as_array(p, shape=(n,)).copy() if n else np.zeros(0, dtype=dt))
        return (take(rows, n_edges.value, np.int32), take(cols, n_edges.value, np.int32),
                take(start, n_samples.value + 1, np.uint32))

    def distinct(self):
        """Distinct post-pass on the device rows; returns counts[num_samples, steps]."""
        check(lib().nd_sampler_distinct(self._h))
        p, n = C.POINTER(C.c_int32)(), C.c_int64()
        check(lib().nd_sampler_get_distinct_counts(self._h, C.byref(p), C.byref(n)))
        return np.ctypeslib.as_array(p, shape=(n.value,)).copy().reshape(self.num_samples, self.steps)

    def sample_states(self):
        nbytes = lib().nd_sampler_sample_state_bytes(self._h)
        if nbytes <= 0:
            return None
        buf = np.empty(nbytes, dtype=np.uint8)
        check(lib().nd_sampler_get_sample_states(self._h, buf.ctypes.data_as(C.c_void_p), nbytes))
        return buf

    def set_inversion_period(self, period):
        """Walks: 1 inverts before every step (the reference's behaviour, default); p > 1 keeps
        the walks out of transit order and only drops ended walks every p-th step; 0 lets the
        engine decide.  The samples do not depend on it."""
        check(lib().nd_sampler_set_inversion_period(self._h, int(period)))

    def set_launch_graph(self, mode):
        """1: replay every pass as a recorded HIP graph; 0 (default): enqueue the launches one
        by one.  The samples are the same."""
        check(lib().nd_sampler_set_launch_graph(self._h, int(mode)))

    def set_profiling(self, on):
        check(lib().nd_sampler_set_profiling(self._h, int(on)))

    def phase_times(self):
        out = (C.c_float * 12)()
        check(lib().nd_sampler_phase_times(self._h, out))
        keys = ["end_to_end_ms", "inversion_ms", "load_balancing_ms", "flat_kernel_ms", "workgroup_kernel_ms",
                "flat_launches", "workgroup_launches", "sort_passes", "assemble_ms", "distinct_ms",
                "neighbourhood_ms", "neighbourhood_launches"]
        return dict(zip(keys, list(out)))

    def counter(self, which):
        return lib().nd_sampler_counter(self._h, which)

    def free_device(self):
        lib().nd_sampler_free_device(self._h)

    def close(self):
        if self._h:
            lib().nd_sampler_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class SamplingModule:
    """The functions of one per-app Python module of the reference
    (src/nextDoorPythonModule.cu:40-102), e.g. ``SamplingModule("KHop")`` for
    ``KHopSamplingPy3``.  State is process-wide, as in the reference."""

    def __init__(self, app, seed=42):
        self.app, self.seed = app, seed

    def initSampling(self, graph_path):
        check(lib().nd_init_sampling(self.app.encode(), str(graph_path).encode(), self.seed))

    def initSamplingFromCSR(self, row_ptr, col, weight=None):
        """The same from CSR arrays in memory (no counterpart in the reference's module)."""
        row_ptr, col = _as(row_ptr, np.int32), _as(col, np.int32)
        weight = None if weight is None else _as(weight, np.float32)
        check(lib().nd_init_sampling_from_csr(self.app.encode(), len(row_ptr) - 1, len(col), _ptr(row_ptr, C.c_int32),
                                              _ptr(col, C.c_int32),
                                              None if weight is None else _ptr(weight, C.c_float), self.seed))

    def sample(self):
        check(lib().nd_sample())

    def finalSampleLength(self):
        return lib().nd_final_sample_length()

    def finalSamplesArray(self):
        """numpy view of the library's host vector (no copy), like wrapping the reference's
        ``int* finalSamplesArray()``."""
        p = lib().nd_final_samples_array()
        if not p:
            raise NextDoorError(lib().nd_last_error().decode())
        return np.ctypeslib.as_array(p, shape=(lib().nd_final_sample_length(),))

    def finalSamples(self):
        return self.finalSamplesArray().tolist()

    def freeDeviceMemory(self):
        lib().nd_free_device_memory()


# ---- building blocks (device kernels behind host buffers) ---------------------------------

def philox_fill_uniform(seed, step, first_slot, n_slots, draws_per_slot=1, step_size=1):
    """The random numbers of a step as a buffer: draws_per_slot uniforms for each of n_slots output
    slots from first_slot on.  step_size > 1: the grouped form of the stream such steps use."""
    out = np.empty(n_slots * draws_per_slot, dtype=np.float32)
    check(lib().nd_philox_fill_step(seed, step, step_size, first_slot, n_slots, draws_per_slot, _ptr(out, C.c_float)))
    return out.reshape(n_slots, draws_per_slot)


def sort_pairs(keys, vals, key_bits):
    keys = _as(keys, np.int32)
    v = None if vals is None else _as(vals, np.int32)
    ko, vo = np.empty_like(keys), np.empty_like(keys)
    check(lib().nd_sort_pairs(_ptr(keys, C.c_int32), None if v is None else _ptr(v, C.c_int32), len(keys), key_bits,
                              _ptr(ko, C.c_int32), _ptr(vo, C.c_int32)))
    return ko, vo


def load_balancing_thresholds():
    """(outputs a transit needs for the workgroup kernel, outputs per work item, edges the LDS cache holds)"""
    out = np.zeros(3, np.int32)
    check(lib().nd_load_balancing_thresholds(_ptr(out, C.c_int32)))
    return tuple(int(x) for x in out)


def classify_runs(sorted_keys, degrees, step_size, pairs_per_lane=1, capacity=None):
    """The load-balancing classification over a sorted key array: (items [k, 2] = first pair and
    pairs of every work item, items wanted, taken [n_vertices], counters [5])."""
    keys, degrees = _as(sorted_keys, np.int32), _as(degrees, np.int32)
    capacity = capacity or max(len(keys), 1)
    items = np.zeros((capacity, 2), np.int32)
    taken = np.zeros(len(degrees), np.uint8)
    counters, wanted = np.zeros(5, np.int64), C.c_int64()
    check(lib().nd_classify_runs(_ptr(keys, C.c_int32), len(keys), _ptr(degrees, C.c_int32), len(degrees), step_size,
                                 pairs_per_lane, _ptr(items, C.c_int32), capacity,
                                 C.byref(wanted), _ptr(taken, C.c_uint8), _ptr(counters, C.c_int64)))
    return items[:min(wanted.value, capacity)], wanted.value, taken, counters


SORT_PAIRS_NOALLOC_MAX = 1 << 20  # ND_SORT_PAIRS_NOALLOC_MAX of include/nextdoor_amd.h


def sort_pairs_noalloc(d_keys, d_vals, n, key_bits, d_keys_out, d_vals_out, stream=0):
    """nd_sort_pairs_noalloc: the sort on DEVICE arrays given as addresses (integers; d_vals 0 =
    value is the index), enqueued on `stream` (a hipStream_t as an integer, 0 = default stream)
    with all working memory inside the library; allocates nothing and does not wait."""
    check(lib().nd_sort_pairs_noalloc(d_keys, d_vals or None, n, key_bits, d_keys_out, d_vals_out, stream or None))


def measure_gather_rate(table_bytes, reads_in_flight=2, workgroup_lanes=256):
    """Independent random 8-byte reads per second over a table of ``table_bytes`` (power of two),
    ``reads_in_flight`` (1, 2, 4, 8) issued per lane before any is used, workgroups of 64 or 256 lanes."""
    rate = C.c_double()
    check(lib().nd_measure_gather_rate_shaped(int(table_bytes), reads_in_flight, workgroup_lanes, C.byref(rate)))
    return rate.value


def gather_rate_ceiling(table_bytes):
    """The largest rate over the probe's shapes, and the rate of every shape: (best, {(k, lanes): rate})."""
    rates = {(k, lanes): measure_gather_rate(table_bytes, k, lanes) for k in (1, 2, 4, 8) for lanes in (64, 256)}
    return max(rates.values()), rates


def unique_transits(sorted_keys, invalid):
    k = _as(sorted_keys, np.int32)
    n = len(k)
    uniq, counts, offsets = (np.empty(max(n, 1), dtype=np.int32) for _ in range(3))
    n_runs, n_valid = C.c_int64(), C.c_int64()
    check(lib().nd_unique_transits(_ptr(k, C.c_int32), n, invalid, _ptr(uniq, C.c_int32), _ptr(counts, C.c_int32),
                                   _ptr(offsets, C.c_int32), C.byref(n_runs), C.byref(n_valid)))
    r = n_runs.value
    return uniq[:r], counts[:r], offsets[:r], n_valid.value


def collective_neighborhood(graph, transits, transits_per_sample, invalid, capacity):
    """sizes, offsets, cols, weights, row_offsets of the collective neighbourhoods of the
    samples whose transits are the rows of `transits`."""
    t = _as(transits, np.int32).reshape(-1, transits_per_sample)
    n = t.shape[0]
    sizes, offsets = np.empty(n, np.int32), np.empty(n + 1, np.int32)
    cols, weights = np.empty(capacity, np.int32), np.empty(capacity, np.float32)
    rows = np.empty(n * transits_per_sample, np.int32)
    check(lib().nd_collective_neighborhood(graph._h, _ptr(t, C.c_int32), n, transits_per_sample, invalid,
                                           _ptr(sizes, C.c_int32), _ptr(offsets, C.c_int32), _ptr(cols, C.c_int32),
                                           _ptr(weights, C.c_float), capacity, _ptr(rows, C.c_int32)))
    total = int(offsets[n])
    return sizes, offsets, cols[:total], weights[:total], rows.reshape(n, transits_per_sample)
