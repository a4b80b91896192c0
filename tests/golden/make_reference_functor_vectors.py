"""Writes tests/golden/reference_functor_vectors.json: what the REFERENCE's own sampler functors
produce on the small fixed graph of make_vectors.py.

The samplers are the text of src/apps/khop/khop.cu, src/apps/randomwalks/randomWalks.cu,
src/apps/layer/layerSampling.cu and src/apps/multiRW/multiRW.cu, compiled from the reference tree as host C++ against this repository's App contract
(oracle/Makefile -> oracle/_ref/libreference_apps_host.so, never committed) and run by
oracle/reference_apps_host.cpp in a plain loop over samples with this repository's slot layout
and Philox streams.  So the numbers below are decided by the reference's next() code - its
rejection loops, its comparisons, its special cases - and not by this repository's restatement
of it.  Needs the reference tree at build time; the fixture it writes does not.

    make -C oracle reference && python tests/golden/make_reference_functor_vectors.py

Sizes are the reference's: KHop [25, 10]; Layer [10, 25]; DeepWalk, PPR and Node2Vec 100 steps; two
walks per vertex are kept (samples 0 .. 2V-1 of the 100 walks per vertex the apps ask for: a
sample's values depend on its index and root only); MultiRW 100 walkers and 100 steps per sample,
the walkers starting where this repository's MultiRW app starts them (a fixed Philox stream; the
reference draws them with rand())."""
import ctypes as C
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from tests import oracle_binding as ob  # noqa: E402
from tests.golden import make_vectors  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
REF_LIB = os.path.join(ob.ORACLE_DIR, "_ref", "libreference_apps_host.so")
SEED = 42
APPS = {"KHop": 0, "DeepWalk": 1, "PPR": 2, "Node2Vec": 3, "Layer": 4}  # ref_sample_individual's app numbers


def main():
    lib = C.CDLL(REF_LIB)
    i32p, f32p = C.POINTER(C.c_int32), C.POINTER(C.c_float)
    lib.ref_app_shape.argtypes = [C.c_int, C.c_int32, i32p, i32p, C.POINTER(C.c_int64)]
    lib.ref_sample_individual.argtypes = [C.c_int, C.c_int32, C.c_int64, i32p, i32p, f32p, f32p, C.c_uint64, C.c_int64,
                                          i32p, i32p, i32p]
    row_ptr, col, w = make_vectors.make_graph()
    g = ob.Graph(row_ptr, col, w)
    V = g.n_vertices
    out = {"seed": SEED, "graph": {"row_ptr": row_ptr, "col": col, "weight": w}, "apps": {}}
    for app, number in APPS.items():
        steps, sizes, n = C.c_int32(), (C.c_int32 * 128)(), C.c_int64()
        assert lib.ref_app_shape(number, V, C.byref(steps), sizes, C.byref(n)) == 0
        sizes = [sizes[k] for k in range(steps.value)]
        n_kept = V if app in ("KHop", "Layer") else 2 * V
        roots = (np.arange(n_kept) % V).astype(np.int32)
        F, per = 0, 1
        for m in sizes:
            per *= m
            F += per
        final = np.empty((n_kept, F), np.int32)
        t = np.empty(n_kept, np.int32)
        p = lambda a, ty: a.ctypes.data_as(C.POINTER(ty))  # noqa: E731
        rc = lib.ref_sample_individual(number, V, len(g.col), p(g.row_ptr, C.c_int32), p(g.col, C.c_int32),
                                       p(g.weight, C.c_float), p(g.max_weight, C.c_float), SEED, n_kept,
                                       p(roots, C.c_int32), p(final, C.c_int32), p(t, C.c_int32) if app == "Node2Vec" else None)
        assert rc == 0
        entry = {"steps": steps.value, "step_sizes": sizes, "samples_of_the_app": int(n.value), "initial": roots.tolist(),
                 "final": final.reshape(-1).tolist(), "shape": list(final.shape)}
        if app == "Node2Vec":
            entry["state_t"] = t.tolist()
        out["apps"][app] = entry
    # the multi-dimensional random walk (explicit transits)
    lib.ref_multirw_shape.argtypes = [i32p, i32p]
    lib.ref_sample_multirw.argtypes = [C.c_int32, C.c_int64, i32p, i32p, C.c_uint64, C.c_int64, i32p, i32p, i32p]
    n_roots, steps = C.c_int32(), C.c_int32()
    assert lib.ref_multirw_shape(C.byref(n_roots), C.byref(steps)) == 0
    roots = ob.multirw_roots(V, n_roots.value, V)
    walkers, last, final = roots.copy(), np.empty(V, np.int32), np.empty((V, steps.value), np.int32)
    p = lambda a, ty: a.ctypes.data_as(C.POINTER(ty))  # noqa: E731
    assert lib.ref_sample_multirw(V, len(g.col), p(g.row_ptr, C.c_int32), p(g.col, C.c_int32), SEED, V,
                                  p(walkers, C.c_int32), p(last, C.c_int32), p(final, C.c_int32)) == 0
    out["apps"]["MultiRW"] = {"steps": steps.value, "n_roots": n_roots.value, "roots": roots.reshape(-1).tolist(),
                              "final": final.reshape(-1).tolist(), "shape": list(final.shape),
                              "walkers": walkers.reshape(-1).tolist(), "last_root_idx": last.tolist()}
    path = os.path.join(HERE, "reference_functor_vectors.json")
    with open(path, "w") as f:
        json.dump(out, f, separators=(",", ":"))
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
