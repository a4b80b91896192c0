"""Benchmark of the transit-parallel sampling path on one MI355X.

One "step" is one full pass of the hot path over one batch: doTransitParallelSampling
(load balanced) of the weighted node2vec walk (p=2, q=0.5, length 100, one walk per
vertex) on the symmetrised R-MAT scale-22 graph, i.e. 419,430,400 sampled edges (output
slots).  The graph and all per-run buffers are resident in HBM before the timed region;
the timed region is the step loop only, as the reference's "End to end time"
(src/nextdoor.cu:2363-2963).

Prints one JSON line:  metric / value (sampled edges per second) / roofline (dominant
kernel, algorithmic bytes over its measured launch time) / cpu_baseline (the CPU oracle on
a bounded sample of the same walks, on this box's host cores) for that workload, and under
"configs" the same figures, shorter runs, for all five benchmark configurations (--only: just
the workload named with --workload).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0

# What rocprofv3 counter runs of this script recorded (the summaries under profiles/; a test compares
# these constants with the tables there).  Per profile: the dominant kernel(s), the HBM bytes one
# launch of it moves (FETCH_SIZE / WRITE_SIZE, scaled by a plain copy of known size:
# profiles/step_kernels_<profile>_hbm_traffic.md) and the HBM bytes of all kernels of a pass; where
# recorded, the read and write requests one launch sends past L2 (TCC_EA0_RDREQ_sum - every one of
# them 128 bytes - and TCC_EA0_WRREQ_sum: profiles/step_kernels_<profile>_l2_requests.md).
MEASURED = {
    "weighted_node2vec_rmat22": {
        "kernels": {"nd::step_flat_kernel": 1.123e9}, "bytes_per_pass": 145.38e9,
        "read_requests": {"nd::step_flat_kernel": 8.235e6}, "write_requests": {"nd::step_flat_kernel": 1.698e6}},
    # the same workload with --inversion-period 0 (the engine's choice: walks keep their lanes)
    "weighted_node2vec_rmat22_period0": {
        "kernels": {"nd::walk_stretch_kernel": 3.676e10}, "bytes_per_pass": 150.95e9,
        "read_requests": {"nd::walk_stretch_kernel": 2.843e8}, "write_requests": {"nd::walk_stretch_kernel": 6.536e6}},
    "uniform_walk_chunglu57k": {"kernels": {"nd::step_flat_kernel": 1.224e7}, "bytes_per_pass": 1.27e9},
    # both kernel classes of a hop; the flat kernel is launched for both hops, the workgroup kernel for the second
    "khop_rmat21": {"kernels": {"nd::step_flat_kernel": 1.088e9, "nd::step_workgroup_kernel": 2.385e9},
                    "bytes_per_pass": 8.45e9},
    # collective_mark_binned, average over its 2 launches per pass
    "fastgcn_importance_rmat22": {"kernels": {"nd::collective_mark_binned": 5.268e9}, "bytes_per_pass": 16.41e9},
    "ladies_importance_chunglu3m": {"kernels": {"nd::collective_mark_binned": 6.752e10}, "bytes_per_pass": 161.61e9},
}


def _one(values):
    return next(iter(values.values()))


# HBM bytes per launch of the dominant kernel (k-hop: the step kernels of one hop = the two flat
# launches and the workgroup launch of a pass, over its 2 hops)
MEASURED_TRAFFIC_BYTES_PER_LAUNCH = {name: _one(m["kernels"]) for name, m in MEASURED.items() if len(m["kernels"]) == 1}
MEASURED_TRAFFIC_BYTES_PER_LAUNCH["khop_rmat21"] = (2 * MEASURED["khop_rmat21"]["kernels"]["nd::step_flat_kernel"] +
                                                     MEASURED["khop_rmat21"]["kernels"]["nd::step_workgroup_kernel"]) / 2
MEASURED_TRAFFIC_BYTES_PER_PASS = {name: m["bytes_per_pass"] for name, m in MEASURED.items()}
MEASURED_L2_MISS_REQUESTS_PER_LAUNCH = {name: _one(m["read_requests"]) for name, m in MEASURED.items() if "read_requests" in m}
MEASURED_L2_WRITE_REQUESTS_PER_LAUNCH = {name: _one(m["write_requests"]) for name, m in MEASURED.items() if "write_requests" in m}

WORKLOADS = {
    # name: (app, graph factory kwargs)
    "weighted_node2vec_rmat22": dict(app="WeightedNode2Vec", kind="WEIGHTED_NODE2VEC",
                                     graph=("rmat", dict(scale=22, edge_factor=16, symmetrise=True))),
    "weighted_node2vec_rmat22_4walks": dict(app="WeightedNode2Vec4PerVertex", kind="WEIGHTED_NODE2VEC",
                                            graph=("rmat", dict(scale=22, edge_factor=16, symmetrise=True))),
    "weighted_node2vec_rmat16": dict(app="WeightedNode2Vec", kind="WEIGHTED_NODE2VEC",
                                     graph=("rmat", dict(scale=16, edge_factor=16, symmetrise=True))),
    # the reference's literal node2vec (unweighted acceptance, src/apps/randomwalks/randomWalks.cu:132-178)
    "node2vec_rmat22": dict(app="Node2VecPerVertex", kind="NODE2VEC",
                            graph=("rmat", dict(scale=22, edge_factor=16, symmetrise=True))),
    "uniform_walk_chunglu57k": dict(app="UniformRandomWalk", kind="UNIFORM_WALK",
                                    graph=("chung_lu", dict(n_vertices=56944, n_edges=818000, exponent=2.1))),
    "khop_rmat21": dict(app="KHop", kind="KHOP", graph=("rmat", dict(scale=21, edge_factor=32, symmetrise=False))),
    "fastgcn_importance_rmat22": dict(app="FastGCNImportance", kind="FASTGCN_IMPORTANCE",
                                      graph=("rmat", dict(scale=22, edge_factor=16, symmetrise=True))),
    "fastgcn_importance_rmat22_b128": dict(app="FastGCNImportanceB128", kind="FASTGCN_IMPORTANCE",
                                           graph=("rmat", dict(scale=22, edge_factor=16, symmetrise=True))),
    "ladies_importance_chunglu3m": dict(app="LADIESImportance", kind="LADIES_IMPORTANCE",
                                        graph=("chung_lu", dict(n_vertices=3072441, n_edges=117000000, exponent=2.0))),
    "ladies_importance_chunglu3m_b8": dict(app="LADIESImportanceB8", kind="LADIES_IMPORTANCE",
                                           graph=("chung_lu", dict(n_vertices=3072441, n_edges=117000000,
                                                                   exponent=2.0))),
    # edge-list apps of the reference (src/apps/mvs, src/apps/clustergcn) on the headline graph
    "mvs_rmat22": dict(app="MVS", kind="SUBGRAPH", graph=("rmat", dict(scale=22, edge_factor=16, symmetrise=True))),
    "clustergcn_rmat22": dict(app="ClusterGCN", kind="SUBGRAPH",
                              graph=("rmat", dict(scale=22, edge_factor=16, symmetrise=True))),
}


def make_graph(nd, spec):
    kind, kw = spec
    if kind == "rmat":
        return nd.Graph.rmat(kw["scale"], kw["edge_factor"], seed=42, symmetrise=kw["symmetrise"])
    return nd.Graph.chung_lu(kw["n_vertices"], kw["n_edges"], kw["exponent"], seed=42)


def cpu_baseline(graph, sampler, kind_name, budget_s, seed):
    """Times the CPU oracle on a strided subset of the same samples (whole walks), all host
    cores, growing the subset until it has run for about budget_s seconds."""
    from tests import graphs, oracle_binding as ob
    og = graphs.oracle_view(graph)
    steps = sampler.steps
    desc = ob.app_desc(getattr(ob, kind_name), steps, [sampler.step_size(k) for k in range(steps)],
                       initial_size=sampler.initial_sample_size)
    roots = sampler.initial_contents.reshape(sampler.num_samples, -1)
    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16")))
    outputs_per_sample = sampler.final_sample_size
    stride = max(1, sampler.num_samples // 4096)
    best = None
    while True:
        sub = np.ascontiguousarray(roots[::stride]).reshape(-1)
        t0 = time.perf_counter()
        _, _, stats = ob.sample_individual(og, desc, seed, sub, n_threads=cores, want_stats=True)
        dt = time.perf_counter() - t0
        n = len(sub) // desc.initial_size
        best = dict(seconds=dt, samples=n, stats=stats, stride=stride)
        if dt >= budget_s / 3 or stride == 1:
            break
        stride = max(1, int(stride / min(8.0, max(2.0, budget_s / max(dt, 1e-3) / 2))))
    edges = best["samples"] * outputs_per_sample
    return {
        "value": edges / best["seconds"], "unit": "sampled edges/s", "cores": cores, "kind": "port",
        "sample": f"CPU oracle, every {best['stride']}th walk ({best['samples']} of {sampler.num_samples} samples, "
                  f"all {steps} steps), {best['seconds']:.1f} s",
    }, best


def cpu_baseline_layers(graph, sampler, kind_name, budget_s, seed):
    """Layer-wise apps: times the CPU oracle on the first batches of the same launch, all
    host cores (one batch per thread), doubling the number of batches until it has run for
    about a third of budget_s."""
    from tests import graphs, oracle_binding as ob
    og = graphs.oracle_view(graph)
    steps = sampler.steps
    desc = ob.app_desc(getattr(ob, kind_name), steps, [sampler.step_size(k) for k in range(steps)],
                       initial_size=sampler.initial_sample_size)
    roots = sampler.initial_contents.reshape(sampler.num_samples, -1)
    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16")))
    fn = ob.sample_fastgcn_importance if kind_name == "FASTGCN_IMPORTANCE" else ob.sample_ladies_importance
    n = min(sampler.num_samples, cores)
    while True:
        t0 = time.perf_counter()
        fn(og, desc, seed, roots[:n].reshape(-1), first_sample=0, n_threads=cores)
        dt = time.perf_counter() - t0
        if dt >= budget_s / 3 or n == sampler.num_samples:
            break
        n = min(sampler.num_samples, n * 2)
    return {
        "value": n * sampler.final_sample_size / dt, "unit": "sampled edges/s", "cores": cores, "kind": "port",
        "sample": f"CPU oracle, the first {n} of {sampler.num_samples} batches (all layers), {dt:.1f} s",
    }


def marking_bytes_per_pass(graph, sampler, final, ladies):
    """Bytes the marking kernel (collective_mark_binned) has to move in one pass, counted on
    the host from the transits of every layer.  A transit with fewer edges into a stretch of the
    vertex range than the library's threshold contributes those entries (id 4 B, + weight 4 B
    for LADIES); with more, the stretch's ready-made piece (a bit per vertex, or a 64-bit sum
    per vertex).  Every layer writes its whole per-sample map (bits, or 32-bit sampling keys).
    FastGCN: a vertex that is among a sample's transits more than once counts once."""
    stretch = 7168 if ladies else 65536
    threshold = int(os.environ.get("ND_DENSE_PIECE_ENTRIES", 2048 if ladies else 1024))
    piece_bytes = stretch * 8 if ladies else stretch // 8
    entry_bytes = 8 if ladies else 4
    rp, col = np.asarray(graph.row_ptr), np.asarray(graph.col)
    degree = np.diff(rp).astype(np.int64)
    n_samples, batch = sampler.num_samples, sampler.step_size(0)
    layers = [sampler.initial_contents.reshape(-1)]
    layers += [final[:, k * batch:(k + 1) * batch].reshape(-1) for k in range(sampler.steps - 1)]
    if not ladies:
        # the bitmap form marks a vertex once however often it is among a sample's transits
        firsts = []
        for layer in layers:
            rows = np.sort(layer.reshape(n_samples, -1), axis=1)
            keep = np.ones(rows.shape, bool)
            keep[:, 1:] = rows[:, 1:] != rows[:, :-1]
            firsts.append(rows[keep])
        layers = firsts
    transits = np.concatenate(layers)
    transits = transits[(transits != sampler.invalid_vertex) & (transits >= 0)]
    vertices, uses = np.unique(transits, return_counts=True)
    big = degree[vertices] >= threshold if threshold > 0 else np.zeros(len(vertices), bool)
    entries = int((uses[~big] * degree[vertices[~big]]).sum())
    pieces, distinct_pieces = 0, 0
    for v, c in zip(vertices[big], uses[big]):
        per_stretch = np.bincount(col[rp[v]:rp[v + 1]] // stretch)
        ready = per_stretch >= threshold
        pieces += int(c) * int(ready.sum())
        distinct_pieces += int(ready.sum())
        entries += int(c) * int(per_stretch[~ready].sum())
    words = ((graph.n_vertices + 31) // 32 + 2047) // 2048 * 2048  # a bit per vertex, padded to 2048 words
    per_sample_out = (words + 223) // 224 * 7168 * 4 if ladies else words * 4  # LADIES: a 32-bit key per vertex
    written = sampler.steps * n_samples * per_sample_out
    # from_memory: every entry and every written map once, every piece that is used at all once
    # per layer (the pieces are a few thousand per graph and stay in the caches between uses)
    from_memory = entries * entry_bytes + sampler.steps * distinct_pieces * piece_bytes + written
    return entries * entry_bytes + pieces * piece_bytes + written, entries, pieces, from_memory


def pairs_reaching_the_step_kernels(sampler, final):
    """Pairs every step's kernels are launched over.  Step 0: every root.  Step k > 0: the pairs
    the inversion keeps, i.e. the previous step's outputs that are vertices (the first sort pass
    drops the rest, and their output slots keep the fill value).  Counted on the result rows."""
    live = [sampler.num_samples * sampler.initial_sample_size]
    base, per_sample = 0, sampler.initial_sample_size
    for k in range(sampler.steps - 1):
        per_sample *= sampler.step_size(k)
        live.append(int(np.count_nonzero(final[:, base:base + per_sample] != sampler.invalid_vertex)))
        base += per_sample
    return live


def algorithmic_bytes_per_pass(sampler, oracle_run, live, weighted, second_order, state_travels):
    """Minimal 4-byte-granular HBM traffic of one pass, split by kernel family.  Only pairs that
    reach a kernel are charged (see pairs_reaching_the_step_kernels); the per-candidate counters
    come from the oracle's run over a subset of the samples, scaled to all samples.
    Step kernels, per pair: (transit, slot) 8 (step 0: the root, 4) + row extent 8 (+ 4 largest
    weight); per candidate edge: id 4 (+ 4 weight); second order: previous vertex read + write 8 and
    its row extent 8 per next() call, 4 per binary-search probe; per output: final sample 4 and,
    unless the step is the last, the next step's pair 8.
    `own`: the same with the adjacency test priced as this engine performs it - no row extent of
    the previous vertex, one 8-byte edge-index slot per test, and a test only for the candidates
    whose acceptance depends on the bias - instead of a binary search per candidate.
    Inversion of the pairs entering step k (walks; records of 8 bytes, 12 with a travelling
    state): the first digit pass reads every pair the previous step emitted (histogram 4 +
    scatter 8 or 12) and writes the kept ones; each later pass reads 4 + record and writes the
    record of every kept pair.  Other apps read the previous step's outputs as keys (4) and
    generate the slot."""
    st = oracle_run["stats"]
    scale = sampler.num_samples / oracle_run["samples"]
    steps = sampler.steps
    passes = (sampler.max_bits + 7) // 8
    per_pair = 8 + (4 if weighted else 0)
    step_bytes = live[0] * (4 + per_pair) + sum(live[1:]) * (8 + per_pair)
    outputs = [live[k] * sampler.step_size(k) for k in range(steps)]
    step_bytes += sum(outputs) * 4 + sum(outputs[:-1]) * 8
    step_bytes += scale * (st["edge_reads"] * 4 + st["weight_reads"] * 4)
    own_bytes = step_bytes
    if second_order:
        step_bytes += scale * (st["next_calls"] * 16 + st["search_probes"] * 4)
        own_bytes += scale * (st["next_calls"] * 8 + st["band_tests"] * 8)
    walk = sampler.initial_sample_size == 1 and all(sampler.step_size(k) == 1 for k in range(steps))
    record = 12 if (walk and state_travels) else 8
    sort_bytes = 0
    for k in range(1, steps):
        entering = outputs[k - 1]  # what step k - 1 emitted, dead pairs included
        first_read = 4 + record if walk else 4 + 4
        sort_bytes += entering * first_read + live[k] * record + (passes - 1) * live[k] * (4 + 2 * record)
    return step_bytes, own_bytes, sort_bytes


def measure(args, workload, steps, warmup, cpu_seconds, graphs, engine_choice=True):
    """One workload: graph, sampler, warm-up, `steps` timed passes, one pass with per-phase events,
    the CPU baseline.  Returns the result line as a dict.  graphs: cache of built graphs by spec."""
    import nextdoor_amd as nd
    w = WORKLOADS[workload]
    t0 = time.perf_counter()
    key = json.dumps(w["graph"], sort_keys=True)
    if key not in graphs:
        graphs.clear()  # one large graph in host memory at a time
        graphs[key] = make_graph(nd, w["graph"])
    graph = graphs[key]
    t_graph = time.perf_counter() - t0
    t0 = time.perf_counter()
    sampler = nd.Sampler(w["app"], graph, seed=args.seed)
    t_setup = time.perf_counter() - t0
    sampler.set_inversion_period(args.inversion_period)
    lb = not args.no_load_balancing
    edges_per_pass = sampler.num_samples * sampler.final_sample_size
    skip_cpu_baseline = args.skip_cpu_baseline

    for _ in range(warmup):
        sampler.do_transit_parallel(lb)
    wall0 = time.perf_counter()
    gpu_ms = []
    for _ in range(steps):
        sampler.do_transit_parallel(lb)  # synchronises its stream before returning
        gpu_ms.append(sampler.phase_times()["end_to_end_ms"])
    wall = time.perf_counter() - wall0
    ms_per_step = wall * 1000.0 / steps
    per_transit = w["kind"] not in ("FASTGCN_IMPORTANCE", "LADIES_IMPORTANCE", "SUBGRAPH")
    schedule = None
    if per_transit and lb:
        # since the buffers were allocated: passes, passes whose steps were classified (a pass after
        # one that found no work item is not), and how the classified steps' two kernel classes ran
        passes, classified, merged, forked, serial = (sampler.counter(i) for i in range(5, 10))
        schedule = {"passes": passes, "lb_passes_that_classified": classified, "steps_as_one_launch": merged,
                    "steps_on_two_streams": forked, "steps_one_kernel_after_the_other": serial}

    # per-kernel-family durations: one extra pass with events around every launch group
    sampler.set_profiling(True)
    sampler.do_transit_parallel(lb)
    prof = sampler.phase_times()
    sampler.set_profiling(False)
    if schedule is not None and sampler.step_size(0) == 1 and sampler.steps > 1 and prof["sort_passes"] == 0:
        # a walk over a small map: the kernel that emits a pair places it for the next step, one
        # launch per step, every pair with the flat lanes - nothing is sorted or classified
        schedule["small_map_placed_as_emitted"] = True
    kernel_classes = None
    if per_transit and lb:
        # pairs per kernel class over the steps of the last pass whose classification ran (the
        # reference's printKernelTypes, src/nextdoor.cu:2117-2189)
        looked, single, split, refused, items = (sampler.counter(i) for i in range(5))
        kernel_classes = {"pairs_classified": looked, "flat_pairs": looked - single - split, "workgroup_pairs": single,
                          "grid_wide_pairs": split, "left_to_flat_for_their_degree": refused, "work_items": items}
    final = sampler.final_samples()
    valid = int((final != sampler.invalid_vertex).sum())

    # walks, for information only (not the headline): the same pass when the engine chooses how
    # often to invert; the samples must come out the same
    adaptive = None
    if sampler.step_size(0) == 1 and sampler.steps > 1 and args.inversion_period == 1 and engine_choice:
        sampler.set_inversion_period(0)
        sampler.do_transit_parallel(lb)
        t0 = time.perf_counter()
        for _ in range(steps):
            sampler.do_transit_parallel(lb)
        ms = (time.perf_counter() - t0) * 1000.0 / steps
        same = bool(np.array_equal(sampler.final_samples(), final))
        adaptive = {"ms_per_step": ms, "sampled_edges_per_s": edges_per_pass / (ms / 1000.0), "same_samples": same}
        sampler.set_profiling(True)
        sampler.do_transit_parallel(lb)
        chosen = sampler.phase_times()
        sampler.set_profiling(False)
        adaptive["phases_ms"] = {k: round(v, 3) for k, v in chosen.items()
                                 if k in ("inversion_ms", "flat_kernel_ms", "assemble_ms", "flat_launches", "sort_passes")}
        sampler.set_inversion_period(1)

    result = {
        "metric": "sampled edges/sec on 1 MI355X", "value": edges_per_pass / (ms_per_step / 1000.0),
        "unit": "sampled edges/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int32 ids / f32 weights", "data": "synthetic",
        "config": {"workload": workload, "app": w["app"], "vertices": graph.n_vertices, "edges": graph.n_edges,
                   "samples": sampler.num_samples, "walk_steps": sampler.steps, "load_balancing": lb,
                   "sampled_edges_per_step": edges_per_pass,
                   "value_counts": "output slots of a pass, INVALID ones included (valid_outputs of them hold a vertex)",
                   "valid_outputs": valid,
                   "valid_sampled_edges_per_s": valid / (ms_per_step / 1000.0),
                   "graph_build_s": round(t_graph, 1), "sampler_setup_s": round(t_setup, 1),
                   "gpu_event_ms_per_step": float(np.mean(gpu_ms))},
        "phases_ms": {k: round(v, 3) for k, v in prof.items()},
    }
    if kernel_classes:
        result["config"]["kernel_classes"] = kernel_classes
    if schedule:
        result["config"]["load_balancing_schedule"] = schedule
    result["config"]["inversion_period"] = args.inversion_period
    if adaptive:
        result["config"]["engine_chosen_inversion_period"] = adaptive
    if w["kind"] in ("FASTGCN_IMPORTANCE", "LADIES_IMPORTANCE"):
        entries, distinct = sampler.counter(0), sampler.counter(1)
        result["config"]["neighbourhood_entries"] = entries
        result["config"]["distinct_pairs"] = distinct
        result["config"]["chunks"] = sampler.counter(2)
        result["config"]["hub_bitmaps"] = sampler.counter(3)
        result["config"]["neighbourhood_entries_per_s"] = entries / (ms_per_step / 1000.0)
        # dominant kernel: collective_mark_binned accounts for every entry of every collective
        # neighbourhood once, one by one or through the ready-made pieces of the hubs
        ladies = w["kind"] == "LADIES_IMPORTANCE"
        mark_bytes, read_entries, read_pieces, from_memory = marking_bytes_per_pass(graph, sampler, final, ladies)
        result["config"]["entries_read_one_by_one"] = read_entries
        result["config"]["hub_pieces_read"] = read_pieces
        launches = max(prof["neighbourhood_launches"], 1)
        # `achieved` prices what has to come from or go to HBM: entries read one by one, the
        # maps written, and every ready-made piece once per layer; the repeated uses of the few
        # thousand pieces are served by the caches and are reported apart, not as HBM bytes
        achieved = from_memory / (prof["neighbourhood_ms"] / 1000.0) / 1e9
        all_uses = mark_bytes / (prof["neighbourhood_ms"] / 1000.0) / 1e9
        # what the recorded counters say the launch is bound by: its measured HBM traffic over this
        # run's launch time.  The LADIES form streams (entries in, keys out: near half of the HBM
        # peak); the FastGCN form moves a fifth of the peak - its hubs' pieces and adjacencies come
        # from the caches, and a workgroup spends its time in the chain of searches, LDS table and
        # barriers it goes through per stretch of the vertex range
        recorded = MEASURED_TRAFFIC_BYTES_PER_LAUNCH.get(workload)
        traffic_gbps = recorded / (prof["neighbourhood_ms"] / launches / 1000.0) / 1e9 if recorded else None
        bound = "hbm" if traffic_gbps is None or traffic_gbps / HBM_PEAK_GBS >= 0.3 else \
            "latency (dependent steps per stretch of the vertex range; the caches serve the hubs)"
        result["roofline"] = {
            "bound": bound, "kernel": "collective_mark_binned", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS, "traffic": recorded,
            "measured_traffic_GBps": traffic_gbps,
            "measured_traffic_frac": traffic_gbps / HBM_PEAK_GBS if traffic_gbps else None,
            "algorithmic_bytes_per_launch": from_memory / launches,
            "avg_launch_ms": prof["neighbourhood_ms"] / launches,
            "cache_served": {"bytes_per_launch_with_every_piece_use": mark_bytes / launches,
                             "GBps_with_every_piece_use": all_uses,
                             "note": "piece uses beyond the first per layer come from L2 / Infinity Cache: a cache "
                                     "throughput figure, not an HBM roofline fraction"},
            "whole_pass": {"measured_traffic": MEASURED_TRAFFIC_BYTES_PER_PASS.get(workload)},
        }
        if not skip_cpu_baseline:
            result["cpu_baseline"] = cpu_baseline_layers(graph, sampler, w["kind"], cpu_seconds, args.seed)
        skip_cpu_baseline = True  # the walk/k-hop accounting below does not apply to layer-wise apps
    if w["kind"] == "SUBGRAPH":
        listed = sampler.counter(0)
        result["config"]["edges_listed"] = listed
        result["config"]["edges_listed_per_s"] = listed / (ms_per_step / 1000.0)
        # minimal traffic of a pass: the result rows and the lists written once; MVS also reads
        # every listed edge once, ClusterGCN the 32 row extents and vertices of every sample
        rows_bytes = 4.0 * edges_per_pass
        reads = 4.0 * listed if w["app"] == "MVS" else sampler.num_samples * 32 * 12.0
        achieved = (rows_bytes + 8.0 * listed + reads) / (np.mean(gpu_ms) / 1000.0) / 1e9
        result["roofline"] = {"bound": "hbm", "kernel": "subgraph_step_kernel (count + write passes)",
                              "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                              "frac": achieved / HBM_PEAK_GBS, "traffic": None}
        skip_cpu_baseline = True
    if w["kind"] == "KHOP":
        counts = sampler.distinct()
        result["config"]["distinct_ms"] = sampler.phase_times()["distinct_ms"]
        result["config"]["distinct_kept"] = int(counts.sum())
    if not skip_cpu_baseline:
        base, run = cpu_baseline(graph, sampler, w["kind"], cpu_seconds, args.seed)
        result["cpu_baseline"] = base
        # the reference's only CPU path over the samples is its validator (src/check_results.cu:162-299):
        # ours, over every output of the pass just sampled, on the same host cores
        t0 = time.perf_counter()
        ok, why = sampler.check_results()
        dt = time.perf_counter() - t0
        result["cpu_baseline"]["validator"] = {"passed": bool(ok), "seconds": round(dt, 2),
                                               "outputs_checked_per_s": edges_per_pass / dt,
                                               "report": None if ok else why}
        weighted = w["kind"] in ("WEIGHTED_NODE2VEC", "DEEPWALK", "PPR")
        second = w["kind"] in ("WEIGHTED_NODE2VEC", "NODE2VEC")
        live = pairs_reaching_the_step_kernels(sampler, final)
        step_bytes, own_bytes, sort_bytes = algorithmic_bytes_per_pass(
            sampler, run, live, weighted, second, state_travels=w["kind"] in ("WEIGHTED_NODE2VEC", "NODE2VEC"))
        if w["kind"] != "WEIGHTED_NODE2VEC":
            own_bytes = step_bytes  # the other apps run the reference's algorithm as written
        step_ms = prof["flat_kernel_ms"] + prof["workgroup_kernel_ms"]
        launches = prof["flat_launches"]
        # dominant kernel family: the step kernels (flat + workgroup launched back to back per walk step)
        achieved = step_bytes / (step_ms / 1000.0) / 1e9
        pass_ms = float(np.mean(gpu_ms))
        result["roofline"] = {
            "bound": "hbm", "kernel": "step_flat_kernel + step_workgroup_kernel", "achieved": achieved,
            "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
            "frac_own_algorithm": own_bytes / (step_ms / 1000.0) / 1e9 / HBM_PEAK_GBS,
            "traffic": MEASURED_TRAFFIC_BYTES_PER_LAUNCH.get(workload),
            "algorithmic_bytes_per_launch": step_bytes / max(launches, 1),
            "own_algorithm_bytes_per_launch": own_bytes / max(launches, 1),
            "avg_launch_ms": step_ms / max(launches, 1),
            "pairs_reaching_kernels_per_pass": int(sum(live)),
            "whole_pass": {"algorithmic_bytes": step_bytes + sort_bytes, "inversion_bytes": sort_bytes,
                           "achieved_GBps": (step_bytes + sort_bytes) / (pass_ms / 1000.0) / 1e9,
                           "frac": (step_bytes + sort_bytes) / (pass_ms / 1000.0) / 1e9 / HBM_PEAK_GBS,
                           "measured_traffic": MEASURED_TRAFFIC_BYTES_PER_PASS.get(workload)},
        }
        result["config"]["bytes_per_sampled_edge"] = (step_bytes + sort_bytes) / edges_per_pass
        if adaptive:
            # the same accounting for the pass with the engine-chosen inversion period: the step
            # kernels' algorithmic bytes are those of the algorithm, whatever the schedule
            chosen_ms = adaptive["phases_ms"]["flat_kernel_ms"]
            chosen_launches = max(adaptive["phases_ms"]["flat_launches"], 1)
            period0 = MEASURED.get(workload + "_period0")
            adaptive["roofline"] = {
                "bound": "hbm", "kernel": "walk_stretch_kernel (and step_flat_kernel for step 0)",
                "achieved": step_bytes / (chosen_ms / 1000.0) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": step_bytes / (chosen_ms / 1000.0) / 1e9 / HBM_PEAK_GBS,
                "algorithmic_bytes_per_launch": step_bytes / chosen_launches,
                "avg_launch_ms": chosen_ms / chosen_launches,
                "traffic": _one(period0["kernels"]) if period0 else None,
                "whole_pass": {"measured_traffic": period0["bytes_per_pass"] if period0 else None,
                               "measured_traffic_GBps": period0["bytes_per_pass"] / (adaptive["ms_per_step"] / 1000.0) / 1e9
                               if period0 else None},
            }
        traffic = MEASURED_TRAFFIC_BYTES_PER_LAUNCH.get(workload)
        if traffic and w["kind"] != "KHOP":  # walks: the recorded figure is the flat kernel's launch
            # recorded counter traffic of one launch over this run's launch duration (flat kernel alone)
            flat_launch_s = prof["flat_kernel_ms"] / max(launches, 1) / 1000.0
            result["roofline"]["traffic_frac"] = traffic / flat_launch_s / 1e9 / HBM_PEAK_GBS
        misses = MEASURED_L2_MISS_REQUESTS_PER_LAUNCH.get(workload)
        if misses:
            # The step kernel's reads are dependent random gathers; each one that misses L2 costs a
            # 128-byte request whatever it uses.  The ceiling for such requests is measured here, on
            # this GPU, over a table of the size of the graph's arrays (rounded down to a power of two).
            graph_bytes = 4.0 * graph.n_vertices * 2 + graph.n_edges * (8.0 + 4.0 * 8.0)
            table_bytes = 1 << (int(graph_bytes).bit_length() - 1)
            # the probe in every shape (1, 2, 4, 8 reads in flight per lane; workgroups of 64 and
            # 256 lanes): the ceiling is the best of them
            ceiling, by_shape = nd.gather_rate_ceiling(table_bytes)
            flat_ms = prof["flat_kernel_ms"] / max(launches, 1)
            writes = MEASURED_L2_WRITE_REQUESTS_PER_LAUNCH.get(workload, 0.0)
            result["roofline"]["l2_miss_path"] = {
                "read_requests_per_launch": misses, "bytes_per_read_request": 128,
                "write_requests_per_launch": writes,
                "achieved_read_requests_per_s": misses / (flat_ms / 1000.0),
                "achieved_requests_per_s": (misses + writes) / (flat_ms / 1000.0),
                "ceiling_requests_per_s": ceiling, "ceiling_table_bytes": table_bytes,
                "ceiling_kind": "independent random 8-byte reads, the best of 8 probe shapes, measured in this run",
                "ceiling_by_shape": {f"{k}_in_flight_{lanes}_lanes": round(v / 1e9, 2) for (k, lanes), v in by_shape.items()},
                "frac_of_ceiling": misses / (flat_ms / 1000.0) / ceiling,
                "frac_of_ceiling_note": "read requests over the read ceiling; the launch's write requests are "
                                        "not priced (the probe does not write)",
                "reads_and_writes_over_read_ceiling": (misses + writes) / (flat_ms / 1000.0) / ceiling,
                "ceiling_as_GBps": ceiling * 128 / 1e9,
            }
            period0 = MEASURED.get(workload + "_period0")
            if adaptive and "roofline" in adaptive and period0 and "read_requests" in period0:
                # the stretch kernel against the same ceiling: its recorded requests per launch (the
                # average over a pass's stretches) times the stretches of this pass, over the time
                # of the pass's step kernels (which includes the one flat launch of step 0)
                stretches = max(adaptive["phases_ms"]["flat_launches"] - 1, 1)
                reads = _one(period0["read_requests"]) * stretches
                chosen_s = adaptive["phases_ms"]["flat_kernel_ms"] / 1000.0
                adaptive["roofline"]["l2_miss_path"] = {
                    "read_requests_per_pass": reads, "write_requests_per_pass": _one(period0["write_requests"]) * stretches,
                    "achieved_read_requests_per_s": reads / chosen_s, "ceiling_requests_per_s": ceiling,
                    "frac_of_ceiling": reads / chosen_s / ceiling}
    del final
    sampler.close()
    return result


HEADLINE = "weighted_node2vec_rmat22"
FIVE_CONFIGS = ["uniform_walk_chunglu57k", "weighted_node2vec_rmat22", "khop_rmat21", "fastgcn_importance_rmat22",
                "ladies_importance_chunglu3m"]


def summary(r):
    """The per-config entry of the result line."""
    out = {"workload": r["config"]["workload"], "ms_per_step": r["ms_per_step"], "steps": r["steps"],
           "value": r["value"], "unit": r["unit"], "valid_sampled_edges_per_s": r["config"]["valid_sampled_edges_per_s"],
           "phases_ms": r["phases_ms"]}
    for key in ("neighbourhood_entries_per_s", "distinct_ms", "kernel_classes", "load_balancing_schedule"):
        if key in r["config"]:
            out[key] = r["config"][key]
    if "engine_chosen_inversion_period" in r["config"]:
        e = r["config"]["engine_chosen_inversion_period"]
        out["engine_chosen_inversion_period"] = {k: e[k] for k in ("ms_per_step", "sampled_edges_per_s", "same_samples")}
        if "roofline" in e:
            out["engine_chosen_inversion_period"]["roofline"] = {k: e["roofline"][k] for k in ("kernel", "frac", "avg_launch_ms",
                                                                                              "algorithmic_bytes_per_launch")}
    if "roofline" in r:
        out["roofline"] = {k: r["roofline"][k] for k in ("kernel", "bound", "frac", "achieved", "avg_launch_ms",
                                                         "algorithmic_bytes_per_launch", "traffic") if k in r["roofline"]}
    if "cpu_baseline" in r:
        out["cpu_baseline"] = {k: r["cpu_baseline"][k] for k in ("value", "unit", "cores", "kind", "sample")}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--workload", default=HEADLINE, choices=sorted(WORKLOADS))
    ap.add_argument("--only", action="store_true",
                    help="measure the workload given with --workload alone; by default the other benchmark "
                         "configurations are measured as well (shorter runs) and reported under \"configs\"")
    ap.add_argument("--no-load-balancing", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=15.0)
    ap.add_argument("--skip-cpu-baseline", action="store_true")
    ap.add_argument("--inversion-period", type=int, default=1,
                    help="walks: invert the sample->transit map before every p-th step (1: every step, as the "
                         "reference; 0: the engine decides); the samples do not depend on it")
    ap.add_argument("--skip-engine-choice", action="store_true",
                    help="walks: do not also measure the pass with the engine-chosen inversion period")
    ap.add_argument("--seed", type=int, default=42)
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one MI355X; this build has no multi-GPU path (samples would shard "
                 "by contiguous ranges with the graph replicated). Run with --gpus 1.")

    graphs = {}
    result = measure(args, args.workload, args.steps, args.warmup, args.cpu_seconds, graphs,
                     engine_choice=not args.skip_engine_choice)
    if not args.only and args.workload == HEADLINE:
        # the other configurations: a few timed passes each and a short CPU baseline, so that the
        # whole run stays within minutes; the configuration that shares the headline's graph first
        configs = {args.workload: summary(result)}
        order = ["fastgcn_importance_rmat22", "uniform_walk_chunglu57k", "khop_rmat21", "ladies_importance_chunglu3m"]
        for name in order:
            t0 = time.perf_counter()
            r = measure(args, name, min(args.steps, 5), 1, min(args.cpu_seconds, 3.0), graphs,
                        engine_choice=not args.skip_engine_choice)
            configs[name] = summary(r)
            configs[name]["bench_seconds"] = round(time.perf_counter() - t0, 1)
        result["configs"] = [configs[name] for name in FIVE_CONFIGS]
    print(json.dumps(result))


if __name__ == "__main__":
    main()
