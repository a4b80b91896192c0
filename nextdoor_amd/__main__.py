"""Command line of the sampling applications: ``python -m nextdoor_amd <App> <options>``.

One entry point for every app instead of one binary per app, with the options of the
reference's ``appMain`` (src/main.cu:5-55) and the run of its ``nextdoor()`` driver
(src/nextdoor.cu:3239-3307): load the graph, allocate, sample ``--nruns`` times with the chosen
kernel type, fetch the samples, print their count (and contents), check them.
"""
import argparse
import sys

import numpy as np

from . import Graph, NextDoorError, Sampler, app_names


def build_parser():
    p = argparse.ArgumentParser(prog="python -m nextdoor_amd", description=__doc__.splitlines()[0])
    p.add_argument("app", nargs="?", help="application to run; --list-apps prints the choices")
    p.add_argument("--list-apps", action="store_true", help="print the application names and exit")
    p.add_argument("-g", "--graph-file", help="File containing graph")
    p.add_argument("-t", "--graph-type", help="Format of graph file: 'adj-list' or 'edge-list'")
    p.add_argument("-f", "--graph-format", "--format", dest="graph_format",
                   help="Format of graph file: 'binary' or 'text'")
    p.add_argument("-n", "--nruns", type=int, default=1, help="Number of runs")
    p.add_argument("-c", "--check-results", action="store_true", help="Check results using an algorithm")
    p.add_argument("-p", "--print-samples", action="store_true", help="Print Samples")
    p.add_argument("-k", "--kernel-type", default="TransitParallel",
                   help="Type of Kernel: 'SampleParallel' or 'TransitParallel'")
    p.add_argument("-l", "--load-balancing", action="store_true", help="Enable Load Balancing")
    p.add_argument("--seed", type=int, default=42, help="seed of the counter-based random numbers")
    p.add_argument("--phases", action="store_true",
                   help="also time inversion, load balancing and step kernels (an event wait per launch: "
                        "the end-to-end time of such a run is longer)")
    return p


def run(argv=None, out=sys.stdout):
    parser = build_parser()
    args = parser.parse_args(argv)
    if args.list_apps:
        print("\n".join(app_names()), file=out)
        return 0
    # as appMain: without the three graph options there is nothing to run, print the usage
    if not (args.app and args.graph_file and args.graph_type and args.graph_format):
        parser.print_usage(out)
        return 0
    if args.kernel_type not in ("TransitParallel", "SampleParallel"):
        print("unknown kernel type '%s'" % args.kernel_type, file=sys.stderr)
        return 2
    try:
        graph = Graph.load(args.graph_file, args.graph_type, args.graph_format)
    except NextDoorError as e:
        print(str(e), file=sys.stderr)
        return 1
    print("Graph has %d edges and %d vertices " % (graph.n_edges, graph.n_vertices), file=out)
    try:
        sampler = Sampler(args.app, graph, seed=args.seed)
        sampler.set_profiling(args.phases)
        for _ in range(max(args.nruns, 0)):
            if args.kernel_type == "TransitParallel":
                sampler.do_transit_parallel(load_balancing=args.load_balancing)
            else:
                sampler.do_sample_parallel()
            t = sampler.phase_times()
            if args.phases:
                print("End to end time %.3f ms (inversion %.3f, load balancing %.3f, step kernels %.3f)" % (
                    t["end_to_end_ms"], t["inversion_ms"], t["load_balancing_ms"],
                    t["flat_kernel_ms"] + t["workgroup_kernel_ms"] + t["neighbourhood_ms"]), file=out)
            else:
                print("End to end time %.3f ms" % t["end_to_end_ms"], file=out)
        final = sampler.final_samples()
        if args.print_samples:
            for s in range(final.shape[0]):
                print("Contents of sample %d [%s]" % (s, "".join("%d, " % v for v in final[s])), file=out)
        print("totalSampledVertices %d" % int(np.count_nonzero(final != sampler.invalid_vertex)), file=out)
        ok = True
        if args.check_results:
            print("checking results", file=out)
            ok, why = sampler.check_results()
            print("Results Checked" if ok else why, file=out)
        sampler.free_device()
        return 0 if ok else 1
    except NextDoorError as e:
        print(str(e), file=sys.stderr)
        return 1


if __name__ == "__main__":
    sys.exit(run())
