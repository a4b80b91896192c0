"""The C++ host API header (include/libNextDoor_amd.hpp, the names of the reference's
src/libNextDoor.hpp:39-50) compiles against the library and behaves through a real caller."""
import os
import subprocess

import pytest

from tests.cpp import build_cpp
from tests.cpp.build_cpp import HOST_PROBE as EXE, TEMPLATE_PROBE, build_host_probe as build_probe


def write_graph(path):
    # a ring of 12 vertices with chords, text edge list "src dst"
    with open(path, "w") as f:
        for v in range(12):
            f.write(f"{v} {(v + 1) % 12}\n{(v + 1) % 12} {v}\n{v} {(v + 5) % 12}\n")


def test_header_compiles_and_host_paths_work(tmp_path):
    build_probe()
    graph = tmp_path / "ring.txt"
    write_graph(graph)
    out = subprocess.run([EXE, str(graph)], capture_output=True, text=True, timeout=60)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "vertices 12 edges 36" in out.stdout
    assert "NoSuchApp" in out.stdout  # the unknown app is reported, not aborted on


@pytest.mark.gpu
def test_nextdoor_entry_runs_on_the_gpu(tmp_path):
    assert os.path.exists(EXE), "tests/cpp/host_api_probe is built by __graft_entry__.build() / the CPU test"
    graph = tmp_path / "ring.txt"
    write_graph(graph)
    out = subprocess.run([EXE, str(graph), "gpu"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "totalSampledVertices 96" in out.stdout  # 12 walks x 8 steps, no dead ends
    assert "final_size 8 values 96" in out.stdout
    assert "kernel types agree" in out.stdout
    assert "edge lists 300" in out.stdout  # MVS5: 20 batches of 5 vertices with 3 out-edges each
    assert "reference-style tests pass" in out.stdout  # the testBase.h macro with the template spellings


def test_caller_with_an_app_of_its_own_compiles():
    """A translation unit in the reference's style - an App struct, then
    appMain<SampleType, App>(argc, argv, checkSampledVerticesResult<SampleType, App>) - builds
    with hipcc against the header; so does the testBase.h macro with the template spellings."""
    exe = build_cpp.build_template_probe()
    out = subprocess.run([exe], capture_output=True, text=True, timeout=60)  # no graph: usage text, as src/main.cu:31-47
    assert out.returncode == 0 and "--graph-file" in out.stdout


def parse_samples(text):
    rows = []
    for line in text.splitlines():
        if line.startswith("Contents of sample"):
            rows.append([int(v) for v in line[line.index("[") + 1:line.index("]")].split(",") if v.strip()])
    return rows


@pytest.mark.gpu
def test_caller_with_an_app_of_its_own_samples_what_the_oracle_does(tmp_path):
    import numpy as np
    from tests import oracle_binding as ob
    assert os.path.exists(TEMPLATE_PROBE), "tests/cpp/template_api_probe is built by __graft_entry__.build()"
    graph = tmp_path / "ring.txt"
    write_graph(graph)
    import nextdoor_amd as nd
    from tests import graphs
    loaded = nd.Graph.load(str(graph), "edge-list", "text")  # the same ingest, host only; owns the arrays below
    og = graphs.oracle_view(loaded)
    d = ob.app_desc(ob.UNIFORM_WALK, 6, [1] * 6)
    want, _ = ob.sample_individual(og, d, 42, np.arange(12, dtype=np.int32))
    for flags in (["-k", "TransitParallel", "-l"], ["-k", "TransitParallel"], ["-k", "SampleParallel"]):
        print("template_api_probe", flags, flush=True)
        out = subprocess.run([TEMPLATE_PROBE, "-g", str(graph), "-t", "edge-list", "-f", "text", "-n", "1", "-c", "-p"] + flags,
                             capture_output=True, text=True, timeout=120)
        assert out.returncode == 0, out.stdout + out.stderr
        assert "Graph has 36 edges and 12 vertices" in out.stdout
        assert np.array_equal(np.array(parse_samples(out.stdout), np.int32), want), out.stdout
        assert "totalSampledVertices 72" in out.stdout
        # the caller's checker read NextDoorData::samples: what next() left in every sample's state
        assert "sample states checked 12" in out.stdout, out.stdout
    out = subprocess.run([TEMPLATE_PROBE, "--registry-app", str(graph)], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    assert out.stdout.count("totalSampledVertices 108") == 2  # KHop3x2App: 12 samples x (3 + 6)
