"""The C++ host API header (include/libNextDoor_amd.hpp, the names of the reference's
src/libNextDoor.hpp:39-50) compiles against the library and behaves through a real caller."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "tests", "cpp", "host_api_probe.cpp")
EXE = os.path.join(ROOT, "tests", "cpp", "host_api_probe")


def build_probe():
    from nextdoor_amd.build import LIB_PATH
    assert os.path.exists(LIB_PATH), "build the library first: python -m nextdoor_amd.build"
    lib_dir = os.path.dirname(LIB_PATH)
    cmd = ["g++", "-std=c++17", "-O1", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), SRC, "-o", EXE,
           "-L", lib_dir, "-lnextdoor_amd", "-Wl,-rpath," + lib_dir, "-Wl,-rpath,/opt/rocm/lib"]
    subprocess.run(cmd, check=True, capture_output=True, text=True)


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
