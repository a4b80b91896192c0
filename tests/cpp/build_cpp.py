"""Builds the C++ callers the tests run: a host-only caller (g++), a caller with an App of its
own (hipcc, as the reference's app binaries are built by nvcc), and a shared object that
registers two user apps with the library.  Called by __graft_entry__.build() and by the CPU
tests; the GPU tests run what is built."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
INCLUDE = os.path.join(ROOT, "include")
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HOST_PROBE_SRC = os.path.join(HERE, "host_api_probe.cpp")
HOST_PROBE = os.path.join(HERE, "host_api_probe")
TEMPLATE_PROBE_SRC = os.path.join(HERE, "template_api_probe.hip")
TEMPLATE_PROBE = os.path.join(HERE, "template_api_probe")
USER_APPS_SRC = os.path.join(HERE, "user_apps.hip")
USER_APPS_LIB = os.path.join(HERE, "libuser_apps.so")


def _lib_dir():
    from nextdoor_amd.build import LIB_PATH
    assert os.path.exists(LIB_PATH), "build the library first: python -m nextdoor_amd.build"
    return os.path.dirname(LIB_PATH)


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    log = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError(" ".join(cmd) + "\n" + log)


def _link_flags():
    lib_dir = _lib_dir()
    # $ORIGIN: the built files travel with the tree, wherever it is put
    return ["-L", lib_dir, "-lnextdoor_amd", "-Wl,-rpath,$ORIGIN/../../nextdoor_amd", "-Wl,-rpath,/opt/rocm/lib"]


def build_host_probe():
    _run(["g++", "-std=c++17", "-O1", "-Wall", "-Werror", "-Wno-unknown-pragmas", "-I", INCLUDE, HOST_PROBE_SRC,
          "-o", HOST_PROBE] + _link_flags())
    return HOST_PROBE


def _hipcc_flags():
    from nextdoor_amd.build import HIPCC_FLAGS, find_hipcc
    return [find_hipcc()] + [f for f in HIPCC_FLAGS if f != "-shared"]


def build_template_probe():
    _run(_hipcc_flags() + ["-I", INCLUDE, TEMPLATE_PROBE_SRC, "-o", TEMPLATE_PROBE] + _link_flags())
    return TEMPLATE_PROBE


def build_user_apps():
    _run(_hipcc_flags() + ["-shared", USER_APPS_SRC, "-o", USER_APPS_LIB] + _link_flags())
    return USER_APPS_LIB


def build_all():
    return [build_host_probe(), build_template_probe(), build_user_apps()]


if __name__ == "__main__":
    for path in build_all():
        print(path)
