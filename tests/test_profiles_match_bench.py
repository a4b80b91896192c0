"""bench.py quotes figures that rocprofv3 counter runs recorded (its MEASURED table); the summaries
of those runs are the tables under profiles/.  The two must say the same: every constant is looked
up in its table and compared to the table's four significant digits."""
import os
import re

import pytest

import bench

PROFILES = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "profiles")


def table_rows(path):
    """kernel name (up to its template arguments) -> cells of its row, from the first table of the file."""
    rows = {}
    for line in open(path):
        if not line.startswith("| ") or line.startswith("| kernel") or line.startswith("|---"):
            continue
        cells = [c.strip() for c in line.strip().strip("|").split("|")]
        rows.setdefault(cells[0].split("<")[0], cells)
    return rows


def close(a, b):
    return abs(a - b) <= 2e-3 * abs(b)


@pytest.mark.parametrize("profile", sorted(bench.MEASURED))
def test_recorded_traffic_is_what_the_summary_says(profile):
    m = bench.MEASURED[profile]
    path = os.path.join(PROFILES, f"step_kernels_{profile}_hbm_traffic.md")
    rows = table_rows(path)
    header = [c.strip() for c in next(l for l in open(path) if l.startswith("| kernel")).strip().strip("|").split("|")]
    column = header.index("HBM bytes/dispatch (scaled)")
    for kernel, value in m["kernels"].items():
        assert kernel in rows, f"{kernel} has no row in {path}"
        assert close(value, float(rows[kernel][column])), (kernel, value, rows[kernel][column])
    per_pass = re.search(r"([0-9.]+) GB per pass", open(path).read())
    assert per_pass and close(m["bytes_per_pass"], float(per_pass.group(1)) * 1e9)
    # the command the summary gives runs this repository's bench.py on the profile's workload
    text = open(path).read()
    workload = profile.replace("_period0", "")
    assert f"python3 bench.py --workload {workload} " in text
    assert ("--inversion-period 0" in text) == profile.endswith("_period0")


@pytest.mark.parametrize("profile", sorted(p for p, m in bench.MEASURED.items() if "read_requests" in m))
def test_recorded_requests_are_what_the_summary_says(profile):
    m = bench.MEASURED[profile]
    path = os.path.join(PROFILES, f"step_kernels_{profile}_l2_requests.md")
    rows = table_rows(path)
    header = [c.strip() for c in next(l for l in open(path) if l.startswith("| kernel")).strip().strip("|").split("|")]
    reads, writes = header.index("RDREQ"), header.index("WRREQ (write requests to memory)")
    for kernel, value in m["read_requests"].items():
        assert close(value, float(rows[kernel][reads])), (kernel, value, rows[kernel][reads])
        # nearly all of them are 128-byte requests, which is what bench.py prices them as
        assert float(rows[kernel][header.index("of them 128 B")]) >= 0.999 * float(rows[kernel][reads])
    for kernel, value in m["write_requests"].items():
        assert close(value, float(rows[kernel][writes])), (kernel, value, rows[kernel][writes])


def test_derived_tables_follow_the_recorded_ones():
    khop = bench.MEASURED["khop_rmat21"]["kernels"]
    assert bench.MEASURED_TRAFFIC_BYTES_PER_LAUNCH["khop_rmat21"] == \
        (2 * khop["nd::step_flat_kernel"] + khop["nd::step_workgroup_kernel"]) / 2
    assert set(bench.MEASURED_TRAFFIC_BYTES_PER_PASS) == set(bench.MEASURED)
    for name in bench.FIVE_CONFIGS:
        assert name in bench.MEASURED


def test_every_profile_summary_names_its_command():
    for name in sorted(os.listdir(PROFILES)):
        text = open(os.path.join(PROFILES, name)).read()
        assert "rocprofv3 " in text or "python -c" in text, name
        assert "_work/" not in text, name  # commands run committed files only
