"""The `traffic` figures bench.py attaches to its kernel rows are constants read
off rocprofv3 counter runs; the summaries of those runs are kept under
profiles/. The two must say the same, or the benchmark line would quote
traffic nobody measured."""

import ast
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def bench_table():
    tree = ast.parse(open(os.path.join(ROOT, "bench.py")).read())
    for node in tree.body:
        if isinstance(node, ast.Assign) and getattr(node.targets[0], "id", "") == "MEASURED_TRAFFIC":
            return ast.literal_eval(node.value)
    raise AssertionError("bench.py has no MEASURED_TRAFFIC")


def profile_table():
    rows = {}
    for line in open(os.path.join(ROOT, "profiles", "bench_kernels_hbm_traffic.md")):
        cells = [c.strip() for c in line.strip().strip("|").split("|")]
        if len(cells) == 7 and re.fullmatch(r"[\d,]+", cells[4]):
            rows[cells[0]] = (int(cells[4].replace(",", "")), float(cells[2]), float(cells[3]))
    return rows


def test_bench_traffic_constants_equal_the_profile_summary():
    bench, prof = bench_table(), profile_table()
    assert len(prof) >= 20
    assert set(bench) == set(prof), sorted(set(bench) ^ set(prof))
    for name, nbytes in bench.items():
        traffic, fetch_kib, write_kib = prof[name]
        assert nbytes == traffic, name
        # and the summary's own arithmetic: FETCH_SIZE x 2 + WRITE_SIZE x 1, in KiB
        assert abs((2.0 * fetch_kib + write_kib) * 1024 - traffic) <= 1024, name
