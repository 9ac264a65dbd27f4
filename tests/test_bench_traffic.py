"""bench.py's traffic figures are rows of the committed counter summary: the constants in bench.py against the table in
profiles/gemm_f16_4096_and_transpose_f32_16384_counters.txt, the calibration factor against the plain copy's row, and the
bytes bench.py derives from them."""
import os
import re
import sys

ROOT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..")
sys.path.insert(0, ROOT)
import bench  # noqa: E402

PROFILE = os.path.join(ROOT, "profiles", "gemm_f16_4096_and_transpose_f32_16384_counters.txt")


def table_rows():
    rows, inside = {}, False
    with open(PROFILE) as f:
        for line in f:
            if line.startswith("kernel") and "FETCH_SIZE" in line and "WRITE_SIZE" in line and "dispatches" in line:
                inside = True
                continue
            if inside:
                m = re.match(r"^(\S.*?\S)\s{2,}(\d+)\s+([\d.]+)\s+([\d.]+)\s*$", line)
                if not m:
                    break
                rows[m.group(1)] = (int(m.group(2)), float(m.group(3)), float(m.group(4)))
    return rows


def test_the_profile_has_the_table():
    rows = table_rows()
    assert len(rows) >= 8 and "copy_flat_b128" in rows and all(n > 0 for n, _, _ in rows.values())


def test_every_constant_is_a_row_of_the_profile():
    rows = table_rows()
    for key, (kernel, fetch_kib, write_kib) in bench.MEASURED_TRAFFIC.items():
        assert kernel in rows, (key, kernel)
        assert rows[kernel][1:] == (fetch_kib, write_kib), (key, rows[kernel], fetch_kib, write_kib)
    name, fetch_kib, write_kib = bench.TRAFFIC_CALIBRATION
    assert rows[name][1:] == (fetch_kib, write_kib)


def test_the_scale_is_what_the_plain_copy_shows():
    _, fetch_kib, write_kib = bench.TRAFFIC_CALIBRATION
    gib = 1048576.0
    assert abs(gib / fetch_kib - bench.FETCH_SCALE) < 1e-3 * bench.FETCH_SCALE      # FETCH_SIZE reads half of what the copy moved
    assert abs(write_kib / gib - 1.0) < 2e-3                                         # WRITE_SIZE reads true


def test_traffic_bytes_and_the_source_string():
    for key, (_, fetch_kib, write_kib) in bench.MEASURED_TRAFFIC.items():
        want = fetch_kib * bench.FETCH_SCALE * 1024 + write_kib * 1024
        assert abs(bench.traffic_bytes(key) - want) <= 1.0
    assert os.path.basename(PROFILE) in bench.TRAFFIC_SOURCE
    # the transpose moves its 2 GiB once; the headline GEMM fetches its operands three times (eight private L2s)
    assert abs(bench.traffic_bytes("transpose_f32_16384") / 2.0 ** 31 - 1.0) < 2e-3
    assert 2.9 < (bench.MEASURED_TRAFFIC["gemm_f16_4096_tile256"][1] * bench.FETCH_SCALE) / 65536.0 < 3.1
