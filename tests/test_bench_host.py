"""Host-side checks of bench.py that need no GPU: the counter summaries under profiles/ that it reads are well formed,
the figures derived from them follow the stated formulas, and the one-GPU contract is enforced."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def bench():
    sys.path.insert(0, ROOT)
    import bench
    return bench


@pytest.mark.parametrize("name,keys", [
    ("search_kernel_c4_acp_prodigal_4x256_counters.md", ["commit", "calibration", "traffic_bytes_per_launch", "sq_insts_valu_per_root", "batched_64_roots", "trees_512"]),
    ("search_kernel_solo_c4_768_searches.md", ["commit", "searches", "sq_insts_valu_per_pass", "traffic_bytes_per_launch"]),
    ("search_kernel_gomoku_ocp_thrifty_4x128_counters.md", ["commit", "sq_insts_valu_per_root", "batched_32_roots", "traffic_bytes_per_launch"]),
    ("search_kernel_puct_gomoku_16_trees_x16.md", ["commit", "sq_insts_valu_per_launch", "traffic_bytes_per_launch"]),
    ("select_kernel_puct_eq256_d1024.md", ["commit", "traffic_bytes_per_launch"]),
])
def test_counter_summaries_carry_what_bench_reads(bench, name, keys):
    prof = bench.profile_json(name)
    assert prof is not None, f"profiles/{name} has no json block"
    for k in keys:
        assert k in prof, (name, k)
    assert prof["file"] == "profiles/" + name
    text = open(os.path.join(ROOT, "profiles", name)).read()
    assert "rocprofv3" in text and "bench.py" in text            # the command that made it, on committed files
    cal = prof.get("calibration") or {}
    if "fetch_reading" in cal:                                   # the factors follow from the copy readings in the same file
        assert abs(cal["fetch_factor"] - cal["copy_KiB"] / cal["fetch_reading"]) < 1e-9
        assert abs(cal["write_factor"] - cal["copy_KiB"] / cal["write_reading"]) < 1e-9


def test_per_root_instruction_counts_cover_the_workload(bench):
    prof = bench.profile_json("search_kernel_c4_acp_prodigal_4x256_counters.md")
    assert len(prof["sq_insts_valu_per_root"]) == bench.N_ROOTS == len(bench.make_roots(bench.N_ROOTS))
    expected = (prof["fetch_KiB_per_launch"] * prof["calibration"]["fetch_factor"] + prof["write_KiB_per_launch"] * prof["calibration"]["write_factor"]) * 1024
    assert abs(prof["traffic_bytes_per_launch"] - expected) < 2


def test_valu_roofline_formula(bench):
    r = bench.valu_roofline(614.4e9 * 0.5, 1.0, {"file": "f", "commit": "c"}, "x")
    assert abs(r["frac"] - 0.5) < 1e-12 and r["peak"] == 614.4 and r["bound"] == "valu"
    assert bench.valu_roofline(None, 1.0, {}, "x") is None
    assert bench.profile_json("no_such_summary.md") is None


def test_algorithmic_bytes_of_one_known_step(bench):
    """One tree-step that walks 2 levels over 7 + 3 children, creates 7 children and plays all of them out."""
    class R:
        stat_levels, stat_children, stat_expanded, stat_played = 2, 10, 7, 7
    b = bench.algorithmic_bytes(R, 1)
    assert b["select"] == 2 * (1 + 4 + 28) + 80 + 5 + 4 * 3
    assert b["expand"] == (49 + 6 + 28 + 18) + 7 * (49 + 18)
    assert b["playout"] == 7 * (49 + 2 + 32 * 256 + 8)
    assert b["backup"] == 7 * 29 + 3 * 21
    assert b["total"] == b["select"] + b["expand"] + b["playout"] + b["backup"]


def test_more_than_one_gpu_is_refused_with_a_message():
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert res.returncode != 0 and "one GPU" in (res.stderr + res.stdout)
