"""Host-side logic of bench.py that needs no GPU: the HBM-traffic table behind roofline.traffic, the
workload registry, and the refusal of more than one GPU."""
import os
import re
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

import bench  # noqa: E402

# entry points of the five configurations and the bytes (cfg1-4) their kernels must at least move
EXPECTED = {
    ("cfg1", "dw_updateOutput"): 2 * 32 * 32 * 112 * 112 * 4,
    ("cfg2", "dw_updateOutput"): 64 * 128 * (56 * 56 + 28 * 28) * 4,
    ("cfg2", "dw_updateGradInput"): 64 * 128 * (56 * 56 + 28 * 28) * 4,
    ("cfg2", "dw_accGradParameters"): 64 * 128 * (56 * 56 + 28 * 28) * 4,
    ("cfg3", "bn_updateOutput"): 2 * 64 * 256 * 28 * 28 * 4,
    ("cfg3", "bn_backward"): 3 * 64 * 256 * 28 * 28 * 4,
    ("cfg4", "maxpool_updateOutput"): 64 * 64 * (112 * 112 + 3 * 56 * 56) * 4,
    ("cfg4", "maxpool_updateGradInput"): 64 * 64 * (112 * 112 + 3 * 56 * 56) * 4,
    ("cfg4", "avgpool_updateOutput"): 64 * 64 * (112 * 112 + 56 * 56) * 4,
    ("cfg4", "avgpool_updateGradInput"): 64 * 64 * (112 * 112 + 56 * 56) * 4,
    ("cfg5", "convmm_updateOutput"): None,
    ("cfg5", "convmm_updateGradInput"): None,
    ("cfg5", "convmm_accGradParameters"): None,
}


def test_traffic_table_rows_name_existing_summaries_and_commits():
    table = bench.load_traffic()
    assert set(EXPECTED) <= set(table)
    for key, row in table.items():
        assert os.path.exists(os.path.join(ROOT, "profiles", row["source"])), (key, row["source"])
        assert re.fullmatch(r"[0-9a-f]{7,40}", row["commit"]), (key, row["commit"])
        assert row["bytes"] > 0


def test_traffic_of_the_streaming_kernels_is_close_to_their_algorithmic_bytes():
    """Counters within -1 % ... +10 % of what the kernel has to move: a stale or mis-scaled row would not be."""
    table = bench.load_traffic()
    for key, algorithmic in EXPECTED.items():
        if algorithmic is None:
            continue
        ratio = table[key]["bytes"] / algorithmic
        assert 0.99 < ratio < 1.10, (key, ratio)


def test_traffic_table_parser_sums_the_kernels_of_an_entry_point(tmp_path):
    p = tmp_path / "t.txt"
    p.write_text("# comment\n"
                 "w e k1 100.0 50.0 s.txt abc1234\n"
                 "w e k2 1.5 2.0 s.txt abc1234   # trailing comment\n"
                 "malformed row\n")
    t = bench.load_traffic(str(p))
    assert list(t) == [("w", "e")]
    assert t[("w", "e")]["bytes"] == int((100.0 * 2 + 50.0) * 1024) + int((1.5 * 2 + 2.0) * 1024)
    assert bench.load_traffic(str(tmp_path / "missing.txt")) == {}


def test_workload_registry_holds_the_five_configurations_and_the_block():
    for name in ("cfg1", "cfg2", "cfg3", "cfg4", "cfg5", "mbv1_block", "copy"):
        assert name in bench.WORKLOADS


def test_more_than_one_gpu_is_refused_before_anything_touches_a_gpu():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode == 2
    assert "one GPU" in r.stderr and r.stdout.strip() == ""
