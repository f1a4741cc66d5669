"""Host-side behaviour of bench.py that needs no GPU: the one-GPU rule, the legs that report beside the headline, and
the tie between the HBM traffic table and the kernel sources."""
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

import bench  # noqa: E402


def test_more_than_one_gpu_is_refused_with_a_message():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert proc.returncode == 2 and "ONE GPU" in proc.stderr and not proc.stdout.strip()


def test_a_side_leg_that_fails_is_reported_in_its_place(capsys):
    def dies():
        raise SystemExit("bench: child failed:\nline one\nline two")

    def hangs():
        raise subprocess.TimeoutExpired(["megray_performance"], 600)

    assert bench.side_leg(lambda: {"ok": 1}) == {"ok": 1}
    assert bench.side_leg(dies) == {"error": "bench: child failed: line one line two"}
    assert "timed out" in bench.side_leg(hangs)["error"]
    assert "dies failed" in capsys.readouterr().err


def test_the_traffic_table_names_the_kernel_sources_it_was_measured_on():
    table = json.load(open(os.path.join(ROOT, "profiles", "hbm_traffic.json")))
    for name in table["kernel_sources"]:
        assert os.path.exists(os.path.join(ROOT, "megray_amd", "csrc", name))
    assert len(bench.kernel_source_hash()) == len(table["kernel_source_hash"])
