"""Host logic of bench.py that needs no GPU: the traffic figure comes from the committed counter
summary and is withheld when that summary was taken on another launch."""
import subprocess
import sys
from pathlib import Path

import bench

ROOT = Path(__file__).resolve().parents[1]


def test_traffic_comes_from_the_counter_summary_and_only_for_the_launch_it_was_taken_on():
    text = bench.TRAFFIC_SUMMARY.read_text()
    line = next(l for l in text.splitlines() if l.startswith("bench-traffic:"))
    fields = dict(item.strip().split("=", 1) for item in line[len("bench-traffic:"):].split(";"))
    launch = ((int(fields["grid"]), 1, 1), (int(fields["block"]), 1, 1), int(fields["lds"]))
    traffic, kernel = bench.measured_traffic(launch)
    assert kernel == fields["kernel"] and kernel in text
    # the figure is the calibrated sum the summary states in words
    stated = next(l for l in text.splitlines() if "traffic =" in l)
    assert int(stated.split("=")[1].split("bytes")[0].replace(" ", "")) == traffic
    # config 1, one row: every code once plus row, scales, table and output; counters may not fall below that
    algorithmic = 17408 * 5120 // 2
    assert algorithmic <= traffic <= 1.1 * algorithmic
    other = (launch[0], launch[1], launch[2] + 16)
    assert bench.measured_traffic(other) == (None, None)


def test_more_than_one_gpu_is_refused_with_a_message():
    run = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert run.returncode != 0 and "one GPU" in (run.stdout + run.stderr)
