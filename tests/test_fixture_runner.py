"""The C++ fixture runner drives liborx the way the engine's `run-artifact` harness drives a kernel
package (crates/orinfer-engine/src/backend/cuda/mod.rs:359-720): upload, launch, relative L2 against
an fp32 reference, graph capture, poisoned-output replay, zero-input replay, restored replay, timed
replays.  The references written here come from the oracle."""
import json
import subprocess
from pathlib import Path

import numpy as np
import pytest

from oracle import reference as orc
from orinfer_amd import build, codebook, lib

RUNNER = build.FIXTURE_RUNNER


def runner():
    if not RUNNER.exists():
        build.build(verbose=False)
    return str(RUNNER)


def run_manifest(directory, manifest):
    path = Path(directory) / "manifest.json"
    path.write_text(json.dumps(manifest))
    done = subprocess.run([runner(), str(path)], capture_output=True, text=True, timeout=120)
    report = json.loads(done.stdout.strip().splitlines()[-1])
    return done.returncode, report, done.stderr


def put(directory, name, array):
    array = np.ascontiguousarray(array)
    array.tofile(Path(directory) / f"{name}.bin")
    return {"name": name, "file": f"{name}.bin", "bytes": array.nbytes}


def test_runner_reports_usage_and_bad_manifests(tmp_path):
    done = subprocess.run([runner()], capture_output=True, text=True)
    assert done.returncode == 2 and "usage" in done.stderr
    (tmp_path / "manifest.json").write_text("{not json")
    done = subprocess.run([runner(), str(tmp_path / "manifest.json")], capture_output=True, text=True)
    assert done.returncode == 3
    assert json.loads(done.stdout.strip())["ok"] is False


@pytest.mark.gpu
@pytest.mark.parametrize("rows,capacity,algorithm", [(1, 1, "gemv"), (5, 64, "auto"), (130, 256, "auto"), (300, 512, "auto")])
def test_q4_projection_fixture(tmp_path, rows, capacity, algorithm):
    rng = np.random.default_rng(orc.SEED + rows)
    n, k = 320, 512
    x = rng.normal(size=(capacity, k)).astype(np.float16)
    a_q, a_s = orc.a8(x)
    packed = rng.integers(0, 2**32, (n, k // 8), dtype=np.uint32)
    scales = rng.uniform(0.005, 0.02, n).astype(np.float16)
    want = orc.project(a_q[:rows], a_s[:rows, 0], orc.q4_integers(packed, orc.basis()), scales, np.float32)
    want.astype(np.float32).tofile(tmp_path / "Out.f32")
    variant = {"M": capacity, "N": n, "K": k, "algorithm": algorithm}
    args = [{"buffer": "A"}, {"buffer": "AS"}, {"buffer": "Book"}, {"buffer": "Out"}, {"buffer": "S"}, {"buffer": "W"}]
    record = {"symbol": "e8p_q4_projection", "variant": variant, "args": args}
    if capacity != rows:
        variant["dynamic_rows"] = True
        args.append({"i32": rows})
        record["rows"] = rows
    manifest = {
        "schema_version": 1, "target": "gfx950",
        "buffers": [put(tmp_path, "A", a_q), put(tmp_path, "AS", a_s[:, 0].copy()), put(tmp_path, "Book", codebook.book()),
                    put(tmp_path, "S", scales), put(tmp_path, "W", packed),
                    {"name": "Out", "bytes": capacity * n * 2, "fill": 0}],
        "kernels": [record],
        "validation": {"output": "Out", "output_dtype": "f16", "reference": "Out.f32", "relative_l2_tolerance": 1e-3,
                       "zero_input": "A", "repetitions": 10},
    }
    code, report, err = run_manifest(tmp_path, manifest)
    assert code == 0 and report["ok"], (report, err)
    assert report["relative_l2"] < 1e-3 and report["graph_replay_identical"] and report["zero_input_gives_zero"]
    assert report["restored_input_identical"] and report["output_bytes_written"] > 0


@pytest.mark.gpu
def test_two_record_program_and_rejected_record(tmp_path):
    """A8 quantisation feeding a W8A8 projection: two kernel records in one fixture, zeroing the
    fp16 input zeroes the final output.  A record with a wrong grid is refused before anything runs."""
    rng = np.random.default_rng(orc.SEED + 4)
    m, n, k = 48, 192, 384
    x = rng.normal(size=(m, k)).astype(np.float16)
    weight = rng.integers(-127, 128, (n, k), dtype=np.int8)
    ws = rng.uniform(0.001, 0.01, n).astype(np.float16)
    a_q, a_s = orc.a8(x)
    want = orc.project(a_q, a_s[:, 0], weight, ws, np.float32)
    want.tofile(tmp_path / "Out.f32")
    buffers = [put(tmp_path, "X", x), put(tmp_path, "Weight", weight), put(tmp_path, "WS", ws),
               {"name": "Q", "bytes": m * k, "fill": 0}, {"name": "S", "bytes": m * 2, "fill": 0},
               {"name": "Out", "bytes": m * n * 2, "fill": 0}]
    quant = {"symbol": "activation_quantization", "variant": {"K": k, "M": m, "omit": "Mask"},  # no mask: out of the list
             "args": [{"buffer": "Q"}, {"buffer": "S"}, {"buffer": "X"}, {"i32": m}], "rows": m}
    project = {"symbol": "int8_projection", "variant": {"M": m, "N": n, "K": k},
               "args": [{"buffer": "Q"}, {"buffer": "Out"}, {"buffer": "S"}, {"buffer": "Weight"}, {"buffer": "WS"}]}
    validation = {"output": "Out", "output_dtype": "f16", "reference": "Out.f32", "relative_l2_tolerance": 1e-3,
                  "zero_input": "X", "repetitions": 5}
    manifest = {"schema_version": 1, "buffers": buffers, "kernels": [quant, project], "validation": validation}
    code, report, err = run_manifest(tmp_path, manifest)
    assert code == 0 and report["ok"] and report["kernels"] == 2, (report, err)
    bad = dict(project, grid=[3, 1, 1], block=[256, 1, 1], shared=0)
    manifest["kernels"] = [quant, bad]
    code, report, err = run_manifest(tmp_path, manifest)
    assert code == 3 and not report["ok"] and str(lib.ORX_ERR_BAD_GEOMETRY) in report["error"]
