"""Weight container `orinfer-e8p-q4-v1` and package records (host side).  The container round trip
follows python/orinfer_build/quantization/e8p_q4.py:80-112; records follow the `Kernel` schema of
crates/orinfer-model-sdk/src/artifact.rs:87-110 and the naming rule of operators/rows.rs:14-58."""
import json
import subprocess

import numpy as np
import pytest

from oracle import reference as orc
from orinfer_amd import build, codebook, container, lib


def weights(rng, n=48, k=256):
    return container.Q4Weights(rng.integers(0, 2**32, (n, k // 8), dtype=np.uint32),
                               rng.uniform(0.005, 0.02, n).astype(np.float16),
                               rng.choice(np.array([-1, 1], np.int8), k))


def test_container_round_trip_and_contract_checks(tmp_path):
    from safetensors.numpy import save_file
    rng = np.random.default_rng(orc.SEED)
    w = weights(rng)
    container.save_q4(tmp_path / "w.safetensors", w)
    back = container.load_q4(tmp_path / "w.safetensors")
    for a, b in ((w.packed, back.packed), (w.scales, back.scales), (w.signs, back.signs)):
        np.testing.assert_array_equal(a, b)
    np.testing.assert_array_equal(back.k_major(), orc.q4_pack_k(w.packed, 128))
    good = dict(codec=container.CODEC, coefficients="4,1", layout=container.LAYOUT, rotation=container.ROTATION)
    tensors = dict(packed=w.packed, scales=w.scales, signs=w.signs, basis=codebook.basis())
    for key, value in (("codec", "orinfer-e8p-q4-v2"), ("coefficients", "7,2"), ("layout", "u32"), ("rotation", "none")):
        save_file(tensors, str(tmp_path / "bad.safetensors"), metadata=dict(good, **{key: value}))
        with pytest.raises(ValueError):
            container.load_q4(tmp_path / "bad.safetensors")
    wrong_basis = codebook.basis().copy()
    wrong_basis[0, 0] = 6
    save_file(dict(tensors, basis=wrong_basis), str(tmp_path / "bad.safetensors"), metadata=good)
    with pytest.raises(ValueError):
        container.load_q4(tmp_path / "bad.safetensors")
    save_file(dict(tensors, extra=w.signs), str(tmp_path / "bad.safetensors"), metadata=good)
    with pytest.raises(ValueError):
        container.load_q4(tmp_path / "bad.safetensors")
    for broken in (container.Q4Weights(w.packed.astype(np.int32), w.scales, w.signs),
                   container.Q4Weights(w.packed, w.scales[:-1], w.signs),
                   container.Q4Weights(w.packed, w.scales, np.zeros_like(w.signs)),
                   container.Q4Weights(w.packed[:, :5], w.scales, w.signs[:40])):
        with pytest.raises(ValueError):
            broken.validate()


def test_symbol_carries_its_variant():
    plain = lib.Kernel("e8p_q4_projection", M=4, N=9728, K=2560, dynamic_rows=True)
    packed = lib.Kernel(container.symbol_with_variant("e8p_q4_projection", M=4, N=9728, K=2560, dynamic_rows=True))
    assert packed.arg_names == plain.arg_names and packed.geometry(1) == plain.geometry(1)
    assert lib.Kernel("int8_projection?M=8192&N=4096&K=4096&output_dtype=float32").geometry() == \
        lib.Kernel("int8_projection", M=8192, N=4096, K=4096, output_dtype="float32").geometry()
    for bad in ("e8p_q4_projection?M=1&N", "e8p_q4_projection?=3", "nothing?M=1"):
        with pytest.raises(lib.OrxError):
            lib.Kernel(bad)
    with pytest.raises(lib.OrxError):
        lib.Kernel("e8p_q4_projection?M=1&N=128&K=128", M=1)


def test_kernel_records_follow_the_package_schema():
    program = container.projection_program("decoder.0.qkv", 7168, 5120, 8192)
    records, dynamic = program["kernels"], {d["name"]: d for d in program["dynamic"]}
    # the ranges partition 1..capacity (operators/rows.rs:14-58 parses MIN-MAX out of the name)
    bounds = [tuple(int(v) for v in r["name"].rsplit("/", 1)[1].split("-")) for r in records]
    assert bounds[0][0] == 1 and bounds[-1][1] == 8192
    assert all(a[1] + 1 == b[0] for a, b in zip(bounds, bounds[1:])) and all(lo <= hi for lo, hi in bounds)
    assert all(r["name"].startswith("decoder.0.qkv/rows/") for r in records)
    keys = {"name", "module", "source", "host_abi", "symbol", "grid", "block", "shared_memory_bytes", "cooperative", "args"}
    for record, (low, high) in zip(records, bounds):
        assert set(record) == keys and record["cooperative"] is False
        assert record["symbol"].startswith("e8p_q4_projection?M=")
        for identity in (record["module"], record["source"], record["host_abi"]):
            assert set(identity) == {"file", "sha256"} and len(identity["sha256"]) == 64
        assert [a.get("name", "m") for a in record["args"]] == ["A", "AS", "Book", "Out", "S", "W", "Workspace", "m"]
        assert record["args"][-1]["kind"] == "i32" and all(a["kind"] == "buffer" for a in record["args"][:-1])
        threads = record["block"][0] * record["block"][1] * record["block"][2]
        assert 0 < threads <= 1024 and all(g > 0 for g in record["grid"])   # artifact.rs validate_geometry
        # the record resolves; block and LDS bytes hold for EVERY row count of its range, and the grid is
        # the record's RowExpression of the rows: what DynamicBatchKernel::launch computes (dynamic.rs:93-118)
        # is a launch the library accepts, with no query of its own per launch
        kernel = lib.Kernel(record["symbol"])
        assert record["args"][-1]["value"] == high == kernel.variant.get("M", high)
        assert kernel.geometry(high) == (tuple(record["grid"]), tuple(record["block"]), record["shared_memory_bytes"])
        contract = dynamic.get(record["name"])
        assert (contract is None) == (low == high)
        for rows in sorted({low, high, (low + high) // 2, min(high, low + 1), max(low, high - 1)}):
            grid, block, shared = kernel.geometry(rows)
            assert (block, shared) == (tuple(record["block"]), record["shared_memory_bytes"])
            if contract is not None:
                assert tuple(container.evaluate_rows(e, rows) for e in contract["grid"]) == grid
        if contract is not None:
            assert contract["capacity"] == high and contract["arguments"] == [{"index": 7, "value": {"op": "rows"}}]
            assert [container.evaluate_rows(e, high) for e in contract["grid"]] == record["grid"]  # validate_binding
    assert len(records) <= 8
    with pytest.raises(ValueError):
        container.evaluate_rows({"op": "subtract", "lhs": {"op": "constant", "value": 1}, "rhs": {"op": "rows"}}, 2)
    plain = container.projection_records("decoder.0.o", 5120, 5120, 4, workspace=False)
    assert [a.get("name", "m") for a in plain[0]["args"]] == ["A", "AS", "Book", "Out", "S", "W", "m"]
    json.loads(container.dumps(records[0]))
    sliced = container.kernel_record("embed", "e8p_q4_embedding", dict(M=8, vocab=100, hidden=256),
                                     dict(Book="Book", IDs=("Tokens", 64), Output="Hidden", Scale="Scale", Signs="Signs",
                                          Weight="Bank", m=3), rows=3)
    assert sliced["args"][1] == {"kind": "buffer_slice", "name": "Tokens", "offset": 64}
    buffer = container.buffer_record("W", np.zeros((4, 8), np.uint32), layout="e8p-q4-k128-u32")
    assert buffer["dtype"] == "u32" and buffer["shape"] == [4, 8] and buffer["access"] == "read"


def test_every_emitted_argument_is_one_the_engine_deserialises():
    # crates/orinfer-model-sdk/src/artifact.rs:184-194: `Argument` is tagged by `kind`, denies unknown fields and knows
    # buffer, buffer_slice, i32, u32, i64, u64 and f32; a program's unused optional buffers are named in `omit`
    fields = {"buffer": {"kind", "name"}, "buffer_slice": {"kind", "name", "offset"}, "i32": {"kind", "value"},
              "u32": {"kind", "value"}, "i64": {"kind", "value"}, "u64": {"kind", "value"}, "f32": {"kind", "value"}}
    layer, _ = container.expert_layer_program("moe.0", 256, 128, 8, 2048, 512)
    exact, _ = container.exact_expert_program("moe.1", 4, 8, 2, 128, 256)
    dense = container.projection_program("decoder.0.o", 512, 512, 64)["kernels"]
    for record in [*layer, *exact, *dense]:
        for arg in record["args"]:
            assert arg["kind"] in fields and set(arg) == fields[arg["kind"]], (record["name"], arg)
        assert len(record["args"]) == len(lib.Kernel(record["symbol"]).arg_names)
    by_name = {r["name"]: r for r in layer}
    assert "omit=C" in by_name["moe.0.gate_up"]["symbol"] and "omit=AS,Q" in by_name["moe.0.down"]["symbol"]
    assert "omit=Shared,SharedGate" in by_name["moe.0.combine"]["symbol"]


def test_row_ranges_are_the_longest_the_geometry_allows():
    """One record per stretch of rows with one block size, one LDS size and one grid expression: the scalar Q4 slot of
    config 1's shape changes kernel at 2, 3, 65, 257 (whole tiles instead of split ones) and 512 rows, nowhere else."""
    program = container.projection_program("layer0.q", 17408, 5120, 1024, family="q4_projection")
    assert [k["name"].rsplit("/", 1)[1] for k in program["kernels"]] == ["1-1", "2-2", "3-64", "65-256", "257-511", "512-1024"]
    for entry in program["dynamic"]:
        low, high = (int(x) for x in entry["name"].rsplit("/", 1)[1].split("-"))
        kernel = lib.Kernel("q4_projection", M=high, N=17408, K=5120, dynamic_rows=True, workspace=True)
        for rows in {low, (low + high) // 2, high}:
            assert tuple(container.evaluate_rows(e, rows) for e in entry["grid"]) == kernel.geometry(rows)[0]


@pytest.mark.gpu
def test_container_to_records_to_fixture_run(tmp_path):
    """File -> container -> records -> launch through the fixture runner, checked against the oracle."""
    rng = np.random.default_rng(orc.SEED + 8)
    n, k, rows = 320, 640, 3
    w = weights(rng, n, k)
    container.save_q4(tmp_path / "layer.safetensors", w)
    loaded = container.load_q4(tmp_path / "layer.safetensors")
    x = rng.normal(size=(rows, k)).astype(np.float16)
    # the model rotates activations with the container's signs before A8
    a_q, a_s = orc.rotate_a8(x, loaded.signs)
    want = orc.project(a_q, a_s[:, 0], orc.q4_integers(loaded.packed, orc.basis()), loaded.scales, np.float32)
    want.tofile(tmp_path / "Out.f32")
    arrays = {"X": x, "Signs": loaded.signs, "Book": codebook.book(), "S": loaded.scales, "W": loaded.packed}
    buffers = []
    for name, array in arrays.items():
        np.ascontiguousarray(array).tofile(tmp_path / f"{name}.bin")
        buffers.append({"name": name, "file": f"{name}.bin", "bytes": int(np.asarray(array).nbytes)})
    buffers += [{"name": "A", "bytes": 4 * k, "fill": 0}, {"name": "AS", "bytes": 8, "fill": 0},
                {"name": "Out", "bytes": 4 * n * 2, "fill": 0}]
    rotate = container.kernel_record("layer.rotate/rows/1-4", "rotate_activation_a8", dict(M=4, K=k, dynamic_rows=True),
                                     dict(Q="A", S="AS", Signs="Signs", X="X", m=rows), rows=rows)
    project = [r for r in container.projection_records("layer.proj", n, k, 4, workspace=False,
                                                        bindings=dict(A="A", AS="AS", Book="Book", Out="Out", S="S", W="W"))
               if int(r["name"].rsplit("/", 1)[1].split("-")[0]) <= rows <= r["args"][-1]["value"]][0]
    project["args"][-1]["value"] = rows
    manifest = container.fixture_manifest(buffers, [rotate, project],
                                          dict(output="Out", output_dtype="f16", reference="Out.f32",
                                               relative_l2_tolerance=1e-3, zero_input="X", repetitions=5), rows=rows)
    (tmp_path / "manifest.json").write_text(json.dumps(manifest))
    done = subprocess.run([str(build.FIXTURE_RUNNER), str(tmp_path / "manifest.json")], capture_output=True, text=True,
                          timeout=120)
    report = json.loads(done.stdout.strip().splitlines()[-1])
    assert done.returncode == 0 and report["ok"] and report["relative_l2"] < 1e-3, (report, done.stderr)


@pytest.mark.gpu
def test_expert_layer_records_run_through_the_fixture_runner(tmp_path):
    """The five-launch expert layer as package records, resolved and launched by the C++ fixture runner
    (a separate process that knows only the C ABI): oracle output within the expert-FFN bar of
    flash_next_quantized.py:117-135, graph capture, poisoned-output, zero-input and restored replays."""
    from orinfer_amd import workloads
    c = workloads.config3(tokens=70, experts=16, top_k=4, hidden=768, intermediate=384)
    records, sizes = container.expert_layer_program("layer.moe", c["tokens"], c["experts"], c["top_k"], c["hidden"],
                                                    c["intermediate"], grouped_algorithm="resident")
    assert [r["name"].rsplit(".", 1)[1] for r in records] == ["router", "metadata", "gate_up", "down", "combine"]
    want = orc.moe_layer(c["x"], c["logits"], c["gate_up"], c["gate_up_scales"], c["down"], c["down_scales"], orc.basis(),
                         c["top_k"], 32)["out"].astype(np.float32)
    want.tofile(tmp_path / "Output.f32")
    data = {"X": c["x"], "Logits": c["logits"], "Book": codebook.book(),
            "GateUpCodes": codebook.q2_to_k_major(np.asarray(c["gate_up"])), "GateUpScales": c["gate_up_scales"],
            "DownCodes": codebook.q2_to_k_major(np.asarray(c["down"])), "DownScales": c["down_scales"]}
    buffers = []
    for name, size in sizes.items():
        if name in data:
            array = np.ascontiguousarray(data[name])
            assert array.nbytes == size, name
            array.tofile(tmp_path / f"{name}.bin")
            buffers.append({"name": name, "file": f"{name}.bin", "bytes": size})
        else:
            buffers.append({"name": name, "bytes": size, "fill": 0})
    manifest = container.fixture_manifest(buffers, records,
                                          dict(output="Output", output_dtype="f16", reference="Output.f32",
                                               relative_l2_tolerance=3e-3, zero_input="X", repetitions=5))
    (tmp_path / "manifest.json").write_text(json.dumps(manifest))
    done = subprocess.run([str(build.FIXTURE_RUNNER), str(tmp_path / "manifest.json")], capture_output=True, text=True,
                          timeout=120)
    report = json.loads(done.stdout.strip().splitlines()[-1])
    assert done.returncode == 0 and report["ok"] and report["relative_l2"] < 3e-3, (report, done.stderr)


@pytest.mark.gpu
def test_exact_expert_records_run_through_the_fixture_runner(tmp_path):
    """The reference's decode pairing on nibble planes (split_a8 -> e8p_exact_grouped, 8-row tiles) as package records,
    resolved and launched by the C++ fixture runner: the oracle's output exactly, graph capture and the replays."""
    rng = np.random.default_rng(orc.SEED + 31)
    rows, experts, top_k, n, k, bm = 9, 8, 4, 320, 640, 8
    slots = rows * top_k
    ids = np.stack([rng.choice(experts, top_k, replace=False) for _ in range(rows)]).astype(np.int32)
    counts, _ = orc.expert_histogram(ids, experts)
    offsets, tile_offsets, total = orc.expert_offsets(counts, bm)
    records, sizes = container.exact_expert_program("flash_decode.layer0.post", rows, experts, top_k, n, k, block_m=bm)
    tiles = sizes["TE"] // 4
    te, tr = orc.expert_tiles(counts, tile_offsets, bm, tiles)
    a = rng.integers(-128, 128, (slots, k), dtype=np.int8)
    scale = rng.uniform(0.01, 0.03, slots).astype(np.float16)
    codes = rng.integers(0, 65536, (experts, n, k // 8), dtype=np.uint16)
    ws = rng.uniform(0.005, 0.02, (experts, n)).astype(np.float16)
    weights = np.stack([orc.q2_integers(c, orc.basis()) for c in codes])
    want = orc.grouped_project(a, scale[:, None], weights, ws, counts, offsets).astype(np.float32)
    want.tofile(tmp_path / "Out.f32")
    data = {"A": a, "AS": scale, "Book": codebook.nibble_book(), "Counts": counts, "Offsets": offsets, "TC": total, "TE": te,
            "TR": tr, "P": codebook.q2_to_k64(codebook.q2_to_k_major(codes)), "WS": ws}
    buffers = []
    for name, size in sizes.items():
        if name in data:
            array = np.ascontiguousarray(data[name])
            assert array.nbytes == size, name
            array.tofile(tmp_path / f"{name}.bin")
            buffers.append({"name": name, "file": f"{name}.bin", "bytes": size})
        else:
            buffers.append({"name": name, "bytes": size, "fill": 0})
    manifest = container.fixture_manifest(buffers, records,
                                          dict(output="Out", output_dtype="f16", reference="Out.f32",
                                               relative_l2_tolerance=1e-7, zero_input="A", repetitions=5))
    (tmp_path / "manifest.json").write_text(json.dumps(manifest))
    done = subprocess.run([str(build.FIXTURE_RUNNER), str(tmp_path / "manifest.json")], capture_output=True, text=True,
                          timeout=120)
    report = json.loads(done.stdout.strip().splitlines()[-1])
    assert done.returncode == 0 and report["ok"] and report["relative_l2"] == 0, (report, done.stderr)
