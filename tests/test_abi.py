"""CPU checks of the C-ABI library and of the host-side helpers: every symbol declared in
include/orx.h is exported, resolve / geometry / argument order / error codes behave like the
engine's catalog (crates/orinfer-engine/src/backend/cuda/kernels.rs:47-61,114-192), and the
package-side codebook and workload generators agree with the oracle.  Nothing here computes on a
device."""
import ctypes
import json
import re
from pathlib import Path

import numpy as np
import pytest

from oracle import reference as ref
from orinfer_amd import codebook, lib, workloads

ROOT = Path(__file__).resolve().parent.parent


def declared_symbols():
    text = (ROOT / "include" / "orx.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(orx_[a-z_]+)\s*\(", text)))


def test_header_symbols_are_exported():
    names = declared_symbols()
    assert len(names) == len(lib.EXPORTS) and set(names) == set(lib.EXPORTS)
    raw = ctypes.CDLL(str(lib.LIBRARY_PATH))
    for name in names:
        assert getattr(raw, name) is not None, name


def test_catalog_lists_every_symbol_and_resolves():
    catalog = lib.catalog()["kernels"]
    symbols = [entry["symbol"] for entry in catalog]
    assert len(symbols) == len(set(symbols))
    for needed in ("activation_quantization", "swiglu", "rotate_activation_a8", "residual_norm_rotate_a8", "e8p_q4_projection",
                   "int8_projection",
                   "e8p_decode_grouped", "integer_vq_grouped", "integer_e8p_gemv", "e8p_q4_unpack", "e8p_q2_unpack", "router_topk",
                   "expert_histogram", "expert_offsets", "expert_tiles", "expert_dispatch", "moe_combine"):
        assert needed in symbols


ABI = {
    # symbol, variant -> expected argument order (buffers in ASCII order, scalars, m last)
    ("activation_quantization", (("K", 2560),)): ["Mask", "Q", "S", "X", "rows"],
    ("swiglu", (("I", 512),)): ["X", "Y", "rows"],
    ("rotate_activation_a8", (("M", 8), ("K", 5120))): ["Q", "S", "Signs", "X"],
    ("residual_norm_rotate_a8", (("M", 8),)): ["Q", "R", "RO", "S", "Signs", "W", "X", "Y"],
    ("residual_norm_rotate_a8", (("M", 4096), ("K", 2560), ("dynamic_rows", True), ("zero_centered", False))):
        ["Q", "R", "RO", "S", "Signs", "W", "X", "Y", "m"],
    ("e8p_q4_embedding", (("M", 8), ("vocab", 1000), ("hidden", 5120))): ["Book", "IDs", "Output", "Scale", "Signs", "Weight", "m"],
    ("rotate_activation_a8", (("M", 8), ("K", 256), ("swiglu", True), ("dynamic_rows", True))): ["Q", "S", "Signs", "X", "m"],
    ("e8p_q4_projection", (("M", 1), ("N", 9728), ("K", 2560))): ["A", "AS", "Book", "Out", "S", "W"],
    ("e8p_q4_projection", (("M", 1), ("N", 9728), ("K", 2560), ("input_dtype", "float16"), ("rotate", True))):
        ["A", "AS", "Book", "Out", "S", "Signs", "W"],
    ("e8p_q4_projection", (("M", 64), ("N", 256), ("K", 256), ("dynamic_rows", True))):
        ["A", "AS", "Book", "Out", "S", "W", "m"],
    ("int8_projection", (("M", 8192), ("N", 4096), ("K", 4096))):
        ["A", "Output", "TokenScale", "Weight", "WeightScale"],
    ("int8_swiglu", (("M", 32), ("N", 512), ("K", 2048), ("dynamic_rows", True))):
        ["A", "Gate", "GateScale", "Output", "TokenScale", "Up", "UpScale", "m"],
    ("e8p_decode_grouped", (("rows", 640), ("E", 512), ("tiles", 552), ("N", 1024), ("K", 2048))):
        ["A", "AS", "Book", "C", "Counts", "Offsets", "P", "TileCount", "TileExpert", "TileRow", "WS"],
    ("integer_e8p_gemv", (("E", 128), ("routes", 8), ("N", 1024), ("K", 2048), ("shared_input", True))):
        ["A", "AS", "Book", "C", "IDs", "P", "WS"],
    ("single_route_metadata", ()): ["Counts", "IDs", "Offsets", "Relative", "TileCount", "TileExpert", "TileOffsets", "TileRow"],
    ("expert_partition_offsets", (("experts", 128), ("hot_m", 32), ("cold_m", 8), ("cold_rows", 8))):
        ["ColdCount", "ColdOffsets", "Counts", "RowOffsets", "TileCount", "TileOffsets"],
    ("expert_partition_tiles", (("M", 64), ("experts", 128), ("top_k", 8), ("hot_m", 32), ("cold_m", 8), ("cold_rows", 8),
                                ("dynamic_rows", True))):
        ["ColdExpert", "ColdOffsets", "ColdRow", "Counts", "TileExpert", "TileOffsets", "TileRow", "m"],
    ("integer_experts", (("M", 64), ("N", 1024), ("K", 2048), ("E", 128), ("top_k", 8), ("dynamic_rows", True))):
        ["A", "AS", "Book", "Counts", "Offsets", "Out", "TileCount", "TileExpert", "TileRow", "W", "WS", "m"],
    ("integer_experts", (("M", 64), ("N", 1024), ("K", 2048), ("E", 128), ("top_k", 8), ("codec", "w8"))):
        ["A", "AS", "Book", "Counts", "Offsets", "Out", "TileCount", "TileExpert", "TileRow", "W", "WS"],
    ("router_topk_warp", (("M", 64), ("E", 128), ("top_k", 8), ("dynamic_rows", True))): ["IDs", "Logits", "Prob", "m"],
    ("rotate_activation", (("M", 8), ("K", 5120), ("swiglu", True))): ["Signs", "X", "Y"],
    ("int8_small_projection", (("M", 4), ("N", 4096), ("K", 4096), ("dynamic_rows", True))):
        ["A", "Output", "TokenScale", "Weight", "WeightScale", "m"],
    ("router_topk", (("M", 64), ("dynamic_rows", True))): ["IDs", "Logits", "Prob", "m"],
    ("expert_histogram", (("M", 64),)): ["Counts", "IDs", "RelativeSlot"],
    ("expert_offsets", ()): ["Counts", "RowOffsets", "TileCount", "TileOffsets"],
    ("expert_tiles", (("M", 64),)): ["Counts", "TileExpert", "TileOffsets", "TileRow"],
    ("route_metadata", (("M", 64), ("E", 128), ("top_k", 8), ("block_m", 32), ("dynamic_rows", True))):
        ["Counts", "IDs", "RelativeSlot", "RowOffsets", "TileCount", "TileExpert", "TileOffsets", "TileRow", "m"],
    ("expert_dispatch", (("M", 64), ("H", 2048))):
        ["A", "D", "DS", "IDs", "RelativeSlot", "RowOffsets", "Scale", "SlotMap"],
    ("moe_combine", (("M", 64), ("H", 2048), ("dynamic_rows", True))):
        ["Expert", "Output", "Prob", "Shared", "SharedGate", "SlotMap", "m"],
    # the nibble-plane family: crates/orinfer-models/src/flash_next/experts.rs:207-215 binds the exact kernel as
    # AS, Book, Counts, High, Low, Offsets, Out, P, Sum, TC, TE, TR, WS and the split as A, High, Low, Sum
    ("split_a8", (("rows", 64), ("K", 2048))): ["A", "High", "Low", "Sum"],
    ("split_prefill_a8", (("rows", 64), ("K", 2048), ("dynamic_rows", True))): ["A", "High", "Low", "Sum", "m"],
    ("split_routed_prefill_a8", (("rows", 640), ("K", 2048), ("experts", 128), ("block_m", 16))):
        ["A", "Counts", "High", "Low", "Offsets", "Sum", "TC", "TE", "TR"],
    ("dispatch_prefill_a8", (("M", 64),)):
        ["A", "DS", "High", "IDs", "Low", "RelativeSlot", "RowOffsets", "Scale", "SlotMap", "Sum"],
    ("pack_expert_tokens", (("M", 64), ("K", 2048), ("E", 128), ("top_k", 8))):
        ["A", "High", "IDs", "Low", "RelativeSlot", "RowOffsets", "SlotMap", "Sources", "Sum", "m"],
    ("expand_expert_slots", (("M", 64), ("K", 2048), ("top_k", 8))):
        ["DS", "High", "Low", "Scale", "Sources", "SrcHigh", "SrcLow", "SrcSum", "Sum", "m"],
    ("e8p_exact_grouped", (("rows", 640), ("E", 128), ("tiles", 200), ("N", 1024), ("K", 2048), ("block_m", 8), ("stages", 3),
                           ("warp_private", True))):
        ["AS", "Book", "Counts", "High", "Low", "Offsets", "Out", "P", "Sum", "TC", "TE", "TR", "WS"],
    ("e8p_prefill_grouped", (("rows", 640), ("E", 128), ("tiles", 200), ("N", 1024), ("K", 2048), ("dynamic_rows", True),
                             ("codec", "e8p_q4"), ("block_m", 32))):
        ["AS", "Book", "Counts", "High", "Low", "Offsets", "Out", "P", "Sum", "TC", "TE", "TR", "WS", "m"],
}


@pytest.mark.parametrize("key", list(ABI), ids=lambda k: k[0])
def test_argument_order_is_the_reference_host_abi(key):
    symbol, variant = key
    kernel = lib.Kernel(symbol, **dict(variant))
    assert kernel.arg_names == ABI[key]
    buffers = [n for n, kind in zip(kernel.arg_names, kernel.arg_kinds) if kind == 0]
    assert buffers == sorted(buffers)
    assert all(kind == 1 for n, kind in zip(kernel.arg_names, kernel.arg_kinds) if n in ("m", "rows"))
    grid, block, shared = kernel.geometry()
    assert block[0] * block[1] * block[2] <= 1024
    assert all(g >= 1 for g in grid) and shared <= 160 * 1024


def test_resolve_errors():
    with pytest.raises(lib.OrxError) as err:
        lib.Kernel("no_such_kernel", M=1)
    assert err.value.code == lib.ORX_ERR_UNKNOWN_SYMBOL
    for variant in (dict(M=1, N=9728), dict(M=1, N=9728, K=2500), dict(M=0, N=128, K=128),
                    dict(M=1, N=128, K=128, algorithm="cublas"), dict(M=1, N=128, K=128, output_dtype="bfloat16"),
                    dict(M=8, N=128, K=128, packed_k=96), dict(M=1, N="x", K=128)):
        with pytest.raises(lib.OrxError) as err:
            lib.Kernel("e8p_q4_projection", **variant)
        assert err.value.code == lib.ORX_ERR_BAD_VARIANT, variant
        assert "e8p_q4_projection" in str(err.value) or "variant" in str(err.value)
    # K-major blocks of 64 resolve (e8p_q4.py:78-80), for the one-row GEMV by name as well while K is a multiple of 256
    assert lib.Kernel("e8p_q4_projection", M=8, N=128, K=256, packed_k=64).arg_names[-1] == "W"
    by_name = lib.Kernel("e8p_q4_projection", M=1, N=128, K=256, packed_k=64, algorithm="gemv")
    assert by_name.geometry(1) == lib.Kernel("e8p_q4_projection", M=1, N=128, K=256, packed_k=128, algorithm="gemv").geometry(1)
    with pytest.raises(lib.OrxError) as err:
        lib.Kernel("e8p_q4_projection", M=1, N=128, K=384, packed_k=64, algorithm="gemv")
    assert err.value.code == lib.ORX_ERR_BAD_VARIANT
    with pytest.raises(lib.OrxError):
        lib.Kernel("int8_projection", M=8, N=128, K=256, packed_k=64)
    handle = ctypes.c_void_p()
    code = lib.library().orx_resolve(b"swiglu", b"{not json", ctypes.byref(handle))
    assert code == lib.ORX_ERR_BAD_VARIANT and not handle.value
    assert lib.library().orx_resolve(None, b"{}", ctypes.byref(handle)) == lib.ORX_ERR_BAD_ARGUMENT
    assert lib.last_error()


def test_dynamic_geometry_follows_live_rows():
    kernel = lib.Kernel("e8p_q4_projection", M=64, N=9728, K=2560, dynamic_rows=True)
    one, many, big = kernel.geometry(1), kernel.geometry(64), lib.Kernel(
        "e8p_q4_projection", M=512, N=9728, K=2560, dynamic_rows=True).geometry(512)
    assert one != many                        # batch-1 and batch-64 take different kernels
    # 257..512 rows of a matrix that gives every CU at least 2.25 blocks of 16 channels: one workgroup per CU (256 where
    # no device answers) owns all rows and a run of channels, the decode in its K loop (608 and 1088 blocks here)
    assert big[0] == (256, 1, 1) and big[1] == (512, 1, 1)
    tall = lib.Kernel("e8p_q4_projection", M=512, N=17408, K=5120, dynamic_rows=True).geometry(512)
    assert tall[0] == (256, 1, 1) and tall[1] == (512, 1, 1)
    # a narrow matrix (320 blocks) keeps the 128 x 128 tiles
    narrow = lib.Kernel("e8p_q4_projection", M=512, N=5120, K=5120, dynamic_rows=True).geometry(512)
    assert narrow[1] == (256, 1, 1)
    with pytest.raises(lib.OrxError) as err:
        kernel.geometry(65)
    assert err.value.code == lib.ORX_ERR_ROWS
    fixed = lib.Kernel("int8_projection", M=8192, N=4096, K=4096)
    grid, block, shared = fixed.geometry()
    # int8 weights: persistent workgroups, one per CU (256 where no device answers), walk the 512 tiles
    assert grid[0] * grid[1] * grid[2] in (256, (8192 // 256) * (4096 // 256)) and grid[0] <= 512 and block == (512, 1, 1)
    assert shared > 64 * 1024                 # two LDS stages of the 256x256 tile
    few = lib.Kernel("int8_projection", M=512, N=1024, K=1024, split_k=False).geometry()
    assert few[0] == (8, 1, 1)                # never more workgroups than tiles


def test_launch_record_is_validated_before_anything_is_enqueued():
    kernel = lib.Kernel("e8p_q4_projection", M=2, N=256, K=256)
    grid, block, shared = kernel.geometry()
    fake = [256] * 6                           # aligned, never dereferenced: every call below is rejected
    for bad in ((grid[0] + 1, 1, 1), (0, 1, 1)):
        with pytest.raises(lib.OrxError) as err:
            kernel.launch_raw(bad, block, shared, 0, fake)
        assert err.value.code == lib.ORX_ERR_BAD_GEOMETRY
    with pytest.raises(lib.OrxError) as err:
        kernel.launch_raw(grid, (block[0] // 2, 1, 1), shared, 0, fake)
    assert err.value.code == lib.ORX_ERR_BAD_GEOMETRY
    with pytest.raises(lib.OrxError) as err:
        kernel.launch_raw(grid, block, shared + 16, 0, fake)
    assert err.value.code == lib.ORX_ERR_BAD_GEOMETRY
    for position in range(6):
        for pointer in (0, 257):                # null, misaligned
            values = list(fake)
            values[position] = pointer
            with pytest.raises(lib.OrxError) as err:
                kernel.launch_raw(grid, block, shared, 0, values)
            assert err.value.code == lib.ORX_ERR_BAD_ARGUMENT, (position, pointer)
    assert lib.library().orx_launch(None, None, None, 0, None, None) == lib.ORX_ERR_BAD_ARGUMENT
    dynamic = lib.Kernel("e8p_q4_projection", M=4, N=256, K=256, dynamic_rows=True)
    grid, block, shared = dynamic.geometry(4)
    for rows in (0, 5, -1):
        with pytest.raises(lib.OrxError) as err:
            dynamic.launch_raw(grid, block, shared, 0, fake + [rows])
        assert err.value.code == lib.ORX_ERR_ROWS


def test_handles_own_no_device_memory_and_say_what_workspace_they_need():
    """orx_resolve allocates nothing: scratch is a `Workspace` buffer the engine sizes from
    orx_workspace_bytes (AGENTS.md:41: the engine owns every buffer).  A thousand handles resolve in
    host memory only (the GPU test of the same name checks the device's free memory)."""
    plain = lib.Kernel("e8p_q4_projection", M=8192, N=7168, K=5120, dynamic_rows=True)
    assert plain.arg_names == ["A", "AS", "Book", "Out", "S", "W", "m"]           # the reference's list, unchanged
    assert plain.workspace_bytes(0) == 0 and plain.workspace() is None
    q4 = lib.Kernel("e8p_q4_projection", M=8192, N=7168, K=5120, dynamic_rows=True, workspace=True)
    assert q4.arg_names == ["A", "AS", "Book", "Out", "S", "W", "Workspace", "m"]
    assert q4.workspace_bytes(8192) == 7168 * 5120                                # int8 weights decoded once per launch
    assert q4.workspace_bytes(1) == 0 and q4.workspace_bytes(32) == 0             # GEMV / batched decode: none
    split = q4.workspace_bytes(256)                                                # 2 x 56 tiles of 128: K steps split over the CUs
    assert split > 0 and split % (2 * 128 * 128 * 4) == 0 and split <= 512 * 2 * 128 * 128 * 4
    # 2560 rows: 10 x 28 tiles of 256, a few more than the 256 CUs this library assumes without a device, so the channels
    # behind one round run as split tiles and their partial tiles sit behind the decoded weights
    peeled = q4.workspace_bytes(2560)
    assert peeled > 7168 * 5120 and (peeled - 7168 * 5120) % (2 * 128 * 128 * 4) == 0
    assert q4.workspace_bytes(0) == max(split, peeled)
    assert q4.geometry(256) != plain.geometry(256)                                 # whole tiles without a workspace
    w8 = lib.Kernel("int8_projection", M=512, N=5120, K=17408, workspace=True)
    assert w8.arg_names == ["A", "Output", "TokenScale", "Weight", "WeightScale", "Workspace"]
    assert w8.workspace_bytes(0) == w8.workspace_bytes(512) > 0
    for off in (dict(split_k=False), dict(algorithm="gemv", M=4)):
        assert lib.Kernel("int8_projection", **{**dict(M=256, N=5120, K=5120, workspace=True), **off}).workspace_bytes(0) == 0
    with pytest.raises(lib.OrxError) as err:
        q4.workspace_bytes(8193)
    assert err.value.code == lib.ORX_ERR_ROWS
    # a launch that needs the buffer refuses a null one before anything is enqueued; one that does not, takes it
    grid, block, shared = q4.geometry(8192)
    fake = [256] * 6
    with pytest.raises(lib.OrxError) as err:
        q4.launch_raw(grid, block, shared, 0, fake + [0, 8192])
    assert err.value.code == lib.ORX_ERR_WORKSPACE and str(7168 * 5120) in str(err.value)
    with pytest.raises(lib.OrxError) as err:
        q4.launch_raw(grid, block, shared, 0, fake + [128, 8192])                 # not 256-byte aligned
    assert err.value.code == lib.ORX_ERR_BAD_ARGUMENT
    handles = [lib.Kernel("e8p_q4_projection", M=64 + i, N=17408, K=5120, dynamic_rows=True, workspace=True)
               for i in range(1000)]
    # up to 512 rows no launch of such a handle needs scratch (K = 5120: the channel-run kernel serves 65..128 rows, and
    # this matrix gives every CU 4.25 blocks of 16 channels: the 512-row channel runs serve 129..512)
    assert all(h.workspace_bytes(0) == 0 for h in handles[:449]) and all(h.workspace_bytes(0) > 0 for h in handles[449:])
    assert lib.library().orx_workspace_bytes(None, 0, None) == lib.ORX_ERR_BAD_ARGUMENT


def test_variant_integers_are_range_checked():
    for variant in (dict(M=4294967297, N=128, K=128), dict(M=1, N=2**31, K=128), dict(M=1, N=128, K=-2**40)):
        with pytest.raises(lib.OrxError) as err:
            lib.Kernel("e8p_q4_projection", **variant)
        assert err.value.code == lib.ORX_ERR_BAD_VARIANT, variant


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(lib, "_lib", None)
    monkeypatch.setattr(lib, "LIBRARY_PATH", tmp_path / "liborx.so")
    with pytest.raises(FileNotFoundError):
        lib.Kernel("swiglu", I=128)


def test_package_codebook_matches_oracle(golden_basis):
    assert np.array_equal(codebook.basis(), golden_basis)
    assert np.array_equal(codebook.selector_table(codebook.basis()), ref.selector_table(ref.basis()))
    book = codebook.book()
    assert book.shape == (256, 1) and book.dtype == np.uint32
    rng = np.random.default_rng(5)
    q4 = rng.integers(0, 2**32, size=(48, 32), dtype=np.uint32)            # N=48, K=256
    assert np.array_equal(codebook.q4_to_k_major(q4), ref.q4_pack_k(q4, 128))
    q2 = rng.integers(0, 2**16, size=(3, 32, 32), dtype=np.uint16)          # E=3, N=32, K=256
    assert np.array_equal(codebook.q2_to_k_major(q2), np.stack([ref.q2_pack_k128(e) for e in q2]))
    assert np.array_equal(codebook.raw_book(), ref.raw_table_words(golden_basis))
    assert np.array_equal(codebook.raw_book(golden_basis[::-1]), ref.raw_table_words(golden_basis[::-1]))


def test_package_nibble_book_and_k64_blocks_match_oracle(golden_basis):
    assert np.array_equal(codebook.nibble_book().reshape(256, 1), ref.nibble_table(ref.selector_table(golden_basis)))
    raw = np.random.default_rng(3).integers(0, 65536, (2, 3, 5, 16), dtype=np.uint16)
    assert np.array_equal(codebook.q2_to_k64(raw), ref.q2_repack_k64(raw))
    zeros = golden_basis.copy()
    zeros[7, 1] = 0
    with pytest.raises(ValueError):
        codebook.nibble_book(zeros)


def test_workload_sizes_and_algorithmic_bytes():
    # N*K/2 + 2N + M*K + 2M + 2*M*N + 1024 (Q4) and N*K + 2N + M*K + 2M + 2*M*N (W8)
    assert workloads.algorithmic_bytes_q4(1, 9728, 2560) == 12_494_338
    assert workloads.algorithmic_bytes_q4(1, 17408, 5120) == 44_640_258
    assert workloads.algorithmic_bytes_w8(8192, 4096, 4096) == 117_465_088
    assert workloads.algorithmic_ops(8192, 4096, 4096) == 2 * 8192 * 4096 * 4096
    case = workloads.config0()
    assert case["packed"].shape == (9728, 320) and case["packed"].dtype == np.uint32
    assert case["x"].shape == (1, 2560) and case["x"].dtype == np.float16 and case["scales"].shape == (9728,)
    again = workloads.config0()
    assert np.array_equal(case["packed"], again["packed"]) and np.array_equal(case["x"], again["x"])
    small = workloads.config1(8, n=256, k=256)
    assert small["x"].shape == (8, 256) and np.array_equal(small["packed"], workloads.config1(1, n=256, k=256)["packed"])


def test_argument_lists_of_the_fused_expert_layer_forms():
    """Buffer names stay in ASCII order when a form adds buffers, and forms the resident expert kernel
    does not serve are refused at resolve time (so a program can fall back to the separate launches)."""
    def names(symbol, **variant):
        return lib.Kernel(symbol, **variant).arg_names

    assert names("router_topk", M=8, E=64, top_k=4, quantize_hidden=256) == ["IDs", "Logits", "Prob", "Q", "S", "X"]
    assert names("router_topk", M=8, E=64, top_k=4, dynamic_rows=True) == ["IDs", "Logits", "Prob", "m"]
    assert names("route_metadata", M=8, E=64, top_k=4, block_m=32, slot_maps=True) == [
        "Counts", "IDs", "RelativeSlot", "RowMax", "RowOffsets", "SlotMap", "SlotToken", "TileCount", "TileExpert",
        "TileOffsets", "TileRow"]
    grouped = dict(rows=2048, E=128, tiles=192, block_m=32, algorithm="resident")
    plain = ["A", "AS", "Book", "C", "Counts", "Offsets", "P", "TileCount", "TileExpert", "TileRow", "WS"]
    assert names("e8p_decode_grouped", N=1024, K=2048, **grouped) == plain
    assert names("e8p_decode_grouped", N=1024, K=2048, gather=True, epilogue="swiglu", **grouped) == [
        "A", "AS", "Act", "Book", "C", "Counts", "Offsets", "P", "RowMax", "SlotToken", "TileCount", "TileExpert",
        "TileRow", "WS"]
    assert names("e8p_decode_grouped", N=2048, K=512, input_dtype="float16", **grouped) == [
        "A", "AS", "Book", "C", "Counts", "Offsets", "P", "Q", "RowMax", "TileCount", "TileExpert", "TileRow", "WS"]
    for listed in (plain, names("rotate_expert_a8", M=4, K=256, routing="scatter", top_k=2, experts=8)):
        assert listed == sorted(listed)
    # the reference's lists (kernels/cuda/model/rotation_a8.py:536-589 in generated-ABI order): nibble planes Low and High
    routed = ["DS", "High", "IDs", "Low", "Q", "RelativeSlot", "RowOffsets", "S", "Signs", "SlotMap", "Sum", "X"]
    assert names("rotate_expert_a8", M=4, K=256, routing="shared", top_k=2, experts=8, dynamic_rows=True) == routed + ["m"]
    assert names("rotate_expert_a8", M=4, K=256, routing="scatter", top_k=2, experts=8) == routed
    assert names("rotate_expert_a8", M=4, K=256) == ["High", "Low", "Q", "S", "Signs", "Sum", "X"]
    assert names("rotate_expert_a8", M=4, K=256, group_major=True) == ["High", "Low", "S", "Signs", "Sum", "X"]
    # whole int8 rows for the int8 expert GEMMs: D (scatter) in place of the planes
    assert names("rotate_expert_a8", M=4, K=256, routing="scatter", top_k=2, experts=8, hand_over="int8") == [
        "D", "DS", "IDs", "Q", "RelativeSlot", "RowOffsets", "S", "Signs", "SlotMap", "Sum", "X"]
    assert names("rotate_expert_a8", M=4, K=256, routing="shared", top_k=2, experts=8, hand_over="int8") == [
        "DS", "IDs", "Q", "RelativeSlot", "RowOffsets", "S", "Signs", "SlotMap", "Sum", "X"]
    assert names("rotate_expert_a8", M=4, K=256, hand_over="int8") == ["Q", "S", "Signs", "Sum", "X"]
    refused = (
        ("e8p_decode_grouped", dict(N=1024, K=2048, gather=True, rows=8200, E=128, tiles=512, block_m=32, algorithm="resident")),
        # without the SwiGLU epilogue the kernel keeps its phase-two sums in LDS, which leaves room for fewer slots
        ("e8p_decode_grouped", dict(N=1024, K=2048, gather=True, rows=8192, E=128, tiles=512, block_m=32, algorithm="resident")),
        ("e8p_decode_grouped", dict(N=2048, K=2048, input_dtype="float16", **grouped)),          # K > 1024 for fp16 rows
        ("e8p_decode_grouped", dict(N=2048, K=512, input_dtype="float16", epilogue="swiglu", **grouped)),
        ("e8p_decode_grouped", dict(N=1024, K=2048, gather=True, rows=2048, E=128, tiles=192, block_m=64)),
        ("e8p_decode_grouped", dict(N=1024, K=2048, epilogue="swiglu", rows=2048, E=128, tiles=192, block_m=32,
                                    algorithm="stream")),
        ("rotate_expert_a8", dict(M=4, K=256, group_major=True, routing="shared", top_k=2, experts=8)),  # rotation_a8.py:409
        ("rotate_expert_a8", dict(M=4, K=256, group_major=True, hand_over="int8")),
        ("rotate_expert_a8", dict(M=4, K=256, hand_over="fp8")),
        ("rotate_expert_a8", dict(M=4, K=256, routing="scatter", top_k=65, experts=128)),
        ("router_topk", dict(M=8, E=64, top_k=4, quantize_hidden=100)),
    )
    for symbol, variant in refused:
        with pytest.raises(lib.OrxError) as err:
            lib.Kernel(symbol, **variant)
        assert err.value.code == lib.ORX_ERR_BAD_VARIANT, (symbol, variant)


def test_static_scratch_launch_refuses_before_it_enqueues():
    # host-only checks of orx_launch_static_scratch: nothing reaches a device, so made-up addresses are safe here
    big = lib.Kernel("e8p_q4_projection", M=8192, N=17408, K=5120, workspace=True)
    assert big.workspace_bytes(8192) == 17408 * 5120 > 64 << 20
    grid, block, shared = big.geometry(8192)
    with pytest.raises(lib.OrxError) as err:  # beyond the static array
        big.launch_raw(grid, block, shared, 0, [256] * 6 + [None], static_scratch=True)
    assert err.value.code == lib.ORX_ERR_WORKSPACE and "static scratch" in str(err.value)
    with pytest.raises(lib.OrxError) as err:  # geometry is checked as orx_launch checks it
        big.launch_raw((grid[0] + 1, 1, 1), block, shared, 0, [256] * 6 + [None], static_scratch=True)
    assert err.value.code == lib.ORX_ERR_BAD_GEOMETRY


def test_omit_takes_optional_buffers_out_of_the_argument_list():
    # a package record cannot say "null" (artifact.rs:184-194): buffers a program does not use are named in `omit`
    full = lib.Kernel("moe_combine", M=4, E=8, top_k=2, H=64, slots=8)
    short = lib.Kernel("moe_combine", M=4, E=8, top_k=2, H=64, slots=8, omit="Shared,SharedGate")
    assert [n for n in full.arg_names if n not in ("Shared", "SharedGate")] == short.arg_names
    assert len(short.arg_kinds) == len(short.arg_names)
    assert short.geometry() == full.geometry()
    for bad in ("Expert", "Nothing", "Shared,Shared"):  # required, unknown, named twice
        with pytest.raises(lib.OrxError) as err:
            lib.Kernel("moe_combine", M=4, E=8, top_k=2, H=64, slots=8, omit=bad)
        assert err.value.code == lib.ORX_ERR_BAD_VARIANT
    inline = lib.Kernel("moe_combine?M=4&E=8&top_k=2&H=64&slots=8&omit=Shared,SharedGate")
    assert inline.arg_names == short.arg_names


def test_session_threads_resolve_and_query_concurrently():
    """Two or more session threads may resolve, inspect and release handles at the same time (one-time
    set-up is atomic, errors are thread-local): every thread sees the answers a single thread sees."""
    import threading

    variants = [("e8p_q4_projection", dict(M=1, N=9728, K=2560)), ("int8_projection", dict(M=256, N=5120, K=5120, workspace=True)),
                ("router_topk", dict(M=64, E=128, top_k=8, quantize_hidden=2048)),
                ("e8p_decode_grouped", dict(rows=2048, E=128, tiles=192, N=1024, K=2048, block_m=32, algorithm="resident")),
                ("rotate_expert_a8", dict(M=16, K=512, routing="scatter", top_k=4, experts=32))]
    expected = []
    for symbol, variant in variants:
        kern = lib.Kernel(symbol, **variant)
        expected.append((kern.arg_names, kern.geometry(), kern.workspace_bytes() if "workspace" in variant else 0))
    catalog = lib.catalog()
    failures = []

    def session(index):
        try:
            for round_ in range(40):
                symbol, variant = variants[(index + round_) % len(variants)]
                kern = lib.Kernel(symbol, **variant)
                want = expected[(index + round_) % len(variants)]
                got = (kern.arg_names, kern.geometry(), kern.workspace_bytes() if "workspace" in variant else 0)
                if got != want or lib.catalog() != catalog:
                    failures.append((index, symbol))
                try:
                    lib.Kernel("e8p_q4_projection", M=1, N=128, K=100 + index)  # a refusal with a thread-local message
                    failures.append((index, "accepted a bad K"))
                except lib.OrxError as error:
                    if str(100 + index) not in str(error) and "K" not in str(error):
                        failures.append((index, str(error)))
                del kern
        except Exception as error:  # noqa: BLE001 - reported below
            failures.append((index, repr(error)))

    threads = [threading.Thread(target=session, args=(i,)) for i in range(8)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not failures, failures[:5]


def test_integer_vq_grouped_takes_the_reference_patch_buffer():
    """integer_vq_grouped lists Patch like the reference's routed prim_func (integer_vq.py:230-258) in the
    sorted host order; e8p_decode_grouped has none (e8p_decode.py:64).  The decoder options that the XOR
    kernels do not take run on the MFMA tiles and refuse the other algorithms."""
    shape = dict(rows=99, E=3, tiles=16, N=65, K=256)
    want = ["A", "AS", "Book", "C", "Counts", "Offsets", "P", "Patch", "TileCount", "TileExpert", "TileRow", "WS"]
    for extra in (dict(shared_table=True), dict(patched=True), dict(), dict(shared_table=True, basis="any"), dict(block_m=8),
                  dict(block_m=16, patched=True, shared_table=True), dict(packed_k=64), dict(packed_k=0, patched=True)):
        kern = lib.Kernel("integer_vq_grouped", **shape, **extra)
        assert kern.arg_names == want, extra
        grid, block, _ = kern.geometry()
        # the reference's defaults (a raw basis table per expert, 16-row tiles: integer_vq.py:304-314) are the general decode
        assert tuple(grid)[:2] == (1, 16) and tuple(block)[0] == 256, extra
    # the selector Book of one table for all on 32-row tiles is what the XOR kernels take
    xor = lib.Kernel("integer_vq_grouped", **shape, shared_table=True, shortbook=True, selectorbook=True, block_m=32)
    assert xor.arg_names == want and xor.geometry()[1][0] == 512
    assert "Patch" not in lib.Kernel("e8p_decode_grouped", **shape).arg_names
    # tile lists in steps of 8 rows, as the reference's decode kernel and route_metadata's default build them
    assert lib.Kernel("e8p_decode_grouped", **shape, block_m=8).geometry()[1][0] == 512
    for symbol, bad in (("integer_vq_grouped", dict(patched=True, algorithm="stream")),
                        ("integer_vq_grouped", dict(algorithm="stream")),
                        ("integer_vq_grouped", dict(shared_table=True, basis="any", algorithm="resident")),
                        ("integer_vq_grouped", dict(basis="e8")),
                        ("integer_vq_grouped", dict(block_m=24)),
                        ("integer_vq_grouped", dict(selectorbook=True)),           # integer_vq.py:95-97: needs shortbook
                        ("integer_vq_grouped", dict(byte_permute=True)),
                        ("integer_vq_grouped", dict(packed_k=32)),
                        ("e8p_decode_grouped", dict(block_m=8, algorithm="resident")),  # 8-row lists: the streaming kernel only
                        ("e8p_decode_grouped", dict(block_m=16, epilogue="swiglu", gather=True)),
                        ("e8p_decode_grouped", dict(block_m=24)),
                        ("e8p_decode_grouped", dict(packed_k=32)),
                        ("e8p_decode_grouped", dict(packed_k=64, algorithm="stream")),  # 64-wide blocks: the MFMA tiles only
                        ("e8p_decode_grouped", dict(packed_k=64, algorithm="resident")),
                        ("e8p_decode_grouped", dict(packed_k=64, epilogue="swiglu"))):
        with pytest.raises(lib.OrxError):
            lib.Kernel(symbol, **shape, **bad)
    # K-major blocks of 64 codes per channel, which the reference's decode kernel takes too (e8p_decode.py:43), at every list step
    for bm in (8, 16, 32, 64, 128):
        assert lib.Kernel("e8p_decode_grouped", **shape, packed_k=64, block_m=bm).geometry()[1][0] == 256
    # the fused forms keep their places around Patch
    xor_book = dict(shared_table=True, shortbook=True, selectorbook=True, block_m=32)
    fused = lib.Kernel("integer_vq_grouped", rows=2048, E=128, tiles=192, N=2048, K=512, input_dtype="float16", **xor_book)
    assert fused.arg_names == ["A", "AS", "Book", "C", "Counts", "Offsets", "P", "Patch", "Q", "RowMax", "TileCount",
                               "TileExpert", "TileRow", "WS"]
    with pytest.raises(lib.OrxError):
        lib.Kernel("integer_vq_grouped", rows=2048, E=128, tiles=192, N=2048, K=512, input_dtype="float16", patched=True, **xor_book)
    with pytest.raises(lib.OrxError):  # the fused forms are forms of the XOR kernels: not with the default raw Book
        lib.Kernel("integer_vq_grouped", rows=2048, E=128, tiles=192, N=2048, K=512, input_dtype="float16", shared_table=True)
    # the form without a tile list: every expert multiplies its own M rows (integer_vq.py:217-228)
    direct = lib.Kernel("integer_vq", E=3, M=17, N=65, K=256, block_m=16, patched=True)
    assert direct.arg_names == ["A", "AS", "Book", "C", "P", "Patch", "WS"]
    grid, block, _ = direct.geometry()
    assert tuple(grid) == (1, 1, 3) and tuple(block)[0] == 256
    for bad in (dict(block_m=128), dict(K=200), dict(packed_k=32), dict(M=0)):
        variant = dict(E=3, M=17, N=65, K=256)
        variant.update(bad)
        with pytest.raises(lib.OrxError):
            lib.Kernel("integer_vq", **variant)


def test_int8_weights_take_k_in_steps_of_64():
    """int8_projection.py:29 accepts K % 64 == 0; codes come in whole groups of 128 only."""
    kern = lib.Kernel("int8_projection", M=512, N=130, K=192, dynamic_rows=True)
    for rows, tile in ((1, 32), (33, 64), (500, 128)):
        grid, block, shared = kern.geometry(rows)
        assert tuple(grid)[:2] == (2, -(-rows // tile)) and tuple(block)[0] == 256, rows
    for symbol, bad in (("int8_projection", dict(K=192, algorithm="gemv")), ("int8_projection", dict(K=192, block_m=256)),
                        ("int8_projection", dict(K=96)), ("e8p_q4_projection", dict(K=192))):
        variant = dict(M=8, N=130, K=128)
        variant.update(bad)
        with pytest.raises(lib.OrxError):
            lib.Kernel(symbol, **variant)


def test_projections_take_the_reference_factories_schedule_names():
    """e8p_q4.projection(algorithm="tensor_core"|"dp4a"|"int4_direct", block_m=8.., split_k=1|2|4, ...) and
    int8_projection(block_m=16.., block_n, block_k, stages, ...) (e8p_q4.py:143-215, int8_projection.py:15-48) pick
    among SM87 kernels; the same keyword set resolves here, and the schedule name and the row tile choose among this
    library's kernels: dp4a keeps the dot-product (GEMV) family where it serves the rows, tensor_core keeps off it,
    int4_direct and tiles of 1-8 rows leave the choice to the row count, and a tile of 16, 96 or 192 rows asks for the
    MFMA tile that holds it (32, 128, 256) while the live rows fit one such tile."""
    shape = dict(M=512, N=17408, K=5120, dynamic_rows=True)
    plain = lib.Kernel("e8p_q4_projection", **shape)

    def q4(**extra):
        return lib.Kernel("e8p_q4_projection", **shape, **extra)

    for extra in (dict(algorithm="int4_direct", block_m=8, block_n=128, basis_nonzero=True, split_k=2),
                  dict(algorithm="int4_direct", block_m=4, group_m=4, cache_scales=True, tail_m=16)):
        for rows in (1, 3, 8, 64, 100, 200, 512):
            assert q4(**extra).geometry(rows) == plain.geometry(rows), (extra, rows)
    gemv = lib.Kernel("e8p_q4_projection", **dict(shape, M=4), algorithm="gemv")
    mma = q4(algorithm="tensor_core", block_m=8, block_n=64, block_k=128, stages=2)
    dot = q4(algorithm="dp4a", block_m=4, block_n=8)
    assert plain.geometry(1) == gemv.geometry(1) == dot.geometry(1) != mma.geometry(1)
    assert mma.geometry(1) == lib.Kernel("e8p_q4_projection", **dict(shape, M=64), algorithm="stream").geometry(1)
    for rows in (2, 3, 4):  # by row count these go to the batched-decode kernel; dp4a keeps the GEMV, tensor_core does not
        assert dot.geometry(rows) == gemv.geometry(rows) != plain.geometry(rows) == mma.geometry(rows), rows
    for rows in (5, 64, 300):
        assert dot.geometry(rows) == plain.geometry(rows) == mma.geometry(rows), rows
    for hint, tile, fits, beyond in ((16, 32, (5, 20, 32), (33, 200)), (96, 128, (20, 100, 128), (129, 400)),
                                     (192, 256, (20, 200, 256), (257, 300))):
        hinted, forced = q4(block_m=hint), q4(block_m=tile)
        for rows in fits:
            assert hinted.geometry(rows) == forced.geometry(rows), (hint, rows)
        for rows in beyond:
            assert hinted.geometry(rows) == plain.geometry(rows), (hint, rows)
    assert q4(block_m=96).geometry(20) != plain.geometry(20) and q4(block_m=192).geometry(100) != plain.geometry(100)
    w8_shape = dict(M=256, N=512, K=1024, dynamic_rows=True)
    w8 = lib.Kernel("int8_projection", **w8_shape, block_m=16, block_n=64, block_k=64, stages=2)
    assert w8.geometry(20) == lib.Kernel("int8_projection", **w8_shape, block_m=32).geometry(20)
    assert w8.geometry(200) == lib.Kernel("int8_projection", **w8_shape).geometry(200)
    # a K of a single step, or one that ends in half a step, has no 256-row tile: 192 then names the 128-row tile
    short = dict(M=256, N=512, K=192, dynamic_rows=True)
    assert lib.Kernel("int8_projection", **short, block_m=192).geometry(100) == \
        lib.Kernel("int8_projection", **short, block_m=128).geometry(100)


def test_tall_tiles_by_name_and_for_handles_without_scratch():
    """512 rows x channel runs with the decode in the K loop: by name at any row count; what `auto` launches from 257
    to 512 rows of a wide matrix whether or not there is a Workspace; and what a two-stage handle without one (or with
    decode_in_gemm) launches above 512 rows.  K in whole blocks of 128, two-stage codes only."""
    shape = dict(M=1024, N=17408, K=5120, dynamic_rows=True)
    tall = lib.Kernel("e8p_q4_projection", **shape, algorithm="tall")
    plain = lib.Kernel("e8p_q4_projection", **shape)
    in_loop = lib.Kernel("e8p_q4_projection", **shape, workspace=True, decode_in_gemm=True)
    scratch = lib.Kernel("e8p_q4_projection", **shape, workspace=True)
    for rows, row_tiles in ((3, 1), (512, 1), (513, 2), (1024, 2)):
        grid, block, lds = tall.geometry(rows)
        assert grid == (row_tiles * 256, 1, 1) and block == (512, 1, 1) and 128 * 1024 < lds <= 160 * 1024
    for rows in (257, 385, 512, 1024):
        assert plain.geometry(rows) == tall.geometry(rows) == in_loop.geometry(rows)
        assert in_loop.workspace_bytes(rows) == 0
    for rows in (257, 384, 512):
        assert scratch.geometry(rows) == tall.geometry(rows) and scratch.workspace_bytes(rows) == 0
    assert scratch.geometry(513) != tall.geometry(513) and scratch.workspace_bytes(513) >= 17408 * 5120
    # 129..256 rows: only where every CU gets 4.25 blocks of 16 channels in one round (17408 = 16 * 4.25 * 256)
    for rows in (129, 256):
        assert plain.geometry(rows) == tall.geometry(rows) == scratch.geometry(rows) and scratch.workspace_bytes(rows) == 0
    assert plain.geometry(128) != tall.geometry(128) and scratch.geometry(128) != tall.geometry(128)
    narrower = lib.Kernel("e8p_q4_projection", **dict(shape, N=17408 - 16))
    assert narrower.geometry(256) != tall.geometry(256) and narrower.geometry(257)[1] == (512, 1, 1)
    for symbol, bad in (("int8_projection", dict(M=8, N=256, K=512)), ("e8p_q4_projection", dict(M=8, N=256, K=128))):
        with pytest.raises(lib.OrxError) as err:
            lib.Kernel(symbol, **bad, algorithm="tall")
        assert err.value.code == lib.ORX_ERR_BAD_VARIANT and "tall" in str(err.value)


def test_two_stage_coefficients_other_than_4_1_are_refused():
    """quantization/e8p_q4.py:19-29 allows other coprime pairs, the model builder only [4, 1]
    (models/qwen35/test_build.py:695-709): the kernels decode 4 * coarse + residual and say so."""
    shape = dict(M=4, N=256, K=512)
    for good in (dict(), dict(coefficients=[4, 1]), dict(coefficients="4,1"), dict(coefficients="4, 1")):
        lib.Kernel("e8p_q4_projection", **shape, **good)
    for symbol, base in (("e8p_q4_projection", shape), ("e8p_q4_unpack", dict(N=256, K=512))):
        for bad in ([3, 1], [7, 2], "5,2", [4], [4, 1, 0]):
            with pytest.raises(lib.OrxError) as err:
                lib.Kernel(symbol, **base, coefficients=bad)
            assert err.value.code == lib.ORX_ERR_BAD_VARIANT and "coefficients" in str(err.value)
    with pytest.raises(lib.OrxError):
        lib.Kernel("e8p_q4_projection", **shape, coefficients=[4.5, 1])


def test_unknown_variant_keys_are_refused():
    """A key no factory reads (a typo, an option of another symbol) fails the resolve and the message lists the
    symbol's keys, as a reference factory raises on an unknown keyword; the reference's own tile hints are known."""
    for symbol, variant, stray in (("e8p_q4_projection", dict(M=4, N=256, K=512), dict(output_strid=300)),
                                   ("e8p_q4_projection", dict(M=4, N=256, K=512), dict(patched=True)),
                                   ("int8_projection", dict(M=4, N=256, K=512), dict(packed=128)),
                                   ("router_topk", dict(M=4, E=64, top_k=4), dict(quantise_hidden=512)),
                                   ("e8p_decode_grouped", dict(rows=64, E=4, tiles=8, N=256, K=256), dict(shared_table=True)),
                                   ("activation_quantization", dict(K=512), dict(groups=4)),
                                   ("moe_combine", dict(M=4, top_k=2, H=256), dict(shared=True))):
        lib.Kernel(symbol, **variant)
        with pytest.raises(lib.OrxError) as err:
            lib.Kernel(symbol, **variant, **stray)
        key = next(iter(stray))
        assert err.value.code == lib.ORX_ERR_BAD_VARIANT and key in str(err.value) and "keys:" in str(err.value), (symbol, str(err.value))
    with pytest.raises(lib.OrxError):
        lib.Kernel("swiglu?I=128&J=3")
    # hints of the reference factories that choose among its own kernels are accepted and change nothing
    lib.Kernel("e8p_q4_projection", M=4, N=256, K=512, block_n=64, block_k=128, stages=2, tail_m=0, group_m=0, cache_scales=False,
               basis_nonzero=True, split_k=1)
    lib.Kernel("int8_projection", M=64, N=256, K=512, block_n=128, block_k=64, stages=2)


def test_routed_decode_symbols_take_the_reference_factories_keywords():
    """integer_vq_grouped(..., kind="e8p", shortbook=True, selectorbook=True, byte_permute=True, num_stages, block_n)
    as tests/cuda/operators/e8p_selector.py:66-79 calls it; the reference's other Book forms are refused."""
    shape = dict(rows=99, E=3, tiles=16, N=65, K=256)
    hints = dict(kind="e8p", shared_table=True, patched=False, block_m=32, block_n=128, shortbook=True, selectorbook=True,
                 num_stages=1, byte_permute=True)
    assert lib.Kernel("integer_vq_grouped", **shape, **hints).geometry()[1][0] == 512  # the XOR kernels (streaming)
    assert lib.Kernel("integer_vq_grouped", **shape, shared_table=True).geometry()[1][0] == 256  # raw Book: the general decode
    lib.Kernel("integer_vq", E=3, M=17, N=65, K=256, kind="e8p", shortbook=True, selectorbook=True, num_stages=2, block_n=128, byte_permute=True)
    lib.Kernel("e8p_decode_grouped", **shape, block_n=32, split_k=2, parity_xor=True)
    dynamic = lib.Kernel("integer_vq_grouped", **shape, shared_table=True, dynamic_rows=True)
    assert dynamic.arg_names[-1] == "m" and dynamic.arg_names[:-1] == lib.Kernel("integer_vq_grouped", **shape, shared_table=True).arg_names
    for bad in (dict(selectorbook=True, shortbook=False), dict(byte_permute=True, shortbook=False), dict(kind="scalar")):
        with pytest.raises(lib.OrxError):
            lib.Kernel("integer_vq_grouped", **shape, **bad)
        with pytest.raises(lib.OrxError):
            lib.Kernel("integer_vq", E=3, M=17, N=65, K=256, **bad)
    # the other two forms of Book resolve: signed values (shortbook alone) and raw basis values (the default)
    for book in (dict(shortbook=True), dict(shortbook=True, byte_permute=True), dict()):
        lib.Kernel("integer_vq_grouped", **shape, **book)
        lib.Kernel("integer_vq", E=3, M=17, N=65, K=256, **book)


REFERENCE_KEYWORDS = {
    # every keyword of the reference's factory with a value it accepts (signatures read from kernels/cuda/model/*.py and
    # kernels/cuda/operators/op30_activation_quantization.py): a package record written for the reference resolves here
    "activation_quantization": dict(K=512, group_size=128, masked=False, threads=512),
    "rotate_activation_a8": dict(M=8, K=512, swiglu=False, reciprocal=False, dynamic_rows=True, registers=True),
    "rotate_expert_a8": dict(M=8, K=512, swiglu=False, reciprocal=True, dynamic_rows=False, routing="scatter", top_k=2, experts=8,
                             group_major=False),
    "residual_norm_rotate_a8": dict(M=8, K=512, dynamic_rows=True, zero_centered=True),
    "integer_experts": dict(M=8, N=256, K=512, E=8, top_k=2, codec="e8p_q4", block_m=16, block_n=64, block_k=128, stages=2,
                            dynamic_rows=False, tail_m=0, minimum_blocks=1),
    "expert_histogram": dict(M=8, E=8, top_k=2, dynamic_rows=True),
    "expert_offsets": dict(E=8, block_m=16),
    "expert_tiles": dict(M=8, E=8, top_k=2, block_m=16, dynamic_rows=True),
    "expert_dispatch": dict(M=8, H=512, E=8, top_k=2, scale_group=512, dynamic_rows=True),
    "router_topk_warp": dict(M=8, E=64, top_k=4, dynamic_rows=True, warps=4),
    "router_topk": dict(M=8, E=64, top_k=4, renormalize=True, dynamic_rows=True),
    "moe_combine": dict(M=8, H=512, slots=16, top_k=2, dynamic_rows=False),
    "single_route_metadata": dict(E=64, top_k=8, capacity=16),
    "route_metadata": dict(M=8, E=64, top_k=8, block_m=16, dynamic_rows=True),
    "int8_swiglu": dict(M=8, N=256, K=512, block_n=64, dynamic_rows=True, algorithm="tensor_core", block_m=16),
    "int8_projection": dict(M=64, N=256, K=512, output_dtype="float16", block_m=64, block_n=128, block_k=64, group_m=4,
                            dynamic_rows=True, output_stride=260, tail_m=16, cache_scales=True),
    "int8_small_projection": dict(M=4, N=256, K=512, output_dtype="float32", dynamic_rows=True, block_m=4, block_n=8,
                                  output_stride=256),
    "expert_partition_offsets": dict(experts=8, hot_m=64, cold_m=16, cold_rows=16),
    "expert_partition_tiles": dict(M=8, experts=8, top_k=2, hot_m=64, cold_m=16, cold_rows=16, dynamic_rows=True),
    "e8p_decode_grouped": dict(rows=64, E=8, tiles=16, N=256, K=512, block_n=32, split_k=2, parity_xor=True, packed_k=128),
    "integer_vq": dict(E=3, M=17, N=65, K=256, kind="e8p", shared_table=True, block_n=128, patched=True, shortbook=True,
                       num_stages=2, block_m=16, byte_permute=True, selectorbook=True, packed_k=64),
    "integer_vq_grouped": dict(rows=64, E=8, tiles=16, N=256, K=512, kind="e8p", shared_table=False, block_n=128, patched=True,
                               shortbook=True, num_stages=1, block_m=8, byte_permute=True, selectorbook=True, warp_decode=True,
                               split_k=2, parity_xor=True, group_n=2, packed_k=64, dynamic_rows=True),
    "integer_e8p_gemv": dict(E=8, routes=2, N=256, K=512, shared_input=True, block_n=8),
    "rotate_activation": dict(M=8, K=512, swiglu=True),
    "rotate_activation_tiles": dict(M=8, K=1024, block_k=1024, swiglu=True, dynamic_rows=True, plane_rows=8, registers=True,
                                    threads=256),
    "quantize_rotation_tiles": dict(M=8, K=1024, block_k=256, dynamic_rows=True),
    "expert_histogram_local": dict(M=64, E=16, K=4, block=512, dynamic_rows=True),
    "expert_histogram_offsets": dict(M=64, E=16, K=4, block=2048, dynamic_rows=False),
    "expert_histogram_finish": dict(M=64, E=16, K=4, block=1024, dynamic_rows=True),
    "expand_experts": dict(N=256, K=512, E=8, block_n=64, block_k=256),
    "e8p_q4_embedding": dict(capacity=8, vocab=1000, hidden=512),
    "e8p_q4_projection": dict(M=8, N=256, K=512, coefficients=[4, 1], algorithm="tensor_core", block_m=8, block_n=64, block_k=128,
                              stages=2, dynamic_rows=False, output_dtype="float16", output_stride=256, packed_k=0,
                              basis_nonzero=False, split_k=1, tail_m=0, group_m=0, cache_scales=False),
    "e8p_q4_unpack": dict(N=256, K=512, coefficients=[4, 1], packed_k=64),
    "q4_projection": dict(M=64, N=256, K=512, BN=64, BK=256, output_dtype="float32", magnitudes=[3, 10, 19, 31, 46, 67, 93, 127],
                          block_m=16, dynamic_rows=True, stages=1, output_stride=260, tail_m=8, group_m=4),
    "q4_gemv": dict(M=4, N=256, K=512, BN=8, output_dtype="float16", magnitudes=[1, 2, 3, 4, 5, 6, 7, 8], dynamic_rows=True,
                    block_m=4, output_stride=256),
    "unpack_q4": dict(N=256, K=512, magnitudes=[3, 10, 19, 31, 46, 67, 93, 127]),
    "router_projection": dict(M=64, H=2048, E=128, dynamic_rows=True, block_m=32, block_n=64, block_k=256, stages=1),
    "split_a8": dict(rows=8, K=512, dynamic_rows=True),
    "split_prefill_a8": dict(rows=8, K=512, dynamic_rows=False),
    "split_routed_prefill_a8": dict(rows=64, K=512, experts=8, block_m=16, dynamic_rows=True),
    "dispatch_prefill_a8": dict(M=8, K=512, E=8, top_k=2, dynamic_rows=True),
    "pack_expert_tokens": dict(M=8, K=512, E=8, top_k=2),
    "expand_expert_slots": dict(M=8, K=512, top_k=2),
    "e8p_exact_grouped": dict(rows=64, E=8, tiles=16, N=256, K=512, block_m=16, stages=4, dynamic_rows=True, warp_private=False),
    "e8p_prefill_grouped": dict(rows=64, E=8, tiles=16, N=256, K=512, dynamic_rows=False, sparse_rows=True, row_major=False,
                                codec="e8p_q2", minimum_blocks=2, block_m=32, block_n=64, specialize_tails=True,
                                merge_routed_tiles=True),
}


@pytest.mark.parametrize("symbol", list(REFERENCE_KEYWORDS))
def test_every_keyword_of_the_reference_factory_resolves(symbol):
    kernel = lib.Kernel(symbol, **REFERENCE_KEYWORDS[symbol])
    assert kernel.arg_names
    with pytest.raises(lib.OrxError, match="unknown variant key"):
        lib.Kernel(symbol, **REFERENCE_KEYWORDS[symbol], no_such_option=1)


def test_plane_kernels_refuse_what_the_reference_refuses():
    # e8p_exact.py:57-70, e8p_prefill.py:160-183
    shape = dict(rows=64, E=8, tiles=16, N=256, K=512)
    for bad in (dict(block_m=32), dict(stages=5), dict(stages=1), dict(K=500), dict(K=131200)):
        with pytest.raises(lib.OrxError):
            lib.Kernel("e8p_exact_grouped", **{**shape, **bad})
    for bad in (dict(block_m=8), dict(block_n=32), dict(codec="w8"), dict(codec="e8p_q4", block_n=64), dict(minimum_blocks=17),
                dict(specialize_tails=True, block_m=16), dict(specialize_tails=True, block_m=32, codec="e8p_q4"),
                dict(merge_routed_tiles=True, block_m=32)):
        with pytest.raises(lib.OrxError):
            lib.Kernel("e8p_prefill_grouped", **{**shape, **bad})
    for bad in (dict(rows=0, K=512), dict(rows=8, K=192)):
        with pytest.raises(lib.OrxError):
            lib.Kernel("split_a8", **bad)
    with pytest.raises(lib.OrxError):
        lib.Kernel("split_routed_prefill_a8", rows=64, K=512, experts=8, block_m=6)
    with pytest.raises(lib.OrxError):
        lib.Kernel("dispatch_prefill_a8", M=8, K=512, E=4, top_k=5)
    # the exact kernel launches no more tiles than the live rows can fill (e8p_exact.py:76)
    dynamic = lib.Kernel("e8p_exact_grouped", **shape, block_m=8, dynamic_rows=True)
    assert dynamic.geometry(8)[0][1] == 1 + 8 and dynamic.geometry(64)[0][1] == 16
    # two kernels behind the symbols: 512-thread weight-streaming workgroups from K = 1024, 256-thread LDS tiles below
    assert lib.Kernel("e8p_exact_grouped", **{**shape, "K": 2048}).geometry()[1][0] == 512 and dynamic.geometry()[1][0] == 256
    assert lib.Kernel("e8p_exact_grouped", **shape, algorithm="stream").geometry()[1][0] == 512
    with pytest.raises(lib.OrxError):
        lib.Kernel("e8p_exact_grouped", **shape, algorithm="mfma")


def test_scalar_q4_symbols_bind_as_the_reference_does_and_refuse_what_it_refuses():
    # crates/orinfer-models/src/flash_next/q4.rs:176-196 binds A, AS, Out, S, W; kernels/cuda/model/q4_projection.py:17-35, :53-54, :142-150
    assert lib.Kernel("q4_projection", M=8, N=256, K=512).arg_names == ["A", "AS", "Out", "S", "W"]
    assert lib.Kernel("q4_gemv", M=8, N=256, K=512, dynamic_rows=True).arg_names == ["A", "AS", "Out", "S", "W", "m"]
    big = lib.Kernel("q4_projection", M=1024, N=256, K=512, workspace=True, dynamic_rows=True)
    assert big.arg_names == ["A", "AS", "Out", "S", "W", "Workspace", "m"]
    assert big.workspace_bytes(64) == 0 and big.workspace_bytes(600) == 256 * 512
    # 511 rows are 8 tiles of 128 x 128 over 4 K steps: 4 workgroups with two partial slots each
    assert big.workspace_bytes(511) == 4 * 2 * 128 * 128 * 4 == big.workspace_bytes()
    # 65..511 rows: int32 partial tiles of a split launch where whole tiles would not spread evenly over the CUs
    mid = lib.Kernel("q4_projection", M=256, N=17408, K=5120, workspace=True, dynamic_rows=True)
    assert mid.workspace_bytes(128) == 512 * 2 * 128 * 128 * 4 == mid.workspace_bytes() and mid.workspace_bytes(64) == 0
    assert mid.geometry(128)[0][0] == 512 and lib.Kernel("q4_projection", M=128, N=17408, K=5120).geometry()[0] == (136, 1, 1)
    assert lib.Kernel("unpack_q4", N=256, K=512).arg_names == ["Output", "W"]
    shape = dict(M=8, N=256, K=512)
    for bad in (dict(magnitudes=[3, 10, 19, 31, 46, 67, 93]), dict(magnitudes=[3, 10, 19, 31, 46, 67, 93, 128]),
                dict(magnitudes=[0, 10, 19, 31, 46, 67, 93, 127]), dict(magnitudes=[3, 3, 19, 31, 46, 67, 93, 127]),
                dict(magnitudes=[3, 10, 19, 31, 46, 67, 93, 127, 127]), dict(K=500), dict(K=133120), dict(BN=48), dict(BK=384),
                dict(block_m=4), dict(stages=3), dict(group_m=3), dict(output_stride=255), dict(output_dtype="bfloat16")):
        with pytest.raises(lib.OrxError):
            lib.Kernel("q4_projection", **{**shape, **bad})
    for bad in (dict(block_m=9), dict(BN=32), dict(block_m=0)):
        with pytest.raises(lib.OrxError):
            lib.Kernel("q4_gemv", **{**shape, **bad})


# Values that the reference's factories take for a keyword (the `not in (...)` checks of kernels/cuda/model/e8p_q4.py:79-196,
# e8p_decode.py:43-49, integer_vq.py:87-99, int8_projection.py:33-39, q4_projection.py:143-149, e8p_exact.py:63-66,
# e8p_prefill.py:167-171, moe.py:77,216,562): each resolves here, on top of the other keywords of the same factory.
REFERENCE_VALUES = [
    ("e8p_q4_projection", "block_m", (8, 16, 32, 64, 96, 128, 192, 256)), ("e8p_q4_projection", "block_n", (32, 64, 128)),
    ("e8p_q4_projection", "split_k", (1, 2, 4)), ("e8p_q4_projection", "group_m", (0, 1, 2, 4, 8)),
    ("e8p_q4_projection", "packed_k", (0, 64, 128)), ("int8_projection", "block_m", (16, 32, 64, 128, 256)),
    ("int8_projection", "block_n", (64, 128)), ("int8_projection", "block_k", (64, 128)),
    ("int8_projection", "group_m", (0, 1, 2, 4, 8)), ("q4_projection", "block_m", (8, 16, 32, 64, 128)),
    ("q4_projection", "group_m", (0, 1, 2, 4, 8)), ("integer_vq", "block_m", (8, 16, 32, 64)), ("integer_vq", "block_n", (64, 128)),
    ("integer_vq", "num_stages", (1, 2)), ("integer_vq", "packed_k", (64, 128)), ("integer_vq_grouped", "block_m", (8, 16, 32, 64)),
    ("integer_vq_grouped", "packed_k", (64, 128)), ("e8p_decode_grouped", "packed_k", (64, 128)),
    ("e8p_decode_grouped", "block_n", (32, 64, 128)), ("e8p_decode_grouped", "split_k", (1, 2, 4)),
    ("e8p_exact_grouped", "block_m", (8, 16)), ("e8p_exact_grouped", "stages", (2, 3, 4)),
    ("integer_experts", "block_m", (8, 16, 32, 64, 128, 256)), ("integer_experts", "codec", ("w8", "e8p_q4")),
    ("expert_offsets", "block_m", (8, 16, 32, 64, 128, 256)), ("expert_tiles", "block_m", (8, 16, 32, 64, 128, 256)),
    ("expert_histogram_local", "block", (512, 1024, 2048)), ("router_topk_warp", "warps", (1, 2, 4)),
    ("activation_quantization", "threads", (128, 256, 512)),
]


@pytest.mark.parametrize("symbol,key,values", REFERENCE_VALUES, ids=[f"{s}-{k}" for s, k, _ in REFERENCE_VALUES])
def test_every_value_the_reference_factory_takes_resolves(symbol, key, values):
    for value in values:
        variant = dict(REFERENCE_KEYWORDS[symbol])
        variant[key] = value
        if symbol == "integer_experts" and (variant.get("codec") == "w8") and variant.get("block_m") == 8:
            variant["block_m"] = 16  # moe.py:80: W8 banks take no 8-row tiles
        lib.Kernel(symbol, **variant)
