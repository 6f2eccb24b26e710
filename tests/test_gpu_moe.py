"""GPU parity for the MoE expert path: routing, metadata, dispatch, grouped Q2A8 GEMM, combine."""
import numpy as np
import pytest
import torch

from oracle import reference as orc
from orinfer_amd import programs, workloads

from . import gpu_util as gu

pytestmark = pytest.mark.gpu
TABLE = orc.basis()
I32 = dict(dtype=torch.int32, device=gu.DEV)


@pytest.mark.parametrize("m,e,k", [(1, 512, 10), (8, 512, 10), (17, 37, 10), (512, 512, 10), (3, 5, 5), (1, 1, 1),
                                   (256, 128, 8)])
@pytest.mark.parametrize("renormalize", [False, True])
def test_router_topk_ties_zero_and_extremes(m, e, k, renormalize):
    # tests/cuda/operators/moe.py:25-57
    rng = np.random.default_rng(orc.SEED + m + e)
    logits = (rng.normal(size=(m, e)) * 5).astype(np.float32)
    logits[0] = 0
    if m > 1:
        logits[1] = -10000
        logits[1, -1] = 10000
    if m > 2:
        logits[2] = -1
        logits[2, :k] = 0
        logits[2, 0] = -0.0
    ids = torch.full((m, k), -1, **I32)
    prob = torch.full((m, k), float("nan"), dtype=torch.float32, device=gu.DEV)
    gu.kernel("router_topk", M=m, E=e, top_k=k, renormalize=renormalize)(IDs=ids, Logits=gu.dev(logits), Prob=prob)
    want_ids, want_prob = orc.router_topk(logits, k, renormalize)
    np.testing.assert_array_equal(gu.host(ids), want_ids)
    np.testing.assert_allclose(gu.host(prob), want_prob, atol=2e-6, rtol=2e-5)


@pytest.mark.parametrize("m,e,k,bm", [(256, 128, 8, 32), (37, 16, 4, 8), (1, 512, 10, 16), (300, 7, 3, 64), (5, 3, 3, 128)])
def test_routing_metadata_and_dispatch(m, e, k, bm):
    rng = np.random.default_rng(orc.SEED + m)
    weights = 1.0 / np.arange(1, e + 1) ** 1.1
    ids_np = np.stack([rng.choice(e, k, replace=False, p=weights / weights.sum()) for _ in range(m)]).astype(np.int32)
    ids = gu.dev(ids_np)
    counts = torch.full((e,), -1, **I32)
    relative = torch.full((m, k), -1, **I32)
    gu.kernel("expert_histogram", M=m, E=e, top_k=k)(Counts=counts, IDs=ids, RelativeSlot=relative)
    want_counts, want_rel = orc.expert_histogram(ids_np, e)
    np.testing.assert_array_equal(gu.host(counts), want_counts)
    np.testing.assert_array_equal(gu.host(relative), want_rel)
    rows = torch.full((e,), -1, **I32)
    tiles = torch.full((e,), -1, **I32)
    total = torch.full((1,), -1, **I32)
    gu.kernel("expert_offsets", E=e, block_m=bm)(Counts=counts, RowOffsets=rows, TileCount=total, TileOffsets=tiles)
    want_rows, want_tiles, want_total = orc.expert_offsets(want_counts, bm)
    np.testing.assert_array_equal(gu.host(rows), want_rows)
    np.testing.assert_array_equal(gu.host(tiles), want_tiles)
    np.testing.assert_array_equal(gu.host(total), want_total)
    cap = orc.tile_capacity(m * k, e, bm)
    tile_expert = torch.full((cap,), -1, **I32)
    tile_row = torch.full((cap,), -1, **I32)
    gu.kernel("expert_tiles", M=m, E=e, top_k=k, block_m=bm)(Counts=counts, TileExpert=tile_expert, TileOffsets=tiles,
                                                           TileRow=tile_row)
    want_te, want_tr = orc.expert_tiles(want_counts, want_tiles, bm, cap)
    np.testing.assert_array_equal(gu.host(tile_expert), want_te)  # untouched tail keeps the -1 sentinel
    np.testing.assert_array_equal(gu.host(tile_row), want_tr)
    h = 192
    a_q = rng.integers(-127, 128, (m, h), dtype=np.int8)
    a_s = rng.uniform(0.01, 0.02, (m, 1)).astype(np.float16)
    d = torch.zeros((m * k, h), dtype=torch.int8, device=gu.DEV)
    ds = torch.zeros((m * k, 1), dtype=torch.float16, device=gu.DEV)
    slot = torch.full((m, k), -1, **I32)
    gu.kernel("expert_dispatch", M=m, H=h, E=e, top_k=k, scale_group=h)(A=gu.dev(a_q), D=d, DS=ds, IDs=ids, RelativeSlot=relative,
                                                                       RowOffsets=rows, Scale=gu.dev(a_s), SlotMap=slot)
    want_d, want_ds, want_slot = orc.expert_dispatch(a_q, a_s, ids_np, want_rel, want_rows)
    np.testing.assert_array_equal(gu.host(slot), want_slot)
    np.testing.assert_array_equal(gu.host(d), want_d)
    np.testing.assert_array_equal(gu.host(ds), want_ds)


@pytest.mark.parametrize("m,e,k,bm", [(256, 128, 8, 32), (37, 16, 4, 8), (1, 512, 10, 16), (300, 7, 3, 64), (5, 3, 3, 128),
                                      (1024, 1024, 10, 16), (17, 64, 64, 8), (40, 100, 100, 16)])
@pytest.mark.parametrize("repeats", [False, True], ids=["unique-routes", "repeated-routes"])
def test_route_metadata_one_launch(m, e, k, bm, repeats):
    """The fused form must write exactly what histogram + offsets + tiles write, also for dynamic
    rows and when a token names one expert twice (ranked by route order)."""
    rng = np.random.default_rng(orc.SEED + m + e)
    ids_np = np.stack([rng.choice(e, k, replace=False) for _ in range(m)]).astype(np.int32)
    if repeats and k > 1:
        ids_np[:, -1] = ids_np[:, 0]
        ids_np[0, :] = ids_np[0, 0]
    cap_rows = m + 3
    kern = gu.kernel("route_metadata", M=cap_rows, E=e, top_k=k, block_m=bm, dynamic_rows=True)
    padded = np.full((cap_rows, k), 0, np.int32)
    padded[:m] = ids_np
    cap = orc.tile_capacity(cap_rows * k, e, bm)
    out = {name: torch.full(shape, -1, **I32) for name, shape in
           (("Counts", (e,)), ("RelativeSlot", (cap_rows, k)), ("RowOffsets", (e,)), ("TileCount", (1,)),
            ("TileExpert", (cap,)), ("TileOffsets", (e,)), ("TileRow", (cap,)))}
    kern(IDs=gu.dev(padded), m=m, **out)
    want_counts, want_rel = orc.expert_histogram(ids_np, e)
    want_rows, want_tiles, want_total = orc.expert_offsets(want_counts, bm)
    want_te, want_tr = orc.expert_tiles(want_counts, want_tiles, bm, cap)
    np.testing.assert_array_equal(gu.host(out["Counts"]), want_counts)
    np.testing.assert_array_equal(gu.host(out["RelativeSlot"])[:m], want_rel)
    assert (gu.host(out["RelativeSlot"])[m:] == -1).all()
    np.testing.assert_array_equal(gu.host(out["RowOffsets"]), want_rows)
    np.testing.assert_array_equal(gu.host(out["TileOffsets"]), want_tiles)
    np.testing.assert_array_equal(gu.host(out["TileCount"]), want_total)
    np.testing.assert_array_equal(gu.host(out["TileExpert"]), want_te)
    np.testing.assert_array_equal(gu.host(out["TileRow"]), want_tr)


@pytest.mark.parametrize("algorithm", ["auto", "mfma"])
@pytest.mark.parametrize("packed_k", [128, 64, 0])
@pytest.mark.parametrize("bm", [32, 64, 128])
def test_grouped_q2_gemm_counts_tiles_and_masks(bm, packed_k, algorithm):
    # count mixes in the spirit of tests/cuda/operators/e8p_exact.py:141-198: empty experts,
    # single rows, exact tile multiples, tails, one hot expert
    rng = np.random.default_rng(orc.SEED + bm)
    e, n, k = 9, 200, 384
    counts_np = np.array([0, 1, bm, bm + 1, 0, 3 * bm - 1, 7, 0, 2], np.int32)
    rows = int(counts_np.sum())
    codes = rng.integers(0, 65536, (e, n, k // 8), dtype=np.uint16)
    ws = rng.uniform(0.005, 0.02, (e, n)).astype(np.float16)
    a_q = rng.integers(-127, 128, (rows, k), dtype=np.int8)
    a_q[0, :2] = [-128, 127]
    a_s = rng.uniform(0.01, 0.03, rows).astype(np.float16)
    offsets_np, tile_offsets, total = orc.expert_offsets(counts_np, bm)
    cap = orc.tile_capacity(rows, e, bm)
    te, tr = orc.expert_tiles(counts_np, tile_offsets, bm, cap)
    stored = codes if packed_k == 0 else np.stack([orc.q2_pack_k128(c) for c in codes])
    if packed_k == 64:  # e8p_decode.py:43,62: blocks of 64 codes per channel
        stored = orc.q2_repack_k64(stored)
    out = torch.full((rows + 1, n), 55.0, dtype=torch.float16, device=gu.DEV)
    kern = gu.kernel("e8p_decode_grouped", rows=rows, E=e, tiles=cap, N=n, K=k, block_m=bm, packed_k=packed_k,
                     algorithm=algorithm)
    counts, offsets = gu.dev(counts_np), gu.dev(offsets_np)
    tile_count = gu.dev(total)
    args = dict(A=gu.dev(a_q), AS=gu.dev(a_s), Book=gu.book(), C=out, Counts=counts, Offsets=offsets, P=gu.dev(stored),
                TileCount=tile_count, TileExpert=gu.dev(te), TileRow=gu.dev(tr), WS=gu.dev(ws))
    kern(**args)
    w = np.stack([orc.q2_integers(c, TABLE) for c in codes])
    want = orc.grouped_project(a_q, a_s[:, None], w, ws, counts_np, offsets_np)
    got = gu.host(out)
    np.testing.assert_array_equal(got[:rows], want)
    assert (got[rows] == 55).all()
    # routing masks (tests/cuda/operators/e8p_decode.py:100-137): a zero tile count leaves C untouched
    out.fill_(55)
    tile_count.zero_()
    kern(**args)
    assert bool((out == 55).all())
    # zeroing one expert's count skips exactly its rows
    tile_count.copy_(gu.dev(total))
    hot = 5
    counts[hot] = 0
    kern(**args)
    got = gu.host(out)
    lo, hi = offsets_np[hot], offsets_np[hot] + counts_np[hot]
    assert (got[lo:hi] == 55).all()
    np.testing.assert_array_equal(got[:lo], want[:lo])
    np.testing.assert_array_equal(got[hi:rows], want[hi:])


# Cases of the resident routed kernel (one 16-wave workgroup per CU, units of one tile x 512
# channels).  With 256 CUs: whole units plus a K-split rest for three ring depths and both split
# widths, a launch that is K-split only, one extra unit for some workgroups, and runs of three
# units that change tile in the middle.
RESIDENT_CASES = {
    "units-and-rest-k512": dict(e=64, n=1536, k=512, high=70),
    "units-and-rest-k384": dict(e=9, n=14848, k=384, counts=[0, 1, 32, 33, 0, 95, 7, 0, 2]),
    "rest-only-k256": dict(e=40, n=512, k=256, high=40),
    "extra-unit-k2048": dict(e=50, n=1024, k=2048, high=20),
    "tile-change-k512": dict(e=128, n=1536, k=512, high=80),
}


@pytest.mark.parametrize("packed_k", [128, 0])
@pytest.mark.parametrize("case", list(RESIDENT_CASES))
def test_grouped_q2_resident_kernel(case, packed_k):
    spec = RESIDENT_CASES[case]
    e, n, k, bm = spec["e"], spec["n"], spec["k"], 32
    rng = np.random.default_rng(orc.SEED + e + k)
    if "counts" in spec:
        counts_np = np.array(spec["counts"], np.int32)
    else:
        counts_np = rng.integers(0, spec["high"] + 1, e).astype(np.int32)
        counts_np[rng.integers(0, e, max(1, e // 10))] = 0
    rows = int(counts_np.sum())
    codes = rng.integers(0, 65536, (e, n, k // 8), dtype=np.uint16)
    ws = rng.uniform(0.005, 0.02, (e, n)).astype(np.float16)
    a_q = rng.integers(-127, 128, (rows, k), dtype=np.int8)
    a_q[0, :2] = [-128, 127]
    a_s = rng.uniform(0.01, 0.03, rows).astype(np.float16)
    offsets_np, tile_offsets, total = orc.expert_offsets(counts_np, bm)
    cap = orc.tile_capacity(rows, e, bm)
    te, tr = orc.expert_tiles(counts_np, tile_offsets, bm, cap)
    stored = codes if packed_k == 0 else np.stack([orc.q2_pack_k128(c) for c in codes])
    out = torch.full((rows + 1, n), 55.0, dtype=torch.float16, device=gu.DEV)
    kern = gu.kernel("e8p_decode_grouped", rows=rows, E=e, tiles=cap, N=n, K=k, block_m=bm, packed_k=packed_k,
                     algorithm="resident")
    assert tuple(kern.geometry()[1])[0] == 1024
    counts = gu.dev(counts_np)
    tile_count = gu.dev(total)
    args = dict(A=gu.dev(a_q), AS=gu.dev(a_s), Book=gu.book(), C=out, Counts=counts, Offsets=gu.dev(offsets_np),
                P=gu.dev(stored), TileCount=tile_count, TileExpert=gu.dev(te), TileRow=gu.dev(tr), WS=gu.dev(ws))
    kern(**args)
    w = np.stack([orc.q2_integers(c, TABLE) for c in codes])
    want = orc.grouped_project(a_q, a_s[:, None], w, ws, counts_np, offsets_np)
    got = gu.host(out)
    np.testing.assert_array_equal(got[:rows], want)
    assert (got[rows] == 55).all()
    # the streaming kernel gives the same bytes
    other = torch.full_like(out, 55.0)
    gu.kernel("e8p_decode_grouped", rows=rows, E=e, tiles=cap, N=n, K=k, block_m=bm, packed_k=packed_k,
              algorithm="stream")(**{**args, "C": other})
    assert torch.equal(out, other)
    # a zero tile count leaves C untouched; a zeroed expert count skips exactly its rows
    out.fill_(55)
    tile_count.zero_()
    kern(**args)
    assert bool((out == 55).all())
    tile_count.copy_(gu.dev(total))
    hot = int(np.argmax(counts_np))
    counts[hot] = 0
    kern(**args)
    got = gu.host(out)
    lo, hi = offsets_np[hot], offsets_np[hot] + counts_np[hot]
    assert (got[lo:hi] == 55).all()
    np.testing.assert_array_equal(got[:lo], want[:lo])
    np.testing.assert_array_equal(got[hi:rows], want[hi:])


def test_grouped_resident_rejects_shapes_it_cannot_take():
    for bad in (dict(N=200, K=384), dict(N=256, K=128), dict(N=256, K=3072), dict(N=256, K=512, block_m=64)):
        variant = dict(rows=64, E=4, tiles=6, block_m=32, packed_k=128, algorithm="resident")
        variant.update(bad)
        with pytest.raises(Exception, match="resident"):
            gu.kernel("e8p_decode_grouped", **variant)


@pytest.mark.parametrize("m,h,slots", [(1, 2560, 10), (8, 2560, 80), (17, 257, 37), (512, 2560, 5120)])
def test_combine_invalid_slots_and_shared_expert(m, h, slots):
    # tests/cuda/operators/moe.py:98-118
    rng = np.random.default_rng(orc.SEED + m)
    k = 10
    ex = rng.normal(size=(slots, h)).astype(np.float16)
    sm = rng.integers(0, slots, (m, k)).astype(np.int32)
    sm[0, :2] = [-1, slots]
    prob = rng.dirichlet(np.ones(k), m).astype(np.float32)
    shared = rng.normal(size=(m, h)).astype(np.float16)
    gate = rng.normal(size=m).astype(np.float16)
    out = torch.empty((m, h), dtype=torch.float16, device=gu.DEV)
    kern = gu.kernel("moe_combine", M=m, H=h, slots=slots, top_k=k)
    kern(Expert=gu.dev(ex), Output=out, Prob=gu.dev(prob), Shared=gu.dev(shared), SharedGate=gu.dev(gate), SlotMap=gu.dev(sm))
    want = orc.moe_combine(ex, sm, prob, shared, gate).astype(np.float32)
    got = gu.host(out).astype(np.float32)
    assert (np.abs(got - want) <= 1e-2 + 1e-3 * np.abs(want)).all()
    rel = np.linalg.norm(got - want) / np.linalg.norm(want)
    assert rel < 1e-3
    kern(Expert=gu.dev(ex), Output=out, Prob=gu.dev(prob), Shared=None, SharedGate=None, SlotMap=gu.dev(sm))
    want = orc.moe_combine(ex, sm, prob).astype(np.float32)
    got = gu.host(out).astype(np.float32)
    assert (np.abs(got - want) <= 1e-2 + 1e-3 * np.abs(want)).all()
    # an output that is only 8-byte aligned takes the element-wise stores: same bytes
    flat = torch.zeros(m * h + 8, dtype=torch.float16, device=gu.DEV)
    shifted = flat[4 : 4 + m * h].view(m, h)
    kern(Expert=gu.dev(ex), Output=shifted, Prob=gu.dev(prob), Shared=None, SharedGate=None, SlotMap=gu.dev(sm))
    assert torch.equal(shifted, out) and not flat[:4].any() and not flat[4 + m * h :].any()


def run_layer(c, bm, packed_k=128, fused_dispatch=True, signs=None, fused_stages=False, **more):
    layer = programs.MoeLayer(c["tokens"], c["experts"], c["top_k"], c["hidden"], c["intermediate"], c["gate_up"],
                              c["gate_up_scales"], c["down"], c["down_scales"], block_m=bm, packed_k=packed_k,
                              fused_dispatch=fused_dispatch, signs=signs, fused_stages=fused_stages,
                              keep_intermediates=True, **more)
    assert fused_stages is None or layer.fused_stages == bool(fused_stages)
    layer.run(gu.dev(c["x"]), gu.dev(c["logits"]))
    gu.sync()
    return layer


def check_layer(c, layer, bm):
    e = c["experts"]
    ids, prob = orc.router_topk(c["logits"], c["top_k"], True)
    np.testing.assert_array_equal(gu.host(layer.ids), ids)
    np.testing.assert_allclose(gu.host(layer.prob), prob, atol=2e-6, rtol=2e-5)
    counts, rel = orc.expert_histogram(ids, e)
    rows, tiles, total = orc.expert_offsets(counts, bm)
    np.testing.assert_array_equal(gu.host(layer.counts), counts)
    np.testing.assert_array_equal(gu.host(layer.row_offsets), rows)
    np.testing.assert_array_equal(gu.host(layer.tile_count), total)
    a_q, a_s = orc.a8(c["x"]) if layer.signs is None else orc.rotate_a8(c["x"], gu.host(layer.signs))
    if layer.signs is None and not layer.fused_dispatch:  # else the rows are quantised on their way to the slots
        np.testing.assert_array_equal(gu.host(layer.a_q), a_q)
    d, ds, slot = orc.expert_dispatch(a_q, a_s, ids, rel, rows)
    np.testing.assert_array_equal(gu.host(layer.slot_map), slot)
    if layer.fused_stages:  # the rows stay per token; the projection gathers them through the slot -> token map
        np.testing.assert_array_equal(gu.host(layer.a_q), a_q)
        np.testing.assert_array_equal(gu.host(layer.a_s), a_s)
        token_of = np.empty(slot.size, np.int32)
        token_of[slot.ravel()] = np.repeat(np.arange(slot.shape[0], dtype=np.int32), slot.shape[1])
        np.testing.assert_array_equal(gu.host(layer.slot_token), token_of)
    else:
        np.testing.assert_array_equal(gu.host(layer.d), d)
        np.testing.assert_array_equal(gu.host(layer.ds), ds)
    w1 = np.stack([orc.q2_integers(x, TABLE) for x in c["gate_up"]])
    w2 = np.stack([orc.q2_integers(x, TABLE) for x in c["down"]])
    gate_up = orc.grouped_project(d, ds, w1, c["gate_up_scales"], counts, rows)
    np.testing.assert_array_equal(gu.host(layer.gate_up_out), gate_up)  # fp16 bit-exact: same integers, same multiplies
    # SwiGLU uses exp(): from here on check each stage exactly on the GPU's own input, and the
    # whole layer against the oracle chain within the output tolerance
    act_gpu_q, act_gpu_s = gu.host(layer.h_q), gu.host(layer.h_s)
    act = orc.swiglu_fp16(gate_up)
    want_q, want_s = orc.a8(act)
    assert (act_gpu_q == want_q).mean() > 0.999 and (act_gpu_s == want_s).mean() > 0.99
    if layer.fused_stages:
        # the fp16 values between the two projections and their per-slot maxima; the codes are the
        # A8 rule applied to exactly those values
        act_gpu = gu.host(layer.act)
        assert (act_gpu == act).mean() > 0.999
        np.testing.assert_array_equal(gu.host(layer.row_max).view(np.float32), np.abs(act_gpu.astype(np.float32)).max(1))
        exact_q, exact_s = orc.a8(act_gpu)
        np.testing.assert_array_equal(act_gpu_q, exact_q)
        np.testing.assert_array_equal(act_gpu_s, exact_s)
    down = orc.grouped_project(act_gpu_q, act_gpu_s, w2, c["down_scales"], counts, rows)
    np.testing.assert_array_equal(gu.host(layer.down_out), down)
    got = gu.host(layer.out).astype(np.float32)
    staged = orc.moe_combine(down, slot, gu.host(layer.prob)).astype(np.float32)
    assert (np.abs(got - staged) <= 1e-2 + 1e-3 * np.abs(staged)).all()
    full = orc.moe_layer(c["x"], c["logits"], c["gate_up"], c["gate_up_scales"], c["down"], c["down_scales"], TABLE,
                         c["top_k"], bm, signs=None if layer.signs is None else gu.host(layer.signs))["out"].astype(np.float32)
    rel_l2 = np.linalg.norm(got - full) / np.linalg.norm(full)
    assert rel_l2 < 0.003  # flash_next_quantized.py:117-135 accepts the expert FFN at this bar
    # element by element against the whole oracle chain, at the output tolerance (1e-3 relative + 1e-2 absolute): the
    # only arithmetic that is not bit-exact in between is exp() inside SwiGLU, which moves a few A8 codes by one step
    error = np.abs(got - full)
    beyond = error > 1e-2 + 1e-3 * np.abs(full)
    assert not beyond.any(), (int(beyond.sum()), beyond.size, float(error.max()))


def test_moe_layer_small_end_to_end():
    c = workloads.config3(tokens=40, experts=16, top_k=4, hidden=256, intermediate=128)
    for bm in (32, 64):
        check_layer(c, run_layer(c, bm), bm)
    check_layer(c, run_layer(c, 32, fused_dispatch=False), 32)  # quantiser and dispatch as two launches
    signs = np.random.default_rng(3).choice(np.array([-1, 1], np.int8), c["hidden"])
    check_layer(c, run_layer(c, 32, signs=signs), 32)  # rotated input: rotation, A8 and scatter in one launch
    # five launches: no dispatch copy, no SwiGLU->A8 launch between the two expert projections
    wide = workloads.config3(tokens=70, experts=16, top_k=4, hidden=768, intermediate=384)  # K/128 = 6 and 3
    for packed_k in (128, 0):
        check_layer(wide, run_layer(wide, 32, packed_k=packed_k, fused_stages=True, grouped_algorithm="resident"), 32)


def test_config3_full_size_end_to_end():
    c = workloads.config3()
    check_layer(c, run_layer(c, 32), 32)


def test_config3_full_size_end_to_end_in_five_launches():
    """What `MoeLayer` runs by default at this size: router that also quantises the token rows, metadata
    with the slot tables, gate_up that gathers the rows by slot and ends in SwiGLU, down that quantises the
    fp16 rows while it stages them, combine."""
    c = workloads.config3()
    layer = run_layer(c, 32, fused_stages=None)
    assert layer.fused_stages
    check_layer(c, layer, 32)
    lean = programs.MoeLayer(c["tokens"], c["experts"], c["top_k"], c["hidden"], c["intermediate"], c["gate_up"],
                             c["gate_up_scales"], c["down"], c["down_scales"], block_m=32)  # no intermediates kept
    lean.run(gu.dev(c["x"]), gu.dev(c["logits"]))
    gu.sync()
    assert lean.fused_stages and torch.equal(lean.out, layer.out)


def test_moe_layer_graph_replay_with_new_routing():
    c = workloads.config3(tokens=64, experts=32, top_k=4, hidden=256, intermediate=128)
    layer = programs.MoeLayer(c["tokens"], c["experts"], c["top_k"], c["hidden"], c["intermediate"], c["gate_up"],
                              c["gate_up_scales"], c["down"], c["down_scales"], block_m=32)
    x, logits = gu.dev(c["x"]), gu.dev(c["logits"])
    layer.run(x, logits)
    gu.sync()
    eager = layer.out.clone()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            layer.run(x, logits, stream=stream.cuda_stream)
    for step in range(3):
        layer.out.fill_(float("nan"))
        graph.replay()
        gu.sync()
        assert torch.equal(layer.out, eager)
        layer.counts.fill_(-7)  # stale metadata must be rebuilt by the replay itself
    rng = np.random.default_rng(5)
    logits.copy_(gu.dev(rng.normal(size=c["logits"].shape).astype(np.float32)))
    graph.replay()
    gu.sync()
    replayed = layer.out.clone()
    layer.run(x, logits)
    gu.sync()
    assert torch.equal(layer.out, replayed)
    assert not torch.equal(replayed, eager)


# ---- single-token routes: every route indexes its expert's bank directly -----------------------
def route_case(rng, e, routes, n, k, table, shared):
    codes = rng.integers(0, 65536, (e, n, k // 8), dtype=np.uint16)
    weights = np.stack([orc.q2_integers(c, table) for c in codes])
    stored = np.stack([orc.q2_pack_k128(c) for c in codes])
    rows = 1 if shared else routes
    a_q = rng.integers(-128, 128, (rows, k), dtype=np.int8)
    return codes, weights, stored, a_q


@pytest.mark.parametrize("n,k", [(65, 256), (1280, 2560), (2560, 640)])
@pytest.mark.parametrize("shared", [True, False])
def test_route_gemv_random_even_tables(n, k, shared):
    """The reference's own check (tests/cuda/operators/flash_mtp_optimization.py:131-175): a random
    even table (zeros and negative bytes included), int8 rows down to -128, power-of-two scales, a
    guard row behind the output, then other ids and negated rows through the same handle."""
    rng = np.random.default_rng(20261002 + n)
    e, routes = 12, 3
    table = (rng.integers(-63, 64, (256, 8)) * 2).astype(np.int8)
    table[5] = 0
    _, weights, stored, a_q = route_case(rng, e, routes, n, k, table, shared)
    rows = a_q.shape[0]
    ws = np.full((e, n), 0.015625, np.float16)
    scale = np.full(rows, 0.0078125, np.float16)
    ids = np.array([[11, 2, 7]], np.int32)
    out = torch.full((routes + 1, n), 91.0, dtype=torch.float16, device=gu.DEV)
    kern = gu.kernel("integer_e8p_gemv", E=e, routes=routes, N=n, K=k, shared_input=shared)
    d_a, d_ids = gu.dev(a_q), gu.dev(ids)
    args = dict(A=d_a, AS=gu.dev(scale), Book=gu.dev(orc.raw_table_words(table)), C=out, IDs=d_ids, P=gu.dev(stored),
                WS=gu.dev(ws))
    kern(**args)
    np.testing.assert_array_equal(gu.host(out)[:routes], orc.route_project(a_q, scale, weights, ws, ids, shared))
    assert (gu.host(out)[routes] == 91).all()
    a_q = np.where(a_q == -128, 127, -a_q).astype(np.int8)
    ids = np.array([[0, 9, 3]], np.int32)
    d_a.copy_(gu.dev(a_q))
    d_ids.copy_(gu.dev(ids))
    kern(**args)
    np.testing.assert_array_equal(gu.host(out)[:routes], orc.route_project(a_q, scale, weights, ws, ids, shared))
    assert (gu.host(out)[routes] == 91).all()


@pytest.mark.parametrize("n,k,shared", [(1024, 2048, True), (2048, 512, False)])
def test_route_gemv_production_table_and_repeated_experts(n, k, shared):
    # the shapes of one routed token: gate/up from the shared row, down from one row per route
    rng = np.random.default_rng(orc.SEED + n)
    e, routes = 128, 8
    codes = rng.integers(0, 65536, (e, n, k // 8), dtype=np.uint16)
    stored = np.stack([orc.q2_pack_k128(c) for c in codes])
    rows = 1 if shared else routes
    a_q = rng.integers(-127, 128, (rows, k), dtype=np.int8)
    a_s = rng.uniform(0.01, 0.03, rows).astype(np.float16)
    ws = rng.uniform(0.005, 0.02, (e, n)).astype(np.float16)
    ids = np.array([[127, 0, 5, 5, 64, 31, 127, 2]], np.int32)
    out = torch.full((routes + 1, n), 91.0, dtype=torch.float16, device=gu.DEV)
    kern = gu.kernel("integer_e8p_gemv", E=e, routes=routes, N=n, K=k, shared_input=shared, block_n=16)
    d_ids = gu.dev(ids)
    args = dict(A=gu.dev(a_q), AS=gu.dev(a_s), Book=gu.dev(orc.raw_table_words(TABLE)), C=out, IDs=d_ids,
                P=gu.dev(stored), WS=gu.dev(ws))
    kern(**args)
    used = sorted(set(ids.ravel().tolist()))
    weights = np.zeros((e, n, k), np.int8)
    for x in used:
        weights[x] = orc.q2_integers(codes[x], TABLE)
    want = orc.route_project(a_q, a_s, weights, ws, ids, shared)
    np.testing.assert_array_equal(gu.host(out)[:routes], want)
    # the routed batch of one token through the grouped kernel gives the same bytes
    if shared:
        counts = np.bincount(ids.ravel(), minlength=e).astype(np.int32)
        offsets, tile_offsets, total = orc.expert_offsets(counts, 32)
        cap = orc.tile_capacity(routes, e, 32)
        te, tr = orc.expert_tiles(counts, tile_offsets, 32, cap)
        grouped = torch.zeros((routes, n), dtype=torch.float16, device=gu.DEV)
        gu.kernel("e8p_decode_grouped", rows=routes, E=e, tiles=cap, N=n, K=k, block_m=32)(
            A=gu.dev(np.repeat(a_q, routes, 0)), AS=gu.dev(np.repeat(a_s, routes)), Book=gu.book(), C=grouped,
            Counts=gu.dev(counts), Offsets=gu.dev(offsets), P=gu.dev(stored), TileCount=gu.dev(total),
            TileExpert=gu.dev(te), TileRow=gu.dev(tr), WS=gu.dev(ws))
        order = np.argsort(ids.ravel(), kind="stable")
        np.testing.assert_array_equal(gu.host(grouped), want[order])
    # an id outside the bank leaves its row as it was
    out.fill_(91)
    bad = ids.copy()
    bad[0, 3], bad[0, 6] = e, -1
    d_ids.copy_(gu.dev(bad))
    kern(**args)
    got = gu.host(out)
    assert (got[3] == 91).all() and (got[6] == 91).all() and (got[routes] == 91).all()
    keep = [0, 1, 2, 4, 5, 7]
    np.testing.assert_array_equal(got[keep], want[keep])


def test_route_gemv_quantises_a_shared_fp16_row():
    rng = np.random.default_rng(orc.SEED + 55)
    e, routes, n, k = 16, 4, 200, 2304
    codes = rng.integers(0, 65536, (e, n, k // 8), dtype=np.uint16)
    weights = np.stack([orc.q2_integers(c, TABLE) for c in codes])
    stored = gu.dev(np.stack([orc.q2_pack_k128(c) for c in codes]))
    ws = rng.uniform(0.005, 0.02, (e, n)).astype(np.float16)
    ids = np.array([[3, 15, 0, 3]], np.int32)
    kern = gu.kernel("integer_e8p_gemv", E=e, routes=routes, N=n, K=k, shared_input=True, input_dtype="float16")
    out = torch.full((routes + 1, n), 91.0, dtype=torch.float16, device=gu.DEV)
    scale = torch.full((2,), 5.0, dtype=torch.float16, device=gu.DEV)
    for case in range(3):
        x = rng.normal(size=(1, k)).astype(np.float16)
        if case == 1:
            x[0, :3] = [700, -700, 1e-7]
        if case == 2:
            x[:] = 0
        kern(A=gu.dev(x), AS=scale, Book=gu.dev(orc.raw_table_words(TABLE)), C=out, IDs=gu.dev(ids), P=stored, WS=gu.dev(ws))
        a_q, a_s = orc.a8(x)
        np.testing.assert_array_equal(gu.host(scale)[:1], a_s[:, 0])
        np.testing.assert_array_equal(gu.host(out)[:routes], orc.route_project(a_q, a_s[:, 0], weights, ws, ids, True))
        assert float(gu.host(scale)[1]) == 5.0 and (gu.host(out)[routes] == 91).all()
    with pytest.raises(Exception):
        gu.kernel("integer_e8p_gemv", E=e, routes=routes, N=n, K=k, shared_input=False, input_dtype="float16")


def test_route_gemv_refuses_bad_variants():
    for variant in (dict(E=4, routes=2, N=64, K=192, shared_input=True),
                    dict(E=4, routes=2, N=64, K=256),
                    dict(E=0, routes=2, N=64, K=256, shared_input=False),
                    dict(E=4, routes=2, N=64, K=256, shared_input=False, block_n=32),
                    dict(E=4, routes=2, N=64, K=131072, shared_input=False)):
        with pytest.raises(Exception):
            gu.kernel("integer_e8p_gemv", **variant)


@pytest.mark.parametrize("experts,top_k,capacity", [(512, 10, 11), (128, 8, 8), (16, 16, 20), (300, 1, 4)])
def test_single_route_metadata_matches_oracle(experts, top_k, capacity):
    rng = np.random.default_rng(orc.SEED + experts)
    kern = gu.kernel("single_route_metadata", E=experts, top_k=top_k, capacity=capacity)
    out = {name: torch.full((size,), 77, dtype=torch.int32, device=gu.DEV)
           for name, size in (("Counts", experts), ("Relative", top_k), ("Offsets", experts), ("TileOffsets", experts),
                              ("TileExpert", capacity), ("TileRow", capacity), ("TileCount", 1))}
    d_ids = torch.zeros((1, top_k), dtype=torch.int32, device=gu.DEV)
    for _ in range(2):  # the same handle and buffers with other ids
        ids = rng.permutation(experts)[:top_k].astype(np.int32)[None, :]
        d_ids.copy_(gu.dev(ids))
        kern(IDs=d_ids, **out)
        counts, relative, offsets, tile_offsets, tile_expert, tile_row, tile_count = orc.single_route_metadata(
            ids, experts, capacity)
        np.testing.assert_array_equal(gu.host(out["Counts"]), counts)
        np.testing.assert_array_equal(gu.host(out["Relative"]), relative[0])
        np.testing.assert_array_equal(gu.host(out["Offsets"]), offsets)
        np.testing.assert_array_equal(gu.host(out["TileOffsets"]), tile_offsets)
        np.testing.assert_array_equal(gu.host(out["TileCount"]), tile_count)
        np.testing.assert_array_equal(gu.host(out["TileExpert"])[:top_k], tile_expert[:top_k])
        np.testing.assert_array_equal(gu.host(out["TileRow"])[:top_k], tile_row[:top_k])
        # the unused tile tail is preserved (moe.py:663)
        assert (gu.host(out["TileExpert"])[top_k:] == 77).all() and (gu.host(out["TileRow"])[top_k:] == 77).all()
    for variant in (dict(E=4, top_k=5), dict(E=8, top_k=4, capacity=3), dict(E=0)):
        with pytest.raises(Exception):
            gu.kernel("single_route_metadata", **variant)


@pytest.mark.parametrize("experts,hot_m,cold_m,cold_rows", [(23, 16, 4, 8), (300, 32, 8, 8), (128, 64, 16, 100)])
def test_expert_partition_matches_oracle(experts, hot_m, cold_m, cold_rows):
    rng = np.random.default_rng(orc.SEED + experts + hot_m)
    m, top_k = 96, min(8, experts)
    ids, _ = orc.router_topk(rng.normal(size=(m, experts)).astype(np.float32), top_k)
    counts, _ = orc.expert_histogram(ids, experts)
    counts[0] = cold_rows  # on the threshold: cold
    hot_cap = orc.tile_capacity(m * top_k, experts, hot_m)
    cold_cap = orc.tile_capacity(m * top_k, experts, cold_m)
    want = orc.expert_partition(counts, hot_m, cold_m, cold_rows, hot_cap, cold_cap)
    sizes = dict(RowOffsets=experts, TileOffsets=experts, ColdOffsets=experts, TileCount=1, ColdCount=1,
                 TileExpert=hot_cap, TileRow=hot_cap, ColdExpert=cold_cap, ColdRow=cold_cap)
    out = {name: torch.full((size,), -1, dtype=torch.int32, device=gu.DEV) for name, size in sizes.items()}
    d_counts = gu.dev(counts)
    shape = dict(experts=experts, hot_m=hot_m, cold_m=cold_m, cold_rows=cold_rows)
    gu.kernel("expert_partition_offsets", **shape)(
        Counts=d_counts, **{name: out[name] for name in ("ColdCount", "ColdOffsets", "RowOffsets", "TileCount", "TileOffsets")})
    gu.kernel("expert_partition_tiles", M=m, top_k=top_k, dynamic_rows=True, **shape)(
        Counts=d_counts, m=m,
        **{name: out[name] for name in ("ColdExpert", "ColdOffsets", "ColdRow", "TileExpert", "TileOffsets", "TileRow")})
    for name in sizes:
        np.testing.assert_array_equal(gu.host(out[name]), want[name], err_msg=name)
    assert int(want["TileCount"][0]) > 0 or cold_rows >= counts.max()
    for variant in (dict(experts=0, hot_m=8, cold_m=8, cold_rows=1), dict(experts=4, hot_m=8, cold_m=0, cold_rows=1),
                    dict(experts=4, hot_m=8, cold_m=8)):
        with pytest.raises(Exception):
            gu.kernel("expert_partition_offsets", **variant)
    with pytest.raises(Exception):
        gu.kernel("expert_partition_tiles", M=4, top_k=9, experts=8, hot_m=8, cold_m=8, cold_rows=2)


# ---- routed Q4 / W8 banks (integer_experts) -----------------------------------------------------
@pytest.mark.parametrize("codec,bm", [("e8p_q4", 8), ("e8p_q4", 16), ("e8p_q4", 64), ("e8p_q4", 128), ("w8", 16),
                                      ("w8", 32), ("w8", 128), ("e8p_q4", 256), ("w8", 256)])
def test_integer_experts_q4_and_w8_banks(codec, bm):
    rng = np.random.default_rng(orc.SEED + bm + len(codec))
    e, n, k, top_k = 9, 200, 384, 3
    m = 300 if bm == 256 else 40  # 256-row lists (moe.py:77): the hot expert fills both halves of a listed tile and a tail
    logits = rng.normal(size=(m, e)).astype(np.float32)
    logits[:, 4] = -50  # an expert nobody picks
    logits[:, 2] += 3   # a hot one
    ids, _ = orc.router_topk(logits, top_k)
    counts_np, relative = orc.expert_histogram(ids, e)
    rows = m * top_k
    offsets_np, tile_offsets, total = orc.expert_offsets(counts_np, bm)
    cap = orc.tile_capacity(rows, e, bm)
    te, tr = orc.expert_tiles(counts_np, tile_offsets, bm, cap)
    if codec == "e8p_q4":
        packed = rng.integers(0, 2**32, (e, n, k // 8), dtype=np.uint32)
        weights = np.stack([orc.q4_integers(x, TABLE) for x in packed])
        stored = np.stack([orc.q4_pack_k(x, 128) for x in packed])
    else:
        weights = rng.integers(-128, 128, (e, n, k), dtype=np.int8)
        stored = weights
    ws = rng.uniform(0.005, 0.02, (e, n)).astype(np.float16)
    a_q = rng.integers(-127, 128, (rows, k), dtype=np.int8)
    a_q[0, :2] = [-128, 127]
    a_s = rng.uniform(0.01, 0.03, rows).astype(np.float16)
    out = torch.full((rows + 1, n), 55.0, dtype=torch.float16, device=gu.DEV)
    kern = gu.kernel("integer_experts", M=m, N=n, K=k, E=e, top_k=top_k, codec=codec, block_m=bm,
                     block_n=64 if codec == "w8" else 32)
    counts, tile_count = gu.dev(counts_np), gu.dev(total)
    args = dict(A=gu.dev(a_q), AS=gu.dev(a_s), Book=gu.book(), Counts=counts, Offsets=gu.dev(offsets_np), Out=out,
                TileCount=tile_count, TileExpert=gu.dev(te), TileRow=gu.dev(tr), W=gu.dev(stored), WS=gu.dev(ws))
    kern(**args)
    want = orc.grouped_project(a_q, a_s[:, None], weights, ws, counts_np, offsets_np)
    got = gu.host(out)
    np.testing.assert_array_equal(got[:rows], want)
    assert (got[rows] == 55).all()
    # a zero tile count leaves the output untouched; zeroing one expert's count skips exactly its rows
    out.fill_(55)
    tile_count.zero_()
    kern(**args)
    assert bool((out == 55).all())
    tile_count.copy_(gu.dev(total))
    counts[2] = 0
    kern(**args)
    got = gu.host(out)
    lo, hi = offsets_np[2], offsets_np[2] + counts_np[2]
    assert (got[lo:hi] == 55).all()
    np.testing.assert_array_equal(np.delete(got[:rows], np.s_[lo:hi], 0), np.delete(want, np.s_[lo:hi], 0))


def test_integer_experts_dynamic_rows_and_refusals():
    rng = np.random.default_rng(orc.SEED + 5)
    e, n, k, cap_m, top_k, bm = 6, 128, 256, 64, 2, 16
    kern = gu.kernel("integer_experts", M=cap_m, N=n, K=k, E=e, top_k=top_k, block_m=bm, dynamic_rows=True)
    packed = rng.integers(0, 2**32, (e, n, k // 8), dtype=np.uint32)
    weights = np.stack([orc.q4_integers(x, TABLE) for x in packed])
    stored = gu.dev(np.stack([orc.q4_pack_k(x, 128) for x in packed]))
    ws = rng.uniform(0.005, 0.02, (e, n)).astype(np.float16)
    cap = orc.tile_capacity(cap_m * top_k, e, bm)
    for m in (64, 5, 1):
        ids, _ = orc.router_topk(rng.normal(size=(m, e)).astype(np.float32), top_k)
        counts_np, _ = orc.expert_histogram(ids, e)
        rows = m * top_k
        offsets_np, tile_offsets, total = orc.expert_offsets(counts_np, bm)
        te, tr = orc.expert_tiles(counts_np, tile_offsets, bm, cap)
        a_q = rng.integers(-127, 128, (cap_m * top_k, k), dtype=np.int8)
        a_s = rng.uniform(0.01, 0.03, cap_m * top_k).astype(np.float16)
        out = torch.full((cap_m * top_k, n), 55.0, dtype=torch.float16, device=gu.DEV)
        kern(A=gu.dev(a_q), AS=gu.dev(a_s), Book=gu.book(), Counts=gu.dev(counts_np), Offsets=gu.dev(offsets_np), Out=out,
             TileCount=gu.dev(total), TileExpert=gu.dev(te), TileRow=gu.dev(tr), W=stored, WS=gu.dev(ws), m=m)
        want = orc.grouped_project(a_q[:rows], a_s[:rows, None], weights, ws, counts_np, offsets_np)
        np.testing.assert_array_equal(gu.host(out)[:rows], want)
        assert (gu.host(out)[rows:] == 55).all()
    for variant in (dict(block_m=512), dict(block_m=12), dict(codec="w8", block_m=8), dict(codec="w8", block_n=32),
                    dict(codec="q2"), dict(K=192), dict(top_k=7), dict(block_k=256, K=384), dict(stages=3)):
        base = dict(M=8, N=64, K=256, E=6, top_k=2)
        base.update(variant)
        with pytest.raises(Exception):
            gu.kernel("integer_experts", **base)


@pytest.mark.parametrize("m,e,k,warps", [(5, 128, 8, 4), (64, 512, 10, 2), (1, 32, 32, 1)])
def test_router_topk_warp_symbol(m, e, k, warps):
    # kernels/cuda/model/moe.py:332-409: same ranking rule, probabilities over the selected routes
    rng = np.random.default_rng(orc.SEED + e + k)
    logits = (rng.normal(size=(m, e)) * 5).astype(np.float32)
    logits[0, :4] = [0.0, -0.0, 0.0, 3.0]
    ids = torch.full((m, k), -1, **I32)
    prob = torch.full((m, k), float("nan"), dtype=torch.float32, device=gu.DEV)
    gu.kernel("router_topk_warp", M=m, E=e, top_k=k, warps=warps)(IDs=ids, Logits=gu.dev(logits), Prob=prob)
    want_ids, want_prob = orc.router_topk(logits, k, True)
    np.testing.assert_array_equal(gu.host(ids), want_ids)
    np.testing.assert_allclose(gu.host(prob), want_prob, atol=2e-6, rtol=2e-5)
    np.testing.assert_allclose(gu.host(prob).sum(axis=1), 1.0, rtol=1e-6)
    for variant in (dict(E=100, top_k=4), dict(E=128, top_k=33), dict(E=128, top_k=4, warps=3)):
        with pytest.raises(Exception):
            gu.kernel("router_topk_warp", M=4, **variant)


@pytest.mark.parametrize("m,e,k,h", [(37, 16, 4, 2048), (256, 128, 8, 2048), (5, 8, 2, 4096 + 8), (3, 4, 1, 64)])
def test_expert_dispatch_quantises_fp16_rows(m, e, k, h):
    """input_dtype=float16: the dispatch gives what activation_quantization + expert_dispatch give."""
    rng = np.random.default_rng(orc.SEED + m + h)
    x = rng.normal(size=(m, h)).astype(np.float16)
    x[0] = 0
    ids_np, _ = orc.router_topk(rng.normal(size=(m, e)).astype(np.float32), k)
    counts, relative = orc.expert_histogram(ids_np, e)
    offsets, _, _ = orc.expert_offsets(counts, 32)
    a_q, a_s = orc.a8(x)
    want_d, want_ds, want_map = orc.expert_dispatch(a_q, a_s, ids_np, relative, offsets)
    d = torch.full((m * k + 1, h), 7, dtype=torch.int8, device=gu.DEV)
    ds = torch.full((m * k + 1,), 3.0, dtype=torch.float16, device=gu.DEV)
    slot_map = torch.full((m, k), -1, **I32)
    gu.kernel("expert_dispatch", M=m, H=h, E=e, top_k=k, input_dtype="float16")(
        A=gu.dev(x), D=d, DS=ds, IDs=gu.dev(ids_np), RelativeSlot=gu.dev(relative), RowOffsets=gu.dev(offsets), Scale=None,
        SlotMap=slot_map)
    np.testing.assert_array_equal(gu.host(d)[: m * k], want_d)
    np.testing.assert_array_equal(gu.host(ds)[: m * k], want_ds[:, 0])
    np.testing.assert_array_equal(gu.host(slot_map), want_map)
    assert (gu.host(d)[m * k] == 7).all() and float(gu.host(ds)[m * k]) == 3.0
    for variant in (dict(H=h, scale_group=h // 2), dict(H=36)):
        with pytest.raises(Exception):
            gu.kernel("expert_dispatch", M=m, E=e, top_k=k, input_dtype="float16", **variant)


def test_moe_token_layer_matches_the_routed_layer_of_one_token():
    """One token through direct bank indexing gives what the token-sorted layer gives for it."""
    c = workloads.config3(tokens=1, experts=32, top_k=4, hidden=512, intermediate=256)
    layer = programs.MoeTokenLayer(c["experts"], c["top_k"], c["hidden"], c["intermediate"], c["gate_up"],
                                   c["gate_up_scales"], c["down"], c["down_scales"], fused=False)
    assert not layer.fused
    x, logits = gu.dev(c["x"]), gu.dev(c["logits"])
    layer.run(x, logits)
    gu.sync()
    ids, prob = orc.router_topk(c["logits"], c["top_k"], True)
    np.testing.assert_array_equal(gu.host(layer.ids), ids)
    a_q, a_s = orc.a8(c["x"])
    w1 = np.stack([orc.q2_integers(m, TABLE) for m in c["gate_up"]])
    w2 = np.stack([orc.q2_integers(m, TABLE) for m in c["down"]])
    gate_up = orc.route_project(a_q, a_s[:, 0], w1, c["gate_up_scales"], ids, True)
    np.testing.assert_array_equal(gu.host(layer.a_s), a_s)
    np.testing.assert_array_equal(gu.host(layer.gate_up_out), gate_up)
    # SwiGLU uses exp(): from here each stage is checked on the GPU's own input
    h_q, h_s = gu.host(layer.h_q), gu.host(layer.h_s)
    want_q, want_s = orc.a8(orc.swiglu_fp16(gate_up))
    assert (h_q == want_q).mean() > 0.999
    down = orc.route_project(h_q, h_s[:, 0], w2, c["down_scales"], ids, False)
    np.testing.assert_array_equal(gu.host(layer.down_out), down)
    staged = orc.moe_combine(down, np.arange(c["top_k"], dtype=np.int32)[None, :], gu.host(layer.prob)).astype(np.float32)
    got = gu.host(layer.out).astype(np.float32)
    assert (np.abs(got - staged) <= 1e-2 + 1e-3 * np.abs(staged)).all()
    # and the token-sorted program on the same token
    sorted_layer = run_layer(c, 32)
    assert torch.equal(sorted_layer.out, layer.out)
    # three launches (gate/up selects the routes itself, down applies SwiGLU -> A8 to its input): same bits
    three = programs.MoeTokenLayer(c["experts"], c["top_k"], c["hidden"], c["intermediate"], c["gate_up"],
                                   c["gate_up_scales"], c["down"], c["down_scales"])
    assert three.fused
    three.ids.fill_(-1)
    three.run(x, logits)
    gu.sync()
    for name in ("ids", "prob", "a_s", "gate_up_out", "h_s", "down_out", "out"):
        assert torch.equal(getattr(three, name), getattr(layer, name)), name
    layer = three  # the graph replay below runs the three-launch program
    # graph replay with another token
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            layer.run(x, logits, stream=stream.cuda_stream)
    rng = np.random.default_rng(9)
    logits.copy_(gu.dev(rng.normal(size=c["logits"].shape).astype(np.float32)))
    x.copy_(gu.dev(rng.normal(size=c["x"].shape).astype(np.float16)))
    graph.replay()
    gu.sync()
    replayed = layer.out.clone()
    layer.run(x, logits)
    gu.sync()
    assert torch.equal(layer.out, replayed)


@pytest.mark.parametrize("swiglu", [False, True], ids=["rows", "swiglu"])
@pytest.mark.parametrize("m,e,k,h", [(37, 64, 10, 640), (5, 512, 10, 5120), (300, 16, 2, 128), (3, 128, 64, 256)])
def test_rotate_expert_a8_rotates_quantises_and_scatters_in_one_launch(m, e, k, h, swiglu):
    """rotate_expert_a8: bit-exact against the oracle for every routing form, and the same bits as
    rotate_activation_a8 followed by expert_dispatch; rows beyond the live count stay untouched."""
    rng = np.random.default_rng(orc.SEED + 3 * m + h + swiglu)
    x = rng.normal(size=(m, 2 * h if swiglu else h)).astype(np.float16)
    x[1] = 0
    signs = rng.choice(np.array([-1, 1], np.int8), h)
    ids_np, _ = orc.router_topk(rng.normal(size=(m, e)).astype(np.float32), k)
    counts, relative = orc.expert_histogram(ids_np, e)
    offsets, _, _ = orc.expert_offsets(counts, 32)
    want_q, want_s, want_d, want_ds, want_map, want_sum = orc.rotate_expert_a8(x, signs, ids_np, relative, offsets, swiglu)
    cap = m + 3
    pad = lambda a: np.concatenate([a, np.zeros((cap - m,) + a.shape[1:], a.dtype)])
    d_x, d_signs = gu.dev(pad(x)), gu.dev(signs)
    d_ids, d_rel, d_off = gu.dev(pad(ids_np)), gu.dev(pad(relative)), gu.dev(offsets)
    fresh = lambda: dict(
        q=torch.full((cap, h), 7, dtype=torch.int8, device=gu.DEV), s=torch.full((cap,), 3.0, dtype=torch.float16, device=gu.DEV),
        d=torch.full((cap * k, h), 7, dtype=torch.int8, device=gu.DEV),
        ds=torch.full((cap * k,), 3.0, dtype=torch.float16, device=gu.DEV), slot_map=torch.full((cap, k), -1, **I32),
        total=torch.full((cap * k,), -5, **I32))
    common = dict(M=cap, K=h, swiglu=swiglu, dynamic_rows=True)
    int8 = dict(hand_over="int8", **common)

    # scatter: codes, scale and sum land in every slot of the row
    o = fresh()
    kern = gu.kernel("rotate_expert_a8", routing="scatter", top_k=k, experts=e, **int8)
    kern(D=o["d"], DS=o["ds"], IDs=d_ids, Q=o["q"], RelativeSlot=d_rel, RowOffsets=d_off, S=o["s"], Signs=d_signs,
         SlotMap=o["slot_map"], Sum=o["total"], X=d_x, m=m)
    np.testing.assert_array_equal(gu.host(o["q"])[:m], want_q)
    np.testing.assert_array_equal(gu.host(o["s"])[:m], want_s[:, 0])
    np.testing.assert_array_equal(gu.host(o["d"])[: m * k], want_d)
    np.testing.assert_array_equal(gu.host(o["ds"])[: m * k], want_ds[:, 0])
    np.testing.assert_array_equal(gu.host(o["slot_map"])[:m], want_map)
    np.testing.assert_array_equal(gu.host(o["total"])[: m * k], want_sum)
    assert (gu.host(o["q"])[m:] == 7).all() and (gu.host(o["d"])[m * k:] == 7).all()
    assert (gu.host(o["ds"])[m * k:] == 3).all() and (gu.host(o["slot_map"])[m:] == -1).all()
    assert (gu.host(o["total"])[m * k:] == -5).all() and (gu.host(o["s"])[m:] == 3).all()
    # Q and Sum are optional under scatter
    lean = fresh()
    kern(D=lean["d"], DS=lean["ds"], IDs=d_ids, Q=None, RelativeSlot=d_rel, RowOffsets=d_off, S=lean["s"], Signs=d_signs,
         SlotMap=lean["slot_map"], Sum=None, X=d_x, m=m)
    assert torch.equal(lean["d"], o["d"]) and torch.equal(lean["ds"], o["ds"]) and torch.equal(lean["slot_map"], o["slot_map"])

    # the two launches it replaces give the same bits
    two = fresh()
    gu.kernel("rotate_activation_a8", **common)(Q=two["q"], S=two["s"], Signs=d_signs, X=d_x, m=m)
    gu.kernel("expert_dispatch", M=cap, H=h, E=e, top_k=k, scale_group=h, dynamic_rows=True)(
        A=two["q"], D=two["d"], DS=two["ds"], IDs=d_ids, RelativeSlot=d_rel, RowOffsets=d_off, Scale=two["s"],
        SlotMap=two["slot_map"], m=m)
    for name in ("q", "s", "d", "ds", "slot_map"):
        assert torch.equal(two[name], o[name]), name

    # shared: the codes stay in Q, every assignment gets its scale and slot
    sh = fresh()
    gu.kernel("rotate_expert_a8", routing="shared", top_k=k, experts=e, **int8)(
        DS=sh["ds"], IDs=d_ids, Q=sh["q"], RelativeSlot=d_rel, RowOffsets=d_off, S=sh["s"], Signs=d_signs,
        SlotMap=sh["slot_map"], Sum=sh["total"], X=d_x, m=m)
    assert torch.equal(sh["q"], o["q"]) and torch.equal(sh["ds"], o["ds"]) and torch.equal(sh["slot_map"], o["slot_map"])
    np.testing.assert_array_equal(gu.host(sh["total"])[:m], want_q.astype(np.int32).sum(1))
    assert (gu.host(sh["total"])[m:] == -5).all()

    # no routing: codes, scale and the row sum
    plain = fresh()
    gu.kernel("rotate_expert_a8", **int8)(Q=plain["q"], S=plain["s"], Signs=d_signs, Sum=plain["total"], X=d_x, m=m)
    assert torch.equal(plain["q"], o["q"]) and torch.equal(plain["s"], o["s"])
    np.testing.assert_array_equal(gu.host(plain["total"])[:m], want_q.astype(np.int32).sum(1))

    # the reference's own hand-over (rotation_a8.py:489-531): the same codes as two planes of nibble words
    def planes(rows, group_major=False):
        shape = (h // 64, rows, 8) if group_major else (rows, h // 8)
        return torch.full(shape, -1, **I32), torch.full(shape, -1, **I32)

    def check(low, high, codes, group_major=False):
        want_low, want_high, _ = orc.split_planes(codes)
        got_low, got_high = gu.host(low, np.uint32), gu.host(high, np.uint32)
        rows = codes.shape[0]
        if group_major:  # the stride is the live row count
            words = h // 64 * rows * 8
            assert (got_low.reshape(-1)[words:] == 0xFFFFFFFF).all() and (got_high.reshape(-1)[words:] == 0xFFFFFFFF).all()
            got_low = orc.planes_row_major(got_low.reshape(-1)[:words].reshape(h // 64, rows, 8))
            got_high = orc.planes_row_major(got_high.reshape(-1)[:words].reshape(h // 64, rows, 8))
        else:
            assert (got_low[rows:] == 0xFFFFFFFF).all() and (got_high[rows:] == 0xFFFFFFFF).all()
        np.testing.assert_array_equal(got_low[:rows], want_low)
        np.testing.assert_array_equal(got_high[:rows], want_high)

    p = fresh()
    low, high = planes(cap * k)
    gu.kernel("rotate_expert_a8", routing="scatter", top_k=k, experts=e, **common)(
        DS=p["ds"], High=high, IDs=d_ids, Low=low, Q=p["q"], RelativeSlot=d_rel, RowOffsets=d_off, S=p["s"], Signs=d_signs,
        SlotMap=p["slot_map"], Sum=p["total"], X=d_x, m=m)
    check(low, high, want_d)
    for name in ("q", "s", "ds", "slot_map", "total"):
        assert torch.equal(p[name], o[name]), name
    p = fresh()
    low, high = planes(cap)
    gu.kernel("rotate_expert_a8", routing="shared", top_k=k, experts=e, **common)(
        DS=p["ds"], High=high, IDs=d_ids, Low=low, Q=p["q"], RelativeSlot=d_rel, RowOffsets=d_off, S=p["s"], Signs=d_signs,
        SlotMap=p["slot_map"], Sum=p["total"], X=d_x, m=m)
    check(low, high, want_q)
    for name in ("q", "s", "ds", "slot_map", "total"):
        assert torch.equal(p[name], sh[name]), name
    p = fresh()
    low, high = planes(cap)
    gu.kernel("rotate_expert_a8", **common)(High=high, Low=low, Q=p["q"], S=p["s"], Signs=d_signs, Sum=p["total"], X=d_x, m=m)
    check(low, high, want_q)
    assert torch.equal(p["q"], plain["q"]) and torch.equal(p["s"], plain["s"]) and torch.equal(p["total"], plain["total"])
    p = fresh()
    low, high = planes(cap, True)
    gu.kernel("rotate_expert_a8", group_major=True, **common)(High=high, Low=low, S=p["s"], Signs=d_signs, Sum=p["total"], X=d_x, m=m)
    check(low, high, want_q, True)
    assert torch.equal(p["s"], plain["s"]) and torch.equal(p["total"], plain["total"])


def test_rotate_expert_a8_refuses_what_it_does_not_serve():
    for variant in (dict(K=192), dict(routing="broadcast"), dict(routing="scatter", top_k=9, experts=8),
                    dict(routing="scatter", top_k=65, experts=128), dict(group_major=True, routing="shared", top_k=1, experts=2),
                    dict(M=0)):
        with pytest.raises(Exception):
            gu.kernel("rotate_expert_a8", **{**dict(M=4, K=256), **variant})


@pytest.mark.parametrize("m,e,k,h", [(256, 128, 8, 2048), (5, 64, 4, 4096), (33, 512, 10, 136), (7, 1024, 8, 256)])
def test_router_quantises_the_hidden_rows_in_the_same_launch(m, e, k, h):
    """quantize_hidden: ids and probabilities as without it, plus the A8 codes and scales of the rows."""
    rng = np.random.default_rng(orc.SEED + m + h)
    logits = rng.normal(size=(m, e)).astype(np.float32)
    x = (rng.normal(size=(m, h)) * rng.uniform(0.1, 4.0, (m, 1))).astype(np.float16)
    x[m // 2] = 0
    cap = m + 2
    ids = torch.full((cap, k), -1, **I32)
    prob = torch.full((cap, k), -1.0, dtype=torch.float32, device=gu.DEV)
    q = torch.full((cap, h), 7, dtype=torch.int8, device=gu.DEV)
    s = torch.full((cap,), 3.0, dtype=torch.float16, device=gu.DEV)
    pad = lambda a: np.concatenate([a, np.zeros((cap - m,) + a.shape[1:], a.dtype)])
    gu.kernel("router_topk", M=cap, E=e, top_k=k, dynamic_rows=True, quantize_hidden=h)(
        IDs=ids, Logits=gu.dev(pad(logits)), Prob=prob, Q=q, S=s, X=gu.dev(pad(x)), m=m)
    plain_ids = torch.full((cap, k), -1, **I32)
    plain_prob = torch.full((cap, k), -1.0, dtype=torch.float32, device=gu.DEV)
    gu.kernel("router_topk", M=cap, E=e, top_k=k, dynamic_rows=True)(IDs=plain_ids, Logits=gu.dev(pad(logits)),
                                                                     Prob=plain_prob, m=m)
    assert torch.equal(ids, plain_ids) and torch.equal(prob, plain_prob)
    want_ids, _ = orc.router_topk(logits, k, True)
    np.testing.assert_array_equal(gu.host(ids)[:m], want_ids)
    want_q, want_s = orc.a8(x)
    np.testing.assert_array_equal(gu.host(q)[:m], want_q)
    np.testing.assert_array_equal(gu.host(s)[:m], want_s[:, 0])
    assert (gu.host(q)[m:] == 7).all() and (gu.host(s)[m:] == 3).all() and (gu.host(ids)[m:] == -1).all()


def test_every_form_reports_a_thread_limit_that_holds_its_own_block():
    """`orx_query` is what an engine checks a record's block against before it accepts the record
    (backend/cuda/kernels.rs:150-170): every form's limit must hold the block its geometry asks for."""
    grouped = dict(rows=2048, E=128, tiles=192, block_m=32)
    forms = [
        ("router_topk", dict(M=256, E=128, top_k=8)),
        ("router_topk", dict(M=256, E=128, top_k=8, quantize_hidden=2048)),
        ("router_topk", dict(M=256, E=1024, top_k=8, quantize_hidden=2048)),
        ("route_metadata", dict(M=256, E=128, top_k=8, block_m=32, slot_maps=True)),
        ("e8p_decode_grouped", dict(N=1024, K=2048, gather=True, epilogue="swiglu", **grouped)),
        ("e8p_decode_grouped", dict(N=2048, K=512, input_dtype="float16", **grouped)),
        ("e8p_decode_grouped", dict(N=2048, K=512, **grouped)),
        ("rotate_expert_a8", dict(M=256, K=2048, routing="scatter", top_k=8, experts=128, hand_over="int8")),
        ("rotate_expert_a8", dict(M=8192, K=5120)),
        ("expert_dispatch", dict(M=256, H=2048, E=128, top_k=8, input_dtype="float16")),
        ("moe_combine", dict(M=256, H=2048, slots=2048, E=128, top_k=8)),
        ("int8_swiglu", dict(M=64, N=512, K=256)),
        ("e8p_q4_projection", dict(M=8192, N=5120, K=5120, dynamic_rows=True, workspace=True)),
    ]
    for symbol, variant in forms:
        kern = gu.lib.Kernel(symbol, **variant)
        for rows in ({1, variant["M"]} if variant.get("dynamic_rows") else {0}):
            threads, _ = kern.query(rows)
            block = kern.geometry(rows)[1]
            assert block[0] * block[1] * block[2] <= threads, (symbol, variant, rows, block, threads)
    # a projection handle starts a different kernel per row range: the limits are those of the kernel that the rows
    # start (every kernel here is compiled for exactly the block it is launched with), not a device-wide constant
    for symbol, variant in (("e8p_q4_projection", dict(M=8192, N=17408, K=5120, dynamic_rows=True, workspace=True)),
                            ("int8_projection", dict(M=8192, N=4096, K=4096, dynamic_rows=True, workspace=True)),
                            ("e8p_q4_projection", dict(M=4096, N=5120, K=5120, dynamic_rows=True))):
        kern = gu.lib.Kernel(symbol, **variant)
        limits = {}
        for rows in (1, 3, 8, 32, 48, 100, 128, 256, 384, 512, variant["M"]):
            grid, block, shared = kern.geometry(rows)
            threads, static_lds = kern.query(rows)
            assert threads == block[0] * block[1] * block[2], (symbol, rows, block, threads)
            assert static_lds + shared <= 160 * 1024
            limits[rows] = threads
        assert kern.query() == kern.query(variant["M"]) and len(set(limits.values())) >= 2, limits
        with pytest.raises(gu.lib.OrxError):
            kern.query(variant["M"] + 1)


@pytest.mark.parametrize("e,k,h,i", [(128, 8, 2048, 512), (512, 10, 1024, 384), (64, 64, 256, 128)])
def test_one_token_layer_in_three_launches_gives_the_bits_of_five(e, k, h, i):
    c = workloads.config3(tokens=1, experts=e, top_k=k, hidden=h, intermediate=i)
    x, logits = gu.dev(c["x"]), gu.dev(c["logits"])
    layers = []
    for fused in (False, True):
        layer = programs.MoeTokenLayer(e, k, h, i, c["gate_up"], c["gate_up_scales"], c["down"], c["down_scales"],
                                       fused=fused)
        layer.run(x, logits)
        gu.sync()
        layers.append(layer)
    want_ids, want_prob = orc.router_topk(c["logits"], k, True)
    np.testing.assert_array_equal(gu.host(layers[1].ids), want_ids)
    np.testing.assert_allclose(gu.host(layers[1].prob), want_prob, atol=2e-6, rtol=2e-5)
    for name in ("ids", "prob", "a_s", "gate_up_out", "h_s", "down_out", "out"):
        assert torch.equal(getattr(layers[1], name), getattr(layers[0], name)), name
    for variant in (dict(shared_input=True, input_dtype="float16", fused_swiglu=True), dict(shared_input=False, input_dtype="float16"),
                    dict(shared_input=False, fused_swiglu=True), dict(shared_input=True, route_logits=True, E=1024)):
        with pytest.raises(Exception):
            gu.kernel("integer_e8p_gemv", **{**dict(E=e, routes=k, N=h, K=i), **variant})


@pytest.mark.parametrize("fused_stages", [False, True], ids=["seven-launches", "five-launches"])
def test_expert_layer_when_every_token_names_the_same_experts(fused_stages):
    """The skew a router can produce: all 150 tokens choose the same four of sixteen experts, so those
    experts have five tiles each (the last one ragged) and the other twelve none."""
    c = workloads.config3(tokens=150, experts=16, top_k=4, hidden=768, intermediate=384)
    logits = np.random.default_rng(11).normal(size=c["logits"].shape).astype(np.float32) * 0.01
    logits[:, [3, 7, 8, 15]] += 5.0
    c = dict(c, logits=logits)
    layer = run_layer(c, 32, fused_stages=fused_stages, grouped_algorithm="resident")
    counts = gu.host(layer.counts)
    assert sorted(np.nonzero(counts)[0].tolist()) == [3, 7, 8, 15] and (counts[[3, 7, 8, 15]] == 150).all()
    assert int(gu.host(layer.tile_count)[0]) == 20
    check_layer(c, layer, 32)


def test_five_launches_at_the_largest_gathered_batch_give_the_bits_of_seven():
    """1024 tokens x top-8 = 8192 slots, the most the slot -> token table in LDS holds; one token more and
    the layer keeps the seven-launch order by itself."""
    c = workloads.config3(tokens=1024)
    x, logits = gu.dev(c["x"]), gu.dev(c["logits"])
    outs = []
    for fused in (False, None):
        layer = programs.MoeLayer(c["tokens"], c["experts"], c["top_k"], c["hidden"], c["intermediate"], c["gate_up"],
                                  c["gate_up_scales"], c["down"], c["down_scales"], block_m=32, fused_stages=fused)
        assert layer.fused_stages == (fused is None)
        layer.run(x, logits)
        gu.sync()
        outs.append(layer.out.clone())
        del layer
    assert torch.equal(outs[0], outs[1])
    bigger = workloads.config3(tokens=1025)
    layer = programs.MoeLayer(1025, bigger["experts"], bigger["top_k"], bigger["hidden"], bigger["intermediate"],
                              bigger["gate_up"], bigger["gate_up_scales"], bigger["down"], bigger["down_scales"], block_m=32)
    assert not layer.fused_stages


# The selector decoder's whole domain, after tests/cuda/operators/e8p_selector.py:23-94: tables drawn from
# {0, +-2, +-6, +-10} (zero coordinates included), one table per expert or one for all, patch words on or
# off (with the word that test plants: valid, value -128, last position), tile lists of 8 to 64 rows with
# one row more than a tile, N = 65, unit power-of-two scales so that the result is the integer itself.
@pytest.mark.parametrize("packed_k", [128, 64, 0])
@pytest.mark.parametrize("bm,m,patched,shared", [(8, 1, False, True), (8, 3, True, False), (16, 17, True, True),
                                                 (32, 33, False, False), (64, 65, False, True), (128, 130, True, False)])
def test_integer_vq_grouped_general_decode(bm, m, patched, shared, packed_k):
    # Book in each of the reference's three forms (integer_vq.py:93-107), by case: raw basis values, signed values, selectors
    form = ("raw", "signed", "selector")[(bm // 8 + packed_k // 64) % 3]
    rng = np.random.default_rng(orc.SEED + bm + packed_k)
    e, n, k = 3, 65, 256
    tables, codes, patches = [], [], []
    for expert in range(e):
        t = rng.choice(np.array([-10, -6, -2, 0, 2, 6, 10], np.int8), (256, 8))
        tables.append(tables[0] if shared and expert else t)
        codes.append(rng.integers(0, 65536, (n, k // 8), dtype=np.uint16))
        words = rng.integers(0, 65536, (n, k // 128), dtype=np.uint16)
        words[0, 0] = 32768 | (128 << 7) | 127
        patches.append(words)
    codes = np.stack(codes)
    patch_np = np.stack([w.T for w in patches])  # (E, K/128, N)
    book_of = dict(raw=orc.basis_words, signed=orc.sign_table, selector=orc.selector_table)[form]
    book_flags = dict(raw={}, signed=dict(shortbook=True), selector=dict(shortbook=True, selectorbook=True))[form]
    book_np = np.stack([book_of(t) for t in (tables[:1] if shared else tables)])
    weights = np.stack([orc.q2_integers(codes[x], tables[x], patches[x] if patched else None) for x in range(e)])
    ws = np.full((e, n), 0.015625, np.float16)
    counts_np = np.full(e, m, np.int32)
    rows = e * m
    a_q = rng.integers(-128, 128, (rows, k), dtype=np.int8)
    a_s = np.full(rows, 0.0078125, np.float16)
    offsets_np, tile_offsets, total = orc.expert_offsets(counts_np, bm)
    cap = orc.tile_capacity(rows, e, bm)
    te, tr = orc.expert_tiles(counts_np, tile_offsets, bm, cap)
    k128 = np.stack([orc.q2_pack_k128(c) for c in codes])
    stored = codes if packed_k == 0 else k128 if packed_k == 128 else orc.q2_repack_k64(k128)
    kern = gu.kernel("integer_vq_grouped", rows=rows, E=e, tiles=cap, N=n, K=k, block_m=bm, packed_k=packed_k,
                     patched=patched, shared_table=shared, basis="any", **book_flags)
    out = torch.full((rows + 1, n), 91.0, dtype=torch.float16, device=gu.DEV)
    book, patch = gu.dev(book_np), gu.dev(patch_np) if patched else None
    counts = gu.dev(counts_np)
    args = dict(A=gu.dev(a_q), AS=gu.dev(a_s), Book=book, C=out, Counts=counts, Offsets=gu.dev(offsets_np),
                P=gu.dev(stored), Patch=patch, TileCount=gu.dev(total), TileExpert=gu.dev(te), TileRow=gu.dev(tr), WS=gu.dev(ws))
    kern(**args)
    want = orc.grouped_project(a_q, a_s[:, None], weights, ws, counts_np, offsets_np)
    got = gu.host(out)
    np.testing.assert_array_equal(got[:rows], want)
    assert (got[rows] == 91).all()
    # every result is the exact integer dot product: 2^-6 * 2^-7 * sum, |sum| < 2^24 / ... fits fp16 only if small,
    # so compare the integers where they are representable
    exact = np.stack([a_q[x * m:(x + 1) * m].astype(np.int64) @ weights[x].astype(np.int64).T for x in range(e)]).reshape(rows, n)
    small = np.abs(exact) < 2048
    np.testing.assert_array_equal(got[:rows][small].astype(np.float64) * 8192, exact[small])
    # tables and patches are read at launch time: an all-zero table leaves 1 - 2p and the patches
    book.copy_(gu.dev(np.stack([book_of(np.zeros((256, 8), np.int8))] * book_np.shape[0])))
    zero_w = np.stack([orc.q2_integers(codes[x], np.zeros((256, 8), np.int8), patches[x] if patched else None) for x in range(e)])
    kern(**args)
    np.testing.assert_array_equal(gu.host(out)[:rows], orc.grouped_project(a_q, a_s[:, None], zero_w, ws, counts_np, offsets_np))
    book.copy_(gu.dev(book_np))
    if patched:
        patch.zero_()
        plain = np.stack([orc.q2_integers(codes[x], tables[x]) for x in range(e)])
        kern(**args)
        np.testing.assert_array_equal(gu.host(out)[:rows], orc.grouped_project(a_q, a_s[:, None], plain, ws, counts_np, offsets_np))
        patch.copy_(gu.dev(patch_np))
    # an expert without rows is skipped
    out.fill_(91)
    counts[0] = 0
    kern(**args)
    got = gu.host(out)
    assert (got[:m] == 91).all()
    np.testing.assert_array_equal(got[m:rows], want[m:])


def test_integer_vq_grouped_default_form_matches_e8p_decode_grouped():
    # with one table for all experts and no other decoder option the symbol runs the same kernels as
    # e8p_decode_grouped; Patch may be null or a dummy
    rng = np.random.default_rng(orc.SEED + 5)
    e, n, k, bm = 6, 160, 256, 32
    counts_np = np.array([3, 0, 40, 32, 1, 9], np.int32)
    rows = int(counts_np.sum())
    codes = rng.integers(0, 65536, (e, n, k // 8), dtype=np.uint16)
    ws = rng.uniform(0.005, 0.02, (e, n)).astype(np.float16)
    a_q = rng.integers(-127, 128, (rows, k), dtype=np.int8)
    a_s = rng.uniform(0.01, 0.03, rows).astype(np.float16)
    offsets_np, tile_offsets, total = orc.expert_offsets(counts_np, bm)
    cap = orc.tile_capacity(rows, e, bm)
    te, tr = orc.expert_tiles(counts_np, tile_offsets, bm, cap)
    stored = np.stack([orc.q2_pack_k128(c) for c in codes])
    want = orc.grouped_project(a_q, a_s[:, None], np.stack([orc.q2_integers(c, TABLE) for c in codes]), ws, counts_np, offsets_np)
    for patch in (None, gu.dev(np.zeros(1, np.uint16))):
        out = torch.full((rows, n), 55.0, dtype=torch.float16, device=gu.DEV)
        gu.kernel("integer_vq_grouped", rows=rows, E=e, tiles=cap, N=n, K=k, block_m=bm, shared_table=True, shortbook=True,
                  selectorbook=True)(
            A=gu.dev(a_q), AS=gu.dev(a_s), Book=gu.book(), C=out, Counts=gu.dev(counts_np), Offsets=gu.dev(offsets_np),
            P=gu.dev(stored), Patch=patch, TileCount=gu.dev(total), TileExpert=gu.dev(te), TileRow=gu.dev(tr), WS=gu.dev(ws))
        np.testing.assert_array_equal(gu.host(out), want)


@pytest.mark.parametrize("packed_k", [128, 64, 0])
@pytest.mark.parametrize("bm,m,patched,shared", [(8, 1, False, True), (8, 3, True, False), (16, 17, True, True),
                                                 (32, 33, False, False), (64, 65, False, True)])
def test_integer_vq_direct_form(bm, m, patched, shared, packed_k):
    # the cases of tests/cuda/operators/e8p_selector.py:23-94 through the symbol without a tile list:
    # expert e multiplies rows [e*m, (e+1)*m)
    rng = np.random.default_rng(orc.SEED + 3 * bm + packed_k)
    e, n, k = 3, 65, 256
    tables, patches = [], []
    for expert in range(e):
        t = rng.choice(np.array([-10, -6, -2, 0, 2, 6, 10], np.int8), (256, 8))
        tables.append(tables[0] if shared and expert else t)
        words = rng.integers(0, 65536, (n, k // 128), dtype=np.uint16)
        words[0, 0] = 32768 | (128 << 7) | 127
        patches.append(words)
    codes = rng.integers(0, 65536, (e, n, k // 8), dtype=np.uint16)
    weights = np.stack([orc.q2_integers(codes[x], tables[x], patches[x] if patched else None) for x in range(e)])
    ws = np.full((e, n), 0.015625, np.float16)
    a_q = rng.integers(-128, 128, (e * m, k), dtype=np.int8)
    a_s = np.full(e * m, 0.0078125, np.float16)
    k128 = np.stack([orc.q2_pack_k128(c) for c in codes])
    stored = codes if packed_k == 0 else k128 if packed_k == 128 else orc.q2_repack_k64(k128)
    form = ("signed", "selector", "raw")[(bm // 8 + packed_k // 64) % 3]  # integer_vq.py:93-107
    book_of = dict(raw=orc.basis_words, signed=orc.sign_table, selector=orc.selector_table)[form]
    book_flags = dict(raw={}, signed=dict(shortbook=True, byte_permute=True), selector=dict(shortbook=True, selectorbook=True))[form]
    book_np = np.stack([book_of(t) for t in (tables[:1] if shared else tables)])
    out = torch.full((e * m + 1, n), 91.0, dtype=torch.float16, device=gu.DEV)
    kern = gu.kernel("integer_vq", E=e, M=m, N=n, K=k, block_m=bm, packed_k=packed_k, patched=patched, shared_table=shared,
                     **book_flags)
    kern(A=gu.dev(a_q), AS=gu.dev(a_s), Book=gu.dev(book_np), C=out, P=gu.dev(stored),
         Patch=gu.dev(np.stack([w.T for w in patches])) if patched else None, WS=gu.dev(ws))
    counts = np.full(e, m, np.int32)
    want = orc.grouped_project(a_q, a_s[:, None], weights, ws, counts, np.arange(e, dtype=np.int32) * m)
    got = gu.host(out)
    np.testing.assert_array_equal(got[:e * m], want)
    assert (got[e * m] == 91).all()


@pytest.mark.parametrize("symbol", ["e8p_decode_grouped", "integer_vq_grouped"])
def test_grouped_q2_with_dynamic_rows_takes_m_last(symbol):
    # dynamic_rows (integer_vq.py:234-258): the same launch with the live row count as a trailing scalar
    rng = np.random.default_rng(orc.SEED + 17)
    e, n, k, bm = 5, 160, 256, 32
    counts_np = np.array([3, 0, 40, 32, 9], np.int32)
    rows, cap_rows = int(counts_np.sum()), 128
    codes = rng.integers(0, 65536, (e, n, k // 8), dtype=np.uint16)
    ws = rng.uniform(0.005, 0.02, (e, n)).astype(np.float16)
    a_q = rng.integers(-127, 128, (cap_rows, k), dtype=np.int8)
    a_s = rng.uniform(0.01, 0.03, cap_rows).astype(np.float16)
    offsets_np, tile_offsets, total = orc.expert_offsets(counts_np, bm)
    cap = orc.tile_capacity(cap_rows, e, bm)
    te, tr = orc.expert_tiles(counts_np, tile_offsets, bm, cap)
    stored = np.stack([orc.q2_pack_k128(c) for c in codes])
    extra = dict(shared_table=True, shortbook=True, selectorbook=True) if symbol == "integer_vq_grouped" else {}
    kern = gu.kernel(symbol, rows=cap_rows, E=e, tiles=cap, N=n, K=k, block_m=bm, dynamic_rows=True, **extra)
    assert kern.arg_names[-1] == "m"
    out = torch.full((cap_rows, n), 55.0, dtype=torch.float16, device=gu.DEV)
    args = dict(A=gu.dev(a_q), AS=gu.dev(a_s), Book=gu.book(), C=out, Counts=gu.dev(counts_np), Offsets=gu.dev(offsets_np),
                P=gu.dev(stored), TileCount=gu.dev(total), TileExpert=gu.dev(te), TileRow=gu.dev(tr), WS=gu.dev(ws), m=rows)
    if symbol == "integer_vq_grouped":
        args["Patch"] = None
    kern(**args)
    want = orc.grouped_project(a_q[:rows], a_s[:rows, None], np.stack([orc.q2_integers(c, TABLE) for c in codes]), ws, counts_np, offsets_np)
    got = gu.host(out)
    np.testing.assert_array_equal(got[:rows], want)
    assert (got[rows:] == 55).all()
    with pytest.raises(gu.lib.OrxError):
        kern(**{**args, "m": cap_rows + 1})


@pytest.mark.parametrize("m,e,k,block,capacity", [(300, 16, 4, 512, 300), (1, 8, 2, 1024, 1), (700, 64, 10, 2048, 900),
                                                  (513, 5, 1, 512, 513)])
def test_segmented_histogram_in_three_launches_gives_expert_histogram(m, e, k, block, capacity):
    # kernels/cuda/model/moe.py:556-656: per-segment ranks and partial counts, their prefixes, the final slots
    rng = np.random.default_rng(orc.SEED + m)
    ids_np = np.stack([rng.choice(e, k, replace=False) for _ in range(m)]).astype(np.int32)
    want_counts, want_rel = orc.expert_histogram(ids_np, e)
    segments = (m * k + block - 1) // block
    ids = torch.full((capacity, k), -1, **I32)
    ids[:m] = gu.dev(ids_np)
    partial, offsets = torch.full((e, segments), -3, **I32), torch.full((e, segments), -3, **I32)
    slots, counts = torch.full((capacity, k), -3, **I32), torch.full((e,), -3, **I32)
    common = dict(M=capacity, E=e, K=k, block=block, dynamic_rows=capacity != m)
    live = dict(m=m) if capacity != m else {}
    gu.kernel("expert_histogram_local", **common)(IDs=ids, Partial=partial, Slots=slots, **live)
    flat = ids_np.reshape(-1)
    want_partial = np.stack([[np.count_nonzero(flat[s * block:(s + 1) * block] == x) for s in range(segments)] for x in range(e)])
    np.testing.assert_array_equal(gu.host(partial), want_partial)
    local = gu.host(slots)[:m].reshape(-1)
    for i in (0, m * k // 2, m * k - 1):  # rank of an assignment among those of its expert inside its segment
        assert local[i] == np.count_nonzero(flat[i // block * block:i] == flat[i])
    gu.kernel("expert_histogram_offsets", **common)(Counts=counts, Offsets=offsets, Partial=partial, **live)
    np.testing.assert_array_equal(gu.host(offsets), np.cumsum(want_partial, axis=1) - want_partial)
    np.testing.assert_array_equal(gu.host(counts), want_counts)
    gu.kernel("expert_histogram_finish", **common)(IDs=ids, Offsets=offsets, Slots=slots, **live)
    np.testing.assert_array_equal(gu.host(slots)[:m], want_rel)
    assert (gu.host(slots)[m:] == -3).all()


def test_expand_experts_decodes_the_banks_of_experts_with_rows():
    # kernels/cuda/model/moe.py:146-173
    rng = np.random.default_rng(orc.SEED + 8)
    e, n, k = 5, 128, 512
    packed = rng.integers(0, 2**32, (e, n, k // 8), dtype=np.uint32)
    stored = np.stack([orc.q4_pack_k(p, 128) for p in packed])
    counts = np.array([3, 0, 1, 0, 40], np.int32)
    out = torch.full((e, n, k), 99, dtype=torch.int8, device=gu.DEV)
    gu.kernel("expand_experts", N=n, K=k, E=e)(Book=gu.book(), Counts=gu.dev(counts), Out=out, W=gu.dev(stored))
    got = gu.host(out)
    for x in range(e):
        if counts[x]:
            np.testing.assert_array_equal(got[x], orc.q4_integers(packed[x], TABLE))
        else:
            assert (got[x] == 99).all()
    for bad in (dict(N=100), dict(K=384), dict(E=0), dict(block_n=48)):
        with pytest.raises(Exception):
            gu.kernel("expand_experts", **{**dict(N=n, K=k, E=e), **bad})


@pytest.mark.parametrize("m,h,e", [(1, 128, 1), (37, 2048, 128), (256, 2048, 128), (130, 2560, 512), (5, 384, 33)])
def test_router_projection_logits_and_shared_gate(m, h, e):
    # floating point (fp16 operands, fp32 accumulation): every logit within 2^-15 of the sum of the magnitudes of its
    # products (H fp32 roundings of partial sums would allow H * 2^-24 of it; H <= 2560 here), the gate within one fp16 step
    rng = np.random.default_rng(orc.SEED + m + e)
    x = rng.normal(size=(m, h)).astype(np.float16)
    w = (rng.normal(size=(e + 1, h)) * 0.05).astype(np.float16)
    cap = m + 3
    logits = torch.full((cap, e), 7.0, dtype=torch.float32, device=gu.DEV)
    gate = torch.full((cap,), 7.0, dtype=torch.float16, device=gu.DEV)
    gu.kernel("router_projection", M=cap, H=h, E=e, dynamic_rows=True)(
        Logits=logits, SharedGate=gate, W=gu.dev(w), X=gu.dev(np.concatenate([x, np.zeros((cap - m, h), np.float16)])), m=m)
    want_logits, want_gate = orc.router_projection(x, w)
    bound = (np.abs(x.astype(np.float64)) @ np.abs(w.astype(np.float64)).T) * 2.0 ** -15
    got = gu.host(logits)
    assert (np.abs(got[:m].astype(np.float64) - want_logits) <= bound[:, :e] + 1e-30).all()
    got_gate = gu.host(gate)[:m].astype(np.float64)
    assert (np.abs(got_gate - want_gate.astype(np.float64)) <= np.abs(want_gate.astype(np.float64)) * 2.0 ** -10 + bound[:, e]).all()
    assert (got[m:] == 7).all() and (gu.host(gate)[m:] == 7).all()
    # the ranking that follows is the one of the exact logits wherever they are farther apart than the bound
    ids = torch.empty((m, min(4, e)), **I32)
    prob = torch.empty((m, min(4, e)), dtype=torch.float32, device=gu.DEV)
    gu.kernel("router_topk", M=m, E=e, top_k=min(4, e))(IDs=ids, Logits=logits[:m].contiguous(), Prob=prob)
    want_ids, _ = orc.router_topk(got[:m], min(4, e))
    np.testing.assert_array_equal(gu.host(ids), want_ids)
    for bad in (dict(H=100), dict(block_k=512), dict(block_m=8), dict(stages=3), dict(E=0)):
        with pytest.raises(Exception):
            gu.kernel("router_projection", **{**dict(M=4, H=256, E=8), **bad})


def test_integer_vq_raw_basis_with_values_beyond_the_e8p_palette():
    # the default Book is the (256, 2) table of raw int8 basis values (integer_vq.py:104-107, :188-192): any even value
    # decodes as +-t + (1 - 2p) in int8 arithmetic, -128 included (its negative wraps to itself, as in the reference's
    # word arithmetic, integer_vq.py:26-39); the signed-value table gives the same weights
    rng = np.random.default_rng(orc.SEED + 41)
    e, m, n, k = 2, 9, 96, 256
    table = (rng.integers(-64, 64, (256, 8)) * 2).astype(np.int8)
    table[0] = [-128, 126, 0, -2, 4, 100, -100, 8]
    codes = rng.integers(0, 65536, (e, n, k // 8), dtype=np.uint16)
    codes[0, 0, :4] = [0x0000, 0x00FF, 0x0001, 0x0080]  # row 0 with no sign, every sign, odd parity with one sign each way
    wide = np.stack([orc.e8p_decode(c, table).reshape(n, k) for c in codes]).astype(np.int64)
    weights = ((wide + 128) % 256 - 128).astype(np.int8)
    a_q = rng.integers(-128, 128, (e * m, k), dtype=np.int8)
    a_s = np.full(e * m, 0.0078125, np.float16)
    ws = np.full((e, n), 0.015625, np.float16)
    want = orc.grouped_project(a_q, a_s[:, None], weights, ws, np.full(e, m, np.int32), np.arange(e, dtype=np.int32) * m)
    stored = np.stack([orc.q2_pack_k128(c) for c in codes])
    for flags, book in ((dict(), orc.basis_words(table)), (dict(shortbook=True), orc.sign_table(table))):
        out = torch.full((e * m, n), 91.0, dtype=torch.float16, device=gu.DEV)
        gu.kernel("integer_vq", E=e, M=m, N=n, K=k, shared_table=True, **flags)(
            A=gu.dev(a_q), AS=gu.dev(a_s), Book=gu.dev(book[None]), C=out, P=gu.dev(stored), Patch=None, WS=gu.dev(ws))
        np.testing.assert_array_equal(gu.host(out), want)


def test_expert_dispatch_default_scale_groups_of_64_channels():
    # moe.py:286-329: a record without scale_group carries one scale per 64 channels, Scale (M, H / 64) -> DS (slots, H / 64)
    rng = np.random.default_rng(orc.SEED + 51)
    m, e, k, h = 13, 8, 3, 192
    ids_np = np.stack([rng.choice(e, k, replace=False) for _ in range(m)]).astype(np.int32)
    counts, relative = orc.expert_histogram(ids_np, e)
    offsets, _, _ = orc.expert_offsets(counts, 16)
    a_q = rng.integers(-127, 128, (m, h), dtype=np.int8)
    a_s = rng.uniform(0.01, 0.02, (m, h // 64)).astype(np.float16)
    d = torch.zeros((m * k, h), dtype=torch.int8, device=gu.DEV)
    ds = torch.zeros((m * k, h // 64), dtype=torch.float16, device=gu.DEV)
    slot = torch.full((m, k), -1, **I32)
    gu.kernel("expert_dispatch", M=m, H=h, E=e, top_k=k)(A=gu.dev(a_q), D=d, DS=ds, IDs=gu.dev(ids_np), RelativeSlot=gu.dev(relative),
                                                       RowOffsets=gu.dev(offsets), Scale=gu.dev(a_s), SlotMap=slot)
    want_d, want_ds, want_slot = orc.expert_dispatch(a_q, a_s, ids_np, relative, offsets)
    np.testing.assert_array_equal(gu.host(slot), want_slot)
    np.testing.assert_array_equal(gu.host(d), want_d)
    np.testing.assert_array_equal(gu.host(ds), want_ds)
    assert gu.lib.Kernel("route_metadata", M=64, E=16, top_k=2).geometry() == gu.lib.Kernel("route_metadata", M=64, E=16, top_k=2, block_m=8).geometry()


@pytest.mark.parametrize("packed_k", [128, 64])
@pytest.mark.parametrize("bm", [8, 16])
def test_e8p_decode_grouped_takes_tile_lists_in_steps_of_8_and_16_rows(bm, packed_k):
    # the reference's decode kernel multiplies 8-row tiles (e8p_decode.py:36-58) and route_metadata builds such lists by
    # default (moe.py:714): here the workgroup of the first tile of every stretch of 32 rows takes the whole stretch
    rng = np.random.default_rng(orc.SEED + 61 + bm)
    e, n, k = 6, 160, 512
    counts_np = np.array([3, 0, 41, 32, 1, 17], np.int32)
    rows = int(counts_np.sum())
    codes = rng.integers(0, 65536, (e, n, k // 8), dtype=np.uint16)
    ws = rng.uniform(0.005, 0.02, (e, n)).astype(np.float16)
    a_q = rng.integers(-127, 128, (rows, k), dtype=np.int8)
    a_s = rng.uniform(0.01, 0.03, rows).astype(np.float16)
    meta = {name: torch.full(shape, -1, **I32) for name, shape in
            dict(Counts=(e,), RelativeSlot=(rows, 1), RowOffsets=(e,), TileCount=(1,), TileOffsets=(e,)).items()}
    ids = np.repeat(np.arange(e, dtype=np.int32), counts_np)[:, None]
    cap = orc.tile_capacity(rows, e, bm)
    meta["TileExpert"], meta["TileRow"] = torch.full((cap,), -1, **I32), torch.full((cap,), -1, **I32)
    gu.kernel("route_metadata", M=rows, E=e, top_k=1, block_m=bm)(IDs=gu.dev(ids), **meta)
    assert int(meta["TileCount"].cpu()[0]) == int(np.sum((counts_np + bm - 1) // bm))
    out = torch.full((rows + 1, n), 55.0, dtype=torch.float16, device=gu.DEV)
    stored = np.stack([orc.q2_pack_k128(c) for c in codes])
    if packed_k == 64:  # blocks of 64 codes per channel (e8p_decode.py:43,62): the 8- and 16-row tiles of the MFMA kernel
        stored = orc.q2_repack_k64(stored)
    gu.kernel("e8p_decode_grouped", rows=rows, E=e, tiles=cap, N=n, K=k, block_m=bm, packed_k=packed_k)(
        A=gu.dev(a_q), AS=gu.dev(a_s), Book=gu.book(), C=out, Counts=meta["Counts"], Offsets=meta["RowOffsets"],
        P=gu.dev(stored), TileCount=meta["TileCount"], TileExpert=meta["TileExpert"],
        TileRow=meta["TileRow"], WS=gu.dev(ws))
    want = orc.grouped_project(a_q, a_s[:, None], np.stack([orc.q2_integers(c, TABLE) for c in codes]), ws, counts_np,
                               gu.host(meta["RowOffsets"]))
    got = gu.host(out)
    np.testing.assert_array_equal(got[:rows], want)
    assert (got[rows] == 55).all()
