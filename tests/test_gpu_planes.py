"""GPU parity for the nibble-plane hand-over (A8 as two planes of 4-bit words) and the grouped GEMMs that take it.

The cases follow the reference's own test of these kernels (tests/cuda/operators/e8p_exact.py): random bases from
{+-2, +-6, +-10}, extreme codes planted in every row, tile lists with tails, the plane words checked through
low + 16 high == permuted codes, outputs equal to the int8 grouped kernel's on the same code bank.
"""
import numpy as np
import pytest
import torch

from oracle import reference as orc

from . import gpu_util as gu

pytestmark = pytest.mark.gpu
I32 = dict(dtype=torch.int32, device=gu.DEV)

SHAPES = [  # (block_m, counts, N, K): tests/cuda/operators/e8p_exact.py:35-45
    (8, [1, 0], 160, 640),
    (8, [7, 8], 160, 640),
    (16, [17, 16], 160, 640),
    (32, [33, 32], 160, 640),
    (16, [3, 0], 129, 128),
    (16, [5, 9], 257, 2560),
    (8, [9, 17], 1280, 2560),
    (16, [17, 33], 2560, 640),
]


def planted_rows(rng, rows, k):
    a = rng.integers(-128, 128, (rows, k), dtype=np.int8)
    a[:, :4] = np.array([-128, -1, 0, 127], np.int8)
    return a


def tile_list(counts, bm):
    offsets, tile_offsets, total = orc.expert_offsets(np.asarray(counts, np.int32), bm)
    cap = sum(counts) // bm + len(counts) + 1
    te, tr = orc.expert_tiles(np.asarray(counts, np.int32), tile_offsets, bm, cap)
    return offsets, te, tr, total, cap


def empty_planes(rows, k, group_major):
    shape = (k // 64, rows, 8) if group_major else (rows, k // 8)
    return torch.full(shape, -1, **I32), torch.full(shape, -1, **I32)


@pytest.mark.parametrize("rows,k", [(1, 128), (5, 640), (67, 2560), (130, 5120)])
@pytest.mark.parametrize("group_major", [False, True])
def test_split_a8_words_and_sums(rows, k, group_major):
    rng = np.random.default_rng(orc.SEED + rows)
    a = planted_rows(rng, rows, k)
    low, high = empty_planes(rows + 1, k, group_major) if not group_major else empty_planes(rows, k, True)
    total = torch.full((rows + 1,), -7, **I32)
    symbol = "split_prefill_a8" if group_major else "split_a8"
    gu.kernel(symbol, rows=rows, K=k)(A=gu.dev(a), High=high, Low=low, Sum=total)
    want_low, want_high, want_sum = orc.split_planes(a)
    got_low, got_high = gu.host(low, np.uint32), gu.host(high, np.uint32)
    if group_major:
        got_low, got_high = orc.planes_row_major(got_low), orc.planes_row_major(got_high)
    else:
        assert (got_low[rows] == 0xFFFFFFFF).all() and (got_high[rows] == 0xFFFFFFFF).all()
        got_low, got_high = got_low[:rows], got_high[:rows]
    np.testing.assert_array_equal(got_low, want_low)
    np.testing.assert_array_equal(got_high, want_high)
    np.testing.assert_array_equal(gu.host(total)[:rows], want_sum)
    assert gu.host(total)[rows] == -7
    # the reference's own statement of the planes (e8p_exact.py:196-206)
    shifts = np.arange(0, 32, 4, dtype=np.uint64)
    lo = ((got_low.astype(np.uint64)[..., None] >> shifts) & 15).astype(np.int64).reshape(rows, k)
    hi = ((got_high.astype(np.uint64)[..., None] >> shifts) & 15).astype(np.int64).reshape(rows, k)
    hi = np.where(hi >= 8, hi - 16, hi)
    permuted = a.reshape(rows, k // 8, 8)[:, :, [0, 2, 1, 3, 4, 6, 5, 7]].reshape(rows, k)
    np.testing.assert_array_equal(lo + 16 * hi, permuted.astype(np.int64))


def test_split_a8_dynamic_rows_strides_follow_the_live_rows():
    rng = np.random.default_rng(orc.SEED)
    capacity, m, k = 40, 13, 256
    a = planted_rows(rng, capacity, k)
    low, high = empty_planes(capacity, k, True)
    total = torch.full((capacity,), -7, **I32)
    gu.kernel("split_prefill_a8", rows=capacity, K=k, dynamic_rows=True)(A=gu.dev(a), High=high, Low=low, Sum=total, m=m)
    want_low, want_high, want_sum = orc.split_planes(a[:m])
    words = k // 64 * m * 8
    np.testing.assert_array_equal(gu.host(low, np.uint32).reshape(-1)[:words], orc.planes_group_major(want_low).reshape(-1))
    np.testing.assert_array_equal(gu.host(high, np.uint32).reshape(-1)[:words], orc.planes_group_major(want_high).reshape(-1))
    assert (gu.host(low, np.uint32).reshape(-1)[words:] == 0xFFFFFFFF).all()
    np.testing.assert_array_equal(gu.host(total)[:m], want_sum)
    assert (gu.host(total)[m:] == -7).all()


def test_split_routed_prefill_a8_touches_the_rows_of_the_tiles_only():
    rng = np.random.default_rng(orc.SEED + 1)
    counts, bm, k = [5, 0, 9, 3], 8, 384
    rows = sum(counts) + 2  # two rows that belong to no expert
    a = planted_rows(rng, rows, k)
    offsets, tile_offsets, total = orc.expert_offsets(np.asarray(counts, np.int32), bm)
    cap = (rows + bm - 1) // bm + min(len(counts), rows)
    te, tr = orc.expert_tiles(np.asarray(counts, np.int32), tile_offsets, bm, cap)
    low, high = empty_planes(rows, k, True)
    sums = torch.full((rows,), -7, **I32)
    gu.kernel("split_routed_prefill_a8", rows=rows, K=k, experts=len(counts), block_m=bm)(
        A=gu.dev(a), Counts=gu.dev(np.asarray(counts, np.int32)), High=high, Low=low, Offsets=gu.dev(offsets), Sum=sums,
        TC=gu.dev(total), TE=gu.dev(te), TR=gu.dev(tr))
    want_low, want_high, want_sum = orc.split_planes(a)
    live = sum(counts)
    got_low, got_high = orc.planes_row_major(gu.host(low, np.uint32)), orc.planes_row_major(gu.host(high, np.uint32))
    np.testing.assert_array_equal(got_low[:live], want_low[:live])
    np.testing.assert_array_equal(got_high[:live], want_high[:live])
    np.testing.assert_array_equal(gu.host(sums)[:live], want_sum[:live])
    assert (got_low[live:] == 0xFFFFFFFF).all() and (gu.host(sums)[live:] == -7).all()


def routed(rng, m, e, top_k):
    ids = np.stack([rng.choice(e, top_k, replace=False) for _ in range(m)]).astype(np.int32)
    counts, relative = orc.expert_histogram(ids, e)
    offsets, _, _ = orc.expert_offsets(counts, 16)
    return ids, relative, offsets


@pytest.mark.parametrize("m,k,e,top_k", [(1, 128, 4, 1), (9, 640, 16, 4), (33, 2560, 64, 10)])
def test_dispatch_prefill_a8(m, k, e, top_k):
    rng = np.random.default_rng(orc.SEED + m)
    a = planted_rows(rng, m, k)
    scale = rng.uniform(0.01, 0.03, (m, 1)).astype(np.float16)
    ids, relative, offsets = routed(rng, m, e, top_k)
    slots = m * top_k
    low, high = empty_planes(slots, k, True)
    sums, slot_map = torch.full((slots,), -7, **I32), torch.full((m, top_k), -7, **I32)
    ds = torch.zeros((slots, 1), dtype=torch.float16, device=gu.DEV)
    gu.kernel("dispatch_prefill_a8", M=m, K=k, E=e, top_k=top_k)(
        A=gu.dev(a), DS=ds, High=high, IDs=gu.dev(ids), Low=low, RelativeSlot=gu.dev(relative), RowOffsets=gu.dev(offsets),
        Scale=gu.dev(scale), SlotMap=slot_map, Sum=sums)
    want = orc.dispatch_planes(a, scale, ids, relative, offsets)
    for got, expected in zip((gu.host(low, np.uint32), gu.host(high, np.uint32), gu.host(sums), gu.host(ds), gu.host(slot_map)), want):
        np.testing.assert_array_equal(got, expected)


def test_pack_expert_tokens_then_expand_expert_slots_equals_dispatch():
    rng = np.random.default_rng(orc.SEED + 2)
    capacity, m, k, e, top_k = 24, 19, 640, 16, 4
    a = planted_rows(rng, capacity, k)
    scale = rng.uniform(0.01, 0.03, (capacity, 1)).astype(np.float16)
    ids, relative, offsets = routed(rng, m, e, top_k)
    slots = m * top_k
    src_low, src_high = empty_planes(m, k, True)
    src_sum, sources = torch.full((m,), -7, **I32), torch.full((slots,), -7, **I32)
    slot_map = torch.full((m, top_k), -7, **I32)
    gu.kernel("pack_expert_tokens", M=capacity, K=k, E=e, top_k=top_k)(
        A=gu.dev(a), High=src_high, IDs=gu.dev(ids), Low=src_low, RelativeSlot=gu.dev(relative), RowOffsets=gu.dev(offsets),
        SlotMap=slot_map, Sources=sources, Sum=src_sum, m=m)
    want_low, want_high, want_sum = orc.split_planes(a[:m])
    np.testing.assert_array_equal(gu.host(src_low, np.uint32), orc.planes_group_major(want_low))
    np.testing.assert_array_equal(gu.host(src_high, np.uint32), orc.planes_group_major(want_high))
    np.testing.assert_array_equal(gu.host(src_sum), want_sum)
    want = orc.dispatch_planes(a[:m], scale[:m], ids, relative, offsets)
    np.testing.assert_array_equal(gu.host(slot_map), want[4])
    inverse = np.empty(slots, np.int32)
    inverse[want[4]] = np.arange(m, dtype=np.int32)[:, None]
    np.testing.assert_array_equal(gu.host(sources), inverse)
    low, high = empty_planes(slots, k, True)
    sums = torch.full((slots,), -7, **I32)
    ds = torch.zeros((slots, 1), dtype=torch.float16, device=gu.DEV)
    gu.kernel("expand_expert_slots", M=capacity, K=k, top_k=top_k)(
        DS=ds, High=high, Low=low, Scale=gu.dev(scale), Sources=sources, SrcHigh=src_high, SrcLow=src_low, SrcSum=src_sum,
        Sum=sums, m=m)
    for got, expected in zip((gu.host(low, np.uint32), gu.host(high, np.uint32), gu.host(sums), gu.host(ds)), want[:4]):
        np.testing.assert_array_equal(got, expected)


def grouped_case(rng, counts, n, k, basis):
    e, rows = len(counts), sum(counts)
    a = planted_rows(rng, rows, k)
    raw = rng.integers(0, 65536, (e, k // 128, n, 16), dtype=np.uint16)  # K128 blocks, as the reference's bank
    codes = np.ascontiguousarray(raw.transpose(0, 2, 1, 3)).reshape(e, n, k // 8)
    ws = (rng.random((e, n)) / 16).astype(np.float16)
    scale = (rng.random(rows) / 16).astype(np.float16)
    weights = np.stack([orc.q2_integers(c, basis) for c in codes])
    return a, raw, codes, ws, scale, weights


@pytest.mark.parametrize("bm,counts,n,k", SHAPES)
def test_exact_and_prefill_grouped_match_the_int8_kernel(bm, counts, n, k):
    rng = np.random.default_rng(orc.SEED + bm + n)
    basis = rng.choice(np.array([-10, -6, -2, 2, 6, 10], np.int8), (256, 8))
    selector = orc.selector_table(basis)
    nibble = orc.nibble_table(selector)
    e, rows = len(counts), sum(counts)
    a, raw, codes, ws, scale, weights = grouped_case(rng, counts, n, k, basis)
    offsets, te, tr, total, cap = tile_list(counts, bm)
    counts_np = np.asarray(counts, np.int32)
    want = orc.grouped_project(a, scale[:, None], weights, ws, counts_np, offsets)
    routing = dict(Counts=gu.dev(counts_np), Offsets=gu.dev(offsets))
    # the int8 kernel on the same bank in K64 blocks
    ref = torch.full((rows, n), float("nan"), dtype=torch.float16, device=gu.DEV)
    gu.kernel("integer_vq_grouped", rows=rows, E=e, tiles=cap, N=n, K=k, kind="e8p", shared_table=True, block_m=bm,
              block_n=128, shortbook=True, selectorbook=True, packed_k=64, basis="any")(
        A=gu.dev(a), AS=gu.dev(scale), Book=gu.dev(selector[None]), C=ref, P=gu.dev(orc.q2_repack_k64(raw)), Patch=None,
        TileCount=gu.dev(total), TileExpert=gu.dev(te), TileRow=gu.dev(tr), WS=gu.dev(ws), **routing)
    np.testing.assert_array_equal(gu.host(ref), want)
    a_dev = gu.dev(a)
    forms = []  # both kernels behind the symbols: codes decoded into MFMA operands (stream) or staged in LDS (tiles)
    if bm <= 16:
        forms += [("e8p_exact_grouped", dict(block_m=bm, stages=s, algorithm=("stream", "tiles", "auto")[s - 2]), False)
                  for s in (2, 3, 4) if k // 64 >= s - 1]
    if bm >= 16:
        forms += [("e8p_prefill_grouped", dict(block_m=bm, algorithm="stream"), True),
                  ("e8p_prefill_grouped", dict(block_m=bm, algorithm="tiles"), True),
                  ("e8p_prefill_grouped", dict(block_m=bm, row_major=True), False)]
    for symbol, options, group_major in forms:
        low, high = empty_planes(rows, k, group_major)
        sums = torch.full((rows,), -7, **I32)
        gu.kernel("split_prefill_a8" if group_major else "split_a8", rows=rows, K=k)(A=a_dev, High=high, Low=low, Sum=sums)
        out = torch.full((rows, n), float("nan"), dtype=torch.float16, device=gu.DEV)
        kern = gu.kernel(symbol, rows=rows, E=e, tiles=cap, N=n, K=k, **options)
        args = dict(AS=gu.dev(scale), Book=gu.dev(nibble[None]), High=high, Low=low, Out=out, P=gu.dev(orc.q2_repack_k64(raw)),
                    Sum=sums, TC=gu.dev(total), TE=gu.dev(te), TR=gu.dev(tr), WS=gu.dev(ws), **routing)
        kern(**args)
        assert torch.equal(out, ref), (symbol, options)
        # Sum is an input like any other: the kernels add what they are given (e8p_core.py:186)
        planted = rng.integers(-1000, 1000, rows).astype(np.int32)
        sums.copy_(gu.dev(planted))
        kern(**args)
        half = np.stack([orc.nibble_decode(c, nibble).reshape(n, k) for c in codes])
        expected = np.zeros((rows, n), np.float16)
        got_low, got_high = gu.host(low, np.uint32), gu.host(high, np.uint32)
        if group_major:
            got_low, got_high = orc.planes_row_major(got_low), orc.planes_row_major(got_high)
        for x, c in enumerate(counts):
            r = slice(int(offsets[x]), int(offsets[x]) + c)
            expected[r] = orc.plane_project(got_low[r], got_high[r], planted[r], half[x], ws[x], scale[r])
        np.testing.assert_array_equal(gu.host(out), expected)
        # zero activations with their sums give zero (the reference's graph replay on a.zero_())
        low.zero_(), high.zero_(), sums.zero_()
        kern(**args)
        assert bool((out == 0).all())


@pytest.mark.parametrize("bm,counts,n,k", [(16, [17, 16], 160, 640), (32, [33, 5, 0, 70], 257, 1280), (16, [3, 0], 129, 128)])
def test_prefill_grouped_two_stage_codes(bm, counts, n, k):
    # codec e8p_q4: K-major blocks of 128 u32 codes, Book = selector words (e8p_prefill.py:468-469, :492-493)
    rng = np.random.default_rng(orc.SEED + bm + k)
    basis = orc.basis()
    e, rows = len(counts), sum(counts)
    a = planted_rows(rng, rows, k)
    packed = rng.integers(0, 2**32, (e, n, k // 8), dtype=np.uint32)
    weights = np.stack([orc.q4_integers(p, basis) for p in packed])
    stored = np.stack([orc.q4_pack_k(p, 128) for p in packed])
    ws = (rng.random((e, n)) / 64).astype(np.float16)
    scale = (rng.random(rows) / 16).astype(np.float16)
    offsets, te, tr, total, cap = tile_list(counts, bm)
    counts_np = np.asarray(counts, np.int32)
    want = orc.grouped_project(a, scale[:, None], weights, ws, counts_np, offsets)
    low, high = empty_planes(rows, k, True)
    sums = torch.full((rows,), -7, **I32)
    gu.kernel("split_prefill_a8", rows=rows, K=k)(A=gu.dev(a), High=high, Low=low, Sum=sums)
    out = torch.full((rows + 1, n), 91.0, dtype=torch.float16, device=gu.DEV)
    for algorithm in ("stream", "tiles"):
        out.fill_(91.0)
        gu.kernel("e8p_prefill_grouped", rows=rows, E=e, tiles=cap, N=n, K=k, codec="e8p_q4", block_m=bm, algorithm=algorithm)(
            AS=gu.dev(scale), Book=gu.book(), Counts=gu.dev(counts_np), High=high, Low=low, Offsets=gu.dev(offsets), Out=out,
            P=gu.dev(stored), Sum=sums, TC=gu.dev(total), TE=gu.dev(te), TR=gu.dev(tr), WS=gu.dev(ws))
        got = gu.host(out)
        np.testing.assert_array_equal(got[:rows], want)
        assert (got[rows] == 91).all()


def test_prefill_grouped_merges_adjacent_tiles_of_a_shared_list_and_takes_live_rows():
    # merge_routed_tiles: the list steps by 16 rows, a workgroup takes 32 (e8p_prefill.py:188, :497-498);
    # dynamic rows: the plane stride is the live row count (e8p_prefill.py:186-187)
    rng = np.random.default_rng(orc.SEED + 9)
    basis = orc.basis()
    nibble = orc.nibble_table(orc.selector_table(basis))
    counts, n, k, capacity = [40, 0, 16, 7], 192, 512, 80
    e, rows = len(counts), sum(counts)
    a, raw, codes, ws, scale, weights = grouped_case(rng, counts, n, k, basis)
    counts_np = np.asarray(counts, np.int32)
    offsets, tile_offsets, total = orc.expert_offsets(counts_np, 16)
    cap = capacity // 16 + e + 1
    te, tr = orc.expert_tiles(counts_np, tile_offsets, 16, cap)
    want = orc.grouped_project(a, scale[:, None], weights, ws, counts_np, offsets)
    low, high = empty_planes(capacity, k, True)
    sums = torch.full((capacity,), -7, **I32)
    gu.kernel("split_prefill_a8", rows=capacity, K=k, dynamic_rows=True)(A=gu.dev(a), High=high, Low=low, Sum=sums, m=rows)
    out = torch.full((capacity, n), 91.0, dtype=torch.float16, device=gu.DEV)
    for algorithm in ("stream", "tiles"):
        out.fill_(91.0)
        gu.kernel("e8p_prefill_grouped", rows=capacity, E=e, tiles=cap, N=n, K=k, block_m=32, specialize_tails=True,
                  merge_routed_tiles=True, dynamic_rows=True, sparse_rows=True, minimum_blocks=2, algorithm=algorithm)(
            AS=gu.dev(scale), Book=gu.dev(nibble[None]), Counts=gu.dev(counts_np), High=high, Low=low, Offsets=gu.dev(offsets),
            Out=out, P=gu.dev(orc.q2_repack_k64(raw)), Sum=sums, TC=gu.dev(total), TE=gu.dev(te), TR=gu.dev(tr), WS=gu.dev(ws),
            m=rows)
        got = gu.host(out)
        np.testing.assert_array_equal(got[:rows], want)
        assert (got[rows:] == 91).all()


def test_rotated_planes_into_the_exact_kernel_equal_int8_rows_into_the_int8_kernel():
    # one routed expert projection both ways: rotate_expert_a8 writes planes at the slots and e8p_exact_grouped reads them
    # (the reference's pairing, flash_next/experts.rs:207-215), or it writes int8 rows and e8p_decode_grouped reads those
    rng = np.random.default_rng(orc.SEED + 11)
    m, e, top_k, h, n, bm = 21, 8, 2, 512, 192, 16
    basis = orc.basis()
    x = rng.normal(size=(m, h)).astype(np.float16)
    signs = rng.choice(np.array([-1, 1], np.int8), h)
    ids, _ = orc.router_topk(rng.normal(size=(m, e)).astype(np.float32), top_k)
    counts, relative = orc.expert_histogram(ids, e)
    offsets, tile_offsets, total = orc.expert_offsets(counts, bm)
    slots = m * top_k
    cap = orc.tile_capacity(slots, e, bm)
    te, tr = orc.expert_tiles(counts, tile_offsets, bm, cap)
    raw = rng.integers(0, 65536, (e, h // 128, n, 16), dtype=np.uint16)
    ws = rng.uniform(0.005, 0.02, (e, n)).astype(np.float16)
    routing = dict(IDs=gu.dev(ids), RelativeSlot=gu.dev(relative), RowOffsets=gu.dev(offsets), Signs=gu.dev(signs), X=gu.dev(x))
    shape = dict(M=m, K=h, routing="scatter", top_k=top_k, experts=e)
    tiles = dict(Counts=gu.dev(counts), Offsets=gu.dev(offsets))
    q = torch.empty((m, h), dtype=torch.int8, device=gu.DEV)
    s = torch.empty((m,), dtype=torch.float16, device=gu.DEV)
    ds = torch.empty((slots,), dtype=torch.float16, device=gu.DEV)
    slot_map, sums = torch.empty((m, top_k), **I32), torch.empty((slots,), **I32)
    d = torch.empty((slots, h), dtype=torch.int8, device=gu.DEV)
    gu.kernel("rotate_expert_a8", hand_over="int8", **shape)(D=d, DS=ds, Q=q, S=s, SlotMap=slot_map, Sum=sums, **routing)
    ref = torch.full((slots, n), float("nan"), dtype=torch.float16, device=gu.DEV)
    gu.kernel("e8p_decode_grouped", rows=slots, E=e, tiles=cap, N=n, K=h, block_m=32)(
        A=d, AS=ds, Book=gu.book(), C=ref, P=gu.dev(raw), TileCount=gu.dev(total), TileExpert=gu.dev(te), TileRow=gu.dev(tr),
        WS=gu.dev(ws), **tiles)
    low, high = empty_planes(slots, h, False)
    ds2, sums2 = torch.empty_like(ds), torch.empty_like(sums)
    gu.kernel("rotate_expert_a8", **shape)(DS=ds2, High=high, Low=low, Q=q, S=s, SlotMap=slot_map, Sum=sums2, **routing)
    out = torch.full((slots, n), float("nan"), dtype=torch.float16, device=gu.DEV)
    gu.kernel("e8p_exact_grouped", rows=slots, E=e, tiles=cap, N=n, K=h, block_m=bm)(
        AS=ds2, Book=gu.dev(orc.nibble_table(orc.selector_table(basis))[None]), High=high, Low=low, Out=out,
        P=gu.dev(orc.q2_repack_k64(raw)), Sum=sums2, TC=gu.dev(total), TE=gu.dev(te), TR=gu.dev(tr), WS=gu.dev(ws), **tiles)
    assert torch.equal(out, ref) and not bool(torch.isnan(out).any())
    want_q, want_s, want_d, want_ds, want_map, want_sum = orc.rotate_expert_a8(x, signs, ids, relative, offsets)
    codes = np.ascontiguousarray(raw.transpose(0, 2, 1, 3)).reshape(e, n, h // 8)
    weights = np.stack([orc.q2_integers(c, basis) for c in codes])
    np.testing.assert_array_equal(gu.host(out), orc.grouped_project(want_d, want_ds, weights, ws, counts, offsets))


def test_split_then_exact_grouped_replayed_from_a_graph_with_changed_inputs():
    # the replay sequence of tests/cuda/operators/e8p_exact.py:208-227: zeroed rows, new rows, the first rows again;
    # the tile list, the counts and Book are read on the device at every replay
    rng = np.random.default_rng(orc.SEED + 21)
    basis = orc.basis()
    bm, counts, n, k = 16, [17, 33], 320, 640
    e, rows = len(counts), sum(counts)
    a, raw, codes, ws, scale, weights = grouped_case(rng, counts, n, k, basis)
    offsets, te, tr, total, cap = tile_list(counts, bm)
    counts_np = np.asarray(counts, np.int32)
    d_a = gu.dev(a)
    low, high = empty_planes(rows, k, False)
    sums = torch.empty((rows,), **I32)
    out = torch.empty((rows, n), dtype=torch.float16, device=gu.DEV)
    d_counts = gu.dev(counts_np)
    split = gu.kernel("split_a8", rows=rows, K=k)
    gemm = gu.kernel("e8p_exact_grouped", rows=rows, E=e, tiles=cap, N=n, K=k, block_m=bm)
    args = dict(AS=gu.dev(scale), Book=gu.dev(orc.nibble_table(orc.selector_table(basis))[None]), Counts=d_counts, High=high,
                Low=low, Offsets=gu.dev(offsets), Out=out, P=gu.dev(orc.q2_repack_k64(raw)), Sum=sums, TC=gu.dev(total),
                TE=gu.dev(te), TR=gu.dev(tr), WS=gu.dev(ws))
    split(A=d_a, High=high, Low=low, Sum=sums)
    gemm(**args)
    gu.sync()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            split(stream=side.cuda_stream, A=d_a, High=high, Low=low, Sum=sums)
            gemm(stream=side.cuda_stream, **args)
    first = a.copy()
    for rows_now in (np.zeros_like(a), planted_rows(rng, rows, k), first):
        d_a.copy_(gu.dev(rows_now))
        out.fill_(float("nan"))
        gu.sync()
        graph.replay()
        gu.sync()
        np.testing.assert_array_equal(gu.host(out), orc.grouped_project(rows_now, scale[:, None], weights, ws, counts_np, offsets))
    # an expert that lost its rows between replays is skipped
    d_counts[0] = 0
    out.fill_(5.0)
    gu.sync()
    graph.replay()
    gu.sync()
    got = gu.host(out)
    assert (got[:counts[0]] == 5).all()
    np.testing.assert_array_equal(got[counts[0]:], orc.grouped_project(first, scale[:, None], weights, ws, counts_np, offsets)[counts[0]:])
