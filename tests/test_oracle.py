"""Pins the CPU oracle (oracle/reference.py, oracle/e8p_oracle.c) before anything trusts it.

Each check is chosen so that a plausible mistake fails: a wrong SIGN_BITS entry, a
dropped parity shift, a transposed table, a wrong outer-row spread, reciprocal
instead of divide in A8, swapped scale order in the epilogue.
"""
import ctypes
import itertools
import subprocess
from pathlib import Path

import numpy as np
import pytest

from oracle import reference as orc

ROOT = Path(__file__).resolve().parents[1]


@pytest.fixture(scope="module")
def table():
    return orc.basis()


@pytest.fixture(scope="module")
def clib():
    so = ROOT / "oracle" / "libe8p_oracle.so"
    if not so.exists():
        subprocess.check_call(["make", "-C", str(ROOT / "oracle")])
    return ctypes.CDLL(str(so))


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


# ---- codebook ------------------------------------------------------------
def test_basis_matches_reference_golden(table, golden_basis):
    # Row ORDER is fixed only by the reference's source; the golden holds its output.
    np.testing.assert_array_equal(table, golden_basis)


def test_basis_closed_form_invariants(table):
    t = table.astype(np.int32)
    assert table.shape == (256, 8) and table.dtype == np.int8
    assert set(np.unique(np.abs(t))) == {2, 6, 10}
    norms = (t * t).sum(1)
    inner, outer = t[:227], t[227:]
    assert (norms[:227] <= 160).all() and (norms[227:] == 192).all()
    n6 = (np.abs(inner) == 6).sum(1)
    n10 = (np.abs(inner) == 10).sum(1)
    # docs/quantization.md:44-50: 163 rows without a 10, 64 with exactly one 10
    assert ((n10 == 0) & (n6 <= 4)).sum() == 163
    assert ((n10 == 1) & (n6 <= 1)).sum() == 64
    assert ((np.abs(outer) == 6).sum(1) == 5).all() and len(outer) == 29
    # only the last coordinate is ever negative, and sum(B/4 ... ) parity rule holds
    assert (t[:, :7] > 0).all()
    assert ((np.abs(t).sum(1) // 4) % 2 == (t[:, 7] < 0)).all()
    assert (((t.sum(1)) // 4) % 2 == 0).all()  # canonical representative: even sum(B)/4
    assert len({tuple(r) for r in np.abs(t)}) == 256


def test_c_basis_agrees(table, clib):
    out = np.zeros((256, 8), np.int8)
    clib.orc_basis(_ptr(out))
    np.testing.assert_array_equal(out, table)


# ---- decoder ------------------------------------------------------------
ALL = np.arange(65536, dtype=np.uint16)


def test_decode_all_codes_unique_and_odd(table):
    grid = orc.e8p_decode(ALL, table)
    assert grid.shape == (65536, 8)
    assert (grid.astype(np.int32) % 2 != 0).all() and np.abs(grid.astype(np.int32)).max() == 11
    assert len(np.unique(grid, axis=0)) == 65536  # test_e8p.py:12-13


def test_decode_known_answers_by_hand(table):
    # code 0: basis row 0 = all 2, no flips, parity 0 -> all 3
    assert orc.e8p_decode(np.array([0], np.uint16), table)[0].tolist() == [3] * 8
    # code 1: u=1, p=1, m=0 -> no flips, shift -1 -> all 1
    assert orc.e8p_decode(np.array([1], np.uint16), table)[0].tolist() == [1] * 8
    # code 3: u=3, p=0, m=3 -> bits 0,1 flip coords 0 and 2 -> [-1,3,-1,3,3,3,3,3]
    assert orc.e8p_decode(np.array([3], np.uint16), table)[0].tolist() == [-1, 3, -1, 3, 3, 3, 3, 3]
    # code 0x10: u=16, p=1, m=17 -> bits 0,4 flip coords 0 and 1, shift -1
    assert orc.e8p_decode(np.array([0x10], np.uint16), table)[0].tolist() == [-3, -3, 1, 1, 1, 1, 1, 1]


def test_decode_against_scalar_formula_random_table():
    # same construction as test_vq.py:132-147 (random even table incl. zeros and negatives)
    rng = np.random.default_rng(orc.SEED)
    t = (rng.integers(-5, 6, (256, 8)) * 2).astype(np.int8)
    codes = np.array([0, 1, 127, 128, 255, 256, 32768, 65535], np.uint16)
    want = [orc.e8p_decode_scalar(c, t) for c in codes]
    np.testing.assert_array_equal(orc.e8p_decode(codes, t), want)
    some = rng.integers(0, 65536, 512).astype(np.uint16)
    np.testing.assert_array_equal(orc.e8p_decode(some, t), [orc.e8p_decode_scalar(c, t) for c in some])


def test_decode_against_palette_decoder():
    # literal palettes from test_vq.py:32-36: an independent statement of the decoder
    rng = np.random.default_rng(orc.SEED)
    t = rng.choice(np.array([-10, -6, -2, 0, 2, 6, 10], np.int8), (256, 8))
    book = orc.selector_table(t)
    parity = np.array([bin(int(c) & 255).count("1") & 1 for c in ALL], np.uint32)
    even = np.array([3, 7, 11, 1, -1, -5, -9, 1], np.int8)
    odd = np.array([1, 5, 9, -1, -3, -7, -11, -1], np.int8)
    got = np.empty((65536, 8), np.int8)
    base = book[ALL >> 8, 0]
    for lane, bit in enumerate(orc.SIGN_BITS):
        sel = ((base >> np.uint32(4 * lane)) & 7) ^ ((((ALL ^ parity) >> bit) & 1) * 4)
        got[:, lane] = np.where(parity == 1, odd[sel], even[sel])
    np.testing.assert_array_equal(got, orc.e8p_decode(ALL, t))


def test_decode_against_xor_nibble_identity(table):
    # v=(q-1)/2 equals h ^ mask with h=t/2, mask = (flip?0xE:0)^(parity?1:0): the identity behind
    # the reference's nibble decoder (test_vq.py:70-95, magic 0xEEE00E00) on the real basis.
    q = orc.e8p_decode(ALL, table).astype(np.int32)
    u = ALL.astype(np.int32) & 255
    p = np.array([bin(int(x)).count("1") & 1 for x in u])
    m = u ^ p
    h = table.astype(np.int32)[ALL >> 8] // 2
    for j, bit in enumerate(orc.SIGN_BITS):
        mask = np.where((m >> bit) & 1, 0xE, 0) ^ p
        v = ((h[:, j] & 15) ^ mask)
        v = np.where(v >= 8, v - 16, v)
        np.testing.assert_array_equal(2 * v + 1, q[:, j])


def test_decode_negation_symmetry(table):
    # lattice fact: flipping all 8 sign bits and the parity bit negates the vector
    q = orc.e8p_decode(ALL, table).astype(np.int32)
    neg = orc.e8p_decode((ALL ^ np.uint16(0xFE)).astype(np.uint16), table).astype(np.int32)
    np.testing.assert_array_equal(neg, -q)


def test_c_decode_agrees(table, clib):
    out = np.zeros((65536, 8), np.int8)
    clib.orc_decode_all(_ptr(table), _ptr(ALL), ctypes.c_int64(65536), _ptr(out))
    np.testing.assert_array_equal(out, orc.e8p_decode(ALL, table))


def test_selector_table_roundtrip_and_rejects(table):
    book = orc.selector_table(table)
    assert book.shape == (256, 1) and book.dtype == np.uint32 and book.nbytes == 1024
    mags = np.array([2, 6, 10, 0, -2, -6, -10, 0])
    back = np.stack([mags[(book[:, 0] >> np.uint32(4 * j)) & 7] for j in range(8)], 1)
    np.testing.assert_array_equal(back, table)
    assert not (book & np.uint32(0x88888888)).any()
    bad = table.copy()
    bad[0, 0] = 4
    with pytest.raises(ValueError):
        orc.selector_table(bad)


# ---- Q4 two-stage -------------------------------------------------------
def test_q4_exhaustive_fixture(table, clib):
    # quantization/test_e8p_q4.py:13-30: every coarse code once, residual by an LCG
    first = np.arange(65536, dtype=np.uint32).reshape(4096, 16)
    second = (first * np.uint32(32771) + np.uint32(97)) & np.uint32(65535)
    packed = first | (second << np.uint32(16))
    for a, b in ((3, 1), (4, 1), (7, 2)):
        w = orc.q4_integers(packed, table, (a, b))
        want = (a * orc.e8p_decode(first.astype(np.uint16), table).astype(np.int16)
                + b * orc.e8p_decode(second.astype(np.uint16), table).astype(np.int16)).reshape(4096, 128)
        np.testing.assert_array_equal(w, want)
        assert np.abs(want).max() <= 127
        cw = np.zeros((4096, 128), np.int8)
        clib.orc_q4_integers(_ptr(table), _ptr(packed), ctypes.c_int64(4096), ctypes.c_int64(128),
                             ctypes.c_int(a), ctypes.c_int(b), _ptr(cw))
        np.testing.assert_array_equal(cw, w)
    w41 = orc.q4_integers(packed, table, (4, 1)).astype(np.int32)
    assert np.abs(w41).max() == 55 and (w41 % 2 != 0).all()  # 4*odd + odd is odd, |.| <= 44+11


def test_q4_integers_gather_form_for_large_matrices_is_the_same_function(table, clib):
    # above 2^20 codes q4_integers gathers from e8p_decode of all 65 536 codes: same values as the
    # direct form (rows of it evaluated below the threshold) and as the C restatement
    rng = np.random.default_rng(orc.SEED + 17)
    packed = rng.integers(0, 2**32, (2100, 512), dtype=np.uint64).astype(np.uint32)
    big = orc.q4_integers(packed, table)
    assert big.dtype == np.int8 and big.shape == (2100, 4096)
    for first in (0, 777, 2000):
        np.testing.assert_array_equal(big[first:first + 100], orc.q4_integers(packed[first:first + 100], table))
    cw = np.zeros((64, 4096), np.int8)
    clib.orc_q4_integers(_ptr(table), _ptr(np.ascontiguousarray(packed[1500:1564])), ctypes.c_int64(64),
                         ctypes.c_int64(4096), ctypes.c_int(4), ctypes.c_int(1), _ptr(cw))
    np.testing.assert_array_equal(cw, big[1500:1564])


def test_k_major_layouts_are_lossless():
    rng = np.random.default_rng(orc.SEED)
    packed = rng.integers(0, 2**32, (17, 48), dtype=np.uint64).astype(np.uint32)
    for pk in (64, 128):
        km = orc.q4_pack_k(packed, pk)
        assert km.shape == (48 * 8 // pk, 17, pk // 8)
        np.testing.assert_array_equal(km.transpose(1, 0, 2).reshape(17, 48), packed)
    idx = rng.integers(0, 65536, (5, 32), dtype=np.uint16)
    k128 = orc.q2_pack_k128(idx)
    assert k128.shape == (2, 5, 16)
    np.testing.assert_array_equal(k128.transpose(1, 0, 2).reshape(5, 32), idx)
    src = rng.integers(0, 65536, (2, 3, 17, 16), dtype=np.uint16)
    k64 = orc.q2_repack_k64(src)
    np.testing.assert_array_equal(k64.reshape(2, 3, 2, 17, 8).transpose(0, 1, 3, 2, 4).reshape(src.shape), src)


# ---- A8 ------------------------------------------------------------------
def test_a8_edge_cases():
    x = np.zeros((4, 8), np.float16)
    x[1] = [127, -127, 63.5, 0.5, 1.5, 2.5, -0.5, -2.5]     # scale exactly 1: ties go to even
    x[2] = [1e-7, 0, 0, 0, 0, 0, 0, 0]                       # amax/127 under the 2^-24 floor
    x[3] = [254, 1, -1, 3, -3, 5, 127, -254]                 # scale exactly 2: halves tie
    q, s = orc.a8(x)
    assert s.dtype == np.float16 and s.shape == (4, 1) and q.dtype == np.int8
    assert s[0, 0] == 1 and (q[0] == 0).all()
    assert s[1, 0] == 1 and q[1].tolist() == [127, -127, 64, 0, 2, 2, 0, -2]
    assert s[2, 0] == np.float16(2.0**-24)
    assert q[2, 0] == int(np.rint(np.float32(np.float16(1e-7)) / np.float32(2.0**-24)))
    assert s[3, 0] == 2 and q[3].tolist() == [127, 0, 0, 2, -2, 2, 64, -127]


def test_a8_scale_is_divide_then_fp16_and_codes_clamp():
    rng = np.random.default_rng(orc.SEED)
    x = rng.normal(size=(64, 256)).astype(np.float16)
    x[0, 0] = 65504  # fp16 max
    q, s = orc.a8(x)
    amax = np.abs(x.astype(np.float32)).max(1)
    np.testing.assert_array_equal(s[:, 0], (amax / np.float32(127)).astype(np.float16))
    assert np.abs(q.astype(np.int32)).max() <= 127
    # fp16 rounding of the scale can push |x|/scale above 127.5: the clamp must catch it
    ratio = np.abs(x.astype(np.float32)) / s.astype(np.float32)
    assert (np.abs(q.astype(np.int32)) == np.minimum(np.rint(ratio), 127)).all()
    # grouped form
    qg, sg = orc.a8(x, 64)
    assert sg.shape == (64, 4)
    q0, s0 = orc.a8(x[:, :64])
    np.testing.assert_array_equal(qg[:, :64], q0)
    np.testing.assert_array_equal(sg[:, :1], s0)


def test_c_a8_agrees(clib):
    rng = np.random.default_rng(orc.SEED + 1)
    x = rng.normal(size=(9, 384)).astype(np.float16)
    x[3] = 0
    xf = np.ascontiguousarray(x.astype(np.float32))
    raw = np.zeros(9, np.float32)
    clib.orc_a8_scale(_ptr(xf), ctypes.c_int64(9), ctypes.c_int64(384), _ptr(raw))
    s16 = raw.astype(np.float16)
    sf = np.ascontiguousarray(s16.astype(np.float32))
    q = np.zeros((9, 384), np.int8)
    clib.orc_a8_codes(_ptr(xf), _ptr(sf), ctypes.c_int64(9), ctypes.c_int64(384), _ptr(q))
    wq, ws = orc.a8(x)
    np.testing.assert_array_equal(s16, ws[:, 0])
    np.testing.assert_array_equal(q, wq)


# ---- contraction + epilogue ---------------------------------------------
def test_int_dot_matches_bruteforce_at_extremes(clib):
    rng = np.random.default_rng(orc.SEED)
    a = rng.integers(-128, 128, (5, 640), dtype=np.int64).astype(np.int8)
    w = rng.integers(-128, 128, (7, 640), dtype=np.int64).astype(np.int8)
    a[0] = -128
    w[0] = -128
    a[1] = 127
    w[1] = -128
    np.testing.assert_array_equal(orc.int_dot(a, w), orc.int_dot_bruteforce(a, w))
    assert orc.int_dot(a, w)[0, 0] == 128 * 128 * 640
    c = np.zeros((5, 7), np.int32)
    clib.orc_int_dot(_ptr(a), _ptr(w), ctypes.c_int64(5), ctypes.c_int64(7), ctypes.c_int64(640), _ptr(c))
    np.testing.assert_array_equal(c, orc.int_dot(a, w))


def test_project_power_of_two_scales_are_exact():
    # tests/cuda/operators/int8_projection.py:25-41: with 2^-6 and 2^-7 every product is exact
    rng = np.random.default_rng(orc.SEED)
    for m, n, k in ((1, 48, 2560), (3, 65, 128), (17, 129, 640)):
        a = rng.integers(-128, 128, (m, k), dtype=np.int64).astype(np.int8)
        w = rng.integers(-128, 128, (n, k), dtype=np.int64).astype(np.int8)
        ws = np.full(n, 0.015625, np.float16)
        ts = np.full(m, 0.0078125, np.float16)
        out32 = orc.project(a, ts, w, ws, np.float32)
        exact = orc.int_dot_bruteforce(a, w).astype(np.float64) * 2.0**-13
        np.testing.assert_array_equal(out32.astype(np.float64), exact)
        np.testing.assert_array_equal(orc.project(a, ts, w, ws), exact.astype(np.float16))


def test_rescale_order_is_weight_scale_first(clib):
    # (acc*ws)*as and acc*(ws*as) differ in fp32 for suitable values: pin the order
    acc = np.array([[16777217 // 3]], np.int32)
    ws = np.array([0.0123], np.float16)
    ts = np.array([0.0071], np.float16)
    got = orc.rescale(acc, ws, ts, np.float32)[0, 0]
    want = np.float32(np.float32(np.float32(acc[0, 0]) * np.float32(ws[0])) * np.float32(ts[0]))
    assert got == want
    found = False
    rng = np.random.default_rng(1)
    for _ in range(2000):
        a = np.int32(rng.integers(1, 2**24))
        s1, s2 = np.float16(rng.uniform(0.005, 0.02)), np.float16(rng.uniform(0.001, 0.01))
        x = np.float32(np.float32(a) * np.float32(s1)) * np.float32(s2)
        y = np.float32(a) * np.float32(np.float32(s1) * np.float32(s2))
        if x != y:
            assert orc.rescale(np.array([[a]], np.int32), np.array([s1]), np.array([s2]), np.float32)[0, 0] == x
            out = np.zeros(1, np.float32)
            clib.orc_rescale(_ptr(np.array([a], np.int32)), _ptr(np.array([s1], np.float32)),
                             _ptr(np.array([s2], np.float32)), ctypes.c_int64(1), ctypes.c_int64(1), _ptr(out))
            assert out[0] == x
            found = True
            break
    assert found


def test_q4_dot_fused_c_path_agrees(table, clib):
    rng = np.random.default_rng(orc.SEED)
    packed = rng.integers(0, 2**32, (33, 32), dtype=np.uint64).astype(np.uint32)
    a = rng.integers(-128, 128, (3, 256), dtype=np.int64).astype(np.int8)
    acc = np.zeros((3, 33), np.int32)
    clib.orc_q4_dot(_ptr(table), _ptr(packed), _ptr(a), ctypes.c_int64(3), ctypes.c_int64(33),
                    ctypes.c_int64(256), _ptr(acc))
    np.testing.assert_array_equal(acc, orc.int_dot(a, orc.q4_integers(packed, table)))


# ---- MoE -----------------------------------------------------------------
def test_router_topk_ties_signed_zero_and_extremes():
    # tests/cuda/operators/moe.py:25-57
    rng = np.random.default_rng(orc.SEED)
    for m, e, k in ((1, 512, 10), (8, 512, 10), (17, 37, 10), (3, 5, 5), (1, 1, 1)):
        logits = (rng.normal(size=(m, e)) * 5).astype(np.float32)
        logits[0] = 0
        if m > 1:
            logits[1] = -10000
            logits[1, -1] = 10000
        if m > 2:
            logits[2] = -1
            logits[2, :k] = 0
            logits[2, 0] = -0.0
        for renorm in (False, True):
            ids, prob = orc.router_topk(logits, k, renorm)
            assert ids[0].tolist() == list(range(k))
            if m > 1:
                assert ids[1, 0] == e - 1 and ids[1, 1:].tolist() == list(range(k - 1))
            if m > 2:
                assert ids[2].tolist() == list(range(k))
            for row in range(m):
                order = sorted(range(e), key=lambda j: (-float(logits[row, j]) + 0.0, j))[:k]
                assert ids[row].tolist() == order
            soft = np.exp(logits.astype(np.float64) - logits.max(1, keepdims=True))
            soft /= soft.sum(1, keepdims=True)
            want = np.take_along_axis(soft, ids.astype(np.int64), 1)
            if renorm:
                want /= want.sum(1, keepdims=True)
            np.testing.assert_allclose(prob, want, atol=2e-6)


def test_routing_metadata_by_enumeration():
    rng = np.random.default_rng(orc.SEED)
    m, e, k, bm = 37, 16, 4, 8
    ids = np.stack([rng.permutation(e)[:k] for _ in range(m)]).astype(np.int32)
    counts, rel = orc.expert_histogram(ids, e)
    np.testing.assert_array_equal(counts, np.bincount(ids.ravel(), minlength=e))
    flat = ids.ravel()
    for i, ex in enumerate(flat):
        assert rel.ravel()[i] == (flat[:i] == ex).sum()
    rows, tiles, total = orc.expert_offsets(counts, bm)
    assert rows[0] == 0 and (np.diff(rows) == counts[:-1]).all()
    assert total[0] == sum(-(-int(c) // bm) for c in counts)
    cap = orc.tile_capacity(m * k, e, bm)
    te, tr = orc.expert_tiles(counts, tiles, bm, cap)
    listed = [(int(a), int(b)) for a, b in zip(te[: total[0]], tr[: total[0]])]
    assert listed == [(ex, t * bm) for ex in range(e) for t in range(-(-int(counts[ex]) // bm))]
    assert total[0] <= cap
    a_q = rng.integers(-127, 128, (m, 64), dtype=np.int64).astype(np.int8)
    a_s = rng.uniform(0.01, 0.02, (m, 1)).astype(np.float16)
    d, ds, slot = orc.expert_dispatch(a_q, a_s, ids, rel, rows)
    assert sorted(slot.ravel().tolist()) == list(range(m * k))  # a permutation of the slots
    for row, rank in itertools.product(range(m), range(k)):
        s = slot[row, rank]
        assert rows[ids[row, rank]] <= s < rows[ids[row, rank]] + counts[ids[row, rank]]
        np.testing.assert_array_equal(d[s], a_q[row])
        assert ds[s, 0] == a_s[row, 0]


def test_combine_skips_invalid_slots_and_matches_formula():
    rng = np.random.default_rng(orc.SEED)
    m, h, slots, k = 5, 33, 12, 3
    ex = rng.normal(size=(slots, h)).astype(np.float16)
    sm = rng.integers(0, slots, (m, k)).astype(np.int32)
    sm[0, :2] = [-1, slots]
    prob = rng.uniform(0, 1, (m, k)).astype(np.float32)
    shared = rng.normal(size=(m, h)).astype(np.float16)
    gate = rng.normal(size=m).astype(np.float16)
    got = orc.moe_combine(ex, sm, prob, shared, gate)
    want = np.zeros((m, h), np.float64)
    for r in range(m):
        for j in range(k):
            if 0 <= sm[r, j] < slots:
                want[r] += ex[sm[r, j]].astype(np.float64) * prob[r, j]
        want[r] += shared[r].astype(np.float64) / (1 + np.exp(-float(gate[r])))
    np.testing.assert_allclose(got.astype(np.float64), want, atol=2e-3, rtol=2e-3)
    nos = orc.moe_combine(ex, sm, prob)
    assert nos.dtype == np.float16 and nos.shape == (m, h)


def test_swiglu_matches_closed_form():
    g = np.array([[-20, -1, 0, 1, 20, 3.5]], np.float16)
    u = np.array([[2, 2, 2, 2, 2, -1.25]], np.float16)
    got = orc.swiglu_fp16(np.concatenate([g, u], 1)).astype(np.float64)
    gf, uf = g.astype(np.float64), u.astype(np.float64)
    np.testing.assert_allclose(got, gf / (1 + np.exp(-gf)) * uf, rtol=2e-3, atol=1e-7)
    assert got[0, 2] == 0 and abs(got[0, 4] - 40) < 0.05


# ---- rotation (the producer of A8 activations in the real model) --------------------------------
def test_rotate_is_the_scaled_sylvester_hadamard_and_exact_on_integers():
    from scipy.linalg import hadamard
    rng = np.random.default_rng(orc.SEED)
    h = hadamard(128).astype(np.int64)
    x = rng.integers(-64, 65, (3, 256))
    signs = rng.choice(np.array([-1, 1], np.int8), 256)
    got = orc.rotate(x.astype(np.float32), signs)
    # before the final scaling every intermediate is an integer below 2**24: fp32 is exact
    want = np.concatenate([(x * signs)[:, :128] @ h, (x * signs)[:, 128:] @ h], axis=1)
    np.testing.assert_array_equal(got, (want.astype(np.float32) * np.float32(128**-0.5)))
    # a transposed or mis-ordered butterfly fails on a unit vector: column 5 of H, block 1
    e = np.zeros((1, 256), np.float32)
    e[0, 128 + 5] = 1
    np.testing.assert_array_equal(orc.rotate(e, np.ones(256, np.int8))[0, 128:],
                                  h[:, 5].astype(np.float32) * np.float32(128**-0.5))
    assert not orc.rotate(e, np.ones(256, np.int8))[0, :128].any()


def test_rotate_preserves_dots_and_is_an_involution_up_to_signs():
    # python/orinfer_build/quantization/test_vq.py:123-130
    rng = np.random.default_rng(20261002)
    x = rng.normal(size=(5, 256)).astype(np.float32)
    w = rng.normal(size=(7, 256)).astype(np.float32)
    s = rng.choice(np.array([-1, 1], np.int8), 256)
    np.testing.assert_allclose(orc.rotate(x, s) @ orc.rotate(w, s).T, x @ w.T, atol=2e-5, rtol=2e-5)
    inverse = orc.rotate(orc.rotate(x, s), np.ones(256, np.int8)) * s
    np.testing.assert_allclose(inverse, x, atol=1e-6, rtol=1e-5)
    with pytest.raises(ValueError):
        orc.rotate(x[:, :100], s[:100])
    with pytest.raises(ValueError):
        orc.rotate(x, np.zeros(256, np.int8))


def test_rotate_a8_quantises_the_materialised_fp16_values():
    rng = np.random.default_rng(orc.SEED + 3)
    x = rng.normal(size=(4, 384)).astype(np.float16)
    signs = rng.choice(np.array([-1, 1], np.int8), 384)
    q, s = orc.rotate_a8(x, signs)
    rotated = orc.rotate(x.astype(np.float32), signs).astype(np.float16)
    wq, ws = orc.a8(rotated)
    np.testing.assert_array_equal(q, wq)
    np.testing.assert_array_equal(s, ws)
    # a power-of-two row: one non-zero input of 2**-3 gives +-2**-3 * 128**-0.5 everywhere in its block
    x = np.zeros((1, 128), np.float16)
    x[0, 7] = 0.125
    q, s = orc.rotate_a8(x, np.ones(128, np.int8))
    assert set(np.abs(q[0]).tolist()) == {127} and s.shape == (1, 1)
    # zero row: scale 1, codes 0
    q, s = orc.rotate_a8(np.zeros((1, 128), np.float16), np.ones(128, np.int8))
    assert not q.any() and float(s[0, 0]) == 1.0
    # the SwiGLU form rotates fp16(silu(gate) * up)
    gu = rng.normal(size=(2, 256)).astype(np.float16)
    q, s = orc.rotate_a8(gu, signs[:128], swiglu=True)
    wq, ws = orc.rotate_a8(orc.swiglu_fp16(gu), signs[:128])
    np.testing.assert_array_equal(q, wq)
    np.testing.assert_array_equal(s, ws)


def test_residual_norm_closed_forms():
    """Cases the mathematics fixes (kernels/cuda/operators/op02_residual_norm.py:13-38)."""
    k = 256
    # a constant row c with zero weights normalises to c / sqrt(c^2 + eps): +-1 to fp16 accuracy,
    # and the residual sum comes back unrounded in fp32
    x = np.full((1, k), 0.5, np.float16)
    r = np.full((1, k), 2.0 ** -20, np.float32)
    y, total = orc.residual_norm(x, r, np.zeros(k, np.float16))
    assert total.dtype == np.float32 and (total == np.float32(0.5) + np.float32(2.0 ** -20)).all()
    assert (y == np.float16(1.0)).all()
    y, _ = orc.residual_norm(-x, -r, np.zeros(k, np.float16))
    assert (y == np.float16(-1.0)).all()
    # zero-centred weights add one to the gain; plain weights do not
    w = np.full(k, 0.5, np.float16)
    y, _ = orc.residual_norm(x, r, w)
    assert (y == np.float16(1.5)).all()
    y, _ = orc.residual_norm(x, r, w, zero_centered=False)
    assert (y == np.float16(0.5)).all()
    # scale invariance: doubling x and r leaves the normalised row unchanged up to the last place
    # (epsilon and the rounding of the reciprocal root do not scale)
    rng = np.random.default_rng(orc.SEED + 21)
    x = rng.normal(size=(3, 512)).astype(np.float16)
    r = rng.normal(size=(3, 512)).astype(np.float32)
    w = (rng.normal(size=512) * 0.1).astype(np.float16)
    y1, t1 = orc.residual_norm(x, r, w)
    y2, t2 = orc.residual_norm(x * np.float16(2), r * 2, w)
    np.testing.assert_array_equal(t2, 2 * t1)
    np.testing.assert_allclose(y1.astype(np.float64), y2.astype(np.float64), rtol=2 ** -10, atol=2 ** -24)
    # against a float64 evaluation of the formula; unit mean square before the gain
    t64 = x.astype(np.float64) + r.astype(np.float64)
    want = t64 / np.sqrt((t64 ** 2).mean(axis=1, keepdims=True) + 1e-6) * (1.0 + w.astype(np.float64))
    np.testing.assert_allclose(y1.astype(np.float64), want, rtol=2 ** -10, atol=2 ** -24)
    # the zero row: epsilon keeps the reciprocal finite, the row stays zero
    y, t = orc.residual_norm(np.zeros((1, k), np.float16), np.zeros((1, k), np.float32), w[:k])
    assert not y.any() and not t.any()


def test_residual_norm_rotate_a8_is_the_rotation_of_the_normalised_row():
    rng = np.random.default_rng(orc.SEED + 22)
    x = rng.normal(size=(4, 512)).astype(np.float16)
    r = rng.normal(size=(4, 512)).astype(np.float32)
    x[2], r[2] = 0, 0
    w = (rng.normal(size=512) * 0.1).astype(np.float16)
    signs = rng.choice(np.array([-1, 1], np.int8), 512)
    y, total, q, s = orc.residual_norm_rotate_a8(x, r, w, signs)
    wy, wt = orc.residual_norm(x, r, w)
    wq, ws = orc.rotate_a8(wy, signs)
    for got, want in ((y, wy), (total, wt), (q, wq), (s, ws)):
        np.testing.assert_array_equal(got, want)
    assert not q[2].any() and float(s[2, 0]) == 1.0  # models/qwen35/check_rows.py:186-190


def test_route_project_indexes_banks_directly():
    """integer_vq.py:380-444 against a float64 dot (the reference test's oracle, flash_mtp_optimization.py:159-166)."""
    rng = np.random.default_rng(orc.SEED + 31)
    e, routes, n, k = 5, 3, 7, 256
    table = (rng.integers(-63, 64, (256, 8)) * 2).astype(np.int8)
    codes = rng.integers(0, 65536, (e, n, k // 8), dtype=np.uint16)
    weights = np.stack([orc.q2_integers(c, table) for c in codes])
    assert np.abs(weights.astype(np.int32)).max() <= 127 and (weights.astype(np.int32) % 2 != 0).all()
    ws = np.full((e, n), 0.015625, np.float16)
    ids = np.array([[4, 0, 4]], np.int32)
    for shared in (True, False):
        rows = 1 if shared else routes
        a = rng.integers(-128, 128, (rows, k), dtype=np.int8)
        scale = np.full(rows, 0.0078125, np.float16)
        got = orc.route_project(a, scale, weights, ws, ids, shared)
        for route in range(routes):
            row = 0 if shared else route
            acc = (weights[ids[0, route]].astype(np.float64) * a[row].astype(np.float64)).sum(-1)
            want = (np.float32(acc) * np.float32(0.015625)) * np.float32(0.0078125)
            np.testing.assert_array_equal(got[route], want.astype(np.float16))
        if shared:
            np.testing.assert_array_equal(got[0], got[2])  # the same expert twice
    # the raw table words are the table bytes, little endian, coordinates 0-3 then 4-7
    words = orc.raw_table_words(table)
    assert words.shape == (256, 2) and words.dtype == np.uint32
    assert ((words[9, 1] >> 16) & 255) == (int(table[9, 6]) & 255)


def test_single_route_metadata_is_the_general_metadata_of_one_token():
    """moe.py:659-709: with distinct ids the one-token form equals histogram + offsets + tiles
    (moe.py:177-282) at any tile height."""
    rng = np.random.default_rng(orc.SEED + 41)
    for experts, top_k in ((512, 10), (128, 8), (16, 16), (7, 1)):
        ids = rng.permutation(experts)[:top_k].astype(np.int32)[None, :]
        capacity = top_k + 3
        counts, relative, offsets, tile_offsets, tile_expert, tile_row, tile_count = orc.single_route_metadata(
            ids, experts, capacity)
        want_counts, want_relative = orc.expert_histogram(ids, experts)
        np.testing.assert_array_equal(counts, want_counts)
        np.testing.assert_array_equal(relative, want_relative)
        for block_m in (8, 32):
            want_offsets, want_tile_offsets, want_total = orc.expert_offsets(want_counts, block_m)
            want_expert, want_row = orc.expert_tiles(want_counts, want_tile_offsets, block_m, capacity)
            np.testing.assert_array_equal(offsets, want_offsets)
            np.testing.assert_array_equal(tile_offsets, want_tile_offsets)
            np.testing.assert_array_equal(tile_count, want_total)
            np.testing.assert_array_equal(tile_expert, want_expert)
            np.testing.assert_array_equal(tile_row, want_row)
        assert tile_expert[:top_k].tolist() == sorted(ids.ravel().tolist()) and (tile_expert[top_k:] == -1).all()


def test_expert_partition_covers_every_row_once():
    """expert_partition.py:1-5: both lists keep the global row offsets and own disjoint tiles."""
    rng = np.random.default_rng(orc.SEED + 43)
    counts = rng.integers(0, 40, 23).astype(np.int32)
    counts[[0, 5]] = 0
    counts[7], counts[8] = 8, 9  # on and just above the threshold
    hot_m, cold_m, cold_rows = 16, 4, 8
    total = int(counts.sum())
    part = orc.expert_partition(counts, hot_m, cold_m, cold_rows, orc.tile_capacity(total, 23, hot_m),
                                orc.tile_capacity(total, 23, cold_m))
    seen = np.zeros(total, np.int32)
    for experts, rows, count, height, hot in (("TileExpert", "TileRow", "TileCount", hot_m, True),
                                              ("ColdExpert", "ColdRow", "ColdCount", cold_m, False)):
        live = int(part[count][0])
        assert (part[experts][live:] == -1).all()
        for e, first in zip(part[experts][:live], part[rows][:live]):
            assert (counts[e] > cold_rows) == hot
            rows_in_tile = min(height, counts[e] - first)
            assert rows_in_tile > 0
            seen[part["RowOffsets"][e] + first : part["RowOffsets"][e] + first + rows_in_tile] += 1
        assert list(part[experts][:live]) == sorted(part[experts][:live])
    assert (seen == 1).all()
    # a threshold below every count gives the plain tile list of moe.py:214-282 in the hot list
    plain = orc.expert_partition(np.maximum(counts, 1), hot_m, cold_m, 0, 64, 64)
    offsets, tile_offsets, tile_total = orc.expert_offsets(np.maximum(counts, 1), hot_m)
    tile_expert, tile_row = orc.expert_tiles(np.maximum(counts, 1), tile_offsets, hot_m, 64)
    np.testing.assert_array_equal(plain["RowOffsets"], offsets)
    np.testing.assert_array_equal(plain["TileOffsets"], tile_offsets)
    np.testing.assert_array_equal(plain["TileCount"], tile_total)
    np.testing.assert_array_equal(plain["TileExpert"], tile_expert)
    np.testing.assert_array_equal(plain["TileRow"], tile_row)
    assert plain["ColdCount"][0] == 0


def test_q4_embedding_inverts_the_rotation_of_a_rotated_row():
    """Weights that are the rotation of a known vector come back as that vector: the embedding
    kernel's formula is the inverse rotation (H is an involution up to the 1/128 scaling)."""
    rng = np.random.default_rng(orc.SEED + 21)
    table = orc.basis()
    packed = rng.integers(0, 2**32, (6, 32), dtype=np.uint32)          # vocab 6, hidden 256
    weights = orc.q4_integers(packed, table).astype(np.float32)
    scales = np.array([0.5, 0.25, 1.0, 0.125, 2.0, 0.0625], np.float16)  # powers of two: exact scaling
    signs = rng.choice(np.array([-1, 1], np.int8), 256)
    got = orc.q4_embedding(np.array([3, -1, 0, 6, 5]), packed, table, scales, signs)
    assert got.shape == (5, 256) and not got[1].any() and not got[3].any()
    from scipy.linalg import hadamard
    h = hadamard(128).astype(np.float64)
    for row, token in ((0, 3), (2, 0), (4, 5)):
        blocks = weights[token].reshape(2, 128).astype(np.float64) @ h
        want = blocks.reshape(256) * 128**-0.5 * float(scales[token]) * signs
        np.testing.assert_allclose(got[row].astype(np.float64), want, rtol=2e-3, atol=1e-3)
        # rotating the embedding again (with the signs) returns the scaled integer weights
        again = orc.rotate(got[row].astype(np.float32)[None, :], signs)[0]
        np.testing.assert_allclose(again, weights[token] * float(scales[token]), atol=0.03 * float(scales[token]) * 8)


def test_int8_swiglu_is_the_fp16_pair_through_the_swiglu_boundary():
    rng = np.random.default_rng(orc.SEED + 50)
    a_q = rng.integers(-127, 128, (5, 128), dtype=np.int8)
    a_s = rng.uniform(0.01, 0.02, 5).astype(np.float16)
    gate, up = (rng.integers(-127, 128, (24, 128), dtype=np.int8) for _ in range(2))
    gs, us = (rng.uniform(0.001, 0.01, 24).astype(np.float16) for _ in range(2))
    got = orc.int8_swiglu(a_q, a_s, gate, gs, up, us)
    pair = np.concatenate([orc.project(a_q, a_s, gate, gs), orc.project(a_q, a_s, up, us)], axis=1)
    # same boundary as the stand-alone SwiGLU operator, whose sigmoid is written differently:
    # equal to within one fp16 step
    stable = orc.swiglu_fp16(pair).astype(np.float32)
    np.testing.assert_allclose(got.astype(np.float32), stable, rtol=2e-3, atol=1e-6)
    # hand-computed entry in float64
    g, u = float(pair[2, 3]), float(pair[2, 24 + 3])
    assert abs(float(got[2, 3]) - g / (1 + np.exp(-g)) * u) <= 1e-3 * abs(g * u) + 1e-7
    # a very negative gate gives (signed) zero, not NaN
    big = orc.int8_swiglu(np.full((1, 128), 127, np.int8), np.array([1.0], np.float16), -np.full((1, 128), 127, np.int8),
                          np.array([2.0**-6], np.float16), np.ones((1, 128), np.int8), np.array([1.0], np.float16))
    assert float(orc.project(np.full((1, 128), 127, np.int8), np.array([1.0], np.float16), -np.full((1, 128), 127, np.int8),
                             np.array([2.0**-6], np.float16))[0, 0]) == -32256.0  # fp16(-32258.0)
    assert float(big[0, 0]) == 0.0


def test_rotate_expert_a8_is_rotation_then_dispatch_and_its_sum_closes_the_nibble_identity():
    """The fused hand-over adds no arithmetic: its pieces are `rotate_a8` (pinned by the Sylvester
    matrix above) and `expert_dispatch` (pinned by enumeration).  What is new is Sum; the reference
    needs it because its planes are unsigned nibbles: sum_k (low + 16 high) - 256 [q < 0] = sum_k q,
    and an int dot with unsigned planes is repaired by exactly that term."""
    rng = np.random.default_rng(orc.SEED + 77)
    m, k, e, top_k = 9, 256, 6, 3
    x = rng.normal(size=(m, k)).astype(np.float16)
    x[4] = 0
    signs = rng.choice(np.array([-1, 1], np.int8), k)
    ids = np.stack([rng.choice(e, top_k, replace=False) for _ in range(m)]).astype(np.int32)
    counts, relative = orc.expert_histogram(ids, e)
    offsets, _, _ = orc.expert_offsets(counts, 16)
    q, s, d, ds, slot_map, slot_sum = orc.rotate_expert_a8(x, signs, ids, relative, offsets)
    want_q, want_s = orc.rotate_a8(x, signs)
    assert np.array_equal(q, want_q) and np.array_equal(s, want_s)
    assert sorted(slot_map.ravel().tolist()) == list(range(m * top_k))  # a permutation of the slots
    for row in range(m):
        for rank in range(top_k):
            slot = slot_map[row, rank]
            assert offsets[ids[row, rank]] <= slot < offsets[ids[row, rank]] + counts[ids[row, rank]]
            assert np.array_equal(d[slot], q[row]) and ds[slot, 0] == s[row, 0]
            assert slot_sum[slot] == int(q[row].astype(np.int64).sum())
    low, high = orc.nibble_planes(q)
    assert low.max() <= 15 and high.max() <= 15
    unsigned = low.astype(np.int64) + 16 * high.astype(np.int64)
    assert np.array_equal(unsigned - 256 * (q < 0), q.astype(np.int64))
    w = rng.integers(-8, 8, (5, k)).astype(np.int64)
    repaired = unsigned @ w.T - 256 * ((q < 0).astype(np.int64) @ w.T)
    assert np.array_equal(repaired, q.astype(np.int64) @ w.T)
    # shared routing and no routing keep the per-row sum
    q2, s2, ds2, map2, row_sum = orc.rotate_expert_a8(x, signs, ids, relative, offsets, scatter=False)
    assert np.array_equal(map2, slot_map) and np.array_equal(ds2, ds) and np.array_equal(row_sum, q.astype(np.int32).sum(1))
    q3, s3, sum3 = orc.rotate_expert_a8(x, signs)
    assert np.array_equal(sum3, row_sum) and row_sum[4] == 0 and s[4, 0] == 1


def test_q2_patches_override_one_weight_per_row_and_group(table):
    """Patch words (vq.py:184-194; the word the reference's own test plants, tests/cuda/operators/e8p_selector.py:38):
    checked against a scalar loop over every (row, group) and on hand-built words."""
    rng = np.random.default_rng(orc.SEED + 77)
    n, k = 11, 384
    codes = rng.integers(0, 65536, (n, k // 8), dtype=np.uint16)
    words = rng.integers(0, 65536, (n, k // 128), dtype=np.uint16)
    words[0, 0] = 32768 | (128 << 7) | 127  # valid, value byte 0x80 = -128, last position of group 0
    words[1, 1] = (5 << 7) | 3              # not valid: ignored
    plain = orc.q2_integers(codes, table)
    got = orc.q2_integers(codes, table, words)
    assert got[0, 127] == -128 and got[1, 128 + 3] == plain[1, 128 + 3]
    want = plain.copy()
    changed = 0
    for row in range(n):
        for group in range(k // 128):
            word = int(words[row, group])
            if word & 0x8000:
                value = (word >> 7) & 0xFF
                want[row, group * 128 + (word % 128)] = value - 256 if value >= 128 else value
                changed += 1
    np.testing.assert_array_equal(got, want)
    assert int((got != plain).sum()) <= changed and changed > 5
    # no valid bit anywhere: nothing changes; wrong shape is refused
    np.testing.assert_array_equal(orc.q2_integers(codes, table, words & np.uint16(0x7FFF)), plain)
    with pytest.raises(ValueError):
        orc.q2_integers(codes, table, words[:, :2])


def test_decode_with_zero_coordinates_and_the_selector_table_for_them():
    """Tables with zeros (the selector decoder's domain, vq.py:74-93): a zero coordinate decodes to 1 - 2p
    whatever its sign bit says, and its selector nibble is 3."""
    rng = np.random.default_rng(orc.SEED + 78)
    general = rng.choice(np.array([-10, -6, -2, 0, 2, 6, 10], np.int8), (256, 8))
    general[7] = 0
    book = orc.selector_table(general)
    assert int(book[7, 0]) == 0x33333333
    decoded = orc.e8p_decode(ALL, general).reshape(256, 256, 8)  # [basis row, low byte, coordinate]
    parity = np.array([bin(u).count("1") & 1 for u in range(256)])
    for u in (0, 1, 2, 0x55, 0xFE, 0xFF):
        assert decoded[7, u].tolist() == [1 - 2 * parity[u]] * 8
    zero_row, zero_col = np.nonzero(general == 0)
    np.testing.assert_array_equal(decoded[zero_row, :, zero_col], np.broadcast_to(1 - 2 * parity, (len(zero_row), 256)))
    some = rng.integers(0, 65536, 300)
    np.testing.assert_array_equal(orc.e8p_decode(some.astype(np.uint16), general),
                                  [orc.e8p_decode_scalar(c, general) for c in some])


def test_plane_words_follow_the_reference_masks_and_its_test():
    """split_planes against the mask-and-shift form of kernels/cuda/model/e8p_core.py:63-78 and against the statement of
    tests/cuda/operators/e8p_exact.py:196-206 (low + 16 high == codes permuted by [0, 2, 1, 3, 4, 6, 5, 7])."""
    rng = np.random.default_rng(orc.SEED)
    a = rng.integers(-128, 128, (7, 256), dtype=np.int8)
    a[:, :4] = np.array([-128, -1, 0, 127], np.int8)
    low, high, total = orc.split_planes(a)
    x = a.view("<u4").reshape(7, 32, 2)[:, :, 0]
    y = a.view("<u4").reshape(7, 32, 2)[:, :, 1]
    np.testing.assert_array_equal(low, (x & 0x0F0F) | ((x >> 12) & 0xF0F0) | ((y << 16) & 0x0F0F0000) | ((y << 4) & 0xF0F00000))
    np.testing.assert_array_equal(high, ((x >> 4) & 0x0F0F) | ((x >> 16) & 0xF0F0) | ((y << 12) & 0x0F0F0000) | (y & 0xF0F00000))
    # a word by hand: codes -128, -1, 0, 127, 5, -3, 17, -16 are bytes 80 FF 00 7F 05 FD 11 F0; low nibbles
    # 0 F 0 F 5 D 1 0 and high nibbles 8 F 0 7 0 F 1 F land at positions [0, 2, 1, 3, 4, 6, 5, 7]
    hand = np.array([[-128, -1, 0, 127, 5, -3, 17, -16] * 16], np.int8)
    hl, hh, ht = orc.split_planes(hand)
    assert hl[0, 0] == 0x0D15FF00 and hh[0, 0] == 0xFF107F08 and ht[0] == 16
    shifts = np.arange(0, 32, 4, dtype=np.uint64)
    lo = ((low.astype(np.uint64)[..., None] >> shifts) & 15).astype(np.int64).reshape(7, 256)
    hi = ((high.astype(np.uint64)[..., None] >> shifts) & 15).astype(np.int64).reshape(7, 256)
    hi = np.where(hi >= 8, hi - 16, hi)
    np.testing.assert_array_equal(lo + 16 * hi, a.reshape(7, 32, 8)[:, :, [0, 2, 1, 3, 4, 6, 5, 7]].reshape(7, 256))
    np.testing.assert_array_equal(orc.planes_values(low, high), a)
    np.testing.assert_array_equal(total, a.astype(np.int64).sum(axis=1))
    grouped = orc.planes_group_major(low)
    assert grouped.shape == (4, 7, 8) and grouped[2, 5, 3] == low[5, 19]
    np.testing.assert_array_equal(orc.planes_row_major(grouped), low)


def test_nibble_table_and_decode_are_the_selector_decode_halved(table):
    """2 y + 1 == e8p_decode over all 65 536 codes, on the real basis and on a random nonzero one
    (python/orinfer_build/quantization/vq.py:105-118, kernels/cuda/model/e8p_core.py:7-10); the table itself against
    the literal palette of vq.py:115 for one row; zero coordinates are refused."""
    codes = np.arange(65536, dtype=np.uint16)
    rng = np.random.default_rng(orc.SEED)
    for basis in (table, rng.choice(np.array([-10, -6, -2, 2, 6, 10], np.int8), (256, 8))):
        nibbles = orc.nibble_table(orc.selector_table(basis))
        assert nibbles.shape == (256, 1) and nibbles.dtype == np.uint32
        np.testing.assert_array_equal(2 * orc.nibble_decode(codes, nibbles) + 1, orc.e8p_decode(codes, basis))
    row = np.array([[2, -6, 10, -2, 6, -10, 2, 6]] * 256, np.int8)
    # halves 1 -3 5 -1 3 -5 1 3 in the order [0, 2, 1, 3, 4, 6, 5, 7]: 1, 5, -3, -1, 3, 1, -5, 3
    assert orc.nibble_table(orc.selector_table(row))[0, 0] == 0x3B13FD51
    zeros = table.copy()
    zeros[3, 2] = 0
    with pytest.raises(ValueError):
        orc.nibble_table(orc.selector_table(zeros))


def test_plane_project_is_project_when_sum_is_the_row_sum_and_adds_what_it_is_given(table):
    """2 (y . a) + Sum == w . a for w = 2 y + 1 (kernels/cuda/model/e8p_exact.py:3-4); two-stage codes:
    y = 4 y_coarse + y_fine and 5 Sum (e8p_core.py:154-170); a planted Sum moves every integer by its difference."""
    rng = np.random.default_rng(orc.SEED + 4)
    n, k, rows = 9, 256, 5
    a = rng.integers(-128, 128, (rows, k), dtype=np.int8)
    low, high, total = orc.split_planes(a)
    ws = np.full(n, 2.0 ** -7, np.float16)
    scale = np.full(rows, 2.0 ** -6, np.float16)
    codes = rng.integers(0, 65536, (n, k // 8), dtype=np.uint16)
    nibbles = orc.nibble_table(orc.selector_table(table))
    y = orc.nibble_decode(codes, nibbles).reshape(n, k)
    np.testing.assert_array_equal(orc.plane_project(low, high, total, y, ws, scale), orc.project(a, scale, orc.q2_integers(codes, table), ws))
    packed = rng.integers(0, 2**32, (n, k // 8), dtype=np.uint32)
    y4 = 4 * orc.nibble_decode((packed & 0xFFFF).astype(np.uint16), nibbles) + orc.nibble_decode((packed >> 16).astype(np.uint16), nibbles)
    np.testing.assert_array_equal(orc.plane_project(low, high, total, y4.reshape(n, k), ws, scale, 5),
                                  orc.project(a, scale, orc.q4_integers(packed, table), ws))
    moved = orc.plane_project(low, high, total + 64, y, ws, scale).astype(np.float64)
    plain = orc.project(a, scale, orc.q2_integers(codes, table), ws).astype(np.float64)
    exact = np.abs(a.astype(np.int64) @ orc.q2_integers(codes, table).astype(np.int64).T) < 1900
    np.testing.assert_array_equal((moved - plain)[exact] * 8192, 64)


def test_dispatch_planes_copies_every_token_to_its_slots():
    rng = np.random.default_rng(orc.SEED + 6)
    m, k, e, top_k = 6, 128, 5, 2
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    scale = rng.uniform(0.01, 0.03, (m, 1)).astype(np.float16)
    ids = np.stack([rng.choice(e, top_k, replace=False) for _ in range(m)]).astype(np.int32)
    counts, relative = orc.expert_histogram(ids, e)
    offsets, _, _ = orc.expert_offsets(counts, 16)
    low, high, total, ds, slot_map = orc.dispatch_planes(a, scale, ids, relative, offsets)
    assert low.shape == (k // 64, m * top_k, 8) and sorted(slot_map.reshape(-1)) == list(range(m * top_k))
    wl, wh, wt = orc.split_planes(a)
    for row in range(m):
        for rank in range(top_k):
            slot = slot_map[row, rank]
            np.testing.assert_array_equal(orc.planes_row_major(low)[slot], wl[row])
            np.testing.assert_array_equal(orc.planes_row_major(high)[slot], wh[row])
            assert total[slot] == wt[row] and ds[slot, 0] == scale[row, 0]
            assert offsets[ids[row, rank]] <= slot < offsets[ids[row, rank]] + counts[ids[row, rank]]


def test_row_q4_every_signed_nibble_and_the_byte_permute_form():
    """The reference's known answer (python/orinfer_build/quantization/test_row_q4.py:11-16) and its kernel's decode
    (kernels/cuda/model/q4_projection.py:23-29: two byte permutes, xor with the sign bytes, + 1 where negative)
    emulated on every u16 word."""
    codes = np.tile(np.arange(16, dtype=np.uint8), (1, 8))
    packed = codes[:, ::2] | (codes[:, 1::2] << 4)
    expected = np.tile(np.r_[orc.ROW_Q4_MAGNITUDES, -np.asarray(orc.ROW_Q4_MAGNITUDES)], (1, 8))
    np.testing.assert_array_equal(orc.row_q4_integers(packed), expected)
    magnitudes = (1, 2, 5, 9, 33, 64, 100, 126)
    table = np.array(magnitudes, np.uint8)
    words = np.arange(65536, dtype=np.uint32)
    selector = words & 0x7777
    sign_selector = (words >> 1) & 0x4444
    got = np.empty((65536, 4), np.int64)
    for i in range(4):
        value = table[(selector >> (4 * i)) & 7].astype(np.uint32)           # __byte_perm(lo, hi, selector), byte i
        sign = np.where(((sign_selector >> (4 * i)) & 7) >= 4, 0xFF, 0).astype(np.uint32)  # __byte_perm(0, ~0, ...)
        byte = ((value ^ sign) + (sign & 1)) & 0xFF
        got[:, i] = byte.astype(np.uint8).view(np.int8)
    want = orc.row_q4_integers(words.astype(np.uint16).reshape(-1, 1), magnitudes)
    np.testing.assert_array_equal(got, want)


def test_sign_table_rows_are_the_decodes_with_no_and_with_every_sign(table):
    """python/orinfer_build/quantization/vq.py:44-69: row p * 256 + b holds +t + (1 - 2p) and -t + (1 - 2p) for the two halves
    of basis row b, which is what the codes with sign byte 0x00 / 0xFF (even parity) and 0x01 / 0xFE (odd parity: the
    parity bit itself is flipped back) decode to; a hand-made row with -128 wraps as int8 arithmetic does."""
    signs = orc.sign_table(table)
    assert signs.shape == (512, 4) and signs.dtype == np.uint32
    rows = np.arange(256, dtype=np.uint16) << 8
    for parity, plain, flipped in ((0, 0x00, 0xFF), (1, 0x01, 0xFE)):
        positive = orc.e8p_decode(rows | plain, table)
        negative = orc.e8p_decode(rows | flipped, table)
        block = signs[parity * 256:(parity + 1) * 256]
        np.testing.assert_array_equal(block[:, 0], np.ascontiguousarray(positive[:, :4]).view("<u4").reshape(256))
        np.testing.assert_array_equal(block[:, 1], np.ascontiguousarray(negative[:, :4]).view("<u4").reshape(256))
        np.testing.assert_array_equal(block[:, 2], np.ascontiguousarray(positive[:, 4:]).view("<u4").reshape(256))
        np.testing.assert_array_equal(block[:, 3], np.ascontiguousarray(negative[:, 4:]).view("<u4").reshape(256))
    odd = np.zeros((256, 8), np.int8)
    odd[0] = [-128, 126, 0, -2, 4, 100, -100, 8]
    hand = orc.sign_table(odd)
    assert hand[0, 0] == 0xFF017F81 and hand[0, 1] == 0x03018381  # +t + 1: 81 7F 01 FF;  -t + 1: 81 83 01 03
    assert hand[256, 0] == 0xFDFF7D7F and hand[256, 1] == 0x01FF817F  # +t - 1: 7F 7D FF FD;  -t - 1: 7F 81 FF 01
