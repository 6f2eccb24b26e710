"""GPU parity: decode, A8 and the dense Q4A8 / W8A8 projections against the CPU oracle.

Integer results (decoded weights, int8 activations, int32 accumulators) must be bit-exact.
fp16/fp32 outputs are produced by the same two fp32 multiplies as the oracle, so they are
compared for equality as well; the contract tolerance (1e-3 relative / 1e-2 absolute) is
asserted separately so a reader sees the stated bar.
"""
import numpy as np
import pytest
import torch

from oracle import reference as orc
from orinfer_amd import codebook, workloads

from . import gpu_util as gu

pytestmark = pytest.mark.gpu
TABLE = orc.basis()
RTOL, ATOL = 1e-3, 1e-2  # fp16 output tolerance stated by the benchmark contract


def assert_close_fp16(got, want):
    got = np.asarray(got, np.float32)
    want = np.asarray(want, np.float32)
    assert np.isfinite(got).all()
    assert (np.abs(got - want) <= ATOL + RTOL * np.abs(want)).all()


def exhaustive_q4():
    first = np.arange(65536, dtype=np.uint32).reshape(4096, 16)
    second = (first * np.uint32(32771) + np.uint32(97)) & np.uint32(65535)
    return first | (second << np.uint32(16))


# ---- decode ---------------------------------------------------------------
@pytest.mark.parametrize("packed_k", [0, 64, 128])
def test_q4_unpack_every_code(packed_k):
    packed = exhaustive_q4()  # every coarse code once, residual by an LCG (test_e8p_q4.py:13-30)
    want = orc.q4_integers(packed, TABLE)
    stored = packed if packed_k == 0 else orc.q4_pack_k(packed, packed_k)
    out = torch.zeros((4096, 128), dtype=torch.int8, device=gu.DEV)
    gu.kernel("e8p_q4_unpack", N=4096, K=128, packed_k=packed_k)(Book=gu.book(), Output=out, W=gu.dev(stored))
    np.testing.assert_array_equal(gu.host(out), want)


def test_q4_unpack_residual_every_code():
    # swap the halves so that every code also appears as the residual stage
    packed = exhaustive_q4()
    swapped = (packed >> np.uint32(16)) | (packed << np.uint32(16))
    out = torch.zeros((4096, 128), dtype=torch.int8, device=gu.DEV)
    gu.kernel("e8p_q4_unpack", N=4096, K=128)(Book=gu.book(), Output=out, W=gu.dev(swapped))
    np.testing.assert_array_equal(gu.host(out), orc.q4_integers(swapped, TABLE))


def test_q2_unpack_every_code():
    codes = np.arange(65536, dtype=np.uint16).reshape(4096, 16)
    out = torch.zeros((4096, 128), dtype=torch.int8, device=gu.DEV)
    gu.kernel("e8p_q2_unpack", N=4096, K=128)(Book=gu.book(), Output=out, W=gu.dev(codes))
    np.testing.assert_array_equal(gu.host(out), orc.q2_integers(codes, TABLE))
    k128 = orc.q2_pack_k128(codes)
    out.zero_()
    gu.kernel("e8p_q2_unpack", N=4096, K=128, packed_k=128)(Book=gu.book(), Output=out, W=gu.dev(k128))
    np.testing.assert_array_equal(gu.host(out), orc.q2_integers(codes, TABLE))


# ---- A8 -------------------------------------------------------------------
def test_a8_edges_and_random():
    rng = np.random.default_rng(orc.SEED)
    x = rng.normal(size=(67, 2560)).astype(np.float16)
    x[0] = 0
    x[1, :8] = [127, -127, 63.5, 0.5, 1.5, 2.5, -0.5, -2.5]
    x[1, 8:] = 0
    x[2] = 0
    x[2, 5] = 1e-7
    x[3, :8] = [254, 1, -1, 3, -3, 5, 127, -254]
    x[3, 8:] = 0
    x[4, 0] = 65504
    x[5] *= 20
    q, s = gu.a8(gu.dev(x))
    wq, ws = orc.a8(x)
    np.testing.assert_array_equal(gu.host(s), ws)
    np.testing.assert_array_equal(gu.host(q), wq)


@pytest.mark.parametrize("k,group", [(2560, 64), (384, 128), (100, 25), (7, 7), (5120, 5120), (16384, 8192), (9001, 9001),
                                     (1024, 512), (4096, 4096)])
def test_a8_groups_and_odd_shapes(k, group):
    rng = np.random.default_rng(orc.SEED + k)
    x = (rng.normal(size=(5, k)) * 3).astype(np.float16)
    q, s = gu.a8(gu.dev(x), group=group)
    wq, ws = orc.a8(x, group)
    np.testing.assert_array_equal(gu.host(s), ws)
    np.testing.assert_array_equal(gu.host(q), wq)


@pytest.mark.parametrize("rows,k,group", [(300, 17408, 17408), (260, 16384, 8192), (259, 5120, 5120), (257, 24576, 24576), (258, 24584, 24584)])
def test_a8_many_rows_of_long_groups(rows, k, group):
    # above 256 rows, groups of 4608 to 24576 values wait in LDS between the maximum and the quantise
    # pass; the last shape is just past that range and reads its input twice
    rng = np.random.default_rng(orc.SEED + rows + k)
    x = (rng.normal(size=(rows, k)) * 2).astype(np.float16)
    x[1] = 0
    x[2, -1] = 1000
    q, s = gu.a8(gu.dev(x), group=group)
    wq, ws = orc.a8(x, group)
    np.testing.assert_array_equal(gu.host(s), ws)
    np.testing.assert_array_equal(gu.host(q), wq)


def test_a8_masked_columns():
    rng = np.random.default_rng(orc.SEED)
    x = rng.normal(size=(9, 512)).astype(np.float16)
    mask = (rng.uniform(size=512) < 0.1).astype(np.uint8)
    x[:, 3] = 1000  # would dominate amax if the mask were ignored
    mask[3] = 7
    q, s = gu.a8(gu.dev(x), masked=gu.dev(mask))
    xm = x.copy()
    xm[:, mask != 0] = 0
    wq, ws = orc.a8(xm)
    np.testing.assert_array_equal(gu.host(s), ws)
    np.testing.assert_array_equal(gu.host(q), wq)


def test_swiglu_then_a8_and_fused_form_agree():
    rng = np.random.default_rng(orc.SEED)
    gu_in = (rng.normal(size=(33, 2 * 512)) * 2).astype(np.float16)
    x = gu.dev(gu_in)
    y = torch.empty((33, 512), dtype=torch.float16, device=gu.DEV)
    gu.kernel("swiglu", I=512)(X=x, Y=y, rows=33)
    want = orc.swiglu_fp16(gu_in)
    got = gu.host(y)
    # exp() differs by an ulp between libraries: tolerance on the fp16 boundary value
    np.testing.assert_allclose(got.astype(np.float32), want.astype(np.float32), rtol=2e-3, atol=1e-6)
    assert (got == want).mean() > 0.99
    q1, s1 = gu.a8(y)
    wq, ws = orc.a8(got)  # the quantiser itself must be exact on the GPU's own fp16 values
    np.testing.assert_array_equal(gu.host(q1), wq)
    np.testing.assert_array_equal(gu.host(s1), ws)
    q2, s2 = gu.a8(x, fused=True)
    assert torch.equal(q1, q2) and torch.equal(s1, s2)


# ---- signed block-128 rotation fused with A8 -------------------------------------------------
@pytest.mark.parametrize("m,k", [(1, 128), (3, 384), (5, 2560), (2, 5120), (1, 17408), (260, 2304)])
@pytest.mark.parametrize("swiglu", [False, True])
def test_rotate_activation_a8_matches_oracle(m, k, swiglu):
    rng = np.random.default_rng(orc.SEED + m + k)
    x = rng.normal(size=(m, 2 * k if swiglu else k)).astype(np.float16)
    x[0, :3] = [0, 60000, -60000] if not swiglu else [3, -2, 0]
    signs = rng.choice(np.array([-1, 1], np.int8), k)
    want_q, want_s = orc.rotate_a8(x, signs, swiglu=swiglu)
    variant = dict(M=m, K=k)
    if swiglu:
        variant["swiglu"] = True
    q = torch.full((m + 1, k), 77, dtype=torch.int8, device=gu.DEV)
    s = torch.full((m + 1,), 5.0, dtype=torch.float16, device=gu.DEV)
    gu.kernel("rotate_activation_a8", **variant)(Q=q, S=s, Signs=gu.dev(signs), X=gu.dev(x))
    if swiglu:
        # the exponential of the SwiGLU boundary may differ in the last place between libm and the
        # device: compare the codes on the device's own fp16 SwiGLU values
        mid = torch.empty((m, k), dtype=torch.float16, device=gu.DEV)
        gu.kernel("swiglu", I=k)(X=gu.dev(x), Y=mid, rows=m)
        want_q, want_s = orc.rotate_a8(gu.host(mid), signs)
    np.testing.assert_array_equal(gu.host(s)[:m], want_s[:, 0])
    np.testing.assert_array_equal(gu.host(q)[:m], want_q)
    assert (gu.host(q)[m:] == 77).all() and float(gu.host(s)[m]) == 5.0


def test_rotate_activation_a8_dynamic_rows_zero_row_and_graph():
    rng = np.random.default_rng(orc.SEED + 12)
    k = 1024
    x = rng.normal(size=(9, k)).astype(np.float16)
    x[4] = 0
    signs = rng.choice(np.array([-1, 1], np.int8), k)
    kern = gu.kernel("rotate_activation_a8", M=16, K=k, dynamic_rows=True)
    d_x, d_signs = gu.dev(x), gu.dev(signs)
    q = torch.zeros((16, k), dtype=torch.int8, device=gu.DEV)
    s = torch.zeros((16,), dtype=torch.float16, device=gu.DEV)
    for rows in (9, 1):
        q.fill_(9)
        kern(Q=q, S=s, Signs=d_signs, X=d_x, m=rows)
        want_q, want_s = orc.rotate_a8(x[:rows], signs)
        np.testing.assert_array_equal(gu.host(q)[:rows], want_q)
        np.testing.assert_array_equal(gu.host(s)[:rows], want_s[:, 0])
        assert (gu.host(q)[rows:] == 9).all()
    assert float(gu.host(s)[0]) > 0
    kern(Q=q, S=s, Signs=d_signs, X=d_x, m=9)
    assert not gu.host(q)[4].any() and float(gu.host(s)[4]) == 1.0
    # rotated activations against rotated weights reproduce the un-rotated dot products
    w = rng.normal(size=(6, k)).astype(np.float32)
    rotated_w = orc.rotate(w, signs)
    codes, scales = gu.host(q)[:9].astype(np.float32), gu.host(s)[:9].astype(np.float32)
    approx = (codes * scales[:, None]) @ rotated_w.T
    np.testing.assert_allclose(approx, x.astype(np.float32) @ w.T, atol=0.6, rtol=0.05)


def ulps_fp16(a, b):
    """Distance in fp16 units in the last place (both finite)."""
    def key(v):
        bits = np.asarray(v, np.float16).view(np.int16).astype(np.int32)
        return np.where(bits < 0, -(bits & 0x7FFF), bits)
    return np.abs(key(a) - key(b))


@pytest.mark.parametrize("m,k,zero_centered", [(1, 256, True), (3, 1536, True), (5, 5120, True), (2, 5120, False),
                                               (1, 17408, True)])
def test_residual_norm_rotate_a8_matches_oracle(m, k, zero_centered):
    rng = np.random.default_rng(orc.SEED + 3 * m + k)
    x = rng.normal(size=(m, k)).astype(np.float16)
    r = rng.normal(size=(m, k)).astype(np.float32)
    w = (rng.normal(size=k) * 0.1 + (0.0 if zero_centered else 1.0)).astype(np.float16)
    signs = rng.choice(np.array([-1, 1], np.int8), k)
    variant = dict(M=m, K=k)
    if not zero_centered:
        variant["zero_centered"] = False
    # one spare row behind every output, as in the reference's check (check_rows.py:156-161,172)
    y = torch.full((m + 1, k), 91, dtype=torch.float16, device=gu.DEV)
    ro = torch.full((m + 1, k), 91, dtype=torch.float32, device=gu.DEV)
    q = torch.full((m + 1, k), 91, dtype=torch.int8, device=gu.DEV)
    s = torch.full((m + 1,), 91, dtype=torch.float16, device=gu.DEV)
    gu.kernel("residual_norm_rotate_a8", **variant)(Q=q, R=gu.dev(r), RO=ro, S=s, Signs=gu.dev(signs), W=gu.dev(w),
                                                    X=gu.dev(x), Y=y)
    want_y, want_ro, _, _ = orc.residual_norm_rotate_a8(x, r, w, signs, zero_centered=zero_centered)
    np.testing.assert_array_equal(gu.host(ro)[:m], want_ro)  # one fp32 add: exact
    got_y = gu.host(y)[:m]
    # fp16((sum * rsqrt(mean + eps)) * gain): the fp32 sum of squares and the reciprocal square root
    # may differ in the last place from the float64 restatement, which moves an fp16 rounding by
    # at most one unit in the last place
    distance = ulps_fp16(got_y, want_y)
    assert distance.max() <= 1 and (distance > 0).mean() < 0.02
    # the rotation and the quantiser read the fp16 row the kernel wrote: codes and scales are exact
    want_q, want_s = orc.rotate_a8(got_y, signs)
    np.testing.assert_array_equal(gu.host(q)[:m], want_q)
    np.testing.assert_array_equal(gu.host(s)[:m], want_s[:, 0])
    for spare in (y, ro, q, s):
        assert (gu.host(spare)[m:] == 91).all()


def test_residual_norm_rotate_a8_dynamic_rows_zero_rows_and_composition():
    rng = np.random.default_rng(orc.SEED + 77)
    k, cap = 5120, 32
    x = rng.normal(size=(17, k)).astype(np.float16)
    r = rng.normal(size=(17, k)).astype(np.float32)
    x[6], r[6] = 0, 0
    w = (rng.normal(size=k) * 0.1).astype(np.float16)
    signs = rng.choice(np.array([-1, 1], np.int8), k)
    kern = gu.kernel("residual_norm_rotate_a8", M=cap, K=k, dynamic_rows=True)
    rotation = gu.kernel("rotate_activation_a8", M=cap, K=k, dynamic_rows=True)
    d = dict(R=gu.dev(r), Signs=gu.dev(signs), W=gu.dev(w), X=gu.dev(x))
    y = torch.zeros((cap, k), dtype=torch.float16, device=gu.DEV)
    ro = torch.zeros((cap, k), dtype=torch.float32, device=gu.DEV)
    q = torch.zeros((cap, k), dtype=torch.int8, device=gu.DEV)
    s = torch.zeros((cap,), dtype=torch.float16, device=gu.DEV)
    for rows in (17, 1, 8):
        for out in (y, ro, q, s):
            out.fill_(91)
        kern(Q=q, RO=ro, S=s, Y=y, m=rows, **d)
        # the reference's own check: the fused kernel equals the rotation kernel run on Y
        q2 = torch.zeros_like(q)
        s2 = torch.zeros_like(s)
        rotation(Q=q2, S=s2, Signs=d["Signs"], X=y, m=rows)
        assert torch.equal(q[:rows], q2[:rows]) and torch.equal(s[:rows], s2[:rows])
        assert (gu.host(q)[rows:] == 91).all() and (gu.host(y)[rows:] == 91).all()
        np.testing.assert_array_equal(gu.host(ro)[:rows], x[:rows].astype(np.float32) + r[:rows])
    kern(Q=q, RO=ro, S=s, Y=y, m=17, **d)
    # an all-zero row: zero codes, scale one (check_rows.py:186-190)
    assert not gu.host(q)[6].any() and float(gu.host(s)[6]) == 1.0 and not gu.host(y)[6].any()
    # unit RMS before the gain: mean(Y / (1 + w))^2 is 1 to fp16 accuracy
    unit = gu.host(y)[:17].astype(np.float64) / (1.0 + w.astype(np.float64))
    live = [i for i in range(17) if i != 6]
    np.testing.assert_allclose((unit[live] ** 2).mean(axis=1), 1.0, rtol=2e-3)


def test_residual_norm_rotate_a8_refuses_incomplete_tiles():
    for k in (128, 5120 + 128, 0, 32768 + 256):
        with pytest.raises(Exception):
            gu.kernel("residual_norm_rotate_a8", M=4, K=k)


@pytest.mark.parametrize("m,k,swiglu", [(1, 128, False), (3, 2560, False), (2, 5120, True), (4, 384, True)])
def test_rotate_activation_gives_the_values_the_fused_kernel_quantises(m, k, swiglu):
    # kernels/cuda/model/integer_vq.py:447-486
    rng = np.random.default_rng(orc.SEED + m + k)
    x = rng.normal(size=(m, 2 * k if swiglu else k)).astype(np.float16)
    signs = rng.choice(np.array([-1, 1], np.int8), k)
    y = torch.full((m + 1, k), 7.0, dtype=torch.float16, device=gu.DEV)
    variant = dict(M=m, K=k, swiglu=True) if swiglu else dict(M=m, K=k)
    gu.kernel("rotate_activation", **variant)(Signs=gu.dev(signs), X=gu.dev(x), Y=y)
    values = x
    if swiglu:  # the device's own fp16 SwiGLU values (the exponential may differ from libm in the last place)
        mid = torch.empty((m, k), dtype=torch.float16, device=gu.DEV)
        gu.kernel("swiglu", I=k)(X=gu.dev(x), Y=mid, rows=m)
        values = gu.host(mid)
    want = orc.rotate(values.astype(np.float32), signs).astype(np.float16)
    np.testing.assert_array_equal(gu.host(y)[:m], want)
    assert (gu.host(y)[m] == 7).all()
    # A8 of these values is what rotate_activation_a8 writes
    q = torch.zeros((m, k), dtype=torch.int8, device=gu.DEV)
    s = torch.zeros((m,), dtype=torch.float16, device=gu.DEV)
    gu.kernel("rotate_activation_a8", **variant)(Q=q, S=s, Signs=gu.dev(signs), X=gu.dev(x))
    want_q, want_s = orc.a8(gu.host(y)[:m])
    np.testing.assert_array_equal(gu.host(q), want_q)
    np.testing.assert_array_equal(gu.host(s), want_s[:, 0])
    with pytest.raises(Exception):
        gu.kernel("rotate_activation", M=2, K=192)


@pytest.mark.parametrize("m,block_m", [(1, None), (3, None), (8, 8), (6, 2)])
def test_int8_small_projection_symbol(m, block_m):
    # kernels/cuda/model/int8_projection.py:65-107: same buffers and arithmetic as int8_projection
    rng = np.random.default_rng(orc.SEED + m)
    n, k = 136, 384
    w = rng.integers(-128, 128, (n, k), dtype=np.int8)
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    ws = rng.uniform(0.005, 0.02, n).astype(np.float16)
    ts = rng.uniform(0.01, 0.03, m).astype(np.float16)
    variant = dict(M=m, N=n, K=k, block_n=8, output_stride=n + 8)
    if block_m:
        variant["block_m"] = block_m
    out = torch.full((m, n + 8), 9.0, dtype=torch.float16, device=gu.DEV)
    gu.kernel("int8_small_projection", **variant)(A=gu.dev(a), Output=out, TokenScale=gu.dev(ts), Weight=gu.dev(w),
                                                  WeightScale=gu.dev(ws))
    np.testing.assert_array_equal(gu.host(out)[:, :n], orc.project(a, ts, w, ws))
    assert (gu.host(out)[:, n:] == 9).all()
    for bad in (dict(block_m=9), dict(block_n=32), dict(block_m=0)):
        with pytest.raises(Exception):
            gu.kernel("int8_small_projection", M=4, N=n, K=k, **bad)


@pytest.mark.parametrize("n,k,packed_k", [(9728, 2560, 0), (17408, 5120, 0), (200, 1024, 0), (4096, 8192, 0),
                                          (17408, 5120, 128), (136, 2048, 128)])
def test_q4_gemv_quantises_fp16_input_itself(n, k, packed_k):
    """input_dtype=float16: one launch gives what activation_quantization + e8p_q4_projection give."""
    rng = np.random.default_rng(orc.SEED + n + k)
    packed = rng.integers(0, 2**32, (n, k // 8), dtype=np.uint32)
    scales = rng.uniform(0.005, 0.02, n).astype(np.float16)
    stored = gu.dev(packed if packed_k == 0 else orc.q4_pack_k(packed, packed_k))
    kern = gu.kernel("e8p_q4_projection", M=1, N=n, K=k, packed_k=packed_k, input_dtype="float16")
    weights = orc.q4_integers(packed, TABLE)
    out = torch.full((2, n), 9.0, dtype=torch.float16, device=gu.DEV)
    a_scale = torch.full((2,), 7.0, dtype=torch.float16, device=gu.DEV)
    for case in range(3):
        x = rng.normal(size=(1, k)).astype(np.float16)
        if case == 1:
            x[0, :4] = [900, -900, 0, 1e-7]  # a large maximum: most codes are zero
        if case == 2:
            x[:] = 0                              # zero row: scale one, zero output
        kern(A=gu.dev(x), AS=a_scale, Book=gu.book(), Out=out, S=gu.dev(scales), W=stored)
        a_q, a_s = orc.a8(x)
        np.testing.assert_array_equal(gu.host(a_scale)[:1], a_s[:, 0])
        np.testing.assert_array_equal(gu.host(out)[:1], orc.project(a_q, a_s, weights, scales))
        assert float(gu.host(a_scale)[1]) == 7.0 and (gu.host(out)[1] == 9).all()


@pytest.mark.parametrize("n,k,packed_k", [(9728, 2560, 0), (17408, 5120, 0), (200, 1024, 0), (17408, 5120, 128)])
def test_q4_gemv_rotates_and_quantises_fp16_input(n, k, packed_k):
    """input_dtype=float16, rotate=true: one launch gives what rotate_activation_a8 + e8p_q4_projection give."""
    rng = np.random.default_rng(orc.SEED + n + k + 1)
    packed = rng.integers(0, 2**32, (n, k // 8), dtype=np.uint32)
    scales = rng.uniform(0.005, 0.02, n).astype(np.float16)
    signs = rng.choice(np.array([-1, 1], np.int8), k)
    stored = gu.dev(packed if packed_k == 0 else orc.q4_pack_k(packed, packed_k))
    kern = gu.kernel("e8p_q4_projection", M=1, N=n, K=k, packed_k=packed_k, input_dtype="float16", rotate=True,
                     workspace=False)
    assert kern.arg_names == ["A", "AS", "Book", "Out", "S", "Signs", "W"]
    weights = orc.q4_integers(packed, TABLE)
    out = torch.full((2, n), 9.0, dtype=torch.float16, device=gu.DEV)
    a_scale = torch.full((2,), 7.0, dtype=torch.float16, device=gu.DEV)
    for case in range(3):
        x = rng.normal(size=(1, k)).astype(np.float16)
        if case == 1:
            x[0, :4] = [900, -900, 0, 1e-7]
        if case == 2:
            x[:] = 0
        kern(A=gu.dev(x), AS=a_scale, Book=gu.book(), Out=out, S=gu.dev(scales), Signs=gu.dev(signs), W=stored)
        a_q, a_s = orc.rotate_a8(x, signs)
        np.testing.assert_array_equal(gu.host(a_scale)[:1], a_s[:, 0])
        np.testing.assert_array_equal(gu.host(out)[:1], orc.project(a_q, a_s, weights, scales))
        assert float(gu.host(a_scale)[1]) == 7.0 and (gu.host(out)[1] == 9).all()
    with pytest.raises(Exception):
        gu.kernel("e8p_q4_projection", M=1, N=n, K=k, rotate=True)


def test_q4_fp16_input_is_refused_where_no_kernel_serves_it():
    for variant in (dict(M=2, N=256, K=1024), dict(M=1, N=256, K=1024, algorithm="mfma"), dict(M=1, N=256, K=16384),
                    dict(M=1, N=256, K=1024, input_dtype="bfloat16")):
        variant.setdefault("input_dtype", "float16")
        with pytest.raises(Exception):
            gu.kernel("e8p_q4_projection", **variant)


@pytest.mark.parametrize("codec,m,n,k,dtype", [("q4", 128, 8704, 512, "float16"), ("q4", 70, 8300, 384, "float16"),
                                               ("w8", 128, 8704, 256, "float16"), ("w8", 300, 8450, 384, "float32"),
                                               ("q4", 256, 17408, 256, "float16"), ("w8", 40, 2048, 1024, "float16"),
                                               ("w8", 17, 5120, 512, "float32")])
def test_mid_row_projections_split_k_steps_evenly(codec, m, n, k, dtype):
    """65-384 rows on the 128-row tiles: the K steps of the tiles are dealt evenly to one workgroup per
    CU, runs that do not cover a whole tile meet as int32 partial sums.  Same bytes as whole tiles."""
    rng = np.random.default_rng(orc.SEED + m + n)
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    a_s = rng.uniform(0.01, 0.03, m).astype(np.float16)
    scales = rng.uniform(0.005, 0.02, n).astype(np.float16)
    torch_dtype = torch.float16 if dtype == "float16" else torch.float32
    stride = n + 8
    if codec == "q4":
        packed = rng.integers(0, 2**32, (n, k // 8), dtype=np.uint32)
        weights = orc.q4_integers(packed, TABLE)
        symbol, stored = "e8p_q4_projection", gu.dev(packed)
        call = lambda kern, out: kern(A=gu.dev(a), AS=gu.dev(a_s), Book=gu.book(), Out=out, S=gu.dev(scales), W=stored)
    else:
        weights = rng.integers(-128, 128, (n, k), dtype=np.int8)
        symbol, stored = "int8_projection", gu.dev(weights)
        call = lambda kern, out: kern(A=gu.dev(a), Output=out, TokenScale=gu.dev(a_s), Weight=stored, WeightScale=gu.dev(scales))
    variant = dict(M=m, N=n, K=k, output_dtype=dtype, output_stride=stride)
    if m <= 64 or codec == "q4":
        # `auto` gives so few rows of so small a matrix to the streaming kernel, 65..128 rows of two-stage codes with a
        # short K to the channel-run kernel, and more rows of a matrix this wide to the 512-row channel runs
        variant["algorithm"] = "mfma"
    split = gu.kernel(symbol, **variant)
    whole = gu.kernel(symbol, split_k=False, **variant)
    grid_split, grid_whole = tuple(split.geometry()[0]), tuple(whole.geometry()[0])
    assert grid_split[1] == 1 and grid_whole[0] == -(-n // 128) and grid_whole[1] == -(-m // 128)
    out = torch.full((m + 1, stride), 9.0, dtype=torch_dtype, device=gu.DEV)
    other = torch.full((m + 1, stride), 9.0, dtype=torch_dtype, device=gu.DEV)
    call(split, out)
    call(whole, other)
    assert torch.equal(out, other)
    want = orc.project(a, a_s, weights, scales, out_dtype=np.float16 if dtype == "float16" else np.float32)
    np.testing.assert_array_equal(gu.host(out)[:m, :n], want)
    assert (gu.host(out)[m] == 9).all() and (gu.host(out)[:, n:] == 9).all()
    # again into the same buffers: the partial slots carry nothing over
    out.fill_(9)
    call(split, out)
    assert torch.equal(out, other)


@pytest.mark.parametrize("packed_k", [128, 64])
def test_split_launches_serve_k_major_codes_and_dynamic_rows(packed_k):
    rng = np.random.default_rng(orc.SEED + 91)
    n, k, cap = 8704, 384, 256
    packed = rng.integers(0, 2**32, (n, k // 8), dtype=np.uint32)
    weights = orc.q4_integers(packed, TABLE)
    scales = rng.uniform(0.005, 0.02, n).astype(np.float16)
    kern = gu.kernel("e8p_q4_projection", M=cap, N=n, K=k, packed_k=packed_k, dynamic_rows=True)
    stored = gu.dev(orc.q4_pack_k(packed, packed_k))
    for m in (200, 65, 130):
        a = rng.integers(-128, 128, (cap, k), dtype=np.int8)
        a_s = rng.uniform(0.01, 0.03, cap).astype(np.float16)
        out = torch.full((cap, n), 9.0, dtype=torch.float16, device=gu.DEV)
        assert tuple(kern.geometry(m)[0])[1] == 1  # one workgroup list: the split form
        kern(A=gu.dev(a), AS=gu.dev(a_s), Book=gu.book(), Out=out, S=gu.dev(scales), W=stored, m=m)
        np.testing.assert_array_equal(gu.host(out)[:m], orc.project(a[:m], a_s[:m], weights, scales))
        assert (gu.host(out)[m:] == 9).all()


def test_q4_embedding_gather_matches_oracle():
    rng = np.random.default_rng(orc.SEED + 40)
    vocab, hidden, cap = 50, 640, 16
    packed = rng.integers(0, 2**32, (vocab, hidden // 8), dtype=np.uint32)
    scales = rng.uniform(0.005, 0.02, vocab).astype(np.float16)
    signs = rng.choice(np.array([-1, 1], np.int8), hidden)
    ids = np.array([0, 49, 7, -1, 50, 7, 2**31 - 1, 13, 1], np.int32)
    kern = gu.kernel("e8p_q4_embedding", M=cap, vocab=vocab, hidden=hidden)
    out = torch.full((cap, hidden), 3.0, dtype=torch.float16, device=gu.DEV)
    padded = np.zeros(cap, np.int32)
    padded[: len(ids)] = ids
    kern(Book=gu.book(), IDs=gu.dev(padded), Output=out, Scale=gu.dev(scales), Signs=gu.dev(signs),
         Weight=gu.dev(orc.q4_pack_k(packed, 128)), m=len(ids))
    got = gu.host(out)
    np.testing.assert_array_equal(got[: len(ids)], orc.q4_embedding(ids, packed, TABLE, scales, signs))
    assert not got[3].any() and not got[4].any() and not got[6].any() and (got[len(ids):] == 3).all()


@pytest.mark.parametrize("m,n,k", [(1, 96, 256), (6, 200, 1024), (70, 130, 384), (300, 260, 256), (64, 512, 2048),
                                   (129, 64, 128)])
def test_int8_swiglu_gate_up_boundary(m, n, k):
    rng = np.random.default_rng(orc.SEED + m + n)
    a_q = rng.integers(-127, 128, (m, k), dtype=np.int8)
    a_s = rng.uniform(0.005, 0.02, m).astype(np.float16)
    gate, up = (rng.integers(-127, 128, (n, k), dtype=np.int8) for _ in range(2))
    gs, us = (rng.uniform(0.001, 0.004, n).astype(np.float16) for _ in range(2))
    out = torch.full((m + 1, n), 2.0, dtype=torch.float16, device=gu.DEV)
    gu.kernel("int8_swiglu", M=m, N=n, K=k)(A=gu.dev(a_q), Gate=gu.dev(gate), GateScale=gu.dev(gs), Output=out,
                                            TokenScale=gu.dev(a_s), Up=gu.dev(up), UpScale=gu.dev(us))
    got = gu.host(out)
    want = orc.int8_swiglu(a_q, a_s, gate, gs, up, us)
    # the two projections inside are exact integers rounded to fp16 as the oracle rounds them; only exp()
    # may differ in the last place between the device and libm: one fp16 step at most, rarely
    np.testing.assert_allclose(got[:m].astype(np.float32), want.astype(np.float32), rtol=1e-3, atol=1e-2)
    assert ulps_fp16(got[:m], want).max() <= 1
    assert np.mean(got[:m] == want) > 0.99 and (got[m:] == 2).all()


# ---- Q4A8 projections -----------------------------------------------------
def q4_case(rng, m, n, k):
    x = (rng.normal(size=(m, k))).astype(np.float16)
    a_q, a_s = orc.a8(x)
    packed = rng.integers(0, 2**32, (n, k // 8), dtype=np.uint32)
    scales = rng.uniform(0.005, 0.02, n).astype(np.float16)
    return a_q, a_s[:, 0].copy(), packed, scales


@pytest.mark.parametrize("m", [1, 2, 3, 4])
@pytest.mark.parametrize("n,k", [(65, 256), (257, 2560), (1024, 5120), (130, 17408), (33, 8192 + 512), (70, 1536)])
def test_q4_gemv_matches_oracle(m, n, k):
    rng = np.random.default_rng(orc.SEED + m + n)
    a_q, a_s, packed, scales = q4_case(rng, m, n, k)
    a_q[0, :4] = [-128, -1, 0, 127]  # extremes outside the A8 range must still be exact
    w = orc.q4_integers(packed, TABLE)
    acc = orc.int_dot(a_q, w)
    ones_n, ones_m = np.ones(n, np.float16), np.ones(m, np.float16)
    got_acc = gu.q4_project(gu.dev(a_q), gu.dev(ones_m), gu.dev(packed), gu.dev(ones_n), dtype=torch.float32,
                            algorithm="gemv")
    np.testing.assert_array_equal(gu.host(got_acc).astype(np.int64), acc.astype(np.int64))
    got = gu.q4_project(gu.dev(a_q), gu.dev(a_s), gu.dev(packed), gu.dev(scales), algorithm="gemv")
    want = orc.rescale(acc, scales, a_s)
    assert_close_fp16(gu.host(got), want)
    np.testing.assert_array_equal(gu.host(got), want)


@pytest.mark.parametrize("blocks_of", [128, 64])
@pytest.mark.parametrize("m", [1, 2, 3, 4])
@pytest.mark.parametrize("n,k", [(65, 256), (257, 2560), (1024, 5120), (130, 16384), (33, 8192 + 512), (7, 1536), (17408, 5120),
                                 (40, 17408), (9, 768)])
def test_q4_gemv_k_major_codes_match_oracle(m, n, k, blocks_of):
    """The reference's storage layouts (K/128 blocks of N rows, or K/64: e8p_q4.py:78-80): 16 lanes per row and tasks of 4
    adjacent rows, or 8 lanes and 8 rows when K is a multiple of 256 only."""
    rng = np.random.default_rng(orc.SEED + 500 + m + n)
    a_q, a_s, packed, scales = q4_case(rng, m, n, k)
    a_q[0, :4] = [-128, -1, 0, 127]
    stored = orc.q4_pack_k(packed, blocks_of)
    w = orc.q4_integers(packed, TABLE)
    acc = orc.int_dot(a_q, w)
    ones_n, ones_m = np.ones(n, np.float16), np.ones(m, np.float16)
    planes_fit = 131072 + (1 if m == 1 else 2 if m == 2 else 4) * (k // 8) * 12 + 256 + k // 32 + 16 <= 160 * 1024
    if not planes_fit:  # the activation planes of so many rows do not fit beside the tables: refused at launch
        with pytest.raises(Exception, match="K-major"):
            gu.q4_project(gu.dev(a_q), gu.dev(ones_m), gu.dev(stored), gu.dev(ones_n), algorithm="gemv", packed_k=blocks_of)
        return
    got_acc = gu.q4_project(gu.dev(a_q), gu.dev(ones_m), gu.dev(stored), gu.dev(ones_n), dtype=torch.float32,
                            algorithm="gemv", packed_k=blocks_of)
    np.testing.assert_array_equal(gu.host(got_acc).astype(np.int64), acc.astype(np.int64))
    storage = torch.full((m + 1, n + 5), 91.0, dtype=torch.float16, device=gu.DEV)
    gu.q4_project(gu.dev(a_q), gu.dev(a_s), gu.dev(stored), gu.dev(scales), out=storage, stride=n + 5,
                  algorithm="gemv", packed_k=blocks_of)
    got = gu.host(storage)
    np.testing.assert_array_equal(got[:m, :n], orc.rescale(acc, scales, a_s))
    assert (got[m:] == 91).all() and (got[:m, n:] == 91).all()
    if m <= 2:  # what `auto` picks for K-major codes at 1 and 2 rows
        auto = gu.q4_project(gu.dev(a_q), gu.dev(a_s), gu.dev(stored), gu.dev(scales), packed_k=blocks_of)
        np.testing.assert_array_equal(gu.host(auto), orc.rescale(acc, scales, a_s))


def test_q4_gemv_k_major_refuses_what_it_cannot_read():
    with pytest.raises(Exception, match="gemv"):
        gu.kernel("e8p_q4_projection", M=1, N=64, K=384, packed_k=128, algorithm="gemv")


@pytest.mark.parametrize("variant", [{}, {"gemv_passes": 1}], ids=["replicated-tables", "compact-tables"])
@pytest.mark.parametrize("m", [1, 2, 4])
@pytest.mark.parametrize("pattern", ["all_max", "band", "sparse", "negative"])
def test_q4_gemv_activation_extremes(m, pattern, variant):
    """Activations at and around the top of the int8 range: the GEMV splits them into signed
    nibbles, and values of 120..127 take a separate path that random data visits rarely."""
    n, k = 193, 5120
    rng = np.random.default_rng(orc.SEED + 77 + m)
    if pattern == "all_max":
        a_q = np.full((m, k), 127, np.int8)
    elif pattern == "band":                       # every boundary value, many times
        a_q = rng.choice(np.array([111, 112, 119, 120, 121, 126, 127, -120, -121, -127, -128, 7, 8, -8, -9, 0], np.int8),
                         size=(m, k))
    elif pattern == "sparse":                     # one overflow in the last chunk of the last row only
        a_q = rng.integers(-119, 120, (m, k)).astype(np.int8)
        a_q[m - 1, k - 1] = 124
    else:
        a_q = rng.integers(-128, -119, (m, k)).astype(np.int8)
    packed = rng.integers(0, 2**32, (n, k // 8), dtype=np.uint32)
    acc = orc.int_dot(a_q, orc.q4_integers(packed, TABLE))
    np.testing.assert_array_equal(acc, orc.int_dot_bruteforce(a_q[:, :256], orc.q4_integers(packed[:, :32], TABLE))
                                  + orc.int_dot(a_q[:, 256:], orc.q4_integers(packed[:, 32:], TABLE)))
    got = gu.q4_project(gu.dev(a_q), gu.dev(np.ones(m, np.float16)), gu.dev(packed), gu.dev(np.ones(n, np.float16)),
                        dtype=torch.float32, algorithm="gemv", **variant)
    np.testing.assert_array_equal(gu.host(got).astype(np.int64), acc.astype(np.int64))


@pytest.mark.parametrize("packed_k", [0, 64, 128])
@pytest.mark.parametrize("m", [1, 7, 32, 33, 64, 65, 128, 129, 300])
def test_q4_mfma_rows_tails_stride_and_sentinels(m, packed_k):
    # check_e8p_q4.py:123-193: N=65, K=256, fp32 out, stride N+3, sentinel 91 beyond the tails
    rng = np.random.default_rng(orc.SEED + m)
    n, k = 65, 256
    a_q, a_s, packed, scales = q4_case(rng, m, n, k)
    a_q[0, :2] = [-128, 127]
    stored = packed if packed_k == 0 else orc.q4_pack_k(packed, packed_k)
    storage = torch.full((m + 2, n + 3), 91.0, dtype=torch.float32, device=gu.DEV)
    gu.q4_project(gu.dev(a_q), gu.dev(a_s), gu.dev(stored), gu.dev(scales), out=storage, stride=n + 3,
                  dtype=torch.float32, algorithm="mfma", packed_k=packed_k)
    got = gu.host(storage)
    want = orc.project(a_q, a_s, orc.q4_integers(packed, TABLE), scales, np.float32)
    np.testing.assert_array_equal(got[:m, :n], want)
    assert (got[m:] == 91).all() and (got[:m, n:] == 91).all()


@pytest.mark.parametrize("packed_k", [0, 64, 128])
@pytest.mark.parametrize("m", [5, 8, 31, 32, 33, 64])
def test_q4_stream_rows_tails_stride_and_sentinels(m, packed_k):
    # same construction as the MFMA tail test, through the weight-streaming kernel; K=640 gives the
    # eight K slices of a workgroup uneven shares (5 blocks over 8 waves, three of them empty)
    rng = np.random.default_rng(orc.SEED + 100 + m)
    n, k = 97, 640
    a_q, a_s, packed, scales = q4_case(rng, m, n, k)
    a_q[0, :2] = [-128, 127]
    stored = packed if packed_k == 0 else orc.q4_pack_k(packed, packed_k)
    w = orc.q4_integers(packed, TABLE)
    storage = torch.full((m + 2, n + 3), 91.0, dtype=torch.float32, device=gu.DEV)
    gu.q4_project(gu.dev(a_q), gu.dev(a_s), gu.dev(stored), gu.dev(scales), out=storage, stride=n + 3,
                  dtype=torch.float32, algorithm="stream", packed_k=packed_k)
    got = gu.host(storage)
    np.testing.assert_array_equal(got[:m, :n], orc.project(a_q, a_s, w, scales, np.float32))
    assert (got[m:] == 91).all() and (got[:m, n:] == 91).all()
    ones_n, ones_m = np.ones(n, np.float16), np.ones(m, np.float16)
    acc = gu.q4_project(gu.dev(a_q), gu.dev(ones_m), gu.dev(stored), gu.dev(ones_n), dtype=torch.float32,
                        algorithm="stream", packed_k=packed_k)
    np.testing.assert_array_equal(gu.host(acc).astype(np.int64), orc.int_dot(a_q, w).astype(np.int64))
    half = gu.q4_project(gu.dev(a_q), gu.dev(a_s), gu.dev(stored), gu.dev(scales), algorithm="stream", packed_k=packed_k)
    np.testing.assert_array_equal(gu.host(half), orc.project(a_q, a_s, w, scales))


# The resident two-stage kernels (K split over the waves of one workgroup per CU, channel blocks of
# 16; K up to 5120 in steps of 512 with loader waves, up to 8192 in steps of 1024 without): every K
# they take, one and two token tiles, channel counts that leave CUs
# without work, with a part block or with several rounds of held blocks, more than 32 rows (several
# launches), the contract shape, fp32 and fp16 outputs with a stride and sentinels around them.
@pytest.mark.parametrize("m,n,k", [(5, 97, 1024), (16, 300, 2048), (17, 1000, 3072), (8, 5000, 4096), (32, 17408, 5120),
                                   (9, 4100, 6144), (31, 600, 7168), (32, 9000, 8192), (33, 513, 1024), (128, 2050, 5120),
                                   (1, 40, 2048), (3, 9728, 2560), (20, 70, 512), (7, 1111, 1536), (32, 4099, 3584),
                                   (16, 257, 4608)])
def test_q4_resident_rows_blocks_and_tails(m, n, k):
    rng = np.random.default_rng(orc.SEED + 300 + m + n)
    a_q, a_s, packed, scales = q4_case(rng, m, n, k)
    a_q[0, :2] = [-128, 127]
    w = orc.q4_integers(packed, TABLE)
    storage = torch.full((m + 2, n + 3), 91.0, dtype=torch.float32, device=gu.DEV)
    gu.q4_project(gu.dev(a_q), gu.dev(a_s), gu.dev(packed), gu.dev(scales), out=storage, stride=n + 3,
                  dtype=torch.float32, algorithm="resident")
    got = gu.host(storage)
    np.testing.assert_array_equal(got[:m, :n], orc.project(a_q, a_s, w, scales, np.float32))
    assert (got[m:] == 91).all() and (got[:m, n:] == 91).all()
    ones_n, ones_m = np.ones(n, np.float16), np.ones(m, np.float16)
    acc = gu.q4_project(gu.dev(a_q), gu.dev(ones_m), gu.dev(packed), gu.dev(ones_n), dtype=torch.float32,
                        algorithm="resident")
    np.testing.assert_array_equal(gu.host(acc).astype(np.int64), orc.int_dot(a_q, w).astype(np.int64))
    half = gu.q4_project(gu.dev(a_q), gu.dev(a_s), gu.dev(packed), gu.dev(scales), algorithm="resident")
    np.testing.assert_array_equal(gu.host(half), orc.project(a_q, a_s, w, scales))
    # launched again into the same buffers (the sums in LDS start from zero every time)
    again = gu.q4_project(gu.dev(a_q), gu.dev(a_s), gu.dev(packed), gu.dev(scales), algorithm="resident")
    assert torch.equal(half, again)


@pytest.mark.parametrize("m,n,k", [(3, 97, 1024), (16, 300, 2048), (17, 1000, 3072), (8, 5000, 4096), (32, 17408, 5120),
                                   (64, 2050, 5120), (5, 40, 2048)])
@pytest.mark.parametrize("blocks_of", [128, 64])
def test_q4_resident_k_major_codes(m, n, k, blocks_of):
    """The loader/decoder kernel on the reference's storage layouts (K/128 blocks of N rows x 64 bytes, K/64 x 32)."""
    rng = np.random.default_rng(orc.SEED + 400 + m + n)
    a_q, a_s, packed, scales = q4_case(rng, m, n, k)
    a_q[0, :2] = [-128, 127]
    stored = orc.q4_pack_k(packed, blocks_of)
    w = orc.q4_integers(packed, TABLE)
    storage = torch.full((m + 2, n + 3), 91.0, dtype=torch.float32, device=gu.DEV)
    gu.q4_project(gu.dev(a_q), gu.dev(a_s), gu.dev(stored), gu.dev(scales), out=storage, stride=n + 3,
                  dtype=torch.float32, algorithm="resident", packed_k=blocks_of)
    got = gu.host(storage)
    np.testing.assert_array_equal(got[:m, :n], orc.project(a_q, a_s, w, scales, np.float32))
    assert (got[m:] == 91).all() and (got[:m, n:] == 91).all()
    half = gu.q4_project(gu.dev(a_q), gu.dev(a_s), gu.dev(stored), gu.dev(scales), packed_k=blocks_of)  # what `auto` picks
    np.testing.assert_array_equal(gu.host(half), orc.project(a_q, a_s, w, scales))


def test_q4_resident_dynamic_rows_and_refusals():
    rng = np.random.default_rng(orc.SEED + 77)
    n, k = 777, 2048
    a_q, a_s, packed, scales = q4_case(rng, 100, n, k)
    w = orc.q4_integers(packed, TABLE)
    for rows in (5, 32, 33, 64, 100):
        got = gu.q4_project(gu.dev(a_q), gu.dev(a_s), gu.dev(packed), gu.dev(scales), rows=rows, dynamic=True,
                            capacity=100, algorithm="resident")
        np.testing.assert_array_equal(gu.host(got)[:rows], orc.project(a_q[:rows], a_s[:rows], w, scales))
    for bad in (dict(K=1280), dict(K=9216), dict(packed_k=128, K=1536), dict(M=129)):
        variant = dict(M=8, N=256, K=1024, algorithm="resident")
        variant.update(bad)
        with pytest.raises(Exception, match="resident"):
            gu.kernel("e8p_q4_projection", **variant)
    with pytest.raises(Exception, match="resident"):
        gu.kernel("int8_projection", M=8, N=256, K=1024, algorithm="resident")


@pytest.mark.parametrize("m,n,k", [(7, 48, 2560), (40, 65, 128), (64, 129, 640)])
def test_w8_stream_matches_oracle(m, n, k):
    rng = np.random.default_rng(orc.SEED + m)
    x = rng.integers(-128, 128, (m, k), dtype=np.int8)
    w = rng.integers(-128, 128, (n, k), dtype=np.int8)
    ws = rng.uniform(0.001, 0.01, n).astype(np.float16)
    ts = rng.uniform(0.001, 0.01, m).astype(np.float16)
    out = torch.full((m + 1, n), 99.0, dtype=torch.float16, device=gu.DEV)
    gu.w8_project(gu.dev(x), gu.dev(ts), gu.dev(w), gu.dev(ws), out=out, algorithm="stream")
    got = gu.host(out)
    np.testing.assert_array_equal(got[:m], orc.project(x, ts, w, ws))
    assert (got[m] == 99).all()


@pytest.mark.parametrize("hints", [dict(algorithm="dp4a", block_m=4, block_n=8), dict(algorithm="tensor_core", block_m=8),
                                   dict(algorithm="int4_direct", block_m=16), dict(algorithm="tensor_core", block_m=96),
                                   dict(block_m=192)], ids=lambda h: "-".join(str(v) for v in h.values()))
def test_reference_schedule_names_and_row_tiles_give_the_same_outputs(hints):
    """The reference's schedule names and row tiles (e8p_q4.py:143-215, int8_projection.py:15-48) choose among this
    library's kernels; whichever kernel a launch then runs, the output is the oracle's to the bit."""
    rng = np.random.default_rng(orc.SEED + 77)
    n, k, capacity = 449, 1024, 300
    a_q, a_s, packed, scales = q4_case(rng, capacity, n, k)
    w = orc.q4_integers(packed, TABLE)
    want = orc.project(a_q, a_s, w, scales)
    x8 = rng.integers(-128, 128, (capacity, k), dtype=np.int8)
    w8 = rng.integers(-128, 128, (n, k), dtype=np.int8)
    want8 = orc.project(x8, a_s, w8, scales)
    for rows in (1, 2, 4, 5, 20, 33, 100, 129, 200, 300):
        got = gu.q4_project(gu.dev(a_q[:rows]), gu.dev(a_s[:rows]), gu.dev(packed), gu.dev(scales), dynamic=True,
                            capacity=capacity, **hints)
        np.testing.assert_array_equal(gu.host(got), want[:rows], err_msg=f"q4 rows {rows}")
        got = gu.w8_project(gu.dev(x8[:rows]), gu.dev(a_s[:rows]), gu.dev(w8), gu.dev(scales), dynamic=True,
                            capacity=capacity, **hints)
        np.testing.assert_array_equal(gu.host(got), want8[:rows], err_msg=f"w8 rows {rows}")


@pytest.mark.parametrize("block_m", [32, 64, 128, 256])
def test_q4_mfma_tiles_and_accumulators(block_m):
    rng = np.random.default_rng(orc.SEED + block_m)
    m, n, k = 300, 384 + 65, 1024
    a_q, a_s, packed, scales = q4_case(rng, m, n, k)
    acc = orc.int_dot(a_q, orc.q4_integers(packed, TABLE))
    got = gu.q4_project(gu.dev(a_q), gu.dev(np.ones(m, np.float16)), gu.dev(packed), gu.dev(np.ones(n, np.float16)),
                        dtype=torch.float32, algorithm="mfma", block_m=block_m)
    np.testing.assert_array_equal(gu.host(got).astype(np.int64), acc.astype(np.int64))
    got16 = gu.q4_project(gu.dev(a_q), gu.dev(a_s), gu.dev(packed), gu.dev(scales), algorithm="mfma", block_m=block_m)
    np.testing.assert_array_equal(gu.host(got16), orc.rescale(acc, scales, a_s))


def test_q4_dynamic_rows_one_handle_many_lengths():
    rng = np.random.default_rng(orc.SEED)
    n, k, cap = 257, 640 + 128, 128
    _, _, packed, scales = q4_case(rng, 1, n, k)
    w = orc.q4_integers(packed, TABLE)
    for m in (1, 2, 4, 5, 31, 64, 127, 128):
        x = rng.normal(size=(m, k)).astype(np.float16)
        a_q, a_s = orc.a8(x)
        out = torch.full((cap + 1, n), 7.0, dtype=torch.float16, device=gu.DEV)
        gu.q4_project(gu.dev(a_q), gu.dev(a_s[:, 0].copy()), gu.dev(packed), gu.dev(scales), dynamic=True,
                      capacity=cap, out=out)
        got = gu.host(out)
        np.testing.assert_array_equal(got[:m], orc.project(a_q, a_s[:, 0], w, scales))
        assert (got[m:] == 7).all()


# ---- W8A8 -----------------------------------------------------------------
@pytest.mark.parametrize("m,n,k", [(1, 48, 2560), (3, 65, 128), (17, 129, 640)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("algorithm", ["auto", "mfma"])
def test_w8_power_of_two_scales_exact(m, n, k, dtype, algorithm):
    # tests/cuda/operators/int8_projection.py:25-41
    rng = np.random.default_rng(orc.SEED + m)
    x = rng.integers(-128, 128, (m, k), dtype=np.int8)
    w = rng.integers(-128, 128, (n, k), dtype=np.int8)
    ws = np.full(n, 0.015625, np.float16)
    ts = np.full(m, 0.0078125, np.float16)
    out = torch.full((m + 1, n), 99.0, dtype=dtype, device=gu.DEV)
    gu.w8_project(gu.dev(x), gu.dev(ts), gu.dev(w), gu.dev(ws), out=out, dtype=dtype, algorithm=algorithm)
    want = orc.project(x, ts, w, ws, np.float32 if dtype == torch.float32 else np.float16)
    got = gu.host(out)
    np.testing.assert_array_equal(got[:m], want)
    assert (got[m] == 99).all()


@pytest.mark.parametrize("m", [1, 3, 17, 63, 65, 129, 511])
def test_w8_dynamic_capacity_stride_extremes(m):
    # int8_projection.py:125-193: capacity 512, N=257, stride 272, forced extremes, ws[0]=0
    rng = np.random.default_rng(orc.SEED + m)
    n, k, stride = 257, 640, 272
    x = rng.integers(-128, 128, (m, k), dtype=np.int8)
    w = rng.integers(-128, 128, (n, k), dtype=np.int8)
    x[:, :4] = [-128, -1, 0, 127]
    ws = (rng.uniform(size=n) * 0.003).astype(np.float16)
    ts = (rng.uniform(size=m) * 0.005).astype(np.float16)
    ws[0] = 0
    storage = torch.full((m + 2, stride), 99.0, dtype=torch.float16, device=gu.DEV)
    gu.w8_project(gu.dev(x), gu.dev(ts), gu.dev(w), gu.dev(ws), dynamic=True, capacity=512, out=storage, stride=stride)
    got = gu.host(storage)
    np.testing.assert_array_equal(got[:m, :n], orc.project(x, ts, w, ws))
    assert (got[m:] == 99).all() and (got[:m, n:] == 99).all()


@pytest.mark.parametrize("k", [64, 192, 2752])
@pytest.mark.parametrize("m", [1, 5, 33, 100, 200, 500])
def test_w8_k_ends_in_half_a_step(m, k):
    # int8_projection.py:29 takes any K that is a multiple of 64; the last K step is then half empty.
    # A sentinel row sits right behind the activations and the weights, so a read past K would change the sums.
    rng = np.random.default_rng(orc.SEED + m + k)
    n, stride = 130, 136
    x = rng.integers(-128, 128, (m + 1, k), dtype=np.int8)
    w = rng.integers(-128, 128, (n + 1, k), dtype=np.int8)
    x[m], w[n] = 127, 127
    ws = (rng.uniform(0.2, 1.0, n) * 0.003).astype(np.float16)
    ts = (rng.uniform(0.2, 1.0, m) * 0.005).astype(np.float16)
    storage = torch.full((m + 2, stride), 99.0, dtype=torch.float32, device=gu.DEV)
    gu.w8_project(gu.dev(x)[:m], gu.dev(ts), gu.dev(w)[:n], gu.dev(ws), dynamic=True, capacity=512, out=storage, stride=stride,
                  dtype=torch.float32)
    got = gu.host(storage)
    np.testing.assert_array_equal(got[:m, :n], orc.project(x[:m], ts, w[:n], ws, np.float32))
    assert (got[m:] == 99).all() and (got[:m, n:] == 99).all()


# Channel runs per CU over the whole K (`algorithm=wide`): one and two row passes, a last pass of one row,
# runs of 2, 97 (two channel passes, the second with one channel) and 100 channels per CU, a K of one step
# and of many, both code layouts, strided fp32 output with sentinels, extremes outside the A8 range.
@pytest.mark.parametrize("packed_k", [0, 128, 64])
@pytest.mark.parametrize("m,n,k", [(33, 300, 384), (64, 24832, 128), (100, 1000, 640), (128, 300, 5120), (129, 515, 256),
                                   (200, 25600, 256), (256, 300, 1024)])
def test_q4_channel_run_kernel(m, n, k, packed_k):
    rng = np.random.default_rng(orc.SEED + m + n + k)
    a_q, a_s, packed, scales = q4_case(rng, m, n, k)
    a_q[0, :4] = [-128, -1, 0, 127]
    a_q[m - 1, -2:] = [127, -128]
    stored = packed if packed_k == 0 else orc.q4_pack_k(packed, packed_k)
    storage = torch.full((m + 2, n + 3), 91.0, dtype=torch.float32, device=gu.DEV)
    gu.q4_project(gu.dev(a_q), gu.dev(a_s), gu.dev(stored), gu.dev(scales), out=storage, stride=n + 3, dtype=torch.float32,
                  algorithm="wide", packed_k=packed_k)
    got = gu.host(storage)
    np.testing.assert_array_equal(got[:m, :n], orc.project(a_q, a_s, orc.q4_integers(packed, TABLE), scales, np.float32))
    assert (got[m:] == 91).all() and (got[:m, n:] == 91).all()
    out16 = gu.q4_project(gu.dev(a_q), gu.dev(a_s), gu.dev(stored), gu.dev(scales), algorithm="wide", packed_k=packed_k)
    np.testing.assert_array_equal(gu.host(out16), orc.project(a_q, a_s, orc.q4_integers(packed, TABLE), scales))


@pytest.mark.parametrize("packed_k", [0, 64, 128])
def test_q4_big_tile_tails_stride_sentinels(packed_k):
    rng = np.random.default_rng(orc.SEED + 9)
    m, n, k = 257 + 130, 300, 384
    a_q, a_s, packed, scales = q4_case(rng, m, n, k)
    a_q[0, :2] = [-128, 127]
    stored = packed if packed_k == 0 else orc.q4_pack_k(packed, packed_k)
    storage = torch.full((m + 2, n + 5), 91.0, dtype=torch.float32, device=gu.DEV)
    gu.q4_project(gu.dev(a_q), gu.dev(a_s), gu.dev(stored), gu.dev(scales), out=storage, stride=n + 5,
                  dtype=torch.float32, algorithm="mfma", packed_k=packed_k, block_m=256)
    got = gu.host(storage)
    np.testing.assert_array_equal(got[:m, :n], orc.project(a_q, a_s, orc.q4_integers(packed, TABLE), scales, np.float32))
    assert (got[m:] == 91).all() and (got[:m, n:] == 91).all()


@pytest.mark.parametrize("packed_k", [0, 64, 128])
@pytest.mark.parametrize("m,n,k", [(512, 256, 512), (500, 333, 640), (700, 130, 256), (3, 128, 384), (300, 17400, 256)])
def test_q4_tall_tiles_decode_in_the_k_loop(m, n, k, packed_k):
    """512 rows x channel runs with the decode in the K loop (`algorithm=tall`): K of an even and an odd number of
    128-blocks, one and two row tiles, ragged rows and channels, runs of one block and (N = 17400 on 256 CUs) of four
    and five blocks with a ragged last block, every layout, fp16 and fp32 output with a stride and sentinels."""
    rng = np.random.default_rng(orc.SEED + m + n + k + packed_k)
    a_q, a_s, packed, scales = q4_case(rng, m, n, k)
    a_q[0, :2] = [-128, 127]
    stored = packed if packed_k == 0 else orc.q4_pack_k(packed, packed_k)
    weights = orc.q4_integers(packed, TABLE)
    for dtype, np_dtype in ((torch.float16, np.float16), (torch.float32, np.float32)):
        storage = torch.full((m + 2, n + 8), 91.0, dtype=dtype, device=gu.DEV)
        gu.q4_project(gu.dev(a_q), gu.dev(a_s), gu.dev(stored), gu.dev(scales), out=storage, stride=n + 8, dtype=dtype,
                      algorithm="tall", packed_k=packed_k)
        got = gu.host(storage)
        np.testing.assert_array_equal(got[:m, :n], orc.project(a_q, a_s, weights, scales, np_dtype))
        assert (got[m:] == 91).all() and (got[:m, n:] == 91).all()


def test_q4_tall_tiles_two_rounds_of_units_and_graph_replay():
    """More blocks of 16 channels than five per CU: the units come in two rounds.  One handle, live rows from a trailing
    scalar, replayed from a graph while the weight bits change in place and the row count changes between captures."""
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    n, k = 16 * (5 * cus + 9) + 3, 256
    rng = np.random.default_rng(orc.SEED + 123)
    a_q, a_s, packed, scales = q4_case(rng, 512, n, k)
    other = rng.integers(0, 2**32, packed.shape, dtype=np.uint32)
    kern = gu.lib.Kernel("e8p_q4_projection", M=512, N=n, K=k, dynamic_rows=True, algorithm="tall")
    assert kern.geometry(300)[0] == (2 * cus, 1, 1)
    d_a, d_as, d_s, d_book, d_w = gu.dev(a_q), gu.dev(a_s), gu.dev(scales), gu.book(), gu.dev(packed)
    out = torch.full((512, n), 7.0, dtype=torch.float16, device=gu.DEV)
    side = torch.cuda.Stream()
    for rows in (300, 512):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                kern(stream=side.cuda_stream, A=d_a, AS=d_as, Book=d_book, Out=out, S=d_s, W=d_w, m=rows)
        for bits in (other, packed, other):
            d_w.copy_(gu.dev(bits))
            out.fill_(7.0)
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            got = gu.host(out)
            np.testing.assert_array_equal(got[:rows], orc.project(a_q[:rows], a_s[:rows], orc.q4_integers(bits, TABLE), scales))
            assert (got[rows:] == 7).all()


@pytest.mark.parametrize("workspace", [False, True])
def test_q4_auto_takes_channel_runs_from_257_rows_of_a_wide_matrix(workspace):
    """257..512 rows of a matrix with at least 2.25 blocks of 16 channels per CU: `auto` decodes in the K loop of the
    512-row channel runs and leaves the Workspace alone; 256 rows and a narrow matrix keep the other kernels."""
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    n, k = 16 * (9 * cus // 4) + 16 + 8, 256
    rng = np.random.default_rng(orc.SEED + 77 + workspace)
    a_q, a_s, packed, scales = q4_case(rng, 512, n, k)
    weights = orc.q4_integers(packed, TABLE)
    variant = dict(M=512, N=n, K=k, dynamic_rows=True, output_stride=n + 8)
    if workspace:
        variant["workspace"] = True
    kern = gu.lib.Kernel("e8p_q4_projection", **variant)
    by_name = gu.lib.Kernel("e8p_q4_projection", **variant, algorithm="tall")
    narrow = [gu.lib.Kernel("e8p_q4_projection", **dict(variant, N=16 * 2 * cus), **extra) for extra in ({}, {"algorithm": "tall"})]
    scratch = torch.zeros(max(kern.workspace_bytes(0), 16), dtype=torch.uint8, device=gu.DEV) if workspace else None
    assert narrow[0].geometry(257) != narrow[1].geometry(257)      # two blocks per CU: the 128 x 128 tiles
    out = torch.full((513, n + 8), 7.0, dtype=torch.float16, device=gu.DEV)
    for rows in (257, 400, 512, 256):
        same = kern.geometry(rows) == by_name.geometry(rows)
        assert same == (rows > 256)
        if rows > 256:
            assert kern.workspace_bytes(rows) == 0
        out.fill_(7.0)
        args = dict(A=gu.dev(a_q), AS=gu.dev(a_s), Book=gu.book(), Out=out, S=gu.dev(scales), W=gu.dev(packed), m=rows)
        if workspace:
            args["Workspace"] = scratch
        kern(**args)
        got = gu.host(out)
        np.testing.assert_array_equal(got[:rows, :n], orc.project(a_q[:rows], a_s[:rows], weights, scales))
        assert (got[rows:] == 7).all() and (got[:rows, n:] == 7).all()


@pytest.mark.parametrize("codec", ["w8", "q4"])
def test_a_few_tiles_more_than_cus_go_to_split_tiles(codec):
    """A handful of 256 x 256 tiles beyond one round of the persistent kernel: it takes the column tiles that fill the
    round and the channels behind them run as split 128 x 128 tiles from the same Workspace (behind the decoded weights
    of two-stage codes).  Ragged last tile, output stride, sentinels; rows checked in every row tile."""
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    rows, k = 1000, 256
    row_tiles = -(-rows // 256)
    main_columns = cus // row_tiles
    n = main_columns * 256 + 2 * 256 + 70          # two whole column tiles and a ragged one behind the round
    assert cus < row_tiles * -(-n // 256) <= cus + cus // 8
    rng = np.random.default_rng(orc.SEED + 91)
    scales = rng.uniform(0.005, 0.02, n).astype(np.float16)
    a_q = rng.integers(-127, 128, (rows, k), dtype=np.int8)
    a_s = rng.uniform(0.005, 0.02, rows).astype(np.float16)
    out = torch.full((rows + 1, n + 5), 7.0, dtype=torch.float16, device=gu.DEV)
    variant = dict(M=rows, N=n, K=k, output_stride=n + 5, workspace=True)
    if codec == "q4":
        packed = rng.integers(0, 2**32, (n, k // 8), dtype=np.uint32)
        weights = orc.q4_integers(packed, TABLE)
        kern = gu.lib.Kernel("e8p_q4_projection", **variant)
        decoded = n * k
        args = dict(A=gu.dev(a_q), AS=gu.dev(a_s), Book=gu.book(), Out=out, S=gu.dev(scales), W=gu.dev(packed))
    else:
        weights = rng.integers(-128, 128, (n, k), dtype=np.int8)
        kern = gu.lib.Kernel("int8_projection", **variant)
        decoded = 0
        args = dict(A=gu.dev(a_q), Output=out, TokenScale=gu.dev(a_s), Weight=gu.dev(weights), WeightScale=gu.dev(scales))
    assert kern.geometry(rows)[0][0] == row_tiles * main_columns     # the persistent launch: one round
    assert kern.workspace_bytes(rows) > decoded                        # partial tiles of the split launch behind it
    assert gu.lib.Kernel(kern.symbol, **dict(variant, split_k=False)).workspace_bytes(rows) == decoded
    kern(**args)
    got = gu.host(out)
    sample = np.unique(np.concatenate([np.arange(0, rows, 37), [127, 128, 255, 256, 511, 512, 767, 768, rows - 1]]))
    want = orc.project(a_q[sample], a_s[sample], weights, scales)
    np.testing.assert_array_equal(got[sample, :n], want)
    assert (got[rows:] == 7).all() and (got[:rows, n:] == 7).all()
    # every row and channel was written, and column sums agree with the oracle's on the sampled rows' complement check
    assert not (got[:rows, :n] == 7).all(axis=0).any()
    # the whole-tile launch of the same handle family gives the same bits
    whole = torch.full_like(out, 7.0)
    other = gu.lib.Kernel(kern.symbol, **dict(variant, split_k=False))
    other(**dict(args, **({"Out": whole} if codec == "q4" else {"Output": whole})))
    np.testing.assert_array_equal(gu.host(whole), got)
    # a dynamic handle of larger capacity: one Workspace sized for any row count serves this launch and a shorter one
    dynamic = gu.lib.Kernel(kern.symbol, **dict(variant, M=1024, dynamic_rows=True))
    space = torch.empty(dynamic.workspace_bytes(0), dtype=torch.uint8, device=gu.DEV)
    assert dynamic.workspace_bytes(0) >= dynamic.workspace_bytes(rows) == kern.workspace_bytes(rows)
    for live in (rows, 300):
        again = torch.full_like(out, 7.0)
        dynamic(**dict(args, Workspace=space, m=live, **({"Out": again} if codec == "q4" else {"Output": again})))
        result = gu.host(again)
        np.testing.assert_array_equal(result[:live], got[:live])
        assert (result[live:] == 7).all()


@pytest.mark.parametrize("packed_k", [0, 64, 128])
@pytest.mark.parametrize("decode_in_gemm", [False, True], ids=["decode-once", "decode-in-gemm"])
def test_q4_many_rows_both_decode_paths(packed_k, decode_in_gemm):
    """From 512 rows on the two-stage weights are decoded once into the caller's Workspace and the
    int8 kernel runs on them; `decode_in_gemm` keeps the decode inside the GEMM.  Same bits either
    way, also when the weights change between launches of one handle and under graph replay."""
    rng = np.random.default_rng(orc.SEED + 31 + packed_k)
    m, n, k = 700, 333, 640
    a_q, a_s, packed, scales = q4_case(rng, m, n, k)
    other = rng.integers(0, 2**32, packed.shape, dtype=np.uint32)
    store = (lambda p: p) if packed_k == 0 else (lambda p: orc.q4_pack_k(p, packed_k))
    # split_k=False: so few 256-row tiles would otherwise go to the split 128-row tiles
    variant = dict(M=1024, N=n, K=k, dynamic_rows=True, output_stride=n + 3, split_k=False)
    if packed_k:
        variant["packed_k"] = packed_k
    if decode_in_gemm:
        variant["decode_in_gemm"] = True
    kern = gu.lib.Kernel("e8p_q4_projection", workspace=True, **variant)
    assert kern.workspace_bytes(700) == (0 if decode_in_gemm else n * k) and kern.workspace_bytes(3) == 0
    d_a, d_as, d_s, d_book = gu.dev(a_q), gu.dev(a_s), gu.dev(scales), gu.book()
    d_w = gu.dev(store(packed))
    out = torch.full((1024, n + 3), 7.0, dtype=torch.float16, device=gu.DEV)
    for rows in (700, 512, 511, 3):        # 511 and 3 take the other kernels of the same handle
        out.fill_(7.0)
        kern(A=d_a, AS=d_as, Book=d_book, Out=out, S=d_s, W=d_w, m=rows)
        got = gu.host(out)
        want = orc.project(a_q[:rows], a_s[:rows], orc.q4_integers(packed, TABLE), scales)
        np.testing.assert_array_equal(got[:rows, :n], want)
        assert (got[rows:] == 7).all() and (got[:rows, n:] == 7).all()
    # same handle, new weight bits in the same buffer, replayed from a graph
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            kern(stream=side.cuda_stream, A=d_a, AS=d_as, Book=d_book, Out=out, S=d_s, W=d_w, m=700)
    for bits in (other, packed, other):
        d_w.copy_(gu.dev(store(bits)))
        out.fill_(7.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want = orc.project(a_q, a_s, orc.q4_integers(bits, TABLE), scales)
        np.testing.assert_array_equal(gu.host(out)[:700, :n], want)


@pytest.mark.parametrize("m,n,k", [(384, 512, 4096), (1000, 777, 640)])
def test_w8_mid_size_accumulators(m, n, k):
    rng = np.random.default_rng(orc.SEED)
    x = rng.integers(-127, 128, (m, k), dtype=np.int8)
    w = rng.integers(-127, 128, (n, k), dtype=np.int8)
    got = gu.w8_project(gu.dev(x), gu.dev(np.ones(m, np.float16)), gu.dev(w), gu.dev(np.ones(n, np.float16)),
                        dtype=torch.float32)
    acc = orc.int_dot(x, w)
    assert np.abs(acc).max() < 2**24
    np.testing.assert_array_equal(gu.host(got).astype(np.int64), acc.astype(np.int64))


# ---- launch contract -------------------------------------------------------
def test_graph_capture_replays_with_changed_contents():
    # Every reference operator test captures once and replays after mutating inputs in place.
    rng = np.random.default_rng(orc.SEED)
    m, n, k = 3, 129, 512
    a_q, a_s, packed, scales = q4_case(rng, m, n, k)
    ta, ts_, tw, tsc = gu.dev(a_q), gu.dev(a_s), gu.dev(packed), gu.dev(scales)
    book = gu.book()
    out = torch.empty((m, n), dtype=torch.float16, device=gu.DEV)
    for algorithm in ("gemv", "mfma"):
        kern = gu.kernel("e8p_q4_projection", M=m, N=n, K=k, algorithm=algorithm)
        args = dict(A=ta, AS=ts_, Book=book, Out=out, S=tsc, W=tw)
        kern(**args)  # warm-up outside capture
        gu.sync()
        stream = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(stream):
            with torch.cuda.graph(graph, stream=stream):
                kern(stream=stream.cuda_stream, **args)
        w = orc.q4_integers(packed, TABLE)
        for step in range(3):
            out.fill_(float("nan"))
            graph.replay()
            gu.sync()
            np.testing.assert_array_equal(gu.host(out), orc.project(gu.host(ta), gu.host(ts_), w, gu.host(tsc)))
            ta.copy_(gu.dev(rng.integers(-127, 128, (m, k), dtype=np.int8)))  # new contents, same addresses
            tsc.mul_(1.5)
        ta.zero_()
        graph.replay()
        gu.sync()
        assert bool((out == 0).all())  # zero-input replay (backend/cuda/mod.rs:649-678)
        ta.copy_(gu.dev(a_q))
        tsc.copy_(gu.dev(scales))


def test_launch_rejects_bad_geometry_rows_and_alignment():
    from orinfer_amd import lib

    kern = gu.kernel("e8p_q4_projection", M=8, N=128, K=256, dynamic_rows=True)
    a = torch.zeros((8, 256), dtype=torch.int8, device=gu.DEV)
    s = torch.ones(8, dtype=torch.float16, device=gu.DEV)
    w = torch.zeros((128, 32), dtype=torch.int32, device=gu.DEV)
    ws = torch.ones(128, dtype=torch.float16, device=gu.DEV)
    out = torch.zeros((8, 128), dtype=torch.float16, device=gu.DEV)
    values = [a, s, gu.book(), out, ws, w, None, 8]    # 8 rows use no Workspace: a null one is taken
    grid, block, shared = kern.geometry(8)
    stream = torch.cuda.current_stream().cuda_stream
    with pytest.raises(lib.OrxError) as e:
        kern.launch_raw((grid[0] + 1, 1, 1), block, shared, stream, values)
    assert e.value.code == lib.ORX_ERR_BAD_GEOMETRY
    with pytest.raises(lib.OrxError) as e:
        kern.launch_raw(grid, block, shared, stream, values[:-1] + [9])
    assert e.value.code == lib.ORX_ERR_ROWS
    with pytest.raises(lib.OrxError) as e:
        kern.launch_raw(grid, block, shared, stream, [a.data_ptr() + 1] + values[1:])
    assert e.value.code == lib.ORX_ERR_BAD_ARGUMENT
    kern.launch_raw(grid, block, shared, stream, values)
    gu.sync()


# ---- benchmark configurations at full size ---------------------------------
def test_config0_full_size_bit_exact():
    c = workloads.config0()
    x = gu.dev(c["x"])
    a_q, a_s = gu.a8(x)
    wq, ws = orc.a8(c["x"])
    np.testing.assert_array_equal(gu.host(a_q), wq)
    np.testing.assert_array_equal(gu.host(a_s), ws)
    out = gu.q4_project(a_q, a_s, gu.dev(c["packed"]), gu.dev(c["scales"]))
    w = orc.q4_integers(c["packed"], TABLE)
    want = orc.project(wq, ws[:, 0], w, c["scales"])
    assert_close_fp16(gu.host(out), want)
    np.testing.assert_array_equal(gu.host(out), want)


@pytest.mark.parametrize("rows", [1, 8, 32, 128, 512])
def test_config1_full_size_bit_exact(rows):
    c = workloads.config1(rows)
    a_q, a_s = gu.a8(gu.dev(c["x"]))
    wq, ws = orc.a8(c["x"])
    np.testing.assert_array_equal(gu.host(a_q), wq)
    out = gu.q4_project(a_q, a_s, gu.dev(c["packed"]), gu.dev(c["scales"]))
    w = _config1_weights(c)
    want = orc.project(wq, ws[:, 0], w, c["scales"])
    assert_close_fp16(gu.host(out), want)
    np.testing.assert_array_equal(gu.host(out), want)


def test_config1_full_size_512_rows_without_scratch():
    """The same 512 rows through a handle without a Workspace: the same 512-row channel runs with the decode in the K
    loop (one workgroup per CU), K-major codes as the package stores them, against the oracle on every row."""
    c = workloads.config1(512)
    a_q, a_s = gu.a8(gu.dev(c["x"]))
    wq, ws = orc.a8(c["x"])
    stored = orc.q4_pack_k(c["packed"], 128)
    kern = gu.lib.Kernel("e8p_q4_projection", M=512, N=c["n"], K=c["k"], packed_k=128)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    assert kern.geometry(512)[1] == (512, 1, 1) and kern.geometry(512)[0] == (min(c["n"] // 16, cus), 1, 1)
    out = torch.empty((512, c["n"]), dtype=torch.float16, device=gu.DEV)
    kern(A=a_q, AS=a_s, Book=gu.book(), Out=out, S=gu.dev(c["scales"]), W=gu.dev(stored))
    np.testing.assert_array_equal(gu.host(out), orc.project(wq, ws[:, 0], _config1_weights(c), c["scales"]))


_weights_cache = {}


def _config1_weights(c):
    if "w" not in _weights_cache:
        _weights_cache["w"] = orc.q4_integers(c["packed"], TABLE)
    return _weights_cache["w"]


def test_config2_full_size_sampled_rows_and_linearity():
    c = workloads.config2()
    a_q, a_s = gu.a8(gu.dev(c["x"]))
    out = gu.w8_project(a_q, a_s, gu.dev(c["weight"]), gu.dev(c["scales"]))
    rows = np.random.default_rng(0).choice(c["rows"], 96, replace=False)
    wq, ws = orc.a8(c["x"][rows])
    np.testing.assert_array_equal(gu.host(a_q)[rows], wq)
    want = orc.project(wq, ws[:, 0], c["weight"], c["scales"])
    np.testing.assert_array_equal(gu.host(out)[rows], want)
    # size-independent property on ALL rows: the int32 accumulators are linear in the activations,
    # so acc(a) + acc(-a) == 0 and acc(a) with unit scales summed over N equals a . colsum(W)
    ones_m = torch.ones(c["rows"], dtype=torch.float16, device=gu.DEV)
    ones_n = torch.ones(c["n"], dtype=torch.float16, device=gu.DEV)
    acc = gu.w8_project(a_q, ones_m, gu.dev(c["weight"]), ones_n, dtype=torch.float32)
    neg = gu.w8_project(-a_q, ones_m, gu.dev(c["weight"]), ones_n, dtype=torch.float32)
    assert bool((acc + neg == 0).all())
    colsum = c["weight"].astype(np.int64).sum(0)
    checksum = gu.host(a_q).astype(np.int64) @ colsum
    np.testing.assert_array_equal(gu.host(acc.double().sum(1)).astype(np.int64), checksum)


# ---- configuration 4: one decoder layer's four projections at M = 8192 --------------------------
_config4_cache = {}


def _config4():
    if "c" not in _config4_cache:
        _config4_cache["c"] = workloads.config4()
    return _config4_cache["c"]


@pytest.mark.parametrize("name", [p[0] for p in workloads.LAYER_PROJECTIONS])
def test_config4_full_size_sampled_rows_and_checksums(name):
    """A8 with outlier channels + projection of every linear of the layer at M = 8192: the codes and
    scales of the quantiser and the fp16 output bit-exact on 96 sampled rows x all N (oracle in
    column blocks: the float64 form of the gate/up matrix alone would be 1.4 GB), and on ALL rows
    acc(a) + acc(-a) == 0, row sums == a . colsum(W), column sums == colsum(a) . W."""
    spec = _config4()[name]
    rows_total, n, k = spec["rows"], spec["n"], spec["k"]
    x = gu.dev(spec["x"])
    a_q, a_s = gu.a8(x)
    del x
    rng = np.random.default_rng(4)
    rows = np.sort(rng.choice(rows_total, 96, replace=False))
    rows[0], rows[-1] = 0, rows_total - 1
    wq, ws = orc.a8(spec["x"][rows])
    got_q = gu.host(a_q)
    np.testing.assert_array_equal(got_q[rows], wq)
    np.testing.assert_array_equal(gu.host(a_s)[rows], ws)
    # the outlier channels (x20) are where the row maxima sit: they must be the +-127 codes
    outliers = np.argsort(np.abs(spec["x"][:64].astype(np.float32)).mean(0))[-max(1, k // 1000):]
    assert (np.abs(got_q[rows][:, outliers]).max(1) == 127).all()
    if spec["codec"] == "q4":
        w_int = orc.q4_integers(spec["packed"], TABLE)
        w_dev, s_dev = gu.dev(spec["packed"]), gu.dev(spec["scales"])
        project = lambda a, s_tok, s_w, **kw: gu.q4_project(a, s_tok, w_dev, s_w, **kw)
    else:
        w_int = spec["weight"]
        w_dev, s_dev = gu.dev(spec["weight"]), gu.dev(spec["scales"])
        project = lambda a, s_tok, s_w, **kw: gu.w8_project(a, s_tok, w_dev, s_w, **kw)
    out = project(a_q, a_s, s_dev)
    got = gu.host(out[torch.from_numpy(rows).to(gu.DEV)])
    del out
    for first in range(0, n, 4096):
        want = orc.project(wq, ws[:, 0], w_int[first:first + 4096], spec["scales"][first:first + 4096])
        assert_close_fp16(got[:, first:first + 4096], want)
        np.testing.assert_array_equal(got[:, first:first + 4096], want)
    # size-independent properties over ALL rows, on the int32 accumulators (fp32 output, unit scales)
    ones_m = torch.ones(rows_total, dtype=torch.float16, device=gu.DEV)
    ones_n = torch.ones(n, dtype=torch.float16, device=gu.DEV)
    acc = project(a_q, ones_m, ones_n, dtype=torch.float32)
    assert float(acc.abs().max()) < 2.0 ** 24  # every accumulator is an exact fp32 value
    neg = project(-a_q, ones_m, ones_n, dtype=torch.float32)
    assert bool((acc + neg == 0).all())
    del neg
    row_sums = gu.host(acc.sum(1, dtype=torch.float64)).astype(np.int64)
    col_sums = gu.host(acc.sum(0, dtype=torch.float64)).astype(np.int64)
    del acc
    w_colsum = np.zeros(k, np.int64)
    for first in range(0, n, 4096):
        w_colsum += w_int[first:first + 4096].sum(0, dtype=np.int64)
    np.testing.assert_array_equal(row_sums, got_q.astype(np.int64) @ w_colsum)
    a_colsum = got_q.sum(0, dtype=np.int64).astype(np.float64)
    want_cols = np.concatenate([(w_int[first:first + 4096].astype(np.float64) @ a_colsum)
                                for first in range(0, n, 4096)]).astype(np.int64)
    np.testing.assert_array_equal(col_sums, want_cols)
    torch.cuda.empty_cache()


# ---- scratch is the caller's ---------------------------------------------------------------------
def test_resolving_handles_takes_no_device_memory():
    torch.cuda.synchronize()
    gu.lib.Kernel("int8_projection", M=8, N=128, K=128)  # the library's one-time set-up, if any
    free_before = torch.cuda.mem_get_info()[0]
    handles = [gu.lib.Kernel("e8p_q4_projection", M=4096 + i, N=17408, K=5120, dynamic_rows=True, workspace=True)
               for i in range(1000)]
    handles += [gu.lib.Kernel("int8_swiglu", M=512 + i, N=1024, K=2048, dynamic_rows=True) for i in range(100)]
    assert torch.cuda.mem_get_info()[0] == free_before
    # the decoded int8 weights, and at 1024 rows (272 tiles of 256 for 256 CUs) the partial tiles of the channels that
    # the persistent launch leaves to the split tiles behind them
    assert handles[0].workspace_bytes(4096) == 17408 * 5120
    assert 17408 * 5120 <= handles[0].workspace_bytes(0) <= 17408 * 5120 + 512 * 2 * 128 * 128 * 4


def test_two_handles_on_two_streams_with_their_own_workspaces_stay_bit_exact():
    """Launches of different handles (and of one handle) overlap on distinct streams as long as their
    buffers, the Workspace included, are distinct: split tiles on one stream, decode-once on the other."""
    rng = np.random.default_rng(orc.SEED + 77)
    cases = []
    for m, n, k in ((256, 5120, 1024), (640, 777, 640)):
        a_q, a_s, packed, scales = q4_case(rng, m, n, k)
        kern = gu.lib.Kernel("e8p_q4_projection", M=m, N=n, K=k, workspace=True)
        assert kern.workspace_bytes(m) > 0
        want = orc.project(a_q, a_s, orc.q4_integers(packed, TABLE), scales)
        cases.append((kern, gu.dev(a_q), gu.dev(a_s), gu.dev(packed), gu.dev(scales), want))
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    # two launches of each handle in flight at once: each (handle, stream) pair has its own workspace and output
    outs, spaces = {}, {}
    for c, (kern, a, s, w, ws, want) in enumerate(cases):
        for t in range(2):
            outs[c, t] = torch.zeros(want.shape, dtype=torch.float16, device=gu.DEV)
            spaces[c, t] = torch.empty(kern.workspace_bytes(0), dtype=torch.uint8, device=gu.DEV)
    torch.cuda.synchronize()
    for repeat in range(6):
        for c, (kern, a, s, w, ws, want) in enumerate(cases):
            for t in range(2):
                kern(stream=streams[t].cuda_stream, A=a, AS=s, Book=gu.book(), Out=outs[c, t], S=ws, W=w,
                     Workspace=spaces[c, t])
    torch.cuda.synchronize()
    for c, (kern, a, s, w, ws, want) in enumerate(cases):
        for t in range(2):
            np.testing.assert_array_equal(gu.host(outs[c, t]), want)


@pytest.mark.parametrize("m,k,block_k,swiglu,planes", [(3, 5120, 512, False, False), (1, 17408, 2048, False, False),
                                                       (5, 640, 256, True, False), (4, 1152, 1024, True, True),
                                                       (2, 128, 128, False, False)])
def test_rotation_in_tiles_gives_the_one_launch_codes(m, k, block_k, swiglu, planes):
    # kernels/cuda/model/rotation_a8.py:266-365: rotate_activation_tiles then quantize_rotation_tiles
    rng = np.random.default_rng(orc.SEED + m + k)
    x = (rng.normal(size=(m, 2 * k if swiglu else k)) * rng.uniform(0.2, 3.0, (m, 1))).astype(np.float16)
    signs = rng.choice(np.array([-1, 1], np.int8), k)
    cap = m + 2
    blocks = (k + block_k - 1) // block_k
    plane_rows = cap + 1 if planes else 0
    if planes:  # gate rows, then the up rows as a second plane
        stacked = np.zeros((cap + plane_rows, k), np.float16)
        stacked[:m], stacked[plane_rows:plane_rows + m] = x[:, :k], x[:, k:]
        d_x = gu.dev(stacked)
    else:
        d_x = gu.dev(np.concatenate([x, np.zeros((cap - m, x.shape[1]), np.float16)]))
    rotated = torch.full((cap, k), 9.0, dtype=torch.float16, device=gu.DEV)
    maxima = torch.full((m, blocks), -1.0, dtype=torch.float32, device=gu.DEV)
    variant = dict(M=cap, K=k, block_k=block_k, dynamic_rows=True)
    gu.kernel("rotate_activation_tiles", swiglu=swiglu, plane_rows=plane_rows, **variant)(
        Maxima=maxima, Rotated=rotated, Signs=gu.dev(signs), X=d_x, m=m)
    single = torch.empty((m, k), dtype=torch.float16, device=gu.DEV)
    gu.kernel("rotate_activation", M=m, K=k, swiglu=swiglu)(Signs=gu.dev(signs), X=gu.dev(x), Y=single)
    assert torch.equal(rotated[:m], single) and bool((rotated[m:] == 9).all())
    values = np.abs(gu.host(single).astype(np.float32))
    padded = np.zeros((m, blocks * block_k), np.float32)
    padded[:, :k] = values
    np.testing.assert_array_equal(gu.host(maxima), padded.reshape(m, blocks, block_k).max(axis=2))
    q = torch.full((cap, k), 77, dtype=torch.int8, device=gu.DEV)
    s = torch.full((cap,), 5.0, dtype=torch.float16, device=gu.DEV)
    gu.kernel("quantize_rotation_tiles", **variant)(Maxima=maxima, Q=q, Rotated=rotated, S=s, m=m)
    want_q = torch.empty((m, k), dtype=torch.int8, device=gu.DEV)
    want_s = torch.empty((m,), dtype=torch.float16, device=gu.DEV)
    gu.kernel("rotate_activation_a8", M=m, K=k, swiglu=swiglu)(Q=want_q, S=want_s, Signs=gu.dev(signs), X=gu.dev(x))
    assert torch.equal(q[:m], want_q) and torch.equal(s[:m], want_s)
    assert bool((q[m:] == 77).all()) and bool((s[m:] == 5).all())
    if not swiglu:
        oracle_q, oracle_s = orc.rotate_a8(x, signs)
        np.testing.assert_array_equal(gu.host(q)[:m], oracle_q)
        np.testing.assert_array_equal(gu.host(s)[:m], oracle_s[:, 0])


def test_rotation_tiles_refuse_what_the_reference_refuses():
    for bad in (dict(block_k=384), dict(K=192), dict(plane_rows=8), dict(swiglu=True, plane_rows=2), dict(threads=256),
                dict(registers=True, threads=512, block_k=1024), dict(registers=True, threads=96)):
        with pytest.raises(Exception):
            gu.kernel("rotate_activation_tiles", **{**dict(M=4, K=1024), **bad})
    gu.kernel("rotate_activation_tiles", M=4, K=1024, registers=True, threads=256, block_k=1024)
    with pytest.raises(Exception):
        gu.kernel("quantize_rotation_tiles", M=4, K=1024, block_k=64)


@pytest.mark.parametrize("m,n,k,symbol", [(3, 333, 640, "q4_projection"), (3, 333, 640, "q4_gemv"), (1, 9728, 2560, "q4_gemv"),
                                          (2, 333, 640, "q4_gemv"), (1, 129, 128, "q4_projection"), (2, 5000, 3200, "q4_projection"),
                                          (33, 200, 1024, "q4_projection"), (64, 129, 256, "q4_projection"),
                                          (65, 260, 384, "q4_projection"), (130, 1000, 1280, "q4_projection"),
                                          (700, 300, 512, "q4_projection")])
def test_scalar_q4_projection_at_every_row_range(m, n, k, symbol):
    # kernels/cuda/model/q4_projection.py; the check of python/orinfer_build/quantization/check_e8p_q4.py:195-214
    # (random u16 words, rows in -128..127, unit token scales, fp32 out) plus fp16 with scales, strides and live rows
    rng = np.random.default_rng(orc.SEED + m + n)
    words = rng.integers(0, 65536, (n, k // 4), dtype=np.uint16)
    weights = orc.row_q4_integers(words)
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    ws = rng.uniform(0.005, 0.02, n).astype(np.float16)
    cap, stride = m + 3, n + 5
    pad = np.concatenate([a, np.zeros((cap - m, k), np.int8)])
    ones = np.ones(cap, np.float16)
    extra = {} if symbol == "q4_gemv" else dict(workspace=True)
    kern = gu.kernel(symbol, M=cap, N=n, K=k, dynamic_rows=True, output_dtype="float32", output_stride=stride, **extra)
    out = torch.full((cap, stride), -7.0, dtype=torch.float32, device=gu.DEV)
    args = dict(A=gu.dev(pad), AS=gu.dev(ones), Out=out, S=gu.dev(ws), W=gu.dev(words), m=m)
    kern(**args)
    got = gu.host(out)
    np.testing.assert_array_equal(got[:m, :n], orc.project(a, ones[:m], weights, ws, np.float32))
    assert (got[m:] == -7).all() and (got[:, n:] == -7).all()
    # unit weight scales: the int32 accumulators themselves
    args["S"] = gu.dev(np.ones(n, np.float16))
    kern(**args)
    np.testing.assert_array_equal(gu.host(out)[:m, :n], (a.astype(np.int64) @ weights.astype(np.int64).T).astype(np.float32))
    scales = rng.uniform(0.01, 0.03, cap).astype(np.float16)
    half = torch.full((cap, n), 9.0, dtype=torch.float16, device=gu.DEV)
    plain = gu.kernel(symbol, M=cap, N=n, K=k, dynamic_rows=True)
    plain(A=gu.dev(pad), AS=gu.dev(scales), Out=half, S=gu.dev(ws), W=gu.dev(words), m=m)
    np.testing.assert_array_equal(gu.host(half)[:m], orc.project(a, scales[:m], weights, ws))
    assert bool((half[m:] == 9).all())


def test_scalar_q4_other_magnitudes_extremes_and_unpack():
    rng = np.random.default_rng(orc.SEED + 77)
    n, k, m = 160, 512, 5
    magnitudes = [1, 2, 5, 9, 33, 64, 100, 127]
    words = rng.integers(0, 65536, (n, k // 4), dtype=np.uint16)
    words[0] = 0xFFFF  # -127 everywhere
    words[1] = 0x7777  # +127 everywhere
    weights = orc.row_q4_integers(words, magnitudes)
    assert (weights[0] == -127).all() and (weights[1] == 127).all()
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    a[0] = -128
    out = torch.empty((m, n), dtype=torch.float32, device=gu.DEV)
    gu.kernel("q4_projection", M=m, N=n, K=k, magnitudes=magnitudes, output_dtype="float32")(
        A=gu.dev(a), AS=gu.dev(np.ones(m, np.float16)), Out=out, S=gu.dev(np.ones(n, np.float16)), W=gu.dev(words))
    np.testing.assert_array_equal(gu.host(out), (a.astype(np.int64) @ weights.astype(np.int64).T).astype(np.float32))
    assert gu.host(out)[0, 0] == 128 * 127 * k
    unpacked = torch.full((n + 1, k), 55, dtype=torch.int8, device=gu.DEV)
    gu.kernel("unpack_q4", N=n, K=k, magnitudes=magnitudes)(Output=unpacked, W=gu.dev(words))
    np.testing.assert_array_equal(gu.host(unpacked)[:n], weights)
    assert bool((unpacked[n] == 55).all())
