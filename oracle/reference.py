"""CPU oracle for the quantized linear-layer path (TEST INFRASTRUCTURE ONLY).

This module restates, in plain numpy, the arithmetic that iMMIQ/orinfer's E8P
Q4A8 / Q2A8 / W8A8 kernels implement.  It is the checker for the HIP kernels
and the timed CPU baseline; it is never imported by the product package
(`orinfer_amd`).  Only tests/, __graft_entry__.smoke() and bench.py's
cpu_baseline leg may import it.

Every function cites the reference file:line it follows.  Pinning status:

* basis()                pinned by tests/golden/e8p_basis.npy (written from the
                         reference's own basis()), plus closed-form invariants
* e8p_decode()           pinned by the scalar formula, the palette decoders and
                         the XOR/nibble identities of the reference's test_vq.py
* q4_integers()          pinned by the exhaustive 65 536-code fixture
* q2_integers()          decode as above; the patch words by a scalar loop over every
                         (row, group) and the word the reference's own test plants
                         (tests/cuda/operators/e8p_selector.py:38); tables with zero
                         coordinates by the scalar decode and the 1 - 2p rule
* row_q4_integers()      pinned by the reference's own known answer (every signed nibble,
                         quantization/test_row_q4.py:11-16) and by the byte-permute form of
                         kernels/cuda/model/q4_projection.py:23-29 emulated on all 65 536 words
* a8()                   pinned by closed-form edge cases (ties, clamp, floor)
* project()/rescale()    pinned by brute-force int64 dots and power-of-two KATs
* router_topk()/metadata pinned by stable argsort / enumeration
* swiglu(), combine()    pinned by direct formula on tiny inputs
* split_planes(), nibble_table(), nibble_decode(), plane_project()
                         the plane words by the reference's mask-and-shift form and its
                         test's low + 16 high == permuted codes; the nibble decode by
                         2y + 1 == e8p_decode() over all 65 536 codes; plane_project by
                         project() on the same integers and a planted Sum
* rotate(), rotate_a8()  pinned by the Sylvester Hadamard matrix (exact on small
                         integers), dot preservation and the involution of the
                         reference's test_vq.py:123-130
"""

import itertools

import numpy as np

# Coordinate j of a codeword takes its sign from bit SIGN_BITS[j] of the
# parity-adjusted low byte (python/orinfer_build/quantization/vq.py:17).
SIGN_BITS = (0, 4, 1, 5, 2, 6, 3, 7)
SEED = 20261002  # python/orinfer_build/compiler/cuda/common.py:18


# --------------------------------------------------------------------------
# Codebook
# --------------------------------------------------------------------------
def basis():
    """256x8 int8 E8P basis (python/orinfer_build/quantization/e8p.py:15-25).

    Inner rows: magnitudes in {2,6,10}, lexicographic product order, squared
    norm <= 160 (227 rows).  Outer rows: 29 patterns of five 6s and three 2s,
    taken at positions i*56//29 of the 56 five-subsets of range(8).  The last
    coordinate is negated when sum(row)//4 is odd.
    """
    inner = [r for r in itertools.product((2, 6, 10), repeat=8) if sum(v * v for v in r) <= 160]
    subsets = list(itertools.combinations(range(8), 5))
    outer = []
    for i in range(29):
        chosen = subsets[i * len(subsets) // 29]
        outer.append(tuple(6 if j in chosen else 2 for j in range(8)))
    rows = np.array(inner + outer, dtype=np.int16)
    flip = (rows.sum(axis=1) // 4) % 2 == 1
    rows[flip, 7] = -rows[flip, 7]
    assert rows.shape == (256, 8)
    return rows.astype(np.int8)


def e8p_decode(codes, table):
    """u16 code -> 8 int8 lattice coordinates (vq.py:34-43, docs/quantization.md:66-72).

    b = code>>8, u = code&255, p = popcount(u)&1, m = u^p,
    q[j] = table[b,j] * (1 - 2*bit(m, SIGN_BITS[j])) + (1 - 2p).
    """
    c = np.asarray(codes).astype(np.uint16).astype(np.int32)
    u = c & 255
    p = np.zeros_like(u)
    for bit in range(8):
        p ^= (u >> bit) & 1
    m = u ^ p
    sign = np.stack([1 - 2 * ((m >> s) & 1) for s in SIGN_BITS], axis=-1)
    t = np.asarray(table).astype(np.int32)[c >> 8]
    return (t * sign + (1 - 2 * p)[..., None]).astype(np.int8)


def e8p_decode_scalar(code, table):
    """Pure-Python scalar decode of one code (test_vq.py:132-147); small cases only."""
    code = int(code)
    u = code & 255
    p = bin(u).count("1") & 1
    m = u ^ p
    return [
        int(table[code >> 8][j]) * (-1 if (m >> SIGN_BITS[j]) & 1 else 1) + (1 - 2 * p)
        for j in range(8)
    ]


def selector_table(table):
    """(256,1) u32 selector LUT the engine binds as `Book` (vq.py:74-93).

    Nibble j = magnitude id ((|t|-2)/4, or 3 for zero) | 4 if t<0.
    """
    t = np.asarray(table)
    if t.dtype != np.int8 or t.shape != (256, 8) or not np.isin(t, (-10, -6, -2, 0, 2, 6, 10)).all():
        raise ValueError("selector table needs values in {0,+-2,+-6,+-10}")
    v = t.astype(np.int64)
    ident = np.where(v == 0, 3, (np.abs(v) - 2) // 4) + 4 * (v < 0)
    word = np.zeros(256, np.uint64)
    for j in range(8):
        word |= ident[:, j].astype(np.uint64) << np.uint64(4 * j)
    return word.astype(np.uint32).reshape(256, 1)


def sign_table(table):
    """(512, 4) u32: for basis row b at parity p (row p * 256 + b) the words [low half +, low half -, high half +,
    high half -] of the values +-t + (1 - 2p), int8 wrap-around (python/orinfer_build/quantization/vq.py:44-69)."""
    t = np.asarray(table, np.int8).astype(np.int16)
    values = np.empty((512, 8, 2), np.int8)
    for parity in (0, 1):
        shift = 1 - 2 * parity
        values[parity * 256:(parity + 1) * 256, :, 0] = (t + shift).astype(np.int8)
        values[parity * 256:(parity + 1) * 256, :, 1] = (-t + shift).astype(np.int8)
    columns = [np.ascontiguousarray(values[:, half * 4:half * 4 + 4, sign]).view("<u4").reshape(512)
               for half in range(2) for sign in range(2)]
    return np.stack(columns, axis=-1)


def basis_words(table):
    """(256,2) u32 raw int8 basis view used by the single-token Q2 kernel (vq.py:203)."""
    return np.ascontiguousarray(np.asarray(table, np.int8)).view("<u4").reshape(256, 2)


# --------------------------------------------------------------------------
# Weights
# --------------------------------------------------------------------------
def q4_integers(packed, table, coefficients=(4, 1)):
    """Two-stage Q4 int8 weights (quantization/e8p_q4.py:61-67).

    packed u32 [N, K/8]: low half = coarse code, high half = residual code.
    w = a*decode(lo) + b*decode(hi); (a,b)=(4,1) gives |w| <= 55.
    """
    packed = np.asarray(packed)
    if packed.dtype != np.uint32 or packed.ndim != 2:
        raise ValueError("expected u32 [N, K/8]")
    a, b = coefficients
    if packed.size > (1 << 20):
        # large matrices: e8p_decode is a function of the code alone, so it is evaluated once for
        # each of the 65 536 codes and gathered (same values, minutes -> seconds at 10^8 weights)
        every = e8p_decode(np.arange(65536, dtype=np.uint32).astype(np.uint16), table).astype(np.int16)
        w = np.empty((packed.shape[0], packed.shape[1], 8), np.int8)
        step = max(1, (1 << 22) // packed.shape[1])
        for first in range(0, packed.shape[0], step):
            block = packed[first:first + step]
            value = a * every[block & 0xFFFF] + b * every[block >> 16]
            assert np.abs(value).max() <= 127
            w[first:first + step] = value
        return w.reshape(packed.shape[0], packed.shape[1] * 8)
    lo = e8p_decode((packed & 0xFFFF).astype(np.uint16), table).astype(np.int16)
    hi = e8p_decode((packed >> 16).astype(np.uint16), table).astype(np.int16)
    w = a * lo + b * hi
    assert np.abs(w).max() <= 127
    return w.reshape(packed.shape[0], packed.shape[1] * 8).astype(np.int8)


def q2_integers(indices, table, patches=None):
    """Single-stage int8 weights from u16 [N, K/8] (vq.py:184-194).

    `patches` [N, K/128] u16 overrides at most one weight per row and group of 128: bit 15 says the
    word is valid, bits 0-6 give the position inside the group, bits 7-14 the int8 value.
    """
    indices = np.asarray(indices)
    if indices.dtype != np.uint16 or indices.ndim != 2:
        raise ValueError("expected u16 [N, K/8]")
    weights = e8p_decode(indices, table).reshape(indices.shape[0], indices.shape[1] * 8).copy()
    if patches is not None:
        words = np.asarray(patches)
        if words.dtype != np.uint16 or words.shape != (weights.shape[0], weights.shape[1] // 128):
            raise ValueError("expected one u16 patch word per row and group of 128")
        for row, group in zip(*np.nonzero(words >> 15)):
            word = int(words[row, group])
            stored = (word >> 7) & 255
            weights[row, 128 * group + (word & 127)] = stored - 256 if stored > 127 else stored
    return weights


ROW_Q4_MAGNITUDES = (3, 10, 19, 31, 46, 67, 93, 127)  # python/orinfer_build/quantization/row_q4.py:15


def row_q4_integers(packed, magnitudes=ROW_Q4_MAGNITUDES):
    """Row-scaled scalar Q4: uint8 (N, K/2), two nibbles per byte, low nibble first -> int8 (N, K).

    python/orinfer_build/quantization/row_q4.py:45-51: weight = magnitudes[nibble & 7], negated for
    nibbles 8..15.  The kernels bind the same bytes as (N, K/4) u16
    (kernels/cuda/model/q4_projection.py:66, :165).
    """
    packed = np.asarray(packed)
    if packed.dtype == np.uint16:
        packed = np.ascontiguousarray(packed).view(np.uint8)
    codes = np.stack((packed & 15, packed >> 4), axis=-1).reshape(packed.shape[0], -1)
    values = np.asarray(magnitudes, np.int8)[codes & 7]
    return np.where(codes < 8, values, -values).astype(np.int8)


def q4_pack_k(packed, packed_k):
    """Row-major (N,K/8) u32 -> K-major (K/pk, N, pk/8) (models/qwen35/storage.py:69-76)."""
    n, vectors = packed.shape
    per = packed_k // 8
    return np.ascontiguousarray(packed.reshape(n, vectors // per, per).transpose(1, 0, 2))


def q2_pack_k128(indices):
    """(N,K/8) u16 -> (K/128, N, 16) (vq.py:199-202)."""
    n, vectors = indices.shape
    return np.ascontiguousarray(indices.reshape(n, vectors // 16, 16).transpose(1, 0, 2))


def q2_repack_k64(packed):
    """(E,K/128,N,16) u16 -> (E,K/64,N,8), codes unchanged (vq.py:121-128): K block 2g holds the first
    eight codes of every row of group g, block 2g + 1 the other eight."""
    experts, groups, rows, per_row = packed.shape
    if per_row != 16:
        raise ValueError("expected sixteen codes per row and group of 128")
    blocks = np.empty((experts, 2 * groups, rows, 8), packed.dtype)
    blocks[:, 0::2] = packed[..., :8]
    blocks[:, 1::2] = packed[..., 8:]
    return blocks


# --------------------------------------------------------------------------
# Activations
# --------------------------------------------------------------------------
def a8(x, group=None):
    """fp16 -> int8 codes + fp16 scale per (row, group).

    quantization/reference_math.py:6-20 and
    kernels/cuda/operators/op30_activation_quantization.py:14-18,49-65:
    scale = fp16(max(amax/127, 2^-24)) or 1 when amax == 0;
    code = clamp(rint(x / fp32(scale)), -127, 127), ties to even.
    Returns (codes int8 [M,K], scale fp16 [M, groups]).
    """
    x = np.asarray(x).astype(np.float16).astype(np.float32)
    if x.ndim != 2 or not np.isfinite(x).all():
        raise ValueError("a8 wants a finite 2-D fp16 matrix")
    width = x.shape[1] if group is None else group
    if x.shape[1] % width:
        raise ValueError("group must divide K")
    g = x.reshape(x.shape[0], -1, width)
    amax = np.abs(g).max(axis=-1)
    floor = np.float32(2.0**-24)
    raw = np.maximum(amax / np.float32(127.0), floor).astype(np.float32)
    scale = np.where(amax > 0, raw, np.float32(1.0)).astype(np.float16)
    ratio = g / scale.astype(np.float32)[..., None]
    codes = np.clip(np.rint(ratio), -127, 127).astype(np.int8)
    return codes.reshape(x.shape), scale


def swiglu_fp16(gu):
    """fp16 [M,2I] -> fp16 [M,I]: silu(gate)*up in fp32 with a stable sigmoid, one fp16 cast.

    kernels/cuda/operators/op04_swiglu.py:6-17, reference_math.py:31-35.
    """
    gu = np.asarray(gu).astype(np.float16).astype(np.float32)
    g, u = np.split(gu, 2, axis=-1)
    e = np.exp(-np.abs(g)).astype(np.float32)
    one = np.float32(1.0)
    sig = np.where(g >= 0, one / (one + e), e / (one + e)).astype(np.float32)
    return ((g * sig) * u).astype(np.float16)


def rotate(x, signs):
    """Signed block-128 Hadamard rotation in fp32 (python/orinfer_build/quantization/vq.py:20-31).

    y = x * signs, then seven butterfly stages with partner distance 1, 2, .. 64 inside every block
    of 128: the element whose distance bit is clear becomes itself + partner, the other one
    partner - itself; then one multiply by fp32(128 ** -0.5).  Every step is a single fp32
    operation, so a kernel that runs the stages in the same order is bit-exact.
    """
    values = np.asarray(x, dtype=np.float32)
    flips = np.asarray(signs)
    width = values.shape[-1]
    if width % 128 != 0 or flips.shape != (width,) or np.any(np.abs(flips) != 1):
        raise ValueError("block-128 rotation needs one +-1 sign per input channel")
    y = values * flips.astype(np.float32)
    position = np.arange(width)
    for distance in (1, 2, 4, 8, 16, 32, 64):
        partner = y[..., position ^ distance]
        upper = (position & distance) != 0
        y = np.where(upper, partner - y, y + partner).astype(np.float32)
    return (y * np.float32(128**-0.5)).astype(np.float32)


def rotate_a8(x, signs, swiglu=False):
    """fp16 activations -> rotated int8 codes + one fp16 scale per row.

    kernels/cuda/model/rotation_a8.py:188-224 (load, optional fp16 SwiGLU boundary, signs,
    butterflies, fp16 materialisation of the scaled result), :144-164 and :369-383 (row scale
    and codes: the A8 rule on the materialised fp16 values; the reciprocal form there falls
    back to the exact divide near ties, so it produces the same codes).
    """
    x = np.asarray(x).astype(np.float16)
    values = swiglu_fp16(x) if swiglu else x
    rotated = rotate(values.astype(np.float32), signs).astype(np.float16)
    return a8(rotated)


def residual_norm(x, residual, weight, epsilon=1e-6, zero_centered=True):
    """Residual add and RMSNorm: (fp16 normalised row, fp32 residual sum).

    kernels/cuda/operators/op02_residual_norm.py:13-38: sum = fp32(x) + residual is returned
    unrounded; the row is normalised as fp16((sum * rsqrt(mean(sum^2) + epsilon)) * (fp32(w) + 1))
    (+0 when the weights are not stored zero-centred), the two products in fp32 in that order.
    The mean is taken in float64 here: the order of the fp32 partial sums is the reference
    kernel's own business, so a kernel is compared to one fp16 unit in the last place.
    """
    x = np.asarray(x).astype(np.float16)
    total = (x.astype(np.float32) + np.asarray(residual, dtype=np.float32)).astype(np.float32)
    mean = (total.astype(np.float64) ** 2).sum(axis=-1, keepdims=True) / x.shape[-1]
    inverse = (1.0 / np.sqrt(mean.astype(np.float32).astype(np.float64) + np.float32(epsilon))).astype(np.float32)
    gain = (np.asarray(weight).astype(np.float16).astype(np.float32) + np.float32(1.0 if zero_centered else 0.0))
    scaled = (total * inverse).astype(np.float32)
    return (scaled * gain).astype(np.float32).astype(np.float16), total


def residual_norm_rotate_a8(x, residual, weight, signs, epsilon=1e-6, zero_centered=True):
    """Fused residual RMSNorm + rotation + A8: (Y fp16, RO fp32, codes, row scales).

    kernels/cuda/model/rotation_a8.py:607-659: the rotation reads the fp16 normalised row, so the
    result equals rotate_a8 of Y (the reference's own check, models/qwen35/check_rows.py:167-172).
    """
    y, total = residual_norm(x, residual, weight, epsilon, zero_centered)
    codes, scales = rotate_a8(y, signs)
    return y, total, codes, scales


def q4_embedding(ids, packed, table, scales, signs):
    """Token ids -> fp16 rows of the un-rotated embedding (kernels/cuda/model/e8p_q4.py:83-140).

    `packed` is the row-major (vocab, hidden/8) u32 code matrix (the kernel reads its K-major
    form).  Per row: int8 weights, unsigned block-128 butterflies and * fp32(128**-0.5) (that is
    rotate() with all signs +1), * fp32(scale[id]), * sign, one fp16 cast; ids outside
    [0, vocab) give zero rows.
    """
    ids = np.asarray(ids)
    weights = q4_integers(packed, table)
    vocab, hidden = weights.shape
    out = np.zeros((ids.shape[0], hidden), np.float16)
    ones = np.ones(hidden, np.int8)
    for row, token in enumerate(ids.tolist()):
        if 0 <= token < vocab:
            value = rotate(weights[token].astype(np.float32)[None, :], ones)[0]
            value = (value * np.float32(np.float16(scales[token]))).astype(np.float32)
            out[row] = (value * np.asarray(signs, np.float32)).astype(np.float16)
    return out


# --------------------------------------------------------------------------
# Contraction + epilogue
# --------------------------------------------------------------------------
def int_dot(a_q, w_q):
    """Exact int32 accumulators [M,N] via fp64 BLAS (tests/cuda/operators/quantized_reference.py:12-15).

    Exact because |sum| <= 128*128*K < 2^53 for every K on this path.
    """
    a = np.asarray(a_q)
    w = np.asarray(w_q)
    assert a.dtype == np.int8 and w.dtype == np.int8 and a.shape[1] == w.shape[1]
    dot = a.astype(np.float64) @ w.astype(np.float64).T
    return dot.astype(np.int64).astype(np.int32)


def int_dot_bruteforce(a_q, w_q):
    """Pure integer dot, no floating point anywhere; for pinning int_dot on small shapes."""
    a = np.asarray(a_q).astype(np.int64)
    w = np.asarray(w_q).astype(np.int64)
    return np.einsum("mk,nk->mn", a, w).astype(np.int32)


def rescale(acc, weight_scale, token_scale, out_dtype=np.float16):
    """(fp32(acc) * fp32(ws)) * fp32(as), one cast (kernels/cuda/model/integer_core.py:19-22)."""
    value = np.asarray(acc).astype(np.float32) * np.asarray(weight_scale).astype(np.float32)[None, :]
    value = value * np.asarray(token_scale).astype(np.float32).reshape(-1)[:, None]
    return value.astype(out_dtype)


def project(a_q, a_scale, w_q, w_scale, out_dtype=np.float16):
    """int8 x int8 -> int32 -> rescale (tests/cuda/operators/flash_next_quantized.py:30-37)."""
    return rescale(int_dot(a_q, w_q), w_scale, a_scale, out_dtype)


# --------------------------------------------------------------------------
# MoE routing (kernels/cuda/model/moe.py)
# --------------------------------------------------------------------------
def int8_swiglu(a_q, token_scale, gate, gate_scale, up, up_scale):
    """Shared-expert W8 gate/up projections with the SwiGLU boundary
    (kernels/cuda/model/int8_swiglu.py:10-57, integer_core.py:19-28): both projections are
    rounded to fp16, then fp16((g / (1 + exp(-g))) * u) evaluated in fp32."""
    g = project(a_q, token_scale, gate, gate_scale).astype(np.float32)
    u = project(a_q, token_scale, up, up_scale).astype(np.float32)
    with np.errstate(over="ignore"):
        value = (g / (np.float32(1.0) + np.exp(-g).astype(np.float32))).astype(np.float32) * u
    return value.astype(np.float16)


def router_topk(logits, top_k, renormalize=True):
    """fp32 logits [M,E] -> ids int32 [M,k], prob fp32 [M,k] (moe.py:413-494).

    Descending logit, exact ties -> lower id, -0 == +0 (stable descending
    argsort, tests/cuda/operators/moe.py:51-57).  prob = exp(l-max)/den with
    den over the selected experts (renormalize) or over all E.
    """
    logits = np.asarray(logits, np.float32)
    m, e = logits.shape
    key = np.where(logits == 0, np.float32(0.0), logits)  # fold signed zero
    ids = np.argsort(-key.astype(np.float64), axis=1, kind="stable")[:, :top_k].astype(np.int32)
    top = logits.max(axis=1, keepdims=True)
    picked = np.take_along_axis(logits, ids.astype(np.int64), axis=1)
    num = np.exp((picked - top).astype(np.float32)).astype(np.float32)
    if renormalize:
        den = num.sum(axis=1, keepdims=True, dtype=np.float32)
    else:
        den = np.exp((logits - top).astype(np.float32)).sum(axis=1, keepdims=True, dtype=np.float32)
    return ids, (num / den).astype(np.float32)


def router_projection(x, w):
    """Logits fp32 (m, E) and SharedGate fp16 (m,) = x (m, H) . w (E + 1, H)^T (kernels/cuda/model/moe.py:15-49).

    fp16 operands with fp32 accumulation in the kernels; here the products are summed in float64 and
    rounded once, and the tests bound the difference by the fp32 rounding of the partial sums.
    """
    full = np.asarray(x, np.float16).astype(np.float64) @ np.asarray(w, np.float16).astype(np.float64).T
    return full[:, :-1].astype(np.float32), full[:, -1].astype(np.float16)


def expert_histogram(ids, experts):
    """Counts[E], RelativeSlot[M,k]; assignment order token-major, rank-minor (moe.py:177-210)."""
    ids = np.asarray(ids, np.int32)
    counts = np.zeros(experts, np.int32)
    relative = np.zeros_like(ids)
    for row in range(ids.shape[0]):
        for rank in range(ids.shape[1]):
            e = int(ids[row, rank])
            relative[row, rank] = counts[e]
            counts[e] += 1
    return counts, relative


def expert_offsets(counts, block_m):
    """RowOffsets, TileOffsets (exclusive prefixes) and TileCount (moe.py:214-244)."""
    counts = np.asarray(counts, np.int64)
    tiles = (counts + block_m - 1) // block_m
    rows = np.cumsum(counts) - counts
    tile_offsets = np.cumsum(tiles) - tiles
    return rows.astype(np.int32), tile_offsets.astype(np.int32), np.array([tiles.sum()], np.int32)


def expert_tiles(counts, tile_offsets, block_m, capacity):
    """(TileExpert, TileRow) lists; entries beyond TileCount stay -1 here (moe.py:248-282)."""
    tile_expert = np.full(capacity, -1, np.int32)
    tile_row = np.full(capacity, -1, np.int32)
    for e, c in enumerate(np.asarray(counts)):
        for t in range((int(c) + block_m - 1) // block_m):
            tile_expert[tile_offsets[e] + t] = e
            tile_row[tile_offsets[e] + t] = t * block_m
    return tile_expert, tile_row


def single_route_metadata(ids, experts, capacity):
    """One token's routes in expert-id order (moe.py:659-709): every selected expert owns one row
    and one tile.  Returns counts, relative slots (all zero), row offsets, tile offsets (equal to
    the row offsets), tile experts and tile rows (entries from top_k on stay -1 here: the kernel
    leaves them as they were) and the tile count (top_k).  ids distinct and inside [0, experts).
    """
    ids = np.asarray(ids, np.int32).reshape(-1)
    experts_axis = np.arange(experts)[:, None]
    counts = (ids[None, :] == experts_axis).sum(axis=1).astype(np.int32)
    offsets = (ids[None, :] < experts_axis).sum(axis=1).astype(np.int32)
    tile_expert = np.full(capacity, -1, np.int32)
    tile_row = np.full(capacity, -1, np.int32)
    for expert in ids:
        position = int((ids < expert).sum())
        tile_expert[position] = expert
        tile_row[position] = 0
    return (counts, np.zeros((1, len(ids)), np.int32), offsets, offsets.copy(), tile_expert, tile_row,
            np.array([len(ids)], np.int32))


def expert_partition(counts, hot_m, cold_m, cold_rows, hot_capacity, cold_capacity):
    """Hot / cold tile lists over common row offsets (kernels/cuda/model/expert_partition.py:16-89).

    Experts with more than cold_rows rows get tiles of hot_m rows, the others tiles of cold_m rows.
    Returns a dict of RowOffsets, TileOffsets, TileCount, ColdOffsets, ColdCount and the four tile
    lists (entries past the counts stay -1 here; the kernel leaves them as they were).
    """
    counts = np.asarray(counts, np.int64)
    is_hot = counts > cold_rows
    hot = np.where(is_hot, (counts + hot_m - 1) // hot_m, 0)
    cold = np.where(~is_hot, (counts + cold_m - 1) // cold_m, 0)
    out = {
        "RowOffsets": (np.cumsum(counts) - counts).astype(np.int32),
        "TileOffsets": (np.cumsum(hot) - hot).astype(np.int32),
        "ColdOffsets": (np.cumsum(cold) - cold).astype(np.int32),
        "TileCount": np.array([hot.sum()], np.int32),
        "ColdCount": np.array([cold.sum()], np.int32),
        "TileExpert": np.full(hot_capacity, -1, np.int32), "TileRow": np.full(hot_capacity, -1, np.int32),
        "ColdExpert": np.full(cold_capacity, -1, np.int32), "ColdRow": np.full(cold_capacity, -1, np.int32),
    }
    for e, c in enumerate(counts):
        names, height, base = (("TileExpert", "TileRow"), hot_m, out["TileOffsets"][e]) if is_hot[e] else (
            ("ColdExpert", "ColdRow"), cold_m, out["ColdOffsets"][e])
        for tile in range((int(c) + height - 1) // height):
            out[names[0]][base + tile] = e
            out[names[1]][base + tile] = tile * height
    return out


def tile_capacity(assignments, experts, block_m):
    """ceil(M*k/bm) + min(E, M*k) (moe.py:263-264)."""
    return (assignments + block_m - 1) // block_m + min(experts, assignments)


def expert_dispatch(a_q, a_scale, ids, relative, row_offsets):
    """Copy int8 rows + scales to expert-sorted slots; returns (D, DS, SlotMap) (moe.py:286-329)."""
    m, k = ids.shape
    slot_map = (np.asarray(row_offsets)[ids] + relative).astype(np.int32)
    d = np.zeros((m * k, a_q.shape[1]), np.int8)
    scale = np.asarray(a_scale).reshape(m, -1)
    ds = np.zeros((m * k, scale.shape[1]), np.float16)
    for row in range(m):
        for rank in range(k):
            d[slot_map[row, rank]] = a_q[row]
            ds[slot_map[row, rank]] = scale[row]
    return d, ds, slot_map


def rotate_expert_a8(x, signs, ids=None, relative=None, row_offsets=None, swiglu=False, scatter=True):
    """Rotation + A8 with the routed hand-over of the same launch (rotation_a8.py:452-531, :558-604).

    The row's codes and scale are those of `rotate_a8`.  Without `ids`: (Q, S, Sum) with Sum the
    integer sum of each row's codes (:499, :530).  With routing, slot = RowOffsets[IDs] +
    RelativeSlot (:502, :597): scatter gives (Q, S, D, DS, SlotMap, Sum) with the codes, the scale
    and the sum copied to every slot of the row (:503-510); shared gives (Q, S, DS, SlotMap, Sum)
    with Sum per row (:596-599).  The reference leaves the codes as two planes of unsigned
    nibbles, low = q & 15 and high = (q >> 4) & 15 (:489-491): `nibble_planes` gives those.
    """
    q, s = rotate_a8(x, signs, swiglu)
    total = q.astype(np.int32).sum(axis=1).astype(np.int32)
    if ids is None:
        return q, s, total
    d, ds, slot_map = expert_dispatch(q, s, ids, relative, row_offsets)
    if not scatter:
        return q, s, ds, slot_map, total
    slot_sum = np.zeros(d.shape[0], np.int32)
    slot_sum[slot_map] = total[:, None]
    return q, s, d, ds, slot_map, slot_sum


def nibble_planes(q):
    """int8 codes -> (low, high) unsigned nibbles of the two's-complement byte (rotation_a8.py:489-491)."""
    b = np.asarray(q, np.int8).view(np.uint8)
    return b & 15, b >> 4


# --------------------------------------------------------------------------
# Nibble planes: the A8 hand-over of the reference's INT4 expert kernels
# --------------------------------------------------------------------------
# Nibble i of a plane word holds coordinate PLANE_ORDER[i] of its eight codes
# (kernels/cuda/model/e8p_core.py:63-78, rotation_a8.py:489-491).
PLANE_ORDER = (0, 2, 1, 3, 4, 6, 5, 7)


def split_planes(a_q):
    """int8 (rows, K) -> (Low, High, Sum): u32 (rows, K/8) words and the int32 row sums.

    a = low + 16 * high with low the unsigned and high the signed nibble of the byte
    (kernels/cuda/model/e8p_exact.py:3-4, :18-46); the words take the eight nibbles in
    PLANE_ORDER.  Sum is what the exact kernels add back for w = 2y + 1.
    """
    a_q = np.asarray(a_q, np.int8)
    rows, k = a_q.shape
    b = a_q.view(np.uint8).reshape(rows, k // 8, 8)[:, :, list(PLANE_ORDER)].astype(np.uint32)
    shifts = np.arange(0, 32, 4, dtype=np.uint32)
    low = np.bitwise_or.reduce((b & 15) << shifts, axis=-1).astype(np.uint32)
    high = np.bitwise_or.reduce((b >> 4) << shifts, axis=-1).astype(np.uint32)
    return low, high, a_q.astype(np.int32).sum(axis=1).astype(np.int32)


def planes_group_major(words):
    """(rows, K/8) plane words -> (K/64, rows, 8): K64-major (kernels/cuda/model/e8p_prefill.py:55-56, :79-80)."""
    rows, w = words.shape
    return np.ascontiguousarray(words.reshape(rows, w // 8, 8).transpose(1, 0, 2))


def planes_row_major(words):
    """Inverse of `planes_group_major`."""
    g, rows, _ = words.shape
    return np.ascontiguousarray(words.transpose(1, 0, 2)).reshape(rows, g * 8)


def planes_values(low, high):
    """(rows, K/8) words -> int64 (rows, K) values low_u4 + 16 * high_s4 in K order."""
    shifts = np.arange(0, 32, 4, dtype=np.uint32)
    lo = ((np.asarray(low, np.uint32)[..., None] >> shifts) & 15).astype(np.int64)
    hi = ((np.asarray(high, np.uint32)[..., None] >> shifts) & 15).astype(np.int64)
    hi = np.where(hi >= 8, hi - 16, hi)
    inverse = np.argsort(PLANE_ORDER)
    return (lo + 16 * hi)[..., inverse].reshape(low.shape[0], low.shape[1] * 8)


def nibble_table(selectors):
    """Selector words -> words of signed nibbles (w - 1) / 2 at even parity, in PLANE_ORDER.

    python/orinfer_build/quantization/vq.py:105-118 (and `direct_nibble_basis`,
    kernels/cuda/model/e8p_core.py:45-60): id 0..2 are +1, +3, +5, id 4..6 their negatives;
    zero coordinates (id 3, 7) have no nibble form and are refused.
    """
    sel = np.asarray(selectors, np.uint32).reshape(-1)
    shifts = np.arange(0, 32, 4, dtype=np.uint32)
    ids = (sel[:, None] >> shifts) & 7
    if np.any((ids & 3) == 3) or np.any(sel & np.uint32(0x88888888)):
        raise ValueError("the nibble form needs a nonzero spread29 basis")
    half = np.array([1, 3, 5, 0, -1, -3, -5, 0], np.int32)[ids]
    words = np.bitwise_or.reduce((half[:, list(PLANE_ORDER)] & 15).astype(np.uint32) << shifts, axis=1)
    return words.astype(np.uint32).reshape(-1, 1)


def nibble_decode(codes, nibbles):
    """u16 codes -> int64 (..., 8) values y = (w - 1) / 2 in K order, from a nibble table.

    kernels/cuda/model/e8p_core.py:7-10: sign bit SIGN_BITS[j] negates coordinate j's nibble
    (xor 0xe: the stored values are odd), odd parity lowers every nibble by one (xor 1) and
    flips the first coordinate's sign as well.
    """
    codes = np.asarray(codes, np.uint16).astype(np.uint32)
    book = np.asarray(nibbles, np.uint32).reshape(-1)[codes >> 8]
    low = codes & 255
    parity = np.zeros_like(low)
    for bit in range(8):
        parity ^= (low >> bit) & 1
    out = np.empty(codes.shape + (8,), np.int64)
    for position, coordinate in enumerate(PLANE_ORDER):
        nib = (book >> np.uint32(4 * position)) & 15
        flip = (low >> SIGN_BITS[coordinate]) & 1
        nib = nib ^ (flip * 0xE) ^ parity
        if position == 0:
            nib = nib ^ (parity * 0xE)
        out[..., coordinate] = np.where(nib >= 8, nib.astype(np.int64) - 16, nib.astype(np.int64))
    return out


def plane_project(low, high, total, half_weights, weight_scale, token_scale, coefficient_sum=1):
    """Out = rescale(2 * sum_k y[n, k] * (low + 16 high)[m, k] + coefficient_sum * Sum[m]).

    kernels/cuda/model/e8p_core.py:173-189 (single-stage, coefficient_sum 1) and :154-170
    (two-stage: y = 4 y_coarse + y_fine, coefficient_sum 5); `total` is taken as given, as
    the kernels take their Sum argument.  Integer arithmetic wraps at 32 bits as theirs does.
    """
    a = planes_values(low, high)
    acc = a @ np.asarray(half_weights, np.int64).T
    value = 2 * acc + coefficient_sum * np.asarray(total, np.int64)[:, None]
    value = ((value + 2**31) % 2**32 - 2**31).astype(np.int32)
    return rescale(value, weight_scale, token_scale)


def dispatch_planes(a_q, a_scale, ids, relative, row_offsets):
    """A8 rows -> K64-major planes at their routed slots (kernels/cuda/model/e8p_prefill.py:565-622).

    Returns (Low, High, Sum, DS, SlotMap) with slot = RowOffsets[IDs] + RelativeSlot.
    """
    m, top_k = ids.shape
    low, high, total = split_planes(a_q)
    slot_map = (np.asarray(row_offsets)[ids] + relative).astype(np.int32)
    slots = m * top_k
    out_low = np.zeros((slots, low.shape[1]), np.uint32)
    out_high = np.zeros_like(out_low)
    out_sum = np.zeros(slots, np.int32)
    ds = np.zeros((slots, 1), np.float16)
    scale = np.asarray(a_scale, np.float16).reshape(m)
    for row in range(m):
        for rank in range(top_k):
            slot = slot_map[row, rank]
            out_low[slot], out_high[slot], out_sum[slot], ds[slot, 0] = low[row], high[row], total[row], scale[row]
    return planes_group_major(out_low), planes_group_major(out_high), out_sum, ds, slot_map


def moe_combine(expert_out, slot_map, prob, shared=None, shared_gate=None):
    """out = sum_rank fp32(Expert[slot])*prob (+ sigmoid(gate)*shared), one fp16 cast (moe.py:498-554).

    fp32 accumulation in rank order; slots < 0 or >= slots are skipped.
    """
    expert_out = np.asarray(expert_out)
    slots = expert_out.shape[0]
    m, k = slot_map.shape
    acc = np.zeros((m, expert_out.shape[1]), np.float32)
    for rank in range(k):
        s = slot_map[:, rank]
        ok = (s >= 0) & (s < slots)
        rows = expert_out[np.clip(s, 0, slots - 1)].astype(np.float32)
        term = (rows * np.asarray(prob, np.float32)[:, rank : rank + 1]).astype(np.float32)
        acc = np.where(ok[:, None], (acc + term).astype(np.float32), acc)
    if shared is not None:
        gate = np.asarray(shared_gate).astype(np.float32)
        sig = (np.float32(1.0) / (np.float32(1.0) + np.exp(-gate).astype(np.float32))).astype(np.float32)
        acc = (acc + sig[:, None] * np.asarray(shared).astype(np.float32)).astype(np.float32)
    return acc.astype(np.float16)


def grouped_project(d, ds, weights_int8, weight_scales, counts, row_offsets):
    """Per-expert project over the sorted rows (integer_vq.py:205-214 epilogue)."""
    out = np.zeros((d.shape[0], weights_int8.shape[1]), np.float16)
    for e, c in enumerate(np.asarray(counts)):
        if c:
            lo = int(row_offsets[e])
            out[lo : lo + c] = project(d[lo : lo + c], ds[lo : lo + c, 0], weights_int8[e], weight_scales[e])
    return out


def route_project(a_q, a_scale, weights_int8, weight_scales, ids, shared_input):
    """Single-token expert routes: C[route] = project(A[row], W[ids[route]]) (integer_vq.py:380-444).

    Every route indexes its expert's bank directly; row = 0 when all routes share one token row,
    else row = route.  Same int32 dot and rescale as every other projection here.
    """
    ids = np.asarray(ids).reshape(-1)
    a_q = np.asarray(a_q)
    scale = np.asarray(a_scale).reshape(-1)
    out = np.zeros((len(ids), weights_int8.shape[1]), np.float16)
    for route, expert in enumerate(ids):
        row = 0 if shared_input else route
        acc = int_dot(a_q[row : row + 1], weights_int8[expert])
        out[route] = rescale(acc, weight_scales[expert], scale[row : row + 1])[0]
    return out


def raw_table_words(table):
    """The 256x8 int8 table as (256, 2) u32, the Book of the raw-basis kernels (vq.py:203)."""
    return np.ascontiguousarray(np.asarray(table, np.int8)).view("<u4").reshape(256, 2)


def moe_layer(x, logits, gate_up_codes, gate_up_scales, down_codes, down_scales, table, top_k, block_m=16, signs=None):
    """Whole Q2A8 expert layer in the reference's program order
    (tests/cuda/operators/flash_next_quantized.py:117-135; kernels/cuda/model/moe.py):
    top-k -> histogram/offsets -> A8 -> dispatch -> grouped gate_up -> SwiGLU fp16 -> A8 ->
    grouped down -> weighted combine.

    gate_up_codes u16 [E, 2I, H/8], down_codes u16 [E, H, I/8] (row-major per expert).
    `signs`: the input is rotated before the A8 (rotation_a8.py:558-604).
    Returns a dict of every intermediate so kernels can be checked stage by stage.
    """
    e = gate_up_codes.shape[0]
    ids, prob = router_topk(logits, top_k, True)
    counts, relative = expert_histogram(ids, e)
    row_offsets, tile_offsets, tile_count = expert_offsets(counts, block_m)
    a_q, a_s = a8(x) if signs is None else rotate_a8(x, signs)
    d, ds, slot_map = expert_dispatch(a_q, a_s, ids, relative, row_offsets)
    w1 = np.stack([q2_integers(gate_up_codes[i], table) for i in range(e)])
    w2 = np.stack([q2_integers(down_codes[i], table) for i in range(e)])
    gu = grouped_project(d, ds, w1, gate_up_scales, counts, row_offsets)
    act = swiglu_fp16(gu)
    h_q, h_s = a8(act)
    dn = grouped_project(h_q, h_s, w2, down_scales, counts, row_offsets)
    out = moe_combine(dn, slot_map, prob)
    return dict(ids=ids, prob=prob, counts=counts, relative=relative, row_offsets=row_offsets,
                tile_offsets=tile_offsets, tile_count=tile_count, a_q=a_q, a_s=a_s, d=d, ds=ds,
                slot_map=slot_map, gate_up=gu, act=act, h_q=h_q, h_s=h_s, down=dn, out=out)
