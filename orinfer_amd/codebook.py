"""Host-side E8P codebook data and weight layouts (numpy only; no device code).

What the engine would load from a package: the 256x8 int8 basis
(python/orinfer_build/quantization/e8p.py:15-25), the (256,1) u32 selector table it binds as
`Book` (quantization/vq.py:74-93, models/qwen35/build.py:385-389) and the K-major physical
layouts of the code tensors (models/qwen35/storage.py:56-81, quantization/vq.py:199-204).
"""
import itertools

import numpy as np


def basis():
    """The 256 E8P basis rows: 227 inner magnitude patterns, 29 spread outer patterns."""
    rows = []
    for pattern in itertools.product((2, 6, 10), repeat=8):
        if sum(v * v for v in pattern) <= 160:
            rows.append(list(pattern))
    five_sets = list(itertools.combinations(range(8), 5))
    for i in range(29):
        row = [2] * 8
        for j in five_sets[i * 56 // 29]:
            row[j] = 6
        rows.append(row)
    table = np.asarray(rows, np.int32)
    odd = (table.sum(1) // 4) % 2 == 1
    table[odd, 7] *= -1
    if table.shape != (256, 8):
        raise AssertionError("E8P basis must have 256 rows")
    return table.astype(np.int8)


def selector_table(table):
    """(256,1) u32: nibble j = {2:0, 6:1, 10:2, 0:3}[|t_j|] | 4*(t_j < 0)."""
    t = np.asarray(table)
    if t.dtype != np.int8 or t.shape != (256, 8):
        raise ValueError("expected the int8 [256,8] basis")
    magnitude = np.abs(t.astype(np.int32))
    if not np.isin(magnitude, (0, 2, 6, 10)).all():
        raise ValueError("E8P selector decoder requires values in {0, +-2, +-6, +-10}")
    ident = np.where(magnitude == 0, 3, (magnitude - 2) // 4) | ((t < 0) * 4)
    shifts = (4 * np.arange(8)).astype(np.uint32)
    return (ident.astype(np.uint32) << shifts).sum(1, dtype=np.uint32).reshape(256, 1)


def book():
    """Selector table of the production basis: the `Book` buffer of every E8P kernel."""
    return selector_table(basis())


def nibble_book(table=None):
    """(1, 256, 1) u32 nibble words, the `Book` of `e8p_exact_grouped` and of `e8p_prefill_grouped` with single-stage
    codes: nibble i = (t_j / 2) & 15 for j = [0, 2, 1, 3, 4, 6, 5, 7][i] (python/orinfer_build/quantization/vq.py:105-118).
    Needs a basis without zeros."""
    t = np.asarray(basis() if table is None else table)
    if t.dtype != np.int8 or t.shape != (256, 8) or not np.isin(np.abs(t.astype(np.int32)), (2, 6, 10)).all():
        raise ValueError("the nibble form needs the int8 [256,8] basis with entries of +-2, +-6, +-10")
    half = (t.astype(np.int32) // 2)[:, [0, 2, 1, 3, 4, 6, 5, 7]] & 15
    shifts = np.arange(0, 32, 4, dtype=np.uint32)
    return np.bitwise_or.reduce(half.astype(np.uint32) << shifts, axis=1).astype(np.uint32).reshape(1, 256, 1)


def q2_to_k64(blocks):
    """(E, K/128, N, 16) u16 -> (E, K/64, N, 8): the K-major blocks of 64 the plane kernels read (vq.py:121-128)."""
    e, g, n, _ = blocks.shape
    return np.ascontiguousarray(blocks.reshape(e, g, n, 2, 8).transpose(0, 1, 3, 2, 4)).reshape(e, g * 2, n, 8)


def raw_book(table=None):
    """The 256 x 8 int8 table as (256, 2) u32 words: the `Book` of the raw-table kernels
    (`integer_e8p_gemv`; python/orinfer_build/quantization/vq.py:203)."""
    table = basis() if table is None else np.asarray(table, np.int8)
    return np.ascontiguousarray(table).view("<u4").reshape(256, 2)


def q4_to_k_major(packed, packed_k=128):
    """(N, K/8) u32 -> (K/packed_k, N, packed_k/8), tag e8p-q4-k128-u32."""
    n, vectors = packed.shape
    per = packed_k // 8
    return np.ascontiguousarray(packed.reshape(n, vectors // per, per).transpose(1, 0, 2))


def q2_to_k_major(indices):
    """(E, N, K/8) u16 -> (E, K/128, N, 16)."""
    e, n, vectors = indices.shape
    return np.ascontiguousarray(indices.reshape(e, n, vectors // 16, 16).transpose(0, 2, 1, 3))
