"""Seeded synthetic inputs for the five benchmark configurations (numpy only).

RNG: numpy.random.default_rng(20261002 + config index); the seed value is the reference's
universal SEED (python/orinfer_build/compiler/cuda/common.py:18).  Draw order inside each
generator is fixed and is the order of the statements below; changing it changes every
fixture.  Shapes default to the full benchmark sizes and can be shrunk for tests.
"""
import numpy as np

SEED = 20261002


def _activations(rng, rows, k, outlier_channels=False):
    """fp16 ~N(0,1) with 0.1 % outliers x20 (entries, or whole channels for the layer config)."""
    x = rng.standard_normal((rows, k), dtype=np.float32)
    if outlier_channels:
        count = max(1, k // 1000)
        x[:, rng.choice(k, count, replace=False)] *= 20.0
    else:
        count = max(1, (rows * k) // 1000)
        flat = rng.choice(rows * k, count, replace=False)
        x.reshape(-1)[flat] *= 20.0
    return x.astype(np.float16)


def _codes_u32(rng, n, k):
    return rng.integers(0, 2**32, (n, k // 8), dtype=np.uint32)


def _scales(rng, shape, low, high):
    return rng.uniform(low, high, shape).astype(np.float16)


def q4_linear(config_index, rows, n, k, outlier_channels=False):
    """x fp16 [rows,k]; packed u32 [n,k/8] (low half coarse, high half residual); S fp16 [n]."""
    rng = np.random.default_rng(SEED + config_index)
    x = _activations(rng, rows, k, outlier_channels)
    packed = _codes_u32(rng, n, k)
    scales = _scales(rng, n, 0.005, 0.02)
    return dict(x=x, packed=packed, scales=scales, rows=rows, n=n, k=k)


def config0(n=9728, k=2560):
    """Single E8P two-stage Q4A8 linear, batch-1 decode GEMV."""
    return q4_linear(0, 1, n, k)


def config1(rows, n=17408, k=5120):
    """Q4A8 at a larger projection; rows in {1, 8, 32, 128, 512}.  The weights do not depend on
    `rows`: activations are drawn for 512 rows and the first `rows` are used."""
    full = q4_linear(1, 512, n, k)
    full["x"] = full["x"][:rows]
    full["rows"] = rows
    return full


def config2(rows=8192, n=4096, k=4096):
    """W8A8 prefill GEMM: int8 weights in [-127,127], WS ~U(0.001,0.01)."""
    rng = np.random.default_rng(SEED + 2)
    weight = rng.integers(-127, 128, (n, k), dtype=np.int8)
    scales = _scales(rng, n, 0.001, 0.01)
    x = rng.standard_normal((rows, k), dtype=np.float32).astype(np.float16)
    return dict(x=x, weight=weight, scales=scales, rows=rows, n=n, k=k)


def config3(tokens=256, experts=128, top_k=8, hidden=2048, intermediate=512):
    """MoE layer with single-stage Q2A8 experts and Zipf(1.1)-skewed routing."""
    rng = np.random.default_rng(SEED + 3)
    x = rng.standard_normal((tokens, hidden), dtype=np.float32).astype(np.float16)
    order = rng.permutation(experts)
    bias = np.empty(experts, np.float32)
    bias[order] = -1.1 * np.log(np.arange(1, experts + 1, dtype=np.float32))
    logits = (rng.standard_normal((tokens, experts), dtype=np.float32) + bias[None, :]).astype(np.float32)
    gate_up = rng.integers(0, 65536, (experts, 2 * intermediate, hidden // 8), dtype=np.uint16)
    down = rng.integers(0, 65536, (experts, hidden, intermediate // 8), dtype=np.uint16)
    gate_up_scales = _scales(rng, (experts, 2 * intermediate), 0.005, 0.02)
    down_scales = _scales(rng, (experts, hidden), 0.005, 0.02)
    return dict(x=x, logits=logits, gate_up=gate_up, down=down, gate_up_scales=gate_up_scales,
                down_scales=down_scales, tokens=tokens, experts=experts, top_k=top_k, hidden=hidden,
                intermediate=intermediate)


LAYER_PROJECTIONS = (  # name, codec, N, K at 27B-class shapes
    ("qkv", "q4", 7168, 5120),
    ("o", "q4", 5120, 5120),
    ("gate_up", "q4", 34816, 5120),
    ("down", "w8", 5120, 17408),
)


def config4(rows=8192, shrink=1):
    """One decoder layer's quantized projections; activations have 0.1 % outlier channels x20.
    `shrink` divides every N (tests); K keeps its real value."""
    rng = np.random.default_rng(SEED + 4)
    out = {}
    for name, codec, n, k in LAYER_PROJECTIONS:
        n //= shrink
        x = _activations(rng, rows, k, outlier_channels=True)
        if codec == "q4":
            out[name] = dict(codec=codec, x=x, packed=_codes_u32(rng, n, k), scales=_scales(rng, n, 0.005, 0.02),
                             rows=rows, n=n, k=k)
        else:
            out[name] = dict(codec=codec, x=x, weight=rng.integers(-127, 128, (n, k), dtype=np.int8),
                             scales=_scales(rng, n, 0.001, 0.01), rows=rows, n=n, k=k)
    return out


def algorithmic_bytes_q4(rows, n, k):
    """codes + weight scales + int8 activations + token scales + fp16 output + 1 KiB LUT."""
    return n * (k // 8) * 4 + n * 2 + rows * k + rows * 2 + rows * n * 2 + 1024


def algorithmic_bytes_w8(rows, n, k):
    return n * k + n * 2 + rows * k + rows * 2 + rows * n * 2


def algorithmic_ops(rows, n, k):
    return 2 * rows * n * k
