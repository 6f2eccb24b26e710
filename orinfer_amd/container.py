"""Weight containers and package records for the quantized linear path (host side, numpy only).

Two things the engine's packaging layer does for this path:

* the E8P two-stage weight container `orinfer-e8p-q4-v1`: a safetensors file with tensors
  `packed` (N, K/8) u32, `scales` (N) f16, `signs` (K) i8, `basis` (256, 8) i8 and metadata
  `codec`, `coefficients`, `layout`, `rotation`
  (python/orinfer_build/quantization/e8p_q4.py:33-58 validation, :80-112 save/load);
* `Kernel` records: one launch of one symbol with ordered arguments
  (crates/orinfer-model-sdk/src/artifact.rs:87-110, arguments :176-186, buffers :60-72), named by
  the row-specialisation rule `slot/rows/MIN-MAX`
  (crates/orinfer-model-sdk/src/operators/rows.rs:14-58).

A record has no field for a variant, so the symbol carries it
(`family?M=1&N=9728&K=2560`), which `orx_resolve` accepts.
"""
import hashlib
import json
from dataclasses import dataclass
from pathlib import Path

import numpy as np

from . import codebook, lib

CODEC = "orinfer-e8p-q4-v1"
LAYOUT = "u32-low-coarse-high-residual"
ROTATION = "signed-block128"
COEFFICIENTS = (4, 1)

_DTYPES = {np.dtype(np.uint8): "u8", np.dtype(np.int8): "i8", np.dtype(np.uint16): "u16", np.dtype(np.float16): "f16",
           np.dtype(np.float32): "f32", np.dtype(np.float64): "f64", np.dtype(np.uint32): "u32", np.dtype(np.int32): "i32",
           np.dtype(np.uint64): "u64", np.dtype(np.int64): "i64"}


@dataclass
class Q4Weights:
    """One two-stage E8P matrix: row-major codes, one scale per output row, one sign per input."""
    packed: np.ndarray   # (N, K/8) u32, low half coarse code, high half residual code
    scales: np.ndarray   # (N,) f16
    signs: np.ndarray    # (K,) i8, +-1: the rotation the activations must undergo

    def validate(self):
        p, s, g = self.packed, self.scales, self.signs
        if p.dtype != np.uint32 or p.ndim != 2 or min(p.shape) <= 0 or (p.shape[1] * 8) % 128:
            raise ValueError("E8P-Q4 codes must be (N, K/8) uint32 with K a multiple of 128")
        n, k = p.shape[0], p.shape[1] * 8
        if s.dtype != np.float16 or s.shape != (n,) or not np.isfinite(s).all() or (s <= 0).any():
            raise ValueError("E8P-Q4 scales must be N positive finite float16 values")
        if g.dtype != np.int8 or g.shape != (k,) or not np.isin(g, (-1, 1)).all():
            raise ValueError("E8P-Q4 signs must be K int8 values of +-1")
        return n, k

    def k_major(self, packed_k=128):
        """(K/packed_k, N, packed_k/8) u32, tag e8p-q4-k128-u32 (models/qwen35/storage.py:56-81)."""
        return codebook.q4_to_k_major(self.packed, packed_k)


def save_q4(path, weights):
    from safetensors.numpy import save_file

    weights.validate()
    save_file(dict(packed=weights.packed, scales=weights.scales, signs=weights.signs, basis=codebook.basis()), str(path),
              metadata=dict(codec=CODEC, coefficients=",".join(map(str, COEFFICIENTS)), layout=LAYOUT, rotation=ROTATION))


def load_q4(path):
    """Reads a container; refuses any codec, layout, rotation, coefficient or basis it does not implement."""
    from safetensors import safe_open

    with safe_open(str(path), framework="numpy") as source:
        metadata = source.metadata() or {}
        if (metadata.get("codec") != CODEC or metadata.get("layout") != LAYOUT or metadata.get("rotation") != ROTATION
                or set(source.keys()) != {"packed", "scales", "signs", "basis"}):
            raise ValueError("E8P-Q4 codec contract mismatch")
        if not np.array_equal(source.get_tensor("basis"), codebook.basis()):
            raise ValueError("E8P-Q4 basis differs from the one the kernels decode")
        coefficients = tuple(int(v) for v in metadata.get("coefficients", "").split(",") if v)
        if coefficients != COEFFICIENTS:
            raise ValueError(f"E8P-Q4 coefficients {coefficients}: the kernels implement {COEFFICIENTS}")
        weights = Q4Weights(source.get_tensor("packed"), source.get_tensor("scales"), source.get_tensor("signs"))
    weights.validate()
    return weights


# ---- package records -------------------------------------------------------------------------
def file_identity(path):
    data = Path(path).read_bytes()
    return {"file": Path(path).name, "sha256": hashlib.sha256(data).hexdigest()}


def buffer_record(name, array=None, *, dtype=None, shape=None, layout="row-major", access="read", data=None,
                  alignment=256):
    """`Buffer` of artifact.rs:60-72.  Either an array (dtype and shape are taken from it) or both."""
    if array is not None:
        dtype, shape = _DTYPES[np.asarray(array).dtype], list(np.asarray(array).shape)
    if access not in ("read", "write", "read_write"):
        raise ValueError("access must be read, write or read_write")
    return {"name": name, "dtype": dtype, "shape": list(shape), "layout": layout, "alignment": alignment,
            "access": access, "data": data}


def symbol_with_variant(family, **variant):
    def text(value):
        return "true" if value is True else "false" if value is False else str(value)
    return family + "?" + "&".join(f"{key}={text(value)}" for key, value in variant.items()) if variant else family


def kernel_record(name, family, variant, bindings, rows=0):
    """`Kernel` of artifact.rs:87-110 for one launch of `family` with `variant`.

    bindings: argument name -> buffer name | (buffer name, byte offset) | int (scalar).  The grid,
    block and LDS bytes are the library's own for `rows` live rows (0 = the variant's M)."""
    # An optional buffer that this program does not use (bound to None) leaves the argument list through the
    # variant's `omit` key: the record's arguments stay within the engine's `Argument` kinds (artifact.rs:184-194).
    unused = [arg_name for arg_name, bound in bindings.items() if bound is None]
    if unused:
        variant = dict(variant, omit=",".join(sorted(unused)))
    kernel = lib.Kernel(family, **variant)
    grid, block, shared = kernel.geometry(rows)
    args = []
    for arg_name, kind in zip(kernel.arg_names, kernel.arg_kinds):
        if arg_name not in bindings:
            raise KeyError(f"{family}: no binding for argument {arg_name}")
        bound = bindings[arg_name]
        if kind == 1:
            args.append({"kind": "i32", "value": int(bound)})
        elif isinstance(bound, tuple):
            args.append({"kind": "buffer_slice", "name": bound[0], "offset": int(bound[1])})
        else:
            args.append({"kind": "buffer", "name": bound})
    root = Path(__file__).resolve().parent
    return {
        "name": name,
        "module": file_identity(lib.LIBRARY_PATH),
        "source": file_identity(root / "csrc" / "orx_api.cpp"),
        "host_abi": file_identity(root.parent / "include" / "orx.h"),
        "symbol": symbol_with_variant(family, **variant),
        "grid": list(grid), "block": list(block), "shared_memory_bytes": shared, "cooperative": False,
        "args": args,
    }


# ---- dynamic-row launch contracts (crates/orinfer-model-sdk/src/operators/dynamic.rs:5-118) ---------
def _constant(value):
    return {"op": "constant", "value": int(value)}


def _ceil_div_rows(divisor):
    return {"op": "divide", "lhs": {"op": "add", "lhs": {"op": "rows"}, "rhs": _constant(divisor - 1)},
            "rhs": _constant(divisor)}


def evaluate_rows(expression, rows):
    """RowExpression::evaluate (dynamic.rs:27-64): checked u32 arithmetic over the live row count."""
    op = expression["op"]
    if op == "constant":
        return int(expression["value"])
    if op == "rows":
        return int(rows)
    a, b = evaluate_rows(expression["lhs"], rows), evaluate_rows(expression["rhs"], rows)
    if op in ("divide", "remainder") and b == 0:
        raise ValueError("Invalid row expression arithmetic")
    value = {"add": a + b, "subtract": a - b, "multiply": a * b, "divide": a // b if b else 0,
             "remainder": a % b if b else 0, "minimum": min(a, b)}[op]
    if not 0 <= value < 2**32:
        raise ValueError("Invalid row expression arithmetic")
    return value


def _fit_rows(values):
    """A RowExpression that gives values[rows] for every key of `values`, or None: a constant,
    c * ceil(rows / d), min(cap, c * ceil(rows / d)) (persistent workgroups), or
    min(cap, c * ceil(rows / d) / 8) (the workgroups of a split launch)."""
    rows = sorted(values)
    if len({values[r] for r in rows}) == 1:
        return _constant(values[rows[0]])
    for d in (32, 64, 128, 256):
        tiles = {r: -(-r // d) for r in rows}
        if all(values[r] % tiles[r] == 0 for r in rows) and len({values[r] // tiles[r] for r in rows}) == 1:
            c = values[rows[0]] // tiles[rows[0]]
            expr = _ceil_div_rows(d) if c == 1 else {"op": "multiply", "lhs": _constant(c), "rhs": _ceil_div_rows(d)}
            return expr
    cap = max(values.values())
    # min(cap, c * ceil(rows / d)): persistent workgroups, one per tile up to one per compute unit
    for d in (32, 64, 128, 256):
        tiles = {r: -(-r // d) for r in rows}
        below = [r for r in rows if values[r] < cap]
        if below and values[below[0]] % tiles[below[0]] == 0:
            c = values[below[0]] // tiles[below[0]]
            if all(values[r] == min(cap, c * tiles[r]) for r in rows):
                return {"op": "minimum", "lhs": _constant(cap),
                        "rhs": {"op": "multiply", "lhs": _constant(c), "rhs": _ceil_div_rows(d)}}
    for d in (128,):
        below = [r for r in rows if values[r] < cap]
        if not below:
            continue
        r0 = below[0]
        for c in range(values[r0] * 8 // -(-r0 // d), (values[r0] + 1) * 8 // -(-r0 // d) + 1):
            expr = {"op": "minimum", "lhs": _constant(cap),
                    "rhs": {"op": "divide", "lhs": {"op": "multiply", "lhs": _constant(c), "rhs": _ceil_div_rows(d)},
                            "rhs": _constant(8)}}
            if all(evaluate_rows(expr, r) == values[r] for r in rows):
                return expr
    return None


def projection_program(slot, n, k, capacity, *, family="e8p_q4_projection", bindings=None, workspace=True, **extra):
    """Row-specialised records of one projection slot under the naming rule `slot/rows/MIN-MAX`
    (crates/orinfer-model-sdk/src/operators/rows.rs:14-58), each a separately resolvable symbol.

    The library picks a kernel by the live row count, and kernels differ in block size and LDS
    bytes.  A `Kernel` record fixes block and shared memory and a `DynamicBatchKernel` varies only the
    grid and the `m` scalar (dynamic.rs:74-118), so the row domain 1..capacity is cut wherever block
    or LDS bytes change, and further wherever the grid stops being one RowExpression of the rows.
    Every range is checked row by row against the library's own geometry before it is emitted.
    Returns {"kernels": [Kernel...], "dynamic": [DynamicBatchKernel...]} (ranges of one row count have
    no dynamic entry: their grid is static)."""
    def handle(top):
        variant = dict(M=top, N=n, K=k, dynamic_rows=True, **extra)
        if workspace:
            variant["workspace"] = True
        return variant, lib.Kernel(family, **variant)

    _, whole = handle(capacity)
    kernels, dynamic = [], []
    low = 1
    while low <= capacity:
        block, shared = whole.geometry(low)[1:]
        high = low
        while high < capacity and whole.geometry(high + 1)[1:] == (block, shared):
            high += 1
        # the record of a range is resolved at the top of the range: its own dispatch must agree, and the
        # grid over the range must be one expression per dimension; take the longest range for which both hold
        def attempt(top):
            variant, kernel = handle(top)
            geometry = {r: kernel.geometry(r) for r in range(low, top + 1)}
            if not all(g[1:] == (block, shared) for g in geometry.values()):
                return None
            fits = [_fit_rows({r: g[0][d] for r, g in geometry.items()}) for d in range(3)]
            return (variant, kernel, fits) if all(f is not None for f in fits) else None

        found = attempt(high)
        if found is None:
            good, bad = low, high  # a single row count always fits (constants)
            while bad - good > 1:
                middle = (good + bad) // 2
                if attempt(middle) is not None:
                    good = middle
                else:
                    bad = middle
            high, found = good, attempt(good)
        variant, kernel, fits = found
        names = kernel.arg_names
        bound = dict(bindings or {a: a for a in names})
        bound["m"] = high
        name = f"{slot}/rows/{low}-{high}"
        kernels.append(kernel_record(name, family, variant, bound, rows=high))
        if high > low:
            dynamic.append({"name": name, "capacity": high, "grid": fits,
                            "arguments": [{"index": names.index("m"), "value": {"op": "rows"}}]})
        low = high + 1
    return {"kernels": kernels, "dynamic": dynamic}


def projection_records(slot, n, k, capacity, **options):
    """The `Kernel` records of projection_program()."""
    return projection_program(slot, n, k, capacity, **options)["kernels"]


def expert_layer_program(slot, tokens, experts, top_k, hidden, intermediate, *, block_m=32, packed_k=128,
                         grouped_algorithm="auto", buffers=None):
    """The routed Q2A8 expert layer as five `Kernel` records in launch order (the program of
    `programs.MoeLayer` where the resident expert kernel applies): router top-k that also quantises
    the token rows, routing metadata with the slot tables, gate_up (rows gathered by slot, SwiGLU
    epilogue), down (fp16 rows quantised while staged), weighted combine.

    buffers: overrides of the default buffer names, which are the argument names prefixed where two
    launches would collide (`GateUpCodes`/`DownCodes`, `GateUpScales`/`DownScales`, ...).  Returns the
    records and a dict name -> byte size of every buffer the program touches."""
    assignments = tokens * top_k
    tiles = (assignments + block_m - 1) // block_m + min(experts, assignments)
    common = dict(M=tokens, E=experts, top_k=top_k)
    grouped = dict(rows=assignments, E=experts, tiles=tiles, block_m=block_m, packed_k=packed_k,
                   algorithm=grouped_algorithm)
    name = dict(buffers or {})
    b = lambda key: name.get(key, key)
    routed = dict(Book=b("Book"), Counts=b("Counts"), Offsets=b("RowOffsets"), TileCount=b("TileCount"),
                  TileExpert=b("TileExpert"), TileRow=b("TileRow"))
    records = [
        kernel_record(f"{slot}.router", "router_topk", dict(renormalize=True, quantize_hidden=hidden, **common),
                      dict(IDs=b("IDs"), Logits=b("Logits"), Prob=b("Prob"), Q=b("A8"), S=b("A8Scale"), X=b("X"))),
        kernel_record(f"{slot}.metadata", "route_metadata", dict(block_m=block_m, slot_maps=True, **common),
                      dict(Counts=b("Counts"), IDs=b("IDs"), RelativeSlot=b("RelativeSlot"), RowMax=b("RowMax"),
                           RowOffsets=b("RowOffsets"), SlotMap=b("SlotMap"), SlotToken=b("SlotToken"),
                           TileCount=b("TileCount"), TileExpert=b("TileExpert"), TileOffsets=b("TileOffsets"),
                           TileRow=b("TileRow"))),
        kernel_record(f"{slot}.gate_up", "e8p_decode_grouped",
                      dict(N=2 * intermediate, K=hidden, gather=True, epilogue="swiglu", **grouped),
                      dict(A=b("A8"), AS=b("A8Scale"), Act=b("Act"), C=None, P=b("GateUpCodes"), RowMax=b("RowMax"),
                           SlotToken=b("SlotToken"), WS=b("GateUpScales"), **routed)),
        kernel_record(f"{slot}.down", "e8p_decode_grouped",
                      dict(N=hidden, K=intermediate, input_dtype="float16", **grouped),
                      dict(A=b("Act"), AS=None, C=b("ExpertOut"), P=b("DownCodes"), Q=None, RowMax=b("RowMax"),
                           WS=b("DownScales"), **routed)),
        kernel_record(f"{slot}.combine", "moe_combine", dict(H=hidden, slots=assignments, **common),
                      dict(Expert=b("ExpertOut"), Output=b("Output"), Prob=b("Prob"), Shared=None, SharedGate=None,
                           SlotMap=b("SlotMap"))),
    ]
    sizes = {
        b("X"): tokens * hidden * 2, b("Logits"): tokens * experts * 4, b("IDs"): assignments * 4,
        b("Prob"): assignments * 4, b("A8"): tokens * hidden, b("A8Scale"): tokens * 2, b("Counts"): experts * 4,
        b("RelativeSlot"): assignments * 4, b("RowMax"): assignments * 4, b("RowOffsets"): experts * 4,
        b("SlotMap"): assignments * 4, b("SlotToken"): assignments * 4, b("TileCount"): 4, b("TileExpert"): tiles * 4,
        b("TileOffsets"): experts * 4, b("TileRow"): tiles * 4, b("Act"): assignments * intermediate * 2,
        b("ExpertOut"): assignments * hidden * 2, b("Output"): tokens * hidden * 2, b("Book"): 1024,
        b("GateUpCodes"): experts * 2 * intermediate * hidden // 4, b("DownCodes"): experts * hidden * intermediate // 4,
        b("GateUpScales"): experts * 2 * intermediate * 2, b("DownScales"): experts * hidden * 2,
    }
    return records, sizes


def exact_expert_program(slot, rows, experts, top_k, n, k, *, block_m=8, stages=4, warp_private=True, buffers=None):
    """One routed expert projection on nibble planes as the reference's decode programs record it
    (python/orinfer_build/models/flash_next/expert_decode.py:23-75: `e8p_exact_grouped` with 8-row tiles behind the
    split of the A8 rows): `split_a8` writes Low / High / Sum, `e8p_exact_grouped` multiplies them with the
    K-major blocks of 64 (`codebook.q2_to_k64`) and the nibble Book (`codebook.nibble_book`).

    rows: token rows; the projection sees rows * top_k routed rows.  Returns the two records and a dict
    name -> byte size of every buffer they touch."""
    slots = rows * top_k
    tiles = (slots + block_m - 1) // block_m + min(experts, slots)
    name = dict(buffers or {})
    b = lambda key: name.get(key, key)
    records = [
        kernel_record(f"{slot}.split", "split_a8", dict(rows=slots, K=k),
                      dict(A=b("A"), High=b("High"), Low=b("Low"), Sum=b("Sum"))),
        kernel_record(f"{slot}.project", "e8p_exact_grouped",
                      dict(rows=slots, E=experts, tiles=tiles, N=n, K=k, block_m=block_m, stages=stages,
                           warp_private=warp_private),
                      dict(AS=b("AS"), Book=b("Book"), Counts=b("Counts"), High=b("High"), Low=b("Low"), Offsets=b("Offsets"),
                           Out=b("Out"), P=b("P"), Sum=b("Sum"), TC=b("TC"), TE=b("TE"), TR=b("TR"), WS=b("WS"))),
    ]
    sizes = {b("A"): slots * k, b("High"): slots * k // 2, b("Low"): slots * k // 2, b("Sum"): slots * 4, b("AS"): slots * 2,
             b("Book"): 1024, b("Counts"): experts * 4, b("Offsets"): experts * 4, b("Out"): slots * n * 2,
             b("P"): experts * n * k // 4, b("TC"): 4, b("TE"): tiles * 4, b("TR"): tiles * 4, b("WS"): experts * n * 2}
    return records, sizes


def fixture_manifest(buffers, records, validation, *, rows=None):
    """The same records as a manifest of the `orx_run_fixture` runner (buffers: name -> bytes | array file)."""
    kernels = []
    for record in records:
        family, _, query = record["symbol"].partition("?")
        args = []
        for arg in record["args"]:
            if arg["kind"] == "buffer":
                args.append({"buffer": arg["name"]})
            elif arg["kind"] == "buffer_slice":
                args.append({"buffer": arg["name"], "offset": arg["offset"]})
            else:
                args.append({"i32": arg["value"]})
        entry = {"symbol": record["symbol"], "grid": record["grid"], "block": record["block"],
                 "shared": record["shared_memory_bytes"], "args": args}
        if rows is not None:
            entry["rows"] = rows
        kernels.append(entry)
    return {"schema_version": 1, "target": "gfx950", "buffers": buffers, "kernels": kernels, "validation": validation}


def dumps(record):
    return json.dumps(record, indent=1, sort_keys=False)
