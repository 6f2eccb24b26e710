"""ctypes binding of liborx.so and a Python mirror of the engine's launch path.

`Kernel` plays the part of the engine's `Kernel` record plus `launch_kernel`
(crates/orinfer-engine/src/backend/cuda/mod.rs:312-341): it resolves a symbol + variant to a
handle, asks the library for the launch geometry, marshals arguments as `void**` exactly the
way `Value::address` does (mod.rs:282-299) and enqueues on the caller's stream.  There is no
CPU fallback: a missing library raises.
"""
import ctypes
import json
from pathlib import Path

LIBRARY_PATH = Path(__file__).resolve().parent / "liborx.so"

ORX_OK = 0
ORX_ERR_UNKNOWN_SYMBOL = 10001
ORX_ERR_BAD_VARIANT = 10002
ORX_ERR_BAD_GEOMETRY = 10003
ORX_ERR_BAD_ARGUMENT = 10004
ORX_ERR_ROWS = 10005
ORX_ERR_WORKSPACE = 10006
ORX_ERR_INTERNAL = 10007

EXPORTS = (
    "orx_resolve", "orx_release", "orx_query", "orx_geometry", "orx_arg_count", "orx_arg_name",
    "orx_arg_kind", "orx_launch", "orx_last_error", "orx_catalog", "orx_workspace_bytes",
    "orx_launch_static_scratch", "orx_query_rows",
)


class OrxError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"{message} [code {code}]")
        self.code = code


_lib = None


def library():
    """Loads liborx.so once.  Raises if it has not been built: there is no other path."""
    global _lib
    if _lib is None:
        if not LIBRARY_PATH.exists():
            raise FileNotFoundError(
                f"{LIBRARY_PATH} is missing: build it with `python -m orinfer_amd.build` (hipcc, gfx950)"
            )
        try:
            # liborx must bind to the HIP runtime torch has already loaded: two runtimes in one
            # process do not share devices or streams
            import torch  # noqa: F401
        except ImportError:
            pass
        lib = ctypes.CDLL(str(LIBRARY_PATH))
        u32x3 = ctypes.POINTER(ctypes.c_uint32)
        lib.orx_resolve.argtypes = [ctypes.c_char_p, ctypes.c_char_p, ctypes.POINTER(ctypes.c_void_p)]
        lib.orx_resolve.restype = ctypes.c_int
        lib.orx_release.argtypes = [ctypes.c_void_p]
        lib.orx_release.restype = ctypes.c_int
        lib.orx_query.argtypes = [ctypes.c_void_p, u32x3, u32x3]
        lib.orx_query.restype = ctypes.c_int
        lib.orx_query_rows.argtypes = [ctypes.c_void_p, ctypes.c_int32, u32x3, u32x3]
        lib.orx_query_rows.restype = ctypes.c_int
        lib.orx_geometry.argtypes = [ctypes.c_void_p, ctypes.c_int32, u32x3, u32x3, u32x3]
        lib.orx_geometry.restype = ctypes.c_int
        lib.orx_arg_count.argtypes = [ctypes.c_void_p]
        lib.orx_arg_count.restype = ctypes.c_int
        lib.orx_arg_name.argtypes = [ctypes.c_void_p, ctypes.c_int]
        lib.orx_arg_name.restype = ctypes.c_char_p
        lib.orx_arg_kind.argtypes = [ctypes.c_void_p, ctypes.c_int]
        lib.orx_arg_kind.restype = ctypes.c_int
        lib.orx_launch.argtypes = [ctypes.c_void_p, u32x3, u32x3, ctypes.c_uint32, ctypes.c_void_p,
                                   ctypes.POINTER(ctypes.c_void_p)]
        lib.orx_launch.restype = ctypes.c_int
        lib.orx_launch_static_scratch.argtypes = lib.orx_launch.argtypes
        lib.orx_launch_static_scratch.restype = ctypes.c_int
        lib.orx_workspace_bytes.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.POINTER(ctypes.c_uint64)]
        lib.orx_workspace_bytes.restype = ctypes.c_int
        lib.orx_last_error.argtypes = []
        lib.orx_last_error.restype = ctypes.c_char_p
        lib.orx_catalog.argtypes = []
        lib.orx_catalog.restype = ctypes.c_char_p
        _lib = lib
    return _lib


def last_error():
    return library().orx_last_error().decode()


def catalog():
    return json.loads(library().orx_catalog().decode())


def _check(code):
    if code != ORX_OK:
        raise OrxError(code, last_error())


def _pointer_of(value):
    if value is None:
        return 0
    if hasattr(value, "data_ptr"):
        return int(value.data_ptr())
    return int(value)


class Kernel:
    """A resolved kernel: symbol + variant -> handle, argument order, geometry, launch."""

    def __init__(self, symbol, **variant):
        self.symbol = symbol
        self.variant = dict(variant)
        self._handle = ctypes.c_void_p()
        self._workspace = None
        lib = library()
        _check(lib.orx_resolve(symbol.encode(), json.dumps(self.variant).encode(), ctypes.byref(self._handle)))
        count = lib.orx_arg_count(self._handle)
        self.arg_names = [lib.orx_arg_name(self._handle, i).decode() for i in range(count)]
        self.arg_kinds = [lib.orx_arg_kind(self._handle, i) for i in range(count)]

    def __del__(self):
        handle = getattr(self, "_handle", None)
        if handle and _lib is not None:
            _lib.orx_release(handle)
            self._handle = None

    def query(self, rows=0):
        """(thread limit, static LDS bytes) of the kernel that a launch of `rows` rows starts (0: the variant's M)."""
        threads, lds = ctypes.c_uint32(), ctypes.c_uint32()
        _check(library().orx_query_rows(self._handle, int(rows), ctypes.byref(threads), ctypes.byref(lds)))
        return threads.value, lds.value

    def geometry(self, rows=0):
        grid, block = (ctypes.c_uint32 * 3)(), (ctypes.c_uint32 * 3)()
        shared = ctypes.c_uint32()
        _check(library().orx_geometry(self._handle, int(rows), grid, block, ctypes.byref(shared)))
        return tuple(grid), tuple(block), shared.value

    def workspace_bytes(self, rows=0):
        """Bytes of `Workspace` a launch of `rows` rows uses (rows = 0: the most any row count needs)."""
        need = ctypes.c_uint64()
        _check(library().orx_workspace_bytes(self._handle, int(rows), ctypes.byref(need)))
        return need.value

    def workspace(self):
        """This caller's Workspace buffer for the kernel, allocated once at the largest need (torch memory:
        the caller owns it, as the engine owns every buffer).  None when the kernel takes or needs none."""
        if "Workspace" not in self.arg_names:
            return None
        if self._workspace is None:
            need = self.workspace_bytes(0)
            if need:
                import torch

                self._workspace = torch.empty(need, dtype=torch.uint8, device="cuda")
        return self._workspace

    def launch_raw(self, grid, block, shared, stream, values, static_scratch=False):
        """values: ABI-ordered list of device addresses (int) / int32 scalars.  Mirrors launch_kernel.
        static_scratch: through orx_launch_static_scratch (the library's scratch replaces Workspace)."""
        if len(values) != len(self.arg_names):
            raise OrxError(ORX_ERR_BAD_ARGUMENT,
                           f"{self.symbol} takes {len(self.arg_names)} arguments {self.arg_names}, got {len(values)}")
        storage = []
        for kind, value in zip(self.arg_kinds, values):
            storage.append(ctypes.c_uint64(_pointer_of(value)) if kind == 0 else ctypes.c_int32(int(value)))
        pointers = (ctypes.c_void_p * len(storage))(*[ctypes.cast(ctypes.byref(s), ctypes.c_void_p) for s in storage])
        g, b = (ctypes.c_uint32 * 3)(*grid), (ctypes.c_uint32 * 3)(*block)
        entry = library().orx_launch_static_scratch if static_scratch else library().orx_launch
        _check(entry(self._handle, g, b, int(shared), ctypes.c_void_p(int(stream)), pointers))

    def launch(self, *values, rows=0, stream=None):
        """Launch with ABI-ordered arguments on `stream` (default: torch's current stream)."""
        if stream is None:
            import torch

            stream = torch.cuda.current_stream().cuda_stream
        if rows == 0 and self.arg_names and self.arg_names[-1] in ("m", "rows"):
            rows = int(values[-1])
        grid, block, shared = self.geometry(rows)
        self.launch_raw(grid, block, shared, stream, values)

    def __call__(self, stream=None, **named):
        """Launch with arguments given by name (any order); unknown or missing names raise."""
        if "Workspace" in self.arg_names and "Workspace" not in named:
            named["Workspace"] = self.workspace()
        unknown = set(named) - set(self.arg_names)
        if unknown:
            raise OrxError(ORX_ERR_BAD_ARGUMENT, f"{self.symbol} has no arguments {sorted(unknown)}")
        missing = [n for n in self.arg_names if n not in named]
        if missing:
            raise OrxError(ORX_ERR_BAD_ARGUMENT, f"{self.symbol} needs arguments {missing}")
        self.launch(*[named[n] for n in self.arg_names], stream=stream)
