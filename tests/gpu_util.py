"""Helpers for the GPU parity tests: run liborx kernels through the C ABI on torch tensors."""
import numpy as np
import torch

from orinfer_amd import codebook, lib

DEV = "cuda"
_cache = {}


WORKSPACE_SYMBOLS = ("e8p_q4_projection", "int8_projection", "int8_small_projection")


def kernel(symbol, **variant):
    # projections are resolved the way a package would record them: with a Workspace buffer, so that
    # the split-tile and decode-once launches are what the tests run (workspace=False asks for the rest)
    if symbol in WORKSPACE_SYMBOLS:
        variant.setdefault("workspace", True)
    key = (symbol, tuple(sorted((k, tuple(v) if isinstance(v, list) else v) for k, v in variant.items())))
    if key not in _cache:
        _cache[key] = lib.Kernel(symbol, **variant)
    return _cache[key]


def dev(array):
    a = np.ascontiguousarray(array)
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).to(DEV)
    if a.dtype == np.uint32:
        return torch.from_numpy(a.view(np.int32)).to(DEV)
    return torch.from_numpy(a).to(DEV)


def host(tensor, dtype=None):
    a = tensor.detach().cpu().numpy()
    return a.view(dtype) if dtype is not None else a


def book():
    return dev(codebook.book())


def a8(x16, group=None, masked=None, fused=False):
    """x16: torch fp16 [rows, K] (or [rows, 2K] when fused) -> (int8 [rows,K], fp16 [rows,groups])."""
    rows = x16.shape[0]
    k = x16.shape[1] // (2 if fused else 1)
    g = k if group is None else group
    q = torch.empty((rows, k), dtype=torch.int8, device=DEV)
    s = torch.empty((rows, (k + g - 1) // g), dtype=torch.float16, device=DEV)
    variant = dict(K=k)
    if group is not None:
        variant["group_size"] = group
    if masked is not None:
        variant["masked"] = True
    if fused:
        variant["fused"] = True
    kernel("activation_quantization", **variant)(Mask=masked, Q=q, S=s, X=x16, rows=rows)
    return q, s


def q4_project(a_q, a_s, packed, scales, *, rows=None, dynamic=False, capacity=None, out=None, stride=None,
               dtype=torch.float16, packed_k=0, **variant):
    m = a_q.shape[0] if rows is None else rows
    n = scales.shape[0]
    k = a_q.shape[1]
    if out is None:
        out = torch.empty((m, n if stride is None else stride), dtype=dtype, device=DEV)
    v = dict(M=capacity or m, N=n, K=k, **variant)
    if dynamic:
        v["dynamic_rows"] = True
    if stride is not None:
        v["output_stride"] = stride
    if dtype == torch.float32:
        v["output_dtype"] = "float32"
    if packed_k:
        v["packed_k"] = packed_k
    kern = kernel("e8p_q4_projection", **v)
    args = dict(A=a_q, AS=a_s, Book=book(), Out=out, S=scales, W=packed)
    if dynamic:
        args["m"] = m
    kern(**args)
    return out


def w8_project(a_q, a_s, weight, scales, *, rows=None, dynamic=False, capacity=None, out=None, stride=None,
               dtype=torch.float16, **variant):
    m = a_q.shape[0] if rows is None else rows
    n, k = weight.shape
    if out is None:
        out = torch.empty((m, n if stride is None else stride), dtype=dtype, device=DEV)
    v = dict(M=capacity or m, N=n, K=k, **variant)
    if dynamic:
        v["dynamic_rows"] = True
    if stride is not None:
        v["output_stride"] = stride
    if dtype == torch.float32:
        v["output_dtype"] = "float32"
    kern = kernel("int8_projection", **v)
    args = dict(A=a_q, Output=out, TokenScale=a_s, Weight=weight, WeightScale=scales)
    if dynamic:
        args["m"] = m
    kern(**args)
    return out


def sync():
    torch.cuda.synchronize()
