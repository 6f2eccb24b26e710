"""orx_launch_static_scratch: the launch that uses the library's static scratch instead of a caller's
Workspace, for callers that cannot allocate.  Checked through the C ABI against orx_launch (same handle,
a Workspace of the caller's) and against the oracle, bit for bit, on two calls in a row, the second
smaller, for both uses of the scratch: int32 partial tiles of a split launch and two-stage weights
decoded once per launch."""
import numpy as np
import pytest
import torch

from oracle import reference as orc
from orinfer_amd import codebook, lib

pytestmark = pytest.mark.gpu
TABLE = orc.basis()
DEV = "cuda"


def dev(array):
    a = np.ascontiguousarray(array)
    view = {np.dtype(np.uint16): np.int16, np.dtype(np.uint32): np.int32}.get(a.dtype)
    return torch.from_numpy(a.view(view) if view else a).to(DEV)


def case(rng, m, n, k):
    x = rng.normal(size=(m, k)).astype(np.float16)
    a_q, a_s = orc.a8(x)
    packed = rng.integers(0, 2**32, (n, k // 8), dtype=np.uint32)
    scales = rng.uniform(0.005, 0.02, n).astype(np.float16)
    return a_q, a_s[:, 0].copy(), packed, scales


@pytest.mark.parametrize("use", ["split-tiles", "decode-once"])
def test_static_scratch_launch_matches_the_workspace_launch_twice_in_a_row(use):
    rng = np.random.default_rng(orc.SEED + 707)
    if use == "split-tiles":
        capacity, n, k, variant = 256, 5120, 1024, {}
        calls = (256, 130)                       # 80 and 80 tiles of 128 rows, K steps dealt over the CUs
    else:
        capacity, n, k, variant = 1024, 2048, 640, {"split_k": False}
        calls = (1000, 600)                      # 256-row tiles on weights decoded into the scratch
    kern = lib.Kernel("e8p_q4_projection", M=capacity, N=n, K=k, dynamic_rows=True, workspace=True, **variant)
    a_q, a_s, packed, scales = case(rng, capacity, n, k)
    book = dev(codebook.book())
    d_a, d_as, d_w, d_s = dev(a_q), dev(a_s), dev(packed), dev(scales)
    weights = orc.q4_integers(packed, TABLE)
    stream = torch.cuda.current_stream().cuda_stream
    workspace = torch.empty(kern.workspace_bytes(0), dtype=torch.uint8, device=DEV)
    outs = [torch.empty((capacity, n), dtype=torch.float16, device=DEV) for _ in range(2)]
    # one launch up front: the HIP runtime loads a kernel's code object on its first launch
    grid, block, shared = kern.geometry(capacity)
    kern.launch_raw(grid, block, shared, stream, [d_a, d_as, book, outs[0], d_s, d_w, workspace, capacity])
    for rows in calls:
        need = kern.workspace_bytes(rows)
        assert 0 < need <= 64 << 20
        grid, block, shared = kern.geometry(rows)
        for out in outs:
            out.fill_(3.0)
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        # the existing entry point with the caller's Workspace, then the new one with none (null slot)
        kern.launch_raw(grid, block, shared, stream, [d_a, d_as, book, outs[0], d_s, d_w, workspace, rows])
        kern.launch_raw(grid, block, shared, stream, [d_a, d_as, book, outs[1], d_s, d_w, None, rows], static_scratch=True)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before  # the launches took no device memory
        assert torch.equal(outs[0], outs[1])
        got = outs[1].cpu().numpy()
        np.testing.assert_array_equal(got[:rows], orc.project(a_q[:rows], a_s[:rows], weights, scales))
        assert (got[rows:] == 3).all()


def test_static_scratch_launch_runs_plain_kernels_as_orx_launch_does():
    # a launch that needs no scratch (one row: the GEMV), and a kernel without a Workspace argument, run as they do
    # through orx_launch
    rng = np.random.default_rng(orc.SEED + 708)
    a_q, a_s, packed, scales = case(rng, 1, 384, 1024)
    weights = orc.q4_integers(packed, TABLE)
    want = orc.project(a_q, a_s, weights, scales)
    stream = torch.cuda.current_stream().cuda_stream
    for workspace in (True, False):
        kern = lib.Kernel("e8p_q4_projection", M=1, N=384, K=1024, workspace=workspace)
        out = torch.zeros((1, 384), dtype=torch.float16, device=DEV)
        values = [dev(a_q), dev(a_s), dev(codebook.book()), out, dev(scales), dev(packed)] + ([None] if workspace else [])
        kern.launch_raw(*kern.geometry(1), stream, values, static_scratch=True)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(out.cpu().numpy(), want)
