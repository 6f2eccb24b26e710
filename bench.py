"""Benchmark of the quantized linear-layer path on one MI355X.

Contract line (one JSON object on stdout): metric = Q4A8 GEMV achieved HBM GB/s on
BASELINE configuration 1 at M=1 (K=5120, N=17408), one step = A8 quantisation of the token row
plus the E8P-Q4 projection, weights rotating over enough distinct copies that they cannot stay
in the 256 MB Infinity Cache.  `roofline` prices the projection kernel alone against 8 TB/s;
`extra` carries the other configurations (GEMV config 0, the M sweep, W8A8 and layer GEMM TOPS
against the int8 MFMA peak, the MoE layer).  `cpu_baseline` times the oracle's C restatement on the same
workload on this box's host cores.
"""
import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0          # MI355X published HBM3E bandwidth
INT8_PEAK_TOPS = 5000.0        # MI355X published dense int8 MFMA (5.0 POP/s)
CACHE_BYTES = 256 << 20        # Infinity Cache
# Untimed replays in front of every timed region, beside the W warm-up steps: after the idle time in which the host
# prepares a workload the GPU's clocks take a few tenths of a second of work to settle (config 1 at 8 / 32 rows reads
# 17.2 / 20.5 us in the first replays after a pause and 15.1 / 18.2 us from 0.5 s on), and a few warm-up steps of some
# microseconds each do not cover that.
CLOCK_WARMUP_SECONDS = 0.6

# HBM bytes per launch of the contract kernel come from the committed counter summary (two
# `rocprofv3 --pmc` runs of `bench.py --profile-traffic`: FETCH_SIZE, then WRITE_SIZE, each scaled by what
# the same counter reads for a device copy of known size in the same run).  The summary records the
# launch it was taken on; `measured_traffic` gives nothing when that is not what the handle launches now.
TRAFFIC_SUMMARY = ROOT / "profiles" / "gemv_q4_config1_m1_hbm_traffic.txt"


def measured_traffic(geometry):
    """(bytes per launch, kernel name) from the counter summary, or (None, None) when the summary is
    absent, unreadable or was taken on a launch with another grid, block or LDS size."""
    try:
        fields = {}
        for line in TRAFFIC_SUMMARY.read_text().splitlines():
            if line.startswith("bench-traffic:"):
                for item in line[len("bench-traffic:"):].split(";"):
                    key, _, value = item.strip().partition("=")
                    fields[key] = value.strip()
        grid, block, shared = geometry
        if (int(fields["grid"]), int(fields["block"]), int(fields["lds"])) != (grid[0], block[0], shared):
            return None, None
        copy_kib = float(fields["copy_kib"])
        fetch = float(fields["kernel_fetch"]) * copy_kib / float(fields["copy_fetch"])
        write = float(fields["kernel_write"]) * copy_kib / float(fields["copy_write"])
        return int(round((fetch + write) * 1024)), fields["kernel"]
    except (OSError, KeyError, ValueError, ZeroDivisionError):
        return None, None


def parse():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=2000)
    p.add_argument("--warmup", type=int, default=100)
    p.add_argument("--no-extra", action="store_true", help="only the contract workload")
    p.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    p.add_argument("--settle", type=float, default=CLOCK_WARMUP_SECONDS, metavar="SECONDS",
                   help="untimed graph replays in front of every timed region (0 under a profiler: they only add dispatches)")
    p.add_argument("--profile-rows", type=int, default=0, metavar="ROWS",
                   help="workload for a rocprofv3 counter run: config 1's projection at ROWS rows once per weight copy, "
                        "eagerly, then exit")
    p.add_argument("--profile-traffic", action="store_true",
                   help="workload for `rocprofv3 --pmc FETCH_SIZE|WRITE_SIZE`: a plain copy of known size, then the "
                        "contract kernel once per weight copy, eagerly; no timing")
    return p.parse_args()


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (--gpus must be 1)", file=sys.stderr)
        sys.exit(2)
    import numpy as np
    import torch

    from orinfer_amd import codebook, lib, workloads
    from orinfer_amd.lib import Kernel

    lib.library()
    torch.cuda.set_device(0)
    stream = torch.cuda.current_stream()

    def dev(a):
        a = np.ascontiguousarray(a)
        view = {np.dtype(np.uint16): np.int16, np.dtype(np.uint32): np.int32}.get(a.dtype)
        return torch.from_numpy(a.view(view) if view else a).cuda()

    def settle(graph):
        """Untimed replays: the graph's upload, then work until the clocks have settled."""
        t0 = time.perf_counter()
        while True:
            graph.replay()
            torch.cuda.synchronize()
            if time.perf_counter() - t0 >= args.settle:
                return

    def timed_graph(enqueue, launches, replays=3):
        """Captures `launches` calls of enqueue(i) in one graph; returns mean seconds per launch over
        `replays` replays behind the untimed ones of settle()."""
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            enqueue(0, side.cuda_stream)  # warm-up outside capture (first-launch setup)
            side.synchronize()
            with torch.cuda.graph(graph, stream=side):
                for i in range(launches):
                    enqueue(i, side.cuda_stream)
        settle(graph)
        total = 0.0
        for replay in range(replays):
            start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            start.record()
            graph.replay()
            stop.record()
            torch.cuda.synchronize()
            total += start.elapsed_time(stop) * 1e-3 / launches
        return total / replays

    book = dev(codebook.book())

    class Q4Case:
        """One Q4A8 linear at (rows, n, k) with `copies` distinct weight tensors."""

        def __init__(self, case, copies, algorithm="auto", packed_k=0, fused_input=False):
            self.rows, self.n, self.k = case["rows"], case["n"], case["k"]
            rng = np.random.default_rng(7)
            first = case["packed"] if packed_k == 0 else codebook.q4_to_k_major(case["packed"], packed_k)
            self.weights = [dev(first)]
            for _ in range(copies - 1):  # same shape and statistics, different bits
                self.weights.append(dev(rng.integers(0, 2**32, first.shape, dtype=np.uint32)))
            self.scales = dev(case["scales"])
            self.x = dev(case["x"])
            self.a_q = torch.empty((self.rows, self.k), dtype=torch.int8, device="cuda")
            self.a_s = torch.empty((self.rows, 1), dtype=torch.float16, device="cuda")
            self.out = torch.empty((self.rows, self.n), dtype=torch.float16, device="cuda")
            self.quant = Kernel("activation_quantization", K=self.k)
            self.proj = Kernel("e8p_q4_projection", M=self.rows, N=self.n, K=self.k, algorithm=algorithm, workspace=True,
                               **({"packed_k": packed_k} if packed_k else {}))
            self.proj.workspace()  # the caller's scratch, allocated before anything is captured
            # one row: the projection can quantise its fp16 row itself (one launch instead of two)
            self.fused = Kernel("e8p_q4_projection", M=1, N=self.n, K=self.k, input_dtype="float16",
                                **({"packed_k": packed_k} if packed_k else {})) if fused_input else None

        def quantize(self, s):
            self.quant(stream=s, Mask=None, Q=self.a_q, S=self.a_s, X=self.x, rows=self.rows)

        def project(self, i, s):
            self.proj(stream=s, A=self.a_q, AS=self.a_s, Book=book, Out=self.out, S=self.scales,
                      W=self.weights[i % len(self.weights)])

        def project_fp16(self, i, s):
            self.fused(stream=s, A=self.x, AS=self.a_s, Book=book, Out=self.out, S=self.scales,
                       W=self.weights[i % len(self.weights)])

        def step(self, i, s):
            if self.fused is not None:
                self.project_fp16(i, s)
            else:
                self.quantize(s)
                self.project(i, s)

    # ---- contract workload: config 1, M=1 ----
    c1 = workloads.config1(1)
    bytes_c1 = workloads.algorithmic_bytes_q4(1, c1["n"], c1["k"])
    copies = -(-2 * CACHE_BYTES // (c1["n"] * c1["k"] // 2))  # aggregate footprint >= 2x the cache
    main_case = Q4Case(c1, copies, fused_input=True)
    if args.profile_rows:
        case = Q4Case(workloads.config1(args.profile_rows), copies)
        case.quantize(stream.cuda_stream)
        for i in range(copies):
            case.project(i, stream.cuda_stream)
        torch.cuda.synchronize()
        grid, block, shared = case.proj.geometry(args.profile_rows)
        print(json.dumps({"profile_rows": {"rows": args.profile_rows, "launches": copies, "grid": list(grid), "block": list(block), "lds": shared}}))
        return
    if args.profile_traffic:
        # counter calibration: a device copy reads and writes exactly `probe.numel()` bytes
        probe = torch.empty(c1["n"] * c1["k"] // 2, dtype=torch.uint8, device="cuda").random_(0, 256)
        target = torch.empty_like(probe)
        for _ in range(4):
            target.copy_(probe)
        for i in range(copies):
            main_case.step(i, stream.cuda_stream)
        torch.cuda.synchronize()
        grid, block, shared = main_case.fused.geometry(1)
        print(json.dumps({"profile_traffic": {"copy_bytes_read": probe.numel(), "copy_bytes_written": probe.numel(),
                                            "projection_launches": copies, "algorithmic_bytes": bytes_c1,
                                            "grid": grid[0], "block": block[0], "lds": shared}}))
        return
    for i in range(args.warmup):
        main_case.step(i, stream.cuda_stream)
    torch.cuda.synchronize()
    # exactly K steps, bracketed by synchronize on both sides, replayed as one graph
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            for i in range(args.steps):
                main_case.step(i, side.cuda_stream)
    settle(graph)  # graph upload and clocks
    t0 = time.perf_counter()
    graph.replay()
    torch.cuda.synchronize()
    step_seconds = (time.perf_counter() - t0) / args.steps
    # the step is one launch: the GEMV that quantises its fp16 row during set-up
    # (260 launches per graph whatever K is: the events bracket the graph's own launch as well, which is 0.3 us per
    # kernel in a graph of 20 and nothing in one of 260)
    kernel_seconds = timed_graph(lambda i, s: main_case.project_fp16(i, s), max(260, copies))
    achieved = bytes_c1 / kernel_seconds / 1e9
    # for comparison: the same GEMV on a row that is already int8 (the quantiser is then a launch of its own)
    main_case.quantize(stream.cuda_stream)
    plain_seconds = timed_graph(lambda i, s: main_case.project(i, s), max(260, copies))
    traffic_bytes, traffic_kernel = measured_traffic(main_case.fused.geometry(1))
    # config 0 (the reference's own CPU-runnable shape) on the same kernel: a second roofline entry
    c0 = workloads.config0()
    b0 = workloads.algorithmic_bytes_q4(1, c0["n"], c0["k"])
    case0 = Q4Case(c0, -(-2 * CACHE_BYTES // (c0["n"] * c0["k"] // 2)), fused_input=True)
    t0_fused = timed_graph(lambda i, s: case0.project_fp16(i, s), 480)
    case0.quantize(stream.cuda_stream)
    t0_plain = timed_graph(lambda i, s: case0.project(i, s), 480)
    del case0
    result = {
        "metric": "Q4A8 GEMV HBM GB/s (% of peak) + GEMM int8 TOPS (% MFMA peak), 1 GPU",
        "value": round(bytes_c1 / step_seconds / 1e9, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(step_seconds * 1e3, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8 x int8 -> int32 (u16 E8P codes), fp16 rescale",
        "data": "synthetic (seeded uniform codes, N(0,1) activations, random-init scales)",
        "config": {"workload": "BASELINE config 1: Q4A8 linear K=5120 N=17408, M=1 decode GEMV, step = A8 + projection "
                               "of one fp16 row (one launch: the GEMV quantises the row during its set-up)",
                   "weight_copies_rotated": copies, "algorithmic_bytes_per_step": bytes_c1,
                   "untimed_replays_before_timing_seconds": args.settle},
        "roofline": {"bound": "hbm", "kernel": traffic_kernel or "gemv_banked_kernel<Q4, 1 row, fp16 input>",
                     "achieved": round(achieved, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "us_per_launch": round(kernel_seconds * 1e6, 3), "traffic": traffic_bytes,
                     "same_kernel_int8_input": {"us_per_launch": round(plain_seconds * 1e6, 3),
                                                "achieved": round(bytes_c1 / plain_seconds / 1e9, 1),
                                                "frac": round(bytes_c1 / plain_seconds / 1e9 / HBM_PEAK_GBS, 4)},
                     "config0": {"workload": "BASELINE config 0: Q4A8 linear K=2560 N=9728, M=1, fp16 row in",
                                 "bound": "hbm", "algorithmic_bytes": b0, "us_per_launch": round(t0_fused * 1e6, 3),
                                 "achieved": round(b0 / t0_fused / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                 "frac": round(b0 / t0_fused / 1e9 / HBM_PEAK_GBS, 4),
                                 "int8_input_us_per_launch": round(t0_plain * 1e6, 3)}},
    }

    extra = {}
    # launches per graph for kernels of tens of microseconds: at least a hundred, so that a replay lasts milliseconds
    # (a 26-launch graph of the 128-row projection reads 38-40 us per launch, a 260-launch one settles at 34.6)
    short_graph = 8 * copies
    if not args.no_extra:
        # config 0 GEMV (int8 row in; the fp16-row form is `roofline.config0`)
        extra["config0_q4a8_gemv_m1"] = {"us": round(t0_plain * 1e6, 3), "GBps": round(b0 / t0_plain / 1e9, 1),
                                         "frac_hbm": round(b0 / t0_plain / 1e9 / HBM_PEAK_GBS, 4), "bytes": b0}
        # config 1 sweep
        sweep = {}
        for rows in (1, 8, 32, 128, 512, 1024):
            case = Q4Case(workloads.config1(rows), copies)
            t = timed_graph(lambda i, s: case.project(i, s), short_graph)
            b = workloads.algorithmic_bytes_q4(rows, case.n, case.k)
            ops = workloads.algorithmic_ops(rows, case.n, case.k)
            sweep[str(rows)] = {"us": round(t * 1e6, 3), "GBps": round(b / t / 1e9, 1),
                                "frac_hbm": round(b / t / 1e9 / HBM_PEAK_GBS, 4), "TOPS": round(ops / t / 1e12, 2),
                                "frac_int8": round(ops / t / 1e12 / INT8_PEAK_TOPS, 4)}
            del case
        extra["config1_q4a8_sweep"] = sweep
        # the same decode step as two launches (quantiser, then the projection on int8 rows)
        t_a8 = timed_graph(lambda i, s: main_case.quantize(s), short_graph)
        t_both = timed_graph(lambda i, s: (main_case.quantize(s), main_case.project(i, s)), short_graph)
        extra["config1_m1_two_launches"] = {"a8_us": round(t_a8 * 1e6, 3), "gemv_us": sweep["1"]["us"],
                                            "both_us": round(t_both * 1e6, 3)}
        # the production form of the step: signed block-128 rotation in front of the quantiser
        signs1 = (torch.randint(0, 2, (main_case.k,), device="cuda", dtype=torch.int8) * 2 - 1)
        rot1 = Kernel("rotate_activation_a8", M=1, K=main_case.k)
        fused_rot = Kernel("e8p_q4_projection", M=1, N=main_case.n, K=main_case.k, input_dtype="float16", rotate=True)

        def rotate_then_project(i, s):
            rot1(stream=s, Q=main_case.a_q, S=main_case.a_s, Signs=signs1, X=main_case.x)
            main_case.project(i, s)

        t_rot_two = timed_graph(rotate_then_project, short_graph)
        t_rot_one = timed_graph(lambda i, s: fused_rot(stream=s, A=main_case.x, AS=main_case.a_s, Book=book,
                                                       Out=main_case.out, S=main_case.scales, Signs=signs1,
                                                       W=main_case.weights[i % copies]), short_graph)
        extra["config1_m1_rotated_input"] = {"rotate_a8_then_gemv_us": round(t_rot_two * 1e6, 3),
                                             "one_launch_us": round(t_rot_one * 1e6, 3)}
        # the same projection on the reference's storage layout (K-major blocks of 128)
        k_major = {}
        for rows in (1, 8, 32):
            case = Q4Case(workloads.config1(rows), copies, packed_k=128)
            t = timed_graph(lambda i, s: case.project(i, s), short_graph)
            b = workloads.algorithmic_bytes_q4(rows, case.n, case.k)
            k_major[str(rows)] = {"us": round(t * 1e6, 3), "GBps": round(b / t / 1e9, 1),
                                  "frac_hbm": round(b / t / 1e9 / HBM_PEAK_GBS, 4)}
            del case
        extra["config1_q4a8_k_major_codes"] = k_major
        del main_case
        torch.cuda.empty_cache()
        # config 2 W8A8
        c2 = workloads.config2()
        x2 = dev(c2["x"])
        a2 = torch.empty((c2["rows"], c2["k"]), dtype=torch.int8, device="cuda")
        s2 = torch.empty((c2["rows"], 1), dtype=torch.float16, device="cuda")
        o2 = torch.empty((c2["rows"], c2["n"]), dtype=torch.float16, device="cuda")
        w2, ws2 = dev(c2["weight"]), dev(c2["scales"])
        quant2 = Kernel("activation_quantization", K=c2["k"])
        proj2 = Kernel("int8_projection", M=c2["rows"], N=c2["n"], K=c2["k"], workspace=True)
        proj2.workspace()
        quant2(Mask=None, Q=a2, S=s2, X=x2, rows=c2["rows"])
        t = timed_graph(lambda i, s: proj2(stream=s, A=a2, Output=o2, TokenScale=s2, Weight=w2, WeightScale=ws2), 20)
        tq = timed_graph(lambda i, s: quant2(stream=s, Mask=None, Q=a2, S=s2, X=x2, rows=c2["rows"]), 20)
        ops = workloads.algorithmic_ops(c2["rows"], c2["n"], c2["k"])
        extra["config2_w8a8_gemm"] = {"us": round(t * 1e6, 2), "TOPS": round(ops / t / 1e12, 1),
                                      "frac_int8": round(ops / t / 1e12 / INT8_PEAK_TOPS, 4),
                                      "a8_us": round(tq * 1e6, 2)}
        del x2, a2, s2, o2, w2
        torch.cuda.empty_cache()
        # config 3 MoE layer
        from orinfer_amd import programs

        c3 = workloads.config3()
        layer = programs.MoeLayer(c3["tokens"], c3["experts"], c3["top_k"], c3["hidden"], c3["intermediate"],
                                  c3["gate_up"], c3["gate_up_scales"], c3["down"], c3["down_scales"], block_m=32)
        x3, l3 = dev(c3["x"]), dev(c3["logits"])
        t = timed_graph(lambda i, s: layer.run(x3, l3, stream=s), 100)
        counts = layer.counts.cpu().numpy()
        touched = int((counts > 0).sum())
        code_bytes = touched * (c3["hidden"] * 2 * c3["intermediate"] + c3["intermediate"] * c3["hidden"]) // 4
        extra["config3_moe_q2a8_layer"] = {"us": round(t * 1e6, 2), "experts_touched": touched,
                                           "code_bytes_touched": code_bytes,
                                           "GBps_codes": round(code_bytes / t / 1e9, 1)}
        del layer
        # one token of the same layer: its 8 routes index the banks directly (no sorting, no tiles)
        raw_book = dev(codebook.raw_book())
        e3, h3, i3, k3 = c3["experts"], c3["hidden"], c3["intermediate"], c3["top_k"]
        routes = torch.tensor([[3, 77, 12, 100, 64, 31, 127, 2]], dtype=torch.int32, device="cuda")
        single = {}
        for name, codes, scales, n, k, shared in (("gate_up", c3["gate_up"], c3["gate_up_scales"], 2 * i3, h3, True),
                                                  ("down", c3["down"], c3["down_scales"], h3, i3, False)):
            bank = dev(codes).view(e3, n, k // 128, 16).permute(0, 2, 1, 3).contiguous()
            rows = 1 if shared else k3
            a = torch.randint(-127, 128, (rows, k), dtype=torch.int8, device="cuda")
            a_scale = torch.full((rows,), 0.01, dtype=torch.float16, device="cuda")
            out = torch.empty((k3, n), dtype=torch.float16, device="cuda")
            kern = Kernel("integer_e8p_gemv", E=e3, routes=k3, N=n, K=k, shared_input=shared)
            ws_dev = dev(scales)
            t = timed_graph(lambda i, st: kern(stream=st, A=a, AS=a_scale, Book=raw_book, C=out, IDs=routes, P=bank,
                                               WS=ws_dev), 100)
            moved = k3 * n * k // 4
            single[name] = {"us": round(t * 1e6, 2), "GBps_codes": round(moved / t / 1e9, 1)}
            del bank
        extra["config3_single_token_routes"] = single
        # the whole layer for one token: direct bank indexing against the token-sorted program
        token_layer = programs.MoeTokenLayer(e3, k3, h3, i3, c3["gate_up"], c3["gate_up_scales"], c3["down"],
                                             c3["down_scales"])
        sorted_layer = programs.MoeLayer(1, e3, k3, h3, i3, c3["gate_up"], c3["gate_up_scales"], c3["down"],
                                         c3["down_scales"], block_m=32)
        x1, l1 = x3[:1].contiguous(), l3[:1].contiguous()
        t_direct = timed_graph(lambda i, s: token_layer.run(x1, l1, stream=s), 100)
        t_sorted = timed_graph(lambda i, s: sorted_layer.run(x1, l1, stream=s), 100)
        extra["config3_single_token_layer"] = {"direct_routes_us": round(t_direct * 1e6, 2),
                                               "token_sorted_us": round(t_sorted * 1e6, 2)}
        del token_layer, sorted_layer
        torch.cuda.empty_cache()
        # config 4 layer linears
        c4 = workloads.config4()
        layer_us, per = 0.0, {}
        for name, spec in c4.items():
            rows, n, k = spec["rows"], spec["n"], spec["k"]
            x = dev(spec["x"])
            a = torch.empty((rows, k), dtype=torch.int8, device="cuda")
            sc = torch.empty((rows, 1), dtype=torch.float16, device="cuda")
            o = torch.empty((rows, n), dtype=torch.float16, device="cuda")
            ws = dev(spec["scales"])
            quant = Kernel("activation_quantization", K=k)
            if spec["codec"] == "q4":
                w = dev(spec["packed"])
                proj = Kernel("e8p_q4_projection", M=rows, N=n, K=k, workspace=True)
                run = lambda i, s: proj(stream=s, A=a, AS=sc, Book=book, Out=o, S=ws, W=w)
            else:
                w = dev(spec["weight"])
                proj = Kernel("int8_projection", M=rows, N=n, K=k, workspace=True)
                run = lambda i, s: proj(stream=s, A=a, Output=o, TokenScale=sc, Weight=w, WeightScale=ws)
            proj.workspace()
            tq = timed_graph(lambda i, s: quant(stream=s, Mask=None, Q=a, S=sc, X=x, rows=rows), 5)
            tp = timed_graph(run, 5)
            ops = workloads.algorithmic_ops(rows, n, k)
            per[name] = {"codec": spec["codec"], "a8_us": round(tq * 1e6, 1), "gemm_us": round(tp * 1e6, 1),
                         "TOPS": round(ops / tp / 1e12, 1), "frac_int8": round(ops / tp / 1e12 / INT8_PEAK_TOPS, 4)}
            layer_us += (tq + tp) * 1e6
            del x, a, o, w
            torch.cuda.empty_cache()
        extra["config4_layer_linears_m8192"] = {"layer_us": round(layer_us, 1), "per_gemm": per}

        # signed block-128 rotation fused with A8: the real producer of the int8 activations
        rows, width = 8192, 5120
        x = torch.randn((rows, width), dtype=torch.float16, device="cuda")
        signs = (torch.randint(0, 2, (width,), device="cuda", dtype=torch.int8) * 2 - 1)
        q = torch.empty((rows, width), dtype=torch.int8, device="cuda")
        sc = torch.empty((rows,), dtype=torch.float16, device="cuda")
        rot = Kernel("rotate_activation_a8", M=rows, K=width)
        tr = timed_graph(lambda i, st: rot(stream=st, Q=q, S=sc, Signs=signs, X=x), 20)
        moved = rows * width * 3 + rows * 2 + width
        extra["rotate_a8_m8192_k5120"] = {"us": round(tr * 1e6, 2), "GBps": round(moved / tr / 1e9, 1),
                                          "frac_hbm": round(moved / tr / 1e9 / HBM_PEAK_GBS, 4), "bytes": moved}
        # the same with the residual add and RMSNorm in front: fp16 + fp32 in, fp16 + fp32 + int8 out
        res = torch.randn((rows, width), dtype=torch.float32, device="cuda")
        res_out = torch.empty_like(res)
        gain = torch.randn((width,), dtype=torch.float16, device="cuda") * 0.1
        y = torch.empty_like(x)
        fused = Kernel("residual_norm_rotate_a8", M=rows, K=width)
        tf = timed_graph(lambda i, st: fused(stream=st, Q=q, R=res, RO=res_out, S=sc, Signs=signs, W=gain, X=x, Y=y), 20)
        moved = rows * width * (2 + 4 + 2 + 4 + 1) + rows * 2 + width * 3
        extra["residual_norm_rotate_a8_m8192_k5120"] = {"us": round(tf * 1e6, 2), "GBps": round(moved / tf / 1e9, 1),
                                                        "frac_hbm": round(moved / tf / 1e9 / HBM_PEAK_GBS, 4),
                                                        "bytes": moved}
        del x, q, res, res_out, y

        # ---- the reference's other factories on the path, at the same shapes ----
        # row-scaled scalar Q4 (q4_projection): config 1's matrix as nibbles, six weight copies in rotation
        rng = np.random.default_rng(11)
        n4, k4 = c1["n"], c1["k"]
        nibbles = [dev(rng.integers(0, 65536, (n4, k4 // 4), dtype=np.uint16)) for _ in range(6)]
        s4 = dev(c1["scales"])
        scalar = {}
        for rows in (1, 32, 512):
            a4 = torch.randint(-127, 128, (rows, k4), dtype=torch.int8, device="cuda")
            as4 = torch.rand((rows,), dtype=torch.float16, device="cuda") * 0.02 + 0.01
            o4 = torch.empty((rows, n4), dtype=torch.float16, device="cuda")
            kern = Kernel("q4_projection", M=rows, N=n4, K=k4, workspace=True)
            ws4 = kern.workspace()
            t = timed_graph(lambda i, st: kern(stream=st, A=a4, AS=as4, Out=o4, S=s4, W=nibbles[i % 6], Workspace=ws4), 24)
            code_bytes = n4 * k4 // 2
            scalar[str(rows)] = {"us": round(t * 1e6, 2), "weight_GBps": round(code_bytes / t / 1e9, 1),
                                 "TOPS": round(2 * rows * n4 * k4 / t / 1e12, 1)}
        extra["scalar_q4_projection_config1_shape"] = scalar
        del nibbles
        # nibble planes: config 3's gate_up through split_prefill_a8 + e8p_prefill_grouped (16-row tiles)
        e3, slots3, h3, n3 = 128, 2048, 2048, 1024
        ids3 = dev(np.stack([rng.choice(e3, 8, replace=False) for _ in range(256)]).astype(np.int32))
        cap3 = (slots3 + 15) // 16 + min(e3, slots3)
        i32 = dict(dtype=torch.int32, device="cuda")
        counts3, relative3 = torch.zeros((e3,), **i32), torch.zeros((256, 8), **i32)
        offsets3, tile_offsets3, total3 = torch.zeros((e3,), **i32), torch.zeros((e3,), **i32), torch.zeros((1,), **i32)
        te3, tr3 = torch.zeros((cap3,), **i32), torch.zeros((cap3,), **i32)
        Kernel("route_metadata", M=256, E=e3, top_k=8, block_m=16)(
            Counts=counts3, IDs=ids3, RelativeSlot=relative3, RowOffsets=offsets3, TileCount=total3, TileExpert=te3,
            TileOffsets=tile_offsets3, TileRow=tr3)
        a3 = torch.randint(-127, 128, (slots3, h3), dtype=torch.int8, device="cuda")
        low3 = torch.empty((h3 // 64, slots3, 8), dtype=torch.int32, device="cuda")
        high3, sum3 = torch.empty_like(low3), torch.empty((slots3,), dtype=torch.int32, device="cuda")
        split = Kernel("split_prefill_a8", rows=slots3, K=h3)
        t_split = timed_graph(lambda i, st: split(stream=st, A=a3, High=high3, Low=low3, Sum=sum3), 40)
        p3 = dev(rng.integers(0, 65536, (e3, h3 // 64, n3, 8), dtype=np.uint16))
        nib3 = dev(codebook.nibble_book())
        ws3 = dev(rng.uniform(0.005, 0.02, (e3, n3)).astype(np.float16))
        as3 = torch.rand((slots3,), dtype=torch.float16, device="cuda") * 0.02 + 0.01
        o3 = torch.empty((slots3, n3), dtype=torch.float16, device="cuda")
        grouped = Kernel("e8p_prefill_grouped", rows=slots3, E=e3, tiles=cap3, N=n3, K=h3, block_m=16)
        routing3 = dict(Counts=counts3, Offsets=offsets3, TC=total3, TE=te3, TR=tr3)
        t_planes = timed_graph(lambda i, st: grouped(stream=st, AS=as3, Book=nib3, High=high3, Low=low3, Out=o3, P=p3, Sum=sum3,
                                                     WS=ws3, **routing3), 40)
        extra["config3_gate_up_on_nibble_planes"] = {"split_prefill_a8_us": round(t_split * 1e6, 2),
                                                     "e8p_prefill_grouped_us": round(t_planes * 1e6, 2),
                                                     "tiles_of_16_rows": int(total3.cpu()[0])}
        # router projection: 256 tokens x 2048 -> 128 logits + the shared expert's gate
        xr = torch.randn((256, 2048), dtype=torch.float16, device="cuda")
        wr = torch.randn((129, 2048), dtype=torch.float16, device="cuda") * 0.05
        lr = torch.empty((256, 128), dtype=torch.float32, device="cuda")
        gr = torch.empty((256,), dtype=torch.float16, device="cuda")
        proj = Kernel("router_projection", M=256, H=2048, E=128)
        t_proj = timed_graph(lambda i, st: proj(stream=st, Logits=lr, SharedGate=gr, W=wr, X=xr), 100)
        extra["config3_router_projection"] = {"us": round(t_proj * 1e6, 2)}
    result["extra"] = extra

    # ---- CPU baseline: the oracle's C restatement on the contract workload, all host cores ----
    if not args.no_cpu:
        import ctypes
        from concurrent.futures import ThreadPoolExecutor

        from oracle import reference as orc

        so = Path(__file__).resolve().parent / "oracle" / "libe8p_oracle.so"
        if not so.exists():  # the checker's own build step (gcc), as the tests do
            import subprocess

            subprocess.check_call(["make", "-C", str(so.parent)], stdout=subprocess.DEVNULL)
        clib = ctypes.CDLL(str(so))
        table = np.ascontiguousarray(orc.basis())
        packed = np.ascontiguousarray(c1["packed"])
        n, k = c1["n"], c1["k"]
        threads = max(1, min(16, os.cpu_count() or 1))  # the box's CPU share for one GPU
        bounds = [n * i // threads for i in range(threads + 1)]
        acc = np.zeros((1, n), np.int32)
        pointer = lambda a: a.ctypes.data_as(ctypes.c_void_p)

        def slice_dot(i, a_q):  # rows [bounds[i], bounds[i + 1]) of the matrix; ctypes releases the GIL
            lo, hi = bounds[i], bounds[i + 1]
            part = np.zeros((1, hi - lo), np.int32)
            clib.orc_q4_dot(pointer(table), pointer(packed[lo:hi]), pointer(a_q), ctypes.c_int64(1),
                            ctypes.c_int64(hi - lo), ctypes.c_int64(k), pointer(part))
            acc[0, lo:hi] = part[0]

        pool = ThreadPoolExecutor(threads)

        def cpu_once():
            a_q, a_s = orc.a8(c1["x"])
            a_q = np.ascontiguousarray(a_q)
            list(pool.map(lambda i: slice_dot(i, a_q), range(threads)))
            return orc.rescale(acc, c1["scales"], a_s[:, 0])

        check_q, check_s = orc.a8(c1["x"])
        expected = orc.project(check_q, check_s[:, 0], orc.q4_integers(packed[:64], table), c1["scales"][:64])
        if not np.array_equal(cpu_once()[:, :64], expected):
            raise SystemExit("the C restatement disagrees with the numpy oracle")
        calls, spent = 0, 0.0
        while spent < 10.0 and calls < 5000:         # bounded sample: about 10 s of host work
            t0 = time.perf_counter()
            cpu_once()
            spent += time.perf_counter() - t0
            calls += 1
        pool.shutdown()
        cpu_seconds = spent / calls
        result["cpu_baseline"] = {
            "value": round(bytes_c1 / cpu_seconds / 1e9, 4), "unit": "GB/s", "cores": threads, "kind": "port",
            "seconds_per_call": round(cpu_seconds, 4), "host_cpus": os.cpu_count(), "calls": calls,
            "sample": "mean of `calls` full calls on config 1, M=1: A8 (numpy), decode of 11.1M two-stage codes fused "
                      "with the exact dot (oracle/e8p_oracle.c, scalar C, the matrix rows split over `cores` threads), "
                      "rescale (numpy); about 10 s in total",
        }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
