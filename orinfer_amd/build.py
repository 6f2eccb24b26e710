"""Builds liborx.so (HIP kernels + C ABI) for gfx950 with hipcc.  Usage: python -m orinfer_amd.build"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

HERE = Path(__file__).resolve().parent
CSRC = HERE / "csrc"
LIBRARY = HERE / "liborx.so"
SOURCES = ["orx_api.cpp", "k_quant.hip", "k_gemv.hip", "k_gemm.hip", "k_gemm_big.hip", "k_stream.hip", "k_dense.hip", "k_wide.hip", "k_grouped.hip", "k_moe.hip", "k_planes.hip", "k_rowq4.hip"]
# -packed-fp32-ops off: this pool has seen wrong results from compiler-made v_pk_*_f32.
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-x", "hip",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # no contraction: the epilogue's two fp32 multiplies and the fp16 cast must each round on their
    # own (a fused multiply+convert rounds once and differs from the reference in the last bit)
    "-ffp-contract=off",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes", "-Wno-unused-command-line-argument",
]
FIXTURE_RUNNER = HERE / "orx_run_fixture"


def hipcc():
    return os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


def build(verbose=True):
    objects = []

    def compile_one(name):
        obj = CSRC / (Path(name).stem + ".o")
        cmd = [hipcc(), *FLAGS, "-c", str(CSRC / name), "-o", str(obj)]
        if verbose:
            print(" ".join(cmd), flush=True)
        done = subprocess.run(cmd, capture_output=True, text=True)
        text = "\n".join(l for l in (done.stdout + done.stderr).splitlines()
                         if "packed-fp32-ops" not in l and "is not a recognized feature" not in l)
        if done.returncode != 0:
            raise RuntimeError(f"hipcc failed on {name}:\n{text}")
        if verbose and text.strip():
            print(text)
        return obj

    with ThreadPoolExecutor(max_workers=4) as pool:
        objects = list(pool.map(compile_one, SOURCES))
    link = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIBRARY), *map(str, objects)]
    if verbose:
        print(" ".join(link), flush=True)
    subprocess.check_call(link)
    runner_src = CSRC / "orx_run_fixture.cpp"
    if runner_src.exists():
        cmd = [hipcc(), "--offload-arch=gfx950", "-O2", "-std=c++17", "-x", "hip",
               "-Wno-unused-command-line-argument", str(runner_src),
               "-o", str(FIXTURE_RUNNER), f"-L{HERE}", "-lorx", f"-Wl,-rpath,$ORIGIN"]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd)
    return LIBRARY


if __name__ == "__main__":
    build()
    print("built", LIBRARY)
    sys.exit(0)
