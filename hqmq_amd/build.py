"""Builds hqmq_amd/libhqmq_amd.so from hqmq_amd/csrc/*.hip with hipcc for gfx950, and beside it
hqmq_amd/libhqmq_bench.so from hqmq_amd/csrc_bench/*.hip: the read-only measurement kernels that bench.py and
hqmq_amd/bench_ceiling.py time (nothing in the product path loads that one).

    python -m hqmq_amd.build            # compile (always) and link
    python -m hqmq_amd.build --stamps   # also hqmq_amd/libhqmq_amd_stamps.so: the same library with attention_fast.hip compiled
                                        # with -DHQMQ_STAMPS (time stamps inside the LDS-landing attention kernel, read by
                                        # hqmq_amd/bench_stamps.py; a measurement build, never loaded by the package itself)

The kernels that decide integers (codeword index, radius code, Med3x mask) are
compiled with -ffp-contract=off so that every written float operation rounds
on its own; the attention kernels keep the default contraction.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

HERE = Path(__file__).resolve().parent
CSRC = HERE / "csrc"
OUT = HERE / "libhqmq_amd.so"
BENCH_SRC = HERE / "csrc_bench"
BENCH_OUT = HERE / "libhqmq_bench.so"

COMMON = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-function",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
EXACT = {"joint.hip", "quantize.hip", "med3x.hip", "dequant.hip"}


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(exe).exists():
        raise RuntimeError("hipcc not found; libhqmq_amd.so cannot be built")
    return exe


def build(verbose: bool = False, stamps: bool = False) -> Path:
    cc = hipcc()
    objdir = HERE / "build"
    objdir.mkdir(exist_ok=True)
    srcs = sorted(CSRC.glob("*.hip"))
    if not srcs:
        raise RuntimeError(f"no sources under {CSRC}")

    def compile_one(src: Path) -> Path:
        obj = objdir / (src.stem + ".o")
        cmd = [cc, *COMMON, "-c", str(src), "-o", str(obj)]
        if src.name in EXACT:
            cmd.insert(1, "-ffp-contract=off")
        if src.name == "quantize.hip":      # MFMA results straight into VGPRs: the search loop reads them at once
            cmd[1:1] = ["-mllvm", "-amdgpu-mfma-vgpr-form"]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if verbose or r.returncode:
            sys.stderr.write(" ".join(cmd) + "\n" + r.stdout + r.stderr)
        if r.returncode:
            raise RuntimeError(f"hipcc failed on {src.name}")
        return obj

    bench_srcs = sorted(BENCH_SRC.glob("*.hip"))
    with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as ex:
        all_objs = list(ex.map(compile_one, srcs + bench_srcs))
    objs, bench_objs = all_objs[:len(srcs)], all_objs[len(srcs):]
    cmd = [cc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(OUT), *map(str, objs)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode:
        sys.stderr.write(r.stdout + r.stderr)
        raise RuntimeError("link failed")
    if bench_objs:
        cmd = [cc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(BENCH_OUT), *map(str, bench_objs)]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode:
            sys.stderr.write(r.stdout + r.stderr)
            raise RuntimeError("link of the measurement library failed")
    if stamps:
        obj = objdir / "attention_fast_stamps.o"
        cmd = [cc, *COMMON, "-DHQMQ_STAMPS", "-c", str(CSRC / "attention_fast.hip"), "-o", str(obj)]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode:
            sys.stderr.write(r.stdout + r.stderr)
            raise RuntimeError("hipcc failed on attention_fast.hip (stamps)")
        others = [o for o in objs if o.name != "attention_fast.o"]
        cmd = [cc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(HERE / "libhqmq_amd_stamps.so"), *map(str, others), str(obj)]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode:
            sys.stderr.write(r.stdout + r.stderr)
            raise RuntimeError("link of the stamps build failed")
    return OUT


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv, stamps="--stamps" in sys.argv))
