"""Builds libzllm_attn.so (the C-ABI library) for gfx950 with hipcc, in-tree."""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libzllm_attn.so")
SOURCES = ["api.hip", "append.hip", "gqa_decode.hip", "mla_decode.hip", "mla_partial_x32.hip", "mla_generic.hip", "gqa_prefill.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    # packed-FP32 VALU forms are kept out of all device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-Wno-unknown-warning-option",
]


def _compile(src: str) -> str:
    obj = os.path.join(CSRC, src.replace(".hip", ".o"))
    cmd = [HIPCC, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    result = subprocess.run(cmd, capture_output=True, text=True)
    if result.returncode != 0:
        sys.stderr.write(result.stdout + result.stderr)
        raise RuntimeError(f"hipcc failed on {src}")
    noise = "'-packed-fp32-ops' is not a recognized feature"
    for line in result.stderr.splitlines():
        if line.strip() and noise not in line and "warning generated" not in line and "warnings generated" not in line:
            sys.stderr.write(line + "\n")
    return obj


def build_library(jobs: int = 6) -> str:
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objects = list(pool.map(_compile, SOURCES))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objects]
    subprocess.check_call(cmd)
    return LIB


BACKEND_LIB = os.path.join(HERE, "libzllm_backend.so")
HOST_TEST = os.path.join(os.path.dirname(HERE), "tests", "host", "backend_parity")


def build_host_layer() -> str:
    """The C++ host layer above the C ABI (zllm_amd/host) as libzllm_backend.so; needs libzllm_attn.so."""
    cmd = [HIPCC, "--offload-arch=gfx950", "-O2", "-std=c++17", "-fPIC", "-shared", "-o", BACKEND_LIB,
           os.path.join(HERE, "host", "rocm_backend.cpp"), "-L" + HERE, "-lzllm_attn", "-Wl,-rpath,$ORIGIN"]
    subprocess.check_call(cmd)
    return BACKEND_LIB


def build_host_test(oracle_dir: str) -> str:
    """tests/host/backend_parity: the host layer's parity driver; links the CPU oracle (checker only)."""
    cmd = [HIPCC, "--offload-arch=gfx950", "-O2", "-std=c++17", "-o", HOST_TEST, HOST_TEST + ".cpp", "-L" + HERE, "-lzllm_backend",
           "-lzllm_attn", "-L" + oracle_dir, "-lzllm_oracle", "-Wl,-rpath,$ORIGIN/../../zllm_amd", "-Wl,-rpath,$ORIGIN/../../oracle"]
    subprocess.check_call(cmd)
    return HOST_TEST


BENCH_PROBE = os.path.join(os.path.dirname(HERE), "libbench_probe.so")


def build_bench_probe() -> str:
    """bench.py's plain-read measurement kernels (bench_probe.hip beside bench.py); not part of the attention library."""
    cmd = [HIPCC, *FLAGS, "-shared", "-o", BENCH_PROBE, os.path.join(os.path.dirname(HERE), "bench_probe.hip")]
    subprocess.check_call(cmd, stderr=subprocess.DEVNULL)
    return BENCH_PROBE


if __name__ == "__main__":
    print(build_library())
    print(build_host_layer())
    print(build_bench_probe())
