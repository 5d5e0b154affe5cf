"""Contracts that hold without a GPU: the bench refuses more than one GPU, the product has no CPU fallback, and nothing
outside tests/, the smoke entry and the bench's CPU-baseline leg touches the oracle."""
import os
import re
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_bench_refuses_more_than_one_gpu():
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, cwd=ROOT)
    assert out.returncode != 0
    assert "--gpus must be 1" in out.stderr
    assert out.stdout.strip() == ""


def test_missing_library_is_an_error_not_a_fallback(monkeypatch, tmp_path):
    from zllm_amd import capi

    monkeypatch.setattr(capi, "_lib", None)
    monkeypatch.setattr(capi, "LIB_PATH", str(tmp_path / "libzllm_attn.so"))
    with pytest.raises(FileNotFoundError, match="no CPU fallback"):
        capi.load()


def test_product_code_does_not_use_the_oracle():
    """Only tests/, __graft_entry__.smoke() and the benches' cpu_baseline leg may import or link anything under oracle/."""
    offenders = []
    for folder, _, files in os.walk(os.path.join(ROOT, "zllm_amd")):
        for name in files:
            if not name.endswith((".py", ".hip", ".hpp", ".cpp", ".h")):
                continue
            path = os.path.join(folder, name)
            text = open(path, encoding="utf-8", errors="replace").read()
            for number, line in enumerate(text.splitlines(), 1):
                if re.search(r"^\s*(import oracle|from oracle)\b|zllm_oracle|oracle/", line):
                    offenders.append((os.path.relpath(path, ROOT), number, line.strip()))
    # the build script links the host layer's parity driver (a test) against the oracle; nothing else may name it
    allowed = {"zllm_amd/build.py"}
    assert [o for o in offenders if o[0] not in allowed] == []
    assert "oracle_dir" in open(os.path.join(ROOT, "zllm_amd", "build.py")).read()


def test_the_probe_kernels_are_not_part_of_the_library():
    """bench.py's plain-read kernels live in their own shared object; the drop-in ABI exports no measurement aid."""
    header = open(os.path.join(ROOT, "include", "zllm_attn.h")).read()
    assert "probe" not in header
    for folder, _, files in os.walk(os.path.join(ROOT, "zllm_amd")):
        for name in files:
            if name.endswith((".py", ".hip", ".hpp", ".cpp", ".h")):
                assert "stream_read" not in open(os.path.join(folder, name), encoding="utf-8", errors="replace").read(), name
