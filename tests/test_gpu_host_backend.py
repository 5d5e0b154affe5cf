"""Runs the C++ host layer's parity driver (tests/host/backend_parity.cpp): the reference-shaped backend methods
(gqa_prefill_attention and its _visible form over dense K/V, gqa_prefill_attention_cached and its _visible / _from forms,
block_attention and its prefix + suffix form with the reference's own vectors, append_mla, append_mla_rope,
mla_decode_attention, mla_prefill_attention) over the C ABI, compared with the CPU oracle inside the driver, plus their
error behaviour, the grow-by-doubling rule of the cache planes, the ring of a sliding-window layer, and the counters that
show a decode loop in steady state neither allocating, nor uploading rotary tables again, nor waiting for its stream.  The binary is built by __graft_entry__.build()."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BINARY = os.path.join(ROOT, "tests", "host", "backend_parity")


def test_cpp_backend_mirror_matches_oracle():
    assert os.path.exists(BINARY), f"{BINARY} is missing: run `python -c 'import __graft_entry__ as g; g.build()'`"
    done = subprocess.run([BINARY], capture_output=True, text=True, timeout=110)
    print(done.stdout)
    print(done.stderr)
    assert done.returncode == 0, done.stdout[-2000:] + done.stderr[-2000:]
    assert "ALL PASSED" in done.stdout
