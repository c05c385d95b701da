"""The C ABI from a C++ host program (tests/cabi/cabi_check.cpp): no Python between the caller and
the library.  The CPU test compiles it against the header and the built library; the GPU test runs
the prebuilt binary, which checks prefill, decode steps and a captured HIP graph of them against the
CPU oracle byte for byte."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "tests", "cabi", "cabi_check.cpp")
BIN = os.path.join(ROOT, "tests", "cabi", "cabi_check")
LIBDIR = os.path.join(ROOT, "viby-model_amd", "causal_conv1d")


def test_cpp_host_program_compiles_and_links(tmp_path):
    out = tmp_path / "cabi_check"
    subprocess.check_call([
        "/opt/rocm/bin/hipcc", "-O1", "-std=c++17", "--offload-arch=gfx950", f"-I{ROOT}/include", "-o", str(out), SRC,
        f"-L{LIBDIR}", "-lcanon_conv1d", "-ldl"], stderr=subprocess.DEVNULL)
    assert out.exists()


@pytest.mark.gpu
def test_cpp_host_program_matches_the_oracle():
    assert os.path.exists(BIN), f"{BIN} is not built: run `make -C tests/cabi` (or __graft_entry__.build())"
    from oracle import canon_oracle
    r = subprocess.run([BIN, canon_oracle.build()], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and "cabi_check: OK" in r.stdout, r.stdout + r.stderr
