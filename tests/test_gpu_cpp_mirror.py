"""GPU parity of the C++ host mirror (include/ckks_llm_amd.hpp): runs the test program built from tests/cpp, which calls
the mirror's member functions the way the reference's test programs call the reference's and compares every result with
the CPU oracle bit for bit."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))


def test_cpp_mirror_program_passes():
    exe = os.path.join(HERE, "cpp", "test_cpp_mirror.bin")
    assert os.path.exists(exe), "tests/cpp/test_cpp_mirror.bin is not built (run __graft_entry__.build())"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    print(r.stdout[-3000:], r.stderr[-2000:])
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-2000:]
    assert "all C++ mirror checks passed" in r.stdout


def test_reference_pcmm_test_program_flow_passes():
    """tests/cpp/test_rlwe_decomp_flow.cpp: the reference's test_rlwe_decomp.cu replayed against the mirror (no oracle involved:
    its check is the program's own comparison with the plain matrix product)."""
    exe = os.path.join(HERE, "cpp", "test_rlwe_decomp_flow.bin")
    assert os.path.exists(exe), "tests/cpp/test_rlwe_decomp_flow.bin is not built (run __graft_entry__.build())"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    print(r.stdout[-3000:], r.stderr[-2000:])
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-2000:]
    assert "the reference's PCMM test flow passed" in r.stdout
