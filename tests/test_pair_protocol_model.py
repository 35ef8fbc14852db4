"""The hand-over protocol of the one-launch transforms (claim, take over, defer, finish: ckks_llm_amd/csrc/pair_protocol.hpp) run on
the host with one thread per workgroup: tests/cpp/pair_protocol_model.cpp compiles the device header's decision functions for the CPU
and drives them through residency limits down to a single workgroup, every start order, late starters, spin limits from zero
upwards, the form that never takes a tile over, launches in a row on the same words and two sets of words that share the residency
slots.  CPU only."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
CPP = os.path.join(HERE, "cpp")


def test_protocol_model_finds_no_violation():
    exe = os.path.join(CPP, "pair_protocol_model.bin")
    if not os.path.exists(exe):
        subprocess.check_call(["make", "-C", CPP, "pair_protocol_model.bin"], stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    r = subprocess.run([exe, "3"], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, (r.stdout[-2000:], r.stderr[-2000:])
    assert " 0 violations" in r.stdout, r.stdout
