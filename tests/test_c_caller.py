"""tests/c_caller/guard_sequence.c is a C11 program that includes include/cwick_hip.h, links
-lcwick_hip and runs the guard sequence an engine would (create -> write_f32 -> decode ->
deselect -> decline -> CPU loop -> select again), checking every result against its own
double-precision loops.  __graft_entry__.build() compiles it; the tests run the binary."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "c_caller", "guard_sequence")


def _run():
    assert os.path.exists(EXE), "build it first: make -C tests/c_caller (or __graft_entry__.build())"
    return subprocess.run([EXE], capture_output=True, text=True, timeout=120)


def test_c_program_builds_against_the_header_and_library():
    subprocess.check_call(["make", "-C", os.path.join(ROOT, "tests", "c_caller"), "-B"])
    out = subprocess.check_output(["ldd", EXE], text=True)
    assert "libcwick_hip.so" in out and "not found" not in out


@pytest.mark.skipif(os.path.exists("/dev/kfd"), reason="a GPU is present")
def test_c_program_declines_cleanly_without_a_gpu():
    r = _run()
    assert r.returncode == 0, r.stdout + r.stderr
    assert "backend: unavailable" in r.stdout and "declines: clean" in r.stdout


@pytest.mark.gpu
def test_c_program_guard_sequence_on_the_gpu():
    print("[case] C caller: guard sequence", flush=True)
    r = _run()
    print(r.stdout, flush=True)
    assert r.returncode == 0, r.stdout + r.stderr
    for line in ("mla_decode (GPU)", "mla_decode after force(0)", "declined", "untouched", "mla_decode after force(1)",
                 "mla_decode over sel[] with -1", "kv_write_f32 narrows with RNE", "bit-equal", "gqa_decode (GPU)"):
        assert line in r.stdout, line
    assert r.stdout.strip().endswith("OK")
