"""The C-ABI library loads, exports every symbol include/cwick_hip.h declares and
nothing else, and declines cleanly where there is no GPU (no compute is called here)."""
import ctypes
import os
import re
import subprocess
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "cwick_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cwick_hip_[a-z0-9_]+)\s*\(", text)))


def test_header_compiles_as_c(tmp_path):
    src = tmp_path / "t.c"
    src.write_text('#include "cwick_hip.h"\nint main(void){return sizeof(cwick_hip_kv*) ? 0 : 1;}\n')
    subprocess.check_call(["gcc", "-std=c11", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"),
                           "-c", str(src), "-o", str(tmp_path / "t.o")])


def test_library_exports_exactly_the_header():
    from cwick_amd import hip
    L = hip.lib()
    names = declared_symbols()
    assert len(names) >= 38
    for n in names:
        assert hasattr(L, n), "libcwick_hip.so does not export " + n
        assert n in hip.SIGNATURES, "cwick_amd/hip.py has no binding for " + n
    out = subprocess.check_output(["nm", "-D", "--defined-only", hip.LIB_PATH], text=True)
    exported = sorted(l.split()[-1] for l in out.splitlines() if " T " in l)
    assert exported == names, set(exported) ^ set(names)


def test_no_torch_and_no_oracle_in_the_product():
    """The shipped package must not route through the CPU oracle or any fallback."""
    for dirpath, _, files in os.walk(os.path.join(ROOT, "cwick_amd")):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.replace("the CPU oracle", ""), f
    out = subprocess.check_output(["ldd", os.path.join(ROOT, "cwick_amd", "lib", "libcwick_hip.so")],
                                  text=True)
    assert "torch" not in out and "oracle" not in out


@pytest.mark.skipif(os.path.exists("/dev/kfd"), reason="a GPU is present")
def test_declines_without_a_gpu():
    from cwick_amd import hip
    L = hip.lib()
    assert L.cwick_hip_ready() == 0
    assert hip.last_error() != ""
    out = np.zeros(4, np.float32)
    got = ctypes.c_int64(-1)
    rc = L.cwick_hip_topk(out.ctypes.data, 4, 2, out.ctypes.data, ctypes.byref(got))
    assert rc == 0 and got.value == -1            # outputs untouched
    assert L.cwick_hip_kv_create(16, 4, 256) is None
    assert L.cwick_hip_force(0) == 0 and L.cwick_hip_ready() == 0
    assert "not selected" in hip.last_error() or "unavailable" in hip.last_error()


def test_bench_refuses_more_than_one_gpu():
    """bench.py shows one GPU's share of the path: --gpus N with N above 1 ends with a message
    that says so, before anything touches a device."""
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0
    assert "--gpus 2 is not run" in r.stderr + r.stdout
    assert not r.stdout.strip().startswith("{")
