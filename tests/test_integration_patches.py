"""The guards of INTEGRATION.md as patches against the engine's own files (integration/*.patch:
added lines only): each applies to a copy of the reference file it names and the patched file
compiles as C11 against the engine's headers and include/cwick_hip.h, with the backend compiled in
(-DCWICK_WITH_HIP) and without it.  No link step: the engine cannot be linked here.  Runs only
where the reference tree is present."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF = "/root/reference/src"
PATCHES = {"attention.c": "attention_hip.patch", "ds_model.c": "ds_model_hip.patch", "main.c": "main_hip.patch"}

pytestmark = pytest.mark.skipif(not os.path.isdir(REF), reason="the reference tree is not on this machine")


@pytest.mark.parametrize("name", sorted(PATCHES))
def test_guard_patch_applies_and_compiles(name, tmp_path):
    patch = os.path.join(ROOT, "integration", PATCHES[name])
    text = open(patch).read()
    body = [l for l in text.splitlines() if not l.startswith(("---", "+++", "@@"))]
    assert body and all(l.startswith("+") for l in body), "the patch must hold added lines only"
    src = tmp_path / "src"
    src.mkdir()
    shutil.copy(os.path.join(REF, name), src / name)
    r = subprocess.run(["patch", "-p1", "--no-backup-if-mismatch", "-i", patch], cwd=tmp_path, capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "cwick_hip_" in (src / name).read_text()
    for defs in (["-DCWICK_WITH_HIP"], []):
        cmd = ["gcc", "-std=gnu11", "-c", "-Wall", "-Werror=implicit-function-declaration",
               "-Werror=incompatible-pointer-types", "-Werror=int-conversion", "-Werror=jump-misses-init",
               "-I", str(src), "-I", REF, "-I", os.path.join(ROOT, "include")] + defs + [
               str(src / name), "-o", str(tmp_path / "out.o")]
        r = subprocess.run(cmd, capture_output=True, text=True)
        assert r.returncode == 0, " ".join(cmd) + "\n" + r.stderr[-4000:]
