"""The backend's guards as patches against the engine's own files (integration/*.patch:
added lines only): each applies to a copy of the reference file it names and the patched file
compiles as C11 against the engine's headers and include/cwick_hip.h, with the backend compiled in
(-DCWICK_WITH_HIP) and without it.  No link step: the engine cannot be linked here.  Runs only
where the reference tree is present.

src/q35_model.c is written for NEON and does not compile on this machine as it stands (vector types
and intrinsics outside any #if); its patch is applied and the compiler is run over the patched file
for diagnostics only: none of them may lie inside the added lines, and the patched file may not
have more errors than the original."""
import os
import re
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


def _diagnostics(path, inc, defs):
    cmd = ["gcc", "-std=gnu11", "-fsyntax-only", "-fmax-errors=0", "-Wall", "-I", inc, "-I", REF,
           "-I", os.path.join(ROOT, "include")] + defs + [path]
    r = subprocess.run(cmd, capture_output=True, text=True)
    out = []
    for l in r.stderr.splitlines():
        m = re.match(r"^%s:(\d+):\d+: (error|warning): (.*)$" % re.escape(path), l)
        if m:
            out.append((int(m.group(1)), m.group(2), m.group(3)))
    return out


def test_q35_guard_patch_applies_and_its_lines_draw_no_diagnostics(tmp_path):
    patch = os.path.join(ROOT, "integration", "q35_model_hip.patch")
    text = open(patch).read()
    body = [l for l in text.splitlines() if not l.startswith(("---", "+++", "@@"))]
    assert body and all(l.startswith("+") for l in body), "the patch must hold added lines only"
    src = tmp_path / "src"
    src.mkdir()
    shutil.copy(os.path.join(REF, "q35_model.c"), src / "q35_model.c")
    base = _diagnostics(str(src / "q35_model.c"), str(src), ["-DCWICK_WITH_HIP"])
    r = subprocess.run(["patch", "-p1", "--no-backup-if-mismatch", "-i", patch], cwd=tmp_path, capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
    # the added line ranges in the patched file, from the hunk headers (@@ -a,0 +b,n @@)
    added = []
    for m in re.finditer(r"^@@ -\d+(?:,\d+)? \+(\d+)(?:,(\d+))? @@", text, re.M):
        added.append((int(m.group(1)), int(m.group(1)) + int(m.group(2) or 1)))
    assert len(added) == 3
    patched = (src / "q35_model.c").read_text().splitlines()
    assert any("cwick_hip_gqa_prefill" in patched[i - 1] for a, b in added for i in range(a, b))
    diags = _diagnostics(str(src / "q35_model.c"), str(src), ["-DCWICK_WITH_HIP"])
    inside = [d for d in diags if any(a <= d[0] < b for a, b in added)]
    assert not inside, inside
    n_err = lambda ds: sum(1 for d in ds if d[1] == "error")
    assert n_err(base) > 0                      # the file does not build here even unpatched
    assert n_err(diags) == n_err(base), (n_err(diags), n_err(base))
    # and with the backend compiled out the patch changes nothing for the compiler
    assert n_err(_diagnostics(str(src / "q35_model.c"), str(src), [])) == n_err(base)
