"""Build libcwick_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

    python -m cwick_amd.build            # compile what changed, link
    python -m cwick_amd.build --force    # recompile everything

The library lands in cwick_amd/lib/ so that it travels with the source tree.
"""
import concurrent.futures as cf
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
OBJDIR = os.path.join(LIBDIR, "obj")
LIB = os.path.join(LIBDIR, "libcwick_hip.so")

SOURCES = ["runtime.hip", "misc.hip", "gqa_decode.hip", "gqa_prefill.hip", "mla_roles.hip",
           "indexer.hip", "indexer_band.hip", "topk.hip", "probe.hip", "prep.hip", "mla_prefill64.hip", "mm_select.hip"]

COMMON = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
          "-Wall", "-Wno-unused-function",
          # packed-fp32 VALU forms are kept out of every kernel in this library
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
# the indexer's summation order is a contract: nothing may be fused behind its back
PER_FILE = {"indexer.hip": ["-ffp-contract=off"], "indexer_band.hip": ["-ffp-contract=off"]}


def _hipcc():
    for c in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if c and (os.path.isabs(c) and os.path.exists(c) or not os.path.isabs(c)):
            return c
    return "hipcc"


def _compile(src, force):
    obj = os.path.join(OBJDIR, src.replace(".hip", ".o"))
    path = os.path.join(CSRC, src)
    deps = [path, os.path.join(HERE, "..", "include", "cwick_hip.h"), os.path.abspath(__file__)]
    deps += [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hpp")]
    if not force and os.path.exists(obj) and all(
            os.path.getmtime(obj) >= os.path.getmtime(d) for d in deps):
        return obj, ""
    cmd = [_hipcc()] + COMMON + PER_FILE.get(src, []) + ["-c", path, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    log = "\n".join(l for l in (r.stdout + r.stderr).splitlines()
                    if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, log))
    return obj, log


def build(force=False, verbose=True):
    os.makedirs(OBJDIR, exist_ok=True)
    with cf.ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        results = list(ex.map(lambda s: _compile(s, force), SOURCES))
    objs = [o for o, _ in results]
    for (_, log), src in zip(results, SOURCES):
        if verbose and log.strip():
            print("[%s]\n%s" % (src, log))
    need_link = force or not os.path.exists(LIB) or any(
        os.path.getmtime(o) > os.path.getmtime(LIB) for o in objs)
    if need_link:
        # only the C ABI of include/cwick_hip.h leaves the library
        cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC",
               "-Wl,--version-script=" + os.path.join(CSRC, "exports.map"), "-o", LIB] + objs
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed:\n" + r.stdout + r.stderr)
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build(force="--force" in sys.argv)
