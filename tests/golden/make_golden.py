"""Writes tests/golden/ref_vectors.npz from oracle/_ref/libcwick_ref.so, i.e. from the
reference's own C files (src/ds_ops.c, src/tensor.c, src/util.c) compiled where they lie
by oracle/Makefile.  Run in a container that has /root/reference:

    make -C oracle && python tests/golden/make_golden.py

The vectors are data (inputs and the outputs the reference's object code gave); they let
the oracle be checked on machines where the reference tree does not exist.
"""
import ctypes as C
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import orc  # noqa: E402

R = orc.ref()
assert R is not None, "build oracle/_ref first (make -C oracle)"
out = {}

# E4M3 decode: cwick_fp8_e4m3_to_f32 (src/tensor.c:354-368) on all 256 bytes
out["e4m3_table"] = np.array([R.cwick_fp8_e4m3_to_f32(b) for b in range(256)], np.float32)

# bf16: cwick_f32_to_bf16 (src/util.c:202-210), ds_bf16_round (src/ds_ops.c:89-96)
g = np.random.Generator(np.random.Philox(2024))
x = np.concatenate([g.standard_normal(2000) * 5, [0.0, -0.0, 0.5, 1.0, 1.5, -2.0, 3.5, 123.25, 1e-5],
                    np.float32(1.0) + np.arange(64) * np.float32(2.0 ** -9)]).astype(np.float32)
out["bf16_in"] = x
out["bf16_cwick"] = np.array([R.cwick_f32_to_bf16(float(v)) for v in x], np.uint16)
out["bf16_round"] = np.array([R.ds_bf16_round(float(v)) for v in x], np.float32)

# softmax: cwick_softmax (src/tensor.c:793-803) and ds_softmax (src/ds_ops.c:100-107)
s = (g.standard_normal(3000) * 4).astype(np.float32)
out["softmax_in"] = s
a = s.copy()
R.cwick_softmax(a.ctypes.data_as(C.POINTER(C.c_float)), C.c_int64(a.size))
out["softmax_out"] = a
b = s.copy()
R.ds_softmax(b.ctypes.data_as(C.POINTER(C.c_float)), C.c_int(b.size))
out["ds_softmax_out"] = b

# ds_topk_scores (src/ds_ops.c:310-338): tie-free, tied, all-equal, -inf, k >= n
cases = []
cases.append((g.standard_normal(4096).astype(np.float32), 512))
cases.append((g.integers(-5, 5, 3000).astype(np.float32), 512))
cases.append((np.full(100, 2.0, np.float32), 10))
cases.append((np.array([5, 5, 7], np.float32), 2))
cases.append((np.array([3, 9, 3, 3, 8, 3], np.float32), 4))
c = g.standard_normal(1000).astype(np.float32)
c[g.random(1000) < 0.6] = -np.inf
cases.append((c, 512))
cases.append((g.standard_normal(20).astype(np.float32), 20))
cases.append((g.integers(0, 3, 65536).astype(np.float32), 2048))
out["topk_ncases"] = np.int64(len(cases))
for i, (sc, k) in enumerate(cases):
    out["topk_sc_%d" % i] = sc
    out["topk_k_%d" % i] = np.int64(k)
    out["topk_out_%d" % i] = orc.ref_topk_scores(sc, k)

np.savez_compressed(os.path.join(ROOT, "tests", "golden", "ref_vectors.npz"), **out)
print("wrote", len(out), "arrays")
