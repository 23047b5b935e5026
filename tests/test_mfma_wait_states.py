"""The kernels that issue matrix instructions from inline assembly (to pin their accumulators to
VGPRs) hide them from the compiler's hazard recognizer, which would otherwise put two wait states
between a vector-ALU write of a register and the MFMA that reads it as an operand.  The sources
place `s_nop 1` where such a write comes last; this test compiles them to assembly and checks the
rule on what the compiler scheduled: no vector-ALU instruction that writes an MFMA's A or B operand
may be one of the two instructions in front of it, and no instruction may read an MFMA's result
within nineteen wait states of it (thirteen for the eight-pass scaled FP8 instruction) unless it is an MFMA accumulating into it.  (Violations give wrong numbers only now and
then, depending on timing, which is why the rule is checked on the code and not on results.)"""
import os
import re
import subprocess
import tempfile

import pytest

from cwick_amd import build as B

ASM_MFMA_SOURCES = ["gqa_prefill.hip", "indexer_band.hip", "mla_prefill64.hip"]


def _regs(tok):
    m = re.match(r"v\[(\d+):(\d+)\]", tok)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"v(\d+)$", tok)
    return {int(m.group(1))} if m else set()


@pytest.mark.parametrize("src", ASM_MFMA_SOURCES)
def test_no_valu_write_right_before_an_mfma_reads_it(src):
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "k.s")
        cmd = [B._hipcc()] + B.COMMON + B.PER_FILE.get(src, []) + [
            "-w", "-S", "--cuda-device-only", os.path.join(B.CSRC, src), "-o", out]
        r = subprocess.run(cmd, capture_output=True, text=True)
        assert r.returncode == 0, r.stderr[-2000:]
        ins, from_asm, in_asm = [], [], False
        for line in open(out):
            t = line.strip()
            if t.startswith(";;#ASMSTART"):
                in_asm = True
            elif t.startswith(";;#ASMEND"):
                in_asm = False
            if not t or t.startswith((";", ".")) or t.endswith(":"):
                continue
            ins.append(t)
            from_asm.append(in_asm)
    n_mfma, bad, early = 0, [], []
    for i, t in enumerate(ins):
        if not t.startswith("v_mfma"):
            continue
        n_mfma += from_asm[i]
        ops = [o.strip() for o in t.split(None, 1)[1].split(",")]
        src_regs = _regs(ops[1]) | _regs(ops[2])
        for back in (1, 2):
            p = ins[i - back]
            # (an MFMA that the compiler issued itself is its own business: it knows what it wrote)
            if from_asm[i] and p.startswith("v_") and not p.startswith("v_mfma"):
                dst = _regs(p.split(None, 1)[1].split(",")[0].strip())
                if dst & src_regs:
                    bad.append((p, t))
        # The other direction: a result must not be read by anything but an MFMA that accumulates
        # into it before the matrix pipe has written it.  The compiler's own figure for the
        # longest MFMA is 19 wait states (an s_nop N counts N + 1, any other instruction 1);
        # the scan follows straight-line code and stops at a branch or after 24.
        dst_regs = _regs(ops[0])
        waited = 0
        for q in ins[i + 1:i + 64]:
            if q.startswith(("s_cbranch", "s_branch", "s_endpgm")) or waited >= 24:
                break
            qops = [o.strip() for o in q.split(None, 1)[1].split(",")] if " " in q else []
            reads = set()
            for o in (qops[1:] if q.startswith("v_") and not q.startswith("v_mfma") else qops):
                reads |= _regs(o.split()[0]) if o else set()
            if q.startswith("v_mfma"):
                reads = _regs(qops[1]) | _regs(qops[2])          # accumulating into the result is allowed
            # (the scaled FP8 16x16x128 instruction takes eight passes: the compiler's figure for an
            # eight-pass result is eleven wait states, twelve on this chip; thirteen are asked here)
            need = 13 if t.startswith("v_mfma_scale_f32_16x16x128") else 19
            if reads & dst_regs and waited < need:
                early.append((t[:60], q[:60], waited))
                break
            m = re.match(r"s_nop (\d+)", q)
            waited += int(m.group(1)) + 1 if m else 1
    assert n_mfma > 0
    assert not bad, "VALU write within two instructions of the MFMA that reads it: %r" % bad[:3]
    assert not early, "MFMA result read before the matrix pipe has written it: %r" % early[:3]


LDS_DMA_SOURCES = ["mla_roles.hip", "mla_prefill64.hip", "gqa_prefill.hip"]


@pytest.mark.parametrize("src", LDS_DMA_SOURCES)
def test_m0_belongs_to_the_lds_copies_only(src):
    """The global -> LDS copies are issued from inline assembly that sets M0 (the LDS address)
    itself.  M0 is reserved to the compiler and cannot be declared clobbered, so the sources rely
    on the compiler having no use of M0 of its own in these kernels: on the compiled code, every
    instruction that names m0 must be the `s_mov_b32 m0, sN` of a copy statement, followed by its
    `s_nop 0` and its `global_load_lds_*`, and every such load must follow one."""
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "k.s")
        cmd = [B._hipcc()] + B.COMMON + B.PER_FILE.get(src, []) + [
            "-w", "-S", "--cuda-device-only", os.path.join(B.CSRC, src), "-o", out]
        r = subprocess.run(cmd, capture_output=True, text=True)
        assert r.returncode == 0, r.stderr[-2000:]
        ins = []
        for line in open(out):
            t = line.split(";")[0].strip()
            if not t or t.startswith(".") or t.endswith(":"):
                continue
            ins.append(t)
    n_copies = 0
    for i, t in enumerate(ins):
        if re.search(r"\bm0\b", t):
            assert re.match(r"s_mov_b32 m0, s\d+$", t), "compiler-generated use of m0: " + t
            assert ins[i + 1] == "s_nop 0" and ins[i + 2].startswith("global_load_lds_"), ins[i:i + 3]
        if t.startswith("global_load_lds_"):
            n_copies += 1
            assert ins[i - 2].startswith("s_mov_b32 m0,") and ins[i - 1] == "s_nop 0", ins[i - 2:i + 1]
    assert n_copies > 0
