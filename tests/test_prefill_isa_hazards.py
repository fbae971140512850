"""The fast loop of the prefill kernel issues its MFMAs from inline assembly, which the compiler's hazard recogniser
does not see.  This test compiles prefill.hip to gfx950 ISA and checks, for every MFMA that sits inside an inline
assembly block, that
  * no vector-ALU instruction writes one of its source registers in the two instructions before it (the compiler
    rebuilding a constant or copying a register right in front of the MFMA), and
  * no other instruction touches its result in the six instructions after it.
Loads from LDS / scratch into the sources are ordered by s_waitcnt, which the compiler does insert for inline assembly."""
import os
import re
import shutil
import subprocess
import tempfile

import pytest

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


def _regs(tok):
    m = re.fullmatch(r"[av]\[(\d+):(\d+)\]", tok)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.fullmatch(r"-?\|?v(\d+)\|?", tok)
    return {int(m.group(1))} if m else set()


def _instructions(text):
    """(line number, opcode, operands, inside inline assembly) for every instruction line."""
    out, in_asm = [], False
    for i, raw in enumerate(text.split("\n")):
        if "#ASMSTART" in raw:
            in_asm = True
            continue
        if "#ASMEND" in raw:
            in_asm = False
            continue
        line = raw.split(";")[0].strip()
        if not line or line.endswith(":") or line.startswith("."):
            continue
        parts = line.split(None, 1)
        ops = [t.strip().split(" ")[0] for t in parts[1].split(",")] if len(parts) > 1 else []
        out.append((i + 1, parts[0], ops, in_asm))
    return out


def find_hazards(text):
    ins, bad = _instructions(text), []
    for idx, (ln, op, ops, in_asm) in enumerate(ins):
        if not (in_asm and op.startswith("v_mfma")):
            continue
        dst = _regs(ops[0])
        srcs = set().union(*[_regs(t) for t in ops[1:4]])
        for back in (1, 2):
            if idx - back < 0:
                break
            l2, op2, ops2, _ = ins[idx - back]
            if op2.startswith("v_") and not op2.startswith(("v_mfma", "v_cmp")) and ops2 and (_regs(ops2[0]) & srcs):
                bad.append("line %d: source of the MFMA written by %s at line %d" % (ln, op2, l2))
        for fwd in range(1, 7):
            if idx + fwd >= len(ins):
                break
            l2, op2, ops2, _ = ins[idx + fwd]
            if op2.startswith(("v_mfma", "s_")):
                continue
            if set().union(*[_regs(t) for t in ops2] or [set()]) & dst:
                bad.append("line %d: result of the MFMA touched by %s at line %d" % (ln, op2, l2))
    return ins, bad


def test_scanner_flags_the_patterns_it_is_meant_to():
    text = """
	v_mov_b64_e32 v[112:113], s[10:11]
	;;#ASMSTART
	v_mfma_f32_16x16x32_f16 v[62:65], v[110:113], v[218:221], v[62:65]
	;;#ASMEND
	v_mul_f32_e32 v62, v1, v62
	;;#ASMSTART
	v_mfma_f32_16x16x32_f16 v[50:53], v[114:117], v[218:221], v[50:53]
	;;#ASMEND
	ds_read_b128 v[114:117], v3
	v_mfma_f32_16x16x32_f16 v[10:13], v[114:117], v[218:221], v[10:13]
	v_add_f32_e32 v10, v10, v10
"""
    _, bad = find_hazards(text)
    assert len(bad) == 2 and "written by v_mov_b64_e32" in bad[0] and "touched by v_mul_f32_e32" in bad[1], bad


@pytest.mark.skipif(shutil.which(HIPCC) is None, reason="hipcc not available")
def test_no_vector_write_next_to_an_inline_assembly_mfma():
    # the library's own compile flags, from the build recipe (loaded by path: it does not need the built library)
    import importlib.util
    spec = importlib.util.spec_from_file_location("_lsattn_build_flags", os.path.join(REPO, "loongserve_amd", "build.py"))
    recipe = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(recipe)
    src = os.path.join(REPO, "loongserve_amd", "csrc", "prefill.hip")
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "prefill.s")
        cmd = [recipe.HIPCC, *recipe.FLAGS, *recipe.FILE_FLAGS.get("prefill.hip", []), "-S", "--cuda-device-only", src, "-o", out]
        subprocess.run(cmd, check=True, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
        text = open(out).read()
    ins, bad = find_hazards(text)
    n_asm_mfma = sum(1 for _, op, _, in_asm in ins if in_asm and op.startswith("v_mfma"))
    assert n_asm_mfma >= 9 * 8 * 34, n_asm_mfma   # nine kernels (dtype / V route x three epilogues), eight unrolled phases of 34 MFMAs
    assert not bad, "\n".join(bad[:20])
