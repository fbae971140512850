"""The fast loop of the prefill kernel issues its MFMAs from inline assembly, which the compiler's hazard recogniser
does not see.  This test compiles prefill.hip to gfx950 ISA and checks, for every MFMA that sits inside an inline
assembly block, that
  * no vector-ALU instruction writes one of its source registers in the two instructions before it (the compiler
    rebuilding a constant or copying a register right in front of the MFMA), and
  * no other instruction touches its result in the six instructions after it.
Loads from LDS / scratch into the sources are ordered by s_waitcnt, which the compiler does insert for inline assembly.

The K/V tile loads (global -> LDS, and global -> registers for a bfloat16 V) are issued from inline assembly too, with
hand-placed `s_waitcnt vmcnt(N)`: the compiler neither counts them nor waits for them.  For every loop of every kernel
that holds such loads the test checks the budget the pipeline is built on: after a group of tile loads, and before the
next group is issued, there is a wait that leaves at most that one group in flight (so the group before it has landed),
and a workgroup barrier follows that wait before the next group goes out (the other waves' parts have landed too before
anyone reads the tile, and nobody still reads the slot the next loads overwrite).  In the kernels that take fp16 V tiles
no other vector-memory instruction (a register spill) sits in those loops: its compiler-placed vmcnt(0) would wait for
the tile loads just issued.

decode.hip orders DPP additions by hand: a DPP operand needs two wait states after a vector write of it, so no vector
instruction may write the DPP source of an inline-assembly DPP instruction in the two instructions before it."""
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


_DEVICE_ASM = {}


def _device_asm(source):
    """The device assembly of a file of loongserve_amd/csrc under the library's own compile flags, from the build recipe
    (loaded by path: it does not need the built library); compiled once per session."""
    if source not in _DEVICE_ASM:
        import importlib.util
        spec = importlib.util.spec_from_file_location("_lsattn_build_flags", os.path.join(REPO, "loongserve_amd", "build.py"))
        recipe = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(recipe)
        src = os.path.join(REPO, "loongserve_amd", "csrc", source)
        with tempfile.TemporaryDirectory() as tmp:
            out = os.path.join(tmp, source + ".s")
            cmd = [recipe.HIPCC, *recipe.FLAGS, *recipe.FILE_FLAGS.get(source, []), "-S", "--cuda-device-only", src, "-o", out]
            subprocess.run(cmd, check=True, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
            _DEVICE_ASM[source] = open(out).read()
    return _DEVICE_ASM[source]


@pytest.mark.skipif(shutil.which(HIPCC) is None, reason="hipcc not available")
def test_no_vector_write_next_to_an_inline_assembly_mfma():
    text = _device_asm("prefill.hip")
    ins, bad = find_hazards(text)
    n_asm_mfma = sum(1 for _, op, _, in_asm in ins if in_asm and op.startswith("v_mfma"))
    # twenty-one kernels (dtype / V route / workgroup shape x three epilogues); the 256-row ones hold eight unrolled
    # plain phases of 34 MFMAs and eight masked ones of 32, the four-wave ones four of each
    assert n_asm_mfma >= (15 * 4 + 6 * 2) * (34 + 32), n_asm_mfma
    assert not bad, "\n".join(bad[:20])
    bad = tile_load_budget_violations(text)
    assert not bad, "\n".join(bad[:20])


def _kernels(text):
    """{kernel symbol: its lines} for every prefill_kernel instantiation in the assembly text."""
    out, name = {}, None
    for raw in text.split("\n"):
        m = re.match(r"^(_ZN6lsattn14prefill_kernel\w+):", raw)
        if m:
            name = m.group(1)
            out[name] = []
        elif raw.startswith("\t.end_amdhsa_kernel") or raw.startswith(".Lfunc_end"):
            name = None
        if name:
            out[name].append(raw)
    return out


def _loops(lines):
    """(first line index, last line index) of every loop: a label and a later branch back to it.  (A block that only ends
    the program, placed early in the text and branched back to by later exits, is no loop.)"""
    labels = {}
    loops = []
    for i, raw in enumerate(lines):
        m = re.match(r"^(\.LBB\d+_\d+):", raw)
        if m:
            labels[m.group(1)] = i
        m = re.match(r"^\s+s_cbranch_\w+\s+(\.LBB\d+_\d+)", raw) or re.match(r"^\s+s_branch\s+(\.LBB\d+_\d+)", raw)
        if m and m.group(1) in labels:
            first = next((l.split(";")[0].strip() for l in lines[labels[m.group(1)] + 1:] if l.split(";")[0].strip()), "")
            if first != "s_endpgm":
                loops.append((labels[m.group(1)], i))
    return loops


def tile_load_budget_violations(text, min_loops=2 * 21):
    """Plays the vector-memory counter over every loop that issues tile loads (three trips; loads complete in order, a
    wait for vmcnt(n) retires all but the n youngest) and reports, in the steady state:
      * a group of global -> LDS loads issued while a group older than the previous one is still in flight,
      * a group of global -> LDS loads issued after a hand-placed wait (vmcnt(n), n > 0) retired LDS loads with no
        barrier in between,
      * (fp16-V kernels) any other vector-memory instruction in the loop."""
    bad = []
    n_loops = 0
    for name, lines in _kernels(text).items():
        fp16_v = bool(re.search(r"ELi\dELb1ELb[01]E", name))  # DV = true
        for lo, hi in _loops(lines):
            ev, in_asm = [], False  # ("L",) load to LDS, ("R",) load to registers, ("W", n), ("B",), ("X", text) other vmem
            for raw in lines[lo:hi + 1]:
                if "#ASMSTART" in raw:
                    in_asm = True
                    continue
                if "#ASMEND" in raw:
                    in_asm = False
                    continue
                ins = raw.split(";")[0].strip()
                if not ins:
                    continue
                op = ins.split()[0]
                if op.startswith(("global_", "scratch_", "buffer_", "flat_")):
                    if in_asm and op.startswith("global_load_lds"):
                        ev.append(("L",))
                    elif in_asm and op.startswith("global_load"):
                        ev.append(("R",))
                    else:
                        ev.append(("X", ins))
                elif op == "s_waitcnt":
                    m = re.search(r"vmcnt\((\d+)\)", ins)
                    if m:
                        ev.append(("W", int(m.group(1))))
                elif op == "s_barrier":
                    ev.append(("B",))
            if not any(e[0] == "L" for e in ev):
                continue
            n_loops += 1
            if fp16_v:
                bad += ["%s: %s inside a loop with tile loads" % (name, e[1]) for e in ev if e[0] == "X"]
            ev = [e for e in ev if e[0] != "X"]
            queue, group, prev, need_barrier = [], 0, None, False  # queue of (LDS group id or None), oldest first
            found = set()
            for trip in range(3):
                for e in ev:
                    if e[0] == "L":
                        if prev != "L":
                            group += 1
                            older = {g for g in queue if g is not None and g < group - 1}
                            if trip and older:
                                found.add("%s: tile loads issued with more than the previous group still in flight" % name)
                            if trip and need_barrier:
                                found.add("%s: tile loads issued after a wait for earlier ones with no barrier in between" % name)
                        queue.append(group)
                    elif e[0] == "R":
                        queue.append(None)
                    elif e[0] == "W":
                        done, queue = queue[:max(len(queue) - e[1], 0)], queue[max(len(queue) - e[1], 0):]
                        # (a vmcnt(0) in a loop is the compiler's, behind a spill reload: it only makes this wave wait
                        # longer and is not the wait the pipeline relies on)
                        if e[1] > 0 and any(g is not None for g in done):
                            need_barrier = True
                    elif e[0] == "B":
                        need_barrier = False
                    prev = e[0]
            bad += sorted(found)
    assert n_loops >= min_loops, n_loops  # a plain and a masked loop in each of the twenty-one kernels
    return bad


def test_budget_scanner_flags_a_lax_wait():
    ok = """_ZN6lsattn14prefill_kernelINS_3F16ELi0ELb1ELb0EEEvNS_13PrefillParamsE:
.LBB0_1:
	;;#ASMSTART
	global_load_lds_dwordx4 v1, s[2:3]
	global_load_lds_dwordx4 v2, s[2:3]
	;;#ASMEND
	s_barrier
	s_waitcnt vmcnt(%d)
	s_barrier
	s_cbranch_scc1 .LBB0_1
"""
    scan = lambda t: tile_load_budget_violations(t, min_loops=1)
    assert not scan(ok % 2)
    assert any("still in flight" in b for b in scan(ok % 3))
    assert any("no barrier" in b for b in scan((ok % 2).replace("\ts_barrier\n\ts_cbranch", "\ts_cbranch")))
    assert any("inside a loop" in b for b in scan((ok % 2).replace("\ts_barrier\n\ts_waitcnt", "\tscratch_load_dword v3, off, off\n\ts_barrier\n\ts_waitcnt")))


def find_dpp_hazards(text):
    ins, bad = _instructions(text), []
    for idx, (ln, op, ops, in_asm) in enumerate(ins):
        if not (in_asm and op.endswith("_dpp")):
            continue
        srcs = set().union(*[_regs(t) for t in ops[1:3]])
        for back in (1, 2):
            if idx - back < 0:
                break
            l2, op2, ops2, _ = ins[idx - back]
            if op2.startswith("v_") and not op2.startswith("v_cmp") and ops2 and (_regs(ops2[0]) & srcs):
                bad.append("line %d: DPP source written by %s at line %d" % (ln, op2, l2))
    return ins, bad


def test_dpp_scanner_flags_a_close_write():
    text = """
	;;#ASMSTART
	v_dot2c_f32_f16 v5, v1, v2
	;;#ASMEND
	v_mov_b32_e32 v7, v5
	;;#ASMSTART
	v_add_f32_dpp v9, v7, v7 row_ror:8 row_mask:0xf bank_mask:0x3
	;;#ASMEND
	;;#ASMSTART
	v_add_f32_dpp v10, v5, v5 row_ror:8 row_mask:0xf bank_mask:0x3
	;;#ASMEND
"""
    _, bad = find_dpp_hazards(text)
    assert len(bad) == 1 and "written by v_mov_b32_e32" in bad[0], bad


def _decode_asm():
    """The device assembly of decode.hip under the library's own flags (compiled once per session)."""
    return _device_asm("decode.hip")


@pytest.mark.skipif(shutil.which(HIPCC) is None, reason="hipcc not available")
def test_no_vector_write_next_to_an_inline_assembly_dpp_in_decode():
    ins, bad = find_dpp_hazards(_decode_asm())
    assert sum(1 for _, op, _, in_asm in ins if in_asm and op.endswith("_dpp")) >= 1000
    assert not bad, "\n".join(bad[:20])


def loads_in_flight_violations(text, kernel_pattern):
    """The matrix-pipe decode kernel issues its global loads from inline assembly and waits for them with hand-placed
    `s_waitcnt vmcnt(N)`; the compiler knows of neither, so nothing but data flow through the asm operands keeps it from
    using a destination register early.  Walk each matching kernel in program order: a register that such a load is still
    to write (vmcnt retires loads oldest first: `vmcnt(N)` leaves the N youngest in flight) may appear in no instruction,
    not even as the address of the next load.  Returns {kernel: (asm loads seen, violations)}.  The walk is linear over the
    text; a loop's back edge is covered by the prologue putting the counters into the state the loop's end leaves."""
    res, kernels, name = {}, {}, None
    for ln, raw in enumerate(text.split("\n"), 1):
        m = re.match(r"^(_ZN6lsattn\w+):", raw)
        if m:
            name = m.group(1)
            kernels[name] = []
        elif raw.startswith("\t.end_amdhsa_kernel") or raw.startswith(".Lfunc_end"):
            name = None
        if name:
            kernels[name].append((ln, raw))
    for name, lines in kernels.items():
        if kernel_pattern not in name:
            continue
        pending, bad, in_asm, nload = {}, [], False, 0
        for ln, raw in lines:
            if "#ASMSTART" in raw:
                in_asm = True
                continue
            if "#ASMEND" in raw:
                in_asm = False
                continue
            ins = raw.split(";")[0].strip()
            if not ins or ins.endswith(":") or ins.startswith("."):
                continue
            parts = ins.split(None, 1)
            op = parts[0]
            ops = [t.strip().split(" ")[0] for t in parts[1].split(",")] if len(parts) > 1 else []
            if op == "s_waitcnt":
                m = re.search(r"vmcnt\((\d+)\)", ins)
                if m:
                    n = int(m.group(1))
                    pending = {r: v for r, v in pending.items() if v > nload - n}  # (v: the load's number in issue order)
                continue
            touched = set().union(*[_regs(t) for t in ops]) if ops else set()
            if in_asm and op.startswith("global_load_lds_dword"):
                # a load into LDS: it counts for vmcnt like any other and writes no register
                nload += 1
                hit = touched & set(pending)
                if hit:
                    bad.append("line %d: %s addresses with v%s, which a load in flight writes" % (ln, ins, sorted(hit)))
                continue
            if in_asm and op.startswith("global_load_dword"):
                nload += 1
                hit = set().union(*[_regs(t) for t in ops[1:]]) & set(pending) if len(ops) > 1 else set()
                if hit:
                    bad.append("line %d: %s addresses with v%s, which a load in flight writes" % (ln, ins, sorted(hit)))
                for r in _regs(ops[0]):
                    pending[r] = nload
                continue
            hit = touched & set(pending)
            if hit:
                bad.append("line %d: %s touches v%s, which a load in flight writes" % (ln, ins, sorted(hit)))
        res[name] = (nload, bad)
    return res


def test_in_flight_scanner_flags_an_early_use():
    text = """
_ZN6lsattn4demoEv:
	;;#ASMSTART
	global_load_dwordx4 v[4:7], v[20:21], off nt
	;;#ASMEND
	;;#ASMSTART
	global_load_dwordx4 v[8:11], v[22:23], off nt
	;;#ASMEND
	;;#ASMSTART
	s_waitcnt vmcnt(1)
	;;#ASMEND
	v_add_f32_e32 v30, v4, v5
	%s
	;;#ASMSTART
	s_waitcnt vmcnt(0)
	;;#ASMEND
	v_add_f32_e32 v31, v8, v9
	s_endpgm
.Lfunc_end0:
"""
    (n, bad), = loads_in_flight_violations(text % "v_mov_b32_e32 v32, v6", "demo").values()
    assert n == 2 and not bad, bad
    (n, bad), = loads_in_flight_violations(text % "v_mov_b32_e32 v32, v10", "demo").values()
    assert len(bad) == 1 and "touches v[10]" in bad[0], bad


@pytest.mark.skipif(shutil.which(HIPCC) is None, reason="hipcc not available")
def test_decode_matrix_pipe_kernel_touches_no_register_of_a_load_in_flight():
    res = loads_in_flight_violations(_decode_asm(), "decode_stage1_mfma_")
    # fp16 and bf16: plain, with the waves of a workgroup splitting a block, the plain shape over a list of units, and the
    # plain shape over every wave's equal share of the blocks
    assert len(res) == 8 and sum("listed" in name for name in res) == 2 and sum("range" in name for name in res) == 2, list(res)
    for name, (n, bad) in res.items():
        assert n >= 3 * 8 + 3 * 16, (name, n)             # slot and row loads of the prologue and of both halves of the loop
        assert not bad, name + "\n" + "\n".join(bad[:20])


@pytest.mark.skipif(shutil.which(HIPCC) is None, reason="hipcc not available")
def test_inline_assembly_stores_of_a_partial_keep_their_data_registers_for_two_cycles():
    """The matrix-pipe decode kernel stores a partial's row from inline assembly (the compiler has no plain store with the
    system-scope bits).  A vector instruction may not overwrite the data registers of a store of more than 64 bits in
    the two cycles behind it; the compiler's hazard recogniser covers its own stores only, so every such store must be
    followed by `s_nop 1` (or more) inside the same assembly block."""
    for src in ("decode.hip", "ceiling.hip", "prefill.hip"):
        raw = _device_asm(src).split("\n")
        lines = [ln.split(";")[0].strip() for ln in raw]
        seen, in_asm = 0, False
        for i, ins in enumerate(lines):
            if "#ASMSTART" in raw[i]:
                in_asm = True
            if "#ASMEND" in raw[i]:
                in_asm = False
            if in_asm and ins.startswith("global_store_dwordx"):
                seen += 1
                nxt = next(x for x in lines[i + 1:] if x)
                m = re.match(r"s_nop (\d+)", nxt)
                assert m and int(m.group(1)) >= 1, "%s line %d: %s is followed by %s" % (src, i + 1, ins, nxt)
        assert seen >= 8, (src, seen)
