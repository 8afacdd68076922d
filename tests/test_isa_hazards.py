"""Static checks of the generated gfx950 code (CPU only): hazards that the compiler's hazard recogniser
cannot see because the instructions involved are inline assembly.

1. The four-wave GEMM kernels issue their MFMAs as inline assembly (to pin the accumulators to the
   accumulation registers), so the compiler neither knows that they are MFMAs nor inserts the wait states
   that a read of an MFMA result needs.  The source places a wait at the end of a tile's last K iteration
   (`mfma_retire` in triton_amd/csrc/gemm_wave128.h); the test proves on the assembly the build keeps
   that on EVERY control-flow path from an MFMA to a non-MFMA instruction reading an accumulation
   register at least MIN_WAIT issue slots pass (an 8-pass MFMA needs 11 by the CDNA3/CDNA4 ISA guides'
   table of required software wait states; `s_nop N` counts N + 1, any other instruction 1).
2. Every kernel issues its direct global->LDS loads (and some plain loads) as inline assembly with a
   scalar base address.  A vector-memory instruction must not read a scalar register within 5 issue
   slots of a VALU instruction writing it (v_readlane_b32 - which is how the compiler restores a SPILLED
   scalar register -, v_readfirstlane_b32, VALU compares and carries): it would see the old value.  For
   instructions it knows the compiler inserts the wait states itself; for inline assembly nobody does.
   (A block-scaled fp8 product came out wrong in a few per cent of runs on cold caches that way: a
   spilled tile base, restored right in front of a load of the prologue, made the load fetch eight rows
   from a stale address.)
"""
import os
import re

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BUILD = os.path.join(HERE, "..", "triton_amd", "csrc", "_build")
ASM = [os.path.join(BUILD, f"{stem}-hip-amdgcn-amd-amdhsa-gfx950.s") for stem in ("gemm_wave128", "gemm_wave128_mx")]
MIN_WAIT = 12
FAR = 1 << 20

AGPR = re.compile(r"\ba(\d+|\[\d+:\d+\])")


def _functions(text):
    cur, out = None, {}
    for line in text.split("\n"):
        m = re.match(r"^(_Z\w+):", line)
        if m:
            cur = m.group(1)
            out[cur] = []
        elif cur is not None:
            if line.startswith("\t.end_amdhsa_kernel") or line.startswith(".Lfunc_end"):
                cur = None
            else:
                out[cur].append(line)
    return out


def _blocks(lines):
    """[(label, [instruction, ...])] in layout order; instructions are stripped text without comments."""
    blocks = [("entry", [])]
    for line in lines:
        code = line.split(";")[0].rstrip()
        if not code.strip():
            continue
        m = re.match(r"^(\.LBB\w+):", code)
        if m:
            blocks.append((m.group(1), []))
        elif code.startswith("\t") and not code.strip().startswith("."):
            blocks[-1][1].append(code.strip())
    return blocks


def _regs(token_text):
    """Accumulation registers named in an operand string: 'a[4:7], a9' -> {4, 5, 6, 7, 9}."""
    out = set()
    for m in AGPR.finditer(token_text):
        t = m.group(1)
        if t.startswith("["):
            lo, hi = t[1:-1].split(":")
            out.update(range(int(lo), int(hi) + 1))
        else:
            out.add(int(t))
    return out


def check_function(lines):
    """Returns a list of (block label, instruction, wait states since the MFMA that wrote the register)
    violations.  State: for every accumulation register written by an MFMA fewer than MIN_WAIT issue slots
    ago, the number of slots since; merged over control-flow paths by taking the minimum."""
    blocks = _blocks(lines)
    index = {lab: i for i, (lab, _) in enumerate(blocks)}
    succ = []
    for i, (_, ins) in enumerate(blocks):
        s = set()
        fall = True
        for t in ins:
            m = re.match(r"s_c?branch\w*\s+(\.LBB\w+)", t)
            if m:
                s.add(index[m.group(1)])
            if t.startswith("s_branch") or t.startswith("s_endpgm") or t.startswith("s_setpc"):
                fall = False
        if fall and i + 1 < len(blocks):
            s.add(i + 1)
        succ.append(s)

    def walk(ins, state, report, label):
        state = dict(state)
        for t in ins:
            op = t.split()[0]
            operands = t[len(op):]
            if op.startswith("v_mfma") or op.startswith("v_smfmac"):
                # (an MFMA reading its own accumulator as the addend is interlocked by the hardware)
                for r in _regs(operands.split(",", 1)[0]):
                    state[r] = 0
                step = 1
            else:
                is_store = op.startswith(("global_store", "buffer_store", "ds_write", "scratch_store", "flat_store"))
                srcs = operands if is_store else (operands.split(",", 1)[1] if "," in operands else "")
                for r in _regs(srcs):
                    if r in state and report is not None:
                        report.append((label, t, state[r]))
                m = re.match(r"s_nop\s+(\d+)", t)
                step = int(m.group(1)) + 1 if m else 1
            state = {r: d + step for r, d in state.items() if d + step < MIN_WAIT}
        return state

    entry = [dict() for _ in blocks]
    work = list(range(len(blocks)))
    while work:
        i = work.pop()
        out = walk(blocks[i][1], entry[i], None, None)
        for j in succ[i]:
            changed = False
            for r, d in out.items():
                if entry[j].get(r, FAR) > d:
                    entry[j][r] = d
                    changed = True
            if changed:
                work.append(j)
    bad = []
    for i, (lab, ins) in enumerate(blocks):
        walk(ins, entry[i], bad, lab)
    return bad


def test_checker_flags_an_early_read_and_accepts_a_late_one():
    early = ["\tv_mfma_f32_16x16x32_bf16 a[0:3], v[0:3], v[4:7], a[0:3]", "\ts_nop 3", "\tv_accvgpr_read_b32 v9, a0"]
    late = ["\tv_mfma_f32_16x16x32_bf16 a[0:3], v[0:3], v[4:7], a[0:3]", "\ts_nop 15", "\tv_accvgpr_read_b32 v9, a0"]
    loop = ["\ts_branch .LBB0_2", ".LBB0_1:", "\tv_accvgpr_read_b32 v9, a0", "\ts_endpgm", ".LBB0_2:",
            "\tv_mfma_f32_16x16x32_bf16 a[0:3], v[0:3], v[4:7], a[0:3]", "\ts_cbranch_scc1 .LBB0_2", "\ts_branch .LBB0_1"]
    assert check_function(early) and not check_function(late)
    assert check_function(loop)          # the read sits before the loop in the text but behind it in control flow


def test_no_accumulator_is_read_before_the_last_mfmas_retire():
    if not all(os.path.exists(f) for f in ASM):
        pytest.skip("device assembly not kept: build the library first (python -m triton_amd.build)")
    kernels = {}
    for f in ASM:
        kernels.update({k: v for k, v in _functions(open(f).read()).items() if "gemm_wave128" in k})
    assert len(kernels) >= 16, sorted(kernels)
    for name, lines in kernels.items():
        assert sum("v_mfma" in l for l in lines) >= 64, name     # (the smallest form: two K steps of 32, fp8 on 128-row tiles)
        bad = check_function(lines)
        assert not bad, (name, bad[:5])


SGPR_WAIT = 5
VALU_SGPR_WRITERS = ("v_readlane_b32", "v_readfirstlane_b32", "v_cmp", "v_cmpx", "v_add_co", "v_sub_co", "v_subrev_co",
                     "v_addc_co", "v_subb_co", "v_div_scale", "v_mad_u64_u32", "v_mad_i64_i32")
SGPR = re.compile(r"\bs(\d+|\[\d+:\d+\])")


def _sregs(text):
    out = set()
    for m in SGPR.finditer(text):
        t = m.group(1)
        if t.startswith("["):
            lo, hi = t[1:-1].split(":")
            out.update(range(int(lo), int(hi) + 1))
        else:
            out.add(int(t))
    return out


def check_sgpr_to_vmem(lines):
    """Violations (block label, instruction, slots since the VALU write) of rule 2, over all control-flow
    paths (same fixed point as check_function, on scalar registers written by VALU instructions)."""
    blocks = _blocks(lines)
    index = {lab: i for i, (lab, _) in enumerate(blocks)}
    succ = []
    for i, (_, ins) in enumerate(blocks):
        s, fall = set(), True
        for t in ins:
            m = re.match(r"s_c?branch\w*\s+(\.LBB\w+)", t)
            if m:
                s.add(index[m.group(1)])
            if t.startswith("s_branch") or t.startswith("s_endpgm") or t.startswith("s_setpc"):
                fall = False
        if fall and i + 1 < len(blocks):
            s.add(i + 1)
        succ.append(s)

    def walk(ins, state, report, label):
        state = dict(state)
        for t in ins:
            op = t.split()[0]
            operands = t[len(op):]
            if op.startswith(("global_", "buffer_", "scratch_", "flat_")):
                for r in _sregs(operands):
                    if r in state and report is not None:
                        report.append((label, t, state[r]))
            m = re.match(r"s_nop\s+(\d+)", t)
            step = int(m.group(1)) + 1 if m else 1
            state = {r: d + step for r, d in state.items() if d + step < SGPR_WAIT}
            if op.startswith(VALU_SGPR_WRITERS):
                dst = operands.split(",", 1)[0] if op.startswith(("v_readlane", "v_readfirstlane", "v_cmp")) else operands
                for r in _sregs(dst):
                    state[r] = 0
        return state

    entry = [dict() for _ in blocks]
    work = list(range(len(blocks)))
    while work:
        i = work.pop()
        out = walk(blocks[i][1], entry[i], None, None)
        for j in succ[i]:
            changed = False
            for r, d in out.items():
                if entry[j].get(r, FAR) > d:
                    entry[j][r] = d
                    changed = True
            if changed:
                work.append(j)
    bad = []
    for i, (lab, ins) in enumerate(blocks):
        walk(ins, entry[i], bad, lab)
    return bad


def test_sgpr_checker_flags_a_restored_spill_in_front_of_a_load():
    early = ["\tv_readlane_b32 s9, v255, 15", "\tglobal_load_lds_dwordx4 v0, s[8:9] offset:16"]
    late = ["\tv_readlane_b32 s9, v255, 15", "\ts_nop 4", "\tglobal_load_lds_dwordx4 v0, s[8:9] offset:16"]
    other = ["\tv_readlane_b32 s11, v255, 15", "\tglobal_load_lds_dwordx4 v0, s[8:9] offset:16"]
    assert check_sgpr_to_vmem(early) and not check_sgpr_to_vmem(late) and not check_sgpr_to_vmem(other)


def test_no_vector_memory_instruction_reads_a_scalar_register_too_soon_after_a_valu_write():
    import glob

    files = sorted(glob.glob(os.path.join(BUILD, "*-hip-amdgcn-amd-amdhsa-gfx950.s")))
    if len(files) < 10:
        pytest.skip("device assembly not kept: build the library first (python -m triton_amd.build)")
    checked = 0
    for f in files:
        for name, lines in _functions(open(f).read()).items():
            if not any(l.lstrip().startswith(("global_", "buffer_", "scratch_", "flat_")) for l in lines):
                continue
            checked += 1
            bad = check_sgpr_to_vmem(lines)
            assert not bad, (os.path.basename(f), name, bad[:5])
    assert checked >= 40, checked


VGPR = re.compile(r"\bv(\d+|\[\d+:\d+\])")
LDS_QUEUE_CAP = 96


def _vregs(text):
    out = set()
    for m in VGPR.finditer(text):
        t = m.group(1)
        if t.startswith("["):
            lo, hi = t[1:-1].split(":")
            out.update(range(int(lo), int(hi) + 1))
        else:
            out.add(int(t))
    return out


def check_lds_reads_in_flight(lines):
    """Rule 3: violations (block label, instruction, registers) where an instruction reads or writes a vector
    register that an LDS read issued earlier has not delivered yet.  LDS (and scalar memory) operations
    retire in order against one counter; `s_waitcnt lgkmcnt(N)` leaves the N youngest outstanding.  The state
    is the queue of outstanding operations (the destination registers of each), kept per control-flow path."""
    blocks = _blocks(lines)
    index = {lab: i for i, (lab, _) in enumerate(blocks)}
    succ = []
    for i, (_, ins) in enumerate(blocks):
        s, fall = set(), True
        for t in ins:
            m = re.match(r"s_c?branch\w*\s+(\.LBB\w+)", t)
            if m:
                s.add(index[m.group(1)])
            if t.startswith("s_branch") or t.startswith("s_endpgm") or t.startswith("s_setpc"):
                fall = False
        if fall and i + 1 < len(blocks):
            s.add(i + 1)
        succ.append(s)

    def walk(ins, queue, report, label):
        queue = list(queue)
        for t in ins:
            op = t.split()[0]
            operands = t[len(op):]
            if op == "s_waitcnt":
                m = re.search(r"lgkmcnt\((\d+)\)", operands)
                if m:
                    keep = int(m.group(1))
                    queue = queue[len(queue) - keep:] if keep < len(queue) else queue
                    if keep == 0:
                        queue = []
                continue
            flying = set().union(*queue) if queue else set()
            if op.startswith(("ds_read", "ds_load")):
                dst, src = operands.split(",", 1)
                hit = _vregs(src) & flying
                queue.append(frozenset(_vregs(dst)))
            elif op.startswith(("ds_", "s_load", "s_buffer_load")):
                hit = _vregs(operands) & flying
                queue.append(frozenset())
            else:
                hit = _vregs(operands) & flying
            if hit and report is not None:
                report.append((label, t, sorted(hit)))
            queue = queue[-LDS_QUEUE_CAP:]
        return tuple(queue)

    entry = [set() for _ in blocks]
    entry[0].add(())
    work = [(0, ())]
    while work:
        i, q = work.pop()
        out = walk(blocks[i][1], q, None, None)
        for j in succ[i]:
            if out not in entry[j]:
                assert len(entry[j]) < 512, "too many distinct LDS queues reach one block"
                entry[j].add(out)
                work.append((j, out))
    bad = []
    for i, (lab, ins) in enumerate(blocks):
        for q in entry[i]:
            walk(ins, q, bad, lab)
    return bad


def test_lds_checker_flags_a_register_reused_before_the_wait():
    # the shape of the defect it was written for: operands of a step that does not follow are read at the end of a
    # loop, and the epilogue's first values are placed in those registers ahead of the wait
    racy = ["\tds_read_b128 v[32:35], v7 offset:64", "\tv_accvgpr_read_b32 v33, a1", "\ts_waitcnt lgkmcnt(0)"]
    fine = ["\tds_read_b128 v[32:35], v7 offset:64", "\ts_waitcnt lgkmcnt(0)", "\tv_accvgpr_read_b32 v33, a1"]
    partial = ["\tds_read_b128 v[32:35], v7", "\tds_read_b128 v[36:39], v7 offset:64", "\ts_waitcnt lgkmcnt(1)",
               "\tv_mov_b32_e32 v0, v32", "\ts_waitcnt lgkmcnt(0)"]
    partial_bad = partial[:3] + ["\tv_mov_b32_e32 v0, v36"] + partial[4:]
    loop = ["\ts_branch .LBB0_2", ".LBB0_1:", "\tv_mov_b32_e32 v32, 0", "\ts_waitcnt lgkmcnt(0)", "\ts_endpgm", ".LBB0_2:",
            "\ts_waitcnt lgkmcnt(0)", "\tds_read_b128 v[32:35], v7", "\ts_cbranch_scc1 .LBB0_2", "\ts_branch .LBB0_1"]
    assert check_lds_reads_in_flight(racy) and not check_lds_reads_in_flight(fine)
    assert not check_lds_reads_in_flight(partial) and check_lds_reads_in_flight(partial_bad)
    assert check_lds_reads_in_flight(loop)


def test_no_register_is_touched_while_an_lds_read_into_it_is_in_flight():
    import glob

    files = sorted(glob.glob(os.path.join(BUILD, "*-hip-amdgcn-amd-amdhsa-gfx950.s")))
    if len(files) < 10:
        pytest.skip("device assembly not kept: build the library first (python -m triton_amd.build)")
    checked = 0
    for f in files:
        for name, lines in _functions(open(f).read()).items():
            if not any(l.lstrip().startswith("ds_read") for l in lines):
                continue
            checked += 1
            bad = check_lds_reads_in_flight(lines)
            assert not bad, (os.path.basename(f), name, bad[:5])
    assert checked >= 40, checked


def check_m0_owner(lines):
    """Rule 4: an LDS-direct load takes its LDS address from M0.  The kernels set M0 inside inline assembly for
    their own such loads while the compiler sets it for the loads it generates from the builtin; each load must see
    the M0 written by its own side.  Returns (instruction, who wrote M0) for every compiler-generated load whose M0
    was last written inside inline assembly, and for every inline-assembly load whose M0 was last written by the
    compiler (unknown at a label: code reached by a branch is not followed)."""
    bad, in_asm, owner = [], False, None
    for line in lines:
        if "#ASMSTART" in line:
            in_asm = True
            continue
        if "#ASMEND" in line:
            in_asm = False
            continue
        code = line.split(";")[0].strip()
        if not code:
            continue
        if re.match(r"^\.LBB\w+:", code):
            owner = None
            continue
        op = code.split()[0]
        operands = code[len(op):]
        if op.startswith(("global_load_lds", "buffer_load")) and ("lds" in op or " lds" in operands):
            mine = "asm" if in_asm else "compiler"
            if owner is not None and owner != mine:
                bad.append((code, owner))
        elif op.startswith("s_") and re.match(r"\s*m0\b", operands):
            owner = "asm" if in_asm else "compiler"
    return bad


def test_m0_checker_flags_a_compiler_write_moved_in_front_of_an_assembly_copy():
    swapped = ["\ts_add_i32 m0, s9, 0x4000", "\t;;#ASMSTART", "\ts_mov_b32 m0, s33", "\ts_nop 0",
               "\tglobal_load_lds_dwordx4 v147, s[26:27]", "\t;;#ASMEND", "\tglobal_load_lds_dword v[24:25], off"]
    right = swapped[1:6] + [swapped[0], swapped[6]]
    assert check_m0_owner(swapped) == [("global_load_lds_dword v[24:25], off", "asm")]
    assert not check_m0_owner(right)


def test_every_lds_direct_load_sees_the_m0_written_for_it():
    import glob

    files = sorted(glob.glob(os.path.join(BUILD, "*-hip-amdgcn-amd-amdhsa-gfx950.s")))
    if len(files) < 10:
        pytest.skip("device assembly not kept: build the library first (python -m triton_amd.build)")
    checked = 0
    for f in files:
        for name, lines in _functions(open(f).read()).items():
            if not any("global_load_lds" in l for l in lines):
                continue
            checked += 1
            bad = check_m0_owner(lines)
            assert not bad, (os.path.basename(f), name, bad[:5])
    assert checked >= 40, checked


VALU_MFMA_WAIT = 2
ANYREG = re.compile(r"\b([va])(\d+|\[\d+:\d+\])")


def _anyregs(text):
    out = set()
    for m in ANYREG.finditer(text):
        t = m.group(2)
        if t.startswith("["):
            lo, hi = t[1:-1].split(":")
            out.update((m.group(1), i) for i in range(int(lo), int(hi) + 1))
        else:
            out.add((m.group(1), int(t)))
    return out


def check_valu_write_to_assembly_mfma(lines):
    """Rule 5: an MFMA must not read a vector or accumulation register within VALU_MFMA_WAIT issue slots of a VALU
    instruction (v_accvgpr_write, v_mov, conversions ...) writing it.  The compiler keeps that distance for the
    MFMAs it generates; for an MFMA inside inline assembly nobody does, so its operands must come from loads - or
    the statement must start with the idle slots itself.  Returns (block label, instruction, slots) violations
    over all control-flow paths; only MFMAs between #ASMSTART and #ASMEND are examined."""
    blocks = [("entry", [])]
    in_asm = False
    for line in lines:
        if "#ASMSTART" in line:
            in_asm = True
            continue
        if "#ASMEND" in line:
            in_asm = False
            continue
        code = line.split(";")[0].rstrip()
        if not code.strip():
            continue
        m = re.match(r"^(\.LBB\w+):", code)
        if m:
            blocks.append((m.group(1), []))
        elif code.startswith("\t") and not code.strip().startswith("."):
            blocks[-1][1].append((code.strip(), in_asm))
    index = {lab: i for i, (lab, _) in enumerate(blocks)}
    succ = []
    for i, (_, ins) in enumerate(blocks):
        s, fall = set(), True
        for t, _a in ins:
            m = re.match(r"s_c?branch\w*\s+(\.LBB\w+)", t)
            if m:
                s.add(index[m.group(1)])
            if t.startswith("s_branch") or t.startswith("s_endpgm") or t.startswith("s_setpc"):
                fall = False
        if fall and i + 1 < len(blocks):
            s.add(i + 1)
        succ.append(s)

    def walk(ins, state, report, label):
        state = dict(state)
        for t, asm in ins:
            op = t.split()[0]
            operands = t[len(op):]
            mfma = op.startswith(("v_mfma", "v_smfmac"))
            if mfma and asm and report is not None:
                for r in _anyregs(operands.split(",", 1)[1]):
                    if r in state:
                        report.append((label, t, state[r]))
            m = re.match(r"s_nop\s+(\d+)", t)
            step = int(m.group(1)) + 1 if m else 1
            state = {r: d + step for r, d in state.items() if d + step < VALU_MFMA_WAIT}
            if op.startswith("v_") and not mfma:
                for r in _anyregs(operands.split(",", 1)[0]):
                    state[r] = 0
        return state

    entry = [dict() for _ in blocks]
    work = list(range(len(blocks)))
    while work:
        i = work.pop()
        out = walk(blocks[i][1], entry[i], None, None)
        for j in succ[i]:
            changed = False
            for r, d in out.items():
                if entry[j].get(r, FAR) > d:
                    entry[j][r] = d
                    changed = True
            if changed:
                work.append(j)
    bad = []
    for i, (lab, ins) in enumerate(blocks):
        walk(ins, entry[i], bad, lab)
    return bad


def test_valu_mfma_checker_flags_a_copy_right_in_front_of_an_assembly_mfma():
    mfma = "\tv_mfma_f32_32x32x16_f16 v[32:47], v[124:127], a[88:91], 0"
    close = ["\tv_accvgpr_write_b32 a91, v175", "\t;;#ASMSTART", mfma, "\t;;#ASMEND"]
    settled = ["\tv_accvgpr_write_b32 a91, v175", "\t;;#ASMSTART", "\ts_nop 1", mfma, "\t;;#ASMEND"]
    known = ["\tv_accvgpr_write_b32 a91, v175", mfma]     # the compiler's own MFMA: it has counted the slots itself
    assert check_valu_write_to_assembly_mfma(close) and not check_valu_write_to_assembly_mfma(settled)
    assert not check_valu_write_to_assembly_mfma(known)


def test_no_assembly_mfma_reads_a_register_right_after_a_valu_write():
    import glob

    files = sorted(glob.glob(os.path.join(BUILD, "*-hip-amdgcn-amd-amdhsa-gfx950.s")))
    if len(files) < 10:
        pytest.skip("device assembly not kept: build the library first (python -m triton_amd.build)")
    checked = 0
    for f in files:
        text = open(f).read()
        if "#ASMSTART" not in text:
            continue
        for name, lines in _functions(text).items():
            if not any("v_mfma" in l for l in lines):
                continue
            checked += 1
            bad = check_valu_write_to_assembly_mfma(lines)
            assert not bad, (os.path.basename(f), name, bad[:5])
    assert checked >= 30, checked


def check_assembly_mfma_results(lines):
    """Rule 1 for every kernel and both register files: the destination of an MFMA issued inside inline assembly
    (the compiler does not know it is one) must not be read or overwritten by a non-MFMA instruction, nor read as
    the A / B operand of another MFMA, within MIN_WAIT issue slots - on any control-flow path.  (An MFMA taking it
    as its addend is interlocked by the hardware.)"""
    blocks = [("entry", [])]
    in_asm = False
    for line in lines:
        if "#ASMSTART" in line:
            in_asm = True
            continue
        if "#ASMEND" in line:
            in_asm = False
            continue
        code = line.split(";")[0].rstrip()
        if not code.strip():
            continue
        m = re.match(r"^(\.LBB\w+):", code)
        if m:
            blocks.append((m.group(1), []))
        elif code.startswith("\t") and not code.strip().startswith("."):
            blocks[-1][1].append((code.strip(), in_asm))
    index = {lab: i for i, (lab, _) in enumerate(blocks)}
    succ = []
    for i, (_, ins) in enumerate(blocks):
        s, fall = set(), True
        for t, _a in ins:
            m = re.match(r"s_c?branch\w*\s+(\.LBB\w+)", t)
            if m:
                s.add(index[m.group(1)])
            if t.startswith("s_branch") or t.startswith("s_endpgm") or t.startswith("s_setpc"):
                fall = False
        if fall and i + 1 < len(blocks):
            s.add(i + 1)
        succ.append(s)

    def walk(ins, state, report, label):
        state = dict(state)
        for t, asm in ins:
            op = t.split()[0]
            operands = t[len(op):]
            mfma = op.startswith(("v_mfma", "v_smfmac"))
            if mfma:
                parts = [x.strip() for x in operands.split(",")]
                touched = _anyregs(",".join(parts[1:3]))        # A and B operands (the addend is interlocked)
            else:
                touched = _anyregs(operands)
            if report is not None:
                for r in touched:
                    if r in state:
                        report.append((label, t, state[r]))
            if mfma and asm:
                for r in _anyregs(operands.split(",", 1)[0]):
                    state[r] = 0
            # (the MFMA's own slot counts, as in check_function: MIN_WAIT = required wait states + 1)
            m = re.match(r"s_nop\s+(\d+)", t)
            step = int(m.group(1)) + 1 if m else 1
            state = {r: d + step for r, d in state.items() if d + step < MIN_WAIT}
        return state

    entry = [dict() for _ in blocks]
    work = list(range(len(blocks)))
    while work:
        i = work.pop()
        out = walk(blocks[i][1], entry[i], None, None)
        for j in succ[i]:
            changed = False
            for r, d in out.items():
                if entry[j].get(r, FAR) > d:
                    entry[j][r] = d
                    changed = True
            if changed:
                work.append(j)
    bad = []
    for i, (lab, ins) in enumerate(blocks):
        walk(ins, entry[i], bad, lab)
    return bad


def test_assembly_mfma_result_checker_covers_vector_register_destinations():
    mfma = ["\t;;#ASMSTART", "\tv_mfma_f32_32x32x16_f16 v[32:47], v[124:127], a[88:91], 0", "\t;;#ASMEND"]
    assert check_assembly_mfma_results(mfma + ["\tv_fma_f32 v0, v33, v161, -v92"])
    assert not check_assembly_mfma_results(mfma + ["\ts_nop 10", "\tv_fma_f32 v0, v33, v161, -v92"])   # 11 wait states
    assert check_assembly_mfma_results(mfma + ["\ts_nop 9", "\tv_fma_f32 v0, v33, v161, -v92"])
    # accumulating into the same tile right away is fine; feeding it to another MFMA as an operand is not
    assert not check_assembly_mfma_results(mfma + ["\tv_mfma_f32_32x32x16_f16 v[32:47], v[0:3], a[0:3], v[32:47]"])
    assert check_assembly_mfma_results(mfma + ["\tv_mfma_f32_32x32x16_f16 v[48:63], v[32:35], a[0:3], 0"])


def test_no_result_of_an_assembly_mfma_is_touched_before_it_retires_in_any_kernel():
    import glob

    files = sorted(glob.glob(os.path.join(BUILD, "*-hip-amdgcn-amd-amdhsa-gfx950.s")))
    if len(files) < 10:
        pytest.skip("device assembly not kept: build the library first (python -m triton_amd.build)")
    checked = 0
    for f in files:
        text = open(f).read()
        if "#ASMSTART" not in text:
            continue
        for name, lines in _functions(text).items():
            if not any("v_mfma" in l for l in lines):
                continue
            checked += 1
            bad = check_assembly_mfma_results(lines)
            assert not bad, (os.path.basename(f), name, bad[:5])
    assert checked >= 30, checked


# ---------------------------------------------------------------------------------------------
# A performance property of the same family.  The K loops of the four-wave GEMM kernels keep their direct loads in
# flight across iterations and wait for them by hand, once per K step.  The compiler counts only the loads it knows
# (spill reloads, the epilogue's own loads); when one of those is still outstanding by ITS count at the first use of
# the loaded register and that use sits inside the K loop, it guards the use with a wait that in reality drains
# every load of the loop, in every step (seen: -6 to -12 % after the loop's own wait changed from vmcnt(0) to
# vmcnt(2), with correct results).  So: no basic block of a K loop may wait for vector memory more than once.
# ---------------------------------------------------------------------------------------------
def k_loop_blocks_with_extra_waits(lines, min_mfma=64):
    bad = []
    for label, ins in _blocks(lines):
        if sum("v_mfma" in i for i in ins) < min_mfma:
            continue
        # (a block of the pipelined loop meets the other waves once per K step; blocks of MFMAs without a barrier are
        # the K tails of the fp8 / MX forms, fed by plain loads that the compiler waits for itself)
        if not any("s_barrier" in i for i in ins):
            continue
        waits = [i for i in ins if i.startswith("s_waitcnt") and "vmcnt" in i]
        if len(waits) > 1:
            bad.append((label, waits))
    return bad


def test_extra_wait_checker_flags_a_guarded_reload_inside_a_k_loop():
    mf = ["\tv_mfma_f32_16x16x32_bf16 a[0:3], v[0:3], v[4:7], a[0:3]"] * 64
    good = [".LBB0_1:", "\ts_waitcnt vmcnt(2)", "\ts_barrier"] + mf
    guarded = [".LBB0_1:", "\ts_waitcnt vmcnt(2)", "\ts_barrier"] + mf[:60] + ["\ts_waitcnt vmcnt(0)", "\tglobal_load_lds_dwordx4 v147, s[34:35] offset:0xc00"] + mf[60:]
    assert k_loop_blocks_with_extra_waits(good) == []
    assert [b[0] for b in k_loop_blocks_with_extra_waits(guarded)] == [".LBB0_1"]


def test_k_loops_of_the_four_wave_kernels_wait_for_loads_once_per_step():
    if not all(os.path.exists(f) for f in ASM):
        pytest.skip("device assembly not kept: build the library first (python -m triton_amd.build)")
    checked = 0
    for f in ASM:
        for name, lines in _functions(open(f).read()).items():
            if "gemm_wave128" not in name:
                continue
            # (the K-tail instantiations - template arguments <..., EPI, true, 256> - multiply their tail from plain
            # loads that the compiler waits for itself, in blocks of 64 MFMAs of their own)
            if re.search(r"Li\dELb1ELi256EEE", name):
                continue
            # (the K-tail instantiations of the MXFP8 form - <EPI, true> -: with the tail's registers the compiler keeps
            # one B fragment of the next step in scratch memory across the loop's back edge and reloads it once per
            # eight K steps, with a full wait; measured against the eight-wave kernel that these products ran before,
            # the form is still the faster one)
            if re.search(r"gemm_wave128_mxfp8_kernelILi\dELb1EEE", name):
                continue
            checked += 1
            bad = k_loop_blocks_with_extra_waits(lines)
            assert not bad, (name, bad[:3])
    assert checked >= 30, checked
