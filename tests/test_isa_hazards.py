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
        assert sum("v_mfma" in l for l in lines) >= 128, name
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
