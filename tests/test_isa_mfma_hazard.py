"""Static check of the generated gfx950 code of the four-wave GEMM kernels (CPU only).

Those kernels issue their MFMAs as inline assembly (to pin the accumulators to the accumulation
registers), so the compiler neither knows that they are MFMAs nor inserts the wait states that a read of
an MFMA result needs.  The source places a wait at the end of a tile's last K iteration
(`mfma_retire` in triton_amd/csrc/gemm_wave128.hip); this test proves on the assembly the build keeps
that on EVERY control-flow path from an MFMA to a non-MFMA instruction reading an accumulation
register at least MIN_WAIT issue slots pass (an 8-pass MFMA needs 11 by the CDNA3/CDNA4 ISA guides'
table of required software wait states; `s_nop N` counts N + 1, any other instruction 1).
"""
import os
import re

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ASM = os.path.join(HERE, "..", "triton_amd", "csrc", "_build", "gemm_wave128-hip-amdgcn-amd-amdhsa-gfx950.s")
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
    if not os.path.exists(ASM):
        pytest.skip("device assembly not kept: build the library first (python -m triton_amd.build)")
    funcs = _functions(open(ASM).read())
    kernels = {k: v for k, v in funcs.items() if "gemm_wave128" in k}
    assert len(kernels) >= 12, sorted(kernels)
    for name, lines in kernels.items():
        assert sum("v_mfma" in l for l in lines) >= 128, name
        bad = check_function(lines)
        assert not bad, (name, bad[:5])
