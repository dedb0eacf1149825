"""Register hazards around hand-placed matrix instructions.

The dK/dV and dQ kernels with 64 keys / queries per wavefront issue their matrix instructions from asm statements, so
the compiler does not know which registers those read and write and keeps none of the distances gfx950 needs between
them and the vector instructions around them. Two of those distances are not enforced by the hardware either:

  * a matrix instruction that reads, as A or B, a register written by the vector instruction just before it sees the
    old contents (measured: at distance 0 the packed dS operand still held the fp32 product; at distance 1 it was right);
  * a vector instruction (a move out of an accumulation register included), LDS / global store or matrix operand read of
    a register that a matrix instruction wrote less than its pass count + 3 issue slots earlier (8 passes for v_mfma_f32_32x32x16_bf16) sees the old contents. A
    matrix instruction in between counts as 8 slots: it cannot enter the pipe before the writer has left it.

This test compiles the two kernels to assembly and checks both distances on every path the assembler text shows
(straight-line windows; a label or branch ends a window, which errs on the side of missing a hazard across a jump, so
the kernels keep their own s_nop where a phase starts)."""
import os
import re
import shutil
import subprocess

import pytest

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "paperkiln_amd", "csrc")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-I" + os.path.join(CSRC, "..", "..", "include"),
         "-I" + CSRC, "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument",
         "-Wno-unknown-warning-option", "--cuda-device-only", "-S"]
RAW_VALU_TO_MFMA = 2    # idle or unrelated issue slots wanted between a vector write and the matrix read
RAW_MFMA_TO_OTHER = 11  # 8 passes + 3
MFMA_SLOTS = 8          # a matrix instruction in between enters the pipe only when the one before it has left it


def _regs(tok):
    """registers named by one operand, as (file, index) pairs: ordinary (v) and accumulation (a) registers"""
    tok = tok.strip().rstrip(",")
    m = re.fullmatch(r"([va])\[(\d+):(\d+)\]", tok)
    if m:
        return {(m.group(1), i) for i in range(int(m.group(2)), int(m.group(3)) + 1)}
    m = re.fullmatch(r"([va])(\d+)", tok)
    return {(m.group(1), int(m.group(2)))} if m else set()


def scan(path):
    """-> list of 'kernel: writer -> reader (distance)' strings"""
    found, hist, kern = [], [], None  # hist: (slots, vector-written regs, matrix-written regs, text, line)
    for ln, line in enumerate(open(path), 1):
        t = line.split(";")[0].strip()
        m = re.match(r"^(_Z\w+):", t)
        if m:
            kern, hist = m.group(1), []
            continue
        if t.endswith(":") or t.startswith("s_cbranch") or t.startswith("s_branch"):
            hist = []
            continue
        if not t or t.startswith("."):
            continue
        op, _, rest = t.partition(" ")
        ops = [x.strip() for x in rest.split(",")] if rest else []
        is_mfma = op.startswith("v_mfma") or op.startswith("v_smfmac")
        if op == "s_nop":
            hist.append((int(ops[0], 0) + 1, set(), set(), t, ln))
            continue
        if is_mfma:
            ab = _regs(ops[1]) | _regs(ops[2])
            reads = ab  # C of an accumulating chain is forwarded by the hardware
        else:
            first_src = 1 if (op.startswith("v_") or op.startswith("ds_read") or op.startswith("global_load")
                              or op.startswith("buffer_load")) else 0
            reads = set().union(*[_regs(x) for x in ops[first_src:]]) if ops else set()
        dist = 0
        for slots, vw, mw, txt, l0 in reversed(hist):
            if is_mfma and dist < RAW_VALU_TO_MFMA and vw & ab:
                found.append(f"{kern}: {l0}: {txt}  ->  {ln}: {t}  (distance {dist})")
            if dist < RAW_MFMA_TO_OTHER and mw & reads:
                found.append(f"{kern}: {l0}: {txt}  ->  {ln}: {t}  (distance {dist})")
            dist += slots
            if dist >= RAW_MFMA_TO_OTHER:
                break
        vw = mw = set()
        if is_mfma:
            mw = _regs(ops[0])
        elif op.startswith("v_") and not op.startswith("v_cmp") and ops:
            vw = _regs(ops[0])
        hist.append((MFMA_SLOTS if is_mfma else 1, vw, mw, t, ln))
        hist = hist[-(RAW_MFMA_TO_OTHER + 2):]
    return found


@pytest.mark.parametrize("src", ["attn_bwd_dq3.hip", "attn_bwd_dkdv3.hip"])
def test_no_unspaced_register_hazard_around_asm_matrix_instructions(src, tmp_path):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not found")
    out = tmp_path / (src + ".s")
    subprocess.run([hipcc, *FLAGS, os.path.join(CSRC, src), "-o", str(out)], check=True, stdout=subprocess.DEVNULL,
                   stderr=subprocess.DEVNULL)
    text = open(out).read()
    assert "v_mfma_f32_32x32x16_bf16" in text
    found = scan(str(out))
    assert not found, "\n".join(found[:20])
