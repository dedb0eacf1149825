"""Register hazards around hand-placed matrix instructions.

The dK/dV and dQ kernels with 64 keys / queries per wavefront issue their matrix instructions from asm statements, so
the compiler does not know which registers those read and write and keeps none of the distances gfx950 needs between
them and the vector instructions around them. Two of those distances are not enforced by the hardware either:

  * a matrix instruction that reads, as A or B, a register written by the vector instruction just before it sees the
    old contents (measured: at distance 0 the packed dS operand still held the fp32 product; at distance 1 it was right);
  * a vector instruction (a move out of an accumulation register included), LDS / global store or matrix operand read of
    a register that a matrix instruction wrote less than its pass count + 3 issue slots earlier (8 passes for v_mfma_f32_32x32x16_bf16) sees the old contents. A
    matrix instruction in between counts as 8 slots: it cannot enter the pipe before the writer has left it.

  * a vector instruction that WRITES a register which a matrix instruction issued less than 11 slots earlier is still
    going to write (write after write), or which a matrix instruction issued less than 7 slots earlier still reads as
    its C operand from ordinary registers (write after read: the 8-pass instruction reads C over its passes), would
    corrupt that instruction's result or input.

This test compiles the two kernels to assembly and checks these distances on every path of the control-flow graph
that the assembler text shows: fall-through over labels, taken branches and loop back-edges (the tail of a loop body
is followed by its head)."""
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
WAW_MFMA_TO_VALU = 11   # a vector write to a register a matrix instruction is still going to write
WAR_SRCC_TO_VALU = 7    # a vector write to a register a matrix instruction still reads as its C operand
MFMA_SLOTS = 8          # a matrix instruction in between enters the pipe only when the one before it has left it
HORIZON = max(RAW_MFMA_TO_OTHER, WAW_MFMA_TO_VALU, WAR_SRCC_TO_VALU, RAW_VALU_TO_MFMA)


def _regs(tok):
    """registers named by one operand, as (file, index) pairs: ordinary (v) and accumulation (a) registers"""
    tok = tok.strip().rstrip(",")
    m = re.fullmatch(r"([va])\[(\d+):(\d+)\]", tok)
    if m:
        return {(m.group(1), i) for i in range(int(m.group(2)), int(m.group(3)) + 1)}
    m = re.fullmatch(r"([va])(\d+)", tok)
    return {(m.group(1), int(m.group(2)))} if m else set()


class Inst:
    __slots__ = ("text", "line", "op", "slots", "is_mfma", "is_valu", "ab", "reads", "vw", "mw", "srcc", "target",
                 "falls_through")


def parse(path):
    """-> {kernel: (instructions, {label: index of the instruction that follows it})}"""
    kernels, cur, labels, kern = {}, None, None, None
    for ln, line in enumerate(open(path), 1):
        t = line.split(";")[0].strip()
        m = re.match(r"^(_Z\w+):", t)
        if m:
            kern, cur, labels = m.group(1), [], {}
            kernels[kern] = (cur, labels)
            continue
        if cur is None or not t:
            continue
        if t.endswith(":"):
            labels[t[:-1]] = len(cur)
            continue
        if t.startswith("."):
            continue
        op, _, rest = t.partition(" ")
        ops = [x.strip() for x in rest.split(",")] if rest else []
        i = Inst()
        i.text, i.line, i.op = t, ln, op
        i.is_mfma = op.startswith("v_mfma") or op.startswith("v_smfmac")
        i.is_valu = op.startswith("v_") and not i.is_mfma
        i.slots = MFMA_SLOTS if i.is_mfma else (int(ops[0], 0) + 1 if op == "s_nop" else 1)
        i.ab = i.reads = i.vw = i.mw = i.srcc = frozenset()
        i.target = ops[0] if op.startswith("s_cbranch") or op == "s_branch" else None
        i.falls_through = op not in ("s_branch", "s_endpgm", "s_setpc_b64")
        if i.is_mfma:
            i.ab = frozenset(_regs(ops[1]) | _regs(ops[2]))
            i.reads = i.ab  # C of an accumulating chain is forwarded by the hardware
            i.mw = frozenset(_regs(ops[0]))
            i.srcc = frozenset(r for r in _regs(ops[3]) if r[0] == "v") if len(ops) > 3 else frozenset()
        elif op != "s_nop" and ops:
            first_src = 1 if (op.startswith("v_") or op.startswith("ds_read") or op.startswith("global_load")
                              or op.startswith("buffer_load")) else 0
            i.reads = frozenset(set().union(*[_regs(x) for x in ops[first_src:]]))
            if i.is_valu and not op.startswith("v_cmp"):
                i.vw = frozenset(_regs(ops[0]))
        cur.append(i)
        if op == "s_endpgm":
            cur = None
    return kernels


def hazards_between(w, r, dist):
    """hazard kinds between an earlier instruction w and a later one r with `dist` issue slots between them"""
    out = []
    if r.is_mfma and dist < RAW_VALU_TO_MFMA and w.vw & r.ab:
        out.append("vector write, matrix operand read")
    if dist < RAW_MFMA_TO_OTHER and w.mw & r.reads:
        out.append("matrix write, read")
    if r.is_valu and dist < WAW_MFMA_TO_VALU and w.mw & r.vw:
        out.append("matrix write, vector write")
    if r.is_valu and dist < WAR_SRCC_TO_VALU and w.srcc & r.vw:
        out.append("matrix C operand read, vector write")
    return out


def scan(path):
    """-> list of 'kernel: earlier -> later (distance, kind)' strings. Every path of the control-flow graph that
    reaches an instruction is walked backwards up to the hazard horizon: fall-through (labels do not end a window),
    taken forward branches and loop back-edges alike."""
    found = []
    for kern, (ins, labels) in parse(path).items():
        preds = [[] for _ in ins]
        for j, i in enumerate(ins):
            if i.falls_through and j + 1 < len(ins):
                preds[j + 1].append(j)
            if i.target in labels and labels[i.target] < len(ins):
                preds[labels[i.target]].append(j)
        for k, r in enumerate(ins):
            if not (r.reads or r.vw or r.is_mfma):
                continue
            stack, seen = [(j, 0) for j in preds[k]], set()
            while stack:
                j, dist = stack.pop()
                if (j, dist) in seen:
                    continue
                seen.add((j, dist))
                w = ins[j]
                for kind in hazards_between(w, r, dist):
                    found.append(f"{kern}: {w.line}: {w.text}  ->  {r.line}: {r.text}  (distance {dist}: {kind})")
                if dist + w.slots < HORIZON:
                    stack.extend((jj, dist + w.slots) for jj in preds[j])
    return found


def _scan_text(tmp_path, body):
    f = tmp_path / "case.s"
    f.write_text("_Zcase:\n" + body + "\ns_endpgm\n")
    return scan(str(f))


def test_the_scan_itself_sees_each_kind_of_hazard(tmp_path):
    """Known-bad and known-good snippets, so that a scan that silently sees nothing cannot pass."""
    mf = "v_mfma_f32_32x32x16_bf16 v[0:15], v[20:23], v[24:27], v[0:15]"
    nops = "s_nop 7\ns_nop 1"
    assert _scan_text(tmp_path, f"v_mov_b32 v20, v40\n{mf}")                      # vector write just before its use as A
    assert not _scan_text(tmp_path, f"v_mov_b32 v20, v40\ns_nop 1\n{mf}")
    assert _scan_text(tmp_path, f"{mf}\nv_add_f32 v40, v3, v41")                   # result read too early
    assert not _scan_text(tmp_path, f"{mf}\n{nops}\ns_nop 0\nv_add_f32 v40, v3, v41")
    assert _scan_text(tmp_path, f"{mf}\ns_nop 7\nv_mov_b32 v5, v41")              # result overwritten too early
    mc = "v_mfma_f32_32x32x16_bf16 v[0:15], v[20:23], v[24:27], v[32:47]"
    assert _scan_text(tmp_path, f"{mc}\ns_nop 3\nv_mov_b32 v33, v50")             # C operand overwritten while read
    assert not _scan_text(tmp_path, f"{mc}\ns_nop 6\nv_mov_b32 v33, v50")
    # across a loop back-edge: the write at the loop's end meets the matrix instruction at its head
    loop = f".LBB0_1:\n{mf}\n{nops}\ns_nop 7\nv_mov_b32 v21, v40\ns_cbranch_scc1 .LBB0_1"
    assert _scan_text(tmp_path, loop)
    assert not _scan_text(tmp_path, loop.replace("s_cbranch_scc1", "s_nop 0\ns_cbranch_scc1"))
    # fall-through over a label keeps the window open
    assert _scan_text(tmp_path, f"{mf}\n.LBB0_2:\nv_add_f32 v40, v3, v41")


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
