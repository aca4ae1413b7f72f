"""Checks of the generated gfx950 code that the compiler cannot make.

The GEMM kernels issue their MFMAs from inline asm (to keep the accumulators in AGPRs and the
instruction order as written).  The compiler looks after the pipeline hazards of the instructions
it emits itself; an MFMA inside an asm statement is opaque to it.  Two of those hazards are real
on this part (measured with a one-wave probe: a `v_mov_b32` or `v_accvgpr_read_b32` into a source
register directly before the MFMA - the MFMA multiplies the register's OLD contents, every time;
one instruction in between and it sees the new ones):

  A. a vector-ALU instruction writes a register that an asm MFMA reads (a source operand or the
     accumulator) fewer than VALU_TO_MFMA wait states before it.  Typical producer: the register
     allocator reloading a fragment register from its AGPR spill copy right at the use.
  B. an instruction other than an MFMA reads or writes the destination of an asm MFMA fewer than
     MFMA_TO_OTHER wait states after it (the compiler moving an accumulator between registers).

`scan(text)` walks the assembly text (hipcc -S / -save-temps) and returns the findings;
`wmma_extension_amd._lib.build` runs it over the GEMM translation unit and refuses to produce a
library when there is one.
"""
import re

VALU_TO_MFMA = 2      # wait states; the compiler keeps 2 for its own MFMAs, the probe needed 1
MFMA_TO_OTHER = 18    # 16x16x32: eight passes; the compiler's own figure for a VALU read is 11

_REG_RANGE = re.compile(r"^([va])\[(\d+):(\d+)\]$")
_REG_ONE = re.compile(r"^([va])(\d+)$")


def _regs(token):
    token = token.strip()
    m = _REG_RANGE.match(token)
    if m:
        return {(m.group(1), i) for i in range(int(m.group(2)), int(m.group(3)) + 1)}
    m = _REG_ONE.match(token)
    if m:
        return {(m.group(1), int(m.group(2)))}
    return set()


def _operands(text):
    parts = text.split(None, 1)
    if len(parts) < 2:
        return []
    # drop modifiers after the operand list (e.g. "quad_perm:[1,0,3,2] row_mask:0xf")
    ops, depth, cur = [], 0, ""
    for ch in parts[1]:
        if ch == "[":
            depth += 1
        elif ch == "]":
            depth -= 1
        if ch == "," and depth == 0:
            ops.append(cur)
            cur = ""
        else:
            cur += ch
    ops.append(cur)
    return [o.strip().split()[0] if o.strip() else "" for o in ops]


def _instructions(text):
    """(line number, instruction text, inside an asm statement) for every instruction line."""
    out, in_asm = [], False
    for n, line in enumerate(text.split("\n"), 1):
        t = line.strip()
        if t.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if t.startswith(";;#ASMEND"):
            in_asm = False
            continue
        if not t or t[0] in ";." or t.endswith(":"):
            continue
        t = t.split(";")[0].strip()
        if t:
            out.append((n, t, in_asm))
    return out


def _wait_states(text):
    if text.startswith("s_nop"):
        return int(text.split()[1], 0) + 1
    return 1


def _is_valu_write(text):
    return (text.startswith("v_") and not text.startswith("v_mfma") and not text.startswith("v_cmp")
            and not text.startswith("v_readlane") and not text.startswith("v_readfirstlane"))


def scan(text):
    """Findings as dicts {kind, line, mfma, other_line, other, wait_states}; empty when clean.
    The windows follow the text: a look-ahead ends at a branch, labels are passed over (the
    kernels place their loop heads on waits and barriers, never directly on an MFMA)."""
    ins = _instructions(text)
    findings = []
    for idx, (n, t, in_asm) in enumerate(ins):
        if not (in_asm and t.startswith("v_mfma")):
            continue
        ops = _operands(t)
        dst = _regs(ops[0]) if ops else set()
        reads = set()
        for o in ops[1:]:
            reads |= _regs(o)
        # A: producers before
        ws = 0
        k = idx - 1
        while k >= 0 and ws < VALU_TO_MFMA:
            pn, pt, _ = ins[k]
            if not pt.startswith("s_nop") and _is_valu_write(pt):
                pops = _operands(pt)
                written = _regs(pops[0]) if pops else set()
                if written & reads:
                    findings.append(dict(kind="valu-write-before-asm-mfma", line=n, mfma=t,
                                         other_line=pn, other=pt, wait_states=ws))
            ws += _wait_states(pt)
            k -= 1
        # B: consumers after
        ws = 0
        k = idx + 1
        while k < len(ins) and ws < MFMA_TO_OTHER:
            qn, qt, _ = ins[k]
            if qt.startswith(("s_cbranch", "s_branch", "s_endpgm", "s_setpc")):
                break
            if not qt.startswith(("v_mfma", "s_")):
                touched = set()
                for o in _operands(qt):
                    touched |= _regs(o)
                if touched & dst:
                    findings.append(dict(kind="asm-mfma-result-touched-early", line=n, mfma=t,
                                         other_line=qn, other=qt, wait_states=ws))
            ws += _wait_states(qt)
            k += 1
    return findings


def format_findings(findings, limit=20):
    lines = []
    for f in findings[:limit]:
        lines.append(f"{f['kind']}: line {f['line']}: {f['mfma']}\n    {'<-' if 'before' in f['kind'] else '->'} "
                     f"line {f['other_line']}: {f['other']}  ({f['wait_states']} wait states between)")
    if len(findings) > limit:
        lines.append(f"... and {len(findings) - limit} more")
    return "\n".join(lines)


def check_file(path):
    """Raise RuntimeError when the assembly at `path` has a finding."""
    with open(path) as f:
        findings = scan(f.read())
    if findings:
        raise RuntimeError(f"{path}: {len(findings)} pipeline hazard(s) around inline-asm MFMAs that the "
                           f"compiler does not handle:\n" + format_findings(findings) +
                           "\n(change the kernel so that the allocation comes out differently, or, at a cost of up "
                           "to 13 % in the kernel that splits its own operands, put a wait state in front of "
                           "every such MFMA: -DWMMAE_MFMA_GUARD='\"s_nop 0\\n\\t\"')")
    return 0
