"""Static check of the hand-placed waits of the inline-assembly load kernels.

    python -m rknpu2_matmul_open_amd.audit_waits            # compiles the two units to assembly and checks them

gemm_wk_kernel and gemm_stream_kernel issue their loop loads from inline assembly and place
every s_waitcnt by hand; the compiler believes the destination registers of such a load hold
their value as soon as the asm statement has executed.  The kernels are correct only if, in the
code the compiler actually produced, nothing reads or overwrites such a register between the
load and the wait that covers it -- no copy, no spill, no reuse for another value.  That is a
property of one compiler's register allocation and scheduling, so it is re-established after
every build from the device assembly itself (`hipcc -S --cuda-device-only` of the same sources
with the same flags):

  * vector memory loads of a wave return in issue order and s_waitcnt vmcnt(N) returns when at
    most N vector memory operations are outstanding: a load is still outstanding only if every
    younger load is, so the wait that covers a load is the first one behind it with N <= the
    number of loads issued since (stores are not counted: they may complete out of order, which
    can only make a wait stricter than this rule assumes);
  * LDS reads (ds_read from asm) are covered by the next s_waitcnt with lgkmcnt(0);
  * between an asm load and its covering wait no instruction may name one of its destination
    registers.

The check walks the control-flow graph of a kernel (basic blocks split at labels and branches):
from every asm load it follows every path until the covering wait, carrying the number of loads
issued since; a block is visited again only when reached with a smaller count (fewer loads
issued can only make coverage come later), so loops end.
"""
import os
import re
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
UNITS = ["rk_kernels_gemm.hip", "rk_kernels_stream.hip"]

_VM_LOAD = re.compile(r"^\s*(global_load|buffer_load|flat_load|scratch_load)")
_ASM_VLOAD = re.compile(r"^\s*global_load_dwordx?(\d*)\s+(v\[\d+:\d+\]|v\d+)\s*,")
_ASM_DSREAD = re.compile(r"^\s*ds_read_b(\d+)\s+(v\[\d+:\d+\]|v\d+)\s*,")
_VMCNT = re.compile(r"vmcnt\((\d+)\)")
_LGKM0 = re.compile(r"lgkmcnt\(0\)")
_REG = re.compile(r"\bv\[(\d+):(\d+)\]|\bv(\d+)\b")
_LABEL = re.compile(r"^(\.LBB\d+_\d+):")
_BRANCH = re.compile(r"^\s*s_cbranch_\w+\s+(\.LBB\d+_\d+)|^\s*s_branch\s+(\.LBB\d+_\d+)")


def _regs(operand_text):
    """Vector registers named in a piece of assembly text, as a set of numbers."""
    out = set()
    for a, b, c in _REG.findall(operand_text):
        if c:
            out.add(int(c))
        else:
            out.update(range(int(a), int(b) + 1))
    return out


def _instructions(lines):
    """(text, in_asm) for every instruction line of a function body; labels are kept as text."""
    out, in_asm = [], False
    for raw in lines:
        if ";;#ASMSTART" in raw:
            in_asm = True
            continue
        if ";;#ASMEND" in raw:
            in_asm = False
            continue
        text = raw.split(";")[0].rstrip()
        if not text.strip() or text.strip().startswith("."):
            m = _LABEL.match(text.strip())
            if m:
                out.append((m.group(1) + ":", False))
            continue
        out.append((text, in_asm))
    return out


_ENDS = re.compile(r"^\s*(s_endpgm|s_branch\b|s_setpc_b64|s_trap)")


def _blocks(instrs):
    """Basic blocks of a function: (first, last + 1, successor block starts)."""
    label_at = {t[:-1]: i for i, (t, _) in enumerate(instrs) if t.endswith(":")}
    starts = {0}
    for i, (t, _) in enumerate(instrs):
        if t.endswith(":"):
            starts.add(i)
        if _BRANCH.match(t) or _ENDS.match(t):
            starts.add(i + 1)
    order = sorted(x for x in starts if x < len(instrs))
    blocks = {}
    for n, lo in enumerate(order):
        hi = order[n + 1] if n + 1 < len(order) else len(instrs)
        last = instrs[hi - 1][0]
        succ = []
        b = _BRANCH.match(last)
        if b:
            target = b.group(1) or b.group(2)
            if target in label_at:
                succ.append(label_at[target])
        if not _ENDS.match(last) and hi < len(instrs):
            succ.append(hi)
        blocks[lo] = (lo, hi, succ)
    return blocks


def _check_load(instrs, blocks, block_of, at, what, violations, seen):
    """Every path behind the asm load at `at` up to its covering wait."""
    text = instrs[at][0]
    m = _ASM_VLOAD.match(text)
    ds = None if m else _ASM_DSREAD.match(text)
    dst = _regs((m or ds).group(2))
    best = {}                      # block start -> smallest `issued` it was entered with
    work = [(at + 1, 0)]
    uncovered_end = False
    while work:
        pos, issued = work.pop()
        lo, hi, succ = blocks[block_of[pos]] if pos < len(instrs) else (pos, pos, [])
        covered = False
        for j in range(pos, hi):
            t, _ = instrs[j]
            if t.endswith(":"):
                continue
            if "s_waitcnt" in t:
                if m:
                    c = _VMCNT.search(t)
                    if c and int(c.group(1)) <= issued:
                        covered = True
                        break
                elif _LGKM0.search(t):
                    covered = True
                    break
                continue
            if m and _VM_LOAD.match(t):
                issued += 1
            parts = t.split(None, 1)
            hit = dst & _regs(parts[1] if len(parts) > 1 else "")
            if hit:
                key = (what, text.strip(), t.strip())
                if key not in seen:
                    seen.add(key)
                    violations.append("%s: `%s` is followed, before the wait that covers it, by `%s` (v%s)"
                                      % (what, text.strip(), t.strip(), ",".join(map(str, sorted(hit)))))
                covered = True      # (reported once; no need to follow this path further)
                break
        if covered:
            continue
        if not succ:
            uncovered_end = True   # the program ends with the load in flight: nothing reads it
            continue
        issued = min(issued, 64)
        for nxt in succ:
            if nxt not in best or issued < best[nxt]:
                best[nxt] = issued
                work.append((nxt, issued))
    return uncovered_end


def audit_function(name, lines):
    """Violations (strings) of one kernel's assembly."""
    instrs = _instructions(lines)
    violations, seen = [], set()
    loads = [i for i, (t, a) in enumerate(instrs) if a and (_ASM_VLOAD.match(t) or _ASM_DSREAD.match(t))]
    if not loads:
        return violations
    blocks = _blocks(instrs)
    block_of, cur = {}, 0
    for i in range(len(instrs)):
        if i in blocks:
            cur = i
        block_of[i] = cur
    for i in loads:
        _check_load(instrs, blocks, block_of, i, name, violations, seen)
    return violations


def audit_text(asm_text, only=("gemm_wk_kernel", "gemm_stream_kernel")):
    """Violations in every kernel of an assembly file whose (mangled) name contains one of `only`."""
    violations, checked = [], 0
    lines = asm_text.splitlines()
    start, name = None, None
    for n, line in enumerate(lines):
        m = re.match(r"^(_Z\w+):\s", line + " ")
        if m and any(k in m.group(1) for k in only):
            start, name = n + 1, m.group(1)
        elif start is not None and "s_endpgm" in line:
            violations += audit_function(name, lines[start:n + 1])
            checked += 1
            start = None
    return violations, checked


def device_assembly(unit, hipcc, flags):
    src = os.path.join(HERE, "csrc", unit)
    cmd = [hipcc] + [f for f in flags if f not in ("-fPIC",)] + ["-S", "--cuda-device-only", src, "-o", "-"]
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    if p.returncode:
        raise RuntimeError("hipcc -S failed for %s:\n%s" % (unit, p.stderr[-2000:]))
    return p.stdout


def audit(hipcc=None, flags=None):
    """Compiles the asm-load units to assembly and checks them; returns (violations, kernels checked)."""
    from . import build as lib_build
    hipcc = hipcc or os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    flags = flags or lib_build.FLAGS
    from concurrent.futures import ThreadPoolExecutor
    with ThreadPoolExecutor(len(UNITS)) as pool:
        texts = list(pool.map(lambda u: device_assembly(u, hipcc, flags), UNITS))
    violations, checked = [], 0
    for t in texts:
        v, c = audit_text(t)
        violations += v
        checked += c
    return violations, checked


if __name__ == "__main__":
    found, count = audit()
    for line in found:
        print(line)
    print("%d kernels checked, %d violations" % (count, len(found)))
    sys.exit(1 if found or not count else 0)
