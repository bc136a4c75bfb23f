"""A check of the generated GPU code that the compiler cannot make itself.

The global -> LDS copies of the kernels are `buffer_load ... lds` instructions inside inline assembly, so that the compiler
does not order its LDS reads behind them.  The price: the compiler does not know that a memory instruction sits there.
On gfx9-family hardware a memory instruction that reads a scalar register needs five wait states after a *vector*
instruction wrote that register (v_readlane_b32 / v_readfirstlane_b32 / a vector compare with a scalar destination) - the
hardware does not interlock this case, the compiler's hazard pass inserts the wait states for the memory instructions it
sees, and restores spilled scalar registers with exactly such v_readlane_b32 instructions wherever it likes.  A copy that
reads a stale descriptor fetches from wherever that pointed: wrong values, or a memory fault.

`scan_asm` walks the assembly the compiler wrote for a source file (kept with -save-temps while building) and reports every
inline copy with fewer than five wait states between it and a vector write of one of its scalar operands (m0, which holds
the copy's LDS address, among them).  The build fails
on a report; the remedy is a longer `s_nop` in front of the copy in question (sdpa_mfma_common.h, sdpa_decode_ring.h).
"""
import re

NEEDED = 5
_SREG = re.compile(r"\bs(\d+)\b|\bs\[(\d+):(\d+)\]")
_VALU_SGPR_WRITE = re.compile(r"^\s*(v_readlane_b32|v_readfirstlane_b32|v_cmp\w*_e64|v_cmpx\w*_e64)\s+(s\[\d+:\d+\]|s\d+|m0)")
M0 = -1          # (m0, which every copy into LDS reads for its LDS address, stands in the register sets as -1)


def _sregs(text):
    regs = {M0} if re.search(r"\bm0\b", text) else set()
    for m in _SREG.finditer(text):
        if m.group(1) is not None:
            regs.add(int(m.group(1)))
        else:
            regs.update(range(int(m.group(2)), int(m.group(3)) + 1))
    return regs


def _is_instruction(line):
    t = line.strip()
    return bool(t) and not t.startswith((";", ".", "//")) and not t.endswith(":") and not re.match(r"^[\w.$]+:", t)


def scan_asm(text):
    """Returns a list of (function, line number, copy instruction, offending instruction, wait states between them)."""
    lines = text.splitlines()
    found = []
    func = "?"
    for n, line in enumerate(lines):
        m = re.match(r"^([A-Za-z_][\w$.]*):\s*(;.*)?$", line)
        if m and not m.group(1).startswith(".L"):
            func = m.group(1)
        t = line.strip()
        if not (t.startswith("buffer_load") and t.endswith("lds")):
            continue
        operands = t.split(None, 1)[1]
        regs = _sregs(operands) | {M0}
        waits = 0
        k = n - 1
        while k >= 0 and waits < NEEDED:
            prev = lines[k]
            k -= 1
            if re.match(r"^[A-Za-z_][\w$.]*:\s*(;.*)?$", prev) and not prev.startswith(".L"):
                break                                   # start of the function
            if not _is_instruction(prev):
                continue
            p = prev.strip()
            nop = re.match(r"^s_nop\s+(\d+)", p)
            if nop:
                waits += int(nop.group(1)) + 1
                continue
            w = _VALU_SGPR_WRITE.match(p)
            if w and _sregs(w.group(2)) & regs:
                found.append((func, n + 1, t, p, waits))
                break
            waits += 1
    return found


def check_file(path):
    with open(path) as f:
        return scan_asm(f.read())
