"""Static check of a hipcc assembly listing for kernels that issue LDS reads from inline asm.

The compiler does not know that such a read is still in flight, so nothing stops it from reusing the
destination registers (as scratch, or for a value that feeds an address) before the data arrives; the
late write-back then corrupts whatever was put there.  LDS reads return in order, so the set of
registers still being filled after ``s_waitcnt lgkmcnt(N)`` is that of the N youngest reads.  The
check walks a kernel's listing in text order and reports every instruction that reads or writes a
vector register an earlier asm-issued ``ds_read`` is still filling.  Only reads between the
compiler's ``;;#ASMSTART`` / ``;;#ASMEND`` markers are tracked as hazards (the compiler waits for its
own); every LDS or scalar-memory instruction counts for the wait arithmetic.  What is in flight
travels along forward branches to their labels (where several paths meet, the one with the most
reads in flight is kept); backward branches are not followed, the loop body having been seen with
the state it is entered with.
"""
import re

_REG = re.compile(r"\bv\[(\d+):(\d+)\]|\bv(\d+)\b")
_LABEL = re.compile(r"^(\.LBB\w+):")


def _regs(text):
    out = set()
    for m in _REG.finditer(text):
        if m.group(1):
            out.update(range(int(m.group(1)), int(m.group(2)) + 1))
        else:
            out.add(int(m.group(3)))
    return out


def check_kernel(lines):
    """lines: [(line_number, text)] of one kernel; returns a list of findings (strings)."""
    pending = []   # [(registers, line_number)] of LDS reads in flight, oldest first
    findings = []
    at_label = {}  # label -> what was in flight at a forward branch to it
    seen = set()
    unreachable = False  # after an unconditional branch, until the next label
    in_asm = False
    for no, ln in lines:
        if ";;#ASMSTART" in ln:
            in_asm = True
        elif ";;#ASMEND" in ln:
            in_asm = False
        t = ln.split(";")[0].strip()
        if not t:
            continue
        m = _LABEL.match(t)
        if m:
            seen.add(m.group(1))
            carried = at_label.get(m.group(1), [])
            if unreachable or len(carried) > len(pending):
                pending = list(carried)
            unreachable = False
            continue
        if t.startswith(".") or t.endswith(":") or unreachable:
            continue
        op = t.split()[0]
        if op == "s_branch" or op.startswith("s_cbranch"):
            target = t.split()[-1]
            if target not in seen and len(at_label.get(target, [])) <= len(pending):
                at_label[target] = list(pending)
            if op == "s_branch":
                unreachable = True
            continue
        inflight = set().union(*[p[0] for p in pending]) if pending else set()
        if op.startswith("ds_") or op.startswith("s_load") or op.startswith("s_buffer_load"):
            hit = _regs(t) & inflight
            if hit:
                findings.append(f"line {no}: touches in-flight v{sorted(hit)}: {t}")
            tracked = in_asm and (op.startswith("ds_read") or op.startswith("ds_load"))
            pending.append((_regs(t.split(",")[0]) if tracked else set(), no))
            continue
        if op == "s_waitcnt":
            m = re.search(r"lgkmcnt\((\d+)\)", t)
            if m:
                n = int(m.group(1))
                if n < len(pending):
                    pending = pending[len(pending) - n:] if n else []
            continue
        hit = _regs(t) & inflight
        if hit:
            issued = [p[1] for p in pending if p[0] & hit]
            findings.append(f"line {no}: touches in-flight v{sorted(hit)} (read issued at line {issued}): {t}")
    return findings


def check_listing(text, name_contains):
    """Checks every kernel whose mangled name contains ``name_contains``; returns {kernel: findings}."""
    src = text.split("\n")
    out, cur, body = {}, None, []
    for i, ln in enumerate(src, 1):
        m = re.match(r"^(_Z\w+):", ln)
        if m and name_contains in m.group(1):
            cur, body = m.group(1), []
            continue
        if cur:
            body.append((i, ln))
            if "s_endpgm" in ln:
                out[cur] = check_kernel(body)
                cur = None
    return out
