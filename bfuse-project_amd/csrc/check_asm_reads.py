#!/usr/bin/env python3
"""Build-time check of the hand-issued LDS reads in the compiled kernels.

Several operators issue `ds_read_*` from inline asm and wait for the data later with a
hand-written `s_waitcnt lgkmcnt(n)` (the compiler would wait for ALL outstanding reads before the
first use, which throws the read-ahead away).  The compiler does not know that the asm's output
registers are still being written: if it copied, spilled or reused such a register between the
read and its wait, the kernel would read whatever the register held before the data arrived --
wrong results with no error.  No remark reports that, so this script reads the device assembly the
compiler produced (`hipcc -save-temps`) and checks it:

  * every instruction between an asm-issued `ds_read` and the wait that covers it is looked at;
    if it names one of the read's destination registers (as source OR destination), that is an error;
  * a wait `lgkmcnt(n)` with n > 0 retires all but the n youngest LDS operations, which is only
    sound while nothing but LDS operations is in flight (they return in order; scalar loads do
    not): a scalar-memory load in flight together with a tracked read at such a wait is an error;
  * a tracked read still in flight at `s_endpgm` is an error, and so is a backward branch taken with
    other reads in flight (other registers, or another order) than the loop was entered with: a
    software-pipelined K loop carries the first reads of its next step round the branch, in the
    registers that held them on entry.

The scan is linear over each kernel's text (forward branches are passed straight through), which
is how the hand-written sequences are laid out; operations the compiler itself has in flight are
forgotten at basic-block boundaries (see below).  Usage: check_asm_reads.py file.s [...]; exit
status 1 and one line per finding if anything is wrong.
"""
import re
import sys

REG = re.compile(r"\b([va])(?:(\d+)|\[(\d+):(\d+)\])")
LGKM = re.compile(r"lgkmcnt\((\d+)\)")
LABEL = re.compile(r"^([A-Za-z_.$][\w.$]*):")


def regs_of(text):
    out = set()
    for m in REG.finditer(text):
        kind = m.group(1)
        if m.group(2) is not None:
            out.add((kind, int(m.group(2))))
        else:
            for i in range(int(m.group(3)), int(m.group(4)) + 1):
                out.add((kind, i))
    return out


def counts_in_lgkm(mn):
    return (mn.startswith("ds_") or mn.startswith("s_load") or mn.startswith("s_buffer_load") or mn.startswith("flat_")
            or mn in ("s_memtime", "s_memrealtime", "s_sendmsg", "s_sendmsghalt"))


def is_smem(mn):
    return mn.startswith("s_load") or mn.startswith("s_buffer_load") or mn in ("s_memtime", "s_memrealtime")


def check(path):
    findings = []
    func = None
    in_asm = False
    queue = []          # LDS / scalar-memory operations in flight, oldest first: (tracked regs or None, is_smem, line no)
    labels_seen = {}        # label -> destinations of the hand-issued reads in flight when the scan passed it
    n_tracked = 0
    for ln, raw in enumerate(open(path, errors="replace"), 1):
        line = raw.split(";;#", 1)[0] if ";;#" in raw and not raw.strip().startswith(";;#") else raw
        s = line.strip()
        if s.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if s.startswith(";;#ASMEND"):
            in_asm = False
            continue
        m = LABEL.match(line)
        if m:
            name = m.group(1)
            if not name.startswith(".L"):
                func, queue, labels_seen = name, [], {}
            else:
                labels_seen[name] = [q[0] for q in queue if q[0]]
                # A basic-block boundary: what the compiler itself has in flight here depends on the
                # path taken, which a linear scan does not know; its own waits take care of those.
                # Forgetting them is the conservative side for the hand-issued reads (fewer younger
                # operations means a wait retires fewer of them in this model than in the hardware).
                queue = [q for q in queue if q[0]]
            continue
        if not s or s.startswith(";") or s.startswith(".") or s.startswith("//"):
            continue
        s = s.split(";", 1)[0].strip()          # trailing comments
        if not s:
            continue
        parts = s.split(None, 1)
        mn, ops = parts[0], (parts[1] if len(parts) > 1 else "")
        tracked_in_flight = [q for q in queue if q[0]]
        if mn == "s_waitcnt":
            m = LGKM.search(ops)
            if m is None and re.fullmatch(r"(0x[0-9a-fA-F]+|\d+)", ops.strip() or "x"):
                imm = int(ops.strip(), 0)
                n = (imm >> 8) & 0xF          # gfx9 encoding: lgkmcnt in bits 11:8
                m = True
            elif m is not None:
                n = int(m.group(1))
            if m:
                if n > 0 and tracked_in_flight and any(q[1] for q in queue):
                    findings.append(f"{path}:{ln}: {func}: lgkmcnt({n}) with a scalar-memory load in flight beside hand-issued LDS reads "
                                    f"(issued at line {tracked_in_flight[0][2]}): completion order is not guaranteed")
                queue = queue[len(queue) - n:] if n < len(queue) else queue
                if n == 0:
                    queue = []
            continue
        if tracked_in_flight:
            used = regs_of(ops)
            for regs, _, at in tracked_in_flight:
                hit = used & regs
                if hit and not (in_asm and mn.startswith("ds_read")):
                    k, i = sorted(hit)[0]
                    findings.append(f"{path}:{ln}: {func}: `{s}` names {k}{i}, destination of the LDS read issued from asm at line {at}, "
                                    "before the wait that covers it")
                elif hit:
                    k, i = sorted(hit)[0]
                    findings.append(f"{path}:{ln}: {func}: a second asm LDS read targets {k}{i} while the read from line {at} is in flight")
        if mn == "s_endpgm" or mn == "s_setpc_b64":
            for regs, _, at in tracked_in_flight:
                findings.append(f"{path}:{ln}: {func}: the LDS read issued from asm at line {at} is never waited for")
            queue = []
            continue
        if mn.startswith("s_cbranch") or mn == "s_branch":
            target = ops.strip()
            # backward branch: the loop head is entered again with exactly the reads in flight that
            # the code after it was checked with (same registers, same order), or with none
            if target in labels_seen and [q[0] for q in tracked_in_flight] != labels_seen[target]:
                at = tracked_in_flight[0][2] if tracked_in_flight else ln
                findings.append(f"{path}:{ln}: {func}: backward branch to {target} with other hand-issued LDS reads in flight "
                                f"(first from line {at}) than when the loop was entered")
            continue
        if counts_in_lgkm(mn):
            if in_asm and mn.startswith("ds_read"):
                dst = ops.split(",", 1)[0]
                queue.append((frozenset(regs_of(dst)), False, ln))
                n_tracked += 1
            else:
                queue.append((None, is_smem(mn), ln))
    return findings, n_tracked


def main():
    bad = 0
    for path in sys.argv[1:]:
        findings, n = check(path)
        for f in findings[:50]:
            print("error:", f)
        bad += len(findings)
        print(f"{path}: {n} hand-issued LDS reads checked, {len(findings)} findings")
    sys.exit(1 if bad else 0)


if __name__ == "__main__":
    main()
