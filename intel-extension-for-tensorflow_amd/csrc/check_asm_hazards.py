"""Checks the device assembly of the tile kernels for the two hazards their inline assembly can create.

The compiler inserts wait counts and hazard wait states only for memory instructions it emitted itself; the ones
written as inline assembly in qgemm_common.hpp / qgemm_tile.hpp are opaque text to it:

1. The early channel-parameter loads (load_raw_channel_early) return their data some hundred cycles after issue.  Until
   an s_waitcnt vmcnt(n) with n <= (vector memory instructions issued since the load) no instruction may write the
   destination register or consume it.  The kernel waits by hand (wait_vmcnt + settle_raw_channel); this script proves
   that the register allocator put nothing in between, along every control-flow path of every instantiation.
   One pattern is reported as harmless and not counted: a 64-bit multiply-add whose addend pair has the pending register
   as its undefined high half (the compiler pairs a 32-bit offset with whatever register follows it when only the
   low half of the result is used); the script checks that the next instruction naming the high half of that result
   overwrites it.
2. A vector store of more than 8 bytes reads its data registers for two more cycles after issue.  Each write-through
   store in the epilogue must be followed by at least two wait states inside the same assembly statement.

Usage:  python check_asm_hazards.py            compiles every qgemm_tile_*.hip to assembly (minutes) and checks it
        python check_asm_hazards.py a.s b.s    checks assembly files made with the build's flags plus -S --offload-device-only
Exit status 0 when nothing is flagged.
"""
import concurrent.futures
import glob
import os
import re
import subprocess
import sys
import tempfile

VMEM = re.compile(r"^(global_|buffer_|flat_|scratch_)(load|store|atomic)")
EARLY = re.compile(r"global_load_(dword|ushort)\s+v(\d+),")
BRANCH = re.compile(r"(s_branch|s_cbranch_\w+)\s+(\S+)")


def vregs(code):
    regs = set(int(x) for x in re.findall(r"\bv(\d+)\b", code))
    for a, b in re.findall(r"\bv\[(\d+):(\d+)\]", code):
        regs.update(range(int(a), int(b) + 1))
    return regs


def dead_high_half(ins, pc, reg):
    """True when the next instruction after pc (in program order) that names `reg` only writes it."""
    for _, code, _ in ins[pc + 1:]:
        ops = code.split(None, 1)
        if len(ops) < 2 or reg not in vregs(code):
            continue
        dst = ops[1].split(",")[0]
        return reg in vregs(dst) and reg not in vregs(ops[1][len(dst):])
    return True


def check_function(ins, labels):
    """ins: [(line number, instruction text, inside an inline-assembly block)].  Returns (load sites, findings)."""
    sites = [i for i, (_, c, a) in enumerate(ins) if a and EARLY.match(c)]
    findings = set()
    # rule 2: wait states after the assembly store
    for i, (ln, code, in_asm) in enumerate(ins):
        if in_asm and re.match(r"global_store_dwordx[34]\b", code):
            nxt = ins[i + 1] if i + 1 < len(ins) else (0, "", False)
            m = re.match(r"s_nop\s+(\d+)", nxt[1])
            if not (nxt[2] and m and int(m.group(1)) >= 1):
                findings.add((ln, "assembly store without two wait states after it: " + code))
    if not sites:
        return 0, findings
    last = sites[-1]
    seen = set()
    work = [(0, (), (), None)]
    while work:
        pc, pend, kn, vcc = work.pop()
        pending, known = dict(pend), dict(kn)    # register -> vector memory instructions issued after its load
        while pc < len(ins):
            key = (pc, tuple(sorted(pending.items())), tuple(sorted(known.items())), vcc)
            if key in seen or (pc > last and not pending):
                break
            seen.add(key)
            ln, code, in_asm = ins[pc]
            if code.startswith("s_endpgm"):
                break
            mw = re.match(r"s_waitcnt.*vmcnt\((\d+)\)", code)
            if mw:
                pending = {r: k for r, k in pending.items() if k < int(mw.group(1))}
                pc += 1
                continue
            mb = BRANCH.match(code)
            if mb:
                tgt = labels[mb.group(2)]
                if mb.group(1) == "s_branch":
                    pc = tgt
                    continue
                taken = not_taken = True
                # if/else joins are expressed with a 64-bit scalar flag set to 0 or -1 on one side
                if mb.group(1) == "s_cbranch_vccz" and vcc:
                    taken, not_taken = vcc == "z", vcc == "nz"
                if mb.group(1) == "s_cbranch_vccnz" and vcc:
                    taken, not_taken = vcc == "nz", vcc == "z"
                if mb.group(1) == "s_cbranch_execz":
                    taken = False                # a running wavefront has at least one lane
                if taken and not_taken:
                    work.append((tgt, tuple(sorted(pending.items())), tuple(sorted(known.items())), vcc))
                    pc += 1
                else:
                    pc = tgt if taken else pc + 1
                continue
            if code.startswith("s_"):
                mm = re.match(r"s_mov_b64\s+(s\[\d+:\d+\]),\s*(0|-1)$", code)
                ma = re.match(r"s_andn2_b64\s+vcc,\s*exec,\s*(s\[\d+:\d+\])$", code)
                if mm:
                    known[mm.group(1)] = int(mm.group(2))
                elif ma:
                    vcc = {0: "nz", -1: "z"}.get(known.get(ma.group(1)))
                else:
                    md = re.match(r"s_\w+\s+(s\[\d+:\d+\]|vcc)", code)
                    if md and md.group(1) == "vcc":
                        vcc = None
                    elif md:
                        known.pop(md.group(1), None)
                pc += 1
                continue
            if code.startswith("v_cmp") or re.match(r"v_\w+\s+vcc", code):
                vcc = None
            regs = vregs(code)
            ml = EARLY.match(code) if in_asm else None
            if ml:
                dst = int(ml.group(2))
                hit = (regs - {dst}) & set(pending)
                if hit:
                    findings.add((ln, "an early load's address uses pending v%s: %s" % (sorted(hit), code)))
                if dst in pending and "saveexec" not in "".join(c for _, c, _ in ins[max(pc - 8, 0):pc]):
                    findings.add((ln, "an early load overwrites pending v%d: %s" % (dst, code)))
                for r in pending:
                    pending[r] += 1
                pending[dst] = 0
                pc += 1
                continue
            for h in sorted(regs & set(pending)):
                mad = re.match(r"v_mad_u64_u32\s+v\[(\d+):(\d+)\],.*,\s*v\[(\d+):(\d+)\]$", code)
                if mad and int(mad.group(4)) == h and dead_high_half(ins, pc, int(mad.group(2))):
                    continue                     # undefined high half of an addend whose high result is dead
                findings.add((ln, "v%d is used %d vector memory instruction(s) after its load with no wait: %s" % (h, pending[h], code)))
                pending.pop(h)
            if VMEM.match(code):
                for r in pending:
                    pending[r] += 1
            pc += 1
    return len(sites), findings


def check_file(path):
    func, in_asm, ins, labels = None, False, [], {}
    sites = flagged = funcs = 0

    def finish():
        nonlocal sites, flagged, funcs
        if func and ins:
            n, found = check_function(ins, labels)
            for ln, msg in sorted(found):
                print("%s:%d %s: %s" % (path, ln, func[:70], msg))
            sites, flagged, funcs = sites + n, flagged + len(found), funcs + 1

    for ln, line in enumerate(open(path), 1):
        s = line.strip()
        m = re.match(r"^([A-Za-z_.][\w$.]*):", line)
        if m:
            if m.group(1).startswith(".L"):
                labels[m.group(1)] = len(ins)
            else:
                finish()
                func, ins, labels = m.group(1), [], {}
            continue
        if s.startswith(";;#ASMSTART"):
            in_asm = True
        elif s.startswith(";;#ASMEND"):
            in_asm = False
        elif s and not s.startswith(";") and not s.startswith("."):
            code = s.split(";")[0].strip()
            if code:
                ins.append((ln, code, in_asm))
    finish()
    print("%s: %d functions, %d early load sites, %d flagged" % (os.path.basename(path), funcs, sites, flagged))
    return flagged


def compile_to_assembly(out_dir):
    here = os.path.dirname(os.path.abspath(__file__))
    sys.path.insert(0, os.path.dirname(here))
    import build as b
    srcs = sorted(glob.glob(os.path.join(here, "qgemm_tile_*.hip")))

    def one(src):
        out = os.path.join(out_dir, os.path.basename(src) + ".s")
        subprocess.run([b.HIPCC] + b.HIP_FLAGS + ["-S", "--offload-device-only", src, "-o", out], check=True,
                       stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
        return out
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as ex:
        return list(ex.map(one, srcs))


if __name__ == "__main__":
    files = sys.argv[1:]
    tmp = None
    if not files:
        tmp = tempfile.TemporaryDirectory()
        files = compile_to_assembly(tmp.name)
    bad = sum(check_file(f) for f in files)
    sys.exit(1 if bad else 0)
