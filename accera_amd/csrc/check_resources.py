#!/usr/bin/env python3
"""Reads the compiler's kernel-resource-usage remarks of one translation unit (hipcc -Rpass-analysis=kernel-resource-usage,
stderr saved by the Makefile) and fails when a four-wave GEMM kernel uses scratch memory; and reads the assembly the
compiler wrote for the same translation unit (-save-temps) and fails when, in such a kernel, an accumulator register
(a0..a255) appears outside the kernel's own asm statements.

Those kernels keep 256 accumulators in a[0:255] across separate asm statements and pass the K loop ~28 operands; the
registers around the loop are tight by design.  A kernel that touches scratch at all pays for it at every dispatch (a
256-workgroup launch costs ~4 us more), and a lambda that stops being inlined, or address arithmetic hoisted out of the
tile loop, shows up here first: as bytes of scratch per lane.

The accumulators stay in a[0:255] from the statements that set them up, through the K loop, to the statements of the
write-back; the compiler is told that those statements clobber them, not that they carry values, so it must not use
the accumulator file for anything of its own in between (copies of vector registers it has run out of, say).  It does
not today -- the kernels ask for all 256 vector registers and the allocator prefers them -- and the check keeps it so.

    python3 check_resources.py <remarks .txt | assembly .s> [...]
"""
import re
import sys


def kernels(text):
    """(function name, {field: value}) per kernel of the remarks text."""
    out, cur = [], None
    for line in text.splitlines():
        m = re.search(r"remark:\s+(.*?)(?:\s+\[-Rpass-analysis=kernel-resource-usage\])?$", line)
        if not m:
            continue
        body = m.group(1).strip()
        if body.startswith("Function Name:"):
            cur = (body.split(":", 1)[1].strip(), {})
            out.append(cur)
        elif cur and ":" in body:
            k, v = body.split(":", 1)
            cur[1][k.strip()] = v.strip()
    return out


_AREG = re.compile(r"(?<![\w.$])a(\d+|\[\d+:\d+\])(?!\w)")


def agpr_uses_outside_asm(text):
    """{kernel: [lines]} of compiler-written instructions that name an accumulator register, per four-wave kernel of an
    assembly listing; and the number of such kernels seen."""
    cur, in_asm, bad, seen = None, False, {}, set()
    for line in text.splitlines():
        m = re.match(r"^(_ZN6acc950\w+):", line)
        if m:
            cur, in_asm = m.group(1), False
        elif line.startswith(".Lfunc_end"):
            cur = None
        if cur is None or "gemm_mfma16w4_kernel" not in cur:
            continue
        seen.add(cur)
        if ";;#ASMSTART" in line:
            in_asm = True
        elif ";;#ASMEND" in line:
            in_asm = False
        elif not in_asm:
            code = line.split(";")[0]
            if _AREG.search(code) or "v_accvgpr" in code:
                bad.setdefault(cur, []).append(line.strip())
    return bad, len(seen)


def main(paths):
    bad, seen = [], 0
    for path in [p for p in paths if p.endswith(".s")]:
        uses, n = agpr_uses_outside_asm(open(path, errors="replace").read())
        seen += n
        for name, lines in uses.items():
            bad.append(f"{name}: the compiler uses accumulator registers outside the asm statements, e.g. `{lines[0]}` ({len(lines)} places)")
    for path in [p for p in paths if not p.endswith(".s")]:
        for name, f in kernels(open(path, errors="replace").read()):
            if "gemm_mfma16w4_kernel" not in name:
                continue
            seen += 1
            scratch = int(f.get("ScratchSize [bytes/lane]", "0"))
            if scratch:
                bad.append(f"{name}: {scratch} bytes of scratch per lane (VGPRs spilled: {f.get('VGPRs Spill')}, SGPRs spilled: {f.get('SGPRs Spill')})")
    if bad:
        print("four-wave GEMM kernels must not use scratch memory, nor the compiler their accumulator registers:\n  " + "\n  ".join(bad), file=sys.stderr)
        return 1
    if paths and not seen:
        print("no four-wave GEMM kernel found in " + ", ".join(paths), file=sys.stderr)
        return 1
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
