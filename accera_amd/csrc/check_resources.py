#!/usr/bin/env python3
"""Reads the compiler's kernel-resource-usage remarks of one translation unit (hipcc -Rpass-analysis=kernel-resource-usage,
stderr saved by the Makefile) and fails when a four-wave GEMM kernel uses scratch memory.

Those kernels keep 256 accumulators in a[0:255] across separate asm statements and pass the K loop ~28 operands; the
registers around the loop are tight by design.  A kernel that touches scratch at all pays for it at every dispatch (a
256-workgroup launch costs ~4 us more), and a lambda that stops being inlined, or address arithmetic hoisted out of the
tile loop, shows up here first: as bytes of scratch per lane.

    python3 check_resources.py <remarks file> [...]
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


def main(paths):
    bad, seen = [], 0
    for path in paths:
        for name, f in kernels(open(path, errors="replace").read()):
            if "gemm_mfma16w4_kernel" not in name:
                continue
            seen += 1
            scratch = int(f.get("ScratchSize [bytes/lane]", "0"))
            if scratch:
                bad.append(f"{name}: {scratch} bytes of scratch per lane (VGPRs spilled: {f.get('VGPRs Spill')}, SGPRs spilled: {f.get('SGPRs Spill')})")
    if bad:
        print("four-wave GEMM kernels must not use scratch memory:\n  " + "\n  ".join(bad), file=sys.stderr)
        return 1
    if paths and not seen:
        print("no four-wave GEMM kernel found in " + ", ".join(paths), file=sys.stderr)
        return 1
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
