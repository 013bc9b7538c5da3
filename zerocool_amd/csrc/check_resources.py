#!/usr/bin/env python3
"""Build step: reads the compiler's kernel-resource-usage remarks of one translation unit and fails the build when a
kernel uses scratch memory (register spills or a stack).

Why this is enforced: the persistent decode kernel launches one workgroup per compute unit and its workgroups wait for
each other, so ALL of them must be resident at once.  Scratch is handed out per wave from a pool of bounded size; when a
kernel's demand (bytes per lane x 64 lanes x every wave of the grid) exceeds what the runtime grants one dispatch, the
dispatch runs with fewer wave slots than the grid has waves, the held-back workgroups never start, and the resident ones
wait for them for ever.  A 512-thread build that spilled 4.8 KB per lane (629 MB for the grid) ended that way.  Every
kernel of the library is therefore required to need no scratch at all.

usage: check_resources.py <remarks file> [--table]"""
import re
import sys


def parse(text):
    kernels, current = [], None
    for line in text.splitlines():
        m = re.search(r"remark:\s+Function Name:\s+(\S+)", line)
        if m:
            current = {"name": m.group(1)}
            kernels.append(current)
            continue
        m = re.search(r"remark:\s+([A-Za-z ]+?)(?: \[[^\]]*\])?:\s+(\S+) \[-Rpass-analysis", line)
        if m and current is not None:
            current[m.group(1).strip()] = m.group(2)
    return kernels


def main(argv):
    text = open(argv[1], errors="replace").read()
    for line in text.splitlines():      # warnings and errors of the compile stay visible
        if "remark:" not in line and "-Rpass-analysis" not in line and re.search(r"(warning|error):", line):
            print(line, file=sys.stderr)
    kernels = parse(text)
    bad = [k for k in kernels if int(k.get("ScratchSize", "0")) != 0 or int(k.get("VGPRs Spill", "0")) != 0 or k.get("Dynamic Stack") == "True"]
    if "--table" in argv:
        for k in kernels:
            print(f"{k['name'][:70]:70s} vgpr {k.get('VGPRs', '?'):>4s} agpr {k.get('AGPRs', '?'):>4s} lds {k.get('LDS Size', '?'):>6s} "
                  f"waves/SIMD {k.get('Occupancy', '?'):>2s} scratch {k.get('ScratchSize', '?')}")
    for k in bad:
        print(f"{argv[1]}: kernel {k['name']} needs scratch memory ({k.get('ScratchSize')} bytes per lane, "
              f"{k.get('VGPRs Spill')} spilled registers): refused, see the head of check_resources.py", file=sys.stderr)
    return 1 if bad else 0


if __name__ == "__main__":
    sys.exit(main(sys.argv))
