#!/usr/bin/env python3
"""Build-time check that no kernel of a translation unit spills registers.

A kernel that runs out of registers still gives right results, from scratch memory, at a fraction of its speed, and nothing
says so: the build fails instead.  hipcc prints the resources of every kernel with -Rpass-analysis=kernel-resource-usage;
this script reads those remarks and fails when a kernel uses scratch memory ("ScratchSize [bytes/lane]" above zero), unless its
name matches one of the patterns below, which name the kernels that keep a small array in private memory on purpose.

usage: check_spills.py <file with the remarks> [<more files>]
"""
import re
import subprocess
import sys

# (pattern of the demangled name, most bytes per lane, why)
ALLOWED = [
    (r"\bdequant_tiled_kernel<", 256, "load time only: one thread rebuilds one native block in a private array, written for clarity"),
    (r"\bgather_tiled_kernel<", 256, "the same private block, for embedding rows of a table kept in the tiled layout"),
    (r"\bgemv_cs_staged_gateup_kernel<13, 0, 16, 6, 0>", 16, "Q5_K gate / up at 9 .. 16 f32 rows with six tiles per workgroup: four dwords over the register file, accepted as it is"),
]


def demangle(names):
    if not names:
        return {}
    out = subprocess.run(["c++filt"], input="\n".join(names), capture_output=True, text=True, check=True).stdout.splitlines()
    return dict(zip(names, out))


def main(paths):
    found = []          # (file, mangled name, bytes)
    kernels = 0
    for path in paths:
        name = None
        with open(path, errors="replace") as f:
            for line in f:
                m = re.search(r"Function Name: (\S+)", line)
                if m:
                    name = m.group(1)
                    kernels += 1
                    continue
                m = re.search(r"ScratchSize \[bytes/lane\]: (\d+)", line)
                if m and name and int(m.group(1)) > 0:
                    found.append((path, name, int(m.group(1))))
    readable = demangle(sorted({n for _, n, _ in found}))
    bad = []
    for path, name, nbytes in found:
        text = readable.get(name, name)
        if not any(re.search(pat, text) and nbytes <= most for pat, most, _ in ALLOWED):
            bad.append(f"{path}: {text[:160]} uses {nbytes} bytes of scratch per lane")
    if bad:
        print("check_spills: kernels that spill registers (or use private memory):", file=sys.stderr)
        for b in bad:
            print("  " + b, file=sys.stderr)
        return 1
    print(f"check_spills: {kernels} kernels in {len(paths)} file(s), none spills ({len(found)} use private memory as listed)")
    return 0


if __name__ == "__main__":
    if len(sys.argv) < 2:
        print(__doc__, file=sys.stderr)
        sys.exit(2)
    sys.exit(main(sys.argv[1:]))
