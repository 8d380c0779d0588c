#!/usr/bin/env python3
"""Turn hipcc's -Rpass-analysis=kernel-resource-usage remarks (stdin or a file) into a table, one kernel per line:

    name<template arguments>  vgprs  agprs  sgprs  scratch_bytes_per_lane  waves_per_simd  static_lds_bytes

Called by the Makefile after the .hip files are compiled; the table is written next to libtdc_amd.so so that tests can
read what was compiled without a GPU.  With --inc as the first argument the output is a C++ initialiser list instead,

    {"name<template arguments>", vgprs + agprs, sgprs, waves_per_simd},

which tile_model.cpp includes: the tile model's occupancy term uses the registers of the kernels as compiled."""
import re
import subprocess
import sys


def main():
    args = sys.argv[1:]
    as_inc = bool(args) and args[0] == "--inc"
    if as_inc:
        args = args[1:]
    text = open(args[0]).read() if args else sys.stdin.read()
    blocks = re.split(r"remark: Function Name: ", text)[1:]
    names = [b.split()[0] for b in blocks]
    demangled = subprocess.run(["c++filt"] + names, capture_output=True, text=True, check=True).stdout.split("\n")
    rows = []
    for b, dem in zip(blocks, demangled):
        def field(key):
            return int(re.search(re.escape(key) + r": (\d+)", b).group(1))
        name = re.sub(r"^void ", "", dem).replace("tdc::", "")
        name = re.sub(r"\(.*\)$", "", name)
        rows.append((name, field("VGPRs"), field("AGPRs"), field("TotalSGPRs"), field("ScratchSize [bytes/lane]"),
                     field("Occupancy [waves/SIMD]"), field("LDS Size [bytes/block]")))
    if as_inc:
        lines = ['{"%s", %d, %d, %d},' % (r[0], r[1] + r[2], r[3], r[5]) for r in sorted(rows)]
        sys.stdout.write("\n".join(lines) + "\n")
        return
    out = ["# name | vgprs | agprs | sgprs | scratch bytes per lane | waves per SIMD | static LDS bytes"
           "   (hipcc -Rpass-analysis=kernel-resource-usage, gfx950)"]
    for r in sorted(rows):
        out.append("%s | %d | %d | %d | %d | %d | %d" % r)
    sys.stdout.write("\n".join(out) + "\n")


if __name__ == "__main__":
    main()
