#!/usr/bin/env python3
"""Mechanical edits that turn a PTO kernel source written for the Ascend toolchain into a gfx950 translation unit.

    python pto-isa_amd/port_ascend_source.py IN.cpp OUT.hip [--set NAME=VALUE ...] [--lds BYTES]

What a kernel source of the reference needs before `hipcc --offload-arch=gfx950 -I include` accepts it, and what this
script therefore does (nothing else is touched; the tile code itself compiles as it is):

1. Device code is bracketed.  The Ascend dialect marks device functions with `AICORE` only, which is empty here; the
   functions between `PTO_DEVICE_CODE_BEGIN` and `PTO_DEVICE_CODE_END` are compiled for the device.  The opening
   bracket goes after the last `#include` / `using namespace` line that precedes the first function, the closing
   one before the first host function (the first function that holds a `<<<` launch).
2. Launch statements.  `kernel<<<blocks, nullptr, stream>>>(...)` becomes
   `kernel<<<blocks, pto::kBlockThreads, LDS_BYTES, (hipStream_t)stream>>>(...)`: a PTO core is a workgroup of
   pto::kBlockThreads threads, and the Mat tiles it TASSIGNs live in dynamic LDS (--lds, default 160 KiB).
3. `PTO_TILE_COPY_WRITEBACK` is defined in front of everything: tiles passed by value hand their values back
   (see include/pto/common/tile.hpp).
4. `--set NAME=VALUE` rewrites `constexpr <type> NAME = <old>;`: tile-size constants chosen for 512 KiB of L1 have
   to fit the 160 KiB of LDS (the TASSIGN of a tile that does not fit is a compile error, not a silent overrun).
"""
import argparse
import re
import sys

LAUNCH = re.compile(r"<<<\s*([^,<>]+?)\s*,\s*nullptr\s*,\s*([^<>]+?)\s*>>>")


def port(text, sets=(), lds_bytes=160 * 1024):
    notes = []
    for name, value in sets:
        pat = re.compile(r"(constexpr\s+[\w:]+\s+%s\s*=\s*)([^;]+)(;)" % re.escape(name))
        text, n = pat.subn(lambda m: m.group(1) + value + m.group(3), text)
        if n == 0:
            raise SystemExit("port_ascend_source: no `constexpr ... %s = ...;` in the source" % name)
        notes.append("set %s = %s (%d place%s)" % (name, value, n, "" if n == 1 else "s"))

    # 2. launch statements
    text, n = LAUNCH.subn(lambda m: "<<<%s, pto::kBlockThreads, %d, (hipStream_t)(%s)>>>" % (m.group(1), lds_bytes, m.group(2)), text)
    notes.append("%d launch statement%s rewritten" % (n, "" if n == 1 else "s"))

    # 1. brackets: open after the prologue (comments, includes, using-directives, macro definitions and file-scope
    # constants come first in these sources; the first AICORE / template line starts the device code)
    lines = text.split("\n")
    first_dev = next((i for i, l in enumerate(lines) if re.match(r"\s*(template\s*<|AICORE\b|__global__\b|constexpr\s+AICORE|enum\b)", l)), None)
    if first_dev is None:
        raise SystemExit("port_ascend_source: no device function found")
    # the first host function: the first file-scope function whose body launches a kernel
    launch_line = next((i for i, l in enumerate(lines) if "<<<" in l), None)
    host_start = None
    if launch_line is not None:
        # walk back to the first line of the top-level declaration that encloses it: a line that starts at column 0
        # with a name and follows an empty line, a closing brace, a semicolon, a comment or a directive
        i = launch_line
        while i > 0:
            prev = lines[i - 1].strip()
            starts = re.match(r"^[A-Za-z_]", lines[i]) is not None
            if starts and (prev == "" or prev.endswith(("}", ";", "*/")) or prev.startswith(("//", "#"))):
                break
            i -= 1
        host_start = i
    out = lines[:first_dev] + ["PTO_DEVICE_CODE_BEGIN"]
    if host_start is not None and host_start > first_dev:
        out += lines[first_dev:host_start] + ["PTO_DEVICE_CODE_END"] + lines[host_start:]
        notes.append("device code: lines %d-%d" % (first_dev + 1, host_start))
    else:
        out += lines[first_dev:] + ["PTO_DEVICE_CODE_END"]
        notes.append("device code: line %d to the end" % (first_dev + 1))
    head = "#define PTO_TILE_COPY_WRITEBACK 1\n#include <hip/hip_runtime.h>\n"
    return head + "\n".join(out), notes


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("src")
    ap.add_argument("dst")
    ap.add_argument("--set", action="append", default=[], metavar="NAME=VALUE")
    ap.add_argument("--lds", type=int, default=160 * 1024)
    args = ap.parse_args()
    sets = [tuple(s.split("=", 1)) for s in args.set]
    with open(args.src) as f:
        text = f.read()
    out, notes = port(text, sets, args.lds)
    with open(args.dst, "w") as f:
        f.write(out)
    for n in notes:
        print("port_ascend_source:", n, file=sys.stderr)


if __name__ == "__main__":
    main()
