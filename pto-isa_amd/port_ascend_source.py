#!/usr/bin/env python3
"""Mechanical edits that turn a PTO kernel source written for the Ascend toolchain into a gfx950 translation unit.

    python pto-isa_amd/port_ascend_source.py IN.cpp OUT.hip [--set NAME=VALUE ...] [--define NAME[=VALUE] ...]
                                             [--lds BYTES] [--vec-in-memory] [--no-inline] [--l1 OLD=NEW ...]

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
5. Headers that sit next to the source (`#include "name"`) are inlined so that the edits reach them; an inlined `.hpp`
   is device code as a whole.
6. `static T name = init;` inside a function becomes `PTO_CORE_STATIC(T, name, init, number);` (a per-wave slot in LDS,
   numbered per translation unit, at most 32: a GPU function cannot keep a core-private `static`), and every `__global__` function starts with `PTO_KERNEL_PROLOGUE();`.
7. `--define NAME[=VALUE]` puts `#define`s in front of everything (the `__DAV_*` macros by which a source asks which
   kind of core it is compiled for: a workgroup plays both, so both may be defined).
8. `__global__` becomes `__global__ __launch_bounds__(pto::kBlockThreads)`.
9. `--vec-in-memory` defines PTO_VEC_TILES_IN_MEMORY (Vec tiles are addresses in a per-workgroup unified buffer, see
   include/pto/common/tile.hpp) and makes every launch prepare that buffer (`pto::host::LaunchBlocks`).
10. A source that names the Ascend compiler's built-in variables `block_idx` / `block_num` gets them as macros over
    `get_block_idx()` / `get_block_num()`, defined after the library's headers.
11. `--l1 OLD=NEW` rewrites the literal address of `TASSIGN(tile, OLD)`: sources place their L1 tiles at addresses laid
    out for Ascend's 512 KiB (0x20000, 0x40000 ...), which have to move inside the 160 KiB of LDS.  Register tiles ignore
    their address, so rewriting theirs too changes nothing.
12. Reads of Ascend's special scalar registers written as inline assembly, `asm volatile("MOV %0, SYS_CNT\n" : "+l"(x));`
    and `... PC ...`, become `x = get_sys_cnt();` and `x = 0;` (time stamps that the test kernels log, and the program
    counter they hand to an instruction-cache preload, which is a no-op here).
13. Loops over role blocks are split.  A source written for a Cube core and its Vec cores interleaves their work in one
    loop, `for (...) { if constexpr (DAV_CUBE) {A} if constexpr (DAV_VEC) {B} if constexpr (DAV_CUBE) {C} }`, and relies
    on the cores running side by side: B of an iteration may wait (through a FIFO) for what A produces in later
    iterations (the flash-attention kernel's Vec side takes a row slice of a whole score tile of which each iteration of
    its Cube side produces one column block, fa_performance_kernel.cpp:862-907).  One workgroup plays both roles in
    program order, so an innermost loop whose body is nothing but such blocks becomes one loop per block with the same
    header, `for (...) {A}  for (...) {B}  for (...) {C}`: every producer has then run before its consumer.  The blocks
    talk to each other through FIFOs only, which is what makes the order of different roles' blocks free on the NPU too.
"""
import argparse
import os
import re
import sys

LAUNCH = re.compile(r"<<<\s*([^,<>]+?)\s*,\s*nullptr\s*,\s*([^<>]+?)\s*>>>")
LOCAL_INCLUDE = re.compile(r'^[ \t]*#include[ \t]+"([^"]+)"[ \t]*$', re.M)
STATIC_LOCAL = re.compile(r"^([ \t]+)static[ \t]+([A-Za-z_][\w:]*(?:[ \t]+[A-Za-z_][\w:]*)*)[ \t]+([A-Za-z_]\w*)[ \t]*=[ \t]*([^;]+);", re.M)
KERNEL_HEAD = re.compile(r"__global__[^;{}]*?\)\s*\{")
ROLE_BLOCK = re.compile(r"\s*if\s+constexpr\s*\(\s*DAV_(?:CUBE|VEC)\s*\)\s*\{")
FOR_HEAD = re.compile(r"^([ \t]*)for\s*\(", re.M)
BEGIN_MARK, END_MARK = "//@@PTO_INLINED_BEGIN ", "//@@PTO_INLINED_END "


def _match(text, pos, open_ch, close_ch):
    """Index just behind the bracket that closes the one at text[pos] (comments and literals of the sources this script
    sees hold no unbalanced brackets)."""
    depth = 0
    for i in range(pos, len(text)):
        c = text[i]
        if c == open_ch:
            depth += 1
        elif c == close_ch:
            depth -= 1
            if depth == 0:
                return i + 1
    raise SystemExit("port_ascend_source: unbalanced %s" % open_ch)


def split_role_loops(text):
    """Rule 13: innermost `for` loops whose body consists of two or more `if constexpr (DAV_CUBE / DAV_VEC) {...}` blocks
    and nothing else become one loop per block.  Returns the new text and the number of loops split."""
    out, pos, count = [], 0, 0
    for m in FOR_HEAD.finditer(text):
        if m.start() < pos:
            continue
        head_end = _match(text, text.index("(", m.start()), "(", ")")
        brace = re.compile(r"\s*\{").match(text, head_end)
        if not brace:
            continue
        body_begin, body_end = brace.end(), _match(text, brace.end() - 1, "{", "}") - 1
        body = text[body_begin:body_end]
        blocks, at = [], 0
        while True:
            rb = ROLE_BLOCK.match(body, at)
            if not rb:
                break
            end = _match(body, rb.end() - 1, "{", "}")
            blocks.append(body[at:end])
            at = end
        if len(blocks) < 2 or body[at:].strip() or any(re.search(r"\bfor\s*\(", blk) for blk in blocks):
            continue
        indent, header = m.group(1), text[m.start():head_end].lstrip()
        loops = "\n".join("%s%s {%s\n%s}" % (indent, header, blk.rstrip(), indent) for blk in blocks)
        out.append(text[pos:m.start()] + loops)
        pos = body_end + 1
        count += 1
    out.append(text[pos:])
    return "".join(out), count


def inline_local_includes(text, directory, seen=None):
    """Replaces `#include "name"` by the text of `directory/name` where that file exists (headers that sit next to the kernel
    source: the edits below have to reach them too).  Each file once; the rest of its includes are left alone."""
    seen = set() if seen is None else seen

    def repl(m):
        name = m.group(1)
        path = os.path.join(directory, name)
        if not os.path.isfile(path):
            return m.group(0)
        if path in seen:
            return "// (already included above: %s)" % name
        seen.add(path)
        with open(path) as f:
            body = inline_local_includes(f.read(), os.path.dirname(path), seen)
        return BEGIN_MARK + name + "\n" + body + "\n" + END_MARK + name
    return LOCAL_INCLUDE.sub(repl, text)


def kernel_before(text, pos):
    """The kernel expression (`name` or `name<template arguments>`) that ends just before the `<<<` at text[pos]."""
    i = pos
    while i > 0 and text[i - 1].isspace():
        i -= 1
    end = i
    if i > 0 and text[i - 1] == ">":
        depth = 0
        while i > 0:
            i -= 1
            if text[i] == ">":
                depth += 1
            elif text[i] == "<":
                depth -= 1
                if depth == 0:
                    break
            elif text[i] in ";{}":
                return None
        if depth != 0:
            return None
        while i > 0 and text[i - 1].isspace():
            i -= 1
    # a name that a macro call pastes together (`CONCAT(run, CASENAME)<...>`): the call belongs to the expression
    if i > 0 and text[i - 1] == ")":
        depth = 0
        while i > 0:
            i -= 1
            if text[i] == ")":
                depth += 1
            elif text[i] == "(":
                depth -= 1
                if depth == 0:
                    break
            elif text[i] in ";{}":
                return None
        if depth != 0:
            return None
    start = i
    while start > 0 and (text[start - 1].isalnum() or text[start - 1] in "_:"):
        start -= 1
    if start == i:
        return None
    return " ".join(text[start:end].split())


ASCEND_SREG_READ = re.compile(r'asm\s+volatile\s*\(\s*"MOV %0, (SYS_CNT|PC)\\n"\s*:\s*"\+l"\s*\(\s*(\w+)\s*\)\s*\)\s*;')
TASSIGN_LITERAL = re.compile(r"(TASSIGN\(\s*\w+\s*,\s*)(0[xX][0-9a-fA-F]+|\d+)(\s*\))")


def port(text, sets=(), lds_bytes=160 * 1024, defines=(), directory=None, vec_in_memory=False, l1_map=None):
    notes = []
    if directory is not None:
        before = text
        text = inline_local_includes(text, directory)
        notes.append("%d local include%s inlined" % (text.count(BEGIN_MARK), "" if text.count(BEGIN_MARK) == 1 else "s"))
    for name, value in sets:
        pat = re.compile(r"(constexpr\s+[\w:]+\s+%s\s*=\s*)([^;]+)(;)" % re.escape(name))
        text, n = pat.subn(lambda m: m.group(1) + value + m.group(3), text)
        if n == 0:
            raise SystemExit("port_ascend_source: no `constexpr ... %s = ...;` in the source" % name)
        notes.append("set %s = %s (%d place%s)" % (name, value, n, "" if n == 1 else "s"))

    # 11. L1 addresses
    if l1_map:
        table = {int(str(k), 0): int(str(v), 0) for k, v in dict(l1_map).items()}
        hits = [0]

        def move(m):
            a = int(m.group(2), 0)
            if a not in table:
                return m.group(0)
            hits[0] += 1
            return "%s0x%x%s" % (m.group(1), table[a], m.group(3))
        text = TASSIGN_LITERAL.sub(move, text)
        notes.append("%d TASSIGN address%s moved" % (hits[0], "" if hits[0] == 1 else "es"))

    # 12. special-register reads
    text, n = ASCEND_SREG_READ.subn(lambda m: "%s = %s;" % (m.group(2), "get_sys_cnt()" if m.group(1) == "SYS_CNT" else "0"), text)
    if n:
        notes.append("%d special-register read%s rewritten" % (n, "" if n == 1 else "s"))

    # 2. launch statements
    blocks = "pto::host::LaunchBlocks(%s, (hipStream_t)(%s))" if vec_in_memory else "%s"

    unnamed = [0]

    def launch(m):
        b = blocks % (m.group(1), m.group(2)) if vec_in_memory else m.group(1)
        kernel = kernel_before(m.string, m.start())
        # the kernel's own static LDS (staging buffers of the tile library, PTO_CORE_STATIC slots) comes out of the same
        # 160 KiB: the dynamic part shrinks by it, or the dispatch would be refused by the hardware queue
        lds = "pto::host::LaunchLds((const void *)(%s), %d)" % (kernel, lds_bytes) if kernel else "%d" % lds_bytes
        if not kernel:
            unnamed[0] += 1
        return "<<<%s, pto::kBlockThreads, %s, (hipStream_t)(%s)>>>" % (b, lds, m.group(2))
    text, n = LAUNCH.subn(launch, text)
    notes.append("%d launch statement%s rewritten" % (n, "" if n == 1 else "s"))
    if unnamed[0]:
        notes.append("WARNING: %d launch%s whose kernel expression was not recognised keep the full dynamic LDS size; a kernel with "
                     "__shared__ variables of its own then asks for more than a compute unit has" % (unnamed[0], "" if unnamed[0] == 1 else "es"))

    # 9. kernels are launched with pto::kBlockThreads threads: tell the compiler (it assumes 1024 otherwise and has half the
    # registers per thread to work with)
    text, n = re.subn(r"__global__(?!\s*__launch_bounds__)", "__global__ __launch_bounds__(pto::kBlockThreads)", text)

    # 5. function-local statics of device functions, and the prologue that resets them
    numbered = [0]

    def core_static(m):
        numbered[0] += 1
        return "%sPTO_CORE_STATIC(%s, %s, %s, %d);" % (m.group(1), m.group(2), m.group(3), m.group(4).strip(), numbered[0] - 1)
    text, n = STATIC_LOCAL.subn(core_static, text)
    if n > 32:
        raise SystemExit("port_ascend_source: %d function-local statics, the per-wave area has 32 slots" % n)
    if n:
        notes.append("%d function-local static%s rewritten" % (n, "" if n == 1 else "s"))
        text, k = KERNEL_HEAD.subn(lambda m: m.group(0) + "\n    PTO_KERNEL_PROLOGUE();", text)
        notes.append("%d kernel prologue%s inserted" % (k, "" if k == 1 else "s"))
    # 13. the flash-attention kernel: one workgroup plays the Cube and the Vec role of a block in program order
    text, k13 = split_role_loops(text)
    if k13:
        notes.append("%d loop%s over Cube / Vec role blocks split into one loop per block" % (k13, "" if k13 == 1 else "s"))

    # 1. brackets.  Inlined .hpp files are device code as a whole; in the main file the device code opens after the
    # prologue (comments, includes, using-directives, macro definitions and file-scope constants come first in these
    # sources; the first AICORE / template / enum line starts the device code) and closes before the first host function.
    lines = text.split("\n")
    out, depth, main_idx = [], 0, []
    for l in lines:
        if l.startswith(BEGIN_MARK):
            depth += 1
            out.append("// ---- " + l[len(BEGIN_MARK):] + " (inlined)")
            if depth == 1 and l.rstrip().endswith(".hpp"):
                out.append("PTO_DEVICE_CODE_BEGIN")
            continue
        if l.startswith(END_MARK):
            if depth == 1 and l.rstrip().endswith(".hpp"):
                out.append("PTO_DEVICE_CODE_END")
            depth -= 1
            out.append("// ---- end of " + l[len(END_MARK):])
            continue
        if depth == 0:
            main_idx.append(len(out))
        out.append(l)
    lines = out
    is_main = set(main_idx)
    first_dev = next((i for i in main_idx if re.match(r"\s*(template\s*<|AICORE\b|__global__\b|constexpr\s+AICORE|enum\b)", lines[i])), None)
    if first_dev is None:
        raise SystemExit("port_ascend_source: no device function found")
    # Top-level declarations of the main file from there on: a declaration ends where braces and parentheses are balanced
    # and the line ends in `}` or `;`.  A host declaration is one that launches a kernel (`<<<`) or explicitly instantiates
    # a host template (`template void ...;`); device regions are the runs between host declarations (sources that
    # alternate kernels and their launchers get one region per run).
    def strip_code(l):
        l = re.sub(r'"(?:[^"\\]|\\.)*"', '""', l)
        l = re.sub(r"'(?:[^'\\]|\\.)'", "''", l)
        return l.split("//", 1)[0]
    chunks, start, braces, parens, in_comment = [], None, 0, 0, False     # (first line, last line, is host)
    for i in range(first_dev, len(lines)):
        if i not in is_main:
            continue
        l = lines[i]
        if in_comment:
            if "*/" in l:
                in_comment = False
            continue
        code = strip_code(l).strip()
        if code.startswith("/*") and "*/" not in code:
            in_comment = True
            continue
        if start is None:
            if code == "" or code.startswith(("#", "/*")):
                continue
            start = i
        braces += code.count("{") - code.count("}")
        parens += code.count("(") - code.count(")")
        if braces == 0 and parens == 0 and code.endswith(("}", ";")):
            body = "\n".join(lines[start:i + 1])
            host = "<<<" in body or re.match(r"\s*template\s+(?!<)", lines[start]) is not None or \
                re.match(r'\s*extern\s+"C"\s+(?!.*__global__)', lines[start]) is not None and "AICORE" not in lines[start]
            marked = re.search(r"\b(AICORE|__aicore__|__global__|PTO_INTERNAL|PTO_INST)\b", body.split("{", 1)[0]) is not None
            # the declaration of a host function (no body, no device marker: `template <...> void Launch(T *out, void *stream);`,
            # specialised further down with the launches in the bodies) is host code too
            flat = " ".join(strip_code(x) for x in lines[start:i + 1]).strip()
            if not host and not marked and "{" not in flat and \
                    re.match(r"^(template\s*<[^;{}]*>\s*)?(?!static_assert|using|typedef|return)[\w:]+[\w:<>,\*&\s]*?\b\w+\s*\([^;{}]*\)\s*;$", flat):
                host = True
            chunks.append((start, i, host, marked))
            start = None
    res, pos, open_region, regions = lines[:first_dev], first_dev, False, 0
    seen_host = False
    for (c0, c1, host, marked) in chunks:
        if host and open_region:
            res.append("PTO_DEVICE_CODE_END")
            open_region = False
        seen_host = seen_host or host
        res += lines[pos:c0]
        # after the first host declaration only a declaration that carries a device marker opens a region again
        if not host and not open_region and (marked or not seen_host):
            res.append("PTO_DEVICE_CODE_BEGIN")
            open_region = True
            regions += 1
        res += lines[c0:c1 + 1]
        pos = c1 + 1
    res += lines[pos:]
    if open_region:
        res.append("PTO_DEVICE_CODE_END")
    notes.append("device code: %d region%s from line %d" % (regions, "" if regions == 1 else "s", first_dev + 1))
    head = "#define PTO_TILE_COPY_WRITEBACK 1\n"
    if vec_in_memory:
        head += "#define PTO_VEC_TILES_IN_MEMORY 1\n"
    for d in defines:
        name, _, value = d.partition("=")
        head += "#define %s %s\n" % (name, value or "1")
    head += "#include <hip/hip_runtime.h>\n"
    # the Ascend compiler's built-in variables `block_idx` / `block_num`
    # (not where the source declares a variable of that name itself)
    builtins = [n for n in ("block_idx", "block_num")
                if re.search(r"\b%s\b" % n, text) and not re.search(r"\b(?:int|auto|unsigned|u?int(?:32|64)_t)\s+%s\b" % n, text)]
    if builtins:
        head += "#include <pto/pto-inst.hpp>\n" + "".join("#define %s (get_%s())\n" % (n, n) for n in builtins)
        notes.append(" / ".join(builtins) + " -> get_...()")
    return head + "\n".join(res), notes


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("src")
    ap.add_argument("dst")
    ap.add_argument("--set", action="append", default=[], metavar="NAME=VALUE")
    ap.add_argument("--define", action="append", default=[], metavar="NAME[=VALUE]")
    ap.add_argument("--lds", type=int, default=160 * 1024)
    ap.add_argument("--vec-in-memory", action="store_true")
    ap.add_argument("--no-inline", action="store_true", help="leave `#include \"...\"` of files next to the source alone")
    ap.add_argument("--l1", action="append", default=[], metavar="OLD=NEW", help="move the literal address of TASSIGN(tile, OLD)")
    args = ap.parse_args()
    sets = [tuple(s.split("=", 1)) for s in args.set]
    with open(args.src) as f:
        text = f.read()
    out, notes = port(text, sets, args.lds, args.define, None if args.no_inline else os.path.dirname(os.path.abspath(args.src)),
                      args.vec_in_memory, dict(x.split("=", 1) for x in args.l1))
    with open(args.dst, "w") as f:
        f.write(out)
    for n in notes:
        print("port_ascend_source:", n, file=sys.stderr)


if __name__ == "__main__":
    main()
