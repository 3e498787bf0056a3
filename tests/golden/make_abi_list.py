"""Writes tests/golden/reference_abi.json: every function the reference's public headers declare inside the line
ranges that include/boat_api.h cites ("include/boat/<header>.h:A-B" in its section comments), with a normalised
prototype.  tests/test_abi.py holds libboat_amd.so and include/boat_api.h to this list, so a symbol of a cited range
that the library does not export, or declares differently, fails a CPU test.

Each entry also says whether the reference DEFINES the function ("defined": the symbol is exported by
oracle/_ref/libboat_ref.so, the reference's sources compiled by oracle/Makefile).  A function its headers declare but
no source defines cannot be called by any program linked against the reference, so the drop-in owes it nothing; the
test requires the defined ones.

Run where the reference tree is present and `make -C oracle ref` has been run:
    python tests/golden/make_abi_list.py [/root/reference]
The reference's headers are read as text and the compiled reference's symbol table is listed; nothing is run.
"""
from __future__ import annotations

import json
import re
import subprocess
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent.parent
OUT = Path(__file__).resolve().parent / "reference_abi.json"

CITATION = re.compile(r"include/(boat(?:/[a-z_]+)*\.h):(\d+)(?:-(\d+))?((?:\s*,\s*:?\d+(?:-\d+)?)*)")
EXTRA = re.compile(r":?(\d+)(?:-(\d+))?")


def cited_ranges(api_header: str) -> dict[str, list[tuple[int, int]]]:
    """{header path under include/: [(first, last), ...]} from the section comments of boat_api.h."""
    ranges: dict[str, list[tuple[int, int]]] = {}
    for line in api_header.splitlines():
        current = None
        for m in CITATION.finditer(line):
            current = m.group(1)
            a = int(m.group(2))
            b = int(m.group(3) or a)
            ranges.setdefault(current, []).append((a, b))
            for e in EXTRA.finditer(m.group(4) or ""):
                ea = int(e.group(1))
                ranges[current].append((ea, int(e.group(2) or ea)))
        # "layers.h:38-51 (2-D convolution), :68-72 (max pooling), :128-132 (flatten)": bare ranges after a header
        if current:
            for m in re.finditer(r"(?<![\w.]):(\d+)-(\d+)", line):
                span = (int(m.group(1)), int(m.group(2)))
                if span not in ranges[current]:
                    ranges[current].append(span)
    return ranges


def normalise(proto: str) -> str:
    """A prototype with export/calling-convention macros, parameter names and spacing removed."""
    proto = re.sub(r"/\*.*?\*/", " ", proto, flags=re.S)
    proto = re.sub(r"//[^\n]*", " ", proto)
    proto = re.sub(r"\b(BOAT_API|BOAT_CALL|BOAT_NOINLINE|extern)\b", " ", proto)
    proto = " ".join(proto.replace("\n", " ").split()).rstrip(";").strip()
    m = re.match(r"(.*?)\b([a-z_][a-z0-9_]*)\s*\((.*)\)$", proto)
    if not m:
        raise ValueError(proto)
    ret, name, args = m.group(1).strip(), m.group(2), m.group(3).strip()

    def strip_name(arg: str) -> str:
        arg = arg.strip()
        if arg in ("void", "..."):
            return arg
        fn = re.match(r"(.*)\(\s*\*\s*[a-z_0-9]*\s*\)\s*\((.*)\)$", arg)   # function pointer parameter
        if fn:
            inner = ",".join(strip_name(a) for a in split_args(fn.group(2)))
            return f"{squeeze(fn.group(1))}(*)({inner})"
        arr = re.match(r"(.*?)([a-z_][a-z0-9_]*)?\s*(\[[^\]]*\])$", arg)
        if arr:
            return squeeze(arr.group(1)) + "*"
        m2 = re.match(r"(.*?[\s*])([a-z_][a-z0-9_]*)$", arg)
        if m2 and m2.group(2) not in ("int", "float", "double", "char", "bool", "size_t", "void", "long", "short",
                                      "unsigned", "int64_t", "int32_t", "uint8_t", "uint64_t", "uint32_t") \
                and not m2.group(2).endswith("_t"):
            return squeeze(m2.group(1))
        return squeeze(arg)

    return f"{squeeze(ret)} {name}({','.join(strip_name(a) for a in split_args(args))})"


def squeeze(t: str) -> str:
    t = " ".join(t.split())
    return re.sub(r"\s*\*\s*", "*", t).strip()


def split_args(args: str) -> list[str]:
    out, depth, cur = [], 0, ""
    for ch in args:
        if ch == "(":
            depth += 1
        elif ch == ")":
            depth -= 1
        if ch == "," and depth == 0:
            out.append(cur)
            cur = ""
        else:
            cur += ch
    if cur.strip():
        out.append(cur)
    return out or ["void"]


def declarations(text: str):
    """(first line, name, normalised prototype) of every BOAT_API function declaration in a header."""
    lines = text.splitlines()
    i = 0
    while i < len(lines):
        if re.match(r"\s*BOAT_API\b", lines[i]) and "(" in "".join(lines[i:i + 3]):
            j, stmt = i, lines[i]
            while ";" not in stmt and j + 1 < len(lines):
                j += 1
                stmt += "\n" + lines[j]
            stmt = stmt.split(";")[0]
            if "(" in stmt and "typedef" not in stmt:
                proto = normalise(stmt)
                name = re.search(r"\b([a-z_][a-z0-9_]*)\(", proto).group(1)
                yield i + 1, name, proto
            i = j + 1
        else:
            i += 1


def main() -> None:
    ref = Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
    ranges = cited_ranges((ROOT / "include" / "boat_api.h").read_text())
    ref_so = ROOT / "oracle" / "_ref" / "libboat_ref.so"
    nm = subprocess.run(["nm", "-D", "--defined-only", str(ref_so)], check=True, capture_output=True, text=True).stdout
    defined = {line.split()[-1] for line in nm.splitlines() if " T " in line}
    entries = []
    for header, spans in sorted(ranges.items()):
        path = ref / "include" / header
        if not path.exists():
            continue
        for line, name, proto in declarations(path.read_text()):
            if any(a <= line <= b for a, b in spans):
                entries.append({"header": header, "line": line, "name": name, "prototype": proto, "defined": name in defined})
    exports = sorted(n for n in defined if n.startswith("boat_"))      # every boat_* function the reference's library defines
    OUT.write_text(json.dumps({"cited_ranges": {h: s for h, s in sorted(ranges.items())}, "functions": entries, "exports": exports},
                              indent=1) + "\n")
    print(f"{len(entries)} functions ({sum(e['defined'] for e in entries)} defined by the reference) in {len(ranges)} headers -> {OUT}")


if __name__ == "__main__":
    main()
