"""Argument labels of the Swift doors of the quantized-matmul path.

`swift_doors(text)` parses Swift source and returns {"Type.func": [[label, ...], ...]} (one list per overload) for the static
functions of the top-level types in it.  Run as a script in a container that holds the reference checkout, it writes
swift_door_labels.json beside itself: the labels of the reference's doors (Sources/Operators/QWGEMM/*.swift), which are
data about its interface.  The shim's own labels are checked against that fixture by tests/test_swift_shim.py.
"""
import json
import re
import sys
from pathlib import Path

TYPE_RE = re.compile(r"^(?:public\s+)?(?:final\s+)?(?:enum|struct|class|extension)\s+(\w+)", re.M)
FUNC_RE = re.compile(r"(?<!private )\bstatic func\s+(\w+)\s*(?:<[^>]*>)?\s*\(")


def _split_top(params):
    parts, depth, cur = [], 0, ""
    for c in params.replace("->", "to"):                          # a closure's arrow is not a closing angle bracket
        depth += c in "([<"
        depth -= c in ")]>"
        if c == "," and depth == 0:
            parts.append(cur)
            cur = ""
        else:
            cur += c
    if cur.strip():
        parts.append(cur)
    return parts


def swift_doors(text):
    text = re.sub(r"//[^\n]*", "", text)
    types = [(m.start(), m.group(1)) for m in TYPE_RE.finditer(text)]
    doors = {}
    for m in FUNC_RE.finditer(text):
        owner = next((name for pos, name in reversed(types) if pos < m.start()), None)
        if owner is None:
            continue
        i, depth = m.end(), 1
        while depth and i < len(text):
            depth += text[i] == "("
            depth -= text[i] == ")"
            i += 1
        labels = []
        for part in _split_top(re.sub(r"\s+", " ", text[m.end():i - 1])):
            head = part.split(":")[0].split()
            if head:
                labels.append(head[0])
        doors.setdefault(f"{owner}.{m.group(1)}", []).append(labels)
    return doors


def main():
    ref = Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
    doors = {}
    for f in sorted((ref / "Sources" / "Operators" / "QWGEMM").glob("*.swift")):
        for name, overloads in swift_doors(f.read_text(errors="replace")).items():
            if name.split(".")[0] in ("QWGemm", "QWGemmAQ", "QWMoEOperator"):
                doors.setdefault(name, []).extend(overloads)
    out = Path(__file__).with_name("swift_door_labels.json")
    out.write_text(json.dumps(doors, indent=1, sort_keys=True) + "\n")
    print(f"{len(doors)} doors -> {out}")


if __name__ == "__main__":
    main()
