"""Writes ``reference_defined_exports.json``: the names of the functions that the reference's tensor library both
declares ``THCL_API`` in a header and defines in a ``.cpp`` file under ``src/lib`` -- the symbols a binding built
against the reference's headers can expect ``libTHCl`` to resolve.  The reference's files are read as text; nothing
is compiled or run.  Definitions inside ``/* ... */`` or ``#if 0`` blocks do not count.

    python tests/golden/make_reference_exports.py /root/reference
"""
import json
import os
import re
import sys


def strip_comments(text):
    text = re.sub(r"/\*.*?\*/", lambda m: "\n" * m.group(0).count("\n"), text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    out, depth = [], 0          # drop `#if 0 ... #endif`
    for line in text.split("\n"):
        s = line.strip()
        if depth:
            if re.match(r"#\s*if", s):
                depth += 1
            elif re.match(r"#\s*endif", s):
                depth -= 1
            continue
        if re.match(r"#\s*if\s+0\b", s):
            depth = 1
            continue
        out.append(line)
    return "\n".join(out)


def main(root):
    lib = os.path.join(root, "src", "lib")
    declared, defined = {}, {}
    for name in sorted(os.listdir(lib)):
        path = os.path.join(lib, name)
        if name.endswith(".h"):
            text = strip_comments(open(path, errors="replace").read())
            for m in re.finditer(r"THCL_API\s+[^;{]*?\b((?:THCl|TH[A-Z][a-z]+(?:Tensor|Storage)_)\w*)\s*\(", text):
                declared.setdefault(m.group(1), name)
        elif name.endswith(".cpp"):
            text = strip_comments(open(path, errors="replace").read())
            # a definition: the name, a parameter list, then an opening brace (possibly on the next line)
            for m in re.finditer(r"^[A-Za-z_][\w \t\*]*?\b((?:THCl|TH[A-Z][a-z]+(?:Tensor|Storage)_)\w*)\s*\(([^;{}]*?)\)\s*\{", text, flags=re.M | re.S):
                defined.setdefault(m.group(1), name)
    both = sorted(n for n in declared if n in defined)
    out = {"source": "src/lib/*.h (THCL_API declarations) and src/lib/*.cpp (definitions) of the reference, read as text",
           "names": both,
           "declared_in": {n: declared[n] for n in both},
           "defined_in": {n: defined[n] for n in both},
           "declared_but_not_defined": sorted(n for n in declared if n not in defined)}
    here = os.path.dirname(os.path.abspath(__file__))
    with open(os.path.join(here, "reference_defined_exports.json"), "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
        f.write("\n")
    print(len(both), "declared and defined;", len(out["declared_but_not_defined"]), "declared only")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
