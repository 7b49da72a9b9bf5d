"""Writes tests/golden/ref_wrapper_symbols.txt: every C symbol the reference's ctypes front-end
(python/deepracin/__init__.py.in) looks up in libdeepracin.so, one name per line, from its
uncommented `lib.dR_*` attribute accesses; and tests/golden/ref_wrapper_signatures.txt: for every
symbol the wrapper declares (`func = lib.NAME`, `func.argtypes = [...]`, `func.restype = ...`), one
line `NAME | restype | argtype, argtype, ...` with the ctypes type names it uses ("-" where it
declares none).  Run in the build container, where /root/reference exists; the wrapper is read as
text, never imported.  The outputs are lists of names (data), the wrapper's text itself is not kept.
"""
import os
import re
import sys

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
HERE = os.path.dirname(os.path.abspath(__file__))
names = []
with open(os.path.join(REF, "python", "deepracin", "__init__.py.in")) as f:
    for line in f:
        code = line.split("#", 1)[0]
        for m in re.finditer(r"\blib\.(dR_\w+)", code):
            if m.group(1) not in names:
                names.append(m.group(1))
with open(os.path.join(HERE, "ref_wrapper_symbols.txt"), "w") as f:
    f.write("\n".join(names) + "\n")
print("%d symbols written" % len(names))

# declared signatures
sigs, cur = {}, None
with open(os.path.join(REF, "python", "deepracin", "__init__.py.in")) as f:
    for line in f:
        code = line.split("#", 1)[0].strip()
        m = re.match(r"func\s*=\s*lib\.(dR_\w+)$", code)
        if m:
            cur = m.group(1)
            sigs[cur] = {"restype": "-", "argtypes": "-"}
            continue
        m = re.match(r"func\.argtypes\s*=\s*\[(.*)\]$", code)
        if m and cur:
            sigs[cur]["argtypes"] = ", ".join(t.strip() for t in m.group(1).split(",") if t.strip())
            continue
        m = re.match(r"func\.restype\s*=\s*(\w+)$", code)
        if m and cur:
            sigs[cur]["restype"] = m.group(1)
with open(os.path.join(HERE, "ref_wrapper_signatures.txt"), "w") as f:
    for name, s in sigs.items():
        f.write("%s | %s | %s\n" % (name, s["restype"], s["argtypes"]))
print("%d signatures written" % len(sigs))
