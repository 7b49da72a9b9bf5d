"""Writes tests/golden/ref_wrapper_symbols.txt: every C symbol the reference's ctypes front-end
(python/deepracin/__init__.py.in) looks up in libdeepracin.so, one name per line, from its
uncommented `lib.dR_*` attribute accesses.  Run in the build container, where /root/reference
exists; the wrapper is read as text, never imported.  The output is a list of names (data), the
wrapper's text itself is not kept.
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
