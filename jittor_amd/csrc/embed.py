"""Build step: turns csrc/kernels/*.h into embedded_kernels.cpp so that the
run-time specialiser carries its hand-written kernel sources inside libmjt.so."""
import os
import sys

here = os.path.dirname(os.path.abspath(__file__))
out = sys.argv[1] if len(sys.argv) > 1 else os.path.join(here, "embedded_kernels.cpp")
parts = ['#include <cstring>\nnamespace mjt {\n']
names = sorted(f for f in os.listdir(os.path.join(here, "kernels")) if f.endswith(".h"))
for i, f in enumerate(names):
    text = open(os.path.join(here, "kernels", f)).read()
    assert ')MJTSRC"' not in text
    # string literals are limited in length by some compilers: split in chunks
    parts.append("static const char* k_src_%d =\n" % i)
    for j in range(0, len(text), 8000):
        parts.append('R"MJTSRC(' + text[j:j + 8000] + ')MJTSRC"\n')
    parts.append(";\n")
parts.append("const char* embedded_source(const char* name) {\n")
for i, f in enumerate(names):
    parts.append('    if (!strcmp(name, "%s")) return k_src_%d;\n' % (f, i))
parts.append("    return nullptr;\n}\n}  // namespace mjt\n")
open(out, "w").write("".join(parts))
