"""Build step: wrap device/mononn_device.h into a C++ string constant (device/prelude_text.h) so the
host compiler can hand it to hipRTC as the include "headers.h"."""
import sys

src, dst = sys.argv[1], sys.argv[2]
text = open(src).read()
delim = "MONONN_PRELUDE"
assert ")" + delim not in text
chunks = [text[i:i + 12000] for i in range(0, len(text), 12000)]   # stay under compilers' literal limits
with open(dst, "w") as f:
    f.write("// generated from device/mononn_device.h by embed_prelude.py - do not edit\n#pragma once\n")
    f.write("namespace mononn { namespace device {\nstatic const char kPreludeText[] =\n")
    for c in chunks:
        f.write('R"' + delim + "(" + c + ")" + delim + '"\n')
    f.write(";\n} }\n")
