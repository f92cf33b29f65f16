#!/usr/bin/env python3
"""Write tests/golden/libknet8_symbols.txt: every symbol the reference's libknet8 exports.

The reference's library is generated: src/libknet8/build.jl:43-55 lists the generator scripts, each of which loops over an op
table of src/libknet8/ops.jl and prints `NAME` and `NAME_stream` definitions from a fixed pattern.  This script READS those
files as text (nothing of the reference is executed), takes the op names from the tables and applies the patterns, which are
restated here with the line that prints them.  The output is a list of names, one per line; tests/test_abi.py checks that
include/knet8.h declares and libknet8.so exports each of them.

Run in the build container only (the reference tree is not available where the GPU tests run):
    python tests/golden/make_libknet8_symbols.py /root/reference
"""
import os
import re
import sys


def tables(ops_jl):
    """{table name: [op name, ...]} from `name = [ ... ]` blocks; an entry is "f" or ("f", ...)."""
    out, cur = {}, None
    for line in open(ops_jl):
        line = line.split("#")[0].strip()
        m = re.match(r"^(\w+)\s*=\s*\[", line)
        if m:
            cur = out.setdefault(m.group(1), [])
            continue
        if cur is None:
            continue
        if line.startswith("]"):
            cur = None
            continue
        m = re.match(r'^\(?\s*"([^"]+)"', line)
        if m:
            cur.append(m.group(1))
    return out


def main(ref):
    lib = os.path.join(ref, "src", "libknet8")
    t = tables(os.path.join(lib, "ops.jl"))
    built = re.findall(r'\("(\w+)"', open(os.path.join(lib, "build.jl")).read().split("SRC = [")[1].split("]")[0])
    names = []
    for S in ("32", "64"):
        if "cuda1" in built:
            names += ["%s_%s" % (f, S) for f in t["unary_ops"]]                       # cuda1.jl:28-33
            names += ["%s_%s" % (f, S) for f in t["unary_ops_with_int_degree"]]       # cuda1.jl:63-68
            names += ["fill_" + S, "xfill_" + S, "icat_" + S, "concat_" + S, "dropout_" + S, "dropback_" + S]  # cuda1.jl:95-100,127-132,195-212,485-494,519-528
            names += ["%s_%s" % (f, S) for f in ("getcols", "setcols", "addcols", "setcol1", "getrows", "setrows", "addrows", "setrow1",
                                                 "getents", "setents", "addents", "setent1")]                  # cuda1.jl:371-443
        forms = [("cuda01", ["01"]), ("cuda11", ["11"]), ("cuda12", ["12"]), ("cuda13", ["13_x_y", "13_y_x"]),
                 ("cuda14", ["14_x_y", "14_y_x"]), ("cuda16", ["16_3", "16_4", "16_5"]), ("cuda17", ["17"])]
        for script, sufs in forms:                                                    # cudaNN.jl: `for a in binary_ops`
            if script in built:
                names += ["%s_%s_%s" % (f, S, suf) for f in t["binary_ops"] for suf in sufs]
        if "cuda111" in built:
            names += ["%s_%s_111" % (f, S) for f in t["actback_ops"]]                 # cuda111.jl:23-28
        for script, suf in (("cuda20", "20"), ("cuda21", "21"), ("cuda22", "22")):
            if script in built:
                names += ["%s_%s_%s" % (f, S, suf) for f in t["reduction_ops"]]       # cuda20.jl:83-98, cuda21.jl:70-76, cuda22.jl:61-66
        if "relu" in built:
            names += ["relu_%s_1" % S, "reluback_%s_1" % S]                           # relu.jl:27-37
    if "cuda1" in built:
        names.append("xcopy")                                                         # cuda1.jl:157-165
    full = []
    for n in names:
        full += [n, n + "_stream"]
    here = os.path.dirname(os.path.abspath(__file__))
    with open(os.path.join(here, "libknet8_symbols.txt"), "w") as f:
        f.write("\n".join(full) + "\n")
    print("%d symbols from %d generator scripts" % (len(full), len(built)))


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
