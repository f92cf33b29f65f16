#!/usr/bin/env python3
"""Write tests/golden/libknet8_symbols.txt and tests/golden/libknet8_signatures.txt: every symbol the reference's libknet8 exports, and the C
signature the reference's generator prints for each.

The reference's library is generated: src/libknet8/build.jl:43-55 lists the generator scripts, each of which loops over an op
table of src/libknet8/ops.jl and prints `NAME` and `NAME_stream` definitions from a fixed pattern.  This script READS those
files as text (nothing of the reference is executed), takes the op names from the tables and applies the patterns, which are
restated here with the line that prints them.  The output is a list of names, one per line; tests/test_abi.py checks that
include/knet8.h declares and libknet8.so exports each of them.

The signatures come from the same files, again as text: every generator script prints its wrappers from lines of the form
`$DLLEXPORT <ret> <name template>(<parameters>) {` inside a `for (T,F) in [("float",...),("double",...)]` loop (cuda16.jl assembles the
parameter list with print loops over `dim_count`); the script finds those lines, substitutes T, F and the op names of the table the
script's driver loop walks, and writes `name<TAB>return type<TAB>parameter types` (parameter names dropped, `T *x` written `T*`).
tests/test_abi.py compares each with the declaration in include/knet8.h, reading `cudaStream_t` as `hipStream_t`.

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


def c_types(params, T):
    """Parameter list as printed by a generator template -> list of C types without the parameter names."""
    out = []
    for p in params.split(","):
        p = p.strip().replace("$T", T)
        if not p:
            continue
        m = re.match(r"^(.*?)(\w+)$", p)              # the last word is the parameter name
        ty = re.sub(r"\s+", " ", m.group(1)).strip()
        out.append(re.sub(r"\s*\*", "*", ty))
    return out


def signatures(lib, t, built):
    """{symbol: (return type, [parameter types])} from the DLLEXPORT lines of the generator scripts in `built`."""
    sigs = {}
    for script in built:
        text = open(os.path.join(lib, script + ".jl")).read()
        # which op table each generator function is driven with: `for a in TABLE ... print(fp,FUNC(a...`
        table_of = {}
        for m in re.finditer(r"^for a in (\w+)\n(?:.*\n)*?\s*print\(fp,\s*(\w+)\(a\.\.\.", text, flags=re.M):
            table_of[m.group(2)] = m.group(1)
        funcs = [(m.start(), m.group(1)) for m in re.finditer(r"^function (\w+)\(", text, flags=re.M)]
        loops = [(m.start(), m.group(1)) for m in re.finditer(r"for \(T,F[\w,]*\) in (\[.*?\])\s*$", text, flags=re.M)]

        def context(pos):
            func = [name for at, name in funcs if at < pos][-1]
            tuples = re.findall(r'\(("[^"]*"(?:\s*,\s*"[^"]*")*)\)', [l for at, l in loops if at < pos][-1])
            return func, [re.findall(r'"([^"]*)"', tp) for tp in tuples]

        def emit(pos, ret, name_tmpl, params):
            func, tuples = context(pos)
            ops = t[table_of[func]] if func in table_of else [None]
            for tp in tuples:
                T, F = tp[0], tp[1]
                Fback = tp[2] if len(tp) > 2 else None
                for f in ops:
                    Ff = F.replace("$(f)", f or "").replace("$f", f or "")
                    name = name_tmpl.replace("$(Fback)", Fback or "").replace("$(F)", Ff).replace("$F", Ff)
                    assert "$" not in name, (script, name_tmpl, name)
                    sigs[name] = (ret.replace("$T", T), c_types(params, T))
        if script == "cuda16":
            # cuda16.jl:60-83: "void $(F)_16_$(dim_count)[_stream]($T *x,$T *y,$T *z," + dim_count x "int stridex_$counter," + the same for y
            # and z + "int Nz[, cudaStream_t STR]) {"
            head = re.search(r'print\(s, "\$DLLEXPORT (\w+) \$\(F\)_16_\$\(dim_count\)_stream\(([^"]*)"\)', text)
            pieces = re.findall(r'print\(s,"(int stride\w_\$counter,)"\)', text[head.start():] if head else "")   # (the kernel above prints the same list)
            tails = re.findall(r'"""(int Nz[^)]*)\) \{', text)
            dims = re.search(r"for dim_count=(\d+):(\d+)", text)
            assert head and len(pieces) == 3 and len(tails) == 2 and dims, "cuda16.jl does not look as expected"
            for dc in range(int(dims.group(1)), int(dims.group(2)) + 1):
                middle = "".join(pc.replace("$counter", str(c)) for pc in pieces for c in range(dc))
                for tail in tails:
                    suffix = "_stream" if "STR" in tail else ""
                    emit(head.start(), head.group(1), "$(F)_16_%d%s" % (dc, suffix), head.group(2) + middle + tail)
            continue
        for m in re.finditer(r"\$DLLEXPORT\s+(\$?\w+)\s+([\w$()]+)\(([^)]*)\)\s*\{", text):
            if script == "cuda1" and m.group(2).startswith("xcopy"):   # cuda1.jl:157-165, outside any (T,F) loop
                sigs[m.group(2)] = (m.group(1), c_types(m.group(3), ""))
                continue
            emit(m.start(), m.group(1), m.group(2), m.group(3))
    return sigs


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
    sigs = signatures(lib, t, built)
    missing = [n for n in full if n not in sigs]
    extra = [n for n in sigs if n not in set(full)]
    assert not missing and not extra, (missing[:5], extra[:5])
    with open(os.path.join(here, "libknet8_signatures.txt"), "w") as f:
        for n in full:
            f.write("%s\t%s\t%s\n" % (n, sigs[n][0], ",".join(sigs[n][1])))
    print("%d signatures" % len(sigs))


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
