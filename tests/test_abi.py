"""CPU checks of the drop-in boundary: the library loads, exports every symbol the header declares, the
generated files are in sync with the operator tables, and the host-side shape logic agrees with the oracle."""
import ctypes
import importlib.util
import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "knet.jl_amd", "lib", "libknet8.so")


def _load(name, rel):
    spec = importlib.util.spec_from_file_location(name, os.path.join(ROOT, rel))
    m = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(m)
    return m


@pytest.fixture(scope="module")
def built_lib():
    if not os.path.exists(LIB):
        import __graft_entry__ as ge
        ge.build()
    return LIB


def test_library_exports_every_declared_symbol(built_lib):
    lk = _load("lk_for_test", "knet.jl_amd/libknet8.py")
    decls = lk.parse_header()
    assert len(decls) > 400
    lib = ctypes.CDLL(built_lib)
    missing = [n for n in decls if not hasattr(lib, n)]
    assert not missing, missing
    # every kernel entry point has both forms, as the reference's generated sources do
    for n in decls:
        if n.endswith("_stream"):
            assert n[: -len("_stream")] in decls, n
    for needed in ["reluback_32_11_stream", "sigmback_64_11_stream", "sum_32_21_stream", "sum_64_20_stream", "sum_32_22_stream",
                   "logsoftmaxback_32_stream", "softmaxback_64_stream", "nll_logsoftmax_back_32_stream", "dropback_32_stream",
                   "getents_32_stream", "addents_64_stream", "eluback_32_111_stream", "reluback_32_1_stream", "gemm_32_stream",
                   "knet8_malloc", "knet8_free", "knet8_memcpy"]:
        assert needed in decls, needed


def test_every_symbol_of_the_reference_library_is_exported(built_lib):
    """tests/golden/libknet8_symbols.txt lists what the reference's generator scripts export (op tables of
    src/libknet8/ops.jl x the patterns of the scripts src/libknet8/build.jl:43-55 builds): a drop-in libknet8.so has them all."""
    names = open(os.path.join(ROOT, "tests", "golden", "libknet8_symbols.txt")).read().split()
    assert len(names) > 1200
    lk = _load("lk_for_test2", "knet.jl_amd/libknet8.py")
    decls = lk.parse_header()
    lib = ctypes.CDLL(built_lib)
    assert not [n for n in names if n not in decls]
    assert not [n for n in names if not hasattr(lib, n)]


def test_every_signature_matches_the_reference_generators():
    """tests/golden/libknet8_signatures.txt holds, for each of the reference's entry points, the return type and parameter types its generator
    script prints (src/libknet8/cuda01.jl:20-25, cuda1.jl:28-33,63-68,95-100,127-132,157-162,188-200,371-442,482-493,519-524, cuda11.jl:22-27,
    cuda111.jl:23-28, cuda12.jl:28-33, cuda13.jl:99-111,172-184, cuda16.jl:60-83, cuda17.jl:58-63, cuda20.jl:83-104, cuda21.jl:70-76,
    cuda22.jl:61-66, relu.jl:27-38; read as text by tests/golden/make_libknet8_symbols.py).  The header must declare each with the same types in
    the same order, `cudaStream_t` read as `hipStream_t`: a swapped, missing or extra parameter anywhere in the boundary fails here."""
    lk = _load("lk_for_sig", "knet.jl_amd/libknet8.py")
    decls = lk.parse_header()
    names = open(os.path.join(ROOT, "tests", "golden", "libknet8_symbols.txt")).read().split()
    rows = [l.rstrip("\n").split("\t") for l in open(os.path.join(ROOT, "tests", "golden", "libknet8_signatures.txt"))]
    assert [r[0] for r in rows] == names          # one signature per exported symbol
    bad = []
    for name, ret, params in rows:
        want = [p.replace("cudaStream_t", "hipStream_t") for p in params.split(",")] if params else []
        have_ret, have = decls[name]
        if have_ret != ret or have != want:
            bad.append((name, ret, want, have_ret, have))
    assert not bad, bad[:5]
    # the fixture itself distinguishes the shapes an order slip would confuse
    sig = {r[0]: r[2].split(",") for r in rows}
    assert sig["sum_32_22"] == ["int", "int", "float*", "int", "int", "int", "float*"]
    assert sig["setcol1_64_stream"] == ["int", "int", "int", "int*", "double*", "double", "cudaStream_t"]
    assert sig["add_32_16_5"] == ["float*"] * 3 + ["int"] * 16
    assert sig["xcopy_stream"] == ["int", "int", "const void*", "int", "void*", "int", "cudaStream_t"]


def _split_top(text):
    """Split at top-level commas (parentheses, braces and brackets nest; string literals are skipped)."""
    parts, depth, cur, q = [], 0, "", False
    for ch in text:
        if ch == '"':
            q = not q
        if not q:
            if ch in "([{":
                depth += 1
            elif ch in ")]}":
                depth -= 1
            elif ch == "," and depth == 0:
                parts.append(cur.strip())
                cur = ""
                continue
        cur += ch
    if cur.strip():
        parts.append(cur.strip())
    return parts


def test_julia_binding_calls_match_the_header():
    """Every `@knet8(name, (argtypes...), args...)` and `ccall((:name, libknet8), ...)` in knet.jl_amd/julia/*.jl names a symbol
    include/knet8.h declares, with as many argument types as the C declaration has parameters (the files are not executed here)."""
    import glob
    import re
    lk = _load("lk_for_test3", "knet.jl_amd/libknet8.py")
    decls = lk.parse_header()
    acts = ("relu", "sigm", "tanh", "elu", "selu")

    def expand(tmpl):
        names = [tmpl]
        for pat, vals in ((r"\$\(?S\)?", ("32", "64")), (r"\$\(f\)", acts)):
            names = [re.sub(pat, v, n, count=0) for n in names for v in vals] if re.search(pat, names[0]) else names
        return names
    checked = 0
    for path in sorted(glob.glob(os.path.join(ROOT, "knet.jl_amd", "julia", "*.jl"))):
        text = "\n".join(l for l in open(path).read().splitlines() if not l.lstrip().startswith("#"))
        # variables holding symbol templates:  fwd, bwd = "bias$(f)_$S", "$(f)back_biasgrad_$S"   /   g = "gemm_$(S)_stream"
        names = {}
        for m in re.finditer(r"^\s*([\w, ]+?)\s*=\s*(\"[^\n]*\")\s*$", text, flags=re.M):
            vs, ss = [v.strip() for v in m.group(1).split(",")], re.findall(r'"([^"]*)"', m.group(2))
            if len(vs) == len(ss):
                names.update(zip(vs, ss))
        for m in re.finditer(r"\(:(\w+),\s*(?:LibKnet8\.)?libknet8\)", text):
            assert m.group(1) in decls, (os.path.basename(path), m.group(1))
            checked += 1
        for m in re.finditer(r"@knet8r?\(", text):
            depth, i = 1, m.end()
            while depth:
                depth += {"(": 1, ")": -1}.get(text[i], 0)
                i += 1
            args = _split_top(text[m.end():i - 1])
            sym = args[0]
            is_r = text[m.start():m.end()].startswith("@knet8r")
            types = args[2 if is_r else 1]
            if sym.startswith('$("'):
                tmpl = re.match(r'\$\("([^"]*)"\)', sym).group(1)
            elif sym.startswith("$"):
                tmpl = names[sym[1:]]
            else:
                tmpl = sym
            ntypes = len(_split_top(types.strip()[1:-1]))
            for name in expand(tmpl):
                assert name in decls, (os.path.basename(path), name)
                assert len(decls[name][1]) == ntypes, (os.path.basename(path), name, decls[name][1], types)
                checked += 1
        # ccall(($("name_$(S)_stream"), LibKnet8.libknet8), Ret, (types...), args...): the stream is part of the declared signature
        for m in re.finditer(r'ccall\(\(\$\("([^"]*)"\),\s*(?:LibKnet8\.)?libknet8\),', text):
            depth, i = 1, m.start() + len("ccall(")
            while depth:
                depth += {"(": 1, ")": -1}.get(text[i], 0)
                i += 1
            args = _split_top(text[m.start() + len("ccall("):i - 1])
            ntypes = len(_split_top(args[2].strip()[1:-1]))
            for name in expand(m.group(1)):
                assert name in decls, (os.path.basename(path), name)
                assert len(decls[name][1]) == ntypes, (os.path.basename(path), name, decls[name][1], args[2])
                checked += 1
    assert checked >= 46


def test_no_undefined_device_runtime_surprises(built_lib):
    # the product must not link the oracle or anything outside HIP / hipBLASLt / the C++ runtime
    out = subprocess.check_output(["readelf", "-d", built_lib], text=True)
    needed = [l.split("[")[1].rstrip("]") for l in out.splitlines() if "NEEDED" in l]
    assert not any("oracle" in n for n in needed)
    assert any("amdhip64" in n for n in needed)


def test_the_library_loads_beside_the_hipblaslt_that_pytorch_bundles(built_lib):
    """A Python process that imported PyTorch first has libhipblaslt.so.1 resolved to PyTorch's bundled copy, an older build than the one under
    /opt/rocm.  libknet8.so must still load there: every hipblaslt symbol it imports has to exist in both copies (the C++ extension interface is
    then switched off at run time, because its class layout belongs to one build; that check is in the library)."""
    import glob
    import importlib.util
    spec = importlib.util.find_spec("torch")
    if spec is None or not spec.submodule_search_locations:
        pytest.skip("PyTorch is not installed here")
    bundled = glob.glob(os.path.join(list(spec.submodule_search_locations)[0], "lib", "libhipblaslt.so*"))
    if not bundled:
        pytest.skip("this PyTorch bundles no libhipblaslt")

    def syms(path, flag):
        out = subprocess.check_output(["nm", "-D", flag, path], text=True)
        return {l.split()[-1] for l in out.splitlines() if l.strip()}
    wanted = {s for s in syms(built_lib, "--undefined-only") if "hipblaslt" in s.lower()}
    assert len(wanted) >= 10
    have = syms(bundled[0], "--defined-only")
    assert not sorted(wanted - have), sorted(wanted - have)


def test_generated_files_match_the_operator_tables():
    gen = _load("gen_knet8_for_test", "knet.jl_amd/csrc/gen_knet8.py")
    for path, text in gen.generate(write=False).items():
        assert os.path.exists(path), path
        assert open(path).read() == text, "stale generated file: %s (run gen_knet8.py)" % path


def test_findindices_matches_oracle(knet, oracle):
    rng = np.random.default_rng(0)
    for (c, n) in [(3, 4), (10, 100), (1, 5), (7, 1)]:
        labels = rng.integers(0, c + 1, size=n)
        assert np.array_equal(knet.findindices(np.zeros((c, n)), labels, dims=1), oracle.findindices((c, n), labels, dims=1))
        assert np.array_equal(knet.findindices(np.zeros((n, c)), labels, dims=2), oracle.findindices((n, c), labels, dims=2))
    with pytest.raises(ValueError):
        knet.findindices(np.zeros((3, 4)), [1, 2, 3], dims=1)
    with pytest.raises(ValueError):
        knet.findindices(np.zeros((3, 4)), [1, 2, 3, 1], dims=3)


def test_package_fails_loudly_without_the_library(tmp_path):
    lk = _load("lk_for_test2", "knet.jl_amd/libknet8.py")
    with pytest.raises(OSError):
        lk.LibKnet8(str(tmp_path / "libknet8.so"))


def test_header_is_plain_c_and_links(built_lib, tmp_path):
    """include/knet8.h must be usable from C (the boundary is a C ABI): compile and link a C translation unit against the library."""
    src = tmp_path / "use_knet8.c"
    src.write_text('#include "knet8.h"\n'
                   'int main(void) {\n'
                   '  void (*f)(int, float*, float*, float*, hipStream_t) = reluback_32_11_stream;\n'
                   '  float (*g)(int, float*, hipStream_t) = sum_32_20_stream;\n'
                   '  return (f != 0 && g != 0 && knet8_version() > 0) ? 0 : 1;\n'
                   '}\n')
    exe = tmp_path / "use_knet8"
    libdir = os.path.dirname(built_lib)
    subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe),
                           "-L", libdir, "-lknet8", "-Wl,-rpath," + libdir, "-Wl,-rpath,/opt/rocm/lib", "-L/opt/rocm/lib"])
    assert subprocess.call([str(exe)]) == 0


def test_the_binary_carries_the_hash_of_the_sources_it_was_built_from(built_lib, monkeypatch):
    """knet8_build_id() is the hash build.py computes over csrc/*.h, *.hip, gen_knet8.py and build.py: a library left over from other
    sources cannot pass for the current ones, and the loader refuses it."""
    build = _load("knet8_build_for_test", "knet.jl_amd/csrc/build.py")
    lib = ctypes.CDLL(built_lib)
    lib.knet8_build_id.restype = ctypes.c_char_p
    have = lib.knet8_build_id().decode()
    assert have == build.source_id(), "knet.jl_amd/lib/libknet8.so is stale: rebuild it (python __graft_entry__.py build)"
    lk = _load("lk_for_build_id", "knet.jl_amd/libknet8.py")
    assert lk.source_build_id() == have
    assert lk.LibKnet8(built_lib).build_id == have                 # loads: ids agree
    monkeypatch.setattr(lk, "source_build_id", lambda: "0" * 16)
    monkeypatch.delenv("KNET8_ALLOW_STALE", raising=False)
    with pytest.raises(OSError, match="built from other sources"):
        lk.LibKnet8(built_lib)
    monkeypatch.setenv("KNET8_ALLOW_STALE", "1")
    assert lk.LibKnet8(built_lib).build_id == have                 # the override for development
