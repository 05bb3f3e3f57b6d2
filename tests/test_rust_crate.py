"""The Rust FFI crate a maintainer adds to the reference (`xabe-hip/`, source only: no rustc in this image) against
the C headers and the library: the generated declarations are up to date, cover every function the headers declare
and nothing else, and every call the hand-written wrappers make names a declared function."""
import os
import re
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CRATE = os.path.join(ROOT, "xabe-hip")


def _header_functions():
    names = []
    for h in ("xabe_hip.h", "xabe_gguf.h", "xabe_lm_head.h"):
        text = re.sub(r"/\*.*?\*/", " ", open(os.path.join(ROOT, "include", h)).read(), flags=re.S)
        names += re.findall(r"\b(xabe_\w+)\s*\(", text)
    return sorted(set(names))


def test_generated_declarations_are_current_and_complete():
    path = os.path.join(CRATE, "src", "ffi.rs")
    before = open(path).read()
    subprocess.check_call([sys.executable, os.path.join(CRATE, "gen_ffi.py")], stdout=subprocess.DEVNULL)
    assert open(path).read() == before, "xabe-hip/src/ffi.rs is stale: run python xabe-hip/gen_ffi.py"
    declared = sorted(set(re.findall(r"pub fn (xabe_\w+)\(", before)))
    assert declared == _header_functions()


def test_declarations_match_the_library_exports():
    from llmxabe_amd import _ffi

    declared = set(re.findall(r"pub fn (xabe_\w+)\(", open(os.path.join(CRATE, "src", "ffi.rs")).read()))
    assert declared == set(_ffi.EXPORTED_SYMBOLS), declared ^ set(_ffi.EXPORTED_SYMBOLS)


def test_wrappers_call_declared_functions_with_the_declared_arity():
    ffi = open(os.path.join(CRATE, "src", "ffi.rs")).read()
    arity = {}
    for m in re.finditer(r"pub fn (xabe_\w+)\((.*?)\)(?: -> [^;]+)?;", ffi):
        args = m.group(2).strip()
        arity[m.group(1)] = 0 if not args else len(args.split(", "))
    consts = set(re.findall(r"pub const (XABE_\w+):", ffi))
    calls = 0
    for name in ("moe.rs", "block.rs", "layer_ops.rs", "dense.rs", "lm_head.rs", "weights.rs"):
        src = open(os.path.join(CRATE, "src", name)).read()
        for m in re.finditer(r"ffi::(xabe_\w+)\s*\(", src):
            fn = m.group(1)
            assert fn in arity, f"{name}: ffi::{fn} is not declared"
            # count top-level commas of the call's argument list
            i, depth, commas, empty = m.end(), 1, 0, True
            while depth:
                c = src[i]
                if c in "([{":
                    depth += 1
                elif c in ")]}":
                    depth -= 1
                elif c == "," and depth == 1:
                    commas += 1
                if depth and not c.isspace():
                    empty = False
                i += 1
            n = 0 if empty else commas + 1
            assert n == arity[fn], f"{name}: ffi::{fn} called with {n} arguments, declared with {arity[fn]}"
            calls += 1
        for c in re.findall(r"ffi::(XABE_\w+)", src):
            assert c in consts, f"{name}: ffi::{c} is not a declared constant"
    assert calls > 40
