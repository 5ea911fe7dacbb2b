"""CPU-side checks of the C-ABI library: it loads, exports every declared symbol, and
refuses work cleanly when there is no device (no kernel is launched here)."""
import ctypes as C
import os

import pytest

from bunker_amd import runtime as rt


def _lib_or_skip():
    if not os.path.exists(rt.LIB_PATH):
        pytest.fail(f"{rt.LIB_PATH} not built: run `make -C bunker_amd/csrc`")
    return rt.load_library(rt.LIB_PATH)


def test_header_symbols_are_exported():
    lib = _lib_or_skip()
    names = rt.declared_symbols()
    assert len(names) >= 37 and len(set(names)) == len(names)
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing
    # the Python binding table covers the header exactly
    assert set(rt._SIGS) | {"bk_last_error"} == set(names)


_CTYPE = {
    "int": rt.i32, "int64_t": rt.i64, "uint64_t": rt.u64,
    "const char*": C.c_char_p, "char*": C.c_char_p, "const void*": rt.vp, "void*": rt.vp,
    "uint64_t*": C.POINTER(rt.u64), "const uint64_t*": C.POINTER(rt.u64), "int*": C.POINTER(rt.i32),
    "float*": C.POINTER(C.c_float),
}


def _header_prototypes():
    """name -> list of C parameter types, parsed from the BK_API lines of include/bunker_hip.h."""
    import re

    text = open(rt.HEADER_PATH).read()
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    protos = {}
    for ret, name, args in re.findall(r"BK_API\s+([\w\s\*]+?)\b(bk_\w+)\s*\(([^)]*)\)\s*;", text):
        params = []
        args = " ".join(args.split())
        if args and args != "void":
            for a in args.split(","):
                toks = a.strip().replace("*", " * ").split()
                # the last identifier is the parameter name; pointer stars belong to the type
                if toks[-1] != "*":
                    toks = toks[:-1]
                params.append(" ".join(toks).replace(" *", "*"))
        protos[name] = (" ".join(ret.split()), params)
    return protos


def test_binding_signatures_match_the_header():
    """Argument count and type of every ctypes signature against the C declaration (ctypes itself checks nothing)."""
    protos = _header_prototypes()
    assert set(protos) == set(rt.declared_symbols())
    for name, sig in rt._SIGS.items():
        ret, params = protos[name]
        assert ret == "int", (name, ret)
        assert len(params) == len(sig), f"{name}: header has {len(params)} parameters {params}, binding {len(sig)}"
        for i, (ct, py) in enumerate(zip(params, sig)):
            assert ct in _CTYPE, f"{name}: parameter {i} has a type this check does not know: {ct!r}"
            assert _CTYPE[ct] is py or _CTYPE[ct] == py, f"{name}: parameter {i} is {ct!r} in the header, {py} in the binding"
    assert protos["bk_last_error"] == ("const char*", [])


def test_calls_before_init_fail_with_message():
    lib = _lib_or_skip()
    out = C.c_uint64(0)
    rc = lib.bk_alloc(1024, C.byref(out))
    if rc == 0:          # a GPU box where another test already initialised the library
        lib.bk_free(out)
        pytest.skip("library already initialised")
    assert rc < 0
    assert b"bk_init" in lib.bk_last_error()
    assert lib.bk_gemv_q4k_q8_1(0, 0, 0, 16, 256, 1, 0, 0) < 0
    assert lib.bk_kernel_create(b"gemm N=16 K=256") < 0


def test_init_without_gpu_reports_no_device():
    import subprocess, sys
    # run in a child: bk_init touches the HIP runtime
    code = (
        "import sys; sys.path.insert(0, %r)\n"
        "from bunker_amd import runtime as rt\n"
        "lib = rt.load_library()\n"
        "rc = lib.bk_init(0)\n"
        "print(rc, lib.bk_last_error().decode())\n" % os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    rc, _, msg = r.stdout.strip().partition(" ")
    if int(rc) == 0:
        pytest.skip("a GPU is present")
    assert int(rc) < 0 and ("no HIP device" in msg or "gfx950" in msg), r.stdout


def test_missing_library_raises():
    with pytest.raises(rt.BunkerError, match="no CPU fallback"):
        rt.load_library("/nonexistent/libbunker_hip.so")


ABI_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "abi")


def test_c_driver_compiles_against_the_header():
    """tests/abi/abi_driver.c is plain C99 over include/bunker_hip.h (-Wall -Wextra -Werror -pedantic): the compiler
    checks every call against the declarations; without a device the program reports bk_init's error and exits 2."""
    import subprocess
    _lib_or_skip()
    subprocess.check_call(["make", "-C", ABI_DIR, "-B", "abi_driver"], stdout=subprocess.DEVNULL)
    exe = os.path.join(ABI_DIR, "abi_driver")
    blob = os.path.join(ABI_DIR, "_empty.bin")
    try:
        import numpy as np
        np.concatenate([np.array([1, 256], np.int32).view(np.uint8), np.zeros(144 + 256 * 4, np.uint8)]).tofile(blob)
        r = subprocess.run([exe, blob], capture_output=True, text=True, timeout=120)
    finally:
        if os.path.exists(blob):
            os.remove(blob)
    if r.returncode == 0:
        assert r.stdout.strip().endswith("ok")            # a GPU is present
    else:
        assert r.returncode == 2 and r.stdout.startswith("ERROR: bk_init(0)"), (r.returncode, r.stdout, r.stderr)


def test_bun_binding_file_matches_the_header():
    """ts/hip.ts (the bun:ffi binding a maintainer drops next to src/ttir.ts) lists every function of the header with
    the FFI type of every parameter; bun cannot run here, so the table is checked as text."""
    import re
    ffi = {"int": "i32", "int64_t": "i64", "uint64_t": "u64"}
    text = open(os.path.join(os.path.dirname(rt.HEADER_PATH), "..", "ts", "hip.ts")).read()
    table = dict((n, (re.findall(r'"(\w+)"', a), r)) for n, a, r in
                 re.findall(r'^\s*(bk_\w+):\s*\{ args: \[([^\]]*)\], returns: "(\w+)" \},', text, flags=re.M))
    protos = _header_prototypes()
    assert set(table) == set(protos)
    for name, (ret, params) in protos.items():
        args, r = table[name]
        assert r == ("i32" if ret == "int" else "ptr"), name
        assert args == [ffi.get(p, "ptr") for p in params], (name, args, params)
    # the names the call sites import from src/ttir.ts are all exported
    for fn in ("cu", "cuAlloc", "cuHtoD", "cuDtoH", "cuFree", "cuSync", "cuHtoDAsync", "cuDtoHAsync", "cuCopySync",
               "compileAndLoad", "cuLaunch", "profGpuReset", "profGpuReport"):
        assert re.search(r"^export function %s\(" % fn, text, flags=re.M), fn
    assert "export interface LoadedKernel" in text
