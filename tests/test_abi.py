"""The C-ABI library loads and exports every symbol include/tenmo_hip.h declares; host-side
argument checking works without a GPU (no compute calls here)."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "tenmo_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"\b([a-z_][a-z0-9_]*)\s*\(", text)
    return sorted({n for n in names if n.startswith("tenmo_hip_") or n == "cblas_sgemm"})


def test_header_symbols_exported():
    from tenmo_amd import _lib

    lib = C.CDLL(_lib.LIB_PATH)
    names = declared_functions()
    assert len(names) >= 25
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/tenmo_hip.h but not exported"
    # and the Python binding table covers exactly the header
    assert sorted(_lib.SIGNATURES) == names


def test_load_binds_everything():
    from tenmo_amd import _lib

    assert _lib.load() is not None


def test_uninitialised_calls_fail_cleanly():
    """Before tenmo_hip_init every compute entry returns NOT_INITIALIZED with a message; nothing
    touches the GPU."""
    from tenmo_amd import _lib

    L = _lib.load()
    if L.tenmo_hip_get_stream():  # some other test initialised the library on a GPU machine
        pytest.skip("library already initialised in this process")
    assert L.tenmo_hip_sync() == -1
    assert b"not initialised" in L.tenmo_hip_last_error()
    assert L.tenmo_hip_gemm_f32(None, 0, 1, 1, None, 0, 1, 1, None, 1, 1, 1, 0, None, None, None, 0, 0) == -1
    with pytest.raises(_lib.TenmoHipError):
        _lib.check(L.tenmo_hip_dot_f32(None, 0, 1, None, 0, 1, 4, None, 0))


def test_classify_matches_reference_rule():
    """tenmo/matmul.mojo:258-272 — pure host logic, no device needed."""
    from tenmo_amd import _lib

    L = _lib.load()
    f = lambda a, b: L.tenmo_hip_classify_matmul(len(a), _lib.i64(a), len(b), _lib.i64(b))
    assert f((3,), (3,)) == _lib.OP_DOT
    assert f((), (3,)) == _lib.OP_DOT
    assert f((3,), (3, 4)) == _lib.OP_VM
    assert f((2, 3), (3,)) == _lib.OP_MV
    assert f((7, 2, 3), (3, 4)) == _lib.OP_MM
    assert f((2, 3), (4, 4)) == _lib.OP_INVALID


def test_result_shape_and_validation_messages():
    """Shape resolution and the reference's error texts (tenmo/kernels/matmul_kernel.mojo:146-162,
    tenmo/broadcasthelper.mojo:54-61) are host-side and run without a device."""
    from tenmo_amd import _lib

    L = _lib.load()
    mk = lambda shape: _lib.make_view(0, 0, shape, [1] * len(shape))
    out, rank = (C.c_int64 * 10)(), C.c_int32()
    a, b = mk((2, 1, 3, 1, 4, 5)), mk((1, 4, 1, 6, 5, 7))
    n = L.tenmo_hip_result_shape(_lib.OP_MM, C.byref(a), C.byref(b), out, C.byref(rank))
    assert n == 2 * 4 * 3 * 6 * 4 * 7 and [out[i] for i in range(rank.value)] == [2, 4, 3, 6, 4, 7]
    a, b = mk((2, 3)), mk((4, 5))
    assert L.tenmo_hip_result_shape(_lib.OP_MM, C.byref(a), C.byref(b), out, C.byref(rank)) == -2
    assert b"inner dims must match, got 3 and 4" in L.tenmo_hip_last_error()
    a, b = mk((2, 5, 3)), mk((3, 3, 4))
    assert L.tenmo_hip_result_shape(_lib.OP_MM, C.byref(a), C.byref(b), out, C.byref(rank)) == -2
    assert b"cannot broadcast shapes" in L.tenmo_hip_last_error()
    a, b = mk((3,)), mk((3, 4))
    assert L.tenmo_hip_result_shape(_lib.OP_MM, C.byref(a), C.byref(b), out, C.byref(rank)) == -2
    assert b"A must have rank >= 2" in L.tenmo_hip_last_error()
    a, b = mk((4, 2, 3)), mk((3,))
    assert L.tenmo_hip_result_shape(_lib.OP_MV, C.byref(a), C.byref(b), out, C.byref(rank)) == 8
    a, b = mk((5, 3)), mk((2, 3, 4))
    assert L.tenmo_hip_result_shape(_lib.OP_VM, C.byref(a), C.byref(b), out, C.byref(rank)) < 0  # (5,) vs (2,)
    a, b = mk((3,)), mk((2, 3, 4))
    assert L.tenmo_hip_result_shape(_lib.OP_VM, C.byref(a), C.byref(b), out, C.byref(rank)) == 8


def test_missing_library_is_loud(monkeypatch, tmp_path):
    from tenmo_amd import _lib

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(ImportError):
        _lib.load()


def test_the_product_never_touches_the_oracle():
    """The oracle is test infrastructure: nothing in the package, the header or the glue names it, the library does not link
    it, and bench.py imports it only inside the two functions that time / replay the CPU side."""
    import ast
    import subprocess

    for top in ("tenmo_amd", "include", "integration"):
        for folder, _dirs, files in os.walk(os.path.join(ROOT, top)):
            if "__pycache__" in folder:
                continue
            for name in files:
                if name.endswith((".py", ".hip", ".hpp", ".h", ".mojo")):
                    assert "oracle" not in open(os.path.join(folder, name)).read().lower(), os.path.join(folder, name)
    needed = subprocess.run(["readelf", "-d", os.path.join(ROOT, "tenmo_amd", "libtenmo_hip.so")], capture_output=True, text=True).stdout
    assert "NEEDED" in needed and "oracle" not in needed
    tree = ast.parse(open(os.path.join(ROOT, "bench.py")).read())
    importers = set()
    for fn in ast.walk(tree):
        if isinstance(fn, (ast.FunctionDef, ast.AsyncFunctionDef)):
            for node in ast.walk(fn):
                if isinstance(node, ast.ImportFrom) and (node.module or "").startswith("oracle"):
                    importers.add(fn.name)
    assert importers == {"cpu_gemm_baseline", "mlp_step_times"}, importers
    for node in tree.body:  # and never at module level
        assert not (isinstance(node, (ast.Import, ast.ImportFrom)) and "oracle" in ast.dump(node))


def test_blas_handle_load_failure_is_recorded(tmp_path):
    """tenmo/blashandle.mojo:183-191, :227-228"""
    from tenmo_amd.blashandle import BLASHandle
    import numpy as np

    h = BLASHandle(str(tmp_path / "libmissing.so"))
    assert not h.is_initialized() and "Failed to load" in h.error()
    with pytest.raises(RuntimeError):
        h.matmul(np.zeros((2, 2), np.float32), np.zeros((2, 2), np.float32))


def test_conv_padding_parse_matches_reference_shapes(golden):
    """Host-side padding parse of the Conv2dFused mirror (tenmo/cnn.mojo:183-222) against the output shapes
    asserted by tests/test_cnn.mojo; no GPU call is made."""
    from helpers import conv_case_tensors
    from tenmo_amd.cnn import parse_padding

    for case in golden["conv"]["cases"]:
        if "expect_shape" not in case and "expect" not in case:
            continue
        image, kernel, _, kw = conv_case_tensors(case)
        kh, kww = kernel.shape[2:]
        top, bottom, left, right = parse_padding(image.shape[2], image.shape[3], kh, kww, kw["stride"], kw["dilation"], kw["padding"])
        dkh, dkw = kh + (kh - 1) * (kw["dilation"] - 1), kww + (kww - 1) * (kw["dilation"] - 1)
        h_out = (image.shape[2] + top + bottom - dkh) // kw["stride"] + 1
        w_out = (image.shape[3] + left + right - dkw) // kw["stride"] + 1
        want = case.get("expect_shape") or list(__import__("numpy").array(case["expect"]).shape)
        assert [image.shape[0], kernel.shape[0], h_out, w_out] == want, case["name"]


def test_mojo_glue_matches_the_header():
    """integration/mojo/hiphandle.mojo cannot be compiled here; what can be checked is that every symbol it looks up is
    declared in include/tenmo_hip.h and that the function type it is looked up with has as many parameters as the C
    prototype (a maintainer's first build would otherwise fail, or worse, call with a shifted argument list)."""
    header = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "tenmo_hip.h")).read(), flags=re.S)
    glue = open(os.path.join(ROOT, "integration", "mojo", "hiphandle.mojo")).read()

    def top_level_commas(args):
        depth = count = 0
        for ch in args:
            depth += ch in "([" 
            depth -= ch in ")]"
            count += ch == "," and depth == 0
        return count

    def arity(args):
        args = args.strip()
        return 0 if args in ("", "void") else top_level_commas(args) + 1

    c_arity = {m.group(1): arity(m.group(2)) for m in re.finditer(r"\b(tenmo_hip_[a-z0-9_]+|cblas_sgemm)\s*\(([^;{]*?)\)\s*;", header, re.S)}
    types = {m.group(1): arity(m.group(2)) for m in re.finditer(r"comptime\s+(\w+_FN)\s*=\s*def\((.*?)\)\s*thin", glue, re.S)}
    lookups = re.findall(r"get_function\[(\w+)\]\(\"(\w+)\"\)", glue)
    assert len(lookups) >= 15 and len(types) >= 15
    for fn_type, symbol in lookups:
        assert symbol in c_arity, f"{symbol}: looked up by the Mojo glue, not declared in the header"
        assert fn_type in types, fn_type
        assert types[fn_type] == c_arity[symbol], f"{symbol}: {c_arity[symbol]} parameters in C, {types[fn_type]} in {fn_type}"
