"""The C-ABI library: loads, exports exactly what include/waffe2_hip.h declares,
and fails cleanly (error codes, no crash, no fallback) on a machine without a
GPU.  No compute call is made here."""
import ctypes as C
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "waffe2_hip.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(wf2hip_[a-z0-9_]+)\s*\(", text)))


def test_header_compiles_as_c():
    subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Werror", "-fsyntax-only", "-x", "c", HEADER])


def test_every_declared_symbol_is_exported(W):
    lib = W.lib.load()
    names = declared_functions()
    assert len(names) >= 40
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing
    out = subprocess.check_output(["nm", "-D", "--defined-only", W.lib.LIB_PATH], text=True)
    exported = sorted(set(re.findall(r"\b(wf2hip_[a-z0-9_]+)\b", out)))
    assert exported == names, set(exported) ^ set(names)
    # nothing else leaks out of the library
    others = [l.split()[-1] for l in out.splitlines() if " T " in l and "wf2hip_" not in l]
    assert others == [], others


def test_bindings_cover_the_header(W):
    assert sorted(W.lib.EXPORTS) == declared_functions()
    assert W.lib.load().wf2hip_abi_version() == 1
    assert C.sizeof(W.lib.View2) == 8 + 3 * 8 * 8 + 16


def test_library_is_gfx950_only(W):
    """The fat binary carries code objects for gfx950 and nothing else."""
    data = open(W.lib.LIB_PATH, "rb").read()
    targets = set(re.findall(rb"amdgcn-amd-amdhsa--(gfx[0-9a-f]+)", data))
    assert targets == {b"gfx950"}, targets


@pytest.mark.skipif(os.path.exists("/dev/kfd"), reason="a GPU is present")
def test_no_gpu_means_errors_not_fallbacks(W):
    lib = W.lib.load()
    assert lib.wf2hip_init(0) != 0
    assert lib.wf2hip_last_error()
    # every compute entry refuses to run before a successful init
    assert lib.wf2hip_sadd(4, None, 1, None, 1) == -2
    assert lib.wf2hip_sgemm(b"N", b"N", 1, 1, 1, 1.0, None, 1, None, 1, 0.0, None, 1) == -2
    assert lib.wf2hip_dgemm(b"N", b"N", 1, 1, 1, 1.0, None, 1, None, 1, 0.0, None, 1) == -2
    p = C.c_void_p()
    assert lib.wf2hip_malloc(C.byref(p), 16) == -2 and not p.value
    with pytest.raises(W.HIPError):
        W.lib.init(0)


def test_missing_library_is_loud(W, monkeypatch):
    monkeypatch.setattr(W.lib, "_lib", None)
    monkeypatch.setattr(W.lib, "LIB_PATH", "/nonexistent/libwaffe2-hip.so")
    with pytest.raises(W.HIPExtensionMissing):
        W.lib.load()


def test_product_never_touches_the_oracle():
    """The oracle is a checker: nothing under the package may import, link or
    mention it."""
    pkg = os.path.join(ROOT, "cl-waffe2_amd")
    for dirpath, _, files in os.walk(pkg):
        if "build" in dirpath:
            continue
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".lisp", ".asd", "Makefile")):
                text = open(os.path.join(dirpath, f), errors="ignore").read()
                assert "oracle" not in text.lower(), os.path.join(dirpath, f)
