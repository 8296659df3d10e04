"""The C-ABI library loads and exports exactly what include/galvatron_moe.h declares (no GPU)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "galvatron_moe.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(gmoe_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_entry_points():
    names = declared_functions()
    assert "gmoe_gmm" in names and "gmoe_route_topk" in names and len(names) >= 15


def test_library_exports_every_declared_symbol(pkg):
    handle = ctypes.CDLL(pkg._C.LIB_PATH)
    for name in declared_functions():
        assert hasattr(handle, name), "library does not export %s" % name


def test_python_prototypes_cover_header(pkg):
    assert sorted(pkg._C.PROTOTYPES) == declared_functions()


def test_prototype_arity_matches_header(pkg):
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    for name, (_, argtypes) in pkg._C.PROTOTYPES.items():
        m = re.search(r"\b%s\s*\(([^;]*?)\)\s*;" % name, text, flags=re.S)
        assert m, name
        args = m.group(1).strip()
        n = 0 if args in ("", "void") else len(args.split(","))
        assert n == len(argtypes), "%s: header has %d args, Python binds %d" % (name, n, len(argtypes))


def test_abi_version_and_status_strings(pkg):
    lib = pkg._C.lib()
    assert lib.gmoe_abi_version() == pkg._C.ABI_VERSION
    assert lib.gmoe_status_string(0) == b"ok"
    assert b"invalid" in lib.gmoe_status_string(-1)
    # pure host-side helpers, no device needed
    assert lib.gmoe_route_workspace_bytes(1024, 8) > 0
    assert lib.gmoe_permute_plan_workspace_bytes(1024, 8) >= 2 * 8 * 4 * 4


def test_argument_checks_reject_bad_calls_without_a_gpu(pkg):
    lib = pkg._C.lib()
    # k > E, null outputs: refused before anything is launched
    assert lib.gmoe_route_topk(None, 0, 4, 8, 9, 0, 0, 0.0, None, None, 0, 0, None, None, None,
                               None, None, None, None) == -1
    assert lib.gmoe_gmm(None, None, None, None, 1, 0, 8, 8, 1, 1, 1, 1, None, 0, None) == -1


def test_missing_library_fails_loudly(pkg, monkeypatch):
    monkeypatch.setattr(pkg._C, "_lib", None)
    monkeypatch.setattr(pkg._C, "LIB_PATH", "/nonexistent/libgalvatron_moe.so")
    with pytest.raises(pkg._C.LibraryMissingError):
        pkg._C.lib()


def test_cpu_tensors_are_refused(pkg):
    import torch

    with pytest.raises(AssertionError):
        pkg.topk_softmax_with_capacity(torch.randn(4, 8), 2)
    with pytest.raises(AssertionError):
        pkg.permute(torch.randn(4, 8), torch.ones(4, 2, dtype=torch.bool))


def test_dropin_package_imports_as_grouped_gemm():
    """`import grouped_gemm` with hetu-galvatron_amd/dropin on sys.path, in a fresh interpreter, as
    moe/grouped_gemm_util.py:3-6 of the reference does: the name resolves to this package's ops."""
    import subprocess
    import sys

    code = ("import sys; sys.path.insert(0, %r); import grouped_gemm; "
            "assert callable(grouped_gemm.ops.gmm) and callable(grouped_gemm.backend.gmm); "
            "import hetu_galvatron_amd; assert grouped_gemm.ops is hetu_galvatron_amd.grouped_gemm.ops; "
            "print('ok')") % os.path.join(ROOT, "hetu-galvatron_amd", "dropin")
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0 and out.stdout.strip().endswith("ok"), out.stderr
