"""The C-ABI library loads on a machine without a GPU and exports every symbol that
include/litekv.h declares, with a ctypes prototype for each (no compute is called here)."""

import ctypes
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
HEADER = ROOT / "include" / "litekv.h"
PROFILE_HEADER = ROOT / "include" / "litekv_profile.h"     # measurement aid, outside the product ABI


def _declared_in(path):
    text = re.sub(r"/\*.*?\*/", "", path.read_text(), flags=re.S)
    return set(re.findall(r"\b(litekv_[a-z0-9_]+)\s*\(", text))


def declared_symbols():
    return sorted(_declared_in(HEADER) | _declared_in(PROFILE_HEADER))


def test_product_header_holds_no_stateful_entry_point():
    assert _declared_in(PROFILE_HEADER) == {"litekv_profile_next_decode"}
    assert "litekv_profile_next_decode" not in _declared_in(HEADER)


def test_header_declares_the_path():
    names = declared_symbols()
    for must in ("litekv_kv_append", "litekv_page_copy", "litekv_page_gather", "litekv_paged_decode",
                 "litekv_paged_decode_balanced", "litekv_decode_plan", "litekv_paged_prefill",
                 "litekv_varlen_prefill", "litekv_last_error"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from llama_lite_npu_amd import _lib

    if not _lib.LIB_PATH.exists():
        from llama_lite_npu_amd.build import build_library
        build_library()
    lib = ctypes.CDLL(str(_lib.LIB_PATH))
    missing = [n for n in declared_symbols() if not hasattr(lib, n)]
    assert not missing, f"declared in litekv.h but not exported: {missing}"
    unbound = [n for n in declared_symbols() if n not in _lib.SIGNATURES]
    assert not unbound, f"declared in litekv.h but without a ctypes prototype: {unbound}"
    extra = [n for n in _lib.SIGNATURES if n not in declared_symbols()]
    assert not extra, f"bound in _lib.py but not declared in litekv.h: {extra}"


def test_loader_checks_abi_version_and_reports_errors_without_a_gpu():
    from llama_lite_npu_amd import _lib

    lib = _lib.load()
    assert lib.litekv_abi_version() == _lib.ABI_VERSION
    # argument validation happens on the host, before any launch
    rc = lib.litekv_kv_append(None, None, 0, 0, None, None, 4, 8, 128, 16, None)
    assert rc == 1 and b"null pointer" in lib.litekv_last_error()
    with pytest.raises(_lib.LiteKVError, match="null pointer"):
        _lib.check(rc)
    assert lib.litekv_paged_decode_workspace_bytes(32, 64, 128, 16) == 32 * 64 * 16 * 129 * 4
    assert lib.litekv_paged_decode_workspace_bytes(32, 64, 128, 1) == 0
    assert lib.litekv_decode_plan_bytes(32, 257, 8, 256) > 0
    rc = lib.litekv_page_copy(None, None, None, 0, 65536, 10, None)
    assert rc == 0   # empty move list is a no-op
    # the entry point with built-in scratch refuses steps beyond its 32 MiB before touching a device
    rc = lib.litekv_paged_decode_static(None, 0, None, None, 1, None, None, 128, 32, 4, 128, 16, 1000, 16, 1,
                                        0.1, None)
    assert rc == 1 and b"built-in scratch holds 33554432" in lib.litekv_last_error()


def test_product_package_never_imports_the_oracle():
    pkg = ROOT / "llama_lite_npu_amd"
    for path in pkg.rglob("*.py"):
        text = path.read_text()
        assert "import oracle" not in text and "from oracle" not in text, path
