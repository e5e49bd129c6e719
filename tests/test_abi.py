"""The C-ABI library loads without a GPU and exports every symbol the header declares."""
import ctypes
import os
import re

import helpers


def _declared():
    text = open(os.path.join(helpers.ROOT, "include", "hk_rowwise.h")).read()
    return sorted(set(re.findall(r"HK_API\s+[\w\s\*]+?\b(hk_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol(hk):
    names = _declared()
    assert len(names) >= 35
    lib = hk.lib()
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_no_torch_types_in_the_boundary():
    text = open(os.path.join(helpers.ROOT, "include", "hk_rowwise.h")).read()
    assert "torch" not in text and "at::" not in text and 'extern "C"' in text


def test_argument_errors_without_a_gpu(hk):
    lib = hk.lib()
    assert lib.hk_tune_set(b"no_such_key", 1) == -1
    assert b"unknown key" in lib.hk_last_error()
    assert lib.hk_tune_set(b"norm_fwd_threads", 0) == 0
    n = ctypes.c_size_t()
    shape = (ctypes.c_int64 * 2)(4, 8)
    strides = (ctypes.c_int64 * 2)(8, 1)
    axes = (ctypes.c_int64 * 1)(5)
    assert lib.hk_reduce_workspace_bytes(6, 2, shape, strides, 1, axes, ctypes.byref(n)) == -1   # axis out of range
    assert lib.hk_event_record(None, None) == -1


def test_missing_library_fails_loudly(hk, monkeypatch, tmp_path):
    import importlib
    capi = importlib.import_module("hotspa-ae_amd.capi")
    monkeypatch.setattr(capi, "_lib", None)
    monkeypatch.setattr(capi, "_LIB", str(tmp_path / "nope.so"))
    try:
        capi.lib()
    except capi.HkError as e:
        assert "missing" in str(e)
    else:
        raise AssertionError("loading a missing library must raise")
