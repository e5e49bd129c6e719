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


def test_bench_library_is_separate(hk):
    """The streaming yardstick lives in a library of its own: libhk_bench.so exports what include/hk_bench.h
    declares, the operator library exports none of it, and bad arguments come back as codes before anything is
    computed from them (no GPU needed)."""
    import importlib
    capi = importlib.import_module("hotspa-ae_amd.capi")
    text = open(os.path.join(helpers.ROOT, "include", "hk_bench.h")).read()
    names = sorted(set(re.findall(r"HK_API\s+[\w\s\*]+?\b(hk_\w+)\s*\(", text)))
    assert names == ["hk_bench_last_error", "hk_bench_ring_probe", "hk_bench_stream_probe"]
    bench = capi.bench_lib()
    for n in names:
        assert hasattr(bench, n) and not hasattr(hk.lib(), n)
    assert not hasattr(hk.lib(), "hk_stream_probe")
    buf = ctypes.create_string_buffer(64)
    addr = ctypes.c_void_p((ctypes.addressof(buf) + 15) // 16 * 16)
    for threads, vectors in ((0, 1), (-64, 1), (96, 1), (256, 0), (256, 3)):
        rc = bench.hk_bench_stream_probe(addr, None, addr, None, 1, 1, ctypes.c_size_t(32), threads, vectors, 1, 1, 0, None)
        assert rc == -2, (threads, vectors, rc)
        assert b"threads" in bench.hk_bench_last_error() or b"vectors" in bench.hk_bench_last_error()


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


def test_planners_survive_odd_shapes(hk):
    """Host-side launch planning (no kernel is launched): every axis subset of small,
    odd and degenerate shapes, with dense and permuted strides."""
    import itertools
    import numpy as np
    g = np.random.default_rng(0)
    for shape in ([3, 4, 5, 6], [1, 7], [6], [2, 1, 3], [0, 5], [5, 0], [33, 264], [1000, 5], [4, 33, 7],
                  [2, 2, 1 << 20], [70000], [1, 1, 1]):
        dense = [int(np.prod(shape[i + 1:], dtype=np.int64)) for i in range(len(shape))]
        for strides in (dense, list(reversed(dense)), [s * 2 for s in dense]):
            for k in range(0, len(shape) + 1):
                for axes in itertools.combinations(range(len(shape)), k):
                    for dt in (6, 8, 4):
                        assert hk.reduce_workspace_bytes(dt, shape, strides, list(axes)) >= 0
    for dt in (5, 6, 8):
        for _ in range(200):
            rows, cols = int(g.integers(0, 70000)), int(g.integers(0, 70000))
            assert hk.norm_bwd_workspace_bytes(dt, rows, cols) >= 0
