"""CPU checks of the C++ operator layer (libhetu_rowwise.so): the host self-test
binary, the exported C entry points, and loud failure when the library is absent."""
import importlib
import os
import re
import subprocess

import pytest

import helpers

LIBDIR = os.path.join(helpers.ROOT, "hotspa-ae_amd", "lib")


def _ops():
    helpers.load_package()
    return importlib.import_module("hotspa-ae_amd.hetu_ops")


def test_host_selftest_passes():
    exe = os.path.join(LIBDIR, "hetu_host_selftest")
    assert os.path.exists(exe), "run __graft_entry__.build() first"
    proc = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    lines = proc.stdout.splitlines()
    failed = [l for l in lines if l.startswith("[FAIL]")]
    assert proc.returncode == 0 and not failed, proc.stdout[-4000:]
    assert sum(l.startswith("[ OK ]") for l in lines) >= 20


def test_operator_library_exports_every_declared_symbol():
    text = open(os.path.join(helpers.ROOT, "include", "hetu_ops_c.h")).read()
    names = sorted(set(re.findall(r"HT_API\s+[\w\s\*]+?\b(ht_\w+)\s*\(", text)))
    assert len(names) >= 25
    lib = _ops().lib()
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_kernel_link_names_are_exported():
    """The `<Kernel>Cuda` symbols are the link contract of the operator layer."""
    out = subprocess.run(["nm", "-DC", "--defined-only", os.path.join(LIBDIR, "libhetu_rowwise.so")],
                         stdout=subprocess.PIPE, text=True, check=True).stdout
    for name in ["LayerNormCuda", "LayerNormGradientCuda", "FusedLayerNormCuda", "FusedLayerNormGradientCuda",
                 "DropoutAddLnFwdCuda", "DropoutAddLnBwdCuda", "SoftmaxCuda", "SoftmaxGradientCuda",
                 "SoftmaxCrossEntropyCuda", "SoftmaxCrossEntropyGradientCuda", "SoftmaxCrossEntropySparseCuda",
                 "SoftmaxCrossEntropySparseGradientCuda", "ReduceCuda", "ReduceSumCuda", "ReduceMeanCuda"]:
        assert re.search(r"hetu::impl::%s\(" % name, out), name


def test_errors_map_to_exception_kinds_without_a_gpu():
    import torch
    ops = _ops()
    x = torch.zeros(4, 8)
    out = torch.empty(4, 8)
    # host arrays handed to an accelerator-only kernel: the device assertion fires before any GPU call
    with pytest.raises(ops.AssertionError_, match="not on an accelerator"):
        ops.fused_layer_norm(x, torch.ones(8), torch.zeros(8), torch.empty(4), torch.empty(4), out, 1, 1e-5)
    # kernels with a host twin dispatch on the device type and run on the host
    ops.softmax(x, out, 1)
    assert torch.allclose(out, torch.full((4, 8), 0.125))
    ops.ndarray_softmax(x, 1, out)
    assert torch.allclose(out, torch.full((4, 8), 0.125))
    red = torch.empty(8)
    ops.ndarray_reduce(x + 1, "sum", [0], False, red)
    assert torch.equal(red, torch.full((8,), 4.0))
    # a kernel without a host twin reached through the NDArray static: the switch itself refuses the host
    with pytest.raises(ops.NotImplemented_):
        ops.ndarray_layernorm(x, torch.ones(8), torch.zeros(8), 1, 1e-5, True, out)


def test_missing_operator_library_fails_loudly(monkeypatch, tmp_path):
    ops = _ops()
    monkeypatch.setattr(ops, "_lib", None)
    monkeypatch.setattr(ops, "_LIB", str(tmp_path / "nope.so"))
    with pytest.raises(ops.HetuError, match="missing"):
        ops.lib()
