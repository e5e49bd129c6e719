"""MI355X-native row-wise operator kernels behind Hetu's kernel interface.

The compute lives in two native libraries built in-tree by ``build.py``:

* ``lib/libhk_rowwise.so``   — C-ABI device layer + hand-written gfx950 kernels
  (``include/hk_rowwise.h``);
* ``lib/libhetu_rowwise.so`` — C++ host layer with Hetu's own types and kernel
  entry points (``hetu::impl::LayerNormCuda`` ...).

This Python package is only the thin ctypes harness used by the tests and the
benchmark: it loads the libraries and passes raw device pointers.  There is no
CPU fallback: if the library is missing, loading fails with an error.

The directory name contains a hyphen, so import it with
``importlib.import_module("hotspa-ae_amd")``.
"""
from .capi import (  # noqa: F401
    HkError, lib, lib_path, check, DTYPES, dtype_code, torch_dtype,
    layer_norm_fwd, layer_norm_bwd, norm_bwd_workspace_bytes,
    dropout_add_ln_fwd, dropout_add_ln_bwd, dropout_add_ln_bwd_static, dropout_add_ln_fwd_ex, dropout_add_ln_bwd_ex,
    unary, binary_const, binary, broadcast, sce_sparse_bwd_reduced, sce_dense_bwd_reduced, vocab_parallel_ce_gather, vocab_parallel_ce_bwd,
    vocab_parallel_ce_stats, vocab_parallel_ce_combine, vocab_parallel_ce_bwd_fused, UNARY_OPS, BINARY_OPS,
    softmax_fwd, softmax_bwd,
    sce_sparse_fwd, sce_sparse_bwd, sce_dense_fwd, sce_dense_bwd, nll_loss_fwd, nll_loss_bwd,
    reduce, reduce_workspace_bytes, norm, norm_bwd, batch_norm_fwd, batch_norm_bwd, batch_norm_workspace_bytes, tune_set, copy_kernel, strided_copy, strided_scatter, stream_probe, ring_probe, memcpy_d2d,
    Event, current_stream,
)
