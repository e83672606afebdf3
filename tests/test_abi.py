"""The C-ABI library loads on a machine without a GPU and exports every symbol
that include/oslo_hip.h and include/oslo_hip_testing.h declare; argument validation that needs no device is
exercised too (no kernel is launched here)."""
import os
import re

import pytest

from oslo_amd.torch import _C

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols(header=None):
    """Symbols declared by the production header, the testing header, or both."""
    names = []
    for h in ([header] if header else ["oslo_hip.h", "oslo_hip_testing.h"]):
        text = open(os.path.join(ROOT, "include", h)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names += re.findall(r"\b(oslo_[a-z0-9_]+)\s*\(", text)
    return sorted(set(names))


def test_test_hooks_live_in_their_own_header():
    hooks = {"oslo_tune", "oslo_copy_probe", "oslo_philox_words", "oslo_wave_reduce_selftest",
             "oslo_colsum_finalize_probe"}
    assert set(declared_symbols("oslo_hip_testing.h")) == hooks
    assert not hooks & set(declared_symbols("oslo_hip.h"))


def test_header_and_loader_agree():
    assert declared_symbols() == sorted(_C.EXPORTED_SYMBOLS)


def test_library_exports_every_declared_symbol():
    lib = _C.load_library()
    for name in declared_symbols():
        assert hasattr(lib, name), name
    assert lib.oslo_hip_arch() == b"gfx950"
    assert lib.oslo_hip_abi_version() == _C.ABI_VERSION


def test_workspace_bytes_and_errors():
    lib = _C.load_library()
    assert lib.oslo_workspace_bytes(_C.OSLO_OP_LN_BWD, 0, 128) == 0
    ln = lib.oslo_workspace_bytes(_C.OSLO_OP_LN_BWD, 4096, 1024)
    rms = lib.oslo_workspace_bytes(_C.OSLO_OP_RMS_BWD, 4096, 1024)
    assert ln == 2 * rms and rms % (1024 * 4) == 0 and rms > 0
    assert lib.oslo_workspace_bytes(_C.OSLO_OP_BIAS_GELU_BWD, 100, 64) > 0
    assert lib.oslo_workspace_bytes(99, 4, 4) < 0
    assert b"unknown op" in lib.oslo_hip_last_error()


def test_invalid_arguments_are_rejected_before_any_launch():
    lib = _C.load_library()
    # unsupported dtype pair: fp16 input with bf16 output
    rc = lib.oslo_ln_fwd(None, None, None, None, None, None, 4, 8, 1e-5, 1, 2, None)
    assert rc == -2 and b"dtype pair" in lib.oslo_hip_last_error()
    rc = lib.oslo_ln_fwd(None, None, None, None, None, None, 4, 8, 1e-5, 7, 0, None)
    assert rc == -1
    rc = lib.oslo_softmax_causal_fwd(None, None, 2, 4, 0, 1.0, 0, None)
    assert rc == -1 and b"bad shape" in lib.oslo_hip_last_error()
    rc = lib.oslo_softmax_masked_fwd(None, None, None, 2, 2, 4, 8, 3, 1, 1.0, 0, None)
    assert rc == -1 and b"broadcast" in lib.oslo_hip_last_error()
    rc = lib.oslo_bias_dropout_add_fwd(None, None, None, None, None, 4, 8, 1.5, 0, 0, 0, None)
    assert rc == -1 and b"not in [0, 1]" in lib.oslo_hip_last_error()
    rc = lib.oslo_copy_probe(None, None, 24, None)
    assert rc == -1
    assert lib.oslo_tune(b"no_such_knob", 1) == -1
    assert lib.oslo_tune(b"norm_fwd_vpl", 0) == 0
    # values without a kernel build or a valid workgroup shape are refused
    for key, bad in ((b"norm_fwd_vpl", 5), (b"norm_bwd_vpl", 8), (b"norm_fwd_waves", 17),
                     (b"norm_bwd_prefetch", 3), (b"softmax_rows_per_wave", 3),
                     (b"softmax_lanes_per_row", 4), (b"norm_lanes_per_row", 1),
                     (b"softmax_fwd_elems", 4), (b"eltwise_tile_max", 100),
                     (b"eltwise_tile_min", 512), (b"eltwise_unroll", 3), (b"adam_unroll", 8),
                     (b"norm_bwd_blocks_per_cu", -1)):
        assert lib.oslo_tune(key, bad) == -1, key
    assert lib.oslo_tune(b"eltwise_tile_max", 100) == -1 and b"no valid value" in lib.oslo_hip_last_error()
    for key, good in ((b"norm_fwd_vpl", 8), (b"softmax_lanes_per_row", 1), (b"eltwise_tile_min", 64),
                      (b"norm_bwd_waves", 16)):
        assert lib.oslo_tune(key, good) == 0 and lib.oslo_tune(key, 0) == 0, key
    # empty problems succeed without touching any pointer
    assert lib.oslo_ln_fwd(None, None, None, None, None, None, 0, 8, 1e-5, 0, 0, None) == 0
    assert lib.oslo_bias_gelu_fwd(None, None, None, 0, 8, 2, None) == 0


def test_multi_tensor_entry_points_check_their_arguments():
    import ctypes

    lib = _C.load_library()
    one = (ctypes.c_void_p * 1)(None)
    sizes = (ctypes.c_int64 * 1)(8)
    neg = (ctypes.c_int64 * 1)(-8)
    # float32 gradients cannot meet 16-bit weights; a copy needs float32 weights
    rc = lib.oslo_multi_tensor_sgd(one, one, one, None, sizes, 1, 0, 0, 0, 0.1, 0, 1, 0, 1.0, 0, 1, 0, None, None)
    assert rc == -1 and b"weights must" in lib.oslo_hip_last_error()
    rc = lib.oslo_multi_tensor_sgd(one, one, one, one, sizes, 1, 0, 0, 0, 0.1, 0, 1, 0, 1.0, 1, 1, 1, None, None)
    assert rc == -1 and b"16-bit copy" in lib.oslo_hip_last_error()
    # a null tensor pointer and a negative length are caught before any launch
    rc = lib.oslo_multi_tensor_sgd(one, one, one, None, sizes, 1, 0, 0, 0, 0.1, 0, 1, 0, 1.0, 0, 0, 0, None, None)
    assert rc == -1 and b"null pointer" in lib.oslo_hip_last_error()
    rc = lib.oslo_multi_tensor_adagrad(one, one, one, neg, 1, 0.1, 1e-10, 0, 0.0, 0, None)
    assert rc == -1 and b"size -8" in lib.oslo_hip_last_error()
    assert lib.oslo_multi_tensor_adagrad(one, one, one, sizes, 1, 0.1, 1e-10, 2, 0.0, 0, None) == -1
    assert lib.oslo_multi_tensor_novograd(one, one, one, sizes, 1, None, 0.1, 0.9, 0.99, 1e-8, 1, 1, 0.0, 1, 1, 0, None) == -1
    assert lib.oslo_multi_tensor_lamb_stage1(one, one, one, one, sizes, 1, 0.9, 0.99, 1e-6, 1, 1, 0.0, 1, 3,
                                             None, 1.0, 0, None) == -1
    assert lib.oslo_multi_tensor_lamb_stage2(one, one, sizes, 1, None, None, 0.1, 0.0, 0, 0, None) == -1
    assert lib.oslo_multi_tensor_norm(one, sizes, 1, 0, None, 0, None, None, 2, 0, 0.0, 0.0, None, 0, None) == -1
    assert b"no workspace" in lib.oslo_hip_last_error()
    assert lib.oslo_multi_tensor_norm(one, sizes, 1, 0, one, 1, None, None, 1, 0, 0.0, 0.0, None, 0, None) == -1
    assert lib.oslo_multi_tensor_norm(one, sizes, 1, 0, one, 1, None, None, 2, 1, 0.5, 0.5, None, 0, None) == -1
    assert b"blending needs" in lib.oslo_hip_last_error()
    # workspace: one value per piece of 16384 float32 / 32768 16-bit elements, at least one
    three = (ctypes.c_int64 * 3)(16384, 16385, 0)
    assert lib.oslo_multi_tensor_norm_partials(three, 3, 0) == 3
    assert lib.oslo_multi_tensor_norm_partials(three, 3, 2) == 2
    assert lib.oslo_multi_tensor_norm_partials(three, 0, 0) == 1
    assert lib.oslo_multi_tensor_norm_partials(neg, 1, 0) < 0
    # no tensors: nothing to do
    assert lib.oslo_multi_tensor_sgd(None, None, None, None, None, 0, 0, 0, 0, 0.1, 0, 1, 0, 1.0, 0, 0, 0, None, None) == 0


def test_batch_per_block():
    lib = _C.load_library()
    assert lib.oslo_softmax_batch_per_block(1024, 1024, 16, 16) >= 1
    assert lib.oslo_softmax_batch_per_block(0, 8, 1, 1) < 0


def test_missing_library_raises_environment_error(monkeypatch, tmp_path):
    monkeypatch.setattr(_C, "_lib", None)
    bogus = tmp_path / "liboslo_hip.so"
    bogus.write_bytes(b"not an ELF file")
    monkeypatch.setattr(_C, "LIBRARY_PATH", str(bogus))
    with pytest.raises(EnvironmentError):
        _C.load_library()
