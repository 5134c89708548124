"""The C-ABI library loads and exports every function include/fast_rnnt_amd.h declares."""
import ctypes
import os

import pytest

from fast_rnnt_amd import _lib


def test_library_exports_every_declared_symbol():
    if not os.path.exists(_lib.LIB_PATH):
        pytest.fail(f"{_lib.LIB_PATH} not built; run `make -C fast_rnnt_amd/csrc`")
    lib = ctypes.CDLL(_lib.LIB_PATH)
    names = _lib.declared_symbols()
    assert "frnnt_mi_forward_f32" in names and "frnnt_mi_backward_f64" in names
    for name in names:
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    # every declared function also has a ctypes signature in the binding
    assert set(names) == set(_lib._SIGNATURES)


def test_version_and_error_text():
    lib = _lib.load()
    assert lib.frnnt_version() >= 100
    assert isinstance(lib.frnnt_last_error(), bytes)


def test_argument_errors_are_reported_without_a_gpu():
    # validation happens on the host before any launch
    lib = _lib.load()
    rc = lib.frnnt_mi_forward_f32(None, None, None, None, None, 2, 3, 4, 0, None)
    assert rc == -1 and b"null" in lib.frnnt_last_error()
    rc = lib.frnnt_mi_forward_f32(None, None, None, None, None, -1, 3, 4, 0, None)
    assert rc == -1
    assert lib.frnnt_mi_forward_f32(None, None, None, None, None, 0, 3, 4, 0, None) == 0


def test_size_limits_are_reported_without_a_gpu():
    # the float32 simple-loss kernels address an utterance's lm / am rows with 32-bit byte
    # offsets; sizes beyond that are refused on the host, before any pointer is followed
    lib = _lib.load()
    dummy = ctypes.c_void_p(0x1000)
    B, S, T, C = 1, 10, 70000, 8000          # T * C * 4 bytes >= 2 GiB
    rc = lib.frnnt_simple_logprobs_fwd_f32(dummy, dummy, dummy, None, dummy, dummy, dummy, dummy,
                                           None, B, S, T, C, 0, 0, 0, None)
    assert rc == -3 and b"2 GiB" in lib.frnnt_last_error()
    B, S, T = 1, 20000, 20000                # (S+1) * (T+1) * 4 bytes >= 1 GiB
    rc = lib.frnnt_mi_forward_f32(dummy, dummy, None, dummy, dummy, B, S, T, 0, None)
    assert rc == -3 and b"1 GiB" in lib.frnnt_last_error()


def test_cpu_tensors_are_refused():
    import torch
    from fast_rnnt_amd import _fast_rnnt

    px, py, p = torch.zeros(1, 2, 4), torch.zeros(1, 3, 3), torch.zeros(1, 3, 4)
    with pytest.raises(RuntimeError, match="no CPU path"):
        _fast_rnnt.mutual_information_forward(px, py, None, p)
