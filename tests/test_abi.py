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


def test_cpu_tensors_are_refused():
    import torch
    from fast_rnnt_amd import _fast_rnnt

    px, py, p = torch.zeros(1, 2, 4), torch.zeros(1, 3, 3), torch.zeros(1, 3, 4)
    with pytest.raises(RuntimeError, match="no CPU path"):
        _fast_rnnt.mutual_information_forward(px, py, None, p)
