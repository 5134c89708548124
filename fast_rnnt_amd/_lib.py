"""The two native pieces of this package: libfast_rnnt_amd.so (the gfx950 C-ABI
library, bound here with ctypes for the operators that are not on the per-step hot
path and for tests of the raw ABI) and the compiled torch operator module
``fast_rnnt_amd._C`` that sits on top of it (:func:`ops`).

Both are built in-tree by ``make -C fast_rnnt_amd/csrc`` (or
``__graft_entry__.build()``).  There is no fallback: if one is missing, loading
raises, and every operator of this package needs them.
"""
import ctypes
import os
import re

import torch  # noqa: F401  (loads the HIP runtime the library binds to)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libfast_rnnt_amd.so")
HEADER_PATH = os.path.join(os.path.dirname(_HERE), "include", "fast_rnnt_amd.h")

_lib = None

_P = ctypes.c_void_p
_I = ctypes.c_int
_F = ctypes.c_float
_D = ctypes.c_double

# argument lists of the entry points, in header order
_SIGNATURES = {
    "frnnt_version": ([], _I),
    "frnnt_last_error": ([], ctypes.c_char_p),
    "frnnt_set_spin_limit": ([_I], None),
    "frnnt_mi_forward_f32": ([_P, _P, _P, _P, _P, _I, _I, _I, _I, _P], _I),
    "frnnt_mi_forward_f64": ([_P, _P, _P, _P, _P, _I, _I, _I, _I, _P], _I),
    "frnnt_mi_forward_checked_f32": ([_P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P, _P], _I),
    "frnnt_mi_forward_checked_f64": ([_P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P, _P], _I),
    "frnnt_mi_backward_f32": ([_P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P], _I),
    "frnnt_mi_backward_f64": ([_P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P], _I),
    "frnnt_simple_logprobs_fwd_f32": ([_P] * 9 + [_I] * 7 + [_P], _I),
    "frnnt_simple_logprobs_fwd_f64": ([_P] * 9 + [_I] * 7 + [_P], _I),
    "frnnt_simple_logprobs_bwd_f32": ([_P] * 8 + [_I, _D] + [_P] * 8 + [_I] * 7 + [_P], _I),
    "frnnt_simple_logprobs_bwd_f64": ([_P] * 8 + [_I, _D] + [_P] * 8 + [_I] * 7 + [_P], _I),
    "frnnt_simple_logprobs_bwd_noalloc_f32": ([_P] * 8 + [_I, _D] + [_P] * 4 + [_I] * 7 + [_P], _I),
    "frnnt_smoothed_logprobs_fwd_f32": ([_P] * 14 + [_I] * 6 + [_D, _D, _P], _I),
    "frnnt_smoothed_logprobs_fwd_f64": ([_P] * 14 + [_I] * 6 + [_D, _D, _P], _I),
    "frnnt_smoothed_logprobs_bwd_f32": ([_P] * 21 + [_I] * 6 + [_D, _D, _P], _I),
    "frnnt_smoothed_logprobs_bwd_f64": ([_P] * 21 + [_I] * 6 + [_D, _D, _P], _I),
    "frnnt_simple_loss_fwd_f32": ([_P] * 14 + [_I] * 8 + [_P, _P], _I),
    "frnnt_simple_loss_fwd_f64": ([_P] * 14 + [_I] * 8 + [_P, _P], _I),
    "frnnt_mi_loss_fwd_f32": ([_P] * 8 + [_I] * 6 + [_P, _P], _I),
    "frnnt_mi_loss_fwd_f64": ([_P] * 8 + [_I] * 6 + [_P, _P], _I),
    "frnnt_mi_scale_grads_f32": ([_P] * 3 + [_I, _D] + [_I] * 4 + [_P], _I),
    "frnnt_mi_scale_grads_f64": ([_P] * 3 + [_I, _D] + [_I] * 4 + [_P], _I),
    "frnnt_loss_reduce_f32": ([_P, _P, _I, _I, _P], _I),
    "frnnt_loss_reduce_f64": ([_P, _P, _I, _I, _P], _I),
    "frnnt_lattice_logprobs_fwd_f32": ([_P] * 9 + [_I] * 8 + [_P], _I),
    "frnnt_lattice_logprobs_fwd_f64": ([_P] * 9 + [_I] * 8 + [_P], _I),
    "frnnt_lattice_logprobs_bwd_f32": ([_P] * 8 + [_I] * 8 + [_P], _I),
    "frnnt_lattice_logprobs_bwd_f64": ([_P] * 8 + [_I] * 8 + [_P], _I),
    "frnnt_lattice_logprobs_fwd_f16": ([_P] * 9 + [_I] * 8 + [_P], _I),
    "frnnt_lattice_logprobs_fwd_bf16": ([_P] * 9 + [_I] * 8 + [_P], _I),
    "frnnt_lattice_logprobs_bwd_f16": ([_P] * 8 + [_I] * 8 + [_P], _I),
    "frnnt_lattice_logprobs_bwd_bf16": ([_P] * 8 + [_I] * 8 + [_P], _I),
    "frnnt_prune_ranges_f32": ([_P] * 4 + [_I] * 5 + [_P], _I),
    "frnnt_prune_ranges_f64": ([_P] * 4 + [_I] * 5 + [_P], _I),
    "frnnt_prune_gather_f32": ([_P] * 3 + [_I] * 5 + [_P], _I),
    "frnnt_prune_gather_f64": ([_P] * 3 + [_I] * 5 + [_P], _I),
    "frnnt_prune_gather_bwd_f32": ([_P] * 3 + [_I] * 5 + [_P], _I),
    "frnnt_prune_gather_bwd_f64": ([_P] * 3 + [_I] * 5 + [_P], _I),
    "frnnt_prune_gather_f16": ([_P] * 3 + [_I] * 5 + [_P], _I),
    "frnnt_prune_gather_bf16": ([_P] * 3 + [_I] * 5 + [_P], _I),
    "frnnt_prune_gather_bwd_f16": ([_P] * 3 + [_I] * 5 + [_P], _I),
    "frnnt_prune_gather_bwd_bf16": ([_P] * 3 + [_I] * 5 + [_P], _I),
    "frnnt_pruned_joiner_fwd_f32": ([_P] * 4 + [_I] * 6 + [_P], _I),
    "frnnt_pruned_joiner_fwd_f64": ([_P] * 4 + [_I] * 6 + [_P], _I),
    "frnnt_pruned_joiner_bwd_f32": ([_P] * 5 + [_I] * 6 + [_P], _I),
    "frnnt_pruned_joiner_bwd_f64": ([_P] * 5 + [_I] * 6 + [_P], _I),
}


def declared_symbols():
    """Names of every function the public header declares."""
    with open(HEADER_PATH) as f:
        text = re.sub(r"/\*.*?\*/", "", f.read(), flags=re.S)
    return sorted(set(re.findall(r"\b(frnnt_[a-z0-9_]+)\s*\(", text)))


def load():
    """Return the loaded library; raises RuntimeError if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `make -C fast_rnnt_amd/csrc` "
                "(hipcc, gfx950). fast_rnnt_amd has no CPU or eager fallback."
            )
        lib = ctypes.CDLL(LIB_PATH)
        for name, (argtypes, restype) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = restype
        _lib = lib
    return _lib


_ops = None


def ops():
    """The compiled torch operator module ``fast_rnnt_amd._C`` (csrc/torch_ops.cpp): the
    reference's three operator functions and the loss nodes, also registered as
    ``torch.ops.fast_rnnt_amd.*``.  Built in-tree beside the library by
    ``make -C fast_rnnt_amd/csrc``; raises RuntimeError if it is missing."""
    global _ops
    if _ops is None:
        load()  # the module links against the library: fail with the build hint first
        try:
            from . import _C
        except ImportError as e:
            raise RuntimeError(
                f"fast_rnnt_amd/_C*.so cannot be imported ({e}): build it with "
                "`make -C fast_rnnt_amd/csrc` (g++ against the installed torch). "
                "fast_rnnt_amd has no CPU or eager fallback.") from e
        _ops = _C
    return _ops


def call(name, *args):
    """Invoke an int-returning entry point; raise RuntimeError on a non-zero code."""
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise RuntimeError(f"{name} failed ({rc}): {lib.frnnt_last_error().decode()}")


def stream_of(t: "torch.Tensor"):
    """hipStream_t (as an int) torch is currently using on the tensor's device."""
    return torch.cuda.current_stream(t.device).cuda_stream


def suffix(dtype, narrow: bool = False) -> str:
    """Entry-point suffix of a tensor type; `narrow` also admits the 2-byte types, for
    the entry points that have a float16 / bfloat16 form."""
    if dtype == torch.float32:
        return "f32"
    if dtype == torch.float64:
        return "f64"
    if narrow and dtype == torch.float16:
        return "f16"
    if narrow and dtype == torch.bfloat16:
        return "bf16"
    raise RuntimeError(f"fast_rnnt_amd supports float32 and float64 tensors here, got {dtype}")


def ptr(t):
    return None if t is None else t.data_ptr()
