"""RNN-T losses on the gfx950 kernels.

Public functions, argument names, defaults, return shapes and error behaviour
are those of fast_rnnt/python/fast_rnnt/rnnt_loss.py; the tensor algebra of
each px/py builder runs in fused HIP kernels (see fast_rnnt_amd/csrc) behind
autograd Functions instead of chains of stock torch ops.

Conventions (same as the reference): ``lm`` is ``[B][S+1][C]``, ``am`` is
``[B][T][C]``, ``symbols`` int64 ``[B][S]``, ``boundary`` int64 ``[B][4]`` rows
``[begin_symbol, begin_frame, end_symbol, end_frame]`` (``None`` = ``[0,0,S,T]``),
``rnnt_type`` one of ``"regular"`` (a symbol does not consume a frame; px has
T+1 columns, the last one -inf), ``"modified"`` (every step consumes a frame)
and ``"constrained"`` (modified, plus a forced blank after each symbol).
"""
from typing import Optional, Tuple, Union

import contextlib

import torch
from torch import Tensor

from . import _lib
from .mutual_information import (_assert_boundary, boundary_rows,  # noqa: F401
                                 mutual_information_recursion)

_RNNT_TYPES = {"regular": 0, "modified": 1, "constrained": 2}


def validate_st_lengths(S: int, T: int, is_rnnt_type_regular: bool,
                        boundary: Optional[Tensor] = None, on_device: bool = False):
    """fast_rnnt/python/fast_rnnt/rnnt_loss.py:25-42 (same assertions; the boundary
    rows are looked at on the host copy shared with the recursion's own check, so a
    loss call waits for the device at most once).  ``on_device``: the caller hands the
    row tests to the recursion's forward kernel (:func:`_device_checks`), so nothing
    waits for a host copy of the rows here."""
    if boundary is None:
        assert S >= 1, S
        assert is_rnnt_type_regular or T >= S, \
            f"Modified transducer requires T >= S, but got T={T} and S={S}"
    elif on_device:
        return
    else:
        rows = boundary_rows(boundary)
        assert all(r[2] >= 1 for r in rows), boundary[:, 2]
        assert is_rnnt_type_regular or all(r[3] >= r[2] for r in rows), \
            f"Modified transducer requires T >= S, but got T={boundary[:, 3]} and S={boundary[:, 2]}"


def fix_for_boundary(px: Tensor, boundary: Optional[Tensor] = None) -> Tensor:
    """Set ``px[b, :, boundary[b, 3]] = -inf`` in place (rnnt_loss.py:45-63).

    The fused builders of this module already do this inside their kernels; the
    function is kept for callers that assemble px themselves.
    """
    if boundary is None:
        return px
    B, S, T1 = px.shape
    index = boundary[:, 3].reshape(B, 1, 1).expand(B, S, T1)
    return px.scatter_(dim=2, index=index, value=float("-inf"))


def _require_gpu(*tensors: Tensor) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("fast_rnnt_amd runs on GPU tensors only (no CPU path)")


def _check_tensors(floats, indices) -> None:
    """What must hold before raw pointers go to the library: every tensor on one GPU,
    the floating-point ones of one dtype, the index tensors int64.  The kernels read
    index tensors as 64-bit words and all floating-point buffers as one element type, so
    anything else would be read past its end; the reference fails in the same places
    with a RuntimeError from torch.gather / scatter_ / matmul."""
    floats = [(n, t) for n, t in floats if t is not None]
    indices = [(n, t) for n, t in indices if t is not None]
    name0, first = floats[0]
    for name, t in floats + indices:
        if t.device != first.device:
            raise RuntimeError(f"{name} is on {t.device}, {name0} on {first.device}: "
                               "all tensors must be on the same device")
    for name, t in floats:
        if t.dtype != first.dtype:
            raise RuntimeError(f"{name} is {t.dtype}, {name0} is {first.dtype}: "
                               "floating-point tensors must share one dtype")
    for name, t in indices:
        if t.dtype != torch.int64:
            raise RuntimeError(f"{name} must be an int64 tensor, got {t.dtype}")
    _require_gpu(*(t for _, t in floats + indices))


_NARROW = (torch.float16, torch.bfloat16)


def _lattice_dtype(dtype):
    """Element type of px / py (and of the loss) for inputs of type `dtype`: the 2-byte
    types are accumulated in float32 (the reference's recursion has no half form,
    mutual_information_cuda.cu:37-38)."""
    return torch.float32 if dtype in _NARROW else dtype


def _widen(*tensors):
    """float16 / bfloat16 inputs of the additive-joiner losses as float32 (differentiable:
    the gradients come back in the inputs' type); other types pass through."""
    return tuple(t.float() if t is not None and t.dtype in _NARROW else t for t in tensors)


class _SimpleLogprobs(torch.autograd.Function):
    """(px, py) of the additive-joiner loss: frnnt_simple_logprobs_fwd/bwd."""

    @staticmethod
    def forward(ctx, lm, am, symbols, boundary, termination_symbol, rnnt_type):
        B, T, C = am.shape
        S = lm.shape[1] - 1
        kind = _RNNT_TYPES[rnnt_type]
        sfx = _lib.suffix(am.dtype)
        lm_c, am_c = lm.contiguous(), am.contiguous()
        sym_c = symbols.contiguous()
        bnd_c = boundary.contiguous() if boundary is not None else None
        opts = dict(dtype=am.dtype, device=am.device)
        T1 = T + 1 if kind == 0 else T
        need_grad = ctx.needs_input_grad[0] or ctx.needs_input_grad[1]
        with torch.cuda.device(am.device):
            px = torch.empty(B, S, T1, **opts)
            py = torch.empty(B, S + 1, T, **opts)
            lm_max = torch.empty(B, S + 1, **opts)
            am_max = torch.empty(B, T, **opts)
            norm_raw = torch.empty(B, S + 1, T, **opts) if need_grad else None
            _lib.call("frnnt_simple_logprobs_fwd_" + sfx, lm_c.data_ptr(), am_c.data_ptr(),
                      sym_c.data_ptr(), _lib.ptr(bnd_c), px.data_ptr(), py.data_ptr(),
                      lm_max.data_ptr(), am_max.data_ptr(), _lib.ptr(norm_raw), B, S, T, C,
                      int(termination_symbol), kind, 0, _lib.stream_of(am))
        if need_grad:
            ctx.save_for_backward(lm_c, am_c, sym_c, bnd_c, lm_max, am_max, norm_raw)
            ctx.meta = (B, S, T, C, int(termination_symbol), kind, sfx)
        return px, py

    @staticmethod
    def backward(ctx, gpx, gpy):
        lm, am, sym, bnd, lm_max, am_max, norm_raw = ctx.saved_tensors
        B, S, T, C, term, kind, sfx = ctx.meta
        opts = dict(dtype=am.dtype, device=am.device)
        T1 = T + 1 if kind == 0 else T
        with torch.cuda.device(am.device):
            gpx = torch.zeros(B, S, T1, **opts) if gpx is None else gpx.contiguous()
            gpy = torch.zeros(B, S + 1, T, **opts) if gpy is None else gpy.contiguous()
            dmat = torch.empty(B, S + 1, (T + 3) // 4 * 4, **opts)
            row_x = torch.empty(B, S + 1, **opts)
            row_y = torch.empty(B, S + 1, **opts)
            col_y = torch.empty(B, T, **opts)
            lm_grad = torch.empty_like(lm) if ctx.needs_input_grad[0] else None
            am_grad = torch.empty_like(am) if ctx.needs_input_grad[1] else None
            _lib.call("frnnt_simple_logprobs_bwd_" + sfx, lm.data_ptr(), am.data_ptr(),
                      sym.data_ptr(), _lib.ptr(bnd), lm_max.data_ptr(), am_max.data_ptr(),
                      norm_raw.data_ptr(), None, 0, 1.0, gpx.data_ptr(), gpy.data_ptr(),
                      dmat.data_ptr(),
                      row_x.data_ptr(), row_y.data_ptr(), col_y.data_ptr(), _lib.ptr(lm_grad),
                      _lib.ptr(am_grad), B, S, T, C, term, kind, 0, _lib.stream_of(am))
        return lm_grad, am_grad, None, None, None, None


def get_rnnt_logprobs(
    lm: Tensor, am: Tensor, symbols: Tensor, termination_symbol: int,
    rnnt_type: str = "regular", boundary: Optional[Tensor] = None,
) -> Tuple[Tensor, Tensor]:
    """(px, py) for the simple loss whose joiner is ``lm + am``
    (fast_rnnt/python/fast_rnnt/rnnt_loss.py:66-227).

    Returns:
      px ``[B][S][T+1]`` (regular) or ``[B][S][T]``: log-prob of emitting
      ``symbols[b][s]`` at lattice position (s, t); py ``[B][S+1][T]``: log-prob
      of emitting the termination symbol, i.e. moving to the next frame.
    """
    assert lm.ndim == 3, lm.ndim
    assert am.ndim == 3, am.ndim
    assert lm.shape[0] == am.shape[0], (lm.shape[0], am.shape[0])
    assert lm.shape[2] == am.shape[2], (lm.shape[2], am.shape[2])
    (B, T, C) = am.shape
    S = lm.shape[1] - 1
    assert symbols.shape == (B, S), symbols.shape
    validate_st_lengths(S, T, rnnt_type == "regular", boundary)
    assert rnnt_type in ["regular", "modified", "constrained"], rnnt_type
    _check_tensors([("am", am), ("lm", lm)], [("symbols", symbols), ("boundary", boundary)])
    lm, am = _widen(lm, am)
    return _SimpleLogprobs.apply(lm, am, symbols, boundary, termination_symbol, rnnt_type)


def _apply_delay_penalty(px: Tensor, boundary: Optional[Tensor], rnnt_type: str,
                         delay_penalty: float) -> None:
    """``px += ((T_b - 1) / 2 - t) * delay_penalty`` in place (rnnt_loss.py:309-324)."""
    B, S, T0 = px.shape
    T = T0 if rnnt_type != "regular" else T0 - 1
    if boundary is None:
        offset = torch.tensor((T - 1) / 2, dtype=px.dtype, device=px.device).expand(B, 1, 1)
    else:
        offset = (boundary[:, 3] - 1) / 2
    penalty = offset.reshape(B, 1, 1) - torch.arange(T0, device=px.device).reshape(1, 1, T0)
    penalty = penalty * delay_penalty
    px += penalty.to(px.dtype)


_REDUCTIONS = {"none": 0, "mean": 1, "sum": 2}


def _device_checks(rnnt_type: str, boundary: Optional[Tensor]) -> int:
    """FRNNT_CHECK_* bits for the recursion's forward kernel when the boundary rows are to
    be tested on the device (the default, see :func:`set_boundary_checks`): the two
    assertions of validate_st_lengths (rnnt_loss.py:38-42); the window's range
    (mutual_information.py:277-288) is always tested there.  0 = the rows have been
    asserted on the host."""
    if boundary is None or not _lib.ops().deferred_checks():
        return 0
    return 1 | (0 if rnnt_type == "regular" else 2)


def _recursion_and_reduce(px, py, boundary, rnnt_type, delay_penalty, reduction, return_grad):
    """Shared tail of the four losses (e.g. rnnt_loss.py:309-340): one autograd node of the
    operator module (recursion, its eager backward with a gradient of ones, the reduction;
    its backward scales the occupation gradients in place, mutual_information.py:159-181)."""
    if delay_penalty > 0.0:
        _apply_delay_penalty(px, boundary, rnnt_type, delay_penalty)
    if reduction not in _REDUCTIONS:
        # (the reference finds this out after the recursion has run: same exception)
        raise ValueError(f"reduction should be ('none' | 'mean' | 'sum'), given {reduction}")
    # the argument checks of mutual_information_recursion (mutual_information.py:271-289)
    assert px.ndim == 3
    B, S, T1 = px.shape
    T = py.shape[-1]
    assert px.shape[-1] in [T, T + 1]
    assert py.shape == (B, S + 1, T)
    assert px.dtype == py.dtype
    checks = _device_checks(rnnt_type, boundary)
    if boundary is not None:
        _assert_boundary(boundary, B, S, T, on_device=checks != 0)
    _require_gpu(px, py)
    loss, px_grad, py_grad = _lib.ops().recursion_loss(
        px, py, boundary, bool(return_grad), _REDUCTIONS[reduction], checks)
    return (loss, (px_grad, py_grad)) if return_grad else loss


def _on_device(device):
    """Device guard that costs nothing when `device` is already current."""
    if torch.cuda.current_device() == device.index:
        return contextlib.nullcontext()
    return torch.cuda.device(device)


def _carve(sizes):
    """Element offsets of consecutive buffers, each starting 16-byte aligned (for
    4- and 8-byte elements), and the total element count."""
    offsets, total = [], 0
    for n in sizes:
        offsets.append(total)
        total += (n + 3) & ~3
    return offsets, total


def rnnt_loss_simple(
    lm: Tensor, am: Tensor, symbols: Tensor, termination_symbol: int,
    boundary: Optional[Tensor] = None, rnnt_type: str = "regular",
    delay_penalty: float = 0.0, reduction: Optional[str] = "mean", return_grad: bool = False,
) -> Union[Tensor, Tuple[Tensor, Tuple[Tensor, Tensor]]]:
    """RNN-T loss with an additive joiner (rnnt_loss.py:230-340).

    Returns the loss (``[B]`` for ``reduction="none"``, else a scalar) and, with
    ``return_grad=True``, also ``(px_grad, py_grad)``: the occupation
    probabilities of the lattice, used by :func:`get_rnnt_prune_ranges`.
    """
    # the argument checks of get_rnnt_logprobs and mutual_information_recursion
    assert lm.ndim == 3, lm.ndim
    assert am.ndim == 3, am.ndim
    assert lm.shape[0] == am.shape[0], (lm.shape[0], am.shape[0])
    assert lm.shape[2] == am.shape[2], (lm.shape[2], am.shape[2])
    (B, T, C) = am.shape
    S = lm.shape[1] - 1
    assert symbols.shape == (B, S), symbols.shape
    assert rnnt_type in ["regular", "modified", "constrained"], rnnt_type
    checks = _device_checks(rnnt_type, boundary)
    validate_st_lengths(S, T, rnnt_type == "regular", boundary, on_device=checks != 0)
    _check_tensors([("am", am), ("lm", lm)], [("symbols", symbols), ("boundary", boundary)])
    if boundary is not None:
        _assert_boundary(boundary, B, S, T, on_device=checks != 0)
    if reduction not in ("none", "mean", "sum"):
        raise ValueError(f"reduction should be ('none' | 'mean' | 'sum'), given {reduction}")
    lm, am = _widen(lm, am)
    # the whole device pipeline is one autograd node of the operator module: px / py (row
    # maxima + MFMA contraction), the recursion, its backward with a gradient of ones, the
    # reduction; its backward scales the occupation gradients in place and runs the two
    # gradient products
    loss, px_grad, py_grad = _lib.ops().simple_loss(
        lm, am, symbols, boundary, int(termination_symbol), _RNNT_TYPES[rnnt_type],
        float(delay_penalty), bool(return_grad), _REDUCTIONS[reduction], checks)
    return (loss, (px_grad, py_grad)) if return_grad else loss


class _LatticeLogprobs(torch.autograd.Function):
    """(px, py) from joiner logits, pruned (``ranges`` given) or not:
    frnnt_lattice_logprobs_fwd/bwd."""

    @staticmethod
    def forward(ctx, logits, symbols, ranges, boundary, termination_symbol, rnnt_type,
                window_only=False):
        # window_only: the caller feeds (px, py) to the recursion with this same boundary,
        # so cells outside each utterance's window may stay undefined and carry no gradient
        B, T, R, C = logits.shape
        S = symbols.shape[1]
        kind = _RNNT_TYPES[rnnt_type]
        # float16 / bfloat16 logits are read as they are; px, py and everything after
        # them are float32
        sfx = _lib.suffix(logits.dtype, narrow=True)
        lg = logits.contiguous()
        sym_c = symbols.contiguous()
        rng_c = ranges.contiguous() if ranges is not None else None
        bnd_c = boundary.contiguous() if boundary is not None else None
        opts = dict(dtype=_lattice_dtype(logits.dtype), device=logits.device)
        T1 = T + 1 if kind == 0 else T
        windowed = bool(window_only) and bnd_c is not None
        with torch.cuda.device(logits.device):
            px = torch.empty(B, S, T1, **opts)
            py = torch.empty(B, S + 1, T, **opts)
            norm = torch.empty(B, T, R, **opts)
            xr = torch.empty(B, T, R, **opts)
            yr = torch.empty(B, T, R, **opts)
            _lib.call("frnnt_lattice_logprobs_fwd_" + sfx, lg.data_ptr(), sym_c.data_ptr(),
                      _lib.ptr(rng_c), _lib.ptr(bnd_c), px.data_ptr(), py.data_ptr(),
                      norm.data_ptr(), xr.data_ptr(), yr.data_ptr(), B, S, T, R, C,
                      int(termination_symbol), kind, int(windowed), _lib.stream_of(logits))
        if ctx.needs_input_grad[0]:
            ctx.save_for_backward(lg, sym_c, rng_c, bnd_c, norm)
            ctx.meta = (B, S, T, R, C, int(termination_symbol), kind, sfx, int(windowed))
        return px, py

    @staticmethod
    def backward(ctx, gpx, gpy):
        lg, sym, rng, bnd, norm = ctx.saved_tensors
        B, S, T, R, C, term, kind, sfx, windowed = ctx.meta
        opts = dict(dtype=norm.dtype, device=lg.device)
        T1 = T + 1 if kind == 0 else T
        with torch.cuda.device(lg.device):
            gpx = torch.zeros(B, S, T1, **opts) if gpx is None else gpx.contiguous()
            gpy = torch.zeros(B, S + 1, T, **opts) if gpy is None else gpy.contiguous()
            grad = torch.empty_like(lg)
            _lib.call("frnnt_lattice_logprobs_bwd_" + sfx, lg.data_ptr(), sym.data_ptr(),
                      _lib.ptr(rng), _lib.ptr(bnd), norm.data_ptr(), gpx.data_ptr(),
                      gpy.data_ptr(), grad.data_ptr(), B, S, T, R, C, term, kind, windowed,
                      _lib.stream_of(lg))
        return grad, None, None, None, None, None, None


def _joint_logprobs(logits, symbols, termination_symbol, boundary, rnnt_type, window_only):
    assert logits.ndim == 4, logits.ndim
    (B, T, S1, C) = logits.shape
    S = S1 - 1
    assert symbols.shape == (B, S), symbols.shape
    assert rnnt_type in ["regular", "modified", "constrained"], rnnt_type
    # (window_only: the caller is a loss function, whose recursion tests the rows itself)
    on_device = bool(window_only) and _device_checks(rnnt_type, boundary) != 0
    validate_st_lengths(S, T, rnnt_type == "regular", boundary, on_device=on_device)
    _check_tensors([("logits", logits)], [("symbols", symbols), ("boundary", boundary)])
    if window_only and boundary is not None:
        _assert_boundary(boundary, B, S, T, on_device=on_device)
    return _LatticeLogprobs.apply(logits, symbols, None, boundary, termination_symbol, rnnt_type,
                                  window_only)


def get_rnnt_logprobs_joint(
    logits: Tensor, symbols: Tensor, termination_symbol: int,
    boundary: Optional[Tensor] = None, rnnt_type: str = "regular",
) -> Tuple[Tensor, Tensor]:
    """(px, py) from the full joiner output ``logits`` of shape ``(B, T, S+1, C)``
    (fast_rnnt/python/fast_rnnt/rnnt_loss.py:343-449)."""
    return _joint_logprobs(logits, symbols, termination_symbol, boundary, rnnt_type, False)


def rnnt_loss(
    logits: Tensor, symbols: Tensor, termination_symbol: int,
    boundary: Optional[Tensor] = None, rnnt_type: str = "regular",
    delay_penalty: float = 0.0, reduction: Optional[str] = "mean", return_grad: bool = False,
) -> Tensor:
    """The unpruned RNN-T loss on joiner logits ``(B, T, S+1, C)`` (rnnt_loss.py:452-547).
    The logits of cells outside an utterance's boundary window are not read: the
    recursion never visits them and their gradient is exactly zero."""
    px, py = _joint_logprobs(logits, symbols, termination_symbol, boundary, rnnt_type, True)
    return _recursion_and_reduce(px, py, boundary, rnnt_type, delay_penalty, reduction,
                                 return_grad)


def _monotonic_lower_bound(x: Tensor) -> Tensor:
    """Suffix minimum along the last axis: the largest non-decreasing sequence
    below ``x`` (rnnt_loss.py:550-581), e.g. [0,2,1,3,6,5,8] -> [0,1,1,3,5,5,8]."""
    x = torch.flip(x, dims=(-1,))
    x, _ = torch.cummin(x, dim=-1)
    return torch.flip(x, dims=(-1,))


def _adjust_pruning_lower_bound(s_begin: Tensor, s_range: int) -> Tensor:
    """Make ``s_begin`` (B, T) non-decreasing, starting at 0, with steps below
    ``s_range`` (rnnt_loss.py:584-632).  Torch-op form of what the prune-range
    kernel does in LDS; kept for callers that use it on its own."""
    (B, T) = s_begin.shape
    ramp = (s_range - 1) * torch.arange(0, T, device=s_begin.device)
    s_begin = _monotonic_lower_bound(s_begin)
    s_begin = torch.clamp(_monotonic_lower_bound(ramp - s_begin), min=0)
    return ramp - s_begin


def get_rnnt_prune_ranges(px_grad: Tensor, py_grad: Tensor, boundary: Tensor,
                          s_range: int) -> Tensor:
    """Pruning bounds from the occupation gradients (rnnt_loss.py:638-777).

    Returns an int64 tensor ``(B, T, s_range)``: for each frame the ``s_range``
    consecutive symbol positions kept.  As in the reference, ``s_range`` is raised
    (with a printed warning) to the minimum the regular lattice needs and capped
    at ``S + 1``, so the last dimension can differ from the request.
    """
    (B, S, T1) = px_grad.shape
    T = py_grad.shape[-1]
    is_regular = T1 != T
    assert T1 in [T, T + 1], T1
    assert py_grad.shape == (B, S + 1, T), py_grad.shape
    assert boundary.shape == (B, 4), boundary.shape
    validate_st_lengths(S, T, is_regular, boundary)
    _check_tensors([("px_grad", px_grad), ("py_grad", py_grad)], [("boundary", boundary)])

    if is_regular:
        # max over the batch of trunc((S_b - 1) / T_b) + 2 (rnnt_loss.py:696-710), from the
        # host copy of the boundary rows that the loss call before this one has usually left
        # behind: no kernels and no wait for the device here
        s_range_min = None
        for _s_begin, _t_begin, s_end, t_end in boundary_rows(boundary):
            if t_end == 0:
                raise RuntimeError("ZeroDivisionError")  # what the reference's integer division raises
            quotient = abs(s_end - 1) // abs(t_end)
            if (s_end - 1 < 0) != (t_end < 0):
                quotient = -quotient
            s_range_min = quotient + 2 if s_range_min is None else max(s_range_min, quotient + 2)
        if s_range_min is not None and s_range < s_range_min:
            print(f"Warning: get_rnnt_prune_ranges - got s_range={s_range} "
                  f"for boundaries S={boundary[:, 2]}, T={boundary[:, 3]}. "
                  f"Adjusting to {s_range_min}")
            s_range = s_range_min
    if s_range > S:
        s_range = S + 1
    if is_regular:
        assert s_range >= 2, (
            "Pruning range for standard RNN-T should be equal to or greater than 2, "
            "or no valid paths could survive pruning.")
    else:
        assert s_range >= 1, (
            "Pruning range for modified RNN-T should be equal to or greater than 1, "
            "or no valid paths could survive pruning.")

    sfx = _lib.suffix(px_grad.dtype)
    gx, gy = px_grad.detach().contiguous(), py_grad.detach().contiguous()
    bnd = boundary.contiguous()
    with torch.cuda.device(px_grad.device):
        ranges = torch.empty(B, T, int(s_range), dtype=torch.int64, device=px_grad.device)
        _lib.call("frnnt_prune_ranges_" + sfx, gx.data_ptr(), gy.data_ptr(), bnd.data_ptr(),
                  ranges.data_ptr(), B, S, T, int(not is_regular), int(s_range),
                  _lib.stream_of(px_grad))
    return ranges


class _PruneGather(torch.autograd.Function):
    """lm_pruned[b,t,j,:] = lm[b, ranges[b,t,j], :]: frnnt_prune_gather / _bwd."""

    @staticmethod
    def forward(ctx, lm, ranges):
        B, S1, C = lm.shape
        _, T, R = ranges.shape
        sfx = _lib.suffix(lm.dtype, narrow=True)
        lm_c, rng_c = lm.contiguous(), ranges.contiguous()
        with torch.cuda.device(lm.device):
            out = torch.empty(B, T, R, C, dtype=lm.dtype, device=lm.device)
            _lib.call("frnnt_prune_gather_" + sfx, lm_c.data_ptr(), rng_c.data_ptr(),
                      out.data_ptr(), B, S1 - 1, T, R, C, _lib.stream_of(lm))
        ctx.save_for_backward(rng_c)
        ctx.meta = (B, S1, T, R, C, sfx)
        return out

    @staticmethod
    def backward(ctx, grad):
        (rng,) = ctx.saved_tensors
        B, S1, T, R, C, sfx = ctx.meta
        grad = grad.contiguous()
        with torch.cuda.device(grad.device):
            lm_grad = torch.empty(B, S1, C, dtype=grad.dtype, device=grad.device)
            _lib.call("frnnt_prune_gather_bwd_" + sfx, grad.data_ptr(), rng.data_ptr(),
                      lm_grad.data_ptr(), B, S1 - 1, T, R, C, _lib.stream_of(grad))
        return lm_grad, None


def do_rnnt_pruning(am: Tensor, lm: Tensor, ranges: Tensor) -> Tuple[Tensor, Tensor]:
    """Prune encoder and predictor outputs with ``ranges`` (rnnt_loss.py:780-818).

    Returns ``(am_pruned, lm_pruned)``, both ``(B, T, s_range, C)``; ``am_pruned``
    is a zero-copy expanded view of ``am``, as in the reference.
    """
    assert ranges.shape[0] == am.shape[0], (ranges.shape[0], am.shape[0])
    assert ranges.shape[0] == lm.shape[0], (ranges.shape[0], lm.shape[0])
    assert am.shape[1] == ranges.shape[1], (am.shape[1], ranges.shape[1])
    (B, T, s_range) = ranges.shape
    (B, S1, C) = lm.shape
    _check_tensors([("am", am), ("lm", lm)], [("ranges", ranges)])
    am_pruning = am.unsqueeze(2).expand((B, T, s_range, C))
    lm_pruning = _PruneGather.apply(lm, ranges)
    return am_pruning, lm_pruning


_ACTIVATIONS = {None: 0, "none": 0, "tanh": 1}


class _PrunedJoinerInput(torch.autograd.Function):
    """act(am[b,t] + lm[b, ranges[b,t,j]]): frnnt_pruned_joiner_fwd / _bwd."""

    @staticmethod
    def forward(ctx, am, lm, ranges, activation):
        B, S1, C = lm.shape
        _, T, R = ranges.shape
        sfx = _lib.suffix(lm.dtype)
        am_c, lm_c, rng_c = am.contiguous(), lm.contiguous(), ranges.contiguous()
        with _on_device(lm.device):
            out = torch.empty(B, T, R, C, dtype=lm.dtype, device=lm.device)
            _lib.call("frnnt_pruned_joiner_fwd_" + sfx, am_c.data_ptr(), lm_c.data_ptr(),
                      rng_c.data_ptr(), out.data_ptr(), B, S1 - 1, T, R, C, activation,
                      _lib.stream_of(lm))
        ctx.save_for_backward(rng_c, out if activation else None)
        ctx.meta = (B, S1, T, R, C, activation, sfx)
        return out

    @staticmethod
    def backward(ctx, grad):
        rng, out = ctx.saved_tensors
        B, S1, T, R, C, activation, sfx = ctx.meta
        grad = grad.contiguous()
        with _on_device(grad.device):
            am_grad = (torch.empty(B, T, C, dtype=grad.dtype, device=grad.device)
                       if ctx.needs_input_grad[0] else None)
            lm_grad = (torch.empty(B, S1, C, dtype=grad.dtype, device=grad.device)
                       if ctx.needs_input_grad[1] else None)
            _lib.call("frnnt_pruned_joiner_bwd_" + sfx, grad.data_ptr(), _lib.ptr(out),
                      rng.data_ptr(), _lib.ptr(am_grad), _lib.ptr(lm_grad), B, S1 - 1, T, R, C,
                      activation, _lib.stream_of(grad))
        return am_grad, lm_grad, None, None


def pruned_joiner_input(am: Tensor, lm: Tensor, ranges: Tensor,
                        activation: Optional[str] = "tanh") -> Tensor:
    """``act(am_pruned + lm_pruned)`` of shape ``(B, T, s_range, C)`` in one pass.

    The usual joiner starts with ``tanh(am_pruned + lm_pruned)`` on the two tensors
    :func:`do_rnnt_pruning` returns (the reference's recipe, README.md:193-215, with
    rnnt_loss.py:780-818).  This op consumes ``ranges`` directly::

        out[b, t, j, :] = act(am[b, t, :] + lm[b, ranges[b, t, j], :])

    so the gathered copy ``lm_pruned`` (80 MB at B=32, T=250, s_range=5, C=500) is never
    written or read back, and the backward pass sums straight into ``am.grad`` and -- with
    the deterministic per-row segmented sum of the pruning gather's adjoint -- ``lm.grad``.
    ``activation`` is ``"tanh"`` or ``None`` (the plain sum).  It has no counterpart in the
    reference, whose callers obtain the same values with two more passes over
    ``(B, T, s_range, C)``; :func:`do_rnnt_pruning` stays as it is for them.
    """
    assert ranges.shape[0] == am.shape[0], (ranges.shape[0], am.shape[0])
    assert ranges.shape[0] == lm.shape[0], (ranges.shape[0], lm.shape[0])
    assert am.shape[1] == ranges.shape[1], (am.shape[1], ranges.shape[1])
    assert am.shape[2] == lm.shape[2], (am.shape[2], lm.shape[2])
    if activation not in _ACTIVATIONS:
        raise ValueError(f"activation should be ('tanh' | None), given {activation}")
    _check_tensors([("am", am), ("lm", lm)], [("ranges", ranges)])
    return _PrunedJoinerInput.apply(am, lm, ranges, _ACTIVATIONS[activation])


def _roll_by_shifts(src: Tensor, shifts: torch.LongTensor):
    """``out[b,t,s] = src[b,t,(s - shifts[b,t]) mod S]`` (rnnt_loss.py:821-853).
    The fused pruned-logprob kernel applies this roll itself; kept for callers."""
    assert src.dim() == 3, src.dim()
    (B, T, S) = src.shape
    assert shifts.shape == (B, T), shifts.shape
    index = (torch.arange(S, device=src.device).view(1, 1, S) - shifts.reshape(B, T, 1)) % S
    return torch.gather(src, 2, index)


def _pruned_logprobs(logits, symbols, ranges, termination_symbol, boundary, rnnt_type,
                     window_only):
    assert logits.ndim == 4, logits.ndim
    (B, T, s_range, C) = logits.shape
    assert ranges.shape == (B, T, s_range), f"{ranges.shape} == ({B}, {T}, {s_range})"
    (B, S) = symbols.shape
    assert rnnt_type in ["regular", "modified", "constrained"], rnnt_type
    on_device = bool(window_only) and _device_checks(rnnt_type, boundary) != 0
    validate_st_lengths(S, T, rnnt_type == "regular", boundary, on_device=on_device)
    _check_tensors([("logits", logits)],
                   [("symbols", symbols), ("ranges", ranges), ("boundary", boundary)])
    if window_only and boundary is not None:
        _assert_boundary(boundary, B, S, T, on_device=on_device)
    return _LatticeLogprobs.apply(logits, symbols, ranges, boundary, termination_symbol,
                                  rnnt_type, window_only)


def get_rnnt_logprobs_pruned(
    logits: Tensor, symbols: Tensor, ranges: Tensor, termination_symbol: int,
    boundary: Optional[Tensor] = None, rnnt_type: str = "regular",
) -> Tuple[Tensor, Tensor]:
    """(px, py) from pruned joiner logits ``(B, T, s_range, C)`` and the
    ``ranges`` they were computed for (rnnt_loss.py:856-1024); lattice cells
    outside the kept range of their frame are -inf."""
    return _pruned_logprobs(logits, symbols, ranges, termination_symbol, boundary, rnnt_type,
                            False)


def rnnt_loss_pruned(
    logits: Tensor, symbols: Tensor, ranges: Tensor, termination_symbol: int,
    boundary: Optional[Tensor] = None, rnnt_type: str = "regular",
    delay_penalty: float = 0.0, reduction: Optional[str] = "mean", return_grad: bool = False,
) -> Tensor:
    """The pruned RNN-T loss on joiner logits ``(B, T, s_range, C)`` (rnnt_loss.py:1027-1132).
    As in :func:`rnnt_loss`, logits outside an utterance's boundary window are not read."""
    px, py = _pruned_logprobs(logits, symbols, ranges, termination_symbol, boundary, rnnt_type,
                              True)
    return _recursion_and_reduce(px, py, boundary, rnnt_type, delay_penalty, reduction,
                                 return_grad)


class _SmoothedCombine(torch.autograd.Function):
    """Interpolation of the joint (px, py) with the lm-only and am-only models
    (rnnt_loss.py:1264-1355): frnnt_smoothed_logprobs_fwd/bwd."""

    @staticmethod
    def forward(ctx, pxj, pyj, lm, am, symbols, boundary, termination_symbol, regular, k_lm,
                k_am):
        # boundary (regular lattice): px[b, :, t_end] = -inf, the reference's
        # fix_for_boundary after the interpolation (rnnt_loss.py:1364-1365); backward() lets
        # no gradient through those cells, as the scatter_ there does (the recursion leaves
        # 1 in px_grad at them when the lattice has no path at all)
        B, T, C = am.shape
        S = lm.shape[1] - 1
        sfx = _lib.suffix(am.dtype)
        lm_c, am_c, sym_c = lm.contiguous(), am.contiguous(), symbols.contiguous()
        pxj_c, pyj_c = pxj.contiguous(), pyj.contiguous()
        bnd_c = boundary.contiguous() if (boundary is not None and regular) else None
        opts = dict(dtype=am.dtype, device=am.device)
        n_lm, n_am = B * (S + 1), B * T
        # kept for the backward: lm_max | lm_sum | am_max | am_z | unigram
        (o_lmx, o_lms, o_amx, o_amz, o_u), total = _carve([n_lm, n_lm, n_am, n_am, C])
        with _on_device(am.device):
            px = torch.empty_like(pxj_c)
            py = torch.empty_like(pyj_c)
            stats = torch.empty(total, **opts)
            partial = torch.empty((n_lm + 15) // 16 * C, **opts)
            base, item = stats.data_ptr(), stats.element_size()
            _lib.call("frnnt_smoothed_logprobs_fwd_" + sfx, lm_c.data_ptr(), am_c.data_ptr(),
                      sym_c.data_ptr(), _lib.ptr(bnd_c), pxj_c.data_ptr(), pyj_c.data_ptr(),
                      px.data_ptr(),
                      py.data_ptr(), base + o_lmx * item, base + o_lms * item,
                      base + o_amx * item, base + o_amz * item, base + o_u * item,
                      partial.data_ptr(), B, S, T, C, int(termination_symbol), int(regular),
                      k_lm, k_am, _lib.stream_of(am))
        ctx.save_for_backward(lm_c, am_c, sym_c, stats)
        ctx.masked_at = bnd_c
        ctx.meta = (B, S, T, C, int(termination_symbol), int(regular), k_lm, k_am, sfx,
                    (o_lmx, o_lms, o_amx, o_amz, o_u))
        return px, py

    @staticmethod
    def backward(ctx, gpx, gpy):
        lm, am, sym, stats = ctx.saved_tensors
        B, S, T, C, term, regular, k_lm, k_am, sfx, (o_lmx, o_lms, o_amx, o_amz, o_u) = ctx.meta
        opts = dict(dtype=am.dtype, device=am.device)
        T1 = T + 1 if regular else T
        n_lm, n_am = B * (S + 1), B * T
        with _on_device(am.device):
            gpx = torch.zeros(B, S, T1, **opts) if gpx is None else gpx.contiguous()
            gpy = torch.zeros(B, S + 1, T, **opts) if gpy is None else gpy.contiguous()
            gxj, gyj = torch.empty_like(gpx), torch.empty_like(gpy)
            lm_grad, am_grad = torch.empty_like(lm), torch.empty_like(am)
            # scratch: row_x | row_y | col_y | col_g | g_unigram | partial
            (o_rx, o_ry, o_cy, o_cg, o_gu, o_p), total = _carve(
                [n_lm, n_lm, n_am, n_am, C, (n_am + 15) // 16 * C])
            scratch = torch.empty(total, **opts)
            sb, wb, item = scratch.data_ptr(), stats.data_ptr(), stats.element_size()
            _lib.call("frnnt_smoothed_logprobs_bwd_" + sfx, lm.data_ptr(), am.data_ptr(),
                      sym.data_ptr(), _lib.ptr(ctx.masked_at), wb + o_lmx * item,
                      wb + o_lms * item, wb + o_amx * item,
                      wb + o_amz * item, wb + o_u * item, gpx.data_ptr(), gpy.data_ptr(),
                      gxj.data_ptr(), gyj.data_ptr(), lm_grad.data_ptr(), am_grad.data_ptr(),
                      sb + o_rx * item, sb + o_ry * item, sb + o_cy * item, sb + o_cg * item,
                      sb + o_gu * item, sb + o_p * item, B, S, T, C, term, regular, k_lm, k_am,
                      _lib.stream_of(am))
        return gxj, gyj, lm_grad, am_grad, None, None, None, None, None, None


def get_rnnt_logprobs_smoothed(
    lm: Tensor, am: Tensor, symbols: Tensor, termination_symbol: int,
    lm_only_scale: float = 0.1, am_only_scale: float = 0.1,
    boundary: Optional[Tensor] = None, rnnt_type: str = "regular",
) -> Tuple[Tensor, Tensor]:
    """(px, py) interpolating the joint model with an lm-only and an am-only
    (unigram-lm) model (rnnt_loss.py:1135-1369)::

        (1 - lm_only_scale - am_only_scale) * joint + lm_only_scale * lm_only
                                                    + am_only_scale * am_only

    The joint part -- the [B,S+1,C] x [B,C,T] contraction and its px / py -- comes
    from the fused MFMA kernel; the lm-only / am-only models, the unigram over the
    whole batch and the interpolation come from frnnt_smoothed_logprobs_fwd/bwd.
    """
    return _smoothed_logprobs(lm, am, symbols, termination_symbol, lm_only_scale,
                              am_only_scale, boundary, rnnt_type, False)


def _smoothed_logprobs(lm, am, symbols, termination_symbol, lm_only_scale, am_only_scale,
                       boundary, rnnt_type, from_loss):
    # from_loss: the recursion that follows tests the boundary rows on the device
    assert lm.ndim == 3, lm.ndim
    assert am.ndim == 3, am.ndim
    assert lm.shape[0] == am.shape[0], (lm.shape[0], am.shape[0])
    assert lm.shape[2] == am.shape[2], (lm.shape[2], am.shape[2])
    (B, T, C) = am.shape
    S = lm.shape[1] - 1
    assert symbols.shape == (B, S), symbols.shape
    assert rnnt_type in ["regular", "modified", "constrained"], rnnt_type
    validate_st_lengths(S, T, rnnt_type == "regular", boundary,
                        on_device=from_loss and _device_checks(rnnt_type, boundary) != 0)
    _check_tensors([("am", am), ("lm", lm)], [("symbols", symbols), ("boundary", boundary)])

    lm, am = _widen(lm, am)
    # joint part, without the boundary / constrained post-processing (applied last)
    base_type = "regular" if rnnt_type == "regular" else "modified"
    px, py = _SimpleLogprobs.apply(lm, am, symbols, None, termination_symbol, base_type)

    # exact zeros would turn -inf * 0 into nan
    if lm_only_scale == 0.0:
        lm_only_scale = 1.0e-20
    if am_only_scale == 0.0:
        am_only_scale = 1.0e-20
    # fix_for_boundary (rnnt_loss.py:1364-1365) happens inside the node for the regular
    # lattice: its forward kernel writes the -inf of px[b, :, t_end], its backward kernels let
    # no gradient through those cells -- what the reference's in-place scatter_ does in both
    # directions, without the three launches and the index tensor.
    px_interp, py_interp = _SmoothedCombine.apply(
        px, py, lm, am, symbols, boundary if rnnt_type == "regular" else None,
        termination_symbol, rnnt_type == "regular", float(lm_only_scale), float(am_only_scale))

    if rnnt_type == "constrained":
        px_interp += py_interp[:, 1:, :]
    return (px_interp, py_interp)


def rnnt_loss_smoothed(
    lm: Tensor, am: Tensor, symbols: Tensor, termination_symbol: int,
    lm_only_scale: float = 0.1, am_only_scale: float = 0.1,
    boundary: Optional[Tensor] = None, rnnt_type: str = "regular",
    delay_penalty: float = 0.0, reduction: Optional[str] = "mean", return_grad: bool = False,
) -> Union[Tuple[Tensor, Tuple[Tensor, Tensor]], Tensor]:
    """rnnt_loss_simple with lm-only / am-only smoothing (rnnt_loss.py:1372-1494)."""
    px, py = _smoothed_logprobs(lm, am, symbols, termination_symbol, lm_only_scale,
                                am_only_scale, boundary, rnnt_type, True)
    return _recursion_and_reduce(px, py, boundary, rnnt_type, delay_penalty, reduction,
                                 return_grad)
