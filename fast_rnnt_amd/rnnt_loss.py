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

import torch
from torch import Tensor

from . import _lib
from .mutual_information import mutual_information_recursion

_RNNT_TYPES = {"regular": 0, "modified": 1, "constrained": 2}


def validate_st_lengths(S: int, T: int, is_rnnt_type_regular: bool,
                        boundary: Optional[Tensor] = None):
    """fast_rnnt/python/fast_rnnt/rnnt_loss.py:25-42."""
    if boundary is None:
        assert S >= 1, S
        assert is_rnnt_type_regular or T >= S, \
            f"Modified transducer requires T >= S, but got T={T} and S={S}"
    else:
        Ss = boundary[:, 2]
        Ts = boundary[:, 3]
        assert (Ss >= 1).all(), Ss
        assert is_rnnt_type_regular or (Ts >= Ss).all(), \
            f"Modified transducer requires T >= S, but got T={Ts} and S={Ss}"


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
                      int(termination_symbol), kind, _lib.stream_of(am))
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
            dmat = torch.empty(B, S + 1, T, **opts)
            row_x = torch.empty(B, S + 1, **opts)
            row_y = torch.empty(B, S + 1, **opts)
            col_y = torch.empty(B, T, **opts)
            lm_grad = torch.empty_like(lm) if ctx.needs_input_grad[0] else None
            am_grad = torch.empty_like(am) if ctx.needs_input_grad[1] else None
            _lib.call("frnnt_simple_logprobs_bwd_" + sfx, lm.data_ptr(), am.data_ptr(),
                      sym.data_ptr(), _lib.ptr(bnd), lm_max.data_ptr(), am_max.data_ptr(),
                      norm_raw.data_ptr(), gpx.data_ptr(), gpy.data_ptr(), dmat.data_ptr(),
                      row_x.data_ptr(), row_y.data_ptr(), col_y.data_ptr(), _lib.ptr(lm_grad),
                      _lib.ptr(am_grad), B, S, T, C, term, kind, _lib.stream_of(am))
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
    assert lm.dtype == am.dtype, (lm.dtype, am.dtype)
    _require_gpu(lm, am, symbols, boundary)
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


def _recursion_and_reduce(px, py, boundary, rnnt_type, delay_penalty, reduction, return_grad):
    """Shared tail of the four losses (e.g. rnnt_loss.py:309-340)."""
    if delay_penalty > 0.0:
        _apply_delay_penalty(px, boundary, rnnt_type, delay_penalty)
    scores_and_grads = mutual_information_recursion(
        px=px, py=py, boundary=boundary, return_grad=return_grad)
    negated_loss = scores_and_grads[0] if return_grad else scores_and_grads
    if reduction == "none":
        loss = -negated_loss
    elif reduction == "mean":
        loss = -torch.mean(negated_loss)
    elif reduction == "sum":
        loss = -torch.sum(negated_loss)
    else:
        raise ValueError(f"reduction should be ('none' | 'mean' | 'sum'), given {reduction}")
    return (loss, scores_and_grads[1]) if return_grad else loss


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
    px, py = get_rnnt_logprobs(lm=lm, am=am, symbols=symbols,
                               termination_symbol=termination_symbol,
                               boundary=boundary, rnnt_type=rnnt_type)
    return _recursion_and_reduce(px, py, boundary, rnnt_type, delay_penalty, reduction,
                                 return_grad)
