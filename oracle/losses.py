"""torch-CPU restatement of the RNN-T loss layer (TEST INFRASTRUCTURE ONLY).

Follows fast_rnnt/python/fast_rnnt/rnnt_loss.py function by function; the
arithmetic order of every floating-point expression is the reference's (that is
what decides rounding), the indexing is written with direct advanced indexing
and masks instead of the reference's gather / cat / roll chains.

  lattice_logprobs_simple    <- get_rnnt_logprobs           rnnt_loss.py:66-227
  lattice_logprobs_smoothed  <- get_rnnt_logprobs_smoothed  rnnt_loss.py:1135-1369
  lattice_logprobs_joint     <- get_rnnt_logprobs_joint     rnnt_loss.py:343-449
  lattice_logprobs_pruned    <- get_rnnt_logprobs_pruned    rnnt_loss.py:856-1024
  monotonic_lower_bound      <- _monotonic_lower_bound      rnnt_loss.py:550-581
  adjust_lower_bound         <- _adjust_pruning_lower_bound rnnt_loss.py:584-632
  prune_ranges               <- get_rnnt_prune_ranges       rnnt_loss.py:638-777
  prune                      <- do_rnnt_pruning             rnnt_loss.py:780-818
  roll_rows                  <- _roll_by_shifts             rnnt_loss.py:821-853
  loss_simple / loss_smoothed / loss_pruned / loss_joint
                             <- rnnt_loss_simple :230, rnnt_loss_smoothed :1372,
                                rnnt_loss_pruned :1027, rnnt_loss :452
"""
from typing import Optional, Tuple

import torch
from torch import Tensor

from .recursion import mutual_information_recursion

_TYPES = ("regular", "modified", "constrained")
NEG_INF = float("-inf")


def check_lengths(S: int, T: int, regular: bool, boundary: Optional[Tensor]) -> None:
    """rnnt_loss.py:25-42."""
    if boundary is None:
        assert S >= 1, S
        assert regular or T >= S, (T, S)
    else:
        assert bool((boundary[:, 2] >= 1).all()), boundary[:, 2]
        assert regular or bool((boundary[:, 3] >= boundary[:, 2]).all())


def _mask_last_frame(px: Tensor, boundary: Optional[Tensor]) -> Tensor:
    """rnnt_loss.py:45-63: px[b, :, T_b] = -inf (regular lattices only)."""
    if boundary is None:
        return px
    B, S, T1 = px.shape
    cols = torch.arange(T1).reshape(1, 1, T1)
    hit = cols == boundary[:, 3].reshape(B, 1, 1)
    return px.masked_fill_(hit.expand(B, S, T1), NEG_INF)


def _append_neg_inf_column(x: Tensor) -> Tensor:
    B, S, _ = x.shape
    return torch.cat((x, x.new_full((B, S, 1), NEG_INF)), dim=2)


def _joint_normalizers(lm: Tensor, am: Tensor):
    """Shared head of rnnt_loss.py:174-186 and :1262-1296."""
    am_max = am.max(dim=2, keepdim=True)[0]
    lm_max = lm.max(dim=2, keepdim=True)[0]
    am_probs = (am - am_max).exp()
    lm_probs = (lm - lm_max).exp()
    tiny = torch.finfo(am_probs.dtype).tiny
    norm = (torch.matmul(lm_probs, am_probs.transpose(1, 2)) + tiny).log()
    return am_max, lm_max, am_probs, lm_probs, norm


def lattice_logprobs_simple(lm, am, symbols, termination_symbol,
                            rnnt_type="regular", boundary=None) -> Tuple[Tensor, Tensor]:
    assert lm.ndim == 3 and am.ndim == 3
    assert lm.shape[0] == am.shape[0] and lm.shape[2] == am.shape[2]
    B, T, C = am.shape
    S = lm.shape[1] - 1
    assert symbols.shape == (B, S)
    check_lengths(S, T, rnnt_type == "regular", boundary)
    assert rnnt_type in _TYPES, rnnt_type

    am_max, lm_max, _, _, norm = _joint_normalizers(lm, am)
    norm = norm + lm_max + am_max.transpose(1, 2)  # [B,S+1,T]

    rows = torch.arange(B).reshape(B, 1)
    px_am = am[rows, :, symbols]  # [B,S,T] = am[b, t, symbols[b,s]]
    if rnnt_type == "regular":
        px_am = _append_neg_inf_column(px_am)
    px_lm = lm[rows, torch.arange(S).reshape(1, S), symbols].unsqueeze(2)  # [B,S,1]
    px = px_am + px_lm
    px[:, :, :T] -= norm[:, :S, :]

    py = am[:, :, termination_symbol].unsqueeze(1) + lm[:, :, termination_symbol].unsqueeze(2) - norm

    if rnnt_type == "regular":
        px = _mask_last_frame(px, boundary)
    elif rnnt_type == "constrained":
        px += py[:, 1:, :]
    return px, py


def lattice_logprobs_smoothed(lm, am, symbols, termination_symbol, lm_only_scale=0.1,
                              am_only_scale=0.1, boundary=None,
                              rnnt_type="regular") -> Tuple[Tensor, Tensor]:
    assert lm.ndim == 3 and am.ndim == 3
    assert lm.shape[0] == am.shape[0] and lm.shape[2] == am.shape[2]
    B, T, C = am.shape
    S = lm.shape[1] - 1
    assert symbols.shape == (B, S)
    check_lengths(S, T, rnnt_type == "regular", boundary)
    assert rnnt_type in _TYPES, rnnt_type

    am_max, lm_max, am_probs, lm_probs, norm = _joint_normalizers(lm, am)
    tiny = torch.finfo(lm_probs.dtype).tiny

    lm_row_sum = lm_probs.sum(dim=2, keepdim=True)  # [B,S+1,1]
    # mean over every (b, s) row, padding rows included (:1278-1281)
    unigram = torch.mean(lm_probs / lm_row_sum, dim=(0, 1), keepdim=True) + tiny  # [1,1,C]
    am_only_norm = (torch.mv(am_probs.reshape(-1, C), unigram.reshape(C))
                    .reshape(B, T, 1).log() + am_max).transpose(1, 2)  # [B,1,T]
    unigram = unigram.log()
    lm_only_norm = lm_row_sum.log() + lm_max  # [B,S+1,1]
    norm = norm + lm_max + am_max.transpose(1, 2)

    rows = torch.arange(B).reshape(B, 1)
    px_am = am[rows, :, symbols]
    if rnnt_type == "regular":
        px_am = _append_neg_inf_column(px_am)
    px_lm = lm[rows, torch.arange(S).reshape(1, S), symbols].unsqueeze(2)
    px_lm_unigram = unigram.reshape(C)[symbols].unsqueeze(2)  # [B,S,1]

    px = px_am + px_lm
    px[:, :, :T] -= norm[:, :S, :]
    px_amonly = px_am + px_lm_unigram
    px_amonly[:, :, :T] -= am_only_norm
    px_lmonly = px_lm - lm_only_norm[:, :S, :]

    py_am = am[:, :, termination_symbol].unsqueeze(1)
    py_lm = lm[:, :, termination_symbol].unsqueeze(2)
    py = py_am + py_lm - norm
    py_amonly = py_am + unigram[0][0][termination_symbol] - am_only_norm
    py_lmonly = py_lm - lm_only_norm

    combined = 1.0 - lm_only_scale - am_only_scale
    # exact zeros would turn (-inf * 0) into nan (:1346-1351)
    if lm_only_scale == 0.0:
        lm_only_scale = 1.0e-20
    if am_only_scale == 0.0:
        am_only_scale = 1.0e-20
    px_mix = px * combined + px_lmonly * lm_only_scale + px_amonly * am_only_scale
    py_mix = py * combined + py_lmonly * lm_only_scale + py_amonly * am_only_scale

    if rnnt_type == "regular":
        px_mix = _mask_last_frame(px_mix, boundary)
    elif rnnt_type == "constrained":
        px_mix += py_mix[:, 1:, :]
    return px_mix, py_mix


def lattice_logprobs_joint(logits, symbols, termination_symbol, boundary=None,
                           rnnt_type="regular") -> Tuple[Tensor, Tensor]:
    assert logits.ndim == 4
    B, T, S1, C = logits.shape
    S = S1 - 1
    assert symbols.shape == (B, S)
    check_lengths(S, T, rnnt_type == "regular", boundary)
    assert rnnt_type in _TYPES, rnnt_type

    norm = torch.logsumexp(logits, dim=3).permute(0, 2, 1)  # [B,S+1,T]
    rows = torch.arange(B).reshape(B, 1, 1)
    srange = torch.arange(S).reshape(1, 1, S)
    trange = torch.arange(T).reshape(1, T, 1)
    px = logits[rows, trange, srange, symbols.reshape(B, 1, S)].permute(0, 2, 1)  # [B,S,T]
    if rnnt_type == "regular":
        px = _append_neg_inf_column(px)
    else:
        px = px.clone()
    px[:, :, :T] -= norm[:, :S, :]
    py = logits[:, :, :, termination_symbol].permute(0, 2, 1).clone()
    py -= norm
    if rnnt_type == "regular":
        px = _mask_last_frame(px, boundary)
    elif rnnt_type == "constrained":
        px += py[:, 1:, :]
    return px, py


def roll_rows(src: Tensor, shifts: Tensor) -> Tensor:
    """out[b,t,s] = src[b,t,(s - shifts[b,t]) mod S'] (rnnt_loss.py:821-853)."""
    assert src.dim() == 3
    B, T, S = src.shape
    assert shifts.shape == (B, T)
    pos = (torch.arange(S).reshape(1, 1, S) - shifts.reshape(B, T, 1)) % S
    return torch.gather(src, 2, pos)


def lattice_logprobs_pruned(logits, symbols, ranges, termination_symbol, boundary=None,
                            rnnt_type="regular") -> Tuple[Tensor, Tensor]:
    assert logits.ndim == 4
    B, T, R, C = logits.shape
    assert ranges.shape == (B, T, R)
    B, S = symbols.shape
    check_lengths(S, T, rnnt_type == "regular", boundary)
    assert rnnt_type in _TYPES, rnnt_type

    norm = torch.logsumexp(logits, dim=3)  # [B,T,R]
    sym_ext = torch.cat((symbols, symbols.new_full((B, 1), termination_symbol)), dim=1)
    picked = sym_ext[torch.arange(B).reshape(B, 1, 1), ranges]  # [B,T,R]
    px = torch.gather(logits, 3, picked.unsqueeze(3)).squeeze(3) - norm
    filler = px.new_full((B, T, S + 1 - R), NEG_INF)
    px = roll_rows(torch.cat((px, filler), dim=2), ranges[:, :, 0])[:, :, :S]
    px = px.permute(0, 2, 1)
    if rnnt_type == "regular":
        px = _append_neg_inf_column(px)
    py = logits[:, :, :, termination_symbol].clone() - norm
    py = roll_rows(torch.cat((py, filler), dim=2), ranges[:, :, 0]).permute(0, 2, 1)
    if rnnt_type == "regular":
        px = _mask_last_frame(px, boundary)
    elif rnnt_type == "constrained":
        px += py[:, 1:, :]
    return px, py


def monotonic_lower_bound(x: Tensor) -> Tensor:
    """Suffix minimum along the last axis (rnnt_loss.py:550-581)."""
    return torch.flip(torch.cummin(torch.flip(x, dims=(-1,)), dim=-1)[0], dims=(-1,))


def adjust_lower_bound(s_begin: Tensor, r: int) -> Tensor:
    """rnnt_loss.py:584-632: make s_begin non-decreasing with steps < r, start 0."""
    B, T = s_begin.shape
    ramp = (r - 1) * torch.arange(T)
    y = ramp - monotonic_lower_bound(s_begin)
    y = torch.clamp(monotonic_lower_bound(y), min=0)
    return ramp - y


def window_sums_in_torch_cpu_order(py_grad: Tensor, n: int, width: int) -> Tensor:
    """sum_j py_grad[:, s + j, :] for s < n, j < width, added in the order of ATen's CPU
    loop for a sum over a strided axis whose neighbour axis is contiguous
    (aten/src/ATen/native/cpu/SumKernel.cpp, multi_row_sum): left to right in stretches of
    16 into a first accumulator, which is added to a second after every stretch, that one
    to a third after 16 stretches and to a fourth after 256, the remainder left to right,
    and at the end the four added in order.  Up to 16 values this is plain left to right.
    torch.sum itself deviates from this for the last few output elements of each chunk
    of its loop (those that do not fill four SIMD vectors are summed as four interleaved
    partial sums), so which elements those are depends on the host's SIMD width and
    thread count."""
    B, _, T = py_grad.shape
    zero = py_grad.new_zeros(B, n, T)
    acc = [zero.clone() for _ in range(4)]
    i = 0
    while i + 16 <= width:
        for _ in range(16):
            acc[0] = acc[0] + py_grad[:, i:i + n, :]
            i += 1
        for level in range(1, 4):
            acc[level] = acc[level] + acc[level - 1]
            acc[level - 1] = zero.clone()
            if i & (0xF << (4 * level)):
                break
    while i < width:
        acc[0] = acc[0] + py_grad[:, i:i + n, :]
        i += 1
    return ((acc[0] + acc[1]) + acc[2]) + acc[3]


def prune_ranges(px_grad, py_grad, boundary, s_range: int, window_sum: str = "torch") -> Tensor:
    """rnnt_loss.py:638-777.  ``window_sum='torch'`` reduces the strided window
    view with torch.sum exactly as the reference does (:726-734);
    ``'ltr'`` adds the window rows strictly left to right in the input dtype;
    ``'cascade'`` is window_sums_in_torch_cpu_order, the host-independent restatement of
    what torch.sum does there."""
    B, S, T1 = px_grad.shape
    T = py_grad.shape[-1]
    regular = T1 != T
    assert T1 in (T, T + 1)
    assert py_grad.shape == (B, S + 1, T)
    assert boundary.shape == (B, 4)
    check_lengths(S, T, regular, boundary)
    if regular:
        need = int((boundary[:, 2] - 1).div(boundary[:, 3], rounding_mode="trunc").add(2).max())
        if s_range < need:
            print(f"Warning: get_rnnt_prune_ranges - got s_range={s_range} "
                  f"for boundaries S={boundary[:, 2]}, T={boundary[:, 3]}. Adjusting to {need}")
            s_range = need
    if s_range > S:
        s_range = S + 1
    assert s_range >= (2 if regular else 1)
    n = S + 2 - s_range  # number of candidate window starts
    if window_sum == "torch":
        sb, ss, st = py_grad.stride()
        win = torch.as_strided(py_grad, (B, n, s_range, T), (sb, ss, ss, st))
        blk = torch.sum(win, axis=2)
    elif window_sum == "cascade":
        blk = window_sums_in_torch_cpu_order(py_grad, n, s_range)
    else:
        blk = py_grad[:, 0:n, :].clone()
        for j in range(1, s_range):
            blk = blk + py_grad[:, j:j + n, :]
    below = torch.cat((px_grad.new_zeros(B, 1, T1), px_grad), dim=1)[:, :n, :T]
    score = blk - below
    s_begin = torch.argmax(score, dim=1)  # first maximum, [B,T]
    live = torch.arange(T).reshape(1, T) < (boundary[:, 3].reshape(B, 1) - 1)
    tail = torch.clamp(boundary[:, 2].reshape(B, 1) - s_range + 1, min=0)
    s_begin = torch.where(live, s_begin, tail.expand(B, T))
    s_begin = adjust_lower_bound(s_begin, s_range if regular else 2)
    return s_begin.reshape(B, T, 1) + torch.arange(s_range).reshape(1, 1, s_range)


def prune(am: Tensor, lm: Tensor, ranges: Tensor) -> Tuple[Tensor, Tensor]:
    """rnnt_loss.py:780-818."""
    assert ranges.shape[0] == am.shape[0] == lm.shape[0]
    assert am.shape[1] == ranges.shape[1]
    B, T, R = ranges.shape
    C = lm.shape[2]
    am_p = am.unsqueeze(2).expand(B, T, R, C)
    lm_p = lm[torch.arange(B).reshape(B, 1, 1), ranges]  # [B,T,R,C]
    return am_p, lm_p


def _finish(px, py, boundary, rnnt_type, delay_penalty, reduction, return_grad):
    """Common tail of the four loss wrappers (e.g. rnnt_loss.py:309-340)."""
    if delay_penalty > 0.0:
        B, S, T0 = px.shape
        T = T0 if rnnt_type != "regular" else T0 - 1
        if boundary is None:
            offset = torch.tensor((T - 1) / 2, dtype=px.dtype).expand(B, 1, 1)
        else:
            offset = (boundary[:, 3] - 1) / 2
        penalty = offset.reshape(B, 1, 1) - torch.arange(T0).reshape(1, 1, T0)
        penalty = penalty * delay_penalty
        px += penalty.to(px.dtype)
    out = mutual_information_recursion(px=px, py=py, boundary=boundary, return_grad=return_grad)
    scores = out[0] if return_grad else out
    if reduction == "none":
        loss = -scores
    elif reduction == "mean":
        loss = -torch.mean(scores)
    elif reduction == "sum":
        loss = -torch.sum(scores)
    else:
        raise ValueError(f"reduction should be ('none' | 'mean' | 'sum'), given {reduction}")
    return (loss, out[1]) if return_grad else loss


def loss_simple(lm, am, symbols, termination_symbol, boundary=None, rnnt_type="regular",
                delay_penalty=0.0, reduction="mean", return_grad=False):
    px, py = lattice_logprobs_simple(lm, am, symbols, termination_symbol,
                                     rnnt_type=rnnt_type, boundary=boundary)
    return _finish(px, py, boundary, rnnt_type, delay_penalty, reduction, return_grad)


def loss_smoothed(lm, am, symbols, termination_symbol, lm_only_scale=0.1, am_only_scale=0.1,
                  boundary=None, rnnt_type="regular", delay_penalty=0.0, reduction="mean",
                  return_grad=False):
    px, py = lattice_logprobs_smoothed(lm, am, symbols, termination_symbol, lm_only_scale,
                                       am_only_scale, boundary=boundary, rnnt_type=rnnt_type)
    return _finish(px, py, boundary, rnnt_type, delay_penalty, reduction, return_grad)


def loss_pruned(logits, symbols, ranges, termination_symbol, boundary=None,
                rnnt_type="regular", delay_penalty=0.0, reduction="mean", return_grad=False):
    px, py = lattice_logprobs_pruned(logits, symbols, ranges, termination_symbol,
                                     boundary=boundary, rnnt_type=rnnt_type)
    return _finish(px, py, boundary, rnnt_type, delay_penalty, reduction, return_grad)


def loss_joint(logits, symbols, termination_symbol, boundary=None, rnnt_type="regular",
               delay_penalty=0.0, reduction="mean", return_grad=False):
    px, py = lattice_logprobs_joint(logits, symbols, termination_symbol,
                                    boundary=boundary, rnnt_type=rnnt_type)
    return _finish(px, py, boundary, rnnt_type, delay_penalty, reduction, return_grad)
