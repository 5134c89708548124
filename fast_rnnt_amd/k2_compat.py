"""The names under which k2 ships these same functions (the reference's README.md:4: "There
is also a fast RNN-T loss implementation in k2 project, which shares the same code here"),
for recipes written against ``k2.rnnt_loss_pruned`` and friends::

    import fast_rnnt_amd.k2_compat as k2
    simple_loss, (px_grad, py_grad) = k2.rnnt_loss_smoothed(..., return_grad=True)
    ranges = k2.get_rnnt_prune_ranges(px_grad, py_grad, boundary, s_range)
    am_pruned, lm_pruned = k2.do_rnnt_pruning(am, lm, ranges)
    pruned_loss = k2.rnnt_loss_pruned(logits, symbols, ranges, termination_symbol, boundary)

Only the RNN-T loss functions exist here (k2's FSA machinery is not part of this path), and
this module is never installed as a top-level ``k2``.  Signatures, defaults and return values
are those of fast_rnnt/python/fast_rnnt/rnnt_loss.py and mutual_information.py, which k2's
python/k2/rnnt_loss.py and mutual_information.py mirror.
"""
from .mutual_information import (joint_mutual_information_recursion,  # noqa: F401
                                 mutual_information_recursion)
from .rnnt_loss import (do_rnnt_pruning, get_rnnt_logprobs,  # noqa: F401
                        get_rnnt_logprobs_joint, get_rnnt_logprobs_pruned,
                        get_rnnt_logprobs_smoothed, get_rnnt_prune_ranges, rnnt_loss,
                        rnnt_loss_pruned, rnnt_loss_simple, rnnt_loss_smoothed)

__all__ = [
    "do_rnnt_pruning", "get_rnnt_logprobs", "get_rnnt_logprobs_joint",
    "get_rnnt_logprobs_pruned", "get_rnnt_logprobs_smoothed", "get_rnnt_prune_ranges",
    "joint_mutual_information_recursion", "mutual_information_recursion", "rnnt_loss",
    "rnnt_loss_pruned", "rnnt_loss_simple", "rnnt_loss_smoothed",
]
