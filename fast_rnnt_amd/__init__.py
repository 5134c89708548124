"""fast_rnnt on MI355X: the loss hot path of k2-fsa/fast_rnnt as gfx950 kernels.

The export list is the reference's (fast_rnnt/python/fast_rnnt/__init__.py:1-15).
"""
from ._fast_rnnt import with_cuda

from .mutual_information import mutual_information_recursion
from .mutual_information import joint_mutual_information_recursion

from .rnnt_loss import get_rnnt_logprobs
from .rnnt_loss import rnnt_loss_simple
