"""fast_rnnt on MI355X: the loss hot path of k2-fsa/fast_rnnt as gfx950 kernels.

The export list is the reference's (fast_rnnt/python/fast_rnnt/__init__.py:1-15).
"""
# The reference's version (CMakeLists.txt:50, written into the package by setup.py:100-103)
# with a local label for this build.
__version__ = "1.2+mi355x"

from ._fast_rnnt import with_cuda

from .mutual_information import mutual_information_recursion
from .mutual_information import joint_mutual_information_recursion

from .rnnt_loss import do_rnnt_pruning
from .rnnt_loss import get_rnnt_logprobs
from .rnnt_loss import get_rnnt_logprobs_joint
from .rnnt_loss import get_rnnt_logprobs_pruned
from .rnnt_loss import get_rnnt_logprobs_smoothed
from .rnnt_loss import get_rnnt_prune_ranges
from .rnnt_loss import rnnt_loss
from .rnnt_loss import rnnt_loss_pruned
from .rnnt_loss import rnnt_loss_simple
from .rnnt_loss import rnnt_loss_smoothed

# beyond the reference's export list: the joiner's input without the gathered copy, and
# where the rows of a boundary tensor are asserted (on the device, raised later, by default)
from .rnnt_loss import pruned_joiner_input
from .mutual_information import check_boundaries, set_boundary_checks
