"""MI355X-native implementation of k2's RNN-T mutual-information path.

Exports the same names as ``import k2`` does for this path
(k2/python/k2/__init__.py:79-80,98-108), so ``import k2_amd as k2`` drops in for
``mutual_information_recursion``, ``rnnt_loss_simple``, ``get_rnnt_prune_ranges``,
``do_rnnt_pruning``, ``rnnt_loss_pruned``, ``rnnt_loss`` and their log-prob builders.
"""
from .lattice import pruned_ranges_to_lattice
from .mutual_information import joint_mutual_information_recursion
from .mutual_information import mutual_information_recursion
from .rnnt_loss import do_rnnt_pruning
from .rnnt_loss import get_hat_logprobs_pruned
from .rnnt_loss import get_rnnt_logprobs
from .rnnt_loss import get_rnnt_logprobs_joint
from .rnnt_loss import get_rnnt_logprobs_pruned
from .rnnt_loss import get_rnnt_logprobs_smoothed
from .rnnt_loss import get_rnnt_prune_ranges
from .rnnt_loss import get_rnnt_prune_ranges_deprecated
from .rnnt_loss import rnnt_loss
from .rnnt_loss import rnnt_loss_pruned
from .rnnt_loss import rnnt_loss_pruned_joiner
from .rnnt_loss import rnnt_loss_simple
from .rnnt_loss import rnnt_loss_smoothed

with_cuda = True  # the reference's tests read k2.with_cuda to pick devices (k2/python/k2/__init__.py:121)

__all__ = [
    "joint_mutual_information_recursion", "mutual_information_recursion", "do_rnnt_pruning",
    "get_rnnt_logprobs", "get_rnnt_logprobs_joint", "get_rnnt_logprobs_pruned",
    "get_rnnt_prune_ranges", "rnnt_loss", "rnnt_loss_pruned", "rnnt_loss_simple",
    "get_hat_logprobs_pruned", "get_rnnt_logprobs_smoothed", "rnnt_loss_smoothed",
    "get_rnnt_prune_ranges_deprecated", "pruned_ranges_to_lattice", "rnnt_loss_pruned_joiner",
]
