"""k2.pruned_ranges_to_lattice on MI355X (k2/python/k2/__init__.py:122, the binding at
k2/python/csrc/torch/pruned_ranges_to_lattice.cu:265-281).

The reference returns a ``RaggedArc`` that callers wrap in ``k2.Fsa``.  k2's FSA classes are not
part of this package; ``ArcLattice`` carries the same content — the two levels of row splits
(sequence -> states -> arcs) and the arc records — under the accessor names of ``RaggedArc``.
"""
from typing import Tuple

import torch
from torch import Tensor

from . import native


class ArcLattice:
    """A batch of lattices in k2's ragged layout [sequence][state][arc]."""

    def __init__(self, state_splits: Tensor, arc_splits: Tensor, arcs: Tensor):
        self._splits = (state_splits, arc_splits)
        self._arcs = arcs

    @property
    def dim0(self) -> int:
        return self._splits[0].numel() - 1

    @property
    def num_elements(self) -> int:
        return self._arcs.shape[0]

    def row_splits(self, axis: int) -> Tensor:
        """axis 1: sequence -> states; axis 2: state -> arcs (as RaggedShape.row_splits)."""
        assert axis in (1, 2), axis
        return self._splits[axis - 1]

    def values(self) -> Tensor:
        """int32 [num_arcs][4]: src_state, dest_state, label, and the bits of the fp32 score
        (k2's Fsa.arcs.values() has the same four columns)."""
        return self._arcs

    @property
    def scores(self) -> Tensor:
        """fp32 [num_arcs], a view of column 3 of values()."""
        return self._arcs[:, 3].view(torch.float32)


def pruned_ranges_to_lattice(ranges: Tensor, frames: Tensor, symbols: Tensor,
                             logits: Tensor) -> Tuple[ArcLattice, Tensor]:
    """ranges int32 [B][T][s_range], frames int32 [B], symbols int64 [B][S], logits
    [B][T][s_range][C] (float32 / float64 / float16) -> (lattice, arc_map int32 [num_arcs]);
    arc_map[i] indexes logits.reshape(-1), or is -1 for the arcs into the final states."""
    state_splits, arc_splits, arcs, arc_map = native.pruned_ranges_to_lattice(
        ranges, frames, symbols, logits)
    return ArcLattice(state_splits, arc_splits, arcs), arc_map
