"""
Single-rank stand-in for Heat's MPI communicator (heat/core/communication.py:126-284).

This package runs one process per GPU and the k-means path needs no exchange at one rank (every
collective on it is skipped when ``size == 1``, heat/core/_operations.py:509), so the communicator
only carries ``rank``/``size`` and the chunking helpers callers read.
"""

from __future__ import annotations

from typing import Optional, Tuple


class Communication:
    """Base class, as in heat/core/communication.py:85-123."""

    @staticmethod
    def is_distributed() -> bool:
        return False


class SingleRankCommunication(Communication):
    rank = 0
    size = 1

    def Get_rank(self) -> int:
        return 0

    def Get_size(self) -> int:
        return 1

    def is_distributed(self) -> bool:
        return False

    def chunk(self, shape, split: Optional[int], rank: Optional[int] = None, w_size: Optional[int] = None):
        """(offset, local shape, slices) of this rank's part: everything (communication.py:197-254)."""
        return 0, tuple(shape), tuple(slice(0, s) for s in shape)

    def counts_displs_shape(self, shape, axis: int) -> Tuple[tuple, tuple, tuple]:
        """communication.py:256-284 at one rank."""
        return (shape[axis],), (0,), tuple(shape)

    def __repr__(self) -> str:
        return "SingleRankCommunication(size=1)"


MPI_WORLD = SingleRankCommunication()
MPI_SELF = SingleRankCommunication()
_default = MPI_WORLD


def get_comm() -> Communication:
    return _default


def sanitize_comm(comm: Optional[Communication]) -> Communication:
    if comm is None:
        return get_comm()
    if isinstance(comm, Communication):
        return comm
    raise TypeError(f"Unknown communication, must be instance of {Communication}")


def use_comm(comm: Optional[Communication] = None) -> None:
    global _default
    _default = sanitize_comm(comm)


__all__ = ["Communication", "SingleRankCommunication", "MPI_WORLD", "MPI_SELF", "get_comm", "sanitize_comm", "use_comm"]
