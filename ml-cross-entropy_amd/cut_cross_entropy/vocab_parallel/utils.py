"""Vocabulary sharding options (reference: cut_cross_entropy/vocab_parallel/utils.py).

Only the shard bounds are used on one GPU: ``start``/``stop`` select the slice of
the vocabulary that ``c`` holds.  The exchange steps of the reference (MAX/SUM
all-reduce of the shard LSEs, SUM of the correct logits, SUM of the dE partials;
vocab_parallel/utils.py:47-76) are not part of this build; with an initialised
process group of more than one rank the operator raises instead of silently
returning shard-local values.
"""

from dataclasses import dataclass
from typing import Any, Optional, Tuple


def partition_n_into_range(n: int, rank: int, world_size: int) -> Tuple[int, int]:
    """Contiguous split of range(n): every rank gets n // world_size items and the
    first n % world_size ranks one more (reference vocab_parallel/utils.py:9-13)."""
    base, extra = divmod(n, world_size)
    start = rank * base + min(rank, extra)
    return start, start + base + (1 if rank < extra else 0)


@dataclass
class VocabParallelOptions:
    """:param start: first vocabulary index held by this shard.
    :param stop: one past the last index held by this shard.
    :param group: process group of the vocab-parallel ranks (unused on one GPU).
    :param reduce_e_grad: whether dE should be summed over the ranks (unused on one GPU).
    """

    start: int
    stop: int
    group: Optional[Any] = None
    reduce_e_grad: bool = True

    @classmethod
    def from_vocab(cls, vocab_size: int, group: Optional[Any] = None, reduce_e_grad: bool = True):
        """Bounds of this rank's shard (reference vocab_parallel/utils.py:32-44)."""
        import torch.distributed as dist

        rank = dist.get_rank(group)
        world_size = dist.get_world_size(group)
        start, stop = partition_n_into_range(vocab_size, rank, world_size)
        return cls(start, stop, group, reduce_e_grad)


def require_single_rank(opts: "VocabParallelOptions") -> None:
    """Shard partials are exact only when no other rank holds part of the vocabulary
    sum; refuse to run where the reference would have all-reduced."""
    import torch.distributed as dist

    if dist.is_available() and dist.is_initialized() and dist.get_world_size(opts.group) > 1:
        raise NotImplementedError(
            "vocab-parallel collectives are not implemented in this single-GPU build; "
            "use cut_cross_entropy.vocab_parallel.shard_forward / shard_backward and "
            "combine the shard partials yourself"
        )
