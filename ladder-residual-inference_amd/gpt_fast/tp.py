"""Tensor-parallel rank bookkeeping without a process group.

The reference initialises NCCL at import time and shards every layer by the size of the
torch.distributed world (gpt_fast/tp.py:40-63, utils.py:37-40).  This build runs ONE rank's shard
on one GPU: the world size is a plain number ("virtual" tensor parallelism), the row-parallel
outputs stay local partial sums, and no collective is ever issued.  `maybe_init_dist` keeps the
reference's name and return convention so benchmark.py reads the same."""
import os
from typing import Optional

_TP_WORLD_SIZE = 1
_SHARD_VOCAB = False
_TP_RANK = 0


def set_virtual_tp(world_size: int, rank: int = 0, shard_vocab: bool = False) -> None:
    """Shard shapes as rank `rank` of `world_size` (layers are built at size // world_size).  shard_vocab: the
    lm_head keeps vocab_size // world_size rows as well (the reference replicates the whole head on every rank)."""
    global _TP_WORLD_SIZE, _TP_RANK, _SHARD_VOCAB
    assert world_size >= 1 and 0 <= rank < world_size
    _TP_WORLD_SIZE, _TP_RANK, _SHARD_VOCAB = int(world_size), int(rank), bool(shard_vocab)


def get_shard_vocab() -> bool:
    return _SHARD_VOCAB


def get_tp_world_size() -> int:
    return _TP_WORLD_SIZE


def get_tp_rank() -> int:
    return _TP_RANK


def _get_rank() -> int:
    return int(os.environ.get("LOCAL_RANK", "0"))


def _get_world_size() -> int:
    return int(os.environ.get("LOCAL_WORLD_SIZE", "1"))


def is_local() -> bool:
    return _get_rank() == 0


def maybe_init_dist() -> Optional[int]:
    """Reference: tp.py:40-63.  Here: binds the device for this process and returns the local
    rank; never creates a process group.  More than one process is refused because every
    process would compute the same single-rank shard."""
    import torch

    rank = _get_rank()
    if _get_world_size() > 1 or int(os.environ.get("WORLD_SIZE", "1")) > 1:
        raise RuntimeError(
            "this build runs one tensor-parallel rank's shard on one GPU (see set_virtual_tp); "
            "launch a single process")
    if torch.cuda.is_available():
        torch.cuda.set_device(rank)
    return rank
