"""Tensor-parallel coordinates of this process: the two getters the head-block operators of the
reference read from dhellam/adaptor/parallel_state.py (loss.py:32-33, embedding.py:21-23).

This build runs one rank on one GPU and owns no process groups: the coordinates are plain
numbers set by the caller.  With a world size above one the operators compute that rank's
share and every all-reduce of the reference is left to the caller (identity here).
"""
_TP_RANK = 0
_TP_WORLD = 1


def set_tensor_model_parallel(rank: int, world_size: int) -> None:
    global _TP_RANK, _TP_WORLD
    if not (world_size >= 1 and 0 <= rank < world_size):
        raise ValueError(f"rank {rank} outside a tensor-parallel world of {world_size}")
    _TP_RANK, _TP_WORLD = int(rank), int(world_size)


def get_tensor_model_parallel_rank() -> int:
    return _TP_RANK


def get_tensor_model_parallel_world_size() -> int:
    return _TP_WORLD
