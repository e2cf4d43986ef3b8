"""dhellam.operators.comm on one GPU.  The sequence-parallel collectives (comm.py:13-58) are the identity for a
tensor-parallel group of one rank; anything that needs a second rank raises: collectives are outside the
single-GPU operator path."""
import torch


class _Done:
    """Stands for the async work handle the reference returns."""

    def wait(self):
        return None


def _single_rank(gpus, comm_group):
    world = gpus if gpus is not None else 1
    if comm_group is not None and torch.distributed.is_available() and torch.distributed.is_initialized():
        world = torch.distributed.get_world_size(group=comm_group)
    if world != 1:
        raise RuntimeError("collectives across ranks are not part of the single-GPU operator path "
                           f"(tensor-parallel world size {world})")


def gather_along_first_dim(input_, gpus=1, comm_group=None, async_op=False):
    _single_rank(gpus, comm_group)
    return input_, (_Done() if async_op else None)


def reduce_scatter_along_first_dim(input_, gpus=1, comm_group=None, async_op=False):
    _single_rank(gpus, comm_group)
    return input_, (_Done() if async_op else None)


def _needs_ranks(name):
    def fn(*args, **kwargs):
        raise RuntimeError(f"{name} exchanges data between ranks: not part of the single-GPU operator path")
    fn.__name__ = name
    return fn


flash_attn_p2p_communicate = _needs_ranks("flash_attn_p2p_communicate")
chunk_allgather_gemm = _needs_ranks("chunk_allgather_gemm")
chunk_gemm_reduce_scatter = _needs_ranks("chunk_gemm_reduce_scatter")
