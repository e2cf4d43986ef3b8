"""Small helpers of dhellam/common/common.py that the hot path touches."""
import torch

_workspace = {}


def get_workspace() -> torch.Tensor:
    """GEMM workspace, cached per device (the reference re-allocates 4/32 MiB on every
    call, common.py:7-13); hipBLASLt manages its own, so this is only kept for callers."""
    dev = torch.cuda.current_device()
    if dev not in _workspace:
        _workspace[dev] = torch.empty(4_194_304, dtype=torch.uint8, device=f"cuda:{dev}")
    return _workspace[dev]


def print_rank0(*args) -> None:
    if not torch.distributed.is_available() or not torch.distributed.is_initialized() \
            or torch.distributed.get_rank() == 0:
        print(*args)
