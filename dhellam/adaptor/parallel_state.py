"""dhellam.adaptor.parallel_state: the rank / world-size getters the head-block operators use
(parallel_state.py:26-40), backed by dhellam_amd.common.parallel_state (one rank unless told otherwise)."""
from dhellam_amd.common.parallel_state import (get_tensor_model_parallel_rank, get_tensor_model_parallel_world_size,  # noqa: F401
                                               set_tensor_model_parallel)
