"""dhellam.core.dsllm (dsllm.py:10-115)."""
from dhellam_amd.core.dsllm import DSLLM, Stack, pre_backward_hook  # noqa: F401
