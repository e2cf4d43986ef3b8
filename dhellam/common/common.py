"""dhellam.common.common (common.py:2-118)."""
from dhellam_amd.common.common import _get_qkv_layout, get_workspace, print_rank0  # noqa: F401
