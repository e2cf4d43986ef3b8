"""dhellam.operators.moe -> dhellam_amd.operators.moe."""
from dhellam_amd.operators.moe import *  # noqa: F401,F403
