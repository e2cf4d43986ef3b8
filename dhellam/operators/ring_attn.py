"""dhellam.operators.ring_attn -> dhellam_amd.operators.ring_attn."""
from dhellam_amd.operators.ring_attn import *  # noqa: F401,F403
