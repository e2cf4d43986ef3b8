"""dhellam.operators.layernorm -> dhellam_amd.operators.layernorm."""
from dhellam_amd.operators.layernorm import *  # noqa: F401,F403
