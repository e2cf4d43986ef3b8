"""dhellam.operators.rope -> dhellam_amd.operators.rope."""
from dhellam_amd.operators.rope import *  # noqa: F401,F403
