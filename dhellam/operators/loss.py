"""dhellam.operators.loss -> dhellam_amd.operators.loss."""
from dhellam_amd.operators.loss import *  # noqa: F401,F403
