"""dhellam.operators.bda -> dhellam_amd.operators.bda."""
from dhellam_amd.operators.bda import *  # noqa: F401,F403
