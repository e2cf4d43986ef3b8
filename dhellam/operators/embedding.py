"""dhellam.operators.embedding -> dhellam_amd.operators.embedding."""
from dhellam_amd.operators.embedding import *  # noqa: F401,F403
