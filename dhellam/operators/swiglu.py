"""dhellam.operators.swiglu -> dhellam_amd.operators.swiglu."""
from dhellam_amd.operators.swiglu import *  # noqa: F401,F403
