"""dhellam.core.dshb (dshb.py:73-275)."""
from dhellam_amd.core.dshb import DSHB, DSHB_, post_process, pre_process  # noqa: F401
