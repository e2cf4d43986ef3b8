"""dhellam.common.template_launch (template_launch.py:4-72)."""
from dhellam_amd.common.template_launch import template_bwd, template_bwd_new, template_fwd, template_fwd_new  # noqa: F401
