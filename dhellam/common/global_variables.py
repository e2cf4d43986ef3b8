"""dhellam.common.global_variables: the same dict object as dhellam_amd's."""
from dhellam_amd.common.global_variables import GLOBAL_VARIABLES  # noqa: F401
