"""Process-global side channel, as dhellam/common/global_variables.py:3."""
from collections import defaultdict

GLOBAL_VARIABLES = defaultdict(lambda: {})
