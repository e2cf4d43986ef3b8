"""dhellam.common.benchmark (benchmark.py:4-79)."""
from dhellam_amd.common.benchmark import benchmark, benchmark_ms, benchmark_ms_ops  # noqa: F401
