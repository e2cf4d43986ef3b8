"""dhellam.operators.layernorm_column -> dhellam_amd.operators.layernorm_column
(gemm_fwd, gemm_fwd_event, gemm_bwd, dgrad_bwd, wgrad_bwd: layernorm_column.py:7-323)."""
from dhellam_amd.operators.layernorm_column import dgrad_bwd, gemm_bwd, gemm_fwd, gemm_fwd_event, wgrad_bwd  # noqa: F401
