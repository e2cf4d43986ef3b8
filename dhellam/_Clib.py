"""dhellam._Clib: the six names of the reference's pybind11 extension (csrc/torchapi.cpp:2-9) with their
positional signatures (csrc/operators/ops.h:18-81), over the C ABI of libdhellam_hip.so."""
from dhellam_amd._Clib import *  # noqa: F401,F403
from dhellam_amd._Clib import add_tensors, pybda, pygelu, pygemm, pymha_varlen_bwd, pymha_varlen_fwd  # noqa: F401
