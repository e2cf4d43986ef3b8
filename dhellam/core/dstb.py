"""dhellam.core.dstb (dstb.py:24-1468)."""
from dhellam_amd.core.dstb import (DCBlock, DCFunc, DCOP, DCoperation, DSTB, DSTB_, FuncChoice, LayerConfig,  # noqa: F401
                                   exec, init_DCBlocks)
