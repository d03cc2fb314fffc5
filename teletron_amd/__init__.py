"""MI355X-native fused AdaLN / RMSNorm ops with TeleTron's ``teletron_op`` interface.

The compute path is hand-written HIP for gfx950 in ``libteletron_op.so`` (C ABI,
``include/teletron_op.h``); Python only validates, allocates and launches.
"""
from .functional import (AdaLNModelFunction, FusedAdaLN, FusedRMSNorm, RMSNormModelFunction,
                         fused_adaln, fused_rmsnorm)
from . import cabi, ops, workloads

__all__ = ["AdaLNModelFunction", "RMSNormModelFunction", "FusedAdaLN", "FusedRMSNorm",
           "fused_adaln", "fused_rmsnorm", "cabi", "ops", "workloads"]
__version__ = "0.1.0"
