"""MI355X-native fused AdaLN / RMSNorm ops with TeleTron's ``teletron_op`` interface.

The compute path is hand-written HIP for gfx950 in ``libteletron_op.so`` (C ABI,
``include/teletron_op.h``); Python only validates, allocates and launches.
"""
from .functional import (AdaLNGradReduceFunction, AdaLNModelFunction, FusedAdaLN, GateResidualGradReduceFunction, FusedGate, FusedRMSNorm, GateResidualFunction,
                         RMSNormModelFunction, RMSNormRopeFunction, RMSNormRopeHeadsFunction, ResidualNormFunction, adaln_modulate,
                         residual_adaln, residual_layer_norm, rms_norm, rope_table_from_cos_sin)
from . import cabi, ops, swap_in, workloads

__all__ = ["AdaLNModelFunction", "AdaLNGradReduceFunction", "GateResidualGradReduceFunction", "RMSNormModelFunction", "GateResidualFunction", "RMSNormRopeFunction", "FusedAdaLN", "FusedRMSNorm", "FusedGate",
           "ResidualNormFunction", "RMSNormRopeHeadsFunction", "rope_table_from_cos_sin", "residual_adaln", "residual_layer_norm", "adaln_modulate", "rms_norm", "cabi", "ops", "swap_in", "workloads", "install_reference_modules"]


def install_reference_modules() -> None:
    """Make ``import fused_adaln`` / ``import fused_rmsnorm`` (the reference's top-level module
    names, ``teletron_op/README.md:55,133``) resolve to this package's glue modules."""
    import importlib
    import sys
    for name in ("fused_adaln", "fused_rmsnorm"):
        sys.modules.setdefault(name, importlib.import_module(f"{__name__}.{name}"))
__version__ = "0.1.0"
