"""Top-level module name that TeleTron's RMSNorm autograd Function imports
(``teletron_op/README.md:133,165``; built there by ``teletron_op/fused_rmsnorm/rms_setup.py``).
Installed next to the ``teletron_amd`` package by ``setup.py``; the functions are the glue module's."""
from teletron_amd.fused_rmsnorm import torch_launch_rms_backward, torch_launch_rms_forward

__all__ = ["torch_launch_rms_forward", "torch_launch_rms_backward"]
