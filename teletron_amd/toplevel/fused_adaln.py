"""Top-level module name that TeleTron's AdaLN autograd Function imports
(``teletron_op/README.md:55,87``; built there by ``teletron_op/fused_adaln/adaln_setup.py``).
Installed next to the ``teletron_amd`` package by ``setup.py``; the functions are the glue module's."""
from teletron_amd.fused_adaln import torch_launch_adaln_backward, torch_launch_adaln_forward

__all__ = ["torch_launch_adaln_forward", "torch_launch_adaln_backward"]
