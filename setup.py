"""Installs the MI355X fused AdaLN / RMSNorm ops the way TeleTron's ``teletron_op/install.sh`` installs
its own (two ``setup.py install`` runs, ``teletron_op/install.sh:1-9``): afterwards ``import fused_adaln``
and ``import fused_rmsnorm`` work from anywhere, next to the ``teletron_amd`` package that holds the
HIP library.

    pip install --no-build-isolation .        # or: python setup.py install

The HIP library and the torch glue modules are compiled by ``teletron_amd/build.py`` (hipcc for
gfx950, g++ for the glue) before the files are collected, unless what is built in the tree is newer
than every source.
"""
from setuptools import setup
from setuptools.command.build_py import build_py


class BuildWithHip(build_py):
    def run(self):
        import importlib.util
        import os
        import sys
        here = os.path.dirname(os.path.abspath(__file__))
        # load teletron_amd/build.py by path: importing the package itself would need the library it builds
        spec = importlib.util.spec_from_file_location("_teletron_amd_build", os.path.join(here, "teletron_amd", "build.py"))
        tb = importlib.util.module_from_spec(spec)
        sys.modules[spec.name] = tb
        spec.loader.exec_module(tb)
        if not tb.is_current():
            tb.build_library(force=False)
            tb.build_torch_extensions(force=False)
        super().run()


setup(
    name="teletron-op-mi355x",
    version="0.1.0",
    description="MI355X-native fused AdaLN / RMSNorm ops with TeleTron's teletron_op interface",
    packages=["teletron_amd"],
    package_dir={"": "teletron_amd/toplevel", "teletron_amd": "teletron_amd"},
    py_modules=["fused_adaln", "fused_rmsnorm"],
    package_data={"teletron_amd": ["*.so"]},
    include_package_data=False,
    zip_safe=False,
    cmdclass={"build_py": BuildWithHip},
    python_requires=">=3.9",
)
