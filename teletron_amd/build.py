"""Builds the HIP shared library ``libteletron_op.so`` (C ABI, no torch dependency)
in-tree with hipcc for gfx950, and optionally the torch-facing pybind modules.

Usage:  python -m teletron_amd.build [--force] [--define NAME=VALUE ...]
"""
from __future__ import annotations

import argparse
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
REPO_ROOT = PKG_DIR.parent
CSRC = PKG_DIR / "csrc"
OBJ_DIR = CSRC / "build"
LIB_PATH = PKG_DIR / "libteletron_op.so"

HIP_SOURCES = ["capi.hip", "adaln_fwd.hip", "adaln_fwd_xnorm.hip", "adaln_bwd.hip", "adaln_bwd_saved.hip",
               "rms_fwd.hip", "rms_bwd.hip", "rms_bwd_saved.hip", "rms_rope.hip", "gate.hip",
               "resnorm_plain.hip", "resnorm_gated.hip"]

# -packed-fp32-ops is switched off on purpose: the compiler must not form
# v_pk_{add,mul,fma}_f32 from the scalar float code of these kernels.
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; a ROCm toolchain is required to build teletron_amd")
    return exe


def _run(cmd):
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s\n%s" % (" ".join(map(str, cmd)), proc.stdout, proc.stderr))
    return proc


def build_library(force: bool = True, defines=(), jobs: int = 8, verbose: bool = True) -> Path:
    """Compile every HIP translation unit and link libteletron_op.so."""
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    headers = list(CSRC.glob("*.hpp")) + [REPO_ROOT / "include" / "teletron_op.h"]
    newest_header = max(h.stat().st_mtime for h in headers)
    dflags = ["-D" + d for d in defines]

    def compile_one(name: str) -> Path:
        src = CSRC / name
        obj = OBJ_DIR / (Path(name).stem + ".o")
        if (not force and obj.exists() and obj.stat().st_mtime > max(src.stat().st_mtime, newest_header)):
            return obj
        cmd = [hipcc(), *HIP_FLAGS, *dflags, "-I", str(REPO_ROOT / "include"), "-I", str(CSRC),
               "-c", str(src), "-o", str(obj)]
        if verbose:
            print("[teletron_amd.build] hipcc", name, flush=True)
        _run(cmd)
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(compile_one, HIP_SOURCES))
    _run([hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", f"-Wl,-soname,{LIB_PATH.name}", "-o", str(LIB_PATH),
          *map(str, objs)])
    if verbose:
        print("[teletron_amd.build] linked", LIB_PATH, flush=True)
    return LIB_PATH


TORCH_EXT_MODULES = ["fused_adaln", "fused_rmsnorm"]


def torch_ext_path(name: str) -> Path:
    import sysconfig
    return PKG_DIR / (name + sysconfig.get_config_var("EXT_SUFFIX"))


def is_current() -> bool:
    """True when the library and the glue modules exist and each is newer than every source it is built from."""
    glue = [torch_ext_path(n) for n in TORCH_EXT_MODULES]
    if not LIB_PATH.exists() or not all(g.exists() for g in glue):
        return False
    header = REPO_ROOT / "include" / "teletron_op.h"
    newest = lambda files: max(f.stat().st_mtime for f in files)
    lib_srcs = list(CSRC.glob("*.hip")) + list(CSRC.glob("*.hpp")) + [header]
    glue_srcs = list((CSRC / "torch_ext").glob("*")) + [header]
    return LIB_PATH.stat().st_mtime > newest(lib_srcs) and min(g.stat().st_mtime for g in glue) > newest(glue_srcs)


def build_torch_extensions(force: bool = True, verbose: bool = True):
    """Compile the pybind / TORCH_LIBRARY glue modules (host C++ only, g++) against the
    installed torch and link them to libteletron_op.so.  They hold no kernels."""
    import sysconfig
    import torch
    from torch.utils import cpp_extension as ce
    if not LIB_PATH.exists():
        build_library(force=True, verbose=verbose)
    src_dir = CSRC / "torch_ext"
    torch_lib = Path(torch.__file__).resolve().parent / "lib"
    incs = []
    for d in ce.include_paths("cuda") + [sysconfig.get_paths()["include"], str(REPO_ROOT / "include"), str(src_dir)]:
        incs += ["-I", d]
    abi = int(getattr(torch._C, "_GLIBCXX_USE_CXX11_ABI", True))
    cxx = shutil.which("g++") or "g++"

    def compile_one(name: str) -> Path:
        src = src_dir / (name + ".cpp")
        out = torch_ext_path(name)
        deps = [src, src_dir / "glue.hpp", REPO_ROOT / "include" / "teletron_op.h"]
        if not force and out.exists() and out.stat().st_mtime > max(d.stat().st_mtime for d in deps):
            return out
        cmd = [cxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
               f"-DTORCH_EXTENSION_NAME={name}", "-DTORCH_API_INCLUDE_EXTENSION_H",
               f"-D_GLIBCXX_USE_CXX11_ABI={abi}", "-Wno-deprecated-declarations", *incs, str(src), "-o", str(out),
               f"-L{torch_lib}", "-L/opt/rocm/lib", "-ltorch", "-ltorch_cpu", "-ltorch_python", "-lc10", "-lc10_hip",
               "-ltorch_hip", "-lamdhip64", f"-L{PKG_DIR}", f"-l:{LIB_PATH.name}",
               "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{torch_lib}", "-Wl,-rpath,/opt/rocm/lib"]
        if verbose:
            print("[teletron_amd.build] g++", src.name, flush=True)
        _run(cmd)
        return out

    with ThreadPoolExecutor(max_workers=2) as pool:
        return list(pool.map(compile_one, TORCH_EXT_MODULES))


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--force", action="store_true", help="recompile even if objects look current")
    ap.add_argument("--define", action="append", default=[], help="extra -D for hipcc (tuning constants)")
    ap.add_argument("--no-torch-ext", action="store_true", help="skip the pybind/TORCH_LIBRARY glue modules")
    ap.add_argument("--jobs", type=int, default=min(8, os.cpu_count() or 1))
    args = ap.parse_args(argv)
    build_library(force=args.force or bool(args.define), defines=args.define, jobs=args.jobs)
    if not args.no_torch_ext:
        build_torch_extensions(force=args.force)
    return 0


if __name__ == "__main__":
    sys.exit(main())
