"""In-tree build of the gfx950 kernels and the `test_time_training` operator module.

    python ttt-tk_amd/build.py            # kernels + C ABI library + Python module
    python ttt-tk_amd/build.py --lib      # kernels + C ABI library only
    python ttt-tk_amd/build.py --stages   # libttt_mlp_stages.so: the library with stage clocks, for stage_clocks.py

Outputs (next to this file, picked up by `import test_time_training` once this directory is on
sys.path):
    libttt_mlp.so                                   hipcc, --offload-arch=gfx950, the C ABI of include/ttt_mlp.h
    test_time_training.cpython-*.so                 g++, pybind11 module on top of libttt_mlp.so
hipcc cross-compiles for gfx950, so no GPU is needed to build.
"""
from __future__ import annotations

import argparse
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libttt_mlp.so")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")

HIP_SOURCES = ["ttt_mlp_fwd.hip", "ttt_mlp_bwd.hip", "ttt_mlp_export.hip", "ttt_mlp_c_abi.hip"]
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
             # packed-fp32 VALU forms are kept out of the generated code on purpose
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)


def module_path() -> str:
    return os.path.join(HERE, "test_time_training" + sysconfig.get_config_var("EXT_SUFFIX"))


def build_lib(extra_flags=(), lib: str = LIB, objdir: str = "build") -> str:
    """Compiles the four HIP sources and links them into `lib` (objects under `objdir`, next to this file)."""
    objs = []
    os.makedirs(os.path.join(HERE, objdir), exist_ok=True)
    procs = []
    for src in HIP_SOURCES:
        obj = os.path.join(HERE, objdir, src.replace(".hip", ".o"))
        cmd = ["hipcc", *HIP_FLAGS, *extra_flags, "-c", os.path.join(CSRC, src), "-o", obj]
        print("+", " ".join(cmd), flush=True)
        procs.append((cmd, subprocess.Popen(cmd)))
        objs.append(obj)
    for cmd, p in procs:
        if p.wait() != 0:
            raise subprocess.CalledProcessError(p.returncode, cmd)
    _run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", lib])
    return lib


STAGES_LIB = os.path.join(HERE, "libttt_mlp_stages.so")


def build_stages_lib() -> str:
    """The same library with the stage clocks compiled in (-DTTT_STAGE_CLOCKS), for stage_clocks.py only."""
    return build_lib(("-DTTT_STAGE_CLOCKS",), STAGES_LIB, os.path.join("build", "stages"))


def build_module() -> str:
    import torch
    from torch.utils import cpp_extension as ce

    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    out = module_path()
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-DTORCH_EXTENSION_NAME=test_time_training", "-DTORCH_API_INCLUDE_EXTENSION_H",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           *[f"-I{p}" for p in ce.include_paths()], f"-I{sysconfig.get_paths()['include']}", f"-I{ROCM}/include",
           os.path.join(CSRC, "test_time_training.cpp"), "-o", out,
           f"-L{HERE}", "-lttt_mlp", f"-L{torch_lib}", "-lc10", "-lc10_hip", "-ltorch", "-ltorch_cpu", "-ltorch_python",
           f"-L{ROCM}/lib", "-lamdhip64", "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{torch_lib}", f"-Wl,-rpath,{ROCM}/lib"]
    _run(cmd)
    return out


def build_all() -> None:
    build_lib()
    build_module()


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--lib", action="store_true", help="build only libttt_mlp.so")
    ap.add_argument("--stages", action="store_true", help="build only libttt_mlp_stages.so (stage clocks compiled in)")
    a = ap.parse_args()
    if a.stages:
        print("built:", build_stages_lib())
        sys.exit(0)
    build_lib()
    if not a.lib:
        build_module()
    print("built:", LIB, "" if a.lib else module_path())
