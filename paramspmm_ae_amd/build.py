"""Builds the native parts in-tree: libparamsp_hip.so (hipcc, gfx950) and the three PyTorch extension
modules ParamSpMM / ParamSDDMM / ParamSpCONV (g++, linked against the library).  Everything lands in
paramspmm_ae_amd/lib/.  Run as `python -m paramspmm_ae_amd.build` or through paramspmm_ae_amd/build_param.sh.
"""
import os
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "lib")
MODULES = ("ParamSpMM", "ParamSDDMM", "ParamSpCONV")


def build_hip_library(jobs=8, force=False):
    cmd = ["make", "-C", CSRC, "-j%d" % jobs]
    if force:
        cmd.append("-B")
    subprocess.check_call(cmd)
    return os.path.join(LIB, "libparamsp_hip.so")


def _ext_command(name):
    import torch
    from torch.utils import cpp_extension as ce

    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    inc = ["-I" + p for p in ce.include_paths()]
    inc += ["-I" + sysconfig.get_paths()["include"], "-I/opt/rocm/include", "-I" + os.path.join(ROOT, "include")]
    src = os.path.join(CSRC, "torch_ext", name + ".cpp")
    out = os.path.join(LIB, name + ".so")
    return [
        "g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden", "-Wno-attributes",
        "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=" + name,
        "-DTORCH_API_INCLUDE_EXTENSION_H", "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
    ] + inc + [
        src, "-o", out,
        "-L" + LIB, "-lparamsp_hip", "-L" + torch_lib, "-lc10", "-lc10_hip", "-ltorch", "-ltorch_cpu", "-ltorch_hip",
        "-ltorch_python", "-L/opt/rocm/lib", "-lamdhip64", "-lrocsparse",
        "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + torch_lib, "-Wl,-rpath,/opt/rocm/lib",
    ]


def build_extensions(force=False):
    os.makedirs(LIB, exist_ok=True)
    hdr = os.path.join(CSRC, "torch_ext", "glue_common.h")
    hdr2 = os.path.join(CSRC, "torch_ext", "baseline_rocsparse.h")
    todo = []
    for name in MODULES:
        src = os.path.join(CSRC, "torch_ext", name + ".cpp")
        out = os.path.join(LIB, name + ".so")
        newest = max(os.path.getmtime(src), os.path.getmtime(hdr), os.path.getmtime(hdr2), os.path.getmtime(os.path.join(ROOT, "include", "paramsp.h")))
        if force or not os.path.exists(out) or os.path.getmtime(out) < newest:
            todo.append(name)

    def run(name):
        subprocess.check_call(_ext_command(name))
        return name

    with ThreadPoolExecutor(max_workers=3) as pool:
        list(pool.map(run, todo))
    return [os.path.join(LIB, n + ".so") for n in MODULES]


def build_all(force=False):
    build_hip_library(force=force)
    build_extensions(force=force)


if __name__ == "__main__":
    build_all(force="--force" in sys.argv)
    print("built:", ", ".join(sorted(os.listdir(LIB))))
