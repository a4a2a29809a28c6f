#!/usr/bin/env python3
"""Build the gfx950 libraries in-tree by driving hipcc directly.

Counterpart of the reference's build script (setup.py:39-96, a CUDAExtension built
with nvcc): here there is one target architecture (gfx950), no hipify pass and no
CUDA shims, so the compiler is simply invoked on the sources.

Outputs, next to this file (where the reference's wrappers look for the module,
omni-attn-mma/omni_attn_torch.py:548-552):
  libomni_attn_gfx950.so            C ABI (include/omni_attn_gfx950.h), no torch dependency
  omni_attn.cpython-*.so            Python module `omni_attn` (torch tensors in, C ABI underneath)

Usage:  python build.py [--no-ext] [--jobs N]
"""
import argparse
import concurrent.futures
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")
HIPCC = os.path.join(ROCM, "bin", "hipcc")

# Packed-fp32 VALU forms are disabled for every device compile.
DEVICE_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]

INSTANCES = [(bf, d) for bf in (0, 1) for d in (32, 64, 128)]
LIB_NAME = "libomni_attn_gfx950.so"


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(
        line for line in proc.stdout.splitlines()
        if "packed-fp32-ops' is not a recognized feature" not in line
    )
    if proc.returncode != 0:
        raise RuntimeError("command failed (%d): %s\n%s" % (proc.returncode, " ".join(cmd), out))
    return out


def build_capi(jobs):
    os.makedirs(OBJ, exist_ok=True)
    cmds = []
    objs = []
    for bf, d in INSTANCES:
        obj = os.path.join(OBJ, "fwd_inst_%s_d%d.o" % ("bf16" if bf else "f16", d))
        objs.append(obj)
        cmds.append([HIPCC] + DEVICE_FLAGS + [
            "-DOMNI_INST_BF16=%d" % bf, "-DOMNI_INST_D=%d" % d,
            "-c", os.path.join(CSRC, "omni_attn_fwd_inst.hip"), "-o", obj])
    obj = os.path.join(OBJ, "omni_attn_capi.o")
    objs.append(obj)
    cmds.append([HIPCC] + DEVICE_FLAGS + ["-c", os.path.join(CSRC, "omni_attn_capi.hip"), "-o", obj])
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        for out in pool.map(_run, cmds):
            if out.strip():
                print(out)
    lib = os.path.join(HERE, LIB_NAME)
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib] + objs)
    return lib


def build_ext():
    """Python module `omni_attn`: g++-level C++ (no device code) against torch + the C ABI."""
    import torch
    from torch.utils import cpp_extension

    suffix = sysconfig.get_config_var("EXT_SUFFIX")
    out = os.path.join(HERE, "omni_attn" + suffix)
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    includes = cpp_extension.include_paths("cuda") + [sysconfig.get_paths()["include"]]
    cmd = [HIPCC, "-O2", "-std=c++17", "-fPIC", "-shared", "-x", "c++",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=omni_attn",
           "-DTORCH_API_INCLUDE_EXTENSION_H", "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
           "-Wno-unused-command-line-argument"]
    for inc in includes:
        cmd += ["-isystem", inc]
    cmd += ["-I", os.path.join(ROOT, "include"),
            os.path.join(CSRC, "omni_attn_pybind.cpp"), "-o", out,
            "-L", HERE, "-l:" + LIB_NAME, "-Wl,-rpath,$ORIGIN",
            "-L", torch_lib, "-Wl,-rpath," + torch_lib,
            "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-ltorch_python"]
    _run(cmd)
    return out


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.splitlines()[0])
    ap.add_argument("--no-ext", action="store_true", help="build only the C-ABI library")
    ap.add_argument("--jobs", type=int, default=min(8, os.cpu_count() or 1))
    args = ap.parse_args(argv)
    lib = build_capi(args.jobs)
    print("built", lib)
    if not args.no_ext:
        ext = build_ext()
        print("built", ext)
    return 0


if __name__ == "__main__":
    sys.exit(main())
