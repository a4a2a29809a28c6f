#!/usr/bin/env python3
"""Build the gfx950 libraries in-tree by driving hipcc directly.

Counterpart of the reference's build script (setup.py:39-96, a CUDAExtension built
with nvcc): here there is one target architecture (gfx950), no hipify pass and no
CUDA shims, so the compiler is simply invoked on the sources.

Outputs, next to this file (where the reference's wrappers look for the module,
omni-attn-mma/omni_attn_torch.py:548-552):
  libomni_attn_gfx950.so            C ABI (include/omni_attn_gfx950.h), no torch dependency
  omni_attn.cpython-*.so            Python module `omni_attn` (torch tensors in, C ABI underneath)

Every device compile also reports the registers, scratch and occupancy the compiler gave
each kernel instance (-Rpass-analysis=kernel-resource-usage).  The figures are written to
build/kernel_resources.json and checked: an instance that spills to scratch memory or
drops below the waves per SIMD its pipeline is written for fails the build -- the
instruction schedule of the forward kernel depends on both, and a compiler change would
otherwise halve the throughput silently.

Usage:  python build.py [--no-ext] [--jobs N]
"""
import argparse
import concurrent.futures
import json
import os
import re
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
    "-Wno-unused-command-line-argument", "-Wno-inline-asm",
    # LDS addresses are 32-bit integers turned into address-space-3 pointers; the host pass of
    # hipcc, where pointers are 64 bits wide, warns about every such cast
    "-Wno-int-to-pointer-cast",
    "-Rpass-analysis=kernel-resource-usage",
]
RESOURCES_JSON = os.path.join(OBJ, "kernel_resources.json")

# What the kernels of the library must keep: no scratch memory, no spilled registers, and at
# least this many waves per SIMD (kernels are matched by a substring of their mangled name).
# The backward kernels keep scalar values in spare vector lanes here and there (SGPR spills, no
# memory behind them): for them only scratch memory and spilled vector registers fail the build.
MIN_WAVES_PER_SIMD = {"fwd_kernel": 2, "bwd_dq_kernel": 2, "bwd_dkdv_kernel": 2}
SGPR_SPILLS_ALLOWED = ("bwd_dq_kernel", "bwd_dkdv_kernel")
NOT_GATED = ("fwd_generic_kernel",)

INSTANCES = [(bf, d) for bf in (0, 1) for d in (32, 64, 128)]
LIB_NAME = "libomni_attn_gfx950.so"


_REMARK = re.compile(r"remark:\s+(Function Name|TotalSGPRs|VGPRs|AGPRs|ScratchSize \[bytes/lane\]|"
                     r"Occupancy \[waves/SIMD\]|SGPRs Spill|VGPRs Spill|LDS Size \[bytes/block\]):\s+(\S+)")
_KEYS = {"TotalSGPRs": "sgprs", "VGPRs": "vgprs", "AGPRs": "agprs", "ScratchSize [bytes/lane]": "scratch_bytes",
         "Occupancy [waves/SIMD]": "waves_per_simd", "SGPRs Spill": "sgpr_spills", "VGPRs Spill": "vgpr_spills",
         "LDS Size [bytes/block]": "static_lds_bytes"}


def parse_resource_remarks(text):
    """Compiler remarks of one device compile -> {mangled kernel name: {figure: value}}."""
    kernels, cur = {}, None
    for line in text.splitlines():
        m = _REMARK.search(line)
        if not m:
            continue
        key, val = m.group(1), m.group(2)
        if key == "Function Name":
            cur = kernels.setdefault(val, {})
        elif cur is not None:
            cur[_KEYS[key]] = int(val)
    return kernels


def check_resources(kernels):
    """Raise if a kernel uses scratch memory, spills, or falls below its waves per SIMD."""
    problems = []
    for name, r in sorted(kernels.items()):
        if any(tag in name for tag in NOT_GATED):
            continue
        sgpr_spills = 0 if any(tag in name for tag in SGPR_SPILLS_ALLOWED) else r.get("sgpr_spills", 0)
        if r.get("scratch_bytes", 0) or r.get("vgpr_spills", 0) or sgpr_spills:
            problems.append("%s: scratch %d B/lane, %d VGPR / %d SGPR spills" % (
                name, r.get("scratch_bytes", 0), r.get("vgpr_spills", 0), r.get("sgpr_spills", 0)))
        for pattern, waves in MIN_WAVES_PER_SIMD.items():
            if pattern in name and r.get("waves_per_simd", 0) < waves:
                problems.append("%s: %d waves per SIMD, needs %d (%d VGPRs, %d AGPRs)" % (
                    name, r.get("waves_per_simd", 0), waves, r.get("vgprs", -1), r.get("agprs", -1)))
    if problems:
        raise RuntimeError("kernel resource check failed:\n  " + "\n  ".join(problems))


def _run(cmd):
    """Run a compiler command; returns (diagnostics without the resource remarks, remarks)."""
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    lines = proc.stdout.splitlines()
    remarks = "\n".join(l for l in lines if "-Rpass-analysis=kernel-resource-usage" in l)
    keep, skip = [], 0
    for l in lines:
        if "-Rpass-analysis=kernel-resource-usage" in l:
            skip = 2  # the source line and caret that follow a remark
            continue
        if skip and (re.match(r"^\s*\d+ \|", l) or re.match(r"^\s*\|?\s*\^", l)):
            skip -= 1
            continue
        skip = 0
        if "packed-fp32-ops' is not a recognized feature" in l or "In file included from" in l:
            continue
        keep.append(l)
    out = "\n".join(keep)
    if proc.returncode != 0:
        raise RuntimeError("command failed (%d): %s\n%s" % (proc.returncode, " ".join(cmd), proc.stdout))
    return out, remarks


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
    for bf, d in INSTANCES:
        obj = os.path.join(OBJ, "bwd_inst_%s_d%d.o" % ("bf16" if bf else "f16", d))
        objs.append(obj)
        cmds.append([HIPCC] + DEVICE_FLAGS + [
            "-DOMNI_INST_BF16=%d" % bf, "-DOMNI_INST_D=%d" % d,
            "-c", os.path.join(CSRC, "omni_attn_bwd_inst.hip"), "-o", obj])
    for src in ("omni_attn_capi", "omni_attn_probe", "omni_attn_mask_pack", "omni_attn_fwd_generic"):
        obj = os.path.join(OBJ, src + ".o")
        objs.append(obj)
        cmds.append([HIPCC] + DEVICE_FLAGS + ["-c", os.path.join(CSRC, src + ".hip"), "-o", obj])
    kernels = {}
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        for out, remarks in pool.map(_run, cmds):
            if out.strip():
                print(out)
            kernels.update(parse_resource_remarks(remarks))
    with open(RESOURCES_JSON, "w") as f:
        json.dump(kernels, f, indent=1, sort_keys=True)
    check_resources(kernels)
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
