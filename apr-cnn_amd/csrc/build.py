#!/usr/bin/env python3
"""Builds the native libraries in-tree:
     libaprnet_hip.so  HIP operators for gfx950 (hipcc, one translation unit per .hip file)
     libaprcore.so     host-only APR builder (g++ / OpenMP)
     ../_pyaprwrapper.<abi>.so   pybind11 module with the reference's native function names over the C ABI (g++, torch headers)
Usage: python build.py [--force]"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIP_SOURCES = ["plan.hip", "lists.hip", "faces.hip", "need.hip", "tree_ops.hip", "grouped.hip", "conv.hip", "conv_mfma.hip", "conv_narrow.hip", "conv_bwd.hip", "conv_bwd_mfma.hip", "conv111.hip", "restrict.hip", "pixels.hip", "stardist.hip", "norm.hip"]
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-Wno-unused-command-line-argument", "-Wno-unknown-attributes"]
HEADERS = ["common.hpp", "conv_common.hpp", os.path.join("..", "..", "include", "aprnet_hip.h")]


def _newer(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps if os.path.exists(d))


def build(force=False, verbose=True):
    os.chdir(HERE)
    objs, jobs = [], []
    for src in HIP_SOURCES:
        if not os.path.exists(src):
            continue
        obj = src.replace(".hip", ".o")
        objs.append(obj)
        if force or _newer(obj, [src] + HEADERS):
            jobs.append([HIPCC, *HIP_FLAGS, "-c", src, "-o", obj])
    def run(cmd):
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd)
    with ThreadPoolExecutor(max_workers=min(8, max(1, len(jobs)))) as ex:
        list(ex.map(run, jobs))
    if force or jobs or _newer("libaprnet_hip.so", objs):
        run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", "libaprnet_hip.so", *objs])
    if force or _newer("libaprcore.so", ["aprcore.cpp"]):
        run(["g++", "-O3", "-march=x86-64-v3", "-fopenmp", "-shared", "-fPIC", "-std=c++17", "-o", "libaprcore.so", "aprcore.cpp"])
    build_binding(force=force, verbose=verbose)
    return os.path.join(HERE, "libaprnet_hip.so"), os.path.join(HERE, "libaprcore.so")


def build_binding(force=False, verbose=True):
    """pybind/pyaprwrapper.cpp -> apr-cnn_amd/_pyaprwrapper.<abi>.so, linked against libaprnet_hip.so (found through an
    $ORIGIN rpath) and the torch libraries of this interpreter."""
    import sysconfig
    import torch
    tdir = os.path.dirname(torch.__file__)
    src = os.path.join(HERE, "pybind", "pyaprwrapper.cpp")
    out = os.path.join(os.path.dirname(HERE), "_pyaprwrapper" + sysconfig.get_config_var("EXT_SUFFIX"))
    if not (force or _newer(out, [src, os.path.join(HERE, "..", "..", "include", "aprnet_hip.h")])):
        return out
    cmd = ["g++", "-O2", "-std=c++17", "-shared", "-fPIC", "-D__HIP_PLATFORM_AMD__", "-DUSE_ROCM",
           "-DTORCH_EXTENSION_NAME=_pyaprwrapper", "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
           "-I" + os.path.join(tdir, "include"), "-I" + os.path.join(tdir, "include", "torch", "csrc", "api", "include"),
           "-I/opt/rocm/include", "-I" + sysconfig.get_paths()["include"], src, "-o", out,
           "-L" + HERE, "-laprnet_hip", "-L" + os.path.join(tdir, "lib"), "-ltorch", "-ltorch_cpu", "-ltorch_python", "-lc10",
           "-lc10_hip", "-ltorch_hip", "-L/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath,$ORIGIN/csrc", "-Wl,-rpath," + os.path.join(tdir, "lib")]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return out


if __name__ == "__main__":
    build(force="--force" in sys.argv)
