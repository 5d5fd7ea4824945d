#!/usr/bin/env python3
"""Build the native parts of the hip backend in-tree.

  libtfjs_hip.so   HIP kernels + C ABI (include/tfjs_hip.h), gfx950 only
  tfjs_hip.node    N-API addon that exposes the C ABI to Node.js (needs node headers)

Usage: python tfjs-core_amd/build.py [--force] [--no-node]
"""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(ROOT, "include")
LIB = os.path.join(HERE, "libtfjs_hip.so")
ADDON = os.path.join(HERE, "js", "tfjs_hip.node")
NODE_INCLUDE = "/usr/include/node"

HIP_SOURCES = ["context.hip", "gemm.hip", "image.hip", "elementwise.hip", "reduce.hip",
               "shape_ops.hip", "backward.hip", "indexing.hip", "spectral.hip", "separable.hip"]
# Packed fp32 VALU ops are switched off for every kernel (scalar/float2 code only).
HIPCC_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-I" + INCLUDE, "-I" + CSRC,
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-Wno-unused-result", "-Wno-unknown-warning-option"]


def _stale(target, sources):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(s) > t for s in sources)


def build_lib(force=False, verbose=False):
    srcs = [os.path.join(CSRC, s) for s in HIP_SOURCES]
    deps = srcs + [os.path.join(CSRC, "tfhip_internal.h"), os.path.join(CSRC, "tfhip_device.h"), os.path.join(INCLUDE, "tfjs_hip.h")]
    if not force and not _stale(LIB, deps):
        return LIB
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    objs = []
    procs = []
    for s in srcs:
        o = os.path.splitext(s)[0] + ".o"
        objs.append(o)
        if force or _stale(o, [s] + deps[len(srcs):]):
            cmd = [hipcc] + HIPCC_FLAGS + ["-c", s, "-o", o]
            if verbose:
                print(" ".join(cmd))
            procs.append((s, subprocess.Popen(cmd, stderr=subprocess.PIPE, text=True)))
    for s, p in procs:
        _, err = p.communicate()
        err = "\n".join(l for l in err.splitlines()
                        if "packed-fp32-ops" not in l and "is not a recognized feature" not in l)
        if p.returncode != 0:
            raise RuntimeError("hipcc failed on %s:\n%s" % (s, err))
        if err.strip() and verbose:
            print(err)
    subprocess.check_call([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs)
    return LIB


def build_addon(force=False, verbose=False):
    src = os.path.join(CSRC, "napi_addon.c")
    if not os.path.exists(src) or not os.path.isdir(NODE_INCLUDE):
        return None
    if not force and not _stale(ADDON, [src, os.path.join(INCLUDE, "tfjs_hip.h")]):
        return ADDON
    os.makedirs(os.path.dirname(ADDON), exist_ok=True)
    # the addon sits in js/, the library one directory up
    cmd = ["gcc", "-O2", "-fPIC", "-shared", "-Wall", "-DNODE_GYP_MODULE_NAME=tfjs_hip",
           "-I" + NODE_INCLUDE, "-I" + INCLUDE, src, "-o", ADDON, "-L" + HERE, "-ltfjs_hip",
           "-Wl,-rpath,$ORIGIN/.."]
    if verbose:
        print(" ".join(cmd))
    subprocess.check_call(cmd)
    return ADDON


def main(argv):
    force = "--force" in argv
    print(build_lib(force, verbose=True))
    if "--no-node" not in argv:
        print(build_addon(force, verbose=True))


if __name__ == "__main__":
    main(sys.argv[1:])
