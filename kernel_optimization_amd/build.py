"""Builds the native parts in-tree: libko.so (HIP kernels + C ABI, gfx950), libko_harness.so (fills, probes,
tuning and debug views for the tests and the benchmark) and the
pure C++ host layer (Tensor, benchmark drivers) that sits on top of the C ABI.

Usage: python -m kernel_optimization_amd.build [--jobs N] [--only lib|harness|host|vendor] [--cmake]
"""
import argparse
import concurrent.futures
import os
import shutil
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
HOST = os.path.join(PKG, "host")
LIB_DIR = os.path.join(PKG, "lib")
BIN_DIR = os.path.join(PKG, "bin")
OBJ_DIR = os.path.join(PKG, "build")
LIB_PATH = os.path.join(LIB_DIR, "libko.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"

# -packed-fp32-ops is switched off: the compiler must not form v_pk_*_f32 instructions.
HIP_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def _run(cmd):
    proc = subprocess.run(cmd, capture_output=True, text=True)
    out = "\n".join(l for l in (proc.stdout + proc.stderr).splitlines()
                    if "packed-fp32-ops' is not a recognized feature" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def hip_sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def build_lib(jobs=4, verbose=False):
    os.makedirs(LIB_DIR, exist_ok=True)
    os.makedirs(OBJ_DIR, exist_ok=True)
    objs = []
    cmds = []
    for src in hip_sources():
        obj = os.path.join(OBJ_DIR, src[:-4] + ".o")
        objs.append(obj)
        cmds.append([HIPCC, *HIP_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj])
    with concurrent.futures.ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
        for out in pool.map(_run, cmds):
            if verbose and out.strip():
                print(out)
    out = _run([HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", LIB_PATH, *objs])
    if verbose and out.strip():
        print(out)
    return LIB_PATH


def build_harness(jobs=4, verbose=False):
    """libko_harness.so: seeded fills, copy and streaming-probe kernels, tuning knobs and debug views
    (include/ko_harness.h).  Tests and the benchmark load it beside libko.so; it is no part of the product."""
    hdir = os.path.join(PKG, "harness")
    out_path = os.path.join(LIB_DIR, "libko_harness.so")
    os.makedirs(OBJ_DIR, exist_ok=True)
    objs, cmds = [], []
    for src in sorted(f for f in os.listdir(hdir) if f.endswith(".hip")):
        obj = os.path.join(OBJ_DIR, "harness_" + src[:-4] + ".o")
        objs.append(obj)
        cmds.append([HIPCC, *HIP_FLAGS, "-I", CSRC, "-c", os.path.join(hdir, src), "-o", obj])
    with concurrent.futures.ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
        for out in pool.map(_run, cmds):
            if verbose and out.strip():
                print(out)
    _run([HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", out_path, *objs, "-L", LIB_DIR, "-lko",
          "-Wl,-rpath,$ORIGIN"])
    return out_path


def build_vendor(verbose=False):
    """libko_vendor.so: hipBLASLt and rocBLAS timed on the same buffers (comparison harness, not product)."""
    os.makedirs(LIB_DIR, exist_ok=True)
    out_path = os.path.join(LIB_DIR, "libko_vendor.so")
    out = _run([HIPCC, "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden", "-x", "hip",
                f"--offload-arch={ARCH}", os.path.join(PKG, "vendor", "ko_vendor.cpp"), "-o", out_path,
                "-lhipblaslt", "-lrocblas"])
    if verbose and out.strip():
        print(out)
    return out_path


def build_host(verbose=False):
    """Tensor + the three benchmark drivers: plain C++ (g++), linked against libko.so only."""
    if not os.path.isdir(HOST):
        return []
    os.makedirs(BIN_DIR, exist_ok=True)
    cxx = os.environ.get("CXX", "g++")
    inc = os.path.join(ROOT, "include")
    common = [cxx, "-O2", "-std=c++17", "-Wall", "-Wextra", "-I", inc]
    tensor_obj = os.path.join(OBJ_DIR, "tensor.o")
    _run(common + ["-fPIC", "-c", os.path.join(HOST, "tensor.cpp"), "-o", tensor_obj])
    built = []
    for name in ("softmax", "layernorm", "gemm", "host_selftest"):
        src = os.path.join(HOST, name + "_main.cpp")
        if not os.path.exists(src):
            continue
        exe = os.path.join(BIN_DIR, name)
        _run(common + [src, tensor_obj, "-o", exe, "-L", LIB_DIR, "-lko", "-Wl,-rpath,$ORIGIN/../lib"])
        built.append(exe)
    return built


def build_cmake(jobs=4, verbose=False, targets=()):
    """The same build through the CMakeLists.txt at the repository root (targets ko, ko_vendor, common, softmax,
    layernorm, gemm, host_selftest; the names of the reference's CMake tree)."""
    bdir = os.path.join(OBJ_DIR, "cmake")
    out = _run(["cmake", "-S", ROOT, "-B", bdir])
    cmd = ["cmake", "--build", bdir, "-j", str(max(1, jobs))]
    for t in targets:
        cmd += ["--target", t]
    out += _run(cmd)
    if verbose:
        print(out)
    return bdir


def build_all(jobs=4, verbose=False):
    lib = build_lib(jobs=jobs, verbose=verbose)
    harness = build_harness(jobs=jobs, verbose=verbose)
    vendor = build_vendor(verbose=verbose)
    host = build_host(verbose=verbose)
    return lib, harness, vendor, host


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--jobs", type=int, default=min(8, os.cpu_count() or 1))
    ap.add_argument("--only", choices=["lib", "harness", "host", "vendor"])
    ap.add_argument("-v", "--verbose", action="store_true")
    ap.add_argument("--cmake", action="store_true", help="build everything through CMakeLists.txt instead")
    args = ap.parse_args(argv)
    if args.cmake:
        print("built with cmake in", build_cmake(args.jobs, args.verbose))
        return
    if args.only in (None, "lib"):
        print("built", build_lib(args.jobs, args.verbose))
    if args.only in (None, "harness"):
        print("built", build_harness(args.jobs, args.verbose))
    if args.only in (None, "vendor"):
        print("built", build_vendor(args.verbose))
    if args.only in (None, "host"):
        for exe in build_host(args.verbose):
            print("built", exe)


if __name__ == "__main__":
    main()
