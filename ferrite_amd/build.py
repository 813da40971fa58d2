"""Builds libferrite_hip.so for gfx950 with hipcc (in-tree, next to the sources).

`python -m ferrite_amd.build` or ferrite_amd.build.build().  The build id baked into the library is a hash of
every source that goes into it (the same-source gate of the reference, crates/ferrite-kernel/build.rs:1-216).
"""
from __future__ import annotations

import hashlib
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
SO_PATH = os.path.join(HERE, "libferrite_hip.so")
SOURCES = ["layer.hip", "route.hip", "formats.hip", "experts_f32.hip", "experts_mfma.hip", "block_ops.hip"]
HEADERS = ["internal.hpp", "numerics.hpp", "device_utils.hpp"]


def source_hash() -> str:
    h = hashlib.sha256()
    for name in SOURCES + HEADERS:
        with open(os.path.join(CSRC, name), "rb") as f:
            h.update(name.encode())
            h.update(f.read())
    with open(os.path.join(INCLUDE, "ferrite_hip.h"), "rb") as f:
        h.update(f.read())
    return h.hexdigest()[:16]


def build(verbose: bool = False, incremental: bool = False) -> str:
    """Compile every HIP source into libferrite_hip.so: one object per source, compiled side by side, then linked.
    Always recompiles unless `incremental` is set, which keeps the objects whose inputs (the source, the shared
    headers, the flags) have not changed since they were built - a convenience while editing one kernel file."""
    from concurrent.futures import ThreadPoolExecutor
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    build_id = "ferrite-hip-" + source_hash()
    flags = ["-O3", "-std=c++17", "--offload-arch=gfx950", "-fPIC",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             # a*b+c must stay two rounded operations: routing has to reproduce the reference's f32 chains bit
             # for bit (HIP's __fmul_rn/__fadd_rn are plain operators and would otherwise be fused); fmaf() where
             # a fused multiply-add is wanted is written explicitly
             "-ffp-contract=off",
             "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes", "-I", INCLUDE]
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    shared = hashlib.sha256(" ".join(flags).encode())
    for name in HEADERS:
        with open(os.path.join(CSRC, name), "rb") as f:
            shared.update(f.read())
    with open(os.path.join(INCLUDE, "ferrite_hip.h"), "rb") as f:
        shared.update(f.read())

    def compile_one(src: str):
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        with open(os.path.join(CSRC, src), "rb") as f:
            key = hashlib.sha256(shared.digest() + f.read()).hexdigest()
        # the build id is baked into layer.hip only, so the other objects do not depend on it
        extra = [f'-DFERRITE_BUILD_ID="{build_id}"'] if src == "layer.hip" else []
        if src == "layer.hip":
            key = hashlib.sha256((key + build_id).encode()).hexdigest()
        stamp = obj + ".key"
        if incremental and os.path.exists(obj) and os.path.exists(stamp) and open(stamp).read() == key:
            return obj, ""
        cmd = [hipcc] + flags + extra + ["-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd))
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            sys.stderr.write(res.stdout + res.stderr)
            raise RuntimeError(f"hipcc failed on {src}")
        with open(stamp, "w") as f:
            f.write(key)
        return obj, res.stderr

    with ThreadPoolExecutor(max_workers=min(len(SOURCES), os.cpu_count() or 1)) as pool:
        results = list(pool.map(compile_one, SOURCES))
    if verbose:
        for _, err in results:
            if err:
                sys.stderr.write(err)
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", SO_PATH] + [o for o, _ in results]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        sys.stderr.write(res.stdout + res.stderr)
        raise RuntimeError("hipcc link failed")
    return SO_PATH


HOST_DIR = os.path.join(HERE, "host")
HOST_SMOKE = os.path.join(HOST_DIR, "hip_backend_smoke")
HOST_SO = os.path.join(HOST_DIR, "libferrite_host.so")


def build_host(verbose: bool = False) -> str:
    """Compile the C++ host side (HipBackend over the C ABI) and its smoke driver with g++."""
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    common = ["g++", "-O2", "-std=c++17", "-Wall", "-pthread", "-D__HIP_PLATFORM_AMD__", f"-I{rocm}/include"]
    libs = [f"-L{rocm}/lib", "-lamdhip64", "-ldl", f"-Wl,-rpath,{rocm}/lib"]
    src = lambda *names: [os.path.join(HOST_DIR, n) for n in names]
    cmds = [
        common + ["-o", HOST_SMOKE] + src("hip_backend.cpp", "checkpoint.cpp", "smoke_main.cpp") + libs,
        # the same host code as a shared library with a C facade, for bindings (ctypes) that cannot call C++
        common + ["-fPIC", "-shared", "-o", HOST_SO] + src("hip_backend.cpp", "checkpoint.cpp", "host_capi.cpp") + libs,
    ]
    for cmd in cmds:
        if verbose:
            print(" ".join(cmd))
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            sys.stderr.write(res.stdout + res.stderr)
            raise RuntimeError("g++ failed (host side)")
    return HOST_SMOKE


if __name__ == "__main__":
    if "--print-id" in sys.argv:   # what a binding bakes in to refuse a library of another build
        print("ferrite-hip-" + source_hash())
        sys.exit(0)
    print(build(verbose="-v" in sys.argv, incremental="--incremental" in sys.argv))
    print(build_host(verbose=True))
