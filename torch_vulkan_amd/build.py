"""Builds the HIP library for gfx950 in-tree: ``python -m torch_vulkan_amd.build``.

hipcc cross-compiles without a GPU.  Objects go to ``torch_vulkan_amd/_build/`` and the
shared library to ``torch_vulkan_amd/lib/libvkt_mi355.so``; both are kept out of git
(the library still travels with the tree to the GPU machine).
"""
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "_build")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libvkt_mi355.so")
HOSTTEST = os.path.join(LIBDIR, "libvkt_hosttest.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# packed FP32 instructions are switched off for every kernel of this library
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function", "-Wno-pass-failed",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
SOURCES = {
    "core/runtime.hip": [],
    "kernels/qmm8.hip": [],
    # every float32 operation of the int4 path is a single IEEE operation
    # (and its MFMA results go to ordinary registers, where the float32 chain consumes them)
    "kernels/qmm4.hip": ["-ffp-contract=off", "-mllvm", "-amdgpu-mfma-vgpr-form"],
    "kernels/fp8mm.hip": [],
    "kernels/gemm16.hip": [],
    # (single float32 operations in the float8 producer, as specified)
    "kernels/cast.hip": ["-ffp-contract=off"],
    "kernels/move.hip": [],
    # (the CPU's quantisation arithmetic, operation by operation)
    "kernels/quantize.hip": ["-ffp-contract=off"],
    "kernels/util.hip": [],
    "kernels/probe.hip": [],
}


def _headers():
    out = [os.path.join(os.path.dirname(HERE), "include", "vkt.h")]
    for root, _, files in os.walk(CSRC):
        out += [os.path.join(root, f) for f in files if f.endswith(".h")]
    return out


def _stale(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def _compile(job):
    src, obj, extra = job
    cmd = [HIPCC] + FLAGS + extra + ["-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    return r.returncode, " ".join(cmd), err


def build(force=False, verbose=True):
    """Compiles every HIP source and links the library.  Returns the library path."""
    os.makedirs(OUT, exist_ok=True)
    os.makedirs(LIBDIR, exist_ok=True)
    headers = _headers()
    jobs, objs = [], []
    for rel, extra in SOURCES.items():
        src = os.path.join(CSRC, rel)
        obj = os.path.join(OUT, rel.replace("/", "_").replace(".hip", ".o"))
        objs.append(obj)
        if force or _stale(obj, [src] + headers):
            jobs.append((src, obj, extra))
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, max(1, len(jobs)))) as ex:
        for rc, cmd, err in ex.map(_compile, jobs):
            if verbose and err.strip():
                print(err, file=sys.stderr)
            if rc != 0:
                raise RuntimeError("hipcc failed: " + cmd + "\n" + err)
    if force or jobs or _stale(LIB, objs):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs + ["-Wl,--no-undefined"]
        subprocess.check_call(cmd)
    # host-only test shim for the allocator policy (no HIP)
    shim = os.path.join(os.path.dirname(HERE), "tests", "pool_shim.cpp")
    if os.path.exists(shim) and (force or _stale(HOSTTEST, [shim] + headers)):
        subprocess.check_call(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-I", os.path.join(CSRC, "core"), "-I", os.path.join(CSRC, "kernels"), "-o", HOSTTEST, shim])
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
