"""The PyTorch device "vk" on MI355X: ``import torch_vulkan_amd.backend`` does what
``import torch_vulkan`` does in the reference (python/torch_vulkan/__init__.py:29-52,151-210)
for the quantized-matmul path: renames the PrivateUse1 backend to "vk", loads the C++
backend (allocator, device guard, copies, CPU fallback, the five quantised aten ops), and
registers the device module ``torch.vk``.

    import torch, torch_vulkan_amd.backend as tv
    y = torch._weight_int8pack_mm(x.to("vk"), w.to("vk"), s.to("vk")).cpu()
"""
import atexit
import ctypes
import os
import subprocess
import sys
import types

import torch

from . import abi

_HERE = os.path.dirname(os.path.abspath(__file__))
_SRC = os.path.join(_HERE, "csrc", "torch")
LIB_PATH = os.path.join(_HERE, "lib", "libvk_torch_backend.so")
_lib = None


def build(force=False):
    """Compiles the C++ backend against the installed torch (g++; no GPU or HIP needed)."""
    from torch.utils import cpp_extension
    srcs = [os.path.join(_SRC, f) for f in ("backend.cpp", "quant.cpp", "linalg.cpp", "quantized.cpp")]
    deps = srcs + [os.path.join(_SRC, "vk.h"), os.path.join(os.path.dirname(_HERE), "include", "vkt.h")]
    if not force and os.path.exists(LIB_PATH) and all(os.path.getmtime(d) <= os.path.getmtime(LIB_PATH) for d in deps):
        return LIB_PATH
    os.makedirs(os.path.dirname(LIB_PATH), exist_ok=True)
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    objs = []
    jobs = []
    for src in srcs:
        obj = os.path.join(_HERE, "_build", "torch_" + os.path.basename(src).replace(".cpp", ".o"))
        os.makedirs(os.path.dirname(obj), exist_ok=True)
        cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function", "-Wno-unknown-pragmas",
               f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}", "-c", src, "-o", obj]
        for inc in cpp_extension.include_paths():
            cmd += ["-isystem", inc]
        jobs.append(subprocess.Popen(cmd))
        objs.append(obj)
    for j in jobs:
        if j.wait() != 0:
            raise RuntimeError("g++ failed on the torch backend")
    subprocess.check_call(["g++", "-shared", "-fPIC", "-o", LIB_PATH] + objs +
                          [f"-L{tlib}", "-ltorch_cpu", "-lc10", "-ltorch", f"-L{os.path.dirname(abi.LIB_PATH)}",
                           "-lvkt_mi355", "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{tlib}", "-Wl,--no-undefined"])
    return LIB_PATH


def _load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise abi.VktError(f"{LIB_PATH} is missing: build it with `python -c 'import torch_vulkan_amd.backend as b; b.build()'`"
                           if False else f"{LIB_PATH} is missing: run torch_vulkan_amd.backend.build()")
    abi.lib()  # libvkt_mi355.so first, so that both share one runtime
    torch.utils.rename_privateuse1_backend("vk")
    _lib = ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_GLOBAL)
    _lib.vkt_register_backend()
    _lib.vkt_fallback_counts.restype = ctypes.c_size_t
    _lib.vkt_fallback_counts.argtypes = [ctypes.c_char_p, ctypes.c_size_t]
    torch.utils.generate_methods_for_privateuse1_backend(for_tensor=True, for_module=True, for_storage=True)
    torch._register_device_module("vk", _device_module())
    atexit.register(shutdown)
    return _lib


# ------------------------------------------------------------------ the user API of the reference's package
def is_available():
    """True if the library finds a gfx950 device (reference __init__.py:65-70)."""
    return bool(abi.lib().vkt_capabilities())


def synchronize(device=None):
    abi.synchronize()


def memory_stats(device=None):
    a, r = abi.u64(), abi.u64()
    abi.lib().vkt_memory_stats(ctypes.byref(a), ctypes.byref(r))
    return {"allocated_bytes": a.value, "reserved_bytes": r.value}


def empty_cache():
    abi.check(abi.lib().vkt_empty_cache())


def fallback_counts():
    """{op name: times it ran on the CPU instead of the GPU} (reference __init__.py:107-123)."""
    lib = _load()
    n = lib.vkt_fallback_counts(None, 0)
    buf = ctypes.create_string_buffer(n)
    lib.vkt_fallback_counts(buf, n)
    out = {}
    for line in buf.value.decode().splitlines():
        k, _, v = line.rpartition("=")
        out[k] = int(v)
    return out


def capabilities():
    return abi.lib().vkt_capabilities()


def kernel_subgroup_size(name):
    """Lanes per wave the kernel `name` runs with, 0 if the library has no such kernel (reference _native.kernel_subgroup_size)."""
    return abi.lib().vkt_kernel_subgroup_size(name.encode())


def dispatch_count():
    return abi.lib().vkt_dispatch_count()


def shutdown():
    abi.lib().vkt_shutdown()


def _device_module():
    m = types.ModuleType("torch.vk")
    m.is_available = is_available
    m.is_initialized = lambda: True
    m.device_count = lambda: 1
    m.current_device = lambda: 0
    m.set_device = lambda d: None
    m.synchronize = synchronize
    m.memory_stats = memory_stats
    m.empty_cache = empty_cache
    m.fallback_counts = fallback_counts
    m._is_in_bad_fork = lambda: False
    m.manual_seed_all = lambda seed: None
    m.get_rng_state = lambda device=None: torch.empty(0, dtype=torch.uint8)
    m.set_rng_state = lambda state, device=None: None
    return m


if os.environ.get("TORCH_VULKAN_AMD_NO_AUTOLOAD") != "1" and os.path.exists(LIB_PATH):
    _load()
