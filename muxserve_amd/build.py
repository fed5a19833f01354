"""Compile the shared libraries of the package, in-tree.

    libmuxhost.so  - g++,   pure host C++ (allocator + batch builder)
    libmuxattn.so  - hipcc, gfx950 kernels + their C ABI
    libmuxtorch.so - g++,   thin TORCH_LIBRARY operators over libmuxattn.so's C ABI
    libmuxprobe.so - hipcc, a bare gather-read kernel: bench.py's yardstick, not product
    libmuxattn_trace.so - hipcc, libmuxattn.so built with -DMUX_TRACE (per-workgroup phase
                     stamps in the decode kernel) for `bench.py --workload decode_timeline`;
                     built on request only (`python -m muxserve_amd.build trace`), never loaded
                     by the package

Run as ``python -m muxserve_amd.build``.  Nothing here runs at import time of
the package: the loaders in muxserve_amd._lib only open what this step built
and raise if it is missing.
"""
import os
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
INCLUDE = os.path.join(ROOT, "include")
CSRC = os.path.join(PKG, "csrc")

HOST_LIB = os.path.join(PKG, "libmuxhost.so")
ATTN_LIB = os.path.join(PKG, "libmuxattn.so")
TORCH_LIB = os.path.join(PKG, "libmuxtorch.so")
PROBE_LIB = os.path.join(PKG, "libmuxprobe.so")
TRACE_LIB = os.path.join(PKG, "libmuxattn_trace.so")
PROBE_SOURCES = [os.path.join(CSRC, "probe", "probe.hip")]
TORCH_SOURCES = [os.path.join(CSRC, "torch", "mux_torch_ops.cpp")]

HOST_SOURCES = [os.path.join(CSRC, "host", f) for f in ("kv_storage.cpp", "batch_scheduler.cpp")]
HIP_SOURCES = [os.path.join(CSRC, "hip", f) for f in (
    "cache_write.hip", "paged_decode.hip", "prefill.hip", "rotary.hip", "model_ops.hip", "sampler.hip",
    "step_tables.hip", "runtime.hip")]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# Packed-FP32 instruction selection is switched off for every device
# translation unit (ordinary float code otherwise compiles to v_pk_*_f32).
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-fno-gpu-rdc", "-Wno-unused-command-line-argument"]


def _run(cmd):
    print("[build]", " ".join(cmd), flush=True)
    subprocess.check_call(cmd)


def build_host():
    _run(["g++", "-std=c++17", "-O2", "-fPIC", "-shared", "-Wall", "-Wextra",
          f"-I{INCLUDE}", *HOST_SOURCES, "-o", HOST_LIB])
    return HOST_LIB


def _compile_and_link(out, extra=(), tag="o"):
    """One hipcc -c per translation unit, side by side (they are independent:
    -fno-gpu-rdc), then one link step."""
    from concurrent.futures import ThreadPoolExecutor
    objdir = os.path.join(CSRC, "build")
    os.makedirs(objdir, exist_ok=True)
    flags = [f for f in HIP_FLAGS if f != "-shared"]
    jobs = []
    for src in HIP_SOURCES:
        obj = os.path.join(objdir, os.path.basename(src) + "." + tag)
        jobs.append(([HIPCC, *flags, *extra, f"-I{INCLUDE}", f"-I{os.path.join(CSRC, 'hip')}", "-c", src, "-o", obj], obj))
    with ThreadPoolExecutor(max_workers=min(8, len(jobs))) as pool:
        list(pool.map(lambda j: _run(j[0]), jobs))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", *[j[1] for j in jobs], "-o", out])
    return out


def build_hip(extra=()):
    return _compile_and_link(ATTN_LIB, extra)


def build_trace():
    return _compile_and_link(TRACE_LIB, ("-DMUX_TRACE",), tag="trace.o")


def build_probe():
    _run([HIPCC, *HIP_FLAGS, f"-I{os.path.join(CSRC, 'probe')}", *PROBE_SOURCES, "-o", PROBE_LIB])
    return PROBE_LIB


def build_torch():
    """The operator library: host C++ only (no device code), linked against
    torch's libraries and libmuxattn.so next to it."""
    import torch
    from torch.utils import cpp_extension
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = ["g++", "-std=c++17", "-O2", "-fPIC", "-shared", "-w", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}", f"-I{INCLUDE}"]
    for inc in cpp_extension.include_paths() + ["/opt/rocm/include"]:
        cmd += ["-isystem", inc]
    cmd += [*TORCH_SOURCES, "-o", TORCH_LIB, f"-L{tlib}", f"-L{PKG}", "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{tlib}",
            "-l:libmuxattn.so", "-ltorch", "-ltorch_cpu", "-lc10", "-lc10_hip"]
    _run(cmd)
    return TORCH_LIB


def build_all():
    build_host()
    build_hip()
    build_torch()
    build_probe()


if __name__ == "__main__":
    what = sys.argv[1] if len(sys.argv) > 1 else "all"
    {"host": build_host, "hip": build_hip, "torch": build_torch, "probe": build_probe, "trace": build_trace,
     "all": build_all}[what]()
