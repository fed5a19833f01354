"""Build the reference's own host C++ (KVStorage, BatchScheduler) into oracle/_ref/.

TEST INFRASTRUCTURE ONLY.  The two translation units are compiled from where
they lie under the reference checkout (nothing is copied into this
repository); the resulting pybind11 modules are used solely to pin
oracle/host_oracle.py and to generate the fixtures under tests/golden/.

Sources compiled (reference paths):
    csrc/memory_manager.cpp   -> oracle/_ref/memory_manager.so
    csrc/batch_scheduler.cpp  -> oracle/_ref/batch_scheduler.so

The reference declares these as torch extensions (setup.py:130-147) although
they contain only host code, so a plain g++ line against the installed torch /
pybind11 / CPython headers is enough.
"""
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
OUT = os.path.join(HERE, "_ref")
REFERENCE = os.environ.get("MUX_REFERENCE_DIR", "/root/reference")

UNITS = {
    "memory_manager": "csrc/memory_manager.cpp",
    "batch_scheduler": "csrc/batch_scheduler.cpp",
}


def available() -> bool:
    return all(os.path.exists(os.path.join(REFERENCE, p)) for p in UNITS.values())


def build(verbose: bool = True) -> bool:
    """Compile both units.  Returns False (and builds nothing) when the
    reference checkout is not present, e.g. on a GPU box."""
    if not available():
        if verbose:
            print(f"[build_ref] {REFERENCE} not present; keeping prebuilt oracle/_ref")
        return False
    from torch.utils import cpp_extension as ce
    import torch

    os.makedirs(OUT, exist_ok=True)
    inc = ce.include_paths() + [sysconfig.get_paths()["include"]]
    libdir = ce.library_paths()[0]
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    procs = []
    for name, rel in UNITS.items():
        src = os.path.join(REFERENCE, rel)
        out = os.path.join(OUT, name + ".so")
        cmd = ["g++", "-std=c++17", "-O2", "-g0", "-fPIC", "-shared", "-w",
               f"-DTORCH_EXTENSION_NAME={name}", f"-D_GLIBCXX_USE_CXX11_ABI={abi}",
               "-DTORCH_API_INCLUDE_EXTENSION_H"]
        for i in inc:
            cmd += ["-isystem", i]
        cmd += [src, "-o", out, f"-L{libdir}", f"-Wl,-rpath,{libdir}",
                "-ltorch_python", "-ltorch", "-ltorch_cpu", "-lc10"]
        if verbose:
            print("[build_ref]", " ".join(cmd))
        procs.append((name, subprocess.Popen(cmd)))
    ok = True
    for name, p in procs:
        if p.wait() != 0:
            print(f"[build_ref] FAILED: {name}", file=sys.stderr)
            ok = False
    if not ok:
        raise RuntimeError("reference host C++ did not compile")
    return True


def load():
    """Import the two compiled reference modules (None, None if absent)."""
    import importlib.util
    import torch  # noqa: F401  (the modules link against libtorch)

    mods = []
    for name in UNITS:
        path = os.path.join(OUT, name + ".so")
        if not os.path.exists(path):
            return None, None
        spec = importlib.util.spec_from_file_location(name, path)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        mods.append(mod)
    return tuple(mods)


if __name__ == "__main__":
    build()
