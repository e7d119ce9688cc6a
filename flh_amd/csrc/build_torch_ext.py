"""Build the PyTorch-ROCm extension flh_amd/_flh_torch.so (host-only C++ in front of libflh_hip.so).

    python -m flh_amd.csrc.build_torch_ext

It contains no device code: torch_ext.cpp checks tensors, takes torch's current HIP stream, allocates outputs and
calls the C ABI of libflh_hip.so, which must have been built first (flh_amd/csrc/build.py) and is found at run time
next to the extension ($ORIGIN).
"""
import pathlib
import shutil
import subprocess
import sys
import sysconfig

HERE = pathlib.Path(__file__).resolve().parent
PKG = HERE.parent
NAME = "_flh_torch"
OUT = PKG / (NAME + ".so")


def build(verbose=True):
    from torch.utils import cpp_extension as ce
    import torch
    cxx = shutil.which("g++") or "g++"
    inc = [f"-I{p}" for p in ce.include_paths()] + [f"-I{sysconfig.get_paths()['include']}", "-I/opt/rocm/include"]
    lib_dirs = ce.library_paths()
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    cmd = [cxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           f"-DTORCH_EXTENSION_NAME={NAME}", f"-D_GLIBCXX_USE_CXX11_ABI={abi}", "-DTORCH_API_INCLUDE_EXTENSION_H",
           "-Wno-deprecated-declarations", *inc, str(HERE / "torch_ext.cpp"), "-o", str(OUT),
           *[f"-L{d}" for d in lib_dirs], f"-L{PKG}", "-lflh_hip", "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip",
           "-ltorch", "-ltorch_python", "-Wl,-rpath,$ORIGIN", *[f"-Wl,-rpath,{d}" for d in lib_dirs]]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode:
        raise RuntimeError("building the torch extension failed:\n" + r.stdout + r.stderr)
    if verbose and r.stderr.strip():
        print(r.stderr)
    return OUT


if __name__ == "__main__":
    build()
    sys.exit(0)
