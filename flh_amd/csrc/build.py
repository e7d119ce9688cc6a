"""Build libflh_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

    python -m flh_amd.csrc.build          # or: python flh_amd/csrc/build.py

The library lands next to the package (flh_amd/libflh_hip.so), where flh_amd._lib
looks for it.  Packed float32 instructions are disabled for all device code.
"""
import pathlib
import shutil
import subprocess
import sys

HERE = pathlib.Path(__file__).resolve().parent
OUT = HERE.parent / "libflh_hip.so"
SOURCES = ["capi.hip", "reference_abi.hip", "gemm_i4.hip", "gemm_i4_decode.hip", "gemm_f6.hip", "fwht_quant.hip", "fwht_mfma.hip", "rope_cache.hip", "decode_attention.hip", "prefill_attention.hip"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # matrix-core results land in ordinary VGPRs when a kernel fits 256 registers (no copies out of AGPRs)
    "-mllvm", "-amdgpu-mfma-vgpr-form=1",
    "-Wno-unused-command-line-argument", "-Wno-unknown-attributes",
]


def build(verbose=True, extra=(), out=None, tag=""):
    """Compile every source and link the shared library.  `extra` are additional hipcc
    flags (e.g. -D switches for experiments), `out` another output path, `tag` a suffix
    that keeps the object files of such a build apart."""
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    out = pathlib.Path(out) if out else OUT
    objs = []
    for s in SOURCES:
        o = HERE / (s + tag + ".o")
        cmd = [hipcc, *[f for f in FLAGS if f != "-shared"], *extra, "-c", str(HERE / s), "-o", str(o)]
        if verbose:
            print(" ".join(cmd), flush=True)
        r = subprocess.run(cmd, capture_output=True, text=True)
        msgs = [l for l in (r.stdout + r.stderr).splitlines() if "packed-fp32-ops" not in l]
        if r.returncode:
            raise RuntimeError("hipcc failed for %s:\n%s" % (s, "\n".join(msgs)))
        if verbose and msgs:
            print("\n".join(msgs))
        objs.append(str(o))
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", str(out)]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    for o in objs:
        pathlib.Path(o).unlink(missing_ok=True)
    return out


if __name__ == "__main__":
    build(extra=sys.argv[1:])
