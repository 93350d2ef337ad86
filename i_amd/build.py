"""Builds the two native artefacts of the backend, in-tree:

  i_amd/i_kernels_gfx950.hsaco   device code object (hipcc --genco, gfx950 only)
  i_amd/libi_core.so             host runtime + compiler (C++17), linked to libamdhip64

Run as  python -m i_amd.build  (or call build()).  hipcc cross-compiles, no GPU needed.
"""
import os
import subprocess
import sys
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
ROCM = Path(os.environ.get("ROCM_PATH", "/opt/rocm"))
HSACO = PKG / "i_kernels_gfx950.hsaco"
LIB = PKG / "libi_core.so"

# packed-fp32 VALU forms are disabled for all device code on purpose.
HIPCC_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _run(cmd):
    print("+", " ".join(str(c) for c in cmd), flush=True)
    subprocess.run([str(c) for c in cmd], check=True)


def host_sources():
    return sorted(p for p in CSRC.rglob("*.cpp"))


def build_kernels():
    _run([ROCM / "bin" / "hipcc", "--genco", *HIPCC_FLAGS, CSRC / "kernels" / "kernels.hip", "-o", HSACO])


def build_static_scratch():
    """The one host + device source: the fixed device workspace (a file-scope __device__ array) and its lookup."""
    obj = CSRC / "runtime" / "static_scratch.o"
    _run([ROCM / "bin" / "hipcc", "-c", "-fPIC", "-O2", "-std=c++17", "--offload-arch=gfx950",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
          CSRC / "runtime" / "static_scratch.hip", "-o", obj])
    return obj


def build_host():
    scratch_obj = build_static_scratch()
    _run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-fvisibility=hidden", "-Wno-unused-function",
          "-D__HIP_PLATFORM_AMD__", f"-I{ROCM / 'include'}", f"-I{PKG.parent / 'include'}",
          *host_sources(), scratch_obj, "-o", LIB,
          f"-L{ROCM / 'lib'}", "-lamdhip64", f"-Wl,-rpath,{ROCM / 'lib'}", "-ldl", "-lpthread"])


def build():
    build_kernels()
    build_host()


if __name__ == "__main__":
    build()
    sys.exit(0)
