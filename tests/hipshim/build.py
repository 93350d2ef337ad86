"""Builds tests/hipshim/_build/libi_core_shim.so: the product's host sources linked against shim.cpp
instead of the HIP runtime, for the CPU emulation tests."""
import subprocess
import sys
from pathlib import Path

HERE = Path(__file__).resolve().parent
ROOT = HERE.parent.parent
OUT = HERE / "_build" / "libi_core_shim.so"


def build():
    sys.path.insert(0, str(ROOT))
    from i_amd.build import ROCM, host_sources

    srcs = host_sources() + [HERE / "shim.cpp"]
    if OUT.exists() and all(OUT.stat().st_mtime > p.stat().st_mtime for p in srcs + list((ROOT / "i_amd" / "csrc").rglob("*.h"))):
        return OUT
    OUT.parent.mkdir(exist_ok=True)
    subprocess.run(["g++", "-O1", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden", "-Wno-unused-function",
                    "-D__HIP_PLATFORM_AMD__", f"-I{ROCM / 'include'}", f"-I{ROOT / 'include'}",
                    *map(str, srcs), "-o", str(OUT), "-ldl", "-lpthread"], check=True)
    return OUT


if __name__ == "__main__":
    print(build())
