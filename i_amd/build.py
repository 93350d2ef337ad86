"""Builds the two native artefacts of the backend, in-tree:

  i_amd/i_kernels_gfx950.hsaco   device code object (hipcc --genco, gfx950 only)
  i_amd/libi_core.so             host runtime + compiler (C++17), linked to libamdhip64

Run as  python -m i_amd.build  (or call build()).  hipcc cross-compiles, no GPU needed.
"""
import os
import re
import subprocess
import sys
import tempfile
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


def inline_mfma_hazards(asm_text):
    """Kernels whose matrix instructions are inline assembly (the four-wave GEMMs, named ..._w4) are outside the
    compiler's hazard handling: a matrix instruction may read a register two wait states after an ordinary vector
    instruction wrote it at the earliest.  The kernels are written so that no such pair exists; this walks the
    compiled assembly and returns the pairs it finds all the same (a later compiler might place a copy there)."""
    def regs(token):
        m = re.match(r"([va])\[(\d+):(\d+)\]", token)
        if m:
            return {(m.group(1), r) for r in range(int(m.group(2)), int(m.group(3)) + 1)}
        m = re.match(r"([va])(\d+)$", token)
        return {(m.group(1), int(m.group(2)))} if m else set()

    found = []
    for name, body in re.findall(r"^(\w+_w4):\n(.*?)\.end_amdhsa_kernel", asm_text, re.S | re.M):
        lines = [l.strip() for l in body.splitlines()]
        lines = [l for l in lines if l and not l.startswith((";", ".", "//")) and not l.endswith(":")]
        for n, line in enumerate(lines):
            if not line.startswith("v_mfma"):
                continue
            sources = set().union(*[regs(t.strip()) for t in line.split(None, 1)[1].split(",")[1:]])
            waited = 0
            for before in reversed(lines[max(0, n - 8):n]):
                if before.startswith("s_nop"):
                    waited += int(before.split()[1]) + 1
                    continue
                if waited >= 2:
                    break
                if before.startswith("v_") and not before.startswith("v_mfma"):
                    if regs(before.split(None, 1)[1].split(",")[0].strip()) & sources:
                        found.append(f"{name}: {before}  ->  {line}")
                waited += 1
    return found


def build_kernels():
    with tempfile.TemporaryDirectory() as tmp:
        # (the intermediate assembly lands in the working directory: it is read for the check below)
        print("+ cd", tmp, flush=True)
        cmd = [ROCM / "bin" / "hipcc", "--genco", *HIPCC_FLAGS, "-save-temps", CSRC / "kernels" / "kernels.hip", "-o", HSACO]
        print("+", " ".join(str(c) for c in cmd), flush=True)
        subprocess.run([str(c) for c in cmd], check=True, cwd=tmp)
        listings = list(Path(tmp).glob("*gfx950*.s"))
        if not listings:
            raise RuntimeError("hipcc left no gfx950 assembly to check")
        hazards = inline_mfma_hazards(listings[0].read_text())
        if hazards:
            raise RuntimeError("inline matrix instructions too close to a vector write of their operands:\n" + "\n".join(hazards))


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
