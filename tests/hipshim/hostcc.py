#!/usr/bin/env python3
"""Stands in for hipcc in the CPU emulation tests (ILANG_HIPCC points here): compiles the generated HIP
source as host C++ into a shared object.  Takes hipcc's command line (flags, source, -o output)."""
import subprocess
import sys
from pathlib import Path

args = sys.argv[1:]
out = args[args.index("-o") + 1]
src = [a for a in args if a.endswith(".hip")][0]
inc = Path(__file__).resolve().parent / "include"
sys.exit(subprocess.run(["g++", "-shared", "-fPIC", "-O1", "-std=c++17", f"-I{inc}", "-x", "c++", src, "-o", out]).returncode)
