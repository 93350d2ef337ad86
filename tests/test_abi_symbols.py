"""The shared library loads on a machine without a GPU and exports every symbol
that include/*.h declares.  No compute call is made here."""
import ctypes
import re
from pathlib import Path

ROOT = Path(__file__).resolve().parents[1]


def declared_symbols():
    names = set()
    for header in sorted((ROOT / "include").glob("*.h")):
        text = re.sub(r"/\*.*?\*/", "", header.read_text(), flags=re.S)
        text = re.sub(r"//[^\n]*", "", text)
        names |= set(re.findall(r"\b(i_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(str(ROOT / "i_amd" / "libi_core.so"))
    names = declared_symbols()
    assert "i_error" in names and "i_hip_attention" in names
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, f"declared in include/ but not exported: {missing}"


def test_code_object_is_present_and_gfx950():
    blob = (ROOT / "i_amd" / "i_kernels_gfx950.hsaco").read_bytes()
    assert blob[:4] == b"\x7fELF" or blob.startswith(b"__CLANG_OFFLOAD_BUNDLE__")
    assert b"attn_fwd_bf16_d128_bn64" in blob and b"row_softmax_wave_v16" in blob
