"""Writes tests/golden/flashattn_ref.npz.

Runs the reference's own emitted C for the demo FlashAttention component
(ilang-python/annotated-flashattn.c, compiled unmodified into
oracle/_ref/libflashattn_ref.so by oracle/Makefile) on small seeded inputs and
stores inputs and outputs.  Only runs where the reference tree is mounted; the
committed .npz is what travels.

Cases follow the reference's own input recipes:
  uniform(-1,1) seeds 1,2,3        (BASELINE config 1 recipe)
  standard_normal seeds 1,2,3      (ilang-python/flash-attn.py:31-36, test.py:27-29)
"""
import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))
import oracle  # noqa: E402

CASES = [
    ("u_48x24", "uniform", 48, 24),
    ("u_64x64", "uniform", 64, 64),
    ("u_100x40", "uniform", 100, 40),   # ragged: 100 = 6*16 + 4
    ("n_48x24", "normal", 48, 24),
    ("n_33x17", "normal", 33, 17),      # ragged in both tile loops
    ("n_16x130", "normal", 16, 130),    # one tile, wide head
]


def inputs(kind, n, d):
    out = []
    for seed in (1, 2, 3):
        rng = np.random.default_rng(seed)
        if kind == "uniform":
            out.append(rng.uniform(-1, 1, (n, d)).astype(np.float32))
        else:
            out.append(rng.standard_normal((n, d), dtype=np.float32))
    return out


def main():
    oracle.build()
    assert oracle.have_ref(), "reference tree not mounted: cannot regenerate goldens"
    blobs = {}
    for name, kind, n, d in CASES:
        q, k, v = inputs(kind, n, d)
        o = oracle.ref_flash_attention(q, k, v)
        blobs[f"{name}.q"], blobs[f"{name}.k"], blobs[f"{name}.v"], blobs[f"{name}.o"] = q, k, v, o
    np.savez_compressed(Path(__file__).with_name("flashattn_ref.npz"), **blobs)
    print("wrote", len(CASES), "cases")

    # checksum of the reference's emitted C for the demo component, comments and
    # whitespace removed: pins the whole lowering pipeline + C printer byte for byte
    import hashlib
    import re

    text = Path("/root/reference/ilang-python/annotated-flashattn.c").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    text = re.sub(r"\s+", "", text)
    Path(__file__).with_name("flashattn_emitted.sha256").write_text(
        f"{hashlib.sha256(text.encode()).hexdigest()}  {len(text)}\n")


if __name__ == "__main__":
    main()
