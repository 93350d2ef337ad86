"""Runs components through the product's executor with every kernel in its generated form, on the CPU
emulation of the HIP runtime (shim.cpp), and compares with the C the oracle backend emits for the same
component.  Started as a subprocess by tests/test_generated_kernels_cpu.py with
ILANG_CORE_LIB, ILANG_HIPCC, ILANG_NO_TORCH and ILANG_NO_DISK_CACHE set; ILANG_SHIM_WAVE=1 asks for the
wavefront-per-iteration form of reduction nests (the program option generated.wave), ILANG_SHIM_PARTS=n for
reduction nests with their outermost sequential loop in n parts (generated.parts).
Prints the case name before running it, so a crash (a guard page hit = out-of-bounds access) names its case."""
import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent.parent.parent
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "tests"))

import oracle  # noqa: E402
from i_amd import Component as i, I  # noqa: E402


def rnd(shape, seed):
    return np.random.default_rng(seed).standard_normal(shape, dtype=np.float32)


def flash(split="i:16,j:16", p=""):
    mm_t = i(f"{p}ik*{p}jk~{p}ijk | {split} | {p}jii'j'k") >> i(f"+{p}ijk~{p}ij | {split} | {p}jii'j'k0")
    row_max_shift = (I & i(f">{p}ij~{p}i | {split} | {p}ji0i'j'")) >> i(f"{p}ij-{p}i~{p}ij | {split} | {p}ji01i'j'")
    exp = i(f"^{p}ij~{p}ij | {split} | {p}ji0i'j'")
    row_normalize = (I & i(f"+{p}ij~{p}i | {split} | {p}ji0i'j'")) >> i(f"{p}ij/{p}i~{p}ij | {split} | {p}ji01i'j'")
    mm = i(f"{p}ij*{p}jk~{p}ikj | {split} | {p}ji0i'kj'") >> i(f"+{p}ikj~{p}ik | {split} | {p}jii'kj'0")
    return mm_t >> row_max_shift >> exp >> row_normalize >> mm


def naive(split="i:16,j:16"):
    mm_t = i(f"ik*jk~ijk | {split} | jii'j'k") >> i(f"+ijk~ij | {split} | jii'j'k0")
    row_max_shift = (I & i(f">ij~i | {split} | jii'j'")) >> i(f"ij-i~ij | {split} | 1jii'j'")
    exp = i(f"^ij~ij | {split} | jii'j'")
    row_normalize = (I & i(f"+ij~i | {split} | jii'j'")) >> i(f"ij/i~ij | {split} | 1jii'j'")
    mm = i(f"ij*jk~ikj | {split} | jii'kj'") >> i(f"+ikj~ik | {split} | jii'kj'0")
    return mm_t >> row_max_shift >> exp >> row_normalize >> mm


def softmax_naive(s="i:16,j:16"):
    return (((I & i(f">ij~i|{s}|jii'j'")) >> i(f"ij-i~ij|{s}|1jii'j'")) >> i(f"^ij~ij|{s}|jii'j'")
            >> ((I & i(f"+ij~i|{s}|jii'j'")) >> i(f"ij/i~ij|{s}|1jii'j'")))


def softmax_rowstaged():
    return (((I & i(">ij~i|i:16|ii'j")) >> i("ij-i~ij|i:16|ii'1j")) >> i("^ij~ij|i:16|ii'0j")
            >> ((I & i("+ij~i|i:16|ii'0j")) >> i("ij/i~ij|i:16|ii'01j")))


def batched_naive():
    mm_t = i("bhij*bhkj~bhikj | i:16,k:16 | bhkii'k'j") >> i("+bhikj~bhik | i:16,k:16 | bhkii'k'j0")
    row_max_shift = (I & i(">bhik~bhi | i:16,k:16 | bhkii'k'")) >> i("bhik-bhi~bhik | i:16,k:16 | bh1kii'k'")
    exp = i("^bhik~bhik | i:16,k:16 | bhkii'k'")
    row_normalize = (I & i("+bhik~bhi | i:16,k:16 | bhkii'k'")) >> i("bhik/bhi~bhik | i:16,k:16 | bh1kii'k'")
    mm = i("bhik*bhkj~bhijk | i:16,k:16 | bhkii'jk'") >> i("+bhijk~bhij | i:16,k:16 | bhkii'jk'0")
    return mm_t >> row_max_shift >> exp >> row_normalize >> mm


CASES = {
    "flash 33x17": (flash, [(33, 17)] * 3),
    "flash 48x24 i:32,j:8": (lambda: flash("i:32,j:8"), [(48, 24)] * 3),
    "flash one key": (flash, [(17, 3), (1, 3), (1, 5)]),
    "flash batched": (lambda: flash(p="bh"), [(2, 3, 20, 8)] * 3),
    "naive attention 32x40": (naive, [(32, 40)] * 3),
    "naive attention ragged": (naive, [(21, 12), (37, 12), (37, 9)]),
    "batched naive attention": (batched_naive, [(2, 3, 4, 8)] * 3),
    "softmax naive 20x37": (softmax_naive, [(20, 37)]),
    "softmax naive 1x1": (softmax_naive, [(1, 1)]),
    "softmax naive i:4,j:32": (lambda: softmax_naive("i:4,j:32"), [(9, 70)]),
    "softmax row-staged": (softmax_rowstaged, [(20, 37)]),
    "mm_t": (lambda: i("ik*jk~ijk | i:16,j:16 | jii'j'k") >> i("+ijk~ij | i:16,j:16 | jii'j'k0"), [(100, 40), (70, 40)]),
    "mm_t empty": (lambda: i("ik*jk~ijk | i:16,j:16 | jii'j'k") >> i("+ijk~ij | i:16,j:16 | jii'j'k0"), [(0, 5), (3, 5)]),
    "matmul unfused": (lambda: i("ik*kj~ijk") >> i("+ijk~ij"), [(8, 16), (16, 7)]),
    "matmul fused init site": (lambda: i("ik*kj~ijk|i:2,k:2|ii'jkk'") >> i("+ijk~ij|i:2,k:2|ii'j!kk'0"), [(8, 16), (16, 7)]),
    "row sum": (lambda: i("+ij~i"), [(16, 8)]),
    "column max": (lambda: i(">ij~j"), [(9, 14)]),
    "total": (lambda: i("+ij~."), [(6, 11)]),
    "fanout two outputs": (lambda: i("+ij~i") & i(">ij~j"), [(9, 14)]),
    "swapped fanout": (lambda: ~(i("+ij~i") & i(">ij~j")), [(9, 14)]),
    "scalar operand": (lambda: i("ij*.~ij"), [(6, 11), ()]),
    "two-level split mm_t": (lambda: i("ik*jk~ijk | i:4:2,j:8 | jii'i''j'k") >> i("+ijk~ij | i:4:2,j:8 | jii'i''j'k0"), [(37, 12), (21, 12)]),
    "batched row softmax": (lambda: (((I & i(">bij~bi|i:8|bii'j")) >> i("bij-bi~bij|i:8|bii'1j")) >> i("^bij~bij|i:8|bii'0j")
                                     >> ((I & i("+bij~bi|i:8|bii'0j")) >> i("bij/bi~bij|i:8|bii'01j"))), [(3, 11, 19)]),
    "flash i:128,j:64 (dynamic private tiles)": (lambda: flash("i:128,j:64"), [(150, 24), (200, 24), (200, 24)]),
    "pointwise chain": (lambda: i("ij+ij~ij") >> i("^ij~ij") >> i("$ij~ij"), [(5, 7), (5, 7)]),
    "comparison and logic": (lambda: (i("ij>>ij~ij") & i("ij<=ij~ij")) >> i("ij^^ij~ij"), [(5, 7), (5, 7)]),
    "column min": (lambda: i("<ij~j"), [(9, 14)]),
    "product reduction": (lambda: i("*ij~i"), [(6, 5)]),
    "rank-3 output": (lambda: i("ik*jk~ijk | i:7 | jii'k"), [(20, 6), (9, 6)]),
    "column normalize (two nests)": (lambda: (I & i("+ij~j||ij")) >> i("ij/j~ij||1ij"), [(37, 70)]),
    "column max shift, split": (lambda: (I & i(">ij~j|i:8,j:4|ijj'i'")) >> i("ij-j~ij|i:8,j:4|1ijj'i'"), [(21, 9)]),
    "column max shift, i outermost": (lambda: (I & i(">ij~j||ij")) >> i("ij-j~ij||1ij"), [(21, 9)]),
    "column sum normalize, split j": (lambda: (I & i("+ij~j|j:4|ijj'")) >> i("ij/j~ij|j:4|1ijj'"), [(9, 21)]),
    "mlp with pair": (lambda: (i("ij~ij") | ((i("ij*j~ij") >> i("+ij~i")) >> i(">i~i"))) >> (i("ij*j~ij") >> i("+ij~i")),
                      [(7, 16), (16, 8), (8,)]),
    # reductions long enough for several rounds of a wavefront's 64 lanes, with ragged ends
    "row sum 5x300": (lambda: i("+ij~i"), [(5, 300)]),
    "row max 3x130, split j": (lambda: i(">ij~i|j:16|ijj'"), [(3, 130)]),
    "row min 70x129": (lambda: i("<ij~i"), [(70, 129)]),
    "fused matrix-vector product": (lambda: i("ij*j~ij||ij") >> i("+ij~i||ij0"), [(7, 150), (150,)]),
    "batched row sum": (lambda: i("+bij~bi"), [(3, 5, 200)]),
    "sum over the two last axes": (lambda: i("+bij~b"), [(3, 9, 70)]),
}

# the cases with a nest that has a wavefront-per-iteration form (reduction loops spread over 64 lanes)
WAVE_CASES = ["naive attention ragged", "batched naive attention", "mm_t", "mm_t empty", "matmul unfused",
              "matmul fused init site", "row sum", "column max", "total", "fanout two outputs", "swapped fanout",
              "two-level split mm_t", "column min", "product reduction", "mlp with pair", "row sum 5x300",
              "row max 3x130, split j", "row min 70x129", "fused matrix-vector product", "batched row sum",
              "sum over the two last axes"]


# a sample for the runs that repeat the suite under another option: every kind of reduction nest, kernels of several
# nests, fused kernels with private tiles
SAMPLE_CASES = ["flash 33x17", "naive attention ragged", "softmax naive 20x37", "mm_t", "mm_t empty", "matmul fused init site", "column max",
                "total", "fanout two outputs", "two-level split mm_t", "product reduction", "column normalize (two nests)",
                "column sum normalize, split j", "mlp with pair", "row sum 5x300", "row max 3x130, split j", "fused matrix-vector product",
                "sum over the two last axes"]


# Components with a reduced vector staged at the root of its consumer are checked against NumPy as well: the emitted
# C comes out of the same lowering, and the reference's lowering mis-addresses that vector when producer and
# consumer number the shared index differently (fixed here, see compiler/stage_to_kernels.cpp lower_read).
CLOSED_FORMS = {
    "column normalize (two nests)": lambda x: x / x.sum(axis=0),
    "column max shift, split": lambda x: x - x.max(axis=0),
    "column max shift, i outermost": lambda x: x - x.max(axis=0),
    "column sum normalize, split j": lambda x: x / x.sum(axis=0),
}


def run_without_allocating(comp, inputs):
    """The same call through i_exec_into_device_noalloc: on the emulated runtime device memory is host memory, so
    NumPy buffers stand in for device tensors.  Temporaries then come out of the fixed workspace."""
    import ctypes

    from i_amd import _native as nat, ilang

    operands = [ilang._operand(x, "input") for x in inputs]
    outs = [np.full(shape, np.nan, dtype=np.float32) for shape in comp.output_shapes(*inputs)]
    targets = [ilang._operand(o, "output") for o in outs]
    in_records, keep_in = ilang._pack(operands, on_device=True)
    out_records, keep_out = ilang._pack(targets, on_device=True)
    nat.check(nat.core.i_exec_into_device_noalloc(comp._compile(), in_records, len(operands), out_records, len(targets), None))
    return outs[0] if len(outs) == 1 else tuple(outs)


def main():
    import os

    noalloc = os.environ.get("ILANG_SHIM_NOALLOC") == "1"
    which = os.environ.get("ILANG_SHIM_CASES")
    names = sys.argv[1:] or (WAVE_CASES if which == "wave" else SAMPLE_CASES if which == "sample" else list(CASES))
    tolerance = float(os.environ.get("ILANG_SHIM_TOLERANCE", "1e-5"))
    failed = []
    for name in names:
        build, shapes = CASES[name]
        print("CASE", name, flush=True)
        comp = build()
        comp.option("generated.only", 1)
        if os.environ.get("ILANG_SHIM_WAVE") is not None:
            comp.option("generated.wave", int(os.environ["ILANG_SHIM_WAVE"]))
        if os.environ.get("ILANG_SHIM_PARTS") is not None:
            comp.option("generated.parts", int(os.environ["ILANG_SHIM_PARTS"]))
        inputs = [rnd(s, k + 1) for k, s in enumerate(shapes)]
        got = run_without_allocating(comp, inputs) if noalloc else comp.exec_numpy(*inputs)
        ref = oracle.compile_component(comp.handle).run(*inputs)
        got = got if isinstance(got, tuple) else (got,)
        ref = ref if isinstance(ref, tuple) else (ref,)
        if name in CLOSED_FORMS:
            ref = (CLOSED_FORMS[name](*inputs),) + tuple(ref)   # NumPy closed form first, then the emitted C
            got = (got[0],) + tuple(got)
        for g, r in zip(got, ref):
            scale = float(np.abs(r).max()) if r.size else 1.0
            err = float(np.abs(g - r).max()) / (scale or 1.0) if r.size else 0.0
            ok = g.shape == r.shape and (r.size == 0 or (np.isfinite(g).all() and err <= tolerance))
            if not ok:
                failed.append(name)
                print("MISMATCH", name, g.shape, r.shape, err, flush=True)
    print("DONE", len(names), "cases;", "failed:", failed, flush=True)
    sys.exit(1 if failed else 0)


if __name__ == "__main__":
    main()
