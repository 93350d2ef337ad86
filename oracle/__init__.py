"""ctypes access to the CPU oracle (test infrastructure, not product code).

Only the test-suite, the smoke check and the benchmark's cpu_baseline leg may
import this package.  It wraps

* ``liboracle.so``  - oracle.c, the scalar restatement of the loop nests the
  reference C backend emits for the FlashAttention / mm_t / row-softmax
  components, and
* ``_ref/libflashattn_ref.so`` - the reference's own emitted C
  (ilang-python/annotated-flashattn.c) compiled unmodified, reached through
  the generated-library ABI ``count/ranks/shapes/exec`` (ABI.md:4-9).

plus float64 NumPy closed forms used to pin both.
"""
import ctypes
import os
import subprocess
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
_LIB = HERE / "liboracle.so"
_REF = HERE / "_ref" / "libflashattn_ref.so"

_f32p = ctypes.POINTER(ctypes.c_float)
_sz = ctypes.c_size_t


def build():
    """Compile oracle.c (and the reference emission when its tree is mounted)."""
    subprocess.run(["make", "-s", "-C", str(HERE)], check=True)


def _load():
    if not _LIB.exists():
        build()
    lib = ctypes.CDLL(str(_LIB))
    lib.oracle_attention_tiled.argtypes = [_f32p, _f32p, _f32p, _f32p, _sz, _sz, _sz, _sz, _sz,
                                           ctypes.c_int, ctypes.c_float, _sz, _sz]
    lib.oracle_attention_tiled.restype = ctypes.c_int
    lib.oracle_attention_naive.argtypes = [_f32p, _f32p, _f32p, _f32p, _sz, _sz, _sz, _sz, _sz,
                                           ctypes.c_int, ctypes.c_float]
    lib.oracle_attention_naive.restype = ctypes.c_int
    lib.oracle_mm_t.argtypes = [_f32p, _f32p, _f32p, _sz, _sz, _sz, _sz]
    lib.oracle_mm_t.restype = ctypes.c_int
    lib.oracle_row_softmax.argtypes = [_f32p, _f32p, _sz, _sz]
    lib.oracle_row_softmax.restype = ctypes.c_int
    return lib


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = _load()
    return _lib


def _p(a):
    return a.ctypes.data_as(_f32p)


def _c(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def attention_tiled(q, k, v, scale=None, ti=16, tj=16):
    """Blockwise online-softmax attention over the trailing two axes."""
    q, k, v = _c(q), _c(k), _c(v)
    lead = q.shape[:-2]
    bh = int(np.prod(lead)) if lead else 1
    nq, d = q.shape[-2:]
    nk, dv = v.shape[-2:]
    # np.empty on purpose: the reference frontend hands the kernel
    # uninitialised output memory (ilang-python/ilang.py:334).
    o = np.empty(lead + (nq, dv), dtype=np.float32)
    o.fill(np.float32(123.0))
    rc = lib().oracle_attention_tiled(_p(q), _p(k), _p(v), _p(o), bh, nq, nk, d, dv,
                                      0 if scale is None else 1,
                                      0.0 if scale is None else float(np.float32(scale)), ti, tj)
    assert rc == 0
    return o


def attention_naive(q, k, v, scale=None):
    q, k, v = _c(q), _c(k), _c(v)
    lead = q.shape[:-2]
    bh = int(np.prod(lead)) if lead else 1
    nq, d = q.shape[-2:]
    nk, dv = v.shape[-2:]
    o = np.empty(lead + (nq, dv), dtype=np.float32)
    rc = lib().oracle_attention_naive(_p(q), _p(k), _p(v), _p(o), bh, nq, nk, d, dv,
                                      0 if scale is None else 1,
                                      0.0 if scale is None else float(np.float32(scale)))
    assert rc == 0
    return o


def mm_t(a, b):
    a, b = _c(a), _c(b)
    lead = a.shape[:-2]
    bh = int(np.prod(lead)) if lead else 1
    m, kk = a.shape[-2:]
    n = b.shape[-2]
    c = np.empty(lead + (m, n), dtype=np.float32)
    assert lib().oracle_mm_t(_p(a), _p(b), _p(c), bh, m, n, kk) == 0
    return c


def row_softmax(x):
    x = _c(x)
    rows = int(np.prod(x.shape[:-1]))
    y = np.empty_like(x)
    assert lib().oracle_row_softmax(_p(x), _p(y), rows, x.shape[-1]) == 0
    return y


# ---------------------------------------------------------------- reference emission
class _Tensor(ctypes.Structure):
    _fields_ = [("data", _f32p), ("shape", ctypes.POINTER(_sz)), ("rank", _sz)]


def have_ref():
    return _REF.exists()


def ref_flash_attention(q, k, v):
    """Run the compiled reference emission (2-D f32 q, k, v) through ABI #2."""
    r = ctypes.CDLL(str(_REF))
    r.count.restype = _sz
    q, k, v = _c(q), _c(k), _c(v)
    shapes = [(_sz * 2)(*a.shape) for a in (q, k, v)]
    ins = (_Tensor * 3)(*[_Tensor(_p(a), s, 2) for a, s in zip((q, k, v), shapes)])
    assert r.count() == 1
    ranks = (_sz * 1)()
    r.ranks(ranks)
    assert ranks[0] == 2
    oshape = (_sz * 2)()
    oshape_p = (ctypes.POINTER(_sz) * 1)(ctypes.cast(oshape, ctypes.POINTER(_sz)))
    r.shapes(ins, oshape_p)
    o = np.empty((oshape[0], oshape[1]), dtype=np.float32)
    o.fill(np.float32(123.0))
    outs = (_Tensor * 1)(_Tensor(_p(o), oshape, 2))
    r.exec(ins, outs)
    return o


# ---------------------------------------------------------------- closed forms (fp64)
def np_attention64(q, k, v, scale=None):
    q, k, v = (np.asarray(a, dtype=np.float64) for a in (q, k, v))
    s = q @ np.swapaxes(k, -1, -2)
    if scale is not None:
        s = s * float(np.float32(scale))
    s = s - s.max(axis=-1, keepdims=True)
    w = np.exp(s)
    w = w / w.sum(axis=-1, keepdims=True)
    return w @ v


def np_softmax64(x):
    x = np.asarray(x, dtype=np.float64)
    e = np.exp(x - x.max(axis=-1, keepdims=True))
    return e / e.sum(axis=-1, keepdims=True)


def np_mm_t64(a, b):
    return np.asarray(a, np.float64) @ np.swapaxes(np.asarray(b, np.float64), -1, -2)


def to_bf16_f32(x):
    """Round f32 values to the nearest bf16 (ties to even), returned widened to f32."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return r.astype(np.uint32).view(np.float32).reshape(x.shape)


def bf16_bits(x):
    """uint16 bf16 bit patterns of f32 values that are already bf16-representable."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    return (x.view(np.uint32) >> 16).astype(np.uint16).reshape(x.shape)


# ---------------------------------------------------------------- C text backend (arbitrary components)
_CB = HERE / "liboracle_cbackend.so"
_cb = None


def _cbackend():
    global _cb
    if _cb is None:
        if not _CB.exists():
            build()
        _cb = ctypes.CDLL(str(_CB))
        _cb.oracle_emit_c.restype = ctypes.c_void_p
        _cb.oracle_emit_c.argtypes = [ctypes.c_void_p]
        _cb.oracle_c_error.restype = ctypes.c_char_p
    return _cb


def emit_c(component_ptr):
    """C source the reference C backend would print for a component handle
    (an ``i_component*`` made through libi_core's i_parse / combinators)."""
    lib_ = _cbackend()
    raw = lib_.oracle_emit_c(component_ptr)
    if not raw:
        raise RuntimeError(lib_.oracle_c_error().decode())
    try:
        return ctypes.cast(raw, ctypes.c_char_p).value.decode()
    finally:
        ctypes.CDLL(None).free(ctypes.c_void_p(raw))


class CProgram:
    """Emitted C compiled the reference's way (cc -O3 -shared -fPIC -lm,
    core/src/lib.rs:400-406) and driven through count/ranks/shapes/exec."""

    def __init__(self, source):
        import tempfile

        self.source = source
        self._dir = tempfile.TemporaryDirectory(prefix="ilang_oracle_")
        c_path = Path(self._dir.name) / "prog.c"
        so_path = Path(self._dir.name) / "prog.so"
        c_path.write_text(source)
        subprocess.run(["cc", "-O3", "-shared", "-fPIC", str(c_path), "-o", str(so_path), "-lm"], check=True)
        self._lib = ctypes.CDLL(str(so_path))
        self._lib.count.restype = _sz

    def run(self, *inputs):
        arrs = [_c(a) for a in inputs]
        shapes = [(_sz * max(a.ndim, 1))(*a.shape) for a in arrs]
        ins = (_Tensor * len(arrs))(*[_Tensor(_p(a), s, a.ndim) for a, s in zip(arrs, shapes)])
        n = self._lib.count()
        ranks = (_sz * n)()
        self._lib.ranks(ranks)
        oshapes = [(_sz * max(ranks[i], 1))() for i in range(n)]
        optrs = (ctypes.POINTER(_sz) * n)(*[ctypes.cast(s, ctypes.POINTER(_sz)) for s in oshapes])
        self._lib.shapes(ins, optrs)
        outs = [np.full(tuple(oshapes[i][d] for d in range(ranks[i])), 123.0, dtype=np.float32) for i in range(n)]
        otens = (_Tensor * n)(*[_Tensor(_p(o), s, ranks[i]) for i, (o, s) in enumerate(zip(outs, oshapes))])
        self._lib.exec(ins, otens)
        return outs[0] if n == 1 else tuple(outs)


def compile_component(component_ptr):
    return CProgram(emit_c(component_ptr))
