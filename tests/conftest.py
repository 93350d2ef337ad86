import sys
from pathlib import Path

import pytest

import os
import tempfile

ROOT = Path(__file__).resolve().parents[1]
# generated code objects are cached per user under $XDG_CACHE_HOME; the tests keep theirs out of the home directory
os.environ.setdefault("XDG_CACHE_HOME", str(Path(tempfile.gettempdir()) / f"ilang_test_cache_{os.getuid()}"))
Path(os.environ["XDG_CACHE_HOME"]).mkdir(mode=0o700, exist_ok=True)
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box)")


@pytest.fixture(scope="session")
def golden():
    import numpy as np

    return np.load(ROOT / "tests" / "golden" / "flashattn_ref.npz")


def gemm_kernel_knobs(knobs, which):
    """`which` names one product kernel: "256" / "192" (192 x 256) / "256x192" / "128" (the direct kernels' workgroup
    tile; a trailing "w8" is not part of the name), "0" (register-staged)."""
    which = str(which)
    which = which[:-2] if which.endswith("w8") else which
    for name in ("gemm.tile", "gemm.tile_n", "gemm.direct"):
        knobs.pop(name, None)
    if which == "0":
        knobs["gemm.direct"] = 0
    elif "x" in which:
        knobs["gemm.tile"], knobs["gemm.tile_n"] = (int(v) for v in which.split("x"))
    else:
        knobs["gemm.tile"] = int(which)


class LauncherKnobs(dict):
    """Launcher options for the calls of one test ("attention.waves": 8, "gemm.tile": 128, ...): the names of
    i_hip_program_option, handed to the i_hip_*_opt entry points by NativeWithKnobs below."""

    def text(self, prefix):
        return " ".join(f"{k}={v}" for k, v in self.items() if k.startswith(prefix)).encode()


class _CoreWithKnobs:
    """The kernel launchers of libi_core.so; a call made while the test has set knobs goes through the entry
    point that takes options (i_hip_attention_opt, i_hip_gemm_opt), every other call through the plain one."""

    def __init__(self, core, knobs):
        self._core, self._knobs = core, knobs

    def __getattr__(self, name):
        return getattr(self._core, name)

    def i_hip_attention(self, q, k, v, o, in_dtype, out_dtype, bh, nq, nk, d, dv, scale, stream):
        opts = self._knobs.text("attention.")
        if not opts:
            return self._core.i_hip_attention(q, k, v, o, in_dtype, out_dtype, bh, nq, nk, d, dv, scale, stream)
        return self._core.i_hip_attention_opt(q, k, v, o, in_dtype, out_dtype, bh, nq, nk, d, dv, scale, 0, 0, opts, stream)

    def _gemm(self, plain, a, b, c, in_dtype, out_dtype, row_major, bh, m, n, k, stream):
        opts = self._knobs.text("gemm.")
        if not opts:
            return plain()
        return self._core.i_hip_gemm_opt(a, b, c, in_dtype, out_dtype, row_major, bh, m, n, k, opts, stream)

    def i_hip_gemm_nt_bf16(self, a, b, c, bh, m, n, k, stream):
        return self._gemm(lambda: self._core.i_hip_gemm_nt_bf16(a, b, c, bh, m, n, k, stream), a, b, c, 1, 0, 0, bh, m, n, k, stream)

    def i_hip_gemm_nt_bf16_ex(self, a, b, c, out_dtype, bh, m, n, k, tile_m, tile_n, stream):
        if tile_m or tile_n:  # (the schedule's tile spelled out: the plain entry point takes it)
            return self._core.i_hip_gemm_nt_bf16_ex(a, b, c, out_dtype, bh, m, n, k, tile_m, tile_n, stream)
        return self._gemm(lambda: self._core.i_hip_gemm_nt_bf16_ex(a, b, c, out_dtype, bh, m, n, k, 0, 0, stream),
                          a, b, c, 1, out_dtype, 0, bh, m, n, k, stream)

    def i_hip_gemm_nn_bf16(self, a, b, c, bh, m, n, k, stream):
        return self._gemm(lambda: self._core.i_hip_gemm_nn_bf16(a, b, c, bh, m, n, k, stream), a, b, c, 1, 0, 1, bh, m, n, k, stream)

    def i_hip_gemm_nt_f32(self, a, b, c, bh, m, n, k, stream):
        return self._gemm(lambda: self._core.i_hip_gemm_nt_f32(a, b, c, bh, m, n, k, stream), a, b, c, 0, 0, 0, bh, m, n, k, stream)


class NativeWithKnobs:
    """i_amd._native as the GPU tests use it (core, check, last_error, F32, BF16), with `knobs` applied to the launchers."""

    def __init__(self, nat):
        self.knobs = LauncherKnobs()
        self.core = _CoreWithKnobs(nat.core, self.knobs)
        self.check, self.last_error, self.check_ptr = nat.check, nat.last_error, nat.check_ptr
        self.F32, self.BF16 = nat.F32, nat.BF16


@pytest.fixture
def knobs(env):
    """The launcher options of this test's calls; empty again when the test ends."""
    env.nat.knobs.clear()
    yield env.nat.knobs
    env.nat.knobs.clear()
