"""Randomised parity sweep of the hand-written attention, GEMM and row-softmax kernels (through the C ABI of include/i_hip.h)
against the closed forms in f64, computed on the device by torch: many ragged shapes, every workgroup size and
tile the launcher can pick, each case run twice.  The seeds are fixed; a mismatch prints the case.

Tolerance 2e-2 of max |reference| for attention (bf16 in, f32 accumulate), 1e-2 for the GEMMs, 1e-4 for the softmax (f32).
"""
import random

import pytest

from conftest import gemm_kernel_knobs

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def env():
    import torch

    assert torch.cuda.is_available(), "GPU tests need a visible MI355X"
    from i_amd import _native as nat

    class Env:
        pass

    from conftest import NativeWithKnobs

    e = Env()
    e.torch, e.nat = torch, NativeWithKnobs(nat)
    e.stream = lambda: torch.cuda.current_stream().cuda_stream
    return e


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_attention_bf16_random_shapes(env, knobs, seed):
    t, nat = env.torch, env.nat
    rng = random.Random(seed)
    for case in range(40):
        d = rng.choice([64, 128])
        bh = rng.randint(1, 6)
        nq = rng.choice([rng.randint(1, 64), rng.randint(65, 700), rng.randint(700, 1600)])
        nk = rng.choice([rng.randint(1, 64), rng.randint(65, 300), rng.randint(256, 2100)])
        waves = rng.choice([None, "4", "8"] + (["64"] if d == 64 else []))
        amp = rng.choice([0.5, 1.0, 2.0])
        if waves:
            knobs["attention.waves"] = waves
        else:
            knobs.pop("attention.waves", None)
        g = t.Generator(device="cuda").manual_seed(1000 * seed + case)
        q, k, v = ((amp * t.randn(bh, n, d, device="cuda", generator=g)).bfloat16() for n in (nq, nk, nk))
        scale = d ** -0.5
        ref = t.softmax((q.double() @ k.double().transpose(1, 2)) * scale, -1) @ v.double()
        for rep in range(2):
            o = t.full((bh, nq, d), float("nan"), device="cuda")
            nat.check(nat.core.i_hip_attention(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), nat.BF16, nat.F32,
                                               bh, nq, nk, d, d, scale, env.stream()))
            t.cuda.synchronize()
            err = float((o.double() - ref).abs().max() / ref.abs().max())
            assert err <= 2e-2, dict(case=case, d=d, bh=bh, nq=nq, nk=nk, waves=waves, amp=amp, rep=rep, err=err)


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_gemm_bf16_random_shapes(env, knobs, seed):
    t, nat = env.torch, env.nat
    rng = random.Random(seed)
    for case in range(40):
        nn = rng.random() < 0.5  # row-major right operand
        bh = rng.randint(1, 3)
        m = rng.choice([rng.randint(1, 130), rng.randint(130, 700)])
        n = rng.choice([rng.randint(1, 130), rng.randint(130, 700)])
        k = rng.choice([64, 128, 192, 320, 512, 1024]) if (nn or rng.random() < 0.7) else 8 * rng.randint(1, 60)
        if nn:
            n = max(8, n // 8 * 8)
        direct = rng.choice([None, "256", "128"] + ([] if nn else ["0", "192", "256x192"]))
        if direct:
            gemm_kernel_knobs(knobs, direct)
        else:
            knobs.pop("gemm.tile", None); knobs.pop("gemm.tile_n", None); knobs.pop("gemm.direct", None)
        g = t.Generator(device="cuda").manual_seed(1000 * seed + case)
        a = (t.rand(bh, m, k, device="cuda", generator=g) * 2 - 1).bfloat16()
        b = (t.rand(*((bh, k, n) if nn else (bh, n, k)), device="cuda", generator=g) * 2 - 1).bfloat16()
        ref = a.double() @ (b.double() if nn else b.double().transpose(1, 2))
        f = nat.core.i_hip_gemm_nn_bf16 if nn else nat.core.i_hip_gemm_nt_bf16
        for rep in range(2):
            c = t.full((bh, m, n), float("nan"), device="cuda")
            nat.check(f(a.data_ptr(), b.data_ptr(), c.data_ptr(), bh, m, n, k, env.stream()))
            t.cuda.synchronize()
            err = float((c.double() - ref).abs().max() / ref.abs().max().clamp_min(1e-6))
            assert err <= 1e-2, dict(case=case, nn=nn, bh=bh, m=m, n=n, k=k, direct=direct, rep=rep, err=err)


@pytest.mark.parametrize("seed", [1, 2])
def test_row_softmax_random_shapes(env, seed):
    """Row widths from 1 to 300000 columns, i.e. every form of the row kernel (several rows per wavefront, a
    wavefront, a workgroup with the row in registers, a workgroup in two passes), aligned and unaligned, with rows
    that sit far from zero; against softmax in f64.  Each case runs twice and must repeat bit for bit."""
    t, nat = env.torch, env.nat
    rng = random.Random(seed)
    for case in range(60):
        band = rng.choice([(1, 128), (1, 128), (129, 8192), (8193, 65536), (65537, 300000)])
        cols = rng.randint(*band)
        if rng.random() < 0.5:
            cols = max(4, cols // 4 * 4)
        rows = rng.randint(1, max(1, min(700, (1 << 22) // cols)))
        shift = rng.choice([0.0, 30.0, -80.0])
        g = t.Generator(device="cuda").manual_seed(7000 * seed + case)
        offset = rng.choice([0, 0, 1])  # 1: operands start 4 bytes into their allocations
        xbuf = t.randn(rows * cols + 1, device="cuda", generator=g) * 3 + shift
        x = xbuf[offset:offset + rows * cols].view(rows, cols)
        ref = t.softmax(x.double(), dim=-1)
        results = []
        for rep in range(2):
            ybuf = t.full((rows * cols + 2,), float("nan"), device="cuda")
            nat.check(nat.core.i_hip_row_softmax(x.data_ptr(), ybuf.data_ptr() + 4 * offset, rows, cols, env.stream()))
            t.cuda.synchronize()
            y = ybuf[offset:offset + rows * cols].view(rows, cols)
            err = float((y.double() - ref).abs().max() / ref.abs().max())
            assert err <= 1e-4, dict(case=case, rows=rows, cols=cols, offset=offset, shift=shift, rep=rep, err=err)
            assert bool(t.isnan(ybuf[offset + rows * cols:]).all()) and (offset == 0 or bool(t.isnan(ybuf[0])))
            results.append(y.clone())
        assert t.equal(results[0], results[1]), dict(case=case, rows=rows, cols=cols)
