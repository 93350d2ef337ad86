"""Randomised parity sweep of the hand-written attention and GEMM kernels (through the C ABI of include/i_hip.h)
against the closed forms in f64, computed on the device by torch: many ragged shapes, every workgroup size and
tile the launcher can pick, each case run twice.  The seeds are fixed; a mismatch prints the case.

Tolerance 2e-2 of max |reference| for attention (bf16 in, f32 accumulate), 1e-2 for the GEMMs.
"""
import random

import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def env():
    import torch

    assert torch.cuda.is_available(), "GPU tests need a visible MI355X"
    from i_amd import _native as nat

    class Env:
        pass

    e = Env()
    e.torch, e.nat = torch, nat
    e.stream = lambda: torch.cuda.current_stream().cuda_stream
    return e


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_attention_bf16_random_shapes(env, monkeypatch, seed):
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
            monkeypatch.setenv("ILANG_ATTN_WAVES", waves)
        else:
            monkeypatch.delenv("ILANG_ATTN_WAVES", raising=False)
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
def test_gemm_bf16_random_shapes(env, monkeypatch, seed):
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
        direct = rng.choice([None, "256", "128"] + ([] if nn else ["0"]))
        if direct:
            monkeypatch.setenv("ILANG_GEMM_DIRECT", direct)
        else:
            monkeypatch.delenv("ILANG_GEMM_DIRECT", raising=False)
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
