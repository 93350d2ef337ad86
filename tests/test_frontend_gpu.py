"""End-to-end through the drop-in boundary on the GPU: component strings ->
i_parse / combinators -> i_compile -> i_exec / i_exec_into / i_exec_into_device.

The cases are the reference's own integration tests (ilang-python/test.py:131-150,
ilang-python/flash-attn.py:31-77) plus the BASELINE configurations, each
checked against the CPU oracle: the emitted C of the same component where the
oracle finishes in seconds, oracle.c / NumPy closed forms otherwise.
"""
import os

import numpy as np
import pytest

import oracle
from i_amd import Component as i, I, Tensor

pytestmark = pytest.mark.gpu
RTOL_F32, RTOL_BF16 = 1e-4, 2e-2


@pytest.fixture(scope="module")
def torch():
    import torch

    assert torch.cuda.is_available()
    return torch


def rnd(shape, seed):
    return np.random.default_rng(seed).standard_normal(shape, dtype=np.float32)


def close(got, ref, rtol):
    got, ref = np.asarray(got), np.asarray(ref)
    assert got.shape == ref.shape and np.isfinite(got).all()
    scale = max(float(np.abs(ref).max()), 1e-30)
    assert float(np.abs(got - ref).max()) / scale <= rtol
    return True


def as_numpy(t):
    return np.asarray(t.data, dtype=np.float32).reshape(t.shape)


def flash(split="i:16,j:16", prefix="", scaled=False):
    p = prefix
    mm_t = i(f"{p}ik*{p}jk~{p}ijk | {split} | {p}jii'j'k") >> i(f"+{p}ijk~{p}ij | {split} | {p}jii'j'k0")
    row_max_shift = (I & i(f">{p}ij~{p}i | {split} | {p}ji0i'j'")) >> i(f"{p}ij-{p}i~{p}ij | {split} | {p}ji01i'j'")
    exp = i(f"^{p}ij~{p}ij | {split} | {p}ji0i'j'")
    row_normalize = (I & i(f"+{p}ij~{p}i | {split} | {p}ji0i'j'")) >> i(f"{p}ij/{p}i~{p}ij | {split} | {p}ji01i'j'")
    mm = i(f"{p}ij*{p}jk~{p}ikj | {split} | {p}ji0i'kj'") >> i(f"+{p}ikj~{p}ik | {split} | {p}jii'kj'0")
    if scaled:
        return mm_t >> i(f"{p}ij*.~{p}ij | {split} | {p}ji0i'j'") >> row_max_shift >> exp >> row_normalize >> mm
    return mm_t >> row_max_shift >> exp >> row_normalize >> mm


def naive(split="i:16,j:16"):
    mm_t = i(f"ik*jk~ijk | {split} | jii'j'k") >> i(f"+ijk~ij | {split} | jii'j'k0")
    row_max_shift = (I & i(f">ij~i | {split} | jii'j'")) >> i(f"ij-i~ij | {split} | 1jii'j'")
    exp = i(f"^ij~ij | {split} | jii'j'")
    row_normalize = (I & i(f"+ij~i | {split} | jii'j'")) >> i(f"ij/i~ij | {split} | 1jii'j'")
    mm = i(f"ij*jk~ikj | {split} | jii'kj'") >> i(f"+ikj~ik | {split} | jii'kj'0")
    return mm_t >> row_max_shift >> exp >> row_normalize >> mm


def softmax_rowstaged():
    return (((I & i(">ij~i|i:16|ii'j")) >> i("ij-i~ij|i:16|ii'1j")) >> i("^ij~ij|i:16|ii'0j")
            >> ((I & i("+ij~i|i:16|ii'0j")) >> i("ij/i~ij|i:16|ii'01j")))


def softmax_naive():
    s = "i:16,j:16"
    return (((I & i(f">ij~i|{s}|jii'j'")) >> i(f"ij-i~ij|{s}|1jii'j'")) >> i(f"^ij~ij|{s}|jii'j'")
            >> ((I & i(f"+ij~i|{s}|jii'j'")) >> i(f"ij/i~ij|{s}|1jii'j'")))


# ------------------------------------------------------------------ the reference's test.py cases (Tensor in, Tensor out)
def test_reference_matmul_case(torch):
    a, b = rnd((8, 16), 1), rnd((16, 7), 2)
    f = i("ik*kj~ijk|i:2,k:2|ii'jkk'") >> i("+ijk~ij|i:2,k:2|ii'j!kk'0")
    got = as_numpy(f.exec(Tensor(a.tolist()), Tensor(b.tolist())))
    assert np.allclose(got, a @ b, rtol=1e-5, atol=1e-6)


def test_reference_batched_attention_case(torch):
    q, k, v = rnd((2, 3, 4, 8), 1), rnd((2, 3, 4, 8), 2), rnd((2, 3, 4, 8), 3)
    mm_t = i("bhij*bhkj~bhikj | i:16,k:16 | bhkii'k'j") >> i("+bhikj~bhik | i:16,k:16 | bhkii'k'j0")
    row_max_shift = (I & i(">bhik~bhi | i:16,k:16 | bhkii'k'")) >> i("bhik-bhi~bhik | i:16,k:16 | bh1kii'k'")
    exp = i("^bhik~bhik | i:16,k:16 | bhkii'k'")
    row_normalize = (I & i("+bhik~bhi | i:16,k:16 | bhkii'k'")) >> i("bhik/bhi~bhik | i:16,k:16 | bh1kii'k'")
    mm = i("bhik*bhkj~bhijk | i:16,k:16 | bhkii'jk'") >> i("+bhijk~bhij | i:16,k:16 | bhkii'jk'0")
    attn = mm_t >> row_max_shift >> exp >> row_normalize >> mm
    got = as_numpy(attn.exec(*(Tensor(x.tolist()) for x in (q, k, v))))
    assert np.allclose(got, oracle.np_attention64(q, k, v), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("src,fn", [(">ij~i", np.max), ("<ij~i", np.min), ("+ij~i", np.sum)])
def test_reference_row_reductions(torch, src, fn):
    x = rnd((16, 8), 1)
    got = as_numpy(i(src).exec(Tensor(x.tolist())))
    assert np.allclose(got, fn(x, axis=1), rtol=1e-5, atol=1e-6)


def test_reference_mlp_case_with_pair(torch):
    # test.py's mlp spells the pairing with an operator the frontend lacks; `|` is the pair combinator
    x, w1, w2 = rnd((8,), 1), rnd((16, 8), 2), rnd((7, 16), 3)
    mvp = i("ij*j~ij") >> i("+ij~i")
    amvp = mvp >> i(">i~i")
    f = (i("ij~ij") | amvp) >> mvp
    got = as_numpy(f.exec(*(Tensor(t.tolist()) for t in (w2, w1, x))))
    assert np.allclose(got, w2 @ np.maximum(w1 @ x, 0), rtol=1e-5, atol=1e-5)


# ------------------------------------------------------------------ flash-attn.py
def test_reference_demo_flash_and_naive_attention(torch):
    q, k, v = rnd((32, 2048), 1), rnd((32, 2048), 2), rnd((32, 2048), 3)
    ref = oracle.np_attention64(q, k, v)
    for comp in (flash(), naive()):
        got = comp.exec_numpy(q, k, v)
        assert np.allclose(got, ref, rtol=3e-4, atol=5e-5, equal_nan=True)  # the demo's own tolerance


def test_head_sizes_between_and_unequal_through_the_frontend(torch):
    """The compiled component hands the operands' own d and dv to the launcher: bf16 tensors with d = dv = 96 (batch
    axes, score scale), d = 40 without a scale, and d = 64 with dv = 128 run the padded direct kernels; f32 tensors
    with d = dv = 96 the padded f32 kernel.  Against the oracle."""
    for d, dv, nq, nk, kernel in ((96, 96, 300, 500, "attn_fwd_bf16_d128_bn64_direct_pad"),
                                  (64, 128, 130, 333, "attn_fwd_bf16_d128_bn64_direct_pad"),
                                  (40, 40, 77, 200, "attn_fwd_bf16_d64_bn64_direct_pad")):
        qb, kb, vb = (oracle.to_bf16_f32(rnd(shape, seed)) for seed, shape in
                      ((1, (2, 3, nq, d)), (2, (2, 3, nk, d)), (3, (2, 3, nk, dv))))
        scale = np.float32(1.0 / np.sqrt(d))
        comp = flash("i:128,j:64", prefix="bh", scaled=True)
        out = comp.exec_torch(torch.from_numpy(qb).cuda().bfloat16(), torch.from_numpy(kb).cuda().bfloat16(),
                              torch.tensor(scale, device="cuda"), torch.from_numpy(vb).cuda().bfloat16())
        assert kernel + " " in comp.report() + " ", comp.report()
        close(out.cpu().numpy(), oracle.attention_tiled(qb, kb, vb, scale), RTOL_BF16)
    q, k, v = rnd((200, 96), 1), rnd((333, 96), 2), rnd((333, 96), 3)
    comp = flash()
    out = comp.exec_torch(*(torch.from_numpy(a).cuda() for a in (q, k, v)))
    assert "attn_fwd_f32_d128_bn32_direct_pad" in comp.report()
    close(out.cpu().numpy(), oracle.attention_tiled(q, k, v), RTOL_F32)


def test_head_sizes_above_128(torch):
    """bf16 with d and dv up to 256 runs the fused kernel for 256-column rows (padded below 256), in the f32-scale
    form too.  Everything else above 128 (f32, the demo's own shape [32, 2048] of flash-attn.py:31-36; bf16 above 256) runs as three
    hand-written kernels: scores by the MFMA GEMM, row softmax in place, output by the MFMA GEMM.  f32 at the demo's
    shape against the emitted C; bf16 with batch axes, a score scale and ragged query counts against the oracle."""
    q, k, v = rnd((32, 2048), 1), rnd((32, 2048), 2), rnd((32, 2048), 3)
    comp = flash()
    got = comp.exec_numpy(q, k, v)
    assert "attention in three kernels" in comp.report() and "gemm_nt_f32" in comp.report()
    close(got, oracle.compile_component(comp.handle).run(q, k, v), RTOL_F32)
    for d, dv, nq, nk, fused, f32_scale in ((192, 192, 300, 512, True, False), (256, 256, 130, 700, True, False),
                                            (256, 160, 77, 136, True, False), (192, 192, 300, 512, True, True), (320, 192, 77, 136, False, False)):
        qb, kb, vb = (oracle.to_bf16_f32(rnd(shape, seed)) for seed, shape in
                      ((1, (2, 3, nq, d)), (2, (2, 3, nk, d)), (3, (2, 3, nk, dv))))
        scale = np.float32(1.0 / np.sqrt(d))
        comp = flash("i:128,j:64", prefix="bh", scaled=True)
        if f32_scale:
            comp.option("attention.f32_scale", 1)
        out = comp.exec_torch(torch.from_numpy(qb).cuda().bfloat16(), torch.from_numpy(kb).cuda().bfloat16(),
                              torch.tensor(scale, device="cuda"), torch.from_numpy(vb).cuda().bfloat16())
        if fused:
            assert "attn_fwd_bf16_d256_bn32_direct" + ("_f32scale" if f32_scale else "") + ("_pad" if (d, dv) != (256, 256) else "") + " " in comp.report() + " "
        else:
            assert "attention in three kernels" in comp.report() and "scaled_softmax" in comp.report()
        close(out.cpu().numpy(), oracle.attention_tiled(qb, kb, vb, scale), RTOL_BF16)
    # extents the GEMM kernels cannot take (f32 with a key count that is no multiple of 4) still run generated
    q, k, v = rnd((20, 160), 1), rnd((33, 160), 2), rnd((33, 160), 3)
    comp = flash()
    close(comp.exec_numpy(q, k, v), oracle.attention_tiled(q, k, v), RTOL_F32)
    assert "generated kernel" in comp.report()


# ------------------------------------------------------------------ BASELINE config 1
@pytest.mark.parametrize("split", ["i:16,j:16", "i:32,j:8", "i:128,j:64"])
def test_config1_demo_attention_f32_vs_emitted_c(torch, split):
    q, k, v = (np.random.default_rng(s).uniform(-1, 1, (512, 64)).astype(np.float32) for s in (1, 2, 3))
    comp = flash(split)
    ref = oracle.compile_component(comp.handle).run(q, k, v)  # the C the reference backend would emit for these strings
    close(comp.exec_numpy(q, k, v), ref, RTOL_F32)
    close(comp.exec_torch(*(torch.from_numpy(a) for a in (q, k, v))).numpy(), ref, RTOL_F32)


def test_config1_golden_reference_outputs(torch, golden):
    comp = flash()
    for case in ("u_48x24", "u_64x64", "u_100x40", "n_48x24", "n_33x17", "n_16x130"):
        q, k, v, o = (golden[f"{case}.{x}"] for x in "qkvo")
        close(comp.exec_numpy(q, k, v), o, RTOL_F32)


def test_generated_and_hand_written_forms_agree(torch):
    q, k, v = (np.random.default_rng(s).uniform(-1, 1, (200, 48)).astype(np.float32) for s in (1, 2, 3))
    hand = flash().exec_numpy(q, k, v)

    def generated(comp):
        comp.option("generated.only", 1)
        return comp

    gen = generated(flash()).exec_numpy(q, k, v)
    x = rnd((70, 300), 1)
    sm_gen = generated(softmax_rowstaged()).exec_numpy(x)
    a, b = rnd((50, 24), 1), rnd((30, 24), 2)
    mm_gen = generated(i("ik*jk~ijk | i:16,j:16 | jii'j'k") >> i("+ijk~ij | i:16,j:16 | jii'j'k0")).exec_numpy(a, b)
    ref = oracle.attention_tiled(q, k, v)
    close(hand, ref, RTOL_F32)
    close(gen, ref, RTOL_F32)
    close(sm_gen, oracle.row_softmax(x), RTOL_F32)
    close(mm_gen, oracle.mm_t(a, b), RTOL_F32)


# ------------------------------------------------------------------ BASELINE config 2
@pytest.mark.parametrize("comp_fn", [softmax_rowstaged, softmax_naive])
def test_config2_row_softmax_small_vs_emitted_c(torch, comp_fn):
    x = rnd((50, 70), 1)
    comp = comp_fn()
    close(comp.exec_numpy(x), oracle.compile_component(comp.handle).run(x), RTOL_F32)


def test_config2_row_softmax_full_size_device(torch):
    x = rnd((16384, 4096), 1)
    xd = torch.from_numpy(x).cuda()
    y = softmax_rowstaged().exec_torch(xd)
    assert (y.sum(dim=-1) - 1).abs().max().item() < 1e-4
    rows = np.r_[0:8, 16376:16384]
    close(y[rows].cpu().numpy(), oracle.row_softmax(x[rows]), RTOL_F32)


# ------------------------------------------------------------------ BASELINE config 3
def test_config3_mm_t_bf16_device(torch):
    n = 4096
    a = oracle.to_bf16_f32(np.random.default_rng(1).uniform(-1, 1, (n, n)).astype(np.float32))
    b = oracle.to_bf16_f32(np.random.default_rng(2).uniform(-1, 1, (n, n)).astype(np.float32))
    comp = i("ik*jk~ijk | i:256,j:256 | jii'j'k") >> i("+ijk~ij | i:256,j:256 | jii'j'k0")
    c = comp.exec_torch(torch.from_numpy(a).cuda().bfloat16(), torch.from_numpy(b).cuda().bfloat16())
    rows = np.r_[0:4, n - 4:n]
    close(c[rows].cpu().numpy(), oracle.mm_t(a[rows], b), RTOL_BF16)
    cols = np.r_[0:4, n - 4:n]
    close(c[:, cols].cpu().numpy(), oracle.mm_t(a, b[cols]), RTOL_BF16)


def test_large_host_calls_run_in_slices(torch):
    """The reference's own entry point (host f32 arrays) with operands of tens of MiB: a program that only maps over
    the first index of its outputs runs slice by slice, the rows of one slice on the link while the kernels of the
    slice before run.  Row softmax, attention (all of Q, K, V and O cut along the batch) and mm_t (A and C in
    slices, B whole) against the device entry on the same operands; programs that sum over that index, or use it
    under two names, stay whole and stay right."""
    g = np.random.default_rng(7)

    def on_device(comp, *ins):
        return comp.exec_torch(*(torch.from_numpy(np.asarray(x)).cuda() for x in ins)).cpu().numpy()

    x = g.standard_normal((16384, 1024), dtype=np.float32)                      # 64 MiB in, 64 MiB out
    sm = softmax_rowstaged()
    y = np.empty_like(x)
    sm.into(y, x)
    assert "host: operands in 4 slices of 4096 rows" in sm.report(), sm.report()
    assert np.array_equal(y, on_device(sm, x))                                   # rows do not know how many there are
    picked = np.r_[0:64, 4090:4102, 16320:16384]                                 # (rows on both sides of a slice's edge)
    close(y[picked], oracle.row_softmax(x[picked]), RTOL_F32)
    q, k, v = (g.standard_normal((4, 8, 1024, 128), dtype=np.float32) for _ in range(3))  # 16 MiB each
    attn = flash("i:128,j:32", prefix="bh", scaled=True)
    scale = np.float32(128 ** -0.5)
    o = np.empty_like(q)
    attn.into(o, q, k, scale, v)
    assert "host: operands in 2 slices of 2 rows" in attn.report(), attn.report()
    close(o, on_device(attn, q, k, scale, v), 1e-6)
    close(o[1:3, 7:8, 1000:1024], oracle.attention_tiled(q[1:3, 7:8, 1000:1024], k[1:3, 7:8], v[1:3, 7:8], scale), RTOL_F32)
    a = g.uniform(-1, 1, (4100, 2048)).astype(np.float32)                        # 32 MiB, in slices
    b = g.uniform(-1, 1, (4096, 2048)).astype(np.float32)                        # 32 MiB, whole
    mm = i("ik*jk~ijk | i:16,j:16 | jii'j'k") >> i("+ijk~ij | i:16,j:16 | jii'j'k0")
    c = np.empty((4100, 4096), np.float32)                                       # 64 MiB, in slices
    mm.into(c, a, b)
    assert "host: operands in 3 slices of 1367 rows" in mm.report(), mm.report()
    close(c, on_device(mm, a, b), 1e-5)  # (a slice may take another kernel than the whole: sums in another order)
    rows = np.r_[0:4, 1365:1369, 4096:4100]
    close(c[rows], a[rows].astype(np.float64) @ b.astype(np.float64).T, RTOL_F32)
    close(c[rows], oracle.mm_t(a[rows], b), RTOL_F32)
    # the first index summed over: whole
    xs = np.abs(x[:, :1024]) + 0.1
    colnorm = (I & i("+ij~j||ij")) >> i("ij/j~ij||1ij")
    yn = np.empty_like(xs)
    colnorm.into(yn, xs)
    assert "host:" not in colnorm.report()
    close(yn, xs / xs.sum(0, dtype=np.float64), RTOL_F32)
    # the first index under two names in one expression: one input as both operands of a product
    gram = (I & I) >> i("ik*jk~ijk | i:16,j:16 | jii'j'k") >> i("+ijk~ij | i:16,j:16 | jii'j'k0")
    z = g.uniform(-1, 1, (4096, 1024)).astype(np.float32)
    got = np.empty((4096, 4096), np.float32)                                     # 64 MiB out
    gram.into(got, z)
    assert "host:" not in gram.report()
    close(got[:16], z[:16].astype(np.float64) @ z.astype(np.float64).T, RTOL_F32)


def test_bf16_operands_that_start_off_a_16_byte_boundary(torch):
    """Every bf16 kernel moves 16 bytes per lane (the direct ones straight from global memory into LDS).  Operands
    that are views starting one element (2 bytes) into their allocation are copied into aligned temporaries by the
    executor, a misaligned attention output is written through one; the launchers themselves refuse such operands.
    Attention (d = 128 and a padded head size, f32 and bf16 results into views that are misaligned too), mm_t
    and the product with a row-major right operand, against the oracle."""
    from i_amd import _native as nat

    def shifted(a, dtype):
        buf = torch.zeros(a.size + 1, dtype=dtype, device="cuda")
        view = buf[1:].view(a.shape)
        view.copy_(torch.from_numpy(a))
        assert view.data_ptr() % 16 != 0
        return view

    attn = flash(prefix="b", scaled=True)
    for d, out_dtype in ((128, torch.float32), (72, torch.bfloat16), (64, torch.float32)):
        bh, nq, nk = 2, 200, 333
        q, k, v = (oracle.to_bf16_f32(rnd((bh, n, d), sd)) for sd, n in ((1, nq), (2, nk), (3, nk)))
        scale = np.float32(1.0 / np.sqrt(d))
        ref = oracle.attention_tiled(q, k, v, scale)
        qd, kd, vd = (shifted(x, torch.bfloat16) for x in (q, k, v))
        whole = torch.full((bh * nq * d + 2,), -7.0, dtype=out_dtype, device="cuda")
        out = whole[1:-1].view(bh, nq, d)
        attn.into(out, qd, kd, torch.tensor(scale, device="cuda"), vd)
        assert "attn_fwd_bf16" in attn.report(), attn.report()
        assert whole[0].item() == -7.0 and whole[-1].item() == -7.0
        close(out.float().cpu().numpy(), ref, RTOL_BF16)
    a, b = (oracle.to_bf16_f32(np.random.default_rng(sd).uniform(-1, 1, shape).astype(np.float32)) for sd, shape in ((1, (300, 136)), (2, (260, 136))))
    mm_t = i("ik*jk~ijk | i:16,j:16 | jii'j'k") >> i("+ijk~ij | i:16,j:16 | jii'j'k0")
    got = mm_t.exec_torch(shifted(a, torch.bfloat16), shifted(b, torch.bfloat16))
    assert "gemm_nt_bf16" in mm_t.report(), mm_t.report()
    close(got.cpu().numpy(), oracle.mm_t(a, b), RTOL_BF16)
    mm = i("ik*kj~ijk|i:16,k:16|ii'jkk'") >> i("+ijk~ij|i:16,k:16|ii'j!kk'0")
    bt = np.ascontiguousarray(b[:256].T)  # [136, 256]
    got = mm.exec_torch(shifted(a, torch.bfloat16), shifted(bt, torch.bfloat16))
    assert "gemm_n" in mm.report() and "generated" not in mm.report(), mm.report()
    close(got.cpu().numpy(), oracle.mm_t(a, b[:256]), RTOL_BF16)
    # the launchers say so instead of reading from such an address
    qd = shifted(oracle.to_bf16_f32(rnd((1, 64, 64), 1)), torch.bfloat16)
    o = torch.empty(1, 64, 64, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    assert nat.core.i_hip_attention(qd.data_ptr(), qd.data_ptr(), qd.data_ptr(), o.data_ptr(), nat.BF16, nat.F32, 1, 64, 64, 64, 64, 0.1, stream) == -1
    assert "16-byte aligned" in nat.last_error()
    assert nat.core.i_hip_gemm_nt_bf16(qd.data_ptr(), qd.data_ptr(), o.data_ptr(), 1, 64, 64, 64, stream) == -1
    assert "16-byte aligned" in nat.last_error()


@pytest.mark.parametrize("k", [42, 40, 64])  # 42: operands padded to k = 44 first; 40: a partial last slab; 64: whole slabs
def test_mm_t_f32_small_vs_emitted_c(torch, k):
    a, b = rnd((100, k), 1), rnd((70, k), 2)
    comp = i("ik*jk~ijk | i:16,j:16 | jii'j'k") >> i("+ijk~ij | i:16,j:16 | jii'j'k0")
    close(comp.exec_numpy(a, b), oracle.compile_component(comp.handle).run(a, b), RTOL_F32)
    assert "gemm_nt_f32" in comp.report() and "generated kernel" not in comp.report()
    assert ("_ktail" in comp.report()) == (k != 64)


def test_products_with_any_contracted_extent_run_on_the_matrix_kernels(torch):
    """A contracted extent that is no multiple of what the matrix-instruction kernels read (4 elements in f32, 8 in
    bf16) does not fall back to the generated kernel: the executor pads both operands with zero columns first.
    NT and NN products, f32 and bf16, against float64."""
    mm_t = i("ik*jk~ijk | i:16,j:16 | jii'j'k") >> i("+ijk~ij | i:16,j:16 | jii'j'k0")
    mm = i("ik*kj~ijk|i:2,k:2|ii'jkk'") >> i("+ijk~ij|i:2,k:2|ii'j!kk'0")
    for k in (1, 7, 42, 1001):
        a, b = rnd((150, k), 1), rnd((90, k), 2)
        ref = a.astype(np.float64) @ b.astype(np.float64).T
        close(mm_t.exec_numpy(a, b), ref, RTOL_F32)
        assert "gemm_nt_f32" in mm_t.report(), mm_t.report()
        close(mm.exec_numpy(a, np.ascontiguousarray(b.T)), ref, RTOL_F32)
        assert "gemm_nt_f32" in mm.report(), mm.report()
        ad, bd = torch.from_numpy(a).cuda().bfloat16(), torch.from_numpy(b).cuda().bfloat16()
        ref16 = ad.double() @ bd.double().T
        got = mm_t.exec_torch(ad, bd)
        assert "gemm_nt_bf16" in mm_t.report(), mm_t.report()
        assert float((got.double() - ref16).abs().max()) <= RTOL_BF16 * float(ref16.abs().max())
        got = mm.exec_torch(ad, bd.T.contiguous())
        assert float((got.double() - ref16).abs().max()) <= RTOL_BF16 * float(ref16.abs().max())
    # batched, and an f32 operand that starts 4 bytes into its allocation (rows not 16-byte aligned)
    ab, bb = rnd((3, 40, 30), 3), rnd((3, 50, 30), 4)
    bmm = i("bik*bjk~bijk | i:16,j:16 | bjii'j'k") >> i("+bijk~bij | i:16,j:16 | bjii'j'k0")
    close(bmm.exec_numpy(ab, bb), np.einsum("bik,bjk->bij", ab.astype(np.float64), bb.astype(np.float64)), RTOL_F32)
    buf = torch.zeros(100 * 64 + 1, device="cuda")
    x = rnd((100, 64), 5)
    buf[1:] = torch.from_numpy(x).cuda().reshape(-1)
    shifted = buf[1:].view(100, 64)
    got = mm_t.exec_torch(shifted, shifted)
    assert float((got.double().cpu() - torch.from_numpy(x.astype(np.float64) @ x.astype(np.float64).T)).abs().max()) <= 1e-4 * 64


def test_products_with_few_tiles_and_a_long_k_loop_are_split_over_workgroups(torch, monkeypatch):
    """One small extent against a long contraction leaves most CUs without an output tile: the executor then splits
    the k loop over workgroups (partial products in a temporary, added up by a second kernel).  Against float64,
    with whole and partial last slabs, several batches, f32 and bf16 results; the program option gemm.k_parts = 1 gives the
    unsplit kernel and the same numbers to within the order of the sums."""
    mm_t = i("ik*jk~ijk | i:16,j:16 | jii'j'k") >> i("+ijk~ij | i:16,j:16 | jii'j'k0")
    bmm = i("bik*bjk~bijk | i:16,j:16 | bjii'j'k") >> i("+bijk~bij | i:16,j:16 | bjii'j'k0")
    for shape_a, shape_b, comp in (((64, 8192), (1000, 8192), mm_t), ((100, 5000), (1000, 5000), mm_t),
                                   ((300, 16424), (260, 16424), mm_t), ((2, 64, 8192), (2, 512, 8192), bmm)):
        g = torch.Generator(device="cuda").manual_seed(shape_a[-1])
        a = (torch.rand(*shape_a, device="cuda", generator=g) * 2 - 1).bfloat16()
        b = (torch.rand(*shape_b, device="cuda", generator=g) * 2 - 1).bfloat16()
        ref = a.double() @ b.double().transpose(-1, -2)
        comp.option("gemm.k_parts", 0)
        got = comp.exec_torch(a, b)
        assert "parts)" in comp.report(), comp.report()
        assert float((got.double() - ref).abs().max()) <= 1e-2 * float(ref.abs().max())
        got16 = comp.exec_torch(a, b, out_dtype=torch.bfloat16)
        assert float((got16.double() - ref).abs().max()) <= 2e-2 * float(ref.abs().max())
        comp.option("gemm.k_parts", 1)
        plain = comp.exec_torch(a, b)
        assert "parts)" not in comp.report()
        assert float((plain - got).abs().max()) <= 1e-4 * float(ref.abs().max())
    # a row-major right operand (c = a b): the same kernels' NN forms split the same way
    mm = i("ik*kj~ijk|i:16,k:16|ii'jkk'") >> i("+ijk~ij|i:16,k:16|ii'j!kk'0")
    for m, k, n in ((64, 8192, 1000), (300, 5000, 264), (40, 4104, 72)):
        g = torch.Generator(device="cuda").manual_seed(k + 2)
        a = (torch.rand(m, k, device="cuda", generator=g) * 2 - 1).bfloat16()
        b = (torch.rand(k, n, device="cuda", generator=g) * 2 - 1).bfloat16()
        ref = a.double() @ b.double()
        mm.option("gemm.k_parts", 0)
        got = mm.exec_torch(a, b)
        assert "gemm_nn_bf16" in mm.report() and "parts)" in mm.report(), mm.report()
        assert float((got.double() - ref).abs().max()) <= 1e-2 * float(ref.abs().max())
        got16 = mm.exec_torch(a, b, out_dtype=torch.bfloat16)
        assert float((got16.double() - ref).abs().max()) <= 2e-2 * float(ref.abs().max())
        mm.option("gemm.k_parts", 1)
        plain = mm.exec_torch(a, b)
        assert "parts)" not in mm.report()
        assert float((plain - got).abs().max()) <= 1e-4 * float(ref.abs().max())
    # f32 operands: the same through the f32 kernels, to the f32 bar
    for shape_a, shape_b, comp in (((64, 2048), (300, 2048), mm_t), ((100, 1000), (100, 1000), mm_t), ((2, 128, 4100), (2, 64, 4100), bmm)):
        g = torch.Generator(device="cuda").manual_seed(shape_a[-1] + 1)
        a = torch.rand(*shape_a, device="cuda", generator=g) * 2 - 1
        b = torch.rand(*shape_b, device="cuda", generator=g) * 2 - 1
        ref = a.double() @ b.double().transpose(-1, -2)
        comp.option("gemm.k_parts", 0)
        got = comp.exec_torch(a, b)
        assert "_f32_" in comp.report() and "parts)" in comp.report(), comp.report()
        assert float((got.double() - ref).abs().max()) <= RTOL_F32 * float(ref.abs().max())
        comp.option("gemm.k_parts", 1)
        plain = comp.exec_torch(a, b)
        assert "parts)" not in comp.report()
        assert float((plain - got).abs().max()) <= 1e-5 * float(ref.abs().max())
    # a product that fills the chip is left alone
    mm_t.option("gemm.k_parts", 0)
    a = torch.randn(2048, 4096, device="cuda").bfloat16()
    mm_t.exec_torch(a, a)
    assert "parts)" not in mm_t.report()


def test_config3_mm_t_through_the_host_f32_abi(torch):
    """BASELINE configs[2] the way the unchanged reference frontend would run it: host f32 arrays holding
    bf16-representable values through i_exec_into (upload, f32 MFMA kernel, download)."""
    n = 4096
    a = oracle.to_bf16_f32(np.random.default_rng(1).uniform(-1, 1, (n, n)).astype(np.float32))
    b = oracle.to_bf16_f32(np.random.default_rng(2).uniform(-1, 1, (n, n)).astype(np.float32))
    comp = i("ik*jk~ijk | i:16,j:16 | jii'j'k") >> i("+ijk~ij | i:16,j:16 | jii'j'k0")
    c = comp.exec_numpy(a, b)
    rows = np.r_[0:4, n - 4:n]
    close(c[rows], oracle.mm_t(a[rows], b), RTOL_F32)
    cols = np.r_[0:4, n - 4:n]
    close(c[:, cols], oracle.mm_t(a, b[cols]), RTOL_F32)


# ------------------------------------------------------------------ NN products: row-major right operand (read in place, or transposed on the device first)
MATMUL = "ik*kj~ijk|i:16,k:16|ii'jkk'", "+ijk~ij|i:16,k:16|ii'j!kk'0"  # test.py's matmul with larger splits


@pytest.mark.parametrize("m,k,n", [(100, 64, 70), (64, 96, 200), (1, 32, 1), (130, 160, 65)])
def test_matmul_nn_f32_vs_emitted_c(torch, m, k, n):
    a, b = rnd((m, k), 1), rnd((k, n), 2)
    comp = i(MATMUL[0]) >> i(MATMUL[1])
    assert "row-major right operand" in comp._code()
    close(comp.exec_numpy(a, b), oracle.compile_component(comp.handle).run(a, b), RTOL_F32)


@pytest.mark.parametrize("m,k,n", [(300, 256, 200), (128, 64, 128), (77, 1024, 513)])
def test_matmul_nn_bf16_device_vs_torch(torch, m, k, n):
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev).manual_seed(3)
    a = (torch.rand(m, k, device=dev, generator=gen) * 2 - 1).bfloat16()
    b = (torch.rand(k, n, device=dev, generator=gen) * 2 - 1).bfloat16()
    comp = i(MATMUL[0]) >> i(MATMUL[1])
    got = comp.exec_torch(a, b)
    ref = a.double() @ b.double()
    assert float((got.double() - ref).abs().max() / ref.abs().max()) <= RTOL_BF16


def test_matmul_nn_batched_and_the_demo_mm(torch):
    a, b = rnd((2, 3, 40, 64), 1), rnd((2, 3, 64, 50), 2)
    batched = i("bhik*bhkj~bhijk | i:16,k:16 | bhkii'jk'") >> i("+bhijk~bhij | i:16,k:16 | bhkii'jk'0")
    assert "row-major right operand" in batched._code()
    close(batched.exec_numpy(a, b), np.einsum("bhik,bhkj->bhij", a.astype(np.float64), b.astype(np.float64)), RTOL_F32)
    p_, v_ = rnd((48, 96), 3), rnd((96, 64), 4)
    mm = i("ij*jk~ikj | i:16,j:16 | jii'kj'") >> i("+ikj~ik | i:16,j:16 | jii'kj'0")
    close(mm.exec_numpy(p_, v_), oracle.compile_component(mm.handle).run(p_, v_), RTOL_F32)


@pytest.mark.parametrize("rows,cols", [(37, 100), (64, 4096), (5, 9000), (300, 33), (1000, 16), (3, 70000), (2, 70002)])
def test_row_max_shift_and_row_normalize_kernels(torch, rows, cols):
    x = rnd((rows, cols), 1)
    shift = (I & i(">ij~i|i:16,j:16|jii'j'")) >> i("ij-i~ij|i:16,j:16|1jii'j'")
    assert "x - row max" in shift._code()
    got = shift.exec_numpy(x)
    assert np.array_equal(got, x - x.max(axis=1, keepdims=True))  # one exact subtraction per element
    pos = np.abs(x) + 0.1
    norm = (I & i("+ij~i|i:16,j:16|jii'j'")) >> i("ij/i~ij|i:16,j:16|1jii'j'")
    assert "x / row sum" in norm._code()
    close(norm.exec_numpy(pos), pos.astype(np.float64) / pos.astype(np.float64).sum(axis=1, keepdims=True), RTOL_F32)
    ex = i("^ij~ij|i:16,j:16|jii'j'")
    assert "exp x" in ex._code()
    small = np.clip(x, -20.0, 5.0)
    close(ex.exec_numpy(small), oracle.compile_component(ex.handle).run(small), RTOL_F32)
    # the three-kernel naive softmax of the reference's demo runs on them
    close(softmax_naive().exec_numpy(x), oracle.row_softmax(x), RTOL_F32)


def test_wide_rows_through_the_naive_and_the_row_staged_schedules(torch):
    """Rows wider than 8192: the fused softmax and the three row kernels of the naive schedule all keep the row in the
    registers of one workgroup; the report names the kernels."""
    x = rnd((6, 20000), 4)
    fused = softmax_rowstaged()
    close(fused.exec_numpy(x), oracle.row_softmax(x), RTOL_F32)
    assert "row_softmax_group_v8" in fused.report()
    three = softmax_naive()
    close(three.exec_numpy(x), oracle.row_softmax(x), RTOL_F32)
    assert all(name in three.report() for name in ("row_shift_group_v8", "row_exp_group_v8", "row_norm_group_v8"))
    ragged = rnd((3, 9001), 5)  # cols % 4 != 0: element-wise loads
    close(three.exec_numpy(ragged), oracle.row_softmax(ragged), RTOL_F32)
    assert "row_shift_group_s4" in three.report()


def test_products_write_bf16_outputs_themselves(torch):
    """bf16 operands with out_dtype bf16: mm_t and the row-major product (k a multiple of 64, and not)
    store bf16 from the kernel, with no f32 staging and no conversion pass; results equal the f32 results rounded."""
    a = torch.from_numpy(oracle.to_bf16_f32(rnd((300, 128), 1))).cuda().bfloat16()
    b = torch.from_numpy(oracle.to_bf16_f32(rnd((264, 128), 2))).cuda().bfloat16()
    mm_t = i("ik*jk~ijk | i:128,j:128 | jii'j'k") >> i("+ijk~ij | i:128,j:128 | jii'j'k0")
    assert torch.equal(mm_t.exec_torch(a, b, out_dtype=torch.bfloat16), mm_t.exec_torch(a, b).bfloat16())
    nn = i("ik*kj~ijk|i:16,j:16|jii'j'k") >> i("+ijk~ij|i:16,j:16|jii'j'k0")
    for kk in (128, 72):  # whole slabs / a partial last slab
        bt = torch.from_numpy(oracle.to_bf16_f32(rnd((kk, 264), 3))).cuda().bfloat16()
        a2 = torch.from_numpy(oracle.to_bf16_f32(rnd((300, kk), 4))).cuda().bfloat16()
        assert torch.equal(nn.exec_torch(a2, bt, out_dtype=torch.bfloat16), nn.exec_torch(a2, bt).bfloat16())


def test_naive_attention_uses_both_gemm_forms(torch):
    """The reference's naive attention (flash-attn.py:57-65): mm_t and mm on the MFMA kernels, the rest generated."""
    q, k, v = rnd((96, 64), 1), rnd((96, 64), 2), rnd((96, 64), 3)
    comp = naive()
    code = comp._code()
    assert "transposed right operand" in code and "row-major right operand" in code
    assert np.allclose(comp.exec_numpy(q, k, v), oracle.np_attention64(q, k, v), rtol=3e-4, atol=5e-5)
    # bf16 operands: S = Q K^T on the bf16 kernel; the probabilities are an f32 intermediate, so P V is an f32 product
    # with V widened on the device (not a generated kernel), sums in f32 as the emitted C has them
    for n, d in ((96, 64), (300, 72), (1000, 128)):
        q, k, v = (oracle.to_bf16_f32(rnd((n, d), s) * 0.5) for s in (1, 2, 3))
        qd, kd, vd = (torch.from_numpy(a).cuda().bfloat16() for a in (q, k, v))
        got = comp.exec_torch(qd, kd, vd)
        lines = comp.report().splitlines()
        assert lines[0].startswith("f0: gemm_nt_bf16") and "gemm_nt_f32" in lines[-1], comp.report()
        close(got.cpu().numpy(), oracle.np_attention64(q, k, v), 3e-4)
        got16 = comp.exec_torch(qd, kd, vd, out_dtype=torch.bfloat16)
        close(got16.float().cpu().numpy(), oracle.np_attention64(q, k, v), 1e-2)


# ------------------------------------------------------------------ BASELINE configs 4 and 5 (bf16 in, f32 accumulate)
def test_config4_attention_slice_vs_oracle(torch):
    """B8 H32 N4096 d128 recipe; two heads on the GPU, one (b,h) slice of query rows against the oracle."""
    B, H, N, D = 1, 2, 4096, 128
    q, k, v = (oracle.to_bf16_f32(rnd((B, H, N, D), s)) for s in (1, 2, 3))
    scale = np.float32(1.0 / np.sqrt(D))
    comp = flash("i:128,j:64", prefix="bh", scaled=True)
    qd, kd, vd = (torch.from_numpy(a).cuda().bfloat16() for a in (q, k, v))
    sd = torch.tensor(scale, device="cuda")
    got = comp.exec_torch(qd, kd, sd, vd).cpu().numpy()
    rows = np.r_[0:64, N - 64:N]
    ref = oracle.attention_tiled(q[:, 1:2, rows], k[:, 1:2], v[:, 1:2], scale)
    close(got[:, 1:2, rows], ref, RTOL_BF16)
    got16 = comp.exec_torch(qd, kd, sd, vd, out_dtype=torch.bfloat16).float().cpu().numpy()
    close(got16[:, 1:2, rows], ref, RTOL_BF16)


def test_schedule_tiles_select_kernel_variants_with_equal_results(torch):
    """The i split of the attention schedule picks the workgroup size (128 or 256 query rows) and the
    i, j splits of mm_t pick the 128 x 128, 192 x 256 or 256 x 256 kernel; the variants agree (attention bitwise)."""
    B, H, N, D = 1, 4, 1024, 128
    q, k, v = (torch.from_numpy(oracle.to_bf16_f32(rnd((B, H, N, D), s))).cuda().bfloat16() for s in (1, 2, 3))
    sd = torch.tensor(np.float32(1.0 / np.sqrt(D)), device="cuda")
    o128 = flash("i:128,j:64", prefix="bh", scaled=True).exec_torch(q, k, sd, v)
    o256 = flash("i:256,j:64", prefix="bh", scaled=True).exec_torch(q, k, sd, v)
    assert torch.equal(o128, o256)
    a = torch.from_numpy(oracle.to_bf16_f32(rnd((512, 256), 1))).cuda().bfloat16()
    b = torch.from_numpy(oracle.to_bf16_f32(rnd((300, 256), 2))).cuda().bfloat16()
    c128 = (i("ik*jk~ijk | i:128,j:128 | jii'j'k") >> i("+ijk~ij | i:128,j:128 | jii'j'k0")).exec_torch(a, b)
    c256 = (i("ik*jk~ijk | i:256,j:256 | jii'j'k") >> i("+ijk~ij | i:256,j:256 | jii'j'k0")).exec_torch(a, b)
    ref = a.float() @ b.float().T
    assert (c128 - ref).abs().max() <= 1e-3 * ref.abs().max()
    assert (c256 - ref).abs().max() <= 1e-3 * ref.abs().max()
    m192 = i("ik*jk~ijk | i:192,j:256 | jii'j'k") >> i("+ijk~ij | i:192,j:256 | jii'j'k0")
    c192 = m192.exec_torch(a, b)
    assert "gemm_nt_bf16_192x256x64_direct_w4" in m192.report(), m192.report()
    assert "the schedule tile selects the kernel" in m192._code()
    assert torch.equal(c192, c256)  # the same sums in the same order, whatever the tile
    m256x192 = i("ik*jk~ijk | i:256,j:192 | jii'j'k") >> i("+ijk~ij | i:256,j:192 | jii'j'k0")
    assert torch.equal(m256x192.exec_torch(a, b), c256) and "gemm_nt_bf16_256x192x64_direct_w4" in m256x192.report()
    # the launcher's own choice: a size whose 256 x 256 tiles leave a partly empty round takes the 192 x 256 tile
    g = torch.Generator(device="cuda").manual_seed(4)
    a, b = ((torch.rand(3072, 1024, device="cuda", generator=g) * 2 - 1).bfloat16() for _ in range(2))
    free = i("ik*jk~ijk | i:16,j:16 | jii'j'k") >> i("+ijk~ij | i:16,j:16 | jii'j'k0")
    c = free.exec_torch(a, b)
    assert "192x256" in free.report(), free.report()
    ref = a.float() @ b.float().T
    assert (c - ref).abs().max() <= 1e-5 * ref.abs().max()


def test_few_heads_under_a_long_key_loop_split_the_keys_of_a_head_over_workgroups(torch, monkeypatch):
    """A single head (or a few sequences) leaves most CUs without a query tile: the executor then runs parts of the
    key loop side by side (each part's normalised rows and the logarithm of its row sums in a temporary) and a
    second kernel merges them.  The program option attention.kv_parts forces a number of parts, so that small operands reach the
    path: every direct bf16 kernel family (d = 128 without a reference, d = 64 with prescaled scores, padded head
    sizes, d = 256), ragged query and key counts, f32 and bf16 results, against the oracle and against the
    unsplit kernel; then the launcher's own choice for one long head."""
    comp = flash(prefix="b", scaled=True)
    for BH, NQ, NK, D, DV in ((1, 300, 4100, 128, 128), (2, 200, 2500, 72, 40), (1, 130, 3000, 256, 256), (3, 257, 2111, 64, 64)):
        q, k, v = (oracle.to_bf16_f32(rnd(shape, s)) for s, shape in ((1, (BH, NQ, D)), (2, (BH, NK, D)), (3, (BH, NK, DV))))
        scale = np.float32(1.0 / np.sqrt(D))
        qd, kd, vd = (torch.from_numpy(a).cuda().bfloat16() for a in (q, k, v))
        sd = torch.tensor(scale, device="cuda")
        rows = np.r_[0:8, NQ - 8:NQ]
        ref = oracle.attention_tiled(q[:, rows], k, v, scale)
        comp.option("attention.kv_parts", 1)
        plain = comp.exec_torch(qd, kd, sd, vd)
        assert "keys in" not in comp.report()
        for parts in (2, 3, 16):
            comp.option("attention.kv_parts", parts)
            got = comp.exec_torch(qd, kd, sd, vd)
            assert "(keys in " in comp.report(), comp.report()
            close(got.cpu().numpy()[:, rows], ref, RTOL_BF16)
            assert float((got - plain).abs().max()) <= 2e-3
            got16 = comp.exec_torch(qd, kd, sd, vd, out_dtype=torch.bfloat16)
            close(got16.float().cpu().numpy()[:, rows], ref, RTOL_BF16)
    # parts whose scores lie far apart: the first third of the keys adds `offset` nats to the scores of rows 0..95, which
    # sends that part of the d = 128 kernel (exponentials without a reference) through its second pass with the
    # running max, and the merge then weighs parts whose sums differ by 2^115 or 2^-430
    plain_flash = flash(prefix="b")
    plain_flash.option("attention.kv_parts", 3)
    comp.option("attention.kv_parts", 3)
    for d in (128, 64):
        for offset in (80.0, -300.0):
            nq, nk = 300, 1500
            q = oracle.to_bf16_f32(rnd((2, nq, d), 1) * 0.5)
            k = oracle.to_bf16_f32(rnd((2, nk, d), 2) * 0.5)
            q[:, :, 0] = 0.0
            q[:, :96, 0] = 1.0
            k[:, :, 0] = 0.0
            k[:, :nk // 3, 0] = oracle.to_bf16_f32(np.full((2, nk // 3), offset, np.float32))
            v = oracle.to_bf16_f32(rnd((2, nk, d), 3))
            ref = oracle.attention_tiled(q, k, v)
            assert np.isfinite(ref).all()
            got = plain_flash.exec_torch(*(torch.from_numpy(a).cuda().bfloat16() for a in (q, k, v)))
            assert "(keys in 3 parts)" in plain_flash.report(), plain_flash.report()
            close(got.cpu().numpy(), ref, RTOL_BF16)
    # f32 operands (the f32 direct kernel, plain and with padded rows), to the f32 bar
    for BH, NQ, NK, D in ((1, 300, 1000, 96), (2, 130, 777, 64), (1, 64, 2100, 128)):
        q, k, v = (rnd(shape, s) for s, shape in ((1, (BH, NQ, D)), (2, (BH, NK, D)), (3, (BH, NK, D))))
        scale = np.float32(1.0 / np.sqrt(D))
        ref = oracle.attention_tiled(q, k, v, scale)
        got = comp.exec_torch(*(torch.from_numpy(a).cuda() for a in (q, k)), torch.tensor(scale, device="cuda"), torch.from_numpy(v).cuda())
        assert "_f32_" in comp.report() and "(keys in 3 parts)" in comp.report(), comp.report()
        close(got.cpu().numpy(), ref, RTOL_F32)
    comp.option("attention.kv_parts", 0)
    # the reference's demo (one f32 head of 512 x 64, 4 workgroups as it is): 8 parts of 64 keys
    q, k, v = (np.random.default_rng(s).uniform(-1, 1, (512, 64)).astype(np.float32) for s in (1, 2, 3))
    demo = flash()
    got = demo.exec_torch(*(torch.from_numpy(a).cuda() for a in (q, k, v)))
    assert "(keys in 8 parts)" in demo.report(), demo.report()
    close(got.cpu().numpy(), oracle.attention_tiled(q, k, v), RTOL_F32)
    # the launcher's choice: one head of 8192 x 128 in 4 parts (64 query tiles for 256 CUs); short key loops and grids that fill
    # the chip as they are
    g = torch.Generator(device="cuda").manual_seed(5)
    q, k, v = (torch.randn(1, 8192, 128, device="cuda", generator=g).bfloat16() for _ in range(3))
    sd = torch.tensor(128 ** -0.5, device="cuda")
    got = comp.exec_torch(q, k, sd, v)
    assert "(keys in 4 parts)" in comp.report(), comp.report()
    ref = torch.softmax((q[:, :64].double() @ k.double().transpose(1, 2)) * 128 ** -0.5, -1) @ v.double()
    assert float((got[:, :64].double() - ref).abs().max()) <= 2e-3
    comp.exec_torch(q[:, :1024].contiguous(), k[:, :1024].contiguous(), sd, v[:, :1024].contiguous())
    assert "keys in" not in comp.report()
    comp.exec_torch(q[:, :100].contiguous(), k, sd, v)  # a few queries against many keys: 16 parts of 512
    assert "(keys in 16 parts)" in comp.report(), comp.report()
    q, k, v = (torch.randn(64, 8192, 128, device="cuda", generator=g).bfloat16() for _ in range(3))
    comp.exec_torch(q, k, sd, v)
    assert "keys in" not in comp.report()


def test_random_shapes_through_the_split_loops(torch, monkeypatch):
    """Forty random attentions (bf16 and f32, head sizes of every kernel family, 1 to 400 queries, 130 to 3000 keys)
    with their keys in 2 to 32 parts, and forty random products (NT and NN, bf16 and f32, every extent ragged) with
    their k loop in 2 to 32 parts, against float64."""
    import random

    rng = random.Random(7)
    fa = flash(prefix="b", scaled=True)
    mm_t = i("bik*bjk~bijk | i:16,j:16 | bjii'j'k") >> i("+bijk~bij | i:16,j:16 | bjii'j'k0")
    mm = i("bik*bkj~bijk|i:16,k:16|bii'jkk'") >> i("+bijk~bij|i:16,k:16|bii'j!kk'0")
    split = 0
    for case in range(40):
        bf16 = rng.random() < 0.6
        bh, nq, nk = rng.choice([1, 1, 2, 3]), rng.randint(1, 400), rng.randint(130, 3000)
        d = rng.choice([64, 128, 72, 40, 256, 96] if bf16 else [64, 128, 96, 40])
        dv = d if rng.random() < 0.7 else rng.choice([64, 128, 32 + 8 * rng.randint(0, 8)])
        if not bf16 and dv > 128:
            dv = d
        dt = torch.bfloat16 if bf16 else torch.float32
        g = torch.Generator(device="cuda").manual_seed(case)
        q, k, v = ((torch.randn(bh, n, w, device="cuda", generator=g) * 0.7).to(dt) for n, w in ((nq, d), (nk, d), (nk, dv)))
        ref = torch.softmax((q.double() @ k.double().transpose(1, 2)) * d ** -0.5, -1) @ v.double()
        fa.option("attention.kv_parts", rng.choice([2, 3, 5, 8, 13, 32]))
        print("case attention", case, bf16, bh, nq, nk, d, dv, flush=True)
        got = fa.exec_torch(q, k, torch.tensor(d ** -0.5, device="cuda"), v)
        split += "(keys in" in fa.report()
        assert float((got.double() - ref).abs().max()) <= (RTOL_BF16 if bf16 else RTOL_F32) * float(ref.abs().max()), fa.report()
    assert split >= 30  # (head sizes no direct kernel has run unsplit)
    split = 0
    for case in range(40):
        kind = rng.choice(["nt16", "nn16", "nt32", "nn32"])
        bh, m, n, k = rng.choice([1, 1, 2, 5]), rng.randint(1, 500), rng.randint(1, 500), rng.randint(64, 6000)
        k = k // 8 * 8 if kind.endswith("16") else k // 4 * 4
        if kind == "nn16":
            n = max(8, n // 8 * 8)
        dt = torch.bfloat16 if kind.endswith("16") else torch.float32
        g = torch.Generator(device="cuda").manual_seed(100 + case)
        a = (torch.rand(bh, m, k, device="cuda", generator=g) * 2 - 1).to(dt)
        b = (torch.rand(*((bh, n, k) if kind.startswith("nt") else (bh, k, n)), device="cuda", generator=g) * 2 - 1).to(dt)
        ref = a.double() @ (b.double().transpose(1, 2) if kind.startswith("nt") else b.double())
        print("case product", case, kind, bh, m, n, k, flush=True)
        comp = mm_t if kind.startswith("nt") else mm
        comp.option("gemm.k_parts", rng.choice([2, 3, 4, 7, 16, 32]))
        got = comp.exec_torch(a, b)
        split += "(k in" in comp.report()
        bar = 1e-2 if kind.endswith("16") else RTOL_F32
        assert float((got.double() - ref).abs().max()) <= bar * max(float(ref.abs().max()), 1e-30), comp.report()
    assert split >= 25  # (m * n that is no multiple of 4 runs unsplit)


def test_softmax_of_a_few_very_long_rows_runs_every_row_in_parts(torch):
    """Fewer rows than half the CUs, 2^17 columns and more: every row in parts over workgroups (a first launch leaves
    each part's running max and sum of exponentials, a second combines them and writes).  Aligned and unaligned
    widths, one row and several, a row whose largest element sits in its last part, against float64; rows that are
    many or short keep the one-workgroup-per-row kernels."""
    sm = softmax_rowstaged()
    for rows, cols in ((1, 1 << 20), (3, 1 << 17), (8, (1 << 18) + 3), (100, 200001), (5, 150000)):
        g = torch.Generator(device="cuda").manual_seed(rows)
        x = torch.randn(rows, cols, device="cuda", generator=g) * 3
        x[0, cols - 7] = 40.0
        y = sm.exec_torch(x)
        assert "(rows in " in sm.report(), sm.report()
        ref = torch.softmax(x.double(), -1)
        assert float((y.double() - ref).abs().max()) <= RTOL_F32 * float(ref.abs().max())
        assert float((y.double().sum(-1) - 1).abs().max()) <= 1e-4
    for rows, cols in ((200, 1 << 17), (8, 70000)):
        sm.exec_torch(torch.randn(rows, cols, device="cuda"))
        assert "rows in" not in sm.report()


def test_attention_with_operands_of_both_types_runs_on_the_f32_kernels(torch):
    """Q in bf16 against K and V in f32 (and the other way round): an f32 attention, the bf16 operands widened on the
    device first, not a generated kernel; head sizes of the fused f32 kernel and of the three-kernel form."""
    comp = flash(prefix="b", scaled=True)
    for d, types in ((64, (torch.bfloat16, torch.float32, torch.float32)), (128, (torch.float32, torch.bfloat16, torch.bfloat16)),
                     (160, (torch.bfloat16, torch.float32, torch.bfloat16))):
        g = torch.Generator(device="cuda").manual_seed(d)
        q, k, v = ((torch.randn(2, n, d, device="cuda", generator=g) * 0.5).to(t) for n, t in zip((200, 332, 332), types))
        got = comp.exec_torch(q, k, torch.tensor(d ** -0.5, device="cuda"), v)
        assert "generated" not in comp.report() and "f32" in comp.report(), comp.report()
        ref = torch.softmax((q.double() @ k.double().transpose(1, 2)) * d ** -0.5, -1) @ v.double()
        assert float((got.double() - ref).abs().max()) <= RTOL_F32 * float(ref.abs().max())


def test_temporaries_are_kept_from_call_to_call_on_a_stream(torch):
    """Calls enqueued back to back on one stream carve their temporaries (here the two [rows, cols] intermediates
    of the naive softmax) from one block that the library keeps and replaces when a call needs more: operands that
    grow and shrink from call to call without a synchronisation in between, then two streams interleaved, each
    with a block of its own."""
    comp = softmax_naive()
    g = torch.Generator(device="cuda").manual_seed(11)
    xs = [torch.randn(*shape, device="cuda", generator=g) for shape in ((64, 100), (2048, 3000), (300, 77), (2048, 3000), (5, 9), (4096, 2000))]
    torch.cuda.synchronize()
    outs = [comp.exec_torch(x) for x in xs]
    torch.cuda.synchronize()
    for x, y in zip(xs, outs):
        assert float((y.double() - torch.softmax(x.double(), -1)).abs().max()) <= 1e-6
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    results = []
    for rep in range(3):
        for stream, x in zip(streams, (xs[1], xs[5])):
            with torch.cuda.stream(stream):
                results.append((x, comp.exec_torch(x)))
    torch.cuda.synchronize()
    for x, y in results:
        assert float((y.double() - torch.softmax(x.double(), -1)).abs().max()) <= 1e-6


def test_config4_full_size_properties(torch):
    B, H, N, D = 8, 32, 4096, 128
    g = torch.Generator(device="cuda").manual_seed(1)
    q, k, v = (torch.randn(B, H, N, D, device="cuda", generator=g).bfloat16() for _ in range(3))
    v[..., 5] = -0.75            # a constant column must come out constant: rows are convex combinations
    q[3, 7], k[3, 7], v[3, 7] = q[0, 1], k[0, 1], v[0, 1]
    sd = torch.tensor(D ** -0.5, device="cuda")
    out = flash("i:128,j:64", prefix="bh", scaled=True).exec_torch(q, k, sd, v)
    assert out.shape == (B, H, N, D) and torch.isfinite(out).all()
    assert (out[..., 5] + 0.75).abs().max().item() < 1e-2
    assert torch.equal(out[3, 7], out[0, 1])
    assert (out <= v.float().amax(dim=2, keepdim=True) + 1e-3).all()


def test_config5_long_sequence_slice_vs_oracle(torch):
    """B1 H16 N32768 d64, inputs x2.0: full length on the GPU, a few query rows against the oracle."""
    N, D = 32768, 64
    q, k, v = (oracle.to_bf16_f32(rnd((1, 1, N, D), s) * 2.0) for s in (1, 2, 3))
    scale = np.float32(1.0 / np.sqrt(D))
    comp = flash("i:128,j:64", prefix="bh", scaled=True)
    got = comp.exec_torch(*(torch.from_numpy(a).cuda().bfloat16() for a in (q, k)), torch.tensor(scale, device="cuda"),
                          torch.from_numpy(v).cuda().bfloat16()).cpu().numpy()
    rows = np.r_[0:16, N - 16:N]
    ref = oracle.attention_tiled(q[:, :, rows], k, v, scale)
    close(got[:, :, rows], ref, RTOL_BF16)


def np_inputs(shape, amp=1.0):
    """The operand recipe of the BASELINE configurations: NumPy default_rng(seed).standard_normal, seeds 1, 2, 3."""
    return [oracle.to_bf16_f32(np.random.default_rng(seed).standard_normal(shape, dtype=np.float32) * np.float32(amp))
            for seed in (1, 2, 3)]


def test_config4_full_size_with_the_benchmark_schedule_vs_oracle(torch):
    """B8 H32 N4096 d128 with the schedule bench.py times, i:256,j:64 (the 8-wave direct kernel), at full size:
    four (b, h) slices, first and last 32 query rows of each (the first and the last workgroup of a head, and rows
    of its first and last wave), against the oracle on identical inputs."""
    B, H, N, D = 8, 32, 4096, 128
    q, k, v = np_inputs((B, H, N, D))
    scale = np.float32(1.0 / np.sqrt(D))
    comp = flash("i:256,j:64", prefix="bh", scaled=True)
    got = comp.exec_torch(torch.from_numpy(q).cuda().bfloat16(), torch.from_numpy(k).cuda().bfloat16(),
                          torch.tensor(scale, device="cuda"), torch.from_numpy(v).cuda().bfloat16())
    assert "attn_fwd_bf16_d128_bn64_direct_w8 (tile 256 x 64)" in comp.report()
    rows = np.r_[0:32, N - 32:N]
    for b, h in ((0, 0), (3, 17), (7, 31), (5, 8)):
        ref = oracle.attention_tiled(q[b, h][rows], k[b, h], v[b, h], scale)
        close(got[b, h][torch.from_numpy(rows).cuda()].cpu().numpy(), ref, RTOL_BF16)


def test_config5_full_size_with_the_benchmark_schedule_vs_oracle(torch):
    """B1 H16 N32768 d64, inputs x 2.0, with the schedule bench.py times, i:512,j:32 (64 queries per wave), on all
    16 heads at once: three heads x first and last 32 query rows against the oracle."""
    B, H, N, D = 1, 16, 32768, 64
    q, k, v = np_inputs((B, H, N, D), amp=2.0)
    scale = np.float32(1.0 / np.sqrt(D))
    comp = flash("i:512,j:32", prefix="bh", scaled=True)
    got = comp.exec_torch(torch.from_numpy(q).cuda().bfloat16(), torch.from_numpy(k).cuda().bfloat16(),
                          torch.tensor(scale, device="cuda"), torch.from_numpy(v).cuda().bfloat16())
    assert "attn_fwd_bf16_d64_bn32_q64 (tile 512 x 32)" in comp.report()
    rows = np.r_[0:32, N - 32:N]
    for h in (0, 7, 15):
        ref = oracle.attention_tiled(q[0, h][rows], k[0, h], v[0, h], scale)
        close(got[0, h][torch.from_numpy(rows).cuda()].cpu().numpy(), ref, RTOL_BF16)


def test_schedule_tiles_reach_the_kernels_and_unknown_tiles_are_reported(torch):
    """The i and j splits of the attention schedule select the kernel with that workgroup tile; a tile that no
    kernel has is reported, in the plan and after the run, instead of being replaced silently."""
    B, H, N, D = 1, 2, 640, 128
    q, k, v = (torch.from_numpy(a).cuda().bfloat16() for a in np_inputs((B, H, N, D)))
    sd = torch.tensor(np.float32(1.0 / np.sqrt(D)), device="cuda")
    outs = {}
    for ti, tj, name in ((64, 32, "d128_bn32_direct_w2"), (64, 64, "d128_bn64_direct_w2"), (128, 32, "d128_bn32_direct "),
                         (128, 64, "d128_bn64_direct "), (256, 32, "d128_bn32_direct_w8"), (256, 64, "d128_bn64_direct_w8")):
        comp = flash(f"i:{ti},j:{tj}", prefix="bh", scaled=True)
        outs[ti, tj] = comp.exec_torch(q, k, sd, v)
        assert f"attn_fwd_bf16_{name}" in comp.report() and f"(tile {ti} x {tj})" in comp.report()
        assert "the schedule tile selects the kernel" in comp._code()
    ref = outs[128, 64]
    for out in outs.values():
        assert (out - ref).abs().max() <= 2e-2 * ref.abs().max()
    odd = flash("i:16,j:16", prefix="bh", scaled=True)
    assert "no hand-written kernel has this tile" in odd._code()
    odd.exec_torch(q, k, sd, v)
    assert "the schedule asks for 16 x 16, which no hand-written kernel has" in odd.report()
    # the f32-scale form is a program option
    precise = flash("i:256,j:64", prefix="bh", scaled=True).option("attention.f32_scale", 1)
    out = precise.exec_torch(q, k, sd, v)
    assert "attn_fwd_bf16_d128_bn64_direct_w8_f32scale" in precise.report()
    assert (out - ref).abs().max() <= 2e-2 * ref.abs().max()
    with pytest.raises(RuntimeError):
        precise.option("no.such.option", 1)


def test_rescale_stress_max_in_last_tile(torch):
    # every key tile raises the running max of every row
    nq, nk, d = 100, 700, 16
    q = np.ones((nq, d), np.float32)
    k = (np.arange(nk, dtype=np.float32)[:, None] * np.ones((1, d), np.float32)) * 0.125
    v = rnd((nk, d), 3)
    close(flash().exec_numpy(q, k, v), oracle.attention_tiled(q, k, v), RTOL_F32)
    qb, kb, vb = (torch.from_numpy(oracle.to_bf16_f32(a)).cuda().bfloat16() for a in (q, k, v))
    ref = oracle.attention_tiled(*(oracle.to_bf16_f32(a) for a in (q, k, v)))
    close(flash().exec_torch(qb, kb, vb).cpu().numpy(), ref, RTOL_BF16)


# ------------------------------------------------------------------ edge cases and the ABI on a live device
def test_multi_output_and_swap(torch):
    x = rnd((9, 14), 1)
    two = i("+ij~i") & i(">ij~j")
    a, b = two.exec_numpy(x)
    assert np.allclose(a, x.sum(1), rtol=1e-5, atol=1e-5) and np.array_equal(b, x.max(0))
    b2, a2 = (~two).exec_numpy(x)
    assert np.array_equal(b2, b) and np.array_equal(a2, a)


def test_scalar_output_and_scalar_input(torch):
    x = rnd((6, 11), 1)
    assert np.allclose(i("+ij~.").exec_numpy(x), x.sum(dtype=np.float64), rtol=1e-5, atol=1e-5)
    got = i("ij*.~ij").exec_numpy(x, np.array(2.5, np.float32))
    assert np.array_equal(got, x * np.float32(2.5))


def test_all_pointwise_ops(torch):
    x, y = rnd((5, 7), 1), rnd((5, 7), 2)
    ax, ay = np.abs(x) + 0.5, np.abs(y) + 0.5
    cases = [("ij+ij~ij", x + y), ("ij*ij~ij", x * y), ("ij-ij~ij", x - y), ("ij/ij~ij", x / ay if False else None),
             ("ij>ij~ij", np.maximum(x, y)), ("ij<ij~ij", np.minimum(x, y)), ("ij>>ij~ij", (x > y) * 1.0),
             ("ij>=ij~ij", (x >= y) * 1.0), ("ij<<ij~ij", (x < y) * 1.0), ("ij<=ij~ij", (x <= y) * 1.0),
             ("ij==ij~ij", (x == y) * 1.0), ("ij!=ij~ij", (x != y) * 1.0)]
    for src, ref in cases:
        if ref is not None:
            assert np.allclose(i(src).exec_numpy(x, y), ref.astype(np.float32), rtol=1e-6, atol=0), src
    assert np.allclose(i("ij/ij~ij").exec_numpy(x, ay), x / ay, rtol=1e-6)
    assert np.allclose(i("ij^ij~ij").exec_numpy(ax, y), np.power(ax, y), rtol=1e-5)
    bx, by = (x > 0) * 1.0, (y > 0) * 1.0
    assert np.array_equal(i("ij&&ij~ij").exec_numpy(bx, by), np.logical_and(bx, by) * 1.0)
    assert np.array_equal(i("ij||ij~ij").exec_numpy(bx, by), np.logical_or(bx, by) * 1.0)
    assert np.array_equal(i("ij^^ij~ij").exec_numpy(bx, by), np.logical_xor(bx, by) * 1.0)
    unary = [("-ij~ij", -x), ("/ij~ij", 1 / ax), (">ij~ij", np.maximum(x, 0)), ("<ij~ij", np.minimum(x, 0)),
             ("^ij~ij", np.exp(x)), ("$ij~ij", np.log(ax)), ("!!ij~ij", (bx == 0) * 1.0), (">>ij~ij", (x > 0) * 1.0)]
    for src, ref in unary:
        arg = ax if src[0] in "/$" else bx if src.startswith("!!") else x
        assert np.allclose(i(src).exec_numpy(arg), ref.astype(np.float32), rtol=1e-5, atol=1e-6), src


def test_empty_and_ragged_extents(torch):
    mm = i("ik*jk~ijk | i:16,j:16 | jii'j'k") >> i("+ijk~ij | i:16,j:16 | jii'j'k0")
    assert mm.exec_numpy(np.zeros((0, 5), np.float32), np.zeros((3, 5), np.float32)).shape == (0, 3)
    a, b = rnd((1, 1), 1), rnd((1, 1), 2)
    assert np.allclose(mm.exec_numpy(a, b), a @ b.T)
    q, k, v = rnd((17, 3), 1), rnd((1, 3), 2), rnd((1, 5), 3)
    close(flash().exec_numpy(q, k, v), np.broadcast_to(v, (17, 5)), RTOL_F32)  # one key: output is that value row


def test_exec_rejects_wrong_rank_and_missing_inputs(torch):
    mm = i("ik*kj~ijk") >> i("+ijk~ij")
    with pytest.raises(RuntimeError):
        mm.exec_numpy(np.zeros((4,), np.float32), np.zeros((4, 3), np.float32))
    with pytest.raises(RuntimeError):
        mm.exec_numpy(np.zeros((4, 4), np.float32))


def test_device_entry_is_stream_ordered_and_repeatable(torch):
    x = torch.randn(64, 256, device="cuda")
    sm = softmax_naive()  # three generated kernels with two stream-ordered intermediates
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        outs = [sm.exec_torch(x) for _ in range(5)]
    side.synchronize()
    ref = torch.softmax(x, -1)
    for o in outs:
        assert (o - ref).abs().max().item() < 1e-5


def test_non_f32_host_inputs_are_converted_like_the_reference(torch):
    x = np.arange(12, dtype=np.int64).reshape(3, 4)
    assert np.array_equal(i("+ij~i").exec_numpy(x), x.sum(1).astype(np.float32))
    xt = np.asfortranarray(rnd((5, 6), 1))
    assert np.allclose(i("+ij~i").exec_numpy(xt), xt.sum(1), rtol=1e-5, atol=1e-6)


def test_every_loop_nest_of_a_generated_kernel_is_a_kernel_of_its_own(torch):
    """Kernels whose body is a sequence of loop nests and that no hand-written kernel covers run as one kernel per
    nest, each with a grid of its own (the vectors they share are intermediates of the plan, the stream orders them).
    A column normalisation (no hand-written form), and the naive three-kernel softmax and the naive attention with
    every kernel forced into its generated form, against the emitted C."""
    x = rnd((300, 70), 1)
    colnorm = (I & i("+ij~j||ij")) >> i("ij/j~ij||1ij")  # the column sums staged at the root: one kernel, two nests
    close(colnorm.exec_numpy(x), x / x.sum(axis=0), RTOL_F32)
    close(colnorm.exec_numpy(x), oracle.compile_component(colnorm.handle).run(x), RTOL_F32)
    assert "2 loop nests, a kernel each: generated kernel f0" in colnorm.report() and "; generated kernel f1" in colnorm.report()
    xd = torch.from_numpy(x).cuda()
    assert torch.equal(colnorm.exec_torch(xd), colnorm.exec_torch(xd))  # repeatable
    sm = softmax_naive()
    sm.option("generated.only", 1)
    y = rnd((130, 257), 2)
    close(sm.exec_numpy(y), oracle.row_softmax(y), RTOL_F32)
    assert sm.report().count("2 loop nests, a kernel each") == 2  # row_max_shift and row_normalize
    q, k, v = rnd((40, 24), 1), rnd((50, 24), 2), rnd((50, 24), 3)
    nv = naive()
    nv.option("generated.only", 1)
    close(nv.exec_numpy(q, k, v), oracle.compile_component(nv.handle).run(q, k, v), RTOL_F32)


def test_generated_reductions_that_the_parallel_loops_alone_cannot_spread_over_the_chip(torch):
    """A sum to a single element, a column sum of a few thousand columns, a column normalisation: the parallel loops
    of the reduction nest are 1, 4096 and 4096 iterations, so its outermost sequential loop runs in parts over
    groups of work-items, each part on copies of its own of the accumulated buffer, which a second kernel folds in
    part order.  Against the emitted C (sums in another order: the bar is relative to the sum of magnitudes), at sizes
    the C finishes in seconds and with the number of parts forced as well as left to the launcher; then the full
    sizes against float64 on the device, with a bound on the time: before, these ran as one wavefront's or one
    workgroup's work (21 ms, 0.43 ms and 2.6 ms)."""
    x = np.abs(rnd((1000, 700), 1)) + 0.1
    for src, ref, bar in (("+ij~.", x.astype(np.float64).sum(), x.sum()), ("+ij~j", x.astype(np.float64).sum(0), x.sum(0).max()),
                          (">ij~j", x.max(0), 1.0), ("*ij~j|i:4|ii'j", None, None)):
        for parts in (0, 7, 64, 1):
            comp = i(src)
            comp.option("generated.parts", parts)
            data = x if not src.startswith("*") else (x[:40] * 0.5 + 0.7)
            got = comp.exec_numpy(data)
            emitted = oracle.compile_component(comp.handle).run(data)
            assert np.abs(got - emitted).max() <= RTOL_F32 * (bar if bar is not None else np.abs(emitted).max()), (src, parts)
            if ref is not None:
                assert np.abs(got - ref).max() <= RTOL_F32 * bar, (src, parts)
            assert ("in 7 parts" in comp.report()) == (parts == 7), comp.report()
            if parts == 1:
                assert "parts" not in comp.report()
    colnorm = (I & i("+ij~j||ij")) >> i("ij/j~ij||1ij")
    for parts in (0, 5):
        colnorm.option("generated.parts", parts)
        close(colnorm.exec_numpy(x), oracle.compile_component(colnorm.handle).run(x), RTOL_F32)
        close(colnorm.exec_numpy(x), x / x.sum(0), RTOL_F32)
    # full sizes
    import bench

    g = torch.Generator(device="cuda").manual_seed(3)
    big = torch.rand(4096, 4096, device="cuda", generator=g) + 0.1
    total = i("+ij~.")
    out = torch.empty((), device="cuda")
    total.into(out, big)
    assert "parts over wavefronts" in total.report(), total.report()
    assert abs(float(out) - float(big.double().sum())) <= RTOL_F32 * float(big.double().sum())
    _, ms = bench.time_steps(torch, lambda: total.into(out, big), 50, 10)
    assert ms <= 0.1, f"sum of 4096 x 4096 to one element takes {ms * 1000:.0f} us"
    tall = torch.rand(16384, 4096, device="cuda", generator=g) + 0.1
    col = i("+ij~j")
    sums = torch.empty(4096, device="cuda")
    col.into(sums, tall)
    assert "parts over work-items" in col.report(), col.report()
    assert float((sums.double() - tall.double().sum(0)).abs().max()) <= RTOL_F32 * float(tall.double().sum(0).max())
    _, ms = bench.time_steps(torch, lambda: col.into(sums, tall), 30, 5)
    assert ms <= 0.2, f"column sums of 16384 x 4096 take {ms * 1000:.0f} us"
    colnorm.option("generated.parts", 0)
    normed = torch.empty_like(tall)
    colnorm.into(normed, tall)
    ref = tall.double() / tall.double().sum(0)
    assert float((normed.double() - ref).abs().max()) <= RTOL_F32 * float(ref.max())
    _, ms = bench.time_steps(torch, lambda: colnorm.into(normed, tall), 30, 5)
    assert ms <= 0.5, f"column normalisation of 16384 x 4096 takes {ms * 1000:.0f} us"


@pytest.mark.parametrize("wave", ["1", "0", None])
def test_reduction_nests_in_the_wavefront_form(torch, monkeypatch, wave):
    """Generated reduction nests have a second form in which a wavefront stands where a work-item stood (the
    reduction loop spread over 64 lanes, lane shares combined by a butterfly).  Forced on, forced off and left to
    the launcher (the program option generated.wave), against NumPy in float64 and, at sizes it finishes quickly, the
    emitted C."""
    x = rnd((300, 2500), 1)
    x64 = x.astype(np.float64)
    for src, ref in ((">ij~i", x64.max(1)), ("<ij~i", x64.min(1)), ("+ij~i", x64.sum(1)), ("+ij~j", x64.sum(0)),
                     (">ij~j", x64.max(0)), ("+ij~i|j:16|ijj'", x64.sum(1)), ("+ij~.", x64.sum())):
        comp = i(src)
        if wave is not None:
            comp.option("generated.wave", int(wave))
        got = comp.exec_numpy(x)
        # sums of 2500 unit normals: the bar is relative to the sum of magnitudes, which bounds the rounding error
        assert np.abs(got - ref).max() <= RTOL_F32 * np.abs(x64).sum(1).max(), src
        if wave is None and src in (">ij~i", "+ij~i"):  # (300 rows: the lanes over the columns, and the columns in parts too)
            assert "_w: one wavefront per iteration" in comp.report() or "parts over wavefronts" in comp.report(), comp.report()
        if wave is None and src == "+ij~j":  # (strided reads: a work-item per column, the rows in parts)
            assert "parts over work-items" in comp.report(), comp.report()
        if wave == "0":
            assert "_w:" not in comp.report() and "wavefronts" not in comp.report()
    small = rnd((37, 130), 2)
    for src in ("+ij~i", ">ij~j", "*ij~i"):
        comp = i(src)  # (kept alive: the oracle reads the component behind the handle)
        close(comp.exec_numpy(small * 0.5 + 1), oracle.compile_component(comp.handle).run(small * 0.5 + 1), RTOL_F32)
    # a product fused into its row sum (a matrix-vector product), then the reference's mlp at a size with long rows
    w1, v, w2 = rnd((200, 1500), 3), rnd((1500,), 4), rnd((70, 200), 5)
    fused = i("ij*j~ij||ij") >> i("+ij~i||ij0")
    close(fused.exec_numpy(w1, v), w1.astype(np.float64) @ v.astype(np.float64), RTOL_F32)
    mvp = i("ij*j~ij") >> i("+ij~i")
    mlp = (i("ij~ij") | (mvp >> i(">i~i"))) >> mvp
    close(mlp.exec_numpy(w2, w1, v), w2.astype(np.float64) @ np.maximum(w1.astype(np.float64) @ v, 0), RTOL_F32)
    # batched rows, sums over two axes, short rows (which stay with one work-item per row)
    xb = rnd((5, 33, 700), 6)
    close(i("+bij~bi").exec_numpy(xb), xb.astype(np.float64).sum(2), RTOL_F32)
    close(i("+bij~b").exec_numpy(xb), xb.astype(np.float64).sum((1, 2)), 5e-4)
    close(i(">ij~i").exec_numpy(rnd((5000, 20), 7)), rnd((5000, 20), 7).max(1), RTOL_F32)
    # the device entry, twice: same bits
    xd = torch.from_numpy(x).cuda()
    assert torch.equal(i("+ij~i").exec_torch(xd), i("+ij~i").exec_torch(xd))
