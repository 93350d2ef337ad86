"""Parity of the hand-written gfx950 kernels (called through the C ABI of
include/i_hip.h) against the CPU oracle on identical seeded inputs.

Tolerances (relative to max|oracle|): 1e-4 for f32 paths, 2e-2 for bf16 inputs
with f32 accumulation.
"""
import numpy as np
import pytest

import oracle
from conftest import gemm_kernel_knobs

pytestmark = pytest.mark.gpu

RTOL_F32 = 1e-4
RTOL_BF16 = 2e-2


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


def rnd(shape, seed, kind="normal"):
    rng = np.random.default_rng(seed)
    if kind == "uniform":
        return rng.uniform(-1, 1, shape).astype(np.float32)
    return rng.standard_normal(shape, dtype=np.float32)


def relerr(got, ref):
    return float(np.abs(got - ref).max() / np.abs(ref).max())


def assert_close(got, ref, rtol):
    assert got.shape == ref.shape
    assert np.isfinite(got).all()
    err = relerr(got, ref)
    assert err <= rtol, f"relative error {err} > {rtol}"
    assert np.allclose(got, ref, rtol=rtol, atol=rtol * np.abs(ref).max())


def gpu_attention(env, q, k, v, scale, bf16, out_bf16=False):
    t = env.torch
    lead = q.shape[:-2]
    bh = int(np.prod(lead)) if lead else 1
    nq, d = q.shape[-2:]
    nk, dv = v.shape[-2:]
    dt = t.bfloat16 if bf16 else t.float32
    qd, kd, vd = (t.from_numpy(a).cuda().to(dt).contiguous() for a in (q, k, v))
    od = t.full(lead + (nq, dv), float("nan"), device="cuda", dtype=t.bfloat16 if out_bf16 else t.float32)
    env.nat.check(env.nat.core.i_hip_attention(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), od.data_ptr(),
                                               env.nat.BF16 if bf16 else env.nat.F32,
                                               env.nat.BF16 if out_bf16 else env.nat.F32,
                                               bh, nq, nk, d, dv, 1.0 if scale is None else scale, env.stream()))
    t.cuda.synchronize()
    return od.float().cpu().numpy()


def gpu_attention_ex(env, q, k, v, scale, query_tile=0, key_tile=0, f32_scale=False):
    """bf16 operands, f32 output, through i_hip_attention_ex (the schedule's tile and the scale mode spelled out)."""
    t = env.torch
    lead = q.shape[:-2]
    bh = int(np.prod(lead)) if lead else 1
    nq, d = q.shape[-2:]
    nk, dv = v.shape[-2:]
    qd, kd, vd = (t.from_numpy(a).cuda().to(t.bfloat16).contiguous() for a in (q, k, v))
    od = t.full(lead + (nq, dv), float("nan"), device="cuda", dtype=t.float32)
    env.nat.check(env.nat.core.i_hip_attention_ex(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), od.data_ptr(), env.nat.BF16,
                                                  env.nat.F32, bh, nq, nk, d, dv, scale, query_tile, key_tile,
                                                  int(f32_scale), env.stream()))
    t.cuda.synchronize()
    return od.cpu().numpy()


# ------------------------------------------------------------------ attention, f32
@pytest.mark.parametrize("case", ["u_48x24", "u_64x64", "u_100x40", "n_48x24", "n_33x17"])
def test_attention_f32_vs_reference_golden(env, golden, case):
    q, k, v, o = (golden[f"{case}.{x}"] for x in "qkvo")
    assert_close(gpu_attention(env, q, k, v, None, bf16=False), o, RTOL_F32)


@pytest.mark.parametrize("shape,kind", [((512, 64), "uniform"), ((500, 60), "uniform"), ((1, 1), "normal"),
                                        ((2, 3, 4, 8), "normal"), ((6, 100, 40), "normal"), ((2, 130, 128), "normal")])
def test_attention_f32_vs_oracle(env, shape, kind):
    q, k, v = (rnd(shape, s, kind) for s in (1, 2, 3))
    assert_close(gpu_attention(env, q, k, v, None, bf16=False), oracle.attention_tiled(q, k, v), RTOL_F32)


def test_attention_f32_ragged_nq_nk_dv_and_scale(env):
    q, k, v = rnd((3, 77, 24), 1), rnd((3, 130, 24), 2), rnd((3, 130, 40), 3)
    assert_close(gpu_attention(env, q, k, v, 0.2, bf16=False), oracle.attention_tiled(q, k, v, 0.2), RTOL_F32)


def test_attention_f32_online_rescale_stress(env):
    nq, nk, d = 40, 300, 8
    q = np.ones((nq, d), np.float32)
    k = (np.arange(nk, dtype=np.float32)[:, None] * np.ones((1, d), np.float32)) * 0.25
    v = rnd((nk, d), 3)
    assert_close(gpu_attention(env, q, k, v, None, bf16=False), oracle.attention_tiled(q, k, v), RTOL_F32)


@pytest.mark.parametrize("d", [64, 128, 36, 60, 96, 100, 124])
@pytest.mark.parametrize("direct", [True, False])
def test_attention_f32_direct_and_staged_kernels_vs_oracle(env, knobs, d, direct):
    """f32 operands with d == dv that is a multiple of 4 above 32 run the kernel that moves K/V tiles global -> LDS directly
    (with its LDS rows padded when d is neither 64 nor 128), everything else (and the launcher option attention.direct=0) the
    register-staged one: both against the oracle on one tile, partial tiles, several heads (more than the 8 XCDs),
    ragged query counts, negative and zero scales, and a longer key loop."""
    if not direct:
        knobs["attention.direct"] = 0
    for bh, nq, nk, scale in ((1, 128, 32, 1.0), (3, 200, 333, 0.11), (2, 77, 130, -0.2), (9, 130, 64, 0.0), (1, 1, 1, 1.0),
                              (2, 512, 1024, float(np.float32(1.0 / np.sqrt(d))))):
        q, k, v = (rnd((bh, n, d), sd) for sd, n in ((1, nq), (2, nk), (3, nk)))
        assert_close(gpu_attention(env, q, k, v, scale, bf16=False), oracle.attention_tiled(q, k, v, scale), RTOL_F32)


@pytest.mark.parametrize("d,dv", [(64, 128), (128, 64), (40, 72), (100, 36), (24, 64)])
def test_attention_f32_different_head_sizes_of_k_and_v(env, d, dv):
    """f32 with d != dv (multiples of 4, the larger above 32): the padded form of the direct kernel."""
    for bh, nq, nk, scale in ((1, 128, 32, 1.0), (3, 200, 333, 0.11), (9, 130, 64, -0.2)):
        q, k, v = (rnd((bh, n, w), sd) for sd, n, w in ((1, nq, d), (2, nk, d), (3, nk, dv)))
        assert_close(gpu_attention(env, q, k, v, scale, bf16=False), oracle.attention_tiled(q, k, v, scale), RTOL_F32)


def test_attention_f32_operands_not_16_byte_aligned(env):
    """The direct f32 kernel moves 16 bytes per lane; operands that start off a 16-byte boundary take the
    register-staged kernel and give the same result."""
    t = env.torch
    bh, n, d = 2, 100, 64
    q, k, v = (rnd((bh, n, d), sd) for sd in (1, 2, 3))
    ref = oracle.attention_tiled(q, k, v, 0.3)
    bufs = [t.zeros(bh * n * d + 1, device="cuda") for _ in range(4)]
    views = [b[1:] for b in bufs]
    for view, a in zip(views[:3], (q, k, v)):
        view.copy_(t.from_numpy(a).reshape(-1))
    assert all(x.data_ptr() % 16 != 0 for x in views)
    env.nat.check(env.nat.core.i_hip_attention(views[0].data_ptr(), views[1].data_ptr(), views[2].data_ptr(), views[3].data_ptr(),
                                               env.nat.F32, env.nat.F32, bh, n, n, d, d, 0.3, env.stream()))
    t.cuda.synchronize()
    assert_close(views[3].cpu().numpy().reshape(bh, n, d), ref, RTOL_F32)


# ------------------------------------------------------------------ attention, bf16 in / f32 accumulate
@pytest.mark.parametrize("bh,nq,nk,d", [(1, 64, 64, 64), (2, 128, 128, 128), (3, 200, 333, 128), (2, 77, 130, 64),
                                        (1, 512, 512, 64), (2, 100, 100, 40), (1, 1, 1, 8)])
def test_attention_bf16_vs_oracle(env, bh, nq, nk, d):
    q, k, v = (oracle.to_bf16_f32(rnd((bh, n, d), s)) for s, n in ((1, nq), (2, nk), (3, nk)))
    scale = float(np.float32(1.0 / np.sqrt(d)))
    ref = oracle.attention_tiled(q, k, v, scale)
    assert_close(gpu_attention(env, q, k, v, scale, bf16=True), ref, RTOL_BF16)
    assert_close(gpu_attention(env, q, k, v, scale, bf16=True, out_bf16=True), ref, RTOL_BF16)


@pytest.mark.parametrize("d", [8, 24, 40, 56, 72, 80, 96, 112, 120])
@pytest.mark.parametrize("waves", ["4", "8", "staged"])
def test_attention_bf16_head_sizes_between_the_kernel_sizes(env, knobs, d, waves):
    """d == dv that is a multiple of 8 but neither 64 nor 128 runs the direct-to-LDS kernels with LDS rows padded to
    64 or 128 columns (4 and 8 waves per workgroup forced in turn; "staged": the register-staged kernel these
    shapes used to take).  Short and long key loops (the steady state needs four full tiles), partial tiles, ragged
    query counts, more heads than XCDs, both output types."""
    if waves == "staged":
        knobs["attention.direct"] = 0
    else:
        knobs["attention.waves"] = waves
    scale = float(np.float32(1.0 / np.sqrt(d)))
    for bh, nq, nk in ((1, 64, 64), (3, 200, 333), (9, 130, 700), (2, 300, 1024)):
        q, k, v = (oracle.to_bf16_f32(rnd((bh, n, d), s)) for s, n in ((1, nq), (2, nk), (3, nk)))
        ref = oracle.attention_tiled(q, k, v, scale)
        assert_close(gpu_attention(env, q, k, v, scale, bf16=True), ref, RTOL_BF16)
        assert_close(gpu_attention(env, q, k, v, scale, bf16=True, out_bf16=True), ref, RTOL_BF16)


def test_attention_bf16_padded_head_size_keeps_its_neighbours_untouched(env):
    """The padded kernels store only the first d columns of an output row: the next row's first elements and the
    element after the last row stay as they were (checked with a guard element around a d = 72 output)."""
    t = env.torch
    bh, nq, nk, d = 2, 150, 400, 72
    q, k, v = (oracle.to_bf16_f32(rnd((bh, n, d), s)) for s, n in ((1, nq), (2, nk), (3, nk)))
    qd, kd, vd = (t.from_numpy(a).cuda().bfloat16().contiguous() for a in (q, k, v))
    whole = t.full((bh * nq * d + 8,), -7.0, device="cuda")
    od = whole[4:-4]
    env.nat.check(env.nat.core.i_hip_attention(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), od.data_ptr(), env.nat.BF16,
                                               env.nat.F32, bh, nq, nk, d, d, 0.1, env.stream()))
    t.cuda.synchronize()
    assert (whole[:4] == -7.0).all().item() and (whole[-4:] == -7.0).all().item()
    assert_close(od.cpu().numpy().reshape(bh, nq, d), oracle.attention_tiled(q, k, v, 0.1), RTOL_BF16)


@pytest.mark.parametrize("d,dv", [(128, 64), (64, 128), (192, 128), (40, 72), (256, 136), (96, 256), (8, 16), (128, 120)])
@pytest.mark.parametrize("f32_scale", [False, True])
def test_attention_bf16_different_head_sizes_of_k_and_v(env, d, dv, f32_scale):
    """d != dv: the padded direct-to-LDS kernels with K rows of d and V rows of dv elements in LDS rows of 64, 128 or
    256 columns (the larger of the two decides).  Partial tiles, long key loops, ragged query counts, several heads."""
    scale = float(np.float32(1.0 / np.sqrt(d)))
    for bh, nq, nk in ((1, 64, 64), (3, 200, 333), (9, 130, 700)):
        q, k, v = (oracle.to_bf16_f32(rnd((bh, n, w), s)) for s, n, w in ((1, nq, d), (2, nk, d), (3, nk, dv)))
        ref = oracle.attention_tiled(q, k, v, scale)
        assert_close(gpu_attention_ex(env, q, k, v, scale, f32_scale=f32_scale), ref, RTOL_BF16)
    if not f32_scale:
        assert_close(gpu_attention(env, q, k, v, scale, bf16=True, out_bf16=True), ref, RTOL_BF16)


@pytest.mark.parametrize("d", [136, 160, 192, 224, 256])
def test_attention_bf16_head_sizes_above_128(env, d):
    """d == dv in 136 .. 256 (multiples of 8) runs the direct-to-LDS kernel for 256-column rows: one wave per SIMD,
    32-key tiles, LDS rows padded when d < 256.  One tile, partial tiles, long key loops (the steady state needs four
    full tiles), ragged query counts, more heads than XCDs, both output types, and scores large enough that the pass
    without a reference overflows and the second pass takes over."""
    scale = float(np.float32(1.0 / np.sqrt(d)))
    for bh, nq, nk, amp in ((1, 32, 32, 1.0), (3, 200, 333, 1.0), (9, 130, 700, 1.0), (2, 300, 1024, 1.0), (2, 128, 512, 4.0)):
        q, k, v = (oracle.to_bf16_f32(rnd((bh, n, d), s) * np.float32(a)) for s, n, a in ((1, nq, amp), (2, nk, amp), (3, nk, 1.0)))
        ref = oracle.attention_tiled(q, k, v, scale)
        assert_close(gpu_attention(env, q, k, v, scale, bf16=True), ref, RTOL_BF16 if amp == 1.0 else 6e-2)
        assert_close(gpu_attention(env, q, k, v, scale, bf16=True, out_bf16=True), ref, RTOL_BF16 if amp == 1.0 else 6e-2)


@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("force", [None, "waves8", "q64", "staged"])
def test_attention_bf16_every_kernel_vs_oracle(env, knobs, d, force):
    """The launcher picks between the direct-to-LDS kernel (4 or 8 waves per workgroup), the 64-queries-per-wave
    kernel (d = 64) and the register-staged kernel; force each of them on one ragged problem (7 full 64-key
    tiles + a partial one, so the steady-state loop, its drain and the masked tail all run)."""
    if force == "q64" and d != 64:
        pytest.skip("the 64-queries-per-wave kernel exists for d = 64 only")
    if force == "waves8":
        knobs["attention.waves"] = "8"
    elif force == "q64":
        knobs["attention.waves"] = "64"
    elif force == "staged":
        knobs["attention.direct"] = 0
    bh, nq, nk = 2, 300, 450
    q, k, v = (oracle.to_bf16_f32(rnd((bh, n, d), s)) for s, n in ((1, nq), (2, nk), (3, nk)))
    scale = float(np.float32(1.0 / np.sqrt(d)))
    ref = oracle.attention_tiled(q, k, v, scale)
    assert_close(gpu_attention(env, q, k, v, scale, bf16=True), ref, RTOL_BF16)
    assert_close(gpu_attention(env, q, k, v, scale, bf16=True, out_bf16=True), ref, RTOL_BF16)


def test_attention_bf16_workgroup_sizes_agree_bitwise(env, knobs):
    """A wave does the same arithmetic whether its workgroup has 4 or 8 waves."""
    bh, n, d = 16, 1024, 128
    q, k, v = (oracle.to_bf16_f32(rnd((bh, n, d), s)) for s in (1, 2, 3))
    knobs["attention.waves"] = "4"
    a = gpu_attention(env, q, k, v, 0.1, bf16=True)
    knobs["attention.waves"] = "8"
    b = gpu_attention(env, q, k, v, 0.1, bf16=True)
    assert np.array_equal(a, b)
    knobs["attention.waves"] = "3"
    t = env.torch
    x = t.zeros(1, 8, 128, device="cuda", dtype=t.bfloat16)
    rc = env.nat.core.i_hip_attention(x.data_ptr(), x.data_ptr(), x.data_ptr(), x.data_ptr(), 1, 1, 1, 8, 8, 128, 128,
                                      1.0, env.stream())
    assert rc == -1 and "attention.waves" in env.nat.last_error()


@pytest.mark.parametrize("q64", [False, True])
@pytest.mark.parametrize("span", [20.0, 45.0, 90.0])
def test_attention_bf16_reference_max_moves_slowly_and_fast(env, knobs, span, q64):
    """Scores rise steadily along the keys by `span` nats in total over 10 tiles.  The direct kernel
    moves a row's reference max only when a tile exceeds it by 2^8: span 20 never reaches that after
    the first tile, 45 reaches it every other tile, 90 at every tile."""
    if q64:
        knobs["attention.waves"] = "64"
    nq, nk, d = 64, 640, 64
    q = np.ones((1, nq, d), np.float32)
    k = oracle.to_bf16_f32((np.arange(nk, dtype=np.float32)[None, :, None] * np.ones((1, 1, d), np.float32))
                           * np.float32(span / (nk * d)))
    v = oracle.to_bf16_f32(rnd((1, nk, d), 3))
    ref = oracle.attention_tiled(q, k, v, 1.0)
    assert_close(gpu_attention(env, q, k, v, 1.0, bf16=True), ref, RTOL_BF16)


@pytest.mark.parametrize("d", [64, 128, "64 (64 queries per wave)"])
@pytest.mark.parametrize("jump_tile", [1, 6, 11])
def test_attention_bf16_score_jump_overflows_the_stale_reference(env, knobs, d, jump_tile):
    """All scores are ~0 except in one key tile, where they are ~+300 nats: exp against the reference of the
    earlier tiles overflows to inf there.  The steady-state loop takes no row max; its row-sum guard has to
    catch this before the tile's PV product and move the reference.  Rows 32.. keep small scores throughout."""
    if d == "64 (64 queries per wave)":
        knobs["attention.waves"] = "64"
        d = 64
    nq, nk = 64, 12 * 64 + 40
    q = np.zeros((1, nq, d), np.float32)
    q[:, :32, 0] = 1.0
    q[:, 32:, 1] = 0.5
    k = oracle.to_bf16_f32(rnd((1, nk, d), 2) * 0.25)
    k[:, :, 0] = 0.0
    k[:, 64 * jump_tile:64 * jump_tile + 64, 0] = oracle.to_bf16_f32(np.linspace(296, 304, 64, dtype=np.float32))
    v = oracle.to_bf16_f32(rnd((1, nk, d), 3))
    ref = oracle.attention_tiled(q, k, v, 1.0)
    assert np.isfinite(ref).all()
    assert_close(gpu_attention(env, q, k, v, 1.0, bf16=True), ref, RTOL_BF16)


@pytest.mark.parametrize("waves,d", [("4", 128), ("8", 128), ("64", 64)])
@pytest.mark.parametrize("offset", [-300.0, -75.0, -60.0, 0.0, 25.0, 50.0, 60.0, 80.0])
def test_attention_bf16_scores_far_from_zero(env, knobs, waves, d, offset):
    """Every score of rows 0..95 is `offset` nats plus noise.  The steady state of these kernels takes exp of the score
    as it is, with no reference: within range (-75 .. 50) it must stay accurate, and where a tile's row sum
    leaves the range (60, 80) or the whole row underflows (-300) the workgroup has to notice and compute the item
    again with the running max.  The other rows keep scores near zero, next to the affected ones in the same
    workgroup; the last query tile is a partial one."""
    knobs["attention.waves"] = waves
    nq, nk = 300, 7 * 64 + 10
    q = oracle.to_bf16_f32(rnd((2, nq, d), 1) * 0.5)
    k = oracle.to_bf16_f32(rnd((2, nk, d), 2) * 0.5)
    q[:, :, 0] = 0.0
    q[:, :96, 0] = 1.0
    k[:, :, 0] = oracle.to_bf16_f32(np.full((2, nk), offset, np.float32))
    v = oracle.to_bf16_f32(rnd((2, nk, d), 3))
    ref = oracle.attention_tiled(q, k, v, 1.0)
    assert np.isfinite(ref).all()
    assert_close(gpu_attention(env, q, k, v, 1.0, bf16=True), ref, RTOL_BF16)


@pytest.mark.parametrize("d,waves", [(128, "8"), (64, "8"), (64, "64")])
def test_attention_bf16_large_scores_error_growth(env, knobs, d, waves):
    """The direct kernels fold scale * log2(e) into Q, rounded to bf16 once more: a perturbation of the scores that
    grows with their magnitude.  Inputs x 1, x 2 (the recipe of the long-sequence configuration) and x 3 (scores of
    +-35 nats, far more peaked than attention): the error against the f64 closed form stays below 1e-2, 1.5e-2
    and 3e-2 of max |reference|; the last is looser than the 2e-2 bar of the other tests and states where it ends."""
    knobs["attention.waves"] = waves
    bh, nq, nk = 2, 200, 1100
    for amp, bound in ((1.0, 1e-2), (2.0, 1.5e-2), (3.0, 3e-2)):
        q, k, v = (oracle.to_bf16_f32(rnd((bh, n, d), s) * np.float32(amp)) for s, n in ((1, nq), (2, nk), (3, nk)))
        scale = float(np.float32(1.0 / np.sqrt(d)))
        s = np.einsum("bik,bjk->bij", q.astype(np.float64), k.astype(np.float64)) * scale
        p = np.exp(s - s.max(axis=-1, keepdims=True))
        ref = np.einsum("bij,bjk->bik", p / p.sum(axis=-1, keepdims=True), v.astype(np.float64))
        got = gpu_attention(env, q, k, v, scale, bf16=True)
        err = np.abs(got - ref).max() / np.abs(ref).max()
        assert err <= bound, f"inputs x {amp}: error {err} > {bound}"


@pytest.mark.parametrize("d,tile", [(128, 128), (128, 256), (64, 128), (64, 256), (96, 128), (96, 256), (40, 128), (40, 256),
                                    (192, 128), (256, 128)])
def test_attention_bf16_f32_scale_keeps_the_bar_at_any_score_magnitude(env, d, tile):
    """f32_scale: the score scale multiplies every score in f32 (the reference's arithmetic) and Q is not rounded a
    second time (head sizes 64 and 128, and the padded and the 256-column kernels for the others).  Same inputs as above, x 1, x 2 and x 3: the error stays inside the 2e-2 bar, and does not grow
    with the magnitude of the scores the way the folded form's does."""
    bh, nq, nk = 2, 200, 1100
    for amp in (1.0, 2.0, 3.0):
        q, k, v = (oracle.to_bf16_f32(rnd((bh, n, d), s) * np.float32(amp)) for s, n in ((1, nq), (2, nk), (3, nk)))
        scale = float(np.float32(1.0 / np.sqrt(d)))
        s = np.einsum("bik,bjk->bij", q.astype(np.float64), k.astype(np.float64)) * scale
        p = np.exp(s - s.max(axis=-1, keepdims=True))
        ref = np.einsum("bij,bjk->bik", p / p.sum(axis=-1, keepdims=True), v.astype(np.float64))
        got = gpu_attention_ex(env, q, k, v, scale, query_tile=tile, key_tile=64, f32_scale=True)
        err = np.abs(got - ref).max() / np.abs(ref).max()
        assert err <= 1e-2, f"inputs x {amp}: error {err}"


@pytest.mark.parametrize("d,query_tile,key_tile", [(128, 64, 64), (128, 64, 32), (128, 128, 32), (128, 256, 32),
                                                   (128, 128, 64), (128, 256, 64), (64, 64, 64), (64, 64, 32),
                                                   (64, 128, 32), (64, 128, 64), (64, 256, 64), (64, 512, 32)])
@pytest.mark.parametrize("f32_scale", [False, True])
def test_attention_bf16_every_schedule_tile_vs_oracle(env, d, query_tile, key_tile, f32_scale):
    """Every (query tile, key tile) kernel of the direct-to-LDS family, and the f32-scale form of the tiles that
    have one, on a ragged problem long enough for the steady-state loop (9 full 64-key tiles + 10 keys), a second
    problem that is too short for it, and one with a single query and a single key."""
    scale = float(np.float32(1.0 / np.sqrt(d)))
    for nq, nk in ((300, 9 * 64 + 10), (70, 100), (1, 1)):
        q, k, v = (oracle.to_bf16_f32(rnd((3, n, d), s)) for s, n in ((1, nq), (2, nk), (3, nk)))
        ref = oracle.attention_tiled(q, k, v, scale)
        got = gpu_attention_ex(env, q, k, v, scale, query_tile, key_tile, f32_scale)
        assert_close(got, ref, RTOL_BF16)


@pytest.mark.parametrize("q64", [False, True])
def test_attention_bf16_direct_negative_and_zero_scale(env, knobs, q64):
    if q64:
        knobs["attention.waves"] = "64"
    q, k, v = (oracle.to_bf16_f32(rnd((2, n, 64), s)) for s, n in ((1, 70), (2, 400), (3, 400)))
    for scale in (-0.3, 0.0):
        ref = oracle.np_attention64(q, k, v, scale).astype(np.float32)
        assert_close(gpu_attention(env, q, k, v, scale, bf16=True), ref, RTOL_BF16)


def test_attention_bf16_config4_slice_vs_oracle(env):
    """One (b, h) slice of B8 H32 N4096 d128 at full sequence length, against the oracle on 256 query rows."""
    n, d = 4096, 128
    q, k, v = (oracle.to_bf16_f32(rnd((1, n, d), s)) for s in (1, 2, 3))
    scale = float(np.float32(1.0 / np.sqrt(d)))
    got = gpu_attention(env, q, k, v, scale, bf16=True)
    rows = np.r_[0:128, n - 128:n]
    ref = oracle.attention_tiled(q[:, rows], k, v, scale)
    assert_close(got[:, rows], ref, RTOL_BF16)


@pytest.mark.parametrize("waves", ["8", "64"])
def test_attention_bf16_long_sequence_rescale_stress(env, knobs, waves):
    """Config 5 recipe (inputs x2.0, d=64) at N=8192: heavy running-max movement; the 8-wave kernel and the
    64-queries-per-wave kernel that the launcher picks at the full size."""
    knobs["attention.waves"] = waves
    n, d = 8192, 64
    q, k, v = (oracle.to_bf16_f32(rnd((1, n, d), s) * 2.0) for s in (1, 2, 3))
    scale = float(np.float32(1.0 / np.sqrt(d)))
    got = gpu_attention(env, q, k, v, scale, bf16=True)
    rows = np.r_[0:64, n - 64:n]
    ref = oracle.attention_tiled(q[:, rows], k, v, scale)
    assert_close(got[:, rows], ref, RTOL_BF16)


def test_attention_full_size_properties(env):
    """Size-independent properties at B8 H32 N4096 d128: rows are convex combinations of V
    (constant V column -> constant output), and identical heads give identical outputs."""
    t = env.torch
    bh, n, d = 256, 4096, 128
    g = t.Generator(device="cuda").manual_seed(1)
    q = t.randn(bh, n, d, device="cuda", generator=g).bfloat16()
    k = t.randn(bh, n, d, device="cuda", generator=g).bfloat16()
    v = t.randn(bh, n, d, device="cuda", generator=g).bfloat16()
    v[:, :, 0] = 1.5
    q[7], k[7], v[7] = q[200], k[200], v[200]
    o = t.empty(bh, n, d, device="cuda", dtype=t.float32)
    env.nat.check(env.nat.core.i_hip_attention(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), 1, 0,
                                               bh, n, n, d, d, d ** -0.5, env.stream()))
    t.cuda.synchronize()
    assert t.isfinite(o).all()
    assert (o[:, :, 0] - 1.5).abs().max().item() < 2e-2
    assert t.equal(o[7], o[200])
    vmax = v.float().amax(dim=1, keepdim=True)
    vmin = v.float().amin(dim=1, keepdim=True)
    assert (o <= vmax + 1e-3).all() and (o >= vmin - 1e-3).all()


def test_attention_rejects_unsupported(env):
    t = env.torch
    x = t.zeros(1, 8, 256, device="cuda")
    rc = env.nat.core.i_hip_attention(x.data_ptr(), x.data_ptr(), x.data_ptr(), x.data_ptr(), 0, 0, 1, 8, 8, 256, 256,
                                      1.0, env.stream())
    assert rc == -1 and "unsupported" in env.nat.last_error()
    rc = env.nat.core.i_hip_attention(x.data_ptr(), x.data_ptr(), x.data_ptr(), x.data_ptr(), 0, 0, 1, 8, 8, 64, 64,
                                      float("inf"), env.stream())
    assert rc == -1 and "scale" in env.nat.last_error()
    rc = env.nat.core.i_hip_attention(x.data_ptr(), x.data_ptr(), x.data_ptr(), x.data_ptr(), 1, 0, 1, 8, 8, 60, 60,
                                      1.0, env.stream())
    assert rc == -1  # bf16 rows must be 16-byte multiples
    # above 128: bf16 with d, dv <= 256, multiples of 8
    xb = t.zeros(1, 8, 320, device="cuda", dtype=t.bfloat16)
    for d, dv, f32_scale in ((192, 132, 0), (264, 264, 0), (136, 260, 1)):
        rc = env.nat.core.i_hip_attention_ex(xb.data_ptr(), xb.data_ptr(), xb.data_ptr(), x.data_ptr(), 1, 0, 1, 8, 8, d, dv,
                                             1.0, 0, 0, f32_scale, env.stream())
        assert rc == -1 and "unsupported" in env.nat.last_error(), (d, dv, f32_scale)


def test_attention_negative_and_zero_scale(env):
    q, k, v = rnd((2, 70, 32), 1), rnd((2, 90, 32), 2), rnd((2, 90, 32), 3)
    for scale in (-0.4, 0.0):
        ref = oracle.np_attention64(q, k, v, scale).astype(np.float32)
        assert_close(gpu_attention(env, q, k, v, scale, bf16=False), ref, RTOL_F32)
    qb, kb, vb = (oracle.to_bf16_f32(a) for a in (q, k, v))
    ref = oracle.np_attention64(qb, kb, vb, -0.4).astype(np.float32)
    assert_close(gpu_attention(env, qb, kb, vb, -0.4, bf16=True), ref, RTOL_BF16)


# ------------------------------------------------------------------ mm_t
@pytest.mark.parametrize("bh,m,n,k", [(1, 128, 128, 64), (1, 100, 70, 40), (2, 300, 260, 136), (1, 1, 1, 8),
                                      (1, 512, 384, 1024)])
def test_gemm_nt_bf16_vs_oracle(env, bh, m, n, k):
    t = env.torch
    a = oracle.to_bf16_f32(rnd((bh, m, k), 1, "uniform"))
    b = oracle.to_bf16_f32(rnd((bh, n, k), 2, "uniform"))
    ad, bd = t.from_numpy(a).cuda().bfloat16(), t.from_numpy(b).cuda().bfloat16()
    cd = t.full((bh, m, n), float("nan"), device="cuda")
    env.nat.check(env.nat.core.i_hip_gemm_nt_bf16(ad.data_ptr(), bd.data_ptr(), cd.data_ptr(), bh, m, n, k, env.stream()))
    t.cuda.synchronize()
    assert_close(cd.cpu().numpy(), oracle.mm_t(a, b), RTOL_BF16)


@pytest.mark.parametrize("bh,m,n,k", [(1, 256, 256, 64), (1, 300, 260, 128), (2, 600, 520, 192), (1, 1, 1, 256),
                                      (3, 257, 255, 320)])
@pytest.mark.parametrize("direct", ["256", "256w8", "192", "256x192", "128", "0"])
def test_gemm_nt_bf16_every_kernel_vs_oracle(env, knobs, bh, m, n, k, direct):
    """The launcher picks between the 256 x 256 (four waves; "w8": the form with eight), 192 x 256 and 128 x 128
    direct-to-LDS kernels and the register-staged kernel by problem size; force each of them on small ragged
    problems with 1 to 5 k-slabs, edge tiles on both axes and several batches."""
    gemm_kernel_knobs(knobs, direct)
    if direct.endswith("w8"):
        knobs["gemm.waves"] = 8
    t = env.torch
    a = oracle.to_bf16_f32(rnd((bh, m, k), 1, "uniform"))
    b = oracle.to_bf16_f32(rnd((bh, n, k), 2, "uniform"))
    ad, bd = t.from_numpy(a).cuda().bfloat16(), t.from_numpy(b).cuda().bfloat16()
    cd = t.full((bh, m, n), float("nan"), device="cuda")
    env.nat.check(env.nat.core.i_hip_gemm_nt_bf16(ad.data_ptr(), bd.data_ptr(), cd.data_ptr(), bh, m, n, k, env.stream()))
    t.cuda.synchronize()
    assert_close(cd.cpu().numpy(), oracle.mm_t(a, b), RTOL_BF16)


@pytest.mark.parametrize("bh,m,n,k", [(1, 256, 256, 8), (1, 300, 264, 40), (2, 600, 520, 136), (1, 1, 8, 200), (3, 257, 256, 1000),
                                      (1, 128, 128, 72)])
@pytest.mark.parametrize("nn", [False, True])
@pytest.mark.parametrize("tile", ["128", "192", "256x192", "256", "256w8"])
def test_gemm_bf16_k_that_is_no_multiple_of_64(env, knobs, bh, m, n, k, nn, tile):
    """k % 8 == 0 but k % 64 != 0: the direct kernels with a partial last slab (the lanes past k clear their LDS
    slots), every tile size (and both forms of the largest) forced here at small sizes; NT and NN (which has no
    192 x 256 tile and takes 256 x 256 for it), f32 and bf16 output."""
    gemm_kernel_knobs(knobs, tile)
    if tile.endswith("w8"):
        knobs["gemm.waves"] = 8
    t = env.torch
    a = oracle.to_bf16_f32(rnd((bh, m, k), 1, "uniform"))
    b = oracle.to_bf16_f32(rnd((bh, n, k), 2, "uniform"))
    ref = oracle.mm_t(a, b)
    ad = t.from_numpy(a).cuda().bfloat16()
    bd = t.from_numpy(np.ascontiguousarray(b.transpose(0, 2, 1)) if nn else b).cuda().bfloat16()
    cd = t.full((bh, m, n), float("nan"), device="cuda")
    core = env.nat.core
    if nn:
        env.nat.check(core.i_hip_gemm_nn_bf16(ad.data_ptr(), bd.data_ptr(), cd.data_ptr(), bh, m, n, k, env.stream()))
    else:
        env.nat.check(core.i_hip_gemm_nt_bf16(ad.data_ptr(), bd.data_ptr(), cd.data_ptr(), bh, m, n, k, env.stream()))
        c16 = t.full((bh, m, n), float("nan"), device="cuda", dtype=t.bfloat16)
        env.nat.check(core.i_hip_gemm_nt_bf16_ex(ad.data_ptr(), bd.data_ptr(), c16.data_ptr(), env.nat.BF16, bh, m, n, k, 0, 0,
                                                  env.stream()))
    t.cuda.synchronize()
    assert_close(cd.cpu().numpy(), ref, RTOL_BF16)
    if not nn:
        assert t.equal(c16, cd.bfloat16())


def test_gemm_four_wave_form_does_not_read_what_registers_held_before(env, knobs):
    """The four-wave form of the 256 x 256 tile spells its matrix instructions as inline assembly and carries its own
    wait states.  Its first matrix instructions multiply zeroed operands; issued too soon after the zeroing they read
    what the registers held before, which is visible when that was NaN: products of NaN operands run first here, so
    that the register file is full of NaN, then several small multi-batch products (many short-lived workgroups)."""
    t = env.torch
    poison = t.full((2048, 512), float("nan"), device="cuda", dtype=t.bfloat16)
    sink = t.empty(2048, 2048, device="cuda")
    core = env.nat.core
    for rep in range(6):
        gemm_kernel_knobs(knobs, ("256", "192", "256x192")[rep % 3])  # (the three four-wave tiles)
        env.nat.check(core.i_hip_gemm_nt_bf16(poison.data_ptr(), poison.data_ptr(), sink.data_ptr(), 1, 2048, 2048, 512, env.stream()))
        for bh, m, n, k in ((3, 677, 61, 128), (4, 512, 61, 128), (3, 677, 60, 256), (2, 300, 264, 64)):
            g = t.Generator(device="cuda").manual_seed(100 * rep + m)
            a = (t.rand(bh, m, k, device="cuda", generator=g) * 2 - 1).bfloat16()
            b = (t.rand(bh, n, k, device="cuda", generator=g) * 2 - 1).bfloat16()
            c = t.full((bh, m, n), 12345.0, device="cuda")
            env.nat.check(core.i_hip_gemm_nt_bf16(a.data_ptr(), b.data_ptr(), c.data_ptr(), bh, m, n, k, env.stream()))
            bn = b[:, : n // 8 * 8].transpose(1, 2).contiguous()  # the same product with a row-major right operand
            cn = t.full((bh, m, n // 8 * 8), 12345.0, device="cuda")
            env.nat.check(core.i_hip_gemm_nn_bf16(a.data_ptr(), bn.data_ptr(), cn.data_ptr(), bh, m, n // 8 * 8, k, env.stream()))
            t.cuda.synchronize()
            ref = a.double() @ b.double().transpose(1, 2)
            assert float((c.double() - ref).abs().max()) <= 1e-2 * float(ref.abs().max()), (rep, bh, m, n, k)
            assert float((cn.double() - ref[:, :, : n // 8 * 8]).abs().max()) <= 1e-2 * float(ref.abs().max()), (rep, bh, m, n, k)


@pytest.mark.parametrize("tile", [0, 128, 192, 256, (256, 192)])
def test_gemm_nt_bf16_output_in_bf16(env, knobs, tile):
    """bf16 output: the kernels round their f32 sums to nearest-even on the way out, so the result equals the f32
    result rounded to bf16, bit for bit, for the register-staged kernel (gemm.direct=0) and every tile."""
    t = env.torch
    if tile == 0:
        gemm_kernel_knobs(knobs, "0")
    tile, tile_n = tile if isinstance(tile, tuple) else (tile, 256 if tile == 192 else tile)
    for bh, m, n, k in ((2, 300, 260, 128), (1, 512, 512, 576), (3, 1, 1, 64)):
        a = oracle.to_bf16_f32(rnd((bh, m, k), 1, "uniform"))
        b = oracle.to_bf16_f32(rnd((bh, n, k), 2, "uniform"))
        ad, bd = t.from_numpy(a).cuda().bfloat16(), t.from_numpy(b).cuda().bfloat16()
        c32 = t.full((bh, m, n), float("nan"), device="cuda")
        c16 = t.full((bh, m, n), float("nan"), device="cuda", dtype=t.bfloat16)
        core = env.nat.core
        env.nat.check(core.i_hip_gemm_nt_bf16_ex(ad.data_ptr(), bd.data_ptr(), c32.data_ptr(), env.nat.F32, bh, m, n, k,
                                                  tile, tile_n, env.stream()))
        env.nat.check(core.i_hip_gemm_nt_bf16_ex(ad.data_ptr(), bd.data_ptr(), c16.data_ptr(), env.nat.BF16, bh, m, n, k,
                                                  tile, tile_n, env.stream()))
        t.cuda.synchronize()
        assert t.equal(c16, c32.bfloat16())
        assert_close(c32.cpu().numpy(), oracle.mm_t(a, b), RTOL_BF16)


@pytest.mark.parametrize("tile", [128, 192, 256, (256, 192)])
@pytest.mark.parametrize("out_bf16", [False, True])
def test_gemm_nt_bf16_output_not_16_byte_aligned(env, out_bf16, tile):
    """The direct kernels store four columns per lane when C allows it; a C that starts one element past a
    16-byte boundary takes the element-wise stores instead.  The elements before and after C stay untouched."""
    t = env.torch
    bh, m, n, k = 2, 300, 260, 128
    tile, tile_n = tile if isinstance(tile, tuple) else (tile, 256 if tile == 192 else tile)
    a = oracle.to_bf16_f32(rnd((bh, m, k), 1, "uniform"))
    b = oracle.to_bf16_f32(rnd((bh, n, k), 2, "uniform"))
    ad, bd = t.from_numpy(a).cuda().bfloat16(), t.from_numpy(b).cuda().bfloat16()
    whole = t.full((bh * m * n + 2,), -7.0, device="cuda", dtype=t.bfloat16 if out_bf16 else t.float32)
    cd = whole[1:-1]
    assert cd.data_ptr() % 16 != 0
    env.nat.check(env.nat.core.i_hip_gemm_nt_bf16_ex(ad.data_ptr(), bd.data_ptr(), cd.data_ptr(),
                                                      env.nat.BF16 if out_bf16 else env.nat.F32, bh, m, n, k, tile,
                                                      tile_n, env.stream()))
    t.cuda.synchronize()
    assert whole[0].item() == -7.0 and whole[-1].item() == -7.0
    ref = oracle.mm_t(a, b)
    got = cd.float().cpu().numpy().reshape(bh, m, n)
    assert_close(got, oracle.to_bf16_f32(ref) if out_bf16 else ref, RTOL_BF16)


@pytest.mark.parametrize("bh,m,n,k", [(1, 256, 256, 64), (1, 300, 264, 128), (2, 600, 520, 192), (1, 1, 8, 256),
                                      (3, 257, 248, 320), (1, 130, 1000, 64)])
@pytest.mark.parametrize("direct", ["256", "128"])
def test_gemm_nn_bf16_vs_oracle(env, knobs, bh, m, n, k, direct):
    """Row-major right operand (c = a b, b [k, n]) on the direct kernels: 1 to 5 k-slabs, edge tiles on both
    axes (n a multiple of 8 only), several batches, both workgroup tiles."""
    gemm_kernel_knobs(knobs, direct)
    t = env.torch
    a = oracle.to_bf16_f32(rnd((bh, m, k), 1, "uniform"))
    b = oracle.to_bf16_f32(rnd((bh, k, n), 2, "uniform"))
    ad, bd = t.from_numpy(a).cuda().bfloat16(), t.from_numpy(b).cuda().bfloat16()
    cd = t.full((bh, m, n), float("nan"), device="cuda")
    env.nat.check(env.nat.core.i_hip_gemm_nn_bf16(ad.data_ptr(), bd.data_ptr(), cd.data_ptr(), bh, m, n, k, env.stream()))
    t.cuda.synchronize()
    assert_close(cd.cpu().numpy(), oracle.mm_t(a, np.ascontiguousarray(b.transpose(0, 2, 1))), RTOL_BF16)


def test_gemm_nn_bf16_rejects_what_the_direct_kernels_cannot_read(env):
    t = env.torch
    x = t.zeros(64 * 72, device="cuda", dtype=t.bfloat16)
    c = t.zeros(64 * 72, device="cuda")
    for m, n, k in ((64, 60, 64), (64, 64, 36)):
        rc = env.nat.core.i_hip_gemm_nn_bf16(x.data_ptr(), x.data_ptr(), c.data_ptr(), 1, m, n, k, env.stream())
        assert rc == -1 and "gemm_nn" in env.nat.last_error()


@pytest.mark.parametrize("bh,m,n,k", [(1, 256, 256, 32), (1, 300, 260, 96), (2, 600, 520, 160), (1, 1, 1, 64),
                                      (3, 257, 255, 320), (1, 100, 70, 64),
                                      # k a multiple of 4 but not of 32: a partial last slab
                                      (1, 256, 256, 40), (2, 300, 260, 100), (1, 100, 70, 4), (3, 257, 255, 1004), (1, 64, 64, 28)])
@pytest.mark.parametrize("tile", ["256", "128"])
def test_gemm_nt_f32_vs_oracle(env, knobs, bh, m, n, k, tile):
    """f32 operands, f32 MFMA: the reference's own arithmetic type, against the scalar oracle at the f32 bar."""
    gemm_kernel_knobs(knobs, tile)
    t = env.torch
    a, b = rnd((bh, m, k), 1, "uniform"), rnd((bh, n, k), 2, "uniform")
    ad, bd = t.from_numpy(a).cuda(), t.from_numpy(b).cuda()
    cd = t.full((bh, m, n), float("nan"), device="cuda")
    env.nat.check(env.nat.core.i_hip_gemm_nt_f32(ad.data_ptr(), bd.data_ptr(), cd.data_ptr(), bh, m, n, k, env.stream()))
    t.cuda.synchronize()
    assert_close(cd.cpu().numpy(), oracle.mm_t(a, b), RTOL_F32)


def test_gemm_nt_f32_rejects_ragged_k(env):
    t = env.torch
    x = t.zeros(64, 42, device="cuda")
    c = t.zeros(64, 64, device="cuda")
    rc = env.nat.core.i_hip_gemm_nt_f32(x.data_ptr(), x.data_ptr(), c.data_ptr(), 1, 64, 64, 42, env.stream())
    assert rc == -1 and "multiple of 4" in env.nat.last_error()


def test_gemm_nt_bf16_full_size_linearity(env):
    """M=N=K=4096: C(A1+A2, B) == C(A1,B) + C(A2,B) for bf16-exact sums, and row block vs oracle."""
    t = env.torch
    n = 4096
    a = oracle.to_bf16_f32(rnd((n, n), 1, "uniform"))
    b = oracle.to_bf16_f32(rnd((n, n), 2, "uniform"))
    ad, bd = t.from_numpy(a).cuda().bfloat16(), t.from_numpy(b).cuda().bfloat16()
    cd = t.empty(n, n, device="cuda")
    env.nat.check(env.nat.core.i_hip_gemm_nt_bf16(ad.data_ptr(), bd.data_ptr(), cd.data_ptr(), 1, n, n, n, env.stream()))
    t.cuda.synchronize()
    rows = np.r_[0:8, n - 8:n]
    assert_close(cd[rows].cpu().numpy(), oracle.mm_t(a[rows], b), RTOL_BF16)
    a2 = (ad.float() * 2).bfloat16()  # exact in bf16
    c2 = t.empty(n, n, device="cuda")
    env.nat.check(env.nat.core.i_hip_gemm_nt_bf16(a2.data_ptr(), bd.data_ptr(), c2.data_ptr(), 1, n, n, n, env.stream()))
    t.cuda.synchronize()
    assert t.equal(c2, cd * 2)


# ------------------------------------------------------------------ row softmax
@pytest.mark.parametrize("rows,cols", [(16, 8), (1, 1), (33, 1000), (64, 4096), (7, 4099), (5, 8192), (3, 20000),
                                       (5, 8196), (4, 16384), (3, 16390), (3, 32768), (2, 40001), (3, 65536), (2, 65538),
                                       (2, 100000),
                                       # at most 128 columns: several rows per wavefront
                                       (1000, 16), (777, 4), (5, 3), (300, 2), (100, 30), (129, 100), (64, 128), (1, 128),
                                       (4097, 64), (70, 1), (33, 17),
                                       # beyond 65536 columns: two passes, float4 and element-wise
                                       (2, 100002), (3, 131072), (2, 262148), (1, 1048576), (1, 300001)])
def test_row_softmax_vs_oracle(env, rows, cols):
    t = env.torch
    x = rnd((rows, cols), 1) * 2
    xd = t.from_numpy(x).cuda()
    yd = t.full_like(xd, float("nan"))
    env.nat.check(env.nat.core.i_hip_row_softmax(xd.data_ptr(), yd.data_ptr(), rows, cols, env.stream()))
    t.cuda.synchronize()
    if cols <= 300000:
        assert_close(yd.cpu().numpy(), oracle.row_softmax(x), RTOL_F32)
    else:
        # the reference's nest adds a row's exponentials one after the other in f32; over a million terms that
        # sum is itself off by more than the bar (measured 1e-3), so the closed form in float64 is the referee
        x64 = x.astype(np.float64)
        e = np.exp(x64 - x64.max(axis=1, keepdims=True))
        assert_close(yd.cpu().numpy(), e / e.sum(axis=1, keepdims=True), RTOL_F32)
        assert relerr(oracle.row_softmax(x), e / e.sum(axis=1, keepdims=True)) < 1e-2  # (what the oracle gives)


@pytest.mark.parametrize("rows,cols", [(50, 16), (9, 128), (3, 70000)])
def test_row_softmax_operands_that_are_not_16_byte_aligned(env, rows, cols):
    """The float4 forms need 16-byte aligned rows; operands that start 4 bytes into an allocation take the
    element-wise forms of the same kernels."""
    t = env.torch
    x = rnd((rows, cols), 2)
    xbuf = t.zeros(rows * cols + 1, device="cuda")
    ybuf = t.full((rows * cols + 2,), float("nan"), device="cuda")
    xbuf[1:] = t.from_numpy(x).cuda().reshape(-1)
    env.nat.check(env.nat.core.i_hip_row_softmax(xbuf.data_ptr() + 4, ybuf.data_ptr() + 4, rows, cols, env.stream()))
    t.cuda.synchronize()
    assert bool(t.isnan(ybuf[0])) and bool(t.isnan(ybuf[-1]))  # nothing written outside
    assert_close(ybuf[1:-1].reshape(rows, cols).cpu().numpy(), oracle.row_softmax(x), RTOL_F32)


def test_row_softmax_wide_rows_stay_in_registers(env):
    """8192 < cols <= 65536: one workgroup per row with the row in registers (one read, one write per element);
    [2048, 32768] is the same 256 MiB as the benchmark's [16384, 4096]: rows sum to 1 and sampled rows match the
    oracle.  The three row operations of the naive schedule take the same kernels (checked through the frontend)."""
    t = env.torch
    rows, cols = 2048, 32768
    x = rnd((rows, cols), 1)
    xd = t.from_numpy(x).cuda()
    yd = t.full_like(xd, float("nan"))
    env.nat.check(env.nat.core.i_hip_row_softmax(xd.data_ptr(), yd.data_ptr(), rows, cols, env.stream()))
    t.cuda.synchronize()
    assert float((yd.sum(dim=1) - 1).abs().max()) < 1e-4
    pick = [0, 1, 1023, 2047]
    assert_close(yd[pick].cpu().numpy(), oracle.row_softmax(x[pick]), RTOL_F32)


def test_row_softmax_full_size_properties(env):
    """[16384, 4096] normal(0,1) seed 1: rows sum to 1, shift invariance, sampled rows vs oracle."""
    t = env.torch
    x = rnd((16384, 4096), 1)
    xd = t.from_numpy(x).cuda()
    yd = t.empty_like(xd)
    env.nat.check(env.nat.core.i_hip_row_softmax(xd.data_ptr(), yd.data_ptr(), 16384, 4096, env.stream()))
    t.cuda.synchronize()
    assert (yd.sum(dim=-1) - 1).abs().max().item() < 1e-4
    rows = np.r_[0:16, 16384 - 16:16384]
    assert_close(yd[rows].cpu().numpy(), oracle.row_softmax(x[rows]), RTOL_F32)
    y2 = t.empty_like(xd)
    x2 = xd + 3.0
    env.nat.check(env.nat.core.i_hip_row_softmax(x2.data_ptr(), y2.data_ptr(), 16384, 4096, env.stream()))
    t.cuda.synchronize()
    assert (y2 - yd).abs().max().item() <= 1e-4 * yd.abs().max().item()
