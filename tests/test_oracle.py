"""Pins the CPU oracle (oracle/oracle.c) before anything is compared against it.

Checks, chosen so a plausible slip (dropped correction, wrong sign, transposed
operand, wrong tail guard) fails at least one:
  * bit-exact agreement with golden outputs of the reference's own emitted C
    (tests/golden/flashattn_ref.npz, made by tests/golden/make_golden.py),
    and live against oracle/_ref when that library is present;
  * fp64 closed forms (flash-attn.py:38-43 spelled in float64);
  * invariants: softmax rows sum to 1, attention output inside the convex hull
    of V, key-permutation invariance, tile-size invariance, tiled == naive;
  * brute force on tiny inputs with Python loops.
"""
import numpy as np
import pytest

import oracle

CASES = ["u_48x24", "u_64x64", "u_100x40", "n_48x24", "n_33x17", "n_16x130"]


def rnd(shape, seed, kind="normal"):
    rng = np.random.default_rng(seed)
    if kind == "uniform":
        return rng.uniform(-1, 1, shape).astype(np.float32)
    return rng.standard_normal(shape, dtype=np.float32)


@pytest.mark.parametrize("case", CASES)
def test_attention_tiled_bit_exact_vs_reference_golden(golden, case):
    q, k, v, o = (golden[f"{case}.{x}"] for x in "qkvo")
    got = oracle.attention_tiled(q, k, v)  # 16x16 tiles, no scale: the demo component
    assert got.dtype == np.float32 and got.shape == o.shape
    assert np.array_equal(got, o)


@pytest.mark.skipif(not oracle.have_ref(), reason="compiled reference emission not present")
@pytest.mark.parametrize("n,d,kind", [(512, 64, "uniform"), (500, 60, "uniform"), (32, 2048, "normal")])
def test_attention_tiled_bit_exact_vs_live_reference(n, d, kind):
    q, k, v = (rnd((n, d), s, kind) for s in (1, 2, 3))
    assert np.array_equal(oracle.attention_tiled(q, k, v), oracle.ref_flash_attention(q, k, v))


@pytest.mark.parametrize("case", CASES)
def test_golden_matches_fp64_closed_form(golden, case):
    q, k, v, o = (golden[f"{case}.{x}"] for x in "qkvo")
    ref = oracle.np_attention64(q, k, v)
    assert np.allclose(o, ref, rtol=3e-4, atol=5e-5)  # the reference's own bar, flash-attn.py:8


@pytest.mark.parametrize("bh,nq,nk,d,dv,scale,ti,tj", [
    (1, 40, 40, 8, 8, None, 16, 16),
    (3, 37, 53, 12, 20, 0.25, 16, 16),
    (2, 64, 96, 16, 16, 0.125, 32, 8),
    (1, 5, 3, 4, 6, 2.0, 4, 2),
])
def test_attention_tiled_vs_closed_form_and_naive(bh, nq, nk, d, dv, scale, ti, tj):
    q, k, v = rnd((bh, nq, d), 1), rnd((bh, nk, d), 2), rnd((bh, nk, dv), 3)
    ref = oracle.np_attention64(q, k, v, scale)
    tiled = oracle.attention_tiled(q, k, v, scale, ti, tj)
    naive = oracle.attention_naive(q, k, v, scale)
    assert tiled.shape == (bh, nq, dv)
    assert np.abs(tiled - ref).max() <= 1e-5 * max(1.0, np.abs(ref).max())
    assert np.abs(naive - ref).max() <= 1e-5 * max(1.0, np.abs(ref).max())


def test_attention_tile_size_invariance():
    q, k, v = rnd((70, 24), 1), rnd((90, 24), 2), rnd((90, 24), 3)
    a = oracle.attention_tiled(q, k, v, None, 16, 16)
    b = oracle.attention_tiled(q, k, v, None, 32, 8)
    c = oracle.attention_tiled(q, k, v, None, 7, 90)
    assert np.abs(a - b).max() <= 1e-5 and np.abs(a - c).max() <= 1e-5


def test_attention_key_permutation_invariance_and_convex_hull():
    q, k, v = rnd((33, 16), 1), rnd((50, 16), 2), rnd((50, 16), 3)
    perm = np.random.default_rng(7).permutation(50)
    a = oracle.attention_tiled(q, k, v)
    b = oracle.attention_tiled(q, k[perm], v[perm])
    assert np.abs(a - b).max() <= 1e-5
    assert (a <= v.max(axis=0) + 1e-6).all() and (a >= v.min(axis=0) - 1e-6).all()


def test_attention_online_rescale_stress_max_in_last_tile():
    # every key tile raises the running max, so every exp-shift correction fires
    nq, nk, d = 20, 80, 8
    q = np.ones((nq, d), np.float32)
    k = (np.arange(nk, dtype=np.float32)[:, None] * np.ones((1, d), np.float32)) * 0.5
    v = rnd((nk, d), 3)
    got = oracle.attention_tiled(q, k, v)
    assert np.allclose(got, oracle.np_attention64(q, k, v), rtol=1e-5, atol=1e-6)


def test_attention_brute_force_tiny():
    q, k, v = rnd((3, 2), 1), rnd((4, 2), 2), rnd((4, 3), 3)
    out = np.zeros((3, 3))
    for i in range(3):
        s = [sum(float(q[i, x]) * float(k[j, x]) for x in range(2)) for j in range(4)]
        m = max(s)
        w = [np.exp(t - m) for t in s]
        for c in range(3):
            out[i, c] = sum(w[j] * float(v[j, c]) for j in range(4)) / sum(w)
    assert np.allclose(oracle.attention_tiled(q, k, v, None, 2, 2), out, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("bh,m,n,k", [(1, 8, 7, 16), (2, 33, 17, 40), (1, 1, 1, 1)])
def test_mm_t_vs_closed_form(bh, m, n, k):
    a, b = rnd((bh, m, k), 1), rnd((bh, n, k), 2)
    got = oracle.mm_t(a, b)
    assert got.shape == (bh, m, n)
    assert np.allclose(got, oracle.np_mm_t64(a, b), rtol=1e-5, atol=1e-5)
    # transposed-operand slip would fail this: (A B^T)^T == B A^T
    assert np.allclose(oracle.mm_t(b, a), np.swapaxes(got, -1, -2), rtol=1e-6, atol=1e-6)


def test_mm_t_brute_force_order_is_k_ascending_f32():
    a, b = rnd((3, 5), 1), rnd((2, 5), 2)
    ref = np.zeros((3, 2), np.float32)
    for i in range(3):
        for j in range(2):
            acc = np.float32(0)
            for x in range(5):
                acc = np.float32(acc + np.float32(a[i, x] * b[j, x]))
            ref[i, j] = acc
    assert np.array_equal(oracle.mm_t(a, b), ref)


@pytest.mark.parametrize("rows,cols", [(16, 8), (5, 1), (33, 1000), (2, 4099)])
def test_row_softmax_vs_closed_form(rows, cols):
    x = rnd((rows, cols), 1) * 3
    y = oracle.row_softmax(x)
    assert np.allclose(y, oracle.np_softmax64(x), rtol=1e-5, atol=1e-7)
    assert np.allclose(y.sum(axis=-1), 1.0, atol=1e-5)
    assert np.allclose(oracle.row_softmax(x + 5.0), y, rtol=1e-4, atol=1e-7)  # shift invariance


def test_bf16_rounding_helper():
    x = np.array([1.0, 1.00390625, 1.005859375, -2.5, 3.1415927], np.float32)
    r = oracle.to_bf16_f32(x)
    assert r[0] == 1.0 and r[3] == -2.5
    assert r[1] == 1.0  # tie -> even mantissa
    assert r[2] == np.float32(1.0078125)
    assert (oracle.bf16_bits(r).astype(np.uint32) << 16).view(np.float32).tolist() == r.tolist()
