"""Schedule search scaffolding (i_amd/search.py): enumeration on the CPU, a small search on the GPU."""
import numpy as np
import pytest

import oracle
from i_amd import Component as i
from i_amd.search import Result, grid, option_grid, search


def test_grid_enumerates_split_strings():
    assert grid(i=[16, 32], j=[8]) == ["i:16,j:8", "i:32,j:8"]
    assert grid(i=["16:8"], j=[64, 128]) == ["i:16:8,j:64", "i:16:8,j:128"]
    assert grid() == [""]
    # every string is accepted by the parser as a split clause
    for split in grid(i=[16, "16:8"], j=[64]):
        primes = "i'i''" if "16:8" in split else "i'"
        comp = i(f"ik*jk~ijk | {split} | ji{primes}j'k") >> i(f"+ijk~ij | {split} | ji{primes}j'k0")
        assert "hand-written MFMA GEMM" in comp._code()


def test_option_grid_enumerates_program_options():
    assert option_grid({"gemm.k_parts": [1, 4], "gemm.waves": [4, 8]}) == [
        {"gemm.k_parts": 1, "gemm.waves": 4}, {"gemm.k_parts": 1, "gemm.waves": 8},
        {"gemm.k_parts": 4, "gemm.waves": 4}, {"gemm.k_parts": 4, "gemm.waves": 8}]
    assert option_grid({}) == [{}]
    # every name is one the compiled program knows; a wrong one or a wrong value is refused with its name
    comp = i("ik*jk~ijk | i:16,j:16 | jii'j'k") >> i("+ijk~ij | i:16,j:16 | jii'j'k0")
    for name, value in (("gemm.k_parts", 8), ("gemm.tile", 128), ("gemm.waves", 8), ("gemm.direct", 0), ("attention.kv_parts", 3),
                        ("attention.waves", 64), ("attention.direct", 0), ("attention.f32_scale", 1), ("generated.only", 1),
                        ("generated.wave", -1)):
        comp.option(name, value)
    for name, value, text in (("gemm.kparts", 2, "unknown program option"), ("gemm.tile", 64, "0, 128, 192 .192 x 256. or 256"),
                              ("attention.waves", 3, "attention.waves"), ("gemm.k_parts", -1, "gemm.k_parts")):
        with pytest.raises(RuntimeError, match=text):
            comp.option(name, value)


@pytest.mark.gpu
def test_search_over_the_parts_of_a_split_loop():
    """What a schedule has no spelling for is searched as program options: the number of parts the k loop of a product
    with few output tiles (64 x 8192 x 8192) is cut into, and the number of parts of the keys of one head of 8192,
    each ranked by device time with the C the reference backend emits as the referee (on a slice of the result)."""
    import torch

    from i_amd import I

    g = torch.Generator(device="cuda").manual_seed(3)
    a = (torch.rand(64, 8192, device="cuda", generator=g) * 2 - 1).bfloat16()
    b = (torch.rand(8192, 8192, device="cuda", generator=g) * 2 - 1).bfloat16()

    def mm_t(split):
        return i(f"ik*jk~ijk | {split} | jii'j'k") >> i(f"+ijk~ij | {split} | jii'j'k0")

    cols = slice(4000, 4032)

    def referee(a_, b_):
        comp = mm_t("i:16,j:16")
        out = oracle.compile_component(comp.handle).run(a_.float().cpu().numpy(), np.ascontiguousarray(b_[cols].float().cpu().numpy()))
        return torch.from_numpy(out).cuda()

    ranked = search(mm_t, ["i:16,j:16"], inputs=(a, b), rtol=1e-2, referee=referee, repeats=7, view=lambda c: c[:, cols],
                    options=option_grid({"gemm.k_parts": [1, 2, 4, 8, 16, 32]}))
    assert all(r.failure is None for r in ranked), [(r.options, r.failure, r.error) for r in ranked]
    assert len({r.options["gemm.k_parts"] for r in ranked}) >= 4 and ranked == sorted(ranked, key=lambda r: r.ms)
    by = {r.options["gemm.k_parts"]: r for r in ranked}
    assert "parts)" not in by[1].kernels and "(k in 8 parts)" in by[8].kernels
    assert ranked[0].options["gemm.k_parts"] > 1 and ranked[0].ms < by[1].ms  # 32 output tiles for 256 CUs: some split wins
    # the launcher's own choice (no option set) is within 25 % of the best of the search
    own = search(mm_t, ["i:16,j:16"], inputs=(a, b), rtol=1e-2, referee=referee, repeats=7, view=lambda c: c[:, cols])[0]
    assert own.ms <= 1.25 * ranked[0].ms, (own.ms, own.kernels, ranked[0].ms, ranked[0].options)

    q, k, v = (torch.randn(1, 8192, 128, device="cuda", generator=g).bfloat16() for _ in range(3))
    scale = torch.tensor(np.float32(128 ** -0.5), device="cuda")

    def attn(split):
        p = "b"
        first = i(f"{p}ik*{p}jk~{p}ijk | {split} | {p}jii'j'k") >> i(f"+{p}ijk~{p}ij | {split} | {p}jii'j'k0")
        sc = i(f"{p}ij*.~{p}ij | {split} | {p}ji0i'j'")
        shift = (I & i(f">{p}ij~{p}i | {split} | {p}ji0i'j'")) >> i(f"{p}ij-{p}i~{p}ij | {split} | {p}ji01i'j'")
        ex = i(f"^{p}ij~{p}ij | {split} | {p}ji0i'j'")
        norm = (I & i(f"+{p}ij~{p}i | {split} | {p}ji0i'j'")) >> i(f"{p}ij/{p}i~{p}ij | {split} | {p}ji01i'j'")
        last = i(f"{p}ij*{p}jk~{p}ikj | {split} | {p}ji0i'kj'") >> i(f"+{p}ikj~{p}ik | {split} | {p}jii'kj'0")
        return first >> sc >> shift >> ex >> norm >> last

    rows = slice(5000, 5032)

    def attn_referee(q_, k_, s_, v_):
        comp = attn("i:16,j:16")
        out = oracle.compile_component(comp.handle).run(np.ascontiguousarray(q_[:, rows].float().cpu().numpy()), k_.float().cpu().numpy(),
                                                        np.float32(s_.item()), v_.float().cpu().numpy())
        return torch.from_numpy(out).cuda()

    ranked = search(attn, ["i:128,j:64"], inputs=(q, k, scale, v), rtol=2e-2, referee=attn_referee, repeats=7,
                    view=lambda o: o[:, rows], options=option_grid({"attention.kv_parts": [1, 2, 4, 8, 16]}))
    assert all(r.failure is None for r in ranked), [(r.options, r.failure, r.error) for r in ranked]
    assert len({r.options["attention.kv_parts"] for r in ranked}) >= 4 and ranked == sorted(ranked, key=lambda r: r.ms)
    by = {r.options["attention.kv_parts"]: r for r in ranked}
    assert "keys in" not in by[1].kernels and "(keys in 4 parts)" in by[4].kernels
    assert ranked[0].options["attention.kv_parts"] > 1 and ranked[0].ms < by[1].ms  # 64 query tiles for 256 CUs


@pytest.mark.gpu
def test_search_ranks_schedules_and_flags_failures():
    import torch

    a = torch.from_numpy(oracle.to_bf16_f32(np.random.default_rng(1).uniform(-1, 1, (1024, 512)).astype(np.float32)))
    b = torch.from_numpy(oracle.to_bf16_f32(np.random.default_rng(2).uniform(-1, 1, (768, 512)).astype(np.float32)))
    a, b = a.cuda().bfloat16(), b.cuda().bfloat16()

    def mm_t(split):
        if split == "i:7,j:7":
            return i("ik*jk~ijk | i:7 | jii'k")  # a rank-3 product, not the matmul: must be flagged
        return i(f"ik*jk~ijk | {split} | jii'j'k") >> i(f"+ijk~ij | {split} | jii'j'k0")

    ranked = search(mm_t, grid(i=[128, 256, 7], j=[128, 256, 7])[::4] + ["i:,j:1"], inputs=(a, b), rtol=2e-2,
                    referee=lambda x, y: x.float() @ y.float().T, repeats=5)
    by_name = {r.schedule: r for r in ranked}
    assert set(by_name) == {"i:128,j:128", "i:256,j:256", "i:7,j:7", "i:,j:1"}
    good = [r for r in ranked if r.failure is None]
    assert [r.schedule for r in ranked[:len(good)]] == [r.schedule for r in good]  # survivors first
    assert {r.schedule for r in good} == {"i:128,j:128", "i:256,j:256"}
    assert all(isinstance(r, Result) and r.ms > 0 and r.error < 2e-2 and "MFMA GEMM" in r.plan for r in good)
    assert good == sorted(good, key=lambda r: r.ms)
    assert by_name["i:7,j:7"].failure.startswith("mismatch")
    assert by_name["i:,j:1"].failure and by_name["i:,j:1"].ms is None  # rejected by the compiler

    # without a referee the first candidate that runs is the reference
    again = search(mm_t, ["i:128,j:128", "i:256,j:256"], inputs=(a, b), rtol=2e-2, repeats=3)
    assert all(r.failure is None for r in again)


@pytest.mark.gpu
def test_search_over_attention_tiles_with_the_emitted_c_as_referee():
    """B8 H32 N4096 d128 (the benchmark's shape): every (query tile, key tile) kernel is a point of the search, the
    referee is the C the reference backend would emit for the component, run on the host for 64 query rows of one
    (b, h) slice."""
    import torch

    from i_amd import I

    B, H, N, D = 8, 32, 4096, 128
    g = torch.Generator(device="cuda").manual_seed(7)
    q, k, v = (torch.randn(B, H, N, D, device="cuda", generator=g).bfloat16() for _ in range(3))
    scale = torch.tensor(np.float32(1.0 / np.sqrt(D)), device="cuda")

    def attn(split):
        p = "bh"
        mm_t = i(f"{p}ik*{p}jk~{p}ijk | {split} | {p}jii'j'k") >> i(f"+{p}ijk~{p}ij | {split} | {p}jii'j'k0")
        sc = i(f"{p}ij*.~{p}ij | {split} | {p}ji0i'j'")
        shift = (I & i(f">{p}ij~{p}i | {split} | {p}ji0i'j'")) >> i(f"{p}ij-{p}i~{p}ij | {split} | {p}ji01i'j'")
        ex = i(f"^{p}ij~{p}ij | {split} | {p}ji0i'j'")
        norm = (I & i(f"+{p}ij~{p}i | {split} | {p}ji0i'j'")) >> i(f"{p}ij/{p}i~{p}ij | {split} | {p}ji01i'j'")
        mm = i(f"{p}ij*{p}jk~{p}ikj | {split} | {p}ji0i'kj'") >> i(f"+{p}ikj~{p}ik | {split} | {p}jii'kj'0")
        return mm_t >> sc >> shift >> ex >> norm >> mm

    b0, h0, rows = 5, 19, slice(4000, 4064)

    def referee(q_, k_, s_, v_):
        cpu = [t[b0:b0 + 1, h0:h0 + 1].float().cpu().numpy() for t in (q_, k_, v_)]
        demo_tiles = attn("i:16,j:16")  # owns the handle while the C is emitted; the emitted nest is shape-generic
        prog = oracle.compile_component(demo_tiles.handle)
        out = prog.run(np.ascontiguousarray(cpu[0][:, :, rows]), cpu[1], np.float32(s_.item()), cpu[2])
        return torch.from_numpy(out).cuda()

    ranked = search(attn, grid(i=[64, 128, 256], j=[32, 64]) + ["i:16,j:16"], inputs=(q, k, scale, v), rtol=2e-2,
                    referee=referee, repeats=5, view=lambda o: o[b0:b0 + 1, h0:h0 + 1, rows])
    assert all(r.failure is None for r in ranked), [(r.schedule, r.failure, r.error) for r in ranked]
    names = {r.kernels.split()[1] for r in ranked}
    assert len(names) >= 6, names
    assert ranked == sorted(ranked, key=lambda r: r.ms)
    by = {r.schedule: r for r in ranked}
    assert "the schedule asks for 16 x 16" in by["i:16,j:16"].kernels
    assert by["i:256,j:64"].ms < by["i:64,j:32"].ms  # one workgroup per CU with 64-key tiles beats 64-query workgroups
