"""Schedule search scaffolding (i_amd/search.py): enumeration on the CPU, a small search on the GPU."""
import numpy as np
import pytest

import oracle
from i_amd import Component as i
from i_amd.search import Result, grid, search


def test_grid_enumerates_split_strings():
    assert grid(i=[16, 32], j=[8]) == ["i:16,j:8", "i:32,j:8"]
    assert grid(i=["16:8"], j=[64, 128]) == ["i:16:8,j:64", "i:16:8,j:128"]
    assert grid() == [""]
    # every string is accepted by the parser as a split clause
    for split in grid(i=[16, "16:8"], j=[64]):
        primes = "i'i''" if "16:8" in split else "i'"
        comp = i(f"ik*jk~ijk | {split} | ji{primes}j'k") >> i(f"+ijk~ij | {split} | ji{primes}j'k0")
        assert "hand-written MFMA GEMM" in comp._code()


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
