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
