"""i_exec_into_device_noalloc (the entry point that allocates no device memory) against i_exec_into_device, through
the C ABI, on programs whose temporaries are real: the two [rows, cols] intermediates of the naive three-kernel
softmax, the f32 staging of bf16 operands and outputs, the transposed right operand of a ragged f32 product, and
the [i, j, k] intermediate of an unfused product run on generated kernels.  Both entries launch the same kernels,
so the results are compared bit for bit; each case runs twice in a row, the second time on a smaller input, because
every call reuses the same fixed array and finds the previous call's contents in it."""
import ctypes

import numpy as np
import pytest

from i_amd import Component as i, I
from i_amd import _native as nat
from i_amd import ilang

pytestmark = pytest.mark.gpu
LIMIT = 64 << 20  # I_HIP_STATIC_WORKSPACE_BYTES


@pytest.fixture(scope="module")
def torch():
    import torch

    assert torch.cuda.is_available()
    return torch


def softmax_naive(s="i:16,j:16"):
    return (((I & i(f">ij~i|{s}|jii'j'")) >> i(f"ij-i~ij|{s}|1jii'j'")) >> i(f"^ij~ij|{s}|jii'j'")
            >> ((I & i(f"+ij~i|{s}|jii'j'")) >> i(f"ij/i~ij|{s}|1jii'j'")))


def call(entry, comp, inputs, outputs, torch):
    """One call of a device entry point of the C ABI on torch tensors, on the current stream."""
    in_records, keep_in = ilang._pack([ilang._operand(x, "input") for x in inputs], on_device=True)
    out_records, keep_out = ilang._pack([ilang._operand(x, "output") for x in outputs], on_device=True)
    stream = torch.cuda.current_stream().cuda_stream
    rc = entry(comp._compile(), in_records, len(inputs), out_records, len(outputs), stream)
    torch.cuda.synchronize()
    return rc


def both(comp, inputs, torch, out_dtype=None):
    shapes = comp.output_shapes(*inputs)
    outs_a = [torch.full(s, float("nan"), dtype=out_dtype or torch.float32, device="cuda") for s in shapes]
    outs_b = [torch.full(s, float("nan"), dtype=out_dtype or torch.float32, device="cuda") for s in shapes]
    assert call(nat.core.i_exec_into_device, comp, inputs, outs_a, torch) == 0, nat.last_error()
    assert call(nat.core.i_exec_into_device_noalloc, comp, inputs, outs_b, torch) == 0, nat.last_error()
    for a, b in zip(outs_a, outs_b):
        assert torch.isfinite(a.float()).all()
        assert torch.equal(a, b)
    return outs_b


def randn(torch, shape, seed, dtype=None):
    g = torch.Generator(device="cpu").manual_seed(seed)
    x = torch.randn(shape, generator=g, dtype=torch.float32)
    return x.cuda().to(dtype) if dtype else x.cuda()


def test_naive_softmax_twice_second_smaller(torch):
    comp = softmax_naive()
    for shape in ((1024, 2000), (100, 37)):  # 2 x 7.8 MiB of intermediates, then a smaller problem in the same array
        print("case naive softmax", shape, flush=True)
        (y,) = both(comp, [randn(torch, shape, 1)], torch)
        ref = torch.softmax(randn(torch, shape, 1).double(), dim=-1)
        assert float((y.double() - ref).abs().max() / ref.abs().max()) <= 1e-4


def test_bf16_operands_and_outputs_are_staged_in_the_workspace(torch):
    comp = softmax_naive()
    for shape in ((512, 768), (33, 40)):
        print("case bf16 staging", shape, flush=True)
        both(comp, [randn(torch, shape, 2, torch.bfloat16)], torch, out_dtype=torch.bfloat16)


def test_transposed_operand_and_generated_kernels(torch):
    plain = i("ik*kj~ijk|i:16,j:16|jii'j'k") >> i("+ijk~ij|i:16,j:16|jii'j'k0")  # f32, ragged: transpose + NT kernel
    unfused = i("ik*kj~ijk") >> i("+ijk~ij")                                        # two generated kernels, [i,j,k] between
    for m, k, n in ((300, 96, 77), (40, 32, 9)):
        print("case products", (m, k, n), flush=True)
        a, b = randn(torch, (m, k), 3), randn(torch, (k, n), 4)
        (c,) = both(plain, [a, b], torch)
        ref = a.double() @ b.double()
        assert float((c.double() - ref).abs().max() / ref.abs().max()) <= 1e-4
        (c2,) = both(unfused, [a, b], torch)
        assert float((c2.double() - ref).abs().max() / ref.abs().max()) <= 1e-4


def test_split_loops_keep_their_partial_results_in_the_workspace(torch, monkeypatch):
    """A product whose k loop and an attention whose key loop are split over workgroups: the parts' results are
    temporaries like any other (up to 20 MiB of the fixed array; above that the unsplit kernel runs)."""
    mm_t = i("ik*jk~ijk | i:16,j:16 | jii'j'k") >> i("+ijk~ij | i:16,j:16 | jii'j'k0")
    for m, n, k in ((64, 1000, 8192), (40, 300, 4104)):
        print("case split product", (m, n, k), flush=True)
        both(mm_t, [randn(torch, (m, k), 7, torch.bfloat16), randn(torch, (n, k), 8, torch.bfloat16)], torch)
        assert "parts)" in mm_t.report(), mm_t.report()
    s = "i:16,j:16"
    attention = ((i(f"ik*jk~ijk | {s} | jii'j'k") >> i(f"+ijk~ij | {s} | jii'j'k0"))
                 >> ((I & i(f">ij~i | {s} | ji0i'j'")) >> i(f"ij-i~ij | {s} | ji01i'j'")) >> i(f"^ij~ij | {s} | ji0i'j'")
                 >> ((I & i(f"+ij~i | {s} | ji0i'j'")) >> i(f"ij/i~ij | {s} | ji01i'j'"))
                 >> (i(f"ij*jk~ikj | {s} | ji0i'kj'") >> i(f"+ikj~ik | {s} | jii'kj'0")))
    attention.option("attention.kv_parts", 3)
    for nq, nk, d in ((300, 2500, 128), (70, 1000, 64)):
        print("case split attention", (nq, nk, d), flush=True)
        q, k, v = (randn(torch, shape, seed, torch.bfloat16) for seed, shape in ((9, (nq, d)), (10, (nk, d)), (11, (nk, d))))
        both(attention, [q * d ** -0.25, k * d ** -0.25, v], torch)
        assert "(keys in 3 parts)" in attention.report(), attention.report()


def test_temporaries_that_a_launch_can_do_without_are_left_out_when_the_rest_only_fits_without_them(torch):
    """An f32 product whose contracted extent is no multiple of 4: both operands are copied into temporaries with
    padded rows (61.4 MiB here, which the kernels cannot run without), and its k loop would be split over workgroups
    (partial products of a few MiB more, which they can).  Together that exceeds the fixed array; the call then
    runs the loop whole instead of being refused, and a smaller problem afterwards splits again."""
    mm_t = i("ik*jk~ijk | i:16,j:16 | jii'j'k") >> i("+ijk~ij | i:16,j:16 | jii'j'k0")
    for m, n, k, splits in ((64, 1900, 8190, False), (64, 300, 4102, True)):
        print("case optional temporaries", (m, n, k), flush=True)
        a, b = randn(torch, (m, k), 5), randn(torch, (n, k), 6)
        out = torch.full((m, n), float("nan"), device="cuda")
        assert call(nat.core.i_exec_into_device_noalloc, mm_t, [a, b], [out], torch) == 0, nat.last_error()
        assert ("parts)" in mm_t.report()) == splits, mm_t.report()
        ref = a.double() @ b.double().T
        assert float((out.double() - ref).abs().max() / ref.abs().max()) <= 1e-4
        whole = torch.full((m, n), float("nan"), device="cuda")
        assert call(nat.core.i_exec_into_device, mm_t, [a, b], [whole], torch) == 0, nat.last_error()
        assert "parts)" in mm_t.report(), mm_t.report()
        assert float((out - whole).abs().max()) <= 1e-4 * float(ref.abs().max())


def test_cached_memory_can_be_released_and_comes_back(torch):
    """i_hip_release_cached_memory frees the blocks the library keeps from call to call (per-stream temporaries, the
    device copies and page-locked chunks of host operands, its pool of freed temporaries); the calls after it
    allocate again and give the same results."""
    comp = softmax_naive()
    x = randn(torch, (512, 1000), 7)
    first = comp.exec_torch(x)
    host = comp.exec_numpy(x.cpu().numpy())  # the host entry: a kept device block for the operands' copies
    big = np.ones((2100, 1024), np.float32)  # 8.2 MiB: through the page-locked chunks
    assert np.array_equal(i("ij+ij~ij").exec_numpy(big, big), big + big)
    torch.cuda.synchronize()
    released = nat.core.i_hip_release_cached_memory()
    assert released >= (2 * 512 * 1000 * 4) + (4 << 23), released  # the softmax intermediates' block and the four 8 MiB chunks at least
    assert nat.core.i_hip_release_cached_memory() == 0  # nothing left to give back
    assert torch.equal(comp.exec_torch(x), first)
    assert np.array_equal(comp.exec_numpy(x.cpu().numpy()), host)
    assert np.array_equal(i("ij+ij~ij").exec_numpy(big, big), big + big)


def test_both_device_entry_points_under_graph_capture(torch):
    """What the entry point that allocates nothing is for: captured into a HIP graph (after one eager call, which
    loads the code object and compiles the generated kernels) and replayed three times, with new input values,
    eager work and a synchronisation between the replays, every replay checked.  The allocating entry point is
    captured too: under capture its temporaries are plain stream-ordered allocations, which the graph records."""
    sm = softmax_naive()
    s = "i:16,j:16"
    attention = ((i(f"bik*bjk~bijk | {s} | bjii'j'k") >> i(f"+bijk~bij | {s} | bjii'j'k0"))
                 >> ((I & i(f">bij~bi | {s} | bji0i'j'")) >> i(f"bij-bi~bij | {s} | bji01i'j'")) >> i(f"^bij~bij | {s} | bji0i'j'")
                 >> ((I & i(f"+bij~bi | {s} | bji0i'j'")) >> i(f"bij/bi~bij | {s} | bji01i'j'"))
                 >> (i(f"bij*bjk~bikj | {s} | bji0i'kj'") >> i(f"+bikj~bik | {s} | bjii'kj'0")))
    x, y = randn(torch, (512, 777), 12), torch.empty(512, 777, device="cuda")
    q, k, v = (randn(torch, (2, 300, 128), seed, torch.bfloat16) * 0.3 for seed in (13, 14, 15))
    o = torch.empty(2, 300, 128, device="cuda")
    for static in (True, False):
        print("case graph capture, static workspace", static, flush=True)
        sm.into(y, x, static_workspace=static)
        attention.into(o, q, k, v, static_workspace=static)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            sm.into(y, x, static_workspace=static)
            attention.into(o, q, k, v, static_workspace=static)
        for rep in range(3):
            x.copy_(randn(torch, (512, 777), 20 + rep))
            q.copy_(randn(torch, (2, 300, 128), 30 + rep, torch.bfloat16) * 0.3)
            y.fill_(float("nan"))
            o.fill_(float("nan"))
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert float((y.double() - torch.softmax(x.double(), -1)).abs().max()) <= 1e-6
            ref = torch.softmax(q.double() @ k.double().transpose(1, 2), -1) @ v.double()
            assert float((o.double() - ref).abs().max()) <= 2e-2 * float(ref.abs().max())


def test_operands_beyond_the_workspace_are_refused_before_anything_runs(torch):
    comp = softmax_naive()
    x = randn(torch, (8192, 4096), 5)  # two 128 MiB intermediates
    y = torch.full((8192, 4096), 7.0, device="cuda")
    print("case refusal", flush=True)
    assert call(nat.core.i_exec_into_device_noalloc, comp, [x], [y], torch) == -1
    message = nat.last_error()
    assert str(2 * 8192 * 4096 * 4) in message and str(LIMIT) in message
    assert bool((y == 7.0).all())  # nothing was enqueued
    # and the entry point still works afterwards
    both(comp, [randn(torch, (64, 64), 6)], torch)
