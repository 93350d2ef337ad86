"""Schedule search scaffolding: time the same computation under different schedules.

The reference's stated bet is that splits, loop orders and staging are a search
space over one fixed meaning (README.md:41-48).  This module enumerates
candidate schedules of a component, runs each on the GPU with the operands
resident in device memory, checks every candidate's outputs against a referee
and ranks the survivors by time.

The referee is any callable that returns the expected outputs for the given
inputs (torch tensors), or, when none is given, the first candidate: schedules
never change what is computed, so every candidate must agree with it.  The
tolerance is relative to the largest magnitude of the referee's output.
A referee that is slow (the C the reference backend emits, on one host core)
may cover only part of each output: `view` cuts that part out of a candidate's
outputs before the comparison.

    from i_amd import Component as i
    from i_amd.search import grid, search

    def mm_t(split):
        return i(f"ik*jk~ijk | {split} | jii'j'k") >> i(f"+ijk~ij | {split} | jii'j'k0")

    ranked = search(mm_t, grid(i=[128, 256], j=[128, 256]), inputs=(a, b), rtol=2e-2)
    best = ranked[0]          # Result(schedule='i:256,j:256', ms=..., error=..., plan='hand-written ...')

What a schedule has no spelling for, but what matters on this chip (into how many parts the k loop of a product or
the keys of a head are cut over workgroups, how many waves a workgroup has), is a second axis of the search: program
options (``Component.option``, ``i_hip_program_option``), every candidate schedule under every combination of them.

    ranked = search(mm_t, ["i:16,j:16"], inputs=(a, b), rtol=2e-2, options=option_grid({"gemm.k_parts": [1, 2, 4, 8, 16]}))
    best.options              # {'gemm.k_parts': 8}
"""
import itertools
from dataclasses import dataclass, field
from typing import Callable, Dict, Iterable, List, Optional, Sequence


@dataclass
class Result:
    schedule: str            # the split string handed to the builder
    ms: Optional[float]      # median device time of one run, None when the candidate failed
    error: Optional[float]   # max |out - referee| / max |referee| over all outputs
    plan: str                # first line of the backend plan for kernel f0 (which kernel form runs)
    failure: Optional[str] = None  # compile / run error text, or "mismatch"
    kernels: str = ""        # what the run dispatched (Component.report()): kernel names and their tiles
    options: Dict[str, int] = field(default_factory=dict)  # the program options the candidate ran under


def grid(**factors: Sequence) -> List[str]:
    """All combinations of split factors, as split strings: grid(i=[16, 32], j=[8]) -> ['i:16,j:8', 'i:32,j:8'].
    A factor may itself be a multi-level split written as a string, e.g. i=['16', '16:8']."""
    names = list(factors)
    out = []
    for combo in itertools.product(*(factors[n] for n in names)):
        out.append(",".join(f"{n}:{f}" for n, f in zip(names, combo)))
    return out


def option_grid(values: Dict[str, Sequence[int]]) -> List[Dict[str, int]]:
    """All combinations of program option values: option_grid({"gemm.k_parts": [1, 4], "gemm.waves": [4, 8]}) ->
    [{'gemm.k_parts': 1, 'gemm.waves': 4}, {'gemm.k_parts': 1, 'gemm.waves': 8}, ...]."""
    names = list(values)
    return [dict(zip(names, combo)) for combo in itertools.product(*(values[n] for n in names))]


def _plan_line(component) -> str:
    try:
        for line in component._code().splitlines():
            if line.startswith("// f0:"):
                return line[len("// f0:"):].strip()
    except RuntimeError as e:  # the plan is informative only
        return f"(no plan: {e})"
    return ""


def _time_ms(torch, fn, repeats: int, warmup: int) -> float:
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    times = []
    for _ in range(repeats):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        b.synchronize()
        times.append(a.elapsed_time(b))
    times.sort()
    return times[len(times) // 2]


def search(build: Callable[[str], object], schedules: Iterable[str], inputs: Sequence, rtol: float,
           referee: Optional[Callable[..., Sequence]] = None, repeats: int = 10, warmup: int = 2,
           out_dtype=None, view: Optional[Callable] = None, options: Optional[Iterable[Dict[str, int]]] = None) -> List[Result]:
    """Run build(schedule) for every schedule on `inputs` (ROCm torch tensors), under every set of program options
    in `options` when given (each a dict of option name -> value, see option_grid).

    Returns one Result per candidate, fastest first; candidates that fail to compile, fail to run or
    disagree with the referee by more than `rtol` come last with `failure` set.
    """
    import torch

    expected = None
    if referee is not None:
        expected = referee(*inputs)
        if torch.is_tensor(expected):
            expected = [expected]
        expected = [e.float() for e in expected]

    results = []
    for schedule, opts in itertools.product(list(schedules), [dict(o) for o in options] if options is not None else [{}]):
        try:
            comp = build(schedule)
            for name, value in opts.items():
                comp.option(name, value)
            got = comp.exec_torch(*inputs, out_dtype=out_dtype)
            got = [got] if torch.is_tensor(got) else list(got)
            full = got
            got = [(view(g) if view else g).float() for g in got]
            kernels = comp.report().strip()
        except RuntimeError as e:
            results.append(Result(schedule, None, None, "", failure=str(e), options=opts))
            continue
        plan = _plan_line(comp)
        if expected is None:
            expected = got  # first candidate that runs is the referee
        if len(got) != len(expected) or any(g.shape != e.shape for g, e in zip(got, expected)):
            results.append(Result(schedule, None, None, plan, failure="mismatch (output count or shape)", options=opts))
            continue
        err = 0.0
        for g, e in zip(got, expected):
            if e.numel():
                scale = float(e.abs().max()) or 1.0
                err = max(err, float((g - e).abs().max()) / scale)
        if not err <= rtol:  # also catches NaN
            results.append(Result(schedule, None, err, plan, failure="mismatch", kernels=kernels, options=opts))
            continue
        outs = [torch.empty_like(g, dtype=out_dtype or torch.float32) for g in full]
        target = outs[0] if len(outs) == 1 else outs
        ms = _time_ms(torch, lambda: comp.into(target, *inputs), repeats, warmup)
        results.append(Result(schedule, ms, err, plan, kernels=kernels, options=opts))
    results.sort(key=lambda r: (r.failure is not None, r.ms if r.ms is not None else float("inf")))
    return results
