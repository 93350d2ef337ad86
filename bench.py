#!/usr/bin/env python3
"""Benchmark of the north-star path on one MI355X.

One step = one forward pass of the 𝚒 FlashAttention component
(mm_t >> scale >> row_max_shift >> exp >> row_normalize >> mm), compiled from
its expression strings through i_parse/i_compile and run with
i_exec_into_device on operands resident in HBM: B=8, H=32, N=4096, d=128,
bf16 inputs, f32 accumulation, f32 output, scores scaled by 1/sqrt(d).

Prints ONE JSON line.  Besides the headline TFLOP/s it carries
  roofline      achieved vs MI355X dense bf16 MFMA peak for the attention kernel,
                from HIP events recorded on the launch stream
  cpu_baseline  the C the reference backend emits for the benchmark's own
                component strings, compiled with the reference's command
                (cc -O3 -shared -fPIC -lm) and timed on one host core on a
                bounded sample, with the GPU result checked against it
  secondary     row-softmax [16384,4096] f32 (HBM bound), mm_t 4096^3 bf16, the
                long-sequence attention B1 H16 N32768 d64 (inputs x 2.0) and the
                reference's own demo (attention f32 [512,64]) and the attention workload
                in the reference's own arithmetic type (f32 operands, two of the eight
                batches), each with its own roofline, cpu_baseline and rel_err

Operands follow the recipe of the reference's scripts (NumPy default_rng(seed),
seeds 1, 2, 3 for the first, second, third operand; ilang-python/flash-attn.py:33-35).

roofline.shader_clock_ghz is measured inside the timed region: the attention kernels count, per workgroup, the
cycles of the shader clock (the frequency the power manager grants) and the ticks of the constant 100 MHz clock
that pass while they are resident (i_hip_program_clock_probe); for kernels that cannot count for themselves
(the vendor library's GEMM, mm_t) a one-wavefront kernel on a second stream reads the same two clocks while a
second batch of launches runs (i_hip_shader_clock_probe; its own line, not the timed one, because the wavefront
keeps one compute unit from taking a workgroup that needs all of it).  frac_at_measured_clock is the roofline
fraction with the peak scaled to that clock (peak * clock / 2.4 GHz): the share of the matrix cores' cycles the
kernel fills.

roofline.traffic is the HBM traffic per launch measured with rocprofv3
(FETCH_SIZE + WRITE_SIZE passes, scaled by a plain copy of known size); it is read
from the committed summary under profiles/ and is null when that is missing.
"""
import argparse
import json
import re
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E
PEAK_F32_TFLOPS = 157.3    # MI355X dense f32 MFMA
# launches of the headline kernel before the W warm-up steps: the compile-and-first-run call plus 40 more.  The
# launch time of a fresh process keeps falling over its first two dozen launches (2.2 ms -> 1.8 ms while the
# clocks settle); this brings the device to that steady state whatever W is.
PRE_WARMUP_LAUNCHES = 41


def flash_component(i, I, split):
    mm_t = i(f"bhik*bhjk~bhijk | {split} | bhjii'j'k") >> i(f"+bhijk~bhij | {split} | bhjii'j'k0")
    scale = i(f"bhij*.~bhij | {split} | bhji0i'j'")
    row_max_shift = (I & i(f">bhij~bhi | {split} | bhji0i'j'")) >> i(f"bhij-bhi~bhij | {split} | bhji01i'j'")
    exp = i(f"^bhij~bhij | {split} | bhji0i'j'")
    row_normalize = (I & i(f"+bhij~bhi | {split} | bhji0i'j'")) >> i(f"bhij/bhi~bhij | {split} | bhji01i'j'")
    mm = i(f"bhij*bhjk~bhikj | {split} | bhji0i'kj'") >> i(f"+bhikj~bhik | {split} | bhjii'kj'0")
    return mm_t >> scale >> row_max_shift >> exp >> row_normalize >> mm


def flash_demo_component(i, I):
    # the demo's strings (ilang-python/flash-attn.py:45-53): single head, no score scale
    s = "i:16,j:16"
    mm_t = i(f"ik*jk~ijk | {s} | jii'j'k") >> i(f"+ijk~ij | {s} | jii'j'k0")
    row_max_shift = (I & i(f">ij~i | {s} | ji0i'j'")) >> i(f"ij-i~ij | {s} | ji01i'j'")
    exp = i(f"^ij~ij | {s} | ji0i'j'")
    row_normalize = (I & i(f"+ij~i | {s} | ji0i'j'")) >> i(f"ij/i~ij | {s} | ji01i'j'")
    mm = i(f"ij*jk~ikj | {s} | ji0i'kj'") >> i(f"+ikj~ik | {s} | jii'kj'0")
    return mm_t >> row_max_shift >> exp >> row_normalize >> mm


def softmax_component(i, I):
    # row-staged single-kernel schedule: max and sum fold to scalars, the row stays on chip
    return (((I & i(">ij~i|i:16|ii'j")) >> i("ij-i~ij|i:16|ii'1j")) >> i("^ij~ij|i:16|ii'0j")
            >> ((I & i("+ij~i|i:16|ii'0j")) >> i("ij/i~ij|i:16|ii'01j")))


def mm_t_component(i):
    return i("ik*jk~ijk | i:256,j:256 | jii'j'k") >> i("+ijk~ij | i:256,j:256 | jii'j'k0")


def measured_traffic(summary):
    """HBM bytes per launch from a committed rocprofv3 summary, or None."""
    try:
        text = (ROOT / "profiles" / summary).read_text()
    except OSError:
        return None
    m = re.search(r"Scaled traffic per launch: (\d+) MiB fetched \+ (\d+) MiB written", text)
    return (int(m.group(1)) + int(m.group(2))) * 2 ** 20 if m else None


def profile_cycles(kernel):
    """Shader cycles per launch of `kernel` from the committed SQ-counter summary (GRBM_GUI_ACTIVE / 8), or None."""
    try:
        text = (ROOT / "profiles" / "sq_counters_bench_kernels.md").read_text()
    except OSError:
        return None
    header = next((l for l in text.splitlines() if l.startswith("| figure |")), None)
    row = next((l for l in text.splitlines() if l.startswith("| cycles per launch")), None)
    if not header or not row:
        return None
    names = [c.strip() for c in header.strip("|").split("|")]
    cells = [c.strip() for c in row.strip("|").split("|")]
    return int(cells[names.index(kernel)]) if kernel in names else None


NOMINAL_GHZ = 2.4  # the shader clock the published matrix-core peaks are quoted at


def clock_fields(ghz, frac, kernel, kernel_ms):
    """The roofline fields that make a power-limited reading checkable: the measured shader clock, the fraction of
    the peak at that clock, and the kernel time that the committed profile's cycle count predicts at that clock."""
    if not ghz:
        return {"shader_clock_ghz": None, "frac_at_measured_clock": None}
    out = {"shader_clock_ghz": ghz, "frac_at_measured_clock": frac * NOMINAL_GHZ / ghz,
           "cycles_per_launch": kernel_ms * 1e-3 * ghz * 1e9}
    cycles = profile_cycles(kernel)
    if cycles:
        out["cycles_per_launch_profile"] = cycles
        out["kernel_ms_from_profile_cycles"] = cycles / (ghz * 1e9) * 1e3
        out["kernel_ms_measured_over_predicted"] = kernel_ms / out["kernel_ms_from_profile_cycles"]
    return out


def time_steps(torch, fn, steps, warmup, before_timed=None):
    """Wall time per step over exactly `steps` calls, and the average launch duration from one pair of events
    on the launch stream around the timed region (the launches queue back to back on the stream).

    Python's cyclic garbage collector is switched off for the duration: a full collection in a process that has
    imported torch pauses the host for 30-40 ms, and when that falls into a window of 200 launches of a 0.1 ms
    kernel the stream runs dry and the window reads twice its real time (seen as 0.2-0.26 ms for mm_t 4096^3
    and row softmax, always at the same launch count)."""
    import gc

    gc.collect()
    gc.disable()
    try:
        for _ in range(warmup):
            fn()
        if before_timed:
            before_timed()  # (enqueued work, e.g. clearing counters: ordered before the first timed launch)
        torch.cuda.synchronize()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        start.record()
        for _ in range(steps):
            fn()
        end.record()
        torch.cuda.synchronize()
    finally:
        gc.enable()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    kernel_ms = start.elapsed_time(end) / steps
    return wall_ms, kernel_ms


def sm_bytes_of(rows, cols):
    return 2.0 * rows * cols * 4  # one read and one write per element


def host_cpu_model():
    try:
        for line in Path("/proc/cpuinfo").read_text().splitlines():
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def rel_err(got, ref):
    import numpy as np

    return float(np.abs(got - ref).max() / max(float(np.abs(ref).max()), 1e-30))


def emitted_c_baseline(oracle, component, operands, work, unit, sample, got, repeats=1):
    """Times the C emitted for `component` (compiled the reference's way) on `operands` (NumPy, f32) on one host
    core, and compares `got` (the GPU's result for the same operands) with what it computes."""
    prog = oracle.compile_component(component.handle)
    t0 = time.perf_counter()
    for _ in range(repeats):
        ref = prog.run(*operands)
    seconds = (time.perf_counter() - t0) / repeats
    err = rel_err(got, ref)
    return {"value": work / seconds, "unit": unit, "cores": 1, "kind": "port",
            "form": "emitted-c: the C that the restated reference C backend prints for this line's own component "
                    "strings, built with cc -O3 -shared -fPIC -lm and run through count/ranks/shapes/exec",
            "host_cpu": host_cpu_model(), "seconds": seconds, "sample": sample}, err


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # defaults: the launch time keeps falling over the first two dozen launches of a process (2.2 ms -> 1.8 ms
    # while the clocks settle), so the warm-up is longer than the launch count alone would suggest
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=30)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-full", action="store_true",
                    help="time the emitted C of mm_t on the whole workload instead of a sample (about four minutes)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain 256 MiB device copy, a kernel of known traffic for scaling profiler counters")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    import numpy as np
    import torch

    from i_amd import Component as i, I
    from i_amd import _native as nat

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")

    def normal(shape, seed, amp=1.0):
        return np.random.default_rng(seed).standard_normal(shape, dtype=np.float32) * np.float32(amp)

    def to_dev_bf16(a):
        return torch.from_numpy(a).to(dev).bfloat16()

    import oracle  # the CPU side of the checks at the end (and bf16 rounding of host data); never on a timed path

    # All operands are generated on the host and moved to HBM before anything is timed: seconds of host-only work
    # between two timed regions would let the device clock down, and the kernels timed next would read slow.
    B, H, N, D = 8, 32, 4096, 128
    q, k, v = (to_dev_bf16(normal((B, H, N, D), seed)) for seed in (1, 2, 3))
    rows, cols = 16384, 4096
    xs = [torch.from_numpy(normal((rows, cols), seed)).to(dev) for seed in (1, 11, 12, 13)]
    M = 4096
    a_host = oracle.to_bf16_f32(np.random.default_rng(1).uniform(-1, 1, (M, M)).astype(np.float32))
    b_host = oracle.to_bf16_f32(np.random.default_rng(2).uniform(-1, 1, (M, M)).astype(np.float32))
    a, b = to_dev_bf16(a_host), to_dev_bf16(b_host)
    B5, H5, N5, D5 = 1, 16, 32768, 64
    q5, k5, v5 = (to_dev_bf16(normal((B5, H5, N5, D5), seed, 2.0)) for seed in (1, 2, 3))
    demo_in = [np.random.default_rng(sd).uniform(-1, 1, (512, 64)).astype(np.float32) for sd in (1, 2, 3)]
    dq, dk, dv_ = (torch.from_numpy(t).to(dev) for t in demo_in)

    # ------------------------------------------------------------------ headline: attention B8 H32 N4096 d128
    scale = torch.tensor(np.float32(1.0 / np.sqrt(D)), dtype=torch.float32, device=dev)
    out = torch.empty(B, H, N, D, dtype=torch.float32, device=dev)
    attn = flash_component(i, I, "i:256,j:64")
    attn.into(out, q, k, scale, v)  # compile + first run outside the timed region
    for _ in range(PRE_WARMUP_LAUNCHES - 1):
        attn.into(out, q, k, scale, v)
    torch.cuda.synchronize()
    # the kernel's own clock accounting, cleared after the warm-up: it covers exactly the timed launches
    ticks = torch.zeros(2, dtype=torch.int64, device=dev)
    attn.clock_probe(ticks)
    wall_ms, kernel_ms = time_steps(torch, lambda: attn.into(out, q, k, scale, v), args.steps, args.warmup, ticks.zero_)
    attn.clock_probe(None)

    def ghz_of(counters):
        shader, constant = (int(x) for x in counters.tolist())
        return shader / constant / 10.0 if constant > 0 else None

    attn_ghz = ghz_of(ticks)
    side = torch.cuda.Stream()

    def clock_beside(fn, ms_per_call):
        """The shader clock while `fn`'s launches run, read by a one-wavefront kernel on a second stream over the
        middle of a batch of launches of its own (about 30 ms of them, never the timed ones)."""
        n = max(20, int(30.0 / ms_per_call))
        counters = torch.zeros(2, dtype=torch.int64, device=dev)
        torch.cuda.synchronize()
        for _ in range(n // 4):
            fn()
        nat.check(nat.core.i_hip_shader_clock_probe(counters.data_ptr(), int(n * ms_per_call * 1000 * 0.4), side.cuda_stream))
        for _ in range(n - n // 4):
            fn()
        torch.cuda.synchronize()
        return ghz_of(counters)

    attn_ghz_beside = clock_beside(lambda: attn.into(out, q, k, scale, v), kernel_ms)
    attn_kernel = attn.report().split()[1]
    flop = 4.0 * B * H * N * N * D
    tflops = flop / (wall_ms * 1e-3) / 1e12
    achieved = flop / (kernel_ms * 1e-3) / 1e12

    # Same launch, same instruction stream and cycle count, but operands that barely toggle the datapath
    # (every element 0.01): what the kernel does when the chip can hold its clock.  Reported beside the
    # headline, never as the headline; the gap between the two is power management, not scheduling.
    qc, kc, vc = (torch.full_like(q, 0.01) for _ in range(3))
    attn.clock_probe(ticks)
    _, const_ms = time_steps(torch, lambda: attn.into(out, qc, kc, scale, vc), max(args.steps // 2, 5), 2, ticks.zero_)
    attn.clock_probe(None)
    const_ghz = ghz_of(ticks)
    del qc, kc, vc
    attn.into(out, q, k, scale, v)  # leave the seeded result in `out` for the parity check below

    # ------------------------------------------------------------------ row softmax [16384, 4096] f32 (HBM bound)
    x = xs[0]
    y = torch.empty_like(x)
    sm = softmax_component(i, I)
    sm.into(y, x)
    sm_kernel = sm.report().split()[1]
    # The timed calls walk four input/output pairs (2 GiB): one pair alone (512 MiB) would be re-read partly out of
    # the 256 MiB Infinity Cache from one step to the next, and that is not HBM bandwidth.
    ys = [y] + [torch.empty_like(x) for _ in range(3)]
    turn = [0]

    def softmax_step():
        k_ = turn[0] % 4
        turn[0] += 1
        sm.into(ys[k_], xs[k_])

    # ~0.1 ms kernels: enough launches for a timed window of tens of milliseconds, after as long a warm-up
    # (short runs, as the profiler's counter passes use them, stay short)
    short_steps, short_warmup = (max(args.steps, 200), max(args.warmup, 100)) if args.steps >= 20 else (args.steps, args.warmup)
    _, sm_ms = time_steps(torch, softmax_step, short_steps, short_warmup)
    sm.into(y, x)  # the parity check below reads y
    # the same 256 MiB as rows of 32768 columns: one workgroup of 16 wavefronts per row, the row in registers
    wide_rows, wide_cols = 2048, 32768
    xw, yw = [t_.view(wide_rows, wide_cols) for t_ in xs], [t_.view(wide_rows, wide_cols) for t_ in ys]
    sm.into(yw[0], xw[0])
    smw_kernel = sm.report().split()[1]

    def wide_step():
        k_ = turn[0] % 4
        turn[0] += 1
        sm.into(yw[k_], xw[k_])

    _, smw_ms = time_steps(torch, wide_step, short_steps, short_warmup)
    smw_gbs = sm_bytes_of(wide_rows, wide_cols) / (smw_ms * 1e-3) / 1e9
    sm.into(yw[1], xw[1])
    wide_got = yw[1][:64].cpu().numpy()   # rows 0..63 of the second buffer pair, checked on the host below
    wide_in = xw[1][:64].cpu().numpy()
    sm.into(y, x)
    del xs, ys, xw, yw
    sm_bytes = sm_bytes_of(rows, cols)
    sm_gbs = sm_bytes / (sm_ms * 1e-3) / 1e9

    # ------------------------------------------------------------------ mm_t 4096^3 bf16 (MFMA bound)
    c = torch.empty(M, M, device=dev)
    mm = mm_t_component(i)
    mm.into(c, a, b)
    mm_kernel = mm.report().split()[1]
    _, mm_ms = time_steps(torch, lambda: mm.into(c, a, b), short_steps, short_warmup)
    mm_tflops = 2.0 * M ** 3 / (mm_ms * 1e-3) / 1e12
    mm_ghz = clock_beside(lambda: mm.into(c, a, b), mm_ms) if args.steps >= 20 else None

    # ------------------------------------------------------------------ long-sequence attention B1 H16 N32768 d64, x 2.0
    scale5 = torch.tensor(np.float32(1.0 / np.sqrt(D5)), dtype=torch.float32, device=dev)
    out5 = torch.empty(B5, H5, N5, D5, dtype=torch.float32, device=dev)
    attn5 = flash_component(i, I, "i:512,j:32")  # 512 query rows per workgroup, 32-key LDS tiles: the d = 64 kernel
    attn5.into(out5, q5, k5, scale5, v5)
    c5_kernel = attn5.report().split()[1]
    attn5.clock_probe(ticks)
    _, c5_ms = time_steps(torch, lambda: attn5.into(out5, q5, k5, scale5, v5), max(args.steps // 2, 5), 2, ticks.zero_)
    attn5.clock_probe(None)
    c5_ghz = ghz_of(ticks)
    c5_tflops = 4.0 * B5 * H5 * N5 * N5 * D5 / (c5_ms * 1e-3) / 1e12
    # The second bound of this line: at d = 64 there are only 256 matrix-core FLOP per exponential.  Per pair of scores
    # a lane's wave issues two v_exp_f32 (8 cycles each, a quarter of the vector rate), one v_cvt_pk_bf16_f32 and
    # one v_dot2c_f32_bf16 (4 cycles each): 12 vector cycles per score and wave instruction of 64 lanes, on 1024
    # SIMDs.  The matrix cores need 256 / 1024 = 0.25 cycles per score and lane, the vector pipe 12 / 64 = 0.1875.
    c5_scores = float(B5 * H5) * N5 * N5
    c5_valu_ms_nominal = c5_scores * 12.0 / 64.0 / 1024.0 / (NOMINAL_GHZ * 1e9) * 1e3
    c5_mfma_ms_nominal = 4.0 * c5_scores * D5 / (PEAK_BF16_TFLOPS * 1e12) * 1e3

    # ------------------------------------------------------------------ the reference's own demo: attention f32 [512, 64]
    # (BASELINE configs[0]): no scale, i:16,j:16, through the f32 kernel.  Timed here, with the other GPU work and
    # before the host legs below: after seconds of CPU-only work the device has clocked down, and a 70 us kernel
    # timed then reads ten times slower.
    demo = flash_demo_component(i, I)
    dout = torch.empty(512, 64, device=dev)
    demo.into(dout, dq, dk, dv_)
    c1_kernel = demo.report().split()[1]
    _, c1_ms = time_steps(torch, lambda: demo.into(dout, dq, dk, dv_), short_steps, short_warmup)
    c1_flop = 4.0 * 512 * 512 * 64
    c1_launches = demo.report().strip()

    # ------------------------------------------------------------------ one head of the headline's size class on its own
    # (bf16 [1, 8192, 128]: 64 query tiles of 128 rows for 256 CUs): the keys of the head in parts over workgroups, and the same
    # call with the split switched off.  (On the 128-row kernel, so that the profiles of the headline's kernel hold the
    # headline's launches only.)
    attn_one = flash_component(i, I, "i:128,j:64")
    q1, k1, v1 = (t_[0:1, 0:1].repeat(1, 1, 2, 1).contiguous() for t_ in (q, k, v))
    one_out = torch.empty(1, 1, 2 * N, D, dtype=torch.float32, device=dev)
    attn_one.into(one_out, q1, k1, scale, v1)
    one_launches = attn_one.report().strip()
    _, one_ms = time_steps(torch, lambda: attn_one.into(one_out, q1, k1, scale, v1), short_steps, short_warmup)
    one_split = one_out.clone()
    attn_one.option("attention.kv_parts", 1)  # the same program with its key loops left whole
    attn_one.into(one_out, q1, k1, scale, v1)
    one_err = float((one_split - one_out).abs().max() / one_out.abs().max())
    _, one_whole_ms = time_steps(torch, lambda: attn_one.into(one_out, q1, k1, scale, v1), short_steps, short_warmup)
    attn_one.option("attention.kv_parts", 0)
    one_flop = 4.0 * (2 * N) * (2 * N) * D

    # ------------------------------------------------------------------ the attention workload in f32 (the reference's
    # arithmetic type): batches 2 and 3 of the headline operands as f32, through the same compiled component
    BF = 2
    q32, k32, v32 = (t_[2:2 + BF].float() for t_ in (q, k, v))
    out32 = torch.empty(BF, H, N, D, dtype=torch.float32, device=dev)
    attn.into(out32, q32, k32, scale, v32)
    f32_kernel = attn.report().split()[1]
    _, f32_ms = time_steps(torch, lambda: attn.into(out32, q32, k32, scale, v32), max(args.steps // 5, 3), 2)
    f32_tflops = 4.0 * BF * H * N * N * D / (f32_ms * 1e-3) / 1e12

    # What this box's matrix cores deliver to the vendor's own GEMM (torch.matmul -> hipBLASLt, bf16 in, bf16 out)
    # on the same operands as the mm_t line: a practical ceiling for dense bf16 on random data on this box, next to
    # which the MFMA lines can be read.  Not part of the product path; the shader clock under dense MFMA work on
    # random operands stays well below the 2.4 GHz the 2.5 PFLOP/s peak is quoted at.
    lib_ms = lib_ghz = lib32_ms = None
    if args.steps >= 20:
        bt_ = b.t()
        torch.matmul(a, bt_)
        _, lib_ms = time_steps(torch, lambda: torch.matmul(a, bt_), short_steps, short_warmup)
        lib_ghz = clock_beside(lambda: torch.matmul(a, bt_), lib_ms)
        # the same product with an f32 result, which is what the mm_t line writes (twice the bytes stored)
        try:
            torch.mm(a, bt_, out_dtype=torch.float32)
            _, lib32_ms = time_steps(torch, lambda: torch.mm(a, bt_, out_dtype=torch.float32), short_steps, short_warmup)
        except (TypeError, RuntimeError):
            lib32_ms = None

    # ------------------------------------------------------------------ the reference's own entry point: mm_t 4096^3 on
    # host f32 buffers through i_exec_into (upload, f32 MFMA kernel, download, wait).  The operands cross PCIe in
    # page-locked chunks that several host threads fill and empty while the chunk before is in flight.
    host_c = np.empty((M, M), np.float32)
    for _ in range(3):  # (the first two calls size the blocks the library keeps from call to call: 130 and 10 ms)
        mm.into(host_c, a_host, b_host)
    host_kernel = mm.report().split()[1]
    host_calls = 5 if args.steps >= 20 else 1
    t0 = time.perf_counter()
    for _ in range(host_calls):
        mm.into(host_c, a_host, b_host)
    host_s = (time.perf_counter() - t0) / host_calls
    host_err = float(np.abs(host_c[:64] - (a_host[:64].astype(np.float64) @ b_host.astype(np.float64).T)).max() / np.abs(host_c[:64]).max())

    if args.calibrate_copy:
        y.copy_(x)  # 256 MiB read + 256 MiB written
        torch.cuda.synchronize()

    # ------------------------------------------------------------------ host legs: emitted C on one core, and the checks
    cpu = cpu2 = cpu2w = cpu3 = cpu5 = cpu1 = cpuf = None
    err4 = err2 = err2w = err3 = err5 = err1 = errf = None
    if not args.no_cpu_baseline:
        # C4: one (b, h) slice of the workload, 1024 of its 4096 query rows (query tiles and (b, h) pairs are the
        # outermost independent loops of the emitted nest, so the rate carries over to the whole workload)
        b0, h0, r4 = 3, 17, 2048
        ops = [q[b0:b0 + 1, h0:h0 + 1, :r4].float().cpu().numpy(), k[b0:b0 + 1, h0:h0 + 1].float().cpu().numpy(),
               np.float32(scale.item()), v[b0:b0 + 1, h0:h0 + 1].float().cpu().numpy()]
        cpu, err4 = emitted_c_baseline(
            oracle, attn, ops, 4.0 * r4 * N * D / 1e12, "TFLOP/s",
            f"(b,h) = ({b0},{h0}), query rows 0..{r4 - 1} against all {N} keys: 1/{B * H * N // r4} of the workload "
            "(independent outer loops: the rate carries over)", out[b0:b0 + 1, h0:h0 + 1, :r4].cpu().numpy())
        # C2: rows are independent
        r2 = rows  # the whole workload: a few seconds
        cpu2, err2 = emitted_c_baseline(
            oracle, sm, [x[:r2].cpu().numpy()], 2.0 * r2 * cols * 4 / 1e9, "GB/s",
            f"rows 0..{r2 - 1} of {rows} (algorithmic bytes of those rows)", y[:r2].cpu().numpy())
        cpu2w, err2w = emitted_c_baseline(
            oracle, sm, [wide_in], sm_bytes_of(64, wide_cols) / 1e9, "GB/s",
            f"rows 0..63 of {wide_rows} (algorithmic bytes of those rows)", wide_got)
        # C3: output tiles are independent; all of k
        m3 = M if args.cpu_full else 2048  # (a quarter of the output: about 40 s; --cpu-full: all of it, four minutes)
        cpu3, err3 = emitted_c_baseline(
            oracle, mm, [a_host[:m3], b_host[:m3]], 2.0 * m3 * m3 * M / 1e12, "TFLOP/s",
            f"rows 0..{m3 - 1} of A against rows 0..{m3 - 1} of B, all {M} of k: 1/{(M // m3) ** 2} of the workload",
            c[:m3, :m3].cpu().numpy())
        # C5: one head, 512 of its 32768 query rows against all keys
        h5, r5 = 7, 512
        ops5 = [q5[:, h5:h5 + 1, :r5].float().cpu().numpy(), k5[:, h5:h5 + 1].float().cpu().numpy(),
                np.float32(scale5.item()), v5[:, h5:h5 + 1].float().cpu().numpy()]
        cpu5, err5 = emitted_c_baseline(
            oracle, attn5, ops5, 4.0 * r5 * N5 * D5 / 1e12, "TFLOP/s",
            f"head {h5}, query rows 0..{r5 - 1} against all {N5} keys: 1/{H5 * N5 // r5} of the workload",
            out5[:, h5:h5 + 1, :r5].cpu().numpy())
        # the f32 attention line: (b, h) = (3, 17) of the headline operands again, fewer rows (the emitted C does
        # the same work per row whatever the operands' origin)
        rf = 256
        opsf = [q32[1:2, h0:h0 + 1, :rf].cpu().numpy(), k32[1:2, h0:h0 + 1].cpu().numpy(), np.float32(scale.item()),
                v32[1:2, h0:h0 + 1].cpu().numpy()]
        cpuf, errf = emitted_c_baseline(
            oracle, attn, opsf, 4.0 * rf * N * D / 1e12, "TFLOP/s",
            f"(b,h) = (3,{h0}), query rows 0..{rf - 1} against all {N} keys: 1/{BF * H * N // rf} of the workload",
            out32[1:2, h0:h0 + 1, :rf].cpu().numpy())
        # C1: the whole workload; the reference's own committed emission when it was built, else the C emitted here
        got1 = dout.cpu().numpy()
        if oracle.have_ref():
            oracle.ref_flash_attention(*demo_in)
            t0 = time.perf_counter()
            for _ in range(5):
                ref1 = oracle.ref_flash_attention(*demo_in)
            c1_s = (time.perf_counter() - t0) / 5
            err1 = rel_err(got1, ref1)
            cpu1 = {"value": c1_flop / c1_s / 1e12, "unit": "TFLOP/s", "cores": 1, "kind": "reference",
                    "form": "the reference's committed emission ilang-python/annotated-flashattn.c, built unmodified",
                    "host_cpu": host_cpu_model(), "seconds": c1_s, "sample": "the whole workload"}
        else:
            cpu1, err1 = emitted_c_baseline(oracle, demo, demo_in, c1_flop / 1e12, "TFLOP/s", "the whole workload", got1, 5)

    def roof(bound, achieved_, peak, unit, summary, kernel, ms, ghz=None):
        fields = {"bound": bound, "achieved": achieved_, "peak": peak, "unit": unit, "frac": achieved_ / peak,
                  "traffic": measured_traffic(summary), "kernel": kernel, "kernel_ms": ms}
        if bound == "mfma":
            fields.update(clock_fields(ghz, achieved_ / peak, kernel, ms))
        return fields

    line = {
        "metric": "attn TFLOP/s & %MFMA peak (B8,H32,N4096,d128); row-softmax HBM GB/s",
        "value": tflops, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "pre_warmup_launches": PRE_WARMUP_LAUNCHES,
        "ms_per_step": wall_ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic (NumPy default_rng seeds 1, 2, 3: standard_normal -> bf16)",
        "config": {"workload": "flash_attention_fwd B8 H32 N4096 d128, bf16 in / f32 accumulate / f32 out, "
                               "1/sqrt(d) scale, non-causal (BASELINE configs[3]); compiled from 𝚒 component strings",
                   "schedule": "i:256,j:64 (256 query rows per workgroup, 64-key LDS tiles)", "entry": "i_exec_into_device"},
        "roofline": dict(roof("mfma", achieved, PEAK_BF16_TFLOPS, "TFLOP/s", "flash_attention_B8_H32_N4096_d128_bf16.md",
                              attn_kernel, kernel_ms, attn_ghz),
                         shader_clock_source="counted by the kernel's own workgroups over the timed launches "
                                             "(s_memtime / s_memrealtime, i_hip_program_clock_probe)",
                         shader_clock_ghz_beside=attn_ghz_beside),
        "cpu_baseline": cpu, "rel_err": err4,
        "constant_operand_probe": {
            "workload": "the same launch with every element of Q, K, V equal to 0.01 (not the benchmark data)",
            "value": flop / (const_ms * 1e-3) / 1e12, "unit": "TFLOP/s", "kernel_ms": const_ms,
            "frac_of_peak": flop / (const_ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
            **clock_fields(const_ghz, flop / (const_ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, attn_kernel, const_ms)},
        "library_gemm_probe": None if lib_ms is None else {
            "workload": "torch.matmul (hipBLASLt) bf16 4096^3, bf16 out, on the operands of the mm_t line: the vendor "
                        "library's dense bf16 rate on this box, for reading the MFMA fractions against",
            "value": 2.0 * M ** 3 / (lib_ms * 1e-3) / 1e12, "unit": "TFLOP/s", "kernel_ms": lib_ms,
            "frac_of_peak": 2.0 * M ** 3 / (lib_ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
            "shader_clock_ghz": lib_ghz,
            "frac_at_measured_clock": None if not lib_ghz else 2.0 * M ** 3 / (lib_ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS * NOMINAL_GHZ / lib_ghz,
            "shader_clock_source": "a one-wavefront kernel on a second stream beside a second batch of launches (i_hip_shader_clock_probe)",
            "f32_out": None if lib32_ms is None else {
                "workload": "the same product with an f32 result (torch.mm, out_dtype float32), as the mm_t line writes it",
                "value": 2.0 * M ** 3 / (lib32_ms * 1e-3) / 1e12, "kernel_ms": lib32_ms,
                "frac_of_peak": 2.0 * M ** 3 / (lib32_ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS}},
        "secondary": [
            {"workload": "row_softmax f32 [16384,4096] (BASELINE configs[1]); the steps rotate over 4 input/output pairs (2 GiB) so that nothing is re-read from the Infinity Cache", "value": sm_gbs, "unit": "GB/s",
             "roofline": roof("hbm", sm_gbs, PEAK_HBM_GBS, "GB/s", "row_softmax_16384x4096_f32.md", sm_kernel, sm_ms),
             "steps": short_steps, "warmup": short_warmup,
             "cpu_baseline": cpu2, "rel_err": err2},
            {"workload": "row_softmax f32 [2048,32768]: the same 256 MiB as rows eight times as wide (not a BASELINE "
                         "configuration; rows of 8192 < cols <= 65536 keep the row in the registers of one workgroup)",
             "value": smw_gbs, "unit": "GB/s",
             "roofline": roof("hbm", smw_gbs, PEAK_HBM_GBS, "GB/s", "row_softmax_2048x32768_f32.md", smw_kernel, smw_ms),
             "steps": short_steps, "warmup": short_warmup, "cpu_baseline": cpu2w, "rel_err": err2w},
            {"workload": "mm_t bf16 M=N=K=4096, f32 out (BASELINE configs[2])", "value": mm_tflops, "unit": "TFLOP/s",
             "roofline": roof("mfma", mm_tflops, PEAK_BF16_TFLOPS, "TFLOP/s", "gemm_nt_4096x4096x4096_bf16.md", mm_kernel, mm_ms, mm_ghz),
             "steps": short_steps, "warmup": short_warmup,
             "cpu_baseline": cpu3, "rel_err": err3},
            {"workload": "flash_attention_fwd B1 H16 N32768 d64, bf16 inputs x 2.0 (BASELINE configs[4])",
             "schedule": "i:512,j:32 (512 query rows per workgroup, 64 per wave; 32-key LDS tiles)",
             "value": c5_tflops, "unit": "TFLOP/s",
             "roofline": roof("mfma", c5_tflops, PEAK_BF16_TFLOPS, "TFLOP/s", "flash_attention_B1_H16_N32768_d64_bf16.md",
                              c5_kernel, c5_ms, c5_ghz),
             "second_bound": {
                 "what": "vector pipe: per pair of scores two v_exp_f32 (8 cycles), one v_cvt_pk_bf16_f32 and one "
                         "v_dot2c_f32_bf16 (4 cycles each) per 64 lanes on 1024 SIMDs; the matrix cores need 0.25 cycles "
                         "per score and lane at d = 64, the vector pipe 0.1875",
                 "valu_ms_at_2.4GHz": c5_valu_ms_nominal, "mfma_ms_at_2.4GHz": c5_mfma_ms_nominal,
                 "frac_of_valu_bound": c5_valu_ms_nominal / c5_ms,
                 "frac_of_max_bound": max(c5_valu_ms_nominal, c5_mfma_ms_nominal) / c5_ms,
                 "frac_of_max_bound_at_measured_clock": None if not c5_ghz else max(c5_valu_ms_nominal, c5_mfma_ms_nominal) / c5_ms * NOMINAL_GHZ / c5_ghz,
                 "frac_of_sum_of_bounds_at_measured_clock": None if not c5_ghz else (c5_valu_ms_nominal + c5_mfma_ms_nominal) / c5_ms * NOMINAL_GHZ / c5_ghz,
                 "binds": "mfma" if c5_mfma_ms_nominal >= c5_valu_ms_nominal else "valu"},
             "cpu_baseline": cpu5, "rel_err": err5},
            {"workload": "demo flash_attention f32 [512,64], no scale, i:16,j:16 (BASELINE configs[0])",
             "value": c1_flop / (c1_ms * 1e-3) / 1e12, "unit": "TFLOP/s", "kernel": c1_kernel, "kernel_ms": c1_ms,
             "steps": short_steps, "warmup": short_warmup, "launches": c1_launches,
             "cpu_baseline": cpu1, "rel_err": err1},
            {"workload": f"flash_attention_fwd B{BF} H32 N4096 d128 with f32 operands (batches 2 and 3 of the headline "
                         "operands as f32, full f32 arithmetic: the reference's own type; not a BASELINE configuration)",
             "value": f32_tflops, "unit": "TFLOP/s", "dtype": "f32",
             "roofline": roof("mfma", f32_tflops, PEAK_F32_TFLOPS, "TFLOP/s", "flash_attention_B2_H32_N4096_d128_f32.md",
                              f32_kernel, f32_ms),
             "cpu_baseline": cpuf, "rel_err": errf},
            {"workload": "mm_t f32 M=N=K=4096 through the host entry point i_exec_into (host f32 buffers in pageable memory: the "
                         "reference's own ABI; PCIe-inclusive, never the headline)",
             "value": 2.0 * M ** 3 / host_s / 1e12, "unit": "TFLOP/s", "ms_per_call": host_s * 1e3, "kernel": host_kernel,
             "pcie_GBps": 3.0 * M * M * 4 / host_s / 1e9, "bytes_over_pcie": 3 * M * M * 4, "calls": host_calls,
             "rel_err_against_f64": host_err},
            {"workload": f"flash_attention_fwd of one head, bf16 [1,{2 * N},{D}] (not a BASELINE configuration): 64 query "
                         "tiles of 128 rows for 256 CUs, so the keys of the head run in parts over workgroups",
             "value": one_flop / (one_ms * 1e-3) / 1e12, "unit": "TFLOP/s", "ms_per_call": one_ms, "launches": one_launches,
             "ms_per_call_unsplit": one_whole_ms, "rel_err_against_unsplit": one_err, "steps": short_steps, "warmup": short_warmup},
        ],
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
