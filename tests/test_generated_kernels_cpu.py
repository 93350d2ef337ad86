"""The generic code generator and the program executor on the CPU.

tests/hipshim replaces the HIP runtime with a host implementation (guard pages around every allocation,
NaN-filled memory, work-items run one after the other) and hipcc with g++, so every component below runs
through the product's executor with all kernels in their *generated* form and is compared with the C that
the oracle backend emits for the same component.  An out-of-bounds access by a generated kernel or a
buffer the executor sized wrongly ends the subprocess with SIGSEGV, after the case name was printed."""
import os
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
SHIM = ROOT / "tests" / "hipshim"
# the library's kept blocks (temporaries per stream, device copies of host operands) switched off: every buffer is
# then an allocation of its own, with the emulation's guard pages around it
ONE_ALLOCATION_EACH = {"ILANG_HIP_ARENA_MB": "0", "ILANG_HIP_STAGING_MB": "0"}


@pytest.fixture(scope="module")
def shim_lib():
    sys.path.insert(0, str(SHIM))
    import build as shim_build

    return shim_build.build()


def run_cases(shim_lib, extra_env, names=()):
    env = dict(os.environ)
    # ILANG_HIP_UNCHECKED: plain accesses instead of the bounds-checked ones the product emits, so that an access
    # outside a buffer still hits a guard page here and names a lowering that is not sound
    env.update({"ILANG_CORE_LIB": str(shim_lib), "ILANG_HIPCC": str(SHIM / "hostcc.py"),
                "ILANG_NO_TORCH": "1", "ILANG_NO_DISK_CACHE": "1", "ILANG_HIP_UNCHECKED": "1", **ONE_ALLOCATION_EACH})
    env.update(extra_env)
    r = subprocess.run([sys.executable, str(SHIM / "run_cases.py"), *names], env=env, capture_output=True, text=True, timeout=900)
    last = [l for l in r.stdout.splitlines() if l.startswith("CASE")][-1:] or ["(none started)"]
    assert r.returncode == 0, f"exit {r.returncode}; last case: {last[0]}\n{r.stdout[-2000:]}\n{r.stderr[-2000:]}"
    assert "failed: []" in r.stdout


def test_generated_kernels_match_the_emitted_c_on_the_cpu(shim_lib):
    run_cases(shim_lib, {})


def test_reduction_nests_with_their_outer_loop_in_parts_match_too(shim_lib):
    """The program option generated.parts (ILANG_SHIM_PARTS to the case runner) deals the outermost sequential loop of
    every nest that only accumulates out over that many groups of work-items, each with copies of its own of the
    accumulated buffers, and a second kernel folds the copies: 3 parts (one pass of the fold, ragged shares), 256
    parts (two passes; most parts get no iteration at these sizes), both forms of a nest (a work-item or a wavefront
    per iteration), and work-items last to first.  (3 parts on every case; the other settings on a few.)"""
    run_cases(shim_lib, {"ILANG_SHIM_PARTS": "3", "ILANG_SHIM_TOLERANCE": "1e-4"})
    few = ["total", "column max", "row sum 5x300", "column normalize (two nests)", "fused matrix-vector product", "mm_t"]
    run_cases(shim_lib, {"ILANG_SHIM_PARTS": "16", "ILANG_SHIM_TOLERANCE": "1e-4", "ILANG_HIP_UNCHECKED": "0"}, names=few)
    run_cases(shim_lib, {"ILANG_SHIM_PARTS": "256", "ILANG_SHIM_TOLERANCE": "1e-4"}, names=few[:4])
    run_cases(shim_lib, {"ILANG_SHIM_PARTS": "5", "ILANG_SHIM_WAVE": "1", "ILANG_SHIM_TOLERANCE": "1e-4"}, names=few[:3] + ["sum over the two last axes"])
    run_cases(shim_lib, {"ILANG_SHIM_PARTS": "4", "ILANG_SHIM_ORDER": "reverse", "ILANG_SHIM_TOLERANCE": "1e-4"}, names=few)


def test_generated_kernels_do_not_depend_on_work_item_order(shim_lib):
    """Work-items run last to first: a dependency between work-items would change the result."""
    run_cases(shim_lib, {"ILANG_SHIM_ORDER": "reverse", "ILANG_SHIM_CASES": "sample"})


def test_wavefront_form_of_reduction_nests_matches_too(shim_lib):
    """The program option generated.wave = 1 (ILANG_SHIM_WAVE=1 to the case runner) takes the form of a nest in which a wavefront stands where a work-item stood (reduction
    loops spread over its 64 lanes, lane shares combined by a butterfly) wherever a nest has one; the emulation
    runs the lanes as 64 threads.  The order of a sum changes, hence the f32 bar instead of 1e-5."""
    run_cases(shim_lib, {"ILANG_SHIM_WAVE": "1", "ILANG_SHIM_CASES": "wave", "ILANG_SHIM_TOLERANCE": "1e-4"})
    run_cases(shim_lib, {"ILANG_SHIM_WAVE": "1", "ILANG_SHIM_TOLERANCE": "1e-4", "ILANG_HIP_UNCHECKED": "0"},
              names=["row sum 5x300", "fused matrix-vector product", "column max", "mlp with pair"])


def test_checked_accesses_give_the_same_results(shim_lib):
    """The form the product emits by default: every access checked against its buffer's element count."""
    run_cases(shim_lib, {"ILANG_HIP_UNCHECKED": "0", "ILANG_SHIM_CASES": "sample"})


def test_schedules_with_unsound_lowerings_cannot_fault(shim_lib):
    """Schedules the reference accepts but lowers to loop nests that read past their buffers (a column reduction
    recomputed under its consumer's loops over the reduced index: its tail guard mixes the loops of both stages;
    found by random schedules on this emulation).  The reference reads heap garbage there; the generated kernels
    check every access, so on a device this is a wrong result for a schedule that was wrong already, not a memory
    fault.  Unchecked, each of these hits a guard page."""
    env = dict(os.environ, ILANG_CORE_LIB=str(shim_lib), ILANG_HIPCC=str(SHIM / "hostcc.py"),
               ILANG_NO_TORCH="1", ILANG_NO_DISK_CACHE="1", **ONE_ALLOCATION_EACH)
    code = """
import sys
import numpy as np
from i_amd import Component as i, I
cases = [(">ij~j|i:4:2,j:4|jij'i'i''", "ij-j~ij|i:4:2,j:4|jij'i'i''1", (13, 10)),
         (">ij~j|i:2,j:3|jii'j'", "ij-j~ij|i:2,j:3|jii'1j'", (5, 6)),
         ("+ij~j|i:8|ii'j", "ij-j~ij|i:8|ii'j1", (10, 9))]
a, b, shape = cases[int(sys.argv[1])]
x = np.random.default_rng(1).standard_normal(shape).astype(np.float32)
comp = (I & i(a)) >> i(b)
comp.option("generated.only", 1)
out = comp.exec_numpy(x)
print("ran", out.shape == shape)
"""
    for n in range(3):
        r = subprocess.run([sys.executable, "-c", code, str(n)], env=env, capture_output=True, text=True, cwd=ROOT, timeout=300)
        assert r.returncode == 0 and "ran True" in r.stdout, (n, r.returncode, r.stderr[-500:])
        unchecked = subprocess.run([sys.executable, "-c", code, str(n)], env=dict(env, ILANG_HIP_UNCHECKED="1"),
                                   capture_output=True, text=True, cwd=ROOT, timeout=300)
        assert unchecked.returncode == -11, (n, unchecked.returncode)  # SIGSEGV on a guard page: the access is real


def test_fixed_workspace_entry_matches_on_the_cpu(shim_lib):
    """i_exec_into_device_noalloc: every temporary comes out of one fixed block (here a guarded host block of the
    product's size), also with reduction loops in parts (whose copies are temporaries too); results must equal the
    emitted C as through the allocating entry."""
    run_cases(shim_lib, {"ILANG_SHIM_NOALLOC": "1"})
    run_cases(shim_lib, {"ILANG_SHIM_NOALLOC": "1", "ILANG_SHIM_PARTS": "3", "ILANG_SHIM_TOLERANCE": "1e-4", "ILANG_SHIM_CASES": "sample"})


def test_operands_that_disagree_on_a_shared_index_are_refused_before_any_launch(shim_lib):
    """A kernel takes each loop bound from one operand; another operand with a smaller extent for the same index
    would be read out of bounds (a GPU memory fault on the device, a guard-page hit here)."""
    env = dict(os.environ, ILANG_CORE_LIB=str(shim_lib), ILANG_HIPCC=str(SHIM / "hostcc.py"),
               ILANG_NO_TORCH="1", ILANG_NO_DISK_CACHE="1", **ONE_ALLOCATION_EACH)
    code = """
import numpy as np
from i_amd import Component as i
ones = lambda *s: np.ones(s, np.float32)
cases = [
    (i('ij+ij~ij'), [ones(64, 64), ones(2, 2)], 'inputs 0 and 1 disagree'),
    (i("ik*jk~ijk | i:16,j:16 | jii'j'k") >> i("+ijk~ij | i:16,j:16 | jii'j'k0"), [ones(8, 4), ones(8, 5)], 'inputs 0 and 1 disagree'),
    (i('ij+ij~ij') >> i('ij*ij~ij'), [ones(8, 4), ones(8, 4), ones(8, 5)], 'disagree'),   # tied through an intermediate result
    (i('ik*kj~ijk') >> i('+ijk~ij'), [ones(8, 4), ones(5, 3)], 'dimension 1 of input 0 is 4, dimension 0 of input 1 is 5'),
]
for comp, operands, text in cases:
    try:
        comp.exec_numpy(*operands)
        print('NOT REFUSED')
    except RuntimeError as e:
        print('ok' if text in str(e) else 'WRONG TEXT: ' + str(e))
print(i('ij+ij~ij').exec_numpy(ones(3, 2), ones(3, 2)).sum())
"""
    r = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, cwd=ROOT, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert r.stdout.split() == ["ok"] * 4 + ["12.0"], r.stdout


def test_generated_sources_compile_for_the_device():
    """The emulation compiles the generated source with the host compiler, which does not see what only the device
    compiler refuses (a pragma in the wrong place, a builtin spelled wrongly): hipcc cross-compiles the source of a
    few components with every form of a nest for gfx950 here, without a GPU."""
    import tempfile

    from i_amd import Component as i, I

    hipcc = Path(os.environ.get("ROCM_PATH", "/opt/rocm")) / "bin" / "hipcc"
    if not hipcc.exists():
        pytest.skip("no hipcc here")
    s = "i:16,j:16"
    comps = [i("+ij~."), i("+ij~j"), (I & i("+ij~j||ij")) >> i("ij/j~ij||1ij"), i("+bij~b"), i(">ij~i|j:16|ijj'"),
             i("ij*j~ij||ij") >> i("+ij~i||ij0"),
             (I & i(f">ij~i|{s}|jii'j'")) >> i(f"ij-i~ij|{s}|1jii'j'"), i(f"ik*jk~ijk | {s} | jii'j'k") >> i(f"+ijk~ij | {s} | jii'j'k0")]
    with tempfile.TemporaryDirectory() as tmp:
        for n, comp in enumerate(comps):
            code = comp._code()
            src = Path(tmp) / f"c{n}.hip"
            src.write_text(code[code.index("// generated by the i gfx950 backend"):])
            r = subprocess.run([str(hipcc), "--genco", "--offload-arch=gfx950", "-O1", "-std=c++17", str(src), "-o", str(src) + ".hsaco"],
                               capture_output=True, text=True, timeout=600)
            assert r.returncode == 0, (n, r.stderr[-1500:])


def test_every_loop_nest_of_a_kernel_is_a_kernel_of_its_own():
    """A kernel whose body is a sequence of loop nests is generated as one kernel per nest, each with the buffers its
    nest touches and a grid of its own; the initialisation of a scalar stays with the nest that accumulates into it.
    Nests that only accumulate also get the form with their outermost sequential loop in parts."""
    env = dict(os.environ, ILANG_NO_TORCH="1")
    code = ("from i_amd import Component as i, I\n"
            "print(((I & i('+ij~j||ij')) >> i('ij/j~ij||1ij'))._code())\n"
            "print('=====')\n"
            "print(i('+ij~.')._code())")
    out = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, cwd=ROOT, timeout=300).stdout
    colnorm, total = out.split("=====")
    assert "1 kernel(s)" in colnorm and "loop nest as kernel f0, work-items: i3" in colnorm and "loop nest as kernel f1, work-items: i0 i1" in colnorm
    assert "f0_g, loop i2 in parts" in colnorm and "__syncthreads" not in colnorm
    assert 'void __launch_bounds__(64) f0_g(Args_f0_g args)' in colnorm and "ilang_combine" in colnorm
    # the column sums stay in a register across the rows: one load before the loop over i2 and one store after it
    assert "float h0_i2 = " in colnorm
    assert "generated as f0, work-items: 1 (no independent outer loop)" in total
    assert "f0_g / f0_gw, loop i0 in parts" in total and "for (size_t i0 = part * share_i0; i0 < end_i0; ++i0)" in total
