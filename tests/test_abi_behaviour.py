"""Behaviour of the C ABI that needs no GPU: handle ownership, NULL handling and
error reporting as in the reference runtime (core/src/lib.rs:61-351), shape
queries, and loud failure when no device can run the program."""
import ctypes
import threading

import numpy as np
import pytest

from i_amd import Component as i, I
from i_amd import _native as nat
from i_amd import ilang

core = nat.core


def test_null_handles_report_reference_errors():
    assert not core.i_chain(None, I.handle) and nat.last_error() == "null left component"
    assert not core.i_chain(I.handle, None) and nat.last_error() == "null right component"
    assert not core.i_swap(None) and nat.last_error() == "null component"
    assert not core.i_code(None) and nat.last_error() == "null component"
    assert not core.i_compile(None) and nat.last_error() == "null component"
    assert core.i_output_count(None) == 0 and nat.last_error() == "null program"
    assert core.i_output_ranks(None, None) == -1 and nat.last_error() == "null program"
    assert core.i_exec_into(None, None, 0, None, 0) == -1 and nat.last_error() == "null program"
    out = core.i_exec(None, None, 0)
    assert out.count == 0 and not out.tensors and nat.last_error() == "null program"
    # frees accept NULL
    core.i_component_free(None)
    core.i_program_free(None)
    core.i_string_free(None)
    core.i_outputs_free(ilang._COutputs(None, 0))


def test_error_is_thread_local_and_sticky():
    assert not core.i_swap(None)
    assert nat.last_error() == "null component"
    assert i("ij~ij").handle  # success does not clear the slot
    assert nat.last_error() == "null component"
    seen = {}

    def other():
        err = core.i_error()
        seen["fresh"] = err
        core.i_swap(None)
        seen["after"] = core.i_error()

    t = threading.Thread(target=other)
    t.start()
    t.join()
    assert seen["fresh"] is None and seen["after"] == b"null component"


def test_combinators_clone_operands():
    a, b = i("ij~ij"), i("+ij~i")
    c = a >> b
    del a, b  # operands freed; the combined tree must stay valid
    assert "1 kernel(s)" in c._code() or "2 kernel(s)" in c._code()


def test_output_shapes_and_ranks_without_running():
    mm = i("ik*jk~ijk | i:16,j:16 | jii'j'k") >> i("+ijk~ij | i:16,j:16 | jii'j'k0")
    a, b = np.zeros((33, 20), np.float32), np.zeros((17, 20), np.float32)
    assert mm.output_shapes(a, b) == [(33, 17)]
    two = i("+ij~i") & i(">ij~j")
    assert two.output_shapes(np.zeros((4, 9), np.float32)) == [(4,), (9,)]
    assert (~two).output_shapes(np.zeros((4, 9), np.float32)) == [(9,), (4,)]
    scalar = i("+ij~.")
    assert scalar.output_shapes(np.zeros((4, 9), np.float32)) == [()]


def test_output_shapes_rejects_low_rank_inputs():
    mm = i("ik*kj~ijk") >> i("+ijk~ij")
    with pytest.raises(RuntimeError) as err:
        mm.output_shapes(np.zeros((4, 3), np.float32), np.zeros((4,), np.float32))
    assert "rank" in str(err.value)
    # like the reference's emitted `shapes`, only the dimensions an output is sized by are read
    assert mm.output_shapes(np.zeros((4,), np.float32), np.zeros((4, 3), np.float32)) == [(4, 3)]


def test_exec_into_checks_output_count_before_touching_the_device():
    prog = i("+ij~i")
    program = prog._compile()
    x = np.zeros((4, 9), np.float32)
    arr, keep = ilang._pack([ilang._operand(x, "input")], on_device=False)
    assert core.i_exec_into(program, arr, 1, None, 0) == -1
    assert nat.last_error() == "wrong output count"
    assert core.i_exec_into(program, None, 1, None, 1) == -1
    assert nat.last_error() == "null inputs"
    assert core.i_exec_into(program, arr, 1, None, 1) == -1
    assert nat.last_error() == "null outputs"


def test_exec_into_refuses_an_output_whose_stated_extents_are_not_what_the_program_writes():
    """A caller that states the extents of its output buffer (i_tensor_mut.shape) and states them too small would
    have its buffer overrun by the copy back to the host; the call is refused before anything runs.  The Python
    frontend states the extents of every NumPy output."""
    prog = i("+ij~i")
    program = prog._compile()
    x = np.zeros((4, 9), np.float32)
    arr, keep = ilang._pack([ilang._operand(x, "input")], on_device=False)
    for wrong in (np.zeros((3,), np.float32), np.zeros((4, 1), np.float32), np.zeros((5,), np.float32)):
        out, keep_out = ilang._pack([ilang._operand(wrong, "output")], on_device=False)
        assert core.i_exec_into(program, arr, 1, out, 1) == -1
        assert "the program writes [4]" in nat.last_error() and "output 0 has shape" in nat.last_error()
    with pytest.raises(RuntimeError, match="the program writes"):
        prog.into(np.zeros((2,), np.float32), x)


def test_which_programs_may_run_on_their_rows_in_slices():
    """i_hip_program_row_slices: the first index of the outputs has to be one that the program only maps over."""
    mm_t = i("ik*jk~ijk | i:16,j:16 | jii'j'k") >> i("+ijk~ij | i:16,j:16 | jii'j'k0")
    assert mm_t.row_slices() == [True, False]                      # rows of A and of C; all of B for every slice
    assert (i("ik*kj~ijk") >> i("+ijk~ij")).row_slices() == [True, False]
    softmax = (I & i(">ij~i")) >> i("ij-i~ij") >> i("^ij~ij") >> (I & i("+ij~i")) >> i("ij/i~ij")
    assert softmax.row_slices() == [True]                          # the reductions are over j
    s = "i:16,j:16"
    attn = (i(f"bhik*bhjk~bhijk | {s} | bhjii'j'k") >> i(f"+bhijk~bhij | {s} | bhjii'j'k0") >> i(f"bhij*.~bhij | {s} | bhji0i'j'")
            >> (I & i(f">bhij~bhi | {s} | bhji0i'j'")) >> i(f"bhij-bhi~bhij | {s} | bhji01i'j'") >> i(f"^bhij~bhij | {s} | bhji0i'j'")
            >> (I & i(f"+bhij~bhi | {s} | bhji0i'j'")) >> i(f"bhij/bhi~bhij | {s} | bhji01i'j'")
            >> i(f"bhij*bhjk~bhikj | {s} | bhji0i'kj'") >> i(f"+bhikj~bhik | {s} | bhjii'kj'0"))
    assert attn.row_slices() == [True, True, False, True]          # Q, K, V by batch; the scale whole
    assert i("+ij~i").row_slices() == [True] and i("^ij~ij").row_slices() == [True]
    # summed over, second dimension of the input, or under two names in one expression: whole
    assert i("+ij~j").row_slices() is None and i("+ij~.").row_slices() is None and i("ij~ji").row_slices() is None
    assert ((I & i("+ij~j||ij")) >> i("ij/j~ij||1ij")).row_slices() is None
    gram = (I & I) >> i("ik*jk~ijk | i:16,j:16 | jii'j'k") >> i("+ijk~ij | i:16,j:16 | jii'j'k0")
    assert gram.row_slices() is None
    # arguments
    flags = (ctypes.c_ubyte * 1)()
    assert nat.core.i_hip_program_row_slices(None, flags, 1) == -1 and "null program" in nat.last_error()
    assert nat.core.i_hip_program_row_slices(mm_t._compile(), flags, 1) == -1 and "2 inputs" in nat.last_error()
    assert nat.core.i_hip_program_row_slices(mm_t._compile(), None, 0) == 2


def test_identity_program_is_rejected_like_the_reference():
    # a program output that is a program input has no kernel to produce it
    with pytest.raises(RuntimeError) as err:
        I._compile()
    assert "output 0 references Input buffer 0" in str(err.value)


def test_no_device_fails_loudly():
    import torch

    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    x = np.ones((4, 9), np.float32)
    with pytest.raises(RuntimeError) as err:
        i("+ij~i").exec_numpy(x)
    assert "hip" in str(err.value).lower()
    with pytest.raises(RuntimeError):
        i("+ij~i").exec(x.tolist())


def test_generated_source_builds_for_gfx950_without_a_gpu():
    # i_compile runs hipcc for kernels that have no hand-written form
    prog = i("ik*kj~ijk|i:2,k:2|ii'jkk'") >> i("+ijk~ij|i:2,k:2|ii'j!kk'0")
    assert prog._compile()


def test_tensor_from_python_data():
    from i_amd import Tensor

    t = Tensor([[1, 2, 3], [4, 5, 6]])
    assert t.shape == (2, 3) and t.data == [1.0, 2.0, 3.0, 4.0, 5.0, 6.0]
    assert Tensor(2.5).shape == () and Tensor(2.5).data == [2.5]
    assert Tensor([]).shape == (0,) and Tensor([[], []]).shape == (2, 0)
    assert Tensor([1, 2, 3, 4], shape=(2, 2)).shape == (2, 2)
    assert "shape=(2, 3)" in repr(t)
    with pytest.raises(ValueError):
        Tensor([[1, 2], [3]])
    with pytest.raises(ValueError):
        Tensor([1, 2, 3], shape=(2, 2))
    with pytest.raises(TypeError):
        Tensor([["a"]])


def test_operands_must_share_a_place_and_outputs_are_written_in_place():
    prog = i("+ij~i")
    x = np.ones((4, 9), np.float32)
    with pytest.raises(TypeError):
        prog.into(np.zeros((4,), np.float64), x)           # an output is never converted
    with pytest.raises(TypeError):
        prog.into([1.0, 2.0, 3.0, 4.0], x)                 # a list cannot be written in place
    with pytest.raises(TypeError):
        prog.into(np.zeros((4,), np.float32), x, static_workspace=True)  # host operands have no workspace


def test_noalloc_entry_checks_arguments_before_touching_the_device():
    comp = i("+ij~i")  # owns the program
    program = comp._compile()
    assert core.i_exec_into_device_noalloc(None, None, 0, None, 0, None) == -1 and nat.last_error() == "null program"
    assert core.i_exec_into_device_noalloc(program, None, 1, None, 1, None) == -1 and nat.last_error() == "null inputs"
    assert core.i_exec_into_device_noalloc(program, None, 0, None, 0, None) == -1 and nat.last_error() == "wrong output count"
