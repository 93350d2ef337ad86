"""Python frontend of the 𝚒 gfx950 backend.

The public surface is the reference frontend's (ilang-python/ilang.py:147-394): ``Component`` / ``i(src)``
with the operators ``>> << & | ~``, the identity ``I``, ``Tensor`` for plain Python data, and the methods
``exec``, ``exec_numpy``, ``exec_torch``, ``into``, ``output_shapes``, ``_code``; failures of the library
surface as ``RuntimeError(i_error())``.

Underneath, every operand of a call (a ``Tensor``, a NumPy array, a CPU or ROCm torch tensor, a Python number
or nested list) is first reduced to one record, ``_Operand``: address, extents, element type, and whether
the address is host or device memory.  A call is then routed by where its operands live: host operands take
the reference's f32 path (``i_exec_into`` / ``i_exec``), ROCm tensors (float32 or bfloat16) are passed by
device pointer to ``i_exec_into_device`` and never leave the GPU.
"""
import array
import ctypes
import numbers
import sys

from . import _native as nat

core = nat.core
_sz = ctypes.c_size_t
_f32p = ctypes.POINTER(ctypes.c_float)
_vp = ctypes.c_void_p


# ---------------------------------------------------------------- the structs and prototypes of i.h / i_hip.h
class _CTensor(ctypes.Structure):
    _fields_ = [("data", _f32p), ("shape", ctypes.POINTER(_sz)), ("rank", _sz)]


class _COwnedTensor(ctypes.Structure):
    _fields_ = [("data", _f32p), ("shape", ctypes.POINTER(_sz)), ("rank", _sz), ("len", _sz)]


class _COutputs(ctypes.Structure):
    _fields_ = [("tensors", ctypes.POINTER(_COwnedTensor)), ("count", _sz)]


class _CDeviceTensor(ctypes.Structure):
    _fields_ = [("data", _vp), ("shape", ctypes.POINTER(_sz)), ("rank", _sz), ("dtype", ctypes.c_int)]


_PROTOTYPES = {
    "i_parse": ([ctypes.c_char_p], _vp),
    "i_identity": ([], _vp),
    "i_chain": ([_vp, _vp], _vp),
    "i_compose": ([_vp, _vp], _vp),
    "i_fanout": ([_vp, _vp], _vp),
    "i_pair": ([_vp, _vp], _vp),
    "i_swap": ([_vp], _vp),
    "i_code": ([_vp], _vp),
    "i_compile": ([_vp], _vp),
    "i_output_count": ([_vp], _sz),
    "i_output_ranks": ([_vp, ctypes.POINTER(_sz)], ctypes.c_int),
    "i_output_shapes": ([_vp, ctypes.POINTER(_CTensor), _sz, ctypes.POINTER(ctypes.POINTER(_sz))], ctypes.c_int),
    "i_exec_into": ([_vp, ctypes.POINTER(_CTensor), _sz, ctypes.POINTER(_CTensor), _sz], ctypes.c_int),
    "i_exec": ([_vp, ctypes.POINTER(_CTensor), _sz], _COutputs),
    "i_exec_into_device": ([_vp, ctypes.POINTER(_CDeviceTensor), _sz, ctypes.POINTER(_CDeviceTensor), _sz, _vp], ctypes.c_int),
    "i_exec_into_device_noalloc": ([_vp, ctypes.POINTER(_CDeviceTensor), _sz, ctypes.POINTER(_CDeviceTensor), _sz, _vp], ctypes.c_int),
    "i_component_free": ([_vp], None),
    "i_program_free": ([_vp], None),
    "i_outputs_free": ([_COutputs], None),
    "i_string_free": ([_vp], None),
}
for _name, (_args, _res) in _PROTOTYPES.items():
    getattr(core, _name).argtypes = _args
    getattr(core, _name).restype = _res


# ---------------------------------------------------------------- operands
class _Operand:
    """One operand of a call, whatever object it came from."""

    __slots__ = ("address", "extents", "dtype", "device", "anchor")

    def __init__(self, address, extents, dtype, device, anchor):
        self.address = address              # integer address of the first element (0 for an empty operand is fine)
        self.extents = tuple(extents) if type(extents).__name__ == "Size" else tuple(int(n) for n in extents)
        self.dtype = dtype                  # nat.F32 or nat.BF16
        self.device = device                # None: host memory; otherwise the torch device the address belongs to
        self.anchor = anchor                # whatever must stay alive while the address is in use


def _torch_like(x):
    torch = sys.modules.get("torch")
    if torch is not None and isinstance(x, torch.Tensor):
        return True
    return all(hasattr(x, name) for name in ("data_ptr", "device", "is_contiguous", "dtype"))


def _on_gpu(x):
    return _torch_like(x) and x.device.type != "cpu"


def _from_numpy(x, role):
    import numpy as np

    if role == "output":
        if x.dtype != np.float32 or not x.flags.c_contiguous:
            raise TypeError("a NumPy output has to be a C-contiguous float32 array (it is written in place)")
        if not x.flags.writeable:
            raise TypeError("a NumPy output has to be writeable")
    elif x.dtype != np.float32 or not x.flags.c_contiguous:
        x = np.ascontiguousarray(x, dtype=np.float32)  # the host ABI carries f32 only: other inputs are copied
    return _Operand(x.ctypes.data, x.shape, nat.F32, None, x)


_TORCH_DTYPES = {"torch.float32": nat.F32, "torch.bfloat16": nat.BF16}


def _from_torch(x, role):
    dtype = _TORCH_DTYPES.get(str(x.dtype))
    if x.device.type == "cpu":
        if dtype != nat.F32:
            raise TypeError(f"a CPU torch {role} has to be float32, got {x.dtype}")
        if not x.is_contiguous():
            if role == "output":
                raise TypeError("a torch output has to be contiguous (it is written in place)")
            x = x.contiguous()
        return _Operand(x.data_ptr(), x.shape, nat.F32, None, x)
    if dtype is None:
        raise TypeError(f"a GPU {role} has to be float32 or bfloat16, got {x.dtype}")
    if not x.is_contiguous():
        raise TypeError(f"a GPU {role} has to be contiguous")
    return _Operand(x.data_ptr(), x.shape, dtype, x.device, x)


def _operand(x, role):
    if isinstance(x, Tensor):
        return x._operand()
    if _torch_like(x):
        return _from_torch(x, role)
    if type(x).__module__.split(".")[0] == "numpy" and hasattr(x, "ctypes"):
        return _from_numpy(x, role)
    if role == "output":
        raise TypeError(f"an output has to be a NumPy array or a torch tensor, got {type(x).__name__}")
    return Tensor(x)._operand()


def _extent_buffer(extents):
    return (_sz * max(len(extents), 1))(*extents)


def _pack(operands, on_device):
    """The C array for a list of operands, plus the objects that must outlive the call."""
    keep = [op.anchor for op in operands]
    records = []
    for op in operands:
        dims = _extent_buffer(op.extents)
        keep.append(dims)
        if on_device:
            records.append(_CDeviceTensor(op.address, dims, len(op.extents), op.dtype))
        else:
            records.append(_CTensor(ctypes.cast(op.address, _f32p), dims, len(op.extents)))
    kind = _CDeviceTensor if on_device else _CTensor
    return (kind * max(len(records), 1))(*records), keep


def _current_stream(torch, device):
    """The raw handle of torch's current stream on `device` (the device is current when this is called)."""
    raw = getattr(torch._C, "_cuda_getCurrentRawStream", None)
    if raw is not None:
        return raw(torch.cuda.current_device() if device.index is None else device.index)
    return torch.cuda.current_stream().cuda_stream


def _placement(operands, what):
    """None when every operand is host memory, the torch device when every operand is on one GPU."""
    devices = {op.device for op in operands}
    if len(devices) > 1:
        raise TypeError(f"{what} live in different places ({', '.join(sorted(str(d or 'host') for d in devices))}); "
                        "move them all to one GPU or all to the host")
    return devices.pop() if devices else None


# ---------------------------------------------------------------- Tensor
def _measure(x):
    """Extents of a number or of rectangular nested sequences, judged along the first element of each level."""
    extents = []
    while isinstance(x, (list, tuple)):
        extents.append(len(x))
        if not x:
            break
        x = x[0]
    else:
        if not isinstance(x, numbers.Real):
            raise TypeError(f"Tensor data has to be a number or nested lists of numbers, found {type(x).__name__}")
    return tuple(extents)


def _pour(x, extents, level, out):
    if level == len(extents):
        if not isinstance(x, numbers.Real):
            raise TypeError(f"Tensor data has to be a number or nested lists of numbers, found {type(x).__name__}")
        out.append(float(x))
        return
    if not isinstance(x, (list, tuple)) or len(x) != extents[level]:
        raise ValueError(f"Tensor data is not rectangular: expected {extents[level]} items at depth {level}")
    for item in x:
        _pour(item, extents, level + 1, out)


class Tensor:
    """A host f32 tensor made from a Python number or nested lists (reference: ilang-python/ilang.py:147-199).
    ``Tensor(values, shape)`` takes flat values.  ``.shape`` is a tuple, ``.data`` the flat list of values."""

    def __init__(self, x, shape=None):
        values = array.array("f")
        if shape is None:
            self.shape = _measure(x)
            _pour(x, self.shape, 0, values)
        else:
            self.shape = tuple(int(n) for n in shape)
            values.extend(float(v) for v in x)
            count = 1
            for n in self.shape:
                count *= n
            if len(values) != count:
                raise ValueError(f"shape {self.shape} holds {count} values, got {len(values)}")
        self._values = values

    @classmethod
    def _take(cls, owned):
        """Copies one library-owned output record (i_owned_tensor) into a Tensor."""
        self = cls.__new__(cls)
        self.shape = tuple(owned.shape[d] for d in range(owned.rank))
        self._values = array.array("f", bytes(ctypes.string_at(owned.data, owned.len * 4)) if owned.len else b"")
        return self

    @property
    def data(self):
        return self._values.tolist()

    def _operand(self):
        address, _ = self._values.buffer_info()
        return _Operand(address, self.shape, nat.F32, None, self._values)

    def __repr__(self):
        return f"Tensor(shape={self.shape}, data={self.data})"


# ---------------------------------------------------------------- Component
class Component:
    """An 𝚒 component: an expression ``i("ik*jk~ijk | i:16 | ii'jk")`` or a combination of components."""

    def __init__(self, src=None, *, _handle=None):
        self._ptr = None
        self._program = None
        self._extents_seen = {}  # output extents by input extents
        if _handle is None:
            if not isinstance(src, str):
                raise TypeError("Component takes the source text of one expression")
            _handle = core.i_parse(src.encode())
        self._ptr = nat.check_ptr(_handle)

    def __del__(self, _core=core):  # bound at definition: module globals may be gone at interpreter shutdown
        if getattr(self, "_program", None):
            _core.i_program_free(self._program)
        if getattr(self, "_ptr", None):
            _core.i_component_free(self._ptr)
        self._program = self._ptr = None

    @property
    def handle(self):
        """The ``i_component*`` behind this object (owned by it)."""
        return self._ptr

    # combinators: each returns a new component; the operands stay valid (the library clones them)
    def _with(self, other, combine):
        if isinstance(other, str):
            other = Component(other)
        if not isinstance(other, Component):
            return NotImplemented
        return Component(_handle=combine(self._ptr, other._ptr))

    def chain(self, other):
        return self._with(other, core.i_chain)

    def compose(self, other):
        return self._with(other, core.i_compose)

    def fanout(self, other):
        return self._with(other, core.i_fanout)

    def pair(self, other):
        return self._with(other, core.i_pair)

    def swap(self):
        return Component(_handle=core.i_swap(self._ptr))

    __rshift__ = chain
    __lshift__ = compose
    __and__ = fanout
    __or__ = pair
    __invert__ = swap

    def _compile(self):
        """The compiled program, built on first use and kept for the life of the component."""
        if not self._program:
            self._program = nat.check_ptr(core.i_compile(self._ptr))
        return self._program

    def _code(self):
        """The backend's source for this component: the kernel plan and the generated HIP."""
        text = nat.check_ptr(core.i_code(self._ptr))
        try:
            return ctypes.string_at(text).decode()
        finally:
            core.i_string_free(text)

    def option(self, name, value):
        """Sets an option of the compiled program (``i_hip_program_option``), e.g. ``"attention.f32_scale", 1``."""
        nat.check(core.i_hip_program_option(self._compile(), name.encode(), int(value)))
        return self

    def clock_probe(self, ticks):
        """Shader-clock accounting for the program's attention kernels (``i_hip_program_clock_probe``): ``ticks`` is
        a ROCm tensor of two int64 that the caller clears (or None: off); workgroups add shader-clock cycles to
        ``ticks[0]`` and ticks of the constant 100 MHz clock to ``ticks[1]``."""
        if ticks is not None and (ticks.numel() < 2 or ticks.element_size() != 8 or not ticks.is_cuda):
            raise ValueError("clock_probe takes a ROCm tensor of two 64-bit integers")
        nat.check(core.i_hip_program_clock_probe(self._compile(), None if ticks is None else ticks.data_ptr()))
        return self

    def row_slices(self):
        """Whether the program may be run on its outputs' first index slice by slice (``i_hip_program_row_slices``):
        None if it has to run whole, else one flag per input, True for the inputs that are cut along their first
        dimension with the outputs and False for those that every slice needs whole."""
        flags = (ctypes.c_ubyte * 256)()
        n = core.i_hip_program_row_slices(self._compile(), flags, 256)
        if n < 0:
            nat.check(n)
        return None if n == 0 else [bool(flags[k]) for k in range(n)]

    def report(self):
        """The kernels the last run dispatched, one line per kernel of the plan (``i_hip_program_report``)."""
        text = nat.check_ptr(core.i_hip_program_report(self._compile()))
        try:
            return ctypes.string_at(text).decode()
        finally:
            core.i_string_free(text)

    def _result_extents(self, program, operands):
        # (asked of the library once per combination of input shapes: a serving loop calls with the same ones)
        key = tuple(op.extents for op in operands)
        cache = self._extents_seen
        found = cache.get(key)
        if found is None:
            if len(cache) >= 64:
                cache.clear()
            found = cache[key] = self._ask_result_extents(program, operands)
        return list(found)

    def _ask_result_extents(self, program, operands):
        count = core.i_output_count(program)
        ranks = (_sz * max(count, 1))()
        nat.check(core.i_output_ranks(program, ranks))
        rows = [_extent_buffer([0] * ranks[o]) for o in range(count)]
        table = (ctypes.POINTER(_sz) * max(count, 1))(*(ctypes.cast(r, ctypes.POINTER(_sz)) for r in rows))
        # only the extents of the inputs are read here, so device operands are described without their data
        described = [_Operand(0, op.extents, nat.F32, None, None) for op in operands]
        records, keep = _pack(described, on_device=False)
        nat.check(core.i_output_shapes(program, records, len(operands), table))
        del keep
        return [tuple(rows[o][d] for d in range(ranks[o])) for o in range(count)]

    def output_shapes(self, *inputs):
        return self._result_extents(self._compile(), [_operand(x, "input") for x in inputs])

    def exec(self, *inputs):
        """Runs on host data; the library allocates the outputs, which come back as ``Tensor``s."""
        program = self._compile()
        records, keep = _pack([_operand(x, "input") for x in inputs], on_device=False)
        produced = core.i_exec(program, records, len(inputs))
        del keep
        if not produced.tensors:
            raise RuntimeError(nat.last_error())
        try:
            results = [Tensor._take(produced.tensors[o]) for o in range(produced.count)]
        finally:
            core.i_outputs_free(produced)
        return results[0] if len(results) == 1 else tuple(results)

    def exec_numpy(self, *inputs):
        import numpy as np

        operands = [_operand(x, "input") for x in inputs]
        results = [np.empty(extents, dtype=np.float32) for extents in self._result_extents(self._compile(), operands)]
        self._run(operands, [_operand(r, "output") for r in results], False)
        return results[0] if len(results) == 1 else tuple(results)

    def exec_torch(self, *inputs, out_dtype=None, static_workspace=False):
        """Host tensors: as the reference (CPU float32 results).  ROCm tensors: runs on their device and on the
        current stream; results are float32 unless ``out_dtype`` says bfloat16.  ``static_workspace`` (ROCm
        tensors only) runs through ``i_exec_into_device_noalloc``: no device memory is allocated."""
        import torch

        operands = [_operand(x, "input") for x in inputs]
        device = _placement(operands, "inputs")
        extents = self._result_extents(self._compile(), operands)
        if device is None:
            results = [torch.empty(e, dtype=torch.float32) for e in extents]
        else:
            results = [torch.empty(e, dtype=out_dtype or torch.float32, device=device) for e in extents]
        self._run(operands, [_operand(r, "output") for r in results], static_workspace)
        return results[0] if len(results) == 1 else tuple(results)

    def into(self, outputs, *inputs, static_workspace=False):
        """Runs into caller-provided outputs (one object or a sequence of them) and returns them."""
        targets = list(outputs) if isinstance(outputs, (tuple, list)) else [outputs]
        self._run([_operand(x, "input") for x in inputs], [_operand(t, "output") for t in targets], static_workspace)
        return targets[0] if len(targets) == 1 else tuple(targets)

    def _run(self, operands, targets, static_workspace):
        program = self._compile()
        device = _placement(operands + targets, "inputs and outputs")
        in_records, keep_in = _pack(operands, device is not None)
        out_records, keep_out = _pack(targets, device is not None)
        if device is None:
            if static_workspace:
                raise TypeError("static_workspace applies to GPU tensors only")
            nat.check(core.i_exec_into(program, in_records, len(operands), out_records, len(targets)))
        else:
            import torch

            entry = core.i_exec_into_device_noalloc if static_workspace else core.i_exec_into_device
            if device.index is None or device.index == torch.cuda.current_device():
                nat.check(entry(program, in_records, len(operands), out_records, len(targets), _current_stream(torch, device)))
            else:
                with torch.cuda.device(device):
                    nat.check(entry(program, in_records, len(operands), out_records, len(targets), _current_stream(torch, device)))
        del keep_in, keep_out


I = Component(_handle=core.i_identity())


def i(src):
    return Component(src)
