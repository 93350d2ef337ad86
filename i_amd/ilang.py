"""Python frontend of the 𝚒 gfx950 backend.

Same surface as the reference frontend (ilang-python/ilang.py:147-394):
``Component`` / ``i(src)`` with the operators ``>> << & | ~``, the identity
``I``, ``Tensor`` for plain Python data, ``exec``, ``exec_numpy``,
``exec_torch``, ``into``, ``output_shapes`` and ``_code``; errors surface as
``RuntimeError(i_error())``.  Host data takes the reference's f32 path through
``i_exec_into`` / ``i_exec``.  In addition, ROCm torch tensors (float32 or
bfloat16) are passed by device pointer to ``i_exec_into_device`` and never
leave the GPU.
"""
import ctypes

from . import _native as nat

core = nat.core
_sz = ctypes.c_size_t
_f32p = ctypes.POINTER(ctypes.c_float)


class _CTensor(ctypes.Structure):
    _fields_ = [("data", _f32p), ("shape", ctypes.POINTER(_sz)), ("rank", _sz)]


class _COwnedTensor(ctypes.Structure):
    _fields_ = [("data", _f32p), ("shape", ctypes.POINTER(_sz)), ("rank", _sz), ("len", _sz)]


class _COutputs(ctypes.Structure):
    _fields_ = [("tensors", ctypes.POINTER(_COwnedTensor)), ("count", _sz)]


class _CDeviceTensor(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("shape", ctypes.POINTER(_sz)), ("rank", _sz), ("dtype", ctypes.c_int)]


_vp = ctypes.c_void_p
core.i_parse.argtypes = [ctypes.c_char_p]
core.i_parse.restype = _vp
core.i_identity.argtypes = []
core.i_identity.restype = _vp
for _name in ("i_chain", "i_compose", "i_fanout", "i_pair"):
    getattr(core, _name).argtypes = [_vp, _vp]
    getattr(core, _name).restype = _vp
core.i_swap.argtypes = [_vp]
core.i_swap.restype = _vp
core.i_code.argtypes = [_vp]
core.i_code.restype = _vp
core.i_compile.argtypes = [_vp]
core.i_compile.restype = _vp
core.i_output_count.argtypes = [_vp]
core.i_output_count.restype = _sz
core.i_output_ranks.argtypes = [_vp, ctypes.POINTER(_sz)]
core.i_output_ranks.restype = ctypes.c_int
core.i_output_shapes.argtypes = [_vp, ctypes.POINTER(_CTensor), _sz, ctypes.POINTER(ctypes.POINTER(_sz))]
core.i_output_shapes.restype = ctypes.c_int
core.i_exec_into.argtypes = [_vp, ctypes.POINTER(_CTensor), _sz, ctypes.POINTER(_CTensor), _sz]
core.i_exec_into.restype = ctypes.c_int
core.i_exec.argtypes = [_vp, ctypes.POINTER(_CTensor), _sz]
core.i_exec.restype = _COutputs
core.i_exec_into_device.argtypes = [_vp, ctypes.POINTER(_CDeviceTensor), _sz, ctypes.POINTER(_CDeviceTensor), _sz, _vp]
core.i_exec_into_device.restype = ctypes.c_int
core.i_component_free.argtypes = [_vp]
core.i_program_free.argtypes = [_vp]
core.i_outputs_free.argtypes = [_COutputs]
core.i_string_free.argtypes = [_vp]

_check, _check_ptr = nat.check, nat.check_ptr


def _shape_array(shape):
    shape = tuple(int(d) for d in shape)
    return shape, (_sz * max(len(shape), 1))(*shape)


def _flatten(x):
    if isinstance(x, (int, float)):
        return (), [float(x)]
    if not isinstance(x, (list, tuple)):
        raise TypeError("Tensor expects a scalar or nested Python lists")
    if not x:
        return (0,), []
    child_shape, _ = _flatten(x[0])
    data = []
    for item in x:
        item_shape, item_data = _flatten(item)
        if item_shape != child_shape:
            raise ValueError("ragged Tensor input")
        data.extend(item_data)
    return (len(x),) + child_shape, data


class Tensor:
    """Host tensor built from a scalar or nested lists (ilang-python/ilang.py:147-199)."""

    def __init__(self, x, shape=None):
        if shape is None:
            shape, data = _flatten(x)
        else:
            shape = tuple(int(d) for d in shape)
            data = [float(v) for v in x]
        self.shape = tuple(shape)
        self._len = len(data)
        self._data = (ctypes.c_float * max(self._len, 1))(*data)
        self._shape, self._shape_buf = _shape_array(self.shape)
        self._owner = None

    @classmethod
    def _from_owned(cls, owner, index):
        raw = owner.outputs.tensors[index]
        self = cls.__new__(cls)
        self.shape = tuple(raw.shape[i] for i in range(raw.rank))
        self._len = raw.len
        self._data = raw.data
        self._shape, self._shape_buf = _shape_array(self.shape)
        self._owner = owner
        return self

    @property
    def data(self):
        return [self._data[i] for i in range(self._len)]

    def _view(self):
        return _CTensor(ctypes.cast(self._data, _f32p), self._shape_buf, len(self.shape))

    def __repr__(self):
        return f"Tensor(shape={self.shape}, data={self.data})"


class _OwnedOutputs:
    def __init__(self, outputs):
        self.outputs = outputs

    def __del__(self, _core=core):
        outputs = getattr(self, "outputs", None)
        if outputs is not None:
            self.outputs = None
            _core.i_outputs_free(outputs)


def _is_torch(x):
    return hasattr(x, "data_ptr") and hasattr(x, "shape") and hasattr(x, "device")


def _is_device_tensor(x):
    return _is_torch(x) and str(x.device) != "cpu"


def _input(x):
    """(ctypes view, keepalive) for one host operand; non-f32 / non-contiguous data is copied to f32."""
    if isinstance(x, Tensor):
        return x._view(), x
    try:
        import numpy as np

        if isinstance(x, np.ndarray):
            arr = x
            if arr.dtype != np.float32 or not arr.flags.c_contiguous:
                arr = np.ascontiguousarray(arr, dtype=np.float32)
            shape, shape_buf = _shape_array(arr.shape)
            return _CTensor(arr.ctypes.data_as(_f32p), shape_buf, len(shape)), (arr, shape_buf)
    except ImportError:
        pass
    if _is_torch(x):
        if str(x.device) != "cpu":
            raise TypeError("mixing host and device operands is not supported; move all tensors to the GPU")
        if str(x.dtype) != "torch.float32":
            raise TypeError("Torch tensors must be float32")
        if not x.is_contiguous():
            x = x.contiguous()
        shape, shape_buf = _shape_array(tuple(x.shape))
        return _CTensor(ctypes.cast(x.data_ptr(), _f32p), shape_buf, len(shape)), (x, shape_buf)
    return _input(Tensor(x))


def _inputs(xs):
    views = [_input(x) for x in xs]
    return (_CTensor * max(len(views), 1))(*(v[0] for v in views)), views


def _output(x):
    try:
        import numpy as np

        if isinstance(x, np.ndarray):
            if x.dtype != np.float32 or not x.flags.c_contiguous:
                raise TypeError("NumPy outputs must be float32 and C-contiguous")
            shape, shape_buf = _shape_array(x.shape)
            return _CTensor(x.ctypes.data_as(_f32p), shape_buf, len(shape)), (x, shape_buf)
    except ImportError:
        pass
    if _is_torch(x):
        if str(x.device) != "cpu":
            raise TypeError("Torch outputs for host inputs must be on CPU")
        if str(x.dtype) != "torch.float32":
            raise TypeError("Torch outputs must be float32")
        if not x.is_contiguous():
            raise TypeError("Torch outputs must be contiguous")
        shape, shape_buf = _shape_array(tuple(x.shape))
        return _CTensor(ctypes.cast(x.data_ptr(), _f32p), shape_buf, len(shape)), (x, shape_buf)
    raise TypeError("outputs must be NumPy arrays or Torch tensors")


_TORCH_DTYPES = {"torch.float32": nat.F32, "torch.bfloat16": nat.BF16}


def _device_views(tensors, what):
    views, keep = [], []
    for t in tensors:
        if not _is_device_tensor(t):
            raise TypeError(f"{what} must all be GPU tensors")
        if str(t.dtype) not in _TORCH_DTYPES:
            raise TypeError(f"{what} must be float32 or bfloat16")
        if not t.is_contiguous():
            raise TypeError(f"{what} must be contiguous")
        shape, shape_buf = _shape_array(tuple(t.shape))
        views.append(_CDeviceTensor(t.data_ptr(), shape_buf, len(shape), _TORCH_DTYPES[str(t.dtype)]))
        keep.append((t, shape_buf))
    return (_CDeviceTensor * max(len(views), 1))(*views), keep


class Component:
    def __init__(self, src=None, _ptr=None):
        if _ptr is None:
            if src is None:
                raise TypeError("Component needs source")
            _ptr = core.i_parse(src.encode())
        self._ptr = _check_ptr(_ptr)
        self._program = None

    def __del__(self, _core=core):  # bound at definition: module globals may be gone at interpreter shutdown
        program, ptr = getattr(self, "_program", None), getattr(self, "_ptr", None)
        if program:
            _core.i_program_free(program)
            self._program = None
        if ptr:
            _core.i_component_free(ptr)
            self._ptr = None

    def _bin(self, other, fn):
        if not isinstance(other, Component):
            other = Component(other)
        return Component(_ptr=_check_ptr(fn(self._ptr, other._ptr)))

    def chain(self, other):
        return self._bin(other, core.i_chain)

    def compose(self, other):
        return self._bin(other, core.i_compose)

    def fanout(self, other):
        return self._bin(other, core.i_fanout)

    def pair(self, other):
        return self._bin(other, core.i_pair)

    def swap(self):
        return Component(_ptr=_check_ptr(core.i_swap(self._ptr)))

    __rshift__ = chain
    __lshift__ = compose
    __and__ = fanout
    __or__ = pair

    def __invert__(self):
        return self.swap()

    def _compile(self):
        if self._program is None:
            self._program = _check_ptr(core.i_compile(self._ptr))
        return self._program

    def _code(self):
        s = _check_ptr(core.i_code(self._ptr))
        try:
            return ctypes.cast(s, ctypes.c_char_p).value.decode()
        finally:
            core.i_string_free(s)

    def output_shapes(self, *inputs):
        program = self._compile()
        if inputs and all(_is_device_tensor(x) for x in inputs):
            views = [(_CTensor(None, _shape_array(tuple(x.shape))[1], len(x.shape)), None) for x in inputs]
            input_arr = (_CTensor * len(views))(*(v[0] for v in views))
        else:
            input_arr, views = _inputs(inputs)
        count = core.i_output_count(program)
        ranks = (_sz * max(count, 1))()
        _check(core.i_output_ranks(program, ranks))
        shape_bufs = [(_sz * max(ranks[i], 1))() for i in range(count)]
        shape_ptrs = (ctypes.POINTER(_sz) * max(count, 1))(*(ctypes.cast(b, ctypes.POINTER(_sz)) for b in shape_bufs))
        _check(core.i_output_shapes(program, input_arr, len(inputs), shape_ptrs))
        return [tuple(buf[j] for j in range(ranks[i])) for i, buf in enumerate(shape_bufs)]

    def exec(self, *inputs):
        program = self._compile()
        input_arr, keepalive = _inputs(inputs)
        outputs = core.i_exec(program, input_arr, len(inputs))
        if outputs.count == 0:
            _check(-1)
        owner = _OwnedOutputs(outputs)
        tensors = [Tensor._from_owned(owner, i) for i in range(outputs.count)]
        return tensors[0] if len(tensors) == 1 else tuple(tensors)

    def exec_numpy(self, *inputs):
        import numpy as np

        outs = [np.empty(shape, dtype=np.float32) for shape in self.output_shapes(*inputs)]
        self.into(outs if len(outs) != 1 else outs[0], *inputs)
        return outs[0] if len(outs) == 1 else tuple(outs)

    def exec_torch(self, *inputs, out_dtype=None):
        """Host tensors: as the reference (CPU float32).  GPU tensors: runs on their device
        and stream; outputs are float32 unless ``out_dtype`` says otherwise."""
        import torch

        shapes = self.output_shapes(*inputs)
        if inputs and all(_is_device_tensor(x) for x in inputs):
            outs = [torch.empty(shape, dtype=out_dtype or torch.float32, device=inputs[0].device) for shape in shapes]
        else:
            outs = [torch.empty(shape, dtype=torch.float32, device="cpu") for shape in shapes]
        self.into(outs if len(outs) != 1 else outs[0], *inputs)
        return outs[0] if len(outs) == 1 else tuple(outs)

    def into(self, outputs, *inputs):
        program = self._compile()
        if not isinstance(outputs, (tuple, list)):
            outputs = (outputs,)
        if inputs and all(_is_device_tensor(x) for x in inputs):
            import torch

            in_arr, keep_in = _device_views(inputs, "inputs")
            out_arr, keep_out = _device_views(outputs, "outputs")
            with torch.cuda.device(inputs[0].device):
                stream = torch.cuda.current_stream().cuda_stream
                _check(core.i_exec_into_device(program, in_arr, len(inputs), out_arr, len(outputs), stream))
        else:
            input_arr, keepalive = _inputs(inputs)
            out_views = [_output(out) for out in outputs]
            output_arr = (_CTensor * max(len(out_views), 1))(*(v[0] for v in out_views))
            _check(core.i_exec_into(program, input_arr, len(inputs), output_arr, len(out_views)))
        return outputs[0] if len(outputs) == 1 else tuple(outputs)


I = Component(_ptr=core.i_identity())


def i(src):
    return Component(src)
