"""𝚒 on MI355X: the gfx950 HIP backend and runtime behind the 𝚒 C ABI.

``from i_amd import Component as i, Tensor, I`` mirrors the reference's
``from ilang import Component as i, Tensor, I``.
"""
from .ilang import Component, I, Tensor, i  # noqa: F401
