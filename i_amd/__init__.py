"""𝚒 on MI355X: the gfx950 HIP backend and runtime behind the 𝚒 C ABI.

``from i_amd import Component as i, Tensor, I`` mirrors the reference's
``from ilang import Component as i, Tensor, I``.
"""
_FRONTEND = ("Component", "I", "Tensor", "i")
__all__ = list(_FRONTEND)


def __getattr__(name):
    # resolved on first use, so that ``i_amd.build`` can (re)build the native library before anything loads it
    if name in _FRONTEND:
        from . import ilang
        return getattr(ilang, name)
    raise AttributeError(f"module 'i_amd' has no attribute {name!r}")
