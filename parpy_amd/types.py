"""Short names for element types: `parpy.types.F32` is `ElemSize.F32`, and so on for every member
(python/parpy/types.py:1-20 of the reference), plus the pointer type of an external's parameter."""
from .options import ElemSize, ExtType

globals().update({member.name: member for member in ElemSize})
__all__ = [member.name for member in ElemSize] + ["pointer"]


def pointer(ty):
    """Type of a pointer parameter of an external function whose elements have type `ty`."""
    if not isinstance(ty, ElemSize):
        raise RuntimeError(f"Provided type {ty} must be an ExtType.")
    return ExtType.Pointer(ty)
