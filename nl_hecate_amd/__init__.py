"""MI355X (gfx950) memory-rule kernels behind the NL_Hecate kernel FFI.

`ffi` binds the C ABI (include/nl_hecate_ffi.h); `dispatch` mirrors the
reference's device-pointer dispatch functions on torch device tensors.
"""
from . import ffi  # noqa: F401

__all__ = ["ffi", "dispatch"]
