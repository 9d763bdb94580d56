"""Host mirror of the tape's opaque-block registry (core/src/opaque_adapters.rs:1731-1760
register_opaque_vjps, core/src/tape.rs:141-150 OpaqueBackwardFn) for the blocks the GPU library
serves.  Buffers are float32 numpy arrays on the host, in the reference's saved-buffer order; the
backward ADDS into `d_inputs` (what the tape does with an adapter's result, tape.rs:839-866)."""
import ctypes

import numpy as np

from .ffi import lib

# OpaqueKey (tape.rs:100-134), the subset with a GPU adapter
DELTA_RULE, TITANS_LMM, DGD, SWA, FROZEN_DELTA_RULE, FROZEN_TITANS_LMM = 0, 1, 9, 10, 11, 12


class OpaqueBlockError(RuntimeError):
    pass


def _slices(arrays, writable=False):
    ptrs, lens = [], []
    for a in arrays:
        if not isinstance(a, np.ndarray) or a.dtype != np.float32 or not a.flags["C_CONTIGUOUS"]:
            raise ValueError("opaque block buffers are contiguous float32 numpy arrays")
        if writable and not a.flags["WRITEABLE"]:
            raise ValueError("d_inputs buffers must be writable")
        ptrs.append(a.ctypes.data)
        lens.append(a.size)
    n = len(arrays)
    return (ctypes.c_void_p * n)(*ptrs), (ctypes.c_longlong * n)(*lens), n


def opaque_backward(key, d_outputs, saved, d_inputs):
    """d_inputs[i] += gradient of input i.  Raises OpaqueBlockError with the library's message when the
    block's metadata names a configuration that has no GPU adapter or a buffer has the wrong size."""
    po, lo, no = _slices(d_outputs)
    ps, ls, ns = _slices(saved)
    pi, li, ni = _slices(d_inputs, writable=True)
    lib.nlh_set_error_mode(1)
    try:
        lib.nlh_clear_error()
        rc = lib.nlh_opaque_backward(key, po, lo, no, ps, ls, ns, pi, li, ni)
        if rc:
            raise OpaqueBlockError(f"nlh_opaque_backward rc={rc}: {lib.nlh_last_error().decode()}")
    finally:
        lib.nlh_clear_error()
        lib.nlh_set_error_mode(0)
