"""The C-ABI library loads and exports every symbol the header declares; the
drop-in names of the reference's FFI are present.  No compute calls (CPU only).
"""
import ctypes
import os
import re

from nl_hecate_amd import ffi

REF_SYMBOLS_SCOPED = """
titans_forward_f32_cuda titans_backward_f32_cuda titans_forward_ckpt_f32_cuda
titans_backward_segment_f32_cuda delta_forward_f32_cuda delta_backward_f32_cuda
delta_forward_ckpt_f32_cuda delta_backward_segment_f32_cuda dgd_forward_f32_cuda
dgd_backward_f32_cuda dgd_forward_ckpt_f32_cuda dgd_backward_segment_f32_cuda
""".split()


def test_header_parses_and_library_exports_every_declared_symbol():
    protos = ffi.parse_header()
    assert len(protos) >= 20
    cdll = ctypes.CDLL(ffi.LIB_PATH)
    missing = [n for n in protos if not hasattr(cdll, n)]
    assert not missing, f"declared in include/nl_hecate_ffi.h but not exported: {missing}"


def test_reference_ffi_names_are_declared():
    protos = ffi.parse_header()
    for name in REF_SYMBOLS_SCOPED:
        assert name in protos, name


def test_signature_arity_matches_reference_ffi():
    """Argument counts of the reference's extern "C" block (core/src/cuda_ffi.rs),
    transcribed: a drop-in must take exactly these."""
    arity = {
        "titans_forward_f32_cuda": 18, "titans_backward_f32_cuda": 21,
        "titans_forward_ckpt_f32_cuda": 16, "titans_backward_segment_f32_cuda": 25,
        "delta_forward_f32_cuda": 15, "delta_backward_f32_cuda": 17,
        "delta_forward_ckpt_f32_cuda": 13, "delta_backward_segment_f32_cuda": 20,
        "dgd_forward_f32_cuda": 14, "dgd_backward_f32_cuda": 16,
        "dgd_forward_ckpt_f32_cuda": 12, "dgd_backward_segment_f32_cuda": 20,
    }
    protos = ffi.parse_header()
    for name, n in arity.items():
        assert len(protos[name][1]) == n, (name, len(protos[name][1]), n)


def test_library_is_loadable_and_reports_version():
    assert b"gfx950" in ffi.lib.nlh_version()
    assert ffi.lib.nlh_last_error() == b""


def test_product_package_never_imports_the_oracle():
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    pkg = os.path.join(root, "nl_hecate_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert not re.search(r"\boracle\b", text), f"{f} mentions the oracle"


def test_every_function_of_the_reference_ffi_is_exported():
    """tests/golden/cuda_ffi_symbols.txt lists the `pub(crate) fn` names of core/src/cuda_ffi.rs (names only:
    data, made with grep).  Each must be declared in the header and exported by the library."""
    import ctypes
    import os
    here = os.path.dirname(os.path.abspath(__file__))
    names = open(os.path.join(here, "golden", "cuda_ffi_symbols.txt")).read().split()
    assert len(names) == 87
    from nl_hecate_amd.ffi import LIB_PATH, parse_header
    protos = parse_header()
    cdll = ctypes.CDLL(LIB_PATH)
    missing = [n for n in names if n not in protos or not hasattr(cdll, n)]
    assert not missing, missing
