"""The Titans backward entry point that allocates nothing
(titans_backward_noalloc_f32_rocm: work buffers in a fixed device array inside the library)
against titans_backward_f32_cuda on the same inputs, through the C ABI.  Two calls in a row, the
second on a smaller input, so that what the first call left in the shared array is seen not to
leak into the second; then d = 128, where the array also holds the partial sums of a chain's
workgroups.  Tolerance: relative 1e-4 (fp32 path) in max norm and in L2 norm; the oracle is the
second opinion on the first case.  The size limit is checked without touching the GPU.
"""
import numpy as np
import pytest
import torch

from nl_hecate_amd import dispatch as D
from nl_hecate_amd.ffi import lib
from oracle import pyoracle as orc
from tests.gpu_util import assert_close, dev, host, rule_inputs, zeros

NAMES = ("d_k", "d_v", "d_q", "d_alpha", "d_theta", "d_eta", "d_m_initial", "d_s_initial")


def _backward(entry, x, ms, ss, clip=0.0):
    B, s, d = x["k"].shape
    g = [zeros(B, s, d), zeros(B, s, d), zeros(B, s, d), zeros(B, s), zeros(B, s), zeros(B, s),
         zeros(d, d), zeros(d, d)]
    D.call(entry, dev(x["k"]), dev(x["v"]), dev(x["q"]), dev(x["alpha"]), dev(x["theta"]), dev(x["eta"]),
           dev(ms), dev(ss), dev(x["dy"]), *g, s, d, B, clip)
    torch.cuda.synchronize()
    return dict(zip(NAMES, (host(t) for t in g)))


def _case(B, s, d, seed, clip=0.0, oracle=False):
    x = rule_inputs(B, s, d, seed, m0_scale=0.3)
    if clip > 0:
        x["v"] *= 4.0
    _, ms, ss = orc.titans_forward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"],
                                         x["m0"], x["s0"], clip, orc.F32_MAX)
    got = _backward("titans_backward_noalloc_f32_rocm", x, ms, ss, clip)
    want = _backward("titans_backward_f32_cuda", x, ms, ss, clip)
    for n in NAMES:
        assert np.abs(want[n]).max() > 0, n
        assert_close(f"{n} B={B} s={s} d={d}", got[n], want[n])
    if oracle:
        go = orc.titans_backward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"], ms, ss,
                                       x["dy"], clip)
        for n in go:
            assert_close(f"{n} vs oracle", got[n], go[n])


@pytest.mark.gpu
def test_noalloc_backward_matches_the_allocating_entry_point_on_two_calls_in_a_row():
    _case(12, 96, 64, 901, oracle=True)   # fills 12 chains' worth of the array
    _case(5, 40, 64, 902)                 # smaller: stale contents beyond 5 chains must not matter
    _case(3, 33, 32, 903, clip=1.0)       # clipped errors (whole chain in one workgroup)
    _case(2, 24, 128, 904)                # four workgroups per chain: partial sums in the array
    _case(1, 9, 128, 905)


@pytest.mark.gpu
def test_noalloc_backward_allocates_nothing():
    """The property the entry point exists for: with the library's scratch arena released, a call neither grows the
    arena (its generation stays) nor takes device memory (the free byte count stays), for a chain kept in one
    workgroup, for a chain split over four (partial sums in the fixed array) and for the clipped d = 128 case that the
    general kernel serves."""
    from nl_hecate_amd.ffi import lib
    cases = [(6, 50, 64, 0.0), (2, 24, 128, 0.0), (2, 12, 128, 1.0)]
    bufs = []
    for B, s, d, clip in cases:
        x = rule_inputs(B, s, d, 950 + d, m0_scale=0.3)
        _, ms, ss = orc.titans_forward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"], x["m0"], x["s0"],
                                             error_clip=clip)
        g = [zeros(B, s, d), zeros(B, s, d), zeros(B, s, d), zeros(B, s), zeros(B, s), zeros(B, s), zeros(d, d), zeros(d, d)]
        bufs.append(([dev(x[n]) for n in ("k", "v", "q", "alpha", "theta", "eta")] + [dev(ms), dev(ss), dev(x["dy"])] + g,
                     (s, d, B, clip)))
    # once beforehand: the array's address is looked up once per device, and the runtime loads a kernel's code (and
    # sizes its own launch resources) on first use, which is not this library's doing
    for args, dims in bufs:
        D.call("titans_backward_noalloc_f32_rocm", *args, *dims)
    torch.cuda.synchronize()
    lib.nlh_release_workspace()
    gen, free = lib.nlh_workspace_generation(), torch.cuda.mem_get_info()[0]
    for args, dims in bufs:
        D.call("titans_backward_noalloc_f32_rocm", *args, *dims)
    torch.cuda.synchronize()
    assert lib.nlh_workspace_generation() == gen, "the scratch arena grew"
    assert torch.cuda.mem_get_info()[0] == free, "device memory was taken"
    # the clipped d = 128 case is within the size limit where the unclipped one of the same shape counts partial sums
    assert torch.isfinite(bufs[2][0][9]).all()


@pytest.mark.gpu
def test_noalloc_backward_accumulates_into_the_initial_state_gradients():
    """d_m_initial / d_s_initial are += targets, as in titans_backward_f32_cuda."""
    x = rule_inputs(3, 20, 16, 906, m0_scale=0.3)
    _, ms, ss = orc.titans_forward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"], x["m0"], x["s0"])
    B, s, d = x["k"].shape
    g = [zeros(B, s, d), zeros(B, s, d), zeros(B, s, d), zeros(B, s), zeros(B, s), zeros(B, s),
         torch.full((d, d), 2.0, device="cuda"), torch.full((d, d), -1.0, device="cuda")]
    D.call("titans_backward_noalloc_f32_rocm", dev(x["k"]), dev(x["v"]), dev(x["q"]), dev(x["alpha"]),
           dev(x["theta"]), dev(x["eta"]), dev(ms), dev(ss), dev(x["dy"]), *g, s, d, B, 0.0)
    torch.cuda.synchronize()
    go = orc.titans_backward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"], ms, ss, x["dy"])
    assert_close("d_m_initial", host(g[6]) - 2.0, go["d_m_initial"])
    assert_close("d_s_initial", host(g[7]) + 1.0, go["d_s_initial"])


def test_noalloc_backward_rejects_sizes_beyond_the_fixed_buffer():
    """The size check precedes every GPU call: runs without a GPU.  257 chains at d = 64 need
    2 * 257 * 4096 floats > 2 097 152; so does d = 128 with long partial sums."""
    lib.nlh_set_error_mode(1)
    try:
        for (s, d, B) in ((8, 64, 257), (4096, 128, 8)):
            lib.nlh_clear_error()
            lib.titans_backward_noalloc_f32_rocm(*([None] * 17), s, d, B, 0.0)
            msg = lib.nlh_last_error().decode()
            assert "fixed buffer" in msg and "titans_backward_noalloc_f32_rocm" in msg, msg
        lib.nlh_clear_error()
        lib.titans_backward_noalloc_f32_rocm(*([None] * 17), 8, 48, 2, 0.0)
        assert "d=48" in lib.nlh_last_error().decode()
    finally:
        lib.nlh_clear_error()
        lib.nlh_set_error_mode(0)
