"""Head sizes outside {8, 16, 32, 64, 128}, and clip / projection at d = 128: the general kernels
behind the same entry points (the reference's kernels take any d: core/kernels/titans_forward.cu:83-210,
titans_backward.cu:66-341, delta_forward.cu, delta_backward.cu; its own test uses d = 4,
core/tests/test_cuda_titans.rs:99-128).  Same oracle and tolerances as the tiled sizes."""
import numpy as np
import pytest
import torch

from nl_hecate_amd import dispatch as D
from oracle import pyoracle as orc
from tests.gpu_util import assert_close, dev, host, rule_inputs, zeros
from tests.test_gpu_chunkwise import gpu_chunkwise, oracle_chunkwise
from tests.test_gpu_memory_rules import (_gpu_ckpt_fwd_bwd, _oracle_ckpt_grads, gpu_delta_backward,
                                         gpu_delta_forward, gpu_titans_backward, gpu_titans_forward)

pytestmark = pytest.mark.gpu
F32_MAX = float(np.finfo(np.float32).max)


@pytest.mark.parametrize("B,s,d", [(2, 9, 1), (3, 21, 4), (2, 17, 5), (3, 30, 12), (2, 26, 24), (2, 19, 48),
                                   (2, 11, 100), (1, 7, 257)])
def test_titans_and_delta_any_head_size(B, s, d):
    x = rule_inputs(B, s, d, 12000 + d + B, m0_scale=0.2)
    y, ms, ss = gpu_titans_forward(x)
    yo, mo, so = orc.titans_forward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"],
                                          x["m0"], x["s0"])
    assert_close("y", y, yo)
    assert_close("m_states", ms, mo)
    assert_close("s_states", ss, so)
    g = gpu_titans_backward(x, mo, so)
    go = orc.titans_backward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"],
                                   mo, so, x["dy"])
    for n in go:
        assert_close(n, g[n], go[n])
    yd, md = gpu_delta_forward(x)
    ydo, mdo = orc.delta_forward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["m0"])
    assert_close("delta y", yd, ydo)
    assert_close("delta m_states", md, mdo)
    gd = gpu_delta_backward(x, mdo)
    gdo = orc.delta_backward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], mdo, x["dy"])
    for n in gdo:
        assert_close("delta " + n, gd[n], gdo[n])
    yg, mg = gpu_delta_forward(x, dgd=True)
    assert np.array_equal(yg, yd) and np.array_equal(mg, md)


@pytest.mark.parametrize("clip,mx", [(0.7, F32_MAX), (0.0, 1.5), (0.7, 1.5)])
@pytest.mark.parametrize("d", [4, 24, 128])
def test_clip_and_projection_any_head_size(clip, mx, d):
    """d = 128 splits a chain over workgroups in the tiled kernels, so the coupled reductions of clip
    and projection run in the general kernels there too."""
    x = rule_inputs(3, 23, d, 12100 + d, m0_scale=0.3)
    x["v"] *= 2.0
    y, ms, ss = gpu_titans_forward(x, clip, mx)
    yo, mo, so = orc.titans_forward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"],
                                          x["m0"], x["s0"], clip, mx)
    yn, _, _ = orc.titans_forward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"],
                                        x["m0"], x["s0"])
    assert np.abs(yo - yn).max() > 1e-4, "clip / projection must be active in this case"
    assert_close("y", y, yo)
    assert_close("m_states", ms, mo)
    assert_close("s_states", ss, so)
    if mx < 1e30:
        assert np.sqrt((ms[:, 1:] ** 2).sum((2, 3))).max() <= mx * (1 + 1e-5)
    g = gpu_titans_backward(x, mo, so, clip)
    go = orc.titans_backward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"],
                                   mo, so, x["dy"], clip)
    for n in go:
        assert_close(n, g[n], go[n])
    yd, md = gpu_delta_forward(x, clip, mx)
    ydo, mdo = orc.delta_forward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["m0"], clip, mx)
    assert_close("delta y", yd, ydo)
    gd = gpu_delta_backward(x, mdo, clip)
    gdo = orc.delta_backward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], mdo, x["dy"], clip)
    for n in gdo:
        assert_close("delta " + n, gd[n], gdo[n])


@pytest.mark.parametrize("entry", ["", "_replay"])
@pytest.mark.parametrize("B,s,d,C", [(2, 37, 4, 8), (2, 50, 24, 16), (2, 19, 48, 5), (1, 9, 100, 64)])
def test_checkpointed_backward_any_head_size(entry, B, s, d, C):
    x = rule_inputs(B, s, d, 12200 + s + d + C, m0_scale=0.2)
    for has_s in (True, False):
        g = _gpu_ckpt_fwd_bwd(x, C, has_s, entry)
        go = _oracle_ckpt_grads(x, C, has_s)
        for n in g:
            assert_close(f"{n} has_s={has_s}", g[n], go[n])


def test_checkpointed_backward_with_clip_at_d128_and_d24():
    for d in (24, 128):
        x = rule_inputs(2, 21, d, 12300 + d, m0_scale=0.3)
        x["v"] *= 2.0
        g = _gpu_ckpt_fwd_bwd(x, 8, True, "", 0.7, 1.5)
        go = _oracle_ckpt_grads(x, 8, True, 0.7, 1.5)
        for n in g:
            assert_close(f"{n} d={d}", g[n], go[n])


@pytest.mark.parametrize("has_s", [True, False])
@pytest.mark.parametrize("B,s,d,C", [(2, 40, 4, 8), (2, 50, 24, 16), (2, 23, 48, 5), (1, 20, 100, 64)])
def test_chunkwise_rule_any_head_size(has_s, B, s, d, C):
    """Frozen-M0 rule through the reference's chunkwise symbols
    (core/kernels/titans_chunkwise_forward.cu, titans_chunkwise_backward.cu)."""
    x = rule_inputs(B, s, d, 12400 + s + d + C, m0_scale=0.2)
    f, g = gpu_chunkwise(x, C, has_s)
    fo, go = oracle_chunkwise(x, C, has_s)
    assert_close("y", f["y"], fo["y"])
    assert_close("m_chunk_states", f["mc"], fo["mc"])
    if has_s:
        assert_close("s_chunk_states", f["sc"], fo["sc"])
    for n in go:
        assert_close(n, g[n], go[n])


def test_chunkwise_rule_with_clip_and_projection_d24_and_d128():
    for d in (24, 128):
        x = rule_inputs(2, 30, d, 12500 + d, m0_scale=0.3)
        x["v"] *= 2.0
        f, g = gpu_chunkwise(x, 8, True, 0.7, 1.5)
        fo, go = oracle_chunkwise(x, 8, True, 0.7, 1.5)
        assert_close(f"y d={d}", f["y"], fo["y"])
        for n in go:
            assert_close(f"{n} d={d}", g[n], go[n])


def test_segment_backward_accumulates_like_the_tiled_path():
    """d_m_initial / d_s_initial are added into the caller's buffers (core/kernels/titans_backward.cu:337-341)."""
    B, s, d = 3, 13, 12
    x = rule_inputs(B, s, d, 12600, m0_scale=0.2)
    _, mo, so = orc.titans_forward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"],
                                         x["m0"], x["s0"])
    g1 = gpu_titans_backward(x, mo, so)
    acc = torch.ones(d, d, device="cuda")
    junk = [zeros(B, s, d) for _ in range(3)] + [zeros(B, s) for _ in range(3)]
    D.titans_backward_dd(dev(x["k"]), dev(x["v"]), dev(x["q"]), dev(x["alpha"]), dev(x["theta"]),
                         dev(x["eta"]), dev(mo), dev(so), dev(x["dy"]), *junk, acc, zeros(d, d),
                         s, d, B, 0.0)
    torch.cuda.synchronize()
    assert_close("accumulated", host(acc) - 1.0, g1["d_m_initial"], 1e-4)
